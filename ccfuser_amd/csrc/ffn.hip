// Expert FFN as two grouped fp16 GEMMs for gfx950.
//
// FFN1: h[j, :]          = gelu(x[src_row[j], :] * w1[e]^T + b1[e])
// FFN2: y[dst_row[j], :] = (h[j, :] * w2[e]^T + b2[e]) * row_scale[j]
// for the rows offsets[e] <= j < offsets[e+1] of every expert e.
//
// They replace the reference's moe_first_mm / moe_second_mm
// (mix_moe/csrc/cuda/mix_gemm.cu:282-436, 439-555) and what surrounds them:
// the row scatter kernel that fills the staging buffer
// (mix_moe/csrc/cuda/mix_moe_kernel.cu:18-42) becomes a row index applied
// while the A tile is fetched, the separate GELU kernel
// (mix_moe/mix_moe/transformer.py:88) and the bias become the FFN1 epilogue,
// and the index_copy_ after the second GEMM (mix_moe/csrc/mix_moe.h:433)
// becomes the FFN2 epilogue's destination row.  The reference plans 64-row
// blocks on the host in Python (mix_moe/mix_moe/transformer.py:150-250) and
// copies seven arrays to the device per call; here a one-workgroup kernel
// derives the tile list from the offsets on the device.
#include "ccf_common.h"
#include "gemm_tile.h"

namespace ccf {
namespace {

// ---- tile plan ---------------------------------------------------------------
// plan[0] = number of M tiles, then three arrays of max_tiles entries.
struct PlanView {
  const int32_t *n_tiles;
  const int32_t *expert;
  const int32_t *row0;
  const int32_t *rows;
};

__host__ __device__ inline size_t plan_ints(int max_tiles) { return 64 + 3 * static_cast<size_t>(max_tiles); }

__device__ inline PlanView plan_view(const int32_t *plan, int max_tiles) {
  return PlanView{plan, plan + 64, plan + 64 + max_tiles, plan + 64 + 2 * max_tiles};
}

__global__ void __launch_bounds__(256)
plan_kernel(const int32_t *__restrict__ offsets, int E, int BM, int max_tiles, int max_rows,
            int32_t *__restrict__ plan) {
  __shared__ int s_base[1025];
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      s_base[e] = run;
      int lo = offsets[e], hi = offsets[e + 1];
      if (hi > max_rows) hi = max_rows;              // never plan past the caller's bound
      int cnt = hi > lo ? hi - lo : 0;
      run += (cnt + BM - 1) / BM;
    }
    s_base[E] = run;
    plan[0] = run < max_tiles ? run : max_tiles;
  }
  __syncthreads();
  int32_t *expert = plan + 64, *row0 = expert + max_tiles, *rows = row0 + max_tiles;
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int lo = offsets[e], hi = offsets[e + 1];
    if (hi > max_rows) hi = max_rows;
    int cnt = hi > lo ? hi - lo : 0;
    int nt = s_base[e + 1] - s_base[e];
    for (int i = 0; i < nt; ++i) {
      int t = s_base[e] + i;
      if (t >= max_tiles) break;
      expert[t] = e;
      row0[t] = lo + i * BM;
      rows[t] = (cnt - i * BM) < BM ? (cnt - i * BM) : BM;
    }
  }
}

// ---- grouped GEMM kernel -------------------------------------------------------
struct GroupedArgs {
  const half_t *A;          // [*, K] rows
  const int32_t *a_rows;    // row of A for sorted row j, or NULL (identity)
  const half_t *B;          // [E, N, K]
  const half_t *bias;       // [E, N]
  half_t *C;                // [*, N]
  const int32_t *c_rows;    // row of C for sorted row j, or NULL (identity)
  const half_t *row_scale;  // [rows] or NULL
  const int32_t *plan;
  int max_tiles;
  int n_tiles_n;
  int N, K;
};

constexpr int kGroupM = 4;

__device__ __forceinline__ float gelu_erf(float v) {
  return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
}

template <class Cfg, bool kGelu>
__global__ void __launch_bounds__(Cfg::THREADS)
grouped_gemm_kernel(GroupedArgs p) {
  using ML = GemmMainloop<Cfg>;
  // Hardware hands consecutive workgroup ids to the 8 XCDs in turn; undo that so
  // that one XCD (one L2) works on a contiguous run of logical tile ids.
  const int per_xcd = gridDim.x >> 3;               // grid is a multiple of 8
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  // Runs of kGroupM M tiles x all N tiles: neighbours share A rows and B rows.
  const int group_sz = kGroupM * p.n_tiles_n;
  const int first_m = (logical / group_sz) * kGroupM;
  const int gm = (p.max_tiles - first_m) < kGroupM ? (p.max_tiles - first_m) : kGroupM;
  if (gm <= 0) return;
  const int in_group = logical % group_sz;
  const int tile_m = first_m + in_group % gm;
  const int tile_n = in_group / gm;
  const PlanView pv = plan_view(p.plan, p.max_tiles);
  if (tile_m >= pv.n_tiles[0] || tile_n >= p.n_tiles_n) return;

  const int e = pv.expert[tile_m];
  const int row0 = pv.row0[tile_m];
  const int rows = pv.rows[tile_m];
  const int n0 = tile_n * Cfg::BN;
  const half_t *Be = p.B + static_cast<size_t>(e) * p.N * p.K;

  const half_t *a_src[Cfg::A_DMA];
  const half_t *b_src[Cfg::B_DMA];
#pragma unroll
  for (int i = 0; i < Cfg::A_DMA; ++i) {
    const int r = ML::dma_row(i);
    const int rc = r < rows ? r : rows - 1;          // padded rows re-read a valid row
    const int g = p.a_rows ? p.a_rows[row0 + rc] : row0 + rc;
    a_src[i] = p.A + static_cast<size_t>(g) * p.K + ML::dma_chunk(r) * 8;
  }
#pragma unroll
  for (int i = 0; i < Cfg::B_DMA; ++i) {
    const int r = ML::dma_row(i);
    const int n = (n0 + r) < p.N ? (n0 + r) : p.N - 1;
    b_src[i] = Be + static_cast<size_t>(n) * p.K + ML::dma_chunk(r) * 8;
  }

  typename ML::acc_t acc[Cfg::TM][Cfg::TN];
#pragma unroll
  for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < Cfg::TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;

  ML::run(acc, a_src, b_src, p.K);

  // Epilogue: bias (+ GELU) (+ row scale), fp16 store through the row index.
  const half_t *bias_e = p.bias + static_cast<size_t>(e) * p.N;
  float bias_v[Cfg::TN];
  int col[Cfg::TN];
#pragma unroll
  for (int tn = 0; tn < Cfg::TN; ++tn) {
    col[tn] = n0 + acc_col<Cfg>(tn);
    bias_v[tn] = col[tn] < p.N ? static_cast<float>(bias_e[col[tn]]) : 0.0f;
  }
#pragma unroll
  for (int tm = 0; tm < Cfg::TM; ++tm) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int lr = acc_row<Cfg>(tm, r);
      if (lr < rows) {
        const int j = row0 + lr;
        const size_t crow = p.c_rows ? static_cast<size_t>(p.c_rows[j]) : static_cast<size_t>(j);
        const float sc = p.row_scale ? static_cast<float>(p.row_scale[j]) : 1.0f;
        half_t *dst = p.C + crow * p.N;
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn) {
          float v = acc[tm][tn][r] + bias_v[tn];
          if (kGelu) v = gelu_erf(v);
          v *= sc;
          if (col[tn] < p.N) dst[col[tn]] = static_cast<half_t>(v);
        }
      }
    }
  }
}

// ---- variants -------------------------------------------------------------------
using CfgA = GemmCfg<256, 256, 64, 2, 4, 2>;   // 8 wavefronts, 128x64 each, 128 KB LDS
using CfgB = GemmCfg<256, 128, 64, 2, 2, 3>;   // 4 wavefronts, 128x64 each, 144 KB LDS
using CfgC = GemmCfg<128, 128, 64, 2, 2, 2>;   // 4 wavefronts, 64x64 each, 64 KB LDS (2 per CU)
using CfgD = GemmCfg<256, 256, 64, 4, 2, 2>;   // 8 wavefronts, 64x128 each

int g_variant = 0;

struct Launch {
  int bm, bn, threads;
  void (*plain)(GroupedArgs);
  void (*gelu)(GroupedArgs);
};

const Launch kVariants[] = {
    {CfgA::BM, CfgA::BN, CfgA::THREADS, grouped_gemm_kernel<CfgA, false>, grouped_gemm_kernel<CfgA, true>},
    {CfgB::BM, CfgB::BN, CfgB::THREADS, grouped_gemm_kernel<CfgB, false>, grouped_gemm_kernel<CfgB, true>},
    {CfgC::BM, CfgC::BN, CfgC::THREADS, grouped_gemm_kernel<CfgC, false>, grouped_gemm_kernel<CfgC, true>},
    {CfgD::BM, CfgD::BN, CfgD::THREADS, grouped_gemm_kernel<CfgD, false>, grouped_gemm_kernel<CfgD, true>},
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
constexpr int kMinBM = 128;

int max_tiles_for(int max_rows, int E, int bm) { return (max_rows + bm - 1) / bm + E; }

size_t plan_bytes(int max_rows, int E) {
  return round_up(sizeof(int32_t) * plan_ints(max_tiles_for(max_rows, E, kMinBM)), 256);
}

int grouped_gemm(const half_t *A, const int32_t *a_rows, const int32_t *offsets, int max_rows, int E,
                 int N, int K, const half_t *B, const half_t *bias, bool gelu, half_t *C,
                 const int32_t *c_rows, const half_t *row_scale, int32_t *plan, hipStream_t stream,
                 const char *what) {
  CCF_REQUIRE(A && offsets && B && bias && C && plan, CCF_ERR_ARG, "%s: null pointer", what);
  CCF_REQUIRE(max_rows >= 0 && E > 0 && N > 0 && K > 0, CCF_ERR_ARG, "%s: bad size", what);
  CCF_REQUIRE(E <= 1024, CCF_ERR_SHAPE, "%s: num_expert=%d exceeds 1024", what, E);
  CCF_REQUIRE(K % 64 == 0, CCF_ERR_SHAPE, "%s: K=%d is not a multiple of 64", what, K);
  CCF_REQUIRE(N % 8 == 0, CCF_ERR_SHAPE, "%s: N=%d is not a multiple of 8", what, N);
  CCF_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), CCF_ERR_ARG,
              "%s: operands must be 16-byte aligned", what);
  if (max_rows == 0) return CCF_OK;
  const Launch &v = kVariants[g_variant];
  const int max_tiles = max_tiles_for(max_rows, E, v.bm);
  hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(256), 0, stream, offsets, E, v.bm, max_tiles,
                     max_rows, plan);
  if (int rc = check_launch("plan_kernel")) return rc;
  GroupedArgs p;
  p.A = A;
  p.a_rows = a_rows;
  p.B = B;
  p.bias = bias;
  p.C = C;
  p.c_rows = c_rows;
  p.row_scale = row_scale;
  p.plan = plan;
  p.max_tiles = max_tiles;
  p.n_tiles_n = (N + v.bn - 1) / v.bn;
  p.N = N;
  p.K = K;
  // whole groups of kGroupM M tiles, rounded to a multiple of 8 workgroups
  const long long groups = (max_tiles + kGroupM - 1) / kGroupM;
  long long wgs = groups * kGroupM * p.n_tiles_n;
  wgs = (wgs + 7) / 8 * 8;
  CCF_REQUIRE(wgs < (1ll << 31), CCF_ERR_SHAPE, "%s: grid too large", what);
  hipLaunchKernelGGL(gelu ? v.gelu : v.plain, dim3(static_cast<unsigned>(wgs)), dim3(v.threads), 0,
                     stream, p);
  return check_launch(what);
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_set_option(const char *name, int value) {
  using namespace ccf;
  CCF_REQUIRE(name, CCF_ERR_ARG, "set_option: null name");
  if (!strcmp(name, "gemm_variant")) {
    CCF_REQUIRE(value >= 0 && value < kNumVariants, CCF_ERR_ARG, "set_option: gemm_variant %d outside 0..%d",
                value, kNumVariants - 1);
    g_variant = value;
    return CCF_OK;
  }
  return fail(CCF_ERR_ARG, "set_option: unknown option %s", name);
}

extern "C" size_t ccf_ffn_workspace_bytes(int max_rows, int num_expert, int d_model, int d_ffn) {
  if (max_rows < 0 || num_expert <= 0 || d_model <= 0 || d_ffn <= 0) return 0;
  return ccf::plan_bytes(max_rows, num_expert);
}

extern "C" int ccf_ffn1_forward(const void *x, const int32_t *src_row, const int32_t *dst_row,
                                const int32_t *offsets, int max_rows, int num_expert, int d_model,
                                int d_ffn, const void *w1, const void *b1, int apply_gelu, void *h,
                                void *workspace, size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(workspace && workspace_bytes >= plan_bytes(max_rows, num_expert), CCF_ERR_WORKSPACE,
              "ffn1: workspace of %zu bytes needed, %zu given", plan_bytes(max_rows, num_expert),
              workspace_bytes);
  return grouped_gemm(static_cast<const half_t *>(x), src_row, offsets, max_rows, num_expert, d_ffn,
                      d_model, static_cast<const half_t *>(w1), static_cast<const half_t *>(b1),
                      apply_gelu != 0, static_cast<half_t *>(h), dst_row, nullptr,
                      static_cast<int32_t *>(workspace), as_stream(stream), "ffn1");
}

extern "C" int ccf_ffn2_forward(const void *h, const int32_t *src_row, const int32_t *dst_row,
                                const int32_t *offsets, int max_rows, int num_expert, int d_model,
                                int d_ffn, const void *w2, const void *b2, const void *row_scale,
                                void *y, void *workspace, size_t workspace_bytes,
                                ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(workspace && workspace_bytes >= plan_bytes(max_rows, num_expert), CCF_ERR_WORKSPACE,
              "ffn2: workspace of %zu bytes needed, %zu given", plan_bytes(max_rows, num_expert),
              workspace_bytes);
  return grouped_gemm(static_cast<const half_t *>(h), src_row, offsets, max_rows, num_expert, d_model,
                      d_ffn, static_cast<const half_t *>(w2), static_cast<const half_t *>(b2), false,
                      static_cast<half_t *>(y), dst_row, static_cast<const half_t *>(row_scale),
                      static_cast<int32_t *>(workspace), as_stream(stream), "ffn2");
}
