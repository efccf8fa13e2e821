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
#include "gelu.h"
#include "plan.h"

namespace ccf {
namespace {

// The main loop of a tile shape: eight wavefronts (two per SIMD, half the registers each) keep one
// register buffer of token fragments, four wavefronts two.
template <class Cfg, bool kKN, bool kRows = false>
using RingFor = Ring16Mainloop<Cfg, kKN, Cfg::NW == 8, kRows>;

// ---- tile plan ---------------------------------------------------------------
// build_plan() (plan.h) in a launch of its own; the layer's forward call lets the routing
// stage build both of its plans instead.
// Several workgroups share the work (build_plan's `part`): enough that every expert has a wavefront, at most 8.
constexpr int kPlanThreads = 256;
__global__ void __launch_bounds__(kPlanThreads)
plan_kernel(PlanReq rq, const int32_t *__restrict__ offsets, int E) {
  build_plan(rq, offsets, E, blockIdx.x, gridDim.x);
}
// Workgroups that build a plan: a wavefront per expert at least; wavefronts beyond that share the experts'
// entries (the builder is on the critical path of its launch, and the chip is idle beside it).
inline int plan_workgroups(int) { return 8; }

// ---- grouped GEMM kernel -------------------------------------------------------
struct GroupedArgs {
  const half_t *A;          // [*, K] rows
  const int32_t *a_rows;    // row of A for sorted row j, or NULL (identity)
  const half_t *B;          // [E, N, K]
  const half_t *bias;       // [E, N]
  half_t *C;                // [*, N]
  half_t *C2;               // [*, N] in sorted row order: the pre-activation, written by epilogue 2, read by epilogue 3
  const int32_t *c_rows;    // row of C for sorted row j, or NULL (identity)
  const half_t *row_scale;  // [rows] or NULL; NULL with the GELU epilogue
  const int32_t *scale_rows; // epilogue 4: row_scale is read at scale_rows[j]; NULL elsewhere
  const int32_t *plan;
  int N, K;
  // K-segment form (weight gradients): the contraction runs over a per-expert
  // range of columns of A and B, which are then [rows, lda] and [N, ldb] matrices
  // shared by all experts; expert e owns columns k_seg[e] .. k_seg[e+1] (multiples
  // of BK, at least four K tiles) and rows e*seg_rows .. of C.  NULL otherwise.
  const int32_t *k_seg;
  int lda, ldb, seg_rows;
  // split last round (layout in plan.h): header and part entries, fp32 partial tiles
  const int32_t *tail;
  float *partial;
  // rows form (weight gradients without transposed copies): A [rows, lda] and B [rows, ldb] are row-major
  // activation matrices in expert order, the contraction of expert e runs over rows k_seg[e] .. k_seg[e+1]
  // (any number, also none), and rows past the end are fetched from this row of 256 zeros
  const half_t *zero_row;
  // skinny list (layout in plan.h) of this GEMM, or NULL
  const int32_t *skinny;
  float *sk_partial;        // partial tiles of the skinny tiles when they run as a launch of their own
  int tail_inside;          // 1: the persistent launch runs the parts of the split last round itself (no tail launch)
  int sk_positions;         // skinny ranges inside the persistent launch: most points in time they are spread over (0: one per round)
};

// Epilogue forms of the grouped GEMM.
//   0  C = (acc + bias) * row_scale
//   1  C = gelu(acc + bias)
//   2  as 1, and C2 = acc + bias (the pre-activation a later backward needs)
//   3  C = (acc + bias) * gelu'(C2): an input gradient taken straight through the GELU
//   4  C[c_rows[j]] += (acc + bias) * row_scale[scale_rows[j]] with packed fp16 atomic adds: the gate-weighted
//      combine in the second GEMM's epilogue (C zero-filled by the caller, c_rows = token of sorted row j)
constexpr int kEpiPlain = 0, kEpiGelu = 1, kEpiGeluKeep = 2, kEpiGeluGrad = 3, kEpiCombine = 4;

// Row of the tile's row range [0, rows) that tile row r (0 .. BM-1) holds; padded
// tile rows repeat a real one.  The upper and the lower half of the tile (one row
// of wavefronts each) get half of the rows each, so that a partly filled tile
// skips MFMAs in both.
template <class Cfg>
__device__ __forceinline__ int tile_row_to_local(int r, int rows) {
  return RingFor<Cfg, false>::local_row(r, rows);
}

// Global source of every tile load of this lane for the tile of plan entry
// `ent`: K element 0 of the (clamped) A row and B row, at this lane's K chunk.
// Padded A rows re-read the tile's last real row, B rows past N the last row.
// tid: threadIdx.x, or fresh_tid() where what is derived from it must not be kept from an earlier call.
template <class Cfg, bool kSeg = false, bool kKN = false>
__device__ __forceinline__ void tile_sources(const GroupedArgs &p, const int4v ent,
                                             const half_t *(&a_src)[Cfg::A_DMA],
                                             const half_t *(&b_src)[kKN ? 2 : Cfg::B_DMA], int tid) {
  using ML = GemmMainloop<Cfg>;
  const int row0 = ent[1], rows = ent[2], n0 = ent[3] * Cfg::BN;
  const int lda = kSeg ? p.lda : p.K, ldb = kSeg ? p.ldb : p.K;
  const half_t *Ae = p.A, *Be;
  if constexpr (kSeg) {
    const int koff = p.k_seg[ent[0]];
    Ae = p.A + koff;
    Be = p.B + koff;
  } else {
    Be = p.B + static_cast<size_t>(ent[0]) * p.N * p.K;
  }
#pragma unroll
  for (int i = 0; i < Cfg::A_DMA; ++i) {
    const int r = ML::dma_row(i, tid);
    const int rc = tile_row_to_local<Cfg>(r, rows);
    int g = row0 + rc;
    if constexpr (kSeg) g -= ent[0] * p.seg_rows;      // sorted row j of expert e is row j - e*seg_rows of A
    else if (p.a_rows) g = p.a_rows[g];
    if constexpr (kSeg) {
      a_src[i] = Ae + static_cast<size_t>(static_cast<uint32_t>(g)) * static_cast<uint32_t>(lda) + ML::dma_chunk(r, tid) * 8;
    } else {
      a_src[i] = p.A + static_cast<size_t>(g) * p.K + ML::dma_chunk(r, tid) * 8;
    }
  }
  if constexpr (kKN) {
    // B is [E, K, N]: K row r of the tile, the columns LDS unit u of that row holds (N % BN == 0)
    using R = RingFor<Cfg, true>;
#pragma unroll
    for (int i = 0; i < 2; ++i) {                          // loads 0 and 1; load i >= 2 is 16 rows below load i - 2
      const int r = R::kn_dma_row(i, tid);
      b_src[i] = Be + static_cast<size_t>(r) * p.N + n0 + R::kn_col(r, R::kn_dma_unit(tid));
    }
  } else {
#pragma unroll
    for (int i = 0; i < Cfg::B_DMA; ++i) {
      const int r = ML::dma_row(i, tid);
      const int n = (n0 + r) < p.N ? (n0 + r) : p.N - 1;
      if constexpr (kSeg) {
        b_src[i] = Be + static_cast<size_t>(n) * ldb + ML::dma_chunk(r, tid) * 8;
      } else {
        b_src[i] = Be + static_cast<size_t>(n) * p.K + ML::dma_chunk(r, tid) * 8;
      }
    }
  }
}

// Loads through the scalar cache of data no kernel in flight writes (the tile plan, the K
// ranges), complete on return.  Inside the tile loop the compiler would use vector loads for
// them (the kernel's own stores might alias), and a vector load queues behind the epilogue's
// stores.
typedef int int2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ int4v scalar_load4(const int4v *q) {
  int4v r;
  asm volatile("s_load_dwordx4 %0, %1, 0x0\n s_waitcnt lgkmcnt(0)" : "=s"(r) : "s"(q) : "memory");
  return r;
}
// two entries with one wait
__device__ __forceinline__ void scalar_load4x2(const int4v *q0, const int4v *q1, int4v &r0, int4v &r1) {
  asm volatile("s_load_dwordx4 %0, %2, 0x0\n s_load_dwordx4 %1, %3, 0x0\n s_waitcnt lgkmcnt(0)"
               : "=&s"(r0), "=&s"(r1)
               : "s"(q0), "s"(q1)
               : "memory");
}
__device__ __forceinline__ int2v scalar_load2(const int32_t *q) {
  int2v r;
  asm volatile("s_load_dwordx2 %0, %1, 0x0\n s_waitcnt lgkmcnt(0)" : "=s"(r) : "s"(q) : "memory");
  return r;
}

// K tiles [first, first + count) of part `part` of S over k_tiles K tiles.
__device__ __forceinline__ void part_range(int k_tiles, int part, int S, int &first, int &count) {
  const int base = k_tiles / S, rem = k_tiles % S;
  count = base + (part < rem ? 1 : 0);
  first = part * base + (part < rem ? part : rem);
}

// K tiles of expert e's contraction.
template <class Cfg, bool kSeg, bool kRows = false>
__device__ __forceinline__ int k_tiles_of(const GroupedArgs &p, int e) {
  if constexpr (kRows) {
    // rows form: the expert's rows in K tiles, the last one partly masked; never fewer than the pipeline needs
    const int eu = __builtin_amdgcn_readfirstlane(e);
    const int2v r = scalar_load2(p.k_seg + eu);
    const int kt = (r[1] - r[0] + Cfg::BK - 1) / Cfg::BK;
    return kt < 4 ? 4 : kt;
  } else if constexpr (kSeg) {
    const int eu = __builtin_amdgcn_readfirstlane(e);
    const int2v r = scalar_load2(p.k_seg + eu);
    return (r[1] - r[0]) / Cfg::BK;
  } else {
    return p.K / Cfg::BK;
  }
}

// Rows form: sources of the tile loads of both operands for the tile {expert e, first output row row0, N tile},
// and the K mask (the expert's row count seen from this lane's first K row).
template <class Cfg>
__device__ __forceinline__ void rows_sources(const GroupedArgs &p, int e, int row0, int tile_n, const half_t *(&a_src)[2],
                                             const half_t *(&b_src)[2], typename RingFor<Cfg, true, true>::KMask &mk) {
  using R = RingFor<Cfg, true, true>;
  const int eu = __builtin_amdgcn_readfirstlane(e);
  const int2v seg = scalar_load2(p.k_seg + eu);
  const int m0 = row0 - eu * p.seg_rows, n0 = tile_n * Cfg::BN;
  const int tid = fresh_tid();
  const int unit = R::kn_dma_unit(tid);
  const half_t *Ae = p.A + static_cast<size_t>(seg[0]) * p.lda + m0;
  const half_t *Be = p.B + static_cast<size_t>(seg[0]) * p.ldb + n0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {                           // loads 0 and 1; load i >= 2 is 16 rows below load i - 2
    const int r = R::kn_dma_row(i, tid);
    const int col = R::kn_col(r, unit);
    a_src[i] = Ae + static_cast<size_t>(r) * p.lda + col;
    b_src[i] = Be + static_cast<size_t>(r) * p.ldb + col;
  }
  mk.klim = seg[1] - seg[0] - R::kn_dma_row(0, tid);
  mk.zero = p.zero_row + unit * 8;
}

// x, y: this lane's four columns of two neighbouring 16-column blocks.  Lanes 16 apart swap
// (v_permlane16_swap: the odd 16-lane rows of the first operand with the even rows of the
// second), so that an even row ends with columns 4q .. 4q+7 of the first block and an odd
// row with columns 4(q-1) .. 4(q-1)+7 of the second, in order.
__device__ __forceinline__ half8 pair_exchange(half4 x, half4 y) {
  typedef unsigned uint2v __attribute__((ext_vector_type(2)));
  const uint2v xv = __builtin_bit_cast(uint2v, x), yv = __builtin_bit_cast(uint2v, y);
  const uint2v r0 = __builtin_amdgcn_permlane16_swap(xv[0], yv[0], false, false);
  const uint2v r1 = __builtin_amdgcn_permlane16_swap(xv[1], yv[1], false, false);
  typedef unsigned uint4v __attribute__((ext_vector_type(4)));
  const uint4v all = {r0[0], r1[0], r0[1], r1[1]};
  return __builtin_bit_cast(half8, all);
}

// Epilogue of the 16x16x32 accumulator layout: bias (+ GELU) (+ row scale),
// fp16, 8-byte stores through the row index.
template <class Cfg, int kEpi, bool kPlainRows = false>     // kPlainRows: no row index, no row scale, no bias
__device__ __forceinline__ void epilogue16(const GroupedArgs &p, int e, int row0, int rows, int n0) {
  using R = RingFor<Cfg, false>;
  constexpr int TM = R::TM, TN = R::TN;
  const int tid = fresh_tid();
  const half_t *bias_e = p.bias + static_cast<size_t>(e) * p.N;
  float bias_v[TN][4];
  int col[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    col[tn] = n0 + acc16_col4<Cfg>(tn, tid);
    half4 bv = {0, 0, 0, 0};
    if (p.bias && col[tn] < p.N) bv = *reinterpret_cast<const half4 *>(bias_e + col[tn]);
#pragma unroll
    for (int c = 0; c < 4; ++c) bias_v[tn][c] = static_cast<float>(bv[c]);
  }
  // Row data of all TM row blocks is looked up before the first accumulator is touched: one
  // memory round trip for the tile instead of one per row block (padded tile rows look up the
  // real row they repeat, so every index is in range).
  int crow_v[TM];
  float sc_v[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int j = row0 + R::local_row(acc16_row<Cfg>(tm, tid), rows);
    crow_v[tm] = (!kPlainRows && p.c_rows) ? p.c_rows[j] : j;
    if constexpr (kEpi == kEpiCombine) sc_v[tm] = static_cast<float>(p.row_scale[p.scale_rows[j]]);
    else sc_v[tm] = (!kPlainRows && p.row_scale) ? static_cast<float>(p.row_scale[j]) : 1.0f;
  }
  static_for<0, TM>([&](auto T) {
    constexpr int tm = T.value;
    const int tr = acc16_row<Cfg>(tm, tid);               // tile row
    const bool real = R::row_is_real(tr, rows);
    const int lr = R::local_row(tr, rows);
    // the accumulator reads are unconditional (they are asm the compiler must not skip per lane)
    float v[TN][4];
    static_for<0, TN>([&](auto J) {
      constexpr int tn = J.value;
      v[tn][0] = R::template acc_get<tm, tn, 0>();
      v[tn][1] = R::template acc_get<tm, tn, 1>();
      v[tn][2] = R::template acc_get<tm, tn, 2>();
      v[tn][3] = R::template acc_get<tm, tn, 3>();
    });
    const int j = row0 + lr;
    const float sc = sc_v[tm];
    half_t *dst = p.C + static_cast<size_t>(crow_v[tm]) * p.N;
    if constexpr (kEpi == kEpiPlain || kEpi == kEpiCombine) {
      // A lane holds columns 4q .. 4q+3 of every 16-column block (q = lane / 16).  Lanes q and
      // q^1 of a row trade halves of a pair of blocks, after which the even one holds eight
      // consecutive columns of the first block and the odd one of the second: half as many
      // stores, 16 bytes each.  A store costs per instruction and cache line touched, not per
      // byte: 64 eight-byte stores per lane took 9.6 us of a tile's epilogue, 32 sixteen-byte
      // ones 3.4.  Every lane takes part in the exchange, padded rows included.  (The GELU
      // epilogues are bound by their arithmetic, which hides the stores: they keep the plain form.)
      const int q = (tid & 63) >> 4;
#pragma unroll
      for (int tp = 0; tp < TN / 2; ++tp) {
        half4 o[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            o[h][c] = static_cast<half_t>(kPlainRows ? v[2 * tp + h][c]          // weight gradients: no bias, no scale
                                                     : (v[2 * tp + h][c] + bias_v[2 * tp + h][c]) * sc);
        const int c16 = col[2 * tp] - 4 * q + (q & 1) * 16 + 4 * (q & 2);   // first of this lane's 8 columns
        const half8 out = pair_exchange(o[0], o[1]);
        if constexpr (kEpi == kEpiCombine) {
          // eight columns as four packed fp16 atomic adds (no return value)
          if (real && c16 < p.N) {
            typedef unsigned uint4v_ __attribute__((ext_vector_type(4)));
            const uint4v_ bits = __builtin_bit_cast(uint4v_, out);
            half_t *at = dst + c16;
#pragma unroll
            for (int u = 0; u < 4; ++u)
              asm volatile("global_atomic_pk_add_f16 %0, %1, off offset:%2" ::"v"(at), "v"(bits[u]), "n"(4 * u) : "memory");
          }
        } else {
          if (real && c16 < p.N) *reinterpret_cast<half8 *>(dst + c16) = out;
        }
      }
    } else if (real) {
      half_t *row2 = p.C2 + static_cast<size_t>(j) * p.N;           // epilogues 2 and 3 only
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        half4 o, pre = {0, 0, 0, 0};
        if (kEpi == kEpiGeluGrad && col[tn] < p.N) pre = *reinterpret_cast<const half4 *>(row2 + col[tn]);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float x = v[tn][c] + bias_v[tn][c];
          if (kEpi == kEpiGeluGrad) {
            x *= gelu_erf_grad(static_cast<float>(pre[c]));
          } else {
            if (kEpi == kEpiGeluKeep) pre[c] = static_cast<half_t>(x);
            x = gelu_erf(x);                          // FFN1: no row scale
          }
          o[c] = static_cast<half_t>(x);
        }
        if (col[tn] < p.N) {
          *reinterpret_cast<half4 *>(dst + col[tn]) = o;
          if (kEpi == kEpiGeluKeep) *reinterpret_cast<half4 *>(row2 + col[tn]) = pre;
        }
      }
    }
  });
}

// One workgroup per tile (the form used when K is too short for the persistent kernel).
template <class Cfg, int kEpi, bool kSeg = false, bool kKN = false>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::MIN_WAVES_PER_SIMD)
grouped_gemm_kernel(GroupedArgs p) {
  const int4v ent = reinterpret_cast<const int4v *>(p.plan)[blockIdx.x];
  const int e = ent[0];
  if (e < 0) return;                                 // surplus workgroup of the worst-case grid
  const half_t *a_src[Cfg::A_DMA];
  const half_t *b_src[kKN ? 2 : Cfg::B_DMA];
  tile_sources<Cfg, kSeg, kKN>(p, ent, a_src, b_src, threadIdx.x);
  RingFor<Cfg, kKN>::run(a_src, b_src, k_tiles_of<Cfg, kSeg>(p, e) * Cfg::BK, ent[2], p.N);
  epilogue16<Cfg, kEpi, kSeg>(p, e, ent[1], ent[2], ent[3] * Cfg::BN);
}

// ---- skinny tiles -----------------------------------------------------------------
// The rows an expert has beyond its full 256-row tiles, when the plan says so (plan.h tells which
// rows and when), as 64 x 256 tiles over the skinny list.  Such a tile does little arithmetic
// per byte of weights it streams, so this loop is built for memory latency, not for the MFMA
// pipe: four whole-K-tile stages of 40 KB (the persistent kernel's 160 KB of LDS: three K tiles
// in flight while one is read), the same direct-to-LDS loads and XOR swizzle as the main loop,
// four wavefronts side by side along N (64 x 64 each), fragment reads and MFMAs back to back.
// It runs in the few workgroups per XCD of the persistent kernel that the plan sets aside:
// worker `worker` of `ns` on XCD `xcd` takes entries worker, worker + ns, ... of that XCD's
// share of the list.  Accumulation runs over K in the same 32-wide steps and the same order as
// in the main loop, so a skinny tile gives the bits a 256-row tile would give.
struct SkinnyCfg {
  static constexpr int BM = kSkinnyRows, BN = 256, BK = 64;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE_BYTES = A_BYTES + B_BYTES, STAGES = 4;
  static constexpr int A_DMA = BM / 8 / 4, B_DMA = BN / 8 / 4;     // tile loads per wavefront: 8 rows of 128 bytes each
  static constexpr int TM = BM / 16, TN = 4;                       // 16 x 16 blocks per wavefront (64 x 64)
  static constexpr int LOADS = A_DMA + B_DMA;
};

// Layout of a [K][N] weight tile of 64 x 256 in LDS: the one the 256 x 256 main loop uses.
using SkinnyKN = RingFor<GemmCfg<256, 256, 64, 2, 2, 8>, true>;

// acc += w (16 weight rows) x t (16 token rows), K = 32, on ordinary registers
__device__ __forceinline__ void mfma16_v(float4v &acc, const half8 &w, const half8 &t) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(w), "v"(t));
}

// Accumulators of one 64 x 256 skinny tile: wavefront w owns columns 64 w .. 64 w + 63, block (tm, tn) of a lane is
// row 16 tm + lane % 16, columns 64 w + 16 tn + 4 (lane / 16) .. + 3.
typedef float4v SkinnyAcc[SkinnyCfg::TM][SkinnyCfg::TN];

// This lane's fragment chunk of row block 0, per K half (16x16x32 operand: row lane % 16, K chunk lane / 16).
// kKN: the weight tile sits in LDS as [K][N] rows in the main loop's layout of such a tile (its column
// blocks of 16 are XOR-swizzled inside each half of 128 columns; wavefront w reads blocks 4 (w % 2) .. + 3
// of half w / 2 through transposing reads, block tn at the address XOR 32 tn).
template <bool kKN>
__device__ __forceinline__ void skinny_frag_offsets(int tid, uint32_t (&a_off)[2], uint32_t (&b_off)[2]) {
  using C = SkinnyCfg;
  using KN = SkinnyKN;
  const int lane = tid & 63, wave = tid >> 6;
  const int ra = lane & 15, rb = wave * 64 + (lane & 15);
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    const int c = sub * 4 + (lane >> 4);
    a_off[sub] = (ra * 8 + (c ^ swz<8>(ra))) * 16;
    if constexpr (kKN) {
      const int j = lane & 15;
      const int row = sub * 32 + 8 * (lane >> 4) + (j >> 2);
      b_off[sub] = C::A_BYTES + row * KN::KN_PITCH + (wave >> 1) * 256 + ((KN::kn_swz(row) ^ ((wave & 1) * 4)) << 5) + ((j & 3) << 3);
    } else {
      b_off[sub] = C::A_BYTES + (rb * 8 + (c ^ swz<8>(rb))) * 16;
    }
  }
}

// acc = the tile of list entry `ent` over K tiles [kt0, kt0 + nkt) (nkt >= 1), accumulated over K in 32-wide steps
// in ascending order.  All four wavefronts of the workgroup call it together.  kKN: the weights are [E, K, N].
template <bool kKN>
__device__ __forceinline__ void skinny_mainloop(const GroupedArgs &p, const int4v ent, int kt0, int nkt, SkinnyAcc &acc,
                                                const uint32_t (&a_off)[2], const uint32_t (&b_off)[2], int tid,
                                                lds_char *lds, uint32_t lds_base) {
  using C = SkinnyCfg;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // = the wavefront's 64 columns
  const int e = ent[0], row0 = ent[1], rows = ent[2], n0 = ent[3] * C::BN;
  int live_m = (rows + 15) / 16;                                   // 16-row blocks with real rows
  live_m = __builtin_amdgcn_readfirstlane(live_m > C::TM ? C::TM : live_m);
  // global source of every tile load of this lane, at K tile kt0
  const half_t *a_src[C::A_DMA], *b_src[C::B_DMA];
  const half_t *Be = p.B + static_cast<size_t>(e) * p.N * p.K + static_cast<size_t>(kt0) * C::BK * (kKN ? p.N : 1);
  const int bmul = kKN ? p.N : 1;                                  // elements between K rows of the weights
#pragma unroll
  for (int j = 0; j < C::A_DMA; ++j) {
    const int r = (j * 4 + wave) * 8 + (lane >> 3);
    int g = row0 + (r < rows ? r : rows - 1);                      // padded tile rows re-read the last real row
    if (p.a_rows) g = p.a_rows[g];
    a_src[j] = p.A + static_cast<size_t>(g) * p.K + static_cast<size_t>(kt0) * C::BK + ((lane & 7) ^ swz<8>(r)) * 8;
  }
#pragma unroll
  for (int j = 0; j < C::B_DMA; ++j) {
    if constexpr (kKN) {
      // a load is two K rows of 256 columns (N % 256 == 0); which columns a 16-byte unit holds: the main loop's layout
      using KN = SkinnyKN;
      const int r = KN::kn_dma_row(j, tid);
      b_src[j] = Be + static_cast<size_t>(r) * p.N + n0 + KN::kn_col(r, KN::kn_dma_unit(tid));
    } else {
      const int r = (j * 4 + wave) * 8 + (lane >> 3);
      const int n = (n0 + r) < p.N ? (n0 + r) : p.N - 1;
      b_src[j] = Be + static_cast<size_t>(n) * p.K + ((lane & 7) ^ swz<8>(r)) * 8;
    }
  }
  auto issue = [&](int kt, int stage) {                            // K tile kt0 + kt into a stage
    const int k_elem = (kt < nkt ? kt : nkt - 1) * C::BK;          // past the end: the last tile again, into a stage nobody reads
    lds_char *base = lds + stage * C::STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < C::A_DMA; ++j) lds_dma16(a_src[j] + k_elem, base + (j * 4 + wave) * 1024);
#pragma unroll
    for (int j = 0; j < C::B_DMA; ++j)
      lds_dma16(b_src[j] + static_cast<size_t>(k_elem) * bmul, base + C::A_BYTES + (j * 4 + wave) * 1024);
  };
#pragma unroll
  for (int tm = 0; tm < C::TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < C::TN; ++tn) acc[tm][tn] = float4v{0, 0, 0, 0};
  wait_vmcnt<0>();                                                 // the previous tile's stores: the waits below count loads only
  block_barrier();                                                 // and its last LDS reads are done
  issue(0, 0);
  issue(1, 1);
  issue(2, 2);
  int stage = 0;
  for (int kt = 0; kt < nkt; ++kt) {
    // K tile kt has landed for this wavefront (the loads of the two tiles behind it may be in flight), then for all
    wait_vmcnt<2 * C::LOADS>();
    block_barrier();
    // behind the barrier everyone is done with K tile kt-1, whose stage takes K tile kt+3
    issue(kt + 3, stage >= 1 ? stage - 1 : C::STAGES - 1);
    const uint32_t sb = lds_base + stage * C::STAGE_BYTES;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      half8 a[C::TM], b[C::TN];
      static_for<0, C::TN>([&](auto J) {
        if constexpr (kKN) {
          const uint32_t addr = (sb + b_off[sub]) ^ (J.value * 32);
          const half4 lo = lds_read_tr_b64<0>(addr);
          const half4 hi = lds_read_tr_b64<4 * SkinnyKN::KN_PITCH>(addr);
          b[J.value] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
          b[J.value] = lds_read_b128<J.value * 2048>(sb + b_off[sub]);
        }
      });
      static_for<0, C::TM>([&](auto I) { a[I.value] = lds_read_b128<I.value * 2048>(sb + a_off[sub]); });
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int q = 0; q < C::TM; ++q) asm volatile("" : "+v"(a[q]));
#pragma unroll
      for (int q = 0; q < C::TN; ++q) asm volatile("" : "+v"(b[q]));
      static_for<0, C::TM>([&](auto I) {
        constexpr int tm = I.value;
        if (tm < live_m) {                                         // uniform
#pragma unroll
          for (int tn = 0; tn < C::TN; ++tn) mfma16_v(acc[tm][tn], b[tn], a[tm]);
        }
      });
    }
    stage = stage == C::STAGES - 1 ? 0 : stage + 1;
  }
  wait_vmcnt<0>();                                                 // the redundant loads past the end
  // the MFMAs are opaque to the compiler: keep the distance it would keep before their results are read
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");
#pragma unroll
  for (int tm = 0; tm < C::TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < C::TN; ++tn) asm volatile("" : "+v"(acc[tm][tn]));
}

template <int kEpi, bool kKN>
__device__ __forceinline__ void skinny_role(const GroupedArgs &p, int worker, int ns, int xcd, lds_char *lds,
                                            uint32_t lds_base) {
  using C = SkinnyCfg;
  static_assert(C::STAGES * C::STAGE_BYTES <= 5 * 32768, "the stages share the ring's LDS");
  const int T = p.skinny[0], per_x = p.skinny[2];
  const int4v *list = reinterpret_cast<const int4v *>(p.skinny + kSkinnyHead);
  const int tid = fresh_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int KT = p.K / C::BK;
  uint32_t a_off[2], b_off[2];
  skinny_frag_offsets<kKN>(tid, a_off, b_off);
  for (int i = worker; i < per_x; i += ns) {
    const int w = xcd * per_x + i;
    if (w >= T) break;
    const int4v ent = list[w];
    const int e = ent[0], row0 = ent[1], rows = ent[2], n0 = ent[3] * C::BN;
    int live_m = (rows + 15) / 16;
    live_m = __builtin_amdgcn_readfirstlane(live_m > C::TM ? C::TM : live_m);
    SkinnyAcc acc;
    skinny_mainloop<kKN>(p, ent, 0, KT, acc, a_off, b_off, tid, lds, lds_base);
    // epilogue: bias, GELU or row scale, fp16 through the row index; 8-byte stores
    const half_t *bias_e = p.bias + static_cast<size_t>(e) * p.N;
    const int colb = n0 + wave * 64 + 4 * (lane >> 4);             // column of block tn = colb + 16 tn
#pragma unroll
    for (int tm = 0; tm < C::TM; ++tm) {
      if (tm >= live_m) break;                                     // uniform
      const int r = tm * 16 + (lane & 15);
      const bool real = r < rows;
      const int j = row0 + (real ? r : rows - 1);
      const size_t crow = p.c_rows ? static_cast<size_t>(p.c_rows[j]) : static_cast<size_t>(j);
      const float sc = p.row_scale ? static_cast<float>(p.row_scale[j]) : 1.0f;
      half_t *dst = p.C + crow * p.N;
      half_t *row2 = kEpi == kEpiGeluKeep ? p.C2 + static_cast<size_t>(j) * p.N : nullptr;
#pragma unroll
      for (int tn = 0; tn < C::TN; ++tn) {
        const int col = colb + 16 * tn;
        if (!real || col >= p.N) continue;
        half4 bv = {0, 0, 0, 0};
        if (p.bias) bv = *reinterpret_cast<const half4 *>(bias_e + col);
        half4 o, pre;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float x = acc[tm][tn][c] + static_cast<float>(bv[c]);
          if (kEpi == kEpiPlain) {
            x *= sc;
          } else {
            pre[c] = static_cast<half_t>(x);
            x = gelu_erf(x);
          }
          o[c] = static_cast<half_t>(x);
        }
        *reinterpret_cast<half4 *>(dst + col) = o;
        if (kEpi == kEpiGeluKeep) *reinterpret_cast<half4 *>(row2 + col) = pre;
      }
    }
  }
  wait_vmcnt<0>();
}

// The skinny list as a launch of its own (plan.h): workgroup w of W takes K steps [w q, (w + 1) q) of the sequence
// "tile 0's K steps, tile 1's, ..." and leaves one raw fp32 partial tile per list entry it touches, in fragment order
// (block (tm, tn) of thread t at float4 index (4 tm + tn) * 256 + t), in its slots w * kSkTailSegs + 0, 1, ...
// `inside`: called by the persistent launch (1) or by the launch behind it (0); the plan says which of them runs it.
template <bool kKN>
__device__ __forceinline__ void skinny_tail_role(const GroupedArgs &p, int w, int inside, lds_char *lds, uint32_t lds_base) {
  using C = SkinnyCfg;
  if (!p.skinny) return;
  const int T = p.skinny[0], q = p.skinny[3];
  if (T <= 0 || q <= 0 || p.skinny[4] != inside) return;
  const int KT = p.K / C::BK;
  const int total = T * KT;
  const int s0 = w * q;
  if (s0 >= total) return;
  const int s1 = s0 + q < total ? s0 + q : total;
  const int4v *list = reinterpret_cast<const int4v *>(p.skinny + kSkinnyHead);
  const int tid = fresh_tid();
  uint32_t a_off[2], b_off[2];
  skinny_frag_offsets<kKN>(tid, a_off, b_off);
  int t = s0 / KT;
  for (int seg = 0; seg < kSkTailSegs && t * KT < s1; ++seg, ++t) {
    const int k0 = (s0 > t * KT ? s0 : t * KT) - t * KT;
    const int k1 = (s1 < (t + 1) * KT ? s1 : (t + 1) * KT) - t * KT;
    SkinnyAcc acc;
    skinny_mainloop<kKN>(p, list[t], k0, k1 - k0, acc, a_off, b_off, tid, lds, lds_base);
    float4v *out = reinterpret_cast<float4v *>(p.sk_partial) +
                   static_cast<size_t>(w * kSkTailSegs + seg) * (C::TM * C::TN * 256) + tid;
#pragma unroll
    for (int tm = 0; tm < C::TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < C::TN; ++tn) out[(tm * C::TN + tn) * 256] = acc[tm][tn];
  }
  wait_vmcnt<0>();
  block_barrier();                                   // every wavefront is done with LDS before a caller's next tile loads
}

// Row block tm (16 rows) of skinny tile t: the sum of its partial tiles in K order, then the epilogue.
// One workgroup of 256 threads; thread t holds what thread t of the producing workgroup held.
template <int kEpi>
__device__ __forceinline__ void skinny_reduce_block(const GroupedArgs &p, int t, int tm) {
  using C = SkinnyCfg;
  const int q = p.skinny[3];
  const int KT = p.K / C::BK;
  const int4v ent = reinterpret_cast<const int4v *>(p.skinny + kSkinnyHead)[t];
  const int e = ent[0], row0 = ent[1], rows = ent[2], n0 = ent[3] * C::BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = tm * 16 + (lane & 15);
  if (tm * 16 >= rows) return;
  const int w_lo = (t * KT) / q, w_hi = ((t + 1) * KT - 1) / q;
  float4v acc[C::TN];
#pragma unroll
  for (int tn = 0; tn < C::TN; ++tn) acc[tn] = float4v{0, 0, 0, 0};
  // four partial tiles at a time: their loads leave together, the sums stay in K order
  for (int w0 = w_lo; w0 <= w_hi; w0 += 4) {
    float4v v[4][C::TN];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int w = w0 + u <= w_hi ? w0 + u : w_hi;              // past the end: a copy that is not added
      const int seg = t - (w * q) / KT;
      const float4v *src = reinterpret_cast<const float4v *>(p.sk_partial) +
                           static_cast<size_t>(w * kSkTailSegs + seg) * (C::TM * C::TN * 256) + (tm * C::TN) * 256 + tid;
#pragma unroll
      for (int tn = 0; tn < C::TN; ++tn) v[u][tn] = src[tn * 256];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (w0 + u <= w_hi) {
#pragma unroll
        for (int tn = 0; tn < C::TN; ++tn) acc[tn] += v[u][tn];
      }
  }
  if (r >= rows) return;
  const int j = row0 + r;
  const size_t crow = p.c_rows ? static_cast<size_t>(p.c_rows[j]) : static_cast<size_t>(j);
  const float sc = p.row_scale ? static_cast<float>(p.row_scale[j]) : 1.0f;
  const half_t *bias_e = p.bias + static_cast<size_t>(e) * p.N;
#pragma unroll
  for (int tn = 0; tn < C::TN; ++tn) {
    const int col = n0 + wave * 64 + 16 * tn + 4 * (lane >> 4);
    if (col >= p.N) continue;
    half4 bv = {0, 0, 0, 0};
    if (p.bias) bv = *reinterpret_cast<const half4 *>(bias_e + col);
    half4 o, pre;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float x = acc[tn][c] + static_cast<float>(bv[c]);
      if (kEpi == kEpiPlain) {
        x *= sc;
      } else {
        pre[c] = static_cast<half_t>(x);
        x = gelu_erf(x);
      }
      o[c] = static_cast<half_t>(x);
    }
    *reinterpret_cast<half4 *>(p.C + crow * p.N + col) = o;
    if (kEpi == kEpiGeluKeep) *reinterpret_cast<half4 *>(p.C2 + static_cast<size_t>(j) * p.N + col) = pre;
  }
}

// ---- persistent form -------------------------------------------------------------
// One workgroup per CU walks the plan entries of its XCD (entry b belongs to XCD
// b % 8; the workgroup with blockIdx b takes slots b/8, b/8 + gridDim/8, ...).
// What it buys over one workgroup per tile: the first two K tiles of the NEXT
// tile are loaded by the last two K-tile steps of the current one (where the
// plain kernel re-fetches its last K tile into slots nobody reads), so they
// arrive under the epilogue, and the next main loop starts with operands in
// LDS and its first fragments in registers; no workgroup launch, no pipeline
// fill, no drain between tiles.  The ring phase (which slot holds what) simply
// carries on across tiles.
//
// Per tile (K has at least four K tiles): the row indices of the next tile's A
// rows are requested before the first step (plain loads in inline asm, so that
// no compiler-placed wait drains the tile loads in flight; the vmcnt wait of
// the first barrier covers them); steps 0 .. KT-3 run with this tile's sources;
// then the sources of the next tile are computed and the last two steps load
// its K tiles 0 and 1.
template <class Cfg, int kEpi, bool kSeg = false, bool kKN = false>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::MIN_WAVES_PER_SIMD)
grouped_gemm_persistent_kernel(GroupedArgs p, int slots_per_xcd) {
  using ML = GemmMainloop<Cfg>;
  constexpr bool kRows = kSeg && kKN;                 // both operands row-major with the contraction over rows
  using R = RingFor<Cfg, kKN, kRows>;
  const int bmul = kRows ? p.ldb : (kKN ? p.N : 1);   // elements between K rows of a [K][N] B
  const int amul = kRows ? p.lda : 1;                 // and of a [K][M] A
  constexpr int TM = R::TM, TN = R::TN;
  const int4v *plan = reinterpret_cast<const int4v *>(p.plan);
  const int xcd = blockIdx.x & 7;
  int stride = gridDim.x >> 3;
  int slot_j = blockIdx.x >> 3;
  if constexpr (!kSeg && kEpi <= kEpiGeluKeep && Cfg::NW == 4) {
    // the last ns workgroups of each XCD do the skinny tiles (if the plan has any), the others the 256-row tiles
    if (p.skinny) {
      const int ns = __builtin_amdgcn_readfirstlane(p.skinny[1]);
      stride -= ns;
      if (slot_j >= stride) {
        skinny_role<kEpi, kKN>(p, slot_j - stride, ns, xcd, R::lds(), R::lds_addr());
        return;
      }
    }
  }
  // Skinny tiles cut along K inside this launch (plan.h): every workgroup takes its range of their K steps
  // at some point between its 256-row tiles: behind its first sk_pos tiles (0 = in front of all, more than
  // it has = behind all).  The points are spread over the launch by XCD: the workgroups of an XCD pause
  // together, so they stay in step with each other and keep sharing operand tiles through their L2 (spread
  // by groups of slots inside an XCD measured slower), and at any time only about 1 / (rounds + 1) of the
  // chip streams weights for skinny tiles while the rest computes.
  constexpr bool kSkInside = !kSeg && kEpi <= kEpiGeluKeep && Cfg::NW == 4;
  int sk_pos = -1;                                    // -1: no range to run
  if constexpr (kSkInside) {
    if (p.skinny && p.skinny[4] == 1 && p.skinny[0] > 0) {
      const int rounds = __builtin_amdgcn_readfirstlane(p.skinny[5]);
      int npos = rounds + 1;
      npos = (p.sk_positions >= 2 && p.sk_positions < npos) ? p.sk_positions : npos;
      const int at = xcd % npos;
      sk_pos = (at * rounds + (npos - 1) / 2) / (npos - 1);     // npos >= 2: rounds >= 1
    }
    if (sk_pos == 0) {
      skinny_tail_role<kKN>(p, static_cast<int>(blockIdx.x), 1, R::lds(), R::lds_addr());
      sk_pos = -1;
    }
  }
  // Plan entries are read through uniform indices (scalar loads, which do not queue behind the
  // epilogue's stores) and one tile ahead of their use: `ahead` is the entry after the next one.
  // The used slots of an XCD are a prefix; behind a workgroup's last tile comes, once, its part of
  // the split last round (entry blockIdx.x of the split list, expert -1 when there is none, marked by
  // its part count in bits 24..), when the launcher leaves the parts to this launch.  That entry is
  // fetched together with the first plan entry, so it costs no wait of its own.
  constexpr bool kTailInside = !kSeg && kEpi <= kEpiGeluKeep && Cfg::NW == 4;
  int4v tail_ent = int4v{-1, 0, 0, 0};
  int4v ent = int4v{-1, 0, 0, 0};
  {
    const int4v *first = plan + __builtin_amdgcn_readfirstlane((slot_j < slots_per_xcd ? slot_j : 0) * 8 + xcd);
    bool with_tail = false;
    if constexpr (kTailInside) with_tail = p.tail_inside != 0 && p.tail != nullptr;
    if (with_tail) {
      const int me = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x));
      scalar_load4x2(first, reinterpret_cast<const int4v *>(p.tail + 64) + me, ent, tail_ent);
    } else {
      ent = scalar_load4(first);
    }
    if (slot_j >= slots_per_xcd) ent[0] = -1;
  }
  auto take_tail = [&](int4v &t) {
    if constexpr (kTailInside) {
      if (t[0] < 0 && tail_ent[0] >= 0) {
        t = tail_ent;
        tail_ent[0] = -1;
      }
    }
  };
  take_tail(ent);
  auto entry_at = [&](int j) {
    int4v t = int4v{-1, 0, 0, 0};
    if (j < slots_per_xcd) t = scalar_load4(plan + __builtin_amdgcn_readfirstlane(j * 8 + xcd));
    take_tail(t);
    return t;
  };
  // K tiles of an entry and the first of them: all of K, or the part's range
  auto k_span = [&](const int4v &e, int &first) {
    int kt = k_tiles_of<Cfg, kSeg, kRows>(p, e[0]);
    first = 0;
    if constexpr (kTailInside) {
      const int S = e[3] >> 24;
      if (S) part_range(kt, (e[3] >> 16) & 0xff, S, first, kt);
    }
    return kt;
  };
  if (ent[0] < 0) {                                   // neither a 256-row tile nor a part for this workgroup
    if constexpr (kSkInside) {
      if (sk_pos > 0) skinny_tail_role<kKN>(p, static_cast<int>(blockIdx.x), 1, R::lds(), R::lds_addr());
    }
    return;
  }
  int4v ahead = entry_at(slot_j + stride);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const half_t *a_src[R::A_SRCS];
  const half_t *b_src[kKN ? 2 : Cfg::B_DMA];
  typename R::KMask mk{0, nullptr};
  // sources of an entry from scratch (the first tile, and the tile behind a skinny range)
  auto sources_of = [&](const int4v &e, int first, int tid) {
    if constexpr (kRows) {
      rows_sources<Cfg>(p, e[0], e[1], e[3], a_src, b_src, mk);
    } else {
      int4v e2 = e;
      e2[3] &= 0xffff;
      tile_sources<Cfg, kSeg, kKN>(p, e2, a_src, b_src, tid);
      if constexpr (kTailInside) {
        if (first) {
#pragma unroll
          for (int i = 0; i < Cfg::A_DMA; ++i) a_src[i] += first * Cfg::BK;
#pragma unroll
          for (int i = 0; i < (kKN ? 2 : Cfg::B_DMA); ++i) b_src[i] += static_cast<size_t>(first * Cfg::BK) * bmul;
        }
      }
    }
  };
  int k_first0 = 0;
  const int kt0 = k_span(ent, k_first0);
  sources_of(ent, k_first0, threadIdx.x);
  int a_off[2], b_off[2];
  R::frag_offsets(a_off, b_off);
  half8 fa[R::AB][TM], fb[2][TN];
  R::prologue(fa, fb, a_src, b_src, kt0, a_off, b_off, wave, bmul, amul, mk);
  R::reserve();
  int phase = 0;
  int tiles_done = 0;

  for (;;) {
    // the entry after this one; without one, the tail steps re-fetch this tile's first K tiles.  When the
    // skinny range comes behind this tile, the next tile starts from scratch behind it instead.
    const int nj = slot_j + stride;
    const bool real_next = ahead[0] >= 0;
    const bool pause = kSkInside && real_next && tiles_done + 1 == sk_pos;
    const bool has_next = real_next && !pause;
    const int4v nent = has_next ? ahead : ent;
    ahead = has_next ? entry_at(nj + stride) : ahead;  // used by the next tile: its latency hides under this one
    const int n_row0 = nent[1], n_rows = nent[2];
    int k_first = 0, n_first = 0;
    const int KT = k_span(ent, k_first);
    k_span(nent, n_first);
    const int k_end = KT * Cfg::BK;

    R::zero_acc();

    int next_row[kRows ? 1 : Cfg::A_DMA];             // A row of the next tile per tile load
    if constexpr (!kSeg) {
      const int tid0 = fresh_tid();
#pragma unroll
      for (int i = 0; i < Cfg::A_DMA; ++i) {
        const int r = ML::dma_row(i, tid0);
        const int rc = R::local_row(r, n_rows);
        if (p.a_rows) {
          const int32_t *src = p.a_rows + n_row0 + rc;
          asm volatile("global_load_dword %0, %1, off" : "=v"(next_row[i]) : "v"(src) : "memory");
        } else {
          next_row[i] = n_row0 + rc;
        }
      }
    }

    // The eight-wavefront form runs the MFMAs of padded row blocks too (they repeat real rows and are not
    // stored): with half the registers, the branch around each row block makes the compiler park values in
    // accumulation registers, which this kernel owns.
    const int live_m = (Cfg::NW == 8 || kRows) ? TM : R::live_blocks(ent[2]);   // rows form: the tile's rows are weight rows, all real
    R::acc_settle();
    if (live_m == TM) {
      R::template k_range<true>(fa, fb, a_src, b_src, a_off, b_off, KT - 2, 2 * Cfg::BK, k_end, phase, wave, live_m, bmul,
                                amul, mk);
    } else {
      R::template k_range<false>(fa, fb, a_src, b_src, a_off, b_off, KT - 2, 2 * Cfg::BK, k_end, phase, wave, live_m, bmul,
                                 amul, mk);
    }
    if constexpr (kRows) {
      // sources and K mask of the next tile
      int n_e = __builtin_amdgcn_readfirstlane(nent[0]), n_r0 = __builtin_amdgcn_readfirstlane(nent[1]),
          n_tn = __builtin_amdgcn_readfirstlane(nent[3]);
      asm volatile("" : "+s"(n_e), "+s"(n_r0), "+s"(n_tn));
      rows_sources<Cfg>(p, n_e, n_r0, n_tn, a_src, b_src, mk);
    } else {
      // sources of the next tile (tile_sources() with the row indices already at hand); the
      // empty asm keeps the compiler from computing them before the loop above and holding
      // 16 more registers across it
      int n_e = __builtin_amdgcn_readfirstlane(nent[0]), n_tn = __builtin_amdgcn_readfirstlane(nent[3] & 0xffff);
      int n_k0 = __builtin_amdgcn_readfirstlane(n_first * Cfg::BK);      // a part starts inside K
      asm volatile("" : "+s"(n_e), "+s"(n_tn), "+s"(n_k0));
      const int lda = kSeg ? p.lda : p.K, ldb = kSeg ? p.ldb : p.K;
      const half_t *Ae = p.A, *Be;
      if constexpr (kSeg) {
        const int koff = p.k_seg[n_e];
        Ae = p.A + koff;
        Be = p.B + koff;
      } else {
        Be = p.B + static_cast<size_t>(n_e) * p.N * p.K;
      }
      const int n0 = n_tn * Cfg::BN;
      const int tid1 = fresh_tid();
#pragma unroll
      for (int i = 0; i < Cfg::A_DMA; ++i) {
        const int r = ML::dma_row(i, tid1);
        if constexpr (kSeg) {
          // sorted row j of expert e is row j - e*seg_rows of A; nothing to look up, so it is computed here
          int nr0 = __builtin_amdgcn_readfirstlane(nent[1]), nrows = __builtin_amdgcn_readfirstlane(nent[2]);
          asm volatile("" : "+s"(nr0), "+s"(nrows));
          next_row[i] = nr0 - n_e * p.seg_rows + R::local_row(r, nrows);
        } else {
          asm volatile("" : "+v"(next_row[i]));       // requested before step 0, complete at its barrier
        }
        if constexpr (kSeg) {
          a_src[i] = Ae + static_cast<size_t>(static_cast<uint32_t>(next_row[i])) * static_cast<uint32_t>(lda) +
                     ML::dma_chunk(r, tid1) * 8;
        } else {
          a_src[i] = p.A + static_cast<size_t>(next_row[i]) * p.K + (n_k0 + ML::dma_chunk(r, tid1) * 8);
        }
      }
      if constexpr (kKN) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int r = R::kn_dma_row(i, tid1);
          b_src[i] = Be + (static_cast<size_t>(r) + n_k0) * p.N + n0 + R::kn_col(r, R::kn_dma_unit(tid1));
        }
      } else {
#pragma unroll
        for (int i = 0; i < Cfg::B_DMA; ++i) {
          const int r = ML::dma_row(i, tid1);
          const int n = (n0 + r) < p.N ? (n0 + r) : p.N - 1;
          if constexpr (kSeg) {
            b_src[i] = Be + static_cast<size_t>(n) * ldb + ML::dma_chunk(r, tid1) * 8;
          } else {
            b_src[i] = Be + static_cast<size_t>(n) * p.K + (n_k0 + ML::dma_chunk(r, tid1) * 8);
          }
        }
      }
    }
    if (live_m == TM) {
      R::template k_range<true>(fa, fb, a_src, b_src, a_off, b_off, 2, 0, 4 * Cfg::BK, phase, wave, live_m, bmul, amul, mk);
    } else {
      R::template k_range<false>(fa, fb, a_src, b_src, a_off, b_off, 2, 0, 4 * Cfg::BK, phase, wave, live_m, bmul, amul, mk);
    }
    R::acc_settle();
    bool is_part = false;
    if constexpr (kTailInside) is_part = (ent[3] >> 24) != 0;
    if (is_part) {
      // a part of the split last round: raw accumulators for the reduction launch, by workgroup id
      float *out = p.partial + static_cast<size_t>(blockIdx.x) * (Cfg::BM * Cfg::BN);
      const int tid = fresh_tid();
      static_for<0, TM>([&](auto T) {
        constexpr int tm = T.value;
        const int tr = acc16_row<Cfg>(tm, tid);
        static_for<0, TN>([&](auto J) {
          constexpr int tn = J.value;
          float4v v;
          v[0] = R::template acc_get<tm, tn, 0>();
          v[1] = R::template acc_get<tm, tn, 1>();
          v[2] = R::template acc_get<tm, tn, 2>();
          v[3] = R::template acc_get<tm, tn, 3>();
          *reinterpret_cast<float4v *>(out + tr * Cfg::BN + acc16_col4<Cfg>(tn, tid)) = v;
        });
      });
    } else {
      epilogue16<Cfg, kEpi, kSeg>(p, ent[0], ent[1], ent[2], (ent[3] & 0xffff) * Cfg::BN);
    }
    R::acc_settle();
    ++tiles_done;
    if (!real_next) break;
    if constexpr (kSkInside) {
      if (pause) {
        // the skinny range, then the next tile as the first one was started
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_vmcnt<0>();
        skinny_tail_role<kKN>(p, static_cast<int>(blockIdx.x), 1, R::lds(), R::lds_addr());
        sk_pos = -1;
        ent = ahead;
        slot_j = nj;
        ahead = entry_at(nj + stride);
        int first_p = 0;
        const int kt_p = k_span(ent, first_p);
        sources_of(ent, first_p, fresh_tid());
        R::prologue(fa, fb, a_src, b_src, kt_p, a_off, b_off, wave, bmul, amul, mk);
        phase = 0;
        continue;
      }
    }
    ent = nent;
    slot_j = nj;
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  wait_vmcnt<0>();
  if constexpr (kSkInside) {
    if (sk_pos > 0) skinny_tail_role<kKN>(p, static_cast<int>(blockIdx.x), 1, R::lds(), R::lds_addr());
  }
}


// ---- split-K tail -----------------------------------------------------------------
// Tiles all take about the same time, so a launch whose tile count is no multiple of the
// workgroup count ends with a round in which most CUs idle: config 3's FFN2 has 592 tiles for
// 256 workgroups, 2.3 rounds that cost 3.  plan_kernel therefore keeps the tiles of each XCD's
// last, partly filled round out of the plan when they are few enough to matter (at most half a
// round) and cuts each into S parts along K, S = workgroups per XCD / tiles (at most 8, at
// least four K tiles per part).  The parts run as one more launch, one workgroup each, and
// leave raw fp32 accumulators in a scratch area; splitk_reduce adds a tile's parts in part
// order and applies the epilogue.  The area sits in front of the plan in the caller's workspace
// (kTailHead, kTailBytes above).

// One part of one tail tile per workgroup: the main loop over its K range, raw accumulators out.
// Workgroups from `split_wgs` on run the skinny list as a launch of its own (skinny_tail_role).
template <class Cfg, bool kKN = false>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::MIN_WAVES_PER_SIMD)
grouped_gemm_tail_kernel(GroupedArgs p, int split_wgs) {
  using R = RingFor<Cfg, kKN>;
  if (static_cast<int>(blockIdx.x) >= split_wgs) {
    skinny_tail_role<kKN>(p, static_cast<int>(blockIdx.x) - split_wgs, 0, R::lds(), R::lds_addr());
    return;
  }
  const int bmul = kKN ? p.N : 1;                      // elements between K rows of a [K][N] B
  const int tiles = p.tail[0], S = p.tail[1];
  if (static_cast<int>(blockIdx.x) >= tiles * S) return;
  int4v ent = reinterpret_cast<const int4v *>(p.tail + 64)[blockIdx.x];
  if (ent[0] < 0) return;                              // this XCD's last round had fewer tiles
  const int part = (ent[3] >> 16) & 0xff;
  ent[3] &= 0xffff;
  int first, count;
  part_range(p.K / Cfg::BK, part, S, first, count);
  const half_t *a_src[Cfg::A_DMA];
  constexpr int NB = kKN ? 2 : Cfg::B_DMA;
  const half_t *b_src[NB];
  tile_sources<Cfg, false, kKN>(p, ent, a_src, b_src, threadIdx.x);
#pragma unroll
  for (int i = 0; i < Cfg::A_DMA; ++i) a_src[i] += first * Cfg::BK;
#pragma unroll
  for (int i = 0; i < NB; ++i) b_src[i] += static_cast<size_t>(first * Cfg::BK) * bmul;
  R::run(a_src, b_src, count * Cfg::BK, ent[2], bmul);
  float *out = p.partial + static_cast<size_t>(blockIdx.x) * (Cfg::BM * Cfg::BN);
  const int tid = fresh_tid();
  static_for<0, R::TM>([&](auto T) {
    constexpr int tm = T.value;
    const int tr = acc16_row<Cfg>(tm, tid);
    static_for<0, R::TN>([&](auto J) {
      constexpr int tn = J.value;
      float4v v;
      v[0] = R::template acc_get<tm, tn, 0>();
      v[1] = R::template acc_get<tm, tn, 1>();
      v[2] = R::template acc_get<tm, tn, 2>();
      v[3] = R::template acc_get<tm, tn, 3>();
      *reinterpret_cast<float4v *>(out + tr * Cfg::BN + acc16_col4<Cfg>(tn, tid)) = v;
    });
  });
}

// out tile = sum of its S partial tiles (in part order) + bias, then the epilogue kEpi of the
// grouped GEMM.  grid (kReduceX, BM / 16): block (x, q) does tile rows 16q .. 16q+15 of tile slots
// x, x + kReduceX, ... of the split last round, a thread four rows of four columns, and then its share
// of the (tile, row block) pairs of skinny tiles that were cut along K.  It runs at the speed the
// partial tiles stream back in (config 3, FFN2: 63 MB in 13 us when its last round was split).
template <class Cfg, int kEpi>
__device__ __forceinline__ void reduce_split_tile(const GroupedArgs &p, int t, int S) {
  using R = RingFor<Cfg, false>;
  const int first_wg = (t & 7) + 8 * ((t >> 3) * S);   // workgroup id of part 0; part s is 8 s further
  const int4v ent = reinterpret_cast<const int4v *>(p.tail + 64)[first_wg];
  const int e = ent[0], row0 = ent[1], rows = ent[2], n0 = (ent[3] & 0xffff) * Cfg::BN;
  if (e < 0) return;
  const int c4 = threadIdx.x & 63;                     // which group of four columns
  const int col = n0 + 4 * c4;
  if (col >= p.N) return;
  float bias_v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (p.bias) {
    const half4 bv = *reinterpret_cast<const half4 *>(p.bias + static_cast<size_t>(e) * p.N + col);
#pragma unroll
    for (int c = 0; c < 4; ++c) bias_v[c] = static_cast<float>(bv[c]);
  }
  float4v acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
  const int r_first = blockIdx.y * 16 + (threadIdx.x >> 6);
  const float *src = p.partial + static_cast<size_t>(first_wg) * (Cfg::BM * Cfg::BN) + r_first * Cfg::BN + 4 * c4;
  // four parts at a time: their loads leave together, the sums stay in part order
  for (int s0 = 0; s0 < S; s0 += 4) {
    float4v v[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int sp = s0 + u < S ? s0 + u : S - 1;                // past the end: a copy that is not added
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[u][i] = *reinterpret_cast<const float4v *>(src + static_cast<size_t>(8 * sp) * (Cfg::BM * Cfg::BN) + 4 * i * Cfg::BN);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (s0 + u < S) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += v[u][i];
      }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r_first + 4 * i;
    if (!R::row_is_real(r, rows)) continue;
    const int j = row0 + R::local_row(r, rows);
    const size_t crow = p.c_rows ? static_cast<size_t>(p.c_rows[j]) : static_cast<size_t>(j);
    const float sc = p.row_scale ? static_cast<float>(p.row_scale[j]) : 1.0f;
    half4 o, pre;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float x = acc[i][c] + bias_v[c];
      if (kEpi == kEpiGelu || kEpi == kEpiGeluKeep) {
        pre[c] = static_cast<half_t>(x);
        x = gelu_erf(x);
      } else {
        x *= sc;
      }
      o[c] = static_cast<half_t>(x);
    }
    *reinterpret_cast<half4 *>(p.C + crow * p.N + col) = o;
    if (kEpi == kEpiGeluKeep) *reinterpret_cast<half4 *>(p.C2 + static_cast<size_t>(j) * p.N + col) = pre;
  }
}

template <class Cfg, int kEpi>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(GroupedArgs p) {
  const int tiles = p.tail[0], S = p.tail[1];
  for (int t = blockIdx.x; t < tiles; t += gridDim.x) reduce_split_tile<Cfg, kEpi>(p, t, S);
  if (!p.skinny || p.skinny[3] <= 0) return;
  const int pairs = p.skinny[0] * SkinnyCfg::TM;
  const int nblk = gridDim.x * gridDim.y;
  for (int i = blockIdx.x * gridDim.y + blockIdx.y; i < pairs; i += nblk)
    skinny_reduce_block<kEpi>(p, i / SkinnyCfg::TM, i % SkinnyCfg::TM);
}

// ---- kernel table -----------------------------------------------------------------
// 256x256x64 tiles (the most flop per byte pulled from L2 that the register file allows), four
// wavefronts of 128x128.  ccf_set_option("gemm_variant", n): 0 = persistent workgroups (default),
// 1 = one workgroup per tile for every K (otherwise only K below four K tiles runs that way).
using Cfg5 = GemmCfg<256, 256, 64, 2, 2, 8>;
// The same tile with eight wavefronts of 128x64, two per SIMD, half the registers each (gemm_variant 3; the
// forward epilogues only).  Built for GEMMs with few K steps in front of a GELU epilogue; measured, it gives
// the four-wavefront form's bits and is no faster: what two wavefronts per SIMD gain in the epilogue, the main
// loop loses, because a K step then reads 192 KB of fragments from LDS instead of 128 KB next to the 64 KB the
// tile loads write, and the LDS pipe is busy for as long as the MFMAs are.  It is not chosen by default.
using Cfg8 = GemmCfg<256, 256, 64, 2, 4, 8>;
constexpr int kWideMaxKT = 0;        // forward GEMMs with at most this many K tiles take the eight-wavefront form by default

constexpr int kDefaultVariant = 0;
int g_variant = kDefaultVariant;
int g_dgrad_transpose = 0;   // 1: input gradients always on a transposed copy of the weight
int g_wgrad_transpose = 0;   // 1: weight gradients always on transposed copies of the activations
int g_split_tail = 1;        // 0: the last round of tiles is not cut along K
constexpr int kSplitTailMinKT = 64;
int g_split_tail_min_kt = kSplitTailMinKT;
int g_split_max_parts = 8;
int g_fused_combine = 0;     // 1: top-2 layers add the gate-weighted expert outputs in the second GEMM's epilogue
int g_skinny_pct = 70;       // a K step of a skinny tile in percent of a 256-row tile's (plan model); 0: no skinny tiles
int g_skinny_positions = 0;  // skinny ranges inside the persistent launch: 0 = a point per round of tiles, 2 = in front of / behind all tiles
int g_split_inside = 1;      // 1: the parts of a split last round run inside the persistent launch, 0: as a launch of their own
int g_skinny_tail = 0;       // 0: skinny tiles never run as a launch of their own

// The tuning knobs a grouped GEMM's plan and launches depend on, read once per call: the plan
// and the kernels that consume it must agree even if another thread calls ccf_set_option
// between the routing stage (which builds the plans of the layer's forward call) and the GEMMs.
GemmOptions current_options() {
  return GemmOptions{g_variant, g_split_tail, g_split_tail_min_kt, g_split_max_parts, g_skinny_pct, g_fused_combine,
                     g_skinny_tail};
}

// The kernels of one family of epilogues: `first` and `second` are two epilogue forms, each as
// the one-workgroup-per-tile kernel and as the persistent kernel.
struct Launch {
  int bm, bn, threads;
  void (*plain)(GroupedArgs);
  void (*gelu)(GroupedArgs);
  // persistent form (one workgroup per CU), or null; used when K has at least kPersistentMinKT K tiles
  void (*persistent_plain)(GroupedArgs, int);
  void (*persistent_gelu)(GroupedArgs, int);
};
constexpr int kPersistentMinKT = 4;
constexpr int kReduceX = 32;         // x 16 blocks of the reduction launch

const Launch kVariants[] = {// forward: "plain" = bias and row scale, "gelu" = bias and GELU
                            {Cfg5::BM, Cfg5::BN, Cfg5::THREADS, grouped_gemm_kernel<Cfg5, kEpiPlain>,
                             grouped_gemm_kernel<Cfg5, kEpiGelu>, grouped_gemm_persistent_kernel<Cfg5, kEpiPlain>,
                             grouped_gemm_persistent_kernel<Cfg5, kEpiGelu>},
                            // B stored [E, K, N] (input gradients on the stored weight)
                            {Cfg5::BM, Cfg5::BN, Cfg5::THREADS, grouped_gemm_kernel<Cfg5, kEpiPlain, false, true>,
                             grouped_gemm_kernel<Cfg5, kEpiGeluGrad, false, true>,
                             grouped_gemm_persistent_kernel<Cfg5, kEpiPlain, false, true>,
                             grouped_gemm_persistent_kernel<Cfg5, kEpiGeluGrad, false, true>},
                            // training forms: "plain" = GELU that keeps the pre-activation,
                            // "gelu" slot = input gradient through the GELU
                            {Cfg5::BM, Cfg5::BN, Cfg5::THREADS, grouped_gemm_kernel<Cfg5, kEpiGeluKeep>,
                             grouped_gemm_kernel<Cfg5, kEpiGeluGrad>, grouped_gemm_persistent_kernel<Cfg5, kEpiGeluKeep>,
                             grouped_gemm_persistent_kernel<Cfg5, kEpiGeluGrad>},
                            // the combine epilogue ("plain" slot)
                            {Cfg5::BM, Cfg5::BN, Cfg5::THREADS, grouped_gemm_kernel<Cfg5, kEpiCombine>, nullptr,
                             grouped_gemm_persistent_kernel<Cfg5, kEpiCombine>, nullptr},
                            // forward, eight wavefronts (persistent only)
                            {Cfg8::BM, Cfg8::BN, Cfg8::THREADS, nullptr, nullptr, grouped_gemm_persistent_kernel<Cfg8, kEpiPlain>,
                             grouped_gemm_persistent_kernel<Cfg8, kEpiGelu>}};
constexpr int kFwdVariant = 0, kKnVariant = 1, kTrainVariant = 2, kCombineVariant = 3, kFwd8Variant = 4;

// Compute units of the current device, rounded down to whole XCD rounds of 8.
int persistent_grid() {
  static thread_local int cached_dev = -1, cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_dev) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached = cus / 8 * 8;
    cached_dev = dev;
  }
  return cached;
}
constexpr int kNumVariants = 4;                      // what ccf_set_option accepts
constexpr int kMinBM = 256;

int max_tiles_for(int max_rows, int E, int bm) { return (max_rows + bm - 1) / bm + E; }

constexpr int kMinBN = 256;

// Workspace of one grouped GEMM: the split-K tail area, then the tile plan.  A second plan
// (region 1: header and entries of its own, then the plan; the partial tiles are shared) follows
// in the forward workspace, so that the plans of both GEMMs of a layer can exist at once.
size_t plan_core_bytes(int max_rows, int E, int n_max) {
  return round_up(sizeof(int32_t) * plan_ints(launched_wgs(max_tiles_for(max_rows, E, kMinBM),
                                                           (n_max + kMinBN - 1) / kMinBN)), 256);
}
// the tile plan, then the skinny list
size_t plan_only_bytes(int max_rows, int E, int n_max) {
  return plan_core_bytes(max_rows, E, n_max) +
         round_up(sizeof(int32_t) * skinny_ints(max_rows, E, (n_max + kMinBN - 1) / kMinBN), 256);
}
size_t plan_bytes(int max_rows, int E, int n_max) { return kTailBytes + plan_only_bytes(max_rows, E, n_max); }
size_t forward_ws_bytes(int max_rows, int E, int n_max) {
  return plan_bytes(max_rows, E, n_max) + kTailHead + plan_only_bytes(max_rows, E, n_max);
}

// Everything the launches of one grouped GEMM derive from its sizes, and the request that
// builds its plan.
// Epilogue of a 256-row tile in K steps of the main loop (for the plan's cost model): the GELU
// epilogue is ~13 us, the plain one ~7 us, a K step ~1.45 us.
constexpr int kEpiCostGelu = 9, kEpiCostPlain = 5;

struct GemmSetup {
  const Launch *v;
  bool second, split, skinny, cut;
  int32_t *skinny_list;
  int grid;
  long long wgs;
  int32_t *tail, *plan;
  float *partial, *sk_partial;
  PlanReq req;
};

GemmSetup setup_gemm(int max_rows, int E, int N, int K, int epi, bool b_kn, void *workspace, int region,
                     const GemmOptions &opt) {
  GemmSetup g;
  char *ws = static_cast<char *>(workspace);
  g.partial = reinterpret_cast<float *>(ws + kTailHead);
  g.sk_partial = reinterpret_cast<float *>(ws + kTailHead + kSplitPartialBytes);
  if (region == 0) {
    g.tail = reinterpret_cast<int32_t *>(ws);                                       // header and entries
    g.plan = reinterpret_cast<int32_t *>(ws + kTailBytes);
  } else {
    g.tail = reinterpret_cast<int32_t *>(ws + plan_bytes(max_rows, E, N > K ? N : K));
    g.plan = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(g.tail) + kTailHead);
  }
  const bool gelu = epi != kEpiPlain && epi != kEpiCombine;
  const int kt_all = K / 64;
  const int cus = persistent_grid();
  const bool persistent = opt.variant != 1 && kt_all >= kPersistentMinKT && cus >= 8;
  // eight wavefronts: the two plain forward epilogues, short K (or forced)
  const bool wide = persistent && !b_kn && epi <= kEpiGelu && (opt.variant == 3 || (opt.variant == 0 && kt_all <= kWideMaxKT));
  g.v = &kVariants[b_kn ? kKnVariant : (epi == kEpiCombine ? kCombineVariant : (epi >= kEpiGeluKeep ? kTrainVariant :
                                                                                   (wide ? kFwd8Variant : kFwdVariant)))];
  const Launch &v = *g.v;
  // which of the entry's two kernels: the K-N and training entries hold the GELU-gradient form in the second slot
  g.second = b_kn ? epi == kEpiGeluGrad : (epi == kEpiCombine ? false : (epi >= kEpiGeluKeep ? epi == kEpiGeluGrad : gelu));
  const int max_tiles = max_tiles_for(max_rows, E, v.bm);
  const int n_tiles_n = (N + v.bn - 1) / v.bn;
  g.wgs = launched_wgs(max_tiles, n_tiles_n);                   // worst-case tile count
  g.grid = persistent ? cus : 0;
  // the last, partly filled round is cut along K and spread over all workgroups (forward forms;
  // worth its two small launches only where a tile is long: K of 4096 and more)
  g.split = opt.split_tail && (b_kn ? epi == kEpiPlain : epi <= kEpiGeluKeep) && g.grid >= 8 && g.grid <= g.wgs &&
            g.grid <= kTailMaxParts && v.bm == Cfg5::BM && v.bn == Cfg5::BN && K / 64 >= opt.split_tail_min_kt;
  // remainder rows as skinny tiles: forward epilogues of the persistent 256 x 256 kernel (either weight layout)
  g.skinny = opt.skinny_pct != 0 && (b_kn ? epi == kEpiPlain && N % 256 == 0 : epi <= kEpiGeluKeep) && g.grid >= 64 && g.grid <= g.wgs &&
             v.bm == Cfg5::BM && v.bn == Cfg5::BN && v.persistent_plain && (!wide || g.split);
  // skinny tiles may be cut along K (partial tiles in the split scratch, summed by the reduction launch) at any K,
  // also where the last round of 256-row tiles is not split
  g.cut = g.skinny && !wide && g.grid <= kTailMaxParts;
  g.skinny_list = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(g.plan) + plan_core_bytes(max_rows, E, N > K ? N : K));
  static_assert(plan_bm_ok(Cfg5::BM) && plan_bm_ok(Cfg8::BM), "build_plan shifts by the tile height");
  g.req = PlanReq{v.bm, max_tiles, max_rows, n_tiles_n, g.split ? g.grid / 8 : 0, K / 64, opt.split_max_parts, g.plan,
                  (g.split || g.cut) ? g.tail : nullptr, g.skinny ? g.skinny_list : nullptr, g.grid,
                  gelu ? kEpiCostGelu : kEpiCostPlain, opt.skinny_pct, g.cut && opt.skinny_tail, !wide};
  return g;
}

// plan_ready: the plan (and the split list) of this very call was already built in `region`
// by forward_plan_request()'s request.
int grouped_gemm(const half_t *A, const int32_t *a_rows, const int32_t *offsets, int max_rows, int E,
                 int N, int K, const half_t *B, const half_t *bias, int epi, half_t *C,
                 const int32_t *c_rows, const half_t *row_scale, void *workspace, hipStream_t stream,
                 const char *what, bool b_kn = false, half_t *C2 = nullptr, int region = 0,
                 bool plan_ready = false, const GemmOptions *opt = nullptr, const int32_t *scale_rows = nullptr) {
  CCF_REQUIRE(A && offsets && B && C && workspace, CCF_ERR_ARG, "%s: null pointer", what);
  const bool gelu = epi != kEpiPlain && epi != kEpiCombine;
  CCF_REQUIRE(epi >= kEpiPlain && epi <= kEpiCombine &&
                  (epi < kEpiGeluKeep || epi == kEpiCombine || (C2 && aligned16(C2))), CCF_ERR_ARG,
              "%s: epilogue %d needs the pre-activation buffer", what, epi);
  CCF_REQUIRE(epi != kEpiCombine || (c_rows && row_scale && scale_rows && !b_kn && N % 8 == 0), CCF_ERR_ARG,
              "%s: the combine epilogue needs token rows, scores and their index", what);
  // b_kn: B is [E, K, N] (the stored weight of the layer whose input gradient this is); Cfg5 kernels only
  CCF_REQUIRE(!b_kn || (N % Cfg5::BN == 0 && (epi == kEpiPlain || epi == kEpiGeluGrad) &&
                        static_cast<long long>(K) * N < (1ll << 31)), CCF_ERR_SHAPE,
              "%s: the [K][N] weight form needs N=%d to be a multiple of %d", what, N, Cfg5::BN);
  CCF_REQUIRE(max_rows >= 0 && E > 0 && N > 0 && K > 0, CCF_ERR_ARG, "%s: bad size", what);
  CCF_REQUIRE(E <= 1024, CCF_ERR_SHAPE, "%s: num_expert=%d exceeds 1024", what, E);
  CCF_REQUIRE(K % 64 == 0, CCF_ERR_SHAPE, "%s: K=%d is not a multiple of 64", what, K);
  CCF_REQUIRE(N % 8 == 0, CCF_ERR_SHAPE, "%s: N=%d is not a multiple of 8", what, N);
  CCF_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C) && (!bias || aligned16(bias)), CCF_ERR_ARG,
              "%s: operands must be 16-byte aligned", what);
  CCF_REQUIRE(!(gelu && row_scale), CCF_ERR_ARG, "%s: the GELU epilogue takes no row scale", what);
  if (max_rows == 0) return CCF_OK;
  const GemmSetup gs = setup_gemm(max_rows, E, N, K, epi, b_kn, workspace, region, opt ? *opt : current_options());
  const Launch &v = *gs.v;
  const bool second = gs.second, split = gs.split;
  const int grid = gs.grid;
  const long long wgs = gs.wgs;
  CCF_REQUIRE(wgs < (1ll << 24), CCF_ERR_SHAPE, "%s: grid too large", what);
  if (!plan_ready) {
    hipLaunchKernelGGL(plan_kernel, dim3(plan_workgroups(E)), dim3(kPlanThreads), 0, stream, gs.req, offsets, E);
    if (int rc = check_launch("plan_kernel")) return rc;
  }
  int32_t *plan = gs.plan, *tail = gs.tail;
  float *partial = gs.partial;
  GroupedArgs p;
  p.sk_positions = g_skinny_positions;
  p.tail_inside = 0;
  p.A = A;
  p.a_rows = a_rows;
  p.B = B;
  p.bias = bias;
  p.C = C;
  p.C2 = C2;
  p.c_rows = c_rows;
  p.row_scale = row_scale;
  p.scale_rows = scale_rows;
  p.plan = plan;
  p.N = N;
  p.K = K;
  p.k_seg = nullptr;
  p.lda = p.ldb = K;
  p.seg_rows = 0;
  p.tail = tail;
  p.partial = partial;
  p.sk_partial = gs.sk_partial;
  p.zero_row = nullptr;
  p.skinny = gs.skinny ? gs.skinny_list : nullptr;
  if (grid >= 8) {
    const long long g = grid < wgs ? grid : wgs;                // wgs is a multiple of 8
    // the parts of a split last round: run by the persistent workgroups themselves behind their tiles (the
    // four-wavefront kernels; part i is workgroup i's), else by a launch of their own
    const bool parts_inside = split && g_split_inside && gs.v != &kVariants[kFwd8Variant];
    p.tail_inside = parts_inside ? 1 : 0;
    hipLaunchKernelGGL(second ? v.persistent_gelu : v.persistent_plain, dim3(static_cast<unsigned>(g)),
                       dim3(v.threads), 0, stream, p, static_cast<int>(wgs / 8));
    if (split || gs.cut) {
      if (int rc = check_launch(what)) return rc;
      // the skinny list may run as a launch of its own: `grid` more workgroups for it
      const bool sk = gs.req.sk_tail_ok;
      if ((split && !parts_inside) || sk) {
        const int split_wgs = (split && !parts_inside) ? grid : 0;  // workgroups in front of the skinny list's
        const int tail_grid = split_wgs + (sk ? grid : 0);
        if (b_kn) hipLaunchKernelGGL((grouped_gemm_tail_kernel<Cfg5, true>), dim3(tail_grid), dim3(Cfg5::THREADS), 0,
                                     stream, p, split_wgs);
        else hipLaunchKernelGGL((grouped_gemm_tail_kernel<Cfg5, false>), dim3(tail_grid), dim3(Cfg5::THREADS), 0,
                                stream, p, split_wgs);
        if (int rc = check_launch("grouped_gemm_tail_kernel")) return rc;
      }
      const dim3 rgrid(kReduceX, Cfg5::BM / 16);
      if (epi == kEpiPlain) hipLaunchKernelGGL((splitk_reduce_kernel<Cfg5, kEpiPlain>), rgrid, dim3(256), 0, stream, p);
      else if (epi == kEpiGelu) hipLaunchKernelGGL((splitk_reduce_kernel<Cfg5, kEpiGelu>), rgrid, dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((splitk_reduce_kernel<Cfg5, kEpiGeluKeep>), rgrid, dim3(256), 0, stream, p);
      return check_launch("splitk_reduce_kernel");
    }
  } else {
    hipLaunchKernelGGL(second ? v.gelu : v.plain, dim3(static_cast<unsigned>(wgs)), dim3(v.threads), 0,
                       stream, p);
  }
  return check_launch(what);
}

// Plan request of a weight-gradient GEMM: E experts of M output rows each, N columns; the plan sits behind the
// (unused) split scratch in `workspace`.
PlanReq wgrad_plan_request(int E, int M, int N, int32_t *workspace) {
  int32_t *plan = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(workspace) + kTailBytes);
  const int max_rows = E * M;
  return PlanReq{Cfg5::BM, max_tiles_for(max_rows, E, Cfg5::BM), max_rows, (N + Cfg5::BN - 1) / Cfg5::BN, 0, 0, 0, plan,
                 nullptr, nullptr, 0, 0, 0, 0, 0};
}

// C[e*M + m, n] = sum over k in [k_seg[e], k_seg[e+1]) of A[m, k] * B[n, k]: the weight
// gradient of expert e from the two transposed activation matrices.  row_off[e] = e*M.
// plan_ready: wgrad_plan_request()'s plan was already built in `workspace`.
int grouped_gemm_kseg(const half_t *A, int lda, const half_t *B, int ldb, const int32_t *k_seg,
                      const int32_t *row_off, int E, int M, int N, half_t *C, int32_t *workspace,
                      hipStream_t stream, const char *what, bool plan_ready = false) {
  CCF_REQUIRE(A && B && k_seg && row_off && C && workspace, CCF_ERR_ARG, "%s: null pointer", what);
  int32_t *plan = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(workspace) + kTailBytes);
  CCF_REQUIRE(lda % 8 == 0 && ldb % 8 == 0 && N % 8 == 0, CCF_ERR_SHAPE, "%s: strides and N must be multiples of 8", what);
  CCF_REQUIRE(static_cast<long long>(E) * M < (1ll << 31), CCF_ERR_SHAPE, "%s: output too tall", what);
  const int max_rows = E * M;
  const int max_tiles = max_tiles_for(max_rows, E, Cfg5::BM);
  const int n_tiles_n = (N + Cfg5::BN - 1) / Cfg5::BN;
  const long long wgs = launched_wgs(max_tiles, n_tiles_n);
  CCF_REQUIRE(wgs < (1ll << 24), CCF_ERR_SHAPE, "%s: grid too large", what);
  if (!plan_ready) {
    hipLaunchKernelGGL(plan_kernel, dim3(plan_workgroups(E)), dim3(kPlanThreads), 0, stream,
                       wgrad_plan_request(E, M, N, workspace), row_off, E);
    if (int rc = check_launch("plan_kernel")) return rc;
  }
  GroupedArgs p;
  p.sk_positions = g_skinny_positions;
  p.tail_inside = 0;
  p.A = A;
  p.a_rows = nullptr;
  p.B = B;
  p.bias = nullptr;
  p.C = C;
  p.C2 = nullptr;
  p.c_rows = nullptr;
  p.row_scale = nullptr;
  p.scale_rows = nullptr;
  p.plan = plan;
  p.N = N;
  p.K = 0;
  p.k_seg = k_seg;
  p.lda = lda;
  p.ldb = ldb;
  p.seg_rows = M;
  p.tail = nullptr;
  p.partial = nullptr;
  p.sk_partial = nullptr;
  p.zero_row = nullptr;
  p.skinny = nullptr;
  const int grid = persistent_grid();
  if (grid >= 8) {
    const long long g = grid < wgs ? grid : wgs;
    hipLaunchKernelGGL((grouped_gemm_persistent_kernel<Cfg5, kEpiPlain, true>), dim3(static_cast<unsigned>(g)),
                       dim3(Cfg5::THREADS), 0, stream, p, static_cast<int>(wgs / 8));
  } else {
    hipLaunchKernelGGL((grouped_gemm_kernel<Cfg5, kEpiPlain, true>), dim3(static_cast<unsigned>(wgs)),
                       dim3(Cfg5::THREADS), 0, stream, p);
  }
  return check_launch(what);
}

// C[e*M + m, n] = sum over the rows j of expert e (row_lo[e] <= j < row_lo[e+1]) of A[j, m] * B[j, n]: the weight
// gradient of expert e straight from the two row-major activation matrices (no transposed copies): both
// operands go through LDS as [K][*] tiles and transposing reads, rows past an expert's end read as zero.
// M and N multiples of 256; row_off[e] = e*M.
int grouped_gemm_krows(const half_t *A, int lda, const half_t *B, int ldb, const int32_t *row_lo,
                       const int32_t *row_off, int E, int M, int N, half_t *C, int32_t *workspace,
                       const half_t *zero_row, int grid, hipStream_t stream, const char *what, bool plan_ready = false) {
  CCF_REQUIRE(A && B && row_lo && row_off && C && workspace && zero_row, CCF_ERR_ARG, "%s: null pointer", what);
  int32_t *plan = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(workspace) + kTailBytes);
  CCF_REQUIRE(lda % 8 == 0 && ldb % 8 == 0 && M % Cfg5::BM == 0 && N % Cfg5::BN == 0 && grid >= 8, CCF_ERR_SHAPE,
              "%s: the row-major weight-gradient form needs widths that are multiples of 256", what);
  CCF_REQUIRE(static_cast<long long>(E) * M < (1ll << 31), CCF_ERR_SHAPE, "%s: output too tall", what);
  const int max_rows = E * M;
  const int max_tiles = max_tiles_for(max_rows, E, Cfg5::BM);
  const int n_tiles_n = N / Cfg5::BN;
  const long long wgs = launched_wgs(max_tiles, n_tiles_n);
  CCF_REQUIRE(wgs < (1ll << 24), CCF_ERR_SHAPE, "%s: grid too large", what);
  if (!plan_ready) {
    hipLaunchKernelGGL(plan_kernel, dim3(plan_workgroups(E)), dim3(kPlanThreads), 0, stream,
                       wgrad_plan_request(E, M, N, workspace), row_off, E);
    if (int rc = check_launch("plan_kernel")) return rc;
  }
  GroupedArgs p;
  p.sk_positions = g_skinny_positions;
  p.tail_inside = 0;
  p.A = A;
  p.a_rows = nullptr;
  p.B = B;
  p.bias = nullptr;
  p.C = C;
  p.C2 = nullptr;
  p.c_rows = nullptr;
  p.row_scale = nullptr;
  p.scale_rows = nullptr;
  p.plan = plan;
  p.N = N;
  p.K = 0;
  p.k_seg = row_lo;
  p.lda = lda;
  p.ldb = ldb;
  p.seg_rows = M;
  p.tail = nullptr;
  p.partial = nullptr;
  p.sk_partial = nullptr;
  p.zero_row = zero_row;
  p.skinny = nullptr;
  const long long g = grid < wgs ? grid : wgs;
  hipLaunchKernelGGL((grouped_gemm_persistent_kernel<Cfg5, kEpiPlain, true, true>), dim3(static_cast<unsigned>(g)),
                     dim3(Cfg5::THREADS), 0, stream, p, static_cast<int>(wgs / 8));
  return check_launch(what);
}

// Workspace of the backward entry points, carved in this order.
struct BackwardWs {
  int32_t *plan_rows;      // tile plan of the input-gradient GEMM
  int32_t *plan_w;         // tile plan of the weight-gradient GEMM
  int32_t *k_seg, *row_off, *blk_row0, *blk_cnt, *row_lo;
  half_t *zero_row;        // 256 zeros
  half_t *w_t;             // [E, in, out] transposed weight
  half_t *a_t, *b_t;       // [out, ld_t], [in, ld_t] transposed activations
  float *partial;          // [ld_t / 64, out] bias partial sums
  int ld_t, n_blk;
  size_t bytes;
};

BackwardWs carve_backward(void *base, int max_rows, int E, int d, int f) {
  BackwardWs w;
  const int big = d > f ? d : f;
  w.ld_t = padded_rows(max_rows, E);
  w.n_blk = w.ld_t / 64;
  // offsets are added to the base as integers: the size query passes a null base
  uintptr_t p = reinterpret_cast<uintptr_t>(base);
  auto take = [&](size_t bytes) {
    void *r = reinterpret_cast<void *>(p);
    p += round_up(bytes, 256);
    return r;
  };
  w.plan_rows = static_cast<int32_t *>(take(plan_bytes(max_rows, E, big)));
  w.plan_w = static_cast<int32_t *>(take(plan_bytes(E * big, E, big)));
  w.k_seg = static_cast<int32_t *>(take(sizeof(int32_t) * (E + 1)));
  w.row_off = static_cast<int32_t *>(take(sizeof(int32_t) * (E + 1)));
  w.blk_row0 = static_cast<int32_t *>(take(sizeof(int32_t) * w.n_blk));
  w.blk_cnt = static_cast<int32_t *>(take(sizeof(int32_t) * w.n_blk));
  w.row_lo = static_cast<int32_t *>(take(sizeof(int32_t) * (E + 1)));
  w.zero_row = static_cast<half_t *>(take(sizeof(half_t) * 256));
  w.w_t = static_cast<half_t *>(take(sizeof(half_t) * static_cast<size_t>(E) * d * f));
  w.a_t = static_cast<half_t *>(take(sizeof(half_t) * static_cast<size_t>(big) * w.ld_t));
  w.b_t = static_cast<half_t *>(take(sizeof(half_t) * static_cast<size_t>(big) * w.ld_t));
  w.partial = static_cast<float *>(take(sizeof(float) * static_cast<size_t>(w.n_blk) * big));
  w.bytes = static_cast<size_t>(p - reinterpret_cast<uintptr_t>(base));
  return w;
}

// No rows at all: the parameter gradients are zero and there is no input gradient.
int zero_param_grads(void *grad_w, void *grad_b, int E, int n_out, int n_in, hipStream_t stream) {
  CCF_REQUIRE(grad_w && grad_b && E > 0 && n_out > 0 && n_in > 0, CCF_ERR_ARG, "backward: null pointer or bad size");
  CCF_REQUIRE(n_out % 8 == 0 && n_in % 8 == 0 && aligned16(grad_w) && aligned16(grad_b), CCF_ERR_SHAPE,
              "backward: widths must be multiples of 8 and buffers 16-byte aligned");
  if (int rc = launch_zero(static_cast<half_t *>(grad_w), static_cast<size_t>(E) * n_out * n_in, stream)) return rc;
  return launch_zero(static_cast<half_t *>(grad_b), static_cast<size_t>(E) * n_out, stream);
}

// One expert linear layer's backward.  Forward was out[c_row(j)] = in[a_row(j)] * w[e]^T + b[e]
// with w [E, n_out, n_in].  Given grad_out rows (through g_rows) and the forward's input rows
// (through in_rows):
//   grad_in[gi_rows(j)] = grad_out[g_rows(j)] * w[e]            (grouped GEMM on w^T)
//   grad_w[e] = grad_out_e^T * in_e,  grad_b[e] = column sums of grad_out_e
int linear_backward(half_t *grad_out, const int32_t *g_rows, const half_t *in,
                    const int32_t *in_rows, const int32_t *offsets, int max_rows, int E, int n_in,
                    int n_out, const half_t *w, half_t *grad_in, const int32_t *gi_rows,
                    half_t *grad_w, half_t *grad_b, void *workspace, size_t workspace_bytes,
                    int d, int f, hipStream_t stream, const char *what, const half_t *gelu_pre = nullptr,
                    const half_t *pre_inplace = nullptr) {
  CCF_REQUIRE(grad_out && in && offsets && w && grad_in && grad_w && grad_b, CCF_ERR_ARG,
              "%s: null pointer", what);
  CCF_REQUIRE(max_rows >= 0 && E > 0 && E <= 1024 && d > 0 && f > 0, CCF_ERR_ARG, "%s: bad size", what);
  CCF_REQUIRE(d % 64 == 0 && f % 64 == 0, CCF_ERR_SHAPE,
              "%s: d_model=%d and d_ffn=%d must be multiples of 64", what, d, f);
  CCF_REQUIRE(aligned16(grad_out) && aligned16(in) && aligned16(w) && aligned16(grad_in) &&
                  aligned16(grad_w) && aligned16(grad_b) && aligned16(workspace),
              CCF_ERR_ARG, "%s: operands must be 16-byte aligned", what);
  const size_t need = ccf_ffn_backward_workspace_bytes(max_rows, E, d, f);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "%s: workspace of %zu bytes needed, %zu given", what, need, workspace_bytes);
  const BackwardWs ws = carve_backward(workspace, max_rows, E, d, f);
  // The weight gradient contracts over an expert's rows.  Where the widths allow, its GEMM reads the two
  // row-major activation matrices as they are (rows form: transposing LDS reads of both operands); what
  // remains of the data movement is a gather of the operand that arrives through a row index, and one pass
  // over the gradient rows for the bias gradient's partial sums.  Otherwise both matrices are transposed
  // into [columns, padded rows] first.
  const int grid = persistent_grid();
  const int wide = n_out > n_in ? n_out : n_in;
  const bool rows_form = !g_wgrad_transpose && n_out % Cfg5::BM == 0 && n_in % Cfg5::BN == 0 && grid >= 8 &&
                         static_cast<long long>(max_rows + 256) * wide < (1ll << 31);
  // With pre_inplace the incoming rows are gradients of gelu(pre): the pass over them multiplies them by
  // gelu'(pre) and writes them back, so that everything below sees the gradient of the pre-activation.
  CCF_REQUIRE(!pre_inplace || !g_rows, CCF_ERR_ARG, "%s: the in-place GELU gradient needs rows in expert order", what);
  // input gradient: on the stored weight read as [K][N] where the shape allows, else on a transposed copy
  const bool kn = !g_dgrad_transpose && n_in % Cfg5::BN == 0 && static_cast<long long>(n_out) * n_in < (1ll << 31);
  const int dgrad_epi = gelu_pre ? kEpiGeluGrad : kEpiPlain;
  // the launch that lays out the K ranges also builds the tile plans of both GEMMs
  const PlanReq rows_plan = setup_gemm(max_rows, E, n_in, n_out, dgrad_epi, kn, ws.plan_rows, 0, current_options()).req;
  const PlanReq w_plan = wgrad_plan_request(E, n_out, n_in, ws.plan_w);
  const bool plans = max_rows > 0 && static_cast<long long>(E) * n_out < (1ll << 31);
  if (int rc = launch_kseg(offsets, E, max_rows, n_out, ws.n_blk, ws.k_seg, ws.row_off, ws.blk_row0,
                           ws.blk_cnt, ws.row_lo, ws.zero_row, plans ? &rows_plan : nullptr, plans ? &w_plan : nullptr,
                           stream))
    return rc;
  // rows form: gathered gradient rows go to a_t as a plain [rows, n_out] matrix; rows already in expert order stay
  const half_t *g_mat = (rows_form && !g_rows) ? grad_out : ws.a_t;
  if (int rc = launch_transpose_rows(grad_out, g_rows, ws.blk_row0, ws.blk_cnt, ws.n_blk, n_out, ws.ld_t,
                                     (rows_form && !g_rows) ? nullptr : ws.a_t, ws.partial, stream, pre_inplace, !rows_form))
    return rc;
  if (!kn) {
    if (int rc = launch_transpose_weights(w, ws.w_t, E, n_out, n_in, stream)) return rc;
  }
  // gelu_pre: the input was gelu(gelu_pre); the gradient is then taken through the GELU in the epilogue
  CCF_REQUIRE(!gelu_pre || !gi_rows, CCF_ERR_ARG, "%s: the GELU gradient needs rows in expert order", what);
  if (int rc = grouped_gemm(grad_out, g_rows, offsets, max_rows, E, n_in, n_out, kn ? w : ws.w_t, nullptr,
                            dgrad_epi, grad_in, gi_rows, nullptr, ws.plan_rows, stream,
                            what, kn, const_cast<half_t *>(gelu_pre), 0, plans))
    return rc;
  // weight and bias gradients
  const half_t *in_mat = (rows_form && !in_rows) ? in : ws.b_t;
  if (!rows_form || in_rows) {
    if (int rc = launch_transpose_rows(in, in_rows, ws.blk_row0, ws.blk_cnt, ws.n_blk, n_in, ws.ld_t,
                                       ws.b_t, nullptr, stream, nullptr, !rows_form))
      return rc;
  }
  if (int rc = launch_bias_reduce(ws.partial, ws.k_seg, E, n_out, grad_b, stream)) return rc;
  if (rows_form)
    return grouped_gemm_krows(g_mat, n_out, in_mat, n_in, ws.row_lo, ws.row_off, E, n_out, n_in, grad_w, ws.plan_w,
                              ws.zero_row, grid, stream, what, plans);
  return grouped_gemm_kseg(ws.a_t, ws.ld_t, ws.b_t, ws.ld_t, ws.k_seg, ws.row_off, E, n_out, n_in,
                           grad_w, ws.plan_w, stream, what, plans);
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_set_option(const char *name, int value) {
  using namespace ccf;
  CCF_REQUIRE(name, CCF_ERR_ARG, "set_option: null name");
  if (!strcmp(name, "gemm_variant")) {
    CCF_REQUIRE(value >= -1 && value < kNumVariants, CCF_ERR_ARG, "set_option: gemm_variant %d outside -1..%d",
                value, kNumVariants - 1);
    g_variant = value < 0 ? kDefaultVariant : value;     // -1: back to the default (0: the library chooses by K)
    return CCF_OK;
  }
  if (!strcmp(name, "split_tail")) {         // 0 = off, 1 = default, n > 1: for K of n K tiles and more
    g_split_tail = value != 0;
    g_split_tail_min_kt = value > 1 ? value : kSplitTailMinKT;
    return CCF_OK;
  }
  if (!strcmp(name, "split_parts")) {        // most parts a tile of the split last round is cut into
    CCF_REQUIRE(value >= 2 && value <= 8, CCF_ERR_ARG, "set_option: split_parts %d outside 2..8", value);
    g_split_max_parts = value;
    return CCF_OK;
  }
  if (!strcmp(name, "skinny")) {             // 0: off; 1: default; n > 1: cost of a skinny K step in percent (plan model);
                                             // -n: always, with n workgroups per XCD; -(kSkinnyMaxWgs + 1): always, as a
                                             // launch of their own
    CCF_REQUIRE(value >= -kSkinnyMaxWgs - 2 && value <= 400, CCF_ERR_ARG, "set_option: skinny %d outside %d..400", value,
                -kSkinnyMaxWgs - 2);
    g_skinny_pct = value == 1 ? 70 : value;
    return CCF_OK;
  }
  if (!strcmp(name, "skinny_tail")) {
    g_skinny_tail = value != 0;
    return CCF_OK;
  }
  if (!strcmp(name, "dgrad_transpose")) {
    g_dgrad_transpose = value != 0;
    return CCF_OK;
  }
  if (!strcmp(name, "split_inside")) {
    g_split_inside = value != 0;
    return CCF_OK;
  }
  if (!strcmp(name, "skinny_positions")) {
    g_skinny_positions = value < 0 ? 0 : value;
    return CCF_OK;
  }
  if (!strcmp(name, "wgrad_transpose")) {
    g_wgrad_transpose = value != 0;
    return CCF_OK;
  }
  if (!strcmp(name, "gate_waves")) {
    CCF_REQUIRE(value >= 1 && value <= 8, CCF_ERR_ARG, "set_option: gate_waves %d outside 1..8", value);
    g_gate_waves = value;
    return CCF_OK;
  }
  if (!strcmp(name, "gate_stream")) {
    CCF_REQUIRE(value >= -1 && value <= 1, CCF_ERR_ARG, "set_option: gate_stream %d outside -1..1", value);
    g_gate_stream = value;
    return CCF_OK;
  }
  if (!strcmp(name, "fused_combine")) {
    g_fused_combine = value != 0;
    return CCF_OK;
  }
  if (!strcmp(name, "route_rows_max")) {
    CCF_REQUIRE(value >= 0 && value <= 32768, CCF_ERR_ARG, "set_option: route_rows_max %d outside 0..32768", value);
    g_route_rows_max = value;
    return CCF_OK;
  }
  if (!strcmp(name, "gate_slots")) {
    CCF_REQUIRE(value == 0 || value == 1 || value == 2 || value == 4, CCF_ERR_ARG,
                "set_option: gate_slots %d is none of 0, 1, 2, 4", value);
    g_gate_slots = value;
    return CCF_OK;
  }
  return fail(CCF_ERR_ARG, "set_option: unknown option %s", name);
}

extern "C" size_t ccf_ffn_workspace_bytes(int max_rows, int num_expert, int d_model, int d_ffn) {
  if (max_rows < 0 || num_expert <= 0 || d_model <= 0 || d_ffn <= 0) return 0;
  return ccf::forward_ws_bytes(max_rows, num_expert, d_model > d_ffn ? d_model : d_ffn);
}

namespace ccf {

// Plan requests of the layer's two forward GEMMs (which = 1: FFN1 with GELU, 2: FFN2, 3: FFN2 with the
// combine epilogue), for a
// caller that builds the plans itself (the routing stage does) and then passes plan_ready.
// False when the sizes are not ones the GEMM accepts: the caller then leaves the plan to it.
GemmOptions forward_options() { return current_options(); }

bool forward_plan_request(int which, int max_rows, int E, int d, int f, void *workspace, const GemmOptions &opt,
                          PlanReq *out) {
  if (!workspace || max_rows <= 0 || E <= 0 || E > 1024 || d <= 0 || f <= 0 || d % 64 || f % 64) return false;
  const int N = which == 1 ? f : d, K = which == 1 ? d : f;
  const GemmSetup gs = setup_gemm(max_rows, E, N, K, which == 1 ? kEpiGelu : (which == 3 ? kEpiCombine : kEpiPlain),
                                  false, workspace, which == 1 ? 0 : 1, opt);
  if (gs.wgs >= (1ll << 24)) return false;
  *out = gs.req;
  return true;
}

int ffn1_forward(const void *x, const int32_t *src_row, const int32_t *dst_row, const int32_t *offsets,
                 int max_rows, int num_expert, int d_model, int d_ffn, const void *w1, const void *b1,
                 int apply_gelu, void *h, void *workspace, size_t workspace_bytes, hipStream_t stream,
                 const GemmOptions *planned) {
  const bool plan_ready = planned != nullptr;
  const size_t need = ccf_ffn_workspace_bytes(max_rows, num_expert, d_model, d_ffn);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "ffn1: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  return grouped_gemm(static_cast<const half_t *>(x), src_row, offsets, max_rows, num_expert, d_ffn,
                      d_model, static_cast<const half_t *>(w1), static_cast<const half_t *>(b1),
                      apply_gelu != 0 ? kEpiGelu : kEpiPlain, static_cast<half_t *>(h), dst_row, nullptr,
                      workspace, stream, "ffn1", false, nullptr, 0, plan_ready && apply_gelu != 0, planned);
}

int ffn2_forward(const void *h, const int32_t *src_row, const int32_t *dst_row, const int32_t *offsets,
                 int max_rows, int num_expert, int d_model, int d_ffn, const void *w2, const void *b2,
                 const void *row_scale, void *y, void *workspace, size_t workspace_bytes,
                 hipStream_t stream, const GemmOptions *planned) {
  const bool plan_ready = planned != nullptr;
  const size_t need = ccf_ffn_workspace_bytes(max_rows, num_expert, d_model, d_ffn);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "ffn2: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  return grouped_gemm(static_cast<const half_t *>(h), src_row, offsets, max_rows, num_expert, d_model,
                      d_ffn, static_cast<const half_t *>(w2), static_cast<const half_t *>(b2), kEpiPlain,
                      static_cast<half_t *>(y), dst_row, static_cast<const half_t *>(row_scale),
                      workspace, stream, "ffn2", false, nullptr, 1, plan_ready, planned);
}

// FFN2 with the combine in its epilogue: out[token_row[j]] += (h[j] * w2[e]^T + b2[e]) * score[flat_row[j]].
// `out` must be zero; two addends per token make the result independent of their order.
int ffn2_forward_combine(const void *h, const int32_t *token_row, const int32_t *flat_row, const int32_t *offsets,
                         int max_rows, int num_expert, int d_model, int d_ffn, const void *w2, const void *b2,
                         const void *score, void *out, void *workspace, size_t workspace_bytes, hipStream_t stream,
                         const GemmOptions *planned) {
  const size_t need = ccf_ffn_workspace_bytes(max_rows, num_expert, d_model, d_ffn);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "ffn2: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  return grouped_gemm(static_cast<const half_t *>(h), nullptr, offsets, max_rows, num_expert, d_model, d_ffn,
                      static_cast<const half_t *>(w2), static_cast<const half_t *>(b2), kEpiCombine,
                      static_cast<half_t *>(out), token_row, static_cast<const half_t *>(score), workspace, stream,
                      "ffn2 with combine", false, nullptr, 1, planned != nullptr, planned, flat_row);
}

}  // namespace ccf

extern "C" int ccf_ffn1_forward(const void *x, const int32_t *src_row, const int32_t *dst_row,
                                const int32_t *offsets, int max_rows, int num_expert, int d_model,
                                int d_ffn, const void *w1, const void *b1, int apply_gelu, void *h,
                                void *workspace, size_t workspace_bytes, ccf_stream_t stream) {
  return ccf::ffn1_forward(x, src_row, dst_row, offsets, max_rows, num_expert, d_model, d_ffn, w1, b1,
                           apply_gelu, h, workspace, workspace_bytes, ccf::as_stream(stream), nullptr);
}

extern "C" int ccf_ffn2_forward(const void *h, const int32_t *src_row, const int32_t *dst_row,
                                const int32_t *offsets, int max_rows, int num_expert, int d_model,
                                int d_ffn, const void *w2, const void *b2, const void *row_scale,
                                void *y, void *workspace, size_t workspace_bytes,
                                ccf_stream_t stream) {
  return ccf::ffn2_forward(h, src_row, dst_row, offsets, max_rows, num_expert, d_model, d_ffn, w2, b2,
                           row_scale, y, workspace, workspace_bytes, ccf::as_stream(stream), nullptr);
}

extern "C" int ccf_ffn_plan_info(const void *workspace, int max_rows, int num_expert, int d_model, int d_ffn,
                                 int which, int32_t *info, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(workspace && info, CCF_ERR_ARG, "ffn_plan_info: null pointer");
  CCF_REQUIRE(which == 1 || which == 2, CCF_ERR_ARG, "ffn_plan_info: which=%d is neither 1 (first GEMM) nor 2", which);
  CCF_REQUIRE(max_rows > 0 && num_expert > 0 && num_expert <= 1024 && d_model > 0 && d_ffn > 0, CCF_ERR_ARG,
              "ffn_plan_info: bad size");
  const int N = which == 1 ? d_ffn : d_model, K = which == 1 ? d_model : d_ffn;
  const GemmSetup gs = setup_gemm(max_rows, num_expert, N, K, which == 1 ? kEpiGelu : kEpiPlain, false,
                                  const_cast<void *>(workspace), which == 1 ? 0 : 1, current_options());
  for (int i = 0; i < 8; ++i) info[i] = 0;
  hipStream_t st = as_stream(stream);
  hipError_t e = hipSuccess;
  if (gs.split || gs.cut) e = hipMemcpyAsync(info, gs.tail, 2 * sizeof(int32_t), hipMemcpyDeviceToHost, st);
  int32_t where = 0;
  if (gs.skinny && e == hipSuccess) e = hipMemcpyAsync(info + 2, gs.skinny_list, 4 * sizeof(int32_t), hipMemcpyDeviceToHost, st);
  if (gs.skinny && e == hipSuccess) e = hipMemcpyAsync(&where, gs.skinny_list + 4, sizeof(int32_t), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return fail(CCF_ERR_HIP, "ffn_plan_info: %s", hipGetErrorString(e));
  info[6] = gs.grid;
  info[7] = static_cast<int32_t>(gs.wgs < (1ll << 24) ? gs.wgs : -1);
  if (where == 1) info[5] = -info[5];                 // cut along K inside the persistent launch
  return CCF_OK;
}

extern "C" size_t ccf_ffn_backward_workspace_bytes(int max_rows, int num_expert, int d_model, int d_ffn) {
  if (max_rows < 0 || num_expert <= 0 || d_model <= 0 || d_ffn <= 0) return 0;
  return ccf::carve_backward(nullptr, max_rows, num_expert, d_model, d_ffn).bytes;
}

extern "C" int ccf_ffn1_forward_keep(const void *x, const int32_t *src_row, const int32_t *offsets,
                                     int max_rows, int num_expert, int d_model, int d_ffn,
                                     const void *w1, const void *b1, void *h_pre, void *act,
                                     void *workspace, size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  const size_t need = ccf_ffn_workspace_bytes(max_rows, num_expert, d_model, d_ffn);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "ffn1_keep: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CCF_REQUIRE(h_pre && act, CCF_ERR_ARG, "ffn1_keep: null output");
  return grouped_gemm(static_cast<const half_t *>(x), src_row, offsets, max_rows, num_expert, d_ffn,
                      d_model, static_cast<const half_t *>(w1), static_cast<const half_t *>(b1),
                      kEpiGeluKeep, static_cast<half_t *>(act), nullptr, nullptr,
                      workspace, as_stream(stream), "ffn1_keep", false,
                      static_cast<half_t *>(h_pre));
}

extern "C" int ccf_ffn2_backward(const void *grad_y_flat, const void *act, const void *h_pre,
                                 const int32_t *dst_row,
                                 const int32_t *offsets, int max_rows, int num_expert, int d_model,
                                 int d_ffn, const void *w2, void *grad_act, void *grad_w2,
                                 void *grad_b2, void *workspace, size_t workspace_bytes,
                                 ccf_stream_t stream) {
  using namespace ccf;
  if (max_rows == 0) return zero_param_grads(grad_w2, grad_b2, num_expert, d_model, d_ffn, as_stream(stream));
  return linear_backward(const_cast<half_t *>(static_cast<const half_t *>(grad_y_flat)), dst_row,
                         static_cast<const half_t *>(act), nullptr, offsets, max_rows, num_expert,
                         d_ffn, d_model, static_cast<const half_t *>(w2),
                         static_cast<half_t *>(grad_act), nullptr, static_cast<half_t *>(grad_w2),
                         static_cast<half_t *>(grad_b2), workspace, workspace_bytes, d_model, d_ffn,
                         as_stream(stream), "ffn2_backward", static_cast<const half_t *>(h_pre));
}

extern "C" int ccf_ffn1_backward(const void *grad_h, const void *x, const int32_t *src_row,
                                 const int32_t *dst_row, const int32_t *offsets, int max_rows,
                                 int num_expert, int d_model, int d_ffn, const void *w1,
                                 void *grad_x_flat, void *grad_w1, void *grad_b1, void *workspace,
                                 size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  if (max_rows == 0) return zero_param_grads(grad_w1, grad_b1, num_expert, d_ffn, d_model, as_stream(stream));
  return linear_backward(const_cast<half_t *>(static_cast<const half_t *>(grad_h)), nullptr, static_cast<const half_t *>(x),
                         src_row, offsets, max_rows, num_expert, d_model, d_ffn,
                         static_cast<const half_t *>(w1), static_cast<half_t *>(grad_x_flat), dst_row,
                         static_cast<half_t *>(grad_w1), static_cast<half_t *>(grad_b1), workspace,
                         workspace_bytes, d_model, d_ffn, as_stream(stream), "ffn1_backward");
}

extern "C" int ccf_ffn1_backward_gelu(void *grad_act, const void *h_pre, const void *x, const int32_t *src_row,
                                      const int32_t *dst_row, const int32_t *offsets, int max_rows,
                                      int num_expert, int d_model, int d_ffn, const void *w1,
                                      void *grad_x_flat, void *grad_w1, void *grad_b1, void *workspace,
                                      size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(h_pre && aligned16(h_pre), CCF_ERR_ARG, "ffn1_backward_gelu: the pre-activation is missing or unaligned");
  if (max_rows == 0) return zero_param_grads(grad_w1, grad_b1, num_expert, d_ffn, d_model, as_stream(stream));
  return linear_backward(static_cast<half_t *>(grad_act), nullptr, static_cast<const half_t *>(x), src_row, offsets,
                         max_rows, num_expert, d_model, d_ffn, static_cast<const half_t *>(w1),
                         static_cast<half_t *>(grad_x_flat), dst_row, static_cast<half_t *>(grad_w1),
                         static_cast<half_t *>(grad_b1), workspace, workspace_bytes, d_model, d_ffn, as_stream(stream),
                         "ffn1_backward_gelu", nullptr, static_cast<const half_t *>(h_pre));
}
