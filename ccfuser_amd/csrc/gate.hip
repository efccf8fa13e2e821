// Top-k softmax gate for gfx950.
//
// logits[t, e] = sum_k x[t, k] * wg[e, k] + bg[e], then top-k and a softmax
// over the k selected logits (reference mix_moe/mix_moe/gates/naive_gate.py:31-38).
//
// The expert choice has to be reproducible bit for bit, so the fp32 sum is
// taken in one fixed order that a CPU can replay: K is cut into chunks of 8;
// lane l of a 64-lane wavefront owns chunks l, l+64, ... and adds their
// products one element at a time; the 64 partial sums are folded by an xor
// butterfly (32, 16, 8, 4, 2, 1); the bias is added last and the logit is
// rounded once to the input dtype.  Multiplies and adds are kept separate
// (contraction off), which changes nothing for fp16 inputs, whose products are
// exact in fp32, and keeps fp32 inputs replayable without a fused multiply-add.
//
// One wavefront scores TT tokens at a time so that each 16-byte piece of wg it
// reads feeds TT*8 multiply-adds; x is read from HBM once, wg comes from cache.
#include "ccf_common.h"

#include <limits.h>

namespace ccf {
int g_gate_waves = 16;   // wavefronts per gate workgroup when the weights sit in LDS; 4 forces the small one
int g_gate_tt = 0;       // tokens a wavefront scores at a time (1, 2 or 4); 0 = by the token count
namespace {

constexpr int kMaxTopK = 8;
constexpr int kGateEG = 8;   // experts accumulated per pass over x

// Eight consecutive K elements as loaded, and acc += x[j] * w[j] for j = 0..7 in
// order.  For fp16 the product is exact in fp32, so a fused multiply-add on the
// fp16 operands (v_fma_mix_f32, no conversions) gives the same bits as a
// multiply followed by an add; for fp32 the two stay separate.
template <typename T>
struct Chunk;

template <>
struct Chunk<half_t> {
  half8 v;
  __device__ inline void load(const half_t *p) { v = *reinterpret_cast<const half8 *>(p); }
  __device__ inline void mac(const Chunk &w, float &acc) const {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      acc = __builtin_fmaf(static_cast<float>(v[j]), static_cast<float>(w.v[j]), acc);
  }
};

template <>
struct Chunk<float> {
  float4v lo, hi;
  __device__ inline void load(const float *p) {
    lo = reinterpret_cast<const float4v *>(p)[0];
    hi = reinterpret_cast<const float4v *>(p)[1];
  }
  __device__ inline void mac(const Chunk &w, float &acc) const {
#pragma clang fp contract(off)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float p = lo[j] * w.lo[j];
      acc = acc + p;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float p = hi[j] * w.hi[j];
      acc = acc + p;
    }
  }
};

template <typename T>
__device__ inline float round_to(float v) {
  return static_cast<float>(static_cast<T>(v));
}

__device__ inline bool better(float v, int id, float bv, int bid) {
  return v > bv || (v == bv && id < bid);
}

// One level of the lane fold (see gate_kernel): LIVE values remain, partner lane
// is lane ^ OFF.  Everything is resolved at compile time so v stays in registers.
template <int LIVE, int OFF, int N>
__device__ inline void fold_level(float (&v)[N], int lane) {
  if constexpr (OFF >= 1) {
    if constexpr (LIVE > 1) {
      constexpr int HALF = LIVE / 2;
      const bool upper = (lane & OFF) != 0;
#pragma unroll
      for (int j = 0; j < HALF; ++j) {
        const float keep = upper ? v[j + HALF] : v[j];
        const float send = upper ? v[j] : v[j + HALF];
        v[j] = keep + __shfl_xor(send, OFF, kWave);
      }
      fold_level<HALF, OFF / 2, N>(v, lane);
    } else {
      v[0] = v[0] + __shfl_xor(v[0], OFF, kWave);
      fold_level<1, OFF / 2, N>(v, lane);
    }
  }
}

template <int N, int OFF>
__device__ inline void fold_lanes(float (&v)[N], int lane) {
  fold_level<N, OFF, N>(v, lane);
}

// Workgroups are persistent: each stages an expert group's weight rows in LDS
// once (when they fit, kWLds) and then walks over its share of the tokens, one
// wavefront scoring TT tokens at a time.  The x chunks of up to kBatch passes
// are requested together before any arithmetic (one memory round trip for
// d_model <= 4096).  Logits of all experts are parked in LDS until the last
// expert group is done, then each wavefront picks the top-k of its tokens.
// None of this changes the order of the additions.
template <typename T, int TT, bool kWLds, int GW>
__global__ void __launch_bounds__(GW * 64)
gate_kernel(const T *__restrict__ x, const T *__restrict__ wg, const T *__restrict__ bg,
            int tokens, int d, int E, int k, int groups_per_block, int64_t *__restrict__ idx_out,
            T *__restrict__ score_out, T *__restrict__ logits_out) {
#pragma clang fp contract(off)
  constexpr int kBatch = 8 / TT;                   // x chunks requested together per lane
  extern __shared__ float s_logit[];               // [groups_per_block][GW wavefronts][TT][E], then weights
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int nchunk = d >> 3;
  const int niter = (nchunk + kWave - 1) / kWave;
  const int n_groups = (tokens + GW * TT - 1) / (GW * TT);
  T *w_lds = reinterpret_cast<T *>(s_logit + static_cast<size_t>(groups_per_block) * GW * TT * E);

  for (int e0 = 0; e0 < E; e0 += kGateEG) {
    const int ng = (E - e0) < kGateEG ? (E - e0) : kGateEG;
    if (kWLds) {
      __syncthreads();                             // previous group fully consumed
      // always kGateEG rows (rows past E repeat the last expert and are discarded),
      // 16-byte pieces, 8 loads in flight per lane
      const int per_row = static_cast<int>(static_cast<size_t>(d) * sizeof(T) / 16);
      const int total = kGateEG * per_row;
      int4v *dst = reinterpret_cast<int4v *>(w_lds);
      for (int i0 = threadIdx.x; i0 < total; i0 += GW * 64 * 8) {
        int4v tmp[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = i0 + u * GW * 64;
          if (i < total) {
            int row = e0 + i / per_row;
            row = row < E ? row : E - 1;
            tmp[u] = reinterpret_cast<const int4v *>(wg + static_cast<size_t>(row) * d)[i % per_row];
          }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (i0 + u * GW * 64 < total) dst[i0 + u * GW * 64] = tmp[u];
      }
      __syncthreads();
    }
    const T *wbase = kWLds ? w_lds : wg + static_cast<size_t>(e0) * d;

    for (int gi = 0; gi < groups_per_block; ++gi) {
      const int grp = blockIdx.x + gi * gridDim.x;
      if (grp >= n_groups) break;                  // uniform per workgroup
      const int t0 = (grp * GW + wave) * TT;
      float *mine = s_logit + (static_cast<size_t>(gi) * GW + wave) * TT * E;
      const T *xrow[TT];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        int t = t0 + tt;
        if (t > tokens - 1) t = tokens - 1;        // tail waves re-read the last token
        xrow[tt] = x + static_cast<size_t>(t) * d;
      }
      float acc[TT][kGateEG];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int g = 0; g < kGateEG; ++g) acc[tt][g] = 0.0f;

      for (int it0 = 0; it0 < niter; it0 += kBatch) {
        Chunk<T> xv[kBatch][TT];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
          const int c = lane + (it0 + i) * kWave;
          if (c < nchunk) {
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) xv[i][tt].load(xrow[tt] + c * 8);
          }
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
          const int c = lane + (it0 + i) * kWave;
          if (c < nchunk) {                        // lanes past the end of K skip the whole chunk
#pragma unroll
            for (int g = 0; g < kGateEG; ++g) {
              Chunk<T> wv;
              if (kWLds) {
                wv.load(wbase + static_cast<size_t>(g) * d + c * 8);
              } else {
                const int row = (e0 + g) < E ? g : (E - 1 - e0);
                wv.load(wbase + static_cast<size_t>(row) * d + c * 8);
              }
#pragma unroll
              for (int tt = 0; tt < TT; ++tt) xv[i][tt].mac(wv, acc[tt][g]);
            }
          }
        }
      }
      // Fold the 64 lane sums of all TT*kGateEG accumulators at once.  Level by
      // level (xor 32, 16, ...) a lane keeps the half of the values its lane bit
      // selects and adds the partner's copy of them, so N values cost N-1
      // exchanges instead of 6N; the pairs added at each level, and therefore
      // the bits of the result, are those of the plain butterfly.  Value i ends
      // up in the lanes whose top log2(N) lane bits spell i.
      constexpr int N = TT * kGateEG;
      float v[N];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int g = 0; g < kGateEG; ++g) v[tt * kGateEG + g] = acc[tt][g];
      fold_lanes<N, 32>(v, lane);
      {
        constexpr int kBits = N == 32 ? 5 : (N == 16 ? 4 : 3);
        static_assert(N == 8 || N == 16 || N == 32, "TT*kGateEG");
        const int i = lane >> (6 - kBits);                      // value this lane holds
        const int tt = i / kGateEG, g = i % kGateEG;
        if ((lane & ((1 << (6 - kBits)) - 1)) == 0 && g < ng) {
          float b = bg ? static_cast<float>(bg[e0 + g]) : 0.0f;
          mine[tt * E + e0 + g] = round_to<T>(v[0] + b);
        }
      }
    }
  }
  __syncthreads();

  for (int gi = 0; gi < groups_per_block; ++gi) {
    const int grp = blockIdx.x + gi * gridDim.x;
    if (grp >= n_groups) break;
    const int t0 = (grp * GW + wave) * TT;
    const float *mine = s_logit + (static_cast<size_t>(gi) * GW + wave) * TT * E;
#pragma unroll 1
    for (int tt = 0; tt < TT; ++tt) {
      const int t = t0 + tt;
      if (t >= tokens) break;                      // uniform per wave
      const float *lg = mine + tt * E;
      if (logits_out)
        for (int e = lane; e < E; e += kWave)
          logits_out[static_cast<size_t>(t) * E + e] = static_cast<T>(lg[e]);

      float sel_v[kMaxTopK];
      int sel_id[kMaxTopK];
#pragma unroll
      for (int s = 0; s < kMaxTopK; ++s) {
        sel_v[s] = 0.0f;
        sel_id[s] = -1;
      }
#pragma unroll
      for (int s = 0; s < kMaxTopK; ++s) {
        if (s < k) {
          float bv = -INFINITY;
          int bid = INT_MAX;
          for (int e = lane; e < E; e += kWave) {
            bool taken = false;
#pragma unroll
            for (int q = 0; q < kMaxTopK; ++q) taken = taken || (q < s && sel_id[q] == e);
            float v = lg[e];
            if (!taken && better(v, e, bv, bid)) {
              bv = v;
              bid = e;
            }
          }
#pragma unroll
          for (int off = 32; off >= 1; off >>= 1) {
            float ov = __shfl_xor(bv, off, kWave);
            int oi = __shfl_xor(bid, off, kWave);
            if (better(ov, oi, bv, bid)) {
              bv = ov;
              bid = oi;
            }
          }
          sel_v[s] = bv;
          sel_id[s] = bid;
        }
      }
      if (lane == 0) {
        // softmax over the k selected logits; slot 0 holds the maximum
        float ex[kMaxTopK];
        float sum = 0.0f;
#pragma unroll
        for (int s = 0; s < kMaxTopK; ++s) {
          ex[s] = (s < k) ? expf(sel_v[s] - sel_v[0]) : 0.0f;
          sum += ex[s];
        }
#pragma unroll
        for (int s = 0; s < kMaxTopK; ++s) {
          if (s < k) {
            idx_out[static_cast<size_t>(t) * k + s] = static_cast<int64_t>(sel_id[s]);
            score_out[static_cast<size_t>(t) * k + s] = static_cast<T>(ex[s] / sum);
          }
        }
      }
    }
  }
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_gate_topk_softmax(const void *x, const void *wg, const void *bg, int tokens,
                                     int d_model, int tot_expert, int top_k, int dtype,
                                     int64_t *idx_out, void *score_out, void *logits_out,
                                     ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(x && wg && idx_out && score_out, CCF_ERR_ARG, "gate: null pointer");
  CCF_REQUIRE(tokens >= 0 && d_model > 0 && tot_expert > 0, CCF_ERR_ARG, "gate: bad size");
  CCF_REQUIRE(d_model % 8 == 0, CCF_ERR_SHAPE, "gate: d_model=%d is not a multiple of 8", d_model);
  CCF_REQUIRE(top_k >= 1 && top_k <= kMaxTopK && top_k <= tot_expert, CCF_ERR_SHAPE,
              "gate: top_k=%d outside 1..min(%d, tot_expert=%d)", top_k, kMaxTopK, tot_expert);
  CCF_REQUIRE(tot_expert <= 1024, CCF_ERR_SHAPE, "gate: tot_expert=%d exceeds 1024", tot_expert);
  CCF_REQUIRE(dtype == CCF_F16 || dtype == CCF_F32, CCF_ERR_UNSUPPORTED, "gate: dtype %d", dtype);
  CCF_REQUIRE(aligned16(x) && aligned16(wg), CCF_ERR_ARG, "gate: x and wg must be 16-byte aligned");
  if (tokens == 0) return CCF_OK;
  // Enough wavefronts to hide HBM latency: fewer tokens per wavefront when the batch is small.
  const int tt = g_gate_tt ? g_gate_tt : (tokens >= 32768 ? 4 : (tokens >= 8192 ? 2 : 1));
  const size_t esz = dtype == CCF_F16 ? 2 : 4;
  // the kernel always stages kGateEG weight rows (rows past the last expert repeat it)
  const size_t w_bytes = static_cast<size_t>(kGateEG) * d_model * esz;
  const bool w_lds = w_bytes <= 65536;             // one expert group of weights fits next to the logits
  // Wavefronts per workgroup: 16 (one workgroup per CU stages the weights once for 16
  // wavefronts) when the weights sit in LDS, else 4 (two workgroups per CU).
  const int gw = (w_lds && g_gate_waves != 4) ? 16 : 4;
  const int n_groups = (tokens + gw * tt - 1) / (gw * tt);
  const int max_blocks = gw == 16 ? 256 : 512;     // persistent workgroups
  int blocks = n_groups < max_blocks ? n_groups : max_blocks;
  int groups_per_block = (n_groups + blocks - 1) / blocks;
  // the logits of a workgroup's tokens wait in LDS: more workgroups when they would not fit
  const size_t per_group = sizeof(float) * gw * tt * static_cast<size_t>(tot_expert);
  const size_t lds_budget = 160 * 1024 - (w_lds ? w_bytes : 0);
  if (per_group * groups_per_block > lds_budget && per_group <= lds_budget) {
    groups_per_block = static_cast<int>(lds_budget / per_group);
    blocks = (n_groups + groups_per_block - 1) / groups_per_block;
  }
  dim3 grid(blocks), block(gw * 64);
  const size_t lds = per_group * groups_per_block + (w_lds ? w_bytes : 0);
  CCF_REQUIRE(lds <= 160 * 1024, CCF_ERR_SHAPE, "gate: %zu bytes of LDS needed", lds);
#define CCF_GATE_LAUNCH(TYPE, TT, WL, GWV)                                                            \
  do {                                                                                             \
    auto kern = gate_kernel<TYPE, TT, WL, GWV>;                                                    \
    if (lds > 65536) {                                                                             \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize,               \
                                         static_cast<int>(lds));                                   \
      if (e != hipSuccess) return fail(CCF_ERR_HIP, "gate: LDS attribute: %s", hipGetErrorString(e)); \
    }                                                                                              \
    hipLaunchKernelGGL(kern, grid, block, lds, as_stream(stream), static_cast<const TYPE *>(x),    \
                       static_cast<const TYPE *>(wg), static_cast<const TYPE *>(bg), tokens,      \
                       d_model, tot_expert, top_k, groups_per_block, idx_out,                      \
                       static_cast<TYPE *>(score_out),                                             \
                       static_cast<TYPE *>(logits_out));                                           \
  } while (0)
#define CCF_GATE_TT(TYPE, WL, GWV)                    \
  do {                                                \
    if (tt == 4) CCF_GATE_LAUNCH(TYPE, 4, WL, GWV);   \
    else if (tt == 2) CCF_GATE_LAUNCH(TYPE, 2, WL, GWV); \
    else CCF_GATE_LAUNCH(TYPE, 1, WL, GWV);           \
  } while (0)
#define CCF_GATE_W(TYPE)                                              \
  do {                                                                \
    if (!w_lds) CCF_GATE_TT(TYPE, false, 4);                          \
    else if (gw == 16) CCF_GATE_TT(TYPE, true, 16);                   \
    else CCF_GATE_TT(TYPE, true, 4);                                  \
  } while (0)
  if (dtype == CCF_F16) CCF_GATE_W(half_t); else CCF_GATE_W(float);
#undef CCF_GATE_W
#undef CCF_GATE_TT
#undef CCF_GATE_LAUNCH
  return check_launch("gate_kernel");
}
