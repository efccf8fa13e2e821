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
namespace {

constexpr int kMaxTopK = 8;
constexpr int kGateTT = 4;   // tokens per wavefront
constexpr int kGateEG = 8;   // experts accumulated per pass over x

template <typename T>
__device__ inline void load8(const T *p, float (&v)[8]);

template <>
__device__ inline void load8<half_t>(const half_t *p, float (&v)[8]) {
  half8 h = *reinterpret_cast<const half8 *>(p);
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = static_cast<float>(h[j]);
}

template <>
__device__ inline void load8<float>(const float *p, float (&v)[8]) {
  float4v a = reinterpret_cast<const float4v *>(p)[0];
  float4v b = reinterpret_cast<const float4v *>(p)[1];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v[j] = a[j];
    v[4 + j] = b[j];
  }
}

template <typename T>
__device__ inline float round_to(float v) {
  return static_cast<float>(static_cast<T>(v));
}

__device__ inline bool better(float v, int id, float bv, int bid) {
  return v > bv || (v == bv && id < bid);
}

template <typename T>
__global__ void __launch_bounds__(256)
gate_kernel(const T *__restrict__ x, const T *__restrict__ wg, const T *__restrict__ bg,
            int tokens, int d, int E, int k, int64_t *__restrict__ idx_out,
            T *__restrict__ score_out, T *__restrict__ logits_out) {
#pragma clang fp contract(off)
  extern __shared__ float s_logit[];               // [4 waves][kGateTT][E]
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int t0 = (blockIdx.x * 4 + wave) * kGateTT;
  const int nchunk = d >> 3;
  float *mine = s_logit + static_cast<size_t>(wave) * kGateTT * E;

  const T *xrow[kGateTT];
#pragma unroll
  for (int tt = 0; tt < kGateTT; ++tt) {
    int t = t0 + tt;
    if (t > tokens - 1) t = tokens - 1;            // tail waves re-read the last token
    xrow[tt] = x + static_cast<size_t>(t) * d;
  }

  for (int e0 = 0; e0 < E; e0 += kGateEG) {
    float acc[kGateTT][kGateEG];
#pragma unroll
    for (int tt = 0; tt < kGateTT; ++tt)
#pragma unroll
      for (int g = 0; g < kGateEG; ++g) acc[tt][g] = 0.0f;

    for (int c = lane; c < nchunk; c += kWave) {
      float xv[kGateTT][8];
#pragma unroll
      for (int tt = 0; tt < kGateTT; ++tt) load8<T>(xrow[tt] + c * 8, xv[tt]);
#pragma unroll
      for (int g = 0; g < kGateEG; ++g) {
        if (e0 + g < E) {
          float wv[8];
          load8<T>(wg + static_cast<size_t>(e0 + g) * d + c * 8, wv);
#pragma unroll
          for (int tt = 0; tt < kGateTT; ++tt)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              float p = xv[tt][j] * wv[j];
              acc[tt][g] = acc[tt][g] + p;
            }
        }
      }
    }
#pragma unroll
    for (int tt = 0; tt < kGateTT; ++tt)
#pragma unroll
      for (int g = 0; g < kGateEG; ++g) {
        float v = acc[tt][g];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, kWave);
        if (lane == 0 && e0 + g < E) {
          float b = bg ? static_cast<float>(bg[e0 + g]) : 0.0f;
          mine[tt * E + e0 + g] = round_to<T>(v + b);
        }
      }
  }
  __syncthreads();

#pragma unroll 1
  for (int tt = 0; tt < kGateTT; ++tt) {
    const int t = t0 + tt;
    if (t >= tokens) break;                        // uniform per wave
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
  const int tokens_per_block = 4 * kGateTT;
  dim3 grid((tokens + tokens_per_block - 1) / tokens_per_block), block(256);
  size_t lds = sizeof(float) * 4 * kGateTT * static_cast<size_t>(tot_expert);
  if (dtype == CCF_F16) {
    hipLaunchKernelGGL(gate_kernel<half_t>, grid, block, lds, as_stream(stream),
                       static_cast<const half_t *>(x), static_cast<const half_t *>(wg),
                       static_cast<const half_t *>(bg), tokens, d_model, tot_expert, top_k, idx_out,
                       static_cast<half_t *>(score_out), static_cast<half_t *>(logits_out));
  } else {
    hipLaunchKernelGGL(gate_kernel<float>, grid, block, lds, as_stream(stream),
                       static_cast<const float *>(x), static_cast<const float *>(wg),
                       static_cast<const float *>(bg), tokens, d_model, tot_expert, top_k, idx_out,
                       static_cast<float *>(score_out), static_cast<float *>(logits_out));
  }
  return check_launch("gate_kernel");
}
