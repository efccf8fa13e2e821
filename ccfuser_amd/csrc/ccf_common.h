// Shared helpers for the HIP sources of libccfuser_moe.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <string.h>

#include "../../include/ccfuser_moe.h"

namespace ccf {

constexpr int kWave = 64;

// Last error text, per host thread.
char *error_buffer();
int fail(int code, const char *fmt, ...);

inline hipStream_t as_stream(ccf_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Launch check: a failed launch reports through hipGetLastError.
inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(CCF_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return CCF_OK;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef int int4v __attribute__((ext_vector_type(4)));

// bwd.hip: data movement of the backward pass
int padded_rows(int max_rows, int E);
int launch_zero(half_t *dst, size_t halves, hipStream_t stream);
int launch_transpose_weights(const half_t *in, half_t *out, int E, int R, int C, hipStream_t stream);
int launch_transpose_rows(const half_t *in, const int32_t *rows, const int32_t *blk_row0,
                          const int32_t *blk_cnt, int n_blk, int C, int ld_t, half_t *out_t,
                          float *partial, hipStream_t stream, const half_t *gelu_pre_inplace, bool transposed);
int launch_bias_reduce(const float *partial, const int32_t *k_seg, int E, int C, half_t *grad_bias,
                       hipStream_t stream);

// gate.hip
int gate_forward(const void *x, const void *wg, const void *bg, int tokens, int d_model, int tot_expert, int top_k,
                 int dtype, int64_t *idx_out, void *score_out, void *logits_out, ccf_stream_t stream,
                 int32_t *wg_cnt, long long max_cnt, int *tokens_per_wg);

// tuning knobs set through ccf_set_option()
extern int g_gate_waves, g_gate_slots, g_gate_stream;   // gate.hip
extern int g_route_rows_max;             // route.hip

}  // namespace ccf

#define CCF_REQUIRE(cond, code, ...)                 \
  do {                                               \
    if (!(cond)) return ccf::fail(code, __VA_ARGS__); \
  } while (0)
