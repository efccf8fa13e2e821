// The erf GELU and its derivative as the kernels evaluate them (polynomial erf, no library call).
#pragma once

#include <hip/hip_runtime.h>

namespace ccf {

// erf-form GELU, v * Phi(v) with Phi(v) = 0.5 + 0.5*erf(v/sqrt2) = 0.5 + u*Q(u^2), u = v
// clamped to +-3*sqrt2 (beyond it 1 - erf < 2.3e-5).  0.5*erf(u/sqrt2) is an odd minimax
// polynomial u*Q(u^2) of degree 8 in u^2, fitted on [0, 3] in z = u/sqrt2 with the 1/sqrt2
// and the 0.5 folded into the coefficients.  Measured in fp32 against the exact function:
// within 1.4e-5 for |v| <= 2, 5.9e-5 for |v| <= 8 (at -8 the result is -2e-5 instead of -0),
// an eighth of the fp16 rounding step of a result of magnitude 1.  12 full-rate instructions
// with the fp16 conversion and no transcendental (the library erff is ~40, the exp-based form
// 15 plus rcp and exp at quarter rate); the FFN1 epilogue applies it to 256 values per lane
// and tile and is bound by this arithmetic.
__device__ __forceinline__ float gelu_erf(float v) {
  const float u = __builtin_amdgcn_fmed3f(v, -4.2426406871192851464f, 4.2426406871192851464f);
  const float t = u * u;
  float q = 1.1253530e-10f * 0.5f;
  q = fmaf(q, t, -1.0743734e-08f * 0.5f);
  q = fmaf(q, t, 4.5365911e-07f * 0.5f);
  q = fmaf(q, t, -1.1292428e-05f * 0.5f);
  q = fmaf(q, t, 1.8718123e-04f * 0.5f);
  q = fmaf(q, t, -2.2188006e-03f * 0.5f);
  q = fmaf(q, t, 1.9636238e-02f * 0.5f);
  q = fmaf(q, t, -1.3269384e-01f * 0.5f);
  q = fmaf(q, t, 7.9780629e-01f * 0.5f);
  return v * fmaf(u, q, 0.5f);
}

// Derivative of the erf GELU, Phi(v) + v*phi(v), with the same erf polynomial.
__device__ __forceinline__ float gelu_erf_grad(float v) {
  const float u = fminf(fabsf(v), 4.2426406871192851464f);
  const float t = u * u;
  float q = 1.1253530e-10f * 0.5f;
  q = fmaf(q, t, -1.0743734e-08f * 0.5f);
  q = fmaf(q, t, 4.5365911e-07f * 0.5f);
  q = fmaf(q, t, -1.1292428e-05f * 0.5f);
  q = fmaf(q, t, 1.8718123e-04f * 0.5f);
  q = fmaf(q, t, -2.2188006e-03f * 0.5f);
  q = fmaf(q, t, 1.9636238e-02f * 0.5f);
  q = fmaf(q, t, -1.3269384e-01f * 0.5f);
  q = fmaf(q, t, 7.9780629e-01f * 0.5f);
  const float half_erf = copysignf(fminf(q * u, 0.5f), v);        // 0.5 * erf(v / sqrt2)
  // phi(v) = exp(-v^2/2) / sqrt(2 pi) = exp2(-v^2 * log2(e)/2) * 0.3989...
  const float pdf = 0.3989422804014327f * __builtin_amdgcn_exp2f(-0.72134752044448170368f * v * v);
  return fmaf(v, pdf, 0.5f + half_erf);
}

}  // namespace ccf
