// K = 1 fp32 MFMAs of gfx950 as the gate uses them: D = fma(A, B, C) per output element, one
// rounding.  Shared by the gate kernels and by the probe that pins this arithmetic and the
// accumulator layout against a chain of fused multiply-adds on the CPU.
#pragma once

#include <hip/hip_runtime.h>

namespace ccf {

typedef float float16v_ __attribute__((ext_vector_type(16)));
typedef float float32v __attribute__((ext_vector_type(32)));

template <int N>
struct Mfma;

template <>
struct Mfma<32> {
  typedef float32v Acc;
  static constexpr int kRegs = 32;
  __device__ static inline Acc run(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x1f32(a, b, c, 0, 0, 0);
  }
  // accumulator register v of a lane: block and row of that output element (column = lane % 32)
  __device__ static constexpr int block(int v) { return v >> 4; }
  __device__ static inline int row(int v, int lane) { return 8 * ((v & 15) >> 2) + 4 * (lane >> 5) + (v & 3); }
};

template <>
struct Mfma<16> {
  typedef float16v_ Acc;
  static constexpr int kRegs = 16;
  __device__ static inline Acc run(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x1f32(a, b, c, 0, 0, 0);
  }
  __device__ static constexpr int block(int v) { return v >> 2; }
  __device__ static inline int row(int v, int lane) { return 4 * (lane >> 4) + (v & 3); }
};

}  // namespace ccf
