// Measurement probe: what the matrix cores sustain with nothing else in the way.
//
// One workgroup of four wavefronts per CU (the grouped GEMM's shape: one wavefront per SIMD,
// 8 x 8 blocks of v_mfma_f32_16x16x32_f16 per wavefront) issues MFMAs back to back on operand
// fragments held in registers: no memory traffic, no LDS, no epilogue.  With constant operands
// the chip reaches its nominal rate; with random operands the same loop runs slower, because
// the data-dependent switching power makes the power limit lower the clock.  That second
// figure is the ceiling any fp16 GEMM on real data has on this hardware; bench.py reports it
// beside the nominal peak.  No counterpart in the reference.
#include "ccf_common.h"

#include <type_traits>

namespace ccf {
namespace {

__device__ inline half8 probe_fragment(unsigned &x, float scale, int constant) {
  half8 v;
  for (int j = 0; j < 8; j++) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    v[j] = constant ? static_cast<_Float16>(0.0f)
                    : static_cast<_Float16>((static_cast<int>(x & 0xffff) - 32768) / 32768.0f * scale);
  }
  return v;
}

constexpr int kProbeBlocks = 8;          // 8 x 8 MFMA blocks per wavefront, as in the GEMM main loop

// The 64 accumulator blocks live in the accumulation registers a[4 blk .. 4 blk + 3], named
// literally as in the GEMM main loop (as C++ objects the compiler shuffles 256 of them between
// the two register files inside the loop, and the loop then measures those copies).
template <int BLK>
__device__ __forceinline__ void probe_mfma_from(const half8 (&a)[kProbeBlocks], const half8 (&b)[kProbeBlocks]) {
  if constexpr (BLK < kProbeBlocks * kProbeBlocks) {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, a[%2:%3]"
                 :
                 : "v"(b[BLK % kProbeBlocks]), "v"(a[BLK / kProbeBlocks]), "n"(4 * BLK), "n"(4 * BLK + 3));
    probe_mfma_from<BLK + 1>(a, b);
  }
}
template <int R>
__device__ __forceinline__ void probe_zero_from() {
  if constexpr (R < 256) {
    asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(R));
    probe_zero_from<R + 1>();
  }
}
// One register at a time: reading all 256 before adding would need 256 live registers, and the
// compiler would then park values of its own in the accumulation registers this kernel names.
template <int R>
__device__ __forceinline__ float probe_sum_from(float s) {
  if constexpr (R < 256) {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"(R));
    s += v;
    asm volatile("" : "+v"(s));                        // keep the adds in step with the reads
    return probe_sum_from<R + 1>(s);
  } else {
    return s;
  }
}

__global__ void __launch_bounds__(256)
mfma_probe_kernel(float *out, int iters, int constant) {
  unsigned x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  half8 a[kProbeBlocks], b[kProbeBlocks];
  for (int i = 0; i < kProbeBlocks; i++) a[i] = probe_fragment(x, 1.0f, constant);      // token-like values
  for (int i = 0; i < kProbeBlocks; i++) b[i] = probe_fragment(x, 0.03f, constant);     // weight-like values
  asm volatile("" ::: "a255");                                                         // the kernel owns all 256
  probe_zero_from<0>();
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");
  for (int it = 0; it < iters; it++) probe_mfma_from<0>(a, b);
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");
  out[blockIdx.x * blockDim.x + threadIdx.x] = probe_sum_from<0>(0.0f);
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_probe_mfma(int workgroups, int iters, int constant_operands, void *out, double *flop,
                              ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(out && flop, CCF_ERR_ARG, "probe_mfma: null pointer");
  CCF_REQUIRE(workgroups > 0 && workgroups <= 4096 && iters > 0, CCF_ERR_ARG, "probe_mfma: bad size");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(workgroups), dim3(256), 0, as_stream(stream), static_cast<float *>(out),
                     iters, constant_operands);
  // 4 wavefronts x iters x 64 MFMAs of 16 x 16 x 32 x 2 flop
  *flop = static_cast<double>(workgroups) * 4.0 * iters * (kProbeBlocks * kProbeBlocks) * (16.0 * 16.0 * 32.0 * 2.0);
  return check_launch("mfma_probe_kernel");
}
