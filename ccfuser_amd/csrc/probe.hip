// libccfuser_probe.so: two measurement probes, built apart from the product library
// (libccfuser_moe.so exports the MoE path only).  Neither has a counterpart in the reference.
//
// 1. What the matrix cores sustain with nothing else in the way.
//
// One workgroup of four wavefronts per CU (the grouped GEMM's shape: one wavefront per SIMD,
// 8 x 8 blocks of v_mfma_f32_16x16x32_f16 per wavefront) issues MFMAs back to back on operand
// fragments held in registers: no memory traffic, no LDS, no epilogue.  With constant operands
// the chip reaches its nominal rate; with random operands the same loop runs slower, because
// the data-dependent switching power makes the power limit lower the clock.  That second
// figure is the ceiling any fp16 GEMM on real data has on this hardware; bench.py reports it
// beside the nominal peak.
//
// 2. The arithmetic the fp16 gate rests on: a chain of K = 1 fp32 MFMAs on one wavefront, for a
// test that compares every accumulator with a chain of fused multiply-adds on the CPU.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ccfuser_probe.h"
#include "mfma_f32.h"

namespace ccf {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

inline int launch_status() { return hipGetLastError() == hipSuccess ? 0 : 4; }

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
                              void *stream) {
  using namespace ccf;
  if (!out || !flop || workgroups <= 0 || workgroups > 4096 || iters <= 0) return 1;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<float *>(out), iters, constant_operands);
  // 4 wavefronts x iters x 64 MFMAs of 16 x 16 x 32 x 2 flop
  *flop = static_cast<double>(workgroups) * 4.0 * iters * (kProbeBlocks * kProbeBlocks) * (16.0 * 16.0 * 32.0 * 2.0);
  return launch_status();
}

namespace ccf {
namespace {

// One wavefront runs a chain of `steps` K = 1 fp32 MFMAs, acc = mfma(a[s][lane], b[s][lane], acc),
// and leaves its accumulator registers as out[reg][lane].
template <int N>
__global__ void __launch_bounds__(64)
mfma_chain_probe_kernel(const float *__restrict__ a, const float *__restrict__ b, int steps,
                        float *__restrict__ out) {
  using M = Mfma<N>;
  typename M::Acc acc;
#pragma unroll
  for (int v = 0; v < M::kRegs; ++v) acc[v] = 0.0f;
  const int lane = threadIdx.x;
  for (int s = 0; s < steps; ++s) acc = M::run(a[s * 64 + lane], b[s * 64 + lane], acc);
#pragma unroll
  for (int v = 0; v < M::kRegs; ++v) out[v * 64 + lane] = acc[v];
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_probe_mfma_chain(const float *a, const float *b, int steps, int tile, float *out, void *stream) {
  using namespace ccf;
  if (!a || !b || !out || steps < 0 || (tile != 16 && tile != 32)) return 1;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (tile == 32)
    hipLaunchKernelGGL(mfma_chain_probe_kernel<32>, dim3(1), dim3(64), 0, st, a, b, steps, out);
  else
    hipLaunchKernelGGL(mfma_chain_probe_kernel<16>, dim3(1), dim3(64), 0, st, a, b, steps, out);
  return launch_status();
}
