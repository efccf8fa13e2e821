/*
 * libccfuser_probe.so -- measurement probes for the MI355X MoE library, kept out of the product
 * library (libccfuser_moe.so) and its header.  Neither function has a counterpart in the
 * reference: bench.py uses the first for its measured MFMA ceiling, one GPU test uses the second
 * to pin the arithmetic of the gate.  Return 0 on success, 1 for a bad argument, 4 when the
 * launch failed.  `stream` is a hipStream_t (NULL = the default stream).
 */
#ifndef CCFUSER_PROBE_H
#define CCFUSER_PROBE_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * `workgroups` workgroups of four wavefronts issue `iters` x 64 v_mfma_f32_16x16x32_f16 each on
 * register operands, constant (zeros) or pseudo-random, with no memory traffic; *flop receives
 * the flop count of the launch.
 * Timed with events by the caller it gives the rate the matrix cores sustain: the nominal peak
 * with constant operands, a lower, power-limited figure with random ones.
 *   out: device buffer of workgroups * 256 floats (sums that keep the loop alive).
 */
int ccf_probe_mfma(int workgroups, int iters, int constant_operands, void *out, double *flop,
                   void *stream);

/*
 * Probe of the arithmetic the fp16 gate rests on: one wavefront runs a chain of `steps` K = 1
 * fp32 MFMAs, acc = mfma(a[s][lane], b[s][lane], acc),
 * with v_mfma_f32_32x32x1_2b_f32 (tile = 32: two 32 x 32 blocks, 32 accumulator registers) or
 * v_mfma_f32_16x16x1_4b_f32 (tile = 16: four 16 x 16 blocks, 16 registers), and writes its
 * accumulator registers as out[reg][lane].  Block b takes rows from a and columns from b of
 * lanes b*tile .. b*tile + tile - 1.  The tests compare every output with a chain of fused
 * multiply-adds on the CPU.
 *   a, b: device, [steps][64] floats; out: device, [tile][64] floats.
 */
int ccf_probe_mfma_chain(const float *a, const float *b, int steps, int tile, float *out,
                         void *stream);

#ifdef __cplusplus
}
#endif

#endif
