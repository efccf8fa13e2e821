// Data movement of the backward pass for gfx950 (HBM-bound kernels).
//
// The reference's backward pair (mix_moe/csrc/mix_moe.h:300-388, 439-505) runs
// its forward GEMM kernels on the stored [E, out, in] weight for the input
// gradients and a block-CSR kernel on transposed activations
// (`grad_out.transpose(-2, -1).contiguous()`, mix_moe.h:343, 492) for the weight
// gradients.  Here both become calls of the one grouped GEMM, whose operands
// must have the contraction index contiguous:
//   * input gradients contract over the weight's rows: the GEMM's main loop reads
//     the stored weight as a [K][N] operand through transposing LDS reads
//     (gemm_tile.h, B_KN), or, for widths that are no multiple of its column
//     tile, runs on a copy transposed here (transpose_weights);
//   * weight gradients contract over an expert's rows, so the two activation
//     matrices are transposed into [columns, padded rows] with every expert's
//     rows starting at a multiple of 64 and zero-filled up to a multiple of 64
//     and at least 256 (transpose_rows): the expert's range is then a whole
//     number of K tiles and the padding adds zeros to the sum;
//   * bias gradients are column sums over an expert's rows: the row transpose
//     has every element in LDS anyway and writes one partial sum per 64-row
//     block, and bias_reduce adds an expert's partial sums in block order, so
//     the result does not depend on scheduling.
// The reference leaves grad_bias uninitialised (mix_moe.h:342, 488).
#include "ccf_common.h"
#include "gelu.h"
#include "plan.h"

namespace ccf {
namespace {

constexpr int kTile = 64;
constexpr int kPadK = 256;            // shortest K range the persistent GEMM takes (four K tiles)

// Padded K ranges per expert and what each 64-row block of the padded layout holds.
//   k_seg[e]   = start of expert e's columns (multiple of 64); k_seg[E] = total
//   row_off[e] = e * seg_rows (row offsets of the [E * seg_rows, N] output)
//   blk_row0[b], blk_cnt[b]: first sorted row and real rows (0..64) of block b,
//   cnt = -1 for blocks past k_seg[E]
__global__ void __launch_bounds__(1024)
kseg_kernel(const int32_t *__restrict__ offsets, int E, int max_rows, int seg_rows, int n_blk,
            int32_t *__restrict__ k_seg, int32_t *__restrict__ row_off,
            int32_t *__restrict__ blk_row0, int32_t *__restrict__ blk_cnt, int32_t *__restrict__ row_lo,
            half_t *__restrict__ zero_row, PlanReq rows_plan, int rows_plan_wgs, PlanReq w_plan, int w_plan_wgs) {
  // workgroups behind the first build the tile plans of the call's two GEMMs
  if (blockIdx.x > 0) {
    const int b = static_cast<int>(blockIdx.x) - 1;
    if (b < rows_plan_wgs) build_plan(rows_plan, offsets, E, b, rows_plan_wgs);
    else build_plan(w_plan, nullptr, E, b - rows_plan_wgs, w_plan_wgs, seg_rows);
    return;
  }
  __shared__ int s_k[1025];
  const int t = threadIdx.x;
  // for the weight-gradient GEMM on row-major operands: the experts' row ranges, never past max_rows, and a row of zeros
  if (row_lo && t <= E) row_lo[t] = offsets[t] < max_rows ? offsets[t] : max_rows;
  if (zero_row && t < 256) zero_row[t] = static_cast<half_t>(0.0f);
  int lo = 0, cnt = 0;
  if (t < E) {
    lo = offsets[t] < max_rows ? offsets[t] : max_rows;
    const int hi = offsets[t + 1] < max_rows ? offsets[t + 1] : max_rows;
    cnt = hi > lo ? hi - lo : 0;
  }
  int padded = (cnt + kTile - 1) / kTile * kTile;
  padded = padded < kPadK ? kPadK : padded;
  if (t >= E) padded = 0;
  if (t == 0) s_k[0] = 0;
  s_k[t + 1] = padded;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int a = (t + 1 > d) ? s_k[t + 1 - d] : 0;
    __syncthreads();
    s_k[t + 1] += a;
    __syncthreads();
  }
  if (t <= E && t < 1024) k_seg[t] = s_k[t];
  if (t == 0) k_seg[E] = s_k[E];
  if (t <= E && t < 1024) row_off[t] = t * seg_rows;
  if (t == 0) row_off[E] = E * seg_rows;
  const int total_blk = s_k[E] / kTile;
  if (t < E) {
    const int b0 = s_k[t] / kTile, nb = padded / kTile;
    for (int b = 0; b < nb; ++b) {
      if (b0 + b < n_blk) {
        const int left = cnt - b * kTile;
        blk_row0[b0 + b] = lo + b * kTile;
        blk_cnt[b0 + b] = left < 0 ? 0 : (left > kTile ? kTile : left);
      }
    }
  }
  for (int b = total_blk + t; b < n_blk; b += 1024) {
    blk_row0[b] = 0;
    blk_cnt[b] = -1;
  }
}

// out[e][c][r] = in[e][r][c]; R and C multiples of 64.
__global__ void __launch_bounds__(256)
transpose_weights_kernel(const half_t *__restrict__ in, half_t *__restrict__ out, int R, int C) {
  __shared__ half_t tile[kTile][kTile + 8];
  const size_t base = static_cast<size_t>(blockIdx.z) * R * C;
  const int r0 = blockIdx.x * kTile, c0 = blockIdx.y * kTile;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int q = threadIdx.x + it * 256;          // 512 chunks of 8 halves
    const int r = q >> 3, ch = q & 7;
    const half8 v = *reinterpret_cast<const half8 *>(in + base + static_cast<size_t>(r0 + r) * C + c0 + ch * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) tile[r][ch * 8 + j] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int q = threadIdx.x + it * 256;
    const int c = q >> 3, ch = q & 7;
    half8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = tile[ch * 8 + j][c];
    *reinterpret_cast<half8 *>(out + base + static_cast<size_t>(c0 + c) * R + r0 + ch * 8) = v;
  }
}

// out_t[c][64 * b + i] = in[rows[row0_b + i]][c] for i < cnt_b, else 0; one
// workgroup per (64-row block b, 64-column tile).  partial[b][c] (optional) =
// sum over the block's rows of column c, in row order, fp32.
// kGelu: the rows are gradients of gelu(pre) (same layout, no row index): they are multiplied by
// gelu'(pre), written back in place, and what is transposed and summed is the product.
// kT false: nothing is transposed; the (gathered) rows go to out_t as a row-major [rows, C] matrix in sorted
// row order (out_t NULL: nowhere), and the pass is a row gather and / or the partial sums.
template <bool kGelu, bool kT>
__global__ void __launch_bounds__(256)
transpose_rows_kernel(half_t *in, const int32_t *__restrict__ rows,
                      const int32_t *__restrict__ blk_row0, const int32_t *__restrict__ blk_cnt,
                      int C, int ld_t, half_t *__restrict__ out_t, float *__restrict__ partial,
                      const half_t *__restrict__ pre) {
  __shared__ half_t tile[kTile][kTile + 8];
  const int b = blockIdx.x, c0 = blockIdx.y * kTile;
  const int cnt = blk_cnt[b];
  if (cnt < 0) return;                              // past the last expert's range: never read
  const int row0 = blk_row0[b];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int q = threadIdx.x + it * 256;
    const int i = q >> 3, ch = q & 7;
    half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (i < cnt) {
      const size_t r = (!kGelu && rows) ? static_cast<size_t>(rows[row0 + i]) : static_cast<size_t>(row0 + i);
      v = *reinterpret_cast<const half8 *>(in + r * C + c0 + ch * 8);
      if constexpr (kGelu) {
        const half8 p = *reinterpret_cast<const half8 *>(pre + r * C + c0 + ch * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          v[j] = static_cast<half_t>(static_cast<float>(v[j]) * gelu_erf_grad(static_cast<float>(p[j])));
        *reinterpret_cast<half8 *>(in + r * C + c0 + ch * 8) = v;
      }
      if constexpr (!kT) {
        if (out_t) *reinterpret_cast<half8 *>(out_t + static_cast<size_t>(row0 + i) * C + c0 + ch * 8) = v;
      }
    }
    if (kT || partial) {
#pragma unroll
      for (int j = 0; j < 8; ++j) tile[i][ch * 8 + j] = v[j];
    }
  }
  __syncthreads();
  if constexpr (kT) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int q = threadIdx.x + it * 256;
      const int c = q >> 3, ch = q & 7;
      half8 v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = tile[ch * 8 + j][c];
      *reinterpret_cast<half8 *>(out_t + static_cast<size_t>(c0 + c) * ld_t + static_cast<size_t>(b) * kTile + ch * 8) = v;
    }
  }
  if (partial && threadIdx.x < kTile) {
    float s = 0.0f;
    for (int i = 0; i < kTile; ++i) s += static_cast<float>(tile[i][threadIdx.x]);
    partial[static_cast<size_t>(b) * C + c0 + threadIdx.x] = s;
  }
}

// grad_bias[e][c] = sum of partial[b][c] over expert e's blocks, in block order.
__global__ void __launch_bounds__(256)
bias_reduce_kernel(const float *__restrict__ partial, const int32_t *__restrict__ k_seg, int C,
                   half_t *__restrict__ grad_bias) {
  const int e = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int b0 = k_seg[e] / kTile, b1 = k_seg[e + 1] / kTile;
  float s = 0.0f;
  for (int b = b0; b < b1; ++b) s += partial[static_cast<size_t>(b) * C + c];
  grad_bias[static_cast<size_t>(e) * C + c] = static_cast<half_t>(s);
}

// Backward of the gate-weighted combine, one wavefront per flat slot i = t*k + s:
// grad_y_flat[i, :] = score[i] * grad_out[t, :], grad_score[i] = <grad_out[t, :], y_flat[i, :]>;
// both zero for dropped slots.
__global__ void __launch_bounds__(256)
combine_backward_kernel(const half_t *__restrict__ grad_out, const half_t *__restrict__ y_flat,
                        const half_t *__restrict__ score, const int32_t *__restrict__ inv_pos,
                        int n_flat, int top_k, int chunks_per_row, half_t *__restrict__ grad_y_flat,
                        half_t *__restrict__ grad_score) {
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= n_flat) return;
  const size_t t = static_cast<size_t>(i) / top_k;
  const bool kept = !inv_pos || inv_pos[i] >= 0;
  const float g = kept ? static_cast<float>(score[i]) : 0.0f;
  const half8 *go = reinterpret_cast<const half8 *>(grad_out) + t * chunks_per_row;
  const half8 *y = reinterpret_cast<const half8 *>(y_flat) + static_cast<size_t>(i) * chunks_per_row;
  half8 *gy = reinterpret_cast<half8 *>(grad_y_flat) + static_cast<size_t>(i) * chunks_per_row;
  float dot = 0.0f;
  for (int c = lane; c < chunks_per_row; c += 64) {
    const half8 a = go[c];
    half8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = static_cast<half_t>(g * static_cast<float>(a[j]));
    gy[c] = o;
    if (kept) {
      const half8 v = y[c];
#pragma unroll
      for (int j = 0; j < 8; ++j) dot += static_cast<float>(a[j]) * static_cast<float>(v[j]);
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
  if (lane == 0) grad_score[i] = static_cast<half_t>(dot);
}

// dst[0 .. n) = 0, 16 bytes per lane (n a multiple of 8 halves, dst 16-byte aligned)
__global__ void __launch_bounds__(256)
zero_kernel(half_t *__restrict__ dst, size_t chunks) {
  const half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  for (size_t c = blockIdx.x * 256ull + threadIdx.x; c < chunks; c += static_cast<size_t>(gridDim.x) * 256)
    reinterpret_cast<half8 *>(dst)[c] = z;
}

}  // namespace

// A fill kernel rather than a memset node: the call may sit inside a captured graph.
int launch_zero(half_t *dst, size_t halves, hipStream_t stream) {
  if (halves == 0) return CCF_OK;
  const size_t chunks = halves / 8;
  const size_t blocks = (chunks + 255) / 256;
  hipLaunchKernelGGL(zero_kernel, dim3(static_cast<unsigned>(blocks < 4096 ? (blocks ? blocks : 1) : 4096)), dim3(256),
                     0, stream, dst, chunks);
  return check_launch("zero_kernel");
}

int padded_rows(int max_rows, int E) {
  return static_cast<int>(round_up(static_cast<size_t>(max_rows) + static_cast<size_t>(kPadK) * E, kTile));
}

int launch_kseg(const int32_t *offsets, int E, int max_rows, int seg_rows, int n_blk, int32_t *k_seg,
                int32_t *row_off, int32_t *blk_row0, int32_t *blk_cnt, int32_t *row_lo, half_t *zero_row,
                const PlanReq *rows_plan, const PlanReq *w_plan, hipStream_t stream) {
  // a wavefront per expert at least, 4 to 8 workgroups: wavefronts beyond the experts share their entries
  const int per_plan = (E + 15) / 16 > 8 ? 8 : ((E + 15) / 16 < 4 ? 4 : (E + 15) / 16);
  const int na = rows_plan ? per_plan : 0, nb = w_plan ? per_plan : 0;
  const PlanReq none{};
  hipLaunchKernelGGL(kseg_kernel, dim3(1 + na + nb), dim3(1024), 0, stream, offsets, E, max_rows, seg_rows,
                     n_blk, k_seg, row_off, blk_row0, blk_cnt, row_lo, zero_row, rows_plan ? *rows_plan : none, na,
                     w_plan ? *w_plan : none, nb);
  return check_launch("kseg_kernel");
}

int launch_transpose_weights(const half_t *in, half_t *out, int E, int R, int C, hipStream_t stream) {
  hipLaunchKernelGGL(transpose_weights_kernel, dim3(R / kTile, C / kTile, E), dim3(256), 0, stream,
                     in, out, R, C);
  return check_launch("transpose_weights_kernel");
}

int launch_transpose_rows(const half_t *in, const int32_t *rows, const int32_t *blk_row0,
                          const int32_t *blk_cnt, int n_blk, int C, int ld_t, half_t *out_t,
                          float *partial, hipStream_t stream, const half_t *gelu_pre_inplace, bool transposed) {
  half_t *src = const_cast<half_t *>(in);             // written only in the GELU form
  const dim3 grid(n_blk, C / kTile);
  const half_t *none = nullptr;
  if (gelu_pre_inplace && transposed)
    hipLaunchKernelGGL((transpose_rows_kernel<true, true>), grid, dim3(256), 0, stream, src, rows, blk_row0, blk_cnt, C, ld_t,
                       out_t, partial, gelu_pre_inplace);
  else if (gelu_pre_inplace)
    hipLaunchKernelGGL((transpose_rows_kernel<true, false>), grid, dim3(256), 0, stream, src, rows, blk_row0, blk_cnt, C, ld_t,
                       out_t, partial, gelu_pre_inplace);
  else if (transposed)
    hipLaunchKernelGGL((transpose_rows_kernel<false, true>), grid, dim3(256), 0, stream, src, rows, blk_row0, blk_cnt, C, ld_t,
                       out_t, partial, none);
  else
    hipLaunchKernelGGL((transpose_rows_kernel<false, false>), grid, dim3(256), 0, stream, src, rows, blk_row0, blk_cnt, C, ld_t,
                       out_t, partial, none);
  return check_launch("transpose_rows_kernel");
}

int launch_bias_reduce(const float *partial, const int32_t *k_seg, int E, int C, half_t *grad_bias,
                       hipStream_t stream) {
  hipLaunchKernelGGL(bias_reduce_kernel, dim3(E, (C + 255) / 256), dim3(256), 0, stream, partial,
                     k_seg, C, grad_bias);
  return check_launch("bias_reduce_kernel");
}

}  // namespace ccf

extern "C" int ccf_combine_backward(const void *grad_out, const void *y_flat, const void *score,
                                    const int32_t *inv_pos, int tokens, int top_k, int hidden,
                                    void *grad_y_flat, void *grad_score, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(grad_out && y_flat && score && grad_y_flat && grad_score, CCF_ERR_ARG,
              "combine_backward: null pointer");
  CCF_REQUIRE(tokens >= 0 && hidden > 0 && top_k >= 1, CCF_ERR_ARG, "combine_backward: bad size");
  CCF_REQUIRE(hidden % 8 == 0, CCF_ERR_SHAPE, "combine_backward: hidden=%d is not a multiple of 8", hidden);
  CCF_REQUIRE(aligned16(grad_out) && aligned16(y_flat) && aligned16(grad_y_flat), CCF_ERR_ARG,
              "combine_backward: rows must be 16-byte aligned");
  const long long n_flat = static_cast<long long>(tokens) * top_k;
  CCF_REQUIRE(n_flat < (1ll << 31), CCF_ERR_SHAPE, "combine_backward: too many slots");
  if (n_flat == 0) return CCF_OK;
  hipLaunchKernelGGL(combine_backward_kernel, dim3(static_cast<unsigned>((n_flat + 3) / 4)), dim3(256), 0,
                     as_stream(stream), static_cast<const half_t *>(grad_out),
                     static_cast<const half_t *>(y_flat), static_cast<const half_t *>(score), inv_pos,
                     static_cast<int>(n_flat), top_k, hidden / 8, static_cast<half_t *>(grad_y_flat),
                     static_cast<half_t *>(grad_score));
  return check_launch("combine_backward_kernel");
}
