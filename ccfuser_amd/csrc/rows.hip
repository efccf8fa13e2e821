// Row moves and the gate-weighted combine for gfx950 (HBM-bound kernels).
//
// local_scatter / local_gather copy fp16 rows through an index, 16 bytes per
// lane, and replace the reference's memcpy_async row kernels
// (mix_moe/csrc/cuda/mix_moe_kernel.cu:18-42, 56-79).  combine replaces the
// bmm of MixMOE.forward (mix_moe/mix_moe/layers.py:550-559).
#include "ccf_common.h"

namespace ccf {
namespace {

constexpr int kThreads = 256;

// out[j, :] = in[idx[j], :] (GATHER_READ) or out[idx[j], :] = in[j, :]
template <bool kIndexOnRead>
__global__ void __launch_bounds__(kThreads)
row_move_kernel(const half_t *__restrict__ in, half_t *__restrict__ out,
                const int32_t *__restrict__ idx, int n_rows, int chunks_per_row) {
  const size_t total = static_cast<size_t>(n_rows) * chunks_per_row;
  for (size_t c = blockIdx.x * static_cast<size_t>(kThreads) + threadIdx.x; c < total;
       c += static_cast<size_t>(gridDim.x) * kThreads) {
    const int j = static_cast<int>(c / chunks_per_row);
    const int col = static_cast<int>(c % chunks_per_row);
    const size_t other = static_cast<size_t>(idx[j]);
    const size_t src = kIndexOnRead ? other : static_cast<size_t>(j);
    const size_t dst = kIndexOnRead ? static_cast<size_t>(j) : other;
    const half8 v = reinterpret_cast<const half8 *>(in)[src * chunks_per_row + col];
    reinterpret_cast<half8 *>(out)[dst * chunks_per_row + col] = v;
  }
}

template <int K>
__global__ void __launch_bounds__(kThreads)
combine_kernel(const half_t *__restrict__ y_flat, const half_t *__restrict__ score,
               const int32_t *__restrict__ inv_pos, half_t *__restrict__ out, int tokens,
               int top_k, int chunks_per_row) {
  const size_t total = static_cast<size_t>(tokens) * chunks_per_row;
  for (size_t c = blockIdx.x * static_cast<size_t>(kThreads) + threadIdx.x; c < total;
       c += static_cast<size_t>(gridDim.x) * kThreads) {
    const size_t t = c / chunks_per_row;
    const int col = static_cast<int>(c % chunks_per_row);
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
    const int kk = K > 0 ? K : top_k;
#pragma unroll
    for (int s = 0; s < (K > 0 ? K : 8); ++s) {
      if (s < kk) {
        const size_t flat = t * kk + s;
        if (!inv_pos || inv_pos[flat] >= 0) {
          const float g = static_cast<float>(score[flat]);
          const half8 v = reinterpret_cast<const half8 *>(y_flat)[flat * chunks_per_row + col];
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] += g * static_cast<float>(v[j]);
        }
      }
    }
    half8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = static_cast<half_t>(acc[j]);
    reinterpret_cast<half8 *>(out)[t * chunks_per_row + col] = o;
  }
}

int grid_for(size_t total) {
  size_t blocks = (total + kThreads - 1) / kThreads;
  const size_t cap = 256 * 16;                   // 16 workgroups per CU is plenty for a copy
  return static_cast<int>(blocks < cap ? (blocks ? blocks : 1) : cap);
}

int row_move(const void *in, void *out, const int32_t *pos, int pos_len, int hidden,
             bool index_on_read, hipStream_t stream, const char *what) {
  CCF_REQUIRE(in && out && pos, CCF_ERR_ARG, "%s: null pointer", what);
  CCF_REQUIRE(pos_len >= 0 && hidden > 0, CCF_ERR_ARG, "%s: bad size", what);
  CCF_REQUIRE(hidden % 8 == 0, CCF_ERR_SHAPE, "%s: hidden=%d is not a multiple of 8", what, hidden);
  CCF_REQUIRE(aligned16(in) && aligned16(out), CCF_ERR_ARG, "%s: rows must be 16-byte aligned", what);
  if (pos_len == 0) return CCF_OK;
  const int cpr = hidden / 8;
  const int grid = grid_for(static_cast<size_t>(pos_len) * cpr);
  if (index_on_read)
    hipLaunchKernelGGL(row_move_kernel<true>, dim3(grid), dim3(kThreads), 0, stream,
                       static_cast<const half_t *>(in), static_cast<half_t *>(out), pos, pos_len, cpr);
  else
    hipLaunchKernelGGL(row_move_kernel<false>, dim3(grid), dim3(kThreads), 0, stream,
                       static_cast<const half_t *>(in), static_cast<half_t *>(out), pos, pos_len, cpr);
  return check_launch(what);
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_local_scatter(const void *in, void *out, const int32_t *pos, int pos_len,
                                 int hidden, ccf_stream_t stream) {
  return ccf::row_move(in, out, pos, pos_len, hidden, true, ccf::as_stream(stream), "local_scatter");
}

extern "C" int ccf_local_gather(const void *in, void *out, const int32_t *pos, int pos_len,
                                int hidden, ccf_stream_t stream) {
  return ccf::row_move(in, out, pos, pos_len, hidden, false, ccf::as_stream(stream), "local_gather");
}

extern "C" int ccf_combine(const void *y_flat, const void *score, const int32_t *inv_pos, void *out,
                           int tokens, int top_k, int hidden, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(y_flat && score && out, CCF_ERR_ARG, "combine: null pointer");
  CCF_REQUIRE(tokens >= 0 && hidden > 0, CCF_ERR_ARG, "combine: bad size");
  CCF_REQUIRE(top_k >= 1 && top_k <= 8, CCF_ERR_SHAPE, "combine: top_k=%d outside 1..8", top_k);
  CCF_REQUIRE(hidden % 8 == 0, CCF_ERR_SHAPE, "combine: hidden=%d is not a multiple of 8", hidden);
  CCF_REQUIRE(aligned16(y_flat) && aligned16(out), CCF_ERR_ARG, "combine: rows must be 16-byte aligned");
  if (tokens == 0) return CCF_OK;
  const int cpr = hidden / 8;
  const int grid = grid_for(static_cast<size_t>(tokens) * cpr);
  const half_t *y = static_cast<const half_t *>(y_flat);
  const half_t *g = static_cast<const half_t *>(score);
  half_t *o = static_cast<half_t *>(out);
  hipStream_t st = as_stream(stream);
  if (top_k == 1)
    hipLaunchKernelGGL(combine_kernel<1>, dim3(grid), dim3(kThreads), 0, st, y, g, inv_pos, o, tokens, top_k, cpr);
  else if (top_k == 2)
    hipLaunchKernelGGL(combine_kernel<2>, dim3(grid), dim3(kThreads), 0, st, y, g, inv_pos, o, tokens, top_k, cpr);
  else
    hipLaunchKernelGGL(combine_kernel<0>, dim3(grid), dim3(kThreads), 0, st, y, g, inv_pos, o, tokens, top_k, cpr);
  return check_launch("combine_kernel");
}
