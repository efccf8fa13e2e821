// Expert count, offset scan and deterministic pos for gfx950.
//
// Replaces the reference's expert_count_kernel / assign_pos_kernel pair
// (mix_moe/csrc/cuda/local_exchange.cu:6-17, 37-70) and the host-side cumsum,
// .item() and planning between them (mix_moe/mix_moe/functions.py:83-105).
// The reference fills each expert's segment of pos through an atomicSub race;
// here the flat indices inside a segment ascend, which is one of the orders
// that race can produce, and everything stays on the device.
//
// Small launches over chunks of kChunk flat indices:
//   hist   per chunk, per expert counts (wavefront match + LDS integer adds)
//   scan   one workgroup: per expert running sums over chunks, capacity clamp,
//          exclusive scan over experts
//   pos    per chunk: rank of every index inside its expert = chunk base +
//          earlier wavefront passes in the chunk + lanes before it in the
//          wavefront (ballot / popcount), then the scatter of pos and friends
// Integer adds commute, so the results do not depend on scheduling.
//
// When the table of counts is small (at most kRowsMaxInts entries) there is no scan launch:
// every workgroup of the pos launch adds up the rows in front of its chunk and all rows
// itself (a few thousand integers out of L2), which is cheaper than a launch.  The rows are
// then the hist launch's, one per chunk, or, in the layer's forward call, rows the gate
// kernel left, one per gate workgroup (its selection threads hold the expert ids), and the
// routing stage is the pos launch alone.
#include "ccf_common.h"
#include "plan.h"

#include <mutex>

// Scratch of ccf_route_static: the per-chunk count table (the workspace of ccf_route) as a
// device array that lives in the library image, so that the call allocates nothing.  Every
// GPU the library runs on holds its own copy (1 MiB) until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress: kernels are given the address it returns.
constexpr int kStaticScratchInts = 1 << 18;
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];

namespace ccf {
int g_route_rows_max = 16384;   // largest table of counts (entries) that the pos launch sums itself; 0: always a scan launch
namespace {

constexpr int kThreads = 256;
constexpr int kPasses = 4;                       // indices per thread
constexpr int kChunk = kThreads * kPasses;       // flat indices per workgroup
constexpr int kSub = kPasses * (kThreads / 64);  // wavefront passes per chunk
constexpr int kMaxExpert = 1024;
constexpr int kRowsMaxInts = 32768;              // largest table of counts that the pos launch sums itself

__device__ inline uint64_t lanes_below() {
  const int lane = threadIdx.x & 63;
  return lane ? (~0ull >> (64 - lane)) : 0ull;
}

// Lanes of this wavefront that hold the same valid expert id as the caller.
__device__ inline uint64_t peers_of(int e, bool valid, int nbits) {
  uint64_t peers = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    uint64_t m = __ballot((e >> b) & 1);
    peers &= ((e >> b) & 1) ? m : ~m;
  }
  return valid ? peers : 0ull;
}

__device__ inline int load_expert(const int64_t *idx, int i, int n, int E) {
  if (i >= n) return -1;
  int64_t e = idx[i];
  return (e >= 0 && e < E) ? static_cast<int>(e) : -1;
}

__global__ void __launch_bounds__(kThreads)
hist_kernel(const int64_t *__restrict__ idx, int n, int E, int nbits,
            int32_t *__restrict__ chunk_cnt /* [nchunk][E] or NULL */,
            int32_t *__restrict__ accumulate /* [E] or NULL */) {
  extern __shared__ int s_hist[];
  for (int e = threadIdx.x; e < E; e += kThreads) s_hist[e] = 0;
  __syncthreads();
  const int base = blockIdx.x * kChunk;
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int i = base + p * kThreads + threadIdx.x;
    const int e = load_expert(idx, i, n, E);
    const uint64_t peers = peers_of(e, e >= 0, nbits);
    if (e >= 0 && (peers & lanes_below()) == 0) atomicAdd(&s_hist[e], __popcll(peers));
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kThreads) {
    if (chunk_cnt) chunk_cnt[static_cast<size_t>(blockIdx.x) * E + e] = s_hist[e];
    if (accumulate && s_hist[e]) atomicAdd(&accumulate[e], s_hist[e]);
  }
}

// One workgroup.  chunk_cnt becomes, in place, the exclusive running sum over
// chunks (the rank base of each chunk).  If cum_inout is given the segment
// starts come from it (cum[e] - total[e]) and are written back there;
// otherwise they are the exclusive scan of the kept counts.  The table is
// pulled into LDS with parallel loads first when it fits, so that the per
// expert running sum is not a chain of dependent global loads.
constexpr int kScanLdsEntries = 8192;

__global__ void __launch_bounds__(1024)
scan_kernel(int32_t *__restrict__ chunk_cnt, int nchunk, int E, int capacity,
            int32_t *__restrict__ counts, int32_t *__restrict__ offsets,
            int32_t *__restrict__ cum_inout) {
  __shared__ int s_kept[kMaxExpert];
  __shared__ int s_tab[kScanLdsEntries];
  const int entries = nchunk * E;
  const bool in_lds = entries <= kScanLdsEntries;
  if (in_lds) {
    for (int i = threadIdx.x; i < entries; i += blockDim.x) s_tab[i] = chunk_cnt[i];
    __syncthreads();
  }
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int run = 0;
    if (in_lds) {
      for (int c = 0; c < nchunk; ++c) {
        int v = s_tab[c * E + e];
        s_tab[c * E + e] = run;
        run += v;
      }
    } else {
      for (int c = 0; c < nchunk; ++c) {
        int v = chunk_cnt[static_cast<size_t>(c) * E + e];
        chunk_cnt[static_cast<size_t>(c) * E + e] = run;
        run += v;
      }
    }
    int kept = (capacity >= 0 && run > capacity) ? capacity : run;
    s_kept[e] = kept;
    if (counts) counts[e] = kept;
    if (cum_inout) {
      int start = cum_inout[e] - run;
      cum_inout[e] = start;
      offsets[e] = start;
    }
  }
  __syncthreads();
  if (in_lds)
    for (int i = threadIdx.x; i < entries; i += blockDim.x) chunk_cnt[i] = s_tab[i];
  if (!cum_inout && threadIdx.x < 64) {
    // exclusive scan over experts by one wavefront, 64 at a time
    int carry = 0;
    const int lane = threadIdx.x;
    for (int e0 = 0; e0 < E; e0 += 64) {
      int v = (e0 + lane < E) ? s_kept[e0 + lane] : 0;
      int inc = v;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        int o = __shfl_up(inc, off, 64);
        if (lane >= off) inc += o;
      }
      if (e0 + lane < E) offsets[e0 + lane] = carry + inc - v;
      carry += __shfl(inc, 63, 64);
    }
    if (lane == 0) offsets[E] = carry;
  }
}

__global__ void __launch_bounds__(kThreads)
pos_kernel(const int64_t *__restrict__ idx, int n, int E, int nbits, int top_k, int capacity,
           const int32_t *chunk_base, const int32_t *offsets,
           int64_t *__restrict__ pos, int32_t *__restrict__ src_row,
           int32_t *__restrict__ dst_row, int32_t *__restrict__ inv_pos,
           int64_t *__restrict__ idx_kept, int nchunk, int plan_wgs, PlanReq plan0, PlanReq plan1,
           const int32_t *__restrict__ rows, int nrows, int rows_per_chunk, int32_t *__restrict__ counts_out,
           int32_t *__restrict__ offsets_out) {
  extern __shared__ int s_sub[];                 // [kSub][E], then with `rows`: [E] chunk base, [E] totals, [E + 1] offsets
  const bool is_plan = static_cast<int>(blockIdx.x) >= nchunk;
  if (rows) {
    // No scan launch: rows [nrows][E] hold counts of consecutive, equally long runs of flat
    // indices, rows_per_chunk of them per chunk.  Every workgroup adds up the rows in front of
    // its chunk (its rank base) and all rows (the experts' totals, hence the offsets).
    int *s_base = s_sub + kSub * E, *s_tot = s_base + E, *s_off = s_tot + E;
    for (int e = threadIdx.x; e < E; e += kThreads) { s_base[e] = 0; s_tot[e] = 0; }
    __syncthreads();
    const int first = is_plan ? 0 : static_cast<int>(blockIdx.x) * rows_per_chunk;   // rows in front of this chunk
    if (E <= kThreads) {
      // thread t: expert t % E, rows t / E, t / E + G, ...; sums in registers, one LDS add per thread at the end
      const int G = kThreads / E, e = threadIdx.x % E, grp = threadIdx.x / E;
      if (grp < G) {
        int tot = 0, base = 0;
        const int32_t *col = rows + e;
#pragma unroll 8
        for (int g = grp; g < nrows; g += G) {
          const int v = col[static_cast<size_t>(g) * E];
          tot += v;
          base += g < first ? v : 0;
        }
        atomicAdd(&s_tot[e], tot);
        atomicAdd(&s_base[e], base);
      }
    } else {
      for (int e = threadIdx.x; e < E; e += kThreads) {
        int tot = 0, base = 0;
#pragma unroll 8
        for (int g = 0; g < nrows; ++g) {
          const int v = rows[static_cast<size_t>(g) * E + e];
          tot += v;
          base += g < first ? v : 0;
        }
        s_tot[e] = tot;
        s_base[e] = base;
      }
    }
    __syncthreads();
    if (threadIdx.x < 64) {
      // capacity clamp and exclusive scan over experts by one wavefront, 64 at a time
      int carry = 0;
      const int lane = threadIdx.x;
      for (int e0 = 0; e0 < E; e0 += 64) {
        int v = 0;
        if (e0 + lane < E) {
          v = s_tot[e0 + lane];
          v = (capacity >= 0 && v > capacity) ? capacity : v;
          if (blockIdx.x == 0 && counts_out) counts_out[e0 + lane] = v;
        }
        int inc = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          int o = __shfl_up(inc, off, 64);
          if (lane >= off) inc += o;
        }
        if (e0 + lane < E) s_off[e0 + lane] = carry + inc - v;
        carry += __shfl(inc, 63, 64);
      }
      if (lane == 0) s_off[E] = carry;
    }
    __syncthreads();
    if (blockIdx.x == 0)
      for (int e = threadIdx.x; e <= E; e += kThreads) offsets_out[e] = s_off[e];
    chunk_base = nullptr;
    offsets = s_off;
  }
  // Workgroups past the chunks build the tile plans of the GEMMs that follow: the offsets are
  // final, and the plans then cost no launch of their own.
  if (is_plan) {
    const int r = static_cast<int>(blockIdx.x) - nchunk;        // plan_wgs workgroups per plan
    build_plan(r < plan_wgs ? plan0 : plan1, offsets, E, r % plan_wgs, plan_wgs);
    return;
  }
  for (int i = threadIdx.x; i < kSub * E; i += kThreads) s_sub[i] = 0;
  __syncthreads();
  const int base = blockIdx.x * kChunk;
  const int wave = threadIdx.x >> 6;
  int my_e[kPasses];
  int my_rank[kPasses];
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int i = base + p * kThreads + threadIdx.x;
    const int e = load_expert(idx, i, n, E);
    const uint64_t peers = peers_of(e, e >= 0, nbits);
    const uint64_t below = peers & lanes_below();
    my_e[p] = e;
    my_rank[p] = __popcll(below);
    if (e >= 0 && below == 0) s_sub[(p * (kThreads / 64) + wave) * E + e] = __popcll(peers);
  }
  __syncthreads();
  // exclusive running sum over the kSub wavefront passes, per expert
  for (int e = threadIdx.x; e < E; e += kThreads) {
    int run = chunk_base ? chunk_base[static_cast<size_t>(blockIdx.x) * E + e] : s_sub[kSub * E + e];
#pragma unroll
    for (int s = 0; s < kSub; ++s) {
      int v = s_sub[s * E + e];
      s_sub[s * E + e] = run;
      run += v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int i = base + p * kThreads + threadIdx.x;
    if (i >= n) continue;
    const int e = my_e[p];
    int j = -1;
    if (e >= 0) {
      const int rank = s_sub[(p * (kThreads / 64) + wave) * E + e] + my_rank[p];
      if (capacity < 0 || rank < capacity) j = offsets[e] + rank;
      if (j >= n) j = -1;                         // inconsistent caller-given starts
    }
    if (j >= 0) {
      pos[j] = i;
      if (src_row) src_row[j] = i / top_k;
      if (dst_row) dst_row[j] = i;
    }
    if (inv_pos) inv_pos[i] = j;
    if (idx_kept) idx_kept[i] = (j >= 0) ? static_cast<int64_t>(e) : -1;
  }
}

// (start, len, expert) triples -> counts, offsets, row list grouped by expert.
// Inside an expert the rows keep the order of the triple list, then row order.
__global__ void __launch_bounds__(1024)
segments_kernel(const int32_t *__restrict__ seg_start, const int32_t *__restrict__ seg_len,
                const int32_t *__restrict__ seg_expert, int n_seg, int E, int total_rows,
                int32_t *__restrict__ counts, int32_t *__restrict__ offsets,
                int32_t *__restrict__ rows, int plan_wgs, PlanReq plan0, PlanReq plan1) {
  __shared__ int s_cnt[kMaxExpert];
  __shared__ int s_off[kMaxExpert + 1];
  // every workgroup: rows per expert (a thread per triple, integer adds in LDS), then the experts' starts
  for (int e = threadIdx.x; e < E; e += blockDim.x) s_cnt[e] = 0;
  __syncthreads();
  for (int s = threadIdx.x; s < n_seg; s += blockDim.x) {
    const int e = seg_expert[s], len = seg_len[s];
    if (e >= 0 && e < E && len > 0) atomicAdd(&s_cnt[e], len);
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    int carry = 0;
    const int lane = threadIdx.x;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int v = (e0 + lane < E) ? s_cnt[e0 + lane] : 0;
      int inc = v;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        int o = __shfl_up(inc, off, 64);
        if (lane >= off) inc += o;
      }
      if (e0 + lane < E) s_off[e0 + lane] = carry + inc - v;
      carry += __shfl(inc, 63, 64);
    }
    if (lane == 0) s_off[E] = carry;
  }
  __syncthreads();
  // workgroups past the first build the tile plans of the GEMMs that follow (the offsets are final)
  if (blockIdx.x > 0) {
    const int r = static_cast<int>(blockIdx.x) - 1;
    build_plan(r < plan_wgs ? plan0 : plan1, s_off, E, r % plan_wgs, plan_wgs);
    return;
  }
  for (int e = threadIdx.x; e <= E; e += blockDim.x) {
    offsets[e] = s_off[e];
    if (e < E) counts[e] = s_cnt[e];
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nwave = blockDim.x >> 6;
  for (int s = wave; s < n_seg; s += nwave) {
    const int e = seg_expert[s];
    const int len = seg_len[s], st = seg_start[s];
    if (e < 0 || e >= E || len <= 0) continue;     // uniform per wavefront
    int before = 0;                                // rows of earlier triples of this expert
    for (int q = lane; q < s; q += 64)
      if (seg_expert[q] == e && seg_len[q] > 0) before += seg_len[q];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) before += __shfl_xor(before, off, 64);
    const int dst = s_off[e] + before;
    for (int r = lane; r < len; r += 64) {
      int row = st + r;                            // keep malformed triples inside the buffer
      row = row < 0 ? 0 : (row >= total_rows ? total_rows - 1 : row);
      if (dst + r < total_rows) rows[dst + r] = row;
    }
  }
}

int ceil_log2(int v) {
  int b = 0;
  while ((1 << b) < v) ++b;
  return b;
}

size_t route_ws_bytes(int n_flat, int E) {
  int nchunk = (n_flat + kChunk - 1) / kChunk;
  if (nchunk < 1) nchunk = 1;
  size_t ints = static_cast<size_t>(nchunk) * E;
  ints = ints < kRowsMaxInts ? kRowsMaxInts : ints;   // room for the gate's rows (finer than chunks) when the table is small
  return round_up(sizeof(int32_t) * ints, 256);
}

// gate_rows: the table of counts is already in the workspace, one row per gate_row_len flat indices
// (left there by the gate kernel); 0: the hist launch makes it, one row per chunk.
int route_impl(const int64_t *gate_idx, int n_flat, int E, int top_k, int capacity,
               int32_t *counts, int32_t *offsets, int32_t *cum_inout, int64_t *pos,
               int32_t *src_row, int32_t *dst_row, int32_t *inv_pos, int64_t *idx_kept,
               void *ws, size_t ws_bytes, hipStream_t stream, const PlanReq *plans = nullptr,
               int n_plans = 0, int gate_row_len = 0) {
  CCF_REQUIRE(gate_idx && pos, CCF_ERR_ARG, "route: null pointer");
  CCF_REQUIRE(n_plans >= 0 && n_plans <= 2 && (n_plans == 0 || plans), CCF_ERR_ARG, "route: bad plan requests");
  CCF_REQUIRE(n_flat >= 0 && E > 0 && top_k >= 1, CCF_ERR_ARG, "route: bad size");
  CCF_REQUIRE(E <= kMaxExpert, CCF_ERR_SHAPE, "route: num_expert=%d exceeds %d", E, kMaxExpert);
  CCF_REQUIRE(ws && ws_bytes >= route_ws_bytes(n_flat, E), CCF_ERR_WORKSPACE,
              "route: workspace of %zu bytes needed, %zu given", route_ws_bytes(n_flat, E), ws_bytes);
  const int nchunk = n_flat > 0 ? (n_flat + kChunk - 1) / kChunk : 1;
  const int nbits = ceil_log2(E);
  int32_t *chunk_cnt = static_cast<int32_t *>(ws);
  // the table of counts: the gate's rows, or one row per chunk from the hist launch
  int nrows = nchunk, rows_per_chunk = 1;
  if (gate_row_len > 0) {
    CCF_REQUIRE(kChunk % gate_row_len == 0 && !cum_inout, CCF_ERR_ARG, "route: rows of %d indices do not tile a chunk", gate_row_len);
    nrows = (n_flat + gate_row_len - 1) / gate_row_len;
    rows_per_chunk = kChunk / gate_row_len;
    CCF_REQUIRE(static_cast<long long>(nrows) * E <= kRowsMaxInts, CCF_ERR_ARG, "route: table of counts too large");
  } else {
    hipLaunchKernelGGL(hist_kernel, dim3(nchunk), dim3(kThreads), sizeof(int) * E, stream, gate_idx,
                       n_flat, E, nbits, chunk_cnt, static_cast<int32_t *>(nullptr));
    if (int rc = check_launch("hist_kernel")) return rc;
  }
  // small table: the pos launch sums the rows itself; otherwise (or with caller-given segment ends) a scan launch
  const bool sum_rows = !cum_inout && (gate_row_len > 0 || static_cast<long long>(nrows) * E <= g_route_rows_max);
  if (!sum_rows) {
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, stream, chunk_cnt, nchunk, E, capacity,
                       counts, offsets, cum_inout);
    if (int rc = check_launch("scan_kernel")) return rc;
  }
  const PlanReq none{0, 0, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0};
  const size_t pos_lds = sizeof(int) * (static_cast<size_t>(kSub + (sum_rows ? 3 : 0)) * E + 1);
  if (pos_lds > 32768) {
    // with the plan builder's static arrays the kernel passes 64 KB of LDS for many experts
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(pos_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(pos_lds));
    if (e != hipSuccess) return fail(CCF_ERR_HIP, "route: LDS attribute: %s", hipGetErrorString(e));
  }
  // a plan is built by 8 workgroups of kThreads: a wavefront per expert at least, and the wavefronts beyond
  // that share the experts' entries
  const int plan_wgs = 8;
  hipLaunchKernelGGL(pos_kernel, dim3(nchunk + n_plans * plan_wgs), dim3(kThreads), pos_lds, stream,
                     gate_idx, n_flat, E, nbits, top_k, capacity, chunk_cnt, offsets, pos, src_row,
                     dst_row, inv_pos, idx_kept, nchunk, plan_wgs, n_plans > 0 ? plans[0] : none,
                     n_plans > 1 ? plans[1] : none, sum_rows ? chunk_cnt : static_cast<int32_t *>(nullptr), nrows,
                     rows_per_chunk, counts, offsets);
  return check_launch("pos_kernel");
}

// Block plan in the reference's wire format (AsyncExpertAssignment.divide_into_block,
// mix_moe/mix_moe/transformer.py:150-250, at world_size 1 with the identity expert
// plan): per expert the full block_size-row blocks form the "local" list and a
// shorter tail the "remote" list, both in expert order; the lists are interleaved
// l0, r0, l1, r1, ... (transformer.py:199).  Closed form of the interleave: local
// item i sits at 2i while i < nR, else at nR + i; remote item i at 2i + 1 while
// i < nL, else at nL + i.  expert_block_ids / expert_block_id_idxs are the CSR from
// expert to its blocks in plan order (transformer.py:213-219).
// One workgroup; one thread per expert for the scans, then one per block.
__global__ void __launch_bounds__(1024)
blocks_kernel(const int32_t *__restrict__ counts, int E, int bs, int rank, int max_blocks,
              int32_t *__restrict__ expert_ids, int32_t *__restrict__ ranks,
              int32_t *__restrict__ lens, int32_t *__restrict__ start_addrs,
              int32_t *__restrict__ expert_block_ids, int32_t *__restrict__ expert_block_id_idxs,
              int32_t *__restrict__ block_nums) {
  __shared__ int s_start[kMaxExpert + 1], s_full[kMaxExpert + 1], s_tail[kMaxExpert + 1];
  const int t = threadIdx.x;
  const int c = t < E ? counts[t] : 0;
  // inclusive scans of rows, full blocks and tails, shifted by one entry
  if (t == 0) s_start[0] = s_full[0] = s_tail[0] = 0;
  s_start[t + 1] = c;
  s_full[t + 1] = c / bs;
  s_tail[t + 1] = (c % bs) != 0;
  __syncthreads();
  for (int d = 1; d < kMaxExpert; d <<= 1) {
    int a = 0, b = 0, g = 0;
    if (t + 1 > d) {
      a = s_start[t + 1 - d];
      b = s_full[t + 1 - d];
      g = s_tail[t + 1 - d];
    }
    __syncthreads();
    s_start[t + 1] += a;
    s_full[t + 1] += b;
    s_tail[t + 1] += g;
    __syncthreads();
  }
  const int nL = s_full[E], nR = s_tail[E];
  auto pos_local = [&](int i) { return i < nR ? 2 * i : nR + i; };
  auto pos_remote = [&](int i) { return i < nL ? 2 * i + 1 : nL + i; };
  if (t == 0) {
    block_nums[0] = nL + nR;
    block_nums[1] = nR;
    expert_block_id_idxs[E] = nL + nR;
  }
  if (t < E) expert_block_id_idxs[t] = s_full[t] + s_tail[t];
  // full blocks
  for (int i = t; i < nL; i += 1024) {
    int lo = 0, hi = E;                     // expert e with s_full[e] <= i < s_full[e + 1]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_full[mid] <= i) lo = mid; else hi = mid;
    }
    const int e = lo, b = i - s_full[e], p = pos_local(i);
    const bool has_tail = s_tail[e + 1] != s_tail[e];
    const int before = (has_tail && pos_remote(s_tail[e]) < p) ? 1 : 0;
    if (p < max_blocks) {
      expert_ids[p] = e;
      ranks[p] = rank;
      lens[p] = bs;
      start_addrs[p] = s_start[e] + b * bs;
    }
    const int slot = s_full[e] + s_tail[e] + b + before;
    if (slot < max_blocks) expert_block_ids[slot] = p;
  }
  // tails
  if (t < E && (c % bs) != 0) {
    const int e = t, p = pos_remote(s_tail[e]), nfull = c / bs;
    int lo = 0, hi = nfull;                 // full blocks of e planned before the tail
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (pos_local(s_full[e] + mid) < p) lo = mid + 1; else hi = mid;
    }
    if (p < max_blocks) {
      expert_ids[p] = e;
      ranks[p] = rank;
      lens[p] = c % bs;
      start_addrs[p] = s_start[e] + nfull * bs;
    }
    const int slot = s_full[e] + s_tail[e] + lo;
    if (slot < max_blocks) expert_block_ids[slot] = p;
  }
}

}  // namespace
}  // namespace ccf

extern "C" size_t ccf_route_workspace_bytes(int n_flat, int num_expert) {
  if (n_flat < 0 || num_expert <= 0) return 0;
  // chunk counts + room for the offsets ccf_assign_pos keeps internally
  return ccf::route_ws_bytes(n_flat, num_expert) +
         ccf::round_up(sizeof(int32_t) * (static_cast<size_t>(num_expert) + 1), 256);
}

extern "C" int ccf_expert_count(const int64_t *gate_idx, int n_flat, int32_t *expert_count,
                                int num_expert, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(gate_idx && expert_count, CCF_ERR_ARG, "expert_count: null pointer");
  CCF_REQUIRE(n_flat >= 0 && num_expert > 0, CCF_ERR_ARG, "expert_count: bad size");
  CCF_REQUIRE(num_expert <= kMaxExpert, CCF_ERR_SHAPE, "expert_count: num_expert=%d exceeds %d",
              num_expert, kMaxExpert);
  if (n_flat == 0) return CCF_OK;
  const int nchunk = (n_flat + kChunk - 1) / kChunk;
  hipLaunchKernelGGL(hist_kernel, dim3(nchunk), dim3(kThreads), sizeof(int) * num_expert,
                     as_stream(stream), gate_idx, n_flat, num_expert, ceil_log2(num_expert),
                     static_cast<int32_t *>(nullptr), expert_count);
  return check_launch("hist_kernel");
}

extern "C" int ccf_assign_pos(int32_t *cum_count, const int64_t *gate_idx, int n_flat,
                              int num_expert, int64_t *pos, void *workspace,
                              size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(cum_count, CCF_ERR_ARG, "assign_pos: null cum_count");
  CCF_REQUIRE(workspace && workspace_bytes >= ccf_route_workspace_bytes(n_flat, num_expert),
              CCF_ERR_WORKSPACE, "assign_pos: workspace of %zu bytes needed, %zu given",
              ccf_route_workspace_bytes(n_flat, num_expert), workspace_bytes);
  const size_t head = route_ws_bytes(n_flat, num_expert);
  int32_t *offsets = reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + head);
  return route_impl(gate_idx, n_flat, num_expert, 1, -1, nullptr, offsets, cum_count, pos, nullptr,
                    nullptr, nullptr, nullptr, workspace, head, as_stream(stream));
}

namespace ccf {
int route_with_plans(const int64_t *gate_idx, int n_flat, int num_expert, int top_k, int capacity,
                     int32_t *counts, int32_t *offsets, int64_t *pos, int32_t *src_row, int32_t *dst_row,
                     int32_t *inv_pos, int64_t *idx_kept, void *workspace, size_t workspace_bytes,
                     hipStream_t stream, const PlanReq *plans, int n_plans, int gate_row_len) {
  CCF_REQUIRE(counts && offsets, CCF_ERR_ARG, "route: null counts/offsets");
  return route_impl(gate_idx, n_flat, num_expert, top_k, capacity, counts, offsets, nullptr, pos, src_row,
                    dst_row, inv_pos, idx_kept, workspace, workspace_bytes, stream, plans, n_plans, gate_row_len);
}
long long route_rows_max_ints() { return g_route_rows_max < kRowsMaxInts ? g_route_rows_max : kRowsMaxInts; }
}  // namespace ccf

extern "C" int ccf_route(const int64_t *gate_idx, int n_flat, int num_expert, int top_k,
                         int capacity, int32_t *counts, int32_t *offsets, int64_t *pos,
                         int32_t *src_row, int32_t *dst_row, int32_t *inv_pos, int64_t *idx_kept,
                         void *workspace, size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(counts && offsets, CCF_ERR_ARG, "route: null counts/offsets");
  return route_impl(gate_idx, n_flat, num_expert, top_k, capacity, counts, offsets, nullptr, pos,
                    src_row, dst_row, inv_pos, idx_kept, workspace, workspace_bytes,
                    as_stream(stream));
}

namespace ccf {
namespace {
constexpr int kMaxDevices = 64;
int32_t *g_scratch_ptr[kMaxDevices] = {nullptr};   // device address of `scratch`, per device
std::mutex g_scratch_mu;

// Device address of this device's copy of `scratch`, looked up once per device.
int static_scratch(int32_t **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(CCF_ERR_HIP, "route_static: hipGetDevice: %s", hipGetErrorString(e));
  CCF_REQUIRE(dev >= 0 && dev < kMaxDevices, CCF_ERR_UNSUPPORTED, "route_static: device %d outside 0..%d", dev,
              kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(CCF_ERR_HIP, "route_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<int32_t *>(p);
  }
  *out = g_scratch_ptr[dev];
  return CCF_OK;
}
}  // namespace
}  // namespace ccf

extern "C" int ccf_route_static_max_entries(void) { return kStaticScratchInts; }

extern "C" int ccf_route_static(const int64_t *gate_idx, int n_flat, int num_expert, int top_k,
                                int capacity, int32_t *counts, int32_t *offsets, int64_t *pos,
                                int32_t *src_row, int32_t *dst_row, int32_t *inv_pos,
                                int64_t *idx_kept, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(counts && offsets, CCF_ERR_ARG, "route_static: null counts/offsets");
  CCF_REQUIRE(n_flat >= 0 && num_expert > 0 && num_expert <= kMaxExpert, CCF_ERR_ARG, "route_static: bad size");
  const long long nchunk = n_flat > 0 ? (static_cast<long long>(n_flat) + kChunk - 1) / kChunk : 1;
  CCF_REQUIRE(nchunk * num_expert <= kStaticScratchInts, CCF_ERR_SHAPE,
              "route_static: ceil(n_flat / %d) * num_expert = %lld exceeds the built-in scratch of %d entries; "
              "use ccf_route with a workspace", kChunk, nchunk * num_expert, kStaticScratchInts);
  int32_t *ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // hist_kernel writes every entry of the table before scan_kernel reads it: nothing to clear
  return route_impl(gate_idx, n_flat, num_expert, top_k, capacity, counts, offsets, nullptr, pos, src_row,
                    dst_row, inv_pos, idx_kept, ws, sizeof(int32_t) * kStaticScratchInts, as_stream(stream));
}

namespace ccf {
// ccf_segments_to_rows(), whose launch also builds n_plans (0..2) tile plans from the offsets.
int segments_with_plans(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_expert, int n_seg,
                        int num_expert, int total_rows, int32_t *counts, int32_t *offsets, int32_t *rows,
                        hipStream_t stream, const PlanReq *plans, int n_plans) {
  CCF_REQUIRE(seg_start && seg_len && seg_expert && counts && offsets && rows, CCF_ERR_ARG,
              "segments_to_rows: null pointer");
  CCF_REQUIRE(n_seg >= 0 && num_expert > 0 && total_rows >= 0, CCF_ERR_ARG,
              "segments_to_rows: bad size");
  CCF_REQUIRE(num_expert <= kMaxExpert, CCF_ERR_SHAPE, "segments_to_rows: num_expert=%d exceeds %d",
              num_expert, kMaxExpert);
  CCF_REQUIRE(n_plans >= 0 && n_plans <= 2 && (n_plans == 0 || plans), CCF_ERR_ARG, "segments_to_rows: bad plan requests");
  const PlanReq none{0, 0, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0};
  const int plan_wgs = 4;                            // of 1024 threads: 64 wavefronts per plan
  hipLaunchKernelGGL(segments_kernel, dim3(1 + n_plans * plan_wgs), dim3(1024), 0, stream, seg_start, seg_len,
                     seg_expert, n_seg, num_expert, total_rows, counts, offsets, rows, plan_wgs,
                     n_plans > 0 ? plans[0] : none, n_plans > 1 ? plans[1] : none);
  return check_launch("segments_kernel");
}
}  // namespace ccf

extern "C" int ccf_segments_to_rows(const int32_t *seg_start, const int32_t *seg_len,
                                    const int32_t *seg_expert, int n_seg, int num_expert,
                                    int total_rows, int32_t *counts, int32_t *offsets,
                                    int32_t *rows, ccf_stream_t stream) {
  return ccf::segments_with_plans(seg_start, seg_len, seg_expert, n_seg, num_expert, total_rows, counts, offsets,
                                  rows, ccf::as_stream(stream), nullptr, 0);
}

extern "C" int ccf_plan_blocks(const int32_t *counts, int num_expert, int block_size, int rank,
                               int max_blocks, int32_t *expert_ids, int32_t *ranks, int32_t *lens,
                               int32_t *start_addrs, int32_t *expert_block_ids,
                               int32_t *expert_block_id_idxs, int32_t *block_nums,
                               ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(counts && expert_ids && ranks && lens && start_addrs && expert_block_ids &&
                  expert_block_id_idxs && block_nums,
              CCF_ERR_ARG, "plan_blocks: null pointer");
  CCF_REQUIRE(num_expert > 0 && block_size > 0 && max_blocks >= 0, CCF_ERR_ARG,
              "plan_blocks: bad size");
  CCF_REQUIRE(num_expert <= kMaxExpert, CCF_ERR_SHAPE, "plan_blocks: num_expert=%d exceeds %d",
              num_expert, kMaxExpert);
  hipLaunchKernelGGL(blocks_kernel, dim3(1), dim3(1024), 0, as_stream(stream), counts, num_expert,
                     block_size, rank, max_blocks, expert_ids, ranks, lens, start_addrs,
                     expert_block_ids, expert_block_id_idxs, block_nums);
  return check_launch("blocks_kernel");
}
