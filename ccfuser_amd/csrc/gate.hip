// Top-k softmax gate for gfx950.
//
// logits[t, e] = sum_k x[t, k] * wg[e, k] + bg[e], then top-k and a softmax
// over the k selected logits (reference mix_moe/mix_moe/gates/naive_gate.py:31-38).
//
// The expert choice has to be reproducible bit for bit, so the fp32 sum is
// taken in one fixed order that a CPU can replay: K is cut into parts of 128
// consecutive elements (the last may be shorter); a part's sum starts at zero
// and takes its products one at a time in ascending K, acc = fma(x, w, acc);
// the part sums are added one after the other in ascending order, starting from
// the first; the bias is added last and the logit is rounded once to the input
// dtype.  The product of two fp16 values is exact in fp32, so for fp16 inputs
// the fused multiply-add is one rounding of acc + x*w however it is computed.
//
// That chain is what a K = 1 fp32 MFMA computes per output element
// (D = fma(A, B, C), round to nearest even: checked against fmaf chains on a
// CPU), so for fp16 inputs a wavefront runs it for a whole tile of tokens x
// experts at once: v_mfma_f32_32x32x1 (two 32 x 32 blocks) for more than 16
// experts, v_mfma_f32_16x16x1 (four 16 x 16 blocks) otherwise, one instruction
// per K element.  The blocks of an instruction are independent products, so a
// block is either another group of tokens or the same tokens on another part
// of K ("slot"): few tokens still fill the machine.  fp32 inputs keep multiply
// and add separate (two roundings) and run on the vector unit.
#include "ccf_common.h"
#include "mfma_f32.h"

#include <limits.h>

namespace ccf {
int g_gate_waves = 8;    // most wavefronts of a gate workgroup (each takes other parts of K), 1..8
int g_gate_slots = 0;    // parts of K a wavefront works on at a time (1, 2, 4); 0 = by the token count
namespace {

constexpr int kMaxTopK = 8;
constexpr int kPart = 128;          // K elements of a part
constexpr int kMaxWaves = 8;

template <typename T>
__device__ inline float round_to(float v) {
  return static_cast<float>(static_cast<T>(v));
}

__device__ inline bool better(float v, int id, float bv, int bid) {
  return v > bv || (v == bv && id < bid);
}

// The k best of a token so far (k <= KS), best first; ties keep the lower expert id.
template <int KS>
struct Best {
  float v[KS];
  int id[KS];
  __device__ inline void clear() {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      v[s] = -INFINITY;
      id[s] = INT_MAX;
    }
  }
  __device__ inline void offer(float nv, int nid, int k) {
    float lv = v[0];
    int li = id[0];
#pragma unroll
    for (int s = 1; s < KS; ++s)
      if (s == k - 1) {
        lv = v[s];
        li = id[s];
      }
    if (!better(nv, nid, lv, li)) return;          // not among the k best
#pragma unroll
    for (int s = KS - 1; s >= 0; --s) {
      if (s < k) {
        const int up = s > 0 ? s - 1 : 0;
        const bool ahead = s > 0 && better(nv, nid, v[up], id[up]);
        const bool here = better(nv, nid, v[s], id[s]);
        if (ahead) {                               // belongs further up: slot s takes its upper neighbour
          v[s] = v[up];
          id[s] = id[up];
        } else if (here) {
          v[s] = nv;
          id[s] = nid;
        }
      }
    }
  }
  // softmax over the k selected logits (slot 0 holds the maximum) and the writes
  template <typename T>
  __device__ inline void write(int t, int k, int64_t *__restrict__ idx_out, T *__restrict__ score_out) const {
    float ex[KS];
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      ex[s] = (s < k) ? expf(v[s] - v[0]) : 0.0f;
      sum += ex[s];
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      if (s < k) {
        idx_out[static_cast<size_t>(t) * k + s] = static_cast<int64_t>(id[s]);
        score_out[static_cast<size_t>(t) * k + s] = static_cast<T>(ex[s] / sum);
      }
    }
  }
};


// fp16 gate.  An MFMA has 64 / N blocks; with S = 1 << LS slots, block b of a wavefront is
// token block b / S on slot b % S, so a wavefront covers TW = (64 / N / S) * N tokens and
// S parts of K at a time, and the wavefronts of a workgroup (all on the same TW tokens)
// cover waves * S parts per round.  Lane l of block b feeds row l % N of A with its
// token's x and column l % N of B with its expert's weights, zero where K, the tokens or
// the experts end (fma(0, 0, acc) = acc).
//
// A lane needs consecutive K of its own row, which is the opposite of a coalesced load, so
// the operands take the way through LDS: per stage of 32 K elements the wavefront fetches
// the 64 bytes of each of its 64 x rows and of its N*S weight rows with whole-line loads
// (four lanes per row), two stages ahead of their use, parks them in registers, and writes
// them into its own 10 KB of LDS one stage ahead; each lane then reads its row back in
// 16-byte pieces.  Only that wavefront touches the region, so the stage loop has no barrier.
//
// After a round the part sums wait in LDS (the same region) and are added in ascending part
// order onto the running sums; after the last round bias and rounding give the logits of one
// tile of N experts, of which one thread per token keeps the k best (k <= KS).
constexpr int kStageK = 32;                        // K elements of a stage
constexpr int kRowBytes = 80;                      // a row's 64 bytes of a stage + 16: bank spread
constexpr int kTileBytes = 64 * kRowBytes;         // one operand of a stage
constexpr int kRegionFloats = 2 * kTileBytes / 4;  // a wavefront's LDS: two operand tiles, later its part sums

template <int N, int LS, int KS>
__global__ void __launch_bounds__(kMaxWaves * 64)
gate_mfma_kernel(const half_t *__restrict__ x, const half_t *__restrict__ wg, const half_t *__restrict__ bg,
                 int tokens, int d, int E, int k, int64_t *__restrict__ idx_out,
                 half_t *__restrict__ score_out, half_t *__restrict__ logits_out, int32_t *__restrict__ wg_cnt) {
  using M = Mfma<N>;
  constexpr int kBlocks = 64 / N;
  constexpr int S = 1 << LS;
  static_assert(S <= kBlocks, "a slot is a block");
  constexpr int TW = (kBlocks / S) * N;            // tokens of a workgroup
  constexpr int kWLoads = N * S / 16;              // load instructions for the weight rows of a stage
  constexpr int kLd = N + 1;                       // row stride of the logit tile in LDS (bank spread)
  static_assert(64 * N * 4 <= kRegionFloats * 4, "part sums of a wavefront fit its region");
  extern __shared__ float s_mem[];
  const int waves = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  float *region = s_mem + static_cast<size_t>(wave) * kRegionFloats;
  float *s_total = s_mem + static_cast<size_t>(waves) * kRegionFloats;   // [TW][kLd] running sums, then logits
  const int t0 = blockIdx.x * TW;
  const int nparts = (d + kPart - 1) / kPart;
  const int per_round = waves * S;
  const int rounds = (nparts + per_round - 1) / per_round;

  // as a reader: my block, row, slot
  const int blk = lane / N, r = lane % N;
  const int slot = blk & (S - 1);
  char *tile = reinterpret_cast<char *>(region);
  const char *my_x = tile + lane * kRowBytes;                              // x row of lane l is row l of the tile
  const char *my_w = tile + kTileBytes + (slot * N + r) * kRowBytes;       // weight rows: slot-major

  // as a loader: four lanes per row, 16 rows per instruction
  const int l_row = lane >> 2, l_piece = lane & 3;
  char *park_at = tile + l_row * kRowBytes + l_piece * 16;
  const half_t *x_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lr = 16 * i + l_row;
    int t = t0 + ((lr / N) >> LS) * N + lr % N;
    t = t < tokens ? t : tokens - 1;               // rows past the end repeat the last token
    x_src[i] = x + static_cast<size_t>(t) * d + (((lr / N) & (S - 1)) * kPart + l_piece * 8);
  }

  Best<KS> best;
  best.clear();

  for (int e0 = 0; e0 < E; e0 += N) {              // tiles of N experts
    const bool has_w = e0 + r < E;
    // the bias of the column this thread finishes (the same for all its elements: the
    // workgroup size is a multiple of N), asked for before the long part
    float my_bias = 0.0f;
    if (bg && e0 + static_cast<int>(threadIdx.x) % N < E) my_bias = static_cast<float>(bg[e0 + threadIdx.x % N]);
    const half_t *w_src[kWLoads];
#pragma unroll
    for (int i = 0; i < kWLoads; ++i) {
      const int wr = 16 * i + l_row;
      int e = e0 + wr % N;
      e = e < E ? e : E - 1;
      w_src[i] = wg + static_cast<size_t>(e) * d + ((wr / N) * kPart + l_piece * 8);
    }
    for (int rd = 0; rd < rounds; ++rd) {
      const int part0 = rd * per_round + wave * S;               // this wavefront's first part of the round
      if (part0 < nparts) {                        // uniform per wavefront
        int left = d - part0 * kPart;                            // the wavefront's first part is its longest
        left = left < kPart ? left : kPart;
        const int stages = (left + kStageK - 1) / kStageK;       // 1..4
        const int k0 = part0 * kPart;
        const int k_mine = k0 + slot * kPart;                    // where this lane's part starts (may be past d)
        typename M::Acc acc;
#pragma unroll
        for (int v = 0; v < M::kRegs; ++v) acc[v] = 0.0f;

        // Loads of stage s: every lane loads (from the start of the tensor where K has
        // ended) and unwanted pieces become zero when they are used, so there is no branch
        // around a load and the number of loads in flight is known where the waits go.
        int4v xa[4], wa[kWLoads], xb[4], wb[kWLoads];
        auto fetch = [&](int s, int4v (&xv)[4], int4v (&wv)[kWLoads]) {
          const int ks = k0 + s * kStageK;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int kx = ks + (((16 * i + l_row) / N) & (S - 1)) * kPart + l_piece * 8;
            xv[i] = *reinterpret_cast<const int4v *>(kx < d ? x_src[i] + ks : x);
          }
#pragma unroll
          for (int i = 0; i < kWLoads; ++i) {
            const int kw = ks + ((16 * i + l_row) / N) * kPart + l_piece * 8;
            wv[i] = *reinterpret_cast<const int4v *>(kw < d ? w_src[i] + ks : wg);
          }
        };
        auto park = [&](const int4v (&xv)[4], const int4v (&wv)[kWLoads]) {
#pragma unroll
          for (int i = 0; i < 4; ++i) *reinterpret_cast<int4v *>(park_at + 16 * i * kRowBytes) = xv[i];
#pragma unroll
          for (int i = 0; i < kWLoads; ++i)
            *reinterpret_cast<int4v *>(park_at + kTileBytes + 16 * i * kRowBytes) = wv[i];
        };
        auto take = [&](int c, half8 &vx, half8 &vw) {
          vx = *reinterpret_cast<const half8 *>(my_x + c * 16);
          vw = *reinterpret_cast<const half8 *>(my_w + c * 16);
        };
        auto run = [&](int s, int c, const half8 &vx, const half8 &vw) {
          const bool in = k_mine + s * kStageK + c * 8 < d;
          const half8 zero = {};
          const half8 xs = in ? vx : zero;
          const half8 ws = (in && has_w) ? vw : zero;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            acc = M::run(static_cast<float>(xs[j]), static_cast<float>(ws[j]), acc);
        };
        // One stage: its four pieces are read back two at a time; once the last read is on
        // its way (the LDS works in order) the next stage's operands overwrite the tiles
        // and the loads of the stage after that leave.  The scheduling barriers keep loads
        // and LDS traffic where they are written: left alone, the scheduler sinks each
        // load to just before its use.
        half8 ax, aw, bx, bw;
#define CCF_GATE_STAGE(s, PARK_NEXT)                                   \
  do {                                                                 \
    take(0, ax, aw);                                                   \
    take(1, bx, bw);                                                   \
    __builtin_amdgcn_sched_barrier(0);                                 \
    run(s, 0, ax, aw);                                                 \
    __builtin_amdgcn_sched_barrier(0);                                 \
    take(2, ax, aw);                                                   \
    __builtin_amdgcn_sched_barrier(0);                                 \
    run(s, 1, bx, bw);                                                 \
    __builtin_amdgcn_sched_barrier(0);                                 \
    take(3, bx, bw);                                                   \
    __builtin_amdgcn_sched_barrier(0);                                 \
    PARK_NEXT;                                                         \
    __builtin_amdgcn_sched_barrier(0);                                 \
    run(s, 2, ax, aw);                                                 \
    run(s, 3, bx, bw);                                                 \
    __builtin_amdgcn_sched_barrier(0);                                 \
  } while (0)
        fetch(0, xa, wa);
        fetch(1, xb, wb);
        __builtin_amdgcn_sched_barrier(0);
        park(xa, wa);                              // stage 0
        fetch(2, xa, wa);
        __builtin_amdgcn_sched_barrier(0);
        CCF_GATE_STAGE(0, park(xb, wb); fetch(3, xb, wb));
        if (stages > 1) {
          CCF_GATE_STAGE(1, park(xa, wa));
          if (stages > 2) {
            CCF_GATE_STAGE(2, park(xb, wb));
            if (stages > 3) CCF_GATE_STAGE(3, (void)0);
          }
        }
#undef CCF_GATE_STAGE
        // part sums into the same region, [slot][token][expert]
#pragma unroll
        for (int v = 0; v < M::kRegs; ++v) {
          const int ob = M::block(v);
          region[(static_cast<size_t>(ob & (S - 1)) * TW + (ob >> LS) * N + M::row(v, lane)) * N + r] = acc[v];
        }
      }
      __syncthreads();
      // running sums: the parts of this round in ascending order
      for (int i = threadIdx.x; i < TW * N; i += blockDim.x) {
        const int tok = i / N, col = i % N;
        float t = rd == 0 ? 0.0f : s_total[tok * kLd + col];
        for (int q = 0; q < per_round; ++q) {
          const int p = rd * per_round + q;
          if (p >= nparts) break;
          const float ps = s_mem[static_cast<size_t>(q >> LS) * kRegionFloats + (q & (S - 1)) * TW * N + i];
          t = p == 0 ? ps : t + ps;
        }
        if (rd == rounds - 1) {
          const int e = e0 + col;
          if (e < E) {
            if (bg) t = t + my_bias;
            t = round_to<half_t>(t);
            if (logits_out && t0 + tok < tokens)
              logits_out[static_cast<size_t>(t0 + tok) * E + e] = static_cast<half_t>(t);
          }
        }
        s_total[tok * kLd + col] = t;
      }
      __syncthreads();
    }
    // one thread per token: the logits of this tile, ascending expert id
    if (threadIdx.x < TW && t0 + threadIdx.x < tokens) {
      const float *lg = s_total + threadIdx.x * kLd;
      const int ne = (E - e0) < N ? (E - e0) : N;
      for (int c = 0; c < ne; ++c) best.offer(lg[c], e0 + c, k);
    }
    // s_total is next written after the next tile's first barrier, which these threads reach later
  }
  if (threadIdx.x < TW && t0 + threadIdx.x < tokens)
    best.template write<half_t>(t0 + threadIdx.x, k, idx_out, score_out);
  if (wg_cnt) {
    // How many of this workgroup's token slots chose each expert, for the routing stage: the
    // selection threads hold the ids, so the routing needs no pass of its own over idx to count
    // them.  The wavefronts' regions are free since the last barrier.
    int *row = reinterpret_cast<int *>(s_mem);
    for (int e = threadIdx.x; e < E; e += blockDim.x) row[e] = 0;
    __syncthreads();
    if (threadIdx.x < TW && t0 + threadIdx.x < tokens) {
#pragma unroll
      for (int s = 0; s < KS; ++s)
        if (s < k) atomicAdd(&row[best.id[s]], 1);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) wg_cnt[static_cast<size_t>(blockIdx.x) * E + e] = row[e];
  }
}

// fp32 gate on the vector unit, one wavefront per token: a lane takes one (expert, part)
// pair at a time and walks the part in ascending K, multiply and add rounded separately;
// lanes then add each expert's part sums in order.  The logits of the token wait in LDS
// for the selection.
__global__ void __launch_bounds__(64)
gate_f32_kernel(const float *__restrict__ x, const float *__restrict__ wg, const float *__restrict__ bg,
                int tokens, int d, int E, int k, int group, int64_t *__restrict__ idx_out,
                float *__restrict__ score_out, float *__restrict__ logits_out) {
#pragma clang fp contract(off)
  extern __shared__ float s_mem[];
  const int lane = threadIdx.x;
  const int nparts = (d + kPart - 1) / kPart;
  float *s_logit = s_mem;                          // [E]
  float *s_part = s_mem + E;                       // [group][nparts]: `group` experts at a time
  const int t = blockIdx.x;
  const float *xrow = x + static_cast<size_t>(t) * d;
  for (int e0 = 0; e0 < E; e0 += group) {
    const int ne = (E - e0) < group ? (E - e0) : group;
    for (int q = lane; q < ne * nparts; q += kWave) {   // part fastest: neighbours read neighbouring K
      const int e = e0 + q / nparts, p = q % nparts;
      const float *wrow = wg + static_cast<size_t>(e) * d;
      const int k_end = (p + 1) * kPart < d ? (p + 1) * kPart : d;
      float acc = 0.0f;
      for (int kk = p * kPart; kk < k_end; kk += 4) {
        const float4v xv = *reinterpret_cast<const float4v *>(xrow + kk);
        const float4v wv = *reinterpret_cast<const float4v *>(wrow + kk);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float prod = xv[j] * wv[j];
          acc = acc + prod;
        }
      }
      s_part[q] = acc;
    }
    __syncthreads();
    for (int g = lane; g < ne; g += kWave) {
      float s = s_part[g * nparts];
      for (int p = 1; p < nparts; ++p) s = s + s_part[g * nparts + p];
      if (bg) s = s + bg[e0 + g];
      s_logit[e0 + g] = s;
      if (logits_out) logits_out[static_cast<size_t>(t) * E + e0 + g] = s;
    }
    __syncthreads();
  }
  if (lane == 0) {
    Best<kMaxTopK> best;
    best.clear();
    for (int e = 0; e < E; ++e) best.offer(s_logit[e], e, k);
    best.write<float>(t, k, idx_out, score_out);
  }
}

}  // namespace
}  // namespace ccf

namespace ccf {
// The gate; with wg_cnt (room for max_cnt ints) the fp16 kernel also leaves, per workgroup, how many of
// its token slots chose each expert ([workgroups][tot_expert], a workgroup covering *tokens_per_wg
// consecutive tokens), when that table fits; *tokens_per_wg = 0 says it was not written.
int gate_forward(const void *x, const void *wg, const void *bg, int tokens, int d_model, int tot_expert, int top_k,
                 int dtype, int64_t *idx_out, void *score_out, void *logits_out, ccf_stream_t stream,
                 int32_t *wg_cnt, long long max_cnt, int *tokens_per_wg) {
  if (tokens_per_wg) *tokens_per_wg = 0;
  CCF_REQUIRE(x && wg && idx_out && score_out, CCF_ERR_ARG, "gate: null pointer");
  CCF_REQUIRE(tokens >= 0 && d_model > 0 && tot_expert > 0, CCF_ERR_ARG, "gate: bad size");
  CCF_REQUIRE(d_model % 8 == 0, CCF_ERR_SHAPE, "gate: d_model=%d is not a multiple of 8", d_model);
  CCF_REQUIRE(top_k >= 1 && top_k <= kMaxTopK && top_k <= tot_expert, CCF_ERR_SHAPE,
              "gate: top_k=%d outside 1..min(%d, tot_expert=%d)", top_k, kMaxTopK, tot_expert);
  CCF_REQUIRE(tot_expert <= 1024, CCF_ERR_SHAPE, "gate: tot_expert=%d exceeds 1024", tot_expert);
  CCF_REQUIRE(dtype == CCF_F16 || dtype == CCF_F32, CCF_ERR_UNSUPPORTED, "gate: dtype %d", dtype);
  CCF_REQUIRE(aligned16(x) && aligned16(wg), CCF_ERR_ARG, "gate: x and wg must be 16-byte aligned");
  if (tokens == 0) return CCF_OK;
  const int nparts = (d_model + kPart - 1) / kPart;
  if (dtype == CCF_F32) {
    // part sums of as many experts at a time as 32 KB hold
    int group = 8192 / nparts;
    group = group < 1 ? 1 : (group > tot_expert ? tot_expert : group);
    const size_t lds = sizeof(float) * (static_cast<size_t>(tot_expert) + static_cast<size_t>(group) * nparts);
    CCF_REQUIRE(lds <= 64 * 1024, CCF_ERR_SHAPE, "gate: fp32 d_model=%d needs %zu bytes of LDS", d_model, lds);
    hipLaunchKernelGGL(gate_f32_kernel, dim3(tokens), dim3(64), lds, as_stream(stream),
                       static_cast<const float *>(x), static_cast<const float *>(wg),
                       static_cast<const float *>(bg), tokens, d_model, tot_expert, top_k, group, idx_out,
                       static_cast<float *>(score_out), static_cast<float *>(logits_out));
    return check_launch("gate_f32_kernel");
  }
  // Tile and slots.  With S slots a wavefront covers 64 / S tokens, so S grows while there
  // are fewer than four workgroups per CU and K has parts for the slots.
  const int n = tot_expert > 16 ? 32 : 16;
  const int blocks_per_mfma = 64 / n;
  int ls = 0;
  if (g_gate_slots) {
    while ((2 << ls) <= g_gate_slots && (2 << ls) <= blocks_per_mfma) ++ls;
  } else {
    while ((2 << ls) <= blocks_per_mfma && (2 << ls) <= nparts &&
           (tokens + (64 >> ls) - 1) / (64 >> ls) < 1024)
      ++ls;
  }
  const int slots = 1 << ls;
  const int tw = 64 >> ls;
  int waves = (nparts + slots - 1) / slots;
  int cap = g_gate_waves < kMaxWaves ? g_gate_waves : kMaxWaves;
  cap = cap < 1 ? 1 : cap;
  waves = waves < cap ? waves : cap;
  const size_t lds = sizeof(float) * (static_cast<size_t>(waves) * kRegionFloats + static_cast<size_t>(tw) * (n + 1));
  CCF_REQUIRE(lds <= 160 * 1024, CCF_ERR_SHAPE, "gate: %zu bytes of LDS needed", lds);
  dim3 grid((tokens + tw - 1) / tw), block(waves * 64);
  if (wg_cnt && static_cast<long long>(grid.x) * tot_expert <= max_cnt) {
    if (tokens_per_wg) *tokens_per_wg = tw;
  } else {
    wg_cnt = nullptr;
  }
#define CCF_GATE_LAUNCH(NN, LSV, KSV)                                                              \
  do {                                                                                             \
    auto kern = gate_mfma_kernel<NN, LSV, KSV>;                                                    \
    if (lds > 65536) {                                                                             \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize,               \
                                         static_cast<int>(lds));                                   \
      if (e != hipSuccess) return fail(CCF_ERR_HIP, "gate: LDS attribute: %s", hipGetErrorString(e)); \
    }                                                                                              \
    hipLaunchKernelGGL(kern, grid, block, lds, as_stream(stream), static_cast<const half_t *>(x),  \
                       static_cast<const half_t *>(wg), static_cast<const half_t *>(bg), tokens,   \
                       d_model, tot_expert, top_k, idx_out, static_cast<half_t *>(score_out),      \
                       static_cast<half_t *>(logits_out), wg_cnt);                                 \
  } while (0)
#define CCF_GATE_K(NN, LSV)                                                  \
  do {                                                                       \
    if (top_k <= 2) CCF_GATE_LAUNCH(NN, LSV, 2); else CCF_GATE_LAUNCH(NN, LSV, kMaxTopK); \
  } while (0)
  if (n == 32) {
    if (ls == 0) CCF_GATE_K(32, 0); else CCF_GATE_K(32, 1);
  } else {
    if (ls == 0) CCF_GATE_K(16, 0); else if (ls == 1) CCF_GATE_K(16, 1); else CCF_GATE_K(16, 2);
  }
#undef CCF_GATE_K
#undef CCF_GATE_LAUNCH
  return check_launch("gate_mfma_kernel");
}
}  // namespace ccf

namespace ccf {
namespace {

// ---- backward of the softmax over the selected logits and of the selection --------------
// A workgroup takes kGbTokens tokens: thread t computes the k values of its token,
//   g_j = s_j (grad_j - sum_i s_i grad_i)    (fp32),
// the workgroup zero-fills its rows of grad_logits and, behind a barrier, every thread stores its
// k values at their experts' columns.  The bias gradient is the column sum of the unrounded
// values: wavefront w sums experts w, w + 4, ... over the workgroup's tokens (lane l takes
// entries l, l + 64, ... in order, then a fixed tree over the lanes), so the result does not
// depend on scheduling; gate_bias_reduce_kernel adds the workgroups' sums in order.
constexpr int kGbTokens = 256;

__global__ void __launch_bounds__(kGbTokens)
gate_backward_kernel(const half_t *__restrict__ score, const half_t *__restrict__ grad_score,
                     const int64_t *__restrict__ idx, int tokens, int top_k, int E,
                     half_t *__restrict__ grad_logits, float *__restrict__ partial) {
  __shared__ float s_val[kGbTokens * kMaxTopK];
  __shared__ int s_idx[kGbTokens * kMaxTopK];
  const int t = threadIdx.x;
  const int tok0 = blockIdx.x * kGbTokens;
  const int tok = tok0 + t;
  float g[kMaxTopK];
  int ex[kMaxTopK];
  if (tok < tokens) {
    float s[kMaxTopK], dot = 0.0f;
    for (int j = 0; j < top_k; ++j) {
      s[j] = static_cast<float>(score[static_cast<size_t>(tok) * top_k + j]);
      g[j] = static_cast<float>(grad_score[static_cast<size_t>(tok) * top_k + j]);
      dot = fmaf(s[j], g[j], dot);
    }
    for (int j = 0; j < top_k; ++j) {
      g[j] = s[j] * (g[j] - dot);
      const int64_t e = idx[static_cast<size_t>(tok) * top_k + j];
      ex[j] = (e >= 0 && e < E) ? static_cast<int>(e) : -1;
    }
  } else {
    for (int j = 0; j < top_k; ++j) {
      g[j] = 0.0f;
      ex[j] = -1;
    }
  }
  for (int j = 0; j < top_k; ++j) {
    s_val[t * top_k + j] = g[j];
    s_idx[t * top_k + j] = ex[j];
  }
  // this workgroup's rows of grad_logits are one contiguous range
  const int n_tok = tokens - tok0 < kGbTokens ? tokens - tok0 : kGbTokens;
  half_t *rows = grad_logits + static_cast<size_t>(tok0) * E;
  const size_t n_el = static_cast<size_t>(n_tok) * E;
  for (size_t i = t; i < n_el; i += kGbTokens) rows[i] = static_cast<half_t>(0.0f);
  __syncthreads();                                  // the zeros are written (and s_val, s_idx)
  if (tok < tokens) {
    for (int j = 0; j < top_k; ++j)
      if (ex[j] >= 0) rows[static_cast<size_t>(t) * E + ex[j]] = static_cast<half_t>(g[j]);
  }
  if (!partial) return;
  const int lane = t & 63, wave = t >> 6;
  const int n_ent = kGbTokens * top_k;
  for (int e = wave; e < E; e += kGbTokens / 64) {
    float acc = 0.0f;
    for (int i = lane; i < n_ent; i += 64) acc += s_idx[i] == e ? s_val[i] : 0.0f;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) partial[static_cast<size_t>(blockIdx.x) * E + e] = acc;
  }
}

__global__ void __launch_bounds__(256)
gate_bias_reduce_kernel(const float *__restrict__ partial, int n_wg, int E, half_t *__restrict__ grad_bias) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= E) return;
  float acc = 0.0f;
  for (int w = 0; w < n_wg; ++w) acc += partial[static_cast<size_t>(w) * E + e];
  grad_bias[e] = static_cast<half_t>(acc);
}

}  // namespace
}  // namespace ccf

extern "C" size_t ccf_gate_backward_workspace_bytes(int tokens, int tot_expert) {
  if (tokens <= 0 || tot_expert <= 0) return 0;
  return sizeof(float) * static_cast<size_t>((tokens + ccf::kGbTokens - 1) / ccf::kGbTokens) * tot_expert;
}

extern "C" int ccf_gate_backward(const void *score, const void *grad_score, const int64_t *idx, int tokens,
                                 int top_k, int tot_expert, void *grad_logits, void *grad_bias, void *workspace,
                                 size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(tokens >= 0 && tot_expert > 0 && tot_expert <= 1024, CCF_ERR_ARG, "gate_backward: bad size");
  CCF_REQUIRE(top_k >= 1 && top_k <= kMaxTopK && top_k <= tot_expert, CCF_ERR_SHAPE,
              "gate_backward: top_k=%d outside 1..min(%d, tot_expert=%d)", top_k, kMaxTopK, tot_expert);
  if (tokens == 0) {                                 // no rows to write; a sum over nothing
    if (!grad_bias) return CCF_OK;
    hipLaunchKernelGGL(gate_bias_reduce_kernel, dim3((tot_expert + 255) / 256), dim3(256), 0, as_stream(stream),
                       static_cast<const float *>(nullptr), 0, tot_expert, static_cast<half_t *>(grad_bias));
    return check_launch("gate_bias_reduce_kernel");
  }
  CCF_REQUIRE(score && grad_score && idx && grad_logits, CCF_ERR_ARG, "gate_backward: null pointer");
  const size_t need = ccf_gate_backward_workspace_bytes(tokens, tot_expert);
  CCF_REQUIRE(!grad_bias || (workspace && workspace_bytes >= need), CCF_ERR_WORKSPACE,
              "gate_backward: workspace of %zu bytes needed for the bias gradient, %zu given", need, workspace_bytes);
  const int n_wg = (tokens + kGbTokens - 1) / kGbTokens;
  hipLaunchKernelGGL(gate_backward_kernel, dim3(n_wg), dim3(kGbTokens), 0, as_stream(stream),
                     static_cast<const half_t *>(score), static_cast<const half_t *>(grad_score), idx, tokens, top_k,
                     tot_expert, static_cast<half_t *>(grad_logits), grad_bias ? static_cast<float *>(workspace) : nullptr);
  if (int rc = check_launch("gate_backward_kernel")) return rc;
  if (grad_bias) {
    hipLaunchKernelGGL(gate_bias_reduce_kernel, dim3((tot_expert + 255) / 256), dim3(256), 0, as_stream(stream),
                       static_cast<const float *>(workspace), n_wg, tot_expert, static_cast<half_t *>(grad_bias));
    return check_launch("gate_bias_reduce_kernel");
  }
  return CCF_OK;
}

extern "C" int ccf_gate_topk_softmax(const void *x, const void *wg, const void *bg, int tokens,
                                     int d_model, int tot_expert, int top_k, int dtype,
                                     int64_t *idx_out, void *score_out, void *logits_out,
                                     ccf_stream_t stream) {
  return ccf::gate_forward(x, wg, bg, tokens, d_model, tot_expert, top_k, dtype, idx_out, score_out, logits_out, stream,
                           nullptr, 0, nullptr);
}
