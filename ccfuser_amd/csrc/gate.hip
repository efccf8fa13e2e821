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
#include <type_traits>

namespace ccf {
int g_gate_waves = 8;    // most wavefronts of a gate workgroup (each takes other parts of K), 1..8
int g_gate_slots = 0;    // parts of K a wavefront works on at a time (1, 2, 4); 0 = by the token count
int g_gate_stream = -1;  // 1: every wavefront takes its tokens through all of K alone; 0: never; -1: with many tokens
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
    if constexpr (KS > 2) {                        // long lists: most offers end at the last kept entry
      float lv = v[0];
      int li = id[0];
#pragma unroll
      for (int s = 1; s < KS; ++s)
        if (s == k - 1) {
          lv = v[s];
          li = id[s];
        }
      if (!better(nv, nid, lv, li)) return;        // not among the k best
    }
    bool beats[KS];                                // short lists: no branch
#pragma unroll
    for (int s = 0; s < KS; ++s) beats[s] = better(nv, nid, v[s], id[s]);
#pragma unroll
    for (int s = KS - 1; s >= 0; --s) {
      if (s < k) {
        const int up = s > 0 ? s - 1 : 0;
        const bool ahead = s > 0 && beats[up];     // belongs further up: slot s takes its upper neighbour
        v[s] = ahead ? v[up] : (beats[s] ? nv : v[s]);
        id[s] = ahead ? id[up] : (beats[s] ? nid : id[s]);
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
      // running sums: the parts of this round in ascending order.  The part sums are read
      // eight at a time ahead of the additions, which stay one chain in part order.
      int np_round = nparts - rd * per_round;
      np_round = np_round < per_round ? np_round : per_round;
      for (int i = threadIdx.x; i < TW * N; i += blockDim.x) {
        const int tok = i / N, col = i % N;
        float t = rd == 0 ? 0.0f : s_total[tok * kLd + col];
        for (int q0 = 0; q0 < np_round; q0 += 8) {
          float ps[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            int q = q0 + u;
            q = q < np_round ? q : np_round - 1;
            ps[u] = s_mem[static_cast<size_t>(q >> LS) * kRegionFloats + (q & (S - 1)) * TW * N + i];
          }
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const float sum = (rd == 0 && q0 + u == 0) ? ps[u] : t + ps[u];   // the first part starts the chain
            t = q0 + u < np_round ? sum : t;
          }
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
#pragma unroll
      for (int c0 = 0; c0 < N; c0 += 8) {          // eight logits read ahead of their offers
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = lg[c0 + u];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (c0 + u < ne) best.offer(v[u], e0 + c0 + u, k);
      }
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

// fp16 gate for many tokens: every wavefront works alone.  It takes TW tokens through all of
// K, S parts at a time ("round": 4 stages), in one unbroken stream of stages: the loads run
// five stages ahead of the MFMAs in four sets of registers, each set parked in the
// wavefront's LDS one stage ahead of its use, so after the first arrival the matrix pipe
// does not wait for memory again.  At the end of a round the part sums, which are registers
// of this lane, go onto the running sums in ascending part order; the logits of a tile of N
// experts pass through the wavefront's LDS once, for the selection (one lane per token) and
// the coalesced write.  No barrier before the expert counts of the workgroup.
constexpr int kStreamWaves = 4;

template <int N, int LS, int KS>
__global__ void __launch_bounds__(kStreamWaves * 64)
gate_stream_kernel(const half_t *__restrict__ x, const half_t *__restrict__ wg, const half_t *__restrict__ bg,
                   int tokens, int d, int E, int k, int64_t *__restrict__ idx_out,
                   half_t *__restrict__ score_out, half_t *__restrict__ logits_out, int32_t *__restrict__ wg_cnt) {
  using M = Mfma<N>;
  constexpr int kBlocks = 64 / N;
  constexpr int S = 1 << LS;
  static_assert(S <= kBlocks, "a slot is a block");
  constexpr int TB = kBlocks / S;                  // token blocks of a wavefront
  constexpr int TW = TB * N;                       // its tokens
  constexpr int RB = M::kRegs / kBlocks;           // accumulator registers of a block
  constexpr int kWLoads = N * S / 16;
  constexpr int kLd = N + 1;
  static_assert(TW * kLd <= kRegionFloats, "the logits of a tile fit the wavefront's region");
  extern __shared__ float s_mem[];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  float *region = s_mem + static_cast<size_t>(wave) * kRegionFloats;
  const int t0 = (blockIdx.x * kStreamWaves + wave) * TW;
  const int nparts = (d + kPart - 1) / kPart;
  const int rounds = (nparts + S - 1) / S;
  const bool ragged = d % (S * kPart) != 0;        // the last round has K elements to leave out

  const int blk = lane / N, r = lane % N;
  const int slot = blk & (S - 1);
  char *tile = reinterpret_cast<char *>(region);
  const char *my_x = tile + lane * kRowBytes;
  const char *my_w = tile + kTileBytes + (slot * N + r) * kRowBytes;
  const int l_row = lane >> 2, l_piece = lane & 3;
  char *park_at = tile + l_row * kRowBytes + l_piece * 16;

  Best<KS> best;
  best.clear();
  if (t0 < tokens) {                               // uniform per wavefront
    const half_t *x_src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int lr = 16 * i + l_row;
      int t = t0 + ((lr / N) >> LS) * N + lr % N;
      t = t < tokens ? t : tokens - 1;
      x_src[i] = x + static_cast<size_t>(t) * d + (((lr / N) & (S - 1)) * kPart + l_piece * 8);
    }
    for (int e0 = 0; e0 < E; e0 += N) {
      // columns past the last expert repeat its weights; nothing reads their logits
      const bool has_w = e0 + r < E;
      float my_bias = 0.0f;
      if (bg && has_w) my_bias = static_cast<float>(bg[e0 + r]);
      const half_t *w_src[kWLoads];
#pragma unroll
      for (int i = 0; i < kWLoads; ++i) {
        const int wr = 16 * i + l_row;
        int e = e0 + wr % N;
        e = e < E ? e : E - 1;
        w_src[i] = wg + static_cast<size_t>(e) * d + ((wr / N) * kPart + l_piece * 8);
      }
      // stage g of the stream: round g / 4, K offset of the round's first part + (g % 4) * kStageK
      auto stage_k = [&](int g) { return (g >> 2) * (S * kPart) + (g & 3) * kStageK; };
      typedef int4v XSet[4];
      typedef int4v WSet[kWLoads];
      XSet xa, xb, xc, xd;
      WSet wa, wb, wc, wd;
      auto fetch = [&](int g, XSet &xv, WSet &wv) {   // past the end of K the loads read the start of x and wg
        const int ks = stage_k(g);
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
      auto park = [&](const XSet &xv, const WSet &wv) {
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
      typename M::Acc acc;
      // A piece is 8 K elements of a stage.  Its MFMAs run on fp32 copies made during the piece
      // before, in registers that no MFMA in flight reads: a conversion into a register that the
      // running MFMA still reads waits for that MFMA, and one wavefront per SIMD has nothing to
      // cover the wait with.
      auto convert = [&](auto rag, int g, int c, const half8 &vx, const half8 &vw, float (&fx)[8], float (&fw)[8]) {
        half8 xs = vx, ws = vw;
        if constexpr (decltype(rag)::value) {      // K ends inside a round: what lies past it counts as zero
          const bool in = stage_k(g) + slot * kPart + c * 8 < d;
          const half8 zero = {};
          xs = in ? vx : zero;
          ws = in ? vw : zero;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          fx[j] = static_cast<float>(xs[j]);
          fw[j] = static_cast<float>(ws[j]);
        }
      };
      auto mma = [&](const float (&fx)[8], const float (&fw)[8]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc = M::run(fx[j], fw[j], acc);
      };
      float total[TB * RB];
      half8 ax, aw, bx, bw;                        // pieces as read from LDS: even ones in a, odd ones in b
      float fax[8], faw[8], fbx[8], fbw[8];        // their fp32 copies
      // eight MFMAs with the next piece's conversions between them
#define CCF_GATE_PIECE(MMA_F, G, C, RAW, CONV_F)                       \
  do {                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                 \
    mma(MMA_F##x, MMA_F##w);                                           \
    convert(rag, G, C, RAW##x, RAW##w, CONV_F##x, CONV_F##w);          \
    _Pragma("unroll") for (int q_ = 0; q_ < 8; ++q_) {                 \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               \
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);               \
    }                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                 \
  } while (0)
      // One stage, entered with piece 0 converted (fa) and piece 1 read (b).  Reads from LDS
      // run two pieces ahead, conversions one; the next stage is parked once this stage's last
      // read is on its way (the LDS works in order), and its first pieces are read behind that.
#define CCF_GATE_STAGE(g, PARK_NEXT)                                   \
  do {                                                                 \
    take(2, ax, aw);                                                   \
    CCF_GATE_PIECE(fa, g, 1, b, fb);                                   \
    take(3, bx, bw);                                                   \
    __builtin_amdgcn_sched_barrier(0);                                 \
    PARK_NEXT;                                                         \
    CCF_GATE_PIECE(fb, g, 2, a, fa);                                   \
    take(0, ax, aw);                                                   \
    CCF_GATE_PIECE(fa, g, 3, b, fb);                                   \
    take(1, bx, bw);                                                   \
    CCF_GATE_PIECE(fb, (g) + 1, 0, a, fa);                             \
  } while (0)
      auto all_rounds = [&](auto rag) {
      asm volatile("" ::: "memory");               // the tile is free: the previous expert tile's logits have been read
      fetch(0, xa, wa);
      fetch(1, xb, wb);
      fetch(2, xc, wc);
      fetch(3, xd, wd);
      __builtin_amdgcn_sched_barrier(0);
      park(xa, wa);                                // stage 0
      fetch(4, xa, wa);
      __builtin_amdgcn_sched_barrier(0);
      take(0, ax, aw);
      take(1, bx, bw);
      convert(rag, 0, 0, ax, aw, fax, faw);
      __builtin_amdgcn_sched_barrier(0);
      for (int rd = 0; rd < rounds; ++rd) {
        const int g = 4 * rd;
#pragma unroll
        for (int v = 0; v < M::kRegs; ++v) acc[v] = 0.0f;
        CCF_GATE_STAGE(g, park(xb, wb); fetch(g + 5, xb, wb));
        CCF_GATE_STAGE(g + 1, park(xc, wc); fetch(g + 6, xc, wc));
        CCF_GATE_STAGE(g + 2, park(xd, wd); fetch(g + 7, xd, wd));
        if (rd + 1 < rounds)
          CCF_GATE_STAGE(g + 3, park(xa, wa); fetch(g + 8, xa, wa));
        else
          CCF_GATE_STAGE(g + 3, (void)0);            // its reads ahead find the last stage again; nothing uses them
        // the round's part sums onto the running sums, ascending part order
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
          for (int sl = 0; sl < S; ++sl) {
            const int p = rd * S + sl;
            if (p < nparts) {
#pragma unroll
              for (int j = 0; j < RB; ++j) {
                const float ps = acc[(tb * S + sl) * RB + j];
                total[tb * RB + j] = p == 0 ? ps : total[tb * RB + j] + ps;
              }
            }
          }
      }
      };
      if (ragged) all_rounds(std::true_type{}); else all_rounds(std::false_type{});
#undef CCF_GATE_PIECE
#undef CCF_GATE_STAGE
      // logits of the tile: bias, one rounding, into the wavefront's LDS as [token][expert]
      asm volatile("" ::: "memory");
#pragma unroll
      for (int j = 0; j < TB * RB; ++j) {
        float t = total[j];
        if (has_w) {
          if (bg) t = t + my_bias;
          t = round_to<half_t>(t);
        }
        region[((j / RB) * N + M::row(j % RB, lane)) * kLd + r] = t;
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      if (logits_out) {
        for (int i = lane; i < TW * N; i += 64) {
          const int tok = i / N, col = i % N;
          if (e0 + col < E && t0 + tok < tokens)
            logits_out[static_cast<size_t>(t0 + tok) * E + e0 + col] = static_cast<half_t>(region[tok * kLd + col]);
        }
      }
      if (lane < TW && t0 + lane < tokens) {
        const float *lg = region + lane * kLd;
        const int ne = (E - e0) < N ? (E - e0) : N;
#pragma unroll
        for (int c0 = 0; c0 < N; c0 += 8) {
          float v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) v[u] = lg[c0 + u];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (c0 + u < ne) best.offer(v[u], e0 + c0 + u, k);
        }
      }
    }
    if (lane < TW && t0 + lane < tokens) best.template write<half_t>(t0 + lane, k, idx_out, score_out);
  }
  if (wg_cnt) {
    // expert counts of the workgroup's kStreamWaves * TW tokens, as in gate_mfma_kernel
    __syncthreads();
    int *row = reinterpret_cast<int *>(s_mem);
    for (int e = threadIdx.x; e < E; e += blockDim.x) row[e] = 0;
    __syncthreads();
    if (lane < TW && t0 + lane < tokens) {
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
  // With a wavefront or more per SIMD even when each works alone (two with the 16-wide tile, whose
  // MFMAs are shorter), the wavefronts stream through K on their own; with fewer, the wavefronts
  // of a workgroup share the parts of K.
  const int tiles = (tokens + tw - 1) / tw;
  const bool stream_form = g_gate_stream > 0 || (g_gate_stream < 0 && (tiles >= 2048 || (tiles >= 1024 && n == 32)));
  int waves = (nparts + slots - 1) / slots;
  int cap = g_gate_waves < kMaxWaves ? g_gate_waves : kMaxWaves;
  cap = cap < 1 ? 1 : cap;
  waves = waves < cap ? waves : cap;
  if (stream_form) waves = kStreamWaves;
  const int wg_tokens = stream_form ? kStreamWaves * tw : tw;
  const size_t lds = sizeof(float) * (static_cast<size_t>(waves) * kRegionFloats +
                                      (stream_form ? 0 : static_cast<size_t>(tw) * (n + 1)));
  CCF_REQUIRE(lds <= 160 * 1024, CCF_ERR_SHAPE, "gate: %zu bytes of LDS needed", lds);
  dim3 grid((tokens + wg_tokens - 1) / wg_tokens), block(waves * 64);
  if (wg_cnt && static_cast<long long>(grid.x) * tot_expert <= max_cnt) {
    if (tokens_per_wg) *tokens_per_wg = wg_tokens;
  } else {
    wg_cnt = nullptr;
  }
#define CCF_GATE_LAUNCH(NN, LSV, KSV)                                                              \
  do {                                                                                             \
    auto kern = stream_form ? gate_stream_kernel<NN, LSV, KSV> : gate_mfma_kernel<NN, LSV, KSV>;   \
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
    if (top_k == 1) CCF_GATE_LAUNCH(NN, LSV, 1);                             \
    else if (top_k == 2) CCF_GATE_LAUNCH(NN, LSV, 2);                        \
    else CCF_GATE_LAUNCH(NN, LSV, kMaxTopK);                                 \
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
