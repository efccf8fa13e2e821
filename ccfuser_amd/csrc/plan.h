// Tile plan of a grouped GEMM: which workgroup computes which tile, derived on the
// device from the expert offsets.  Shared by the GEMM launcher and by the routing
// kernels, whose last launch can build the plans of the GEMMs that follow.
#pragma once

#include <limits.h>

#include "ccf_common.h"

namespace ccf {

// ---- tile plan ---------------------------------------------------------------
// The plan is one 16-byte entry per launched workgroup, indexed by the hardware
// workgroup id: {expert, first sorted row, rows in the M tile, N tile}, expert
// = -1 for workgroups with nothing to do.  A workgroup learns its whole
// assignment from a single load.
__host__ __device__ inline size_t plan_ints(long long wgs) { return 4 * static_cast<size_t>(wgs); }

__host__ __device__ inline long long launched_wgs(int max_tiles, int n_tiles_n) {
  long long w = static_cast<long long>(max_tiles) * n_tiles_n;
  return ((w + 7) / 8 + 2) * 8;                   // per XCD: a share of each of the two tile classes, rounded up
}

constexpr int kOrderGroupM = 8;
// build_plan divides by the tile height with shifts
__host__ __device__ constexpr bool plan_bm_ok(int bm) { return bm > 0 && (bm & (bm - 1)) == 0; }

// Scratch of the split last round, in front of the plan in the caller's workspace:
//   [0, 16)              header: tile slots T (a multiple of 8; slot t belongs to XCD t % 8), parts S
//   [256, 256 + 16*256)  entries {expert, row0, rows, tile_n | part << 16 | S << 24} by workgroup
//                        id: part s of tile slot t at (t % 8) + 8 * ((t / 8) * S + s); expert -1 = none
//   [kTailHead, ...)     256 partial tiles of 256 x 256 fp32, by the same workgroup id
constexpr int kTailMaxParts = 256;
constexpr int kTailMaxTiles = kTailMaxParts / 2;     // tile slots: every tile has at least two parts
constexpr size_t kTailHead = 256 + 16 * kTailMaxParts;
constexpr size_t kSplitPartialBytes = static_cast<size_t>(kTailMaxParts) * 256 * 256 * 4;
// Behind those partial tiles, the partial tiles of the skinny tiles when they run as a launch of
// their own (below): kSkTailSegs tiles of 64 x 256 fp32 per workgroup of that launch.
constexpr int kSkTailMaxWgs = 256;
constexpr int kSkTailSegs = 4;                       // most skinny tiles the K steps of one workgroup may touch
constexpr size_t kSkTailTileBytes = 64 * 256 * 4;
constexpr size_t kSkTailBytes = static_cast<size_t>(kSkTailMaxWgs) * kSkTailSegs * kSkTailTileBytes;
constexpr size_t kTailBytes = kTailHead + kSplitPartialBytes + kSkTailBytes;

// ---- skinny tiles --------------------------------------------------------------
// An expert's rows rarely fill its last 256-row M tile, and a tile with a few dozen real rows
// costs a CU as much as a full one: its K steps are paced by the tile loads, not by the MFMAs
// it skips.  With a skinny list in the plan request, a remainder of at most kSkinnyRows rows
// (rows % BM, or all rows of an expert smaller than that) may leave the plan of 256-row tiles
// and become one entry per N tile of a second list; a remainder of up to twice that may become
// two (the plan prices both limits and takes the cheaper).  A few workgroups per XCD of the persistent
// kernel (ffn.hip) then do nothing but those entries, as 64 x 256 tiles that stream their
// weight panel through a deep LDS pipeline: little arithmetic, mostly memory latency, so they
// run beside the compute-bound 256-row tiles on bandwidth those leave idle.  Whether that pays
// depends on the tile counts (a CU taken from the 256-row tiles costs them 1/32 of their
// rate; whole rounds of tiles matter more than tiles), so build_plan prices both ways with a
// small model and picks: ns = workgroups per XCD given to skinny tiles, 0 = none.
//
// The third way: the skinny tiles as a launch of their own behind the persistent kernel, which
// then keeps every CU for 256-row tiles (a GEMM whose 256-row tiles fill whole rounds exactly
// loses a round to any CU it gives away).  Alone on the chip the skinny tiles are bound by
// streaming their experts' weights from HBM once more, so the list is cut stream-K fashion: its
// T tiles x k_tiles K steps are one sequence that the W workgroups of the launch cut into equal
// ranges of q = ceil(T k_tiles / W) steps; a workgroup leaves one fp32 partial tile per list
// entry its range touches, and the reduction that follows adds a tile's partial tiles in K
// order and applies the epilogue (no atomics: two runs give the same bits).
//
// Layout of the list (int32):
//   [0] tiles T   [1] ns   [2] tiles per XCD (XCD x owns entries [x * [2], (x + 1) * [2]))
//   [3] q > 0: the tiles are cut along K, q K steps per workgroup; 0 otherwise
//   [4] with q > 0: 0 = as a launch of their own, 1 = inside the persistent launch (each of its
//       workgroups runs its range at some point between its 256-row tiles)
//   [5] most 256-row tiles a workgroup of the persistent launch runs     [6..7] unused
//   [kSkinnyHead + 4 i ...] entry i < T: {expert, first sorted row, rows (1..kSkinnyRows), N tile}
constexpr int kSkinnyRows = 64;
// Skinny M tiles of a remainder of r rows when remainders up to `limit` rows (kSkinnyRows or twice that) leave the
// 256-row tiles.
__host__ __device__ inline int skinny_m_tiles(int r, int limit) {
  return (r > 0 && r <= limit) ? (r + kSkinnyRows - 1) / kSkinnyRows : 0;
}
constexpr int kSkinnyMaxWgs = 4;                     // per XCD
constexpr int kSkinnyHead = 8;                       // header integers in front of the entries
__host__ __device__ inline size_t skinny_ints(int max_rows, int E, int n_tiles_n) {
  const int by_rows = (max_rows + kSkinnyRows - 1) / kSkinnyRows;
  const int most = 2 * E < by_rows ? 2 * E : by_rows;  // at most two skinny M tiles per expert
  return kSkinnyHead + 4 * static_cast<size_t>(most > 0 ? most : 0) * n_tiles_n;
}

// n / d for 0 <= n < 2^24, d > 0 and a quotient below 2^22 (every count a plan divides is far below: at
// most the tiles of an XCD) through the reciprocal of d as a float, made once per divisor: n and d are exact
// as floats, the reciprocal and the product are each within an ulp, so the truncated product is off by at
// most one either way, which the remainder shows.  An integer division proper is ~30 dependent
// instructions, and the plan is built on the critical path of its launch.
struct FastDiv {
  int d;
  float r;
  __device__ inline explicit FastDiv(int dd) : d(dd), r(1.0f / static_cast<float>(dd)) {}
  __device__ inline int div(int n) const {
    int q = static_cast<int>(static_cast<float>(n) * r);
    int rem = n - q * d;
    q += rem >= d ? 1 : 0;
    q -= rem < 0 ? 1 : 0;
    return q;
  }
};

// Time, in K steps of a 256-row tile, that F tiles of k_tiles K steps and an epilogue worth
// `epi` K steps take on spx workgroups: whole rounds, then the last, partly filled round, which
// is cut along K when the request allows it (same rule as the split below).
__device__ inline int rounds_cost(int F, int spx, int k_tiles, int epi, bool may_split, int max_parts) {
  if (spx <= 0) return INT_MAX / 2;
  const int full = FastDiv(spx).div(F);            // every count here is far below 2^24
  const int r = F - full * spx;
  int cost = full * (k_tiles + epi);
  if (r > 0) {
    int S = 0;
    if (may_split && 2 * r <= spx) {
      S = FastDiv(r).div(spx);
      S = S > max_parts ? max_parts : S;
      S = S > k_tiles / 4 ? k_tiles / 4 : S;
      S = (S >= 2 && 8 * r * S <= 256) ? S : 0;
    }
    cost += S ? FastDiv(S).div(k_tiles) + 28 : k_tiles + epi;    // 28: two more launches, pipeline fill, the reduction (measured)
  }
  return cost;
}

// Rows of M tile i of an expert with cnt rows in nt = ceil(cnt / BM) tiles.  When
// the last tile would hold at most BM/2 rows, it and the one before it share
// their rows evenly instead: a nearly empty tile still streams a whole weight
// panel, on its own and from HBM (its siblings have long passed), which costs
// about as much as a full tile; two half-full tiles run in step with their
// siblings, share the panel in L2, and skip half of their MFMAs.
__device__ inline void tile_rows(int cnt, int nt, int i, int BM, int &first_row, int &rows) {
  const int last = cnt - (nt - 1) * BM;
  if (nt >= 2 && last <= BM / 2 && i >= nt - 2) {
    const int both = BM + last;
    const int h = (both + 1) / 2;
    first_row = (nt - 2) * BM + (i == nt - 2 ? 0 : h);
    rows = i == nt - 2 ? h : both - h;
  } else {
    first_row = i * BM;
    rows = (cnt - i * BM) < BM ? (cnt - i * BM) : BM;
  }
}

// Tiles come in two classes.  A "long" M tile holds more than BM/2 rows; a
// "short" one is the only tile of an expert with at most BM/2 rows, skips most
// of its MFMAs and ends early.  Workgroups that share an
// XCD share weight and token tiles through its L2 only while they walk K in
// step, and a workgroup that ends early puts every later one on its CU out of
// step, so all long tiles are launched first and the short ones after them,
// where they also even out the end of the launch.
// What one plan needs besides the offsets; passed by value to the kernel that builds it.
struct PlanReq {
  int BM, max_tiles, max_rows, n_tiles_n;
  int spx;          // persistent workgroups per XCD when the last round may be split, else 0
  int k_tiles;      // K tiles of a tile (bounds the parts of a split)
  int max_parts;    // most parts a tile is cut into
  int32_t *plan;
  int32_t *tail;    // split scratch (header and entries), or NULL
  int32_t *skinny;  // skinny list, or NULL: every row goes through the 256-row tiles
  int cus;          // workgroups of the persistent launch (a multiple of 8)
  int epi_cost;     // the epilogue of a 256-row tile, in K steps
  int skinny_pct;   // a K step of a skinny tile in percent of a K step of a 256-row tile; 0 = never use skinny
                    // tiles; -n (n <= kSkinnyMaxWgs) = always, with n workgroups per XCD; -(kSkinnyMaxWgs + 1) =
                    // always cut along K as a launch of their own, -(kSkinnyMaxWgs + 2) = always cut along K inside
                    // the persistent launch (both need `tail`)
  int sk_tail_ok;   // the skinny tiles may run as a launch of their own (the caller launches the kernels for it)
  int sk_beside_ok; // they may run in workgroups of the persistent launch (its four-wavefront form only)
};

// A K step of a skinny tile, in percent of a 256-row tile's, when the whole chip runs skinny tiles
// and HBM bandwidth bounds them; and the fixed cost of that launch and its reduction, in K steps.
// (Measured on 4096 x 4096 x 14336 layers, 80 and 280 skinny tiles, 70 K steps per workgroup: ~100 K steps'
// worth of time for the launch of its own with its reduction, ~80 inside the persistent launch.)
constexpr int kSkTailStepPct = 115, kSkTailFixed = 16;
// The same when the ranges run inside the persistent launch, half of the chip at a time beside 256-row tiles.
constexpr int kSkInsideStepPct = 105, kSkInsideFixed = 8;

// Most tiles a range of q consecutive K steps can touch when a tile has k_tiles steps.
__host__ __device__ inline int sk_tail_segments(int q, int k_tiles) { return (q - 1 + k_tiles - 1) / k_tiles + 1; }

// Built by `nparts` workgroups of any size that is a multiple of 64 (all threads of each call
// this with the workgroup's `part`).  Every workgroup repeats the small scans and takes a share
// of the experts and of the idle entries; which entries stay idle is known in closed form, so
// no entry is written by two workgroups and their order does not matter.
// uniform_rows > 0: every expert has that many rows (offsets is not read).
__device__ inline void build_plan(const PlanReq &rq, const int32_t *__restrict__ offsets, int E,
                                  int part = 0, int nparts = 1, int uniform_rows = 0) {
  const int BM = rq.BM, max_tiles = rq.max_tiles, max_rows = rq.max_rows, n_tiles_n = rq.n_tiles_n;
  const int k_tiles = rq.k_tiles;
  int spx = rq.spx;                 // lowered below by the workgroups given to skinny tiles
  int32_t *__restrict__ plan = rq.plan;
  int32_t *__restrict__ tail = rq.tail;
  int32_t *__restrict__ skinny = rq.skinny;
  // tile counts and remainders by BM as shifts: BM is a power of two (plan_bm_ok, checked where requests are made)
  const int bm_shift = 31 - __clz(BM);
  auto tiles_of = [&](int cnt) { return (cnt + BM - 1) >> bm_shift; };
  auto rem_of = [&](int cnt) { return cnt & (BM - 1); };
  __shared__ int s_full[8];        // split last round: slots of XCD x from s_full[x] on go to the tail list
  __shared__ int s_used[8];        // tiles of XCD x
  __shared__ int s_parts;          // parts per tail tile, 0 = no split
  __shared__ int s_off[1025];
  __shared__ int s_long[1025];     // exclusive scan of long M tiles per expert
  __shared__ int s_short[1025];    // exclusive scan of short M tiles per expert (0 or 1 each)
  for (int e = threadIdx.x; e <= E; e += blockDim.x) {
    int v = uniform_rows > 0 ? e * uniform_rows : offsets[e];
    s_off[e] = v < max_rows ? v : max_rows;          // never plan past the caller's bound
  }
  __syncthreads();
  __shared__ int s_ns;             // workgroups per XCD given to skinny tiles (0: none)
  __shared__ int s_tail_q;         // > 0: skinny tiles cut along K, K steps per workgroup
  __shared__ int s_tail_inside;    // 1: inside the persistent launch, 0: as a launch of their own
  __shared__ int s_sk_limit;       // remainders of at most this many rows are skinny
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    // Skinny tiles or not: tile counts both ways, then the cheaper plan by the model above.
    int ns_wgs = 0, tail_q = 0, tail_inside = 0, sk_limit = kSkinnyRows;
    if (skinny && rq.skinny_pct != 0 && rq.cus >= 64) {
      // 256-row tiles without skinny tiles; with them, and the skinny M tiles, for both limits on a remainder
      int nl0 = 0, nl1 = 0, nk1 = 0, nl2 = 0, nk2 = 0;
      for (int e = lane; e < E; e += 64) {
        int cnt = s_off[e + 1] - s_off[e];
        cnt = cnt > 0 ? cnt : 0;
        const int nt = tiles_of(cnt), r = rem_of(cnt);
        const int sk1 = skinny_m_tiles(r, kSkinnyRows), sk2 = skinny_m_tiles(r, 2 * kSkinnyRows);
        nl0 += nt;
        nl1 += nt - (sk1 ? 1 : 0);
        nk1 += sk1;
        nl2 += nt - (sk2 ? 1 : 0);
        nk2 += sk2;
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        nl0 += __shfl_xor(nl0, off, 64);
        nl1 += __shfl_xor(nl1, off, 64);
        nk1 += __shfl_xor(nk1, off, 64);
        nl2 += __shfl_xor(nl2, off, 64);
        nk2 += __shfl_xor(nk2, off, 64);
      }
      // candidates 8 .. 15 (below) are candidates 0 .. 7 with the larger limit; forced modes take the larger
      // limit when it gives more skinny tiles (the same answer in every lane)
      const bool wide = rq.skinny_pct < 0 ? nk2 > nk1 : ((lane >> 3) & 1) != 0;
      if (wide) {
        nl1 = nl2;
        nk1 = nk2;
      }
      const int my_limit = wide ? 2 * kSkinnyRows : kSkinnyRows;
      // the launch of their own: possible when the caller launches the split kernels and a
      // workgroup's range stays within kSkTailSegs tiles
      const int tail_wgs = rq.cus < kSkTailMaxWgs ? rq.cus : kSkTailMaxWgs;
      int q_c = 0;
      if (tail && (rq.sk_tail_ok || rq.sk_beside_ok) && nk1 > 0 && k_tiles > 0) {
        const long long steps = static_cast<long long>(nk1) * n_tiles_n * k_tiles;
        // (more than 2^23 steps are more than the workgroups' ranges may hold anyway)
        const int q = steps < (1ll << 23) ? FastDiv(tail_wgs).div(static_cast<int>(steps) + tail_wgs - 1) : (1 << 20);
        if (q < (1 << 20) && FastDiv(k_tiles).div(q - 1 + k_tiles - 1) + 1 <= kSkTailSegs) q_c = q;   // sk_tail_segments(q, k_tiles)
      }
      if (rq.skinny_pct < 0) sk_limit = my_limit;     // uniform: every lane took the same limit
      if (nk1 > 0 && rq.skinny_pct < -kSkinnyMaxWgs) {
        // forced (tests, measurements); 0 = not possible: no skinny tiles
        tail_inside = rq.skinny_pct == -kSkinnyMaxWgs - 2;
        tail_q = (tail_inside ? rq.sk_beside_ok : rq.sk_tail_ok) ? q_c : 0;
      } else if (nk1 > 0 && rq.skinny_pct < 0) {
        ns_wgs = rq.sk_beside_ok ? -rq.skinny_pct : 0; // forced
      } else if (rq.skinny_pct > 0) {
        const int cus_x = rq.cus / 8;
        const bool may_split = spx > 0;
        const int F0 = (nl0 * n_tiles_n + 7) / 8, F1 = (nl1 * n_tiles_n + 7) / 8, T_x = (nk1 * n_tiles_n + 7) / 8;
        // The candidates are priced together, one per lane (the prices are chains of integer divisions, and
        // this wavefront is on the critical path of the launch): 0 = every row in 256-row tiles, 1 ..
        // kSkinnyMaxWgs = that many workgroups per XCD beside them, then the launch of their own and the
        // ranges inside the persistent launch; 8 .. 15 the same with remainders of up to twice kSkinnyRows
        // rows as skinny tiles.  The cheapest wins; of equals, the first in that order.
        const int cand = lane & 7;
        const int n = (cand >= 1 && cand <= kSkinnyMaxWgs) ? cand : 0;
        int cost = rounds_cost(cand == 0 ? F0 : F1, cus_x - n, k_tiles, rq.epi_cost, may_split, rq.max_parts);
        bool ok = cand <= kSkinnyMaxWgs + 2 && (cand == 0 || nk1 > 0);
        if (n > 0) {
          const int sk_tile = (k_tiles * rq.skinny_pct + 99) / 100 + 3;       // one skinny tile, in K steps
          const int sk_c = FastDiv(n).div(T_x + n - 1) * sk_tile;
          cost = cost > sk_c ? cost : sk_c;
          ok = ok && n * 4 <= cus_x && rq.sk_beside_ok;
        } else if (cand == kSkinnyMaxWgs + 1) {
          cost += (q_c * kSkTailStepPct + 99) / 100 + kSkTailFixed;
          ok = ok && q_c > 0 && rq.sk_tail_ok;
        } else if (cand == kSkinnyMaxWgs + 2) {
          cost += (q_c * kSkInsideStepPct + 99) / 100 + kSkInsideFixed;
          ok = ok && q_c > 0 && rq.sk_beside_ok;
        }
        cost = cost < (1 << 26) ? cost : (1 << 26);
        int key = ok ? (cost << 4) | (lane & 15) : INT_MAX;
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) {
          const int other = __shfl_xor(key, off, 64);
          key = other < key ? other : key;
        }
        const int win16 = key & 15, win = win16 & 7;               // candidate 0 is always there
        const int q_win = __shfl(q_c, win16, 64);
        sk_limit = (win16 >> 3) ? 2 * kSkinnyRows : kSkinnyRows;
        ns_wgs = (win >= 1 && win <= kSkinnyMaxWgs) ? win : 0;
        if (win > kSkinnyMaxWgs) {
          tail_q = q_win;
          tail_inside = win == kSkinnyMaxWgs + 2 ? 1 : 0;
        }
      }
    }
    if (lane == 0) { s_ns = ns_wgs; s_tail_q = tail_q; s_tail_inside = tail_inside; s_sk_limit = sk_limit; }
    int carry_l = 0, carry_s = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      int cnt = e < E ? s_off[e + 1] - s_off[e] : 0;
      cnt = cnt > 0 ? cnt : 0;
      const int nt = tiles_of(cnt);
      int ns, nl;
      if (ns_wgs || tail_q) {
        const int r = rem_of(cnt);                                // ns counts skinny M tiles here
        ns = skinny_m_tiles(r, sk_limit);
        nl = nt - (ns ? 1 : 0);
      } else {
        ns = (nt == 1 && cnt <= BM / 2) ? 1 : 0;                  // a short tile only when it is the expert's only one
        nl = nt - ns;
      }
      int inc_l = nl, inc_s = ns;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        int ol = __shfl_up(inc_l, off, 64);
        int os = __shfl_up(inc_s, off, 64);
        if (lane >= off) { inc_l += ol; inc_s += os; }
      }
      if (e < E) { s_long[e] = carry_l + inc_l - nl; s_short[e] = carry_s + inc_s - ns; }
      carry_l += __shfl(inc_l, 63, 64);
      carry_s += __shfl(inc_s, 63, 64);
    }
    if (lane == 0) { s_long[E] = carry_l; s_short[E] = carry_s; }
    // The split last round (run by grouped_gemm_tail_kernel and splitk_reduce_kernel in ffn.hip).
    // XCD x holds used_x tiles; with spx persistent workgroups per XCD the last used_x % spx of
    // them form a partly filled round.
    // When that round is at most half full on every XCD, its tiles leave the plan: tile i of
    // XCD x's last round, part s of S, becomes tail entry x + 8 * (i * S + s), the workgroup id
    // that the hardware places on the same XCD, so the patch of neighbouring tiles keeps sharing
    // its operands through that XCD's L2 (parts of the same K range walk K in step).
    // Lane x < 8 takes XCD x.
    {
      const bool use_sk = ns_wgs > 0 || tail_q > 0;
      const int spx_w = spx > 0 ? spx - ns_wgs : spx;
      const int total_l = carry_l * n_tiles_n, total_s = use_sk ? 0 : carry_s * n_tiles_n;
      const int per_l = (total_l + 7) / 8, per_s = (total_s + 7) / 8;
      const int x = lane & 7;
      int nl_x = total_l - x * per_l, ns_x = total_s - x * per_s;
      nl_x = nl_x < 0 ? 0 : (nl_x > per_l ? per_l : nl_x);
      ns_x = ns_x < 0 ? 0 : (ns_x > per_s ? per_s : ns_x);
      const int used = nl_x + ns_x;
      const int full = spx_w > 0 ? used / spx_w * spx_w : used;
      int max_r = used - full;
#pragma unroll
      for (int off = 4; off >= 1; off >>= 1) {
        const int other = __shfl_xor(max_r, off, 64);
        max_r = other > max_r ? other : max_r;
      }
      int S = 0;
      if (tail && spx_w > 0 && max_r > 0 && max_r * 2 <= spx_w) {
        S = spx_w / max_r;
        S = S > rq.max_parts ? rq.max_parts : S;
        S = S > k_tiles / 4 ? k_tiles / 4 : S;           // at least four K tiles per part
        S = (S >= 2 && 8 * max_r * S <= kTailMaxParts) ? S : 0;
      }
      if (lane < 8) {
        s_used[lane] = used;
        s_full[lane] = S ? full : INT_MAX;
      }
      if (lane == 0) {
        s_parts = S;
        if (tail && part == 0) { tail[0] = S ? 8 * max_r : 0; tail[1] = S; }
      }
    }
  }
  // the launcher checks that the worst-case tile count, and with it every count below, is below 2^24
  const int wgs = static_cast<int>(launched_wgs(max_tiles, n_tiles_n));
  int4v *entry = reinterpret_cast<int4v *>(plan);
  int4v *tent = tail ? reinterpret_cast<int4v *>(tail + 64) : nullptr;
  __syncthreads();
  // Hardware hands consecutive workgroup ids to the 8 XCDs in turn, so XCD x
  // runs ids x, x+8, ... in order.  Each class is cut into eight equal
  // contiguous runs of logical tile ids, one per XCD (one L2): with nl long
  // tiles on XCD x, its slot j is long tile x*per_long + j for j < nl, else
  // short tile x*per_short + (j - nl).  The used slots of an XCD are a prefix:
  // the first idle entry ends its list.
  const int ns_wgs = s_ns;                                       // published by the barrier above
  const bool use_skinny = ns_wgs > 0 || s_tail_q > 0;
  if (spx > 0) spx -= ns_wgs;
  const int total_long = s_long[E] * n_tiles_n;
  const int total_short = use_skinny ? 0 : s_short[E] * n_tiles_n;   // skinny tiles are not in this plan
  if (skinny && part == 0 && threadIdx.x == 0) {
    const int T = use_skinny ? s_short[E] * n_tiles_n : 0;
    skinny[0] = T;
    skinny[1] = ns_wgs;
    skinny[2] = (T + 7) / 8;
    skinny[3] = s_tail_q;
    skinny[4] = s_tail_inside;
    // most 256-row tiles a persistent workgroup runs (full rounds; a split last round goes elsewhere)
    const int cus_x = rq.cus / 8 - ns_wgs;
    const int per_x = ((use_skinny ? s_long[E] : s_long[E] + s_short[E]) * n_tiles_n + 7) / 8;
    const int rounds = cus_x > 0 ? (per_x + cus_x - 1) / cus_x : 1;
    skinny[5] = rounds > 0 ? rounds : 1;
  }
  const int per_long = (total_long + 7) / 8;
  const int per_short = (total_short + 7) / 8;
  const int S = s_parts;
  // idle entries: slot j of XCD x holds a tile while j < used_x (and j < full_x when the last
  // round is split off); tail entry x + 8 * (i * S + s) while i < used_x - full_x
  for (int b = threadIdx.x + part * blockDim.x; b < wgs; b += blockDim.x * nparts) {
    const int x = b & 7, j = b >> 3;
    if (j >= s_used[x] || j >= s_full[x]) entry[b] = int4v{-1, 0, 0, 0};
  }
  if (tail && part == 0)
    for (int b = threadIdx.x; b < kTailMaxParts; b += blockDim.x) {
      const int x = b & 7;
      if (!S || (b >> 3) / S >= s_used[x] - s_full[x]) tent[b] = int4v{-1, 0, 0, 0};
    }
  // slot j of XCD x: into the plan, or cut into S parts on the tail list
  auto place = [&](int j, int x, int4v v) {
    const int b = j * 8 + x;
    if (j >= s_full[x]) {
      const int i = j - s_full[x];
      for (int part = 0; part < S; ++part)
        tent[x + 8 * (i * S + part)] = int4v{v[0], v[1], v[2], v[3] | (part << 16) | (S << 24)};
    } else if (b < wgs) {
      entry[b] = v;
    }
  };
  // A wavefront per expert; with more wavefronts than experts (few experts), `sub_n` wavefronts share an
  // expert's entries.
  const int lane = threadIdx.x & 63, nwave = (blockDim.x >> 6) * nparts;
  const int wave = (threadIdx.x >> 6) * nparts + part;          // interleaved over the workgroups
  const int sub_n = nwave >= 2 * E ? nwave / E : 1;
  const int takers = sub_n > 1 ? sub_n * E : nwave;             // wavefronts that take entries
  const int sub = sub_n > 1 ? wave / E : 0;
  const int l0 = lane + 64 * sub, l_step = 64 * sub_n;
  // per-entry divisions by divisors that are the same for the whole workgroup
  const FastDiv by_run(kOrderGroupM * n_tiles_n), by_long(per_long > 0 ? per_long : 1), by_short(per_short > 0 ? per_short : 1);
  for (int e = sub_n > 1 ? wave % E : wave; wave < takers && e < E; e += nwave) {
    const int lo = s_off[e];
    int cnt = s_off[e + 1] - lo;
    cnt = cnt > 0 ? cnt : 0;
    const int nl = s_long[e + 1] - s_long[e];
    const int ns = s_short[e + 1] - s_short[e];
    // Launch order of an expert's long tiles: runs of up to kOrderGroupM M
    // tiles, and inside a run the M tile varies fastest.  The ~32 workgroups an
    // XCD runs at a time (consecutive logical ids) then form a patch of a M
    // tiles x 32/a N tiles of ONE expert: a weight tile is pulled from HBM once
    // for a M tiles, a token tile once for 32/a N tiles, and HBM traffic per
    // patch, which goes as 1/a + a/32, is near its minimum for a = 4..8.
    const int first = s_long[e] * n_tiles_n;
    const int cnt_long = (use_skinny && ns) ? cnt - rem_of(cnt) : cnt;   // rows the 256-row tiles hold
    for (int l = l0; l < nl * n_tiles_n; l += l_step) {
      const int run = by_run.div(l);                             // which run of M tiles
      const int run_first = run * kOrderGroupM;
      const int run_size = (nl - run_first) < kOrderGroupM ? (nl - run_first) : kOrderGroupM;
      const int in_run = l - run * kOrderGroupM * n_tiles_n;
      const int tn = FastDiv(run_size).div(in_run);
      const int i = run_first + (in_run - tn * run_size);        // M tile within the expert
      const int logical = first + l;
      int first_row, rows;
      tile_rows(cnt_long, nl, i, BM, first_row, rows);
      const int x = by_long.div(logical);
      place(logical - x * per_long, x, int4v{e, lo + first_row, rows, tn});   // hardware id = slot * 8 + XCD
    }
    if (ns && use_skinny) {
      int4v *sk = reinterpret_cast<int4v *>(skinny + kSkinnyHead);
      const int first_s = s_short[e] * n_tiles_n;
      for (int m = 0; m < ns; ++m) {                             // one or two skinny M tiles
        const int r0 = cnt_long + m * kSkinnyRows;
        const int rows = (cnt - r0) < kSkinnyRows ? (cnt - r0) : kSkinnyRows;
        for (int tn = l0; tn < n_tiles_n; tn += l_step) sk[first_s + m * n_tiles_n + tn] = int4v{e, lo + r0, rows, tn};
      }
    } else if (ns) {
      const int i = nl;                                          // the expert's last M tile
      const int first_s = s_short[e] * n_tiles_n;
      for (int tn = l0; tn < n_tiles_n; tn += l_step) {
        const int logical = first_s + tn;
        const int x = by_short.div(logical);
        int nl_x = total_long - x * per_long;              // long tiles on this XCD
        nl_x = nl_x < 0 ? 0 : (nl_x > per_long ? per_long : nl_x);
        place(nl_x + (logical - x * per_short), x, int4v{e, lo + i * BM, cnt - i * BM, tn});
      }
    }
  }
}

// ---- the layer's forward call: plans built by the routing stage ------------------
// ffn.hip
// Snapshot of the tuning knobs (ccf_set_option) that a grouped GEMM's plan and launches depend on.
struct GemmOptions {
  int variant, split_tail, split_tail_min_kt, split_max_parts, skinny_pct, fused_combine, skinny_tail;
};
GemmOptions forward_options();
bool forward_plan_request(int which, int max_rows, int E, int d, int f, void *workspace, const GemmOptions &opt,
                          PlanReq *out);
int ffn1_forward(const void *x, const int32_t *src_row, const int32_t *dst_row, const int32_t *offsets,
                 int max_rows, int num_expert, int d_model, int d_ffn, const void *w1, const void *b1,
                 int apply_gelu, void *h, void *workspace, size_t workspace_bytes, hipStream_t stream,
                 const GemmOptions *planned);   // planned: the options the plan in the workspace was built under, or NULL
int ffn2_forward(const void *h, const int32_t *src_row, const int32_t *dst_row, const int32_t *offsets,
                 int max_rows, int num_expert, int d_model, int d_ffn, const void *w2, const void *b2,
                 const void *row_scale, void *y, void *workspace, size_t workspace_bytes,
                 hipStream_t stream, const GemmOptions *planned);
int ffn2_forward_combine(const void *h, const int32_t *token_row, const int32_t *flat_row, const int32_t *offsets,
                         int max_rows, int num_expert, int d_model, int d_ffn, const void *w2, const void *b2,
                         const void *score, void *out, void *workspace, size_t workspace_bytes, hipStream_t stream,
                         const GemmOptions *planned);
// bwd.hip: the padded K ranges and row blocks of a backward call; the same launch builds the tile plan of its
// input-gradient GEMM (`rows_plan`, from the offsets) and of its weight-gradient GEMM (`w_plan`: every expert
// has seg_rows output rows) when given.
int launch_kseg(const int32_t *offsets, int E, int max_rows, int seg_rows, int n_blk, int32_t *k_seg,
                int32_t *row_off, int32_t *blk_row0, int32_t *blk_cnt, int32_t *row_lo, half_t *zero_row,
                const PlanReq *rows_plan, const PlanReq *w_plan, hipStream_t stream);

// route.hip: ccf_route(), whose last launch also builds n_plans (0..2) tile plans from the offsets.  gate_row_len > 0:
// the head of the workspace already holds the gate kernel's counts, one row per gate_row_len flat indices.
int route_with_plans(const int64_t *gate_idx, int n_flat, int num_expert, int top_k, int capacity,
                     int32_t *counts, int32_t *offsets, int64_t *pos, int32_t *src_row, int32_t *dst_row,
                     int32_t *inv_pos, int64_t *idx_kept, void *workspace, size_t workspace_bytes,
                     hipStream_t stream, const PlanReq *plans, int n_plans, int gate_row_len);
// route.hip: ccf_segments_to_rows(), whose launch also builds n_plans (0..2) tile plans
int segments_with_plans(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_expert, int n_seg,
                        int num_expert, int total_rows, int32_t *counts, int32_t *offsets, int32_t *rows,
                        hipStream_t stream, const PlanReq *plans, int n_plans);
// most entries of a table of per-run expert counts that the routing stage takes from the gate kernel
long long route_rows_max_ints();

}  // namespace ccf
