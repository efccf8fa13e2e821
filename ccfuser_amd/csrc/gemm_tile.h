// Grouped fp16 GEMM main loop for gfx950 (MI355X): C[m, n] = sum_k A[m, k] * B[n, k].
//
// Both operands are K-contiguous ("NT"): A rows are token rows reached through
// an optional row index (the scatter of the MoE layer fused into the tile
// load), B rows are the rows of one expert's weight matrix exactly as the
// reference stores it ([out, in], mix_moe/mix_moe/linear.py:198).  The
// reference's tile kernel (mix_moe/csrc/cuda/mix_gemm.cu:22-244) is a 64x512
// WMMA tile with fp16 accumulators fed by cp.async; this one is built for
// CDNA4 instead:
//
//   * v_mfma_f32_16x16x32_f16, fp32 accumulators in named accumulation
//     registers, 64-lane wavefronts;
//   * tiles go HBM/L2 -> LDS with global_load_lds_dwordx4 (no VGPR staging);
//     the LDS image is forced to be linear in lane order, so the XOR swizzle
//     that keeps ds_read_b128 conflict-free is applied on the global side:
//     the lane that owns LDS slot (row, c') fetches K-chunk c' ^ swz(row);
//   * the A half and the B half of a K tile are slots of a five-slot LDS ring,
//     one workgroup barrier per K tile, in the middle of the tile.
#pragma once

#include "ccf_common.h"

#include <type_traits>

namespace ccf {

// ---- LDS layout ------------------------------------------------------------
// A tile of ROWS x BK halves is ROWS x (BK/8) 16-byte chunks.  Row r, K-chunk c
// lives at byte (r * CPR + (c ^ swz(r))) * 16.  swz depends on r & 15 only, so
// rows 16 apart share it and the per-lane read addresses of the MFMA blocks of
// a wavefront differ by compile-time constants.
template <int CPR>
__device__ __forceinline__ int swz(int r) {
  static_assert(CPR == 8 || CPR == 4, "swizzle written for BK = 64 and BK = 32");
  if constexpr (CPR == 8) {
    // 128-byte rows, so a row's parity picks the half of the 64 banks and chunk ^
    // swz the 16-byte slot in that half.  ds_read_b128 serves 16 lanes per
    // cycle, and not consecutive ones: lanes {0-3, 12-15, 20-23, 24-27} share a
    // cycle, then {4-7, 8-11, 16-19, 28-31}, and the same again 32 lanes up
    // (measured with the bank-conflict counter on lane pairs).  For the
    // 32x32x16 operand (lane l: row l%32, one chunk per half-wave) such a group
    // holds eight even and eight odd rows of one chunk, so swz must be a
    // bijection on the even rows 0..14 and on the odd rows.  For the 16x16x32
    // operand (lane l: row l%16, chunk l/16) it holds rows {0-3, 12-15} of one
    // chunk and rows {4-11} of the chunk that differs in bit 0, so swz ^ [4 <=
    // r%16 < 12] must be such a bijection as well.  (r >> 1) ^ [4 <= r%16 < 12]
    // is both.
    return ((r >> 1) & 7) ^ (((r >> 2) ^ (r >> 3)) & 1);
  } else {
    // 64-byte rows: two rows per 128 bytes; bits of the result are
    // (r>>2)&1 and ((r>>3)^(r>>1))&1
    return (((r >> 2) & 1) << 1) | (((r >> 3) ^ (r >> 1)) & 1);
  }
}

typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) const half8 lds_half8;

template <int S, int BYTES>
__device__ __forceinline__ lds_char *stage_buf() {
  __shared__ __attribute__((aligned(1024))) char buf[BYTES];
  return (lds_char *)buf;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Workgroup barrier without the memory fence __syncthreads() carries: that
// fence makes the compiler drain every tile load in flight (vmcnt(0)), which
// defeats multi-stage buffering.  The callers order their own LDS traffic: the
// tile loads are waited for with wait_vmcnt, the LDS reads have returned
// before the MFMAs that consume them issue.
__device__ __forceinline__ void block_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// Wait until at most N LDS reads are in flight.  The two fragments the next
// MFMA consumes are tied to the wait as in/out operands, so the MFMA cannot be
// scheduled ahead of it.
template <int N>
__device__ __forceinline__ void wait_lgkmcnt(half8 &x, half8 &y) {
  static_assert(N >= 0, "lgkmcnt");
  if constexpr (N < 15) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N));
  } else {
    // the counter has four bits: more than 15 LDS reads are never in flight,
    // so "at most 15" always holds; keep the ordering tie only
    asm volatile("" : "+v"(x), "+v"(y));
  }
}

// 16 bytes per lane from LDS byte address addr + OFF.
template <int OFF>
__device__ __forceinline__ half8 lds_read_b128(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "ds offset");
  half8 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

// 8 bytes per lane from LDS byte address addr + OFF, transposed inside each group
// of 16 lanes: with source lane j = 4*i + r (i, r in 0..3) holding four 16-bit
// elements c = 0..3, lane 4*r + c receives element c of source lanes r, 4 + r,
// 8 + r, 12 + r (measured).  When source lane 4*i + r points at row i, columns
// 4*r .. 4*r+3 of a row-major matrix, lane l receives rows 0..3 of column l:
// four consecutive K elements of a [K][N] operand for the MFMA lane of column l.
template <int OFF>
__device__ __forceinline__ half4 lds_read_tr_b64(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "ds offset");
  half4 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

__device__ __forceinline__ void lds_dma16(const void *gptr, lds_char *lds_wave_base) {
  // 64 lanes x 16 bytes land at lds_wave_base + lane * 16.
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gptr,
                                   (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}

// threadIdx.x as a value the compiler cannot trace back: what is derived from it
// is computed where it is used, not once at kernel start and then held in
// registers across the main loop (the persistent kernel has none to spare).
__device__ __forceinline__ int fresh_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// Tile shape (BM x BN x BK), wavefront grid (WM x WN) and the pacing of the tile loads.
template <int BM_, int BN_, int BK_, int WM_, int WN_, int DMA_EVERY_>
struct GemmCfg {
  static constexpr int DMA_EVERY = DMA_EVERY_;         // one tile load behind every n-th MFMA
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int NW = WM * WN;
  static constexpr int MIN_WAVES_PER_SIMD = (NW + 3) / 4;   // register budget
  static constexpr int THREADS = NW * 64;
  static constexpr int WTM = BM / WM, WTN = BN / WN;   // wavefront tile
  static constexpr int CPR = BK / 8;                   // 16-byte chunks per tile row
  static constexpr int ROWS_PER_DMA = 64 / CPR;        // tile rows one wavefront load covers
  static constexpr int A_DMA = BM / ROWS_PER_DMA / NW; // loads per wavefront per tile
  static constexpr int B_DMA = BN / ROWS_PER_DMA / NW;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "wavefront tile");
  static_assert(BM % (ROWS_PER_DMA * NW) == 0 && BN % (ROWS_PER_DMA * NW) == 0, "dma split");
};

// Which rows of a tile, and which 16-byte K chunk of them, a lane fetches with its tile loads.
template <class Cfg>
struct GemmMainloop {
  // Tile row this lane fetches with its i-th A (or B) load, and the K-chunk.
  // tid: threadIdx.x, or fresh_tid() where the values derived from it must not
  // be computed early and kept in registers.
  static __device__ __forceinline__ int dma_row(int i, int tid) {
    const int wave = tid >> 6, lane = tid & 63;
    return (i * Cfg::NW + wave) * Cfg::ROWS_PER_DMA + lane / Cfg::CPR;
  }
  static __device__ __forceinline__ int dma_chunk(int row, int tid) {
    const int lane = tid & 63;
    return (lane % Cfg::CPR) ^ swz<Cfg::CPR>(row);
  }
  static __device__ __forceinline__ int dma_row(int i) { return dma_row(i, threadIdx.x); }
  static __device__ __forceinline__ int dma_chunk(int row) { return dma_chunk(row, threadIdx.x); }
};

// ---- five-slot ring, v_mfma_f32_16x16x32_f16, barrier in mid-tile ----------------
// 256x256x64 tiles need 64 KB of LDS per K tile, so only two whole tiles fit in
// the CU's 160 KB, and with two whole-tile stages a tile's loads must all have
// landed before the next tile's can be issued: the memory pipe drains once per K
// tile (measured: 12 TB/s into LDS against 16 TB/s when loads of two tiles
// overlap).  Here the A half and the B half of a K tile are separate 32 KB slots
// of a ring of five; every load is a whole 128-byte line.
//
// * The MFMA is the 16x16x32 form.  It moves a quarter of the accumulator
//   registers per flop of the 32x32x16 form, and on data that is not constant
//   the chip is power-limited: measured MFMA-only throughput on random operands
//   is 1.95 PFLOP/s for 16x16x32 against 1.69 for 32x32x16.
// * A K tile is two K=32 substeps, and the operand fragments are double
//   buffered in registers, so every LDS read of tile k has been issued early
//   in substep 0.  The one workgroup barrier per K tile therefore sits BETWEEN
//   the substeps: behind it, tile k's slots are free for the loads of tile
//   k+2 and tile k+1 is complete, so substep 1 prefetches the fragments of
//   tile k+1 under its own MFMAs and no LDS latency is exposed at the tile
//   boundary (one wavefront per SIMD has nobody to hide it behind).
// * A(k+2) is loaded during substep 0 into the fifth slot, B(k+2) during
//   substep 1 into the slot A(k) just left; at the barrier only A(k+2) may
//   still be in flight.
//
// The ring phase (which slot holds what) is a run-time value: one step body
// serves every phase, the slot addresses are a few scalar adds per K tile, and a
// caller that runs tile after tile (the persistent kernel) simply carries the
// phase on.
//
// B_KN: the B operand is stored [K][N] (N contiguous) instead of [N][K].  Its
// half tile then sits in LDS as 64 K rows of BN columns (512 bytes each), and a
// lane's fragment (eight consecutive K of one column) comes from two transposing
// 8-byte reads, four rows apart.  The sixteen rows one such read touches
// (rows 8*g + i for the lane groups g and i = 0..3) would share banks, so the
// 32-byte chunk a row block occupies inside its 256-byte wavefront span is
// XORed with f(row) = row%4 + 4*((row/8)%2): two cycles per read, the minimum
// for 512 bytes.  The XOR sits in address bits 5..7, the column block tn in the
// same bits, so a fragment's address is the lane's base address XOR 32*tn.
//
// ROLL_A (the eight-wavefront form: two wavefronts per SIMD, 128 vector and 128 accumulation
// registers each): the token fragments have ONE register buffer instead of two.  The MFMAs
// of a substep run row block by row block, and as soon as a row block's last MFMA has issued,
// its fragment registers take the NEXT substep's fragment of that row block.  The reads still
// leave during the substep before their use, so the ring schedule above is unchanged; what
// changes is that a row block's new fragment has one substep less one row block of lead
// instead of a whole substep, which the second wavefront of the SIMD covers.
//
// A_KM (with B_KN): the A operand is stored [K][M] as well, read through the same transposing
// reads, and K rows at or past a per-lane limit are fetched from a row of zeros instead (KMask):
// the form of a weight gradient, whose contraction runs over an expert's rows of two row-major
// activation matrices, any number of rows.
template <class Cfg, bool B_KN = false, bool ROLL_A = false, bool A_KM = false>
struct Ring16Mainloop {
  using acc_t = float4v;
  static constexpr int AB = ROLL_A ? 1 : 2;                      // register buffers of the token fragments
  static_assert(!A_KM || (B_KN && !ROLL_A && Cfg::WTM == 128 && Cfg::A_DMA % 2 == 0 && Cfg::BM == Cfg::BN),
                "the [K][M] form of A mirrors the [K][N] form of B");
  static constexpr int A_SRCS = A_KM ? 2 : Cfg::A_DMA;
  // Tile load l of a [K][*] operand fetches K row 8 l + own (own < 8 fixed per lane) of the K tile; with
  // klim = (rows of the contraction) - own, that row exists while (first K row of the tile) + 8 l < klim.
  struct KMask {
    int klim;
    const half_t *zero;        // this lane's 16 bytes of a row of zeros
  };
  static constexpr int KN_PITCH = Cfg::BN * 2;                   // bytes per K row of a [K][N] half tile
  // Source pointers a lane holds for its B tile loads.  [N][K]: one per load.  [K][N]: load i
  // fetches K row 8*i + r0 (r0 < 8 fixed per lane), whose chunk XOR depends on i%2 only, so
  // b_src[i] = b_src2[i % 2] + (i / 2) * 16 rows: two pointers and a scalar offset.
  static constexpr int B_SRCS = B_KN ? 2 : Cfg::B_DMA;
  static_assert(!B_KN || (Cfg::NW == 4 && Cfg::B_DMA % 2 == 0), "[K][N] load pattern");
  static_assert(!B_KN || (Cfg::WTN == 128 && Cfg::BN * Cfg::BK * 2 == Cfg::B_BYTES), "[K][N] layout is written for 128-column wavefront tiles");
  static_assert(Cfg::BK == 64, "two K=32 substeps per K tile");
  static_assert(Cfg::A_BYTES == Cfg::B_BYTES, "ring slots are one size");
  static constexpr int NSLOT = 5;
  static constexpr int SLOT_BYTES = Cfg::A_BYTES;
  static constexpr int TM = Cfg::WTM / 16, TN = Cfg::WTN / 16;   // 16x16 blocks per wavefront
  static constexpr int FRAGS = TM + TN;
  static constexpr int PER_SUB = TM * TN;                        // MFMAs per substep
  // A fragment read goes out behind every READ_EVERY-th MFMA of a substep, a tile
  // load behind every DMA_EVERY-th (measured: spreading both over the substep is
  // ~1 % faster than issuing them back to back at its start).
  static constexpr int READ_EVERY = 2;
  static_assert(PER_SUB >= FRAGS * READ_EVERY, "not enough MFMA slots for the fragment reads");
  static_assert((Cfg::A_DMA - 1) * Cfg::DMA_EVERY + 1 < PER_SUB && (Cfg::B_DMA - 1) * Cfg::DMA_EVERY + 1 < PER_SUB,
                "not enough MFMA slots for the tile loads");

  // One LDS object; slot s is bytes [s * SLOT_BYTES, (s + 1) * SLOT_BYTES).
  static __device__ __forceinline__ lds_char *lds() { return stage_buf<200, NSLOT * SLOT_BYTES>(); }
  static __device__ __forceinline__ uint32_t lds_addr() {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds()));
  }
  // (x mod 5) for 0 <= x < 10
  static __device__ __forceinline__ int mod5(int x) { return x >= NSLOT ? x - NSLOT : x; }

  // Slots of ring phase ph (0..4): K tile kt in a/b, kt+1 in na/nb, A(kt+2) goes to wa, B(kt+2) to a.
  struct Slots {
    int a, b, na, nb, wa;   // byte offsets into lds()
  };
  static __device__ __forceinline__ Slots slots_of(int ph) {
    Slots s;
    const int x = mod5(2 * ph);                      // 2*ph mod 5
    s.a = x * SLOT_BYTES;
    s.b = mod5(x + 1) * SLOT_BYTES;
    s.na = mod5(x + 2) * SLOT_BYTES;
    s.nb = mod5(x + 3) * SLOT_BYTES;
    s.wa = mod5(x + 4) * SLOT_BYTES;
    return s;
  }

  // Source of tile load l: src[l] + k_elem, or for the two-pointer form of a [K][N] operand
  // src[l % 2] + k_elem + (l / 2) * 16 K rows of bmul elements.
  template <bool KN2, int N>
  static __device__ __forceinline__ const half_t *load_src(const half_t *const (&src)[N], int l, int k_elem, int bmul) {
    if constexpr (KN2) {
      return src[l & 1] + (k_elem + (l >> 1) * 16 * bmul);
    } else {
      return src[l] + k_elem;
    }
  }
  // The same with the K mask of the A_KM form: krow = first K row of the tile being loaded.
  template <bool KN2, int N>
  static __device__ __forceinline__ const half_t *load_src_m(const half_t *const (&src)[N], int l, int k_elem, int mul,
                                                             int krow, const KMask &mk) {
    const half_t *p = load_src<KN2>(src, l, k_elem, mul);
    if constexpr (A_KM) p = (krow + 8 * l < mk.klim) ? p : mk.zero;
    return p;
  }
  template <bool KN2, int NLOAD, int N>
  static __device__ __forceinline__ void issue_all(const half_t *const (&src)[N], int k_elem, int slot_off, int wave,
                                                   int bmul = 1, int krow = 0, const KMask &mk = KMask{0, nullptr}) {
    static_for<0, NLOAD>([&](auto I) {
      lds_dma16(load_src_m<KN2>(src, I.value, k_elem, bmul, krow, mk), lds() + slot_off + (I.value * Cfg::NW + wave) * 1024);
    });
  }

  // Fragment I of a substep: the weight fragments first, then the token fragments.
  // ra / rb: LDS address of this lane's chunk of row block 0 in the slots read from.
  template <int I>
  static __device__ __forceinline__ void read_frag(half8 (&a)[TM], half8 (&b)[TN], uint32_t ra, uint32_t rb) {
    if constexpr (I < TN) {
      if constexpr (B_KN) {
        const uint32_t addr = rb ^ (I * 32);
        const half4 lo = lds_read_tr_b64<0>(addr);
        const half4 hi = lds_read_tr_b64<4 * KN_PITCH>(addr);
        b[I] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      } else {
        b[I] = lds_read_b128<I * 16 * Cfg::CPR * 16>(rb);
      }
    } else if constexpr (A_KM) {
      const uint32_t addr = ra ^ ((I - TN) * 32);
      const half4 lo = lds_read_tr_b64<0>(addr);
      const half4 hi = lds_read_tr_b64<4 * KN_PITCH>(addr);
      a[I - TN] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
      a[I - TN] = lds_read_b128<(I - TN) * 16 * Cfg::CPR * 16>(ra);
    }
  }

  // Every LDS read issued so far has returned; the fragments are tied to the
  // wait so that no MFMA reading them is scheduled ahead of it.
  static __device__ __forceinline__ void frags_ready(half8 (&a)[TM], half8 (&b)[TN]) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(a[i]));
#pragma unroll
    for (int i = 0; i < TN; ++i) asm volatile("" : "+v"(b[i]));
  }

  // The accumulators are not C++ objects: block (tm, tn) lives in the accumulation
  // registers a[4*(tm*TN+tn) .. +3], named literally in inline asm.  With 256
  // of them next to 128 fragment registers the register allocator otherwise
  // splits them between the two register files and copies them around inside
  // the loop (or spills) as soon as the control flow is more than one loop.
  // The file is compiled with VGPR-to-AGPR spilling off, so nothing else ever
  // lives there; reserve() makes the kernel own all 256.  Being opaque, the
  // MFMAs get no hazard padding from the compiler: callers keep the required
  // distance to any other instruction that touches an accumulator (settle()).
  static_assert(TM * TN * 4 <= 256, "accumulation registers");
  static __device__ __forceinline__ void reserve() {
    static_assert(TM * TN * 4 == 256 || TM * TN * 4 == 128, "accumulation registers owned by the kernel");
    if constexpr (TM * TN * 4 == 256) asm volatile("" ::: "a255");
    else asm volatile("" ::: "a127");
  }
  // acc(tm, tn) += w (16 weight rows) x t (16 token rows), K = 32
  template <int BLK>
  static __device__ __forceinline__ void mfma16(const half8 &w, const half8 &t) {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, a[%2:%3]"
                 :
                 : "v"(w), "v"(t), "n"(4 * BLK), "n"(4 * BLK + 3));
  }
  static __device__ __forceinline__ void zero_acc() {
    static_for<0, TM * TN * 4>([&](auto R_) { asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(R_.value)); });
  }
  // element c (0..3) of block (tm, tn)
  template <int TM_, int TN_, int C>
  static __device__ __forceinline__ float acc_get() {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"((TM_ * TN + TN_) * 4 + C));
    return v;
  }
  // Distance between an MFMA and the first other reader or writer of an
  // accumulator, or the other way round (a 4-pass MFMA needs at most 11 wait
  // states; this is 32).
  static __device__ __forceinline__ void acc_settle() { asm volatile("s_nop 15\n s_nop 15" ::: "memory"); }

  // One substep: PER_SUB MFMAs on fragment buffer SUB; interleaved with them the
  // reads of the NEXT substep's fragments (LDS addresses ra, rb) into the other
  // buffer and the tile loads into the slot at byte offset ws.
  template <int SUB, int NLOAD, bool FULL, bool KN2 = false, int NSRC>
  static __device__ __forceinline__ void substep(half8 (&a)[AB][TM], half8 (&b)[2][TN],
                                                 const half_t *const (&src)[NSRC], int k_elem, uint32_t ra,
                                                 uint32_t rb, int ws, int wave, int live_m, int bmul = 1, int krow = 0,
                                                 const KMask &mk = KMask{0, nullptr}) {
    constexpr int AS = ROLL_A ? 0 : SUB, AN = ROLL_A ? 0 : SUB ^ 1;     // token fragment buffer in use / being filled
    // what goes out behind MFMA i
    auto behind = [&](auto II) {
      constexpr int i = II.value;
      if constexpr (ROLL_A) {
        // weight fragments early; a row block's token fragment when its last MFMA of this substep has issued
        if constexpr (i % READ_EVERY == 0 && i / READ_EVERY < TN) read_frag<i / READ_EVERY>(a[AN], b[SUB ^ 1], ra, rb);
        if constexpr (i % TN == TN - 1) read_frag<TN + i / TN>(a[AN], b[SUB ^ 1], ra, rb);
      } else if constexpr (i % READ_EVERY == 0 && i / READ_EVERY < FRAGS) {
        read_frag<i / READ_EVERY>(a[AN], b[SUB ^ 1], ra, rb);
      }
      if constexpr (i % Cfg::DMA_EVERY == 1 && i / Cfg::DMA_EVERY < NLOAD) {
        constexpr int l = i / Cfg::DMA_EVERY;
        lds_dma16(load_src_m<KN2>(src, l, k_elem, bmul, krow, mk), lds() + ws + (l * Cfg::NW + wave) * 1024);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    static_for<0, TM>([&](auto T) {
      constexpr int tm = T.value;
      // one (wavefront-uniform) branch per row block, not per MFMA
      if (FULL || tm < live_m) {
        static_for<0, TN>([&](auto J) {
          constexpr int tn = J.value;
          mfma16<tm * TN + tn>(b[SUB][tn], a[AS][tm]);
          behind(std::integral_constant<int, tm * TN + tn>{});
        });
      } else {
        static_for<0, TN>([&](auto J) { behind(std::integral_constant<int, tm * TN + J.value>{}); });
      }
    });
  }

  // K tile kt in ring phase ph; k2 / kb2: element offset from the A / B sources of the K
  // tile that the loads of this step fetch (A into the fifth slot, B into the slot A(kt) leaves);
  // krow: that tile's first K row (for the K mask of the A_KM form).
  template <bool FULL>
  static __device__ __forceinline__ void step(half8 (&a)[AB][TM], half8 (&b)[2][TN],
                                              const half_t *const (&a_src)[A_SRCS],
                                              const half_t *const (&b_src)[B_SRCS], const int (&a_off)[2],
                                              const int (&b_off)[2], int k2, int kb2, int ph, int wave, int live_m, int bmul,
                                              int amul = 1, int krow = 0, const KMask &mk = KMask{0, nullptr}) {
    const Slots s = slots_of(ph);
    const uint32_t base = lds_addr();
    frags_ready(a[0], b[0]);
    __builtin_amdgcn_sched_barrier(0);
    // K half 0; fetch the fragments of K half 1 of this tile; load A(kt+2)
    substep<0, Cfg::A_DMA, FULL, A_KM>(a, b, a_src, k2, base + s.a + a_off[1], base + s.b + b_off[1], s.wa, wave,
                                       live_m, amul, krow, mk);
    // B(kt+1) and everything older have landed; A(kt+2) may stay in flight
    wait_vmcnt<Cfg::A_DMA>();
    block_barrier();
    frags_ready(a[AB - 1], b[1]);
    __builtin_amdgcn_sched_barrier(0);
    // K half 1; fetch the fragments of K half 0 of tile kt+1; load B(kt+2) into A(kt)'s slot
    substep<1, Cfg::B_DMA, FULL, B_KN>(a, b, b_src, kb2, base + s.na + a_off[0], base + s.nb + b_off[0], s.a, wave,
                                       live_m, bmul, krow, mk);
  }

  // `steps` consecutive K-tile steps starting in ring phase `phase` (updated).
  // Step i loads the K tile at element offset min(k2_first + i*BK, k2_max); bmul / amul: elements
  // between consecutive K rows of a [K][N] B / [K][M] A operand.
  template <bool FULL>
  static __device__ __forceinline__ void k_range(half8 (&a)[AB][TM], half8 (&b)[2][TN],
                                                 const half_t *const (&a_src)[A_SRCS],
                                                 const half_t *const (&b_src)[B_SRCS], const int (&a_off)[2],
                                                 const int (&b_off)[2], int steps, int k2_first, int k2_max,
                                                 int &phase, int wave, int live_m, int bmul = 1, int amul = 1,
                                                 const KMask &mk = KMask{0, nullptr}) {
    int ph = phase;
    int k2 = k2_first;
    for (int i = 0; i < steps; ++i) {
      const int kc = k2 < k2_max ? k2 : k2_max;
      step<FULL>(a, b, a_src, b_src, a_off, b_off, A_KM ? kc * amul : kc, B_KN ? kc * bmul : kc, ph, wave, live_m, bmul,
                 amul, kc, mk);
      k2 += Cfg::BK;
      ph = ph == NSLOT - 1 ? 0 : ph + 1;
    }
    phase = ph;
  }

  // Byte offsets in a slot of this lane's operand chunk of row block 0, per K half:
  // lane l of a 16x16x32 operand holds row l%16, K elements 8*(l/16) .. +7 of the 32.
  static __device__ __forceinline__ void frag_offsets(int (&a_off)[2], int (&b_off)[2]) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int ra = (wave / Cfg::WN) * Cfg::WTM + (lane & 15);
    const int rb = (wave % Cfg::WN) * Cfg::WTN + (lane & 15);
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int c = sub * 4 + (lane >> 4);
      if constexpr (A_KM) {
        const int j = lane & 15;
        const int row = sub * 32 + 8 * (lane >> 4) + (j >> 2);
        a_off[sub] = row * KN_PITCH + (wave / Cfg::WN) * (Cfg::WTM * 2) + (kn_swz(row) << 5) + ((j & 3) << 3);
      } else {
        a_off[sub] = (ra * Cfg::CPR + (c ^ swz<Cfg::CPR>(ra))) * 16;
      }
      if constexpr (B_KN) {
        // source lane j of its group of 16 points at K row 8*group + j/4, columns 4*(j%4) ..
        const int j = lane & 15;
        const int row = sub * 32 + 8 * (lane >> 4) + (j >> 2);
        b_off[sub] = row * KN_PITCH + (wave % Cfg::WN) * (Cfg::WTN * 2) + (kn_swz(row) << 5) + ((j & 3) << 3);
      } else {
        b_off[sub] = (rb * Cfg::CPR + (c ^ swz<Cfg::CPR>(rb))) * 16;
      }
    }
  }
  // 32-byte chunk XOR of K row `row` of a [K][N] half tile
  static __device__ __forceinline__ int kn_swz(int row) { return (row & 3) | (((row >> 3) & 1) << 2); }
  // Global column (elements, inside the tile's BN columns) that LDS position
  // (row, 16-byte unit u of the row) of a [K][N] half tile holds.
  static __device__ __forceinline__ int kn_col(int row, int u) {
    const int chunk = u >> 1;                                     // 32-byte chunk of the row
    return (chunk >> 3) * Cfg::WTN + (((chunk & 7) ^ kn_swz(row)) << 4) + ((u & 1) << 3);
  }
  // K row and 16-byte unit of tile load i of this lane for a [K][N] half tile (two rows per load).
  static __device__ __forceinline__ int kn_dma_row(int i, int tid) { return 2 * (i * Cfg::NW + (tid >> 6)) + ((tid & 63) >> 5); }
  static __device__ __forceinline__ int kn_dma_unit(int tid) { return tid & 31; }

  // The tile's rows [0, rows) are split between the two rows of wavefronts: the
  // first (rows+1)/2 sit in tile rows 0 .., the rest in tile rows WTM .., so a
  // partly filled tile has padding, and skips MFMAs, in both halves.
  static_assert(Cfg::WM == 2, "row split written for two rows of wavefronts");
  static __device__ __forceinline__ int local_row(int r, int rows) {
    const int h0 = (rows + 1) >> 1, h1 = rows - h0;
    const int q = r - Cfg::WTM;
    return r < Cfg::WTM ? (r < h0 ? r : h0 - 1) : (q < h1 ? h0 + q : rows - 1);
  }
  static __device__ __forceinline__ bool row_is_real(int r, int rows) {
    const int h0 = (rows + 1) >> 1, h1 = rows - h0;
    return r < Cfg::WTM ? r < h0 : r - Cfg::WTM < h1;
  }
  // 16-row blocks of this wavefront that hold real rows of an M tile with `rows` rows.
  static __device__ __forceinline__ int live_blocks(int rows) {
    const int wm = (threadIdx.x >> 6) / Cfg::WN;
    const int h0 = (rows + 1) >> 1;
    const int mine = wm == 0 ? h0 : rows - h0;
    int live_m = (mine + 15) / 16;
    live_m = live_m > TM ? TM : live_m;
    return __builtin_amdgcn_readfirstlane(live_m);
  }

  // Phase 0: A(0) -> slot 0, B(0) -> slot 1, A(1) -> slot 2, B(1) -> slot 3, then
  // the fragments of K half 0 of tile 0 into a[0], b[0].
  static __device__ __forceinline__ void prologue(half8 (&a)[AB][TM], half8 (&b)[2][TN],
                                                  const half_t *const (&a_src)[A_SRCS],
                                                  const half_t *const (&b_src)[B_SRCS], int KT,
                                                  const int (&a_off)[2], const int (&b_off)[2], int wave,
                                                  int bmul = 1, int amul = 1, const KMask &mk = KMask{0, nullptr}) {
    const int k1 = (KT > 1 ? 1 : 0) * Cfg::BK;
    issue_all<A_KM, Cfg::A_DMA>(a_src, 0, 0 * SLOT_BYTES, wave, amul, 0, mk);
    issue_all<B_KN, Cfg::B_DMA>(b_src, 0, 1 * SLOT_BYTES, wave, bmul, 0, mk);
    issue_all<A_KM, Cfg::A_DMA>(a_src, A_KM ? k1 * amul : k1, 2 * SLOT_BYTES, wave, amul, k1, mk);
    issue_all<B_KN, Cfg::B_DMA>(b_src, B_KN ? k1 * bmul : k1, 3 * SLOT_BYTES, wave, bmul, k1, mk);
    wait_vmcnt<Cfg::A_DMA + Cfg::B_DMA>();
    block_barrier();
    const uint32_t ra = lds_addr() + a_off[0], rb = lds_addr() + SLOT_BYTES + b_off[0];
    static_for<0, FRAGS>([&](auto I) { read_frag<I.value>(a[0], b[0], ra, rb); });
  }

  // rows: real rows of this M tile (1..BM).
  static __device__ __forceinline__ void run(const half_t *const (&a_src)[Cfg::A_DMA],
                                             const half_t *const (&b_src)[B_SRCS], int K, int rows,
                                             int bmul = 1) {
    static_assert(!A_KM, "the [K][M] form runs in the persistent kernel only");
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int KT = K / Cfg::BK;
    const int live_m = live_blocks(rows);
    int a_off[2], b_off[2];
    frag_offsets(a_off, b_off);
    half8 a[AB][TM], b[2][TN];
    prologue(a, b, a_src, b_src, KT, a_off, b_off, wave, bmul);
    int phase = 0;
    reserve();
    zero_acc();
    acc_settle();
    // past the end of K the last K tile is fetched again into slots nobody reads
    if (live_m == TM) {
      k_range<true>(a, b, a_src, b_src, a_off, b_off, KT, 2 * Cfg::BK, (KT - 1) * Cfg::BK, phase, wave, live_m, bmul);
    } else {
      k_range<false>(a, b, a_src, b_src, a_off, b_off, KT, 2 * Cfg::BK, (KT - 1) * Cfg::BK, phase, wave, live_m, bmul);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_vmcnt<0>();
    acc_settle();
  }
};

// Accumulator layout of the 16x16x32 form with the weight fragment first: a
// lane owns ONE token row per 16x16 block and four consecutive output columns:
//   row = wm*WTM + tm*16 + lane%16
//   col = wn*WTN + tn*16 + 4*(lane/16) + r
template <class Cfg>
__device__ __forceinline__ int acc16_row(int tm, int tid) {
  const int wave = tid >> 6, lane = tid & 63;
  return (wave / Cfg::WN) * Cfg::WTM + tm * 16 + (lane & 15);
}
template <class Cfg>
__device__ __forceinline__ int acc16_col4(int tn, int tid) {
  const int wave = tid >> 6, lane = tid & 63;
  return (wave % Cfg::WN) * Cfg::WTN + tn * 16 + 4 * (lane >> 4);
}

}  // namespace ccf
