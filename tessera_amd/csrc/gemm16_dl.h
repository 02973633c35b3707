// Main loop of the 16-bit GEMM tile on v_mfma_f32_16x16x32 with operands loaded from
// global memory STRAIGHT INTO LDS (buffer_load ... lds, 16 bytes per lane).
//
// An alternative to the register-staged 16-wide step of gemm16.h, selected at build time
// (TSR_BIG_DIRECT): no staging registers and no LDS write instructions.  It spends less power
// per FLOP than the 32-wide staged loop and beat it by 5-6 % on random operands, but a stage
// is free for exactly one K step, so its loads have at most that long to land, the matrix
// pipes idle a third of the time, and the staged 16-wide step measures 2 % faster still.
//
// LDS stage = A tile [BM][64] 16-bit (128-byte rows, 16-byte chunks XOR-swizzled by
// (row >> 1) & 7, as in the register-staged loop) + B tile(s) [64][cols] in natural row-major
// form WITHOUT padding, 16-byte chunks XOR-swizzled by 2 * ((k & 3) | ((k >> 3) & 1) << 2): a
// wave's transposing read touches rows {8g + r, r < 4} of four k groups g, 32 bytes each, and
// that swizzle puts the eight rows served together in eight different 32-byte bank slots.
// SwiGLU keeps the gate and the up half as two such sub-tiles, so that every wave
// instruction (1 KB = whole rows of one sub-tile) reads one source matrix.
// A load instruction fills 64 consecutive 16-byte slots; the swizzle is applied on the
// global address (the lane fetches the chunk that belongs in its slot).
//
// Pipeline (two LDS stages, one barrier per K step, KS = 2 MFMA k steps per K step).  The
// barrier sits between the two k steps: before it every wave has read all fragments of the
// current stage (those of the second k step are fetched during the first), after it the stage
// is free and takes the loads of K step kt+2, which are dealt out over the rows of the k step
// that follows the barrier and so have most of a K step to land before the next barrier
// (s_waitcnt vmcnt(0) just ahead of it; loads issued in the k step before that barrier would
// have no time left, and cost a quarter of the rate when tried).  The B fragments are double buffered in registers; the A fragment of a
// row is replaced by the same row's fragment of the next k step as soon as the row's MFMAs
// are issued.
#pragma once
#include <type_traits>
#include "common.h"

namespace tsr950 {

// 16 bytes per lane from a buffer straight into LDS: lane i's data lands at lds_base + 16 i
// (lds_base wave-uniform); an offset at or past the buffer's range stores zeros.  Inline
// assembly, so the compiler does not serialise LDS reads of the other stage behind it; the
// loop waits for these loads itself.
__device__ __forceinline__ void buffer_load16_to_lds(const void* base, uint32_t byte_off, uint32_t lds_base) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const i32x4 rsrc = {(int)(uint32_t)b, (int)(uint32_t)((b >> 32) & 0xffffu), (int)kBufferRange, 0x00020000};
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(lds_base), "v"(byte_off), "s"(rsrc) : "memory");
}
__device__ __forceinline__ void wait_direct_loads() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int BM, int BN>
struct Gemm16DlSmem {
  static constexpr int kAStage = BM * 128;
  static constexpr int kBStage = 64 * BN * 2;
  static constexpr int kStage = kAStage + kBStage;
  static constexpr int kBytes = 2 * kStage;
};

__device__ __forceinline__ int g16_dl_bswz(int krow) { return 2 * ((krow & 3) | (((krow >> 3) & 1) << 2)); }

template <class T, int BM, int BN, int WM, int WN, bool SWIGLU, bool GROUPED, class Acc, class Params>
__device__ __forceinline__ void gemm16_mainloop_dl(const Params& p, char* smem, Acc& acc, const int m_begin,
                                                   const int m_end, const int n_begin, const uint16_t* Ab,
                                                   const uint16_t* Bb, const uint16_t* B2b) {
  using S = Gemm16DlSmem<BM, BN>;
  constexpr int NT = WM * WN * 64;
  static_assert(NT == 256, "four waves");
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int MI = TM / 16, NJ = TN / 16;
  constexpr int BK = 64;
  constexpr int NSRC = SWIGLU ? 2 : 1;
  constexpr int SUBCOLS = BN / NSRC;             // columns of one B sub-tile
  constexpr int BP = SUBCOLS * 2;                // its row pitch in bytes
  constexpr int CPR = SUBCOLS / 8;               // 16-byte chunks per row
  constexpr int SUBBYTES = 64 * BP;
  static_assert(BP % 256 == 0 && CPR >= 16, "B rows must be whole bank lines and hold the swizzle");
  constexpr int A_Q = BM * 128 / 1024 / 4;       // A load instructions per wave and stage
  constexpr int B_Q = S::kBStage / 1024 / 4;     // B load instructions per wave and stage
  constexpr int IPS = SUBBYTES / 1024;           // instructions per sub-tile
  constexpr int RPI = 1024 / BP;                 // B rows per instruction
  static_assert(A_Q >= 1 && B_Q >= 1 && (4 * B_Q) % NSRC == 0, "tile too small for whole-wave loads");
  constexpr int NL = A_Q + B_Q;                  // load instructions per wave and K step

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int lm = lane & 15, lk = lane >> 4;
  const int K = p.K;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(TSR_LDS char*)smem;

  // ---- global -> LDS addressing ----------------------------------------------------
  // A instruction ia = wave A_Q + q fills rows 8 ia .. 8 ia + 7; lane -> (row ia 8 + lane / 8,
  // physical chunk lane % 8).
  const bool gathered = GROUPED && p.gather != nullptr;
  const uint16_t* a_base = gathered ? Ab : Ab + (long)m_begin * p.lda;
  uint32_t a_off[A_Q];
#pragma unroll
  for (int q = 0; q < A_Q; ++q) {
    const int row = (wave * A_Q + q) * 8 + (lane >> 3);
    int gr = row;
    gr = m_begin + gr < m_end ? gr : m_end - 1 - m_begin;   // clamp: rows past the edge are never stored
    if constexpr (GROUPED) {
      if (gathered) gr = p.gather[m_begin + gr];
    }
    const int kc = (lane & 7) ^ g16_aswz(row);
    a_off[q] = ((uint32_t)gr * (uint32_t)p.lda + kc * 8) * 2;
  }
  // B instruction ib = wave B_Q + q: sub-tile ib / IPS, rows RPI (ib % IPS) ...; lane -> (row
  // + lane / CPR, physical chunk lane % CPR).
  uint32_t b_off[B_Q];
#pragma unroll
  for (int q = 0; q < B_Q; ++q) {
    const int il = (wave * B_Q + q) % IPS;
    const int krow = il * RPI + lane / CPR;
    const int logical = (lane % CPR) ^ g16_dl_bswz(krow);
    int col = logical * 8;
    col = n_begin + col < p.N ? col : p.N - 8 - n_begin;    // clamp: columns past the edge are never stored
    b_off[q] = ((uint32_t)krow * (uint32_t)p.ldb + col) * 2;
  }
  // the loads of K step `kt` into stage `stage`: instruction l of the wave (l < A_Q: A)
  auto load = [&](int l, int kt, int stage) __attribute__((always_inline)) {
    const int k0 = kt * BK;
    const uint32_t sbase = lds0 + stage * S::kStage;
    if (l < A_Q) {
      const int row = (wave * A_Q + l) * 8 + (lane >> 3);
      const int kc = (lane & 7) ^ g16_aswz(row);
      const uint32_t off = (k0 + kc * 8 < K) ? a_off[l] : kOutOfRange;
      buffer_load16_to_lds(a_base + k0, off, sbase + (wave * A_Q + l) * 1024);
    } else {
      const int q = l - A_Q;
      const int ib = wave * B_Q + q;
      const int krow = (ib % IPS) * RPI + lane / CPR;
      const uint32_t off = (k0 + krow < K) ? b_off[q] : kOutOfRange;
      const uint16_t* src = (SWIGLU && ib / IPS == 1) ? B2b : Bb;
      buffer_load16_to_lds(src + n_begin + (long)k0 * p.ldb, off, sbase + S::kAStage + ib * 1024);
    }
  };

  // ---- fragment read addressing ------------------------------------------------------
  // A: row wm TM + 16 i + lm, logical chunk 4 ks + lk.
  const int a_sw = g16_aswz(wm * TM + lm);       // (16 i leaves (row >> 1) & 7 unchanged)
  const uint32_t a_row = (wm * TM + lm) * 128;
  auto a_frag = [&](int stage, int ks, int i) __attribute__((always_inline)) -> uint4 {
    return lds_read_b128(smem + stage * S::kStage, a_row + i * 16 * 128 + (((ks * 4 + lk) ^ a_sw) << 4));
  };
  // B: transposing read; the lane supplies k row 32 ks + 8 lk + r16 / 4 (+ 4 for the second
  // read) and columns 4 (r16 % 4) .. + 3 of the wave's j-th 16-column tile.  The row's swizzle
  // is the same for both reads and both k steps.
  const int r16 = lane & 15, rr = r16 >> 2;
  const int c_lane = 2 * (rr | ((lk & 1) << 2));
  uint32_t b_rd[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int sub = (SWIGLU && j >= NJ / 2) ? 1 : 0;
    const int jj = SWIGLU ? j % (NJ / 2) : j;
    const int col = wn * (TN / NSRC) + jj * 16 + 4 * (r16 & 3);
    const int phys = (col >> 3) ^ c_lane;
    b_rd[j] = S::kAStage + sub * SUBBYTES + (8 * lk + rr) * BP + phys * 16 + (col & 7) * 2;
  }
  auto b_frag = [&](int stage, int ks, int j) __attribute__((always_inline)) -> uint4 {
    const char* pb = smem + stage * S::kStage + b_rd[j] + ks * 32 * BP;
    const uint2 lo = lds_read_tr16_b64(pb);
    const uint2 hi = lds_read_tr16_b64(pb + 4 * BP);
    return make_uint4(lo.x, lo.y, hi.x, hi.y);
  };

  uint4 af[MI], bf[2][NJ];
  const int ktiles = (K + BK - 1) / BK;

  // The loads of a K step go out over the SPREAD rows that follow the barrier which frees their
  // stage.  The stage is free for exactly one K step (2 MI rows), and what is issued late in
  // it has no time to land before the next barrier.
  constexpr int SPREAD = 8 < 2 * MI ? 8 : 2 * MI;
  constexpr int H_RAW = (MI * NL + SPREAD - 1) / SPREAD;
  constexpr int H = H_RAW < NL ? H_RAW : NL;    // loads that go out in the first of the two k steps (l SPREAD / NL < MI)
  // one row of the wave tile: its MFMAs, then its share of the fragment reads for the next
  // k step (NEXT) and of the loads [L0, L1) of K step `lkt` into stage `lstage` (GO)
  using std::integral_constant;
  using yes = integral_constant<bool, true>;
  using no = integral_constant<bool, false>;
  auto row = [&](int slot, int i, auto next_c, int fstage, int fks, auto l0_c, auto l1_c, auto go_c, int lkt,
                 int lstage) __attribute__((always_inline)) {
    constexpr bool NEXT = decltype(next_c)::value, GO = decltype(go_c)::value;
    constexpr int L0 = decltype(l0_c)::value, L1 = decltype(l1_c)::value;
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = mfma_16x16x32<T>(bf[slot][j], af[i], acc[i][j]);
    int reads = 0;
    if constexpr (NEXT) {
      af[i] = a_frag(fstage, fks, i);
      ++reads;
#pragma unroll
      for (int j = i * NJ / MI; j < (i + 1) * NJ / MI; ++j) {
        bf[slot ^ 1][j] = b_frag(fstage, fks, j);
        reads += 2;
      }
    }
    if constexpr (GO) {
      // load l of the K step goes out with row l SPREAD / NL after the barrier that freed its
      // stage (rows MI and up are rows of the following k step)
#pragma unroll
      for (int l = L0; l < L1; ++l)
        if (l * SPREAD / NL == i + (L0 == 0 ? 0 : MI)) load(l, lkt, lstage);
    }
    // the reads in the shadow of the row's first MFMAs
#pragma unroll
    for (int x = 0; x < NJ; ++x) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (x < reads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: K steps 0 and 1 on their way, fragments of the first k step in hand ----
#pragma unroll
  for (int l = 0; l < NL; ++l) load(l, 0, 0);
  if (ktiles > 1) {
#pragma unroll
    for (int l = 0; l < NL; ++l) load(l, 1, 1);
  }
  wait_direct_loads();
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MI; ++i) af[i] = a_frag(0, 0, i);
#pragma unroll
  for (int j = 0; j < NJ; ++j) bf[0][j] = b_frag(0, 0, j);

  using c0 = integral_constant<int, 0>;
  using cH = integral_constant<int, H>;
  using cN = integral_constant<int, NL>;
  // One K step.  MORE1: the second half of the loads of K step kt+1 is still to go out (their
  // first half followed the previous barrier; K step 1 was loaded whole by the prologue).
  // HAS1 / HAS2: K steps kt+1 / kt+2 exist.  All compile-time: straight-line code between
  // barriers.
  auto kstep = [&](int kt, auto more1_c, auto has1_c, auto has2_c) __attribute__((always_inline)) {
    const int stage = kt & 1;
#pragma unroll
    for (int i = 0; i < MI; ++i) row(0, i, yes{}, stage, 1, cH{}, cN{}, more1_c, kt + 1, stage ^ 1);
    // Every wave has read all it needs from this stage, and its own loads into the other one
    // have landed; past the barrier the other stage is complete and this one is free.
    wait_direct_loads();
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MI; ++i) row(1, i, has1_c, stage ^ 1, 0, c0{}, cH{}, has2_c, kt + 2, stage);
  };
  int kt = 0;
  if (ktiles == 1) {
    kstep(0, no{}, no{}, no{});
  } else {
    if (ktiles > 2) kstep(0, no{}, yes{}, yes{});
    else kstep(0, no{}, yes{}, no{});
    for (kt = 1; kt + 2 < ktiles; ++kt) kstep(kt, yes{}, yes{}, yes{});
    if (kt + 1 < ktiles) { kstep(kt, yes{}, yes{}, no{}); ++kt; }
    kstep(kt, no{}, no{}, no{});
  }
}

}  // namespace tsr950
