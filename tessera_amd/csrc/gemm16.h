// 16-bit (bf16 / f16) MFMA GEMM for gfx950:  D[M,N] = A[M,K] . B[K,N], row-major,
// f32 accumulate.  One kernel template serves the dense, strided-batched and
// grouped (per-expert, ragged) forms and the fused SwiGLU gate/up form.
//
// Tiling.  A workgroup of WM x WN waves owns a BM x BN output tile and walks K
// in steps of BK = 64.  Each wave owns a (BM/WM) x (BN/WN) sub-tile held as
// MFMA accumulators.  With the default 256x256 tile and 2x2 waves every wave keeps a
// 128x128 f32 accumulator (256 registers) — one wave per SIMD, the full 512-register
// budget — which needs 512 B of LDS operand reads per 32 MFMA cycles, half of the
// 128 B/clk the LDS sustains.
//
// The main loop stages a K step in registers on its way from global memory to LDS and comes
// in two MFMA forms (template parameter MS): v_mfma_f32_32x32x16_{bf16,f16} (4 x 4 tiles per
// wave) and v_mfma_f32_16x16x32 (8 x 8 tiles).  The 256x256 tiles run the 16-wide form, which
// spends less power per FLOP: on operands that toggle the matrix pipes the board then grants
// a higher clock.
// What follows describes the 32-wide step; the 16-wide one (kstep16) differs in how the
// fragment reads are dealt out, see there.
//
// The tile body is a device function (gemm16_tile); the grouped kernel also holds a
// 64 x BN instantiation of it with the four waves side by side along the columns, used
// for a group's last row tile when at most 64 rows are left.
//
// LDS staging (double buffered, one barrier per K step).
//   A tile  [BM][64] 16-bit, 128-byte rows, 16-byte chunks XOR-swizzled by
//           (row & 7): the 8 lanes that read one chunk column of 8 consecutive
//           rows hit 8 different bank groups.  Operand read: ds_read_b128.
//   B tile  [64][BN + 16] 16-bit in its NATURAL row-major form (n contiguous).
//           The MFMA wants 8 consecutive k per lane, so the operand is read
//           with the transposing ds_read_b64_tr_b16: a 16-lane block reads a
//           4(k) x 16(n) patch and every lane receives 4 consecutive k of one
//           column.  The 32-byte row pad makes the 4 rows of a patch fall in
//           4 different bank groups.
// The MFMA is issued with the B fragment as its first operand, so a lane's 16
// accumulators of a 32x32 tile are 4 runs of 4 consecutive n for ONE row m:
// the epilogue stores 8 (16-bit D) or 16 (f32 D) contiguous bytes per lane.
//
// Global loads are 16-byte (global_load_dwordx4), prefetched one K step ahead
// into registers while the MFMAs of the current step run.
#pragma once
#include <type_traits>
#include "common.h"

namespace tsr950 {

enum GemmEpilogue : int {
  EPI_F32 = 0,        // D f32
  EPI_STORE16 = 1,    // D in the storage dtype (RNE)
  EPI_SWIGLU16 = 2,   // D = storage(silu(storage(gate)) * storage(up)); B2 holds "up"
  EPI_GATED_F32 = 3,  // D f32 = act(gate) * up, no intermediate rounding; B2 holds "up"
  EPI_F32_FUSED = 4,  // D f32 = act(acc + bias[n]); tile kernels only (p.bias / p.act)
};

// Pointwise activations of the fused epilogue (the reference's matmul-epilogue
// vocabulary, python/tessera/compiler/fusion_core.py:121-138).
enum Activation : int { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU = 2, ACT_SILU = 3, ACT_SIGMOID = 4, ACT_TANH = 5 };

// All of them but relu are a logistic function of a linear or cubic argument:
//   silu v sig(v); sigmoid sig(v); tanh 2 sig(2v) - 1;
//   gelu (tanh form, argument clamped to +-30) 0.5 v (1 + tanh t) = v sig(2t).
template <int ACT>
__device__ __forceinline__ float activate_as(float v) {
  if constexpr (ACT == ACT_NONE) return v;
  if constexpr (ACT == ACT_RELU) return fmaxf(v, 0.f);
  float x = v;
  if constexpr (ACT == ACT_GELU) x = 2.f * fminf(fmaxf(0.7978845608028654f * (v + 0.044715f * v * v * v), -30.f), 30.f);
  if constexpr (ACT == ACT_TANH) x = 2.f * v;
  const float sg = 1.0f / (1.0f + __expf(-x));
  if constexpr (ACT == ACT_SIGMOID) return sg;
  if constexpr (ACT == ACT_TANH) return 2.f * sg - 1.f;
  return v * sg;
}
__device__ __forceinline__ float activate(float v, int act) {
  if (act == ACT_NONE) return v;
  if (act == ACT_RELU) return fmaxf(v, 0.f);
  float x = v;
  if (act == ACT_GELU) x = 2.f * fminf(fmaxf(0.7978845608028654f * (v + 0.044715f * v * v * v), -30.f), 30.f);
  if (act == ACT_TANH) x = 2.f * v;
  const float sg = 1.0f / (1.0f + __expf(-x));
  if (act == ACT_SIGMOID) return sg;
  if (act == ACT_TANH) return 2.f * sg - 1.f;
  return v * sg;
}

struct Gemm16Params {
  const uint16_t* A;
  const uint16_t* B;
  const uint16_t* B2;     // second weight (SwiGLU "up"), else null
  void* D;
  int M, N, K;
  long lda, ldb, ldd;     // in elements
  long strideA, strideB, strideD;   // batch / expert strides in elements
  const float* bias;      // fused epilogue: f32[N] added to every row, or null
  int act;                // fused epilogue / gate activation (enum Activation)
  const int* offsets;     // grouped: device int32[E+1] row offsets into A and D; else null
  const int* gather;      // grouped: row m of A is row gather[m] of p.A (the dispatch fused
                          // into the A load); null: row m
  int groups;             // E (grouped) or batch count
  int tiles_m, tiles_n;   // tile grid (grouped: tiles_m is an upper bound)
};


constexpr int G16_BK = 64;          // K step, elements
constexpr int G16_APITCH = 128;     // bytes per A row in LDS
constexpr int G16_BPAD = 32;        // B row pad, elements
// s_sleep units (64 shader clocks each) a paced short last tile waits per K step.  Per K step a
// wave of a full 256-row tile issues 128 MFMAs of 16 cycles (2048 cycles), a wave of the 64-row
// tile 32 (512 cycles): the difference, (2048 - 512) / 64 = 24 units, keeps the short tile in step
// with the full tiles of its column.  Both terms are fixed by the tile shapes; the unit is shader
// clocks, so the figure does not depend on K or on the clock the board grants.
constexpr int kTailPace = (2048 - 512) / 64;
// A-tile chunk swizzle: 16 consecutive rows of one chunk column hit 16 different
// 16-byte slots of the 256-byte bank line.
__device__ __forceinline__ int g16_aswz(int row) { return (row >> 1) & 7; }

template <int BM, int BN>
struct Gemm16Smem {
  static constexpr int kAStage = BM * G16_APITCH;
  static constexpr int kBPitch = (BN + G16_BPAD) * 2;
  static constexpr int kBStage = G16_BK * kBPitch;
  static constexpr int kStage = kAStage + kBStage;
  static constexpr int kBytes = 2 * kStage;
};

// Map the linear workgroup id to an output tile.  Workgroups are dealt to the 8
// XCDs round-robin; give every XCD a contiguous run of tiles, walked in bands
// of GROUP_M tile rows, so the tiles resident in one XCD's L2 share A rows and
// B columns.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  constexpr int kXcd = 8;
  int lin = bid;
  if (total % kXcd == 0) {
    const int per = total / kXcd;
    lin = (bid % kXcd) * per + bid / kXcd;
  }
  constexpr int GROUP_M = 4;
  const int band = GROUP_M * tiles_n;
  const int b = lin / band;
  const int first_m = b * GROUP_M;
  const int rows = min(tiles_m - first_m, GROUP_M);
  const int r = lin - b * band;
  tm = first_m + r % rows;
  tn = r / rows;
}

// One BM x BN output tile: rows [m_begin, min(m_begin + BM, m_end)), column tile tn, of
// the product whose operand and output bases are Ab / Bb / B2b / Db.  All threads of the
// workgroup call it with the same arguments.
template <class T, int BM, int BN, int WM, int WN, int EPI, bool GROUPED, int MS = 32>
__device__ __forceinline__ void gemm16_tile(const Gemm16Params& p, char* smem, const int m_begin, const int m_end,
                                            const int tn, const uint16_t* Ab, const uint16_t* Bb,
                                            const uint16_t* B2b, char* Db, const bool paced = false) {
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM, TN = BN / WN;     // wave tile
  // MS: side of the MFMA tile.  32: v_mfma_f32_32x32x16 (16 accumulator registers per lane and
  // tile, k = 16 per instruction); 16: v_mfma_f32_16x16x32 (4 registers, k = 32).  Per FLOP the
  // 16-wide form reads and writes half the accumulator data, and a register-only loop of it runs
  // 14 % faster under the board's power limit on random operands (2010 against 1760 TFLOP/s):
  // the big tiles, which sit on that limit, use it.
  static_assert(MS == 32 || MS == 16, "MFMA tile side");
  constexpr int KD = 512 / MS;                  // k per MFMA instruction
  constexpr int AE = MS * MS / 64;              // accumulator registers per MFMA tile
  constexpr int MI = TM / MS, NJ = TN / MS;     // MFMA tiles per wave
  using acc_t = std::conditional_t<MS == 32, f32x16, f32x4>;
  constexpr bool SWIGLU = (EPI == EPI_SWIGLU16 || EPI == EPI_GATED_F32);   // two-source B tile
  // SwiGLU: the BN columns of the LDS B tile are [gate n0..n0+BN/2) | up n0..n0+BN/2);
  // a wave's first NJ/2 column tiles are gate columns and the rest the matching up
  // columns (wave column wn owns output columns wn*TN/2 .. of the tile).
  static_assert(!SWIGLU || NJ % 2 == 0, "SwiGLU form needs an even number of column tiles per wave");
  using S = Gemm16Smem<BM, BN>;
  constexpr int A_CHUNKS = BM * 8 / NT;         // 16-byte chunks per thread per stage
  constexpr int B_CHUNKS = G16_BK * (BN / 8) / NT;
  static_assert(BM * 8 % NT == 0 && G16_BK * (BN / 8) % NT == 0, "tile/thread mismatch");
  constexpr int DSZ = (EPI == EPI_F32 || EPI == EPI_GATED_F32 || EPI == EPI_F32_FUSED) ? 4 : 2;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;   // output columns per tile
  const int n_begin = tn * BN_OUT;
  const int K = p.K;
  using std::true_type;
  using std::false_type;
  // A lane supplies row / column lm of an MFMA tile and the 8 k of group lk (KD / 8 groups).
  const int lm = lane % MS, lk = lane / MS;
  acc_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < AE; ++r) acc[i][j][r] = 0.f;

  // ---- global load addressing ----------------------------------------------------
  // Buffer loads: a wave-uniform tile base (advanced along K on the scalar unit) plus
  // a fixed 32-bit per-lane byte offset, one address register per chunk.
  // A: chunk v = tid + NT*q  -> row v/8, 16-byte chunk v%8.
  const bool gathered = GROUPED && p.gather != nullptr;
  const uint16_t* a_base = gathered ? Ab : Ab + (long)m_begin * p.lda;
  // A thread's chunks are NT / 8 rows apart, a multiple of 16 rows, so the LDS swizzle is the
  // same for all of them: one LDS address, the others a constant apart.  (The global offsets
  // stay one register each: rows are clamped at the edge and may be gathered.)
  static_assert((NT / 8) % 16 == 0, "a thread's A chunks must share their swizzle");
  uint32_t a_off[A_CHUNKS];
  const int a_chunk = tid & 7;
  const uint32_t a_lds0 = (tid >> 3) * G16_APITCH + ((a_chunk ^ g16_aswz(tid >> 3)) << 4);
  auto a_lds = [&](int q) { return a_lds0 + q * (NT / 8) * G16_APITCH; };
#pragma unroll
  for (int q = 0; q < A_CHUNKS; ++q) {
    const int row = (tid >> 3) + (NT / 8) * q;
    int gr = row;
    gr = m_begin + gr < m_end ? gr : m_end - 1 - m_begin;   // clamp: rows past the edge are never stored
    if constexpr (GROUPED) {
      if (gathered) gr = p.gather[m_begin + gr];            // source row (the launcher bounds rows * lda)
    }
    a_off[q] = ((uint32_t)gr * (uint32_t)p.lda + a_chunk * 8) * 2;
  }
  // B: the tile's columns come from one matrix, or (SwiGLU) half from the gate and
  // half from the up matrix; the first B_CHUNKS / HALVES chunks of a thread belong to
  // the first source.  Within a source: chunk v = tid + NT*q' -> k row v/CPR, n chunk v%CPR:
  // a thread's chunks share their n chunk and are NT / CPR k rows apart, so one global
  // offset and one LDS address serve them all (the k rows enter the scalar tile base).
  constexpr int HALVES = SWIGLU ? 2 : 1;
  constexpr int CPR = BN / HALVES / 8;           // 16-byte chunks per row and source
  constexpr int B_PER = B_CHUNKS / HALVES;
  constexpr int B_KSTRIDE = NT / CPR;            // k rows between a thread's chunks
  static_assert(B_CHUNKS % HALVES == 0, "B chunks must split over the sources");
  static_assert(NT % CPR == 0, "a thread's B chunks must share their column");
  const uint16_t* b_base[HALVES];
  b_base[0] = Bb + n_begin;
  if constexpr (SWIGLU) b_base[1] = B2b + n_begin;
  const int b_krow0 = tid / CPR, b_nch = tid % CPR;
  int b_col0 = b_nch * 8;
  b_col0 = n_begin + b_col0 < p.N ? b_col0 : p.N - 8 - n_begin;   // clamp: columns past the edge are never stored
  const uint32_t b_off0 = ((uint32_t)b_krow0 * (uint32_t)p.ldb + b_col0) * 2;
  const uint32_t b_lds0 = S::kAStage + b_krow0 * S::kBPitch + b_nch * 16;
  auto b_krow = [&](int qb) { return b_krow0 + (qb % B_PER) * B_KSTRIDE; };
  auto b_lds = [&](int qb) { return b_lds0 + (qb % B_PER) * B_KSTRIDE * S::kBPitch + (qb / B_PER) * CPR * 16; };

  // ---- staging registers ------------------------------------------------------
  // st[q] holds one 16-byte chunk on its way from global memory to LDS:
  // q < A_CHUNKS is A chunk q, the rest are B chunks.  The chunks of a K step are
  // split into KS groups; a group is written to LDS and immediately refilled with
  // the same chunks of the K step two ahead, so every global load has a full K
  // step of MFMA time to land and loads / LDS writes are spread evenly over it.
  constexpr int KS = G16_BK / KD;                // MFMA k steps per K step
  constexpr int NC = A_CHUNKS + B_CHUNKS;
  constexpr int CPG = (NC + KS - 1) / KS;       // (the last group is short when KS does not divide NC)
  uint4 st[NC];
  using std::true_type;
  using std::false_type;
  // Load chunk q of the K step starting at k0.  The guarded form is for a step
  // that may be partial: out-of-range K must contribute exact zeros on both
  // operands, which a buffer load returns by itself for an offset past its range.
  auto gfetch = [&](int q, int k0, auto guarded_c) -> uint4 {
    constexpr bool GUARD = decltype(guarded_c)::value;
    if (q < A_CHUNKS) {
      uint32_t off = a_off[q];
      if constexpr (GUARD) off = (k0 + a_chunk * 8 < K) ? off : kOutOfRange;
      return buffer_load_b128(a_base + k0, off);
    } else {
      const int qb = q - A_CHUNKS;
      uint32_t off = b_off0;
      if constexpr (GUARD) off = (k0 + b_krow(qb) < K) ? off : kOutOfRange;
      return buffer_load_b128(b_base[qb / B_PER] + (long)(k0 + (qb % B_PER) * B_KSTRIDE) * p.ldb, off);
    }
  };
  auto gload1 = [&](int q, int k0, auto guarded_c) { st[q] = gfetch(q, k0, guarded_c); };
  auto lstore1 = [&](int q, int buf) {
    char* base = smem + buf * S::kStage;
    if (q < A_CHUNKS) lds_write_b128(base, a_lds(q), st[q]);
    else lds_write_b128(base, b_lds(q - A_CHUNKS), st[q]);
  };
  // Group g: write its chunks (K step `write` done by the caller's choice of
  // buffer) and refill them.  MODE 0 = no refill, 1 = full step, 2 = guarded.
  auto stream_group = [&](int g, int buf_dst, int k0_load, auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int q = g * CPG; q < (g + 1) * CPG; ++q) {
      if (q < NC) {
        lstore1(q, buf_dst);
        if constexpr (MODE == 1) gload1(q, k0_load, false_type{});
        if constexpr (MODE == 2) gload1(q, k0_load, true_type{});
      }
    }
  };

  // ---- operand read addressing --------------------------------------------
  uint32_t a_rd[MI];       // byte offset of this lane's row; chunk applied per k step
  int a_sw[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int row = wm * TM + i * MS + lm;
    a_rd[i] = row * G16_APITCH;
    a_sw[i] = g16_aswz(row);
  }
  // transposing read: lane supplies row (k) = 8*lk + r/4 (+4 for the second half), columns
  // n = MS j + 16*((lane % MS) >> 4) + 4*(r%4), r = lane & 15.
  const int r16 = lane & 15;
  const uint32_t b_rd0 = S::kAStage + (8 * lk + (r16 >> 2)) * S::kBPitch +
                         (wn * (SWIGLU ? TN / 2 : TN) + 16 * (lm >> 4) + 4 * (r16 & 3)) * 2;
  // byte offset of the wave's j-th column tile inside its B rows (SwiGLU: the up
  // columns start BN/2 columns after the gate columns)
  auto b_col = [](int j) constexpr -> int {
    return (SWIGLU && j >= NJ / 2) ? (BN / 2 + (j - NJ / 2) * MS) * 2 : j * MS * 2;
  };


  // Operand fragments are double buffered in registers: the LDS reads of k
  // step s+1 are issued before the MFMAs of step s, which hide their latency.
  uint4 af[2][MI], bf[2][NJ];
  auto frag_load = [&](int buf, int ks, int slot) {
    const char* base = smem + buf * S::kStage;
#pragma unroll
    for (int i = 0; i < MI; ++i)
      af[slot][i] = lds_read_b128(base, a_rd[i] + (((ks * (KD / 8) + lk) ^ a_sw[i]) << 4));
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const char* pb = base + b_rd0 + ks * KD * S::kBPitch + b_col(j);
      const uint2 lo = lds_read_tr16_b64(pb);
      const uint2 hi = lds_read_tr16_b64(pb + 4 * S::kBPitch);
      bf[slot][j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
    }
  };
  auto mma = [&](int slot) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if constexpr (MS == 32) acc[i][j] = mfma_32x32x16<T>(bf[slot][j], af[slot][i], acc[i][j]);
      }
  };
  // Scheduling hint for one k step of NM MFMAs that carries RD operand reads and
  // (when `stream`) CPG LDS writes + CPG global loads.  The writes cannot pass
  // the reads (the compiler cannot prove the two LDS buffers disjoint), so the
  // reads ride the first MFMAs and the write/load pairs the last ones; every
  // memory instruction issues in the shadow of an MFMA instead of in a burst.
  constexpr int NM = MI * NJ, RD = MI + 2 * NJ;
  auto hint_step = [&](auto stream_c, auto loads_c) {
    constexpr bool STREAM = decltype(stream_c)::value;
    constexpr bool LOADS = decltype(loads_c)::value;
    if constexpr (NM >= 4) {
      constexpr int WSLOTS = CPG < NM / 2 ? CPG : NM / 2;
      constexpr int wslots = STREAM ? WSLOTS : 0;
      constexpr int rslots = NM - wslots;
      constexpr int rper = (RD + rslots - 1) / rslots;
      constexpr int wper = (CPG + WSLOTS - 1) / WSLOTS;
#pragma unroll
      for (int x = 0; x < NM; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (x < rslots) {
          __builtin_amdgcn_sched_group_barrier(0x100, rper, 0);
        } else {
          __builtin_amdgcn_sched_group_barrier(0x200, wper, 0);
          if constexpr (LOADS) __builtin_amdgcn_sched_group_barrier(0x020, wper, 0);
        }
      }
    }
  };

  const int ktiles = (K + G16_BK - 1) / G16_BK;
  using mode0 = std::integral_constant<int, 0>;
  using mode1 = std::integral_constant<int, 1>;
  using mode2 = std::integral_constant<int, 2>;

  // ---- prologue: K step 0 in buffer 0, group 0 of step 1 in buffer 1, the rest
  // of step 1 and group 0 of step 2 in registers -------------------------------
  // (the first half of step 1 is requested before step 0 has landed, into registers the
  // operand fragments will use later: group 0 of step 1 is then not a second full
  // memory latency behind step 0)
  constexpr int PRE = NC / 2;
#pragma unroll
  for (int q = 0; q < NC; ++q) gload1(q, 0, true_type{});
  uint4 pre[PRE];
  if (ktiles > 1) {
#pragma unroll
    for (int q = 0; q < PRE; ++q) pre[q] = gfetch(q, G16_BK, true_type{});
  }
#pragma unroll
  for (int q = 0; q < NC; ++q) lstore1(q, 0);
  if (ktiles > 1) {
#pragma unroll
    for (int q = PRE; q < NC; ++q) gload1(q, G16_BK, true_type{});
#pragma unroll
    for (int q = 0; q < PRE; ++q) st[q] = pre[q];
    if (ktiles > 2) stream_group(0, 1, 2 * G16_BK, mode2{});
    else stream_group(0, 1, 0, mode0{});
  }
  __syncthreads();
  frag_load(0, 0, 0);

  // One K step.  HAS1: step kt+1 exists (its groups 1.. go to the other buffer
  // during k steps 0..KS-2).  L2 / L3: how steps kt+2 / kt+3 are fetched
  // (0 absent, 1 full, 2 possibly partial).  All compile-time: the body is one
  // straight-line block per barrier interval.
  auto kstep = [&](int kt, auto has1_c, auto l2_c, auto l3_c) {
    constexpr bool HAS1 = decltype(has1_c)::value;
    constexpr int L2 = decltype(l2_c)::value;
    constexpr int L3 = decltype(l3_c)::value;
    const int buf = kt & 1;
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      frag_load(buf, ks + 1, (ks + 1) & 1);
      if constexpr (HAS1) stream_group(ks + 1, buf ^ 1, (kt + 2) * G16_BK, l2_c);
      mma(ks & 1);
      hint_step(std::integral_constant<bool, HAS1>{}, std::integral_constant<bool, (L2 != 0)>{});
      __builtin_amdgcn_sched_barrier(0);
    }
    // Every wave has issued all its reads of this buffer and all its writes of
    // the other one; past the barrier the other buffer is complete and this one
    // is free to take group 0 of step kt+2.
    __syncthreads();
    if constexpr (HAS1) frag_load(buf ^ 1, 0, KS & 1);
    if constexpr (L2 != 0) stream_group(0, buf, (kt + 3) * G16_BK, l3_c);
    mma((KS - 1) & 1);
    if constexpr (HAS1) hint_step(std::integral_constant<bool, (L2 != 0)>{}, std::integral_constant<bool, (L3 != 0)>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  // The 16-wide MFMA form has twice the operand fragments per k step (8 + 8 of them for a
  // 128 x 128 wave tile).  Double-buffering both sets would not fit the 256 ordinary registers
  // next to the staging registers, so only the B fragments are: the step walks the wave tile
  // row by row, and as soon as a row's MFMAs are issued its A fragment register takes the
  // same row's fragment of the next k step; the next B fragments, the LDS writes and the
  // global loads of the step are dealt out over the rows in the same way.
  auto a_frag = [&](int buf, int ks, int i) __attribute__((always_inline)) -> uint4 {
    return lds_read_b128(smem + buf * S::kStage, a_rd[i] + (((ks * (KD / 8) + lk) ^ a_sw[i]) << 4));
  };
  auto b_frag = [&](int buf, int ks, int j) __attribute__((always_inline)) -> uint4 {
    const char* pb = smem + buf * S::kStage + b_rd0 + ks * KD * S::kBPitch + b_col(j);
    const uint2 lo = lds_read_tr16_b64(pb);
    const uint2 hi = lds_read_tr16_b64(pb + 4 * S::kBPitch);
    return make_uint4(lo.x, lo.y, hi.x, hi.y);
  };
  auto kstep16 = [&](int kt, auto has1_c, auto l2_c, auto l3_c) __attribute__((always_inline)) {
    constexpr bool HAS1 = decltype(has1_c)::value;
    constexpr int L2 = decltype(l2_c)::value;
    static_assert(MS != 16 || KS == 2, "two MFMA k steps per K step");
    const int buf = kt & 1;
    // one row of the wave tile: its MFMAs, then the row's share of the fragment reads for
    // the next k step and of the chunk group `g` (written to LDS buffer `wbuf`, refilled from
    // K offset k0_load in mode `mode_c`)
    auto row = [&](int slot, int i, bool next_frags, int fbuf, int fks, auto stream_c, int g, int wbuf, int k0_load,
                   auto mode_c) __attribute__((always_inline)) {
      constexpr bool STREAM = decltype(stream_c)::value;
      constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if constexpr (MS == 16) acc[i][j] = mfma_16x16x32<T>(bf[slot][j], af[0][i], acc[i][j]);
      }
      int reads = 0, writes = 0;
      if (next_frags) {
        af[0][i] = a_frag(fbuf, fks, i);
        ++reads;
#pragma unroll
        for (int j = i * NJ / MI; j < (i + 1) * NJ / MI; ++j) {
          bf[slot ^ 1][j] = b_frag(fbuf, fks, j);
          reads += 2;
        }
      }
      if constexpr (STREAM) {
#pragma unroll
        for (int q = g * CPG + i * CPG / MI; q < g * CPG + (i + 1) * CPG / MI; ++q) {
          if (q < NC) {
            lstore1(q, wbuf);
            if constexpr (MODE == 1) gload1(q, k0_load, false_type{});
            if constexpr (MODE == 2) gload1(q, k0_load, true_type{});
            ++writes;
          }
        }
      }
      // every memory instruction in the shadow of an MFMA of its row
#pragma unroll
      for (int x = 0; x < NJ; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (x < reads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        else if (x - reads < writes) {
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
          if constexpr (MODE != 0) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // first k step of the K step (fragments in hand); the second's come from the same buffer,
    // and chunk group 1 of K step kt+1 goes to the other buffer
#pragma unroll
    for (int i = 0; i < MI; ++i) row(0, i, true, buf, 1, std::integral_constant<bool, HAS1>{}, 1, buf ^ 1, (kt + 2) * G16_BK, l2_c);
    // Every wave has issued all its reads of this buffer and all its writes of the other one;
    // past the barrier the other buffer is complete and this one is free to take group 0 of
    // step kt+2.
    __syncthreads();
    // A short last row tile of a group issues a quarter of the MFMAs per K step and would run
    // ahead of the full tiles of its column, which started with it on the same XCD: the weight
    // panel they share would then pass through that XCD's L2 twice.  It waits here instead
    // (kTailPace x 64 cycles per K step, about what the full tiles take longer), stays within
    // reach of them, and the panel is fetched once.
    if (paced) __builtin_amdgcn_s_sleep(kTailPace);
#pragma unroll
    for (int i = 0; i < MI; ++i) row(1, i, HAS1, buf ^ 1, 0, std::integral_constant<bool, (L2 != 0)>{}, 0, buf, (kt + 3) * G16_BK, l3_c);
  };
  auto kstep_any = [&](int kt, auto has1_c, auto l2_c, auto l3_c) __attribute__((always_inline)) {
    if constexpr (MS == 16) kstep16(kt, has1_c, l2_c, l3_c);
    else kstep(kt, has1_c, l2_c, l3_c);
  };
  int kt = 0;
  // The first K step stands outside the loop: its MFMAs start from the zero accumulators, and
  // with the loop entered directly the compiler rotates the 16-wide form's accumulators through
  // ordinary registers (hundreds of register moves per K step) instead of updating them in place.
  if (ktiles > 4) { kstep_any(0, true_type{}, mode1{}, mode1{}); kt = 1; }
  for (; kt + 4 < ktiles; ++kt) kstep_any(kt, true_type{}, mode1{}, mode1{});
  if (kt + 3 < ktiles) { kstep_any(kt, true_type{}, mode1{}, mode2{}); ++kt; }
  if (kt + 2 < ktiles) { kstep_any(kt, true_type{}, mode2{}, mode0{}); ++kt; }
  if (kt + 1 < ktiles) { kstep_any(kt, true_type{}, mode0{}, mode0{}); ++kt; }
  kstep_any(kt, false_type{}, mode0{}, mode0{});

  // ---- epilogue -------------------------------------------------------------
  // acc[i][j][r]: row m = MS i + lm, col n = MS j + 8*(r/4) + 4*lk + (r%4): a lane owns
  // runs of four columns of MS different rows.  Stored like that, every store
  // instruction would touch 32 cache lines with 16 bytes each, and the output write
  // would cost a tenth of a long-K product and half of a short-K one.  The wave
  // therefore stages its tile through its share of the (now free) LDS and writes
  // whole row segments: 16 bytes per lane, consecutive lanes along a row.
  constexpr int NJ_OUT = SWIGLU ? NJ / 2 : NJ;
  constexpr int ROWB = NJ_OUT * MS * DSZ;              // bytes of one row of the wave's output tile
  constexpr int PITCH = ROWB + 16;
  constexpr int WAVE_LDS = S::kBytes / (WM * WN);
  constexpr int MB = TM / 32;                          // 32-row blocks of the wave's tile
  constexpr int IB_FIT = WAVE_LDS / (32 * PITCH);      // 32-row blocks that fit the wave's share
  constexpr int IB = IB_FIT >= MB ? MB : (IB_FIT >= 2 ? 2 : 1);
  static_assert(IB_FIT >= 1 && MB % IB == 0, "epilogue staging does not fit");
  constexpr int TPB = 32 / MS;                         // MFMA tiles per 32-row block
  constexpr int QG = AE / 4;                           // runs of four columns per MFMA tile
  constexpr int LPR = ROWB / 16;                       // lanes per row
  constexpr int RPI = 64 / LPR;                        // rows per store instruction
  static_assert(LPR <= 64 && (IB * 32) % RPI == 0, "epilogue row mapping");
  // every wave has consumed its last fragments once its MFMAs are issued: past this
  // barrier nobody reads the operand tiles any more
  __syncthreads();
  char* stg = smem + wave * WAVE_LDS;
  const int nw0 = n_begin + wn * (SWIGLU ? TN / 2 : TN);   // first output column of the wave
  const int st_row = lane / LPR, st_chunk = lane % LPR;
  const int st_n = nw0 + st_chunk * (16 / DSZ);
  // The activation and the presence of a bias are compile-time here: one compact,
  // straight-line instance runs per launch.  (With the choice made per element at run
  // time the epilogue was 23,000 instructions that the plain path hopped through,
  // missing the instruction cache at every hop: 12 us per 256 x 256 tile.)
  auto emit = [&](auto act_c, auto bias_c) __attribute__((always_inline)) {
    constexpr int ACT = decltype(act_c)::value;
    constexpr bool HAS_BIAS = decltype(bias_c)::value;
#pragma unroll
    for (int b0 = 0; b0 < MB; b0 += IB) {
#pragma unroll
      for (int ii = 0; ii < IB * TPB; ++ii) {
        const int i = b0 * TPB + ii;
#pragma unroll
        for (int j = 0; j < NJ_OUT; ++j) {
#pragma unroll
          for (int q = 0; q < QG; ++q) {
            const int n = nw0 + j * MS + q * 8 + lk * 4;
            float v0 = acc[i][j][q * 4 + 0], v1 = acc[i][j][q * 4 + 1];
            float v2 = acc[i][j][q * 4 + 2], v3 = acc[i][j][q * 4 + 3];
            if constexpr (EPI == EPI_F32_FUSED) {
              if constexpr (HAS_BIAS) {
                // (a column past N is never stored; its bias read stays in range)
                const float4 bv = *reinterpret_cast<const float4*>(p.bias + (n < p.N ? n : 0));
                v0 += bv.x; v1 += bv.y; v2 += bv.z; v3 += bv.w;
              }
              v0 = activate_as<ACT>(v0); v1 = activate_as<ACT>(v1);
              v2 = activate_as<ACT>(v2); v3 = activate_as<ACT>(v3);
            }
            if constexpr (EPI == EPI_GATED_F32) {
              const acc_t& u = acc[i][j + NJ / 2];
              v0 = activate_as<ACT>(v0) * u[q * 4 + 0]; v1 = activate_as<ACT>(v1) * u[q * 4 + 1];
              v2 = activate_as<ACT>(v2) * u[q * 4 + 2]; v3 = activate_as<ACT>(v3) * u[q * 4 + 3];
            }
            char* dst = stg + (ii * MS + lm) * PITCH + (j * MS + q * 8 + lk * 4) * DSZ;
            if constexpr (DSZ == 4) {
              *reinterpret_cast<float4*>(dst) = make_float4(v0, v1, v2, v3);
            } else {
              if constexpr (EPI == EPI_SWIGLU16) {
                const acc_t& u = acc[i][j + NJ / 2];
                float g[4] = {v0, v1, v2, v3};
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  // every intermediate lives on the storage grid, as in the reference
                  const float gs = from_storage<T>(to_storage<T>(g[e]));
                  const float us = from_storage<T>(to_storage<T>(u[q * 4 + e]));
                  o[e] = (gs / (1.0f + __expf(-gs))) * us;
                }
                v0 = o[0]; v1 = o[1]; v2 = o[2]; v3 = o[3];
              }
              uint2 pk;
              pk.x = pack2<T>(v0, v1);
              pk.y = pack2<T>(v2, v3);
              *reinterpret_cast<uint2*>(dst) = pk;
            }
          }
        }
      }
      __builtin_amdgcn_wave_barrier();                 // the wave's LDS operations run in order
#pragma unroll
      for (int it = 0; it < IB * 32 / RPI; ++it) {
        const int row = it * RPI + st_row;
        const uint4 v = lds_read_b128(stg, row * PITCH + st_chunk * 16);
        const int m = m_begin + wm * TM + b0 * 32 + row;
        // N % 8 == 0 on this path: a 16-byte chunk is inside or outside as a whole
        if (m < m_end && st_n < p.N)
          *reinterpret_cast<uint4*>(Db + ((long)m * p.ldd + st_n) * DSZ) = v;
      }
      __builtin_amdgcn_wave_barrier();
    }
  };
  using A0 = std::integral_constant<int, ACT_NONE>;
  auto by_activation = [&](auto bias_c) __attribute__((always_inline)) {
    switch (p.act) {
      case ACT_RELU: emit(std::integral_constant<int, ACT_RELU>{}, bias_c); break;
      case ACT_GELU: emit(std::integral_constant<int, ACT_GELU>{}, bias_c); break;
      case ACT_SILU: emit(std::integral_constant<int, ACT_SILU>{}, bias_c); break;
      case ACT_SIGMOID: emit(std::integral_constant<int, ACT_SIGMOID>{}, bias_c); break;
      case ACT_TANH: emit(std::integral_constant<int, ACT_TANH>{}, bias_c); break;
      default: emit(A0{}, bias_c); break;
    }
  };
  if constexpr (EPI == EPI_GATED_F32) {
    by_activation(false_type{});
  } else if constexpr (EPI == EPI_F32_FUSED) {
    if (p.bias) by_activation(true_type{});
    else by_activation(false_type{});
  } else {
    emit(A0{}, false_type{});
  }
}

// MID (grouped 256-row tiles only): a last row tile of 65 to 128 rows runs on the 128-row tile
// body.  A separate instantiation, for launches whose groups average at most a tile of rows: the
// kernel that serves large groups keeps its two bodies.
template <class T, int BM, int BN, int WM, int WN, int EPI, bool GROUPED, int MS = 32, bool MID = false>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm16_kernel(const Gemm16Params p) {
  constexpr bool SWIGLU = (EPI == EPI_SWIGLU16 || EPI == EPI_GATED_F32);
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int lane = threadIdx.x & 63;

  // ---- which tile ---------------------------------------------------------
  int tm, tn, m_begin, m_end;
  const uint16_t* Ab = p.A;
  const uint16_t* Bb = p.B;
  const uint16_t* B2b = p.B2;
  char* Db = (char*)p.D;
  constexpr int DSZ = (EPI == EPI_F32 || EPI == EPI_GATED_F32 || EPI == EPI_F32_FUSED) ? 4 : 2;
  if constexpr (GROUPED) {
    // 1-D grid over the real tiles of all groups, ordered group-major, then n tile,
    // then m tile.  Workgroup ids are dealt to the 8 XCDs round-robin, so XCD j takes
    // the j-th contiguous eighth of that order: the tiles running together on one XCD
    // then belong to one or two experts and share its weight slabs and row tiles in
    // that XCD's L2.  The grid is sized from an upper bound; surplus blocks exit.
    // The decode reads all E + 1 offsets.  Walking them with dependent scalar loads
    // costs microseconds per workgroup, so each wave reads 64 groups per step with one
    // coalesced load, scans their tile counts across its lanes and finds the group of
    // its tile with a ballot.
    auto tiles_of = [&](int g, int& lo, int& hi) -> int {
      lo = g < p.groups ? p.offsets[g] : 0;
      hi = g < p.groups ? p.offsets[g + 1] : 0;
      return ((hi - lo + BM - 1) / BM) * p.tiles_n;
    };
    auto wave_scan = [&](int v) -> int {             // inclusive prefix sum over the 64 lanes
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int u = __shfl_up(v, d, 64);
        if (lane >= d) v += u;
      }
      return v;
    };
    // (the first 64 groups are fetched and scanned once, for the total and for the lookup)
    int lo0, hi0;
    const int cnt0 = tiles_of(lane, lo0, hi0);
    const int incl0 = wave_scan(cnt0);
    int total = __shfl(incl0, 63, 64);
    for (int g0 = 64; g0 < p.groups; g0 += 64) {
      int lo, hi;
      total += __shfl(wave_scan(tiles_of(g0 + lane, lo, hi)), 63, 64);
    }
    total = __builtin_amdgcn_readfirstlane(total);
    const int per = (total + 7) / 8;
    const int slot = blockIdx.x >> 3;
    const int lin = (blockIdx.x & 7) * per + slot;
    if (slot >= per || lin >= total) return;
    int e = -1, acc = 0, g_lo = 0, g_hi = 0, mt = 0;
    for (int g0 = 0, base = 0; g0 < p.groups && e < 0; g0 += 64) {
      int lo = lo0, hi = hi0, cnt = cnt0, incl = incl0;
      if (g0 > 0) {
        cnt = tiles_of(g0 + lane, lo, hi);
        incl = base + wave_scan(cnt);
      }
      const unsigned long long hit = __ballot(lin >= incl - cnt && lin < incl);
      if (hit) {
        const int src = __ffsll((long long)hit) - 1;
        e = g0 + src;
        acc = __shfl(incl - cnt, src, 64);
        g_lo = __shfl(lo, src, 64);
        g_hi = __shfl(hi, src, 64);
        mt = (g_hi - g_lo + BM - 1) / BM;
      }
      base = __shfl(incl, 63, 64);
    }
    if (e < 0) return;
    e = __builtin_amdgcn_readfirstlane(e);
    acc = __builtin_amdgcn_readfirstlane(acc);
    g_lo = __builtin_amdgcn_readfirstlane(g_lo);
    g_hi = __builtin_amdgcn_readfirstlane(g_hi);
    mt = __builtin_amdgcn_readfirstlane(mt);
    const int r = lin - acc;
    tn = r / mt;
    tm = r - tn * mt;
    m_begin = g_lo + tm * BM;
    m_end = g_hi;
    Bb += (long)e * p.strideB;
    if constexpr (SWIGLU) B2b += (long)e * p.strideB;
  } else {
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int z = blockIdx.z;
    Ab += (long)z * p.strideA;
    Bb += (long)z * p.strideB;
    Db += (long)z * p.strideD * DSZ;
    m_begin = tm * BM;
    m_end = p.M;
  }
  if constexpr (GROUPED && BM == 256 && WM * WN == 4) {
    // A group's last row tile is often nearly empty (rows per expert are a little over a
    // multiple of BM about half of the time).  With at most 64 rows left the four waves
    // share the columns of a 64-row tile instead: a quarter of the matrix work of the
    // full tile, whose other 192 rows would be computed and thrown away.
    if (m_end - m_begin <= 64) {
      // (paced when full tiles of the same group and column run beside it; 16-wide step only)
      gemm16_tile<T, 64, BN, 1, 4, EPI, GROUPED, MS>(p, smem, m_begin, m_end, tn, Ab, Bb, B2b, Db, MS == 16 && tm > 0);
      return;
    }
    // (up to 128 rows left — a group of about a hundred rows, a chunk of a thousand tokens over
    // 64 experts — the 128-row tile: half the matrix work)
    if (MID && m_end - m_begin <= 128) {
      gemm16_tile<T, 128, BN, 2, 2, EPI, GROUPED, MS>(p, smem, m_begin, m_end, tn, Ab, Bb, B2b, Db);
      return;
    }
  }
  gemm16_tile<T, BM, BN, WM, WN, EPI, GROUPED, MS>(p, smem, m_begin, m_end, tn, Ab, Bb, B2b, Db);
}

// The tiles that are left when the tile count is not a multiple of the 256 compute units would
// run as a last, mostly empty round.  This kernel takes those tiles (ids first_tile .. in the
// order of tile_of_block) and splits each along K over gridDim.y workgroups, so the round fills
// the chip: workgroup (r, z) computes K range [z ksplit, (z + 1) ksplit) of tile first_tile + r
// and writes the f32 partial tile, row-major 256 x 256, to ws[(z * gridDim.x + r)]; a second
// kernel sums the partials in split order.  Dense, unbatched products only.
template <class T, int MS>
__global__ __launch_bounds__(256, 1) void gemm16_rest_splitk_kernel(const Gemm16Params p, int first_tile, int ksplit,
                                                                    float* __restrict__ ws) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn;
  tile_of_block(first_tile + (int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int z = blockIdx.y;
  const int k0 = z * ksplit;
  Gemm16Params q = p;
  q.K = min(ksplit, p.K - k0);
  q.ldd = 256;
  q.bias = nullptr;
  q.act = ACT_NONE;
  const int m_begin = tm * 256;
  float* tile_ws = ws + ((long)z * gridDim.x + blockIdx.x) * (256 * 256);
  // the tile function stores element (m, n) at Db + (m ldd + n): shift the base so that the
  // tile's first element lands on tile_ws
  char* Db = reinterpret_cast<char*>(tile_ws - ((long)m_begin * 256 + (long)tn * 256));
  gemm16_tile<T, 256, 256, 2, 2, EPI_F32, false, MS>(q, smem, m_begin, p.M, tn, p.A + k0, p.B + (long)k0 * p.ldb, nullptr,
                                                      Db);
}

// D tile = sum over the splits (in split order) of the partial tiles written by the kernel above,
// then bias / activation, stored as f32 or in the storage dtype; four columns per thread.
template <class T, int EPI>
__global__ __launch_bounds__(256) void gemm16_rest_sum_kernel(const float* __restrict__ ws, void* __restrict__ D, int M,
                                                              int N, long ldd, int tiles_m, int tiles_n, int first_tile,
                                                              int splits, const float* __restrict__ bias, int act) {
  int tm, tn;
  tile_of_block(first_tile + (int)blockIdx.y, tiles_m, tiles_n, tm, tn);
  const int quad = blockIdx.x * 256 + threadIdx.x;     // 64 quads of four columns per row
  const int row = quad >> 6, col = (quad & 63) * 4;
  const int m = tm * 256 + row, n = tn * 256 + col;
  if (m >= M || n >= N) return;
  const long tile_elems = 256 * 256;
  const float* src = ws + (long)blockIdx.y * tile_elems + row * 256 + col;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  // (four slices fetched together: every one of these loads is a trip to memory)
  for (int z0 = 0; z0 < splits; z0 += 4) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      v[u] = z0 + u < splits ? *reinterpret_cast<const float4*>(src + (long)(z0 + u) * gridDim.y * tile_elems)
                             : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < 4; ++u) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }   // slice order
  }
  if (bias) {
    const float4 bv = *reinterpret_cast<const float4*>(bias + n);
    acc.x += bv.x; acc.y += bv.y; acc.z += bv.z; acc.w += bv.w;
  }
  acc.x = activate(acc.x, act); acc.y = activate(acc.y, act);
  acc.z = activate(acc.z, act); acc.w = activate(acc.w, act);
  if constexpr (EPI == EPI_F32 || EPI == EPI_F32_FUSED) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(D) + (long)m * ldd + n) = acc;
  } else {
    uint2 pk;
    pk.x = pack2<T>(acc.x, acc.y);
    pk.y = pack2<T>(acc.z, acc.w);
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(D) + (long)m * ldd + n) = pk;
  }
}

}  // namespace tsr950
