// 8-bit MFMA GEMM for gfx950:  D[M,N] = A[M,K] . B[K,N], row-major bytes.
//   I8   int8 x int8 -> int32 (v_mfma_i32_32x32x32_i8), bit-exact.
//   FP8  OCP e4m3 x e4m3 -> f32 (v_mfma_f32_32x32x64_f8f6f4, the full-rate CDNA4
//        fp8 form), scaled by two per-tensor f32 scales in the epilogue.
//
// Same structure as the 16-bit kernel: 256x256 output tile, 2x2 waves of 128x128,
// K walked in steps of 128 bytes, LDS double buffered with one barrier per step,
// operand fragments double buffered in registers.
//   A tile  [256][128 B], 16-byte chunks XOR-swizzled by ((row >> 1) & 7), ds_read_b128.
//   B tile  [128][256 + 32 B] natural layout; the operand (16 or 32 consecutive k
//           bytes of one column per lane) is read with the transposing
//           ds_read_b64_tr_b8: a 16-lane block reads an 8(k) x 16(n) patch and
//           every lane receives 8 consecutive k of one column.  The 32-byte row
//           pad interleaves the two patches a half-wave reads over all 64 banks.
// Both operands enumerate k in the same order, which is all the MFMA needs: for
// the 64-deep fp8 instruction a lane's 32 bytes are bytes [16h,16h+16) of two
// consecutive 32-byte k groups rather than one contiguous run.
#pragma once
#include <type_traits>
#include "common.h"

namespace tsr950 {

struct I8 {};
struct FP8 {};     // OCP e4m3fn
struct BF8 {};     // OCP e5m2
// operand format selector of the f8f6f4 matrix instruction: 0 = e4m3, 1 = e5m2
template <class T> constexpr int f8_format() { return std::is_same<T, BF8>::value ? 1 : 0; }

enum Gemm8Epilogue : int {
  EPI8_I32 = 0,        // I8: int32 accumulators
  EPI8_W8A8_F32 = 1,   // I8: f32(acc) * row_scale[m] * col_scale[n]  (+ optional int32 copy)
  EPI8_SCALED_F32 = 2, // FP8: acc * sa * sb -> f32
  EPI8_SCALED_BF16 = 3 // FP8: acc * sa * sb -> bf16
};

struct Gemm8Params {
  const uint8_t* A;
  const uint8_t* B;
  void* D;
  int32_t* acc_out;          // W8A8: optional raw accumulators
  const float* row_scale;    // W8A8: [M]
  const float* col_scale;    // W8A8: [N]
  float scale_a, scale_b;    // FP8
  int M, N, K;
  int tiles_m, tiles_n;
  int ksplit;                // > 0: workgroup (tile, z = blockIdx.y) computes K range [z ksplit, (z + 1) ksplit)
                             // and stores at D + z M N (partial results, summed by gemm8_split_sum_kernel)
};

constexpr int G8_BK = 128;       // K step in bytes (= elements)
constexpr int G8_BM = 256, G8_BN = 256;
constexpr int G8_APITCH = 128;
constexpr int G8_BPITCH = G8_BN + 32;
constexpr int G8_ASTAGE = G8_BM * G8_APITCH;
constexpr int G8_BSTAGE = G8_BK * G8_BPITCH;
constexpr int G8_STAGE = G8_ASTAGE + G8_BSTAGE;
constexpr int G8_SMEM = 2 * G8_STAGE;
constexpr int g8_smem(int bm) { return 2 * (bm * G8_APITCH + G8_BSTAGE); }   // LDS of a tile of bm rows

__device__ __forceinline__ void tile_of_block8(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  int lin = bid;
  if (total % 8 == 0) lin = (bid % 8) * (total / 8) + bid / 8;
  constexpr int GROUP_M = 4;
  const int band = GROUP_M * tiles_n;
  const int b = lin / band;
  const int first_m = b * GROUP_M;
  const int rows = min(tiles_m - first_m, GROUP_M);
  const int r = lin - b * band;
  tm = first_m + r % rows;
  tn = r / rows;
}

// BM: rows of the workgroup tile, 256 or 128 (the 2 x 2 waves then own 64 rows x 128 columns each: twice the
// tiles to fill the chip with when a product has few of them).
template <class T, int EPI, int BM = G8_BM>
__global__ __launch_bounds__(256, 1) void gemm8_kernel(const Gemm8Params p) {
  static_assert(BM == 256 || BM == 128, "tile rows");
  constexpr int ASTAGE = BM * G8_APITCH, STAGE = ASTAGE + G8_BSTAGE, SMEM = 2 * STAGE;
  constexpr bool IS_I8 = std::is_same<T, I8>::value;
  constexpr int MI = BM / 64, NJ = 4;
  constexpr int NT = 256;
  constexpr int A_CHUNKS = BM * 8 / NT;                 // 8
  constexpr int B_CHUNKS = G8_BK * (G8_BN / 16) / NT;      // 8
  // MFMA k steps per 128-byte tile: 4 x 32 (int8) or 2 x 64 (fp8).
  constexpr int KS = IS_I8 ? 4 : 2;
  constexpr int FR = IS_I8 ? 1 : 2;                        // 16-byte registers per operand fragment
  using acc_t = typename std::conditional<IS_I8, i32x16, f32x16>::type;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  int tm, tn;
  tile_of_block8(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m_begin = tm * BM, n_begin = tn * G8_BN;
  // K range of this workgroup: all of it, or slice blockIdx.y of a split product.  (`K` below is the
  // length of the range; rows of A are p.K bytes apart either way.)
  const int kz = p.ksplit > 0 ? (int)blockIdx.y * p.ksplit : 0;
  const int K = p.ksplit > 0 ? min(p.ksplit, p.K - kz) : p.K;

  // Global addressing: a wave-uniform tile base (advanced along K on the scalar unit)
  // plus a fixed 32-bit per-lane offset, so a chunk costs one address register.
  const uint8_t* a_base = p.A + (long)m_begin * p.K + kz;
  const uint8_t* b_base = p.B + (long)kz * p.N + n_begin;
  uint32_t a_off[A_CHUNKS], a_lds[A_CHUNKS];
  const int a_chunk = tid & 7;
#pragma unroll
  for (int q = 0; q < A_CHUNKS; ++q) {
    const int row = (tid >> 3) + 32 * q;
    int gr = row;
    gr = m_begin + gr < p.M ? gr : p.M - 1 - m_begin;          // clamp: rows past the edge are never stored
    a_off[q] = (uint32_t)gr * (uint32_t)p.K + a_chunk * 16;
    a_lds[q] = row * G8_APITCH + ((a_chunk ^ ((row >> 1) & 7)) << 4);
  }
  uint32_t b_off[B_CHUNKS], b_lds[B_CHUNKS];
  int b_krow[B_CHUNKS];
#pragma unroll
  for (int q = 0; q < B_CHUNKS; ++q) {
    const int v = tid + NT * q;
    const int krow = v / (G8_BN / 16), nch = v % (G8_BN / 16);
    int gc = nch * 16;
    gc = n_begin + gc < p.N ? gc : p.N - 16 - n_begin;         // clamp: columns past the edge are never stored
    b_off[q] = (uint32_t)krow * (uint32_t)p.N + gc;
    b_lds[q] = ASTAGE + krow * G8_BPITCH + nch * 16;
    b_krow[q] = krow;
  }

  // Global -> register -> LDS staging.  Chunk q < A_CHUNKS is A chunk q, the rest are
  // B chunks.  The chunks of a K step are split into KS groups; a group is written
  // to LDS and immediately refilled with the same chunks of the K step two ahead,
  // so every global load has a full K step of MFMA time to land and loads / LDS
  // writes are spread evenly over it.
  constexpr int NC = A_CHUNKS + B_CHUNKS;
  constexpr int CPG = NC / KS;
  static_assert(NC % KS == 0, "chunks must split evenly over the k steps");
  uint4 st[NC];
  using std::true_type;
  using std::false_type;
  // The guarded form is for a step that may be partial: out-of-range K must
  // contribute exact zeros, which a buffer load returns by itself for an offset
  // past the end of its range.
  auto gfetch = [&](int q, int k0, auto guarded_c) -> uint4 {
    constexpr bool GUARD = decltype(guarded_c)::value;
    if (q < A_CHUNKS) {
      uint32_t off = a_off[q];
      if constexpr (GUARD) off = (k0 + a_chunk * 16 < K) ? off : kOutOfRange;
      return buffer_load_b128(a_base + k0, off);
    } else {
      const int qb = q - A_CHUNKS;
      uint32_t off = b_off[qb];
      if constexpr (GUARD) off = (k0 + b_krow[qb] < K) ? off : kOutOfRange;
      return buffer_load_b128(b_base + (long)k0 * p.N, off);
    }
  };
  auto gload1 = [&](int q, int k0, auto guarded_c) { st[q] = gfetch(q, k0, guarded_c); };
  auto lstore1 = [&](int q, int buf) {
    char* base = smem + buf * STAGE;
    if (q < A_CHUNKS) lds_write_b128(base, a_lds[q], st[q]);
    else lds_write_b128(base, b_lds[q - A_CHUNKS], st[q]);
  };
  // Group g: write its chunks and refill them.  MODE 0 = no refill, 1 = full step,
  // 2 = possibly partial step.
  auto stream_group = [&](int g, int buf_dst, int k0_load, auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int q = g * CPG; q < (g + 1) * CPG; ++q) {
      lstore1(q, buf_dst);
      if constexpr (MODE == 1) gload1(q, k0_load, false_type{});
      if constexpr (MODE == 2) gload1(q, k0_load, true_type{});
    }
  };

  uint32_t a_rd[MI];
  int a_sw[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int row = wm * (BM / 2) + i * 32 + l32;
    a_rd[i] = row * G8_APITCH;
    a_sw[i] = (row >> 1) & 7;
  }
  // Transposing byte read: lane r of a 16-lane block supplies row k0 + r/2 and
  // columns n0 + 8 (r % 2) .. +7; lane i receives column n0 + i, k0 .. k0+7.
  const int r16 = lane & 15;
  const uint32_t b_rd0 = ASTAGE + (16 * lh + (r16 >> 1)) * G8_BPITCH +
                         (wn * 128 + 16 * ((lane >> 4) & 1) + 8 * (r16 & 1));

  acc_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // Fragment f (32 k bytes of the tile: bytes 32 f .. 32 f + 31) gives each lane
  // half its 16 bytes [32 f + 16 h, +16).
  uint4 af[2][MI][FR], bf[2][NJ][FR];
  auto frag_load = [&](int buf, int ks, int slot) {
    const char* base = smem + buf * STAGE;
#pragma unroll
    for (int x = 0; x < FR; ++x) {
      const int f = ks * FR + x;
#pragma unroll
      for (int i = 0; i < MI; ++i)
        af[slot][i][x] = lds_read_b128(base, a_rd[i] + ((((f << 1) | lh) ^ a_sw[i]) << 4));
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const char* pb = base + b_rd0 + f * 32 * G8_BPITCH + j * 32;
        const uint2 lo = lds_read_tr8_b64(pb);
        const uint2 hi = lds_read_tr8_b64(pb + 8 * G8_BPITCH);
        bf[slot][j][x] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    }
  };
  auto mma = [&](int slot) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if constexpr (IS_I8) {
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, bf[slot][j][0]),
                                                            __builtin_bit_cast(i32x4, af[slot][i][0]),
                                                            acc[i][j], 0, 0, 0);
        } else {
          i32x8 a8, b8;
          const i32x4 b0 = __builtin_bit_cast(i32x4, bf[slot][j][0]), b1 = __builtin_bit_cast(i32x4, bf[slot][j][1]);
          const i32x4 a0 = __builtin_bit_cast(i32x4, af[slot][i][0]), a1 = __builtin_bit_cast(i32x4, af[slot][i][1]);
          b8 = (i32x8){b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
          a8 = (i32x8){a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
          // format selectors 0 = e4m3, 1 = e5m2; zero scale operands select the unscaled form.
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, a8, acc[i][j], f8_format<T>(), f8_format<T>(),
                                                                      0, 0, 0, 0);
        }
      }
  };

  // Scheduling hint for one k step of NM MFMAs carrying RD operand reads and (when
  // streaming) CPG LDS writes + CPG global loads: the reads ride the first MFMAs,
  // the write/load pairs the last ones, so every memory instruction issues in the
  // shadow of an MFMA instead of in a burst.
  constexpr int NM = MI * NJ, RD = FR * (MI + 2 * NJ);
  auto hint_step = [&](auto stream_c, auto loads_c) {
    constexpr bool STREAM = decltype(stream_c)::value;
    constexpr bool LOADS = decltype(loads_c)::value;
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
  };

  const int ktiles = (K + G8_BK - 1) / G8_BK;
  using mode0 = std::integral_constant<int, 0>;
  using mode1 = std::integral_constant<int, 1>;
  using mode2 = std::integral_constant<int, 2>;

  // ---- prologue: K step 0 in buffer 0, group 0 of step 1 in buffer 1, the rest of
  // step 1 and group 0 of step 2 in registers ---------------------------------------
  // (the first half of step 1 is requested before step 0 has landed, into registers the
  // operand fragments use later: group 0 of step 1 is then not a second full memory
  // latency behind step 0)
  constexpr int PRE = NC / 2;
#pragma unroll
  for (int q = 0; q < NC; ++q) gload1(q, 0, true_type{});
  uint4 pre[PRE];
  if (ktiles > 1) {
#pragma unroll
    for (int q = 0; q < PRE; ++q) pre[q] = gfetch(q, G8_BK, true_type{});
  }
#pragma unroll
  for (int q = 0; q < NC; ++q) lstore1(q, 0);
  if (ktiles > 1) {
#pragma unroll
    for (int q = PRE; q < NC; ++q) gload1(q, G8_BK, true_type{});
#pragma unroll
    for (int q = 0; q < PRE; ++q) st[q] = pre[q];
    if (ktiles > 2) stream_group(0, 1, 2 * G8_BK, mode2{});
    else stream_group(0, 1, 0, mode0{});
  }
  __syncthreads();
  frag_load(0, 0, 0);

  // One K step.  HAS1: step kt+1 exists (its groups 1.. go to the other buffer during
  // k steps 0..KS-2).  L2 / L3: how steps kt+2 / kt+3 are fetched (0 absent, 1 full,
  // 2 possibly partial).  All compile-time: one straight-line block per barrier
  // interval, with a single load form inside the hot loop.
  auto kstep = [&](int kt, auto has1_c, auto l2_c, auto l3_c) {
    constexpr bool HAS1 = decltype(has1_c)::value;
    constexpr int L2 = decltype(l2_c)::value;
    constexpr int L3 = decltype(l3_c)::value;
    const int buf = kt & 1;
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      frag_load(buf, ks + 1, (ks + 1) & 1);
      if constexpr (HAS1) stream_group(ks + 1, buf ^ 1, (kt + 2) * G8_BK, l2_c);
      mma(ks & 1);
      hint_step(std::integral_constant<bool, HAS1>{}, std::integral_constant<bool, (L2 != 0)>{});
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    if constexpr (HAS1) frag_load(buf ^ 1, 0, KS & 1);
    if constexpr (L2 != 0) stream_group(0, buf, (kt + 3) * G8_BK, l3_c);
    mma((KS - 1) & 1);
    if constexpr (HAS1) hint_step(std::integral_constant<bool, (L2 != 0)>{}, std::integral_constant<bool, (L3 != 0)>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  int kt = 0;
  for (; kt + 4 < ktiles; ++kt) kstep(kt, true_type{}, mode1{}, mode1{});
  if (kt + 3 < ktiles) { kstep(kt, true_type{}, mode1{}, mode2{}); ++kt; }
  if (kt + 2 < ktiles) { kstep(kt, true_type{}, mode2{}, mode0{}); ++kt; }
  if (kt + 1 < ktiles) { kstep(kt, true_type{}, mode0{}, mode0{}); ++kt; }
  kstep(kt, false_type{}, mode0{}, mode0{});

  // ---- epilogue ----
  // acc[i][j][r]: row m = 32 i + l32, col n = 32 j + 8 (r / 4) + 4 h + (r % 4): a lane owns
  // runs of four columns of 32 different rows, and a store issued from that layout
  // touches 32 cache lines with 16 (or 8) bytes each.  The wave stages its tile through
  // its share of the (now free) LDS instead and writes whole row segments, 16 bytes per
  // lane with consecutive lanes along a row.
  constexpr int DSZ = EPI == EPI8_SCALED_BF16 ? 2 : 4;
  constexpr int ROWB = NJ * 32 * DSZ;                  // bytes of one row of the wave's 128-column tile
  constexpr int PITCH = ROWB + 16;
  constexpr int WAVE_LDS = SMEM / 4;
  constexpr int IB = WAVE_LDS / (32 * PITCH) >= MI ? MI : (WAVE_LDS / (32 * PITCH) >= 2 ? 2 : 1);   // 32-row blocks staged per pass
  static_assert(IB * 32 * PITCH <= WAVE_LDS && MI % IB == 0, "epilogue staging does not fit");
  constexpr int LPR = ROWB / 16, RPI = 64 / LPR;       // lanes per row, rows per store instruction
  __syncthreads();                                     // nobody reads the operand tiles any more
  char* stg = smem + wave * WAVE_LDS;
  const int st_row = lane / LPR, st_chunk = lane % LPR;
  const int st_n = n_begin + wn * 128 + st_chunk * (16 / DSZ);
  // one staged pass: `raw` stores the int32 accumulators themselves (the plain int8
  // result, or the optional accumulator copy of the W8A8 form) into `out`
  auto pass = [&](char* out, auto raw_c) __attribute__((always_inline)) {
    constexpr bool RAW = decltype(raw_c)::value;
    constexpr int PDSZ = RAW ? 4 : DSZ;
    static_assert(!RAW || DSZ == 4, "raw accumulators are 4 bytes");
#pragma unroll
    for (int i0 = 0; i0 < MI; i0 += IB) {
#pragma unroll
      for (int ii = 0; ii < IB; ++ii) {
        const int i = i0 + ii;
        float rs = 1.f;
        if constexpr (EPI == EPI8_W8A8_F32 && !RAW) {
          const int m = m_begin + wm * (BM / 2) + i * 32 + l32;
          rs = p.row_scale[m < p.M ? m : p.M - 1];
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            char* dst = stg + (ii * 32 + l32) * PITCH + (j * 32 + q * 8 + lh * 4) * PDSZ;
            if constexpr (RAW) {
              *reinterpret_cast<int4*>(dst) =
                  make_int4(acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
            } else if constexpr (EPI == EPI8_W8A8_F32) {
              const int n = n_begin + wn * 128 + j * 32 + q * 8 + lh * 4;
              // (a column past N is never stored; its scale read stays in range)
              const float4 cs = *reinterpret_cast<const float4*>(p.col_scale + (n < p.N ? n : 0));
              float4 o;
              o.x = ((float)acc[i][j][q * 4 + 0] * rs) * cs.x;
              o.y = ((float)acc[i][j][q * 4 + 1] * rs) * cs.y;
              o.z = ((float)acc[i][j][q * 4 + 2] * rs) * cs.z;
              o.w = ((float)acc[i][j][q * 4 + 3] * rs) * cs.w;
              *reinterpret_cast<float4*>(dst) = o;
            } else {
              const float v0 = ((float)acc[i][j][q * 4 + 0] * p.scale_a) * p.scale_b;
              const float v1 = ((float)acc[i][j][q * 4 + 1] * p.scale_a) * p.scale_b;
              const float v2 = ((float)acc[i][j][q * 4 + 2] * p.scale_a) * p.scale_b;
              const float v3 = ((float)acc[i][j][q * 4 + 3] * p.scale_a) * p.scale_b;
              if constexpr (EPI == EPI8_SCALED_F32) {
                *reinterpret_cast<float4*>(dst) = make_float4(v0, v1, v2, v3);
              } else {
                uint2 pk;
                pk.x = pack2<BF16>(v0, v1);
                pk.y = pack2<BF16>(v2, v3);
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
        const int m = m_begin + wm * (BM / 2) + i0 * 32 + row;
        // N % 16 == 0 on this path: a 16-byte chunk is inside or outside as a whole
        if (m < p.M && st_n < p.N) *reinterpret_cast<uint4*>(out + ((long)m * p.N + st_n) * PDSZ) = v;
      }
      __builtin_amdgcn_wave_barrier();
    }
  };
  char* out_base = reinterpret_cast<char*>(p.D);
  if (p.ksplit > 0) out_base += (long)blockIdx.y * p.M * p.N * DSZ;   // this slice's partial result
  if constexpr (EPI == EPI8_I32) {
    pass(out_base, true_type{});
  } else {
    pass(out_base, false_type{});
    if constexpr (EPI == EPI8_W8A8_F32) {
      if (p.acc_out) pass(reinterpret_cast<char*>(p.acc_out), true_type{});
    }
  }
}

// e4m3fn (OCP) byte -> f32: bias 7, no infinities, 0x7f / 0xff are NaN.
__device__ __forceinline__ float e4m3_to_f32(uint8_t c) {
  const uint32_t s = (uint32_t)(c & 0x80) << 24;
  const uint32_t e = (c >> 3) & 0xF, m = c & 7;
  float v;
  if (e == 0) v = (float)m * 0.001953125f;                       // m * 2^-9
  else if (e == 15 && m == 7) v = __builtin_nanf("");
  else v = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
  return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) | s);
}

// e5m2 (OCP) byte -> f32: the byte is the upper half of the IEEE half-precision pattern.
__device__ __forceinline__ float e5m2_to_f32(uint8_t c) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)((uint16_t)c << 8));
}
template <class T> __device__ __forceinline__ float f8_to_f32(uint8_t c) {
  if constexpr (std::is_same<T, BF8>::value) return e5m2_to_f32(c);
  else return e4m3_to_f32(c);
}

// A product split along K: the slices' partial results (int32 accumulators, or f32 ones of the fp8
// form computed with unit scales), [splits][M][N], are summed in slice order and passed through
// the product's epilogue.  int32 sums are exact, so the int8 forms give the bits of the unsplit
// kernel; the f32 sum of the fp8 form is one fixed order.  Four columns per thread.
template <class T, int EPI>
__global__ __launch_bounds__(256) void gemm8_split_sum_kernel(const void* __restrict__ part, int splits, const Gemm8Params p) {
  constexpr bool IS_I8 = std::is_same<T, I8>::value;
  const long quad = (long)blockIdx.x * 256 + threadIdx.x;
  const int nq = p.N / 4;
  if (quad >= (long)p.M * nq) return;
  const int m = (int)(quad / nq), n = (int)(quad - (long)m * nq) * 4;
  const long o = (long)m * p.N + n, mn = (long)p.M * p.N;
  float v[4];
  if constexpr (IS_I8) {
    // (the partials of four slices are fetched together: they were written by other XCDs, so every
    // one of these loads pays a trip to memory)
    int4 acc = make_int4(0, 0, 0, 0);
    for (int z0 = 0; z0 < splits; z0 += 4) {
      int4 a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        a[u] = z0 + u < splits ? *reinterpret_cast<const int4*>(reinterpret_cast<const int32_t*>(part) + (z0 + u) * mn + o)
                               : make_int4(0, 0, 0, 0);
#pragma unroll
      for (int u = 0; u < 4; ++u) { acc.x += a[u].x; acc.y += a[u].y; acc.z += a[u].z; acc.w += a[u].w; }
    }
    if constexpr (EPI == EPI8_I32) {
      *reinterpret_cast<int4*>(reinterpret_cast<int32_t*>(p.D) + o) = acc;
      return;
    } else {
      if (p.acc_out) *reinterpret_cast<int4*>(p.acc_out + o) = acc;
      const float rs = p.row_scale[m];
      const float4 cs = *reinterpret_cast<const float4*>(p.col_scale + n);
      v[0] = ((float)acc.x * rs) * cs.x; v[1] = ((float)acc.y * rs) * cs.y;
      v[2] = ((float)acc.z * rs) * cs.z; v[3] = ((float)acc.w * rs) * cs.w;
    }
  } else {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int z0 = 0; z0 < splits; z0 += 4) {
      float4 a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        a[u] = z0 + u < splits ? *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(part) + (z0 + u) * mn + o)
                               : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 4; ++u) { acc.x += a[u].x; acc.y += a[u].y; acc.z += a[u].z; acc.w += a[u].w; }   // slice order
    }
    v[0] = (acc.x * p.scale_a) * p.scale_b; v[1] = (acc.y * p.scale_a) * p.scale_b;
    v[2] = (acc.z * p.scale_a) * p.scale_b; v[3] = (acc.w * p.scale_a) * p.scale_b;
  }
  if constexpr (EPI == EPI8_SCALED_BF16) {
    uint2 pk;
    pk.x = pack2<BF16>(v[0], v[1]);
    pk.y = pack2<BF16>(v[2], v[3]);
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.D) + o) = pk;
  } else if constexpr (EPI != EPI8_I32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.D) + o) = make_float4(v[0], v[1], v[2], v[3]);
  }
}

// Any-shape fallback, one thread per output element, k in order.
template <class T, int EPI>
__global__ void gemm8_generic_kernel(const Gemm8Params p) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int m = blockIdx.y * blockDim.y + threadIdx.y;
  if (m >= p.M || n >= p.N) return;
  const long o = (long)m * p.N + n;
  if constexpr (std::is_same<T, I8>::value) {
    const int8_t* A = reinterpret_cast<const int8_t*>(p.A) + (long)m * p.K;
    const int8_t* B = reinterpret_cast<const int8_t*>(p.B) + n;
    int32_t acc = 0;
    for (int k = 0; k < p.K; ++k) acc += (int32_t)A[k] * (int32_t)B[(long)k * p.N];
    if constexpr (EPI == EPI8_I32) {
      reinterpret_cast<int32_t*>(p.D)[o] = acc;
    } else {
      reinterpret_cast<float*>(p.D)[o] = ((float)acc * p.row_scale[m]) * p.col_scale[n];
      if (p.acc_out) p.acc_out[o] = acc;
    }
  } else {
    const uint8_t* A = p.A + (long)m * p.K;
    const uint8_t* B = p.B + n;
    float acc = 0.f;
    for (int k = 0; k < p.K; ++k) acc += f8_to_f32<T>(A[k]) * f8_to_f32<T>(B[(long)k * p.N]);
    const float v = (acc * p.scale_a) * p.scale_b;
    if constexpr (EPI == EPI8_SCALED_F32) reinterpret_cast<float*>(p.D)[o] = v;
    else reinterpret_cast<uint16_t*>(p.D)[o] = f32_to_bf16_bits(v);
  }
}

}  // namespace tsr950
