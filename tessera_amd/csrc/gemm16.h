// 16-bit (bf16 / f16) MFMA GEMM for gfx950:  D[M,N] = A[M,K] . B[K,N], row-major,
// f32 accumulate.  One kernel template serves the dense, strided-batched and
// grouped (per-expert, ragged) forms and the fused SwiGLU gate/up form.
//
// Tiling.  A workgroup of WM x WN waves owns a BM x BN output tile and walks K
// in steps of BK = 64.  Each wave owns a (BM/WM) x (BN/WN) sub-tile held as
// 32x32 MFMA accumulators (v_mfma_f32_32x32x16_{bf16,f16}).  With the default
// 256x256 tile and 2x2 waves every wave keeps a 128x128 f32 accumulator (256
// registers) — one wave per SIMD, the full 512-register budget — which needs
// 512 B of LDS operand reads per MFMA, half of the 128 B/clk the LDS sustains.
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
};

struct Gemm16Params {
  const uint16_t* A;
  const uint16_t* B;
  const uint16_t* B2;     // second weight (SwiGLU "up"), else null
  void* D;
  int M, N, K;
  long lda, ldb, ldd;     // in elements
  long strideA, strideB, strideD;   // batch / expert strides in elements
  const int* offsets;     // grouped: device int32[E+1] row offsets into A and D; else null
  int groups;             // E (grouped) or batch count
  int tiles_m, tiles_n;   // tile grid (grouped: tiles_m is an upper bound)
};

#ifndef TSR_NO_SGB
#define TSR_SGB(mask, n, id) __builtin_amdgcn_sched_group_barrier(mask, n, id)
#else
#define TSR_SGB(mask, n, id)
#endif
#ifndef TSR_NO_SB
#define TSR_SB() __builtin_amdgcn_sched_barrier(0)
#else
#define TSR_SB()
#endif

constexpr int G16_BK = 64;          // K step, elements
constexpr int G16_APITCH = 128;     // bytes per A row in LDS
constexpr int G16_BPAD = 16;        // B row pad, elements

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

template <class T, int BM, int BN, int WM, int WN, int EPI, bool GROUPED>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm16_kernel(const Gemm16Params p) {
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM, TN = BN / WN;     // wave tile
  constexpr int MI = TM / 32, NJ = TN / 32;     // 32x32 MFMA tiles per wave
  constexpr bool SWIGLU = (EPI == EPI_SWIGLU16);
  // SwiGLU: the BN columns of the LDS B tile are [gate n0..n0+BN/2) | up n0..n0+BN/2);
  // a wave's first NJ/2 column tiles are gate and the rest the matching up columns.
  static_assert(!SWIGLU || (WN == 1 && NJ % 2 == 0), "SwiGLU form needs WN == 1");
  using S = Gemm16Smem<BM, BN>;
  constexpr int A_CHUNKS = BM * 8 / NT;         // 16-byte chunks per thread per stage
  constexpr int B_CHUNKS = G16_BK * (BN / 8) / NT;
  static_assert(BM * 8 % NT == 0 && G16_BK * (BN / 8) % NT == 0, "tile/thread mismatch");

  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  // ---- which tile ---------------------------------------------------------
  int tm, tn, m_begin, m_end;
  const uint16_t* Ab = p.A;
  const uint16_t* Bb = p.B;
  const uint16_t* B2b = p.B2;
  char* Db = (char*)p.D;
  constexpr int DSZ = (EPI == EPI_F32) ? 4 : 2;
  if constexpr (GROUPED) {
    // blockIdx.x = n tile, blockIdx.y = running m-tile index over all groups.
    tn = blockIdx.x;
    int want = blockIdx.y, e = 0, acc_tiles = 0, g_lo = 0, g_hi = 0;
    bool found = false;
    for (e = 0; e < p.groups; ++e) {
      g_lo = p.offsets[e];
      g_hi = p.offsets[e + 1];
      const int t = (g_hi - g_lo + BM - 1) / BM;
      if (want < acc_tiles + t) { found = true; break; }
      acc_tiles += t;
    }
    if (!found) return;
    tm = want - acc_tiles;
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
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;   // output columns per tile
  const int n_begin = tn * BN_OUT;
  const int K = p.K;

  // ---- global load addressing (fixed per thread, advanced by BK each step) --
  // A: chunk v = tid + NT*q  -> row v/8, 16-byte chunk v%8.
  const uint16_t* a_ptr[A_CHUNKS];
  uint32_t a_lds[A_CHUNKS];
  const int a_chunk = tid & 7;
#pragma unroll
  for (int q = 0; q < A_CHUNKS; ++q) {
    const int row = (tid >> 3) + (NT / 8) * q;
    int gr = m_begin + row;
    gr = gr < m_end ? gr : m_end - 1;            // clamp: rows past the edge are never stored
    a_ptr[q] = Ab + (long)gr * p.lda + a_chunk * 8;
    a_lds[q] = row * G16_APITCH + ((a_chunk ^ (row & 7)) << 4);
  }
  // B: chunk v = tid + NT*q -> k row v/(BN/8), n chunk v%(BN/8).
  const uint16_t* b_ptr[B_CHUNKS];
  uint32_t b_lds[B_CHUNKS];
  int b_krow[B_CHUNKS];
#pragma unroll
  for (int q = 0; q < B_CHUNKS; ++q) {
    const int v = tid + NT * q;
    const int krow = v / (BN / 8);
    const int nch = v % (BN / 8);
    const uint16_t* src = Bb;
    int col = nch * 8;
    if constexpr (SWIGLU) {
      if (col >= BN / 2) { src = B2b; col -= BN / 2; }
    }
    int gc = n_begin + col;
    gc = gc < p.N ? gc : (p.N - 8);              // clamp: columns past the edge are never stored
    b_ptr[q] = src + (long)krow * p.ldb + gc;
    b_lds[q] = S::kAStage + krow * S::kBPitch + nch * 16;
    b_krow[q] = krow;
  }

  uint4 ra[A_CHUNKS], rb[B_CHUNKS];
  // Global -> register prefetch of the K step starting at k0.  The guarded form
  // is for a step that may be partial: out-of-range K must contribute exact
  // zeros on both operands, so the load address is pulled back in range and the
  // value replaced.  Only the last step can be partial; the hot loop uses the
  // plain form.
  auto gload = [&](int k0, auto guarded_c) {
    if constexpr (!decltype(guarded_c)::value) {
#pragma unroll
      for (int q = 0; q < A_CHUNKS; ++q) ra[q] = *reinterpret_cast<const uint4*>(a_ptr[q] + k0);
#pragma unroll
      for (int q = 0; q < B_CHUNKS; ++q) rb[q] = *reinterpret_cast<const uint4*>(b_ptr[q] + (long)k0 * p.ldb);
    } else {
#pragma unroll
      for (int q = 0; q < A_CHUNKS; ++q) {
        const bool ok = k0 + a_chunk * 8 < K;
        const uint4 v = *reinterpret_cast<const uint4*>(a_ptr[q] + (ok ? k0 : -(a_chunk * 8)));
        ra[q].x = ok ? v.x : 0u; ra[q].y = ok ? v.y : 0u; ra[q].z = ok ? v.z : 0u; ra[q].w = ok ? v.w : 0u;
      }
#pragma unroll
      for (int q = 0; q < B_CHUNKS; ++q) {
        const bool ok = k0 + b_krow[q] < K;
        const uint4 v = *reinterpret_cast<const uint4*>(b_ptr[q] + (ok ? (long)k0 : -(long)b_krow[q]) * p.ldb);
        rb[q].x = ok ? v.x : 0u; rb[q].y = ok ? v.y : 0u; rb[q].z = ok ? v.z : 0u; rb[q].w = ok ? v.w : 0u;
      }
    }
  };
  auto lstore = [&](int buf) {
    char* base = smem + buf * S::kStage;
#pragma unroll
    for (int q = 0; q < A_CHUNKS; ++q) lds_write_b128(base, a_lds[q], ra[q]);
#pragma unroll
    for (int q = 0; q < B_CHUNKS; ++q) lds_write_b128(base, b_lds[q], rb[q]);
  };

  // ---- operand read addressing --------------------------------------------
  const int l32 = lane & 31, lh = lane >> 5;
  uint32_t a_rd[MI];       // byte offset of this lane's row; chunk applied per k step
  int a_sw[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int row = wm * TM + i * 32 + l32;
    a_rd[i] = row * G16_APITCH;
    a_sw[i] = row & 7;
  }
  // transposing read: lane supplies row (k) = 8*lh + r/4 (+4 for the second
  // half), columns n = 32j + 16*((lane>>4)&1) + 4*(r%4), r = lane & 15.
  const int r16 = lane & 15;
  const uint32_t b_rd0 = S::kAStage + (8 * lh + (r16 >> 2)) * S::kBPitch +
                         (wn * TN + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3)) * 2;

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Operand fragments are double buffered in registers: the LDS reads of k
  // step s+1 are issued before the MFMAs of step s, which hide their latency.
  uint4 af[2][MI], bf[2][NJ];
  auto frag_load = [&](int buf, int ks, int slot) {
    const char* base = smem + buf * S::kStage;
#pragma unroll
    for (int i = 0; i < MI; ++i)
      af[slot][i] = lds_read_b128(base, a_rd[i] + ((((ks << 1) | lh) ^ a_sw[i]) << 4));
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const char* pb = base + b_rd0 + ks * 16 * S::kBPitch + j * 64;
      const uint2 lo = lds_read_tr16_b64(pb);
      const uint2 hi = lds_read_tr16_b64(pb + 4 * S::kBPitch);
      bf[slot][j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
    }
  };
  auto mma = [&](int slot) {
#ifdef TSR_WAIT_LGKM0
    __builtin_amdgcn_s_waitcnt(0xc07f);
#endif
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = mfma_32x32x16<T>(bf[slot][j], af[slot][i], acc[i][j]);
  };
  // Scheduling hint: pair every LDS read with an MFMA so the reads issue in the
  // shadow of the matrix pipe instead of in a burst in front of it.
  auto interleave_reads = [&]() {
#pragma unroll
    for (int x = 0; x < MI + 2 * NJ; ++x) {
      TSR_SGB(0x008, 1, 0);   // 1 MFMA
      TSR_SGB(0x100, 1, 0);   // 1 DS read
    }
  };

  constexpr int KS = G16_BK / 16;
  const int ktiles = (K + G16_BK - 1) / G16_BK;
  using std::true_type;
  using std::false_type;
  using no_prefetch = std::integral_constant<int, 0>;
  using full_prefetch = std::integral_constant<int, 1>;
  using tail_prefetch = std::integral_constant<int, 2>;
  gload(0, true_type{});
  lstore(0);
  __syncthreads();
  if (ktiles > 1) gload(G16_BK, true_type{});
  frag_load(0, 0, 0);

  // One K step.  MORE: another step follows (its tile is in registers and goes to
  // the other LDS buffer now).  PREFETCH: the step after that exists and is
  // fetched from global memory (1 = known full tile, 2 = possibly partial).
  // Both are compile-time so the body is one straight-line block.
  auto kstep = [&](int kt, auto more_c, auto prefetch_c) {
    constexpr bool MORE = decltype(more_c)::value;
    constexpr int PREFETCH = decltype(prefetch_c)::value;
    const int buf = kt & 1;
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      frag_load(buf, ks + 1, (ks + 1) & 1);
      if (MORE && ks == KS - 2) lstore(buf ^ 1);
      mma(ks & 1);
      if (MORE && ks == KS - 2) {
#pragma unroll
        for (int x = 0; x < MI + 2 * NJ; ++x) {
          TSR_SGB(0x008, 1, 0);
          TSR_SGB(0x100, 1, 0);
          TSR_SGB(0x200, (A_CHUNKS + B_CHUNKS + MI + 2 * NJ - 1) / (MI + 2 * NJ), 0);
        }
      } else {
        interleave_reads();
      }
      TSR_SB();
    }
    // All of this wave's reads of the current buffer are issued; once every wave
    // passes the barrier the other buffer is complete and this one is free.
    __syncthreads();
    if constexpr (MORE) {
      if constexpr (PREFETCH == 1) gload((kt + 2) * G16_BK, false_type{});
      if constexpr (PREFETCH == 2) gload((kt + 2) * G16_BK, true_type{});
      frag_load(buf ^ 1, 0, KS & 1);
    }
    mma((KS - 1) & 1);
    if constexpr (MORE) interleave_reads();
    TSR_SB();
  };
  int kt = 0;
  // Tile kt+2 <= ktiles-2 is always a full tile; only the last one can be partial.
  for (; kt + 3 < ktiles; ++kt) kstep(kt, true_type{}, full_prefetch{});
  if (kt + 2 < ktiles) { kstep(kt, true_type{}, tail_prefetch{}); ++kt; }
  if (kt + 1 < ktiles) { kstep(kt, true_type{}, no_prefetch{}); ++kt; }
  kstep(kt, false_type{}, no_prefetch{});

  // ---- epilogue -------------------------------------------------------------
  // acc[i][j][r]: row m = 32i + l32, col n = 32j + 8*(r/4) + 4*lh + (r%4).
  constexpr int NJ_OUT = SWIGLU ? NJ / 2 : NJ;
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_begin + wm * TM + i * 32 + l32;
    if (m >= m_end) continue;
    char* drow = Db + (long)m * p.ldd * DSZ;
#pragma unroll
    for (int j = 0; j < NJ_OUT; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n_begin + (SWIGLU ? 0 : wn * TN) + j * 32 + q * 8 + lh * 4;
        if (n >= p.N) continue;                  // N % 8 == 0 on this path: all-or-nothing per run of 4
        float v0 = acc[i][j][q * 4 + 0], v1 = acc[i][j][q * 4 + 1];
        float v2 = acc[i][j][q * 4 + 2], v3 = acc[i][j][q * 4 + 3];
        if constexpr (EPI == EPI_F32) {
          *reinterpret_cast<float4*>(drow + (long)n * 4) = make_float4(v0, v1, v2, v3);
        } else {
          if constexpr (SWIGLU) {
            const f32x16& u = acc[i][j + NJ / 2];
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
          *reinterpret_cast<uint2*>(drow + (long)n * 2) = pk;
        }
      }
    }
  }
}

}  // namespace tsr950
