// Flash-attention forward for gfx950: O = softmax(scale * Q K^T, causal) V with
// GQA and the per-row log-sum-exp, 16-bit storage, f32 softmax and accumulate.
//
// The kernel is compiled for a padded head dimension DP in {64, 128, 256} and serves every
// head dimension D <= DP that is a multiple of 16 (the matrix path of the reference's
// kernel, tessera_rocm_flash_attn.cpp:47-144): with D < DP the missing columns of Q, K and
// V are zeros (registers set to zero, LDS columns cleared once and never loaded), which
// leaves the scores unchanged and yields output columns that are not stored.  Q, K, V and O
// are addressed through (batch, head, row) strides, so [B,H,S,D], [B,S,H,D] and column
// slices of a fused projection output are all served without a copy.
//
// One workgroup of 8 waves (two per SIMD) owns 256 query rows of one (batch, q
// head); each wave owns 32 of them as one MFMA tile.  (DP = 256: 128 query rows; two waves
// share each 32-row block, both computing its scores, each accumulating one half of the
// output columns — see FlashGeom.)  K/V are walked in 64-key
// tiles that stream from global memory straight into LDS (two stages each, one
// barrier per tile).  The loop is software-pipelined: the score MFMAs of tile
// t+1 are issued under the softmax arithmetic of tile t, and the exponentials of
// each 8-key group just ahead of the P.V MFMAs that consume it; the second wave
// on each SIMD fills what is left.  (FA_QT = 2, four waves of 64 rows sharing
// each K/V fragment between two query tiles, halves the LDS reads but leaves one
// wave per SIMD and measured 40 % slower.)
//
// Both products are issued TRANSPOSED so that everything a lane holds belongs
// to ONE query row (q = lane % 32):
//   S^T[key][q] = K[key][:] . Q[q][:]      MFMA A-operand = K rows (ds_read_b128),
//                                          B-operand = Q rows (registers, loaded once)
//   O^T[d][q]  += V^T[d][key] . P^T[key][q] A-operand = V columns, read from the
//                                          natural [key][d] LDS tile with the
//                                          transposing ds_read_b64_tr_b16,
//                                          B-operand = P, straight from the S^T
//                                          accumulator registers.
// A lane's 16 accumulators of an S^T tile are keys {8a + 4h + b} (h = lane/32);
// registers 8g..8g+7 are exactly the 8 keys the lane must supply as B-operand of
// the g-th 16-key MFMA step once the V operand uses the same key order — so P
// never leaves its registers and the softmax row statistics (max, sum, rescale)
// are lane-local, with one exchange between the two lane halves per row.
//
// LDS tiles keep the natural row-major layout; 16-byte chunks are XOR-swizzled so
// the K operand reads (16 consecutive rows, one chunk column, per LDS cycle) and
// the V patch reads (4 consecutive rows x 64 bytes) spread over all 64 banks.
#pragma once
#include <type_traits>
#include "common.h"

namespace tsr950 {

// Element (b, h, s, d) of a strided operand X is X[b * batch + h * head + s * row + d].
struct FlashStrides {
  long batch, head, row;
};
struct FlashParams {
  const uint16_t* Q;   // (B, Hq, Sq, D) through qs
  const uint16_t* K;   // (B, Hkv, Sk, D) through ks
  const uint16_t* V;   // (B, Hkv, Sk, D) through vs
  void* O;             // (B, Hq, Sq, D) through os, f32 or storage dtype
  float* LSE;          // [B, Hq, Sq] contiguous, or null
  FlashStrides qs, ks, vs, os;
  int B, Hq, Hkv, Sq, Sk;
  int D;               // head dimension, a multiple of 16, <= the kernel's DP
  float scale;
  int causal;
  int out_storage;     // 0: f32 O, 1: O in the storage dtype
  int window;          // > 0: band of keys per query (see key_bounds); 0: none
  float softcap;       // > 0: scaled scores pass through cap * tanh(s / cap); 0: none
  int ratio;           // Hq / Hkv
  const float* bias;   // additive bias [B, Hq, Sq, Sk] f32 added to the (capped) scaled scores, or null
  // Key splits (few workgroups against a long key range): gridDim.y = query blocks x nsplit;
  // split s of a workgroup covers the 64-key tiles [s tiles_per_split, (s + 1) tiles_per_split)
  // of its key range and writes a normalised partial O (f32, contiguous [B, Hq, Sq, D]) and its
  // log-sum-exp at O + s split_o_elems and LSE + s B Hq Sq; flash_decode_merge_kernel merges them.
  int nsplit;          // 0 or 1: none
  int tiles_per_split;
  long split_o_elems;  // B Hq Sq D
};

// Visible keys [lo, hi] of query row i — the reference's attention_bounds
// (avx512_flash_attn_f32.cpp:180-196): causal masks keys past the bottom-right
// aligned diagonal; a window keeps the `window` keys ending at the diagonal (causal)
// or window/2 keys either side of it.
__host__ __device__ inline void key_bounds(int i, int Sq, int Sk, int causal, int window, int& lo, int& hi) {
  const int off = Sk > Sq ? Sk - Sq : 0;
  lo = 0;
  hi = causal ? i + off : Sk - 1;
  if (window > 0) {
    if (causal) { lo = i + off - window + 1; hi = i + off; }
    else { lo = i + off - window / 2; hi = i + off + window / 2; }
  }
  lo = lo > 0 ? lo : 0;
  hi = hi < Sk - 1 ? hi : Sk - 1;
}

constexpr int FA_QT = 1;               // 32-row query tiles per wave
constexpr int FA_BKV = 64;             // keys per LDS tile
// Per padded head dimension: waves per workgroup (always two per SIMD), how many waves share
// one 32-row block by output columns, query rows per workgroup, 16-byte chunks per LDS row,
// bytes of one K (or V) stage, LDS bytes.
template <int DP> struct FlashGeom {
  static constexpr int WAVES = 8;
  static constexpr int THREADS = WAVES * 64;
  // DP = 256: a wave's 32 rows x 256 output columns would be 128 accumulator registers, which
  // does not fit next to 64 Q and 64 score registers in the 256 a wave has at two per SIMD.
  // Two waves therefore share each 32-row block: both compute its scores and softmax (the same
  // bits), each accumulates one half of the output columns.
  static constexpr int DSPLIT = DP > 128 ? 2 : 1;
  static constexpr int BQ = WAVES / DSPLIT * 32 * FA_QT;
  static constexpr int CHUNKS = DP / 8;
  static constexpr int TILE = FA_BKV * DP * 2;
  static constexpr int STAGE_PITCH = DP / DSPLIT * 4 + 16;     // epilogue staging row, f32
  static constexpr int SMEM = 4 * TILE > WAVES * 32 * FA_QT * STAGE_PITCH ? 4 * TILE : WAVES * 32 * FA_QT * STAGE_PITCH;
};
constexpr float FA_NEG = -1.0e30f;

// Exchange a value with the lane 32 positions away.
__device__ __forceinline__ float swap_half(float v) {
  return __shfl_xor(v, 32, 64);
}
// max of a value and the one held by the lane 32 positions away: one
// v_permlane32_swap (the upper 32 lanes of the first register change places with the
// lower 32 of the second) leaves both halves' values side by side in every lane, with
// no LDS round trip.  The operands are finite, so the raw maximum serves.
__device__ __forceinline__ float max_with_other_half(float v) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  float d;
  asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(__uint_as_float(r[0])), "v"(__uint_as_float(r[1])));
  return d;
}

// max(a, b, c) in one instruction; the operands are finite MFMA results, so the
// NaN canonicalisation fmaxf() would add per operand is not needed.
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}

// 16 bytes per lane from global memory straight into LDS: lane i's data lands at
// lds_base + 16 i (lds_base wave-uniform); the global address is a uniform base
// plus a per-lane byte offset.  Issued as inline assembly so that the compiler
// does not serialise later LDS reads of OTHER stages behind it; the kernel waits
// for these loads itself (fa_wait_loads) before the barrier that publishes the
// stage.
__device__ __forceinline__ void load16_to_lds(const void* base, uint32_t byte_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(byte_off), "s"(base) : "memory");
}
__device__ __forceinline__ void fa_wait_loads() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// acc *= corr for an accumulator element that lives in the accumulation register
// file: the output accumulators are touched by vector arithmetic only here (a rare
// path), so keeping them out of the ordinary register file leaves that file to the
// score tiles and operand fragments.
__device__ __forceinline__ float scale_acc(float acc, float corr) {
  float tmp;
  asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
               : "+a"(acc), "=&v"(tmp) : "v"(corr));
  return acc;
}

template <class T, int DP, bool EXT, bool PAD>
__global__ __launch_bounds__(FlashGeom<DP>::THREADS, 1) void flash_fwd_kernel(const FlashParams p) {
  using G = FlashGeom<DP>;
  constexpr int D = DP;                  // extent the loops are unrolled for
  constexpr int FA_WAVES = G::WAVES, FA_THREADS = G::THREADS, FA_BQ = G::BQ;
  constexpr int FA_KT = FA_BKV / 32;     // 32-key MFMA tiles per LDS tile
  constexpr int QT = FA_QT;
  constexpr int KSTEPS = D / 16;         // MFMA k steps of the score product
  constexpr int KA = (KSTEPS + 3) / 4;   // score k steps issued under the row-max phase
  constexpr int KB = (KSTEPS + KA) / 2;  // ... and up to here under the first exponentials
  constexpr int DS = G::DSPLIT;          // waves that share a row block, splitting the output columns
  constexpr int DT = D / 32 / DS;        // 32-wide d tiles of the output this wave accumulates
  constexpr int ROWB = D * 2;            // bytes per K/V row
  constexpr int CHUNKS = D / 8;          // 16-byte chunks per row
  constexpr int TILE = FA_BKV * ROWB;    // bytes per K (or V) tile
  constexpr int LD_PER_THREAD = FA_BKV * CHUNKS / FA_THREADS;
  static_assert(FA_BKV * CHUNKS % FA_THREADS == 0, "tile/thread mismatch");
  // K swizzle: the 16 rows an LDS cycle serves must hit 16 different 16-byte slots
  // of the 256-byte bank line.  V swizzle: the 4 rows of a patch, 64 bytes each.
  // (Rows of 256 or 512 bytes start in the same bank: 16 different chunks, and four keys a
  // 64-byte step apart; rows of 128 bytes alternate between the two halves of the banks.)
  auto kswz = [](int row) { return CHUNKS % 16 == 0 ? (row & 15) : ((row >> 1) & 7); };
  auto vswz = [](int key) { return CHUNKS % 16 == 0 ? ((key & 3) << 2) : (((key >> 1) & 1) << 2); };

  // LDS: K stages at 0 and TILE, V stages at 2 TILE and 3 TILE.
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const uint32_t lds0 = (uint32_t)(uintptr_t)(TSR_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;

  // Work order.  Workgroups are dealt to the 8 XCDs round-robin by their linear id.
  // The grid is (8 * ratio, query blocks, B * Hkv / 8) when B * Hkv is a multiple of 8:
  // x runs fastest in the dispatch order, so a run of 8 * ratio workgroups puts the
  // query heads that share a KV head on one XCD, where they find its K / V in that
  // XCD's L2; then come the query blocks of those heads, heaviest first (with a causal
  // mask the last block has the longest key range); then the next 8 KV heads.  An XCD
  // therefore works on one or two KV heads at a time (2 MB of K and V each at
  // S = 4096, against 4 MB of L2) instead of on all of its heads at once.  Otherwise
  // the grid is (B * Hq, query blocks, 1), heaviest blocks first.  No index needs a
  // division either way.
  // qlin / kvlin: linear (batch, head) index of the query head / of its KV head.
  const int nsplit = p.nsplit > 1 ? p.nsplit : 1;
  const int split = p.nsplit > 1 ? (int)blockIdx.y % nsplit : 0;
  const int qb = (int)gridDim.y / nsplit - 1 - (int)blockIdx.y / nsplit;
  int qlin, kvlin;
  if (gridDim.z > 1 || (int)gridDim.x == 8 * p.ratio) {
    const int w = blockIdx.x;
    kvlin = blockIdx.z * 8 + (w & 7);
    qlin = kvlin * p.ratio + (w >> 3);
  } else {
    qlin = blockIdx.x;
    kvlin = qlin / p.ratio;
  }
  const int batch = kvlin / p.Hkv;
  const int hkv = kvlin - batch * p.Hkv, hq = qlin - batch * p.Hq;

  const int q0 = qb * FA_BQ;                  // first query row of the workgroup
  // Waves w and w + 4 share a SIMD.  Under a causal mask a wave's key range grows with
  // its row block, so the upper four waves take the row blocks in reverse: every SIMD
  // gets one of the blocks 0-3 and its mirror image 7-4, the same work on all four.
  constexpr int RB = FA_WAVES / DS;            // row blocks of the workgroup
  const int dsel = wave / RB;                  // which part of the output columns this wave accumulates
  const int wrow = wave - dsel * RB;
  const int rblk = wrow < RB / 2 ? wrow : RB + RB / 2 - 1 - wrow;
  const int qw = q0 + rblk * (32 * QT);       // first query row of the wave
  const uint16_t* Qb = p.Q + batch * p.qs.batch + hq * p.qs.head;
  const uint16_t* Kb = p.K + batch * p.ks.batch + hkv * p.ks.head;
  const uint16_t* Vb = p.V + batch * p.vs.batch + hkv * p.vs.head;
  const int ksteps_real = PAD ? p.D / 16 : KSTEPS;      // k steps that hold data; the rest is zero padding

  // Key tiles this workgroup needs: from the first visible key of its first row to
  // the last visible key of its last row (bounds are monotone in the row index).
  // `t` below counts tiles from tile_base.
  int lo_first, hi_first, lo_last, hi_last;
  key_bounds(q0, p.Sq, p.Sk, p.causal, p.window, lo_first, hi_first);
  key_bounds(min(q0 + FA_BQ, p.Sq) - 1, p.Sq, p.Sk, p.causal, p.window, lo_last, hi_last);
  int tile_base = lo_first / FA_BKV;
  int ntiles = max((hi_last + FA_BKV) / FA_BKV - tile_base, 0);
  if (p.nsplit > 1) {                         // this split's share of the tile range (possibly none)
    const int lo = max(tile_base, split * p.tiles_per_split);
    const int hi = min(tile_base + ntiles, (split + 1) * p.tiles_per_split);
    tile_base = lo;
    ntiles = max(hi - lo, 0);
  }
  // Tiles this wave computes on: from (an even number of tiles before) its first
  // row's first key to its last row's last key.
  int nt_w = 0, t_w0 = 0;
  int wlo_first = 0, whi_first = 0, wlo_last = 0, whi_last = 0;   // bounds of the wave's first / last row
  if (qw < p.Sq) {
    key_bounds(qw, p.Sq, p.Sk, p.causal, p.window, wlo_first, whi_first);
    key_bounds(min(qw + 32 * QT, p.Sq) - 1, p.Sq, p.Sk, p.causal, p.window, wlo_last, whi_last);
    nt_w = min(max((whi_last + FA_BKV) / FA_BKV - tile_base, 0), ntiles);
    t_w0 = min(max(wlo_first / FA_BKV - tile_base, 0) & ~1, nt_w);
  }

  // ---- Q fragments: lane (q = l32, h) holds Q[q][16 ks + 8 h .. +7] -----------
  uint4 qf[QT][KSTEPS];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    int row = qw + 32 * qt + l32;
    row = row < p.Sq ? row : p.Sq - 1;
    const uint16_t* src = Qb + (long)row * p.qs.row + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
      qf[qt][ks] = (!PAD || ks < ksteps_real) ? *reinterpret_cast<const uint4*>(src + 16 * ks) : make_uint4(0u, 0u, 0u, 0u);
  }

  // ---- K/V tile loaders: straight from global memory into LDS ----------------------
  // One wave instruction fills 64 consecutive 16-byte LDS slots; slot P is (row
  // P / CHUNKS, physical chunk P % CHUNKS) and holds the row's logical chunk
  // (physical ^ swizzle(row)), so the swizzle is applied on the global address.
  // With D < DP the chunks past the row's end are never loaded (those lanes sit out): their
  // LDS slots keep the zeros written below.
  int ld_row[LD_PER_THREAD];
  uint32_t ld_koff[LD_PER_THREAD], ld_voff[LD_PER_THREAD];   // byte offsets inside a full tile
  bool ld_kok[LD_PER_THREAD], ld_vok[LD_PER_THREAD];
  const uint32_t krow_bytes = (uint32_t)p.ks.row * 2, vrow_bytes = (uint32_t)p.vs.row * 2;
#pragma unroll
  for (int q = 0; q < LD_PER_THREAD; ++q) {
    const int P = (wave * LD_PER_THREAD + q) * 64 + lane;
    const int row = P / CHUNKS, chp = P % CHUNKS;
    ld_row[q] = row;
    ld_koff[q] = row * krow_bytes + ((chp ^ kswz(row)) << 4);
    ld_voff[q] = row * vrow_bytes + ((chp ^ vswz(row)) << 4);
    ld_kok[q] = !PAD || (chp ^ kswz(row)) < 2 * ksteps_real;
    ld_vok[q] = !PAD || (chp ^ vswz(row)) < 2 * ksteps_real;
  }
  if constexpr (PAD) {
    for (int o = tid * 16; o < 4 * TILE; o += FA_THREADS * 16) lds_write_b128(smem, o, make_uint4(0u, 0u, 0u, 0u));
    __syncthreads();
  }
  // Full tiles use the precomputed per-lane offsets on a uniform tile base; the
  // ragged last tile clamps its rows (rows past the end are masked in the scores
  // and meet P = 0 in the second product).
  auto load_tile = [&](const uint16_t* base, long row_elems, uint32_t row_bytes, const uint32_t (&offs)[LD_PER_THREAD],
                       const bool (&ok)[LD_PER_THREAD], int tile, int lds_stage) {
    const uint16_t* tb = base + (long)tile * FA_BKV * row_elems;
    const bool full = (tile + 1) * FA_BKV <= p.Sk;
#pragma unroll
    for (int q = 0; q < LD_PER_THREAD; ++q) {
      uint32_t o = offs[q];
      if (!full) {
        const int last = p.Sk - 1 - tile * FA_BKV;        // last valid row of this tile
        if (ld_row[q] > last) o -= (uint32_t)(ld_row[q] - last) * row_bytes;
      }
      if (!PAD || ok[q]) load16_to_lds(tb, o, lds0 + lds_stage * TILE + (wave * LD_PER_THREAD + q) * 1024);
    }
  };
  auto load_k = [&](int tile, int stage) { load_tile(Kb, p.ks.row, krow_bytes, ld_koff, ld_kok, tile, stage); };
  auto load_v = [&](int tile, int stage) { load_tile(Vb, p.vs.row, vrow_bytes, ld_voff, ld_vok, tile, 2 + stage); };

  // ---- state -----------------------------------------------------------------
  f32x16 o_acc[QT][DT];
  float m_run[QT], l_run[QT];            // running max of the raw scores; this lane half's sum
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m_run[qt] = FA_NEG;
    l_run[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o_acc[qt][dt][r] = 0.f;
  }
  const float c = p.scale * 1.44269504088896340736f;   // scale * log2(e)
  int klo[QT], khi[QT];                  // visible keys of this lane's query rows
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) key_bounds(qw + 32 * qt + l32, p.Sq, p.Sk, p.causal, p.window, klo[qt], khi[qt]);
  // Exponent argument of a raw score, in base 2: scale * log2(e) * s, or with a
  // soft cap  cap * log2(e) * tanh(scale * s / cap)  (tanh y = 1 - 2 / (e^{2y} + 1)).
  const float cap2 = p.softcap * 1.44269504088896340736f;
  const float incap = (EXT && p.softcap > 0.f) ? 2.0f * 1.44269504088896340736f * p.scale / p.softcap : 0.f;
  // The extended variant (soft cap and / or additive bias) turns the score tiles into
  // exponent arguments in place, before masking; the plain variant keeps the raw
  // scores and folds cs = scale * log2(e) into the exponential's FMA.
  const float cs = EXT ? 1.0f : c;
  const float* bias_row[QT];             // this lane's row of the additive bias, or null
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qi = min(qw + 32 * qt + l32, p.Sq - 1);
    bias_row[qt] = (EXT && p.bias) ? p.bias + ((long)qlin * p.Sq + qi) * p.Sk : nullptr;
  }
  auto capped = [&](float sraw) -> float {
    return cap2 * (1.0f - 2.0f * __builtin_amdgcn_rcpf(fast_exp2(sraw * incap) + 1.0f));
  };

  // ---- per-lane LDS read addresses (stage and tile-row offsets are immediates) ----
  // K operand: row l32 (+32 kt), logical chunk 2 ks + lh.
  uint32_t k_rd[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_rd[ks] = l32 * ROWB + ((((ks << 1) | lh) ^ kswz(l32)) << 4);
  // V operand: transposing read; lane r of a 16-lane block supplies key r/4 of a
  // 4-key patch and columns 4 (r % 4) .. +3 of a 16-column slab.
  const int r16 = lane & 15;
  uint32_t v_rd[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int key = 4 * lh + (r16 >> 2);
    const int col = (dsel * DT + dt) * 32 + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);
    v_rd[dt] = 2 * TILE + key * ROWB + (((col >> 3) ^ vswz(key)) << 4) + (col & 7) * 2;
  }

  // S^T(tile in K stage `stage`) = K . Q^T, k steps [ks0, ks1); one K fragment
  // feeds the wave's QT query tiles.
  auto score_steps = [&](f32x16 (&sn)[QT][FA_KT], int stage, int ks0, int ks1) {
#pragma unroll
    for (int ks = ks0; ks < ks1; ++ks)
#pragma unroll
      for (int kt = 0; kt < FA_KT; ++kt) {
        const uint4 kf = lds_read_b128(smem, k_rd[ks] + stage * TILE + kt * 32 * ROWB);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
          if (ks == 0) {
            f32x16 z;
#pragma unroll
            for (int r = 0; r < 16; ++r) z[r] = 0.f;
            sn[qt][kt] = mfma_32x32x16<T>(kf, qf[qt][ks], z);
          } else {
            sn[qt][kt] = mfma_32x32x16<T>(kf, qf[qt][ks], sn[qt][kt]);
          }
        }
      }
  };
  // exp2 of one 8-key group of a score tile (in place), its sum, packed to P.
  auto exp_group = [&](f32x16& sv, int g, float mc, float& sum) -> uint4 {
#pragma unroll
    for (int r = 8 * g; r < 8 * g + 8; ++r) {
      const float e = fast_exp2(fmaf(sv[r], cs, -mc));
      sv[r] = e;
      sum += e;
    }
    uint4 pf;
    pf.x = pack2<T>(sv[8 * g + 0], sv[8 * g + 1]);
    pf.y = pack2<T>(sv[8 * g + 2], sv[8 * g + 3]);
    pf.z = pack2<T>(sv[8 * g + 4], sv[8 * g + 5]);
    pf.w = pack2<T>(sv[8 * g + 6], sv[8 * g + 7]);
    return pf;
  };

  // One pipeline step for tile t.  The score MFMAs of tile t+1 are issued first and
  // run under the softmax arithmetic of tile t (whose scores `sc` were produced one
  // step earlier); the exponentials are produced in 8-key groups, each group just
  // ahead of the P.V MFMAs that consume it.  K(t+2) and V(t+1) stream into the
  // stages the previous step released.
  auto step = [&](auto has_next_c, auto par_c, f32x16 (&sc)[QT][FA_KT], f32x16 (&sn)[QT][FA_KT], int t) {
    constexpr bool HAS_NEXT = decltype(has_next_c)::value;
    constexpr int PAR = decltype(par_c)::value;        // t & 1
    if (t + 2 < ntiles) load_k(tile_base + t + 2, PAR);
    if (t + 1 < ntiles) load_v(tile_base + t + 1, PAR ^ 1);
    const int kv0 = (tile_base + t) * FA_BKV;
    if constexpr (EXT) {
      const bool cap = p.softcap > 0.f;
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int kt = 0; kt < FA_KT; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float x = cap ? capped(sc[qt][kt][r]) : sc[qt][kt][r] * c;
            if (bias_row[qt]) {
              const int key = kv0 + kt * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
              x += bias_row[qt][key < p.Sk ? key : p.Sk - 1] * 1.44269504088896340736f;
            }
            sc[qt][kt][r] = x;
          }
    }
    // mask (only tiles that cross a bound of one of the wave's rows)
    const bool need_mask = (kv0 + FA_BKV - 1 > whi_first) || (kv0 < wlo_last);
    if (need_mask) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int kt = 0; kt < FA_KT; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kv0 + kt * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (key > khi[qt] || key < klo[qt]) sc[qt][kt][r] = FA_NEG;
          }
    }
    if constexpr (HAS_NEXT) score_steps(sn, PAR ^ 1, 0, KA);
    // row max
    float m_new[QT], mc[QT];
    bool grow = false;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      float mx = max3_raw(sc[qt][0][0], sc[qt][0][1], sc[qt][0][2]);
#pragma unroll
      for (int kt = 0; kt < FA_KT; ++kt)
#pragma unroll
        for (int r = (kt == 0 ? 3 : 0); r < 16; r += 2)
          mx = (r + 1 < 16) ? max3_raw(mx, sc[qt][kt][r], sc[qt][kt][r + 1]) : fmaxf(mx, sc[qt][kt][r]);
      mx = max_with_other_half(mx);
      m_new[qt] = fmaxf(m_run[qt], mx);
      grow = grow || (m_new[qt] > m_run[qt]);
    }
    // Rescale the accumulators only when some row of the wave raised its maximum.
    if (__any(grow)) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        const float corr = fast_exp2((m_run[qt] - m_new[qt]) * cs);
        l_run[qt] *= corr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            if constexpr (QT > 1) o_acc[qt][dt][r] = scale_acc(o_acc[qt][dt][r], corr);
            else o_acc[qt][dt][r] *= corr;
          }
        m_run[qt] = m_new[qt];
      }
      if constexpr (QT > 1) asm volatile("s_nop 4");   // accumulator writes settle before the next MFMA
    }
#pragma unroll
    // (a row that has met no visible key yet keeps the sentinel maximum: give it the
    // reference 0 so its masked entries underflow to P = 0 instead of cancelling)
    for (int qt = 0; qt < QT; ++qt) mc[qt] = m_new[qt] > 0.5f * FA_NEG ? m_new[qt] * cs : 0.f;

    // Units of 8 keys x one query tile, in consumption order: i -> (kt, g, qt).
    constexpr int NU = 2 * FA_KT * QT;
    constexpr int AHEAD = 3 < NU ? 3 : NU;             // units exponentiated ahead of their P.V step
    uint4 pf[NU];
    float sum[QT][2];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) sum[qt][0] = sum[qt][1] = 0.f;
    auto unit = [&](int i) {
      const int qt = i % QT, g = (i / QT) & 1, kt = i / (2 * QT);
      pf[i] = exp_group(sc[qt][kt], g, mc[qt], sum[qt][g]);
    };
    if constexpr (HAS_NEXT) score_steps(sn, PAR ^ 1, KA, KB);
    unit(0);
    if (AHEAD > 1) unit(1);
    if constexpr (HAS_NEXT) score_steps(sn, PAR ^ 1, KB, KSTEPS);
    if (AHEAD > 2) unit(2);
    // O^T += V^T . P^T; the 16-key step (kt, g) covers keys
    // 32 kt + 16 g + {4h + 0..3, 8 + 4h + 0..3} and feeds all QT query tiles.
#pragma unroll
    for (int sgi = 0; sgi < 2 * FA_KT; ++sgi) {
      const int kt = sgi >> 1, g = sgi & 1;
      uint4 vf[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const uint32_t a = v_rd[dt] + PAR * TILE + (kt * 32 + g * 16) * ROWB;
        const uint2 lo = lds_read_tr16_b64(smem + a);
        const uint2 hi = lds_read_tr16_b64(smem + a + 8 * ROWB);
        vf[dt] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        const int i = sgi * QT + qt;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] = mfma_32x32x16<T>(vf[dt], pf[i], o_acc[qt][dt]);
        if (i + AHEAD < NU) unit(i + AHEAD);
      }
    }
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) l_run[qt] += sum[qt][0] + sum[qt][1];
    fa_wait_loads();
    __syncthreads();
  };
  using std::true_type;
  using std::false_type;
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;

  // ---- prologue: K(0), V(0), K(1) resident; scores of tile 0 ----------------------
  if (ntiles > 0) {
    load_k(tile_base, 0);
    load_v(tile_base, 0);
  }
  if (ntiles > 1) load_k(tile_base + 1, 1);
  fa_wait_loads();
  __syncthreads();
  f32x16 sA[QT][FA_KT], sB[QT][FA_KT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt)
#pragma unroll
    for (int kt = 0; kt < FA_KT; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) { sA[qt][kt][r] = 0.f; sB[qt][kt][r] = 0.f; }
  // Tiles before the wave's first key (a sliding window): keep the loads going.
  auto idle_step = [&](int t) {
    if (t + 2 < ntiles) load_k(tile_base + t + 2, t & 1);
    if (t + 1 < ntiles) load_v(tile_base + t + 1, (t & 1) ^ 1);
    fa_wait_loads();
    __syncthreads();
  };
  // A wave that starts late computes the scores of its first tile (t_w0, even, so its
  // K tile sits in stage 0) inside the idle step before it: from step t_w0 on the
  // other waves already refill that stage.
  int t = 0;
  if (t_w0 == 0 && nt_w > 0) score_steps(sA, 0, 0, KSTEPS);
  // Step 0 refills K stage 0: every wave must have read tile 0's keys first (a wave
  // that starts late issues those loads without any arithmetic ahead of them).
  __syncthreads();
  for (; t < t_w0; ++t) {
    if (t + 2 < ntiles) load_k(tile_base + t + 2, t & 1);
    if (t + 1 < ntiles) load_v(tile_base + t + 1, (t & 1) ^ 1);
    if (t + 1 == t_w0 && nt_w > t_w0) score_steps(sA, 0, 0, KSTEPS);
    fa_wait_loads();
    __syncthreads();
  }

  for (; t + 2 < nt_w; t += 2) {
    step(true_type{}, P0{}, sA, sB, t);
    step(true_type{}, P1{}, sB, sA, t + 1);
  }
  if (t + 2 == nt_w) {
    step(true_type{}, P0{}, sA, sB, t);
    step(false_type{}, P1{}, sB, sA, t + 1);
    t += 2;
  } else if (t + 1 == nt_w) {
    step(false_type{}, P0{}, sA, sB, t);
    t += 1;
  }
  // Waves past their diagonal keep feeding the loads the others depend on.
  for (; t < ntiles; ++t) idle_step(t);

  // ---- epilogue -------------------------------------------------------------------
  // A lane owns 4-column pieces of ONE output row: stored from the registers, a wave
  // instruction would touch 32 rows with 16 or 32 bytes each.  Every wave therefore passes its
  // 32 x D tile through its own slice of the (now idle) LDS and writes whole rows, 16 bytes per
  // lane with consecutive lanes along a row.  The last loop barrier has passed, so no wave
  // reads K or V any more.
  const int dreal = PAD ? p.D : D;
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qi = qw + 32 * qt + l32;
    float l = l_run[qt] + swap_half(l_run[qt]);
    if (khi[qt] < klo[qt]) l = 0.f;                      // no visible key: O = 0, LSE = -inf
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const long row = (long)qlin * p.Sq + qi + (long)split * p.B * p.Hq * p.Sq;
    if (p.LSE && lh == 0 && dsel == 0 && qi < p.Sq)
      p.LSE[row] = l > 0.f ? (m_run[qt] * cs + __log2f(l)) * 0.69314718055994530942f : -INFINITY;
    char* stage = smem + (wave * QT + qt) * 32 * G::STAGE_PITCH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d = dt * 32 + 8 * a + 4 * lh;
        const float v0 = o_acc[qt][dt][4 * a + 0] * inv, v1 = o_acc[qt][dt][4 * a + 1] * inv;
        const float v2 = o_acc[qt][dt][4 * a + 2] * inv, v3 = o_acc[qt][dt][4 * a + 3] * inv;
        if (p.out_storage) {
          uint2 pk;
          pk.x = pack2<T>(v0, v1);
          pk.y = pack2<T>(v2, v3);
          *reinterpret_cast<uint2*>(stage + l32 * G::STAGE_PITCH + d * 2) = pk;
        } else {
          *reinterpret_cast<float4*>(stage + l32 * G::STAGE_PITCH + d * 4) = make_float4(v0, v1, v2, v3);
        }
      }
    // rows of this wave's share of the dreal columns, 16 bytes per lane
    const int esz = p.out_storage ? 2 : 4;
    const int dcol0 = dsel * DT * 32;                      // first output column of this wave
    const int dcols = min(dreal - dcol0, DT * 32);
    const int per_row = dcols > 0 ? dcols * esz / 16 : 0;  // 16-byte pieces per output row
    const int rows_here = min(32, p.Sq - (qw + 32 * qt));
    char* Ob = reinterpret_cast<char*>(p.O) + (batch * p.os.batch + hq * p.os.head + split * p.split_o_elems) * esz;
    for (int idx = lane; idx < rows_here * per_row; idx += 64) {
      const int r = idx / per_row, c = idx - r * per_row;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + r * G::STAGE_PITCH + c * 16);
      *reinterpret_cast<uint4*>(Ob + ((long)(qw + 32 * qt + r) * p.os.row + dcol0) * esz + c * 16) = v;
    }
  }
}

// Any head dimension and any alignment: one thread per query row, streaming online softmax
// in f32.  Serves only operands the MFMA kernel cannot address (pointers or strides that are
// not multiples of 16 bytes).
template <class T>
__global__ void flash_fwd_generic_kernel(const FlashParams p) {
  const int D = p.D;
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long total = (long)p.B * p.Hq * p.Sq;
  if (row >= total) return;
  const int qi = (int)(row % p.Sq);
  const int hq = (int)((row / p.Sq) % p.Hq);
  const int b = (int)(row / ((long)p.Sq * p.Hq));
  const int hkv = (int)(((long)hq * p.Hkv) / p.Hq);
  const uint16_t* q = p.Q + b * p.qs.batch + hq * p.qs.head + qi * p.qs.row;
  const uint16_t* Kb = p.K + b * p.ks.batch + hkv * p.ks.head;
  const uint16_t* Vb = p.V + b * p.vs.batch + hkv * p.vs.head;
  float acc[256];
  for (int d = 0; d < D; ++d) acc[d] = 0.f;
  float m = -INFINITY, l = 0.f;
  int jmin, jmax;
  key_bounds(qi, p.Sq, p.Sk, p.causal, p.window, jmin, jmax);
  for (int j = jmin; j <= jmax; ++j) {
    float s = 0.f;
    for (int d = 0; d < D; ++d) s += from_storage<T>(q[d]) * from_storage<T>(Kb[(long)j * p.ks.row + d]);
    s *= p.scale;
    if (p.softcap > 0.f) s = p.softcap * tanhf(s / p.softcap);
    if (p.bias) s += p.bias[row * p.Sk + j];
    const float mn = fmaxf(m, s);
    const float cr = __expf(m - mn);       // exp(-inf) = 0 on the first key
    const float e = __expf(s - mn);
    l = l * cr + e;
    for (int d = 0; d < D; ++d) acc[d] = acc[d] * cr + e * from_storage<T>(Vb[(long)j * p.vs.row + d]);
    m = mn;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  if (p.LSE) p.LSE[row] = l > 0.f ? m + __logf(l) : -INFINITY;
  const long o_at = b * p.os.batch + hq * p.os.head + qi * p.os.row;
  for (int d = 0; d < D; ++d) {
    const float v = acc[d] * inv;
    if (p.out_storage) reinterpret_cast<uint16_t*>(p.O)[o_at + d] = to_storage<T>(v);
    else reinterpret_cast<float*>(p.O)[o_at + d] = v;
  }
}

}  // namespace tsr950
