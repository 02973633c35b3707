// Flash-attention backward for gfx950: (dQ, dK, dV) of O = softmax(scale Q K^T, causal) V
// from dO, Q, K, V and the forward's O and log-sum-exp; GQA, 16-bit storage, f32
// accumulate, f32 gradients.
//
// Three kernels, no atomics, results independent of scheduling:
//   flash_bwd_delta_kernel   Delta[q] = sum_d dO[q][d] O[q][d]
//   flash_bwd_dq_kernel      one workgroup per 256 query rows, walks the key tiles
//   flash_bwd_dkdv_kernel    one workgroup per 128 keys of one KV head, walks the
//                            query tiles of every query head that shares the KV head
// Both walkers recompute P = exp(scale S - LSE) and dS = P (dP - Delta) tile by tile.
// As in the forward kernel the products are oriented so that the index a lane owns
// (its query row in the dQ kernel, its key in the dK/dV kernel) is the one the
// second product does NOT contract over, so P and dS go from accumulator registers
// straight into the next MFMA as its B operand:
//   dQ kernel    S^T = K Q^T, dP^T = V dO^T        (lane: one query, 16 keys / tile)
//                dQ^T += K^T dS^T                   (K^T by transposing LDS read)
//   dK/dV kernel S = Q K^T, dP = dO V^T             (lane: one key, 16 queries / tile)
//                dV^T += dO^T P,  dK^T += Q^T dS    (dO^T, Q^T by transposing LDS read)
// Every LDS tile keeps the natural [row][D] layout and is read both by rows
// (ds_read_b128) and transposed (ds_read_b64_tr_b16); one chunk swizzle serves both.
#pragma once
#include "flash_attn.h"

namespace tsr950 {

struct FlashBwdParams {
  const uint16_t* Q;    // [B, Hq, Sq, D]
  const uint16_t* K;    // [B, Hkv, Sk, D]
  const uint16_t* V;    // [B, Hkv, Sk, D]
  const uint16_t* dO;   // [B, Hq, Sq, D]
  const float* O;       // [B, Hq, Sq, D]  forward output
  const float* LSE;     // [B, Hq, Sq]     forward log-sum-exp (natural log, of scaled scores)
  float* Delta;         // [B, Hq, Sq]     workspace: Delta, or -Delta for the MFMA kernels
  float* LSE2;          // [B, Hq, Sq]     workspace of the MFMA kernels: -LSE / scale
  float* dQ;            // [B, Hq, Sq, D]
  float* dK;            // [B, Hkv, Sk, D]
  float* dV;            // [B, Hkv, Sk, D]
  int B, Hq, Hkv, Sq, Sk;
  float scale;
  int causal;
};

constexpr float kLog2e = 1.44269504088896340736f;

// 4 bytes per lane from global memory straight into LDS: lane i lands at lds_base + 4 i.
__device__ __forceinline__ void load4_to_lds(const void* base, uint32_t byte_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :: "s"(lds_base), "v"(byte_off), "s"(base) : "memory");
}

// Chunk swizzle of a [row][D] tile of 16-byte chunks that is conflict-free both for
// row reads (16 consecutive rows, one chunk column) and for transposing reads
// (4 consecutive rows x two adjacent chunks): a bit permutation of the row index
// that is a bijection over the rows sharing a 256-byte bank line and moves the
// row's low bits away from bit 0 of the chunk index.
template <int D>
__device__ __forceinline__ int bwd_swz(int row) {
  if constexpr (D == 128) return ((row & 3) << 2) | ((row >> 2) & 3);
  const int t = (row >> 1) & 7;
  return ((t & 1) << 2) | (t >> 1);
}

// Delta[row] = delta_mul * sum_d dO[row][d] * O[row][d] and LSE2[row] = lse_mul * LSE[row];
// 16 lanes per row, 8 columns per lane per pass.  The MFMA kernels take both negated,
// the log-sum-exp also divided by the softmax scale (multipliers -1 and -1 / scale):
// they start the S and dP accumulators from these values, so that the products come
// out as S - LSE / scale and dP - Delta with no further arithmetic per element.
template <class T>
__global__ void flash_bwd_delta_kernel(const uint16_t* __restrict__ dO, const float* __restrict__ O,
                                       const float* __restrict__ LSE, float* __restrict__ Delta,
                                       float* __restrict__ LSE2, long rows, int D, float delta_mul,
                                       float lse_mul) {
  const long row = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
  const int part = threadIdx.x & 15;
  float acc = 0.f;
  if (row < rows) {
    for (int d = part * 8; d < D; d += 128) {
      const uint4 g = *reinterpret_cast<const uint4*>(dO + row * D + d);
      const float4 o0 = *reinterpret_cast<const float4*>(O + row * D + d);
      const float4 o1 = *reinterpret_cast<const float4*>(O + row * D + d + 4);
      const uint32_t w[4] = {g.x, g.y, g.z, g.w};
      const float ov[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc += from_storage<T>((uint16_t)(w[e] & 0xffff)) * ov[2 * e];
        acc += from_storage<T>((uint16_t)(w[e] >> 16)) * ov[2 * e + 1];
      }
    }
  }
#pragma unroll
  for (int s = 8; s >= 1; s >>= 1) acc += __shfl_xor(acc, s, 64);
  if (row < rows && part == 0) {
    Delta[row] = acc * delta_mul;
    LSE2[row] = LSE[row] * lse_mul;
  }
}

// ---------------------------------------------------------------------------------
// dQ: 8 waves x 32 query rows; K/V tiles of 64 keys stream global -> LDS.
// ---------------------------------------------------------------------------------
constexpr int FB_BQ = 256, FB_BKV = 64, FB_DQ_THREADS = 512;

template <class T, int D>
__global__ __launch_bounds__(FB_DQ_THREADS, 1) void flash_bwd_dq_kernel(const FlashBwdParams p) {
  constexpr int KSTEPS = D / 16, DT = D / 32, ROWB = D * 2, CHUNKS = D / 8;
  constexpr int TILE = FB_BKV * ROWB;
  constexpr int LD_PER_THREAD = FB_BKV * CHUNKS / FB_DQ_THREADS;
  static_assert(FB_BKV * CHUNKS % FB_DQ_THREADS == 0, "tile/thread mismatch");
  extern __shared__ __attribute__((aligned(16))) char smem[];   // K stages 0,1 | V stages 2,3
  const uint32_t lds0 = (uint32_t)(uintptr_t)(TSR_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5, r16 = lane & 15;

  const int qblocks = (p.Sq + FB_BQ - 1) / FB_BQ;
  const int qb = qblocks - 1 - blockIdx.x / (p.B * p.Hq);      // heavy causal blocks first
  const int bh = blockIdx.x % (p.B * p.Hq);
  const int b = bh / p.Hq, hq = bh % p.Hq;
  const int hkv = (int)(((long)hq * p.Hkv) / p.Hq);
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;
  const int q0 = qb * FB_BQ, qw = q0 + wave * 32;
  const long qrow0 = (long)(b * p.Hq + hq) * p.Sq;
  const uint16_t* Kb = p.K + ((long)(b * p.Hkv + hkv) * p.Sk) * D;
  const uint16_t* Vb = p.V + ((long)(b * p.Hkv + hkv) * p.Sk) * D;

  int kv_end = p.Sk;
  if (p.causal) kv_end = min(p.Sk, min(q0 + FB_BQ, p.Sq) - 1 + off + 1);
  const int ntiles = (kv_end + FB_BKV - 1) / FB_BKV;
  int nt_w = 0;
  if (qw < p.Sq) {
    int e = kv_end;
    if (p.causal) e = min(kv_end, min(qw + 32, p.Sq) - 1 + off + 1);
    nt_w = (e + FB_BKV - 1) / FB_BKV;
  }

  // resident operands of this lane's query row
  const int qi = qw + l32;
  const int qrow = qi < p.Sq ? qi : p.Sq - 1;
  uint4 qf[KSTEPS], dof[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    qf[ks] = *reinterpret_cast<const uint4*>(p.Q + (qrow0 + qrow) * D + 16 * ks + 8 * lh);
    dof[ks] = *reinterpret_cast<const uint4*>(p.dO + (qrow0 + qrow) * D + 16 * ks + 8 * lh);
  }
  const float c = p.scale * kLog2e;
  const float neg_lse = p.LSE2[qrow0 + qrow];             // -LSE / scale
  const float neg_delta = p.Delta[qrow0 + qrow];          // -Delta
  const int lim = qi >= p.Sq ? -1 : (p.causal ? min(qi + off, p.Sk - 1) : p.Sk - 1);

  // tile loaders (global -> LDS, swizzle applied on the global address)
  int ld_row[LD_PER_THREAD];
  uint32_t ld_off[LD_PER_THREAD];
#pragma unroll
  for (int q = 0; q < LD_PER_THREAD; ++q) {
    const int P = (wave * LD_PER_THREAD + q) * 64 + lane;
    const int row = P / CHUNKS, chp = P % CHUNKS;
    ld_row[q] = row;
    ld_off[q] = row * ROWB + ((chp ^ bwd_swz<D>(row)) << 4);
  }
  auto load_tile = [&](const uint16_t* base, int tile, int lds_stage) {
    const uint16_t* tb = base + (long)tile * FB_BKV * D;
    const bool full = (tile + 1) * FB_BKV <= p.Sk;
#pragma unroll
    for (int q = 0; q < LD_PER_THREAD; ++q) {
      uint32_t o = ld_off[q];
      if (!full) {
        const int last = p.Sk - 1 - tile * FB_BKV;
        if (ld_row[q] > last) o -= (uint32_t)(ld_row[q] - last) * ROWB;
      }
      load16_to_lds(tb, o, lds0 + lds_stage * TILE + (wave * LD_PER_THREAD + q) * 1024);
    }
  };

  // read addresses: rows (b128) and transposed (tr16) forms of a tile
  uint32_t row_rd[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) row_rd[ks] = l32 * ROWB + ((((ks << 1) | lh) ^ bwd_swz<D>(l32)) << 4);
  uint32_t tr_lo[DT], tr_hi[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int key = 4 * lh + (r16 >> 2);
    const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);
    tr_lo[dt] = key * ROWB + (((col >> 3) ^ bwd_swz<D>(key)) << 4) + (col & 7) * 2;
    tr_hi[dt] = (key + 8) * ROWB + (((col >> 3) ^ bwd_swz<D>(key + 8)) << 4) + (col & 7) * 2;
  }

  f32x16 dq[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[dt][r] = 0.f;

  if (ntiles > 0) {
    load_tile(Kb, 0, 0);
    load_tile(Vb, 0, 2);
  }
  fa_wait_loads();
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const int st = t & 1;
    if (t + 1 < ntiles) {
      load_tile(Kb, t + 1, st ^ 1);
      load_tile(Vb, t + 1, 2 + (st ^ 1));
    }
    if (t < nt_w) {
      const int kv0 = t * FB_BKV;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) { s[r] = neg_lse; dp[r] = neg_delta; }   // S - LSE / scale, dP - Delta
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const uint4 kf = lds_read_b128(smem, row_rd[ks] + st * TILE + kt * 32 * ROWB);
          const uint4 vf = lds_read_b128(smem, row_rd[ks] + (2 + st) * TILE + kt * 32 * ROWB);
          s = mfma_32x32x16<T>(kf, qf[ks], s);
          dp = mfma_32x32x16<T>(vf, dof[ks], dp);
        }
        // lane: query qi, keys kv0 + 32 kt + 8 (r/4) + 4 lh + r % 4.  Only tiles that
        // touch the causal diagonal or the end of Q / K pay for the per-key mask.
        uint4 dsf[2];
        auto ds_part = [&](auto masked_c) {
          constexpr bool MASKED = decltype(masked_c)::value;
          uint32_t w[8];
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            float ds2[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const int rr = r + e;
              float x = s[rr] * c;
              if constexpr (MASKED) {
                const int key = kv0 + kt * 32 + 8 * (rr >> 2) + 4 * lh + (rr & 3);
                x = key <= lim ? x : -INFINITY;          // exponent -inf: P = 0, no branch
              }
              ds2[e] = fast_exp2(x) * dp[rr];
            }
            w[r >> 1] = pack2<T>(ds2[0], ds2[1]);
          }
          dsf[0] = make_uint4(w[0], w[1], w[2], w[3]);
          dsf[1] = make_uint4(w[4], w[5], w[6], w[7]);
        };
        const bool need_mask = (kv0 + kt * 32 + 32 > p.Sk) || (qw + 32 > p.Sq) ||
                               (p.causal && kv0 + kt * 32 + 31 > qw + off);
        if (need_mask) ds_part(std::true_type{});
        else ds_part(std::false_type{});
        // dQ^T += K^T dS^T over the 16-key steps (kt, g)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const uint32_t o = st * TILE + (kt * 32 + g * 16) * ROWB;
            const uint2 lo = lds_read_tr16_b64(smem + tr_lo[dt] + o);
            const uint2 hi = lds_read_tr16_b64(smem + tr_hi[dt] + o);
            dq[dt] = mfma_32x32x16<T>(make_uint4(lo.x, lo.y, hi.x, hi.y), dsf[g], dq[dt]);
          }
      }
    }
    fa_wait_loads();
    __syncthreads();
  }
  if (qi >= p.Sq) return;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int d = dt * 32 + 8 * a + 4 * lh;
      *reinterpret_cast<float4*>(p.dQ + (qrow0 + qi) * D + d) =
          make_float4(dq[dt][4 * a] * p.scale, dq[dt][4 * a + 1] * p.scale, dq[dt][4 * a + 2] * p.scale,
                      dq[dt][4 * a + 3] * p.scale);
    }
}

// ---------------------------------------------------------------------------------
// dK, dV: 4 waves x 32 keys; Q / dO tiles of 64 query rows (plus their LSE and Delta)
// are staged through LDS for every query head of the KV head's group.
// ---------------------------------------------------------------------------------
constexpr int FB_BK = 128, FB_BQT = 64, FB_DKV_THREADS = 256;

template <class T, int D>
__global__ __launch_bounds__(FB_DKV_THREADS, 1) void flash_bwd_dkdv_kernel(const FlashBwdParams p) {
  constexpr int KSTEPS = D / 16, DT = D / 32, ROWB = D * 2, CHUNKS = D / 8;
  constexpr int TILE = FB_BQT * ROWB;                      // bytes of a Q (or dO) tile
  constexpr int STAGE = 2 * TILE + 2 * FB_BQT * 4;         // Q | dO | -LSE/scale [64] | -Delta [64]
  constexpr int LD_PER_WAVE = FB_BQT * CHUNKS / 64 / (FB_DKV_THREADS / 64);
  static_assert(FB_BQT * CHUNKS % FB_DKV_THREADS == 0, "tile/thread mismatch");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(TSR_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5, r16 = lane & 15;

  // heavy key blocks (seen by the most query rows under a causal mask) first
  const int kblocks = (p.Sk + FB_BK - 1) / FB_BK;
  const int kb = blockIdx.x / (p.B * p.Hkv);
  const int bh = blockIdx.x % (p.B * p.Hkv);
  const int b = bh / p.Hkv, hkv = bh % p.Hkv;
  const int ratio = p.Hq / p.Hkv;
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;
  const int k0 = kb * FB_BK;
  const int key = k0 + wave * 32 + l32;                    // this lane's key
  const int krow = key < p.Sk ? key : p.Sk - 1;
  const long kvrow0 = (long)(b * p.Hkv + hkv) * p.Sk;
  (void)kblocks;

  uint4 kf[KSTEPS], vf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    kf[ks] = *reinterpret_cast<const uint4*>(p.K + (kvrow0 + krow) * D + 16 * ks + 8 * lh);
    vf[ks] = *reinterpret_cast<const uint4*>(p.V + (kvrow0 + krow) * D + 16 * ks + 8 * lh);
  }
  const float c = p.scale * kLog2e;

  // first query row that can see this workgroup's keys
  int q_first = 0;
  if (p.causal) q_first = max(0, k0 - off);
  const int t_first = q_first / FB_BQT;
  const int qtiles = (p.Sq + FB_BQT - 1) / FB_BQT;
  const int steps_per_head = max(qtiles - t_first, 0);
  const int nsteps = steps_per_head * ratio;

  // loaders: global -> LDS, one wave instruction = 64 consecutive 16-byte slots
  int ld_row[LD_PER_WAVE];
  uint32_t ld_off[LD_PER_WAVE];
#pragma unroll
  for (int q = 0; q < LD_PER_WAVE; ++q) {
    const int P = (wave * LD_PER_WAVE + q) * 64 + lane;
    const int row = P / CHUNKS, chp = P % CHUNKS;
    ld_row[q] = row;
    ld_off[q] = row * ROWB + ((chp ^ bwd_swz<D>(row)) << 4);
  }
  // Tile of step s: query head hkv * ratio + s / steps_per_head, query tile t_first +
  // s % steps_per_head.  The loop keeps both as counters (no division per step).
  // The loads of a step are issued in two halves (`part`): a burst of 17 per wave
  // sits in the issue queue for over a thousand cycles.
  auto load_part = [&](int head, int tile, int stage, int part) {
    const int qt0 = tile * FB_BQT;
    const long qrow0 = (long)(b * p.Hq + hkv * ratio + head) * p.Sq;
    const uint16_t* qb = p.Q + (qrow0 + qt0) * D;
    const uint16_t* gb = p.dO + (qrow0 + qt0) * D;
    const int last = p.Sq - 1 - qt0;                       // last valid row of this tile
    const uint32_t sbase = lds0 + stage * STAGE;
    constexpr int HALF = LD_PER_WAVE / 2;
    if (last >= FB_BQT - 1) {                              // full tile (uniform): no row clamp
#pragma unroll
      for (int q = part * HALF; q < (part + 1) * HALF; ++q) {
        load16_to_lds(qb, ld_off[q], sbase + (wave * LD_PER_WAVE + q) * 1024);
        load16_to_lds(gb, ld_off[q], sbase + TILE + (wave * LD_PER_WAVE + q) * 1024);
      }
    } else {
#pragma unroll
      for (int q = part * HALF; q < (part + 1) * HALF; ++q) {
        uint32_t o = ld_off[q];
        if (ld_row[q] > last) o -= (uint32_t)(ld_row[q] - last) * ROWB;   // rows past the end: masked later
        load16_to_lds(qb, o, sbase + (wave * LD_PER_WAVE + q) * 1024);
        load16_to_lds(gb, o, sbase + TILE + (wave * LD_PER_WAVE + q) * 1024);
      }
    }
    if (part == 1 && wave < 2) {
      const float* src = (wave == 0 ? p.LSE2 : p.Delta) + qrow0 + qt0;
      const int r = lane <= last ? lane : last;
      load4_to_lds(src, (uint32_t)r * 4, sbase + 2 * TILE + wave * FB_BQT * 4);
    }
  };
  static_assert(LD_PER_WAVE % 2 == 0, "loads are issued in two halves");

  uint32_t row_rd[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) row_rd[ks] = l32 * ROWB + ((((ks << 1) | lh) ^ bwd_swz<D>(l32)) << 4);
  uint32_t tr_lo[DT], tr_hi[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int qq = 4 * lh + (r16 >> 2);
    const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);
    tr_lo[dt] = qq * ROWB + (((col >> 3) ^ bwd_swz<D>(qq)) << 4) + (col & 7) * 2;
    tr_hi[dt] = (qq + 8) * ROWB + (((col >> 3) ^ bwd_swz<D>(qq + 8)) << 4) + (col & 7) * 2;
  }

  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk[dt][r] = 0.f; dv[dt][r] = 0.f; }

  if (nsteps > 0) {
    load_part(0, t_first, 0, 0);
    load_part(0, t_first, 0, 1);
  }
  fa_wait_loads();
  __syncthreads();
  const int wave_k0 = k0 + wave * 32;
  int cur_head = 0, cur_tile = t_first;                    // (head, tile) of this step
  for (int step = 0; step < nsteps; ++step) {
    const int st = step & 1;
    int nxt_head = cur_head, nxt_tile = cur_tile + 1;      // ... and of the next
    if (nxt_tile == qtiles) { nxt_tile = t_first; ++nxt_head; }
    const bool has_next = step + 1 < nsteps;
    if (has_next) load_part(nxt_head, nxt_tile, st ^ 1, 0);
    const char* base = smem + st * STAGE;
    const int qt0 = cur_tile * FB_BQT;
    // do this wave's keys see the tile at all?  (uniform per wave)
    const bool live = wave_k0 < p.Sk && (!p.causal || wave_k0 <= min(qt0 + FB_BQT, p.Sq) - 1 + off);
    if (live) {
      // The step runs as a pipeline over the two 32-row halves of the query tile, so
      // that the softmax arithmetic (VALU) of one half rides in the shadow of the other
      // half's MFMAs — one wave per SIMD has nobody else to overlap with:
      //   first products (S = Q K^T, dP = dO V^T) of half 0
      //   first products of half 1          | softmax of half 0
      //   second products (dV, dK) of half 0 | softmax of half 1
      //   second products of half 1
      // Operand fragments are read one MFMA pair ahead of their use.
      f32x16 s[2], dp[2];
      uint32_t pw[2][8], dw[2][8];                         // packed P and dS per half
      // one eighth of a half's softmax: elements 4 a + 2 h2 + {0, 1} of the lane's 16
      auto softmax_piece = [&](int qt, int piece, auto masked_c) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_c)::value;
        const int a = piece >> 1, h2 = piece & 1;
        const int qoff = 32 * qt + 8 * a + 4 * lh + 2 * h2;
        float pr[2], ds[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int r = 4 * a + 2 * h2 + e;
          float x = s[qt][r] * c;
          if constexpr (MASKED) {
            const int q = qt0 + qoff + e;
            const bool ok = (q < p.Sq) & (key < p.Sk) & (!p.causal | (key <= q + off));
            x = ok ? x : -INFINITY;                        // exponent -inf: P = 0, no branch
          }
          pr[e] = fast_exp2(x);
          ds[e] = pr[e] * dp[qt][r];
        }
        pw[qt][2 * a + h2] = pack2<T>(pr[0], pr[1]);
        dw[qt][2 * a + h2] = pack2<T>(ds[0], ds[1]);
      };
      // S - LSE / scale and dP - Delta of one half: the accumulators start from the
      // staged -LSE / scale and -Delta of their rows (lane's rows 8 a + 4 lh + 0..3),
      // then 8 k steps of two MFMAs; `between(ks)` follows each pair
      auto first_products = [&](int qt, auto&& between) __attribute__((always_inline)) {
        f32x16 s0, dp0;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int qoff = 32 * qt + 8 * a + 4 * lh;
          const float4 l4 = *reinterpret_cast<const float4*>(base + 2 * TILE + qoff * 4);
          const float4 d4 = *reinterpret_cast<const float4*>(base + 2 * TILE + FB_BQT * 4 + qoff * 4);
          s0[4 * a] = l4.x; s0[4 * a + 1] = l4.y; s0[4 * a + 2] = l4.z; s0[4 * a + 3] = l4.w;
          dp0[4 * a] = d4.x; dp0[4 * a + 1] = d4.y; dp0[4 * a + 2] = d4.z; dp0[4 * a + 3] = d4.w;
        }
        uint4 qfr[2], dofr[2];
        qfr[0] = lds_read_b128(base, row_rd[0] + qt * 32 * ROWB);
        dofr[0] = lds_read_b128(base, TILE + row_rd[0] + qt * 32 * ROWB);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int cur = ks & 1;
          if (ks + 1 < KSTEPS) {
            qfr[cur ^ 1] = lds_read_b128(base, row_rd[ks + 1] + qt * 32 * ROWB);
            dofr[cur ^ 1] = lds_read_b128(base, TILE + row_rd[ks + 1] + qt * 32 * ROWB);
          }
          if (ks == 0) {
            s[qt] = mfma_32x32x16<T>(qfr[cur], kf[ks], s0);
            dp[qt] = mfma_32x32x16<T>(dofr[cur], vf[ks], dp0);
          } else {
            s[qt] = mfma_32x32x16<T>(qfr[cur], kf[ks], s[qt]);
            dp[qt] = mfma_32x32x16<T>(dofr[cur], vf[ks], dp[qt]);
          }
          between(ks);
        }
      };
      // dV += dO^T P and dK += Q^T dS of one half: (g, dt) steps of two MFMAs
      auto second_products = [&](int qt, auto&& between) __attribute__((always_inline)) {
        const uint4 pf[2] = {make_uint4(pw[qt][0], pw[qt][1], pw[qt][2], pw[qt][3]),
                             make_uint4(pw[qt][4], pw[qt][5], pw[qt][6], pw[qt][7])};
        const uint4 dsf[2] = {make_uint4(dw[qt][0], dw[qt][1], dw[qt][2], dw[qt][3]),
                              make_uint4(dw[qt][4], dw[qt][5], dw[qt][6], dw[qt][7])};
        auto tr_frags = [&](int i, uint4& qT, uint4& oT) {
          const int dt = i % DT, g = i / DT;
          const uint32_t o = (qt * 32 + g * 16) * ROWB;
          const uint2 qlo = lds_read_tr16_b64(base + tr_lo[dt] + o);
          const uint2 qhi = lds_read_tr16_b64(base + tr_hi[dt] + o);
          const uint2 olo = lds_read_tr16_b64(base + TILE + tr_lo[dt] + o);
          const uint2 ohi = lds_read_tr16_b64(base + TILE + tr_hi[dt] + o);
          qT = make_uint4(qlo.x, qlo.y, qhi.x, qhi.y);
          oT = make_uint4(olo.x, olo.y, ohi.x, ohi.y);
        };
        constexpr int NSTEP = 2 * DT;
        uint4 qT[2], oT[2];
        tr_frags(0, qT[0], oT[0]);
#pragma unroll
        for (int i = 0; i < NSTEP; ++i) {
          const int cur = i & 1;
          if (i + 1 < NSTEP) tr_frags(i + 1, qT[cur ^ 1], oT[cur ^ 1]);
          const int dt = i % DT, g = i / DT;
          dv[dt] = mfma_32x32x16<T>(oT[cur], pf[g], dv[dt]);
          dk[dt] = mfma_32x32x16<T>(qT[cur], dsf[g], dk[dt]);
          between(i);
        }
      };
      static_assert(KSTEPS == 8 || KSTEPS == 4, "softmax pieces are spread over the k steps");
      auto none = [](int) {};
      // lane: key, queries qt0 + 32 qt + 8 (r/4) + 4 lh + r % 4.  Only tiles that touch
      // the causal diagonal or the end of Q / K pay for the per-pair mask.
      const bool need_mask = (qt0 + FB_BQT > p.Sq) || (wave_k0 + 32 > p.Sk) ||
                             (p.causal && wave_k0 + 31 > qt0 + off);
      auto run = [&](auto masked_c) __attribute__((always_inline)) {
        // 8 softmax pieces per half over KSTEPS (first products) or 2 DT (second) slots
        constexpr int PER1 = 8 / KSTEPS, PER2 = 8 / (2 * DT);
        first_products(0, none);
        if (has_next) load_part(nxt_head, nxt_tile, st ^ 1, 1);
        first_products(1, [&](int ks) {
#pragma unroll
          for (int u = 0; u < PER1; ++u) softmax_piece(0, ks * PER1 + u, masked_c);
        });
        second_products(0, [&](int i) {
#pragma unroll
          for (int u = 0; u < PER2; ++u) softmax_piece(1, i * PER2 + u, masked_c);
        });
        second_products(1, none);
      };
      if (need_mask) run(std::true_type{});
      else run(std::false_type{});
    } else if (has_next) {
      load_part(nxt_head, nxt_tile, st ^ 1, 1);
    }
    cur_head = nxt_head;
    cur_tile = nxt_tile;
    fa_wait_loads();
    __syncthreads();
  }
  if (key >= p.Sk) return;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int d = dt * 32 + 8 * a + 4 * lh;
      const long o = (kvrow0 + key) * D + d;
      *reinterpret_cast<float4*>(p.dK + o) = make_float4(dk[dt][4 * a] * p.scale, dk[dt][4 * a + 1] * p.scale,
                                                         dk[dt][4 * a + 2] * p.scale, dk[dt][4 * a + 3] * p.scale);
      *reinterpret_cast<float4*>(p.dV + o) =
          make_float4(dv[dt][4 * a], dv[dt][4 * a + 1], dv[dt][4 * a + 2], dv[dt][4 * a + 3]);
    }
}

// Any head dimension: thread per query row (dQ) and thread per key row (dK, dV),
// f32, recomputing P from the saved LSE.  Serves head dims other than 64 / 128.
template <class T>
__global__ void flash_bwd_generic_dq_kernel(const FlashBwdParams p, int D) {
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= (long)p.B * p.Hq * p.Sq) return;
  const int qi = (int)(row % p.Sq), hq = (int)((row / p.Sq) % p.Hq), b = (int)(row / ((long)p.Sq * p.Hq));
  const int hkv = (int)(((long)hq * p.Hkv) / p.Hq);
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;
  const uint16_t* q = p.Q + row * D;
  const uint16_t* g = p.dO + row * D;
  const uint16_t* Kb = p.K + ((long)(b * p.Hkv + hkv) * p.Sk) * D;
  const uint16_t* Vb = p.V + ((long)(b * p.Hkv + hkv) * p.Sk) * D;
  float acc[256];
  for (int d = 0; d < D; ++d) acc[d] = 0.f;
  const int jmax = p.causal ? min(qi + off, p.Sk - 1) : p.Sk - 1;
  const float lse = p.LSE[row], delta = p.Delta[row];
  for (int j = 0; j <= jmax; ++j) {
    float s = 0.f, dp = 0.f;
    for (int d = 0; d < D; ++d) {
      s += from_storage<T>(q[d]) * from_storage<T>(Kb[(long)j * D + d]);
      dp += from_storage<T>(g[d]) * from_storage<T>(Vb[(long)j * D + d]);
    }
    const float ds = __expf(s * p.scale - lse) * (dp - delta);
    for (int d = 0; d < D; ++d) acc[d] += ds * from_storage<T>(Kb[(long)j * D + d]);
  }
  for (int d = 0; d < D; ++d) p.dQ[row * D + d] = acc[d] * p.scale;
}

template <class T>
__global__ void flash_bwd_generic_dkdv_kernel(const FlashBwdParams p, int D) {
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= (long)p.B * p.Hkv * p.Sk) return;
  const int j = (int)(row % p.Sk), hkv = (int)((row / p.Sk) % p.Hkv), b = (int)(row / ((long)p.Sk * p.Hkv));
  const int ratio = p.Hq / p.Hkv;
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;
  const uint16_t* k = p.K + row * D;
  const uint16_t* v = p.V + row * D;
  float ak[256], av[256];
  for (int d = 0; d < D; ++d) { ak[d] = 0.f; av[d] = 0.f; }
  for (int r = 0; r < ratio; ++r) {
    const int hq = hkv * ratio + r;
    const long qrow0 = (long)(b * p.Hq + hq) * p.Sq;
    const int i0 = p.causal ? max(0, j - off) : 0;
    for (int i = i0; i < p.Sq; ++i) {
      const uint16_t* q = p.Q + (qrow0 + i) * D;
      const uint16_t* g = p.dO + (qrow0 + i) * D;
      float s = 0.f, dp = 0.f;
      for (int d = 0; d < D; ++d) {
        s += from_storage<T>(q[d]) * from_storage<T>(k[d]);
        dp += from_storage<T>(g[d]) * from_storage<T>(v[d]);
      }
      const float pr = __expf(s * p.scale - p.LSE[qrow0 + i]);
      const float ds = pr * (dp - p.Delta[qrow0 + i]);
      for (int d = 0; d < D; ++d) {
        av[d] += pr * from_storage<T>(g[d]);
        ak[d] += ds * from_storage<T>(q[d]);
      }
    }
  }
  for (int d = 0; d < D; ++d) {
    p.dK[row * D + d] = ak[d] * p.scale;
    p.dV[row * D + d] = av[d];
  }
}

}  // namespace tsr950
