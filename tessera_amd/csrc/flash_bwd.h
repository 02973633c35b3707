// Flash-attention backward for gfx950: (dQ, dK, dV) of O = softmax(scale Q K^T, causal) V
// from dO, Q, K, V and the forward's O and log-sum-exp; GQA, 16-bit storage, f32
// accumulate, f32 gradients.
//
// Three kernels, no atomics, results independent of scheduling:
//   flash_bwd_delta_kernel   Delta[q] = sum_d dO[q][d] O[q][d]
//   flash_bwd_dq_kernel      one workgroup per 256 query rows, walks the key tiles
//   flash_bwd_dkdv_kernel    one workgroup per 128 keys of one KV head, walks the
//                            query tiles of every query head that shares the KV head;
//                            producer waves (S, dP, softmax) feed consumer waves (dK, dV)
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
  int qb = qblocks - 1 - blockIdx.x / (p.B * p.Hq);            // heavy causal blocks first
  int bh = blockIdx.x % (p.B * p.Hq);
  if ((p.B * p.Hkv) % 8 == 0) {
    // Workgroups go to the XCDs round robin.  Runs of 8 ratio workgroups take 8 KV heads,
    // one per XCD, with all the query heads of a group on their KV head's XCD; then
    // come the query blocks of those heads, heaviest first, then the next 8 KV heads.
    // The workgroups that walk the same K / V tiles share one L2, and an XCD works on
    // one or two KV heads at a time.
    const int ratio = p.Hq / p.Hkv;
    const int w = blockIdx.x % (8 * ratio), r = blockIdx.x / (8 * ratio);
    qb = qblocks - 1 - r % qblocks;
    bh = ((r / qblocks) * 8 + (w & 7)) * ratio + (w >> 3);
  }
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

constexpr int FB_BK = 128, FB_BQT = 64;                   // keys per workgroup, query rows per tile

// ---------------------------------------------------------------------------------
// dK, dV: one workgroup per 128 keys of a KV head, eight waves.  The four key groups of 32 keys each have a producer wave and a
// consumer wave on the same SIMD (waves g and g + 4).  The producer holds the K and V
// fragments of its keys, computes S and dP of a query tile and the softmax arithmetic,
// and hands P and dS (16-bit, in MFMA operand order) to the consumer through LDS; the
// consumer holds the dK and dV accumulators and does the second products of the tile
// the producer finished one iteration earlier.  Each wave stays under 256 registers
// (no accumulation-file traffic) and the two instruction streams of a SIMD fill each
// other's gaps: the producer's exponentials run under the consumer's MFMAs.
//
// Iteration i: loads of tile i + 1 are issued into stage (i + 1) % 3; the consumer reads
// P / dS of tile i - 1 into registers; barrier; the producer works on tile i (stage
// i % 3) and writes P / dS at its end, the consumer on tile i - 1 (stage (i - 1) % 3);
// barrier.  The exchange buffer is single: it is read before the first barrier and
// written after it.
// ---------------------------------------------------------------------------------
constexpr int FB_DKV_THREADS = 512;

template <int D>
constexpr int flash_bwd_dkdv_lds_bytes() {
  return 3 * (2 * FB_BQT * D * 2 + 2 * FB_BQT * 4) + 4 * 8 * 1024;
}

template <class T, int D>
__global__ __launch_bounds__(FB_DKV_THREADS) void flash_bwd_dkdv_kernel(const FlashBwdParams p) {
  constexpr int KSTEPS = D / 16, DT = D / 32, ROWB = D * 2, CHUNKS = D / 8;
  constexpr int TILE = FB_BQT * ROWB;                      // bytes of a Q (or dO) tile
  constexpr int STAGE = 2 * TILE + 2 * FB_BQT * 4;         // Q | dO | -LSE/scale [64] | -Delta [64]
  constexpr int XCH = 3 * STAGE;                           // exchange: [group][half][P | dS][quad][lane] x 16 B
  constexpr int LD_PER_WAVE = FB_BQT * CHUNKS / 64 / 8;
  static_assert(FB_BQT * CHUNKS % FB_DKV_THREADS == 0, "tile/thread mismatch");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(TSR_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave < 4;
  const int grp = wave & 3;
  const int l32 = lane & 31, lh = lane >> 5, r16 = lane & 15;

  // Heavy key blocks (low indices under a causal mask) first, over all KV heads.  (Giving
  // an XCD one KV head after the other, all of its key blocks together, cuts the Q / dO
  // bytes fetched by the L2 to a third and costs 5 % in time: the blocks of one head
  // differ too much in length.)
  const int kb = blockIdx.x / (p.B * p.Hkv);
  const int bh = blockIdx.x % (p.B * p.Hkv);
  const int b = bh / p.Hkv, hkv = bh % p.Hkv;
  const int ratio = p.Hq / p.Hkv;
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;
  const int k0 = kb * FB_BK;
  const int wave_k0 = k0 + grp * 32;
  const int key = wave_k0 + l32;                           // this lane's key
  const long kvrow0 = (long)(b * p.Hkv + hkv) * p.Sk;
  const float c = p.scale * kLog2e;

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
  auto load_tile = [&](int head, int tile, int stage) {
    const int qt0 = tile * FB_BQT;
    const long qrow0 = (long)(b * p.Hq + hkv * ratio + head) * p.Sq;
    const uint16_t* qb = p.Q + (qrow0 + qt0) * D;
    const uint16_t* gb = p.dO + (qrow0 + qt0) * D;
    const int last = p.Sq - 1 - qt0;                       // last valid row of this tile
    const uint32_t sbase = lds0 + stage * STAGE;
#pragma unroll
    for (int q = 0; q < LD_PER_WAVE; ++q) {
      uint32_t o = ld_off[q];
      if (ld_row[q] > last) o -= (uint32_t)(ld_row[q] - last) * ROWB;     // rows past the end: masked later
      load16_to_lds(qb, o, sbase + (wave * LD_PER_WAVE + q) * 1024);
      load16_to_lds(gb, o, sbase + TILE + (wave * LD_PER_WAVE + q) * 1024);
    }
    if (wave >= 6) {
      const float* src = (wave == 6 ? p.LSE2 : p.Delta) + qrow0 + qt0;
      const int r = lane <= last ? lane : last;
      load4_to_lds(src, (uint32_t)r * 4, sbase + 2 * TILE + (wave - 6) * FB_BQT * 4);
    }
  };
  // does this group's keys see the tile at all?  (uniform per wave, same answer in
  // the producer and the consumer of a group)
  auto tile_live = [&](int tile) {
    const int qt0 = tile * FB_BQT;
    return wave_k0 < p.Sk && (!p.causal || wave_k0 <= min(qt0 + FB_BQT, p.Sq) - 1 + off);
  };
  // Walk order: query tiles from the last one down, the group's query heads innermost.
  // Every key block of a KV head starts at the same tile and moves at the same pace, so
  // the workgroups that share Q / dO tiles (same XCD: blockIdx % 8 is the head's) read
  // them at the same time and the XCD's L2 serves all but one of those reads.
  auto next_of = [&](int& head, int& tile) {
    if (++head == ratio) { head = 0; --tile; }
  };
  const int t_last = qtiles - 1;
  char* xch = smem + XCH + grp * 8192;

  if (nsteps > 0) load_tile(0, t_last, 0);
  fa_wait_loads();
  __syncthreads();

  if (producer) {
    const int krow = key < p.Sk ? key : p.Sk - 1;
    uint4 kf[KSTEPS], vf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      kf[ks] = *reinterpret_cast<const uint4*>(p.K + (kvrow0 + krow) * D + 16 * ks + 8 * lh);
      vf[ks] = *reinterpret_cast<const uint4*>(p.V + (kvrow0 + krow) * D + 16 * ks + 8 * lh);
    }
    uint32_t row_rd[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) row_rd[ks] = l32 * ROWB + ((((ks << 1) | lh) ^ bwd_swz<D>(l32)) << 4);

    int cur_head = 0, cur_tile = t_last, st = 0;           // tile of this iteration and its stage
    for (int i = 0; i <= nsteps; ++i) {
      int nxt_head = cur_head, nxt_tile = cur_tile;
      next_of(nxt_head, nxt_tile);
      const int nst = st == 2 ? 0 : st + 1;
      if (i + 1 < nsteps) load_tile(nxt_head, nxt_tile, nst);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();                        // the consumer has taken P / dS of tile i - 1
      asm volatile("" ::: "memory");
      if (i < nsteps && tile_live(cur_tile)) {
        const char* base = smem + st * STAGE;
        const int qt0 = cur_tile * FB_BQT;
        const bool need_mask = (qt0 + FB_BQT > p.Sq) || (wave_k0 + 32 > p.Sk) ||
                               (p.causal && wave_k0 + 31 > qt0 + off);
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
          // accumulators start from -LSE / scale and -Delta of the lane's rows 8 a + 4 lh + 0..3
          f32x16 sv, dp;
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const int qoff = 32 * qt + 8 * a + 4 * lh;
            const float4 l4 = *reinterpret_cast<const float4*>(base + 2 * TILE + qoff * 4);
            const float4 d4 = *reinterpret_cast<const float4*>(base + 2 * TILE + FB_BQT * 4 + qoff * 4);
            sv[4 * a] = l4.x; sv[4 * a + 1] = l4.y; sv[4 * a + 2] = l4.z; sv[4 * a + 3] = l4.w;
            dp[4 * a] = d4.x; dp[4 * a + 1] = d4.y; dp[4 * a + 2] = d4.z; dp[4 * a + 3] = d4.w;
          }
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            const uint4 qfr = lds_read_b128(base, row_rd[ks] + qt * 32 * ROWB);
            const uint4 dofr = lds_read_b128(base, TILE + row_rd[ks] + qt * 32 * ROWB);
            sv = mfma_32x32x16<T>(qfr, kf[ks], sv);
            dp = mfma_32x32x16<T>(dofr, vf[ks], dp);
          }
          // lane: key, queries qt0 + 32 qt + 8 (r/4) + 4 lh + r % 4
          uint32_t pw[8], dw[8];
          auto softmax = [&](auto masked_c) __attribute__((always_inline)) {
            constexpr bool MASKED = decltype(masked_c)::value;
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
              float pr[2], ds[2];
#pragma unroll
              for (int e = 0; e < 2; ++e) {
                float x = sv[r + e] * c;
                if constexpr (MASKED) {
                  const int q = qt0 + 32 * qt + 8 * ((r + e) >> 2) + 4 * lh + ((r + e) & 3);
                  const bool ok = (q < p.Sq) & (key < p.Sk) & (!p.causal | (key <= q + off));
                  x = ok ? x : -INFINITY;                  // exponent -inf: P = 0, no branch
                }
                pr[e] = fast_exp2(x);
                ds[e] = pr[e] * dp[r + e];
              }
              pw[r >> 1] = pack2<T>(pr[0], pr[1]);
              dw[r >> 1] = pack2<T>(ds[0], ds[1]);
            }
          };
          if (need_mask) softmax(std::true_type{});
          else softmax(std::false_type{});
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            lds_write_b128(xch, ((qt * 2 + 0) * 2 + g) * 1024 + lane * 16,
                           make_uint4(pw[4 * g], pw[4 * g + 1], pw[4 * g + 2], pw[4 * g + 3]));
            lds_write_b128(xch, ((qt * 2 + 1) * 2 + g) * 1024 + lane * 16,
                           make_uint4(dw[4 * g], dw[4 * g + 1], dw[4 * g + 2], dw[4 * g + 3]));
          }
        }
      }
      cur_head = nxt_head;
      cur_tile = nxt_tile;
      st = nst;
      fa_wait_loads();
      __syncthreads();
    }
    return;
  }

  // ---- consumer ----
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

  int ld_head = 0, ld_tile = t_last, lst = 0;              // tile i (whose successor is loaded) and its stage
  int cur_tile = t_last, st = 0;                           // tile i - 1 and its stage (from i = 1 on)
  for (int i = 0; i <= nsteps; ++i) {
    int nxt_head = ld_head, nxt_tile = ld_tile;
    next_of(nxt_head, nxt_tile);
    const int nst = lst == 2 ? 0 : lst + 1;
    if (i + 1 < nsteps) load_tile(nxt_head, nxt_tile, nst);
    const bool live = i >= 1 && tile_live(cur_tile);
    uint4 pf[2][2], dsf[2][2];
    if (live) {
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          pf[qt][g] = lds_read_b128(xch, ((qt * 2 + 0) * 2 + g) * 1024 + lane * 16);
          dsf[qt][g] = lds_read_b128(xch, ((qt * 2 + 1) * 2 + g) * 1024 + lane * 16);
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();                          // P / dS taken: the producer may overwrite them
    asm volatile("" ::: "memory");
    if (live) {
      const char* base = smem + st * STAGE;
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const uint32_t o = (qt * 32 + g * 16) * ROWB;
            const uint2 qlo = lds_read_tr16_b64(base + tr_lo[dt] + o);
            const uint2 qhi = lds_read_tr16_b64(base + tr_hi[dt] + o);
            const uint2 olo = lds_read_tr16_b64(base + TILE + tr_lo[dt] + o);
            const uint2 ohi = lds_read_tr16_b64(base + TILE + tr_hi[dt] + o);
            dv[dt] = mfma_32x32x16<T>(make_uint4(olo.x, olo.y, ohi.x, ohi.y), pf[qt][g], dv[dt]);
            dk[dt] = mfma_32x32x16<T>(make_uint4(qlo.x, qlo.y, qhi.x, qhi.y), dsf[qt][g], dk[dt]);
          }
    }
    cur_tile = ld_tile;
    st = lst;
    ld_head = nxt_head;
    ld_tile = nxt_tile;
    lst = nst;
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
