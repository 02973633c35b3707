// Flash-attention forward for gfx950: O = softmax(scale * Q K^T, causal) V with
// GQA and the per-row log-sum-exp, 16-bit storage, f32 softmax and accumulate.
//
// One workgroup of 8 waves (two per SIMD) owns 256 query rows of one (batch, q
// head); each wave owns 32 of them as one MFMA tile.  K/V are walked in 64-key
// tiles staged through LDS (double buffered, one barrier per tile).  Two waves
// per SIMD let one wave's softmax (VALU) run under the other's MFMAs.
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
#include "common.h"

namespace tsr950 {

struct FlashParams {
  const uint16_t* Q;   // [B, Hq, Sq, D]
  const uint16_t* K;   // [B, Hkv, Sk, D]
  const uint16_t* V;   // [B, Hkv, Sk, D]
  void* O;             // [B, Hq, Sq, D]  f32 or storage dtype
  float* LSE;          // [B, Hq, Sq] or null
  int B, Hq, Hkv, Sq, Sk;
  float scale;
  int causal;
  int out_storage;     // 0: f32 O, 1: O in the storage dtype
};

constexpr int FA_WAVES = 8;
constexpr int FA_THREADS = FA_WAVES * 64;
constexpr int FA_BQ = FA_WAVES * 32;   // query rows per workgroup
constexpr int FA_BKV = 64;             // keys per LDS tile
constexpr float FA_NEG = -1.0e30f;

// Exchange a value with the lane 32 positions away.
__device__ __forceinline__ float swap_half(float v) {
  return __shfl_xor(v, 32, 64);
}

template <class T, int D>
__global__ __launch_bounds__(FA_THREADS, 1) void flash_fwd_kernel(const FlashParams p) {
  constexpr int KSTEPS = D / 16;         // MFMA k steps of the score product
  constexpr int DT = D / 32;             // 32-wide d tiles of the output
  constexpr int ROWB = D * 2;            // bytes per K/V row
  constexpr int CHUNKS = D / 8;          // 16-byte chunks per row
  constexpr int TILE = FA_BKV * ROWB;    // bytes per K (or V) tile
  constexpr int LD_PER_THREAD = FA_BKV * CHUNKS / FA_THREADS;
  static_assert(FA_BKV * CHUNKS % FA_THREADS == 0, "tile/thread mismatch");
  // K swizzle: the 16 rows an LDS cycle serves must hit 16 different 16-byte slots
  // of the 256-byte bank line.  V swizzle: the 4 rows of a patch, 64 bytes each.
  auto kswz = [](int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); };
  auto vswz = [](int key) { return D == 128 ? ((key & 3) << 2) : (((key >> 1) & 1) << 2); };

  extern __shared__ __attribute__((aligned(16))) char smem[];   // [2][K tile | V tile]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;

  // Work order.  Workgroups are dealt to the 8 XCDs round-robin by their linear id.
  // Levels of equal cost (one query block index for every (batch, head)) are
  // issued heaviest first — with a causal mask the last block has the longest key
  // range — so every XCD receives the same mix, and inside a level the (batch,
  // head) pairs are permuted so that all query heads sharing one KV head land on
  // the same XCD and find its K/V in that XCD's L2.
  const int qblocks = (p.Sq + FA_BQ - 1) / FA_BQ;
  const int BH = p.B * p.Hq;
  const int id = blockIdx.x;
  const int qb = qblocks - 1 - id / BH;
  const int u = id % BH;
  const int ratio = p.Hq / p.Hkv;
  int b, hq;
  if ((p.B * p.Hkv) % 8 == 0) {
    const int w = u % (8 * ratio);
    const int g = (u / (8 * ratio)) * 8 + (w & 7);   // kv group = (batch, kv head)
    b = g / p.Hkv;
    hq = (g % p.Hkv) * ratio + (w >> 3);
  } else {
    b = u / p.Hq;
    hq = u % p.Hq;
  }
  const int hkv = (int)(((long)hq * p.Hkv) / p.Hq);
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;

  const int q0 = qb * FA_BQ;             // first query row of the workgroup
  const int qw = q0 + wave * 32;         // first query row of the wave
  const uint16_t* Qb = p.Q + ((long)(b * p.Hq + hq) * p.Sq) * D;
  const uint16_t* Kb = p.K + ((long)(b * p.Hkv + hkv) * p.Sk) * D;
  const uint16_t* Vb = p.V + ((long)(b * p.Hkv + hkv) * p.Sk) * D;

  // Keys this workgroup needs: all of them, or up to the diagonal of its last row.
  int kv_end = p.Sk;
  if (p.causal) {
    const int last_q = min(q0 + FA_BQ, p.Sq) - 1;
    kv_end = min(p.Sk, last_q + off + 1);
  }
  const int ntiles = (kv_end + FA_BKV - 1) / FA_BKV;

  // ---- Q fragments: lane (q = l32, h) holds Q[q][16 ks + 8 h .. +7] -----------
  uint4 qf[KSTEPS];
  {
    int row = qw + l32;
    row = row < p.Sq ? row : p.Sq - 1;
    const uint16_t* src = Qb + (long)row * D + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const uint4*>(src + 16 * ks);
  }

  // ---- K/V tile loaders: chunk v = tid + THREADS q -> row v / CHUNKS, chunk v % CHUNKS
  uint4 rk[LD_PER_THREAD], rv[LD_PER_THREAD];
  auto gload = [&](int tile) {
    const int kv0 = tile * FA_BKV;
#pragma unroll
    for (int q = 0; q < LD_PER_THREAD; ++q) {
      const int v = tid + FA_THREADS * q;
      int row = kv0 + v / CHUNKS;
      row = row < p.Sk ? row : p.Sk - 1;          // rows past the end are masked below
      const long o = (long)row * D + (v % CHUNKS) * 8;
      rk[q] = *reinterpret_cast<const uint4*>(Kb + o);
      rv[q] = *reinterpret_cast<const uint4*>(Vb + o);
    }
  };
  auto lstore = [&](int buf) {
    char* kb = smem + buf * 2 * TILE;
    char* vb = kb + TILE;
#pragma unroll
    for (int q = 0; q < LD_PER_THREAD; ++q) {
      const int v = tid + FA_THREADS * q;
      const int row = v / CHUNKS, ch = v % CHUNKS;
      lds_write_b128(kb, row * ROWB + ((ch ^ kswz(row)) << 4), rk[q]);
      lds_write_b128(vb, row * ROWB + ((ch ^ vswz(row)) << 4), rv[q]);
    }
  };

  // ---- state -----------------------------------------------------------------
  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;
  float m_run = FA_NEG;                  // running max of the raw (unscaled) scores
  float l_run = 0.f;                     // this lane half's share of the running sum
  const float c = p.scale * 1.44269504088896340736f;   // scale * log2(e)

  // Per-wave range: tiles past the wave's own diagonal contribute nothing.
  int wave_kv_end = kv_end;
  if (p.causal) wave_kv_end = min(kv_end, min(qw + 32, p.Sq) - 1 + off + 1);
  const bool wave_active = qw < p.Sq;
  const int qi = qw + l32;               // this lane's query row
  const int lim = p.causal ? min(qi + off, p.Sk - 1) : p.Sk - 1;   // last visible key

  // per-lane LDS read offsets
  const int r16 = lane & 15;
  uint32_t k_rd[2];
  int k_sw[2];
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
    const int row = kt * 32 + l32;
    k_rd[kt] = row * ROWB;
    k_sw[kt] = kswz(row);
  }

  if (ntiles > 0) {
    gload(0);
    lstore(0);
  }
  __syncthreads();

  auto process = [&](int t) {
    const int buf = t & 1;
    const int kv0 = t * FA_BKV;
    const char* kb = smem + buf * 2 * TILE;
    const char* vb = kb + TILE;
    if (wave_active && kv0 < wave_kv_end) {
      // ---- S^T = K . Q^T ------------------------------------------------------
      f32x16 s[2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          const uint4 kf = lds_read_b128(kb, k_rd[kt] + ((((ks << 1) | lh) ^ k_sw[kt]) << 4));
          s[kt] = mfma_32x32x16<T>(kf, qf[ks], s[kt]);
        }
      }

      // ---- mask (only tiles that touch the diagonal or the end of K) ------------
      const bool need_mask = (kv0 + FA_BKV > p.Sk) || (p.causal && (kv0 + FA_BKV - 1 > qw + off));
      if (need_mask) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kv0 + kt * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (key > lim) s[kt][r] = FA_NEG;
          }
      }

      // ---- online softmax; P stays in the S registers -----------------------------
      float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, fmaxf(s[0][r], s[1][r]));
      mx = fmaxf(mx, swap_half(mx));
      const float m_new = fmaxf(m_run, mx);
      const float mc = m_new * c;
      // Rescale the accumulator only when some row of the wave raised its maximum.
      if (__any(m_new > m_run)) {
        const float corr = fast_exp2((m_run - m_new) * c);
        l_run *= corr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o_acc[dt][r] *= corr;
        m_run = m_new;
      }
      float sum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = fast_exp2(fmaf(s[kt][r], c, -mc));
          s[kt][r] = e;
          sum += e;
        }
      l_run += sum;
      uint4 pf[2][2];   // [kt][g]: B operand of the (kt, g) 16-key step
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          pf[kt][g].x = pack2<T>(s[kt][8 * g + 0], s[kt][8 * g + 1]);
          pf[kt][g].y = pack2<T>(s[kt][8 * g + 2], s[kt][8 * g + 3]);
          pf[kt][g].z = pack2<T>(s[kt][8 * g + 4], s[kt][8 * g + 5]);
          pf[kt][g].w = pack2<T>(s[kt][8 * g + 6], s[kt][8 * g + 7]);
        }

      // ---- O^T += V^T . P^T ------------------------------------------------------
      // 16-key step (kt, g) covers keys 32 kt + 16 g + {4h + 0..3, 8 + 4h + 0..3}.
      // Transposing read: lane r of a 16-lane block supplies row (key) r/4 of a
      // 4-key patch and columns 4 (r % 4) .. +3 of a 16-column slab.
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const int key_lo = kt * 32 + g * 16 + 4 * lh + (r16 >> 2);
          const int key_hi = key_lo + 8;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);   // element column
            const int ch = col >> 3, within = (col & 7) * 2;
            const uint2 lo = lds_read_tr16_b64(vb + key_lo * ROWB + ((ch ^ vswz(key_lo)) << 4) + within);
            const uint2 hi = lds_read_tr16_b64(vb + key_hi * ROWB + ((ch ^ vswz(key_hi)) << 4) + within);
            o_acc[dt] = mfma_32x32x16<T>(make_uint4(lo.x, lo.y, hi.x, hi.y), pf[kt][g], o_acc[dt]);
          }
        }
    }
  };
  // Tile t+1 is fetched into registers while tile t is consumed, then stored to
  // the other buffer; the last tile has nothing to fetch.
  for (int t = 0; t + 1 < ntiles; ++t) {
    gload(t + 1);
    process(t);
    lstore((t & 1) ^ 1);
    __syncthreads();
  }
  if (ntiles > 0) process(ntiles - 1);

  // ---- epilogue -------------------------------------------------------------------
  if (!wave_active) return;
  const float l = l_run + swap_half(l_run);
  if (qi >= p.Sq) return;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  const long row = (long)(b * p.Hq + hq) * p.Sq + qi;
  if (p.LSE && lh == 0)
    p.LSE[row] = l > 0.f ? (m_run * c + __log2f(l)) * 0.69314718055994530942f : -INFINITY;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int d = dt * 32 + 8 * a + 4 * lh;
      const float v0 = o_acc[dt][4 * a + 0] * inv, v1 = o_acc[dt][4 * a + 1] * inv;
      const float v2 = o_acc[dt][4 * a + 2] * inv, v3 = o_acc[dt][4 * a + 3] * inv;
      if (p.out_storage) {
        uint2 pk;
        pk.x = pack2<T>(v0, v1);
        pk.y = pack2<T>(v2, v3);
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.O) + row * D + d) = pk;
      } else {
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.O) + row * D + d) = make_float4(v0, v1, v2, v3);
      }
    }
}

// Any head dimension: one thread per query row, streaming online softmax in f32.
// Serves the shapes the MFMA kernel does not (D not 64 or 128).
template <class T>
__global__ void flash_fwd_generic_kernel(const FlashParams p, int D) {
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long total = (long)p.B * p.Hq * p.Sq;
  if (row >= total) return;
  const int qi = (int)(row % p.Sq);
  const int hq = (int)((row / p.Sq) % p.Hq);
  const int b = (int)(row / ((long)p.Sq * p.Hq));
  const int hkv = (int)(((long)hq * p.Hkv) / p.Hq);
  const int off = p.Sk > p.Sq ? p.Sk - p.Sq : 0;
  const uint16_t* q = p.Q + row * D;
  const uint16_t* Kb = p.K + ((long)(b * p.Hkv + hkv) * p.Sk) * D;
  const uint16_t* Vb = p.V + ((long)(b * p.Hkv + hkv) * p.Sk) * D;
  float acc[256];
  for (int d = 0; d < D; ++d) acc[d] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int jmax = p.causal ? min(qi + off, p.Sk - 1) : p.Sk - 1;
  for (int j = 0; j <= jmax; ++j) {
    float s = 0.f;
    for (int d = 0; d < D; ++d) s += from_storage<T>(q[d]) * from_storage<T>(Kb[(long)j * D + d]);
    s *= p.scale;
    const float mn = fmaxf(m, s);
    const float cr = __expf(m - mn);       // exp(-inf) = 0 on the first key
    const float e = __expf(s - mn);
    l = l * cr + e;
    for (int d = 0; d < D; ++d) acc[d] = acc[d] * cr + e * from_storage<T>(Vb[(long)j * D + d]);
    m = mn;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  if (p.LSE) p.LSE[row] = l > 0.f ? m + __logf(l) : -INFINITY;
  for (int d = 0; d < D; ++d) {
    const float v = acc[d] * inv;
    if (p.out_storage) reinterpret_cast<uint16_t*>(p.O)[row * D + d] = to_storage<T>(v);
    else reinterpret_cast<float*>(p.O)[row * D + d] = v;
  }
}

}  // namespace tsr950
