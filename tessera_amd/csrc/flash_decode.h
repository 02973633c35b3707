// Flash-attention forward for few query rows per KV head (decode and short speculative
// steps): O = softmax(scale * Q K^T) V with GQA and the per-row log-sum-exp, 16-bit storage.
//
// The general kernel (flash_attn.h) gives a workgroup 256 query rows of ONE query head.  With
// one query row per head that is one useful row in 256, one workgroup per head however long
// the key range is, and every query head of a GQA group streams the group's K and V again.
// Here the rows of a whole GQA group — (Hq / Hkv) heads x Sq rows, at most 32 NQ — are the
// columns of NQ MFMA tiles that share every K / V fragment, so K and V of a KV head are read once for the group; the key
// range of a (batch, KV head) is split over gridDim.y workgroups and, inside a workgroup, over
// its waves (wave w takes the 32-key tiles w, w + WAVES, ...), so the read of K and V — the
// bound of this problem — is spread over the whole chip.  Every wave runs the online softmax
// of its own tiles (the arithmetic and the register layouts of the general kernel: transposed
// products, exact row maximum, base-2 exponentials); K and V tiles stream from global memory
// straight into a wave-private LDS region, two stages, no workgroup barrier in the loop.  The
// waves' partial (max, sum, O) are merged through LDS at the end; with more than one key split
// the workgroup writes a normalised partial O and its log-sum-exp, and flash_decode_merge_kernel
// merges the splits.
#pragma once
#include "flash_attn.h"

namespace tsr950 {

template <int DP> struct DecodeGeom {
  static constexpr int WAVES = DP > 128 ? 2 : 4;
  static constexpr int THREADS = WAVES * 64;
  static constexpr int BK = 32;                       // keys per tile
  static constexpr int TILE = BK * DP * 2;            // bytes of one K (or V) tile
  static constexpr int WAVE_LDS = 4 * TILE;           // K stage 0, 1, V stage 0, 1
  static constexpr int STAGE_PITCH = DP * 4 + 16;     // a row of the wave's f32 partial O
  static constexpr int SMEM = WAVES * WAVE_LDS;
  static constexpr int ML_AT = SMEM - 2048;           // the waves' (max, sum) and the merged ones
  static_assert(32 * STAGE_PITCH <= WAVE_LDS - 2048, "a wave's partial O must fit its LDS region");
};

struct FlashDecodeParams {
  FlashParams f;
  float* part_o;          // [nsplit][B * Hq * Sq][D] normalised partial O, or null when nsplit == 1
  float* part_lse;        // [nsplit][B * Hq * Sq] natural-log LSE of each partial
  int rows;               // (Hq / Hkv) * Sq <= 32 NQ: the query rows of one KV head
  int tile_lo;            // first 32-key tile any row sees
  int tile_end;           // one past the last
  int tiles_per_split;
};

template <class T, int DP, int NQ>
__global__ __launch_bounds__(DecodeGeom<DP>::THREADS) void flash_decode_kernel(const FlashDecodeParams dp) {
  using G = DecodeGeom<DP>;
  const FlashParams& p = dp.f;
  constexpr int D = DP;
  constexpr int KSTEPS = D / 16, DT = D / 32;
  constexpr int ROWB = D * 2, CHUNKS = D / 8, TILE = G::TILE;
  constexpr int LD = G::BK * CHUNKS / 64;            // 1 KB load instructions per K (or V) tile
  auto kswz = [](int row) { return CHUNKS % 16 == 0 ? (row & 15) : ((row >> 1) & 7); };
  auto vswz = [](int key) { return CHUNKS % 16 == 0 ? ((key & 3) << 2) : (((key >> 1) & 1) << 2); };

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  char* wsm = smem + wave * G::WAVE_LDS;               // this wave's region: K0 K1 V0 V1
  const uint32_t wlds = (uint32_t)(uintptr_t)(TSR_LDS char*)wsm;

  const int kvlin = blockIdx.x, split = blockIdx.y;
  const int batch = kvlin / p.Hkv, hkv = kvlin - batch * p.Hkv;
  // Row i of the group (tile i / 32, column i % 32): query row i % Sq of query head hkv * ratio + i / Sq.
  const uint16_t* Kb = p.K + batch * p.ks.batch + hkv * p.ks.head;
  const uint16_t* Vb = p.V + batch * p.vs.batch + hkv * p.vs.head;

  uint4 qf[NQ][KSTEPS];
  int klo[NQ], khi[NQ];                                // a row past dp.rows sees no key
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    const int i = 32 * qt + l32;
    const bool valid = i < dp.rows;
    const int hsel = valid ? i / p.Sq : 0;
    const int qi = valid ? i - hsel * p.Sq : 0;
    const uint16_t* src = p.Q + batch * p.qs.batch + (hkv * p.ratio + hsel) * p.qs.head + (long)qi * p.qs.row + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
      qf[qt][ks] = valid ? *reinterpret_cast<const uint4*>(src + 16 * ks) : make_uint4(0u, 0u, 0u, 0u);
    klo[qt] = 0;
    khi[qt] = -1;
    if (valid) key_bounds(qi, p.Sq, p.Sk, p.causal, p.window, klo[qt], khi[qt]);
  }
  int lo0, hi0, lo1, hi1;                              // bounds of the first and the last query row
  key_bounds(0, p.Sq, p.Sk, p.causal, p.window, lo0, hi0);
  key_bounds(p.Sq - 1, p.Sq, p.Sk, p.causal, p.window, lo1, hi1);

  // ---- loader: lane's 16-byte slot P = q * 64 + lane of a tile is (row P / CHUNKS, physical
  // chunk P % CHUNKS) and holds the row's logical chunk (physical ^ swizzle(row)).
  int ld_row[LD];
  uint32_t ld_koff[LD], ld_voff[LD];
  const uint32_t krow_bytes = (uint32_t)p.ks.row * 2, vrow_bytes = (uint32_t)p.vs.row * 2;
#pragma unroll
  for (int q = 0; q < LD; ++q) {
    const int P = q * 64 + lane;
    const int row = P / CHUNKS, chp = P % CHUNKS;
    ld_row[q] = row;
    ld_koff[q] = row * krow_bytes + ((chp ^ kswz(row)) << 4);
    ld_voff[q] = row * vrow_bytes + ((chp ^ vswz(row)) << 4);
  }
  auto load_tile = [&](int tile, int stage) {
    const uint16_t* kt = Kb + (long)tile * G::BK * p.ks.row;
    const uint16_t* vt = Vb + (long)tile * G::BK * p.vs.row;
    const int last = p.Sk - 1 - tile * G::BK;          // last valid row of this tile (>= 31: all)
#pragma unroll
    for (int q = 0; q < LD; ++q) {
      uint32_t ko = ld_koff[q], vo = ld_voff[q];
      if (ld_row[q] > last) {                          // clamp: rows past the end are masked below
        ko -= (uint32_t)(ld_row[q] - last) * krow_bytes;
        vo -= (uint32_t)(ld_row[q] - last) * vrow_bytes;
      }
      load16_to_lds(kt, ko, wlds + stage * TILE + q * 1024);
      load16_to_lds(vt, vo, wlds + (2 + stage) * TILE + q * 1024);
    }
  };

  // ---- LDS read addresses (as in the general kernel, one 32-key tile) ----
  uint32_t k_rd[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_rd[ks] = l32 * ROWB + ((((ks << 1) | lh) ^ kswz(l32)) << 4);
  const int r16 = lane & 15;
  uint32_t v_rd[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int key = 4 * lh + (r16 >> 2);
    const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);
    v_rd[dt] = 2 * TILE + key * ROWB + (((col >> 3) ^ vswz(key)) << 4) + (col & 7) * 2;
  }

  // ---- state ----
  f32x16 o_acc[NQ][DT];
  float m_run[NQ], l_run[NQ];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    m_run[qt] = FA_NEG;
    l_run[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o_acc[qt][dt][r] = 0.f;
  }
  const float cs = p.scale * 1.44269504088896340736f;  // scale * log2(e); scale > 0 on this path

  const int t0 = dp.tile_lo + split * dp.tiles_per_split;
  const int t1 = min(t0 + dp.tiles_per_split, dp.tile_end);
  int t = t0 + wave, stage = 0;
  if (t < t1) load_tile(t, 0);
  for (; t < t1; t += G::WAVES) {
    const bool more = t + G::WAVES < t1;
    if (more) {
      load_tile(t + G::WAVES, stage ^ 1);
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * LD) : "memory");   // this tile's loads have landed
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // S^T = K . Q^T for the tile's 32 keys; a K fragment serves the NQ query tiles
    f32x16 sc[NQ];
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[qt][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const uint4 kf = lds_read_b128(wsm, k_rd[ks] + stage * TILE);
#pragma unroll
      for (int qt = 0; qt < NQ; ++qt) sc[qt] = mfma_32x32x16<T>(kf, qf[qt][ks], sc[qt]);
    }
    const int kv0 = t * G::BK;
    const bool need_mask = kv0 + G::BK - 1 > hi0 || kv0 < lo1;
    uint4 pf[NQ][2];
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
      if (need_mask) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kv0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (key > khi[qt] || key < klo[qt]) sc[qt][r] = FA_NEG;
        }
      }
      float mx = max3_raw(sc[qt][0], sc[qt][1], sc[qt][2]);
#pragma unroll
      for (int r = 3; r < 16; r += 2) mx = (r + 1 < 16) ? max3_raw(mx, sc[qt][r], sc[qt][r + 1]) : fmaxf(mx, sc[qt][r]);
      mx = max_with_other_half(mx);
      const float m_new = fmaxf(m_run[qt], mx);
      if (__any(m_new > m_run[qt])) {
        const float corr = fast_exp2((m_run[qt] - m_new) * cs);
        l_run[qt] *= corr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o_acc[qt][dt][r] *= corr;
        m_run[qt] = m_new;
      }
      // (a row that has met no visible key keeps the sentinel: reference 0, so masked entries give P = 0)
      const float mc = m_new > 0.5f * FA_NEG ? m_new * cs : 0.f;
      float sum = 0.f;
#pragma unroll
      for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int r = 8 * g; r < 8 * g + 8; ++r) {
          const float e = fast_exp2(fmaf(sc[qt][r], cs, -mc));
          sc[qt][r] = e;
          sum += e;
        }
        pf[qt][g].x = pack2<T>(sc[qt][8 * g + 0], sc[qt][8 * g + 1]);
        pf[qt][g].y = pack2<T>(sc[qt][8 * g + 2], sc[qt][8 * g + 3]);
        pf[qt][g].z = pack2<T>(sc[qt][8 * g + 4], sc[qt][8 * g + 5]);
        pf[qt][g].w = pack2<T>(sc[qt][8 * g + 6], sc[qt][8 * g + 7]);
      }
      l_run[qt] += sum;
    }
    // O^T += V^T . P^T, 16 keys per step; a V fragment serves the NQ query tiles
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const uint32_t a = v_rd[dt] + stage * TILE + g * 16 * ROWB;
        const uint2 lo = lds_read_tr16_b64(wsm + a);
        const uint2 hi = lds_read_tr16_b64(wsm + a + 8 * ROWB);
        const uint4 vf = make_uint4(lo.x, lo.y, hi.x, hi.y);
#pragma unroll
        for (int qt = 0; qt < NQ; ++qt) o_acc[qt][dt] = mfma_32x32x16<T>(vf, pf[qt][g], o_acc[qt][dt]);
      }
    stage ^= 1;
  }

  // ---- merge the waves' partials through LDS, one 32-row query tile at a time ----
  float* ml = reinterpret_cast<float*>(smem + G::ML_AT);     // m[WAVES][32] | l[WAVES][32] | m_tot[32] | l_tot[32]
  const bool final_out = dp.part_o == nullptr;
  const long total_rows = (long)p.B * p.Hq * p.Sq;
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    __syncthreads();                                         // every wave is done with its tiles / the last pass
    const float l_wave = l_run[qt] + swap_half(l_run[qt]);
    if (lh == 0) {
      ml[wave * 32 + l32] = m_run[qt];
      ml[(G::WAVES + wave) * 32 + l32] = l_wave;
    }
    __syncthreads();
    float m_tot = FA_NEG;
#pragma unroll
    for (int w = 0; w < G::WAVES; ++w) m_tot = fmaxf(m_tot, ml[w * 32 + l32]);
    float l_tot = 0.f;
#pragma unroll
    for (int w = 0; w < G::WAVES; ++w) l_tot += ml[(G::WAVES + w) * 32 + l32] * fast_exp2((ml[w * 32 + l32] - m_tot) * cs);
    const float mine = fast_exp2((m_run[qt] - m_tot) * cs);  // both sentinels: 1, on accumulators that are 0
    if (wave == 0 && lh == 0) {
      ml[2 * G::WAVES * 32 + l32] = m_tot;
      ml[(2 * G::WAVES + 1) * 32 + l32] = l_tot;
    }
    {
      char* stg = wsm;                                       // [32 rows][STAGE_PITCH], f32
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int d = dt * 32 + 8 * a + 4 * lh;
          *reinterpret_cast<float4*>(stg + l32 * G::STAGE_PITCH + d * 4) =
              make_float4(o_acc[qt][dt][4 * a + 0] * mine, o_acc[qt][dt][4 * a + 1] * mine, o_acc[qt][dt][4 * a + 2] * mine,
                          o_acc[qt][dt][4 * a + 3] * mine);
        }
    }
    __syncthreads();
    // every thread sums four columns of one row over the waves and stores them
    const int rows_here = min(32, dp.rows - 32 * qt);
    for (int idx = tid; idx < rows_here * (D / 4); idx += G::THREADS) {
      const int il = idx / (D / 4), d = (idx - il * (D / 4)) * 4;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int w = 0; w < G::WAVES; ++w) {
        const float4 v = *reinterpret_cast<const float4*>(smem + w * G::WAVE_LDS + il * G::STAGE_PITCH + d * 4);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
      }
      const float mt = ml[2 * G::WAVES * 32 + il], lt = ml[(2 * G::WAVES + 1) * 32 + il];
      const float inv = lt > 0.f ? 1.0f / lt : 0.f;
      acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
      const int i = 32 * qt + il;
      const int hs = i / p.Sq, q = i - hs * p.Sq;
      const int hq_i = hkv * p.ratio + hs;
      const long rowlin = ((long)batch * p.Hq + hq_i) * p.Sq + q;
      const float lse = lt > 0.f ? (mt * cs + __log2f(lt)) * 0.69314718055994530942f : -INFINITY;
      if (final_out) {
        const long o_at = batch * p.os.batch + hq_i * p.os.head + (long)q * p.os.row + d;
        if (p.out_storage) {
          uint2 pk;
          pk.x = pack2<T>(acc.x, acc.y);
          pk.y = pack2<T>(acc.z, acc.w);
          *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.O) + o_at) = pk;
        } else {
          *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.O) + o_at) = acc;
        }
        if (p.LSE && d == 0) p.LSE[rowlin] = lse;
      } else {
        *reinterpret_cast<float4*>(dp.part_o + ((long)split * total_rows + rowlin) * D + d) = acc;
        if (d == 0) dp.part_lse[(long)split * total_rows + rowlin] = lse;
      }
    }
  }
}

// O[row] = sum_s w_s O_s[row] / sum_s w_s with w_s = exp(LSE_s - max LSE): the merge of the
// key splits' normalised partials; LSE[row] = max + log(sum_s w_s).  One thread per four columns.
template <class T>
__global__ __launch_bounds__(256) void flash_decode_merge_kernel(const FlashParams p, const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_lse, int nsplit) {
  const int D = p.D, per_row = D / 4;
  const long total_rows = (long)p.B * p.Hq * p.Sq;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total_rows * per_row) return;
  const long row = idx / per_row;
  const int d = (int)(idx - row * per_row) * 4;
  // (four splits fetched together in both passes: every one of these loads is a trip to memory)
  float mx = -INFINITY;
  for (int s0 = 0; s0 < nsplit; s0 += 4) {
    float l[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) l[u] = s0 + u < nsplit ? part_lse[(long)(s0 + u) * total_rows + row] : -INFINITY;
    mx = fmaxf(fmaxf(mx, fmaxf(l[0], l[1])), fmaxf(l[2], l[3]));
  }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float wsum = 0.f;
  if (mx > -INFINITY) {
    for (int s0 = 0; s0 < nsplit; s0 += 4) {
      float l[4];
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool on = s0 + u < nsplit;
        l[u] = on ? part_lse[(long)(s0 + u) * total_rows + row] : -INFINITY;
        v[u] = on ? *reinterpret_cast<const float4*>(part_o + ((long)(s0 + u) * total_rows + row) * D + d)
                  : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {                    // split order
        const float w = __expf(l[u] - mx);             // (exp(-inf) = 0 for the splits past the end)
        acc.x += w * v[u].x; acc.y += w * v[u].y; acc.z += w * v[u].z; acc.w += w * v[u].w;
        wsum += w;
      }
    }
  }
  const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
  acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
  const int q = (int)(row % p.Sq);
  const int hq = (int)((row / p.Sq) % p.Hq);
  const int b = (int)(row / ((long)p.Sq * p.Hq));
  const long o_at = b * p.os.batch + hq * p.os.head + (long)q * p.os.row + d;
  if (p.out_storage) {
    uint2 pk;
    pk.x = pack2<T>(acc.x, acc.y);
    pk.y = pack2<T>(acc.z, acc.w);
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.O) + o_at) = pk;
  } else {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.O) + o_at) = acc;
  }
  if (p.LSE && d == 0) p.LSE[row] = wsum > 0.f ? mx + __logf(wsum) : -INFINITY;
}

// The same merge with one workgroup per row, for many splits (a long single sequence: few rows, up to 512
// splits): the thread-per-four-columns form above walks the splits one dependent memory round trip after
// another.  Here the row's LSE values go through LDS, the weights are formed once, the 256 threads share
// the splits among 256 / (D / 4) groups with all their loads independent, and the groups' sums are added
// in group order.  Every order of summation is fixed, so the result does not depend on scheduling.
constexpr int kMergeMaxSplits = 512;
template <class T>
__global__ __launch_bounds__(256) void flash_decode_merge_rows_kernel(const FlashParams p, const float* __restrict__ part_o,
                                                                      const float* __restrict__ part_lse, int nsplit) {
  __shared__ float sh_w[kMergeMaxSplits];
  __shared__ float4 sh_acc[256];
  __shared__ float sh_red[8];
  const int D = p.D, per_row = D / 4, G = 256 / per_row;
  const long total_rows = (long)p.B * p.Hq * p.Sq;
  const long row = blockIdx.x;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  float mx = -INFINITY;
  for (int s = t; s < nsplit; s += 256) {
    const float l = part_lse[(long)s * total_rows + row];
    sh_w[s] = l;
    mx = fmaxf(mx, l);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  if (lane == 0) sh_red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(sh_red[0], sh_red[1]), fmaxf(sh_red[2], sh_red[3]));
  for (int s = t; s < nsplit; s += 256) sh_w[s] = mx > -INFINITY ? __expf(sh_w[s] - mx) : 0.f;
  __syncthreads();
  if (wave == 0) {                                     // the sum of the weights: lane order, then a fixed tree
    float ws = 0.f;
    for (int s = lane; s < nsplit; s += 64) ws += sh_w[s];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ws += __shfl_xor(ws, o, 64);
    if (lane == 0) sh_red[4] = ws;
  }
  const int g = t / per_row, c = t - g * per_row;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (g < G) {
    const float* src = part_o + row * D + 4 * c;
    const long step = total_rows * D;
    int s = g;
    for (; s + 3 * G < nsplit; s += 4 * G) {
      const float4 v0 = *reinterpret_cast<const float4*>(src + (long)s * step);
      const float4 v1 = *reinterpret_cast<const float4*>(src + (long)(s + G) * step);
      const float4 v2 = *reinterpret_cast<const float4*>(src + (long)(s + 2 * G) * step);
      const float4 v3 = *reinterpret_cast<const float4*>(src + (long)(s + 3 * G) * step);
      const float w0 = sh_w[s], w1 = sh_w[s + G], w2 = sh_w[s + 2 * G], w3 = sh_w[s + 3 * G];
      acc.x += w0 * v0.x; acc.y += w0 * v0.y; acc.z += w0 * v0.z; acc.w += w0 * v0.w;
      acc.x += w1 * v1.x; acc.y += w1 * v1.y; acc.z += w1 * v1.z; acc.w += w1 * v1.w;
      acc.x += w2 * v2.x; acc.y += w2 * v2.y; acc.z += w2 * v2.z; acc.w += w2 * v2.w;
      acc.x += w3 * v3.x; acc.y += w3 * v3.y; acc.z += w3 * v3.z; acc.w += w3 * v3.w;
    }
    for (; s < nsplit; s += G) {
      const float4 v = *reinterpret_cast<const float4*>(src + (long)s * step);
      const float w = sh_w[s];
      acc.x += w * v.x; acc.y += w * v.y; acc.z += w * v.z; acc.w += w * v.w;
    }
  }
  sh_acc[t] = acc;
  __syncthreads();
  if (g != 0) return;
  for (int gg = 1; gg < G; ++gg) {
    const float4 v = sh_acc[gg * per_row + c];
    acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
  }
  const float wsum = sh_red[4];
  const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
  acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
  const int d = 4 * c;
  const int q = (int)(row % p.Sq);
  const int hq = (int)((row / p.Sq) % p.Hq);
  const int b = (int)(row / ((long)p.Sq * p.Hq));
  const long o_at = b * p.os.batch + hq * p.os.head + (long)q * p.os.row + d;
  if (p.out_storage) {
    uint2 pk;
    pk.x = pack2<T>(acc.x, acc.y);
    pk.y = pack2<T>(acc.z, acc.w);
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.O) + o_at) = pk;
  } else {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.O) + o_at) = acc;
  }
  if (p.LSE && c == 0) p.LSE[row] = wsum > 0.f ? mx + __logf(wsum) : -INFINITY;
}

// Launches the merge of `nsplit` partials: a workgroup per row from 8 splits on while the rows are few
// (with many rows the thread-per-four-columns form has the parallelism to hide its round trips).
template <class T>
inline void launch_flash_merge(const FlashParams& p, const float* part_o, const float* part_lse, int nsplit, hipStream_t s) {
  const long rows = (long)p.B * p.Hq * p.Sq;
  if (nsplit >= 8 && nsplit <= kMergeMaxSplits && rows <= 4096) {
    hipLaunchKernelGGL((flash_decode_merge_rows_kernel<T>), dim3((unsigned)rows), dim3(256), 0, s, p, part_o, part_lse, nsplit);
    return;
  }
  const long quads = rows * (p.D / 4);
  hipLaunchKernelGGL((flash_decode_merge_kernel<T>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, p, part_o,
                     part_lse, nsplit);
}

}  // namespace tsr950
