// Skinny 16-bit GEMM for gfx950: D[M,N] = A[M,K] B[K,N] for a handful of rows
// (decode-shaped; the launcher uses it up to M = 8, the kernel handles M <= 32 MI).
//
// The product is bound by streaming B from HBM once, so the kernel is built around
// bytes in flight rather than MFMA rate: a workgroup owns a strip of 64 or 128 columns
// of B and a K range, and each of its waves walks its own slices of that range with
// two slices (8 KB of B per wave) outstanding.  A slice passes through a wave-private LDS
// buffer only to be transposed into MFMA operand order (ds_read_b64_tr_b16); no
// barrier is taken until the waves' partial accumulators are summed through LDS in a
// fixed tree order at the end.  A is read straight from global memory (it is small
// and stays in L2) in operand layout: every lane reads its own row, so one such load
// touches as many cache lines as there are rows, which is why the square-tile kernel
// (A staged through LDS) catches up from M = 16 on.
#pragma once
#include "gemm16.h"

namespace tsr950 {

// Shape of one wave's work: NJ 32-column blocks (a workgroup owns 32 NJ columns) and
// slices of 16 KS rows of K.  A slice row is 64 NJ bytes; the LDS row pitch adds 64
// bytes so that the four rows of a transposing read fall in disjoint banks.
template <int NJ, int KS>
struct SkinnyShape {
  static constexpr int kCols = 32 * NJ;
  static constexpr int kRows = 16 * KS;
  static constexpr int kPitch = 64 * NJ + 64;
  static constexpr int kWaveLds = kRows * kPitch;
  static constexpr int kLoads = KS * NJ;           // 16-byte loads per lane per slice
  static constexpr int kLanesPerRow = 4 * NJ;
  static constexpr int kRowsPerLoad = 64 / kLanesPerRow;
};

template <int MI, int NW, int NJ, int KS>
constexpr int skinny_lds_bytes() {
  constexpr int slices = NW * SkinnyShape<NJ, KS>::kWaveLds;
  constexpr int tree = (NW / 2) * MI * NJ * 16 * 64 * 4;
  constexpr int tile = MI * 32 * (32 * NJ + 4) * 4;  // epilogue staging
  constexpr int big = slices > tree ? slices : tree;
  return big > tile ? big : tile;
}

// EPI: EPI_F32 or EPI_STORE16.  Split z = blockIdx.y covers K rows [z kps, (z+1) kps)
// and writes its tile at D + z strideD.
template <class T, int MI, int NW, int NJ, int KS, int EPI>
__global__ __launch_bounds__(NW * 64) void gemm16_skinny_kernel(Gemm16Params p, int kps) {
  using S = SkinnyShape<NJ, KS>;
  extern __shared__ __align__(16) char smem[];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int n0 = blockIdx.x * S::kCols;
  const int z = blockIdx.y;
  const int kbeg = z * kps;
  const int kend = min(p.K, kbeg + kps);
  const int nslices = kend > kbeg ? (kend - kbeg) / S::kRows : 0;

  // B slice load.  256-byte rows (NJ = 4): a 16-lane write pass is one whole row.
  // 128-byte rows (NJ = 2): the 16-lane groups take rows {0,2},{1,3},{4,6},{5,7} so
  // that one ds_write_b128 pass still covers all 64 banks.
  const int ch = lane % S::kLanesPerRow;
  int brow = lane / S::kLanesPerRow;
  if constexpr (NJ == 2) {
    const int g = lane >> 4, h = (lane >> 3) & 1;
    brow = 4 * (g >> 1) + (g & 1) + 2 * h;
  }
  uint32_t b_off[S::kLoads];
  uint32_t b_wr[S::kLoads];
#pragma unroll
  for (int q = 0; q < S::kLoads; ++q) {
    const int row = brow + S::kRowsPerLoad * q;
    b_off[q] = (n0 + ch * 8 < p.N) ? (uint32_t)(((long)row * p.ldb + n0 + ch * 8) * 2) : kOutOfRange;
    b_wr[q] = w * S::kWaveLds + row * S::kPitch + ch * 16;
  }
  // A operand: lane holds row m = 32 mi + l32, k = 16 ks + 8 lh + (0..7).
  uint32_t a_off[MI];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = mi * 32 + l32;
    a_off[mi] = m < p.M ? (uint32_t)(((long)m * p.lda + 8 * lh) * 2) : kOutOfRange;
  }
  // transposing read: lane supplies k row 8 lh + r16/4 (+4 for the upper half) and
  // columns 32 j + 16 ((lane>>4)&1) + 4 (r16 % 4); it receives column l32, k = 8 lh + (0..7).
  const int r16 = lane & 15;
  const uint32_t b_rd = w * S::kWaveLds + (8 * lh + (r16 >> 2)) * S::kPitch +
                        (16 * ((lane >> 4) & 1) + 4 * (r16 & 3)) * 2;

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mi][j][r] = 0.f;

  uint4 bq[2][S::kLoads], aq[2][KS][MI];
  auto load = [&](int slot, int s) {
    const uint16_t* Bs = p.B + (long)(kbeg + s * S::kRows) * p.ldb;
    const uint16_t* As = p.A + (kbeg + s * S::kRows);
#pragma unroll
    for (int q = 0; q < S::kLoads; ++q) bq[slot][q] = buffer_load_b128(Bs, b_off[q]);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
        aq[slot][ks][mi] = buffer_load_b128(As + ks * 16, a_off[mi]);
  };
  auto consume = [&](int slot, int s_next) {
#pragma unroll
    for (int q = 0; q < S::kLoads; ++q) lds_write_b128(smem, b_wr[q], bq[slot][q]);
    uint4 af[KS][MI];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) af[ks][mi] = aq[slot][ks][mi];
    __builtin_amdgcn_wave_barrier();
    uint4 bf[KS][NJ];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const char* pb = smem + b_rd + ks * 16 * S::kPitch + j * 64;
        const uint2 lo = lds_read_tr16_b64(pb);
        const uint2 hi = lds_read_tr16_b64(pb + 4 * S::kPitch);
        bf[ks][j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    __builtin_amdgcn_wave_barrier();
    if (s_next < nslices) load(slot, s_next);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) acc[mi][j] = mfma_32x32x16<T>(bf[ks][j], af[ks][mi], acc[mi][j]);
  };

  int s = w;
  if (s < nslices) load(0, s);
  if (s + NW < nslices) load(1, s + NW);
  for (; s + NW < nslices; s += 2 * NW) {
    consume(0, s + 2 * NW);
    consume(1, s + 3 * NW);
  }
  if (s < nslices) consume(0, nslices);

  // ---- sum the waves' partial tiles in a fixed order: wave w += wave w + half ----
  __syncthreads();
  float4* red = reinterpret_cast<float4*>(smem);
  constexpr int Q4 = MI * NJ * 4;                    // float4 groups per lane
#pragma unroll
  for (int half = NW / 2; half >= 1; half >>= 1) {
    if (w >= half && w < 2 * half) {
      float4* dst = red + (size_t)(w - half) * Q4 * 64 + lane;
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            dst[((mi * NJ + j) * 4 + q) * 64] = make_float4(acc[mi][j][4 * q], acc[mi][j][4 * q + 1],
                                                           acc[mi][j][4 * q + 2], acc[mi][j][4 * q + 3]);
    }
    __syncthreads();
    if (w < half) {
      const float4* src = red + (size_t)w * Q4 * 64 + lane;
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float4 v = src[((mi * NJ + j) * 4 + q) * 64];
            acc[mi][j][4 * q] += v.x; acc[mi][j][4 * q + 1] += v.y;
            acc[mi][j][4 * q + 2] += v.z; acc[mi][j][4 * q + 3] += v.w;
          }
    }
    __syncthreads();
  }
  if (w != 0) return;

  // ---- epilogue: through LDS into row order, so that every store instruction
  // writes whole 256-byte (f32) or 128-byte (16-bit) row segments ----
  // acc[mi][j][r]: row m = 32 mi + l32, col n = n0 + 32 j + 8 (r/4) + 4 lh + (r%4).
  constexpr int TP = (S::kCols + 4) * 4;               // tile row pitch in bytes (+16: no bank conflicts)
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t off = (mi * 32 + l32) * TP + (j * 32 + q * 8 + lh * 4) * 4;
        *reinterpret_cast<float4*>(smem + off) = make_float4(acc[mi][j][4 * q], acc[mi][j][4 * q + 1],
                                                             acc[mi][j][4 * q + 2], acc[mi][j][4 * q + 3]);
      }
  __builtin_amdgcn_wave_barrier();
  constexpr int DSZ = EPI == EPI_F32 ? 4 : 2;
  constexpr int LPR = S::kCols / 4;                    // lanes per tile row (four columns each)
  constexpr int RPI = 64 / LPR;                        // rows per store instruction
  char* Db = reinterpret_cast<char*>(p.D) + (long)z * p.strideD * DSZ;
  const int n = n0 + (lane % LPR) * 4;
  float4 bv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (p.bias && n < p.N) bv = *reinterpret_cast<const float4*>(p.bias + n);
#pragma unroll
  for (int i = 0; i < MI * 32 / RPI; ++i) {
    const int m = i * RPI + lane / LPR;
    if (m >= p.M || n >= p.N) continue;                // N % 8 == 0: all-or-nothing per run of 4
    const float4 v = *reinterpret_cast<const float4*>(smem + m * TP + (lane % LPR) * 16);
    float v0 = v.x + bv.x, v1 = v.y + bv.y, v2 = v.z + bv.z, v3 = v.w + bv.w;
    if (p.act != ACT_NONE) {
      v0 = activate(v0, p.act); v1 = activate(v1, p.act);
      v2 = activate(v2, p.act); v3 = activate(v3, p.act);
    }
    char* dst = Db + ((long)m * p.ldd + n) * DSZ;
    if constexpr (EPI == EPI_F32) {
      *reinterpret_cast<float4*>(dst) = make_float4(v0, v1, v2, v3);
    } else {
      uint2 pk;
      pk.x = pack2<T>(v0, v1);
      pk.y = pack2<T>(v2, v3);
      *reinterpret_cast<uint2*>(dst) = pk;
    }
  }
}

}  // namespace tsr950
