// Host-side tile selection and launch for the 16-bit MFMA GEMM family.
#pragma once
#include <algorithm>
#include <mutex>
#include "gemm16.h"
#include "gemm16_skinny.h"
#include "host_util.h"
#include "pitch_copy.h"

namespace tsr950 {

// Any-shape fallback: one thread per output element, f32 accumulate in k order.
// Used when rows are not 16-byte aligned (K or N not a multiple of 8), where the
// vector loads of the MFMA kernel do not apply.
template <class T, int EPI>
__global__ void gemm16_generic_kernel(const Gemm16Params p) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int m = blockIdx.y * blockDim.y + threadIdx.y;
  const int z = blockIdx.z;
  if (m >= p.M || n >= p.N) return;
  const uint16_t* A = p.A + (long)z * p.strideA + (long)m * p.lda;
  const uint16_t* B = p.B + (long)z * p.strideB + n;
  float acc = 0.f;
  for (int k = 0; k < p.K; ++k) acc += from_storage<T>(A[k]) * from_storage<T>(B[(long)k * p.ldb]);
  if constexpr (EPI == EPI_GATED_F32) {
    const uint16_t* B2 = p.B2 + (long)z * p.strideB + n;
    float up = 0.f;
    for (int k = 0; k < p.K; ++k) up += from_storage<T>(A[k]) * from_storage<T>(B2[(long)k * p.ldb]);
    acc = activate(acc, p.act) * up;
  } else {
    if (p.bias) acc += p.bias[n];
    acc = activate(acc, p.act);
  }
  const long o = (long)z * p.strideD + (long)m * p.ldd + n;
  if constexpr (EPI == EPI_F32 || EPI == EPI_GATED_F32) reinterpret_cast<float*>(p.D)[o] = acc;
  else reinterpret_cast<uint16_t*>(p.D)[o] = to_storage<T>(acc);
}

// Grouped any-shape fallback: thread per output element, group found by scan.
template <class T, int EPI>
__global__ void gemm16_grouped_generic_kernel(const Gemm16Params p) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int m = blockIdx.y * blockDim.y + threadIdx.y;
  if (m >= p.M || n >= p.N) return;
  int e = 0;
  while (e + 1 < p.groups && m >= p.offsets[e + 1]) ++e;
  if (m < p.offsets[e] || m >= p.offsets[e + 1]) return;
  const uint16_t* A = p.A + (long)(p.gather ? p.gather[m] : m) * p.lda;
  const uint16_t* B = p.B + (long)e * p.strideB + n;
  float acc = 0.f;
  for (int k = 0; k < p.K; ++k) acc += from_storage<T>(A[k]) * from_storage<T>(B[(long)k * p.ldb]);
  if constexpr (EPI == EPI_SWIGLU16) {
    const uint16_t* B2 = p.B2 + (long)e * p.strideB + n;
    float up = 0.f;
    for (int k = 0; k < p.K; ++k) up += from_storage<T>(A[k]) * from_storage<T>(B2[(long)k * p.ldb]);
    const float gs = from_storage<T>(to_storage<T>(acc));
    const float us = from_storage<T>(to_storage<T>(up));
    acc = (gs / (1.0f + __expf(-gs))) * us;
  }
  const long o = (long)m * p.ldd + n;
  if constexpr (EPI == EPI_F32) reinterpret_cast<float*>(p.D)[o] = acc;
  else reinterpret_cast<uint16_t*>(p.D)[o] = to_storage<T>(acc);
}

// The 256 x 256 workgroup tiles, dense and grouped (per expert), use the 16-wide MFMA in the
// register-staged main loop; the smaller tiles use the 32-wide one.
constexpr int kBigTileMfma = 16;
constexpr int kGroupedTileMfma = 16;

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// wg_limit > 0: only the first wg_limit workgroups of a dense product's tile order are launched
// (the caller serves the remaining tiles itself).
template <class T, int BM, int BN, int WM, int WN, int EPI, bool GROUPED, int MS = 32, bool MID = false>
int launch_gemm16_tile(Gemm16Params p, hipStream_t s, int wg_limit = 0) {
  using S = Gemm16Smem<BM, BN>;
  auto kern = gemm16_kernel<T, BM, BN, WM, WN, EPI, GROUPED, MS, MID>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, S::kBytes);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  constexpr int BN_OUT = (EPI == EPI_SWIGLU16 || EPI == EPI_GATED_F32) ? BN / 2 : BN;
  p.tiles_n = ceil_div(p.N, BN_OUT);
  dim3 grid;
  if constexpr (GROUPED) {
    // every group contributes at most ceil(rows/BM) <= rows/BM + 1 tiles
    // (+8: the kernel deals ceil(real tiles / 8) slots to each of the 8 XCDs)
    p.tiles_m = p.M / BM + p.groups;
    grid = dim3(p.tiles_n * p.tiles_m + 8, 1, 1);
  } else {
    p.tiles_m = ceil_div(p.M, BM);
    grid = dim3(wg_limit > 0 ? wg_limit : p.tiles_m * p.tiles_n, 1, p.groups);
  }
  hipLaunchKernelGGL(kern, grid, dim3(WM * WN * 64), S::kBytes, s, p);
  return launch_status();
}

// D[m][n] = sum over splits (in split order) of the f32 partials, stored as f32 or in
// the storage dtype; four columns per thread (N % 8 == 0 on this path).
template <class T, int EPI>
__global__ void splitk_reduce_kernel(const float* __restrict__ ws, void* __restrict__ D, int M, int N, long ldd,
                                     int splits, const float* __restrict__ bias, int act) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int nq = N / 4;
  if (i >= (long)M * nq) return;
  const int m = (int)(i / nq), n = (int)(i % nq) * 4;
  const size_t mn = (size_t)M * N;
  // (the partials of four splits are fetched together: they were written by other
  // XCDs, so every one of these loads pays a trip to memory)
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int z0 = 0; z0 < splits; z0 += 4) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      v[u] = z0 + u < splits ? *reinterpret_cast<const float4*>(ws + (z0 + u) * mn + (size_t)m * N + n)
                             : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < 4; ++u) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }
  }
  if (bias) {
    const float4 bv = *reinterpret_cast<const float4*>(bias + n);
    acc.x += bv.x; acc.y += bv.y; acc.z += bv.z; acc.w += bv.w;
  }
  acc.x = activate(acc.x, act); acc.y = activate(acc.y, act);
  acc.z = activate(acc.z, act); acc.w = activate(acc.w, act);
  if constexpr (EPI == EPI_F32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(D) + (long)m * ldd + n) = acc;
  } else {
    uint2 pk;
    pk.x = pack2<T>(acc.x, acc.y);
    pk.y = pack2<T>(acc.z, acc.w);
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(D) + (long)m * ldd + n) = pk;
  }
}

// Tile and split-K choice of the dense 16-bit GEMM for an aligned problem — the one
// place the decision lives (the launcher below and the schedule query of the C ABI
// both call it).
struct Gemm16Schedule {
  int tile;      // workgroup tile edge: 256, 128 or 64 (square unless tile_m says otherwise)
  int split_k;   // number of K splits (1 = none)
  bool skinny;   // M <= 8: the streaming kernel (32 x 64 workgroup tile, K slices of 32)
  int rest_split = 1;   // 256 tiles, split_k 1: K splits of the tiles beyond the last full round of 256
  int tile_m = 0;       // 128 with tile 256: the 128 x 256 tile (tile rows x tile columns); 0: square
};
constexpr int kSkinnyMaxM = 8;
constexpr long kSplitTargetWgs = 768;
constexpr int kWeightStreamMaxM = 128;   // up to here a product is bound by reading B once

// Time estimates (microseconds) behind the choice for products with more than kWeightStreamMaxM
// rows, fitted to timings of forced (tile, split) pairs on this part over products from 1024^3
// to 7168^3: a 256 x 256 tile spends 9.6 us outside its K loop and 1.09 us per 64-deep K step
// while at most 144 of the 256 compute units are busy, rising to 1.43 us with all of them busy
// (the board's power limit sets the clock); a 128 x 128 tile 5 us and 0.52 us per step, two
// of them sharing a compute unit at half that rate each (512 run at a time); the sum over K splits reads the f32
// partials and writes the result at about 4.4 TB/s.
inline double est_tiles256_us(long tiles, int ksteps) {
  const long full = tiles / 256, rem = tiles % 256;
  double t = (double)full * (9.6 + ksteps * 1.43);
  if (rem) t += 9.6 + ksteps * (1.09 + 0.34 * std::min(1.0, std::max(0.0, (rem - 144) / 112.0)));
  return t;
}
// (a 128 x 256 tile: 7 us and 0.60 us per step up to about 96 tiles at a time, 0.82 with every
// compute unit busy over several rounds — per FLOP a fifth slower than the 256 x 256 tile, but
// twice as many tiles to fill the chip with; a single partial round of 160 to 255 tiles measured
// 0.83 to 0.93 per step)
inline double est_tiles128x256_us(long tiles, int ksteps) {
  const long full = tiles / 256, rem = tiles % 256;
  double t = (double)full * (7.0 + ksteps * 0.82);
  if (rem) t += 7.0 + ksteps * (0.60 + 0.28 * std::min(1.0, std::max(0.0, (rem - 96) / 64.0)));
  return t;
}
inline double est_tiles128_us(long tiles, int ksteps) {
  return 5.0 * (double)((tiles + 511) / 512) + ksteps * 0.52 * (double)((tiles + 255) / 256);
}
inline double est_split_sum_us(long mn, int splits) {
  return splits > 1 ? 2.0 + (double)mn * (4.0 * splits + 2.0) / 4.4e6 : 0.0;
}

// Time estimate (microseconds) for 33 to 128 rows against a weight matrix that streams from HBM,
// fitted (13 % rms) to timings of forced (tile, split) pairs on this part over 19 weight shapes from
// 2048 x 7168 to 32768 x 4096 with the weights cycled through copies: a launch cost, then the larger
// of the busiest compute unit's K steps (its first workgroup at `step`, every further one sharing
// the unit at `shared` per step) and the time to stream the tile columns of B at `tbs` TB/s, which
// takes about 185 workgroups in flight to reach; a split adds 3.4 us and 1.6 us per million
// partial sums.
struct FewRowTile { int tile_m, tile_n; double launch, step, shared, tbs; };
constexpr FewRowTile kFewRowTiles[3] = {{64, 64, 0.26, 0.514, 0.256, 5.39},
                                        {128, 128, 2.31, 0.345, 0.728, 5.46},
                                        {128, 256, 3.97, 0.693, 1.582, 7.01}};
inline double est_few_rows_us(const FewRowTile& t, int M, int N, int K, int splits) {
  const long wgs = (long)ceil_div(M, t.tile_m) * ceil_div(N, t.tile_n) * splits;
  const double steps = (double)K / G16_BK / splits;
  const double busiest = (double)((wgs + 255) / 256);
  const double compute = steps * (t.step + t.shared * (busiest - 1.0));
  const double bytes = 2.0 * K * ceil_div(N, t.tile_n) * t.tile_n;
  const double stream = bytes / (t.tbs * 1e6 * std::min(1.0, wgs / 185.0));
  const double sum = splits > 1 ? 3.4 + (double)M * N * splits * 1.6e-6 : 0.0;
  return t.launch + std::max(compute, stream) + sum;
}

inline Gemm16Schedule select_gemm16_schedule(int M, int N, int K, int batch) {
  if (batch == 1 && M <= kWeightStreamMaxM && N >= 128) {
    // Few rows under a very wide weight matrix (a vocabulary projection, a fused up projection):
    // tiles enough for three quarters of the compute units without a K split, which would add a
    // pass over the partials and little parallelism.  The wider tile reads 512 contiguous bytes
    // of a row of B instead of 256 and streams faster once it, too, fills the chip.
    if ((long)ceil_div(M, 128) * ceil_div(N, 256) >= 192) return {256, 1, false, 1, 128};
    if ((long)ceil_div(M, 128) * ceil_div(N, 128) >= 192) return {128, 1, false};
  }
  if (batch == 1 && M <= kSkinnyMaxM && K % 32 == 0 && K >= 512) {
    // one workgroup per 64-column strip and K split; about one workgroup per CU, and
    // at least two 32-row slices for each of a workgroup's 8 waves
    const int strips = ceil_div(N, 64);
    int splits = std::max(1, std::min((256 + strips / 2) / strips, K / 512));
    return {64, splits, true};
  }
  if (batch == 1 && M > 32 && M <= kWeightStreamMaxM && N >= 2048 && K >= 1024) {
    // the cheapest of the three small tiles with K in 1 to 16 parts, by the estimate above (below
    // 33 rows the rule further down is as good as the estimate: 1 % apart over the same shapes)
    Gemm16Schedule best{128, 1, false};
    double best_us = 1e30;
    for (const FewRowTile& t : kFewRowTiles)
      for (int splits : {1, 2, 3, 4, 6, 8, 12, 16}) {
        if (K % (splits * G16_BK) != 0 || K / splits < 512) continue;
        const double us = est_few_rows_us(t, M, N, K, splits);
        if (us < best_us) {
          best_us = us;
          best = t.tile_n == 256 ? Gemm16Schedule{256, splits, false, 1, 128} : Gemm16Schedule{t.tile_m, splits, false};
        }
      }
    return best;
  }
  const long tiles256 = (long)ceil_div(M, 256) * ceil_div(N, 256) * batch;
  const long tiles128 = (long)ceil_div(M, 128) * ceil_div(N, 128) * batch;
  if (M > kWeightStreamMaxM && N >= 128) {
    // the cheapest of: either tile, K in 1, 2, 3, 4 or 8 parts (a single product only; every
    // part a whole number of K steps and at least 512 deep)
    const int ksteps = ceil_div(K, G16_BK);
    Gemm16Schedule best{256, 1, false};
    double best_us = est_tiles256_us(tiles256, ksteps);
    auto consider = [&](int tile, int splits, double us) {
      if (us < best_us) { best_us = us; best = Gemm16Schedule{tile, splits, false}; }
    };
    consider(128, 1, est_tiles128_us(tiles128, ksteps));
    {
      // (its estimate is the least certain of the three — the per-step figure moved by 13 % between
      // shapes of equal tile count — so it has to win by a margin)
      const double us = 1.06 * est_tiles128x256_us((long)ceil_div(M, 128) * ceil_div(N, 256) * batch, ksteps);
      if (us < best_us) { best_us = us; best = Gemm16Schedule{256, 1, false, 1, 128}; }
    }
    if (batch == 1) {
      for (int splits : {2, 3, 4, 8}) {
        if (K % (splits * G16_BK) != 0 || K / splits < 512) continue;
        const double sum_us = est_split_sum_us((long)M * N, splits);
        consider(256, splits, est_tiles256_us(tiles256 * splits, ksteps / splits) + sum_us);
        consider(128, splits, est_tiles128_us(tiles128 * splits, ksteps / splits) + sum_us);
      }
    }
    // A tile count a little over a multiple of 256 leaves a last round with most compute units
    // idle: those tiles can be split along K among them (one more launch and a sum over the
    // partial tiles).
    const long full = tiles256 / 256, rest = tiles256 % 256;
    if (batch == 1 && full >= 1 && rest > 0 && rest <= 128) {
      const double main_us = (double)full * (9.6 + ksteps * 1.43);
      for (int splits : {2, 3, 4, 6, 8, 12, 16}) {
        const int per = ceil_div(ksteps, splits);
        if (rest * splits > 256 || per < 2 || (long)per * (splits - 1) >= ksteps) continue;
        const double us = main_us + 3.0 + est_tiles256_us(rest * splits, per) +
                          est_split_sum_us(rest * 65536L, splits);
        if (us < best_us) { best_us = us; best = Gemm16Schedule{256, 1, false, splits}; }
      }
    }
    return best;
  }
  // Few rows: the weight matrix streams from HBM once and the tiles are small; for a single
  // product with few tiles and a long K, K is split over about 768 workgroups.
  if (tiles256 >= 192) return {256, 1, false};
  const bool t128 = tiles128 >= 192 || (M > 64 && N >= 128);
  int splits = 1;
  if (batch == 1) {
    const long tiles = t128 ? tiles128 : (long)ceil_div(M, 64) * ceil_div(N, 64);
    splits = (int)std::max<long>(1, std::min<long>((kSplitTargetWgs + tiles - 1) / tiles, K / 512));
    // the f32 partials are written and read once per split (8 M N splits bytes against
    // 2 K (M + N) bytes of operands: B dominates under few rows, A over few columns): beyond two
    // splits keep that under about 0.4 of the operand traffic
    splits = (int)std::min<long>(splits, std::max<long>(2, (long)K * (M + N) / (10L * M * N)));
    while (splits > 1 && K % (splits * G16_BK) != 0) --splits;
  }
  return {t128 ? 128 : 64, splits, false};
}

template <class T, int EPI>
int launch_gemm16_skinny(const Gemm16Params& p, int kps, int splits, hipStream_t s) {
  constexpr int MI = 1, NW = 8, NJ = 2, KS = 2;
  auto kern = gemm16_skinny_kernel<T, MI, NW, NJ, KS, EPI>;
  constexpr int lds = skinny_lds_bytes<MI, NW, NJ, KS>();
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  hipLaunchKernelGGL(kern, dim3(ceil_div(p.N, 32 * NJ), splits), dim3(NW * 64), lds, s, p, kps);
  return launch_status();
}

template <class T, int EPI>
int launch_gemm16(Gemm16Params p, hipStream_t s);

// A product whose operands the tile kernels cannot load as they are (K, N or a pitch not a
// multiple of 8 elements, or a pointer off a 16-byte boundary): the offending operands are
// copied into aligned, zero-padded buffers (K and N rounded up to multiples of 8: zero columns
// of A, zero rows and columns of B), the tile kernels run on those, and the leading N columns
// of the result are copied out.  The buffers live from here to the end of this call's work on
// the stream (stream-ordered allocation).
template <class T, int EPI>
int launch_gemm16_repitched(const Gemm16Params& p, hipStream_t s) {
  constexpr int dsz = (EPI == EPI_F32) ? 4 : 2;
  const int K8 = (p.K + 7) & ~7, N8 = (p.N + 7) & ~7, G = p.groups;
  const bool a_ok = p.K % 8 == 0 && p.lda % 8 == 0 && p.strideA % 8 == 0 && aligned16(p.A) && p.lda < (1L << 21);
  const bool b_ok = p.K % 8 == 0 && p.N % 8 == 0 && p.ldb % 8 == 0 && p.strideB % 8 == 0 && aligned16(p.B) &&
                    p.ldb < (1L << 21);
  const bool d_ok = p.N % 8 == 0 && (p.ldd * dsz) % 16 == 0 && (p.strideD * dsz) % 16 == 0 && aligned16(p.D);
  const bool bias_ok = !p.bias || (p.N % 8 == 0 && aligned16(p.bias));
  const size_t a_bytes = a_ok ? 0 : (size_t)G * p.M * K8 * 2, b_bytes = b_ok ? 0 : (size_t)G * K8 * N8 * 2;
  const size_t d_bytes = d_ok ? 0 : (size_t)G * p.M * N8 * dsz, bias_bytes = bias_ok ? 0 : (size_t)N8 * 4;
  char* ws = nullptr;
  if (hipMallocAsync(reinterpret_cast<void**>(&ws), a_bytes + b_bytes + d_bytes + bias_bytes + 16, s) != hipSuccess) {
    (void)hipGetLastError();
    return kDeviceFailed;
  }
  Gemm16Params q = p;
  q.K = K8;
  q.N = N8;
  char* at = ws;
  if (!a_ok) {
    uint16_t* a2 = reinterpret_cast<uint16_t*>(at);
    at += a_bytes;
    hipLaunchKernelGGL(pad_rows_kernel<uint16_t>, copy_grid(p.M, K8, 8, G), copy_block(), 0, s, a2, (long)K8,
                       (long)p.M * K8, p.A, p.lda, p.strideA, p.M, p.K, p.M);
    q.A = a2; q.lda = K8; q.strideA = (long)p.M * K8;
  }
  if (!b_ok) {
    uint16_t* b2 = reinterpret_cast<uint16_t*>(at);
    at += b_bytes;
    hipLaunchKernelGGL(pad_rows_kernel<uint16_t>, copy_grid(K8, N8, 8, G), copy_block(), 0, s, b2, (long)N8,
                       (long)K8 * N8, p.B, p.ldb, p.strideB, p.K, p.N, K8);
    q.B = b2; q.ldb = N8; q.strideB = (long)K8 * N8;
  }
  void* d2 = nullptr;
  if (!d_ok) {
    d2 = at;
    at += d_bytes;
    q.D = d2; q.ldd = N8; q.strideD = (long)p.M * N8;
  }
  if (!bias_ok) {
    float* bias2 = reinterpret_cast<float*>(at);
    hipLaunchKernelGGL(pad_rows_kernel<float>, copy_grid(1, N8, 4, 1), copy_block(), 0, s, bias2, (long)N8, (long)N8,
                       p.bias, (long)p.N, (long)p.N, 1, p.N, 1);
    q.bias = bias2;
  }
  int rc = launch_status();
  if (rc == kOk) rc = launch_gemm16<T, EPI>(q, s);
  if (rc == kOk && !d_ok) {
    if constexpr (dsz == 4)
      hipLaunchKernelGGL(unpad_rows_kernel<float>, copy_grid(p.M, N8, 4, G), copy_block(), 0, s, static_cast<float*>(p.D),
                         p.ldd, p.strideD, static_cast<const float*>(d2), (long)N8, (long)p.M * N8, p.M, p.N);
    else
      hipLaunchKernelGGL(unpad_rows_kernel<uint16_t>, copy_grid(p.M, N8, 8, G), copy_block(), 0, s,
                         static_cast<uint16_t*>(p.D), p.ldd, p.strideD, static_cast<const uint16_t*>(d2), (long)N8,
                         (long)p.M * N8, p.M, p.N);
    rc = launch_status();
  }
  if (hipFreeAsync(ws, s) != hipSuccess) { (void)hipGetLastError(); rc = rc == kOk ? kDeviceFailed : rc; }
  return rc;
}

// The tiles first_tile .. first_tile + rest - 1 of a dense product on 256 x 256 tiles, each split
// along K over `splits` workgroups, then summed (with the bias / activation of the product).
template <class T, int EPI>
int launch_gemm16_rest(Gemm16Params p, int first_tile, int rest, int splits, hipStream_t s) {
  using S = Gemm16Smem<256, 256>;
  auto kern = gemm16_rest_splitk_kernel<T, kBigTileMfma>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, S::kBytes);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  float* ws = static_cast<float*>(stream_workspace(s, (size_t)rest * splits * 256 * 256 * sizeof(float)));
  if (!ws) return kDeviceFailed;
  p.tiles_m = ceil_div(p.M, 256);
  p.tiles_n = ceil_div(p.N, 256);
  const int ksplit = ceil_div(ceil_div(p.K, G16_BK), splits) * G16_BK;
  hipLaunchKernelGGL(kern, dim3(rest, splits), dim3(256), S::kBytes, s, p, first_tile, ksplit, ws);
  if (int rc = launch_status(); rc != kOk) return rc;
  hipLaunchKernelGGL((gemm16_rest_sum_kernel<T, EPI>), dim3(64, rest), dim3(256), 0, s, ws, p.D, p.M, p.N, p.ldd,
                     p.tiles_m, p.tiles_n, first_tile, splits, p.bias, p.act);
  return launch_status();
}

// Dense / batched.  p.groups = batch count (>= 1).
template <class T, int EPI>
int launch_gemm16(Gemm16Params p, hipStream_t s) {
  const int dsz = (EPI == EPI_F32) ? 4 : 2;
  // (32-bit per-lane byte offsets inside a tile bound the leading dimensions)
  const bool vec = (p.K % 8 == 0) && (p.N % 8 == 0) && (p.lda % 8 == 0) && (p.ldb % 8 == 0) &&
                   (p.lda < (1L << 21)) && (p.ldb < (1L << 21)) &&
                   ((p.ldd * dsz) % 16 == 0) && (p.strideA % 8 == 0) && (p.strideB % 8 == 0) &&
                   ((p.strideD * dsz) % 16 == 0) && aligned16(p.A) && aligned16(p.B) && aligned16(p.D) &&
                   (!p.bias || aligned16(p.bias));
  if (!vec) {
    // small products go one thread per output element; above about 2^24 multiply-adds the
    // copies into aligned buffers cost less than that kernel loses
    if ((double)p.M * p.N * p.K * p.groups >= (double)(1L << 24) && p.M >= 16 && p.N >= 16 &&
        p.K + 8 < (1L << 21) && p.N + 8 < (1L << 21))
      return launch_gemm16_repitched<T, EPI>(p, s);
    dim3 block(32, 8), grid(ceil_div(p.N, 32), ceil_div(p.M, 8), p.groups);
    hipLaunchKernelGGL((gemm16_generic_kernel<T, EPI>), grid, block, 0, s, p);
    return launch_status();
  }
  const Gemm16Schedule sch = select_gemm16_schedule(p.M, p.N, p.K, p.groups);
  // bias / activation: the tile kernels have a separate instantiation for it (f32 out)
  const bool fused = p.bias != nullptr || p.act != ACT_NONE;
  if constexpr (EPI != EPI_F32) {
    if (fused) return kBadShape;
  }
  if (sch.tile == 256 && sch.tile_m == 128 && sch.split_k == 1) {
    if constexpr (EPI == EPI_F32) {
      if (fused) return launch_gemm16_tile<T, 128, 256, 2, 2, EPI_F32_FUSED, false, kBigTileMfma>(p, s);
    }
    return launch_gemm16_tile<T, 128, 256, 2, 2, EPI, false, kBigTileMfma>(p, s);
  }
  if (sch.tile == 256 && sch.split_k == 1) {
    const int tiles = ceil_div(p.M, 256) * ceil_div(p.N, 256);
    const int main_wgs = sch.rest_split > 1 ? tiles / 256 * 256 : 0;     // 0: every tile in one launch
    int rc = kOk;
    if (EPI == EPI_F32 && fused) {
      if constexpr (EPI == EPI_F32)
        rc = launch_gemm16_tile<T, 256, 256, 2, 2, EPI_F32_FUSED, false, kBigTileMfma>(p, s, main_wgs);
    } else {
      rc = launch_gemm16_tile<T, 256, 256, 2, 2, EPI, false, kBigTileMfma>(p, s, main_wgs);
    }
    if (rc != kOk || sch.rest_split <= 1) return rc;
    return launch_gemm16_rest<T, EPI>(p, main_wgs, tiles - main_wgs, sch.rest_split, s);
  }
  const bool t128 = sch.tile == 128;
  if (sch.skinny && sch.split_k == 1) return launch_gemm16_skinny<T, EPI>(p, p.K, 1, s);
  // Every K split is one "batch" of the same kernel writing f32 partials, summed in
  // split order by a second kernel, so the result does not depend on scheduling.
  {
    const int splits = sch.split_k;
    if (splits > 1) {
      const size_t mn = (size_t)p.M * p.N;
      float* ws = static_cast<float*>(stream_workspace(s, mn * splits * sizeof(float)));
      if (!ws) return kDeviceFailed;
      Gemm16Params q = p;
      q.K = p.K / splits;
      q.groups = splits;
      q.strideA = q.K;                       // split z reads A[:, z Ks ..) and B[z Ks .., :)
      q.strideB = (long)q.K * p.ldb;
      q.D = ws;
      q.bias = nullptr;                      // the epilogue runs once, on the summed partials
      q.act = ACT_NONE;
      q.ldd = p.N;
      q.strideD = (long)mn;
      int rc;
      if (sch.skinny) {
        // the skinny kernel takes the whole problem and splits K by blockIdx.y itself
        q.K = p.K;
        rc = launch_gemm16_skinny<T, EPI_F32>(q, ceil_div(ceil_div(p.K, splits), 32) * 32, splits, s);
      } else {
        rc = sch.tile == 256 && sch.tile_m == 128 ? launch_gemm16_tile<T, 128, 256, 2, 2, EPI_F32, false, kBigTileMfma>(q, s)
             : sch.tile == 256 ? launch_gemm16_tile<T, 256, 256, 2, 2, EPI_F32, false, kBigTileMfma>(q, s)
             : t128      ? launch_gemm16_tile<T, 128, 128, 2, 2, EPI_F32, false>(q, s)
                         : launch_gemm16_tile<T, 64, 64, 2, 2, EPI_F32, false>(q, s);
      }
      if (rc == kOk) {
        const long quads = (long)p.M * (p.N / 4);
        hipLaunchKernelGGL((splitk_reduce_kernel<T, EPI>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s,
                           ws, p.D, p.M, p.N, p.ldd, splits, p.bias, p.act);
        rc = launch_status();
      }
      return rc;
    }
  }
  if constexpr (EPI == EPI_F32) {
    if (fused) {
      if (t128) return launch_gemm16_tile<T, 128, 128, 2, 2, EPI_F32_FUSED, false>(p, s);
      return launch_gemm16_tile<T, 64, 64, 2, 2, EPI_F32_FUSED, false>(p, s);
    }
  }
  if (t128) return launch_gemm16_tile<T, 128, 128, 2, 2, EPI, false>(p, s);
  return launch_gemm16_tile<T, 64, 64, 2, 2, EPI, false>(p, s);
}

// D[i] = act(G[i]) * U[i], four elements per thread (n % 4 == 0, 16-byte aligned pointers).
template <int ACT_DYNAMIC = 1>   // (a template so that every translation unit may include this header)
__global__ __launch_bounds__(256) void gate_mul_kernel(float* __restrict__ D, const float* __restrict__ G,
                                                       const float* __restrict__ U, long n4, int act) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const float4 g = reinterpret_cast<const float4*>(G)[i], u = reinterpret_cast<const float4*>(U)[i];
  reinterpret_cast<float4*>(D)[i] =
      make_float4(activate(g.x, act) * u.x, activate(g.y, act) * u.y, activate(g.z, act) * u.z, activate(g.w, act) * u.w);
}

// Dense gated product D f32 = act(A Wg) * (A Wu); p.B = Wg, p.B2 = Wu, p.N = H.
template <class T>
int launch_gemm16_gated(Gemm16Params p, hipStream_t s) {
  // Few rows: both products are bound by reading their weight matrix once, which the dense
  // launcher's decode schedules (small tiles, K split over the chip) do at several times the rate
  // of one 256-row tile per 128 output columns.  Two products into stream-ordered scratch, then
  // the gate.
  if (p.M <= kWeightStreamMaxM && p.N % 8 == 0 && p.K % 8 == 0 && p.ldd == p.N && aligned16(p.D) &&
      (long)p.M * p.N >= 128L * 128L) {
    const size_t mn = (size_t)p.M * p.N;
    float* tmp = nullptr;
    if (hipMallocAsync(reinterpret_cast<void**>(&tmp), 2 * mn * sizeof(float), s) != hipSuccess) {
      (void)hipGetLastError();
      return kDeviceFailed;
    }
    Gemm16Params q = p;
    q.B2 = nullptr;
    q.act = ACT_NONE;
    q.bias = nullptr;
    q.groups = 1;
    q.strideA = q.strideB = q.strideD = 0;
    q.D = tmp;
    int rc = launch_gemm16<T, EPI_F32>(q, s);
    if (rc == kOk) {
      q.B = p.B2;
      q.D = tmp + mn;
      rc = launch_gemm16<T, EPI_F32>(q, s);
    }
    if (rc == kOk) {
      hipLaunchKernelGGL(gate_mul_kernel<1>, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, s,
                         static_cast<float*>(p.D), tmp, tmp + mn, (long)(mn / 4), p.act);
      rc = launch_status();
    }
    if (hipFreeAsync(tmp, s) != hipSuccess) { (void)hipGetLastError(); rc = rc == kOk ? kDeviceFailed : rc; }
    return rc;
  }
  const bool vec = (p.K % 8 == 0) && (p.N % 8 == 0) && (p.lda % 8 == 0) && (p.ldb % 8 == 0) &&
                   (p.lda < (1L << 21)) && (p.ldb < (1L << 21)) && (p.ldd % 4 == 0) && aligned16(p.A) &&
                   aligned16(p.B) && aligned16(p.B2) && aligned16(p.D);
  if (!vec || (long)p.M * p.N < 128L * 128L) {
    dim3 block(32, 8), grid(ceil_div(p.N, 32), ceil_div(p.M, 8), 1);
    hipLaunchKernelGGL((gemm16_generic_kernel<T, EPI_GATED_F32>), grid, block, 0, s, p);
    return launch_status();
  }
  return launch_gemm16_tile<T, 256, 256, 4, 1, EPI_GATED_F32, false, kBigTileMfma>(p, s);
}

// Grouped.  p.M = total rows S, p.groups = E, p.offsets = device int32[E+1].
template <class T, int EPI>
int launch_gemm16_grouped(Gemm16Params p, hipStream_t s) {
  const int dsz = (EPI == EPI_F32) ? 4 : 2;
  // (32-bit per-lane byte offsets inside a tile bound the leading dimensions)
  const bool vec = (p.K % 8 == 0) && (p.N % 8 == 0) && (p.lda % 8 == 0) && (p.ldb % 8 == 0) &&
                   (p.lda < (1L << 21)) && (p.ldb < (1L << 21)) &&
                   ((p.ldd * dsz) % 16 == 0) && (p.strideB % 8 == 0) && aligned16(p.A) &&
                   aligned16(p.B) && aligned16(p.D) && (EPI != EPI_SWIGLU16 || aligned16(p.B2));
  if (!vec) {
    dim3 block(32, 8), grid(ceil_div(p.N, 32), ceil_div(p.M, 8), 1);
    hipLaunchKernelGGL((gemm16_grouped_generic_kernel<T, EPI>), grid, block, 0, s, p);
    return launch_status();
  }
  // groups that average at most a tile of rows (a chunk of a thousand tokens over 64 experts): the
  // instantiation whose last row tile also comes in a 128-row form
  const bool mid = (long)p.M <= 256L * p.groups;
  if constexpr (EPI == EPI_SWIGLU16) {
    if (mid) return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, true, kGroupedTileMfma, true>(p, s);
    return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, true, kGroupedTileMfma>(p, s);
  } else {
    if ((long)p.M < 64L * p.groups) return launch_gemm16_tile<T, 128, 128, 2, 2, EPI, true>(p, s);
    if (mid) return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, true, kGroupedTileMfma, true>(p, s);
    return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, true, kGroupedTileMfma>(p, s);
  }
}

}  // namespace tsr950
