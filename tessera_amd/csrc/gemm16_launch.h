// Host-side tile selection and launch for the 16-bit MFMA GEMM family.
#pragma once
#include <algorithm>
#include <mutex>
#include "gemm16.h"
#include "gemm16_skinny.h"
#include "host_util.h"

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

template <class T, int BM, int BN, int WM, int WN, int EPI, bool GROUPED, int MS = 32>
int launch_gemm16_tile(Gemm16Params p, hipStream_t s) {
  using S = Gemm16Smem<BM, BN>;
  auto kern = gemm16_kernel<T, BM, BN, WM, WN, EPI, GROUPED, MS>;
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
    grid = dim3(p.tiles_m * p.tiles_n, 1, p.groups);
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
// both call it).  256x256 when that alone fills the chip; else 128x128 or 64x64
// tiles, and for a single product with few tiles and a long K (decode-shaped: the
// weight matrix streams from HBM once) K is split over about 768 workgroups.
struct Gemm16Schedule {
  int tile;      // square workgroup tile edge: 256, 128 or 64
  int split_k;   // number of K splits (1 = none)
  bool skinny;   // M <= 8: the streaming kernel (32 x 64 workgroup tile, K slices of 32)
};
constexpr int kSkinnyMaxM = 8;
constexpr long kSplitTargetWgs = 768;
inline Gemm16Schedule select_gemm16_schedule(int M, int N, int K, int batch) {
  if (batch == 1 && M <= kSkinnyMaxM && K % 32 == 0 && K >= 512) {
    // one workgroup per 64-column strip and K split; about one workgroup per CU, and
    // at least two 32-row slices for each of a workgroup's 8 waves
    const int strips = ceil_div(N, 64);
    int splits = std::max(1, std::min((256 + strips / 2) / strips, K / 512));
    return {64, splits, true};
  }
  const long tiles256 = (long)ceil_div(M, 256) * ceil_div(N, 256) * batch;
  const long tiles128 = (long)ceil_div(M, 128) * ceil_div(N, 128) * batch;
  if (tiles256 >= 192) return {256, 1, false};
  const bool t128 = tiles128 >= 192 || (M > 64 && N >= 128);
  int splits = 1;
  if (batch == 1) {
    const long tiles = t128 ? tiles128 : (long)ceil_div(M, 64) * ceil_div(N, 64);
    splits = (int)std::max<long>(1, std::min<long>((kSplitTargetWgs + tiles - 1) / tiles, K / 512));
    // the f32 partials are written and read once per split (8 M N splits bytes against
    // 2 K N bytes of B): beyond two splits keep that under about 0.4 of the weight traffic
    splits = (int)std::min<long>(splits, std::max<long>(2, K / (10L * M)));
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
  if (sch.tile == 256) {
    if constexpr (EPI == EPI_F32) {
      if (fused) return launch_gemm16_tile<T, 256, 256, 2, 2, EPI_F32_FUSED, false, kBigTileMfma>(p, s);
    }
    return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, false, kBigTileMfma>(p, s);
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
        rc = t128 ? launch_gemm16_tile<T, 128, 128, 2, 2, EPI_F32, false>(q, s)
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

// Dense gated product D f32 = act(A Wg) * (A Wu); p.B = Wg, p.B2 = Wu, p.N = H.
template <class T>
int launch_gemm16_gated(Gemm16Params p, hipStream_t s) {
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
  if constexpr (EPI == EPI_SWIGLU16) {
    return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, true, kGroupedTileMfma>(p, s);
  } else {
    if ((long)p.M >= 64L * p.groups) return launch_gemm16_tile<T, 256, 256, 2, 2, EPI, true, kGroupedTileMfma>(p, s);
    return launch_gemm16_tile<T, 128, 128, 2, 2, EPI, true>(p, s);
  }
}

}  // namespace tsr950
