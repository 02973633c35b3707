// C ABI: quantised GEMMs (int8 -> int32, W8A8 with scales, fp8 e4m3 with
// per-tensor scales) and the quantisers that produce their operands.
#include <cmath>
#include <mutex>
#include "../../include/tessera_gfx950.h"
#include "gemm8.h"
#include "gemm8_skinny.h"
#include "gemm8_schedule.h"
#include "host_util.h"
#include "pitch_copy.h"

namespace tsr950 {
namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// The tile kernel needs more dynamic LDS than the default limit: raised once per instantiation.
template <class T, int EPI, int BM = G8_BM>
int gemm8_attr() {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_kernel<T, EPI, BM>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, g8_smem(BM));
  });
  return attr_err == hipSuccess ? kOk : kDeviceFailed;
}

template <class T, int EPI>
int gemm8_dev(Gemm8Params p, hipStream_t s);

// K or N not a multiple of 16, or a pointer off a 16-byte boundary: the operands concerned are
// copied into aligned buffers with K and N rounded up to multiples of 16 (zero columns of A, zero
// rows and columns of B: they add exact zeros), the tile kernel runs on those, and the leading N
// columns of the results are copied out.  Stream-ordered scratch.
template <class T, int EPI>
int gemm8_repitched(const Gemm8Params& p, hipStream_t s) {
  constexpr int dsz = EPI == EPI8_SCALED_BF16 ? 2 : 4;
  const int K16 = (p.K + 15) & ~15, N16 = (p.N + 15) & ~15;
  const bool a_ok = p.K % 16 == 0 && aligned16(p.A);
  const bool b_ok = p.K % 16 == 0 && p.N % 16 == 0 && aligned16(p.B);
  const bool d_ok = p.N % 16 == 0 && aligned16(p.D);
  const bool acc_ok = !p.acc_out || (p.N % 16 == 0 && aligned16(p.acc_out));
  const bool cs_ok = !p.col_scale || (p.N % 16 == 0 && aligned16(p.col_scale));
  const size_t a_bytes = a_ok ? 0 : (size_t)p.M * K16, b_bytes = b_ok ? 0 : (size_t)K16 * N16;
  const size_t d_bytes = d_ok ? 0 : (size_t)p.M * N16 * dsz, acc_bytes = acc_ok ? 0 : (size_t)p.M * N16 * 4;
  const size_t cs_bytes = cs_ok ? 0 : (size_t)N16 * 4;
  char* ws = nullptr;
  if (hipMallocAsync(reinterpret_cast<void**>(&ws), a_bytes + b_bytes + d_bytes + acc_bytes + cs_bytes + 16, s) != hipSuccess) {
    (void)hipGetLastError();
    return kDeviceFailed;
  }
  Gemm8Params q = p;
  q.K = K16;
  q.N = N16;
  char* at = ws;
  if (!a_ok) {
    hipLaunchKernelGGL(pad_rows_kernel<uint8_t>, copy_grid(p.M, K16, 16, 1), copy_block(), 0, s, reinterpret_cast<uint8_t*>(at),
                       (long)K16, 0L, p.A, (long)p.K, 0L, p.M, p.K, p.M);
    q.A = reinterpret_cast<const uint8_t*>(at);
    at += a_bytes;
  }
  if (!b_ok) {
    hipLaunchKernelGGL(pad_rows_kernel<uint8_t>, copy_grid(K16, N16, 16, 1), copy_block(), 0, s, reinterpret_cast<uint8_t*>(at),
                       (long)N16, 0L, p.B, (long)p.N, 0L, p.K, p.N, K16);
    q.B = reinterpret_cast<const uint8_t*>(at);
    at += b_bytes;
  }
  void* d2 = nullptr;
  if (!d_ok) { d2 = at; q.D = d2; at += d_bytes; }
  int32_t* acc2 = nullptr;
  if (!acc_ok) { acc2 = reinterpret_cast<int32_t*>(at); q.acc_out = acc2; at += acc_bytes; }
  if (!cs_ok) {
    hipLaunchKernelGGL(pad_rows_kernel<float>, copy_grid(1, N16, 4, 1), copy_block(), 0, s, reinterpret_cast<float*>(at),
                       (long)N16, 0L, p.col_scale, (long)p.N, 0L, 1, p.N, 1);
    q.col_scale = reinterpret_cast<const float*>(at);
  }
  int rc = launch_status();
  if (rc == kOk) rc = gemm8_dev<T, EPI>(q, s);
  if (rc == kOk && !d_ok) {
    if constexpr (dsz == 4)
      hipLaunchKernelGGL(unpad_rows_kernel<uint32_t>, copy_grid(p.M, N16, 4, 1), copy_block(), 0, s, static_cast<uint32_t*>(p.D),
                         (long)p.N, 0L, static_cast<const uint32_t*>(d2), (long)N16, 0L, p.M, p.N);
    else
      hipLaunchKernelGGL(unpad_rows_kernel<uint16_t>, copy_grid(p.M, N16, 8, 1), copy_block(), 0, s, static_cast<uint16_t*>(p.D),
                         (long)p.N, 0L, static_cast<const uint16_t*>(d2), (long)N16, 0L, p.M, p.N);
    rc = launch_status();
  }
  if (rc == kOk && !acc_ok) {
    hipLaunchKernelGGL(unpad_rows_kernel<int32_t>, copy_grid(p.M, N16, 4, 1), copy_block(), 0, s, p.acc_out, (long)p.N, 0L,
                       static_cast<const int32_t*>(acc2), (long)N16, 0L, p.M, p.N);
    rc = launch_status();
  }
  if (hipFreeAsync(ws, s) != hipSuccess) { (void)hipGetLastError(); rc = rc == kOk ? kDeviceFailed : rc; }
  return rc;
}

template <class T, int EPI>
int gemm8_dev(Gemm8Params p, hipStream_t s) {
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || !p.A || !p.B || !p.D) return kBadShape;
  if (EPI == EPI8_W8A8_F32 && (!p.row_scale || !p.col_scale)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  // (32-bit per-lane byte offsets inside a tile bound K and N)
  const bool vec = (p.K % 16 == 0) && (p.N % 16 == 0) && (p.K < (1 << 22)) && (p.N < (1 << 22)) && aligned16(p.A) && aligned16(p.B) && aligned16(p.D) &&
                   (!p.acc_out || aligned16(p.acc_out)) && (!p.col_scale || aligned16(p.col_scale));
  if (!vec) {
    // small products go one thread per output element; above about 2^24 multiply-adds the copies
    // into aligned, zero-padded buffers cost less than that kernel loses
    if ((double)p.M * p.N * p.K >= (double)(1L << 24) && p.M >= 16 && p.N >= 16 && p.K + 16 < (1 << 22) && p.N + 16 < (1 << 22))
      return gemm8_repitched<T, EPI>(p, s);
    dim3 block(32, 8), grid(ceil_div(p.N, 32), ceil_div(p.M, 8), 1);
    hipLaunchKernelGGL((gemm8_generic_kernel<T, EPI>), grid, block, 0, s, p);
    return launch_status();
  }
  const Gemm8Schedule sch = select_gemm8_schedule(p.M, p.N, p.K);
  if (sch.skinny) {
    // (8 waves and about 256 workgroups measured best for up to 32 rows: 4-wave workgroups, two per
    // compute unit, and 384 or 512 workgroups were level or slower on M = 1 ... 32 against 4096 ...
    // 28672 columns.  33 to 64 rows double the accumulators: 4 waves, one per SIMD.)
    const int nw = p.M <= 32 ? 8 : 4;
    const int smem = p.M <= 32 ? g8s_smem(8, 1) : g8s_smem(4, 2);
    const void* kern = p.M <= 32 ? reinterpret_cast<const void*>(gemm8_skinny_kernel<T, 8, 1>)
                                 : reinterpret_cast<const void*>(gemm8_skinny_kernel<T, 4, 2>);
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
      attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_skinny_kernel<T, 8, 1>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, g8s_smem(8, 1));
      if (attr_err == hipSuccess)
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_skinny_kernel<T, 4, 2>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, g8s_smem(4, 2));
    });
    if (attr_err != hipSuccess) return kDeviceFailed;
    const int strips = ceil_div(p.N, G8S_COLS);
    const int splits = sch.split_k;
    const int kps = ceil_div(ceil_div(p.K, splits), G8S_ROWS) * G8S_ROWS;
    void* ws = stream_workspace(s, (size_t)splits * p.M * p.N * 4);
    if (!ws) return kDeviceFailed;
    void* args[] = {(void*)&p.A, (void*)&p.B, (void*)&ws, (void*)&p.M, (void*)&p.N, (void*)&p.K, (void*)&kps};
    if (hipLaunchKernel(kern, dim3(strips, splits), dim3(nw * 64), args, smem, s) != hipSuccess) {
      (void)hipGetLastError();
      return kDeviceFailed;
    }
    const long quads = (long)p.M * (p.N / 4);
    hipLaunchKernelGGL((gemm8_split_sum_kernel<T, EPI>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, ws,
                       splits, p);
    return launch_status();
  }
  const int bm = sch.tile_m, splits = sch.split_k;
  p.tiles_m = ceil_div(p.M, bm);
  p.tiles_n = ceil_div(p.N, G8_BN);
  p.ksplit = 0;
  const int tiles = p.tiles_m * p.tiles_n;
  auto launch = [&](auto bm_c) -> int {
    constexpr int BM = decltype(bm_c)::value;
    if (splits > 1) {
      // raw accumulators: int32 for int8 operands, f32 with unit scales for fp8
      constexpr int RAW_EPI = std::is_same<T, I8>::value ? EPI8_I32 : EPI8_SCALED_F32;
      if (int rc = gemm8_attr<T, RAW_EPI, BM>(); rc != kOk) return rc;
      void* ws = stream_workspace(s, (size_t)splits * p.M * p.N * 4);
      if (!ws) return kDeviceFailed;
      Gemm8Params q = p;
      q.D = ws;
      q.acc_out = nullptr;
      q.scale_a = q.scale_b = 1.f;
      q.ksplit = ceil_div(ceil_div(p.K, G8_BK), splits) * G8_BK;
      hipLaunchKernelGGL((gemm8_kernel<T, RAW_EPI, BM>), dim3(tiles, splits), dim3(256), g8_smem(BM), s, q);
      if (int rc = launch_status(); rc != kOk) return rc;
      const long quads = (long)p.M * (p.N / 4);
      hipLaunchKernelGGL((gemm8_split_sum_kernel<T, EPI>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, ws,
                         splits, p);
      return launch_status();
    }
    if (int rc = gemm8_attr<T, EPI, BM>(); rc != kOk) return rc;
    hipLaunchKernelGGL((gemm8_kernel<T, EPI, BM>), dim3(tiles), dim3(256), g8_smem(BM), s, p);
    return launch_status();
  };
  return bm == 256 ? launch(std::integral_constant<int, 256>{}) : launch(std::integral_constant<int, 128>{});
}

// ---- quantisers ---------------------------------------------------------------

__device__ __forceinline__ float warp_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Workgroup-wide max of |x| folded into *out with one atomic max on the bit pattern
// (valid for non-negative floats).
// (x 16-byte aligned: the body runs on float4, the last n % 4 elements one by one)
__global__ void absmax_kernel(const float* x, long n, unsigned* out) {
  float m = 0.f;
  const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x, nthreads = (long)gridDim.x * blockDim.x;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  const long n4 = vec ? n / 4 : 0;
  auto fold = [&](const float4& v) {
    m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
  };
  // four independent 16-byte loads in flight per thread (one per trip left the memory
  // system at a third of its rate)
  const float4* x4 = reinterpret_cast<const float4*>(x);
  long i4 = tid;
  for (; i4 + 3 * nthreads < n4; i4 += 4 * nthreads) {
    const float4 v0 = x4[i4], v1 = x4[i4 + nthreads], v2 = x4[i4 + 2 * nthreads], v3 = x4[i4 + 3 * nthreads];
    fold(v0); fold(v1); fold(v2); fold(v3);
  }
  for (; i4 < n4; i4 += nthreads) fold(x4[i4]);
  for (long i = n4 * 4 + tid; i < n; i += nthreads) m = fmaxf(m, fabsf(x[i]));
  // one atomic per workgroup: thousands of them on one address serialise
  __shared__ float red[16];
  m = warp_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x + 63) / 64; ++w) m = fmaxf(m, red[w]);
    atomicMax(out, __builtin_bit_cast(unsigned, m));
  }
}

// f32 (already clipped to +-448) -> e4m3fn byte, round-to-nearest-even with
// gradual underflow below 2^-6.
__device__ __forceinline__ uint8_t f32_to_e4m3(float v) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, v);
  const uint8_t sign = (uint8_t)((bits >> 24) & 0x80);
  const uint32_t ab = bits & 0x7fffffffu;
  if (ab > 0x7f800000u) return (uint8_t)(sign | 0x7f);            // NaN
  const float a = __builtin_bit_cast(float, ab);
  uint32_t code;
  if (a < 0.015625f) {                                            // below the smallest normal 2^-6
    code = (uint32_t)__builtin_rintf(a * 512.0f);                 // multiples of 2^-9; 8 carries into 0x08
  } else {
    const uint32_t r = (ab + 0x7ffffu + ((ab >> 20) & 1u)) >> 20; // (biased exp << 3) | 3-bit mantissa
    code = r - (120u << 3);
    if (code > 0x7eu) code = 0x7eu;                               // saturate at 448
  }
  return (uint8_t)(sign | code);
}

// f32 (already clipped to +-57344) -> e5m2 byte, round-to-nearest-even with gradual
// underflow below 2^-14 (the IEEE half-precision pattern cut to two mantissa bits).
__device__ __forceinline__ uint8_t f32_to_e5m2(float v) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, v);
  const uint8_t sign = (uint8_t)((bits >> 24) & 0x80);
  const uint32_t ab = bits & 0x7fffffffu;
  if (ab > 0x7f800000u) return (uint8_t)(sign | 0x7f);            // NaN
  const float a = __builtin_bit_cast(float, ab);
  uint32_t code;
  if (a < 6.103515625e-05f) {                                     // below the smallest normal 2^-14
    code = (uint32_t)__builtin_rintf(a * 65536.0f);               // multiples of 2^-16; 4 carries into 0x04
  } else {
    const uint32_t r = (ab + 0xfffffu + ((ab >> 21) & 1u)) >> 21; // (biased exp << 2) | 2-bit mantissa
    code = r - (112u << 2);
    if (code > 0x7bu) code = 0x7bu;                               // saturate at 57344
  }
  return (uint8_t)(sign | code);
}

// FMT 0: e4m3 (max 448), 1: e5m2 (max 57344).
// scale_in > 0: use it; else scale = max(amax / max_normal, 1e-12) from *amax_bits.
template <int FMT>
__global__ void quantize_f8_kernel(const float* x, long n, float scale_in, const unsigned* amax_bits,
                                   uint8_t* codes, float* scale_out) {
  constexpr float MAXN = FMT == 0 ? 448.0f : 57344.0f;
  float scale = scale_in;
  if (!(scale_in > 0.f)) {
    const float amax = __builtin_bit_cast(float, *amax_bits);
    scale = fmaxf(__fdiv_rn(amax, MAXN), 1e-12f);
  }
  if (scale_out && blockIdx.x == 0 && threadIdx.x == 0) *scale_out = scale;
  auto clip = [&](float f) { return fminf(fmaxf(__fdiv_rn(f, scale), -MAXN), MAXN); };
  auto code = [&](float f) -> uint32_t {
    if constexpr (FMT == 0) return f32_to_e4m3(clip(f));
    else return f32_to_e5m2(clip(f));
  };
  const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x, nthreads = (long)gridDim.x * blockDim.x;
  // runs of 16 elements: four 16-byte loads, one 16-byte store (both pointers 16-byte aligned)
  const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(codes)) & 15) == 0;
  const long n16 = vec ? n / 16 : 0;
  for (long g = tid; g < n16; g += nthreads) {
    uint32_t w[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float4 v = reinterpret_cast<const float4*>(x)[g * 4 + c];
      // the hardware conversion (OCP formats, round to nearest even, gradual underflow) on
      // values already clipped to the format's range gives the codes of the software one
      int pk;
      if constexpr (FMT == 0) {
        pk = __builtin_amdgcn_cvt_pk_fp8_f32(clip(v.x), clip(v.y), 0, false);
        pk = __builtin_amdgcn_cvt_pk_fp8_f32(clip(v.z), clip(v.w), pk, true);
      } else {
        pk = __builtin_amdgcn_cvt_pk_bf8_f32(clip(v.x), clip(v.y), 0, false);
        pk = __builtin_amdgcn_cvt_pk_bf8_f32(clip(v.z), clip(v.w), pk, true);
      }
      w[c] = (uint32_t)pk;
    }
    reinterpret_cast<uint4*>(codes)[g] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  for (long i = n16 * 16 + tid; i < n; i += nthreads) codes[i] = (uint8_t)code(x[i]);
}

// One workgroup per row: absmax, scale = max(absmax, 1e-12) / 127, q = rint(x / scale).
// `divisor` (f32[N] or null): x[m][n] / divisor[n] takes the place of x[m][n] — the smoothed
// activation of the W8A8 direct-consume path (compiler/smoothquant.py:60-62, 121-122).
__global__ void quantize_i8_rows_kernel(const float* x, int M, int N, int8_t* q, float* scales, const float* divisor) {
  __shared__ float red[4];
  const int m = blockIdx.x;
  if (m >= M) return;
  const float* row = x + (long)m * N;
  auto at = [&](int n) { return divisor ? __fdiv_rn(row[n], divisor[n]) : row[n]; };
  float mx = 0.f;
  for (int n = threadIdx.x; n < N; n += blockDim.x) mx = fmaxf(mx, fabsf(at(n)));
  mx = warp_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float scale = __fdiv_rn(fmaxf(mx, 1e-12f), 127.0f);
  if (threadIdx.x == 0) scales[m] = scale;
  for (int n = threadIdx.x; n < N; n += blockDim.x) {
    float t = __builtin_rintf(__fdiv_rn(at(n), scale));
    t = fminf(fmaxf(t, -127.f), 127.f);
    q[(long)m * N + n] = (int8_t)t;
  }
}

// The same for rows of up to 256 * 16 * GV elements (a multiple of 16, 16-byte aligned):
// a thread keeps its runs of 16 elements in registers between the absmax pass and the
// quantising pass, so x is read from memory once, with 16-byte loads, and every run of
// 16 codes leaves as one 16-byte store.
// (SMOOTH: every element is first divided by its column's entry of `divisor`, 16-byte aligned)
template <int GV, bool SMOOTH = false>
__global__ __launch_bounds__(256) void quantize_i8_rows_vec_kernel(const float* x, int M, int N, int8_t* q,
                                                                   float* scales, const float* divisor = nullptr) {
  __shared__ float red[4];
  const int m = blockIdx.x;
  if (m >= M) return;
  const float4* row = reinterpret_cast<const float4*>(x + (long)m * N);
  const int groups = N / 16;
  float4 v[GV][4];
  float mx = 0.f;
#pragma unroll
  for (int u = 0; u < GV; ++u) {
    const int g = threadIdx.x + 256 * u;
    if (g < groups) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        v[u][c] = row[g * 4 + c];
        if constexpr (SMOOTH) {
          const float4 d = reinterpret_cast<const float4*>(divisor)[g * 4 + c];
          v[u][c] = make_float4(__fdiv_rn(v[u][c].x, d.x), __fdiv_rn(v[u][c].y, d.y), __fdiv_rn(v[u][c].z, d.z),
                                __fdiv_rn(v[u][c].w, d.w));
        }
        mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v[u][c].x), fabsf(v[u][c].y)), fmaxf(fabsf(v[u][c].z), fabsf(v[u][c].w))));
      }
    }
  }
  mx = warp_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float scale = __fdiv_rn(fmaxf(mx, 1e-12f), 127.0f);
  if (threadIdx.x == 0) scales[m] = scale;
  auto code = [&](float f) -> uint32_t {
    float t = __builtin_rintf(__fdiv_rn(f, scale));
    t = fminf(fmaxf(t, -127.f), 127.f);
    return (uint32_t)(uint8_t)(int8_t)t;
  };
  auto pack = [&](const float4& f) -> uint32_t {
    return code(f.x) | (code(f.y) << 8) | (code(f.z) << 16) | (code(f.w) << 24);
  };
#pragma unroll
  for (int u = 0; u < GV; ++u) {
    const int g = threadIdx.x + 256 * u;
    if (g < groups)
      *reinterpret_cast<uint4*>(q + (long)m * N + g * 16) =
          make_uint4(pack(v[u][0]), pack(v[u][1]), pack(v[u][2]), pack(v[u][3]));
  }
}

// Column scales: each thread owns one column and walks the rows (coalesced
// across the wavefront); two passes over x.
__global__ void quantize_i8_cols_kernel(const float* x, int M, int N, int8_t* q, float* scales) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  float mx = 0.f;
  for (int m = 0; m < M; ++m) mx = fmaxf(mx, fabsf(x[(long)m * N + n]));
  const float scale = __fdiv_rn(fmaxf(mx, 1e-12f), 127.0f);
  scales[n] = scale;
  for (int m = 0; m < M; ++m) {
    float t = __builtin_rintf(__fdiv_rn(x[(long)m * N + n], scale));
    t = fminf(fmaxf(t, -127.f), 127.f);
    q[(long)m * N + n] = (int8_t)t;
  }
}

// Column scales for a wide matrix, in two fully parallel passes: a thread owns four
// adjacent columns (16-byte loads, coalesced across the wavefront) and a chunk of
// kColRows rows.  Pass 1 folds the chunk's absmax into amax_bits[n] with an atomic max on
// the bit pattern (non-negative floats order like unsigned integers); pass 2 derives the
// scale and writes the codes, four per 4-byte store.  N % 4 == 0, 16-byte aligned x.
constexpr int kColRows = 64;
__global__ __launch_bounds__(256) void absmax_cols_kernel(const float* x, int M, int N, unsigned* amax_bits) {
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (n >= N) return;
  const int m0 = blockIdx.y * kColRows, m1 = min(m0 + kColRows, M);
  float4 mx = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int m = m0; m < m1; ++m) {
    const float4 v = *reinterpret_cast<const float4*>(x + (long)m * N + n);
    mx.x = fmaxf(mx.x, fabsf(v.x)); mx.y = fmaxf(mx.y, fabsf(v.y));
    mx.z = fmaxf(mx.z, fabsf(v.z)); mx.w = fmaxf(mx.w, fabsf(v.w));
  }
  atomicMax(amax_bits + n + 0, __builtin_bit_cast(unsigned, mx.x));
  atomicMax(amax_bits + n + 1, __builtin_bit_cast(unsigned, mx.y));
  atomicMax(amax_bits + n + 2, __builtin_bit_cast(unsigned, mx.z));
  atomicMax(amax_bits + n + 3, __builtin_bit_cast(unsigned, mx.w));
}
__global__ __launch_bounds__(256) void quantize_i8_cols_vec_kernel(const float* x, int M, int N,
                                                                   const unsigned* amax_bits, int8_t* q,
                                                                   float* scales) {
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (n >= N) return;
  const int m0 = blockIdx.y * kColRows, m1 = min(m0 + kColRows, M);
  float sc[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    sc[e] = __fdiv_rn(fmaxf(__builtin_bit_cast(float, amax_bits[n + e]), 1e-12f), 127.0f);
  if (blockIdx.y == 0) *reinterpret_cast<float4*>(scales + n) = make_float4(sc[0], sc[1], sc[2], sc[3]);
  auto code = [&](float f, float scale) -> uint32_t {
    float t = __builtin_rintf(__fdiv_rn(f, scale));
    t = fminf(fmaxf(t, -127.f), 127.f);
    return (uint32_t)(uint8_t)(int8_t)t;
  };
  for (int m = m0; m < m1; ++m) {
    const float4 v = *reinterpret_cast<const float4*>(x + (long)m * N + n);
    *reinterpret_cast<uint32_t*>(q + (long)m * N + n) =
        code(v.x, sc[0]) | (code(v.y, sc[1]) << 8) | (code(v.z, sc[2]) << 16) | (code(v.w, sc[3]) << 24);
  }
}

template <int FMT = 0>
int quantize_e4m3_dev(const float* x, int64_t n, float scale, void* codes, float* scale_out_dev, hipStream_t s) {
  if (n <= 0 || !x || !codes) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const int blocks = (int)std::min<int64_t>((n + 255) / 256, 4096);
  unsigned* amax = nullptr;
  if (!(scale > 0.f)) {
    // the running maximum lives in the stream's own workspace (work on one stream runs in
    // order, so nothing else on it uses the workspace meanwhile): no allocation per call
    amax = static_cast<unsigned*>(stream_workspace(s, 256));
    if (!amax) return kDeviceFailed;
    zero_words(amax, 1, s);
    // (each workgroup ends in one atomic on the same word and those serialise at about
    // 8 ns each: two workgroups per CU, not sixteen)
    hipLaunchKernelGGL(absmax_kernel, dim3(std::min(blocks, 512)), dim3(256), 0, s, x, (long)n, amax);
  }
  hipLaunchKernelGGL((quantize_f8_kernel<FMT>), dim3(blocks), dim3(256), 0, s, x, (long)n, scale, amax,
                     static_cast<uint8_t*>(codes), scale_out_dev);
  return launch_status();
}

int quantize_i8_dev(const float* x, int M, int N, int axis, void* q, float* scales, hipStream_t s,
                    const float* divisor = nullptr) {
  if (M <= 0 || N <= 0 || !x || !q || !scales || (axis != 0 && axis != 1) || (divisor && axis != 1)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (axis == 1) {
    int8_t* codes = static_cast<int8_t*>(q);
    const int groups = N / 16;
    const bool vec = N % 16 == 0 && groups <= 4 * 256 && aligned16(x) && aligned16(q) && aligned16(divisor);
    if (divisor) {
      if (vec && groups <= 256)
        hipLaunchKernelGGL((quantize_i8_rows_vec_kernel<1, true>), dim3(M), dim3(256), 0, s, x, M, N, codes, scales, divisor);
      else if (vec && groups <= 512)
        hipLaunchKernelGGL((quantize_i8_rows_vec_kernel<2, true>), dim3(M), dim3(256), 0, s, x, M, N, codes, scales, divisor);
      else if (vec)
        hipLaunchKernelGGL((quantize_i8_rows_vec_kernel<4, true>), dim3(M), dim3(256), 0, s, x, M, N, codes, scales, divisor);
      else
        hipLaunchKernelGGL(quantize_i8_rows_kernel, dim3(M), dim3(256), 0, s, x, M, N, codes, scales, divisor);
    } else if (vec && groups <= 256)
      hipLaunchKernelGGL((quantize_i8_rows_vec_kernel<1>), dim3(M), dim3(256), 0, s, x, M, N, codes, scales, nullptr);
    else if (vec && groups <= 512)
      hipLaunchKernelGGL((quantize_i8_rows_vec_kernel<2>), dim3(M), dim3(256), 0, s, x, M, N, codes, scales, nullptr);
    else if (vec)
      hipLaunchKernelGGL((quantize_i8_rows_vec_kernel<4>), dim3(M), dim3(256), 0, s, x, M, N, codes, scales, nullptr);
    else
      hipLaunchKernelGGL(quantize_i8_rows_kernel, dim3(M), dim3(256), 0, s, x, M, N, codes, scales, nullptr);
  } else if (N % 4 == 0 && aligned16(x) && aligned16(scales) && (reinterpret_cast<uintptr_t>(q) & 3) == 0 &&
             ceil_div(M, kColRows) <= 65535) {
    // the per-column running maxima live in the stream's own workspace
    unsigned* amax = static_cast<unsigned*>(stream_workspace(s, (size_t)N * sizeof(unsigned)));
    if (!amax) return kDeviceFailed;
    zero_words(amax, (size_t)N, s);
    const dim3 grid(ceil_div(N, 1024), ceil_div(M, kColRows));
    hipLaunchKernelGGL(absmax_cols_kernel, grid, dim3(256), 0, s, x, M, N, amax);
    hipLaunchKernelGGL(quantize_i8_cols_vec_kernel, grid, dim3(256), 0, s, x, M, N, amax, static_cast<int8_t*>(q),
                       scales);
  } else {
    hipLaunchKernelGGL(quantize_i8_cols_kernel, dim3(ceil_div(N, 64)), dim3(64), 0, s, x, M, N,
                       static_cast<int8_t*>(q), scales);
  }
  return launch_status();
}

// quantization.quantize_int8, symmetric form (python/tessera/quantization.py:24-37): one scale for
// the whole tensor, scale_in if > 0 else max|x| / 127 (1 for an all-zero tensor);
// q = clip(rint(x / scale), -127, 127).  Runs of 16 elements per thread.
__global__ __launch_bounds__(256) void quantize_i8_tensor_kernel(const float* __restrict__ x, long n, float scale_in,
                                                                 const unsigned* amax_bits, int8_t* __restrict__ q,
                                                                 float* scale_out) {
  float scale = scale_in;
  if (!(scale_in > 0.f)) {
    const float amax = __builtin_bit_cast(float, *amax_bits);
    scale = amax == 0.f ? 1.0f : __fdiv_rn(amax, 127.0f);
  }
  if (scale_out && blockIdx.x == 0 && threadIdx.x == 0) *scale_out = scale;
  auto code = [&](float f) -> uint32_t {
    float t = __builtin_rintf(__fdiv_rn(f, scale));
    t = fminf(fmaxf(t, -127.f), 127.f);
    return (uint32_t)(uint8_t)(int8_t)t;
  };
  auto pack = [&](const float4& f) -> uint32_t {
    return code(f.x) | (code(f.y) << 8) | (code(f.z) << 16) | (code(f.w) << 24);
  };
  const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x, nthreads = (long)gridDim.x * blockDim.x;
  const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(q)) & 15) == 0;
  const long n16 = vec ? n / 16 : 0;
  for (long g = tid; g < n16; g += nthreads) {
    const float4* src = reinterpret_cast<const float4*>(x) + g * 4;
    const float4 v0 = src[0], v1 = src[1], v2 = src[2], v3 = src[3];
    reinterpret_cast<uint4*>(q)[g] = make_uint4(pack(v0), pack(v1), pack(v2), pack(v3));
  }
  for (long i = n16 * 16 + tid; i < n; i += nthreads) q[i] = (int8_t)code(x[i]);
}

int quantize_i8_tensor_dev(const float* x, int64_t n, float scale, void* q, float* scale_out_dev, hipStream_t s) {
  if (n <= 0 || !x || !q || scale != scale) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const int blocks = (int)std::min<int64_t>((n / 16 + 255) / 256 + 1, 4096);
  unsigned* amax = nullptr;
  if (!(scale > 0.f)) {
    amax = static_cast<unsigned*>(stream_workspace(s, 256));
    if (!amax) return kDeviceFailed;
    zero_words(amax, 1, s);
    hipLaunchKernelGGL(absmax_kernel, dim3(std::min(blocks, 512)), dim3(256), 0, s, x, (long)n, amax);
  }
  hipLaunchKernelGGL(quantize_i8_tensor_kernel, dim3(blocks), dim3(256), 0, s, x, (long)n, scale, amax,
                     static_cast<int8_t*>(q), scale_out_dev);
  return launch_status();
}

// ---- per-tensor float grids (fp8 / fp6 / fp4) ---------------------------------------------------
// The native lanes' grid rounding, tessera_x86_avx512_fpquant_f32
// (src/compiler/codegen/tessera_x86_backend/src/kernels/avx512_fpquant_f32.cpp:28-41):
//   ax = min(|v|, max_normal); e = max(floor(log2 ax), min_exp); ulp = 2^(e - mantissa_bits);
//   out = sign(v) * min(rne(ax / ulp) * ulp, max_normal); NaN propagates; zero gives +0.
// Both scalings are by powers of two, so ldexp is exact wherever the division and the product are.
__device__ __forceinline__ float fp_grid(float v, float max_normal, int mant, int min_exp) {
  if (v != v) return v;
  const float ax = fminf(fabsf(v), max_normal);
  if (!(ax > 0.f)) return 0.f;
  int e;
  (void)frexpf(ax, &e);                                   // ax = m 2^e with m in [0.5, 1), denormals included
  e = max(e - 1, min_exp);
  const float q = __builtin_rintf(ldexpf(ax, mant - e));
  const float r = fminf(ldexpf(q, e - mant), max_normal);
  return v < 0.f ? -r : r;
}

// ops.quantize_fp8 / quantize_fp6 / quantize_fp4 (python/tessera/__init__.py:3340-3374, 3411-3464):
// scale = scale_in if > 0, else max(amax / max_normal, 1e-12); grid = fp_grid(x / scale) (the
// reference clips x / scale to +-max_normal first, which the grid's own clamp already does);
// dq = grid * scale.  grid16 receives the grid values as bf16 bits: exact for every format of at
// most 7 mantissa bits whose range lies within bf16's.
__global__ __launch_bounds__(256) void fake_quantize_fp_kernel(const float* __restrict__ x, long n, float max_normal,
                                                               int mant, int min_exp, float scale_in,
                                                               const unsigned* amax_bits, float* __restrict__ dq,
                                                               uint16_t* __restrict__ grid16, float* scale_out) {
  float scale = scale_in;
  if (!(scale_in > 0.f)) scale = fmaxf(__fdiv_rn(__builtin_bit_cast(float, *amax_bits), max_normal), 1e-12f);
  if (scale_out && blockIdx.x == 0 && threadIdx.x == 0) *scale_out = scale;
  const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x, nthreads = (long)gridDim.x * blockDim.x;
  const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dq)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(grid16) & 7) == 0;
  const long n4 = vec ? n / 4 : 0;
  auto bf16_bits = [](float g) { return (uint32_t)(__builtin_bit_cast(uint32_t, g) >> 16); };
  for (long i = tid; i < n4; i += nthreads) {
    const float4 v = reinterpret_cast<const float4*>(x)[i];
    const float g0 = fp_grid(__fdiv_rn(v.x, scale), max_normal, mant, min_exp);
    const float g1 = fp_grid(__fdiv_rn(v.y, scale), max_normal, mant, min_exp);
    const float g2 = fp_grid(__fdiv_rn(v.z, scale), max_normal, mant, min_exp);
    const float g3 = fp_grid(__fdiv_rn(v.w, scale), max_normal, mant, min_exp);
    if (dq) reinterpret_cast<float4*>(dq)[i] = make_float4(g0 * scale, g1 * scale, g2 * scale, g3 * scale);
    if (grid16)
      reinterpret_cast<uint2*>(grid16)[i] = make_uint2(bf16_bits(g0) | (bf16_bits(g1) << 16), bf16_bits(g2) | (bf16_bits(g3) << 16));
  }
  for (long i = n4 * 4 + tid; i < n; i += nthreads) {
    const float g = fp_grid(__fdiv_rn(x[i], scale), max_normal, mant, min_exp);
    if (dq) dq[i] = g * scale;
    if (grid16) grid16[i] = (uint16_t)bf16_bits(g);
  }
}

// mantissa_bits 0..23 and min_exp -126..127 keep every power of two the rounding forms a normal
// or denormal f32.
bool bad_fp_format(float max_normal, int mant, int min_exp) {
  return !(max_normal > 0.f) || !std::isfinite(max_normal) || mant < 0 || mant > 23 || min_exp < -126 || min_exp > 127;
}

int fake_quantize_fp_dev(const float* x, int64_t n, float max_normal, int mant, int min_exp, float scale, float* dq,
                         void* grid16, float* scale_out_dev, hipStream_t s) {
  if (n <= 0 || !x || (!dq && !grid16) || bad_fp_format(max_normal, mant, min_exp) || scale != scale) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const int blocks = (int)std::min<int64_t>((n / 4 + 255) / 256 + 1, 4096);
  unsigned* amax = nullptr;
  if (!(scale > 0.f)) {
    amax = static_cast<unsigned*>(stream_workspace(s, 256));
    if (!amax) return kDeviceFailed;
    zero_words(amax, 1, s);
    hipLaunchKernelGGL(absmax_kernel, dim3(std::min(blocks, 512)), dim3(256), 0, s, x, (long)n, amax);
  }
  hipLaunchKernelGGL(fake_quantize_fp_kernel, dim3(blocks), dim3(256), 0, s, x, (long)n, max_normal, mant, min_exp, scale,
                     amax, dq, static_cast<uint16_t*>(grid16), scale_out_dev);
  return launch_status();
}

// ---- NVFP4 (block-scaled E2M1) rounding -------------------------------------------------------
// ops.quantize_nvfp4 followed by dequantize_nvfp4 (python/tessera/__init__.py:3472-3504;
// compiler/microscaling.py:317-384): blocks of 16 along the last axis (a short last block counts
// its missing elements as zeros); raw = max(amax / 6, 1e-30); block scale = raw rounded to e4m3fn
// (a scale that rounds to zero becomes 1); code = x / scale rounded to the E2M1 grid
// {0, .5, 1, 1.5, 2, 3, 4, 6} (nearest even, saturating); value = code * scale.  A value has at
// most 2 + 4 significant bits, so its bf16 form is exact.  One thread per block.
__device__ __forceinline__ float e2m1_round(float v) {
  const float a = fminf(fabsf(v), 6.0f);
  const float ulp = a < 2.0f ? 0.5f : (a < 4.0f ? 1.0f : 2.0f);
  const float r = fminf(__builtin_rintf(__fdiv_rn(a, ulp)) * ulp, 6.0f);
  return copysignf(r, v);
}

__global__ __launch_bounds__(256) void fake_quantize_nvfp4_kernel(const float* __restrict__ x, int rows, int cols,
                                                                  float* __restrict__ dq, uint16_t* __restrict__ dq16,
                                                                  float* __restrict__ scales) {
  const int nb = (cols + 15) / 16;
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long)rows * nb) return;
  const long r = id / nb;
  const int b = (int)(id - r * nb);
  const int c0 = b * 16, n = min(16, cols - c0);
  const float* src = x + r * cols + c0;
  float v[16];
  if (n == 16 && ((reinterpret_cast<uintptr_t>(src) & 15) == 0)) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 t = reinterpret_cast<const float4*>(src)[q];
      v[4 * q] = t.x; v[4 * q + 1] = t.y; v[4 * q + 2] = t.z; v[4 * q + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = i < n ? src[i] : 0.f;
  }
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
  const float raw = fmaxf(__fdiv_rn(amax, 6.0f), 1e-30f);
  const float scale = e4m3_to_f32(f32_to_e4m3(fminf(raw, 448.0f)));
  const float sf = scale == 0.f ? 1.0f : scale;
  if (scales) scales[id] = scale;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (i < n) {
      const float o = e2m1_round(__fdiv_rn(v[i], sf)) * sf;
      if (dq) dq[r * cols + c0 + i] = o;
      if (dq16) dq16[r * cols + c0 + i] = (uint16_t)(__builtin_bit_cast(uint32_t, o) >> 16);
    }
  }
}

int fake_quantize_nvfp4_dev(const float* x, int rows, int cols, float* dq, void* dq16, float* scales, hipStream_t s) {
  if (rows <= 0 || cols <= 0 || !x || (!dq && !dq16)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const long blocks = (long)rows * ((cols + 15) / 16);
  hipLaunchKernelGGL(fake_quantize_nvfp4_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, s, x, rows, cols, dq,
                     static_cast<uint16_t*>(dq16), scales);
  return launch_status();
}

Gemm8Params make_params(const void* A, const void* B, void* D, int M, int N, int K) {
  Gemm8Params p{};
  p.A = static_cast<const uint8_t*>(A);
  p.B = static_cast<const uint8_t*>(B);
  p.D = D;
  p.M = M; p.N = N; p.K = K;
  p.scale_a = p.scale_b = 1.f;
  return p;
}

template <class T, int EPI>
int gemm8_host(const void* A, const void* B, const float* rs, const float* cs, float sa, float sb, void* D,
               void* acc_out, int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || !A || !B || !D) return kBadShape;
  if (EPI == EPI8_W8A8_F32 && (!rs || !cs)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t dsz = (EPI == EPI8_SCALED_BF16) ? 2 : 4;
  const size_t d_bytes = (size_t)M * N * dsz, acc_bytes = (size_t)M * N * 4;
  DeviceScope scope;
  Gemm8Params p = make_params(scope.alloc((size_t)M * K, A), scope.alloc((size_t)K * N, B), scope.alloc(d_bytes),
                              M, N, K);
  if (EPI == EPI8_W8A8_F32) {
    p.row_scale = static_cast<const float*>(scope.alloc((size_t)M * 4, rs));
    p.col_scale = static_cast<const float*>(scope.alloc((size_t)N * 4, cs));
    if (acc_out) p.acc_out = static_cast<int32_t*>(scope.alloc(acc_bytes));
  }
  p.scale_a = sa; p.scale_b = sb;
  if (scope.failed()) return kDeviceFailed;
  int rc = gemm8_dev<T, EPI>(p, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(D, p.D, d_bytes)) return kDeviceFailed;
  if (p.acc_out && !scope.download(acc_out, p.acc_out, acc_bytes)) return kDeviceFailed;
  return kOk;
}

template <int FMT>
int quantize_f8_host(const float* x, int64_t n, float scale, void* codes, float* scale_out) {
  if (n <= 0 || !x || !codes) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  float* dx = static_cast<float*>(scope.alloc((size_t)n * 4, x));
  void* dc = scope.alloc((size_t)n);
  float* ds = static_cast<float*>(scope.alloc(4));
  if (scope.failed()) return kDeviceFailed;
  int rc = quantize_e4m3_dev<FMT>(dx, n, scale, dc, ds, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(codes, dc, (size_t)n)) return kDeviceFailed;
  if (scale_out && !scope.download(scale_out, ds, 4)) return kDeviceFailed;
  return kOk;
}
}  // namespace
}  // namespace tsr950

using namespace tsr950;

extern "C" {

int tessera_gfx950_gemm_i8_i32(const void* A, const void* B, void* C, int M, int N, int K) {
  return gemm8_host<I8, EPI8_I32>(A, B, nullptr, nullptr, 1.f, 1.f, C, nullptr, M, N, K);
}
int tessera_gfx950_gemm_w8a8_f32(const void* A, const void* B, const float* row_scale, const float* col_scale,
                                 void* D, void* acc_out, int M, int N, int K) {
  return gemm8_host<I8, EPI8_W8A8_F32>(A, B, row_scale, col_scale, 1.f, 1.f, D, acc_out, M, N, K);
}
int tessera_gfx950_gemm_e4m3_bf16(const void* A, const void* B, float scale_a, float scale_b, void* D, int M,
                                  int N, int K) {
  return gemm8_host<FP8, EPI8_SCALED_BF16>(A, B, nullptr, nullptr, scale_a, scale_b, D, nullptr, M, N, K);
}
int tessera_gfx950_gemm_e4m3_f32(const void* A, const void* B, float scale_a, float scale_b, void* D, int M,
                                 int N, int K) {
  return gemm8_host<FP8, EPI8_SCALED_F32>(A, B, nullptr, nullptr, scale_a, scale_b, D, nullptr, M, N, K);
}

int tessera_gfx950_gemm_e5m2_bf16(const void* A, const void* B, float scale_a, float scale_b, void* D, int M,
                                  int N, int K) {
  return gemm8_host<BF8, EPI8_SCALED_BF16>(A, B, nullptr, nullptr, scale_a, scale_b, D, nullptr, M, N, K);
}
int tessera_gfx950_gemm_e5m2_f32(const void* A, const void* B, float scale_a, float scale_b, void* D, int M,
                                 int N, int K) {
  return gemm8_host<BF8, EPI8_SCALED_F32>(A, B, nullptr, nullptr, scale_a, scale_b, D, nullptr, M, N, K);
}

int tessera_gfx950_gemm_i8_i32_dev(const void* A, const void* B, void* C, int M, int N, int K, void* stream) {
  return gemm8_dev<I8, EPI8_I32>(make_params(A, B, C, M, N, K), as_stream(stream));
}
int tessera_gfx950_gemm_w8a8_f32_dev(const void* A, const void* B, const float* row_scale,
                                     const float* col_scale, void* D, void* acc_out, int M, int N, int K,
                                     void* stream) {
  Gemm8Params p = make_params(A, B, D, M, N, K);
  p.row_scale = row_scale;
  p.col_scale = col_scale;
  p.acc_out = static_cast<int32_t*>(acc_out);
  return gemm8_dev<I8, EPI8_W8A8_F32>(p, as_stream(stream));
}
int tessera_gfx950_gemm_e4m3_bf16_dev(const void* A, const void* B, float scale_a, float scale_b, void* D,
                                      int M, int N, int K, void* stream) {
  Gemm8Params p = make_params(A, B, D, M, N, K);
  p.scale_a = scale_a; p.scale_b = scale_b;
  return gemm8_dev<FP8, EPI8_SCALED_BF16>(p, as_stream(stream));
}
int tessera_gfx950_gemm_e4m3_f32_dev(const void* A, const void* B, float scale_a, float scale_b, void* D,
                                     int M, int N, int K, void* stream) {
  Gemm8Params p = make_params(A, B, D, M, N, K);
  p.scale_a = scale_a; p.scale_b = scale_b;
  return gemm8_dev<FP8, EPI8_SCALED_F32>(p, as_stream(stream));
}

int tessera_gfx950_gemm_e5m2_bf16_dev(const void* A, const void* B, float scale_a, float scale_b, void* D,
                                      int M, int N, int K, void* stream) {
  Gemm8Params p = make_params(A, B, D, M, N, K);
  p.scale_a = scale_a; p.scale_b = scale_b;
  return gemm8_dev<BF8, EPI8_SCALED_BF16>(p, as_stream(stream));
}
int tessera_gfx950_gemm_e5m2_f32_dev(const void* A, const void* B, float scale_a, float scale_b, void* D,
                                     int M, int N, int K, void* stream) {
  Gemm8Params p = make_params(A, B, D, M, N, K);
  p.scale_a = scale_a; p.scale_b = scale_b;
  return gemm8_dev<BF8, EPI8_SCALED_F32>(p, as_stream(stream));
}

int tessera_gfx950_quantize_e4m3_f32_dev(const float* x, int64_t n, float scale, void* codes,
                                         float* scale_out_dev, void* stream) {
  return quantize_e4m3_dev<0>(x, n, scale, codes, scale_out_dev, as_stream(stream));
}
int tessera_gfx950_quantize_e5m2_f32_dev(const float* x, int64_t n, float scale, void* codes,
                                         float* scale_out_dev, void* stream) {
  return quantize_e4m3_dev<1>(x, n, scale, codes, scale_out_dev, as_stream(stream));
}
int tessera_gfx950_quantize_i8_f32_dev(const float* x, int M, int N, int axis, void* q, float* scales,
                                       void* stream) {
  return quantize_i8_dev(x, M, N, axis, q, scales, as_stream(stream));
}

int tessera_gfx950_quantize_i8_tensor_f32_dev(const float* x, int64_t n, float scale, void* q, float* scale_out_dev,
                                              void* stream) {
  return quantize_i8_tensor_dev(x, n, scale, q, scale_out_dev, as_stream(stream));
}
int tessera_gfx950_quantize_i8_smoothed_f32_dev(const float* x, int M, int N, const float* smoothing, void* q,
                                                float* scales, void* stream) {
  if (!smoothing) return kBadShape;
  return quantize_i8_dev(x, M, N, 1, q, scales, as_stream(stream), smoothing);
}

int tessera_gfx950_fake_quantize_nvfp4_f32_dev(const float* x, int rows, int cols, float* dq, void* dq_bf16,
                                               float* scales, void* stream) {
  return fake_quantize_nvfp4_dev(x, rows, cols, dq, dq_bf16, scales, as_stream(stream));
}

int tessera_gfx950_fake_quantize_nvfp4_f32(const float* x, int rows, int cols, float* dq, void* dq_bf16, float* scales) {
  if (rows <= 0 || cols <= 0 || !x || (!dq && !dq_bf16)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t n = (size_t)rows * cols, ns = (size_t)rows * ((cols + 15) / 16);
  DeviceScope scope;
  float* dx = static_cast<float*>(scope.alloc(n * 4, x));
  float* dd = dq ? static_cast<float*>(scope.alloc(n * 4)) : nullptr;
  void* d16 = dq_bf16 ? scope.alloc(n * 2) : nullptr;
  float* ds = scales ? static_cast<float*>(scope.alloc(ns * 4)) : nullptr;
  if (scope.failed()) return kDeviceFailed;
  int rc = fake_quantize_nvfp4_dev(dx, rows, cols, dd, d16, ds, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (dq && !scope.download(dq, dd, n * 4)) return kDeviceFailed;
  if (dq_bf16 && !scope.download(dq_bf16, d16, n * 2)) return kDeviceFailed;
  if (scales && !scope.download(scales, ds, ns * 4)) return kDeviceFailed;
  return kOk;
}

int tessera_gfx950_fake_quantize_fp_f32_dev(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp,
                                            float scale, float* dq, void* grid_bf16, float* scale_out_dev, void* stream) {
  return fake_quantize_fp_dev(x, n, max_normal, mantissa_bits, min_exp, scale, dq, grid_bf16, scale_out_dev,
                              as_stream(stream));
}
int tessera_gfx950_fpquant_f32_dev(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp, float* out,
                                   void* stream) {
  if (!out) return kBadShape;
  return fake_quantize_fp_dev(x, n, max_normal, mantissa_bits, min_exp, 1.0f, out, nullptr, nullptr, as_stream(stream));
}

int tessera_gfx950_fake_quantize_fp_f32(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp,
                                        float scale, float* dq, void* grid_bf16, float* scale_out) {
  if (n <= 0 || !x || (!dq && !grid_bf16) || bad_fp_format(max_normal, mantissa_bits, min_exp) || scale != scale)
    return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  float* dx = static_cast<float*>(scope.alloc((size_t)n * 4, x));
  float* dd = dq ? static_cast<float*>(scope.alloc((size_t)n * 4)) : nullptr;
  void* d16 = grid_bf16 ? scope.alloc((size_t)n * 2) : nullptr;
  float* ds = static_cast<float*>(scope.alloc(4));
  if (scope.failed()) return kDeviceFailed;
  int rc = fake_quantize_fp_dev(dx, n, max_normal, mantissa_bits, min_exp, scale, dd, d16, ds, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (dq && !scope.download(dq, dd, (size_t)n * 4)) return kDeviceFailed;
  if (grid_bf16 && !scope.download(grid_bf16, d16, (size_t)n * 2)) return kDeviceFailed;
  if (scale_out && !scope.download(scale_out, ds, 4)) return kDeviceFailed;
  return kOk;
}
int tessera_gfx950_fpquant_f32(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp, float* out) {
  if (!out) return kBadShape;
  return tessera_gfx950_fake_quantize_fp_f32(x, n, max_normal, mantissa_bits, min_exp, 1.0f, out, nullptr, nullptr);
}

int tessera_gfx950_quantize_e4m3_f32(const float* x, int64_t n, float scale, void* codes, float* scale_out) {
  return quantize_f8_host<0>(x, n, scale, codes, scale_out);
}
int tessera_gfx950_quantize_e5m2_f32(const float* x, int64_t n, float scale, void* codes, float* scale_out) {
  return quantize_f8_host<1>(x, n, scale, codes, scale_out);
}

int tessera_gfx950_quantize_i8_tensor_f32(const float* x, int64_t n, float scale, void* q, float* scale_out) {
  if (n <= 0 || !x || !q || scale != scale) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  float* dx = static_cast<float*>(scope.alloc((size_t)n * 4, x));
  void* dq = scope.alloc((size_t)n);
  float* ds = static_cast<float*>(scope.alloc(4));
  if (scope.failed()) return kDeviceFailed;
  int rc = quantize_i8_tensor_dev(dx, n, scale, dq, ds, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(q, dq, (size_t)n)) return kDeviceFailed;
  if (scale_out && !scope.download(scale_out, ds, 4)) return kDeviceFailed;
  return kOk;
}

int tessera_gfx950_quantize_i8_smoothed_f32(const float* x, int M, int N, const float* smoothing, void* q, float* scales) {
  if (M <= 0 || N <= 0 || !x || !q || !scales || !smoothing) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t n = (size_t)M * N;
  DeviceScope scope;
  float* dx = static_cast<float*>(scope.alloc(n * 4, x));
  float* dsm = static_cast<float*>(scope.alloc((size_t)N * 4, smoothing));
  void* dq = scope.alloc(n);
  float* ds = static_cast<float*>(scope.alloc((size_t)M * 4));
  if (scope.failed()) return kDeviceFailed;
  int rc = quantize_i8_dev(dx, M, N, 1, dq, ds, nullptr, dsm);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(q, dq, n) || !scope.download(scales, ds, (size_t)M * 4)) return kDeviceFailed;
  return kOk;
}

int tessera_gfx950_quantize_i8_f32(const float* x, int M, int N, int axis, void* q, float* scales) {
  if (M <= 0 || N <= 0 || !x || !q || !scales || (axis != 0 && axis != 1)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t n = (size_t)M * N, ns = (size_t)(axis == 1 ? M : N);
  DeviceScope scope;
  float* dx = static_cast<float*>(scope.alloc(n * 4, x));
  void* dq = scope.alloc(n);
  float* ds = static_cast<float*>(scope.alloc(ns * 4));
  if (scope.failed()) return kDeviceFailed;
  int rc = quantize_i8_dev(dx, M, N, axis, dq, ds, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(q, dq, n) || !scope.download(scales, ds, ns * 4)) return kDeviceFailed;
  return kOk;
}

}  // extern "C"
