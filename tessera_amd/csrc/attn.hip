// C ABI: flash-attention forward (causal, GQA, LSE), 16-bit storage.
#include <cmath>
#include <mutex>
#include "../../include/tessera_gfx950.h"
#include "flash_attn.h"
#include "flash_decode.h"
#include "flash_bwd.h"
#include "host_util.h"

namespace tsr950 {
namespace {

bool bad_attn(int B, int Hq, int Hkv, int Sq, int Sk, int D) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq <= 0 || Sk <= 0 || D <= 0) return true;
  if (D % 16 != 0 || D > 256) return true;       // matrix-core lanes need head_dim % 16 == 0
  if (Hq % Hkv != 0) return true;
  return false;
}

template <class T, int DP, bool EXT, bool PAD>
int launch_flash(const FlashParams& p, hipStream_t s) {
  using G = FlashGeom<DP>;
  auto kern = flash_fwd_kernel<T, DP, EXT, PAD>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, G::SMEM);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  const int qblocks = ceil_div(p.Sq, G::BQ);
  const bool xcd_grouped = (p.B * p.Hkv) % 8 == 0;
  // Few workgroups against a long key range (a chunk of queries against a long context): the key
  // tiles are split over gridDim.y, each split writes a normalised partial O and its log-sum-exp
  // to the stream workspace, and the merge kernel of the decode path combines them.  About two
  // workgroups per compute unit, at least 8 tiles (512 keys) a split.
  const long wgs = (long)p.B * p.Hq * qblocks;
  const int tiles = ceil_div(p.Sk, FA_BKV);
  int nsplit = 1;
  if (wgs < 192 && !p.bias) nsplit = (int)std::max<long>(1, std::min<long>(std::min<long>(ceil_div(512, (int)wgs), tiles / 8), 64));
  if (nsplit > 1) {
    FlashParams q = p;
    q.tiles_per_split = ceil_div(tiles, nsplit);
    q.nsplit = ceil_div(tiles, q.tiles_per_split);
    const size_t rows = (size_t)p.B * p.Hq * p.Sq;
    float* ws = static_cast<float*>(stream_workspace(s, (size_t)q.nsplit * rows * (p.D + 1) * sizeof(float)));
    if (!ws) return kDeviceFailed;
    q.O = ws;
    q.LSE = ws + (size_t)q.nsplit * rows * p.D;
    q.os = FlashStrides{(long)p.Hq * p.Sq * p.D, (long)p.Sq * p.D, (long)p.D};
    q.out_storage = 0;
    q.split_o_elems = (long)rows * p.D;
    const dim3 grid = xcd_grouped ? dim3(8 * p.ratio, qblocks * q.nsplit, p.B * p.Hkv / 8)
                                  : dim3(p.B * p.Hq, qblocks * q.nsplit, 1);
    hipLaunchKernelGGL(kern, grid, dim3(G::THREADS), G::SMEM, s, q);
    if (int rc = launch_status(); rc != kOk) return rc;
    launch_flash_merge<T>(p, static_cast<const float*>(q.O), static_cast<const float*>(q.LSE), q.nsplit, s);
    return launch_status();
  }
  const dim3 grid = xcd_grouped ? dim3(8 * p.ratio, qblocks, p.B * p.Hkv / 8) : dim3(p.B * p.Hq, qblocks, 1);
  hipLaunchKernelGGL(kern, grid, dim3(G::THREADS), G::SMEM, s, p);
  return launch_status();
}

// The kernel for head dimension p.D: compiled for DP = 64 / 128 / 256, exact when D == DP
// or zero-padded to it, each in the plain and the extended form.
template <class T>
int launch_flash_for(const FlashParams& p, bool ext, hipStream_t s) {
  switch (p.D) {
    case 64: return ext ? launch_flash<T, 64, true, false>(p, s) : launch_flash<T, 64, false, false>(p, s);
    case 128: return ext ? launch_flash<T, 128, true, false>(p, s) : launch_flash<T, 128, false, false>(p, s);
    case 256: return ext ? launch_flash<T, 256, true, false>(p, s) : launch_flash<T, 256, false, false>(p, s);
    default: break;
  }
  if (p.D < 64) return ext ? launch_flash<T, 64, true, true>(p, s) : launch_flash<T, 64, false, true>(p, s);
  if (p.D < 128) return ext ? launch_flash<T, 128, true, true>(p, s) : launch_flash<T, 128, false, true>(p, s);
  return ext ? launch_flash<T, 256, true, true>(p, s) : launch_flash<T, 256, false, true>(p, s);
}

// Few query rows per KV head (decode, short speculative steps): the rows of a whole GQA group
// share one MFMA tile and the key range is split over workgroups (flash_decode.h).  Returns
// false when the problem is not of that kind (the general kernel then serves it).
template <class T, int DP, int NQ>
int launch_decode(const FlashParams& p, hipStream_t s) {
  using G = DecodeGeom<DP>;
  auto kern = flash_decode_kernel<T, DP, NQ>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, G::SMEM);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  FlashDecodeParams dp{};
  dp.f = p;
  dp.rows = p.ratio * p.Sq;
  int lo0, hi0, lo1, hi1;
  key_bounds(0, p.Sq, p.Sk, p.causal, p.window, lo0, hi0);
  key_bounds(p.Sq - 1, p.Sq, p.Sk, p.causal, p.window, lo1, hi1);
  dp.tile_lo = lo0 / G::BK;
  dp.tile_end = hi1 / G::BK + 1;
  const int tiles = dp.tile_end - dp.tile_lo;
  // about two workgroups per compute unit, and at least two tiles for every wave of a split
  const int kvheads = p.B * p.Hkv;
  int nsplit = std::max(1, std::min(ceil_div(512, kvheads), tiles / (2 * G::WAVES)));
  dp.tiles_per_split = ceil_div(ceil_div(tiles, nsplit), G::WAVES) * G::WAVES;
  nsplit = ceil_div(tiles, dp.tiles_per_split);
  if (nsplit > 1) {
    const size_t rows = (size_t)p.B * p.Hq * p.Sq;
    float* ws = static_cast<float*>(stream_workspace(s, (size_t)nsplit * rows * (DP + 1) * sizeof(float)));
    if (!ws) return kDeviceFailed;
    dp.part_o = ws;
    dp.part_lse = ws + (size_t)nsplit * rows * DP;
  }
  hipLaunchKernelGGL(kern, dim3(kvheads, nsplit), dim3(G::THREADS), G::SMEM, s, dp);
  if (int rc = launch_status(); rc != kOk || nsplit == 1) return rc;
  launch_flash_merge<T>(p, dp.part_o, dp.part_lse, nsplit, s);
  return launch_status();
}
// (up to 32 rows per KV head at D = 256, 64 at D = 128, 128 at D = 64: one, two or four query
// tiles per wave, what the register file holds of their accumulators)
inline int decode_row_limit(int D) { return D == 64 ? 128 : D == 128 ? 64 : D == 256 ? 32 : 0; }
inline bool decode_shaped(const FlashParams& p) {
  const long rows = (long)p.ratio * p.Sq;
  if (rows > decode_row_limit(p.D)) return false;
  // beyond one query tile the gain is the shared read of K and V by the group's heads (measured: up to
  // 6x with 8 heads a group, a tie or a loss with one)
  if (rows > 32 && p.ratio == 1) return false;
  int lo0, hi0, lo1, hi1;
  key_bounds(0, p.Sq, p.Sk, p.causal, p.window, lo0, hi0);
  key_bounds(p.Sq - 1, p.Sq, p.Sk, p.causal, p.window, lo1, hi1);
  return hi1 >= lo0;                                   // some row sees some key
}

// Contiguous [B, H, S, D].
inline FlashStrides bhsd(int H, int S, int D) { return FlashStrides{(long)H * S * D, (long)S * D, (long)D}; }
// ([B, S, H, D], the rows of a (B * S) x (H * D) matrix one head's D columns at a time, is
// {S * H * D, D, H * D}: callers of the strided entry points pass it themselves.)

bool bad_strides(const FlashStrides& st) {
  return st.batch < 0 || st.head < 0 || st.row <= 0;
}
bool aligned16(const FlashStrides& st) { return ((st.batch | st.head | st.row) & 7) == 0; }

template <class T>
int flash_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B, int Hq, int Hkv,
              int Sq, int Sk, int D, float scale, int causal, int out_storage, hipStream_t s, int window = 0,
              float softcap = 0.f, const float* bias = nullptr, const FlashStrides* strides = nullptr) {
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || !Q || !K || !V || !O) return kBadShape;
  if (window < 0 || !(softcap >= 0.f)) return kBadShape;
  FlashParams p{};
  if (strides) {
    for (int i = 0; i < 4; ++i)
      if (bad_strides(strides[i])) return kBadShape;
    p.qs = strides[0]; p.ks = strides[1]; p.vs = strides[2]; p.os = strides[3];
    if (p.qs.row < D || p.ks.row < D || p.vs.row < D || p.os.row < D) return kBadShape;
    // per-lane byte offsets inside a 64-key tile are 32-bit
    if (p.ks.row > (1L << 23) || p.vs.row > (1L << 23)) return kBadShape;
  } else {
    p.qs = bhsd(Hq, Sq, D); p.ks = bhsd(Hkv, Sk, D); p.vs = p.ks; p.os = p.qs;
  }
  if (probe_device() != kOk) return kNoDevice;
  p.Q = static_cast<const uint16_t*>(Q);
  p.K = static_cast<const uint16_t*>(K);
  p.V = static_cast<const uint16_t*>(V);
  p.O = O;
  p.LSE = static_cast<float*>(LSE);
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Sq = Sq; p.Sk = Sk; p.D = D;
  p.ratio = Hq / Hkv;
  p.scale = scale;
  p.causal = causal ? 1 : 0;
  p.out_storage = out_storage ? 1 : 0;
  p.window = window;
  p.softcap = softcap;
  p.bias = bias;
  // 16-byte accesses: pointers and strides must be multiples of 16 bytes (8 elements of the
  // 16-bit operands; O in f32 is then aligned as well).
  const bool al = ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) |
                    reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(O)) & 15) == 0 &&
                  aligned16(p.qs) && aligned16(p.ks) && aligned16(p.vs) && aligned16(p.os);
  // The plain variant takes row maxima of the raw scores, which needs scale > 0; the
  // extended one scales first and serves every other scale.
  const bool ext = p.softcap > 0.f || p.bias != nullptr || !(scale > 0.f);
  if (al && !ext && decode_shaped(p)) {
    const int rows = p.ratio * p.Sq;
    if (p.D == 64) return rows <= 32 ? launch_decode<T, 64, 1>(p, s) : rows <= 64 ? launch_decode<T, 64, 2>(p, s)
                                                                                  : launch_decode<T, 64, 4>(p, s);
    if (p.D == 128) return rows <= 32 ? launch_decode<T, 128, 1>(p, s) : launch_decode<T, 128, 2>(p, s);
    return launch_decode<T, 256, 1>(p, s);
  }
  if (al) return launch_flash_for<T>(p, ext, s);
  const long rows = (long)B * Hq * Sq;
  hipLaunchKernelGGL((flash_fwd_generic_kernel<T>), dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, p);
  return launch_status();
}

template <class T>
int flash_strided(const void* Q, const void* K, const void* V, void* O, void* LSE, int B, int Hq, int Hkv, int Sq,
                  int Sk, int D, const int64_t* strides, float scale, int causal, int window, float softcap,
                  int out_dtype, void* stream) {
  if (!strides) return kBadShape;
  FlashStrides st[4];
  for (int i = 0; i < 4; ++i) st[i] = FlashStrides{(long)strides[3 * i], (long)strides[3 * i + 1], (long)strides[3 * i + 2]};
  return flash_dev<T>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream), window,
                      softcap, nullptr, st);
}

template <class T>
int flash_host(const void* Q, const void* K, const void* V, void* O, void* LSE, int B, int Hq, int Hkv,
               int Sq, int Sk, int D, float scale, int causal, int window = 0, float softcap = 0.f,
               const float* bias = nullptr) {
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || !Q || !K || !V || !O) return kBadShape;
  if (window < 0 || !(softcap >= 0.f)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t q_bytes = (size_t)B * Hq * Sq * D * 2, kv_bytes = (size_t)B * Hkv * Sk * D * 2;
  const size_t o_bytes = (size_t)B * Hq * Sq * D * 4, l_bytes = (size_t)B * Hq * Sq * 4;
  DeviceScope scope;
  void* dQ = scope.alloc(q_bytes, Q);
  void* dK = scope.alloc(kv_bytes, K);
  void* dV = scope.alloc(kv_bytes, V);
  void* dO = scope.alloc(o_bytes);
  void* dL = LSE ? scope.alloc(l_bytes) : nullptr;
  void* dBias = bias ? scope.alloc((size_t)B * Hq * Sq * Sk * 4, bias) : nullptr;
  if (scope.failed()) return kDeviceFailed;
  int rc = flash_dev<T>(dQ, dK, dV, dO, dL, B, Hq, Hkv, Sq, Sk, D, scale, causal, 0, nullptr, window, softcap,
                        static_cast<const float*>(dBias));
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(O, dO, o_bytes)) return kDeviceFailed;
  if (LSE && !scope.download(LSE, dL, l_bytes)) return kDeviceFailed;
  return kOk;
}

template <class T, int D>
int launch_bwd(const FlashBwdParams& p, hipStream_t s) {
  constexpr int kDqSmem = 4 * FB_BKV * D * 2;
  constexpr int kDkvSmem = flash_bwd_dkdv_lds_bytes<D>();
  auto dq_kern = flash_bwd_dq_kernel<T, D>;
  auto dkv_kern = flash_bwd_dkdv_kernel<T, D>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(dq_kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kDqSmem);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(dkv_kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kDkvSmem);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  hipLaunchKernelGGL(dq_kern, dim3(ceil_div(p.Sq, FB_BQ) * p.B * p.Hq), dim3(FB_DQ_THREADS), kDqSmem, s, p);
  if (int rc = launch_status(); rc != kOk) return rc;
  hipLaunchKernelGGL(dkv_kern, dim3(ceil_div(p.Sk, FB_BK) * p.B * p.Hkv), dim3(FB_DKV_THREADS), kDkvSmem, s, p);
  return launch_status();
}

// Rows of `src_chunks` 16-byte chunks copied into rows of `dst_chunks`: a wider destination is
// zero-filled behind the source's columns, a narrower one takes the leading columns.
__global__ void __launch_bounds__(256) repitch_rows_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                           long rows, int src_chunks, int dst_chunks) {
  const long total = rows * dst_chunks;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long r = i / dst_chunks;
    const int c = (int)(i - r * dst_chunks);
    dst[i] = c < src_chunks ? src[r * src_chunks + c] : make_uint4(0u, 0u, 0u, 0u);
  }
}
inline void repitch_rows(void* dst, const void* src, long rows, int src_bytes, int dst_bytes, hipStream_t s) {
  const long total = rows * (dst_bytes / 16);
  const long blocks = (total + 255) / 256;
  hipLaunchKernelGGL(repitch_rows_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, s,
                     static_cast<uint4*>(dst), static_cast<const uint4*>(src), rows, src_bytes / 16, dst_bytes / 16);
}

template <class T>
int flash_bwd_dev(const void* dO, const void* Q, const void* K, const void* V, const float* O, const float* LSE,
                  float* dQ, float* dK, float* dV, int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                  int causal, hipStream_t s);

// Head dimensions below 128 other than 64: the MFMA kernels are compiled for 64 and 128, so the
// operands are copied into zero-padded rows of the next compiled width (zero columns of Q, K, V
// and dO change no score, no dP and no Delta, and yield zero gradient columns), the kernels run
// at that width, and the leading D columns of the gradients are copied out.  The forward's O
// and log-sum-exp are taken from the caller or recomputed at the real width.
template <class T>
int flash_bwd_padded_dev(const void* dO, const void* Q, const void* K, const void* V, const float* O,
                         const float* LSE, float* dQ, float* dK, float* dV, int B, int Hq, int Hkv, int Sq, int Sk,
                         int D, float scale, int causal, hipStream_t s) {
  const int DP = D < 64 ? 64 : 128;
  const size_t rows = (size_t)B * Hq * Sq, kvrows = (size_t)B * Hkv * Sk;
  const bool recompute = !O || !LSE;
  // 16-bit: Qp dOp (rows) Kp Vp (kvrows); f32: Op dQp (rows) dKp dVp (kvrows) [+ O, LSE at the real width]
  const size_t b16q = rows * DP * 2, b16k = kvrows * DP * 2, f32q = rows * DP * 4, f32k = kvrows * DP * 4;
  const size_t extra = recompute ? rows * D * 4 + rows * 4 : 0;
  char* ws = nullptr;
  if (hipMallocAsync(reinterpret_cast<void**>(&ws), 2 * b16q + 2 * b16k + 2 * f32q + 2 * f32k + extra, s) != hipSuccess) {
    (void)hipGetLastError();
    return kDeviceFailed;
  }
  char* Qp = ws; char* dOp = Qp + b16q; char* Kp = dOp + b16q; char* Vp = Kp + b16k;
  char* Op = Vp + b16k; char* dQp = Op + f32q; char* dKp = dQp + f32q; char* dVp = dKp + f32k;
  int rc = kOk;
  if (recompute) {
    float* o_ws = reinterpret_cast<float*>(dVp + f32k);
    float* lse_ws = o_ws + rows * D;
    rc = flash_dev<T>(Q, K, V, o_ws, lse_ws, B, Hq, Hkv, Sq, Sk, D, scale, causal, 0, s);
    O = o_ws;
    LSE = lse_ws;
  }
  if (rc == kOk) {
    repitch_rows(Qp, Q, (long)rows, D * 2, DP * 2, s);
    repitch_rows(dOp, dO, (long)rows, D * 2, DP * 2, s);
    repitch_rows(Kp, K, (long)kvrows, D * 2, DP * 2, s);
    repitch_rows(Vp, V, (long)kvrows, D * 2, DP * 2, s);
    repitch_rows(Op, O, (long)rows, D * 4, DP * 4, s);
    rc = launch_status();
  }
  if (rc == kOk)
    rc = flash_bwd_dev<T>(dOp, Qp, Kp, Vp, reinterpret_cast<const float*>(Op), LSE, reinterpret_cast<float*>(dQp),
                          reinterpret_cast<float*>(dKp), reinterpret_cast<float*>(dVp), B, Hq, Hkv, Sq, Sk, DP, scale,
                          causal, s);
  if (rc == kOk) {
    repitch_rows(dQ, dQp, (long)rows, DP * 4, D * 4, s);
    repitch_rows(dK, dKp, (long)kvrows, DP * 4, D * 4, s);
    repitch_rows(dV, dVp, (long)kvrows, DP * 4, D * 4, s);
    rc = launch_status();
  }
  if (hipFreeAsync(ws, s) != hipSuccess) { (void)hipGetLastError(); rc = rc == kOk ? kDeviceFailed : rc; }
  return rc;
}

// ---- backward for head dimensions above 128, as dense products ------------------------------
// The flash kernels hold a query (or key) block's accumulators and operand fragments in
// registers, which stops at D = 128.  Above it the backward of one (batch, KV head) group is five
// dense products on the GEMM kernels around one elementwise kernel, with S and dP of the group
// written out (rows = (Hq / Hkv) Sq query rows of the group's heads, one after the other):
//   S  = Qg K^T, dP = dOg V^T                     [rows, Sk] f32   (K^T, V^T: transposed copies)
//   P  = exp(scale S - LSE),  dS = scale P (dP - Delta), masked  -> dS [rows, Sk], P^T, dS^T [Sk, rows]
//   dQg = dS K,   dV = P^T dOg,   dK = dS^T Qg    (the sums over the group's heads are part of
//                                                  the last two contractions)
// At D = 256 a score costs 2 D = 512 multiply-adds per product against 14 bytes of S, dP, P and
// dS traffic, so the dense form stays within a small factor of a fused kernel; it does not skip
// the masked half of a causal problem.  Groups are processed in chunks that bound the scratch.

// dst[z][c][r] = src[z][r][c], 16-bit elements, 64 x 64 tiles through LDS.
__global__ __launch_bounds__(256) void transpose16_kernel(uint16_t* __restrict__ dst, const uint16_t* __restrict__ src,
                                                          int R, int C) {
  __shared__ uint16_t tile[64][66];
  const long z = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4)
    if (r0 + i < R && c0 + tx < C) tile[i][tx] = src[(z * R + r0 + i) * C + c0 + tx];
  __syncthreads();
  for (int i = ty; i < 64; i += 4)
    if (c0 + i < C && r0 + tx < R) dst[(z * C + c0 + i) * R + r0 + tx] = tile[tx][i];
}

// One 64 x 64 tile of (rows, keys) per workgroup: P and dS from S and dP (see above).  Row r of
// group z is query r % Sq of the group's head r / Sq; lse / delta are indexed [z][r].
template <class T>
__global__ __launch_bounds__(256) void bwd_dense_softmax_kernel(const float* __restrict__ S, const float* __restrict__ dP,
                                                                const float* __restrict__ lse,
                                                                const float* __restrict__ delta, uint16_t* __restrict__ dS,
                                                                uint16_t* __restrict__ PT, uint16_t* __restrict__ dST,
                                                                int rows, int Sq, int Sk, float scale, int causal) {
  __shared__ uint16_t pt[64][66], dst[64][66];
  const long z = blockIdx.z;
  const int r0 = blockIdx.y * 64, k0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int off = Sk > Sq ? Sk - Sq : 0;
  const int key = k0 + tx;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i;
    uint16_t pb = 0, db = 0;
    if (r < rows && key < Sk) {
      const long at = (z * rows + r) * Sk + key;
      const int q = r % Sq;
      const bool seen = !causal || key <= q + off;
      float pv = 0.f, dv = 0.f;
      if (seen) {
        pv = __expf(scale * S[at] - lse[z * rows + r]);
        dv = scale * pv * (dP[at] - delta[z * rows + r]);
      }
      pb = to_storage<T>(pv);
      db = to_storage<T>(dv);
      dS[at] = db;
    }
    pt[i][tx] = pb;
    dst[i][tx] = db;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int k = k0 + i, r = r0 + tx;
    if (k < Sk && r < rows) {
      const long at = (z * Sk + k) * rows + r;
      PT[at] = pt[tx][i];
      dST[at] = dst[tx][i];
    }
  }
}

template <class T>
int gemm_f32_batched(const void* A, const void* B, void* D, int batch, int M, int N, int K, long sa, long sb, long sd,
                     hipStream_t s) {
  if constexpr (std::is_same<T, BF16>::value)
    return tessera_gfx950_batched_gemm_strided_bf16_dev(A, B, D, batch, M, N, K, sa, sb, sd, 0, s);
  else
    return tessera_gfx950_batched_gemm_strided_f16_dev(A, B, D, batch, M, N, K, sa, sb, sd, 0, s);
}

// O and LSE as saved by the forward (not null), Delta scratch [B Hq Sq] from the caller.
template <class T>
int flash_bwd_dense_dev(const void* dO, const void* Q, const void* K, const void* V, const float* LSE, const float* Delta,
                        float* dQ, float* dK, float* dV, int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                        int causal, hipStream_t s) {
  const int ratio = Hq / Hkv, groups = B * Hkv;
  const long rows = (long)ratio * Sq;
  // per group: S, dP f32; dS, P^T, dS^T 16-bit; K^T, V^T 16-bit
  const size_t per_group = (size_t)rows * Sk * (4 + 4 + 2 + 2 + 2) + (size_t)2 * Sk * D * 2;
  const size_t budget = (size_t)2 << 30;                                      // aim for 2 GiB of scratch per chunk
  const int gpc = (int)std::max<size_t>(1, std::min<size_t>(groups, budget / per_group));
  char* ws = nullptr;
  if (hipMallocAsync(reinterpret_cast<void**>(&ws), per_group * gpc + 256, s) != hipSuccess) {
    (void)hipGetLastError();
    return kDeviceFailed;
  }
  const size_t e = (size_t)rows * Sk;
  float* Sb = reinterpret_cast<float*>(ws);
  float* dPb = Sb + e * gpc;
  uint16_t* dSb = reinterpret_cast<uint16_t*>(dPb + e * gpc);
  uint16_t* PTb = dSb + e * gpc;
  uint16_t* dSTb = PTb + e * gpc;
  uint16_t* KTb = dSTb + e * gpc;
  uint16_t* VTb = KTb + (size_t)Sk * D * gpc;
  const uint16_t* Qp = static_cast<const uint16_t*>(Q);
  const uint16_t* Kp = static_cast<const uint16_t*>(K);
  const uint16_t* Vp = static_cast<const uint16_t*>(V);
  const uint16_t* dOp = static_cast<const uint16_t*>(dO);
  int rc = kOk;
  for (int g0 = 0; g0 < groups && rc == kOk; g0 += gpc) {
    const int n = std::min(gpc, groups - g0);
    const long qo = (long)g0 * rows * D, ko = (long)g0 * Sk * D;
    const dim3 tgrid(ceil_div(D, 64), ceil_div(Sk, 64), n);
    hipLaunchKernelGGL(transpose16_kernel, tgrid, dim3(256), 0, s, KTb, Kp + ko, Sk, D);
    hipLaunchKernelGGL(transpose16_kernel, tgrid, dim3(256), 0, s, VTb, Vp + ko, Sk, D);
    rc = launch_status();
    if (rc == kOk) rc = gemm_f32_batched<T>(Qp + qo, KTb, Sb, n, (int)rows, Sk, D, rows * D, (long)D * Sk, (long)e, s);
    if (rc == kOk) rc = gemm_f32_batched<T>(dOp + qo, VTb, dPb, n, (int)rows, Sk, D, rows * D, (long)D * Sk, (long)e, s);
    if (rc != kOk) break;
    hipLaunchKernelGGL((bwd_dense_softmax_kernel<T>), dim3(ceil_div(Sk, 64), (unsigned)ceil_div((int)rows, 64), n), dim3(256), 0,
                       s, Sb, dPb, LSE + (long)g0 * rows, Delta + (long)g0 * rows, dSb, PTb, dSTb, (int)rows, Sq, Sk, scale,
                       causal);
    rc = launch_status();
    if (rc == kOk) rc = gemm_f32_batched<T>(dSb, Kp + ko, dQ + qo, n, (int)rows, D, Sk, (long)e, (long)Sk * D, rows * D, s);
    if (rc == kOk) rc = gemm_f32_batched<T>(PTb, dOp + qo, dV + ko, n, Sk, D, (int)rows, (long)e, rows * D, (long)Sk * D, s);
    if (rc == kOk) rc = gemm_f32_batched<T>(dSTb, Qp + qo, dK + ko, n, Sk, D, (int)rows, (long)e, rows * D, (long)Sk * D, s);
  }
  if (hipFreeAsync(ws, s) != hipSuccess) { (void)hipGetLastError(); rc = rc == kOk ? kDeviceFailed : rc; }
  return rc;
}

// (dQ, dK, dV) from (dO, Q, K, V).  O and LSE may be passed in (saved by the forward
// call); when either is null the forward kernel is run first to recompute both.
template <class T>
int flash_bwd_dev(const void* dO, const void* Q, const void* K, const void* V, const float* O, const float* LSE,
                  float* dQ, float* dK, float* dV, int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                  int causal, hipStream_t s) {
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || !dO || !Q || !K || !V || !dQ || !dK || !dV) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t rows = (size_t)B * Hq * Sq;
  const bool recompute = !O || !LSE;
  float* ws = nullptr;                       // Delta (rows) | LSE2 (rows) | [O (rows * D) | LSE (rows)]?
  // The MFMA kernels fold -LSE / scale into their accumulators: they need a scale it
  // can be divided by; anything else takes the generic kernels.
  const bool scale_ok = std::isfinite(scale) && std::fabs(scale) >= 1e-20f;
  {
    const bool al_in = ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(V) |
                         reinterpret_cast<uintptr_t>(dO) | reinterpret_cast<uintptr_t>(dQ) | reinterpret_cast<uintptr_t>(dK) |
                         reinterpret_cast<uintptr_t>(dV) | reinterpret_cast<uintptr_t>(O)) & 15) == 0;
    if (al_in && scale_ok && D < 128 && D != 64)
      return flash_bwd_padded_dev<T>(dO, Q, K, V, O, LSE, dQ, dK, dV, B, Hq, Hkv, Sq, Sk, D, scale, causal, s);
  }
  const size_t ws_floats = 2 * rows + (recompute ? rows * D + rows : 0);
  if (hipMallocAsync(reinterpret_cast<void**>(&ws), ws_floats * sizeof(float), s) != hipSuccess) {
    (void)hipGetLastError();
    return kDeviceFailed;
  }
  int rc = kOk;
  float* delta = ws;
  if (recompute) {
    float* o_ws = ws + 2 * rows;
    float* lse_ws = o_ws + rows * D;
    rc = flash_dev<T>(Q, K, V, o_ws, lse_ws, B, Hq, Hkv, Sq, Sk, D, scale, causal, 0, s);
    O = o_ws;
    LSE = lse_ws;
  }
  if (rc == kOk) {
    FlashBwdParams p{};
    p.Q = static_cast<const uint16_t*>(Q);
    p.K = static_cast<const uint16_t*>(K);
    p.V = static_cast<const uint16_t*>(V);
    p.dO = static_cast<const uint16_t*>(dO);
    p.O = O; p.LSE = LSE; p.Delta = delta; p.LSE2 = ws + rows;
    p.dQ = dQ; p.dK = dK; p.dV = dV;
    p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Sq = Sq; p.Sk = Sk;
    p.scale = scale;
    p.causal = causal ? 1 : 0;
    const bool al = ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) |
                      reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(dO) |
                      reinterpret_cast<uintptr_t>(dQ) | reinterpret_cast<uintptr_t>(dK) |
                      reinterpret_cast<uintptr_t>(dV)) & 15) == 0;
    const bool mfma = al && scale_ok && (D == 128 || D == 64);
    hipLaunchKernelGGL((flash_bwd_delta_kernel<T>), dim3((unsigned)((rows * 16 + 255) / 256)), dim3(256), 0, s,
                       p.dO, p.O, p.LSE, delta, p.LSE2, (long)rows, D, mfma ? -1.f : 1.f,
                       mfma ? -1.f / scale : 1.f);
    rc = launch_status();
    if (rc == kOk) {
      if (mfma && D == 128) rc = launch_bwd<T, 128>(p, s);
      else if (mfma) rc = launch_bwd<T, 64>(p, s);
      else if (al && D > 128 && std::isfinite(scale) && (long)(Hq / Hkv) * Sq * Sk <= (1L << 33))   // (else: 112 GiB of scratch a group)
        rc = flash_bwd_dense_dev<T>(dO, Q, K, V, LSE, delta, dQ, dK, dV, B, Hq, Hkv, Sq, Sk, D, scale, causal, s);
      else {
        const long kvrows = (long)B * Hkv * Sk;
        hipLaunchKernelGGL((flash_bwd_generic_dq_kernel<T>), dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, p, D);
        hipLaunchKernelGGL((flash_bwd_generic_dkdv_kernel<T>), dim3((unsigned)((kvrows + 63) / 64)), dim3(64), 0, s,
                           p, D);
        rc = launch_status();
      }
    }
  }
  if (hipFreeAsync(ws, s) != hipSuccess) { (void)hipGetLastError(); rc = rc == kOk ? kDeviceFailed : rc; }
  return rc;
}

template <class T>
int flash_bwd_host(const void* dO, const void* Q, const void* K, const void* V, void* dQ, void* dK, void* dV, int B,
                   int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal) {
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || !dO || !Q || !K || !V || !dQ || !dK || !dV) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t q_elems = (size_t)B * Hq * Sq * D, kv_elems = (size_t)B * Hkv * Sk * D;
  DeviceScope scope;
  void* ddO = scope.alloc(q_elems * 2, dO);
  void* dQin = scope.alloc(q_elems * 2, Q);
  void* dKin = scope.alloc(kv_elems * 2, K);
  void* dVin = scope.alloc(kv_elems * 2, V);
  void* gQ = scope.alloc(q_elems * 4);
  void* gK = scope.alloc(kv_elems * 4);
  void* gV = scope.alloc(kv_elems * 4);
  if (scope.failed()) return kDeviceFailed;
  int rc = flash_bwd_dev<T>(ddO, dQin, dKin, dVin, nullptr, nullptr, static_cast<float*>(gQ),
                            static_cast<float*>(gK), static_cast<float*>(gV), B, Hq, Hkv, Sq, Sk, D, scale, causal,
                            nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(dQ, gQ, q_elems * 4) || !scope.download(dK, gK, kv_elems * 4) ||
      !scope.download(dV, gV, kv_elems * 4))
    return kDeviceFailed;
  return kOk;
}

}  // namespace
}  // namespace tsr950

using namespace tsr950;

extern "C" {

int tessera_gfx950_flash_attn_f16(const void* Q, const void* K, const void* V, void* O, int B, int H, int Sq,
                                  int Sk, int D, float scale, int causal) {
  return flash_host<F16>(Q, K, V, O, nullptr, B, H, H, Sq, Sk, D, scale, causal);
}
int tessera_gfx950_flash_attn_bf16(const void* Q, const void* K, const void* V, void* O, int B, int H, int Sq,
                                   int Sk, int D, float scale, int causal) {
  return flash_host<BF16>(Q, K, V, O, nullptr, B, H, H, Sq, Sk, D, scale, causal);
}
int tessera_gfx950_flash_attn_gqa_f16(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                      int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal) {
  return flash_host<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal);
}
int tessera_gfx950_flash_attn_gqa_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                       int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal) {
  return flash_host<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal);
}
int tessera_gfx950_flash_attn_gqa_f16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                          int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                          int causal, int out_dtype, void* stream) {
  return flash_dev<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream));
}
int tessera_gfx950_flash_attn_bf16_bench(int B, int Hq, int Hkv, int Sq, int Sk, int D, int causal, int iters,
                                         double* avg_ms) {
  g_last_timer_source = -1;
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || iters <= 0 || !avg_ms) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  const size_t q_bytes = (size_t)B * Hq * Sq * D * 2, kv_bytes = (size_t)B * Hkv * Sk * D * 2;
  void* dQ = scope.alloc(q_bytes);
  void* dK = scope.alloc(kv_bytes);
  void* dV = scope.alloc(kv_bytes);
  void* dO = scope.alloc(q_bytes);
  void* dL = scope.alloc((size_t)B * Hq * Sq * 4);
  if (scope.failed()) return kDeviceFailed;
  // 0x3c3c: finite, non-trivial bf16 values
  if (hipMemset(dQ, 0x3c, q_bytes) != hipSuccess || hipMemset(dK, 0x3c, kv_bytes) != hipSuccess ||
      hipMemset(dV, 0x3c, kv_bytes) != hipSuccess)
    return kDeviceFailed;
  const float scale = 1.0f / std::sqrt((float)D);
  return bench_loop([&](int) { return flash_dev<BF16>(dQ, dK, dV, dO, dL, B, Hq, Hkv, Sq, Sk, D, scale, causal, 1, nullptr); },
                    iters, avg_ms);
}

int tessera_gfx950_flash_attn_gqa_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                           int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                           int causal, int out_dtype, void* stream) {
  return flash_dev<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream));
}

int tessera_gfx950_flash_attn_ext_f16(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                      int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal, int window,
                                      float softcap) {
  return flash_host<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, window, softcap);
}
int tessera_gfx950_flash_attn_ext_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                       int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal, int window,
                                       float softcap) {
  return flash_host<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, window, softcap);
}
int tessera_gfx950_flash_attn_ext_f16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                          int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal,
                                          int window, float softcap, int out_dtype, void* stream) {
  return flash_dev<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream), window,
                        softcap);
}
int tessera_gfx950_flash_attn_ext_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                           int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal,
                                           int window, float softcap, int out_dtype, void* stream) {
  return flash_dev<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream), window,
                         softcap);
}

int tessera_gfx950_flash_attn_strided_f16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                              int Hq, int Hkv, int Sq, int Sk, int D, const int64_t* strides,
                                              float scale, int causal, int window, float softcap, int out_dtype,
                                              void* stream) {
  return flash_strided<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, strides, scale, causal, window, softcap, out_dtype,
                            stream);
}
int tessera_gfx950_flash_attn_strided_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                               int Hq, int Hkv, int Sq, int Sk, int D, const int64_t* strides,
                                               float scale, int causal, int window, float softcap, int out_dtype,
                                               void* stream) {
  return flash_strided<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, strides, scale, causal, window, softcap,
                             out_dtype, stream);
}

int tessera_gfx950_flash_attn_bias_f16(const void* Q, const void* K, const void* V, const float* bias, void* O,
                                       void* LSE, int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                       int causal, int window, float softcap) {
  return flash_host<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, window, softcap, bias);
}
int tessera_gfx950_flash_attn_bias_bf16(const void* Q, const void* K, const void* V, const float* bias, void* O,
                                        void* LSE, int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                        int causal, int window, float softcap) {
  return flash_host<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, window, softcap, bias);
}
int tessera_gfx950_flash_attn_bias_f16_dev(const void* Q, const void* K, const void* V, const float* bias,
                                           void* O, void* LSE, int B, int Hq, int Hkv, int Sq, int Sk, int D,
                                           float scale, int causal, int window, float softcap, int out_dtype,
                                           void* stream) {
  return flash_dev<F16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream), window,
                        softcap, bias);
}
int tessera_gfx950_flash_attn_bias_bf16_dev(const void* Q, const void* K, const void* V, const float* bias,
                                            void* O, void* LSE, int B, int Hq, int Hkv, int Sq, int Sk, int D,
                                            float scale, int causal, int window, float softcap, int out_dtype,
                                            void* stream) {
  return flash_dev<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream), window,
                         softcap, bias);
}

int tessera_gfx950_flash_attn_bwd_f16(const void* dO, const void* Q, const void* K, const void* V, void* dQ,
                                      void* dK, void* dV, int B, int Hq, int Hkv, int Sq, int Sk, int D,
                                      float scale, int causal) {
  return flash_bwd_host<F16>(dO, Q, K, V, dQ, dK, dV, B, Hq, Hkv, Sq, Sk, D, scale, causal);
}
int tessera_gfx950_flash_attn_bwd_bf16(const void* dO, const void* Q, const void* K, const void* V, void* dQ,
                                       void* dK, void* dV, int B, int Hq, int Hkv, int Sq, int Sk, int D,
                                       float scale, int causal) {
  return flash_bwd_host<BF16>(dO, Q, K, V, dQ, dK, dV, B, Hq, Hkv, Sq, Sk, D, scale, causal);
}
int tessera_gfx950_flash_attn_bwd_f16_dev(const void* dO, const void* Q, const void* K, const void* V,
                                          const void* O, const void* LSE, void* dQ, void* dK, void* dV, int B,
                                          int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal,
                                          void* stream) {
  return flash_bwd_dev<F16>(dO, Q, K, V, static_cast<const float*>(O), static_cast<const float*>(LSE),
                            static_cast<float*>(dQ), static_cast<float*>(dK), static_cast<float*>(dV), B, Hq, Hkv,
                            Sq, Sk, D, scale, causal, as_stream(stream));
}
int tessera_gfx950_flash_attn_bwd_bf16_dev(const void* dO, const void* Q, const void* K, const void* V,
                                           const void* O, const void* LSE, void* dQ, void* dK, void* dV, int B,
                                           int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal,
                                           void* stream) {
  return flash_bwd_dev<BF16>(dO, Q, K, V, static_cast<const float*>(O), static_cast<const float*>(LSE),
                             static_cast<float*>(dQ), static_cast<float*>(dK), static_cast<float*>(dV), B, Hq, Hkv,
                             Sq, Sk, D, scale, causal, as_stream(stream));
}

}  // extern "C"
