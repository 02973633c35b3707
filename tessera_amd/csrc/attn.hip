// C ABI: flash-attention forward (causal, GQA, LSE), 16-bit storage.
#include <mutex>
#include "../../include/tessera_gfx950.h"
#include "flash_attn.h"
#include "host_util.h"

namespace tsr950 {
namespace {

bool bad_attn(int B, int Hq, int Hkv, int Sq, int Sk, int D) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq <= 0 || Sk <= 0 || D <= 0) return true;
  if (D % 16 != 0 || D > 256) return true;       // matrix-core lanes need head_dim % 16 == 0
  if (Hq % Hkv != 0) return true;
  return false;
}

template <class T, int D>
int launch_flash(const FlashParams& p, hipStream_t s) {
  constexpr int kSmem = 2 * 2 * FA_BKV * D * 2;
  auto kern = flash_fwd_kernel<T, D>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  });
  if (attr_err != hipSuccess) return kDeviceFailed;
  dim3 grid(ceil_div(p.Sq, FA_BQ) * p.B * p.Hq, 1, 1);
  hipLaunchKernelGGL(kern, grid, dim3(FA_THREADS), kSmem, s, p);
  return launch_status();
}

template <class T>
int flash_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B, int Hq, int Hkv,
              int Sq, int Sk, int D, float scale, int causal, int out_storage, hipStream_t s) {
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || !Q || !K || !V || !O) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  FlashParams p{};
  p.Q = static_cast<const uint16_t*>(Q);
  p.K = static_cast<const uint16_t*>(K);
  p.V = static_cast<const uint16_t*>(V);
  p.O = O;
  p.LSE = static_cast<float*>(LSE);
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Sq = Sq; p.Sk = Sk;
  p.scale = scale;
  p.causal = causal ? 1 : 0;
  p.out_storage = out_storage ? 1 : 0;
  const bool al = ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) |
                    reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(O)) & 15) == 0;
  if (al && D == 128) return launch_flash<T, 128>(p, s);
  if (al && D == 64) return launch_flash<T, 64>(p, s);
  const long rows = (long)B * Hq * Sq;
  hipLaunchKernelGGL((flash_fwd_generic_kernel<T>), dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, p, D);
  return launch_status();
}

template <class T>
int flash_host(const void* Q, const void* K, const void* V, void* O, void* LSE, int B, int Hq, int Hkv,
               int Sq, int Sk, int D, float scale, int causal) {
  if (bad_attn(B, Hq, Hkv, Sq, Sk, D) || !Q || !K || !V || !O) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t q_bytes = (size_t)B * Hq * Sq * D * 2, kv_bytes = (size_t)B * Hkv * Sk * D * 2;
  const size_t o_bytes = (size_t)B * Hq * Sq * D * 4, l_bytes = (size_t)B * Hq * Sq * 4;
  DeviceScope scope;
  void* dQ = scope.alloc(q_bytes, Q);
  void* dK = scope.alloc(kv_bytes, K);
  void* dV = scope.alloc(kv_bytes, V);
  void* dO = scope.alloc(o_bytes);
  void* dL = LSE ? scope.alloc(l_bytes) : nullptr;
  if (scope.failed()) return kDeviceFailed;
  int rc = flash_dev<T>(dQ, dK, dV, dO, dL, B, Hq, Hkv, Sq, Sk, D, scale, causal, 0, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  if (!scope.download(O, dO, o_bytes)) return kDeviceFailed;
  if (LSE && !scope.download(LSE, dL, l_bytes)) return kDeviceFailed;
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
int tessera_gfx950_flash_attn_gqa_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                           int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                           int causal, int out_dtype, void* stream) {
  return flash_dev<BF16>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, out_dtype, as_stream(stream));
}

}  // extern "C"
