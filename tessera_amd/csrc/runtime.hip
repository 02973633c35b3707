// Device management half of the C ABI: probe, raw buffers, event timers.
#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>
#include "../../include/tessera_gfx950.h"
#include "host_util.h"

namespace tsr950 {

thread_local int g_last_timer_source = -1;

std::recursive_mutex& host_call_mutex() {
  static std::recursive_mutex mu;
  return mu;
}

int probe_device() {
  static std::once_flag once;
  static int cached = kNoDevice;
  std::call_once(once, [] {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) { (void)hipGetLastError(); return; }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) { (void)hipGetLastError(); return; }
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) return;
    if (hipSetDevice(0) != hipSuccess) { (void)hipGetLastError(); return; }
    cached = kOk;
    // Device addresses of the library's own device arrays are looked up here, once, so that no
    // entry point does it inside a caller's stream capture.  A failure is reported by the entry
    // point that needs the array.
    (void)route_scratch_warm();
  });
  return cached;
}

namespace {
struct WorkspaceSlot {
  void* ptr = nullptr;
  size_t bytes = 0;
  std::vector<void*> retired;      // outgrown buffers: work queued before the growth may still use them
};
std::mutex g_ws_mu;
std::map<std::pair<int, hipStream_t>, WorkspaceSlot> g_ws_slots;
}  // namespace

void* stream_workspace(hipStream_t s, size_t bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  std::lock_guard<std::mutex> lock(g_ws_mu);
  WorkspaceSlot& slot = g_ws_slots[{dev, s}];
  if (slot.bytes >= bytes && slot.ptr) return slot.ptr;
  // Work already queued on the stream may still use the old buffer, so it is neither
  // freed nor waited for: it is set aside, and the new one is at least twice its size,
  // which bounds everything set aside by the size of the buffer in use.
  size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
  if (want < 2 * slot.bytes) want = 2 * slot.bytes;
  void* p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  if (slot.ptr) slot.retired.push_back(slot.ptr);
  slot.ptr = p;
  slot.bytes = want;
  return p;
}

// Waits for the stream, then frees its workspace (the buffer in use and the outgrown ones).
int stream_workspace_release(hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return kDeviceFailed; }
  if (hipStreamSynchronize(s) != hipSuccess) { (void)hipGetLastError(); return kDeviceFailed; }
  WorkspaceSlot gone;
  {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    auto it = g_ws_slots.find({dev, s});
    if (it == g_ws_slots.end()) return kOk;
    gone = std::move(it->second);
    g_ws_slots.erase(it);
  }
  int rc = kOk;
  if (gone.ptr && hipFree(gone.ptr) != hipSuccess) rc = kDeviceFailed;
  for (void* p : gone.retired)
    if (hipFree(p) != hipSuccess) rc = kDeviceFailed;
  if (rc != kOk) (void)hipGetLastError();
  return rc;
}

struct Timer {
  hipEvent_t start, stop;
};

// Grid-stride 16-byte copy: one coalesced global_load_dwordx4 / store per lane.
__global__ void __launch_bounds__(256) copy16_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

}  // namespace tsr950

using namespace tsr950;

extern "C" {

int tessera_gfx950_abi_version(void) { return 1; }

int tessera_gfx950_probe(void) { return probe_device(); }

int tessera_gfx950_stream_release(void* stream) {
  if (probe_device() != kOk) return kNoDevice;
  return stream_workspace_release(as_stream(stream));
}

int tessera_gfx950_device_name(char* buf, int buflen) {
  if (!buf || buflen <= 0) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return kDeviceFailed;
  char tmp[512];
  snprintf(tmp, sizeof tmp, "%s (%s)", prop.name, prop.gcnArchName);
  std::strncpy(buf, tmp, (size_t)buflen - 1);
  buf[buflen - 1] = 0;
  return kOk;
}

int tessera_gfx950_device_cus(int* cus) {
  if (!cus) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return kDeviceFailed;
  *cus = prop.multiProcessorCount;
  return kOk;
}

int tessera_gfx950_malloc(void** dptr, size_t bytes) {
  if (!dptr) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  return finish(hipMalloc(dptr, bytes < 16 ? 16 : bytes));
}

int tessera_gfx950_free(void* dptr) {
  if (!dptr) return kOk;
  if (probe_device() != kOk) return kNoDevice;
  return finish(hipFree(dptr));
}

int tessera_gfx950_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  if (bytes && (!dst || !src)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  return bytes ? finish(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice)) : kOk;
}

int tessera_gfx950_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  if (bytes && (!dst || !src)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  return bytes ? finish(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost)) : kOk;
}

int tessera_gfx950_memset(void* dst, int value, size_t bytes) {
  if (bytes && !dst) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  return bytes ? finish(hipMemset(dst, value, bytes)) : kOk;
}

int tessera_gfx950_memcpy_d2d_dev(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes && (!dst || !src)) return kBadShape;
  if (bytes % 16 != 0 || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (!bytes) return kOk;
  const size_t n = bytes / 16;
  const size_t want = (n + 255) / 256;
  const unsigned grid = (unsigned)(want < 256 * 32 ? want : 256 * 32);
  hipLaunchKernelGGL(copy16_kernel, dim3(grid), dim3(256), 0, as_stream(stream),
                     static_cast<uint4*>(dst), static_cast<const uint4*>(src), n);
  return launch_status();
}

int tessera_gfx950_synchronize(void) {
  if (probe_device() != kOk) return kNoDevice;
  return finish(hipDeviceSynchronize());
}

int tessera_gfx950_timer_create(void** timer) {
  if (!timer) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  Timer* t = new (std::nothrow) Timer;
  if (!t) return kDeviceFailed;
  if (hipEventCreate(&t->start) != hipSuccess) { delete t; return kDeviceFailed; }
  if (hipEventCreate(&t->stop) != hipSuccess) { (void)hipEventDestroy(t->start); delete t; return kDeviceFailed; }
  *timer = t;
  return kOk;
}

int tessera_gfx950_timer_start(void* timer, void* stream) {
  if (!timer) return kBadShape;
  return finish(hipEventRecord(static_cast<Timer*>(timer)->start, as_stream(stream)));
}

int tessera_gfx950_timer_stop(void* timer, void* stream) {
  if (!timer) return kBadShape;
  return finish(hipEventRecord(static_cast<Timer*>(timer)->stop, as_stream(stream)));
}

int tessera_gfx950_timer_elapsed_ms(void* timer, float* ms) {
  if (!timer || !ms) return kBadShape;
  Timer* t = static_cast<Timer*>(timer);
  if (hipEventSynchronize(t->stop) != hipSuccess) return kDeviceFailed;
  return finish(hipEventElapsedTime(ms, t->start, t->stop));
}

int tessera_gfx950_timer_destroy(void* timer) {
  if (!timer) return kOk;
  Timer* t = static_cast<Timer*>(timer);
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
  return kOk;
}

}  // extern "C"

// ---- the reference C runtime's launch bridge ------------------------------------------
namespace {
constexpr int kTsrSuccess = 0, kTsrInvalidArgument = 1, kTsrNotFound = 2, kTsrDeviceError = 7;
int tsr_status_of(int rc) {
  return rc == tsr950::kOk ? kTsrSuccess : rc == tsr950::kBadShape ? kTsrInvalidArgument : kTsrDeviceError;
}
// every dim must fit the C int the entry points take
bool dims_fit(const int64_t* d, size_t n) {
  for (size_t i = 0; i < n; ++i)
    if (d[i] < 0 || d[i] > 0x7fffffff) return false;
  return true;
}
}  // namespace

extern "C" int tessera_gfx950_gpu_launcher(const char* target, const char* kernel_name,
                                           const tessera_gfx950_launch_params* params, void* user) {
  (void)user;
  if (!target || !kernel_name) return kTsrInvalidArgument;
  if (std::strcmp(target, "rocm") != 0 && std::strcmp(target, "rocm_gfx950") != 0) return kTsrNotFound;
  using Gemm = int (*)(const void*, const void*, void*, int, int, int);
  using Batched = int (*)(const void*, const void*, void*, int, int, int, int);
  using Attn = int (*)(const void*, const void*, const void*, void*, int, int, int, int, int, float, int);
  struct { const char* name; Gemm fn; } const gemms[] = {
      {"tessera_gfx950_gemm_f16", tessera_gfx950_gemm_f16},         {"tessera_gfx950_gemm_bf16", tessera_gfx950_gemm_bf16},
      {"tessera_gfx950_gemm_f16_f16", tessera_gfx950_gemm_f16_f16}, {"tessera_gfx950_gemm_bf16_bf16", tessera_gfx950_gemm_bf16_bf16},
      {"tessera_gfx950_gemm_i8_i32", tessera_gfx950_gemm_i8_i32}};
  struct { const char* name; Batched fn; } const batched[] = {
      {"tessera_gfx950_batched_gemm_f16", tessera_gfx950_batched_gemm_f16},
      {"tessera_gfx950_batched_gemm_bf16", tessera_gfx950_batched_gemm_bf16}};
  struct { const char* name; Attn fn; } const attns[] = {
      {"tessera_gfx950_flash_attn_f16", tessera_gfx950_flash_attn_f16},
      {"tessera_gfx950_flash_attn_bf16", tessera_gfx950_flash_attn_bf16}};
  auto shaped = [&](size_t nbuf, size_t ndim) {
    if (!params || params->num_buffers != nbuf || params->num_dims != ndim || !params->buffers || !params->dims) return false;
    for (size_t i = 0; i < nbuf; ++i)
      if (!params->buffers[i]) return false;
    return dims_fit(params->dims, ndim);
  };
  for (const auto& g : gemms) {
    if (std::strcmp(kernel_name, g.name) != 0) continue;
    if (!shaped(3, 3)) return kTsrInvalidArgument;
    const int64_t* d = params->dims;
    return tsr_status_of(g.fn(params->buffers[0], params->buffers[1], params->buffers[2], (int)d[0], (int)d[1], (int)d[2]));
  }
  for (const auto& g : batched) {
    if (std::strcmp(kernel_name, g.name) != 0) continue;
    if (!shaped(3, 4)) return kTsrInvalidArgument;
    const int64_t* d = params->dims;
    return tsr_status_of(g.fn(params->buffers[0], params->buffers[1], params->buffers[2], (int)d[0], (int)d[1], (int)d[2], (int)d[3]));
  }
  for (const auto& a : attns) {
    if (std::strcmp(kernel_name, a.name) != 0) continue;
    if (!shaped(4, 6)) return kTsrInvalidArgument;
    const int64_t* d = params->dims;
    if (d[4] <= 0) return kTsrInvalidArgument;
    const float scale = 1.0f / std::sqrt((float)d[4]);
    return tsr_status_of(a.fn(params->buffers[0], params->buffers[1], params->buffers[2], params->buffers[3], (int)d[0],
                              (int)d[1], (int)d[2], (int)d[3], (int)d[4], scale, d[5] != 0));
  }
  return kTsrNotFound;
}
