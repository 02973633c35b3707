// Host-side helpers shared by the C-ABI translation units: the cached device
// probe, RAII device buffers for the host-pointer entry points, error mapping.
#pragma once
#include <cmath>
#include <chrono>
#include <hip/hip_runtime.h>
#include <mutex>
#include <stddef.h>
#include <vector>
#include "common.h"

namespace tsr950 {

// 0 when device 0 is a gfx950 part, else kNoDevice.  Cached after the first call.
int probe_device();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Serialises the host-pointer entry points.  Each of them uploads, runs its device-pointer
// twin on the null stream, synchronises and downloads; the twin takes its scratch (split-K
// partials, routing lists, quantiser maxima) from the null stream's workspace at offset 0.
// Two host threads inside such calls at once would share those bytes, so every
// host-pointer call holds this lock from its first allocation to its last download.
// Recursive: a host-pointer entry point may be reached through another (the launcher).
std::recursive_mutex& host_call_mutex();

// Owns device allocations made on behalf of a host-pointer entry point and frees
// them on scope exit, whichever way the call ends.  Holds host_call_mutex() for its
// lifetime, which makes the host-pointer ABI safe to call from several threads.
class DeviceScope {
 public:
  DeviceScope() : lock_(host_call_mutex()) {}
  DeviceScope(const DeviceScope&) = delete;
  DeviceScope& operator=(const DeviceScope&) = delete;
  ~DeviceScope() {
    for (void* p : ptrs_) (void)hipFree(p);
  }
  // Allocates `bytes` (at least 16) and, when `src` is given, copies it in.
  void* alloc(size_t bytes, const void* src = nullptr) {
    void* d = nullptr;
    if (hipMalloc(&d, bytes < 16 ? 16 : bytes) != hipSuccess) { failed_ = true; return nullptr; }
    ptrs_.push_back(d);
    if (src && bytes && hipMemcpy(d, src, bytes, hipMemcpyHostToDevice) != hipSuccess) failed_ = true;
    return d;
  }
  bool download(void* dst, const void* src, size_t bytes) {
    if (!bytes) return true;
    if (hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost) != hipSuccess) { failed_ = true; return false; }
    return true;
  }
  bool failed() const { return failed_; }

 private:
  std::unique_lock<std::recursive_mutex> lock_;   // declared first: released after the frees
  std::vector<void*> ptrs_;
  bool failed_ = false;
};

// Which clock the last bench-ABI call on this thread reported: 0 HIP events, 1 wall clock,
// -1 none yet / the call failed (tessera_gfx950_bench_last_timer_source).
extern thread_local int g_last_timer_source;

// The timing loop of the bench ABI (after tessera_rocm_gemm.cpp:551-667): warm-up of at
// least five launches and 60 ms, so that the clocks, which ramp up over tens of
// milliseconds after idle, are steady; then `iters` launches between two HIP events on the
// null stream, cross-checked against the wall clock (the event figure is used when it lies
// within a factor of two of it, otherwise the wall-clock one, and the source says which).
// `launch(i)` enqueues launch i and returns a status code.
template <class Launch>
int bench_loop(Launch&& launch, int iters, double* avg_ms) {
  const auto warm0 = std::chrono::steady_clock::now();
  for (int w = 0; w < 5 || std::chrono::steady_clock::now() - warm0 < std::chrono::milliseconds(60); ++w) {
    const int rc = launch(w);
    if (rc != kOk) return rc;
    if ((w & 15) == 15 && hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  }
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return kDeviceFailed;
  if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return kDeviceFailed; }
  int rc = kOk;
  const auto t0 = std::chrono::steady_clock::now();
  (void)hipEventRecord(e0, nullptr);
  for (int it = 0; it < iters && rc == kOk; ++it) rc = launch(it);
  (void)hipEventRecord(e1, nullptr);
  const bool synced = hipEventSynchronize(e1) == hipSuccess;
  const double wall_ms =
      std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  float ev_ms = 0.f;
  const bool ev_ok = synced && hipEventElapsedTime(&ev_ms, e0, e1) == hipSuccess && std::isfinite(ev_ms) &&
                     ev_ms > 0.f && ev_ms <= 2.0 * wall_ms && ev_ms >= 0.5 * wall_ms;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != kOk) return rc;
  if (!synced) return kDeviceFailed;
  g_last_timer_source = ev_ok ? 0 : 1;
  *avg_ms = (ev_ok ? (double)ev_ms : wall_ms) / iters;
  return kOk;
}

// Device scratch for kernels that need it between two launches of one call (split-K
// partials, routing and combine lists, quantiser maxima): one buffer per (device,
// stream), grown on demand and kept until the process ends.  Calls on one stream run in
// order, so they share the buffer from offset 0; calls on different streams get
// different buffers.  Growing allocates (hipMalloc) but never frees or synchronises: the
// outgrown buffer is set aside for the work still queued on it.  The host threads that
// enqueue on one stream must be serialised by the caller (two of them would hand the
// same bytes to kernels the stream may then interleave); under stream capture the
// buffer must already have its final size (run the call once outside the capture).
// Returns null on failure.
void* stream_workspace(hipStream_t s, size_t bytes);
// Synchronises `s` and frees its workspace; a later call on the stream allocates afresh.
int stream_workspace_release(hipStream_t s);
// Looks up the device address of the allocation-free routing entry's scratch array for the
// current device (idempotent); called from the device probe.
int route_scratch_warm();

// Clears `words` 32-bit words on the stream with a fill kernel.  (A memset node recorded
// into a captured graph has given wrong results on replays after the first, so nothing a
// caller may capture uses hipMemsetAsync.)
static __global__ void __launch_bounds__(256) zero_words_kernel(uint32_t* p, size_t words) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += stride) p[i] = 0u;
}
inline void zero_words(void* p, size_t words, hipStream_t s) {
  if (!words) return;
  const size_t want = (words + 255) / 256;
  hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)(want < 1024 ? want : 1024)), dim3(256), 0, s,
                     static_cast<uint32_t*>(p), words);
}

inline int finish(hipError_t e) { return e == hipSuccess ? kOk : kDeviceFailed; }

// Launch status of the kernels just enqueued on `s` (does not synchronise).
inline int launch_status() { return finish(hipGetLastError()); }

}  // namespace tsr950
