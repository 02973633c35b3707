// Host-side helpers shared by the C-ABI translation units: the cached device
// probe, RAII device buffers for the host-pointer entry points, error mapping.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <vector>
#include "common.h"

namespace tsr950 {

// 0 when device 0 is a gfx950 part, else kNoDevice.  Cached after the first call.
int probe_device();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Owns device allocations made on behalf of a host-pointer entry point and frees
// them on scope exit, whichever way the call ends.
class DeviceScope {
 public:
  DeviceScope() = default;
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
  std::vector<void*> ptrs_;
  bool failed_ = false;
};

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
