// Copies between a matrix of any pitch and alignment and a 16-byte aligned, zero-padded one:
// how operands that the 16-byte loads of the tile kernels cannot take reach those kernels.
#pragma once
#include <algorithm>
#include "common.h"

namespace tsr950 {

// A thread moves one 16-byte chunk: blockIdx.x / threadIdx.x run along a row, blockIdx.y /
// threadIdx.y over rows, blockIdx.z over the batch.  The side of any alignment is accessed with one
// 16-byte instruction where the whole chunk is inside the row (global memory takes accesses off
// their natural alignment), element by element at the row's end.
// (the field is a plain vector type: a packed attribute is ignored on a field of class type, which would
// leave the struct 16-byte aligned and the access free to assume it)
template <class E> struct __attribute__((packed, aligned(sizeof(E)))) LooseChunk { u32x4 v; };
static_assert(alignof(LooseChunk<uint8_t>) == 1 && alignof(LooseChunk<uint16_t>) == 2 && sizeof(LooseChunk<uint16_t>) == 16,
              "LooseChunk must carry its element's alignment");
constexpr int kCopyRowsPerBlock = 4;

// dst[b][r][c] (rows_dst x ld_dst, 16-byte aligned) = src[b][r][c] inside rows_src x cols_src, else 0.
template <class E>
__global__ void __launch_bounds__(64 * kCopyRowsPerBlock)
pad_rows_kernel(E* __restrict__ dst, long ld_dst, long stride_dst, const E* __restrict__ src, long ld_src,
                long stride_src, int rows_src, int cols_src, int rows_dst) {
  constexpr int V = 16 / sizeof(E);
  const int c0 = (blockIdx.x * 64 + threadIdx.x) * V;
  if (c0 >= ld_dst) return;
  const long b = blockIdx.z;
  for (int r = blockIdx.y * kCopyRowsPerBlock + threadIdx.y; r < rows_dst; r += gridDim.y * kCopyRowsPerBlock) {
    uint4 out = make_uint4(0u, 0u, 0u, 0u);
    if (r < rows_src && c0 < cols_src) {
      const E* sp = src + b * stride_src + (long)r * ld_src + c0;
      if (c0 + V <= cols_src) {
        const u32x4 t = reinterpret_cast<const LooseChunk<E>*>(sp)->v;
        out = make_uint4(t[0], t[1], t[2], t[3]);
      } else {
        alignas(16) E v[V];
#pragma unroll
        for (int u = 0; u < V; ++u) v[u] = c0 + u < cols_src ? sp[u] : E(0);
        out = *reinterpret_cast<const uint4*>(v);
      }
    }
    *reinterpret_cast<uint4*>(dst + b * stride_dst + (long)r * ld_dst + c0) = out;
  }
}
// dst[b][r][c] = src[b][r][c] for r < rows, c < cols; src 16-byte aligned with pitch ld_src, dst any.
template <class E>
__global__ void __launch_bounds__(64 * kCopyRowsPerBlock)
unpad_rows_kernel(E* __restrict__ dst, long ld_dst, long stride_dst, const E* __restrict__ src, long ld_src,
                  long stride_src, int rows, int cols) {
  constexpr int V = 16 / sizeof(E);
  const int c0 = (blockIdx.x * 64 + threadIdx.x) * V;
  if (c0 >= cols) return;
  const long b = blockIdx.z;
  for (int r = blockIdx.y * kCopyRowsPerBlock + threadIdx.y; r < rows; r += gridDim.y * kCopyRowsPerBlock) {
    const uint4 in = *reinterpret_cast<const uint4*>(src + b * stride_src + (long)r * ld_src + c0);
    E* dp = dst + b * stride_dst + (long)r * ld_dst + c0;
    if (c0 + V <= cols) {
      reinterpret_cast<LooseChunk<E>*>(dp)->v = u32x4{in.x, in.y, in.z, in.w};
    } else {
      alignas(16) E v[V];
      *reinterpret_cast<uint4*>(v) = in;
#pragma unroll
      for (int u = 0; u < V; ++u)
        if (c0 + u < cols) dp[u] = v[u];
    }
  }
}
inline dim3 copy_grid(long rows, long ld, int vec, int batch) {
  const long bx = (ld / vec + 63) / 64, by = (rows + kCopyRowsPerBlock - 1) / kCopyRowsPerBlock;
  return dim3((unsigned)bx, (unsigned)std::max<long>(1, std::min<long>(by, 16384)), (unsigned)batch);
}
inline dim3 copy_block() { return dim3(64, kCopyRowsPerBlock, 1); }

}  // namespace tsr950
