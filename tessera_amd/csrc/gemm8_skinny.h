// Skinny 8-bit GEMM for gfx950: raw accumulators of D[M,N] = A[M,K] B[K,N] for M <= 32
// (quantised decode: a few activation rows against a big int8 / e4m3 weight matrix).
//
// The product is bound by streaming B from HBM once.  A workgroup of G8S_NW waves owns a strip of
// 128 columns of B and a K range; each of its waves walks its own 64-row slices of that range with two
// slices (16 KB of B per wave) outstanding.  A slice passes through a wave-private LDS buffer
// only to be transposed into MFMA operand order (ds_read_b64_tr_b8), no barrier is taken until
// the waves' partial accumulators are summed through LDS in a fixed tree order at the end, and
// A is read straight from global memory in operand layout (it is small and stays in L2).
// The result is the tile of raw accumulators (int32, or f32 of unscaled e4m3 products) of K
// split z = blockIdx.y, stored at part + z M N; gemm8_split_sum_kernel sums the splits and
// applies the product's epilogue.
#pragma once
#include "gemm8.h"

namespace tsr950 {

constexpr int G8S_NJ = 4;                       // 32-column blocks per strip
constexpr int G8S_COLS = 32 * G8S_NJ;           // 128
constexpr int G8S_ROWS = 64;                    // k rows per slice
constexpr int G8S_PITCH = G8S_COLS + 32;        // the pad spreads the 8 rows of a transposing read over all banks
constexpr int G8S_WAVE_LDS = G8S_ROWS * G8S_PITCH;
constexpr int G8S_LOADS = G8S_ROWS * G8S_COLS / 16 / 64;     // 16-byte loads per lane per slice: 8
// LDS of a workgroup of NW waves with MI 32-row blocks: the waves' slices (10 KB each), then reused by the
// reduction tree (NW / 2 partial tiles of MI x 16 KB)
constexpr int g8s_smem(int nw, int mi) {
  return nw * G8S_WAVE_LDS > (nw / 2) * mi * 16384 ? nw * G8S_WAVE_LDS : (nw / 2) * mi * 16384;
}

// (taken by value: a bit cast applied directly to an element of a vector-typed accumulator read
// element 0 whatever the index)
template <class E>
__device__ __forceinline__ uint32_t bits_of(E v) { return __builtin_bit_cast(uint32_t, v); }

template <class T, int G8S_NW, int MI>
__global__ __launch_bounds__(G8S_NW * 64) void gemm8_skinny_kernel(const uint8_t* __restrict__ A,
                                                                   const uint8_t* __restrict__ B, void* __restrict__ part,
                                                                   int M, int N, int K, int kps) {
  constexpr bool IS_I8 = std::is_same<T, I8>::value;
  using acc_t = typename std::conditional<IS_I8, i32x16, f32x16>::type;
  extern __shared__ __align__(16) char smem[];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int n0 = blockIdx.x * G8S_COLS;
  const int z = blockIdx.y;
  const int kbeg = z * kps;
  const int kend = min(K, kbeg + kps);
  const int nslices = kend > kbeg ? (kend - kbeg) / G8S_ROWS : 0;

  // B slice load: 8 lanes cover one 128-byte row, one load instruction 8 rows.
  const int ch = lane & 7, brow = lane >> 3;
  uint32_t b_off[G8S_LOADS], b_wr[G8S_LOADS];
#pragma unroll
  for (int q = 0; q < G8S_LOADS; ++q) {
    const int row = brow + 8 * q;
    b_off[q] = (n0 + ch * 16 < N) ? (uint32_t)row * (uint32_t)N + n0 + ch * 16 : kOutOfRange;
    b_wr[q] = w * G8S_WAVE_LDS + row * G8S_PITCH + ch * 16;
  }
  // A operand: lane holds row m = 32 mi + l32, bytes k = 32 f + 16 lh + (0..15) of the slice.
  uint32_t a_off[MI];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
    a_off[mi] = 32 * mi + l32 < M ? (uint32_t)(32 * mi + l32) * (uint32_t)K + 16 * lh : kOutOfRange;
  // transposing read: lane r of a 16-lane block supplies row k0 + r/2 and columns 8 (r%2) .. +7 of a
  // 16-column patch; lane i receives column i, k0 .. k0 + 7.
  const int r16 = lane & 15;
  const uint32_t b_rd = w * G8S_WAVE_LDS + (16 * lh + (r16 >> 1)) * G8S_PITCH + 16 * ((lane >> 4) & 1) + 8 * (r16 & 1);

  acc_t acc[MI][G8S_NJ];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int j = 0; j < G8S_NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mi][j][r] = 0;

  uint4 bq[2][G8S_LOADS], aq[2][MI][2];
  auto load = [&](int slot, int s) {
    const uint8_t* Bs = B + (long)(kbeg + s * G8S_ROWS) * N;
    const uint8_t* As = A + (kbeg + s * G8S_ROWS);
#pragma unroll
    for (int q = 0; q < G8S_LOADS; ++q) bq[slot][q] = buffer_load_b128(Bs, b_off[q]);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      aq[slot][mi][0] = buffer_load_b128(As, a_off[mi]);
      aq[slot][mi][1] = buffer_load_b128(As + 32, a_off[mi]);
    }
  };
  auto consume = [&](int slot, int s_next) {
#pragma unroll
    for (int q = 0; q < G8S_LOADS; ++q) lds_write_b128(smem, b_wr[q], bq[slot][q]);
    uint4 af[MI][2];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) { af[mi][0] = aq[slot][mi][0]; af[mi][1] = aq[slot][mi][1]; }
    // (the transposing read returns bytes other lanes wrote: nothing may move across this point)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    uint4 bf[2][G8S_NJ];
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
      for (int j = 0; j < G8S_NJ; ++j) {
        const char* pb = smem + b_rd + f * 32 * G8S_PITCH + j * 32;
        const uint2 lo = lds_read_tr8_b64(pb);
        const uint2 hi = lds_read_tr8_b64(pb + 8 * G8S_PITCH);
        bf[f][j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    if (s_next < nslices) load(slot, s_next);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int j = 0; j < G8S_NJ; ++j) {
        if constexpr (IS_I8) {
          acc[mi][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, bf[0][j]),
                                                             __builtin_bit_cast(i32x4, af[mi][0]), acc[mi][j], 0, 0, 0);
          acc[mi][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, bf[1][j]),
                                                             __builtin_bit_cast(i32x4, af[mi][1]), acc[mi][j], 0, 0, 0);
        } else {
          const i32x4 b0 = __builtin_bit_cast(i32x4, bf[0][j]), b1 = __builtin_bit_cast(i32x4, bf[1][j]);
          const i32x4 x0 = __builtin_bit_cast(i32x4, af[mi][0]), x1 = __builtin_bit_cast(i32x4, af[mi][1]);
          const i32x8 b8 = (i32x8){b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
          const i32x8 a8 = (i32x8){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
          acc[mi][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, a8, acc[mi][j], f8_format<T>(), f8_format<T>(),
                                                                       0, 0, 0, 0);
        }
      }
  };

  int s = w;
  if (s < nslices) load(0, s);
  if (s + G8S_NW < nslices) load(1, s + G8S_NW);
  for (; s + G8S_NW < nslices; s += 2 * G8S_NW) {
    consume(0, s + 2 * G8S_NW);
    consume(1, s + 3 * G8S_NW);
  }
  if (s < nslices) consume(0, nslices);

  // ---- sum the waves' partial tiles in a fixed order: wave w += wave w + half ----
  __syncthreads();
  uint4* red = reinterpret_cast<uint4*>(smem);
  constexpr int Q4 = MI * G8S_NJ * 4;                // 16-byte groups per lane
#pragma unroll
  for (int half = G8S_NW / 2; half >= 1; half >>= 1) {
    if (w >= half && w < 2 * half) {
      uint4* dst = red + (size_t)(w - half) * Q4 * 64 + lane;
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int j = 0; j < G8S_NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            dst[((mi * G8S_NJ + j) * 4 + q) * 64] = make_uint4(bits_of(acc[mi][j][4 * q]), bits_of(acc[mi][j][4 * q + 1]),
                                                               bits_of(acc[mi][j][4 * q + 2]), bits_of(acc[mi][j][4 * q + 3]));
    }
    __syncthreads();
    if (w < half) {
      const uint4* src = red + (size_t)w * Q4 * 64 + lane;
      using elem_t = typename std::conditional<IS_I8, int32_t, float>::type;
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int j = 0; j < G8S_NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint4 v = src[((mi * G8S_NJ + j) * 4 + q) * 64];
            acc[mi][j][4 * q] += __builtin_bit_cast(elem_t, v.x); acc[mi][j][4 * q + 1] += __builtin_bit_cast(elem_t, v.y);
            acc[mi][j][4 * q + 2] += __builtin_bit_cast(elem_t, v.z); acc[mi][j][4 * q + 3] += __builtin_bit_cast(elem_t, v.w);
          }
    }
    __syncthreads();
  }
  if (w != 0) return;
  // acc[mi][j][r]: row m = 32 mi + l32, column n0 + 32 j + 8 (r / 4) + 4 lh + (r % 4): runs of four columns
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = 32 * mi + l32;
    if (m >= M) continue;
    uint32_t* out = reinterpret_cast<uint32_t*>(part) + ((size_t)z * M + m) * N;
#pragma unroll
    for (int j = 0; j < G8S_NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + 32 * j + 8 * q + 4 * lh;
        if (n < N)                                       // N % 16 == 0: all or nothing per run of four
          *reinterpret_cast<uint4*>(out + n) = make_uint4(bits_of(acc[mi][j][4 * q]), bits_of(acc[mi][j][4 * q + 1]),
                                                          bits_of(acc[mi][j][4 * q + 2]), bits_of(acc[mi][j][4 * q + 3]));
      }
  }
}

}  // namespace tsr950
