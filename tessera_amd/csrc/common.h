// Shared device/host helpers for the gfx950 lane.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tsr950 {

constexpr int kOk = 0;
constexpr int kBadShape = 1;
constexpr int kNoDevice = 2;
constexpr int kDeviceFailed = 3;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

#define TSR_LDS __attribute__((address_space(3)))

// Storage dtypes of the 16-bit kernels.
struct BF16 {};
struct F16 {};

// f32 -> bf16 bits, round-to-nearest-even (the hardware conversion, v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return (float)__builtin_bit_cast(_Float16, b);
}

template <class T> __device__ __forceinline__ uint16_t to_storage(float f);
template <> __device__ __forceinline__ uint16_t to_storage<BF16>(float f) { return f32_to_bf16_bits(f); }
template <> __device__ __forceinline__ uint16_t to_storage<F16>(float f) { return f32_to_f16_bits(f); }
template <class T> __device__ __forceinline__ float from_storage(uint16_t b);
template <> __device__ __forceinline__ float from_storage<BF16>(uint16_t b) { return bf16_bits_to_f32(b); }
template <> __device__ __forceinline__ float from_storage<F16>(uint16_t b) { return f16_bits_to_f32(b); }

// Two f32 -> one dword of two storage values (lo = a, hi = b), one packed convert.
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
template <class T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<BF16>(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
template <> __device__ __forceinline__ uint32_t pack2<F16>(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

// 32x32x16 MFMA on 16-bit operands held as raw 128-bit registers.
template <class T> __device__ __forceinline__ f32x16 mfma_32x32x16(const uint4& a, const uint4& b, f32x16 c);
template <> __device__ __forceinline__ f32x16 mfma_32x32x16<BF16>(const uint4& a, const uint4& b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x16 mfma_32x32x16<F16>(const uint4& a, const uint4& b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// 16x16x32 MFMA on 16-bit operands (four accumulator registers per lane).  Per FLOP it moves
// half the accumulator data of the 32x32x16 form through the register file.
template <class T> __device__ __forceinline__ f32x4 mfma_16x16x32(const uint4& a, const uint4& b, f32x4 c);
template <> __device__ __forceinline__ f32x4 mfma_16x16x32<BF16>(const uint4& a, const uint4& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x4 mfma_16x16x32<F16>(const uint4& a, const uint4& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// LDS accessors on a byte offset into the dynamic LDS window.
__device__ __forceinline__ uint4 lds_read_b128(const char* base, uint32_t byte_off) {
  return *reinterpret_cast<const uint4*>(base + byte_off);
}
__device__ __forceinline__ void lds_write_b128(char* base, uint32_t byte_off, const uint4& v) {
  *reinterpret_cast<uint4*>(base + byte_off) = v;
}
// Transposing 64-bit LDS read of 16-bit elements.  Within each 16-lane block,
// lane r supplies the address of a row of four elements; lane i receives
// element (i % 4) of the rows supplied by lanes i/4, i/4+4, i/4+8, i/4+12.
__device__ __forceinline__ uint2 lds_read_tr16_b64(const char* p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TSR_LDS s16x4*)(p));
  return __builtin_bit_cast(uint2, v);
}
// Transposing 64-bit LDS read of 8-bit elements.  Within each 16-lane block,
// lane r supplies the address of a row of eight bytes; lane i receives byte
// (i % 8) of the rows supplied by lanes i/8, i/8+2, ..., i/8+14.
__device__ __forceinline__ uint2 lds_read_tr8_b64(const char* p) {
  i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((TSR_LDS i32x2*)(p));
  return __builtin_bit_cast(uint2, v);
}

// 16-byte buffer load: wave-uniform base (scalar registers) + 32-bit per-lane byte
// offset.  The range is 2 GiB from the base; any offset at or past it (use
// kOutOfRange) reads as zero without touching memory.
constexpr uint32_t kBufferRange = 0x7fffffffu;
constexpr uint32_t kOutOfRange = 0x80000000u;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 buffer_load_b128(const void* base, uint32_t byte_off) {
  __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, kBufferRange, 0x00020000);
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace tsr950
