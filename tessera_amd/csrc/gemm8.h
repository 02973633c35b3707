// 8-bit MFMA GEMM for gfx950:  D[M,N] = A[M,K] . B[K,N], row-major bytes.
//   I8   int8 x int8 -> int32 (v_mfma_i32_32x32x32_i8), bit-exact.
//   FP8  OCP e4m3 x e4m3 -> f32 (v_mfma_f32_32x32x64_f8f6f4, the full-rate CDNA4
//        fp8 form), scaled by two per-tensor f32 scales in the epilogue.
//
// Same structure as the 16-bit kernel: 256x256 output tile, 2x2 waves of 128x128,
// K walked in steps of 128 bytes, LDS double buffered with one barrier per step,
// operand fragments double buffered in registers.
//   A tile  [256][128 B], 16-byte chunks XOR-swizzled by (row & 7), ds_read_b128.
//   B tile  [128][256 + 16 B] natural layout; the operand (16 or 32 consecutive k
//           bytes of one column per lane) is read with the transposing
//           ds_read_b64_tr_b8: a 16-lane block reads an 8(k) x 16(n) patch and
//           every lane receives 8 consecutive k of one column.  The 16-byte row
//           pad spreads the 8 rows of a patch over all banks.
// Both operands enumerate k in the same order, which is all the MFMA needs: for
// the 64-deep fp8 instruction a lane's 32 bytes are bytes [16h,16h+16) of two
// consecutive 32-byte k groups rather than one contiguous run.
#pragma once
#include <type_traits>
#include "common.h"

namespace tsr950 {

struct I8 {};
struct FP8 {};

enum Gemm8Epilogue : int {
  EPI8_I32 = 0,        // I8: int32 accumulators
  EPI8_W8A8_F32 = 1,   // I8: f32(acc) * row_scale[m] * col_scale[n]  (+ optional int32 copy)
  EPI8_SCALED_F32 = 2, // FP8: acc * sa * sb -> f32
  EPI8_SCALED_BF16 = 3 // FP8: acc * sa * sb -> bf16
};

struct Gemm8Params {
  const uint8_t* A;
  const uint8_t* B;
  void* D;
  int32_t* acc_out;          // W8A8: optional raw accumulators
  const float* row_scale;    // W8A8: [M]
  const float* col_scale;    // W8A8: [N]
  float scale_a, scale_b;    // FP8
  int M, N, K;
  int tiles_m, tiles_n;
};

constexpr int G8_BK = 128;       // K step in bytes (= elements)
constexpr int G8_BM = 256, G8_BN = 256;
constexpr int G8_APITCH = 128;
constexpr int G8_BPITCH = G8_BN + 16;
constexpr int G8_ASTAGE = G8_BM * G8_APITCH;
constexpr int G8_BSTAGE = G8_BK * G8_BPITCH;
constexpr int G8_STAGE = G8_ASTAGE + G8_BSTAGE;
constexpr int G8_SMEM = 2 * G8_STAGE;

__device__ __forceinline__ void tile_of_block8(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  int lin = bid;
  if (total % 8 == 0) lin = (bid % 8) * (total / 8) + bid / 8;
  constexpr int GROUP_M = 4;
  const int band = GROUP_M * tiles_n;
  const int b = lin / band;
  const int first_m = b * GROUP_M;
  const int rows = min(tiles_m - first_m, GROUP_M);
  const int r = lin - b * band;
  tm = first_m + r % rows;
  tn = r / rows;
}

template <class T, int EPI>
__global__ __launch_bounds__(256, 1) void gemm8_kernel(const Gemm8Params p) {
  constexpr bool IS_I8 = std::is_same<T, I8>::value;
  constexpr int MI = 4, NJ = 4;
  constexpr int NT = 256;
  constexpr int A_CHUNKS = G8_BM * 8 / NT;                 // 8
  constexpr int B_CHUNKS = G8_BK * (G8_BN / 16) / NT;      // 8
  // MFMA k steps per 128-byte tile: 4 x 32 (int8) or 2 x 64 (fp8).
  constexpr int KS = IS_I8 ? 4 : 2;
  constexpr int FR = IS_I8 ? 1 : 2;                        // 16-byte registers per operand fragment
  using acc_t = typename std::conditional<IS_I8, i32x16, f32x16>::type;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  int tm, tn;
  tile_of_block8(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m_begin = tm * G8_BM, n_begin = tn * G8_BN;
  const int K = p.K;

  const uint8_t* a_ptr[A_CHUNKS];
  uint32_t a_lds[A_CHUNKS];
  const int a_chunk = tid & 7;
#pragma unroll
  for (int q = 0; q < A_CHUNKS; ++q) {
    const int row = (tid >> 3) + 32 * q;
    int gr = m_begin + row;
    gr = gr < p.M ? gr : p.M - 1;
    a_ptr[q] = p.A + (long)gr * K + a_chunk * 16;
    a_lds[q] = row * G8_APITCH + ((a_chunk ^ (row & 7)) << 4);
  }
  const uint8_t* b_ptr[B_CHUNKS];
  uint32_t b_lds[B_CHUNKS];
  int b_krow[B_CHUNKS];
#pragma unroll
  for (int q = 0; q < B_CHUNKS; ++q) {
    const int v = tid + NT * q;
    const int krow = v / (G8_BN / 16), nch = v % (G8_BN / 16);
    int gc = n_begin + nch * 16;
    gc = gc < p.N ? gc : p.N - 16;
    b_ptr[q] = p.B + (long)krow * p.N + gc;
    b_lds[q] = G8_ASTAGE + krow * G8_BPITCH + nch * 16;
    b_krow[q] = krow;
  }

  uint4 ra[A_CHUNKS], rb[B_CHUNKS];
  auto gload = [&](int k0, auto guarded_c) {
    if constexpr (!decltype(guarded_c)::value) {
#pragma unroll
      for (int q = 0; q < A_CHUNKS; ++q) ra[q] = *reinterpret_cast<const uint4*>(a_ptr[q] + k0);
#pragma unroll
      for (int q = 0; q < B_CHUNKS; ++q) rb[q] = *reinterpret_cast<const uint4*>(b_ptr[q] + (long)k0 * p.N);
    } else {
#pragma unroll
      for (int q = 0; q < A_CHUNKS; ++q) {
        const bool ok = k0 + a_chunk * 16 < K;
        const uint4 v = *reinterpret_cast<const uint4*>(a_ptr[q] + (ok ? k0 : -(a_chunk * 16)));
        ra[q].x = ok ? v.x : 0u; ra[q].y = ok ? v.y : 0u; ra[q].z = ok ? v.z : 0u; ra[q].w = ok ? v.w : 0u;
      }
#pragma unroll
      for (int q = 0; q < B_CHUNKS; ++q) {
        const bool ok = k0 + b_krow[q] < K;
        const uint4 v = *reinterpret_cast<const uint4*>(b_ptr[q] + (ok ? (long)k0 : -(long)b_krow[q]) * p.N);
        rb[q].x = ok ? v.x : 0u; rb[q].y = ok ? v.y : 0u; rb[q].z = ok ? v.z : 0u; rb[q].w = ok ? v.w : 0u;
      }
    }
  };
  auto lstore = [&](int buf) {
    char* base = smem + buf * G8_STAGE;
#pragma unroll
    for (int q = 0; q < A_CHUNKS; ++q) lds_write_b128(base, a_lds[q], ra[q]);
#pragma unroll
    for (int q = 0; q < B_CHUNKS; ++q) lds_write_b128(base, b_lds[q], rb[q]);
  };

  uint32_t a_rd[MI];
  int a_sw[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int row = wm * 128 + i * 32 + l32;
    a_rd[i] = row * G8_APITCH;
    a_sw[i] = row & 7;
  }
  // Transposing byte read: lane r of a 16-lane block supplies row k0 + r/2 and
  // columns n0 + 8 (r % 2) .. +7; lane i receives column n0 + i, k0 .. k0+7.
  const int r16 = lane & 15;
  const uint32_t b_rd0 = G8_ASTAGE + (16 * lh + (r16 >> 1)) * G8_BPITCH +
                         (wn * 128 + 16 * ((lane >> 4) & 1) + 8 * (r16 & 1));

  acc_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // Fragment f (32 k bytes of the tile: bytes 32 f .. 32 f + 31) gives each lane
  // half its 16 bytes [32 f + 16 h, +16).
  uint4 af[2][MI][FR], bf[2][NJ][FR];
  auto frag_load = [&](int buf, int ks, int slot) {
    const char* base = smem + buf * G8_STAGE;
#pragma unroll
    for (int x = 0; x < FR; ++x) {
      const int f = ks * FR + x;
#pragma unroll
      for (int i = 0; i < MI; ++i)
        af[slot][i][x] = lds_read_b128(base, a_rd[i] + ((((f << 1) | lh) ^ a_sw[i]) << 4));
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const char* pb = base + b_rd0 + f * 32 * G8_BPITCH + j * 32;
        const uint2 lo = lds_read_tr8_b64(pb);
        const uint2 hi = lds_read_tr8_b64(pb + 8 * G8_BPITCH);
        bf[slot][j][x] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    }
  };
  auto mma = [&](int slot) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if constexpr (IS_I8) {
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, bf[slot][j][0]),
                                                            __builtin_bit_cast(i32x4, af[slot][i][0]),
                                                            acc[i][j], 0, 0, 0);
        } else {
          i32x8 a8, b8;
          const i32x4 b0 = __builtin_bit_cast(i32x4, bf[slot][j][0]), b1 = __builtin_bit_cast(i32x4, bf[slot][j][1]);
          const i32x4 a0 = __builtin_bit_cast(i32x4, af[slot][i][0]), a1 = __builtin_bit_cast(i32x4, af[slot][i][1]);
          b8 = (i32x8){b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
          a8 = (i32x8){a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
          // format selectors 0 = e4m3; zero scale operands select the unscaled form.
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, a8, acc[i][j], 0, 0, 0, 0, 0, 0);
        }
      }
  };

  const int ktiles = (K + G8_BK - 1) / G8_BK;
  using std::true_type;
  using std::false_type;
  using no_prefetch = std::integral_constant<int, 0>;
  using full_prefetch = std::integral_constant<int, 1>;
  using tail_prefetch = std::integral_constant<int, 2>;
  gload(0, true_type{});
  lstore(0);
  __syncthreads();
  if (ktiles > 1) gload(G8_BK, true_type{});
  frag_load(0, 0, 0);

  auto kstep = [&](int kt, auto more_c, auto prefetch_c) {
    constexpr bool MORE = decltype(more_c)::value;
    constexpr int PREFETCH = decltype(prefetch_c)::value;
    const int buf = kt & 1;
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      frag_load(buf, ks + 1, (ks + 1) & 1);
      if (MORE && ks == KS - 2) lstore(buf ^ 1);
      mma(ks & 1);
    }
    __syncthreads();
    if constexpr (MORE) {
      if constexpr (PREFETCH == 1) gload((kt + 2) * G8_BK, false_type{});
      if constexpr (PREFETCH == 2) gload((kt + 2) * G8_BK, true_type{});
      frag_load(buf ^ 1, 0, KS & 1);
    }
    mma((KS - 1) & 1);
  };
  int kt = 0;
  for (; kt + 3 < ktiles; ++kt) kstep(kt, true_type{}, full_prefetch{});
  if (kt + 2 < ktiles) { kstep(kt, true_type{}, tail_prefetch{}); ++kt; }
  if (kt + 1 < ktiles) { kstep(kt, true_type{}, no_prefetch{}); ++kt; }
  kstep(kt, false_type{}, no_prefetch{});

  // acc[i][j][r]: row m = 32 i + l32, col n = 32 j + 8 (r / 4) + 4 h + (r % 4).
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_begin + wm * 128 + i * 32 + l32;
    if (m >= p.M) continue;
    float rs = 1.f;
    if constexpr (EPI == EPI8_W8A8_F32) rs = p.row_scale[m];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n_begin + wn * 128 + j * 32 + q * 8 + lh * 4;
        if (n >= p.N) continue;
        const long o = (long)m * p.N + n;
        if constexpr (EPI == EPI8_I32) {
          *reinterpret_cast<int4*>(reinterpret_cast<int32_t*>(p.D) + o) =
              make_int4(acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
        } else if constexpr (EPI == EPI8_W8A8_F32) {
          const float4 cs = *reinterpret_cast<const float4*>(p.col_scale + n);
          float4 out;
          out.x = ((float)acc[i][j][q * 4 + 0] * rs) * cs.x;
          out.y = ((float)acc[i][j][q * 4 + 1] * rs) * cs.y;
          out.z = ((float)acc[i][j][q * 4 + 2] * rs) * cs.z;
          out.w = ((float)acc[i][j][q * 4 + 3] * rs) * cs.w;
          *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.D) + o) = out;
          if (p.acc_out)
            *reinterpret_cast<int4*>(p.acc_out + o) =
                make_int4(acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
        } else {
          const float v0 = ((float)acc[i][j][q * 4 + 0] * p.scale_a) * p.scale_b;
          const float v1 = ((float)acc[i][j][q * 4 + 1] * p.scale_a) * p.scale_b;
          const float v2 = ((float)acc[i][j][q * 4 + 2] * p.scale_a) * p.scale_b;
          const float v3 = ((float)acc[i][j][q * 4 + 3] * p.scale_a) * p.scale_b;
          if constexpr (EPI == EPI8_SCALED_F32) {
            *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.D) + o) = make_float4(v0, v1, v2, v3);
          } else {
            uint2 pk;
            pk.x = pack2<BF16>(v0, v1);
            pk.y = pack2<BF16>(v2, v3);
            *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.D) + o) = pk;
          }
        }
      }
  }
}

// e4m3fn (OCP) byte -> f32: bias 7, no infinities, 0x7f / 0xff are NaN.
__device__ __forceinline__ float e4m3_to_f32(uint8_t c) {
  const uint32_t s = (uint32_t)(c & 0x80) << 24;
  const uint32_t e = (c >> 3) & 0xF, m = c & 7;
  float v;
  if (e == 0) v = (float)m * 0.001953125f;                       // m * 2^-9
  else if (e == 15 && m == 7) v = __builtin_nanf("");
  else v = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
  return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) | s);
}

// Any-shape fallback, one thread per output element, k in order.
template <class T, int EPI>
__global__ void gemm8_generic_kernel(const Gemm8Params p) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int m = blockIdx.y * blockDim.y + threadIdx.y;
  if (m >= p.M || n >= p.N) return;
  const long o = (long)m * p.N + n;
  if constexpr (std::is_same<T, I8>::value) {
    const int8_t* A = reinterpret_cast<const int8_t*>(p.A) + (long)m * p.K;
    const int8_t* B = reinterpret_cast<const int8_t*>(p.B) + n;
    int32_t acc = 0;
    for (int k = 0; k < p.K; ++k) acc += (int32_t)A[k] * (int32_t)B[(long)k * p.N];
    if constexpr (EPI == EPI8_I32) {
      reinterpret_cast<int32_t*>(p.D)[o] = acc;
    } else {
      reinterpret_cast<float*>(p.D)[o] = ((float)acc * p.row_scale[m]) * p.col_scale[n];
      if (p.acc_out) p.acc_out[o] = acc;
    }
  } else {
    const uint8_t* A = p.A + (long)m * p.K;
    const uint8_t* B = p.B + n;
    float acc = 0.f;
    for (int k = 0; k < p.K; ++k) acc += e4m3_to_f32(A[k]) * e4m3_to_f32(B[(long)k * p.N]);
    const float v = (acc * p.scale_a) * p.scale_b;
    if constexpr (EPI == EPI8_SCALED_F32) reinterpret_cast<float*>(p.D)[o] = v;
    else reinterpret_cast<uint16_t*>(p.D)[o] = f32_to_bf16_bits(v);
  }
}

}  // namespace tsr950
