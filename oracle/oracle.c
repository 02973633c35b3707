/*
 * oracle.c — plain-C restatement of the reference's CPU kernels for the gfx950
 * lane's hot path.  TEST INFRASTRUCTURE ONLY: linked by tests/, the smoke test
 * and the benchmark's cpu_baseline leg; never by the shipped library.
 *
 * Each function cites the reference file:line it follows (paths relative to
 * the reference checkout, src/compiler/codegen/tessera_x86_backend/src/kernels/
 * unless noted).  Pins: tests/test_oracle_c.py checks every function against
 * the numpy oracle, against closed forms, and — where oracle/_ref builds —
 * against the reference's own compiled kernels.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t v) {      /* avx512_gemm_bf16.cpp:6-11 */
  uint32_t bits = (uint32_t)v << 16;
  float out;
  memcpy(&out, &bits, sizeof out);
  return out;
}

/* Row-major bf16 x bf16 -> f32, sequential k, f32 accumulate.
 * tessera_x86_reference_gemm_bf16, avx512_gemm_bf16.cpp:13-26 (beta = 0). */
void orc_gemm_bf16_f32(const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int k = 0; k < K; ++k)
        acc += bf16_to_f32(A[(size_t)m * K + k]) * bf16_to_f32(B[(size_t)k * N + n]);
      C[(size_t)m * N + n] = acc;
    }
}

/* Same product with the n loop innermost (cache friendly) and an f64
 * accumulator row: the "fp32 or better" reference for larger sizes. */
void orc_gemm_bf16_f64(const uint16_t* A, const uint16_t* B, double* C, int M, int N, int K) {
  for (int m = 0; m < M; ++m) {
    double* c = C + (size_t)m * N;
    for (int n = 0; n < N; ++n) c[n] = 0.0;
    for (int k = 0; k < K; ++k) {
      const double a = bf16_to_f32(A[(size_t)m * K + k]);
      const uint16_t* b = B + (size_t)k * N;
      for (int n = 0; n < N; ++n) c[n] += a * (double)bf16_to_f32(b[n]);
    }
  }
}

/* Row-major s8 x s8 -> s32.  The integer GEMM contract of
 * tessera_x86_reference_gemm_u8s8_s32 (avx512_vnni_gemm_int8.cpp:5-18) with both
 * operands signed, as amx_gemm_int8.cpp:34-100 (s8s8) and smoothquant.py:122. */
void orc_gemm_s8s8_s32(const int8_t* A, const int8_t* B, int32_t* C, int M, int N, int K) {
  for (int m = 0; m < M; ++m) {
    int32_t* c = C + (size_t)m * N;
    for (int n = 0; n < N; ++n) c[n] = 0;
    for (int k = 0; k < K; ++k) {
      const int32_t a = A[(size_t)m * K + k];
      const int8_t* b = B + (size_t)k * N;
      for (int n = 0; n < N; ++n) c[n] += a * (int32_t)b[n];
    }
  }
}

/* Streaming online-softmax attention in f32 with GQA and LSE.
 * tessera_x86_flash_attn_f32 (avx512_flash_attn_f32.cpp:75-107): running max m,
 * denominator l, accumulator rescaled on each new max; causal bound
 * j <= i + max(sk - sq, 0) (attention_bounds, :180-196); kv head = qh*Hkv/Hq and
 * LSE = row_max + log(row_sum) (tessera_x86_flash_attn_ext_lse_f32, :379-422). */
void orc_flash_attn_f32(const float* Q, const float* K, const float* V, int B, int Hq, int Hkv, int sq, int sk,
                        int d, float scale, int causal, float* O, float* LSE) {
  const int off = sk > sq ? sk - sq : 0;
  for (int b = 0; b < B; ++b)
    for (int qh = 0; qh < Hq; ++qh) {
      const int kh = (int)(((long)qh * Hkv) / Hq);
      const float* Qb = Q + ((size_t)(b * Hq + qh) * sq) * d;
      const float* Kb = K + ((size_t)(b * Hkv + kh) * sk) * d;
      const float* Vb = V + ((size_t)(b * Hkv + kh) * sk) * d;
      float* Ob = O + ((size_t)(b * Hq + qh) * sq) * d;
      for (int i = 0; i < sq; ++i) {
        const float* qi = Qb + (size_t)i * d;
        float* oi = Ob + (size_t)i * d;
        for (int t = 0; t < d; ++t) oi[t] = 0.0f;
        const int jmax = causal ? i + off : sk - 1;
        float m = -INFINITY, l = 0.0f;
        for (int j = 0; j <= jmax && j < sk; ++j) {
          float s = 0.0f;
          for (int t = 0; t < d; ++t) s += qi[t] * Kb[(size_t)j * d + t];
          s *= scale;
          const float mn = s > m ? s : m;
          const float c = (m == -INFINITY) ? 0.0f : expf(m - mn);
          const float p = expf(s - mn);
          l = l * c + p;
          for (int t = 0; t < d; ++t) oi[t] = oi[t] * c + p * Vb[(size_t)j * d + t];
          m = mn;
        }
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        for (int t = 0; t < d; ++t) oi[t] *= inv;
        if (LSE) LSE[(size_t)(b * Hq + qh) * sq + i] = l > 0.0f ? m + logf(l) : -INFINITY;
      }
    }
}

/* Low-precision float-grid snap.  scalar_fpquant, avx512_fpquant_f32.cpp:28-41;
 * e4m3 = (448, 3, -6). */
void orc_fpquant_f32(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp, float* out) {
  for (int64_t i = 0; i < n; ++i) {
    const float v = x[i];
    if (isnan(v)) { out[i] = v; continue; }
    const float s = v < 0.0f ? -1.0f : 1.0f;
    const float ax = fminf(fabsf(v), max_normal);
    if (ax <= 0.0f) { out[i] = 0.0f; continue; }
    int e = (int)floorf(log2f(ax));
    if (e < min_exp) e = min_exp;
    const float ulp = ldexpf(1.0f, e - mantissa_bits);
    float r = nearbyintf(ax / ulp) * ulp;            /* RNE under the default rounding mode */
    r = fminf(r, max_normal);
    out[i] = s * r;
  }
}

/* Router + packing plan: f32 max-subtracted softmax, top-k (value descending,
 * ties -> lowest expert id), optional renormalisation, first-come capacity drop
 * in token-major order, kept slots stable-sorted by expert.
 * python/tessera/distributed/moe.py:143-206; python/tessera/nn/functional.py:463-476;
 * int32 ABI of python/tessera/compiler/moe_transport.py:221-227.
 * capacity <= 0 means no limit.  Returns the number of kept slots. */
int orc_moe_route(const float* scores, int T, int E, int k, int normalize, int capacity, int32_t* token_of_slot,
                  int32_t* expert_of_slot, float* combine_weights, int32_t* group_sizes, int32_t* group_offsets) {
  const size_t S = (size_t)T * k;
  int32_t* ids = (int32_t*)malloc(S * sizeof(int32_t));
  float* w = (float*)malloc(S * sizeof(float));
  float* p = (float*)malloc((size_t)E * sizeof(float));
  int32_t* fill = (int32_t*)calloc((size_t)E, sizeof(int32_t));
  if (!ids || !w || !p || !fill) { free(ids); free(w); free(p); free(fill); return -1; }
  for (int t = 0; t < T; ++t) {
    const float* row = scores + (size_t)t * E;
    float mx = row[0];
    for (int e = 1; e < E; ++e) mx = row[e] > mx ? row[e] : mx;
    float sum = 0.0f;
    for (int e = 0; e < E; ++e) { p[e] = expf(row[e] - mx); sum += p[e]; }
    for (int e = 0; e < E; ++e) p[e] /= sum;
    float wsum = 0.0f;
    for (int j = 0; j < k; ++j) {
      int best = -1;
      for (int e = 0; e < E; ++e)
        if (p[e] >= 0.0f && (best < 0 || p[e] > p[best])) best = e;
      ids[(size_t)t * k + j] = best;
      w[(size_t)t * k + j] = p[best];
      wsum += p[best];
      p[best] = -1.0f;
    }
    if (normalize && k > 1) {
      const float dsum = wsum > 0.0f ? wsum : 1.0f;
      for (int j = 0; j < k; ++j) w[(size_t)t * k + j] /= dsum;
    }
  }
  /* capacity drop, token-major then slot-minor; then counting sort by expert */
  for (int e = 0; e < E; ++e) group_sizes[e] = 0;
  for (size_t s = 0; s < S; ++s) {
    const int e = ids[s];
    if (capacity > 0 && fill[e] >= capacity) ids[s] = -1;
    else { fill[e]++; group_sizes[e]++; }
  }
  int off = 0;
  for (int e = 0; e < E; ++e) { group_offsets[e] = off; off += group_sizes[e]; fill[e] = 0; }
  group_offsets[E] = off;
  for (size_t s = 0; s < S; ++s) {
    const int e = ids[s];
    if (e < 0) continue;
    const int pos = group_offsets[e] + fill[e]++;
    token_of_slot[pos] = (int32_t)(s / k);
    expert_of_slot[pos] = e;
    combine_weights[pos] = w[s];
  }
  free(ids); free(w); free(p); free(fill);
  return off;
}
