/*
 * tessera_gfx950.h — C ABI of libtessera_gfx950.so, the MI355X (gfx950 / CDNA4)
 * execution lane for Tessera's dense ops: GEMM (f16 / bf16 / int8 / fp8-e4m3),
 * flash-attention forward (causal, GQA, LSE) and the MoE grouped-GEMM block
 * (routing metadata, dispatch, grouped GEMM, fused SwiGLU, combine).
 *
 * Conventions follow the reference's shipped ROCm libraries
 * (src/compiler/codegen/Tessera_ROCM_Backend/runtime/hip/tessera_rocm_gemm.cpp:843-856,
 *  .../tessera_rocm_flash_attn.cpp:259-278, python/tessera/runtime.py:1987-1988):
 *
 *   - symbols are  tessera_<backend>_<op>_<dtype>  with C linkage;
 *   - every array is contiguous row-major; dims are C int;
 *   - the return code is 0 ok / 1 bad shape or argument (checked before the
 *     device is touched) / 2 no usable gfx950 device / 3 a device operation
 *     failed;
 *   - no C++ exception crosses the boundary.
 *
 * Two families of entry points:
 *
 *   host-pointer  (no suffix)   pointers are HOST memory owned by the caller; the
 *                               library allocates device memory, copies in, runs,
 *                               copies out and frees — the reference's convention,
 *                               a drop-in for its ctypes bindings.
 *   device-pointer (_dev)       pointers are DEVICE memory, the trailing
 *                               `void* stream` is a hipStream_t (NULL = default
 *                               stream); the call enqueues and returns without
 *                               synchronising.  This is the resident-buffer form
 *                               used for chained ops and for timing.
 *
 * Threads.  The host-pointer entry points (and tessera_gfx950_gpu_launcher, which calls
 * them) are re-entrant, like the reference's, which allocate per call: the library
 * serialises them internally (one lock from a call's first allocation to its last
 * download), so any number of host threads may be inside them at once and each gets the
 * result the call gives alone.  They do not overlap with each other on the device.
 *
 * Temporaries of the _dev entry points (split-K partials, routing and combine lists,
 * quantiser maxima) come from one workspace per (device, stream) that the library
 * grows on demand: a call that needs more than any earlier call on its stream makes
 * one hipMalloc (no free, no synchronisation; the outgrown buffer is kept for the
 * work still queued on it), every other call allocates nothing.  All calls on one
 * stream share that workspace from its first byte, so the host threads that enqueue
 * on one stream must be serialised by the caller.  The workspace lives until
 * tessera_gfx950_stream_release(stream) or the end of the process; release a stream's
 * workspace before destroying the stream (a new stream may be given the old handle).
 *
 * HIP graphs.  A _dev call that uses the workspace must have been made once EAGERLY on the
 * stream, with arguments at least as large, before it is recorded into a stream capture:
 * the first call (or a larger one) allocates, which a capture does not allow, and the
 * recorded kernels hold the workspace's address.  Replay such a graph on the stream it was
 * captured on (launched elsewhere it shares that stream's workspace with eager calls on it
 * and races with them), and do not release the stream's workspace while the graph is in
 * use.  tessera_gfx950_moe_layer_bf16_dev takes a caller-owned workspace instead: given the
 * router logits it uses no memory of the library's and has neither restriction (given a router
 * weight, the router product is a GEMM like any other and may split K through the stream's
 * workspace).  Any entry point (tessera_gfx950_probe is the cheapest) must have
 * been called once before the first capture: the first call initialises the device.
 */
#ifndef TESSERA_GFX950_H
#define TESSERA_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TESSERA_GFX950_OK 0
#define TESSERA_GFX950_BAD_SHAPE 1
#define TESSERA_GFX950_NO_DEVICE 2
#define TESSERA_GFX950_DEVICE_FAILED 3

/* ---- lane / device management ------------------------------------------- */

/* ABI version of this header (bumped on incompatible change). */
int tessera_gfx950_abi_version(void);
/* 0 iff device 0 exists and is a gfx950 part; else 2.  The cached host probe the
 * reference's lanes expose through their 16x16x16 zero-GEMM
 * (python/tessera/runtime.py:1992-2033). */
int tessera_gfx950_probe(void);
/* Waits for `stream` (a hipStream_t; NULL = the default stream) and frees the workspace the
 * library keeps for it on the current device.  A later _dev call on the stream allocates a
 * new one.  No counterpart in the reference (its entry points allocate per call). */
int tessera_gfx950_stream_release(void* stream);
/* Writes the gcnArchName / marketing name (NUL-terminated, truncated). */
int tessera_gfx950_device_name(char* buf, int buflen);
int tessera_gfx950_device_cus(int* cus);

/* Raw device buffers for callers without their own allocator (the Python host
 * side is ctypes-only, as Tessera never imports PyTorch).  Mirrors the buffer
 * half of the tsr* runtime ABI (src/runtime/include/tessera/tessera_runtime.h:14-148). */
int tessera_gfx950_malloc(void** dptr, size_t bytes);
int tessera_gfx950_free(void* dptr);
int tessera_gfx950_memcpy_h2d(void* dst, const void* src, size_t bytes);
int tessera_gfx950_memcpy_d2h(void* dst, const void* src, size_t bytes);
int tessera_gfx950_memset(void* dst, int value, size_t bytes);
/* Device-to-device copy kernel on a stream (bytes and both pointers multiples of
 * 16).  Lets a caller chain resident buffers without a host round trip, the role
 * of the device-operand lease in python/tessera/runtime.py:1549-1614; also the
 * known-size kernel HBM byte counters are calibrated against. */
int tessera_gfx950_memcpy_d2d_dev(void* dst, const void* src, size_t bytes, void* stream);
int tessera_gfx950_synchronize(void);

/* Device-event timer on a stream (NULL = default stream): the timing clock the
 * reference's bench ABI uses (tessera_rocm_gemm.cpp:567-667). */
int tessera_gfx950_timer_create(void** timer);
int tessera_gfx950_timer_start(void* timer, void* stream);
int tessera_gfx950_timer_stop(void* timer, void* stream);
/* Blocks until the stop event completed; *ms = elapsed device time. */
int tessera_gfx950_timer_elapsed_ms(void* timer, float* ms);
int tessera_gfx950_timer_destroy(void* timer);

/* ---- GEMM  D[M,N] = A[M,K] . B[K,N]  ------------------------------------- */

/* Call-compatible with tessera_rocm_wmma_gemm_{f16,bf16}
 * (tessera_rocm_gemm.cpp:843-856): 16-bit storage, f32 accumulate, f32 D. */
int tessera_gfx950_gemm_f16(const void* A, const void* B, void* D, int M, int N, int K);
int tessera_gfx950_gemm_bf16(const void* A, const void* B, void* D, int M, int N, int K);
/* Result stored back in the operand storage dtype (RNE) — the ops.gemm rule
 * for reduced-precision operands (python/tessera/__init__.py:5824-5855). */
int tessera_gfx950_gemm_f16_f16(const void* A, const void* B, void* D, int M, int N, int K);
int tessera_gfx950_gemm_bf16_bf16(const void* A, const void* B, void* D, int M, int N, int K);
/* ops.batched_gemm (python/tessera/__init__.py:250-254): `batch` independent
 * products, operands densely stacked; f32 D. */
int tessera_gfx950_batched_gemm_f16(const void* A, const void* B, void* D, int batch, int M, int N, int K);
int tessera_gfx950_batched_gemm_bf16(const void* A, const void* B, void* D, int batch, int M, int N, int K);

/* int8 x int8 -> int32, bit-exact (the int8 contract of the compiled ROCm
 * GEMM executor, python/tessera/runtime.py:6500-6513; integer reference
 * avx512_vnni_gemm_int8.cpp:5-18 / amx_gemm_int8.cpp:34-100). */
int tessera_gfx950_gemm_i8_i32(const void* A, const void* B, void* C, int M, int N, int K);
/* W8A8 direct-consume GEMM (python/tessera/compiler/smoothquant.py:115-124):
 * D[m,n] = f32(acc[m,n]) * row_scale[m] * col_scale[n], two f32 multiplies in
 * that order.  acc_out (int32[M,N]) may be NULL. */
int tessera_gfx950_gemm_w8a8_f32(const void* A, const void* B, const float* row_scale,
                                 const float* col_scale, void* D, void* acc_out,
                                 int M, int N, int K);
/* fp8 e4m3fn (OCP) codes, per-tensor scales: D = f32acc(A.B) * scale_a * scale_b
 * (python/tessera/__init__.py:3340-3374 defines the codes; GEMM over raw fp8
 * bytes as tessera_nvidia_mma_gemm_e4m3, tessera_nvidia_gemm.cpp:555-556).
 * Precision of the accumulation: the fp8 matrix instruction adds each run of 8 consecutive k
 * with the products aligned to the run's largest one, and a product more than 13 binary places
 * below that one is dropped (truncated); runs are added to each other in f32. */
int tessera_gfx950_gemm_e4m3_bf16(const void* A, const void* B, float scale_a, float scale_b,
                                  void* D, int M, int N, int K);
int tessera_gfx950_gemm_e4m3_f32(const void* A, const void* B, float scale_a, float scale_b,
                                 void* D, int M, int N, int K);
/* The same over fp8 e5m2 (OCP) codes, the format table's second fp8 grid
 * (python/tessera/runtime.py:16939-16940; GEMM over raw bytes as tessera_nvidia_mma_gemm_e5m2,
 * compiler/codegen/tessera_gpu_backend_NVIDIA): the matrix instruction's operand format 1. */
int tessera_gfx950_gemm_e5m2_bf16(const void* A, const void* B, float scale_a, float scale_b,
                                  void* D, int M, int N, int K);
int tessera_gfx950_gemm_e5m2_f32(const void* A, const void* B, float scale_a, float scale_b,
                                 void* D, int M, int N, int K);

int tessera_gfx950_gemm_f16_dev(const void* A, const void* B, void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_bf16_dev(const void* A, const void* B, void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_f16_f16_dev(const void* A, const void* B, void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_bf16_bf16_dev(const void* A, const void* B, void* D, int M, int N, int K, void* stream);
int tessera_gfx950_batched_gemm_f16_dev(const void* A, const void* B, void* D, int batch, int M, int N, int K, void* stream);
int tessera_gfx950_batched_gemm_bf16_dev(const void* A, const void* B, void* D, int batch, int M, int N, int K, void* stream);
/* Strided batch: product z of `batch` reads A + z*stride_a and B + z*stride_b and writes
 * D + z*stride_d (strides in elements).  A stride of 0 shares that operand between all
 * products — np.matmul's broadcast of a 2-D weight over a stacked activation, which is
 * what ops.batched_gemm is (python/tessera/__init__.py:250-254) — in one launch and
 * without materialising the copies.  stride_d >= M*N.  out_dtype: 0 = f32 D, 1 = D in the
 * operand storage dtype. */
int tessera_gfx950_batched_gemm_strided_f16_dev(const void* A, const void* B, void* D, int batch, int M, int N, int K,
                                                int64_t stride_a, int64_t stride_b, int64_t stride_d, int out_dtype,
                                                void* stream);
int tessera_gfx950_batched_gemm_strided_bf16_dev(const void* A, const void* B, void* D, int batch, int M, int N, int K,
                                                 int64_t stride_a, int64_t stride_b, int64_t stride_d, int out_dtype,
                                                 void* stream);
int tessera_gfx950_gemm_i8_i32_dev(const void* A, const void* B, void* C, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_w8a8_f32_dev(const void* A, const void* B, const float* row_scale,
                                     const float* col_scale, void* D, void* acc_out,
                                     int M, int N, int K, void* stream);
int tessera_gfx950_gemm_e4m3_bf16_dev(const void* A, const void* B, float scale_a, float scale_b,
                                      void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_e4m3_f32_dev(const void* A, const void* B, float scale_a, float scale_b,
                                     void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_e5m2_bf16_dev(const void* A, const void* B, float scale_a, float scale_b,
                                      void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_e5m2_f32_dev(const void* A, const void* B, float scale_a, float scale_b,
                                     void* D, int M, int N, int K, void* stream);

/* Fused matmul epilogue  D f32 = act(A . B + bias[n]):  the bias operand and
 * `activation` kwarg of the compiled-GEMM executor's tessera.fused_epilogue op
 * (python/tessera/runtime.py:6603-6650) and the (has_bias, activation) epilogue of
 * the matrix-core candidate (python/tessera/compiler/emit/rocm_hip.py:679-699).
 * bias is f32[N] or NULL; activation: 0 none, 1 relu, 2 gelu (tanh form, argument
 * clamped to +-30), 3 silu, 4 sigmoid, 5 tanh — the reference's epilogue
 * vocabulary (python/tessera/compiler/fusion_core.py:121-138).  Any other code is
 * a bad-shape error. */
int tessera_gfx950_gemm_bias_act_f16(const void* A, const void* B, const float* bias, int activation,
                                     void* D, int M, int N, int K);
int tessera_gfx950_gemm_bias_act_bf16(const void* A, const void* B, const float* bias, int activation,
                                      void* D, int M, int N, int K);
int tessera_gfx950_gemm_bias_act_f16_dev(const void* A, const void* B, const float* bias, int activation,
                                         void* D, int M, int N, int K, void* stream);
int tessera_gfx950_gemm_bias_act_bf16_dev(const void* A, const void* B, const float* bias, int activation,
                                          void* D, int M, int N, int K, void* stream);
/* Gated projection  D f32 [M,H] = act(A . Wg) * (A . Wu),  A [M,K], Wg/Wu [K,H]:
 * GatedMatmulRegion (python/tessera/compiler/fusion_core.py:747-782); f32
 * accumulators go through the activation and the product unrounded. */
int tessera_gfx950_gated_gemm_f16(const void* A, const void* Wg, const void* Wu, int activation, void* D,
                                  int M, int H, int K);
int tessera_gfx950_gated_gemm_bf16(const void* A, const void* Wg, const void* Wu, int activation, void* D,
                                   int M, int H, int K);
int tessera_gfx950_gated_gemm_f16_dev(const void* A, const void* Wg, const void* Wu, int activation, void* D,
                                      int M, int H, int K, void* stream);
int tessera_gfx950_gated_gemm_bf16_dev(const void* A, const void* Wg, const void* Wu, int activation, void* D,
                                       int M, int H, int K, void* stream);

/* The schedule the GEMM launcher picks for an aligned problem (workgroup tile and
 * K split), as a host-only query: the gfx950 counterpart of
 * select_rocm_gemm_schedule (python/tessera/compiler/rocm_schedule.py:94-154), which
 * the reference's executor consults before building a kernel
 * (python/tessera/runtime.py:6676-6679).  elem_bytes 2 = f16/bf16, 1 = int8/fp8. */
int tessera_gfx950_gemm_schedule(int M, int N, int K, int batch, int elem_bytes,
                                 int* tile_m, int* tile_n, int* tile_k, int* split_k);

/* A product on 256 x 256 tiles whose tile count is a little over a multiple of the 256 compute
 * units: the tiles beyond the last full round (*rest_tiles of them) are split along K into
 * *rest_split parts each by a second launch and summed by a third, so that round fills the chip.
 * *rest_split == 1: every tile is computed whole by one launch (*rest_tiles is then 0).
 * Host-only query beside tessera_gfx950_gemm_schedule; 16-bit operands.  No counterpart in the
 * reference, whose schedule has no such step. */
int tessera_gfx950_gemm_rest_split(int M, int N, int K, int batch, int* rest_tiles, int* rest_split);

/* Kernel-only benchmark with resident, library-owned buffers: warm-up, `iters`
 * launches between HIP events, cross-checked against wall clock
 * (tessera_rocm_gemm.cpp:551-667).  *avg_ms = mean per-launch ms. */
int tessera_gfx950_gemm_bf16_bench(int M, int N, int K, int iters, double* avg_ms);
/* The f16 form with the parameter list of tessera_rocm_wmma_gemm_f16_bench
 * (tessera_rocm_gemm.cpp:861-866), so a caller of that symbol binds this one unchanged.
 * There mt / nt choose the register blocking of the benchmarked variant; here the
 * launcher picks the tile from the shape (tessera_gfx950_gemm_schedule tells which), so
 * they are validated (> 0, else 1) and otherwise unused.  f16 in, f16 out. */
int tessera_gfx950_gemm_f16_bench(int M, int N, int K, int iters, int mt, int nt, double* avg_ms);
/* The same loop cycling over `weights` (1..64) distinct B matrices: a weight matrix
 * that would fit the memory-side cache is then streamed from HBM on every launch,
 * as the layers of a decode step are.  No counterpart in the reference. */
int tessera_gfx950_gemm_bf16_bench_rotating(int M, int N, int K, int iters, int weights,
                                            double* avg_ms);
/* The bench ABI for the attention forward (the reference has it for the GEMM only): the
 * same warm-up / HIP-event / wall-clock loop over tessera_gfx950_flash_attn_gqa_bf16_dev
 * with bf16 output, scale 1/sqrt(D), on library-owned buffers filled with one constant
 * (on this part a kernel's rate depends on its operand values; this figure is the one for
 * operands that toggle nothing).  tessera_gfx950_bench_last_timer_source() answers for it
 * as well. */
int tessera_gfx950_flash_attn_bf16_bench(int B, int Hq, int Hkv, int Sq, int Sk, int D, int causal, int iters,
                                         double* avg_ms);
/* 0 = device events, 1 = host wall clock, -1 = no measurement yet
 * (tessera_rocm_bench_last_timer_source, tessera_rocm_gemm.cpp:567-580). */
int tessera_gfx950_bench_last_timer_source(void);

/* Register-only matrix-pipe probe for the bench: 1024 workgroups of 4 waves, each wave
 * holding 16 independent 32x32x16 bf16 accumulators and issuing `rounds` rounds of those
 * 16 MFMAs with no memory access inside the loop.  The rate it reaches is what the
 * matrix pipes deliver on the given operand VALUES at the clock the board grants for them
 * (operand toggling sets the power draw, the power limit sets the clock), i.e. the
 * ceiling a GEMM on such data is priced against on this board.  No counterpart in the
 * reference (its bench ABI times whole GEMMs, tessera_rocm_gemm.cpp:551-667).
 * fragments: device memory, 16 wave patterns x 8 fragments x 64 lanes x 16 bytes =
 * 131072 bytes of bf16 values (wave w of the grid uses pattern w % 16: fragments 0-3 as A,
 * 4-7 as B operands); sink: device memory, 1024 * 256 floats; *flop (may be NULL) receives
 * the floating-point operations of one launch. */
int tessera_gfx950_mfma_probe_bf16_dev(const void* fragments, int rounds, void* sink, double* flop, void* stream);
/* The same probe for the other matrix instructions of the lane: kind 0 = 32x32x16 bf16 (the
 * call above), 1 = 32x32x32 int8 (int32 accumulate; the fragments are int8 values), 2 =
 * 32x32x64 fp8 e4m3 in its unscaled form (the fragments are e4m3 codes; a 32-byte operand is
 * two neighbouring 16-byte fragments), 3 = 16x16x32 bf16 (the instruction of the 256 x 256
 * GEMM tile; a quarter of the accumulator registers per instruction, 64 accumulators and
 * MFMAs per round).  *ops receives the operations of one launch (2 * m * n * k per
 * instruction).  No counterpart in the reference. */
int tessera_gfx950_mfma_probe_dev(int kind, const void* fragments, int rounds, void* sink, double* ops, void* stream);

/* ---- quantisers ------------------------------------------------------------ */

/* ops.quantize_fp8(format="e4m3") (python/tessera/__init__.py:3340-3374; grid as
 * scalar_fpquant(v,448,3,-6), avx512_fpquant_f32.cpp:28-41): codes[i] = e4m3fn
 * byte of clip(x[i]/scale, +-448) rounded RNE.  scale <= 0 means "compute
 * max(amax/448, 1e-12)"; the scale used is written to *scale_out. */
int tessera_gfx950_quantize_e4m3_f32(const float* x, int64_t n, float scale, void* codes, float* scale_out);
/* The same to e5m2 codes: scale = max(amax / 57344, 1e-12), clip to +-57344, round to nearest even
 * with gradual underflow below 2^-14 (the grid (57344, 2, -14) of the format table). */
int tessera_gfx950_quantize_e5m2_f32(const float* x, int64_t n, float scale, void* codes, float* scale_out);
/* _quantize_int8_per_channel (python/tessera/compiler/smoothquant.py:79-84):
 * axis=1 -> one scale per row (scales[M]); axis=0 -> one per column (scales[N]). */
int tessera_gfx950_quantize_i8_f32(const float* x, int M, int N, int axis, void* q, float* scales);
/* quantization.quantize_int8, symmetric form (python/tessera/quantization.py:24-37): one scale for
 * the whole tensor — `scale` if > 0, else max|x| / 127 found on the device (1 for an all-zero
 * tensor) — and q = clip(rint(x / scale), -127, 127).  scale_out (optional) receives the scale. */
int tessera_gfx950_quantize_i8_tensor_f32(const float* x, int64_t n, float scale, void* q, float* scale_out);
int tessera_gfx950_quantize_i8_tensor_f32_dev(const float* x, int64_t n, float scale, void* q, float* scale_out_dev,
                                              void* stream);
/* The activation side of smoothquant_matmul (python/tessera/compiler/smoothquant.py:60-62, 115-122):
 * x_hat[m][n] = x[m][n] / smoothing[n] (f32 division), then the per-row quantiser above on x_hat,
 * in one pass over x.  smoothing f32[N]; q int8 [M,N]; scales f32[M]. */
int tessera_gfx950_quantize_i8_smoothed_f32(const float* x, int M, int N, const float* smoothing, void* q, float* scales);
int tessera_gfx950_quantize_i8_smoothed_f32_dev(const float* x, int M, int N, const float* smoothing, void* q,
                                                float* scales, void* stream);
/* ops.quantize_nvfp4 followed by ops.dequantize_nvfp4 (python/tessera/__init__.py:3472-3504, i.e.
 * compiler/microscaling.py:317-384 with the nvfp4 format): x f32 [rows, cols] rounded onto the
 * NVFP4 grid in blocks of 16 along the last axis — block scale = max(amax / 6, 1e-30) rounded to
 * e4m3fn, codes on the E2M1 grid {0, .5, 1, 1.5, 2, 3, 4, 6}, nearest even.  dq (f32) and / or
 * dq_bf16 (the same values as bf16 bit patterns, exact) receive the dequantised values, scales
 * (optional) the block scales, [rows, ceil(cols / 16)].  This is what the reference's
 * grouped_gemm(quant="nvfp4") applies to x and to each expert's weight before its f32 product
 * (compiler/grouped_layout.py:353-392). */
int tessera_gfx950_fake_quantize_nvfp4_f32(const float* x, int rows, int cols, float* dq, void* dq_bf16, float* scales);
int tessera_gfx950_fake_quantize_nvfp4_f32_dev(const float* x, int rows, int cols, float* dq, void* dq_bf16,
                                               float* scales, void* stream);
/* tessera_x86_avx512_fpquant_f32
 * (src/compiler/codegen/tessera_x86_backend/src/kernels/avx512_fpquant_f32.cpp:45-83; the scalar
 * definition at :28-41): out[i] = x[i] snapped to the float grid (max_normal, mantissa_bits,
 * min_exp) — ax = min(|x|, max_normal); e = max(floor(log2 ax), min_exp); ulp = 2^(e - mantissa_bits);
 * out = sign(x) min(rne(ax / ulp) ulp, max_normal); NaN propagates.  The reference's format table
 * (python/tessera/runtime.py:16939-16946): e4m3 (448, 3, -6), e5m2 (57344, 2, -14), e2m3
 * (7.5, 3, -126), e3m2 (28, 2, -126), e2m1 (6, 1, -126).  mantissa_bits in [0, 23], min_exp in
 * [-126, 127], max_normal finite and positive, else TSR_BAD_SHAPE. */
int tessera_gfx950_fpquant_f32(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp, float* out);
int tessera_gfx950_fpquant_f32_dev(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp,
                                   float* out, void* stream);
/* ops.quantize_fp8 / quantize_fp6 / quantize_fp4 (python/tessera/__init__.py:3340-3374, 3411-3464):
 * per-tensor scale = `scale` if > 0, else max(amax|x| / max_normal, 1e-12) found on the device;
 * grid = fpquant(x / scale) as above; dq (f32, optional) receives grid * scale, the reference's
 * return value; grid_bf16 (optional) the unscaled grid values as bf16 bit patterns, exact for
 * every format of the table above, i.e. a ready operand for a 16-bit product that is scaled
 * afterwards; scale_out (optional) the scale used.  With the automatic scale a NaN in x is
 * skipped by the maximum (the reference's numpy maximum would return NaN for everything). */
int tessera_gfx950_fake_quantize_fp_f32(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp,
                                        float scale, float* dq, void* grid_bf16, float* scale_out);
int tessera_gfx950_fake_quantize_fp_f32_dev(const float* x, int64_t n, float max_normal, int mantissa_bits, int min_exp,
                                            float scale, float* dq, void* grid_bf16, float* scale_out_dev, void* stream);
int tessera_gfx950_quantize_e4m3_f32_dev(const float* x, int64_t n, float scale, void* codes, float* scale_out_dev, void* stream);
int tessera_gfx950_quantize_e5m2_f32_dev(const float* x, int64_t n, float scale, void* codes, float* scale_out_dev, void* stream);
int tessera_gfx950_quantize_i8_f32_dev(const float* x, int M, int N, int axis, void* q, float* scales, void* stream);

/* ---- flash-attention forward ---------------------------------------------- */

/* Call-compatible with tessera_rocm_wmma_flash_attn_{f16,bf16}
 * (tessera_rocm_flash_attn.cpp:259-278): Q [B,H,Sq,D], K/V [B,H,Sk,D] 16-bit,
 * O [B,H,Sq,D] f32; causal mask bottom-right aligned (key j visible to query i
 * iff j <= i + max(Sk-Sq,0)); D % 16 == 0, D <= 256. */
int tessera_gfx950_flash_attn_f16(const void* Q, const void* K, const void* V, void* O,
                                  int B, int H, int Sq, int Sk, int D, float scale, int causal);
int tessera_gfx950_flash_attn_bf16(const void* Q, const void* K, const void* V, void* O,
                                   int B, int H, int Sq, int Sk, int D, float scale, int causal);
/* GQA + LSE superset (executor contract python/tessera/runtime.py:7229-7475; GQA
 * head map and LSE as avx512_flash_attn_f32.cpp:379-422): Q [B,Hq,Sq,D],
 * K/V [B,Hkv,Sk,D], kv head = hq*Hkv/Hq; O f32 [B,Hq,Sq,D]; LSE f32 [B,Hq,Sq]
 * (natural log, scaled logits) may be NULL. */
int tessera_gfx950_flash_attn_gqa_f16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                      int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal);
int tessera_gfx950_flash_attn_gqa_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                       int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale, int causal);
/* out_dtype: 0 = f32 O, 1 = O in the input storage dtype. */
int tessera_gfx950_flash_attn_gqa_f16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                          int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                          int causal, int out_dtype, void* stream);
int tessera_gfx950_flash_attn_gqa_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                           int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                           int causal, int out_dtype, void* stream);

/* Sliding window and logit soft cap, the kwargs `window` / `logit_softcap` of the
 * reference's attention executor (python/tessera/runtime.py:7318-7335) with the
 * bounds and score transform of its CPU kernel (avx512_flash_attn_f32.cpp:115-196):
 * window > 0 keeps, per query row i, the `window` keys ending at the causal diagonal
 * i + max(Sk - Sq, 0) (causal != 0) or window/2 keys either side of it (causal == 0);
 * softcap > 0 passes each scaled score through cap * tanh(s / cap) before the
 * softmax.  0 disables either.  A row with no visible key gives O = 0, LSE = -inf. */
int tessera_gfx950_flash_attn_ext_f16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                      int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                      int causal, int window, float softcap);
int tessera_gfx950_flash_attn_ext_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                       int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                       int causal, int window, float softcap);
int tessera_gfx950_flash_attn_ext_f16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                          int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                          int causal, int window, float softcap, int out_dtype,
                                          void* stream);
int tessera_gfx950_flash_attn_ext_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                           int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                           int causal, int window, float softcap, int out_dtype,
                                           void* stream);

/* Attention forward on strided operands, so that a projection GEMM's output feeds the
 * kernel where it lies (the reference copies per op, tessera_rocm_gemm.cpp:450-475; its
 * executor takes [..., H, S, D] only, python/tessera/runtime.py:7229-7475 — no counterpart
 * for other layouts).  strides: 12 element strides, (batch, head, row) for Q, K, V, O in
 * that order; element (b, h, s, d) of X lies at X[b*batch + h*head + s*row + d], the last
 * dimension is contiguous.  [B,S,H,D] is (S*H*D, D, H*D); the Q / K / V column blocks of a
 * fused (B*S) x ((Hq + 2 Hkv) * D) projection are (S*W, D, W) with W the row width and the
 * pointers offset to the block's first column.  Strides must be >= 0 (row >= D); the MFMA
 * kernel needs pointers and strides that are multiples of 8 elements, anything else takes
 * the per-row kernel.  O (f32 for out_dtype 0, else the storage dtype) is written through
 * its own strides; LSE is contiguous [B,Hq,Sq] f32 or NULL.  window / softcap as in the
 * _ext entry points (0 = none). */
int tessera_gfx950_flash_attn_strided_f16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                              int Hq, int Hkv, int Sq, int Sk, int D, const int64_t* strides,
                                              float scale, int causal, int window, float softcap, int out_dtype,
                                              void* stream);
int tessera_gfx950_flash_attn_strided_bf16_dev(const void* Q, const void* K, const void* V, void* O, void* LSE, int B,
                                               int Hq, int Hkv, int Sq, int Sk, int D, const int64_t* strides,
                                               float scale, int causal, int window, float softcap, int out_dtype,
                                               void* stream);

/* Additive attention bias: O = softmax(scale Q K^T + bias, ...) V with bias an f32
 * tensor [B, Hq, Sq, Sk] (the caller broadcasts, as the reference's executor does for
 * its fourth operand, python/tessera/runtime.py:7270-7274); NULL means none.  With a
 * soft cap the bias is added after the cap (avx512_flash_attn_f32.cpp:199-206). */
int tessera_gfx950_flash_attn_bias_f16(const void* Q, const void* K, const void* V, const float* bias,
                                       void* O, void* LSE, int B, int Hq, int Hkv, int Sq, int Sk,
                                       int D, float scale, int causal, int window, float softcap);
int tessera_gfx950_flash_attn_bias_bf16(const void* Q, const void* K, const void* V, const float* bias,
                                        void* O, void* LSE, int B, int Hq, int Hkv, int Sq, int Sk,
                                        int D, float scale, int causal, int window, float softcap);
int tessera_gfx950_flash_attn_bias_f16_dev(const void* Q, const void* K, const void* V, const float* bias,
                                           void* O, void* LSE, int B, int Hq, int Hkv, int Sq, int Sk,
                                           int D, float scale, int causal, int window, float softcap,
                                           int out_dtype, void* stream);
int tessera_gfx950_flash_attn_bias_bf16_dev(const void* Q, const void* K, const void* V, const float* bias,
                                            void* O, void* LSE, int B, int Hq, int Hkv, int Sq, int Sk,
                                            int D, float scale, int causal, int window, float softcap,
                                            int out_dtype, void* stream);

/* ---- flash-attention backward -------------------------------------------- */

/* (dQ, dK, dV) of O = softmax(scale Q K^T, causal) V given dO: the contract of the
 * reference's backward lane (python/tessera/runtime.py:7598-7665: operands
 * (dO, Q, K, V), Q/dO [B,Hq,Sq,D], K/V [B,Hkv,Sk,D], Hq % Hkv == 0, head_dim a
 * multiple of 16, f16/bf16 storage, f32 accumulate) and the arithmetic of
 * vjp_flash_attn (python/tessera/autodiff/vjp.py:1311-1377).  dQ, dK, dV are f32,
 * shaped like Q, K, V; dK / dV of a KV head sum over the query heads of its group.
 * The host-pointer forms recompute the forward (nothing saved), as the reference
 * does.  The _dev forms also accept the forward's saved O (f32) and LSE; pass both
 * NULL to recompute. */
int tessera_gfx950_flash_attn_bwd_f16(const void* dO, const void* Q, const void* K, const void* V,
                                      void* dQ, void* dK, void* dV, int B, int Hq, int Hkv,
                                      int Sq, int Sk, int D, float scale, int causal);
int tessera_gfx950_flash_attn_bwd_bf16(const void* dO, const void* Q, const void* K, const void* V,
                                       void* dQ, void* dK, void* dV, int B, int Hq, int Hkv,
                                       int Sq, int Sk, int D, float scale, int causal);
int tessera_gfx950_flash_attn_bwd_f16_dev(const void* dO, const void* Q, const void* K, const void* V,
                                          const void* O, const void* LSE, void* dQ, void* dK, void* dV,
                                          int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                          int causal, void* stream);
int tessera_gfx950_flash_attn_bwd_bf16_dev(const void* dO, const void* Q, const void* K, const void* V,
                                           const void* O, const void* LSE, void* dQ, void* dK, void* dV,
                                           int B, int Hq, int Hkv, int Sq, int Sk, int D, float scale,
                                           int causal, void* stream);

/* ---- MoE -------------------------------------------------------------------- */

/* Router + packing plan in the canonical int32 device ABI
 * (python/tessera/compiler/moe_transport.py:194-273).  Restates
 * distributed.moe.route_tokens (python/tessera/distributed/moe.py:119-206) and
 * the slot sort of nn.functional.moe_layer (python/tessera/nn/functional.py:463-476):
 * f32 softmax over E experts, top-k descending (ties -> lowest expert id, the
 * rule of models/moe_routing.py:69-70), weights renormalised when
 * normalize != 0 and k > 1, first-come capacity drop in token-major order when
 * capacity > 0, kept slots stable-sorted by expert.
 * Outputs: token_of_slot/expert_of_slot int32[T*k], combine_weights f32[T*k]
 * (first *num_slots entries valid), group_sizes int32[E], group_offsets
 * int32[E+1]. */
int tessera_gfx950_moe_route_f32(const float* scores, int T, int E, int k, int normalize, int capacity,
                                 int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                 int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots);
int tessera_gfx950_moe_route_f32_dev(const float* scores, int T, int E, int k, int normalize, int capacity,
                                     int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                     int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots,
                                     void* stream);

/* The same routing for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Identical arguments, kernels and results as
 * tessera_gfx950_moe_route_f32_dev, but the temporaries (token-major expert ids and
 * weights, per-chunk histograms) live in a fixed 4 MiB device array inside the
 * library image instead of the per-stream workspace: the call makes no hipMalloc,
 * hipFree or other allocating call.  Limit: 2 * roundup(T*k*4, 256) +
 * ceil(T*k / 512) * E * 4 <= 4 MiB (T*k up to about 490,000 slots at E = 64), else
 * rc 1.  Every call on one GPU shares that array, so two such calls that overlap on
 * one GPU (different streams, or different host threads) race; calls on one stream
 * are safe back to back.  The array's device address is looked up when the library first
 * touches the device (any entry point; tessera_gfx950_probe does it), so make one library
 * call before the first stream capture; after that this entry point records into a capture
 * and replays like any kernel launch.  All pointers are device memory. */
int tessera_gfx950_moe_route_f32_noalloc_dev(const float* scores, int T, int E, int k, int normalize, int capacity,
                                             int32_t* token_of_slot, int32_t* expert_of_slot,
                                             float* combine_weights, int32_t* group_sizes,
                                             int32_t* group_offsets, int32_t* num_slots, void* stream);

/* The reference's second router and its packing plan
 * (python/tessera/models/moe_routing.py:54-113, python/tessera/stdlib/moe.py:79-134).
 * With router_logits (f32 [T,E]; k <= 64): route_top_k — the k largest LOGITS per token,
 * descending, ties to the lowest expert id; weights = softmax over the k selected logits
 * (normalize == 1) or 1/k each (normalize == 0); written to expert_ids / weights ([T,k],
 * rank order).  normalize == 2 / 3 select distributed.moe.route_tokens' router instead
 * (python/tessera/distributed/moe.py:164-176): softmax over all E experts, the k largest
 * probabilities, renormalised over the k (2; for k > 1) or as they are (3) — the token-major
 * view (expert_ids, weights, kept_mask) of the routing tessera_gfx950_moe_route_f32 packs,
 * which is what RoutingResult.assignment / weights are made of (any k <= E).  Other values
 * of normalize are rc 1.  With router_logits NULL the selection is given instead (given_expert_ids
 * int32 [T,k] with values in [0,E) — anything else is rc 1 in the host form —
 * given_weights f32 [T,k] or NULL): plan_packing / plan_dispatch on a caller's routing.
 * Then the plan: slots are taken in token-major order, an expert keeps its first
 * `capacity` slots (capacity <= 0: all), kept slots are stable-sorted by expert.
 *   kept_mask     uint8 [T,k]   1 = kept
 *   sort_perm     int32 [S]     kept token-major slot ids in packed order (S = *num_slots)
 *   inverse_perm  int32 [T*k]   packed position of each slot, -1 for a dropped one
 *                               (without a capacity: the inverse permutation of sort_perm)
 *   token_of_slot / expert_of_slot / combine_weights / group_sizes / group_offsets: the
 *   transport descriptor of the same plan, as tessera_gfx950_moe_route_f32.
 * Every output except group_sizes / group_offsets may be NULL. */
int tessera_gfx950_moe_plan_f32(const float* router_logits, const int32_t* given_expert_ids,
                                const float* given_weights, int T, int E, int k, int normalize, int capacity,
                                int32_t* expert_ids, float* weights, uint8_t* kept_mask, int32_t* sort_perm,
                                int32_t* inverse_perm, int32_t* token_of_slot, int32_t* expert_of_slot,
                                float* combine_weights, int32_t* group_sizes, int32_t* group_offsets,
                                int32_t* num_slots);
int tessera_gfx950_moe_plan_f32_dev(const float* router_logits, const int32_t* given_expert_ids,
                                    const float* given_weights, int T, int E, int k, int normalize, int capacity,
                                    int32_t* expert_ids, float* weights, uint8_t* kept_mask, int32_t* sort_perm,
                                    int32_t* inverse_perm, int32_t* token_of_slot, int32_t* expert_of_slot,
                                    float* combine_weights, int32_t* group_sizes, int32_t* group_offsets,
                                    int32_t* num_slots, void* stream);
/* unpack_combine (python/tessera/models/moe_routing.py:103-111): out[t,:] = sum over the
 * token's k slots in rank order of y_packed[inverse_perm[t*k+j],:] * weights[t,j], each
 * product rounded to f32 before the add (numpy's (y_slots * w).sum(axis=1)); a dropped
 * slot (inverse_perm < 0) adds nothing, as in stdlib.moe.combine.  y_packed [S,N] bf16
 * or f32, out f32 [T,N]. */
int tessera_gfx950_moe_unpack_combine_bf16(const void* y_packed, const int32_t* inverse_perm, const float* weights,
                                           float* out, int T, int k, int S, int N);
int tessera_gfx950_moe_unpack_combine_f32(const void* y_packed, const int32_t* inverse_perm, const float* weights,
                                          float* out, int T, int k, int S, int N);
int tessera_gfx950_moe_unpack_combine_bf16_dev(const void* y_packed, const int32_t* inverse_perm,
                                               const float* weights, float* out, int T, int k, int S, int N,
                                               void* stream);
int tessera_gfx950_moe_unpack_combine_f32_dev(const void* y_packed, const int32_t* inverse_perm,
                                              const float* weights, float* out, int T, int k, int S, int N,
                                              void* stream);

/* tessera.moe_dispatch: x_perm[s,:] = x[token_of_slot[s],:]  (exact gather,
 * python/tessera/runtime.py:1791-1806).  elem_bytes = 1, 2 (f16/bf16), 4 (f32) or 8 (f64): rows are copied byte for byte. */
int tessera_gfx950_moe_dispatch(const void* x, const int32_t* token_of_slot, void* x_perm,
                                int T, int S, int H, int elem_bytes);
int tessera_gfx950_moe_dispatch_dev(const void* x, const int32_t* token_of_slot, void* x_perm,
                                    int T, int S, int H, int elem_bytes, void* stream);
/* tessera.moe_combine: out[t,:] = sum_{s: token_of_slot[s]=t} y_perm[s,:]*w[s],
 * f32 accumulation in slot order, out f32 [T,N]
 * (python/tessera/runtime.py:1807-1824; nn/functional.py:487-490). */
int tessera_gfx950_moe_combine_bf16(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                    float* out, int T, int S, int N);
int tessera_gfx950_moe_combine_f32(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                   float* out, int T, int S, int N);
int tessera_gfx950_moe_combine_bf16_dev(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                        float* out, int T, int S, int N, void* stream);
int tessera_gfx950_moe_combine_f32_dev(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                       float* out, int T, int S, int N, void* stream);

/* tessera.grouped_gemm: y[off_e:off_{e+1}] = x[off_e:off_{e+1}] . w[e] in one
 * launch over device offsets[E+1] (python/tessera/runtime.py:26657-26715;
 * python/tessera/__init__.py:291-351).  x [S,K], w [E,K,N] bf16; the _bf16 form
 * stores y in bf16 (storage rule), the _bf16_f32 form keeps f32. */
int tessera_gfx950_grouped_gemm_bf16(const void* x, const void* w, const int32_t* offsets, void* y,
                                     int S, int K, int N, int E);
int tessera_gfx950_grouped_gemm_bf16_f32(const void* x, const void* w, const int32_t* offsets, void* y,
                                         int S, int K, int N, int E);
int tessera_gfx950_grouped_gemm_bf16_dev(const void* x, const void* w, const int32_t* offsets, void* y,
                                         int S, int K, int N, int E, void* stream);
int tessera_gfx950_grouped_gemm_bf16_f32_dev(const void* x, const void* w, const int32_t* offsets, void* y,
                                             int S, int K, int N, int E, void* stream);
/* The same on f16 storage (the reference's grouped product takes any float dtype and applies the
 * storage rule: python/tessera/__init__.py:291-351, 5783-5855). */
int tessera_gfx950_grouped_gemm_f16(const void* x, const void* w, const int32_t* offsets, void* y,
                                    int S, int K, int N, int E);
int tessera_gfx950_grouped_gemm_f16_f32(const void* x, const void* w, const int32_t* offsets, void* y,
                                        int S, int K, int N, int E);
int tessera_gfx950_grouped_gemm_f16_dev(const void* x, const void* w, const int32_t* offsets, void* y,
                                        int S, int K, int N, int E, void* stream);
int tessera_gfx950_grouped_gemm_f16_f32_dev(const void* x, const void* w, const int32_t* offsets, void* y,
                                            int S, int K, int N, int E, void* stream);
/* The per-tensor scales of the reference's quantised grouped product
 * (python/tessera/compiler/grouped_layout.py:373-392: x quantised as one tensor, each expert's
 * weight on its own), applied after the product of the unscaled grid values:
 * out[r, :] = y[r, :] * scale[e] for offsets[e] <= r < offsets[e+1].  y f32 [S, N]; scale f32 [E]
 * (the activation's scale times expert e's); out f32, or bf16 when out_bf16 != 0 (may not alias y
 * then). */
int tessera_gfx950_scale_groups_f32(const float* y, const int32_t* offsets, const float* scale, void* out, int out_bf16,
                                    int S, int N, int E);
int tessera_gfx950_scale_groups_f32_dev(const float* y, const int32_t* offsets, const float* scale, void* out,
                                        int out_bf16, int S, int N, int E, void* stream);
/* ops.silu_mul (python/tessera/__init__.py:559-574): out = silu(a) * b elementwise, silu(a) =
 * a / (1 + exp(-a)); 16-bit storage in and out, f32 arithmetic, n elements.  The stand-alone
 * form of the step the fused block below applies in its epilogue (the reference's quantised
 * block composes grouped_gemm, silu_mul and grouped_gemm: python/tessera/__init__.py:610-616). */
int tessera_gfx950_silu_mul_bf16(const void* a, const void* b, void* out, int64_t n);
int tessera_gfx950_silu_mul_f16(const void* a, const void* b, void* out, int64_t n);
int tessera_gfx950_silu_mul_bf16_dev(const void* a, const void* b, void* out, int64_t n, void* stream);
int tessera_gfx950_silu_mul_f16_dev(const void* a, const void* b, void* out, int64_t n, void* stream);
/* tessera.grouped_swiglu / ops.moe_swiglu_block
 * (python/tessera/runtime.py:20353-20368; python/tessera/__init__.py:592-616):
 * y = gg(bf16(silu(bf16(gg(x,Wg))) * bf16(gg(x,Wu))), Wd), every intermediate
 * rounded to bf16 like the reference's storage rule.  x [S,K], wg/wu [E,K,F],
 * wd [E,F,N], y bf16 [S,N].  hidden (bf16 [S,F]) is workspace; NULL makes the
 * library allocate it (host-pointer form always allocates). */
int tessera_gfx950_moe_swiglu_block_bf16(const void* x, const void* wg, const void* wu, const void* wd,
                                         const int32_t* offsets, void* y, int S, int K, int F, int N, int E);
int tessera_gfx950_moe_swiglu_block_bf16_dev(const void* x, const void* wg, const void* wu, const void* wd,
                                             const int32_t* offsets, void* y, void* hidden,
                                             int S, int K, int F, int N, int E, void* stream);
/* The same block reading its input through the dispatch map: row m of the block's
 * input is x[token_of_slot[m]], x the unpermuted bf16 [T,K] activation, so
 * moe_dispatch (python/tessera/stdlib/moe.py:117-125) needs no pass and no x_perm
 * buffer of its own.  token_of_slot: device int32[S] with values in [0, T) (not read, and
 * may be NULL, when S == 0);
 * T * K * 2 must not exceed 2 GiB - 17 (the range of the buffer load that fetches a
 * token row: rows past it would read as zeros), else rc 1. */
int tessera_gfx950_moe_swiglu_block_gather_bf16_dev(const void* x, const int32_t* token_of_slot,
                                                    const void* wg, const void* wu, const void* wd,
                                                    const int32_t* offsets, void* y, void* hidden,
                                                    int T, int S, int K, int F, int N, int E, void* stream);
/* The whole local layer nn.functional.moe_layer
 * (python/tessera/nn/functional.py:403-490) with the router logits given:
 * route -> swiglu block (reading x through the dispatch map) -> combine.  out f32
 * [T,N].  The five metadata outputs may each be NULL. */
int tessera_gfx950_moe_layer_bf16(const void* x, const float* router_logits, const void* wg, const void* wu,
                                  const void* wd, float* out, int T, int H, int F, int N, int E, int k,
                                  int normalize, int capacity,
                                  int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                  int32_t* group_sizes, int32_t* group_offsets);
/* The same layer starting from the router weight: scores = ops.gemm(x, w_router) stored
 * in bf16 and read as f32 (nn/functional.py:453; w_router bf16 [H,E]), then as above,
 * without a host hop between the router product and the routing.  router_logits_out
 * (f32 [T,E], may be NULL) receives the logits the routing saw. */
int tessera_gfx950_moe_layer_router_bf16(const void* x, const void* w_router, const void* wg, const void* wu,
                                         const void* wd, float* out, int T, int H, int F, int N, int E, int k,
                                         int normalize, int capacity,
                                         int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                         int32_t* group_sizes, int32_t* group_offsets, float* router_logits_out);
/* Device-resident form of the layer: router GEMM (when w_router is not NULL; else
 * router_logits, f32 [T,E], is read) -> routing -> expert block -> combine, enqueued on
 * one stream with no host synchronisation in between — the chained, resident-operand
 * execution the device-operand lease of python/tessera/runtime.py:1549-1614 exists for.
 * All pointers are device memory.  workspace: at least
 * tessera_gfx950_moe_layer_workspace_bytes(...) bytes, 16-byte aligned (router scores and
 * logits, the hidden activation [T k, F], the expert output [T k, N] and each token's packed
 * slot positions [T k]).  The six
 * metadata outputs are required (later stages read them): token_of_slot /
 * expert_of_slot / combine_weights hold T*k entries of which the first *num_slots are
 * valid.  T * H * 2 must stay inside the 2 GiB buffer range (see the gather block above). */
int tessera_gfx950_moe_layer_workspace_bytes(int T, int H, int F, int N, int E, int k, size_t* bytes);
int tessera_gfx950_moe_layer_bf16_dev(const void* x, const void* w_router, const float* router_logits,
                                      const void* wg, const void* wu, const void* wd, float* out,
                                      void* workspace, size_t workspace_bytes,
                                      int T, int H, int F, int N, int E, int k, int normalize, int capacity,
                                      int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                      int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots,
                                      void* stream);

/* ---- C-level launch bridge --------------------------------------------------- */

/* A launcher for the reference's C runtime: a backend registers one function that maps a
 * kernel NAME on a target to a native launch over ordered host buffers and scalar dims
 * (tsrGpuLauncherFn / tsrRegisterGpuLauncher, src/runtime/include/tessera/
 * tessera_runtime.h:81-99; params = tsrGpuLaunchParams, tsr_types.h:83-89: the struct
 * below has the same layout, and the return values are the reference's TsrStatus codes,
 * tsr_status.h:7-14).  tessera_gfx950_gpu_launcher has exactly the tsrGpuLauncherFn
 * signature, so `tsrRegisterGpuLauncher(tessera_gfx950_gpu_launcher, NULL)` is the whole
 * registration.  Targets: "rocm_gfx950" or "rocm".  Kernel names are this library's
 * host-pointer entry points, each with its own buffer / dim order:
 *   tessera_gfx950_gemm_{f16,bf16}, tessera_gfx950_gemm_{f16_f16,bf16_bf16},
 *   tessera_gfx950_gemm_i8_i32                    buffers {A,B,D}      dims {M,N,K}
 *   tessera_gfx950_batched_gemm_{f16,bf16}        buffers {A,B,D}      dims {batch,M,N,K}
 *   tessera_gfx950_flash_attn_{f16,bf16}          buffers {Q,K,V,O}    dims {B,H,Sq,Sk,D,causal}
 *                                                 (scale = 1/sqrt(D), the reference's default)
 * Returns 0 success; 2 (not found) for another target or a name it does not handle, so
 * the runtime reports an unbridged kernel honestly; 1 (invalid argument) for a wrong
 * buffer / dim count, a NULL buffer or dims the entry point rejects; 7 (device error)
 * when no gfx950 device is usable or the launch failed. */
typedef struct {
  void** buffers;
  size_t num_buffers;
  const int64_t* dims;
  size_t num_dims;
} tessera_gfx950_launch_params;
int tessera_gfx950_gpu_launcher(const char* target, const char* kernel_name,
                                const tessera_gfx950_launch_params* params, void* user);

#ifdef __cplusplus
}
#endif
#endif /* TESSERA_GFX950_H */
