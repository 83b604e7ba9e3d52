/*
 * llmq_fp8.h -- C ABI of the MI355X (gfx950) FP8 quantized-matmul path.
 *
 * One entry point per kernel entry point of the reference's src/kernels/kernels.h that lies on the
 * path  abs-max -> scaled bf16->e4m3 quantize (plain / fused transpose) -> e4m3 x e4m3 TN GEMM.
 * Plain pointers and sizes only; bf16 travels as uint16_t bit patterns, e4m3 as uint8_t codes.
 *
 * Conventions shared by every function:
 *   - every pointer is a DEVICE pointer owned by the caller (abs-max / scale slots included);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is enqueued
 *     asynchronously on it, no host synchronisation, no allocation, legal under stream capture;
 *   - the return value is LLMQ_OK or an error code; llmq_last_error() gives the message of the
 *     last failure on the calling thread (the C++ shim turns codes into the reference's exception
 *     types: std::invalid_argument / std::runtime_error);
 *   - tensor base pointers must be 16-byte aligned (src/kernels/matmul.cpp:55-57 has the same rule).
 */
#ifndef LLMQ_FP8_H
#define LLMQ_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* The library is built with hidden visibility: the functions declared here are its whole exported surface. */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

#define LLMQ_OK 0
#define LLMQ_ERR_INVALID_ARGUMENT 1 /* shape / alignment / null-pointer precondition violated */
#define LLMQ_ERR_RUNTIME 2          /* a HIP runtime call failed (message carries hipGetErrorString) */

/* Message of the last error returned on this thread ("" if none). Never NULL. */
const char* llmq_last_error(void);

/* Library version string, and the gfx target the device code was compiled for ("gfx950"). */
const char* llmq_version(void);
const char* llmq_target_arch(void);

/*
 * *out = max_i |in[i]| as fp32 (NaNs ignored, |+-Inf| wins, result >= +0; 0 for n == 0).
 * One kernel launch on `stream`: whatever the slot held before is overwritten (no clearing needed, none done).
 * The workgroups meet in one of LLMQ_ABS_MAX_ARRIVAL_AREAS arrival areas built into the device code, selected by
 * ((uintptr_t)out / 4) % LLMQ_ABS_MAX_ARRIVAL_AREAS.  Calls on one stream, or ordered by events, may share an area.
 * Calls that can run at the same time on one GPU (different streams, nothing ordering them) must use result slots
 * that map to different areas -- any two slots less than 256 bytes apart do -- or they race on the arrival counter
 * (the reference's memset + atomic-max form has no such limit; its abs-max calls all sit on the one compute stream).
 * Replaces: abs_max(float*, const nv_bfloat16*, long, const cudaDeviceProp&, cudaStream_t)
 *           src/kernels/kernels.h:247, src/kernels/quant.cu:107-109 (kernel :11-28).
 * n may be any non-negative count (the reference requires n % 8 == 0).
 */
#define LLMQ_ABS_MAX_ARRIVAL_AREAS 64
int llmq_abs_max_bf16(float* out, const uint16_t* in, int64_t n, void* stream);

/* fp32 input variant.  Replaces abs_max(float*, const float*, long, ...) src/kernels/kernels.h:246,
 * src/kernels/quant.cu:103-105. */
int llmq_abs_max_f32(float* out, const float* in, int64_t n, void* stream);

/*
 * scale = 448.f / fmaxf(*absmax, 1e-10f); out[i] = e4m3_rn_satfinite(scale * (float)in[i]);
 * if scale_or_null: *scale_or_null = 1.f / scale.
 * Replaces: quantize_with_abs_max(__nv_fp8_e4m3*, float*, const nv_bfloat16*, const float*, long,
 *           const cudaDeviceProp&, cudaStream_t)  src/kernels/kernels.h:255, src/kernels/quant.cu:127-129
 *           (kernel :73-93).
 */
int llmq_quantize_e4m3_bf16(uint8_t* out, float* scale_or_null, const uint16_t* in, const float* absmax,
                            int64_t n, void* stream);

/* Same with e5m2 output codes (the gradient dtype option).  Replaces quantize_with_abs_max(
 * __nv_fp8_e5m2*, ...) src/kernels/kernels.h:256, src/kernels/quant.cu:130-132. */
int llmq_quantize_e5m2_bf16(uint8_t* out, float* scale_or_null, const uint16_t* in, const float* absmax,
                            int64_t n, void* stream);

/*
 * fp32-input variants (fp32 master weights / fp32 model dtype); same arithmetic, any n >= 0.
 * Replaces: quantize_with_abs_max(__nv_fp8_e4m3* out, float* scale_ptr, const float* in, ...) src/kernels/kernels.h:251
 *           and the __nv_fp8_e5m2 overload :252, src/kernels/quant.cu:121-126.
 */
int llmq_quantize_e4m3_f32(uint8_t* out, float* scale_or_null, const float* in, const float* absmax, int64_t n,
                           void* stream);
int llmq_quantize_e5m2_f32(uint8_t* out, float* scale_or_null, const float* in, const float* absmax, int64_t n,
                           void* stream);

/*
 * As llmq_quantize_e4m3_bf16 on a row-major [rows, cols] input, written transposed:
 * out[c*rows + r] = q(in[r*cols + c]).  rows % 8 == 0 and cols % 8 == 0 required.
 * Replaces: quantize_and_transpose_with_abs_max(__nv_fp8_e4m3*, float*, const nv_bfloat16*,
 *           const float*, int rows, int cols, const cudaDeviceProp&, cudaStream_t)
 *           src/kernels/kernels.h:263, src/kernels/quant.cu:191-193 (kernel :151-164).
 */
int llmq_quantize_transpose_e4m3_bf16(uint8_t* out, float* scale_or_null, const uint16_t* in,
                                      const float* absmax, int rows, int cols, void* stream);

/* fp32-input variant of the above (fp32 master weights / fp32 model dtype); same arithmetic.
 * Replaces: quantize_and_transpose_with_abs_max(__nv_fp8_e4m3* out, float* scale_ptr, const float* in,
 *           const float* abs_max, int rows, int cols, ...)  src/kernels/kernels.h:261, src/kernels/quant.cu:135-149,175-189. */
int llmq_quantize_transpose_e4m3_f32(uint8_t* out, float* scale_or_null, const float* in, const float* absmax, int rows,
                                     int cols, void* stream);

/*
 * Extension with no counterpart in the reference (it reads the tensor twice instead: quantize_with_abs_max
 * followed by transpose of the codes, src/models/llama_model.cpp:310-331): one read of in[rows, cols] produces
 * both out[r*cols + c] and out_transposed[c*rows + r], the same bytes the two reference calls give.
 * format: 0 = e4m3, 1 = e5m2 (448-based scale for both, as src/kernels/quant.cu:79).  rows, cols multiples of 8.
 */
int llmq_quantize_both_bf16(uint8_t* out, uint8_t* out_transposed, float* scale_or_null, const uint16_t* in,
                            const float* absmax, int rows, int cols, int format, void* stream);

/*
 * Byte transpose: dst[c*rows + r] = src[r*cols + c]  (e4m3 / e5m2 codes).  Any rows, cols >= 0.
 * Replaces: transpose(__nv_fp8_e4m3*, const __nv_fp8_e4m3*, int rows, int cols, cudaStream_t)
 *           src/kernels/kernels.h:267 (and the e5m2 overload :268), src/kernels/transpose.cu:38-43.
 */
int llmq_transpose_u8(uint8_t* dst, const uint8_t* src, int rows, int cols, void* stream);

/*
 * TN GEMM in the reference's matmul convention (column-major cuBLAS view): with ROW-MAJOR
 * a[M,K] and b[N,K] (both e4m3, K contiguous) it writes ROW-MAJOR c[N,M]:
 *     c[n,m] = round( (sum_k b[n,k]*a[m,k]) * (sa*sb) + bias[m] + (accumulate ? c[n,m] : 0) )
 * fp32 accumulation, fp32 epilogue, one rounding to the output type.  sa / sb are device fp32
 * scalars or NULL (= 1).  bias is bf16[M] or NULL.  Any M, N >= 1; K must be a multiple of 16 (16-byte aligned
 * operand rows, the rule of the reference's default backend, src/kernels/matmul.cpp:55-57).  The fast kernels take
 * K % 128 == 0 with M % 128 == 0 (bf16 output without accumulation: also M % 224 == 0 or M % 192 == 0) and all but
 * the last N % 128 rows of c.  Other shapes with M % 8 == 0 run on ragged instances of the same kernels (256 x 256
 * tiles with moved-back edge tiles for large outputs with K >= 384, at about three quarters of the lattice rate;
 * 128 x 128 tiles with clamped rows otherwise); a slow general-shape kernel serves the N % 128 remainder rows of a
 * regular M, K, shapes with M % 8 != 0 and outputs smaller than one 128 x 128 tile.
 * Replaces: matmul(nv_bfloat16* c, const __nv_fp8_e4m3* a, const __nv_fp8_e4m3* b,
 *           const nv_bfloat16* bias, const float* scale_a, const float* scale_b, cublasLtHandle_t,
 *           std::byte* ws, size_t ws_size, int M, int N, int K, EMMTranspose::TN, bool accumulate,
 *           cudaStream_t, EMatmulBackend)  src/kernels/kernels.h:88-90, src/kernels/matmul.cpp:216-220,
 *           and gemm_mma_tn(...) src/kernels/gemm_mma.cu:279-284.
 * workspace: device scratch like the reference's matmul workspace (32 MiB in src/training/model.cpp:69),
 * or NULL with size 0.  It is used in two cases, both deterministic (fp32 partial results go to the workspace and are
 * added in a fixed order by a second kernel): an output with too few tiles to fill the chip has K split over more
 * workgroups (N*M*4 bytes per split), and a large output whose last round of 256 x 256 tiles would leave most of the
 * chip idle has the tiles of that round cut into K segments (256 KiB per segment).  What does not fit the workspace is
 * not split.  Calls that share a workspace must be stream ordered.
 */
int llmq_gemm_tn_e4m3_bf16(uint16_t* c, const uint8_t* a, const uint8_t* b, const uint16_t* bias_or_null,
                           const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                           size_t workspace_bytes, int M, int N, int K, int accumulate, void* stream);

/*
 * The same matmul with the operand layout selected by the reference's EMMTranspose mode (src/kernels/kernels.h:22:
 * TT = 0, TN = 1, NT = 2, NN = 3; in its column-major reading, src/kernels/matmul.cpp:66-67).  With row-major storage:
 *   TN  a[M, K], b[N, K]            (both K contiguous: llmq_gemm_tn_e4m3_bf16 / llmq_gemm_tn_e4m3_e5m2_bf16)
 *   TT  a[M, K], b[K, N]            (b K-major: the output gradient dY[BT, OC] in its stored layout as the second
 *                                    operand of the weight gradient)
 *   NN  a[K, M], b[N, K]            (a K-major: the weight W[OC, C] in its stored layout as the first operand of the dgrad)
 *   NT  a[K, M], b[K, N]            (both K-major: activation X[BT, C] and gradient dY[BT, OC] of the weight gradient)
 * so that the transposed copies the reference's FP8 path materialises (src/models/llama_model.cpp:309-339; its own
 * kernels take TN only) are not needed.  The K-major modes serve M, N and K multiples of 256 (with bf16 output and
 * without accumulation also M a multiple of 224 in modes TT and NN, of 192 in mode NN) and K-major operands below
 * 2 GiB, with bias and accumulation in every mode (llmq_gemm_e4m3_f32_mode: the same with fp32 output,
 * src/kernels/kernels.h:72-78).  Other
 * shapes return LLMQ_ERR_INVALID_ARGUMENT before anything is launched and the caller takes the transposing route.
 * b_format: 0 = e4m3, 1 = e5m2.  The workspace serves the cut of the last round of tiles as in mode TN (the K-major
 * modes have no split-K for few-tile outputs).  Results are bit-identical to mode TN on the transposed copies whenever
 * both run the same plan (256 x 256 tiles of the same kernel family, the same cut).
 */
#define LLMQ_MODE_TT 0
#define LLMQ_MODE_TN 1
#define LLMQ_MODE_NT 2
#define LLMQ_MODE_NN 3
int llmq_gemm_e4m3_bf16_mode(uint16_t* c, const uint8_t* a, const uint8_t* b, const uint16_t* bias_or_null,
                             const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                             size_t workspace_bytes, int M, int N, int K, int mode, int b_format, int accumulate,
                             void* stream);
int llmq_gemm_e4m3_f32_mode(float* c, const uint8_t* a, const uint8_t* b, const void* bias_or_null, int bias_is_bf16,
                            const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                            size_t workspace_bytes, int M, int N, int K, int mode, int b_format, int accumulate,
                            void* stream);

/*
 * fp32-output variant (wgrad into fp32 gradients).  bias may be fp32[M] (bias_is_bf16 == 0) or
 * bf16[M] (bias_is_bf16 != 0) or NULL.
 * Replaces: matmul(float* c, const __nv_fp8_e4m3*, const __nv_fp8_e4m3*, const float* bias, ...)
 *           src/kernels/kernels.h:72-74 and (..., const nv_bfloat16* bias, ...) :76-78,
 *           src/kernels/matmul.cpp:198-208.
 */
int llmq_gemm_tn_e4m3_f32(float* c, const uint8_t* a, const uint8_t* b, const void* bias_or_null,
                          int bias_is_bf16, const float* sa_or_null, const float* sb_or_null,
                          void* workspace_or_null, size_t workspace_bytes, int M, int N, int K, int accumulate,
                          void* stream);

/*
 * Mixed-format variants for the e5m2 gradient dtype: a is e4m3 (weights / activations), b is e5m2 (the
 * quantized output gradient); everything else as above.
 * Replaces: matmul(nv_bfloat16* c, const __nv_fp8_e4m3* a, const __nv_fp8_e5m2* b, const nv_bfloat16* bias, ...)
 *           src/kernels/kernels.h:92-94, src/kernels/matmul.cpp:222-226, and the fp32-output declaration
 *           src/kernels/kernels.h:80-82.
 */
int llmq_gemm_tn_e4m3_e5m2_bf16(uint16_t* c, const uint8_t* a, const uint8_t* b_e5m2, const uint16_t* bias_or_null,
                                const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                                size_t workspace_bytes, int M, int N, int K, int accumulate, void* stream);
int llmq_gemm_tn_e4m3_e5m2_f32(float* c, const uint8_t* a, const uint8_t* b_e5m2, const void* bias_or_null,
                               int bias_is_bf16, const float* sa_or_null, const float* sb_or_null,
                               void* workspace_or_null, size_t workspace_bytes, int M, int N, int K, int accumulate,
                               void* stream);

/*
 * Bias gradient from the (quantized) output gradient: with row-major dout[BT, OC],
 *     dbias[oc] = round_bf16( (float)dbias[oc] + (sa*sb) * sum_bt value(dout[bt, oc]) )
 * i.e. the result is ADDED to dbias.  dout_format: 0 = e4m3, 1 = e5m2, 2 = bf16.  sa / sb: device fp32
 * scalars, both NULL (factor 1) or both non-NULL.  OC must be a multiple of 16 (fp8) or 8 (bf16).
 * scratch: device buffer of at least llmq_backward_bias_scratch_bytes(BT, OC, dout_format) bytes,
 * overwritten by every call (no need to clear it); fp32 sums in a fixed order -> deterministic.
 * Replaces: backward_bias(nv_bfloat16* dbias, const __nv_fp8_e4m3* dout, const float* scale_a,
 *           const float* scale_b, float* dbias_buffer, int B, int T, int OC, const cudaDeviceProp&, cudaStream_t)
 *           src/kernels/kernels.h:104-106, src/kernels/bias.cu:151-195, and
 *           get_bias_backward_scratch_size(ETensorDType, int OC, const cudaDeviceProp&) kernels.h:102, bias.cu:142-148.
 */
int64_t llmq_backward_bias_scratch_bytes(int BT, int OC, int dout_format);
int llmq_backward_bias_bf16(uint16_t* dbias, const void* dout, int dout_format, const float* sa_or_null,
                            const float* sb_or_null, float* scratch, size_t scratch_bytes, int BT, int OC, void* stream);

/*
 * llmq_backward_bias_bf16 for callers that cannot allocate or carry a scratch buffer (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * callers take the scratch from their bump allocator.  Same arguments minus the scratch, same result bit for bit:
 * the band sums go to an array built into the library's device code (LLMQ_BACKWARD_BIAS_STATIC_SCRATCH_BYTES per
 * GPU, held until the process ends); the call allocates and frees nothing.  A shape whose band sums
 * (llmq_backward_bias_scratch_bytes) exceed that size is refused with LLMQ_ERR_INVALID_ARGUMENT.  All calls on one
 * GPU share the array: calls that overlap there (different streams, no ordering between them) race; the array
 * needs no clearing between calls (every call overwrites what it reads).  The first call on a device looks up the
 * array's device address (a host-side query under a mutex, not a stream operation): make one ordinary call per device
 * before capturing this entry point into a HIP graph; every later call enqueues its two kernels and nothing else.
 */
#define LLMQ_BACKWARD_BIAS_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
int llmq_backward_bias_bf16_static_scratch(uint16_t* dbias, const void* dout, int dout_format, const float* sa_or_null,
                                           const float* sb_or_null, int BT, int OC, void* stream);

/*
 * SwiGLU producers adjacent to the quantized matmuls.  inp: row-major [B*T, 2*C] bf16, each row [up(C) | gate(C)].
 *     s = 1 / (1 + exp(-gate));   out[bt, c] = bf16((up * gate) * s)
 * abs_max_or_null: if non-NULL, reset and then set to max |out| over the rounded bf16 outputs (NaNs ignored),
 * bit-identical to llmq_abs_max_bf16(out).  C must be a multiple of 8 and 2*B*T*C < 2^31 (as in the reference;
 * B*T*C need not be a multiple of the launch's block share).  exp and the reciprocal are the hardware's
 * (about 1 ulp each): results lie within one bf16 ulp of the correctly rounded value; the reference's own are
 * not bit-specified either (CUDA expf + approximate reciprocal).
 * Replaces: swiglu_forward(nv_bfloat16* out, const nv_bfloat16* inp, float* abs_max_ptr, int B, int T, int C,
 *           cudaStream_t)  src/kernels/kernels.h:156, src/kernels/swiglu.cu:25-65,104-179,304-346.
 */
int llmq_swiglu_forward_bf16(uint16_t* out, const uint16_t* inp, float* abs_max_or_null, int B, int T, int C,
                             void* stream);

/*
 * SwiGLU written directly as e4m3 codes with a known abs-max: byte-identical to llmq_swiglu_forward_bf16
 * followed by llmq_quantize_e4m3_bf16 with the same abs_max (the invariant the reference tests,
 * src/testing/test-swiglu.cu:243-315), without the bf16 tensor ever reaching memory.
 * scale = 448 / max(*abs_max, 1e-10); *scale_or_null = 1 / scale.
 * Replaces: swiglu_forward_quant(__nv_fp8_e4m3* out, float* scale_ptr, const nv_bfloat16* inp,
 *           const float* abs_max_ptr, int B, int T, int C, cudaStream_t)
 *           src/kernels/kernels.h:160, src/kernels/swiglu.cu:67-98,181-242,348-372.
 */
int llmq_swiglu_forward_quant_bf16(uint8_t* out, float* scale_or_null, const uint16_t* inp, const float* abs_max,
                                   int B, int T, int C, void* stream);

/*
 * SwiGLU backward: dinp [B*T, 2*C] = [dup | dgate] from dout [B*T, C] and the forward input,
 *     dup = bf16(dout * gate * s),   dgate = bf16(dout * up * s * (1 + gate * (1 - s)))
 * (products left to right in fp32).  abs_max_or_null as above, over both halves of dinp.
 * Replaces: swiglu_backward(nv_bfloat16* dinp, const nv_bfloat16* dout, const nv_bfloat16* inp, float* abs_max,
 *           int B, int T, int C, cudaStream_t)  src/kernels/kernels.h:163, src/kernels/swiglu.cu:244-300,374-401.
 */
int llmq_swiglu_backward_bf16(uint16_t* dinp, const uint16_t* dout, const uint16_t* inp, float* abs_max_or_null,
                              int B, int T, int C, void* stream);

/*
 * RMSNorm forward, the producer of the projections' bf16 input.  Per row of C elements of inp [B*T, C]:
 *     s = 1 / sqrt(mean(x^2) + epsilon);  out = bf16((float)bf16(s * x) * (float)weight[c]);  rms[row] = s
 * (the normalised value is rounded to bf16 before the scale, as in the reference).  abs_max_or_null: reset, then
 * max |out| over the rounded outputs, bit-identical to llmq_abs_max_bf16(out).  rms_or_null may be NULL.
 * C must be a multiple of 8 and at most 16384.  The squares are summed in fp32 in a fixed order (deterministic);
 * s is within a few fp32 ulp of the exact value, the reference's own s (approximate rsqrt, launch-dependent
 * summation order) is not bit-specified.
 * Replaces: rmsnorm_forward(nv_bfloat16* out, float* rms, const nv_bfloat16* inp, const nv_bfloat16* weight,
 *           float* abs_max_ptr, float epsilon, int B, int T, int C, cudaStream_t)
 *           src/kernels/kernels.h:46, src/kernels/rmsnorm.cu:17-86,168-178,183-217.
 */
int llmq_rmsnorm_forward_bf16(uint16_t* out, float* rms_or_null, const uint16_t* inp, const uint16_t* weight,
                              float* abs_max_or_null, float epsilon, int B, int T, int C, void* stream);

/*
 * The same with the residual add in front: residual[row] = bf16((float)inp1 + (float)inp2) is stored and normalised;
 * N rows.  residual may be the same buffer as inp1 or inp2.
 * Replaces: fused_residual_rmsnorm_forward(nv_bfloat16* residual, nv_bfloat16* normed, float* rrms,
 *           const nv_bfloat16* inp1, const nv_bfloat16* inp2, const nv_bfloat16* weight, float* abs_max_ptr,
 *           float epsilon, int N, int C, cudaStream_t)  src/kernels/kernels.h:59-60, src/kernels/rmsnorm.cu:88-164,224-227.
 */
int llmq_fused_residual_rmsnorm_forward_bf16(uint16_t* residual, uint16_t* normed, float* rrms, const uint16_t* inp1,
                                             const uint16_t* inp2, const uint16_t* weight, float* abs_max_or_null,
                                             float epsilon, int N, int C, void* stream);

/*
 * RMSNorm backward.  Per row bt of dout / inp [B*T, C], with r = rstd[bt] (the 1/rms the forward stored):
 *     g_c = (float)weight[c] * (float)dout[bt, c];      k = (sum_c g_c * inp[bt, c]) / C * r
 *     dinp[bt, c] = bf16( (float)dresidual[bt, c] + (g_c - inp[bt, c] * r * k) * r )
 *     dweight[c]  = bf16( (float)dweight[c] + sum_bt inp[bt, c] * r * dout[bt, c] )          (ADDED to dweight)
 * dresidual may be the same buffer as dinp (the reference copies it into dinp first when it is not).
 * abs_max_or_null: reset, then max |dinp| over the rounded outputs, bit-identical to llmq_abs_max_bf16(dinp).
 * scratch: device buffer of at least llmq_rmsnorm_backward_scratch_bytes(C) bytes, overwritten by every call (no
 * need to clear it); all sums are fp32 in a fixed order -> deterministic.  C: multiple of 8, at most 8192.
 * Replaces: rmsnorm_backward(nv_bfloat16* dinp, nv_bfloat16* dweight, std::byte* scratch, const nv_bfloat16* dresidual,
 *           const nv_bfloat16* dout, const nv_bfloat16* inp, const nv_bfloat16* weight, const float* rstd,
 *           float* abs_max_ptr, int B, int T, int C, const cudaDeviceProp&, cudaStream_t)
 *           src/kernels/kernels.h:52-53, src/kernels/rmsnorm.cu:229-440,447-470, and
 *           get_rmsnorm_backward_scratch_size(int C, const cudaDeviceProp&) kernels.h:49, rmsnorm.cu:442-445.
 */
int64_t llmq_rmsnorm_backward_scratch_bytes(int C);
int llmq_rmsnorm_backward_bf16(uint16_t* dinp, uint16_t* dweight, void* scratch, size_t scratch_bytes,
                               const uint16_t* dresidual, const uint16_t* dout, const uint16_t* inp,
                               const uint16_t* weight, const float* rstd, float* abs_max_or_null, int B, int T, int C,
                               void* stream);

/*
 * Rotary position embedding on the fused QKV tensor [B, T, Nq + 2*Nkv, head_dim] (bf16); freqs_cis_f16 is [T, head_dim]
 * fp16 with (cos, sin) pairs for d = 0 .. head_dim/2 - 1.  Query and key heads, with real = x[d], imag = x[d + head_dim/2]:
 *     out[d] = bf16(real*cos - imag*sin),  out[d + head_dim/2] = bf16(real*sin + imag*cos)      (backward: sin -> -sin)
 * in fp32; value heads are copied (left alone when out == inp).  abs_max_or_null: reset, then max |out| over all heads
 * including the value heads, bit-identical to llmq_abs_max_bf16(out).  head_dim must be a multiple of 8.
 * Replaces: rope_forward / rope_backward(nv_bfloat16* out, const nv_bfloat16* in, const half* freqs_cis, float* abs_max_ptr,
 *           int B, int T, int Nq, int Nkv, int head_dim, cudaStream_t)  src/kernels/kernels.h:113,116,
 *           src/kernels/rope.cu:42-163.
 */
int llmq_rope_forward_bf16(uint16_t* out, const uint16_t* inp, const uint16_t* freqs_cis_f16, float* abs_max_or_null, int B,
                           int T, int Nq, int Nkv, int head_dim, void* stream);
int llmq_rope_backward_bf16(uint16_t* dinp, const uint16_t* dout, const uint16_t* freqs_cis_f16, float* abs_max_or_null,
                            int B, int T, int Nq, int Nkv, int head_dim, void* stream);
/*
 * Host-side table for the two above: freqs_cis_host[t*dim + 2i] = fp16(cos(t / theta^(2i/dim))), [.. + 2i + 1] = fp16(sin(..)),
 * t < end, i < dim/2, evaluated in fp32 with the C library as the reference does.
 * Replaces: precompute_freqs_cis(half* freqs_cis, int dim, int end, float theta)  src/kernels/kernels.h:111, rope.cu:15-40.
 */
int llmq_precompute_freqs_cis_f16(uint16_t* freqs_cis_host, int dim, int end, float theta);

/*
 * fp32 overloads of the producers above (a model kept in fp32 whose matmuls run in FP8): the same formulas without the
 * roundings to bf16, fp32 tensors throughout; abs_max_or_null as above, bit-identical to llmq_abs_max_f32 of the tensor
 * written.  The fp32 outputs agree with the reference's to a few fp32 ulp, not bit for bit: its float instantiations are
 * compiled with multiply-add contraction and use an exponential and a reciprocal that are not specified to the bit,
 * while these kernels evaluate every product and sum as written (no contraction).  C must be a multiple of 4 (RMSNorm: at most 8192), head_dim a multiple of 8; the rope table is fp32
 * [T, head_dim] of (cos, sin) pairs.  In fp32 RMSNorm the normalised value s * x is the fp32 product itself.
 * Replace the float overloads: swiglu_forward / swiglu_backward  src/kernels/kernels.h:157,164 (src/kernels/swiglu.cu:
 *           304-346,374-401; tested by src/testing/test-swiglu.cu:83-156), rope_forward / rope_backward and
 *           precompute_freqs_cis  kernels.h:110,112,115 (src/kernels/rope.cu:15-40,129-163; src/testing/test-rope.cu:88-183,
 *           303-345), rmsnorm_forward  kernels.h:45, rmsnorm_backward  kernels.h:50-51, fused_residual_rmsnorm_forward
 *           kernels.h:57-58 (src/kernels/rmsnorm.cu:183-227,447-470).
 */
int llmq_swiglu_forward_f32(float* out, const float* inp, float* abs_max_or_null, int B, int T, int C, void* stream);
int llmq_swiglu_backward_f32(float* dinp, const float* dout, const float* inp, float* abs_max_or_null, int B, int T, int C,
                             void* stream);
int llmq_rope_forward_f32(float* out, const float* inp, const float* freqs_cis_f32, float* abs_max_or_null, int B, int T,
                          int Nq, int Nkv, int head_dim, void* stream);
int llmq_rope_backward_f32(float* dinp, const float* dout, const float* freqs_cis_f32, float* abs_max_or_null, int B, int T,
                           int Nq, int Nkv, int head_dim, void* stream);
int llmq_precompute_freqs_cis_f32(float* freqs_cis_host, int dim, int end, float theta);
int llmq_rmsnorm_forward_f32(float* out, float* rms_or_null, const float* inp, const float* weight, float* abs_max_or_null,
                             float epsilon, int B, int T, int C, void* stream);
int llmq_fused_residual_rmsnorm_forward_f32(float* residual, float* normed, float* rrms, const float* inp1, const float* inp2,
                                            const float* weight, float* abs_max_or_null, float epsilon, int N, int C,
                                            void* stream);
int llmq_rmsnorm_backward_f32(float* dinp, float* dweight, void* scratch, size_t scratch_bytes, const float* dresidual,
                              const float* dout, const float* inp, const float* weight, const float* rstd,
                              float* abs_max_or_null, int B, int T, int C, void* stream);

/*
 * AdamW update of bf16 parameters from bf16 gradients, moments in fp32 or bf16 (m_dtype / v_dtype: 0 = fp32, 1 = bf16;
 * supported pairs (m, v): (0, 0), (1, 0), (1, 1)), per element:
 *     grad = *grad_scale * g;  m = fma(beta1, m, fma(-beta1, grad, grad));  v = fma(beta2, v, fma(-beta2, grad^2, grad^2))
 *     p = fma(-lr, fma(wd, p, (m*c1) / (sqrt(v*c2) + eps)), p),   c1 = 1/(1 - beta1^t), c2 = 1/(1 - beta2^t)
 * Values narrower than fp32 are written with the reference's stochastic rounding (SquirrelNoise5 hash of the element
 * index and `seed`; see llmq_amd/csrc/adamw.hip for the threshold of each tensor): reproducible bit for bit.
 * abs_max_or_null: max |new p| is merged into the slot with an atomic max; the slot is NOT reset by this call
 * (as in the reference: the caller clears it, one slot may cover several calls).  num_parameters % 8 == 0.
 * Replaces: adamw_update(nv_bfloat16* params, const nv_bfloat16* grads, {float|nv_bfloat16}* m, {float|nv_bfloat16}* v,
 *           size_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps, float weight_decay,
 *           const float* grad_scale, float* abs_max, unsigned int seed, cudaStream_t)
 *           src/kernels/kernels.h:225-235, src/kernels/adamw.cu:18-195.  The e4m3 first moment is
 *           llmq_adamw_update_bf16_fp8m and fp32 parameters (kernels.h:221) are llmq_adamw_update_f32, both below.
 */
int llmq_adamw_update_bf16(uint16_t* params, const uint16_t* grads, void* m, int m_dtype, void* v, int v_dtype,
                           int64_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps,
                           float weight_decay, const float* grad_scale, float* abs_max_or_null, unsigned int seed,
                           void* stream);

/*
 * The same update with the first moment kept as e4m3 codes and one fp32 scale per 128 consecutive elements
 * (m_scales: ceil(num_parameters / 128) floats), second moment bf16.  m is read as (float)code * m_scales[i / 128];
 * every block of 128 new values gets the scale absmax / 448 (1 when its absmax is not above 1e-10) and is written
 * with the reference's stochastic rounding to e4m3 (values outside [2^-6, 448] in magnitude: round to nearest).
 * Replaces: adamw_update(nv_bfloat16* params, const nv_bfloat16* grads, __nv_fp8_e4m3* m, nv_bfloat16* v,
 *           size_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps, float weight_decay,
 *           const float* grad_scale, float* m_scales, float* abs_max, unsigned int seed, cudaStream_t)
 *           src/kernels/kernels.h:237-239, src/kernels/adamw.cu:22-66,191-195.
 */
int llmq_adamw_update_bf16_fp8m(uint16_t* params, const uint16_t* grads, uint8_t* m_e4m3, float* m_scales, uint16_t* v_bf16,
                                int64_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps,
                                float weight_decay, const float* grad_scale, float* abs_max_or_null, unsigned int seed,
                                void* stream);

/*
 * The same update on fp32 parameters, gradients and moments: nothing is narrower than fp32, so there is no stochastic
 * rounding (seed is accepted for the reference's signature and unused); num_parameters must be a multiple of 4.
 * abs_max_or_null as above (merged, not reset).  Bit exact against the formulas above evaluated operation by operation.
 * Replaces: adamw_update(float* params, const float* grads, float* m, float* v, size_t num_parameters, float learning_rate,
 *           float beta1, float beta2, int t, float eps, float weight_decay, const float* grad_scale, float* abs_max,
 *           unsigned int seed, cudaStream_t)  src/kernels/kernels.h:221-223, src/kernels/adamw.cu:159-163.
 */
int llmq_adamw_update_f32(float* params, const float* grads, float* m, float* v, int64_t num_parameters, float learning_rate,
                          float beta1, float beta2, int t, float eps, float weight_decay, const float* grad_scale,
                          float* abs_max_or_null, unsigned int seed, void* stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* LLMQ_FP8_H */
