/*
 * Multithreaded CPU implementation of the FP8 quantized-matmul path.  TEST INFRASTRUCTURE ONLY:
 * it is the "CPU baseline" timed beside the GPU in the benchmark, and is itself checked against the
 * scalar oracle (llmq_oracle.c) in the CPU test-suite.  The shipped library never calls it.
 *
 * Same arithmetic as the scalar oracle (abs-max: src/kernels/quant.cu:11-28; quantize :73-93;
 * quantize+transpose :151-164; transpose src/kernels/transpose.cu:9-32; GEMM
 * src/kernels/matmul.cpp:47-153), restructured for OpenMP threads and SIMD:
 *   - abs-max / quantize are embarrassingly parallel over elements;
 *   - the GEMM decodes e4m3 through a 256-entry table into fp32 panels and accumulates in fp32
 *     with a register-blocked 4 x 64 micro-kernel (fp32 accumulation in a fixed order, so results
 *     are reproducible but differ from the exact sum by fp32 rounding, like any real backend).
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

uint8_t orc_e4m3_encode(float y);
float orc_e4m3_decode(uint8_t c);
float orc_e5m2_decode(uint8_t c);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);
void orc_quant_scale(float absmax, float* scale, float* dequant);

int mt_num_threads(void) { return omp_get_max_threads(); }
void mt_set_num_threads(int n) { if (n > 0) omp_set_num_threads(n); }

float mt_abs_max_bf16(const uint16_t* in, int64_t n) {
    uint32_t best = 0;
#pragma omp parallel for reduction(max : best) schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        uint32_t a = in[i] & 0x7FFFu;
        if (a <= 0x7F80u && a > best) best = a;
    }
    uint32_t u = best << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Branch-light e4m3 encode of s*x on the fp32 bit pattern; equals orc_e4m3_encode bit for bit
 * (checked exhaustively over all bf16 inputs in the tests). */
static inline uint8_t enc_fast(float y) {
    uint32_t u;
    memcpy(&u, &y, 4);
    uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x7F;
    if (a > 0x43E80000u) return (uint8_t)(sign | 0x7E);
    if (a >= 0x3C800000u) {
        /* round to 3 mantissa bits with the add-and-truncate trick */
        uint32_t r = a + 0x7FFFFu + ((a >> 20) & 1u);
        return (uint8_t)(sign | ((r >> 20) - (120u << 3)));
    }
    /* below 2^-6 (subnormal or zero in e4m3): rare for abs-max scaled data, take the scalar path */
    return orc_e4m3_encode(y);
}

void mt_quantize_e4m3_bf16(uint8_t* out, float* scale_out, const uint16_t* in, float absmax, int64_t n) {
    float s, d;
    orc_quant_scale(absmax, &s, &d);
    if (scale_out) *scale_out = d;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        uint32_t u = (uint32_t)in[i] << 16;
        float x;
        memcpy(&x, &u, 4);
        float y = s * x;
        out[i] = enc_fast(y);
    }
}

void mt_quantize_transpose_e4m3_bf16(uint8_t* out, float* scale_out, const uint16_t* in, float absmax,
                                     int rows, int cols) {
    float s, d;
    orc_quant_scale(absmax, &s, &d);
    if (scale_out) *scale_out = d;
    const int TB = 64;
#pragma omp parallel for collapse(2) schedule(static)
    for (int r0 = 0; r0 < rows; r0 += TB)
        for (int c0 = 0; c0 < cols; c0 += TB) {
            int r1 = r0 + TB < rows ? r0 + TB : rows;
            int c1 = c0 + TB < cols ? c0 + TB : cols;
            for (int c = c0; c < c1; ++c)
                for (int r = r0; r < r1; ++r) {
                    uint32_t u = (uint32_t)in[(int64_t)r * cols + c] << 16;
                    float x;
                    memcpy(&x, &u, 4);
                    float y = s * x;
                    out[(int64_t)c * rows + r] = enc_fast(y);
                }
        }
}

void mt_transpose_u8(uint8_t* dst, const uint8_t* src, int rows, int cols) {
    const int TB = 64;
#pragma omp parallel for collapse(2) schedule(static)
    for (int r0 = 0; r0 < rows; r0 += TB)
        for (int c0 = 0; c0 < cols; c0 += TB) {
            int r1 = r0 + TB < rows ? r0 + TB : rows;
            int c1 = c0 + TB < cols ? c0 + TB : cols;
            for (int c = c0; c < c1; ++c)
                for (int r = r0; r < r1; ++r)
                    dst[(int64_t)c * rows + r] = src[(int64_t)r * cols + c];
        }
}

#define MB 64   /* columns of c (rows of a) per panel */
#define NB 4    /* rows of c (rows of b) per micro-kernel call */

__attribute__((target_clones("avx512f", "avx2,fma", "default")))
static void micro_4x64(float* restrict acc, const float* restrict at, const float* restrict bq, int K) {
    /* acc[4][64] += sum_k bq[j][k] * at[k][0..63] */
    float c0[MB], c1[MB], c2[MB], c3[MB];
    for (int m = 0; m < MB; ++m) { c0[m] = 0.f; c1[m] = 0.f; c2[m] = 0.f; c3[m] = 0.f; }
    for (int k = 0; k < K; ++k) {
        const float* a = at + (size_t)k * MB;
        float b0 = bq[k], b1 = bq[K + k], b2 = bq[2 * K + k], b3 = bq[3 * K + k];
        for (int m = 0; m < MB; ++m) {
            c0[m] += b0 * a[m];
            c1[m] += b1 * a[m];
            c2[m] += b2 * a[m];
            c3[m] += b3 * a[m];
        }
    }
    for (int m = 0; m < MB; ++m) {
        acc[m] = c0[m]; acc[MB + m] = c1[m]; acc[2 * MB + m] = c2[m]; acc[3 * MB + m] = c3[m];
    }
}

/*
 * c[N,M] (row-major) = (b[N,K] . a[M,K]^T) * (sa*sb) (+ bias[m]) (+ c if accumulate).
 * Restricted to c rows n in [n0,n1) so the benchmark can time a bounded slice of a large shape.
 * Requires M % 64 == 0 and (n1-n0) % 4 == 0.  Returns 0, or -1 on unsupported shape.
 */
int mt_gemm_tn_fp8(void* c, int c_is_f32, const uint8_t* a, const uint8_t* b, int b_is_e5m2,
                   const uint16_t* bias_bf16, const float* sa, const float* sb,
                   int M, int N, int K, int accumulate, int n0, int n1) {
    (void)N;
    if (M % MB != 0 || (n1 - n0) % NB != 0) return -1;
    float lut[256], lut_b[256];
    for (int i = 0; i < 256; ++i) {
        lut[i] = orc_e4m3_decode((uint8_t)i);
        lut_b[i] = b_is_e5m2 ? orc_e5m2_decode((uint8_t)i) : lut[i];
    }
    float scale = sa ? *sa : 1.f;
    if (sb) scale = scale * *sb;
#pragma omp parallel
    {
        float* at = (float*)aligned_alloc(64, sizeof(float) * (size_t)K * MB);
        float* bq = (float*)aligned_alloc(64, sizeof(float) * (size_t)K * NB);
        float acc[NB * MB];
#pragma omp for schedule(dynamic, 1)
        for (int m0 = 0; m0 < M; m0 += MB) {
            for (int m = 0; m < MB; ++m) {
                const uint8_t* am = a + (size_t)(m0 + m) * K;
                for (int k = 0; k < K; ++k) at[(size_t)k * MB + m] = lut[am[k]];
            }
            for (int n = n0; n < n1; n += NB) {
                for (int j = 0; j < NB; ++j) {
                    const uint8_t* bn = b + (size_t)(n + j) * K;
                    for (int k = 0; k < K; ++k) bq[(size_t)j * K + k] = lut_b[bn[k]];
                }
                micro_4x64(acc, at, bq, K);
                for (int j = 0; j < NB; ++j)
                    for (int m = 0; m < MB; ++m) {
                        size_t o = (size_t)(n + j) * M + m0 + m;
                        volatile float t = acc[j * MB + m] * scale;
                        if (bias_bf16) t = t + orc_bf16_to_f32(bias_bf16[m0 + m]);
                        if (accumulate)
                            t = t + (c_is_f32 ? ((float*)c)[o] : orc_bf16_to_f32(((uint16_t*)c)[o]));
                        if (c_is_f32) ((float*)c)[o] = t;
                        else ((uint16_t*)c)[o] = orc_f32_to_bf16(t);
                    }
            }
        }
        free(at);
        free(bq);
    }
    return 0;
}

int mt_gemm_tn_e4m3(void* c, int c_is_f32, const uint8_t* a, const uint8_t* b,
                    const uint16_t* bias_bf16, const float* sa, const float* sb,
                    int M, int N, int K, int accumulate, int n0, int n1) {
    return mt_gemm_tn_fp8(c, c_is_f32, a, b, 0, bias_bf16, sa, sb, M, N, K, accumulate, n0, n1);
}
