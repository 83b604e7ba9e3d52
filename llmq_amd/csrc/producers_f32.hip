// fp32 overloads of the producers around the FP8 matmul path for gfx950 (a model kept in fp32 whose matmuls run
// in FP8): SwiGLU forward / backward, rotary embedding forward / backward, RMSNorm forward (plain and with the
// residual add) and backward, each with the abs-max of its own output computed on the way.  The bf16 kernels
// (swiglu.hip, rope.hip, rmsnorm.hip) work on packed bf16 bit patterns; these are their fp32 counterparts with the
// same structure: one trip per lane with independent 16-byte accesses in flight, every wave instruction covering
// 1 KiB contiguous, abs-max folded on bit patterns and finished by block_min_to_atomic_max.
//
// Semantics follow the reference's templates instantiated for float (src/kernels/swiglu.cu:20-65, 244-300;
// src/kernels/rope.cu:42-127; src/kernels/rmsnorm.cu:17-164, 229-440): the arithmetic is the bf16 kernels'
// without the roundings to bf16.  exp is the hardware exp2 (with the argument's rounding error corrected, see
// sigmoid_f32) and the reciprocal the hardware one (about 1 ulp each; the reference's expf / approximate reciprocal are
// not bit-specified either), sums of squares and dot products are fp32 in a fixed order, 1 / sqrt uses the correctly
// rounded square root and division.
#include <cmath>

#include "common.hpp"
#include "absmax_reduce.hpp"

namespace llmq {

typedef float v4f_p __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4f_p ld4(const v4f_p* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st4(v4f_p* p, const v4f_p& v) { __builtin_nontemporal_store(v, p); }

// abs-max fold on fp32 bit patterns: y = +Inf pattern - |x| pattern wraps to a huge value for NaN, so the minimum
// over y ignores NaNs and finds the largest |x|; the start value encodes 0
constexpr uint32_t kFoldStart32 = 0x7F800000u;
__device__ __forceinline__ uint32_t fold32(uint32_t acc, float x) {
    const uint32_t y = kFoldStart32 - (__float_as_uint(x) & 0x7FFFFFFFu);
    return y < acc ? y : acc;
}
__device__ __forceinline__ uint32_t fold32(uint32_t acc, const v4f_p& v) {
    return fold32(fold32(fold32(fold32(acc, v[0]), v[1]), v[2]), v[3]);
}

// 1 / (1 + exp(-gate)).  exp(-gate) = exp2(t * log2(e)) with t = -gate: the product is taken in two pieces (log2(e) =
// hi + lo, the rounding error of t * hi recovered with an fma) and the low piece applied as a first-order correction,
// so that the error of exp stays near one ulp for every gate (rounding t * log2(e) to fp32 alone costs |t| * 0.7 ulp,
// which an fp32 output would show for |gate| of 5 and more).
__device__ __forceinline__ float sigmoid_f32(float gate) {
    const float t = -gate;
    const float hi = t * 1.44269502f;                                                  // 0x3FB8AA3B
    const float lo = __builtin_fmaf(t, 1.44269502f, -hi) + t * 1.92596299e-8f;          // log2(e) - 0x3FB8AA3B
    float e = __builtin_amdgcn_exp2f(hi);
    if (e < __builtin_huge_valf()) e = __builtin_fmaf(e, lo * 0.693147181f, e);       // exp2(hi + lo) ~ exp2(hi) (1 + lo ln 2)
    return __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- SwiGLU ----------------------------------------------------------------------------------------
// chunk number (16 bytes = 4 values of the [rows][C] output) -> offset of its up part in the [rows][2C] input
__device__ __forceinline__ uint32_t input_chunk32(uint32_t idx, uint32_t chunks_per_row) {
    return idx + (idx / chunks_per_row) * chunks_per_row;
}

template <bool ABSMAX, int UNROLL, int THREADS>
__global__ __launch_bounds__(THREADS) void swiglu_forward_f32_kernel(v4f_p* __restrict__ out, const v4f_p* __restrict__ inp,
                                                                 unsigned* __restrict__ absmax_out, uint32_t nchunks,
                                                                 uint32_t chunks_per_row) {
    const uint32_t base = blockIdx.x * ((uint32_t)THREADS * UNROLL) + threadIdx.x;
    v4f_p up[UNROLL], gate[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        up[u] = gate[u] = v4f_p{0.f, 0.f, 0.f, 0.f};
        if (idx < nchunks) {
            const uint32_t src = input_chunk32(idx, chunks_per_row);
            up[u] = ld4(&inp[src]);
            gate[u] = ld4(&inp[src + chunks_per_row]);
        }
    }
    uint32_t acc = kFoldStart32;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        v4f_p r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = (up[u][e] * gate[u][e]) * sigmoid_f32(gate[u][e]);  // zeros when predicated off
        if constexpr (ABSMAX) acc = fold32(acc, r);
        if (idx < nchunks) st4(&out[idx], r);
    }
    if constexpr (ABSMAX) block_min_to_atomic_max(absmax_out, acc, kFoldStart32, 0);
}

template <bool ABSMAX, int UNROLL, int THREADS>
__global__ __launch_bounds__(THREADS) void swiglu_backward_f32_kernel(v4f_p* __restrict__ dinp, const v4f_p* __restrict__ dout,
                                                                  const v4f_p* __restrict__ inp,
                                                                  unsigned* __restrict__ absmax_out, uint32_t nchunks,
                                                                  uint32_t chunks_per_row) {
    const uint32_t base = blockIdx.x * ((uint32_t)THREADS * UNROLL) + threadIdx.x;
    v4f_p d[UNROLL], up[UNROLL], gate[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        d[u] = up[u] = gate[u] = v4f_p{0.f, 0.f, 0.f, 0.f};
        if (idx < nchunks) {
            const uint32_t src = input_chunk32(idx, chunks_per_row);
            d[u] = ld4(&dout[idx]);
            up[u] = ld4(&inp[src]);
            gate[u] = ld4(&inp[src + chunks_per_row]);
        }
    }
    uint32_t acc = kFoldStart32;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        v4f_p g1, g2;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float sg = sigmoid_f32(gate[u][e]);
            g1[e] = d[u][e] * gate[u][e] * sg;
            g2[e] = d[u][e] * up[u][e] * sg * (1.0f + gate[u][e] * (1.0f - sg));
        }
        if constexpr (ABSMAX) acc = fold32(fold32(acc, g1), g2);
        if (idx < nchunks) {
            const uint32_t dst = input_chunk32(idx, chunks_per_row);
            st4(&dinp[dst], g1);
            st4(&dinp[dst + chunks_per_row], g2);
        }
    }
    if constexpr (ABSMAX) block_min_to_atomic_max(absmax_out, acc, kFoldStart32, 0);
}

// C a multiple of 4 (the reference's rule for its fp32 kernels, src/testing/test-swiglu.cu:89-90) and
// 2 * B * T * C below 2^31; B * T * C need not be a multiple of a workgroup's share.
static int check_swiglu_f32(const char* what, int B, int T, int C, int64_t& nchunks) {
    LLMQ_REQUIRE(B >= 0 && T >= 0 && C >= 0, "%s: negative dimension (%d, %d, %d)", what, B, T, C);
    LLMQ_REQUIRE(C % 4 == 0, "%s: C must be divisible by 4 for fp32 tensors (got %d)", what, C);
    const int64_t nelem = (int64_t)B * T * C;
    LLMQ_REQUIRE(2 * nelem < 0x7FFFFFFFLL, "%s: input too large (%lld elements)", what, (long long)(2 * nelem));
    nchunks = nelem / 4;
    return LLMQ_OK;
}

static unsigned blocks_of(int64_t n, int threads, int unroll) {
    return (unsigned)((n + (int64_t)threads * unroll - 1) / ((int64_t)threads * unroll));
}

static int reset_slot(float* abs_max, hipStream_t stream) {
    if (abs_max) {
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(abs_max));
        LLMQ_HIP_TRY(hipGetLastError());
    }
    return LLMQ_OK;
}

// ---- rotary embedding --------------------------------------------------------------------------------
// Lane -> (token bt, head h, group of 4 consecutive d): 16 bytes of the real half, 16 of the imaginary half and the
// 8 table entries (cos, sin) x 4.
template <bool BACKWARD, bool ABSMAX, int THREADS>
__global__ __launch_bounds__(THREADS) void rope_f32_kernel(float* out, const float* inp, const float* __restrict__ freqs,
                                                       unsigned* __restrict__ absmax_out, int64_t total, int T, int Nq,
                                                       int Nkv, int head_dim) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t fold = kFoldStart32;
    if (idx < total) {
        const int groups = head_dim / 8;
        const int N = Nq + 2 * Nkv;
        const int grp = (int)(idx % groups);
        const int h = (int)((idx / groups) % N);
        const int64_t bt = idx / ((int64_t)groups * N);
        const int t = (int)(bt % T);
        const int64_t base = (bt * N + h) * head_dim + (int64_t)grp * 4;
        const bool in_place = out == inp;
        const bool rotated = h < Nq + Nkv;
        if (rotated || ABSMAX || !in_place) {
            v4f_p re = ld4(reinterpret_cast<const v4f_p*>(inp + base));
            v4f_p im = ld4(reinterpret_cast<const v4f_p*>(inp + base + head_dim / 2));
            if (rotated) {
                const float* f = freqs + (int64_t)t * head_dim + 8 * grp;
                const v4f_p cs0 = *reinterpret_cast<const v4f_p*>(f), cs1 = *reinterpret_cast<const v4f_p*>(f + 4);
                const float c[4] = {cs0[0], cs0[2], cs1[0], cs1[2]};
                const float s[4] = {cs0[1], cs0[3], cs1[1], cs1[3]};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float sn = BACKWARD ? -s[e] : s[e];
                    const float r = re[e], i = im[e];
                    re[e] = r * c[e] - i * sn;
                    im[e] = r * sn + i * c[e];
                }
            }
            if (rotated || !in_place) {
                st4(reinterpret_cast<v4f_p*>(out + base), re);
                st4(reinterpret_cast<v4f_p*>(out + base + head_dim / 2), im);
            }
            if constexpr (ABSMAX) fold = fold32(fold32(fold, re), im);
        }
    }
    if constexpr (ABSMAX) block_min_to_atomic_max(absmax_out, fold, kFoldStart32, 0);
}

template <bool BACKWARD>
static int rope_f32_any(const char* what, float* out, const float* inp, const float* freqs, float* abs_max, int B, int T,
                        int Nq, int Nkv, int head_dim, hipStream_t stream) {
    LLMQ_REQUIRE(B >= 0 && T >= 0 && Nq >= 0 && Nkv >= 0 && head_dim >= 0, "%s: negative dimension", what);
    LLMQ_REQUIRE(head_dim % 8 == 0, "%s: head_dim must be divisible by 8 (got %d)", what, head_dim);
    if (int rc = reset_slot(abs_max, stream)) return rc;
    const int64_t heads = (int64_t)B * T * (Nq + 2 * Nkv);
    if (heads == 0 || head_dim == 0) return LLMQ_OK;
    LLMQ_REQUIRE(out && inp && freqs, "%s: null tensor pointer", what);
    LLMQ_REQUIRE(aligned16(out) && aligned16(inp) && aligned16(freqs), "%s: pointers must be 16-byte aligned", what);
    const int64_t total = heads * (head_dim / 8);
    LLMQ_REQUIRE((total + 255) / 256 <= 0x7FFFFFFF, "%s: tensor too large", what);
    if (abs_max)
        hipLaunchKernelGGL((rope_f32_kernel<BACKWARD, true, 1024>), dim3((unsigned)((total + 1023) / 1024)), dim3(1024), 0,
                           stream, out, inp, freqs, reinterpret_cast<unsigned*>(abs_max), total, T, Nq, Nkv, head_dim);
    else
        hipLaunchKernelGGL((rope_f32_kernel<BACKWARD, false, 256>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                           stream, out, inp, freqs, nullptr, total, T, Nq, Nkv, head_dim);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// ---- RMSNorm forward ---------------------------------------------------------------------------------
// One wave per row, the whole row in registers (NCH 16-byte chunks of 4 values per lane), WAVES rows per workgroup.
template <int NCH, bool RESIDUAL, bool ABSMAX, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void rmsnorm_forward_f32_kernel(v4f_p* residual, v4f_p* __restrict__ normed,
                                                                  float* __restrict__ rrms, const v4f_p* __restrict__ inp1,
                                                                  const v4f_p* __restrict__ inp2,
                                                                  const v4f_p* __restrict__ weight,
                                                                  unsigned* __restrict__ absmax_out, float epsilon, int N,
                                                                  int chunks, float c_float) {
    const int lane = threadIdx.x % kWave;
    const int row = blockIdx.x * WAVES + threadIdx.x / kWave;
    const bool valid = row < N;  // no early exit: the abs-max reduction below synchronises the workgroup
    const int64_t base = (int64_t)row * chunks;
    const v4f_p zero = {0.f, 0.f, 0.f, 0.f};

    v4f_p x[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = lane + kWave * k;
        x[k] = (valid && c < chunks) ? ld4(&inp1[base + c]) : zero;
    }
    if constexpr (RESIDUAL) {
        v4f_p y[NCH];
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = lane + kWave * k;
            y[k] = (valid && c < chunks) ? ld4(&inp2[base + c]) : zero;
        }
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = lane + kWave * k;
            x[k] = x[k] + y[k];
            if (valid && c < chunks) st4(&residual[base + c], x[k]);
        }
    }
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = acc + x[k][e] * x[k][e];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc = acc + __shfl_xor(acc, off, kWave);
    const float s = __fdiv_rn(1.0f, sqrt_rn(__fdiv_rn(acc, c_float) + epsilon));

    uint32_t fold = kFoldStart32;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = lane + kWave * k;
        if (c < chunks) {
            const v4f_p w = weight[c];
            v4f_p o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (s * x[k][e]) * w[e];
            if (valid) {
                st4(&normed[base + c], o);
                if constexpr (ABSMAX) fold = fold32(fold, o);
            }
        }
    }
    if (valid && lane == 0 && rrms) rrms[row] = s;
    if constexpr (ABSMAX) block_min_to_atomic_max(absmax_out, fold, kFoldStart32, 0);
}

template <int NCH, bool RESIDUAL>
static void launch_rows_f32(float* residual, float* normed, float* rrms, const float* inp1, const float* inp2,
                            const float* weight, float* abs_max, float epsilon, int N, int C, hipStream_t stream) {
    // rows per workgroup with the abs-max: what 512 registers per SIMD allow for this row width
    constexpr int AM_WAVES = NCH <= 8 ? 16 : NCH == 16 ? 8 : 4;
    auto launch = [&](auto kernel, int waves) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)((N + waves - 1) / waves)), dim3(waves * 64), 0, stream,
                           reinterpret_cast<v4f_p*>(residual), reinterpret_cast<v4f_p*>(normed), rrms,
                           reinterpret_cast<const v4f_p*>(inp1), reinterpret_cast<const v4f_p*>(inp2),
                           reinterpret_cast<const v4f_p*>(weight), reinterpret_cast<unsigned*>(abs_max), epsilon, N, C / 4,
                           (float)C);
    };
    if (abs_max) launch(rmsnorm_forward_f32_kernel<NCH, RESIDUAL, true, AM_WAVES>, AM_WAVES);
    else launch(rmsnorm_forward_f32_kernel<NCH, RESIDUAL, false, 4>, 4);
}

static int rmsnorm_forward_f32_any(const char* what, bool fused, float* residual, float* normed, float* rrms, const float* inp1,
                                   const float* inp2, const float* weight, float* abs_max, float epsilon, int64_t N64, int C,
                                   hipStream_t stream) {
    LLMQ_REQUIRE(N64 >= 0 && C >= 0, "%s: negative dimension (%lld rows, C = %d)", what, (long long)N64, C);
    LLMQ_REQUIRE(N64 <= 0x7FFFFFFF, "%s: too many rows (%lld)", what, (long long)N64);
    LLMQ_REQUIRE(C % 4 == 0, "%s: C must be divisible by 4 for fp32 tensors (got %d)", what, C);
    LLMQ_REQUIRE(C <= 8192, "%s: C up to 8192 is supported for fp32 tensors (got %d)", what, C);
    const int N = (int)N64;
    if (int rc = reset_slot(abs_max, stream)) return rc;
    if (N == 0 || C == 0) return LLMQ_OK;
    LLMQ_REQUIRE(normed && inp1 && weight && (!fused || (residual && inp2)), "%s: null tensor pointer", what);
    LLMQ_REQUIRE(aligned16(residual) && aligned16(normed) && aligned16(inp1) && aligned16(inp2) && aligned16(weight),
                 "%s: tensor pointers must be 16-byte aligned", what);
    const int per_lane = (C / 4 + kWave - 1) / kWave;
#define LLMQ_ROWS32(NCH)                                                                                                  \
    do {                                                                                                                  \
        if (fused) launch_rows_f32<NCH, true>(residual, normed, rrms, inp1, inp2, weight, abs_max, epsilon, N, C, stream); \
        else launch_rows_f32<NCH, false>(nullptr, normed, rrms, inp1, nullptr, weight, abs_max, epsilon, N, C, stream);    \
    } while (0)
    if (per_lane <= 2) LLMQ_ROWS32(2);
    else if (per_lane <= 4) LLMQ_ROWS32(4);
    else if (per_lane <= 8) LLMQ_ROWS32(8);
    else if (per_lane <= 16) LLMQ_ROWS32(16);
    else LLMQ_ROWS32(32);
#undef LLMQ_ROWS32
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// ---- RMSNorm backward --------------------------------------------------------------------------------
// Per row bt with r = rstd[bt]:  g_c = weight[c] * dout[bt, c];  k = (sum_c g_c * inp[bt, c]) / C * r;
//   dinp[bt, c] = dresidual[bt, c] + (g_c - inp[bt, c] * r * k) * r;   dweight[c] += sum_bt inp[bt, c] * r * dout[bt, c].
// Structure of the bf16 kernel: WPR waves share a row (wave `sub` takes the chunks sub * 64 + lane + 64 * WPR * k), a
// lane owns the same columns of every row it sees and keeps their dweight sums in registers; the waves of a workgroup
// add theirs through LDS in a fixed order, workgroup sums go to the caller's scratch [workgroups][C] and a second
// kernel adds them with a fixed tree.  The 4 / WPR rows a workgroup works on at a time advance in lockstep.
template <int NCH, int WPR, bool ABSMAX>
__global__ __launch_bounds__(256) void rmsnorm_backward_f32_kernel(v4f_p* dinp, float* __restrict__ partial, const v4f_p* dresidual,
                                                                   const v4f_p* __restrict__ dout, const v4f_p* __restrict__ inp,
                                                                   const v4f_p* __restrict__ weight,
                                                                   const float* __restrict__ rstd,
                                                                   unsigned* __restrict__ absmax_out, int N, int chunks,
                                                                   float c_float) {
    extern __shared__ float block_dw32[];  // [4 * chunks]
    __shared__ float dot_part[2][4];
    constexpr int ROWS = 4 / WPR;  // rows in flight per workgroup
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int sub = wave % WPR, rslot = wave / WPR;
    const int c_first = sub * kWave + lane;
    const v4f_p zero = {0.f, 0.f, 0.f, 0.f};

    v4f_p dw[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) dw[k] = zero;
    uint32_t fold = kFoldStart32;

    const int step = gridDim.x * ROWS;
    int parity = 0;
    for (int row0 = blockIdx.x * ROWS; row0 < N; row0 += step, parity ^= 1) {  // uniform trip count
        const int row = row0 + rslot;
        const bool valid = row < N;
        const int64_t base = (int64_t)row * chunks;
        const float r = valid ? rstd[row] : 0.f;
        v4f_p d[NCH], x[NCH], old[NCH], w[NCH];
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = c_first + kWave * WPR * k;
            d[k] = x[k] = old[k] = w[k] = zero;
            if (c < chunks) w[k] = weight[c];
            if (valid && c < chunks) {
                d[k] = ld4(&dout[base + c]);
                x[k] = ld4(&inp[base + c]);
                old[k] = ld4(&dresidual[base + c]);
            }
        }
        float dot = 0.f;
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
#pragma unroll
            for (int e = 0; e < 4; ++e) dot = dot + (w[k][e] * d[k][e]) * x[k][e];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) dot = dot + __shfl_xor(dot, off, kWave);
        if constexpr (WPR > 1) {
            // the parts of the waves sharing the row, added in wave order (double-buffered slots: the next row's
            // writes cannot overtake this row's reads)
            if (lane == 0) dot_part[parity][wave] = dot;
            __syncthreads();
            dot = dot_part[parity][rslot * WPR];
#pragma unroll
            for (int p = 1; p < WPR; ++p) dot = dot + dot_part[parity][rslot * WPR + p];
        }
        const float kk = __fdiv_rn(dot, c_float) * r;
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = c_first + kWave * WPR * k;
            if (valid && c < chunks) {
                v4f_p o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float n = x[k][e] * r;
                    dw[k][e] = dw[k][e] + n * d[k][e];
                    o[e] = old[k][e] + (w[k][e] * d[k][e] - n * kk) * r;
                }
                st4(&dinp[base + c], o);
                if constexpr (ABSMAX) fold = fold32(fold, o);
            }
        }
    }

    // workgroup sum of the dweight terms: the row slots add theirs in order (the waves of one slot own disjoint
    // columns, a lane the same columns in every slot), then the whole workgroup writes the row of partial sums
    for (int sl = 0; sl < ROWS; ++sl) {
        if (rslot == sl) {
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                const int c = c_first + kWave * WPR * k;
                if (c < chunks) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float* slot = &block_dw32[(size_t)e * chunks + c];  // [e][chunk]: consecutive lanes, consecutive banks
                        *slot = sl == 0 ? dw[k][e] : *slot + dw[k][e];
                    }
                }
            }
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < 4 * chunks; i += 256) {
        const int e = i / chunks, c = i % chunks;
        partial[(size_t)blockIdx.x * (4 * chunks) + (size_t)c * 4 + e] = block_dw32[i];
    }
    if constexpr (ABSMAX) block_min_to_atomic_max(absmax_out, fold, kFoldStart32, 0);
}

// dweight[c] += sum over workgroups of partial[g][c].  A workgroup takes 32 columns as 8 quads x 32 lanes: lane
// (quad, q) adds workgroups q, q + 32, ... in index order, the 32 lane sums are then added in lane order -- a fixed
// summation tree.
__global__ __launch_bounds__(256) void rmsnorm_dweight_finish_f32_kernel(float* __restrict__ dweight,
                                                                         const float* __restrict__ partial, int groups, int C) {
    __shared__ v4f_p red[32][8];
    const int quad = threadIdx.x % 8, q = threadIdx.x / 8;
    const int col = blockIdx.x * 32 + 4 * quad;  // C is a multiple of 4: a quad is inside or outside as a whole
    v4f_p s = {0.f, 0.f, 0.f, 0.f};
    if (col < C) {
        for (int g = q; g < groups; g += 32) s = s + *reinterpret_cast<const v4f_p*>(partial + (size_t)g * C + col);
    }
    red[q][quad] = s;
    __syncthreads();
    if (q == 0 && col < C) {
        v4f_p t = red[0][quad];
#pragma unroll
        for (int k = 1; k < 32; ++k) t = t + red[k][quad];
        v4f_p* dst = reinterpret_cast<v4f_p*>(dweight + col);
        *dst = *dst + t;
    }
}

static int backward_groups_f32() { return 2 * cu_count(); }

}  // namespace llmq

using namespace llmq;

extern "C" int llmq_swiglu_forward_f32(float* out, const float* inp, float* abs_max_or_null, int B, int T, int C, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int64_t nchunks;
    if (int rc = check_swiglu_f32("swiglu_forward", B, T, C, nchunks)) return rc;
    if (int rc = reset_slot(abs_max_or_null, stream)) return rc;
    if (nchunks == 0) return LLMQ_OK;
    LLMQ_REQUIRE(out && inp, "swiglu_forward: null tensor pointer");
    LLMQ_REQUIRE(aligned16(out) && aligned16(inp), "swiglu_forward: pointers must be 16-byte aligned");
    constexpr int U = 4;
    if (abs_max_or_null)
        hipLaunchKernelGGL((swiglu_forward_f32_kernel<true, U, 512>), dim3(blocks_of(nchunks, 512, U)), dim3(512), 0, stream,
                           reinterpret_cast<v4f_p*>(out), reinterpret_cast<const v4f_p*>(inp),
                           reinterpret_cast<unsigned*>(abs_max_or_null), (uint32_t)nchunks, (uint32_t)(C / 4));
    else
        hipLaunchKernelGGL((swiglu_forward_f32_kernel<false, U, 256>), dim3(blocks_of(nchunks, 256, U)), dim3(256), 0, stream,
                           reinterpret_cast<v4f_p*>(out), reinterpret_cast<const v4f_p*>(inp), nullptr, (uint32_t)nchunks,
                           (uint32_t)(C / 4));
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

extern "C" int llmq_swiglu_backward_f32(float* dinp, const float* dout, const float* inp, float* abs_max_or_null, int B, int T,
                                        int C, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int64_t nchunks;
    if (int rc = check_swiglu_f32("swiglu_backward", B, T, C, nchunks)) return rc;
    if (int rc = reset_slot(abs_max_or_null, stream)) return rc;
    if (nchunks == 0) return LLMQ_OK;
    LLMQ_REQUIRE(dinp && dout && inp, "swiglu_backward: null tensor pointer");
    LLMQ_REQUIRE(aligned16(dinp) && aligned16(dout) && aligned16(inp), "swiglu_backward: pointers must be 16-byte aligned");
    constexpr int U = 2;
    if (abs_max_or_null)
        hipLaunchKernelGGL((swiglu_backward_f32_kernel<true, U, 512>), dim3(blocks_of(nchunks, 512, U)), dim3(512), 0, stream,
                           reinterpret_cast<v4f_p*>(dinp), reinterpret_cast<const v4f_p*>(dout),
                           reinterpret_cast<const v4f_p*>(inp), reinterpret_cast<unsigned*>(abs_max_or_null),
                           (uint32_t)nchunks, (uint32_t)(C / 4));
    else
        hipLaunchKernelGGL((swiglu_backward_f32_kernel<false, U, 256>), dim3(blocks_of(nchunks, 256, U)), dim3(256), 0, stream,
                           reinterpret_cast<v4f_p*>(dinp), reinterpret_cast<const v4f_p*>(dout),
                           reinterpret_cast<const v4f_p*>(inp), nullptr, (uint32_t)nchunks, (uint32_t)(C / 4));
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

extern "C" int llmq_rope_forward_f32(float* out, const float* inp, const float* freqs_cis_f32, float* abs_max_or_null, int B,
                                     int T, int Nq, int Nkv, int head_dim, void* stream) {
    return rope_f32_any<false>("rope_forward", out, inp, freqs_cis_f32, abs_max_or_null, B, T, Nq, Nkv, head_dim,
                               static_cast<hipStream_t>(stream));
}

extern "C" int llmq_rope_backward_f32(float* dinp, const float* dout, const float* freqs_cis_f32, float* abs_max_or_null, int B,
                                      int T, int Nq, int Nkv, int head_dim, void* stream) {
    return rope_f32_any<true>("rope_backward", dinp, dout, freqs_cis_f32, abs_max_or_null, B, T, Nq, Nkv, head_dim,
                              static_cast<hipStream_t>(stream));
}

// Host-side table of (cos, sin) pairs in fp32, [end][dim] (src/kernels/rope.cu:15-31): angle = t / theta^(2i/dim) in
// fp32 with the C library's powf / cosf / sinf, as the reference computes it.
extern "C" int llmq_precompute_freqs_cis_f32(float* freqs_cis_host, int dim, int end, float theta) {
    LLMQ_REQUIRE(freqs_cis_host != nullptr || dim == 0 || end == 0, "precompute_freqs_cis: null output pointer");
    LLMQ_REQUIRE(dim >= 0 && end >= 0 && dim % 2 == 0, "precompute_freqs_cis: dim must be even and non-negative");
    for (int i = 0; i < dim / 2; ++i) {
        const float inv_freq = 1.0f / powf(theta, (float)(2 * i) / (float)dim);
        for (int t = 0; t < end; ++t) {
            const float angle = (float)t * inv_freq;
            freqs_cis_host[(size_t)t * dim + 2 * i] = cosf(angle);
            freqs_cis_host[(size_t)t * dim + 2 * i + 1] = sinf(angle);
        }
    }
    return LLMQ_OK;
}

extern "C" int llmq_rmsnorm_forward_f32(float* out, float* rms_or_null, const float* inp, const float* weight,
                                        float* abs_max_or_null, float epsilon, int B, int T, int C, void* stream) {
    return rmsnorm_forward_f32_any("rmsnorm_forward", false, nullptr, out, rms_or_null, inp, nullptr, weight, abs_max_or_null,
                                   epsilon, (int64_t)B * T, C, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_fused_residual_rmsnorm_forward_f32(float* residual, float* normed, float* rrms, const float* inp1,
                                                       const float* inp2, const float* weight, float* abs_max_or_null,
                                                       float epsilon, int N, int C, void* stream) {
    return rmsnorm_forward_f32_any("fused_residual_rmsnorm_forward", true, residual, normed, rrms, inp1, inp2, weight,
                                   abs_max_or_null, epsilon, N, C, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_rmsnorm_backward_f32(float* dinp, float* dweight, void* scratch, size_t scratch_bytes, const float* dresidual,
                                         const float* dout, const float* inp, const float* weight, const float* rstd,
                                         float* abs_max_or_null, int B, int T, int C, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t N64 = (int64_t)B * T;
    LLMQ_REQUIRE(B >= 0 && T >= 0 && C >= 0, "rmsnorm_backward: negative dimension (%d, %d, %d)", B, T, C);
    LLMQ_REQUIRE(N64 <= 0x7FFFFFFF, "rmsnorm_backward: too many rows (%lld)", (long long)N64);
    LLMQ_REQUIRE(C % 4 == 0, "rmsnorm_backward: C must be divisible by 4 for fp32 tensors (got %d)", C);
    LLMQ_REQUIRE(C <= 8192, "rmsnorm_backward: C up to 8192 is supported (got %d)", C);
    const int N = (int)N64;
    if (int rc = reset_slot(abs_max_or_null, stream)) return rc;
    if (N == 0 || C == 0) return LLMQ_OK;
    LLMQ_REQUIRE(dinp && dweight && dresidual && dout && inp && weight && rstd, "rmsnorm_backward: null tensor pointer");
    LLMQ_REQUIRE(aligned16(dinp) && aligned16(dweight) && aligned16(dresidual) && aligned16(dout) && aligned16(inp) &&
                     aligned16(weight) && aligned16(scratch),
                 "rmsnorm_backward: tensor and scratch pointers must be 16-byte aligned");
    const int chunks = C / 4;
    // waves per row so that a lane holds at most 8 chunks of each operand
    const int wpr = chunks <= 4 * kWave ? 1 : chunks <= 8 * kWave ? 2 : 4;
    const int rows_per_group = 4 / wpr;
    int groups = backward_groups_f32();
    if (groups > (N + rows_per_group - 1) / rows_per_group) groups = (N + rows_per_group - 1) / rows_per_group;
    LLMQ_REQUIRE(scratch != nullptr && scratch_bytes >= (size_t)groups * C * sizeof(float),
                 "rmsnorm_backward: scratch of %zu bytes is too small (need %zu, see llmq_rmsnorm_backward_scratch_bytes)",
                 scratch_bytes, (size_t)groups * C * sizeof(float));
    const int per_lane = (chunks + kWave * wpr - 1) / (kWave * wpr);
    const size_t lds = (size_t)C * sizeof(float);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)groups), dim3(256), lds, stream, reinterpret_cast<v4f_p*>(dinp),
                           reinterpret_cast<float*>(scratch), reinterpret_cast<const v4f_p*>(dresidual),
                           reinterpret_cast<const v4f_p*>(dout), reinterpret_cast<const v4f_p*>(inp),
                           reinterpret_cast<const v4f_p*>(weight), rstd, reinterpret_cast<unsigned*>(abs_max_or_null), N, chunks,
                           (float)C);
    };
#define LLMQ_BWD32(NCH, WPR)                                                      \
    do {                                                                          \
        if (abs_max_or_null) launch(rmsnorm_backward_f32_kernel<NCH, WPR, true>);  \
        else launch(rmsnorm_backward_f32_kernel<NCH, WPR, false>);                 \
    } while (0)
    if (wpr == 1) {
        if (per_lane <= 1) LLMQ_BWD32(1, 1);
        else if (per_lane <= 2) LLMQ_BWD32(2, 1);
        else LLMQ_BWD32(4, 1);
    } else if (wpr == 2) {
        LLMQ_BWD32(4, 2);
    } else if (per_lane <= 4) {
        LLMQ_BWD32(4, 4);
    } else {
        LLMQ_BWD32(8, 4);
    }
#undef LLMQ_BWD32
    LLMQ_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(rmsnorm_dweight_finish_f32_kernel, dim3((unsigned)((C + 31) / 32)), dim3(256), 0, stream, dweight,
                       reinterpret_cast<const float*>(scratch), groups, C);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}
