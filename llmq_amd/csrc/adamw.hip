// AdamW update of bf16 parameters for gfx950 with the abs-max of the updated parameters computed on the
// way: the producer of the weight tensors' abs-max, which the per-step weight quantization consumes (no
// separate pass over the weights).
//
// Semantics follow the reference (src/kernels/adamw.cu:18-170, src/kernels/squirrel_noise.cuh), per element i:
//     grad  = *grad_scale * (float)g[i]
//     m     = fma(beta1, m, fma(-beta1, grad, grad))                  (the reference's two-operation lerp)
//     v     = fma(beta2, v, fma(-beta2, grad*grad, grad*grad))
//     param = p - lr * ( (m * c1) / (sqrt(v * c2) + eps) + wd * p ),   c1 = 1/(1 - beta1^t), c2 = 1/(1 - beta2^t)
// with m, v kept in fp32 or bf16.  Everything narrower than fp32 is written with stochastic rounding: the low
// 16 bits of the fp32 value are compared with a 16-bit threshold from the SquirrelNoise5 hash; above it the
// value rounds away from zero, otherwise towards zero.  Thresholds: parameters hash(i, seed); v the same hash
// rotated left by 20; m hash(first index of i's vector, 51245) rotated left by 7 per position in the vector,
// where the reference's vector has 4 elements unless m and v are both bf16 (then 8).  The hash is integer
// arithmetic and every floating-point operation is correctly rounded, so results are reproducible bit for bit;
// the parameter line is evaluated as fma(-lr, fma(wd, p, quotient), p), the contraction the reference's
// compiler applies by default.  The abs-max slot is NOT reset here (the reference does not either: one slot
// may cover several calls; the caller clears it).
//
// HBM bound: 14 bytes per parameter with bf16 moments (read p, g, m, v; write p, m, v), 22 with fp32 moments.
// A lane takes 8 consecutive parameters: 16-byte accesses throughout.
#include <cmath>

#include "common.hpp"
#include "absmax_reduce.hpp"
#include "fp8_encode.hpp"

namespace llmq {

typedef float f32x2_aw __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_aw __attribute__((ext_vector_type(2)));

__host__ __device__ constexpr uint32_t squirrel_noise_5(uint32_t position, uint32_t seed) {
    uint32_t b = position;
    b *= 0xd2a80a3fu;
    b += seed;
    b ^= b >> 9;
    b += 0xa884f197u;
    b ^= b >> 11;
    b *= 0x6C736F4Bu;
    b ^= b >> 13;
    b += 0xB79F3ABBu;
    b ^= b >> 15;
    b *= 0x1b56c4f5u;
    b ^= b >> 17;
    return b;
}

__device__ __forceinline__ uint32_t rotl32(uint32_t x, int k) { return (x << k) | (x >> (32 - k)); }

// fp32 -> bf16 with the reference's stochastic rounding (squirrel_noise.cuh:47-56): returns the 16-bit pattern
__device__ __forceinline__ uint32_t sr_bf16(float x, uint32_t random) {
    uint32_t bits = __float_as_uint(x);
    bits = (bits & 0xFFFFu) > (random & 0xFFFFu) ? (bits | 0xFFFFu) : (bits & ~0xFFFFu);
    const f32x2_aw p = {__uint_as_float(bits), 0.f};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2_aw)) & 0xFFFFu;
}

// 8 consecutive fp32 values as two streaming 16-byte accesses
__device__ __forceinline__ void load_f32x8(float (&dst)[8], const uint4* p) {
    const uint4 lo = load_nt(p), hi = load_nt(p + 1);
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int k = 0; k < 8; ++k) dst[k] = __uint_as_float(w[k]);
}
__device__ __forceinline__ void store_f32x8(uint4* p, const float (&src)[8]) {
    store_nt(p, make_uint4(__float_as_uint(src[0]), __float_as_uint(src[1]), __float_as_uint(src[2]), __float_as_uint(src[3])));
    store_nt(p + 1, make_uint4(__float_as_uint(src[4]), __float_as_uint(src[5]), __float_as_uint(src[6]), __float_as_uint(src[7])));
}

struct AdamArgs {
    float lr, beta1, beta2, c1, c2, eps, wd;
    unsigned seed;
};

// M_BF16 / V_BF16: storage type of the moments.  THREADS: 1024 with the abs-max (fewer atomics on the slot).
template <bool M_BF16, bool V_BF16, bool ABSMAX, int THREADS>
__global__ __launch_bounds__(THREADS) void adamw_kernel(uint4* __restrict__ params, const uint4* __restrict__ grads,
                                                        void* __restrict__ m_mem, void* __restrict__ v_mem, int64_t nvec,
                                                        AdamArgs a, const float* __restrict__ grad_scale,
                                                        unsigned* __restrict__ absmax_out) {
    constexpr int REF_VEC = (M_BF16 && V_BF16) ? 8 : 4;  // elements per lane in the reference's launch
    const int64_t vec = (int64_t)blockIdx.x * THREADS + threadIdx.x;
    uint32_t fold = 0x7F807F80u;
    if (vec < nvec) {
        const float gs = *grad_scale;
        const uint4 pw = load_nt(&params[vec]), gw = load_nt(&grads[vec]);
        float m[8], v[8];
        if constexpr (M_BF16) {
            const uint4 w = load_nt(&reinterpret_cast<const uint4*>(m_mem)[vec]);
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) { m[2 * k] = bf16_lo(ww[k]); m[2 * k + 1] = bf16_hi(ww[k]); }
        } else {
            load_f32x8(m, reinterpret_cast<const uint4*>(m_mem) + 2 * vec);
        }
        if constexpr (V_BF16) {
            const uint4 w = load_nt(&reinterpret_cast<const uint4*>(v_mem)[vec]);
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) { v[2 * k] = bf16_lo(ww[k]); v[2 * k + 1] = bf16_hi(ww[k]); }
        } else {
            load_f32x8(v, reinterpret_cast<const uint4*>(v_mem) + 2 * vec);
        }
        const uint32_t pws[4] = {pw.x, pw.y, pw.z, pw.w}, gws[4] = {gw.x, gw.y, gw.z, gw.w};
        uint32_t p_out[8], m_out[8], v_out[8];
        const uint32_t first = (uint32_t)(vec * 8);  // the reference hashes the 32-bit truncation of the index
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t pword = pws[e / 2], gword = gws[e / 2];
            const float p_old = (e & 1) ? bf16_hi(pword) : bf16_lo(pword);
            const float grad = gs * ((e & 1) ? bf16_hi(gword) : bf16_lo(gword));
            const float m_new = __builtin_fmaf(a.beta1, m[e], __builtin_fmaf(-a.beta1, grad, grad));
            const float g2 = grad * grad;
            const float v_new = __builtin_fmaf(a.beta2, v[e], __builtin_fmaf(-a.beta2, g2, g2));
            const uint32_t random = squirrel_noise_5(first + e, a.seed);
            const float m_hat = m_new * a.c1, v_hat = v_new * a.c2;
            const float quot = __fdiv_rn(m_hat, sqrt_rn(v_hat) + a.eps);
            const float p_new = __builtin_fmaf(-a.lr, __builtin_fmaf(a.wd, p_old, quot), p_old);
            p_out[e] = sr_bf16(p_new, random);
            m[e] = m_new;
            v[e] = v_new;
            if constexpr (V_BF16) v_out[e] = sr_bf16(v_new, rotl32(random, 20));
            if constexpr (M_BF16) {
                const uint32_t base = squirrel_noise_5(first + (e / REF_VEC) * REF_VEC, 51245u);
                const int pos = e % REF_VEC;
                m_out[e] = sr_bf16(m_new, pos == 0 ? base : rotl32(base, (7 * pos) % 32));
            }
        }
        const uint4 pnew = make_uint4(p_out[0] | (p_out[1] << 16), p_out[2] | (p_out[3] << 16), p_out[4] | (p_out[5] << 16),
                                      p_out[6] | (p_out[7] << 16));
        store_nt(&params[vec], pnew);
        if constexpr (ABSMAX) fold = fold_vec(fold, pnew);
        if constexpr (M_BF16) {
            store_nt(&reinterpret_cast<uint4*>(m_mem)[vec], make_uint4(m_out[0] | (m_out[1] << 16), m_out[2] | (m_out[3] << 16),
                                                              m_out[4] | (m_out[5] << 16), m_out[6] | (m_out[7] << 16)));
        } else {
            store_f32x8(reinterpret_cast<uint4*>(m_mem) + 2 * vec, m);
        }
        if constexpr (V_BF16) {
            store_nt(&reinterpret_cast<uint4*>(v_mem)[vec], make_uint4(v_out[0] | (v_out[1] << 16), v_out[2] | (v_out[3] << 16),
                                                              v_out[4] | (v_out[5] << 16), v_out[6] | (v_out[7] << 16)));
        } else {
            store_f32x8(reinterpret_cast<uint4*>(v_mem) + 2 * vec, v);
        }
    }
    if constexpr (ABSMAX) {
        const uint32_t lo = fold & 0xFFFFu, hi = fold >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

// fp32 parameters, gradients and moments (the reference's all-float overload, src/kernels/adamw.cu:159-163): the same
// formulas; nothing is narrower than fp32, so nothing is stochastically rounded and the seed is unused.  A lane takes 4
// consecutive parameters (16-byte accesses); 28 bytes per parameter.
template <bool ABSMAX, int THREADS>
__global__ __launch_bounds__(THREADS) void adamw_f32_kernel(uint4* __restrict__ params, const uint4* __restrict__ grads,
                                                            uint4* __restrict__ m_mem, uint4* __restrict__ v_mem, int64_t nvec,
                                                            AdamArgs a, const float* __restrict__ grad_scale,
                                                            unsigned* __restrict__ absmax_out) {
    const int64_t vec = (int64_t)blockIdx.x * THREADS + threadIdx.x;
    uint32_t fold = 0x7F800000u;  // +Inf pattern - |x| pattern, minimised: NaNs wrap to huge values and are ignored
    if (vec < nvec) {
        const float gs = *grad_scale;
        const uint4 pw = load_nt(&params[vec]), gw = load_nt(&grads[vec]), mw = load_nt(&m_mem[vec]), vw = load_nt(&v_mem[vec]);
        const uint32_t pws[4] = {pw.x, pw.y, pw.z, pw.w}, gws[4] = {gw.x, gw.y, gw.z, gw.w}, mws[4] = {mw.x, mw.y, mw.z, mw.w},
                       vws[4] = {vw.x, vw.y, vw.z, vw.w};
        uint32_t p_out[4], m_out[4], v_out[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float p_old = __uint_as_float(pws[e]);
            const float grad = gs * __uint_as_float(gws[e]);
            const float m_new = __builtin_fmaf(a.beta1, __uint_as_float(mws[e]), __builtin_fmaf(-a.beta1, grad, grad));
            const float g2 = grad * grad;
            const float v_new = __builtin_fmaf(a.beta2, __uint_as_float(vws[e]), __builtin_fmaf(-a.beta2, g2, g2));
            const float m_hat = m_new * a.c1, v_hat = v_new * a.c2;
            const float quot = __fdiv_rn(m_hat, sqrt_rn(v_hat) + a.eps);
            const float p_new = __builtin_fmaf(-a.lr, __builtin_fmaf(a.wd, p_old, quot), p_old);
            p_out[e] = __float_as_uint(p_new);
            m_out[e] = __float_as_uint(m_new);
            v_out[e] = __float_as_uint(v_new);
            if constexpr (ABSMAX) {
                const uint32_t y = 0x7F800000u - (p_out[e] & 0x7FFFFFFFu);
                fold = y < fold ? y : fold;
            }
        }
        store_nt(&params[vec], make_uint4(p_out[0], p_out[1], p_out[2], p_out[3]));
        store_nt(&m_mem[vec], make_uint4(m_out[0], m_out[1], m_out[2], m_out[3]));
        store_nt(&v_mem[vec], make_uint4(v_out[0], v_out[1], v_out[2], v_out[3]));
    }
    if constexpr (ABSMAX) block_min_to_atomic_max(absmax_out, fold, 0x7F800000u, 0);
}

// fp32 -> e4m3 code with the reference's stochastic rounding (squirrel_noise.cuh:58-75): outside [2^-6, 448] in
// magnitude plain round-to-nearest; inside, the 20 bits below e4m3's three mantissa bits are filled with ones
// (the conversion then rounds away from zero) when they exceed the 20-bit threshold, else cleared.
__device__ __forceinline__ float sr_e4m3_prepare(float x, uint32_t random) {
    const float ax = __builtin_fabsf(x);
    if (ax > 448.f || ax < 0.015625f || x != x) return x;
    uint32_t bits = __float_as_uint(x);
    bits = (bits & 0xFFFFFu) > (random & 0xFFFFFu) ? (bits | 0xFFFFFu) : (bits & ~0xFFFFFu);
    return __uint_as_float(bits);
}

// First moment as e4m3 codes with one fp32 scale per 128 consecutive elements, second moment bf16
// (src/kernels/adamw.cu:22-66).  A lane takes 8 parameters, so 16 consecutive lanes share a block scale: the block's
// abs-max of the new first moment is combined with four xor-shuffles inside each group of 16 lanes.  Lanes beyond
// the tensor contribute 0 to it.
template <bool ABSMAX, int THREADS>
__global__ __launch_bounds__(THREADS) void adamw_fp8m_kernel(uint4* __restrict__ params, const uint4* __restrict__ grads,
                                                             uint2* __restrict__ m_codes, float* __restrict__ m_scales,
                                                             uint4* __restrict__ v_mem, int64_t nvec, AdamArgs a,
                                                             const float* __restrict__ grad_scale,
                                                             unsigned* __restrict__ absmax_out) {
    const int64_t vec = (int64_t)blockIdx.x * THREADS + threadIdx.x;
    const bool active = vec < nvec;
    uint32_t fold = 0x7F807F80u;
    float m[8];
    float blk_max = 0.f;
    uint32_t p_out[8], v_out[8];
    if (active) {
        const float gs = *grad_scale;
        const uint4 pw = load_nt(&params[vec]), gw = load_nt(&grads[vec]), vw = load_nt(&v_mem[vec]);
        const uint2 mw = m_codes[vec];
        const float old_scale = m_scales[vec / 16];
        const uint32_t pws[4] = {pw.x, pw.y, pw.z, pw.w}, gws[4] = {gw.x, gw.y, gw.z, gw.w}, vws[4] = {vw.x, vw.y, vw.z, vw.w};
        const uint32_t mws[2] = {mw.x, mw.y};
        const uint32_t first = (uint32_t)(vec * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const f32x2_aw pair = (e & 2) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)mws[e / 4], true)
                                          : __builtin_amdgcn_cvt_pk_f32_fp8((int)mws[e / 4], false);
            const float m_old = pair[e & 1] * old_scale;
            const float p_old = (e & 1) ? bf16_hi(pws[e / 2]) : bf16_lo(pws[e / 2]);
            const float v_old = (e & 1) ? bf16_hi(vws[e / 2]) : bf16_lo(vws[e / 2]);
            const float grad = gs * ((e & 1) ? bf16_hi(gws[e / 2]) : bf16_lo(gws[e / 2]));
            const float m_new = __builtin_fmaf(a.beta1, m_old, __builtin_fmaf(-a.beta1, grad, grad));
            const float g2 = grad * grad;
            const float v_new = __builtin_fmaf(a.beta2, v_old, __builtin_fmaf(-a.beta2, g2, g2));
            const uint32_t random = squirrel_noise_5(first + e, a.seed);
            const float m_hat = m_new * a.c1, v_hat = v_new * a.c2;
            const float quot = __fdiv_rn(m_hat, sqrt_rn(v_hat) + a.eps);
            const float p_new = __builtin_fmaf(-a.lr, __builtin_fmaf(a.wd, p_old, quot), p_old);
            p_out[e] = sr_bf16(p_new, random);
            v_out[e] = sr_bf16(v_new, rotl32(random, 20));
            m[e] = m_new;
            const float ma = __builtin_fabsf(m_new);
            blk_max = blk_max < ma ? ma : blk_max;  // a NaN never replaces the maximum
        }
    }
    // abs-max of the 128-element block: all lanes take part in the shuffles
#pragma unroll
    for (int d = 1; d < 16; d *= 2) {
        const float other = __shfl_xor(blk_max, d, 16);
        blk_max = blk_max < other ? other : blk_max;
    }
    if (active) {
        float factor = 1.f, scale = 1.f;
        if (blk_max > 1e-10f) {
            factor = __fdiv_rn(448.f, blk_max);
            scale = __fdiv_rn(1.f, factor);
        }
        if (vec % 16 == 0) m_scales[vec / 16] = scale;
        const uint32_t base = squirrel_noise_5((uint32_t)(vec * 8), 51245u);
        float y[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = sr_e4m3_prepare(m[e] * factor, e == 0 ? base : rotl32(base, (7 * e) % 32));
        uint2 codes;
        codes.x = encode4<kE4M3>(y[0], y[1], y[2], y[3]);
        codes.y = encode4<kE4M3>(y[4], y[5], y[6], y[7]);
        m_codes[vec] = codes;
        const uint4 pnew = make_uint4(p_out[0] | (p_out[1] << 16), p_out[2] | (p_out[3] << 16), p_out[4] | (p_out[5] << 16),
                                      p_out[6] | (p_out[7] << 16));
        store_nt(&params[vec], pnew);
        if constexpr (ABSMAX) fold = fold_vec(fold, pnew);
        store_nt(&v_mem[vec], make_uint4(v_out[0] | (v_out[1] << 16), v_out[2] | (v_out[3] << 16), v_out[4] | (v_out[5] << 16),
                                         v_out[6] | (v_out[7] << 16)));
    }
    if constexpr (ABSMAX) {
        const uint32_t lo = fold & 0xFFFFu, hi = fold >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

}  // namespace llmq

// m_dtype / v_dtype: 0 = fp32, 1 = bf16; supported pairs (m, v): (0, 0), (1, 0), (1, 1), as in the reference.
extern "C" int llmq_adamw_update_bf16(uint16_t* params, const uint16_t* grads, void* m, int m_dtype, void* v, int v_dtype,
                                      int64_t num_parameters, float learning_rate, float beta1, float beta2, int t,
                                      float eps, float weight_decay, const float* grad_scale, float* abs_max_or_null,
                                      unsigned int seed, void* stream_) {
    using namespace llmq;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    LLMQ_REQUIRE(num_parameters >= 0, "adamw_update: negative parameter count %lld", (long long)num_parameters);
    LLMQ_REQUIRE(num_parameters % 8 == 0, "adamw_update: num_parameters must be divisible by 8 (got %lld)",
                 (long long)num_parameters);
    LLMQ_REQUIRE((m_dtype == 0 || m_dtype == 1) && (v_dtype == 0 || v_dtype == 1) && !(m_dtype == 0 && v_dtype == 1),
                 "adamw_update: unsupported moment types (m %d, v %d): fp32/fp32, bf16/fp32 or bf16/bf16", m_dtype, v_dtype);
    LLMQ_REQUIRE(grad_scale != nullptr, "adamw_update: grad_scale pointer is null");
    if (num_parameters == 0) return LLMQ_OK;
    LLMQ_REQUIRE(params && grads && m && v, "adamw_update: null tensor pointer");
    LLMQ_REQUIRE(aligned16(params) && aligned16(grads) && aligned16(m) && aligned16(v),
                 "adamw_update: tensors must be 16-byte aligned");
    // bias corrections on the host in fp32, as the reference computes them (adamw.cu:153-158)
    const float c1 = 1.0f / (1.0f - powf(beta1, (float)t)), c2 = 1.0f / (1.0f - powf(beta2, (float)t));
    const AdamArgs a{learning_rate, beta1, beta2, c1, c2, eps, weight_decay, seed};
    const int64_t nvec = num_parameters / 8;
    auto launch = [&](auto kernel, int threads) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)((nvec + threads - 1) / threads)), dim3(threads), 0, stream,
                           reinterpret_cast<uint4*>(params), reinterpret_cast<const uint4*>(grads), m, v, nvec, a, grad_scale,
                           reinterpret_cast<unsigned*>(abs_max_or_null));
    };
    LLMQ_REQUIRE((nvec + 255) / 256 <= 0x7FFFFFFF, "adamw_update: tensor too large");
#define LLMQ_ADAM(MB, VB)                                                     \
    do {                                                                      \
        if (abs_max_or_null) launch(adamw_kernel<MB, VB, true, 1024>, 1024);  \
        else launch(adamw_kernel<MB, VB, false, 256>, 256);                   \
    } while (0)
    if (m_dtype == 0) LLMQ_ADAM(false, false);
    else if (v_dtype == 0) LLMQ_ADAM(true, false);
    else LLMQ_ADAM(true, true);
#undef LLMQ_ADAM
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// fp32 parameters, gradients and moments.  `seed` is accepted for the reference's signature and unused.
extern "C" int llmq_adamw_update_f32(float* params, const float* grads, float* m, float* v, int64_t num_parameters,
                                     float learning_rate, float beta1, float beta2, int t, float eps, float weight_decay,
                                     const float* grad_scale, float* abs_max_or_null, unsigned int seed, void* stream_) {
    using namespace llmq;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    LLMQ_REQUIRE(num_parameters >= 0, "adamw_update: negative parameter count %lld", (long long)num_parameters);
    LLMQ_REQUIRE(num_parameters % 4 == 0, "adamw_update: num_parameters must be divisible by 4 for fp32 tensors (got %lld)",
                 (long long)num_parameters);
    LLMQ_REQUIRE(grad_scale != nullptr, "adamw_update: grad_scale pointer is null");
    if (num_parameters == 0) return LLMQ_OK;
    LLMQ_REQUIRE(params && grads && m && v, "adamw_update: null tensor pointer");
    LLMQ_REQUIRE(aligned16(params) && aligned16(grads) && aligned16(m) && aligned16(v),
                 "adamw_update: tensors must be 16-byte aligned");
    const float c1 = 1.0f / (1.0f - powf(beta1, (float)t)), c2 = 1.0f / (1.0f - powf(beta2, (float)t));
    const AdamArgs a{learning_rate, beta1, beta2, c1, c2, eps, weight_decay, seed};
    const int64_t nvec = num_parameters / 4;
    LLMQ_REQUIRE((nvec + 255) / 256 <= 0x7FFFFFFF, "adamw_update: tensor too large");
    auto launch = [&](auto kernel, int threads) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)((nvec + threads - 1) / threads)), dim3(threads), 0, stream,
                           reinterpret_cast<uint4*>(params), reinterpret_cast<const uint4*>(grads), reinterpret_cast<uint4*>(m),
                           reinterpret_cast<uint4*>(v), nvec, a, grad_scale, reinterpret_cast<unsigned*>(abs_max_or_null));
    };
    if (abs_max_or_null) launch(adamw_f32_kernel<true, 1024>, 1024);
    else launch(adamw_f32_kernel<false, 256>, 256);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// e4m3 first moment with one fp32 scale per 128 elements, bf16 second moment.
extern "C" int llmq_adamw_update_bf16_fp8m(uint16_t* params, const uint16_t* grads, uint8_t* m_e4m3, float* m_scales,
                                           uint16_t* v_bf16, int64_t num_parameters, float learning_rate, float beta1,
                                           float beta2, int t, float eps, float weight_decay, const float* grad_scale,
                                           float* abs_max_or_null, unsigned int seed, void* stream_) {
    using namespace llmq;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    LLMQ_REQUIRE(num_parameters >= 0, "adamw_update: negative parameter count %lld", (long long)num_parameters);
    LLMQ_REQUIRE(num_parameters % 8 == 0, "adamw_update: num_parameters must be divisible by 8 (got %lld)",
                 (long long)num_parameters);
    LLMQ_REQUIRE(grad_scale != nullptr, "adamw_update: grad_scale pointer is null");
    if (num_parameters == 0) return LLMQ_OK;
    LLMQ_REQUIRE(params && grads && m_e4m3 && m_scales && v_bf16, "adamw_update: null tensor pointer");
    LLMQ_REQUIRE(aligned16(params) && aligned16(grads) && aligned16(v_bf16) && (reinterpret_cast<uintptr_t>(m_e4m3) & 7u) == 0,
                 "adamw_update: tensors must be 16-byte aligned (the e4m3 moment 8-byte)");
    const float c1 = 1.0f / (1.0f - powf(beta1, (float)t)), c2 = 1.0f / (1.0f - powf(beta2, (float)t));
    const AdamArgs a{learning_rate, beta1, beta2, c1, c2, eps, weight_decay, seed};
    const int64_t nvec = num_parameters / 8;
    LLMQ_REQUIRE((nvec + 255) / 256 <= 0x7FFFFFFF, "adamw_update: tensor too large");
    auto launch = [&](auto kernel, int threads) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)((nvec + threads - 1) / threads)), dim3(threads), 0, stream,
                           reinterpret_cast<uint4*>(params), reinterpret_cast<const uint4*>(grads), reinterpret_cast<uint2*>(m_e4m3),
                           m_scales, reinterpret_cast<uint4*>(v_bf16), nvec, a, grad_scale,
                           reinterpret_cast<unsigned*>(abs_max_or_null));
    };
    if (abs_max_or_null) launch(adamw_fp8m_kernel<true, 1024>, 1024);
    else launch(adamw_fp8m_kernel<false, 256>, 256);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}
