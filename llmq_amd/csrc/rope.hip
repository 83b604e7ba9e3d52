// Rotary position embedding on the fused QKV tensor for gfx950, forward and backward, with the abs-max of
// the output computed on the way (the backward's abs-max is that of the gradient entering the QKV
// projection's backward matmuls).
//
// Semantics follow the reference (src/kernels/rope.cu:42-127): the tensor is [B, T, Nq + 2 Nkv, head_dim]
// bf16, freqs_cis is [T, head_dim] fp16 holding (cos, sin) pairs for d = 0 .. head_dim/2 - 1.  For query and
// key heads, with real = x[d], imag = x[d + head_dim/2]:
//     out[d]              = bf16(real * cos - imag * sin)
//     out[d + head_dim/2] = bf16(real * sin + imag * cos)          (backward: sin -> -sin)
// in fp32; value heads are copied (not touched when out == inp).  *abs_max = max |out| over all heads,
// value heads included, slot reset first.  Products and sums are separate fp32 operations here (the
// reference's compiler may fuse them), which differs by at most an fp32 rounding.
//
// HBM bound: 4 bytes per element (2 for the value heads when in place with abs-max, 0 without).  A lane takes
// W consecutive d of one head: W * 2 bytes from each half plus the 2 W fp16 factors, with W = 8 (16-byte
// accesses) when head_dim is a multiple of 16 and W = 4 otherwise.
#include <hip/hip_fp16.h>

#include <cmath>

#include "common.hpp"
#include "absmax_reduce.hpp"

namespace llmq {

typedef float f32x2_rp __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_rp __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_rp __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16_rp(float a, float b) {
    const f32x2_rp p = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2_rp));
}

// one dword of the real half, one of the imaginary half, two dwords of (cos, sin) pairs -> rotated dwords
template <bool BACKWARD>
__device__ __forceinline__ void rotate_pair(uint32_t re, uint32_t im, uint32_t cs0, uint32_t cs1, uint32_t& o_re,
                                            uint32_t& o_im) {
    const f16x2_rp f0 = __builtin_bit_cast(f16x2_rp, cs0), f1 = __builtin_bit_cast(f16x2_rp, cs1);
    const float c0 = (float)f0[0], c1 = (float)f1[0];
    const float s0 = BACKWARD ? -(float)f0[1] : (float)f0[1], s1 = BACKWARD ? -(float)f1[1] : (float)f1[1];
    const float r0 = bf16_lo(re), r1 = bf16_hi(re), i0 = bf16_lo(im), i1 = bf16_hi(im);
    o_re = pack_bf16_rp(r0 * c0 - i0 * s0, r1 * c1 - i1 * s1);
    o_im = pack_bf16_rp(r0 * s0 + i0 * c0, r1 * s1 + i1 * c1);
}

template <int DW> struct Words;  // DW dwords moved with one access
template <> struct Words<2> { typedef unsigned int type __attribute__((ext_vector_type(2))); };
template <> struct Words<4> { typedef unsigned int type __attribute__((ext_vector_type(4))); };
// STREAM: non-temporal (the tensor itself; the small factor table is left to the caches)
template <int DW, bool STREAM>
__device__ __forceinline__ void load_words(uint32_t (&dst)[DW], const void* p) {
    typedef typename Words<DW>::type V;
    const V v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const V*>(p)) : *reinterpret_cast<const V*>(p);
#pragma unroll
    for (int k = 0; k < DW; ++k) dst[k] = v[k];
}
template <int DW>
__device__ __forceinline__ void store_words(void* p, const uint32_t (&src)[DW]) {
    typedef typename Words<DW>::type V;
    V v;
#pragma unroll
    for (int k = 0; k < DW; ++k) v[k] = src[k];
    __builtin_nontemporal_store(v, reinterpret_cast<V*>(p));
}

// W: d values per lane (4 or 8).  Lane -> (token bt, head h, group of W d values).
template <bool BACKWARD, bool ABSMAX, int W, int THREADS>
__global__ __launch_bounds__(THREADS) void rope_kernel(uint16_t* out, const uint16_t* inp, const uint16_t* __restrict__ freqs,
                                                   unsigned* __restrict__ absmax_out, int64_t total, int T, int Nq,
                                                   int Nkv, int head_dim) {
    constexpr int DW = W / 2;  // dwords per half and lane
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t fold = 0x7F807F80u;
    if (idx < total) {
        const int groups = head_dim / (2 * W);
        const int N = Nq + 2 * Nkv;
        const int grp = (int)(idx % groups);
        const int h = (int)((idx / groups) % N);
        const int64_t bt = idx / ((int64_t)groups * N);
        const int t = (int)(bt % T);
        const int64_t base = (bt * N + h) * head_dim + (int64_t)grp * W;
        const bool in_place = out == inp;
        const bool rotated = h < Nq + Nkv;
        if (rotated || ABSMAX || !in_place) {
            uint32_t re[DW], im[DW];
            load_words<DW, true>(re, inp + base);
            load_words<DW, true>(im, inp + base + head_dim / 2);
            if (rotated) {
                const uint16_t* f = freqs + (int64_t)t * head_dim + 2 * grp * W;
                uint32_t cs_lo[DW], cs_hi[DW], cs[W];
                load_words<DW, false>(cs_lo, f);
                load_words<DW, false>(cs_hi, f + W);
#pragma unroll
                for (int k = 0; k < DW; ++k) {
                    cs[k] = cs_lo[k];
                    cs[DW + k] = cs_hi[k];
                }
#pragma unroll
                for (int k = 0; k < DW; ++k) rotate_pair<BACKWARD>(re[k], im[k], cs[2 * k], cs[2 * k + 1], re[k], im[k]);
            }
            if (rotated || !in_place) {
                store_words<DW>(out + base, re);
                store_words<DW>(out + base + head_dim / 2, im);
            }
            if constexpr (ABSMAX) {
#pragma unroll
                for (int k = 0; k < DW; ++k) fold = fold_bf16x2(fold_bf16x2(fold, re[k]), im[k]);
            }
        }
    }
    if constexpr (ABSMAX) {
        const uint32_t lo = fold & 0xFFFFu, hi = fold >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

template <bool BACKWARD>
static int rope_any(const char* what, uint16_t* out, const uint16_t* inp, const uint16_t* freqs, float* abs_max, int B,
                    int T, int Nq, int Nkv, int head_dim, hipStream_t stream) {
    LLMQ_REQUIRE(B >= 0 && T >= 0 && Nq >= 0 && Nkv >= 0 && head_dim >= 0, "%s: negative dimension", what);
    LLMQ_REQUIRE(head_dim % 8 == 0, "%s: head_dim must be divisible by 8 (got %d)", what, head_dim);
    if (abs_max) {
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(abs_max));
        LLMQ_HIP_TRY(hipGetLastError());
    }
    const int64_t heads = (int64_t)B * T * (Nq + 2 * Nkv);
    if (heads == 0 || head_dim == 0) return LLMQ_OK;
    LLMQ_REQUIRE(out && inp && freqs, "%s: null tensor pointer", what);
    LLMQ_REQUIRE(aligned16(out) && aligned16(inp) && aligned16(freqs), "%s: pointers must be 16-byte aligned", what);
    const int w = head_dim % 16 == 0 ? 8 : 4;
    const int64_t total = heads * (head_dim / (2 * w));
    LLMQ_REQUIRE((total + 255) / 256 <= 0x7FFFFFFF, "%s: tensor too large", what);
    auto launch = [&](auto kernel, int threads) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)((total + threads - 1) / threads)), dim3(threads), 0, stream, out, inp,
                           freqs, reinterpret_cast<unsigned*>(abs_max), total, T, Nq, Nkv, head_dim);
    };
    // with the abs-max: 1024-thread workgroups (fewer workgroups -> fewer atomics on the one slot)
    if (w == 8) {
        if (abs_max) launch(rope_kernel<BACKWARD, true, 8, 1024>, 1024);
        else launch(rope_kernel<BACKWARD, false, 8, 256>, 256);
    } else {
        if (abs_max) launch(rope_kernel<BACKWARD, true, 4, 1024>, 1024);
        else launch(rope_kernel<BACKWARD, false, 4, 256>, 256);
    }
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

}  // namespace llmq

extern "C" int llmq_rope_forward_bf16(uint16_t* out, const uint16_t* inp, const uint16_t* freqs_cis_f16,
                                      float* abs_max_or_null, int B, int T, int Nq, int Nkv, int head_dim, void* stream) {
    return llmq::rope_any<false>("rope_forward", out, inp, freqs_cis_f16, abs_max_or_null, B, T, Nq, Nkv, head_dim,
                                 static_cast<hipStream_t>(stream));
}

extern "C" int llmq_rope_backward_bf16(uint16_t* dinp, const uint16_t* dout, const uint16_t* freqs_cis_f16,
                                       float* abs_max_or_null, int B, int T, int Nq, int Nkv, int head_dim, void* stream) {
    return llmq::rope_any<true>("rope_backward", dinp, dout, freqs_cis_f16, abs_max_or_null, B, T, Nq, Nkv, head_dim,
                                static_cast<hipStream_t>(stream));
}

// Host-side table of (cos, sin) pairs in fp16, [end][dim] (src/kernels/rope.cu:15-31): angle = t / theta^(2i/dim)
// in fp32 with the C library's powf / cosf / sinf, as the reference computes it.
extern "C" int llmq_precompute_freqs_cis_f16(uint16_t* freqs_cis_host, int dim, int end, float theta) {
    LLMQ_REQUIRE(freqs_cis_host != nullptr || dim == 0 || end == 0, "precompute_freqs_cis: null output pointer");
    LLMQ_REQUIRE(dim >= 0 && end >= 0 && dim % 2 == 0, "precompute_freqs_cis: dim must be even and non-negative");
    for (int i = 0; i < dim / 2; ++i) {
        const float inv_freq = 1.0f / powf(theta, (float)(2 * i) / (float)dim);
        for (int t = 0; t < end; ++t) {
            const float angle = (float)t * inv_freq;
            const _Float16 c = (_Float16)cosf(angle), s = (_Float16)sinf(angle);
            uint16_t cb, sb;
            __builtin_memcpy(&cb, &c, 2);
            __builtin_memcpy(&sb, &s, 2);
            freqs_cis_host[(size_t)t * dim + 2 * i] = cb;
            freqs_cis_host[(size_t)t * dim + 2 * i + 1] = sb;
        }
    }
    return LLMQ_OK;
}
