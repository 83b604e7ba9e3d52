// SwiGLU producers of the FP8 matmul path for gfx950: the activation in front of the down projection
// and its gradient in front of the up projection, each with the abs-max of its own output computed on
// the way, and the variant that writes e4m3 codes directly.
//
// Semantics follow the reference (src/kernels/swiglu.cu:20-23, 25-65, 67-98, 244-300): the input row is
// [up(C) | gate(C)],
//   s   = 1 / (1 + exp(-gate))
//   out = bf16((up * gate) * s)
//   dup = bf16(dout * gate * s),   dgate = bf16(dout * up * s * (1 + gate * (1 - s)))
// with every product taken left to right in fp32, the abs-max taken over the rounded bf16 outputs (slot
// reset first), and the quantizing variant producing exactly quantize_with_abs_max(bf16 out):
// scale = 448 / max(abs_max, 1e-10), code = e4m3(scale * (float)bf16(out)), *scale_ptr = 1 / scale.
// The reference evaluates exp with the CUDA math library and the reciprocal with its approximate
// instruction, so its results are not bit-specified; here exp is the hardware exp2 of gate * -log2(e) and
// the reciprocal the hardware one (both about 1 ulp), which lands within one bf16 ulp of the correctly
// rounded value.
//
// All three kernels are HBM bound (forward 6, quantizing forward 5, backward 10 bytes per activation
// element): one trip per lane with UNROLL independent 16-byte chunks in flight per operand, each wave
// instruction covering 1 KiB contiguous; a chunk never straddles a row because C is a multiple of 8.
#include "common.hpp"
#include "absmax_reduce.hpp"
#include "fp8_encode.hpp"

namespace llmq {

typedef float f32x2_sw __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_sw __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float sigmoid_fast(float gate) {
    const float e = __builtin_amdgcn_exp2f(gate * -1.4426950408889634f);  // exp(-gate)
    return __builtin_amdgcn_rcpf(1.0f + e);
}

// two fp32 values -> packed bf16 pair (round to nearest even), a in the low half
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    const f32x2_sw p = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2_sw));
}

__device__ __forceinline__ uint32_t swiglu_pair(uint32_t up, uint32_t gate) {
    const float g0 = bf16_lo(gate), g1 = bf16_hi(gate);
    return pack_bf16((bf16_lo(up) * g0) * sigmoid_fast(g0), (bf16_hi(up) * g1) * sigmoid_fast(g1));
}

__device__ __forceinline__ uint4 swiglu_chunk(const uint4& up, const uint4& gate) {
    return make_uint4(swiglu_pair(up.x, gate.x), swiglu_pair(up.y, gate.y), swiglu_pair(up.z, gate.z),
                      swiglu_pair(up.w, gate.w));
}

// chunk number -> offset (in 16-byte chunks) of its up part in the [rows][2C] input
__device__ __forceinline__ uint32_t input_chunk(uint32_t idx, uint32_t chunks_per_row) {
    const uint32_t row = idx / chunks_per_row;
    return idx + row * chunks_per_row;  // row * 2 cpr + (idx - row * cpr)
}

// MODE 0: bf16 output; 1: bf16 output + abs-max; 2: e4m3 output with the scale from *absmax_in
// THREADS: 256, or 1024 with the abs-max (fewer workgroups -> fewer atomics on the one slot when the
// workgroups of the first resident round finish together and all find it empty).
template <int MODE, int UNROLL, int THREADS>
__global__ __launch_bounds__(THREADS) void swiglu_forward_kernel(void* __restrict__ out, const uint4* __restrict__ inp,
                                                             unsigned* __restrict__ absmax_out,
                                                             const float* __restrict__ absmax_in,
                                                             float* __restrict__ scale_ptr, uint32_t nchunks,
                                                             uint32_t chunks_per_row) {
    const uint32_t base = blockIdx.x * ((uint32_t)THREADS * UNROLL) + threadIdx.x;
    float s = 0.f;
    if constexpr (MODE == 2) {
        s = quant_scale(*absmax_in);
        if (base == 0 && scale_ptr) *scale_ptr = __fdiv_rn(1.f, s);
    }
    uint4 up[UNROLL], gate[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        up[u] = gate[u] = make_uint4(0, 0, 0, 0);
        if (idx < nchunks) {
            const uint32_t src = input_chunk(idx, chunks_per_row);
            up[u] = load_nt(&inp[src]);
            gate[u] = load_nt(&inp[src + chunks_per_row]);
        }
    }
    uint32_t acc = 0x7F807F80u;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        const uint4 r = swiglu_chunk(up[u], gate[u]);  // zeros for the predicated-off chunks
        if constexpr (MODE == 1) acc = fold_vec(acc, r);
        if (idx < nchunks) {
            if constexpr (MODE == 2) store_nt(&reinterpret_cast<uint2*>(out)[idx], encode8<kE4M3>(r, s));
            else store_nt(&reinterpret_cast<uint4*>(out)[idx], r);
        }
    }
    if constexpr (MODE == 1) {
        const uint32_t lo = acc & 0xFFFFu, hi = acc >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

__device__ __forceinline__ void swiglu_grad_pair(uint32_t dout, uint32_t up, uint32_t gate, uint32_t& dup,
                                                 uint32_t& dgate) {
    float d1[2], d2[2];
    const float dv[2] = {bf16_lo(dout), bf16_hi(dout)}, uv[2] = {bf16_lo(up), bf16_hi(up)},
                gv[2] = {bf16_lo(gate), bf16_hi(gate)};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float sg = sigmoid_fast(gv[k]);
        d1[k] = dv[k] * gv[k] * sg;
        d2[k] = dv[k] * uv[k] * sg * (1.0f + gv[k] * (1.0f - sg));
    }
    dup = pack_bf16(d1[0], d1[1]);
    dgate = pack_bf16(d2[0], d2[1]);
}

template <bool ABSMAX, int UNROLL, int THREADS>
__global__ __launch_bounds__(THREADS) void swiglu_backward_kernel(uint4* __restrict__ dinp, const uint4* __restrict__ dout,
                                                              const uint4* __restrict__ inp,
                                                              unsigned* __restrict__ absmax_out, uint32_t nchunks,
                                                              uint32_t chunks_per_row) {
    const uint32_t base = blockIdx.x * ((uint32_t)THREADS * UNROLL) + threadIdx.x;
    uint4 d[UNROLL], up[UNROLL], gate[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        d[u] = up[u] = gate[u] = make_uint4(0, 0, 0, 0);
        if (idx < nchunks) {
            const uint32_t src = input_chunk(idx, chunks_per_row);
            d[u] = load_nt(&dout[idx]);
            up[u] = load_nt(&inp[src]);
            gate[u] = load_nt(&inp[src + chunks_per_row]);
        }
    }
    uint32_t acc = 0x7F807F80u;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = base + u * (uint32_t)THREADS;
        uint4 g1, g2;
        swiglu_grad_pair(d[u].x, up[u].x, gate[u].x, g1.x, g2.x);
        swiglu_grad_pair(d[u].y, up[u].y, gate[u].y, g1.y, g2.y);
        swiglu_grad_pair(d[u].z, up[u].z, gate[u].z, g1.z, g2.z);
        swiglu_grad_pair(d[u].w, up[u].w, gate[u].w, g1.w, g2.w);
        if constexpr (ABSMAX) acc = fold_vec(fold_vec(acc, g1), g2);
        if (idx < nchunks) {
            const uint32_t dst = input_chunk(idx, chunks_per_row);
            store_nt(&dinp[dst], g1);
            store_nt(&dinp[dst + chunks_per_row], g2);
        }
    }
    if constexpr (ABSMAX) {
        const uint32_t lo = acc & 0xFFFFu, hi = acc >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

// Common argument checks (the reference throws on the same conditions, src/kernels/swiglu.cu:306-318):
// C a multiple of 8 and 2 * B * T * C below 2^31.  Unlike the reference, B * T * C need not be a multiple of
// the workgroup's share.
static int check_shape(const char* what, int B, int T, int C, int64_t& nchunks) {
    LLMQ_REQUIRE(B >= 0 && T >= 0 && C >= 0, "%s: negative dimension (%d, %d, %d)", what, B, T, C);
    LLMQ_REQUIRE(C % 8 == 0, "%s: C must be divisible by 8 (got %d)", what, C);
    const int64_t nelem = (int64_t)B * T * C;
    LLMQ_REQUIRE(2 * nelem < 0x7FFFFFFFLL, "%s: input too large (%lld elements)", what, (long long)(2 * nelem));
    nchunks = nelem / 8;
    return LLMQ_OK;
}

constexpr int kFwdUnroll = 4, kBwdUnroll = 2, kAbsmaxThreads = 512;

static unsigned blocks_for(int64_t nchunks, int threads, int unroll) {
    return (unsigned)((nchunks + (int64_t)threads * unroll - 1) / ((int64_t)threads * unroll));
}

}  // namespace llmq

using namespace llmq;

extern "C" int llmq_swiglu_forward_bf16(uint16_t* out, const uint16_t* inp, float* abs_max_or_null, int B, int T, int C,
                                        void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int64_t nchunks;
    if (int rc = check_shape("swiglu_forward", B, T, C, nchunks)) return rc;
    if (abs_max_or_null) {
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(abs_max_or_null));
        LLMQ_HIP_TRY(hipGetLastError());
    }
    if (nchunks == 0) return LLMQ_OK;
    LLMQ_REQUIRE(out && inp, "swiglu_forward: null tensor pointer");
    LLMQ_REQUIRE(aligned16(out) && aligned16(inp), "swiglu_forward: pointers must be 16-byte aligned");
    if (abs_max_or_null)
        hipLaunchKernelGGL((swiglu_forward_kernel<1, kFwdUnroll, kAbsmaxThreads>),
                           dim3(blocks_for(nchunks, kAbsmaxThreads, kFwdUnroll)), dim3(kAbsmaxThreads), 0, stream, out,
                           reinterpret_cast<const uint4*>(inp), reinterpret_cast<unsigned*>(abs_max_or_null), nullptr,
                           nullptr, (uint32_t)nchunks, (uint32_t)(C / 8));
    else
        hipLaunchKernelGGL((swiglu_forward_kernel<0, kFwdUnroll, 256>), dim3(blocks_for(nchunks, 256, kFwdUnroll)),
                           dim3(256), 0, stream, out,
                           reinterpret_cast<const uint4*>(inp), nullptr, nullptr, nullptr, (uint32_t)nchunks,
                           (uint32_t)(C / 8));
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

extern "C" int llmq_swiglu_forward_quant_bf16(uint8_t* out, float* scale_or_null, const uint16_t* inp,
                                              const float* abs_max, int B, int T, int C, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int64_t nchunks;
    if (int rc = check_shape("swiglu_forward_quant", B, T, C, nchunks)) return rc;
    LLMQ_REQUIRE(abs_max != nullptr, "swiglu_forward_quant: abs_max pointer is null");
    LLMQ_REQUIRE(nchunks == 0 || (out && inp), "swiglu_forward_quant: null tensor pointer");
    LLMQ_REQUIRE(aligned16(inp) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0,
                 "swiglu_forward_quant: inp must be 16-byte and out 8-byte aligned");
    // an empty tensor still gets its scale written, by the same kernel (grid of one workgroup)
    // two chunks per operand and lane: 4 % faster than four for this variant (130 against 134 us on [8192 x 18944],
    // alternating builds, tensors no cache holds); the bf16-output variants measured the other way round
    constexpr int kQuantUnroll = 2;
    const unsigned blocks = nchunks ? blocks_for(nchunks, 256, kQuantUnroll) : 1u;
    hipLaunchKernelGGL((swiglu_forward_kernel<2, kQuantUnroll, 256>), dim3(blocks), dim3(256), 0, stream, out,
                       reinterpret_cast<const uint4*>(inp), nullptr, abs_max, scale_or_null, (uint32_t)nchunks,
                       (uint32_t)(C > 0 ? C / 8 : 1));
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

extern "C" int llmq_swiglu_backward_bf16(uint16_t* dinp, const uint16_t* dout, const uint16_t* inp,
                                         float* abs_max_or_null, int B, int T, int C, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int64_t nchunks;
    if (int rc = check_shape("swiglu_backward", B, T, C, nchunks)) return rc;
    if (abs_max_or_null) {
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(abs_max_or_null));
        LLMQ_HIP_TRY(hipGetLastError());
    }
    if (nchunks == 0) return LLMQ_OK;
    LLMQ_REQUIRE(dinp && dout && inp, "swiglu_backward: null tensor pointer");
    LLMQ_REQUIRE(aligned16(dinp) && aligned16(dout) && aligned16(inp), "swiglu_backward: pointers must be 16-byte aligned");
    if (abs_max_or_null)
        hipLaunchKernelGGL((swiglu_backward_kernel<true, kBwdUnroll, kAbsmaxThreads>),
                           dim3(blocks_for(nchunks, kAbsmaxThreads, kBwdUnroll)), dim3(kAbsmaxThreads), 0, stream,
                           reinterpret_cast<uint4*>(dinp), reinterpret_cast<const uint4*>(dout),
                           reinterpret_cast<const uint4*>(inp), reinterpret_cast<unsigned*>(abs_max_or_null),
                           (uint32_t)nchunks, (uint32_t)(C / 8));
    else
        hipLaunchKernelGGL((swiglu_backward_kernel<false, kBwdUnroll, 256>), dim3(blocks_for(nchunks, 256, kBwdUnroll)),
                           dim3(256), 0, stream,
                           reinterpret_cast<uint4*>(dinp), reinterpret_cast<const uint4*>(dout),
                           reinterpret_cast<const uint4*>(inp), nullptr, (uint32_t)nchunks, (uint32_t)(C / 8));
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}
