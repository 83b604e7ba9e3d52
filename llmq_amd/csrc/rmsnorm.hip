// RMSNorm forward (plain and with the residual add fused in) for gfx950: the producer of the inputs of
// the QKV and gate+up projections, with the abs-max of its output computed on the way.
//
// Semantics follow the reference (src/kernels/rmsnorm.cu:17-86, 88-164, 168-178), per row of C elements:
//   [fused: res = bf16((float)inp1 + (float)inp2), stored to `residual`; otherwise res = inp1]
//   s   = 1 / sqrt(mean(res^2) + epsilon)                          (fp32; stored to rrms[row])
//   out = bf16( (float)bf16(s * res) * (float)weight )             (the normalised value is rounded to
//                                                                   bf16 before the scale, as the reference does)
//   *abs_max = max |out| over the rounded outputs (slot reset first, NaNs ignored).
// The reference sums the squares in an order fixed by its launch geometry and uses the approximate
// reciprocal square root, so s is not bit-specified; here the squares are summed in fp32 per lane and
// combined by a fixed butterfly (deterministic), the mean is divided by C, and s = 1 / sqrtf(.) with the
// correctly rounded square root and division.
//
// HBM bound: 4 bytes per element (8 with the residual: two reads, two writes).  One wave per row and the
// whole row in registers (NCH 16-byte chunks per lane), so every input byte is read once; WAVES rows per
// workgroup; every wave instruction covers 1 KiB contiguous.  The weight row comes through the cache.
// With the abs-max the workgroups are as large as the registers allow (16 rows): tensors of this size run
// with the whole grid resident, all workgroups finish together and find the slot still empty, so each one
// issues its atomic -- 2048 of them on one address cost 10 us on a 15 us kernel; 512 cost a quarter.
#include "common.hpp"
#include "absmax_reduce.hpp"

namespace llmq {

typedef float f32x2_rn __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_rn __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16_rn(float a, float b) {
    const f32x2_rn p = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2_rn));
}

__device__ __forceinline__ uint32_t add_pair(uint32_t a, uint32_t b) {
    return pack_bf16_rn(bf16_lo(a) + bf16_lo(b), bf16_hi(a) + bf16_hi(b));
}

__device__ __forceinline__ float squares(float acc, uint32_t w) {
    const float lo = bf16_lo(w), hi = bf16_hi(w);
    acc = acc + lo * lo;
    return acc + hi * hi;
}

__device__ __forceinline__ uint32_t norm_pair(uint32_t x, uint32_t w, float s) {
    const uint32_t n = pack_bf16_rn(s * bf16_lo(x), s * bf16_hi(x));
    return pack_bf16_rn(bf16_lo(n) * bf16_lo(w), bf16_hi(n) * bf16_hi(w));  // exact products, one rounding
}

template <int NCH, bool RESIDUAL, bool ABSMAX, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void rmsnorm_forward_kernel(uint4* residual, uint4* __restrict__ normed,
                                                              float* __restrict__ rrms, const uint4* __restrict__ inp1,
                                                              const uint4* __restrict__ inp2,
                                                              const uint4* __restrict__ weight,
                                                              unsigned* __restrict__ absmax_out, float epsilon, int N,
                                                              int chunks, float c_float) {
    const int lane = threadIdx.x % kWave;
    const int row = blockIdx.x * WAVES + threadIdx.x / kWave;
    const bool valid = row < N;  // no early exit: the abs-max reduction below synchronises the workgroup
    const int64_t base = (int64_t)row * chunks;

    uint4 x[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = lane + kWave * k;
        x[k] = make_uint4(0, 0, 0, 0);
        if (valid && c < chunks) x[k] = inp1[base + c];
    }
    if constexpr (RESIDUAL) {
        uint4 y[NCH];
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = lane + kWave * k;
            y[k] = make_uint4(0, 0, 0, 0);
            if (valid && c < chunks) y[k] = inp2[base + c];
        }
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = lane + kWave * k;
            x[k] = make_uint4(add_pair(x[k].x, y[k].x), add_pair(x[k].y, y[k].y), add_pair(x[k].z, y[k].z),
                              add_pair(x[k].w, y[k].w));
            if (valid && c < chunks) residual[base + c] = x[k];
        }
    }

    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < NCH; ++k) acc = squares(squares(squares(squares(acc, x[k].x), x[k].y), x[k].z), x[k].w);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc = acc + __shfl_xor(acc, off, kWave);
    const float s = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(acc, c_float) + epsilon));

    uint32_t fold = 0x7F807F80u;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = lane + kWave * k;
        if (c < chunks) {
            const uint4 w = weight[c];
            const uint4 o = make_uint4(norm_pair(x[k].x, w.x, s), norm_pair(x[k].y, w.y, s), norm_pair(x[k].z, w.z, s),
                                       norm_pair(x[k].w, w.w, s));
            if (valid) {
                normed[base + c] = o;
                if constexpr (ABSMAX) fold = fold_vec(fold, o);
            }
        }
    }
    if (valid && lane == 0 && rrms) rrms[row] = s;
    if constexpr (ABSMAX) {
        const uint32_t lo = fold & 0xFFFFu, hi = fold >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

template <int NCH, bool RESIDUAL>
static void launch_rows(uint16_t* residual, uint16_t* normed, float* rrms, const uint16_t* inp1, const uint16_t* inp2,
                        const uint16_t* weight, float* abs_max, float epsilon, int N, int C, hipStream_t stream) {
    // rows per workgroup with the abs-max: what 512 registers per SIMD allow for this row width
    constexpr int AM_WAVES = NCH <= 8 ? 16 : NCH == 16 ? 8 : 4;
    auto launch = [&](auto kernel, int waves) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)((N + waves - 1) / waves)), dim3(waves * 64), 0, stream,
                           reinterpret_cast<uint4*>(residual), reinterpret_cast<uint4*>(normed), rrms,
                           reinterpret_cast<const uint4*>(inp1), reinterpret_cast<const uint4*>(inp2),
                           reinterpret_cast<const uint4*>(weight), reinterpret_cast<unsigned*>(abs_max), epsilon, N,
                           C / 8, (float)C);
    };
    if (abs_max) launch(rmsnorm_forward_kernel<NCH, RESIDUAL, true, AM_WAVES>, AM_WAVES);
    else launch(rmsnorm_forward_kernel<NCH, RESIDUAL, false, 4>, 4);
}

// fused == false is the plain form (residual and inp2 unused); `residual` may be the same buffer as inp1 or inp2
// (every lane reads its chunks before it writes them).
static int rmsnorm_forward_any(const char* what, bool fused, uint16_t* residual, uint16_t* normed, float* rrms,
                               const uint16_t* inp1, const uint16_t* inp2, const uint16_t* weight, float* abs_max,
                               float epsilon, int64_t N64, int C, hipStream_t stream) {
    LLMQ_REQUIRE(N64 >= 0 && C >= 0, "%s: negative dimension (%lld rows, C = %d)", what, (long long)N64, C);
    LLMQ_REQUIRE(N64 <= 0x7FFFFFFF, "%s: too many rows (%lld)", what, (long long)N64);
    LLMQ_REQUIRE(C % 8 == 0, "%s: C must be divisible by 8 (got %d)", what, C);
    LLMQ_REQUIRE(C <= 16384, "%s: C up to 16384 is supported (got %d)", what, C);
    const int N = (int)N64;
    if (abs_max) {
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(abs_max));
        LLMQ_HIP_TRY(hipGetLastError());
    }
    if (N == 0 || C == 0) return LLMQ_OK;
    LLMQ_REQUIRE(normed && inp1 && weight && (!fused || (residual && inp2)), "%s: null tensor pointer", what);
    LLMQ_REQUIRE(aligned16(residual) && aligned16(normed) && aligned16(inp1) && aligned16(inp2) && aligned16(weight),
                 "%s: tensor pointers must be 16-byte aligned", what);
    const int per_lane = (C / 8 + kWave - 1) / kWave;
#define LLMQ_ROWS(NCH)                                                                                              \
    do {                                                                                                            \
        if (fused) launch_rows<NCH, true>(residual, normed, rrms, inp1, inp2, weight, abs_max, epsilon, N, C, stream); \
        else launch_rows<NCH, false>(nullptr, normed, rrms, inp1, nullptr, weight, abs_max, epsilon, N, C, stream);  \
    } while (0)
    if (per_lane <= 2) LLMQ_ROWS(2);
    else if (per_lane <= 4) LLMQ_ROWS(4);
    else if (per_lane <= 8) LLMQ_ROWS(8);
    else if (per_lane <= 16) LLMQ_ROWS(16);
    else LLMQ_ROWS(32);
#undef LLMQ_ROWS
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

}  // namespace llmq

extern "C" int llmq_rmsnorm_forward_bf16(uint16_t* out, float* rms_or_null, const uint16_t* inp, const uint16_t* weight,
                                         float* abs_max_or_null, float epsilon, int B, int T, int C, void* stream) {
    return llmq::rmsnorm_forward_any("rmsnorm_forward", false, nullptr, out, rms_or_null, inp, nullptr, weight, abs_max_or_null,
                                     epsilon, (int64_t)B * T, C, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_fused_residual_rmsnorm_forward_bf16(uint16_t* residual, uint16_t* normed, float* rrms,
                                                        const uint16_t* inp1, const uint16_t* inp2,
                                                        const uint16_t* weight, float* abs_max_or_null, float epsilon,
                                                        int N, int C, void* stream) {
    return llmq::rmsnorm_forward_any("fused_residual_rmsnorm_forward", true, residual, normed, rrms, inp1, inp2, weight,
                                     abs_max_or_null, epsilon, N, C, static_cast<hipStream_t>(stream));
}
