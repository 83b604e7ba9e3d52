// Shared host/device helpers of the gfx950 FP8 path.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "llmq_fp8.h"

namespace llmq {

// Records a message for llmq_last_error() and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int hip_fail(hipError_t e, const char* what) {
    (void)hipGetLastError();  // clear the sticky error, as the reference's CUDA_CHECK does
    return set_error(LLMQ_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
}

#define LLMQ_HIP_TRY(expr)                                           \
    do {                                                             \
        hipError_t _e = (expr);                                      \
        if (_e != hipSuccess) return ::llmq::hip_fail(_e, #expr);    \
    } while (0)

#define LLMQ_REQUIRE(cond, ...)                                                    \
    do {                                                                           \
        if (!(cond)) return ::llmq::set_error(LLMQ_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Number of compute units of the current device (cached per device id).
int cu_count();
// Number of accelerator dies (XCDs) the device's compute units are spread over; workgroup ids are dealt to them
// round-robin and each has an L2 of its own, which the tile walks are laid out for.
int xcd_count();

constexpr int kWave = 64;

// ---- device helpers -----------------------------------------------------------------------------
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

// Streaming accesses: data read for the last time, or written for a consumer that is not the next kernel, is
// marked non-temporal so that it does not displace what the next kernel re-reads from the 256 MB last-level
// cache (measured: abs-max followed by quantize of a 310 MB tensor goes from 151 to 124 us when the quantizer's
// loads are non-temporal, because the tensor the abs-max just read is still cached).  The fp8 codes the
// quantizers and the byte transpose write are the operands of the matmul that follows: those stores stay
// ordinary, which the matmul repays (about 1.4 % per launch in the bench step, measured by alternating builds).
typedef unsigned int llmq_v4u __attribute__((ext_vector_type(4)));
typedef unsigned int llmq_v2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_nt(const uint4* p) {
    const llmq_v4u t = __builtin_nontemporal_load(reinterpret_cast<const llmq_v4u*>(p));
    return make_uint4(t[0], t[1], t[2], t[3]);
}
__device__ __forceinline__ void store_nt(uint4* p, const uint4& v) {
    const llmq_v4u t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<llmq_v4u*>(p));
}
__device__ __forceinline__ void store_nt(uint2* p, const uint2& v) {
    const llmq_v2u t = {v.x, v.y};
    __builtin_nontemporal_store(t, reinterpret_cast<llmq_v2u*>(p));
}

// scale = 448 / max(absmax, 1e-10) with an IEEE-correct fp32 division (src/kernels/quant.cu:79).
__device__ __forceinline__ float quant_scale(float absmax) {
    float a = (absmax > 1e-10f) ? absmax : 1e-10f;  // fmaxf semantics incl. NaN -> 1e-10
    return __fdiv_rn(448.f, a);
}

// Correctly rounded fp32 square root.  The hardware instruction (what sqrtf / __fsqrt_rn compile to on gfx950) is
// within one ulp but not always the nearest value (probed: sqrt(0x370b7c3f) returns 0x3b3cf75c, the nearest is
// 0x3b3cf75d), and the parity claims of the kernels that use a square root are bit for bit.  The neighbours of the
// hardware result are tested with exact residuals: s is the nearest value iff x - (s - ulp) * s > 0 and
// x - (s + ulp) * s <= 0.
__device__ __forceinline__ float sqrt_rn(float x) {
    float s = __builtin_sqrtf(x);
    if (s > 0.f && s < __builtin_huge_valf()) {
        const float down = __uint_as_float(__float_as_uint(s) - 1u), up = __uint_as_float(__float_as_uint(s) + 1u);
        const float r_down = __builtin_fmaf(-down, s, x), r_up = __builtin_fmaf(-up, s, x);
        if (r_down <= 0.f) s = down;
        if (r_up > 0.f) s = up;
    }
    return s;
}

}  // namespace llmq
