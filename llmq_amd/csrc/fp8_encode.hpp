// fp32 / bf16 -> fp8 code conversion shared by the quantizing kernels (gfx950).
//
// The conversion the reference calls is the CUDA toolkit's saturating round-to-nearest-even one
// (src/kernels/quant.cu:88): NaN -> 0x7F (sign dropped), |y| above the largest finite value (and +-Inf)
// -> +-max, zero and underflow keep their sign.  The gfx950 packed conversion instruction (OCP formats)
// does the rounding; saturation is made explicit with a median-of-three clamp and NaNs are patched in a
// rarely-taken branch, so the bytes do not depend on the instruction's overflow/NaN conventions.
#pragma once

#include "common.hpp"

namespace llmq {

enum Fp8Format { kE4M3 = 0, kE5M2 = 1 };

template <int FMT>
__device__ __forceinline__ float clamp_finite(float y) {
    constexpr float lim = FMT == kE4M3 ? 448.f : 57344.f;
    return __builtin_amdgcn_fmed3f(y, -lim, lim);  // +-Inf and overflow -> +-max finite
}

// Packs fp8(a), fp8(b) into the low (hi == false) or high half of `old`.
template <int FMT>
__device__ __forceinline__ uint32_t cvt_pk(float a, float b, uint32_t old, bool hi) {
    if constexpr (FMT == kE4M3) {
        return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true)
                  : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
    } else {
        return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, true)
                  : (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, false);
    }
}

// Four scaled values -> one dword of four codes (y0 in the lowest byte).
template <int FMT>
__device__ __forceinline__ uint32_t encode4(float y0, float y1, float y2, float y3) {
    uint32_t w = cvt_pk<FMT>(clamp_finite<FMT>(y0), clamp_finite<FMT>(y1), 0u, false);
    w = cvt_pk<FMT>(clamp_finite<FMT>(y2), clamp_finite<FMT>(y3), w, true);
    if (__builtin_expect((y0 != y0) | (y1 != y1) | (y2 != y2) | (y3 != y3), 0)) {
        if (y0 != y0) w = (w & 0xFFFFFF00u) | 0x0000007Fu;
        if (y1 != y1) w = (w & 0xFFFF00FFu) | 0x00007F00u;
        if (y2 != y2) w = (w & 0xFF00FFFFu) | 0x007F0000u;
        if (y3 != y3) w = (w & 0x00FFFFFFu) | 0x7F000000u;
    }
    return w;
}

template <int FMT>
__device__ __forceinline__ uint2 encode8(const uint4& v, float s) {
    uint2 r;
    r.x = encode4<FMT>(s * bf16_lo(v.x), s * bf16_hi(v.x), s * bf16_lo(v.y), s * bf16_hi(v.y));
    r.y = encode4<FMT>(s * bf16_lo(v.z), s * bf16_hi(v.z), s * bf16_lo(v.w), s * bf16_hi(v.w));
    return r;
}

}  // namespace llmq
