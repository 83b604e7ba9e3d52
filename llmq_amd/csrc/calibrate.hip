// Calibration kernels for measurements (not part of the drop-in surface).
//
//  * llmq_debug_copy_u8: a plain streaming copy whose HBM bytes are known exactly (n read + n
//    written); hardware traffic counters of the real kernels are scaled by what they read for it.
//  * llmq_debug_read_u8 / llmq_debug_fill_u8: the same access pattern with only the reads (folded into one
//    word per lane that is never stored) resp. only the writes: what a read-only stream (abs-max) and a
//    write-only stream sustain, beside the copy's figure for a read + write stream.
//  * llmq_debug_mfma_ceiling: a loop of fp8 matrix instructions on register operands with no memory
//    traffic at all, 8 waves per compute unit.  With constant operands it runs at the nominal clock;
//    with random fp8 operands that change every iteration (what a real K loop feeds the matrix cores)
//    the chip lowers its clock under power, and the rate it sustains is the practical ceiling any fp8
//    GEMM on this part is measured against.  The 16x16x128 instruction moves half the accumulator
//    registers per flop of the 32x32x64 one and sustains a higher rate under that limit.
#include "common.hpp"

namespace llmq {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void copy_calibration_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                               int64_t nvec) {
    const int64_t base = ((int64_t)blockIdx.x * 256 + threadIdx.x);
    const int64_t stride = (int64_t)gridDim.x * 256;
#pragma unroll 4
    for (int u = 0; u < 4; ++u) {
        const int64_t i = base + u * stride;
        if (i < nvec) dst[i] = src[i];
    }
}

__global__ __launch_bounds__(256) void read_calibration_kernel(uint32_t* __restrict__ sink, const uint4* __restrict__ src,
                                                               int64_t nvec) {
    const int64_t base = ((int64_t)blockIdx.x * 256 + threadIdx.x);
    const int64_t stride = (int64_t)gridDim.x * 256;
    uint4 v[4];
#pragma unroll 4
    for (int u = 0; u < 4; ++u) {
        const int64_t i = base + u * stride;
        v[u] = i < nvec ? src[i] : make_uint4(0, 0, 0, 0);
    }
    uint32_t x = 0;
#pragma unroll 4
    for (int u = 0; u < 4; ++u) x |= (v[u].x & v[u].y) ^ (v[u].z & v[u].w);
    if (x == 0xDEADBEEFu) sink[0] = x;   // practically never true (and harmless if it is): keeps the loads alive
}

__global__ __launch_bounds__(256) void fill_calibration_kernel(uint4* __restrict__ dst, int64_t nvec, uint32_t value) {
    const int64_t base = ((int64_t)blockIdx.x * 256 + threadIdx.x);
    const int64_t stride = (int64_t)gridDim.x * 256;
#pragma unroll 4
    for (int u = 0; u < 4; ++u) {
        const int64_t i = base + u * stride;
        if (i < nvec) dst[i] = make_uint4(value, value + (uint32_t)i, value, value);
    }
}

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

// MODE 0: 32x32x64 instruction, constant operands; 1: 32x32x64, random operands that change every
// iteration; 2: 16x16x128, random operands.  All use 128 accumulator registers per lane like a GEMM
// wave tile, 8 waves per workgroup.
template <int MODE>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(float* out, int iters) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    v8i a[2], b[2];
    for (int s = 0; s < 2; ++s)
        for (int i = 0; i < 8; ++i) {
            if (MODE == 0) {
                a[s][i] = 0x38383838;  // 1.0 in every byte
                b[s][i] = 0x38383838;
            } else {
                const uint32_t ra = mix32(threadIdx.x * 64 + i + 17 * s + blockIdx.x * 77777u), rb = mix32(ra + 12345u);
                a[s][i] = ra & 0xBFBFBFBFu;  // bit 6 of every byte cleared: no NaN code, magnitudes below 2
                b[s][i] = rb & 0xBFBFBFBFu;
            }
        }
    float s = 0;
    if constexpr (MODE != 2) {
        v16f acc[8];
        for (int n = 0; n < 8; ++n)
            for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int n = 0; n < 8; ++n)
                acc[n] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[n & 1], b[(n >> 1) & 1], acc[n], 0, 0, 0, 0, 0, 0);
            if (MODE == 1) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    a[0][i] ^= 0x15150a0a;
                    b[1][i] ^= 0x0a0a1515;
                }
            }
        }
        for (int n = 0; n < 8; ++n)
            for (int i = 0; i < 16; ++i) s += acc[n][i];
    } else {
        v4f acc[32];
        for (int n = 0; n < 32; ++n)
            for (int i = 0; i < 4; ++i) acc[n][i] = 0.f;
        for (int it = 0; it < iters; it += 2) {  // two iterations' worth of flop per trip: 32 x 65536
#pragma unroll
            for (int n = 0; n < 32; ++n)
                acc[n] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[n & 1], b[(n >> 1) & 1], acc[n], 0, 0, 0, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[0][i] ^= 0x15150a0a;
                b[1][i] ^= 0x0a0a1515;
            }
        }
        for (int n = 0; n < 32; ++n)
            for (int i = 0; i < 4; ++i) s += acc[n][i];
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace llmq

extern "C" __attribute__((visibility("default"))) int llmq_debug_copy_u8(uint8_t* dst, const uint8_t* src, int64_t n, void* stream) {
    using namespace llmq;
    LLMQ_REQUIRE(dst && src && n > 0 && n % 16 == 0, "copy: need non-null pointers and a positive multiple of 16 bytes");
    LLMQ_REQUIRE(aligned16(dst) && aligned16(src), "copy: pointers must be 16-byte aligned");
    const int64_t nvec = n / 16;
    const int64_t blocks = (nvec + 1023) / 1024;
    LLMQ_REQUIRE(blocks <= 0x7FFFFFFF, "copy: too large");
    hipLaunchKernelGGL(copy_calibration_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<uint4*>(dst), reinterpret_cast<const uint4*>(src), nvec);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// mode 0: read n bytes of src (dst: at least 4 bytes, never written); mode 1: write n bytes of dst (src unused).
extern "C" __attribute__((visibility("default"))) int llmq_debug_stream_u8(uint8_t* dst, const uint8_t* src, int64_t n, int mode, void* stream) {
    using namespace llmq;
    LLMQ_REQUIRE(dst && n > 0 && n % 16 == 0 && (mode == 1 || src), "stream: need non-null pointers and a positive multiple of 16 bytes");
    LLMQ_REQUIRE(aligned16(dst) && aligned16(src) && (mode == 0 || mode == 1), "stream: 16-byte aligned pointers, mode 0 or 1");
    const int64_t nvec = n / 16;
    const int64_t blocks = (nvec + 1023) / 1024;
    LLMQ_REQUIRE(blocks <= 0x7FFFFFFF, "stream: too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == 0) hipLaunchKernelGGL(read_calibration_kernel, dim3((unsigned)blocks), dim3(256), 0, st, reinterpret_cast<uint32_t*>(dst), reinterpret_cast<const uint4*>(src), nvec);
    else hipLaunchKernelGGL(fill_calibration_kernel, dim3((unsigned)blocks), dim3(256), 0, st, reinterpret_cast<uint4*>(dst), nvec, 0x38383838u);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// Launches one ceiling kernel: `blocks` workgroups of 512 lanes, `iters` (even) iterations of
// 8 * 131072 flop per wave (= blocks * 8 * iters * 1048576 flop).  mode: 0 = 32x32x64 instruction with
// constant operands, 1 = 32x32x64 with random operands, 2 = 16x16x128 with random operands.
// scratch: blocks * 512 floats.
extern "C" __attribute__((visibility("default"))) int llmq_debug_mfma_ceiling(float* scratch, int blocks, int iters, int mode, void* stream) {
    using namespace llmq;
    LLMQ_REQUIRE(scratch != nullptr && blocks > 0 && iters > 0 && iters % 2 == 0 && mode >= 0 && mode <= 2,
                 "mfma_ceiling: bad arguments");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == 0) hipLaunchKernelGGL(mfma_ceiling_kernel<0>, dim3((unsigned)blocks), dim3(512), 0, st, scratch, iters);
    else if (mode == 1) hipLaunchKernelGGL(mfma_ceiling_kernel<1>, dim3((unsigned)blocks), dim3(512), 0, st, scratch, iters);
    else hipLaunchKernelGGL(mfma_ceiling_kernel<2>, dim3((unsigned)blocks), dim3(512), 0, st, scratch, iters);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// What the library's launch plans take as the number of accelerator dies and compute units of the current device.
extern "C" __attribute__((visibility("default"))) int llmq_debug_xcd_count(void) { return llmq::xcd_count(); }
extern "C" __attribute__((visibility("default"))) int llmq_debug_cu_count(void) { return llmq::cu_count(); }
