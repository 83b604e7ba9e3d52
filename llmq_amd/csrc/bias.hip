// Bias gradient from the quantized output gradient, for gfx950:
//     dbias[oc] = round_bf16( (float)dbias[oc] + (sa*sb) * sum_bt dec(dout[bt, oc]) )
//
// Semantics follow the reference's backward_bias for fp8 / bf16 gradients (src/kernels/bias.cu:40-112,
// 151-195; call site src/models/llama_model.cpp:334-336): the column sums of the row-major
// [B*T, OC] gradient are formed in fp32, multiplied by the product of the two dequantisation scales
// (1 when both are absent) and ADDED to the existing dbias.  The result depends on the summation
// order only through fp32 rounding; this implementation uses a fixed order, so it is deterministic.
//
// Design: HBM-bound streaming read (1 byte per fp8 element, 2 per bf16).  A workgroup owns a band of
// rows and up to 256 column chunks of 16 bytes; each lane keeps the partial sums of its chunk in
// registers while walking its rows (several independent 16-byte loads in flight), the lanes that share
// a chunk are combined through LDS, and the band's partial sums go to the caller's scratch buffer
// [bands][OC].  A second small kernel adds the bands in index order, applies the scale and updates
// dbias.
#include <mutex>

#include "common.hpp"

namespace llmq {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kBiasThreads = 256;

enum { kFmtE4M3 = 0, kFmtE5M2 = 1, kFmtBF16 = 2 };

// adds the values of one 16-byte piece to acc[0 .. elements)
template <int FMT>
__device__ __forceinline__ void accumulate_piece(float* acc, const uint4& v) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if constexpr (FMT == kFmtBF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = acc[2 * i] + __uint_as_float(w[i] << 16);
            acc[2 * i + 1] = acc[2 * i + 1] + __uint_as_float(w[i] & 0xFFFF0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f32x2 lo, hi;
            if constexpr (FMT == kFmtE4M3) {
                lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
                hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
            } else {
                lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[i], false);
                hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[i], true);
            }
            acc[4 * i] = acc[4 * i] + lo[0];
            acc[4 * i + 1] = acc[4 * i + 1] + lo[1];
            acc[4 * i + 2] = acc[4 * i + 2] + hi[0];
            acc[4 * i + 3] = acc[4 * i + 3] + hi[1];
        }
    }
}

// chunks: 16-byte pieces per row; cw: chunks handled by this workgroup column (<= 256); rp = 256 / cw
// lanes share a chunk, each taking every rp-th row of the band.
template <int FMT>
__global__ __launch_bounds__(kBiasThreads) void bias_partial_kernel(float* __restrict__ partial,
                                                                    const uint4* __restrict__ dout, int rows,
                                                                    int chunks, int cw, int rows_per_band, int OC) {
    constexpr int EL = FMT == kFmtBF16 ? 8 : 16;   // elements per 16-byte piece
    constexpr int UNROLL = 4;
    __shared__ float red[kBiasThreads * EL];       // [row lane][chunk lane][element]
    const int rp = kBiasThreads / cw;
    const int cl = threadIdx.x % cw, rl = threadIdx.x / cw;
    const int chunk = blockIdx.x * cw + cl;
    const int r_begin = blockIdx.y * rows_per_band;
    const int r_end = min(rows, r_begin + rows_per_band);
    float acc[EL];
#pragma unroll
    for (int e = 0; e < EL; ++e) acc[e] = 0.f;
    if (rl < rp && chunk < chunks) {
        for (int r = r_begin + rl; r < r_end; r += UNROLL * rp) {
            uint4 v[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int rr = r + u * rp;
                v[u] = rr < r_end ? dout[(int64_t)rr * chunks + chunk] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) accumulate_piece<FMT>(acc, v[u]);
        }
    }
    // element-major LDS layout: consecutive lanes -> consecutive words
#pragma unroll
    for (int e = 0; e < EL; ++e) red[e * kBiasThreads + threadIdx.x] = acc[e];
    __syncthreads();
    // lanes 0 .. cw*EL-1 each finish one (chunk lane, element) column
    for (int o = threadIdx.x; o < cw * EL; o += kBiasThreads) {
        const int c = o / EL, e = o % EL;
        float s = 0.f;
        for (int q = 0; q < rp; ++q) s = s + red[e * kBiasThreads + q * cw + c];
        const int col = (blockIdx.x * cw + c) * EL + e;
        if (col < OC) partial[(int64_t)blockIdx.y * OC + col] = s;
    }
}

// 32 columns x 8 band lanes per workgroup: lane (c, q) adds bands q, q+8, ... in index order, the eight
// lane sums are then added in lane order -- a fixed summation tree.
__global__ __launch_bounds__(256) void bias_finish_kernel(uint16_t* __restrict__ dbias, const float* __restrict__ partial,
                                                          int bands, int OC, const float* sa, const float* sb) {
    __shared__ float red[8][32];
    const int c = threadIdx.x % 32, q = threadIdx.x / 32;
    const int col = blockIdx.x * 32 + c;
    float s = 0.f;
    if (col < OC) {
        int b = q;
        for (; b + 24 < bands; b += 32) {
            const float p0 = partial[(int64_t)b * OC + col], p1 = partial[(int64_t)(b + 8) * OC + col];
            const float p2 = partial[(int64_t)(b + 16) * OC + col], p3 = partial[(int64_t)(b + 24) * OC + col];
            s = s + p0;
            s = s + p1;
            s = s + p2;
            s = s + p3;
        }
        for (; b < bands; b += 8) s = s + partial[(int64_t)b * OC + col];
    }
    red[q][c] = s;
    __syncthreads();
    if (q == 0 && col < OC) {
        float t = red[0][c];
#pragma unroll
        for (int k = 1; k < 8; ++k) t = t + red[k][c];
        float scale = 1.f;
        if (sa != nullptr && sb != nullptr) scale = *sa * *sb;
        t = t * scale + __uint_as_float((uint32_t)dbias[col] << 16);
        const f32x2 v = {t, 0.f};
        const bf16x2 h = __builtin_convertvector(v, bf16x2);   // round to nearest even
        dbias[col] = (uint16_t)(__builtin_bit_cast(uint32_t, h) & 0xFFFFu);
    }
}

// Row bands the launch uses for a given shape (also sizes the scratch buffer).
static int bias_bands(int rows, int chunks) {
    const int cw = chunks < kBiasThreads ? chunks : kBiasThreads;
    const int col_blocks = (chunks + cw - 1) / cw;
    int bands = (2 * cu_count() + col_blocks - 1) / col_blocks;
    const int rp = kBiasThreads / cw;
    const int max_bands = (rows + 4 * rp - 1) / (4 * rp);   // at least one unrolled trip per band
    if (bands > max_bands) bands = max_bands;
    return bands < 1 ? 1 : bands;
}

// Scratch of the entry point that allocates nothing: band sums [bands][OC] as in the caller-provided buffer of
// llmq_backward_bias_bf16.  Every GPU the library runs on holds its own copy of this array at its own address
// until the process ends; host code reaches it only through the address hipGetSymbolAddress returns with that
// GPU current (the array's name is a host-side stand-in, not a device address).
constexpr size_t kStaticBiasScratchBytes = LLMQ_BACKWARD_BIAS_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) float static_bias_scratch[kStaticBiasScratchBytes / sizeof(float)];

// Device address of static_bias_scratch on the current device (looked up once per device), or nullptr with the
// error recorded.
static float* static_bias_scratch_ptr() {
    static float* cached[64];
    static std::mutex mu;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        hip_fail(e, "hipGetDevice");
        return nullptr;
    }
    if (dev < 0 || dev >= 64) {
        set_error(LLMQ_ERR_RUNTIME, "backward_bias: device index %d out of range", dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_bias_scratch));
        if (e != hipSuccess || p == nullptr) {
            hip_fail(e, "hipGetSymbolAddress(static_bias_scratch)");
            return nullptr;
        }
        cached[dev] = static_cast<float*>(p);
    }
    return cached[dev];
}

}  // namespace llmq

extern "C" int64_t llmq_backward_bias_scratch_bytes(int BT, int OC, int dout_format) {
    using namespace llmq;
    if (BT <= 0 || OC <= 0) return 0;
    const int el = dout_format == kFmtBF16 ? 8 : 16;
    return (int64_t)bias_bands(BT, (OC + el - 1) / el) * OC * (int64_t)sizeof(float);
}

extern "C" int llmq_backward_bias_bf16(uint16_t* dbias, const void* dout, int dout_format, const float* sa_or_null,
                                       const float* sb_or_null, float* scratch, size_t scratch_bytes, int BT, int OC,
                                       void* stream) {
    using namespace llmq;
    LLMQ_REQUIRE(dout_format == kFmtE4M3 || dout_format == kFmtE5M2 || dout_format == kFmtBF16,
                 "backward_bias: unknown gradient format %d", dout_format);
    LLMQ_REQUIRE((sa_or_null == nullptr) == (sb_or_null == nullptr),
                 "backward_bias: scale_a and scale_b must be both null or both non-null");
    LLMQ_REQUIRE(BT >= 0 && OC >= 0, "backward_bias: negative shape %d x %d", BT, OC);
    const int el = dout_format == kFmtBF16 ? 8 : 16;
    LLMQ_REQUIRE(OC % el == 0, "backward_bias: OC must be a multiple of the vector size (%d)", el);
    if (BT == 0 || OC == 0) return LLMQ_OK;
    LLMQ_REQUIRE(dbias != nullptr && dout != nullptr && scratch != nullptr, "backward_bias: null pointer");
    LLMQ_REQUIRE(aligned16(dout) && aligned16(scratch), "backward_bias: gradient and scratch must be 16-byte aligned");
    const int chunks = OC / el;
    const int bands = bias_bands(BT, chunks);
    LLMQ_REQUIRE(scratch_bytes >= (size_t)bands * OC * sizeof(float),
                 "backward_bias: scratch buffer too small: expected at least %zu bytes, got %zu",
                 (size_t)bands * OC * sizeof(float), scratch_bytes);
    const int cw = chunks < kBiasThreads ? chunks : kBiasThreads;
    const int col_blocks = (chunks + cw - 1) / cw;
    const int rows_per_band = (BT + bands - 1) / bands;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)col_blocks, (unsigned)bands);
    const uint4* src = reinterpret_cast<const uint4*>(dout);
    if (dout_format == kFmtE4M3) {
        hipLaunchKernelGGL(bias_partial_kernel<kFmtE4M3>, grid, dim3(kBiasThreads), 0, st, scratch, src, BT, chunks, cw,
                           rows_per_band, OC);
    } else if (dout_format == kFmtE5M2) {
        hipLaunchKernelGGL(bias_partial_kernel<kFmtE5M2>, grid, dim3(kBiasThreads), 0, st, scratch, src, BT, chunks, cw,
                           rows_per_band, OC);
    } else {
        hipLaunchKernelGGL(bias_partial_kernel<kFmtBF16>, grid, dim3(kBiasThreads), 0, st, scratch, src, BT, chunks, cw,
                           rows_per_band, OC);
    }
    LLMQ_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(bias_finish_kernel, dim3((unsigned)((OC + 31) / 32)), dim3(256), 0, st, dbias, scratch, bands, OC,
                       sa_or_null, sb_or_null);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

extern "C" int llmq_backward_bias_bf16_static_scratch(uint16_t* dbias, const void* dout, int dout_format,
                                                      const float* sa_or_null, const float* sb_or_null, int BT, int OC,
                                                      void* stream) {
    using namespace llmq;
    const int64_t need = llmq_backward_bias_scratch_bytes(BT, OC, dout_format);
    LLMQ_REQUIRE(need <= (int64_t)kStaticBiasScratchBytes,
                 "backward_bias (static scratch): [%d x %d] needs %lld bytes of band sums, the built-in scratch holds %zu; "
                 "use llmq_backward_bias_bf16 with a caller-provided buffer",
                 BT, OC, (long long)need, kStaticBiasScratchBytes);
    float* scratch = static_bias_scratch_ptr();
    if (scratch == nullptr) return LLMQ_ERR_RUNTIME;
    return llmq_backward_bias_bf16(dbias, dout, dout_format, sa_or_null, sb_or_null, scratch, kStaticBiasScratchBytes, BT,
                                   OC, stream);
}
