// Scaled bf16 -> fp8 quantization (plain and with fused transpose) for gfx950.
//
// Semantics follow the reference's quantize_with_abs_max_kernel (src/kernels/quant.cu:73-93) and
// quantize_and_transpose_with_abs_max_kernel (src/kernels/quant.cu:151-164):
//   scale = 448.f / fmaxf(*abs_max, 1e-10f);  out = fp8_rn_satfinite(scale * (float)in);
//   *scale_ptr = 1.f / scale  (written by one lane when the pointer is non-null).
// The conversion the reference calls is the CUDA toolkit's saturating round-to-nearest-even one:
// NaN -> 0x7F (sign dropped), |y| above the largest finite value (and +-Inf) -> +-max, zero and
// underflow keep their sign.  Here the gfx950 packed conversion instruction (OCP formats) does the
// rounding; saturation is made explicit with a median-of-three clamp and NaNs are patched in a
// rarely-taken branch, so the bytes do not depend on the instruction's overflow/NaN conventions.
//
// Both kernels are HBM bound (2 bytes read + 1 byte written per element): every global access is a
// 128-bit (or 64-bit for the plain kernel's stores) per-lane access that is contiguous across the
// wave; the transposing kernel stages a [64 or 128 cols] x [256 rows] tile of fp8 codes in LDS
// (row stride 65 dwords: conflict-free for both the dword writes and the dword reads) so that the
// stores along the transposed rows are 256-byte contiguous per 16 lanes.
#include <type_traits>

#include "common.hpp"
#include "fp8_encode.hpp"

namespace llmq {

// One trip per lane: UNROLL independent 16-byte loads, then UNROLL 8-byte stores.  A workgroup owns a contiguous
// piece of 256 * UNROLL vectors (lane t takes vectors t, t + 256, ...).  Many small workgroups with two loads
// per lane sustain the most HBM bandwidth on tensors no cache holds (310 MB source, rotating buffers:
// UNROLL 8 / 4 / 2 = 5.44 / 5.69 / 5.89 TB/s; a plain copy kernel gets 5.7), hence UNROLL = 2 below.
constexpr int kQuantizeUnroll = 2;

template <int FMT, int UNROLL>
__global__ __launch_bounds__(256) void quantize_kernel(uint2* __restrict__ out, float* __restrict__ scale_ptr,
                                                       const uint4* __restrict__ in,
                                                       const float* __restrict__ absmax, int64_t nvec,
                                                       const uint16_t* __restrict__ tail_in,
                                                       uint8_t* __restrict__ tail_out, int ntail) {
    const float s = quant_scale(*absmax);
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid == 0 && scale_ptr) *scale_ptr = __fdiv_rn(1.f, s);
    const int64_t first = (int64_t)blockIdx.x * (256 * UNROLL) + threadIdx.x;
    uint4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t idx = first + u * 256;
        v[u] = idx < nvec ? load_nt(&in[idx]) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t idx = first + u * 256;
        if (idx < nvec) out[idx] = encode8<FMT>(v[u], s);
    }
    if (tid < ntail) {
        float y = s * __uint_as_float((uint32_t)tail_in[tid] << 16);
        tail_out[tid] = (uint8_t)(encode4<FMT>(y, 0.f, 0.f, 0.f) & 0xFFu);
    }
}

// fp32 input (master weights / activations of an fp32 model): 4 bytes read + 1 written per element.
// Each lane converts 4 values per access (16-byte load, 4-byte store), UNROLL accesses in flight, a workgroup
// owning a contiguous piece of 256 * UNROLL vectors, as in the bf16 kernel above.
template <int FMT, int UNROLL>
__global__ __launch_bounds__(256) void quantize_f32_kernel(uint32_t* __restrict__ out, float* __restrict__ scale_ptr,
                                                           const uint4* __restrict__ in,
                                                           const float* __restrict__ absmax, int64_t nvec,
                                                           const float* __restrict__ tail_in,
                                                           uint8_t* __restrict__ tail_out, int ntail) {
    const float s = quant_scale(*absmax);
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid == 0 && scale_ptr) *scale_ptr = __fdiv_rn(1.f, s);
    const int64_t first = (int64_t)blockIdx.x * (256 * UNROLL) + threadIdx.x;
    uint4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t idx = first + u * 256;
        v[u] = idx < nvec ? load_nt(&in[idx]) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t idx = first + u * 256;
        if (idx < nvec)
            out[idx] = encode4<FMT>(s * __uint_as_float(v[u].x), s * __uint_as_float(v[u].y), s * __uint_as_float(v[u].z),
                                    s * __uint_as_float(v[u].w));
    }
    if (tid < ntail) tail_out[tid] = (uint8_t)(encode4<FMT>(s * tail_in[tid], 0.f, 0.f, 0.f) & 0xFFu);
}

// ---- quantize + transpose -------------------------------------------------------------------------
constexpr int kQtRows = 256;       // tile extent along the input rows (= contiguous bytes of the output)
constexpr int kQtStride = 65;      // LDS row stride in dwords (64 dwords of payload + 1 pad)

// NCH = number of 8-column chunks per tile: the tile is [kQtRows rows] x [8*NCH cols].
// BOTH: the untransposed codes are written as well (out_plain[r*cols + c]), from the same single read of
// the input: 8 bytes per lane and row, 8*NCH contiguous bytes per row segment.
// InT: uint16_t (bf16 patterns) or float (the fp32-input overload, src/kernels/quant.cu:135-149; not with BOTH).
template <int FMT, int NCH, bool ROW_MAJOR_GRID, bool BOTH, typename InT = uint16_t>
__global__ __launch_bounds__(256) void quantize_transpose_kernel(uint8_t* __restrict__ out,
                                                                 uint8_t* __restrict__ out_plain,
                                                                 float* __restrict__ scale_ptr,
                                                                 const InT* __restrict__ in,
                                                                 const float* __restrict__ absmax, int rows,
                                                                 int cols, int rows_mult16) {
    constexpr int TC = 8 * NCH;
    constexpr int QPP = 256 / NCH;            // row quads per pass
    constexpr int PASSES = (kQtRows / 4) / QPP;
    __shared__ uint32_t tile[TC * kQtStride];

    const float s = quant_scale(*absmax);
    const int t = threadIdx.x;
    if (t == 0 && blockIdx.x == 0 && blockIdx.y == 0 && scale_ptr) *scale_ptr = __fdiv_rn(1.f, s);

    const int r0 = (ROW_MAJOR_GRID ? blockIdx.x : blockIdx.y) * kQtRows;
    const int c0 = (ROW_MAJOR_GRID ? blockIdx.y : blockIdx.x) * TC;
    const int chunk = t % NCH;
    const int q = t / NCH;
    const int col = c0 + 8 * chunk;
    // LDS has 64 banks of 4 bytes and the row stride is 65 dwords: the dword written by lane (chunk, q) lands on bank
    // 8 chunk + q + const (mod 64).  With 16 chunks per wave row, chunks c and c + 8 would share banks (a two-way
    // conflict on every write); flipping bit 2 of the row-quad index for the upper eight chunks gives them the other
    // half of each group of eight banks.  The reads below undo it (a group of four consecutive row quads stays a group
    // of four).  Measured: the conflict counter goes from 0.67 to 0.50 of the LDS cycles (the rest are the four-dword
    // reads, which take two passes by themselves); the kernel's rate does not change, it is bound by its global
    // access pattern.
    constexpr int SWZ = NCH == 16 ? 4 : 0;
    const int wr_flip = (chunk >> 3) * SWZ;

    constexpr bool F32 = std::is_same_v<InT, float>;
    static_assert(!(F32 && BOTH), "the plain + transposed variant takes bf16 input");
    if constexpr (F32) {
        // 8 columns of a row are two 16-byte pieces; one pass of 4 rows at a time keeps the registers modest
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int rq = q + QPP * p;
            uint4 lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int row = r0 + 4 * rq + j;
                if (row < rows && col < cols) {
                    const uint4* src = reinterpret_cast<const uint4*>(in + (int64_t)row * cols + col);
                    lo[j] = load_nt(src);
                    hi[j] = load_nt(src + 1);
                } else {
                    lo[j] = hi[j] = make_uint4(0, 0, 0, 0);
                }
            }
            auto val = [&](int j, int c) -> float {  // column c (0..7) of row j
                const uint4& w = c < 4 ? lo[j] : hi[j];
                const uint32_t bits = (c & 3) == 0 ? w.x : (c & 3) == 1 ? w.y : (c & 3) == 2 ? w.z : w.w;
                return __uint_as_float(bits);
            };
#pragma unroll
            for (int c = 0; c < 8; ++c)
                tile[(8 * chunk + c) * kQtStride + (rq ^ wr_flip)] = encode4<FMT>(s * val(0, c), s * val(1, c), s * val(2, c), s * val(3, c));
        }
    }
    uint4 v[F32 ? 1 : PASSES][4];
    if constexpr (!F32) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int rq = q + QPP * p;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = r0 + 4 * rq + j;
            if (row < rows && col < cols) {
                v[p][j] = load_nt(reinterpret_cast<const uint4*>(in + (int64_t)row * cols + col));
            } else {
                v[p][j] = make_uint4(0, 0, 0, 0);
            }
        }
    }
    }
#pragma unroll
    for (int p = 0; p < (F32 ? 0 : PASSES); ++p) {
        const int rq = q + QPP * p;
        const uint32_t w[4][4] = {{v[p][0].x, v[p][0].y, v[p][0].z, v[p][0].w},
                                  {v[p][1].x, v[p][1].y, v[p][1].z, v[p][1].w},
                                  {v[p][2].x, v[p][2].y, v[p][2].z, v[p][2].w},
                                  {v[p][3].x, v[p][3].y, v[p][3].z, v[p][3].w}};
#pragma unroll
        for (int k = 0; k < 4; ++k) {  // word k holds columns 2k (low half) and 2k+1 (high half)
            const uint32_t even = encode4<FMT>(s * bf16_lo(w[0][k]), s * bf16_lo(w[1][k]),
                                               s * bf16_lo(w[2][k]), s * bf16_lo(w[3][k]));
            const uint32_t odd = encode4<FMT>(s * bf16_hi(w[0][k]), s * bf16_hi(w[1][k]),
                                              s * bf16_hi(w[2][k]), s * bf16_hi(w[3][k]));
            tile[(8 * chunk + 2 * k) * kQtStride + (rq ^ wr_flip)] = even;
            tile[(8 * chunk + 2 * k + 1) * kQtStride + (rq ^ wr_flip)] = odd;
        }
        if constexpr (BOTH) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int row = r0 + 4 * rq + j;
                if (row < rows && col < cols)
                    *reinterpret_cast<uint2*>(out_plain + (int64_t)row * cols + col) = encode8<FMT>(v[p][j], s);
            }
        }
    }
    __syncthreads();

    constexpr int ITEMS = TC * (kQtRows / 16);  // 16-byte pieces in the tile
#pragma unroll
    for (int it = 0; it < ITEMS / 256; ++it) {
        const int item = t + 256 * it;
        const int c = item / 16, p = item % 16;
        const int r = r0 + 16 * p;
        if (c0 + c < cols && r < rows) {
            const uint32_t* src = &tile[c * kQtStride + 4 * (p ^ ((c >> 6) * (SWZ / 4)))];
            uint8_t* dst = out + (int64_t)(c0 + c) * rows + r;
            if (rows_mult16) {
                *reinterpret_cast<uint4*>(dst) = make_uint4(src[0], src[1], src[2], src[3]);
            } else {
                *reinterpret_cast<uint2*>(dst) = make_uint2(src[0], src[1]);
                if (r + 8 < rows) *reinterpret_cast<uint2*>(dst + 8) = make_uint2(src[2], src[3]);
            }
        }
    }
}

template <int FMT>
static int launch_quantize(uint8_t* out, float* scale_ptr, const uint16_t* in, const float* absmax, int64_t n,
                           hipStream_t stream) {
    LLMQ_REQUIRE(n >= 0, "quantize_with_abs_max: negative element count %lld", (long long)n);
    LLMQ_REQUIRE(absmax != nullptr, "quantize_with_abs_max: abs_max pointer is null");
    LLMQ_REQUIRE(n == 0 || (out != nullptr && in != nullptr), "quantize_with_abs_max: null tensor pointer");
    LLMQ_REQUIRE(aligned16(in) && aligned16(out), "quantize_with_abs_max: tensors must be 16-byte aligned");
    const int64_t nvec = n / 8;
    const int ntail = (int)(n - nvec * 8);
    auto launch = [&](auto kernel, int unroll) -> int {
        int64_t blocks = (nvec + 256 * unroll - 1) / (256 * unroll);
        LLMQ_REQUIRE(blocks <= 0x7FFFFFFF, "quantize_with_abs_max: %lld elements are too many", (long long)n);
        if (blocks < 1) blocks = 1;  // still writes the scale for n == 0
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<uint2*>(out), scale_ptr,
                           reinterpret_cast<const uint4*>(in), absmax, nvec, in + nvec * 8, out + nvec * 8, ntail);
        return LLMQ_OK;
    };
    const int rc = launch(quantize_kernel<FMT, kQuantizeUnroll>, kQuantizeUnroll);
    if (rc != LLMQ_OK) return rc;
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

}  // namespace llmq

namespace llmq {
template <int FMT>
static int launch_quantize_f32(uint8_t* out, float* scale_ptr, const float* in, const float* absmax, int64_t n,
                               hipStream_t stream) {
    LLMQ_REQUIRE(n >= 0, "quantize_with_abs_max: negative element count %lld", (long long)n);
    LLMQ_REQUIRE(absmax != nullptr, "quantize_with_abs_max: abs_max pointer is null");
    LLMQ_REQUIRE(n == 0 || (out != nullptr && in != nullptr), "quantize_with_abs_max: null tensor pointer");
    LLMQ_REQUIRE(aligned16(in) && aligned16(out), "quantize_with_abs_max: tensors must be 16-byte aligned");
    const int64_t nvec = n / 4;
    const int ntail = (int)(n - nvec * 4);
    auto launch = [&](auto kernel, int unroll) -> int {
        int64_t blocks = (nvec + 256 * unroll - 1) / (256 * unroll);
        LLMQ_REQUIRE(blocks <= 0x7FFFFFFF, "quantize_with_abs_max: %lld elements are too many", (long long)n);
        if (blocks < 1) blocks = 1;  // still writes the scale for n == 0
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(out), scale_ptr,
                           reinterpret_cast<const uint4*>(in), absmax, nvec, in + nvec * 4, out + nvec * 4, ntail);
        return LLMQ_OK;
    };
    const int rc = launch(quantize_f32_kernel<FMT, kQuantizeUnroll>, kQuantizeUnroll);
    if (rc != LLMQ_OK) return rc;
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}
}  // namespace llmq

extern "C" int llmq_quantize_e4m3_f32(uint8_t* out, float* scale_or_null, const float* in, const float* absmax,
                                      int64_t n, void* stream) {
    return llmq::launch_quantize_f32<llmq::kE4M3>(out, scale_or_null, in, absmax, n, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_quantize_e5m2_f32(uint8_t* out, float* scale_or_null, const float* in, const float* absmax,
                                      int64_t n, void* stream) {
    return llmq::launch_quantize_f32<llmq::kE5M2>(out, scale_or_null, in, absmax, n, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_quantize_e4m3_bf16(uint8_t* out, float* scale_or_null, const uint16_t* in,
                                       const float* absmax, int64_t n, void* stream) {
    return llmq::launch_quantize<llmq::kE4M3>(out, scale_or_null, in, absmax, n, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_quantize_e5m2_bf16(uint8_t* out, float* scale_or_null, const uint16_t* in,
                                       const float* absmax, int64_t n, void* stream) {
    return llmq::launch_quantize<llmq::kE5M2>(out, scale_or_null, in, absmax, n, static_cast<hipStream_t>(stream));
}

namespace llmq {

template <int FMT, bool BOTH, typename InT = uint16_t>
static int launch_quantize_transpose(uint8_t* out, uint8_t* out_plain, float* scale_or_null, const InT* in,
                                     const float* absmax, int rows, int cols, hipStream_t st) {
    LLMQ_REQUIRE(rows >= 0 && cols >= 0, "quantize_and_transpose_with_abs_max: negative shape %d x %d", rows, cols);
    LLMQ_REQUIRE(rows % 8 == 0 && cols % 8 == 0,
                 "quantize_and_transpose_with_abs_max: rows (%d) and cols (%d) must be multiples of 8", rows, cols);
    LLMQ_REQUIRE(absmax != nullptr, "quantize_and_transpose_with_abs_max: abs_max pointer is null");
    const bool empty = rows == 0 || cols == 0;
    LLMQ_REQUIRE(empty || (out != nullptr && in != nullptr && (!BOTH || out_plain != nullptr)),
                 "quantize_and_transpose_with_abs_max: null tensor pointer");
    LLMQ_REQUIRE(aligned16(in) && aligned16(out) && aligned16(out_plain),
                 "quantize_and_transpose_with_abs_max: tensors must be 16-byte aligned");
    const int rows_mult16 = rows % 16 == 0;
    const unsigned gy = empty ? 1u : (unsigned)((rows + kQtRows - 1) / kQtRows);
    // Wide tiles (256-byte row segments on the read side) once there are enough of them to fill the chip.
    const int64_t wide_tiles = (int64_t)((cols + 127) / 128) * gy;
    const bool rm = true;  // workgroups walk along the input rows (see the kernel); the other order serves grids beyond 65535
    const int r = empty ? 0 : rows, c = empty ? 0 : cols;
    if (!empty && cols >= 128 && wide_tiles >= 2LL * cu_count()) {
        const unsigned gx = (unsigned)((cols + 127) / 128);
        if (rm && gx <= 65535u)
            hipLaunchKernelGGL((quantize_transpose_kernel<FMT, 16, true, BOTH, InT>), dim3(gy, gx), dim3(256), 0, st, out,
                               out_plain, scale_or_null, in, absmax, r, c, rows_mult16);
        else
            hipLaunchKernelGGL((quantize_transpose_kernel<FMT, 16, false, BOTH, InT>), dim3(gx, gy), dim3(256), 0, st, out,
                               out_plain, scale_or_null, in, absmax, r, c, rows_mult16);
    } else {
        const unsigned gx = empty ? 1u : (unsigned)((cols + 63) / 64);
        if (rm && gx <= 65535u)
            hipLaunchKernelGGL((quantize_transpose_kernel<FMT, 8, true, BOTH, InT>), dim3(gy, gx), dim3(256), 0, st, out,
                               out_plain, scale_or_null, in, absmax, r, c, rows_mult16);
        else
            hipLaunchKernelGGL((quantize_transpose_kernel<FMT, 8, false, BOTH, InT>), dim3(gx, gy), dim3(256), 0, st, out,
                               out_plain, scale_or_null, in, absmax, r, c, rows_mult16);
    }
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

}  // namespace llmq

extern "C" int llmq_quantize_transpose_e4m3_bf16(uint8_t* out, float* scale_or_null, const uint16_t* in,
                                                 const float* absmax, int rows, int cols, void* stream) {
    return llmq::launch_quantize_transpose<llmq::kE4M3, false>(out, nullptr, scale_or_null, in, absmax, rows, cols,
                                                               static_cast<hipStream_t>(stream));
}

extern "C" int llmq_quantize_transpose_e4m3_f32(uint8_t* out, float* scale_or_null, const float* in, const float* absmax,
                                                int rows, int cols, void* stream) {
    return llmq::launch_quantize_transpose<llmq::kE4M3, false, float>(out, nullptr, scale_or_null, in, absmax, rows, cols,
                                                                      static_cast<hipStream_t>(stream));
}

extern "C" int llmq_quantize_both_bf16(uint8_t* out, uint8_t* out_transposed, float* scale_or_null, const uint16_t* in,
                                       const float* absmax, int rows, int cols, int format, void* stream) {
    using namespace llmq;
    LLMQ_REQUIRE(format == kE4M3 || format == kE5M2, "quantize (plain + transposed): unknown fp8 format %d", format);
    LLMQ_REQUIRE(out != out_transposed || out == nullptr, "quantize (plain + transposed): outputs must be distinct");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (format == kE4M3)
        return launch_quantize_transpose<kE4M3, true>(out_transposed, out, scale_or_null, in, absmax, rows, cols, st);
    return launch_quantize_transpose<kE5M2, true>(out_transposed, out, scale_or_null, in, absmax, rows, cols, st);
}
