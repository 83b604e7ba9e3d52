// llmq_kernels.hpp -- C++20 host shim over the C ABI (llmq_fp8.h) that keeps the names, argument
// order and error behaviour of the reference's kernel entry points for the FP8 quantized-matmul path
// (reference: src/kernels/kernels.h:22-23, 72-98, 246-270; Tensor overloads src/kernels/kernels.cpp:
// 224-236, 258-310, 332-374).  A caller written against the reference's kernels.h compiles against this
// header after the type substitutions
//     nv_bfloat16 -> __hip_bfloat16        __nv_fp8_e4m3 -> __hip_fp8_e4m3     __nv_fp8_e5m2 -> __hip_fp8_e5m2
//     cudaStream_t -> hipStream_t          cudaDeviceProp -> hipDeviceProp_t   cublasLtHandle_t -> llmqBlasHandle_t
// The device-property and handle arguments are accepted and ignored.  The matmul workspace is passed
// through: the gfx950 GEMM keeps raw fp32 partial tiles there when it splits K (outputs with too few tiles to fill the
// chip) and when it cuts a last, partial round of tiles into K segments (all operand modes); it works without one.  Errors surface as the reference's exception types:
// std::invalid_argument for shape / dtype / argument errors, std::runtime_error for runtime failures.
#ifndef LLMQ_KERNELS_HPP
#define LLMQ_KERNELS_HPP

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_fp8.h>
#include <hip/hip_runtime_api.h>

#include <array>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "llmq_fp8.h"

// ---- boundary types (reference: src/utilities/dtype.h:16-71, src/utilities/tensor.h:23-132) ----------
enum class ETensorDType : int { FP32, BF16, FP16, INT32, INT8, FP8_E4M3, FP8_E5M2, BYTE };

constexpr int get_dtype_size(ETensorDType t) {
    switch (t) {
        case ETensorDType::FP32: case ETensorDType::INT32: return 4;
        case ETensorDType::BF16: case ETensorDType::FP16: return 2;
        default: return 1;
    }
}

inline const char* dtype_to_str(ETensorDType t) {
    switch (t) {
        case ETensorDType::FP32: return "FP32";
        case ETensorDType::BF16: return "BF16";
        case ETensorDType::FP16: return "FP16";
        case ETensorDType::INT32: return "INT32";
        case ETensorDType::INT8: return "INT8";
        case ETensorDType::FP8_E4M3: return "FP8_E4M3";
        case ETensorDType::FP8_E5M2: return "FP8_E5M2";
        default: return "BYTE";
    }
}

template <class T> constexpr ETensorDType dtype_from_type = ETensorDType::BYTE;
template <> inline constexpr ETensorDType dtype_from_type<float> = ETensorDType::FP32;
template <> inline constexpr ETensorDType dtype_from_type<__hip_bfloat16> = ETensorDType::BF16;
template <> inline constexpr ETensorDType dtype_from_type<__hip_fp8_e4m3> = ETensorDType::FP8_E4M3;
template <> inline constexpr ETensorDType dtype_from_type<__hip_fp8_e5m2> = ETensorDType::FP8_E5M2;
template <> inline constexpr ETensorDType dtype_from_type<std::int8_t> = ETensorDType::INT8;
template <> inline constexpr ETensorDType dtype_from_type<std::int32_t> = ETensorDType::INT32;

constexpr int MAX_TENSOR_DIM = 5;

// A contiguous typed view of device memory; Stats points at two consecutive device floats
// [abs_max, scale] when the tensor takes part in quantization.
struct Tensor {
    ETensorDType DType = ETensorDType::BYTE;
    std::array<long, MAX_TENSOR_DIM> Sizes{};
    std::byte* Data = nullptr;
    float* Stats = nullptr;
    int Rank = 0;
    int Device = -1;

    [[nodiscard]] constexpr bool empty() const { return Data == nullptr; }
    [[nodiscard]] constexpr std::size_t nelem() const {
        std::size_t sz = 1;
        for (int i = 0; i < Rank; ++i) sz *= (std::size_t)Sizes[i];
        return sz;
    }
    [[nodiscard]] constexpr std::size_t bytes() const { return nelem() * (std::size_t)get_dtype_size(DType); }
    constexpr explicit operator bool() const { return !empty(); }

    template <class T> T* get() {
        check<T>();
        return reinterpret_cast<T*>(Data);
    }
    template <class T> const T* get() const {
        check<T>();
        return reinterpret_cast<const T*>(Data);
    }
    template <class T> const T* get_optional() const { return empty() ? nullptr : get<T>(); }

    float* abs_max() { return Stats; }
    float* scale() { return Stats ? Stats + 1 : nullptr; }
    const float* abs_max() const { return Stats; }
    const float* scale() const { return Stats ? Stats + 1 : nullptr; }

    template <typename Container>
    static Tensor from_pointer(std::byte* ptr, int device, ETensorDType dtype, const Container& shape) {
        if (shape.size() > (std::size_t)MAX_TENSOR_DIM) throw std::runtime_error("Tensor rank too large");
        Tensor t;
        t.DType = dtype;
        t.Sizes.fill(1);
        std::size_t i = 0;
        for (auto s : shape) t.Sizes[i++] = (long)s;
        t.Data = ptr;
        t.Rank = (int)shape.size();
        t.Device = device;
        return t;
    }

  private:
    template <class T> void check() const {
        if constexpr (!std::is_same_v<T, std::byte>) {
            if (dtype_from_type<T> != DType)
                throw std::logic_error(std::string("DType mismatch: requested ") + dtype_to_str(dtype_from_type<T>) +
                                       ", tensor is " + dtype_to_str(DType));
        }
    }
};

struct QuantizableTensor {  // reference: src/models/llama_run_state.h:19-24
    Tensor Value;
    Tensor Quant = Tensor{};
};

enum class EMMTranspose { TT, TN, NT, NN };
enum class EMatmulBackend { CuBLAS, Custom };
typedef struct llmqBlasContext* llmqBlasHandle_t;  // stands in for cublasLtHandle_t; always ignored

namespace llmq_detail {
inline void check(int code) {
    if (code == LLMQ_OK) return;
    if (code == LLMQ_ERR_INVALID_ARGUMENT) throw std::invalid_argument(llmq_last_error());
    throw std::runtime_error(llmq_last_error());
}
inline void require_tn(EMMTranspose mode) {
    if (mode != EMMTranspose::TN)
        throw std::invalid_argument("matmul: FP8 operands are only supported in TN layout (both K-contiguous)");
}
// TN, and the K-major modes TT / NN / NT (restricted shapes, see llmq_gemm_e4m3_bf16_mode)
inline int mode_code(EMMTranspose mode) {
    switch (mode) {
        case EMMTranspose::TN: return LLMQ_MODE_TN;
        case EMMTranspose::TT: return LLMQ_MODE_TT;
        case EMMTranspose::NT: return LLMQ_MODE_NT;
        case EMMTranspose::NN: return LLMQ_MODE_NN;
    }
    throw std::invalid_argument("matmul: unknown operand mode");
}
template <class... T> [[noreturn]] void unsupported(const char* func, const T&... t) {
    std::string msg = std::string(func) + ": unsupported dtypes. Got [";
    ((msg += (t.empty() ? std::string("<null>") : std::string(dtype_to_str(t.DType))) + ", "), ...);
    throw std::invalid_argument(msg + "]");
}
inline const uint16_t* u16(const __hip_bfloat16* p) { return reinterpret_cast<const uint16_t*>(p); }
inline uint16_t* u16(__hip_bfloat16* p) { return reinterpret_cast<uint16_t*>(p); }
template <class F8> const uint8_t* u8(const F8* p) { return reinterpret_cast<const uint8_t*>(p); }
template <class F8> uint8_t* u8(F8* p) { return reinterpret_cast<uint8_t*>(p); }
}  // namespace llmq_detail

// ---- quantization (reference: src/kernels/kernels.h:246-264) -----------------------------------------
inline void abs_max(float* scale, const float* in, long N, const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_abs_max_f32(scale, in, N, stream));
}
inline void abs_max(float* scale, const __hip_bfloat16* in, long N, const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_abs_max_bf16(scale, llmq_detail::u16(in), N, stream));
}
inline void abs_max(float* scale, const Tensor& in, long N, const hipDeviceProp_t& dp, hipStream_t stream) {
    if (in.DType == ETensorDType::FP32) abs_max(scale, in.get<float>(), N, dp, stream);
    else if (in.DType == ETensorDType::BF16) abs_max(scale, in.get<__hip_bfloat16>(), N, dp, stream);
    else llmq_detail::unsupported(__func__, in);
}

inline void quantize_with_abs_max(__hip_fp8_e4m3* out, float* scale_ptr, const __hip_bfloat16* in, const float* abs_max,
                                  long N, const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_quantize_e4m3_bf16(llmq_detail::u8(out), scale_ptr, llmq_detail::u16(in), abs_max, N, stream));
}
inline void quantize_with_abs_max(__hip_fp8_e5m2* out, float* scale_ptr, const __hip_bfloat16* in, const float* abs_max,
                                  long N, const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_quantize_e5m2_bf16(llmq_detail::u8(out), scale_ptr, llmq_detail::u16(in), abs_max, N, stream));
}
inline void quantize_with_abs_max(__hip_fp8_e4m3* out, float* scale_ptr, const float* in, const float* abs_max, long N,
                                  const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_quantize_e4m3_f32(llmq_detail::u8(out), scale_ptr, in, abs_max, N, stream));
}
inline void quantize_with_abs_max(__hip_fp8_e5m2* out, float* scale_ptr, const float* in, const float* abs_max, long N,
                                  const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_quantize_e5m2_f32(llmq_detail::u8(out), scale_ptr, in, abs_max, N, stream));
}
inline void quantize_with_abs_max(Tensor& out, float* scale_ptr, const Tensor& in, const float* abs_max, long N,
                                  const hipDeviceProp_t& dp, hipStream_t stream) {
    if (in.DType == ETensorDType::FP32 && out.DType == ETensorDType::FP8_E4M3)
        quantize_with_abs_max(out.get<__hip_fp8_e4m3>(), scale_ptr, in.get<float>(), abs_max, N, dp, stream);
    else if (in.DType == ETensorDType::FP32 && out.DType == ETensorDType::FP8_E5M2)
        quantize_with_abs_max(out.get<__hip_fp8_e5m2>(), scale_ptr, in.get<float>(), abs_max, N, dp, stream);
    else if (in.DType == ETensorDType::BF16 && out.DType == ETensorDType::FP8_E4M3)
        quantize_with_abs_max(out.get<__hip_fp8_e4m3>(), scale_ptr, in.get<__hip_bfloat16>(), abs_max, N, dp, stream);
    else if (in.DType == ETensorDType::BF16 && out.DType == ETensorDType::FP8_E5M2)
        quantize_with_abs_max(out.get<__hip_fp8_e5m2>(), scale_ptr, in.get<__hip_bfloat16>(), abs_max, N, dp, stream);
    else llmq_detail::unsupported(__func__, out, in);
}

inline void quantize_and_transpose_with_abs_max(__hip_fp8_e4m3* out, float* scale_ptr, const __hip_bfloat16* in,
                                                const float* abs_max, int rows, int cols, const hipDeviceProp_t&,
                                                hipStream_t stream) {
    llmq_detail::check(llmq_quantize_transpose_e4m3_bf16(llmq_detail::u8(out), scale_ptr, llmq_detail::u16(in), abs_max,
                                                         rows, cols, stream));
}
// fp32 input (src/kernels/kernels.h:261)
inline void quantize_and_transpose_with_abs_max(__hip_fp8_e4m3* out, float* scale_ptr, const float* in, const float* abs_max,
                                                int rows, int cols, const hipDeviceProp_t&, hipStream_t stream) {
    llmq_detail::check(llmq_quantize_transpose_e4m3_f32(llmq_detail::u8(out), scale_ptr, in, abs_max, rows, cols, stream));
}
inline void quantize_and_transpose_with_abs_max(Tensor& out, float* scale_ptr, const Tensor& in, const float* abs_max,
                                                int rows, int cols, const hipDeviceProp_t& dp, hipStream_t stream) {
    if (out.DType == ETensorDType::FP8_E4M3 && in.DType == ETensorDType::BF16)
        quantize_and_transpose_with_abs_max(out.get<__hip_fp8_e4m3>(), scale_ptr, in.get<__hip_bfloat16>(), abs_max, rows,
                                            cols, dp, stream);
    else if (out.DType == ETensorDType::FP8_E4M3 && in.DType == ETensorDType::FP32)
        quantize_and_transpose_with_abs_max(out.get<__hip_fp8_e4m3>(), scale_ptr, in.get<float>(), abs_max, rows, cols, dp,
                                            stream);
    else llmq_detail::unsupported(__func__, out, in);
}

// ---- transpose (reference: src/kernels/kernels.h:266-270) --------------------------------------------
inline void transpose(__hip_fp8_e4m3* dst, const __hip_fp8_e4m3* src, int rows, int cols, hipStream_t stream) {
    llmq_detail::check(llmq_transpose_u8(llmq_detail::u8(dst), llmq_detail::u8(src), rows, cols, stream));
}
inline void transpose(__hip_fp8_e5m2* dst, const __hip_fp8_e5m2* src, int rows, int cols, hipStream_t stream) {
    llmq_detail::check(llmq_transpose_u8(llmq_detail::u8(dst), llmq_detail::u8(src), rows, cols, stream));
}
inline void transpose(Tensor& dst, const Tensor& src, int rows, int cols, hipStream_t stream) {
    if (dst.DType != src.DType) llmq_detail::unsupported(__func__, dst, src);
    if (src.DType == ETensorDType::FP8_E4M3)
        transpose(dst.get<__hip_fp8_e4m3>(), src.get<__hip_fp8_e4m3>(), rows, cols, stream);
    else if (src.DType == ETensorDType::FP8_E5M2)
        transpose(dst.get<__hip_fp8_e5m2>(), src.get<__hip_fp8_e5m2>(), rows, cols, stream);
    else llmq_detail::unsupported(__func__, dst, src);
}

// Extension (no counterpart in the reference): quantize_with_abs_max and the transpose of its result from
// one read of the input.  out[rows, cols] and out_tp[cols, rows] must have the same fp8 dtype.
inline void quantize_with_abs_max_and_transpose(Tensor& out, Tensor& out_tp, float* scale_ptr, const Tensor& in,
                                                const float* abs_max, int rows, int cols, const hipDeviceProp_t&,
                                                hipStream_t stream) {
    if (in.DType != ETensorDType::BF16 || out.DType != out_tp.DType ||
        (out.DType != ETensorDType::FP8_E4M3 && out.DType != ETensorDType::FP8_E5M2))
        llmq_detail::unsupported(__func__, out, out_tp, in);
    llmq_detail::check(llmq_quantize_both_bf16(reinterpret_cast<uint8_t*>(out.Data), reinterpret_cast<uint8_t*>(out_tp.Data),
                                               scale_ptr, llmq_detail::u16(in.get<__hip_bfloat16>()), abs_max, rows, cols,
                                               out.DType == ETensorDType::FP8_E5M2 ? 1 : 0, stream));
}

// ---- matmul (reference: src/kernels/kernels.h:72-78, 88-90, 96-98) --------------------------------------
// Row-major a[M,K], b[N,K] -> row-major c[N,M] = (b . a^T) * (*scale_a * *scale_b) (+ bias[M]) (+ c).
// Mode TN: any M, N >= 1 and K a multiple of 16 (16-byte aligned fp8 rows).  The K-major modes -- TT (b stored [K, N]:
// e.g. the output gradient dY[B*T, OC] of the weight gradient without its transposed copy), NN (a stored [K, M]: the
// weight W[OC, C] of the dgrad) and NT (both) -- serve M, N and K multiples of 256 (mode TT with bf16 output and without
// accumulation also M of 224), bf16 and fp32 output, with bias and accumulation.  Anything else throws
// std::invalid_argument before a kernel is launched.
inline void matmul(__hip_bfloat16* c, const __hip_fp8_e4m3* a, const __hip_fp8_e4m3* b, const __hip_bfloat16* bias,
                   const float* scale_a, const float* scale_b, llmqBlasHandle_t, std::byte* workspace,
                   std::size_t workspace_size, int M, int N, int K, EMMTranspose mode, bool accumulate,
                   hipStream_t stream, EMatmulBackend = EMatmulBackend::Custom) {
    llmq_detail::check(llmq_gemm_e4m3_bf16_mode(llmq_detail::u16(c), llmq_detail::u8(a), llmq_detail::u8(b),
                                                llmq_detail::u16(bias), scale_a, scale_b, workspace, workspace_size, M, N,
                                                K, llmq_detail::mode_code(mode), 0, accumulate, stream));
}
inline void matmul(float* c, const __hip_fp8_e4m3* a, const __hip_fp8_e4m3* b, const float* bias, const float* scale_a,
                   const float* scale_b, llmqBlasHandle_t, std::byte* workspace, std::size_t workspace_size, int M,
                   int N, int K, EMMTranspose mode, bool accumulate, hipStream_t stream,
                   EMatmulBackend = EMatmulBackend::Custom) {
    llmq_detail::check(llmq_gemm_e4m3_f32_mode(c, llmq_detail::u8(a), llmq_detail::u8(b), bias, 0, scale_a, scale_b, workspace,
                                               workspace_size, M, N, K, llmq_detail::mode_code(mode), 0, accumulate, stream));
}
inline void matmul(float* c, const __hip_fp8_e4m3* a, const __hip_fp8_e4m3* b, const __hip_bfloat16* bias,
                   const float* scale_a, const float* scale_b, llmqBlasHandle_t, std::byte* workspace,
                   std::size_t workspace_size, int M, int N, int K, EMMTranspose mode, bool accumulate,
                   hipStream_t stream, EMatmulBackend = EMatmulBackend::Custom) {
    llmq_detail::check(llmq_gemm_e4m3_f32_mode(c, llmq_detail::u8(a), llmq_detail::u8(b), bias, 1, scale_a, scale_b, workspace,
                                               workspace_size, M, N, K, llmq_detail::mode_code(mode), 0, accumulate, stream));
}
// e4m3 x e5m2 (gradient dtype option; reference: src/kernels/kernels.h:80-82, 92-94)
inline void matmul(__hip_bfloat16* c, const __hip_fp8_e4m3* a, const __hip_fp8_e5m2* b, const __hip_bfloat16* bias,
                   const float* scale_a, const float* scale_b, llmqBlasHandle_t, std::byte* workspace,
                   std::size_t workspace_size, int M, int N, int K, EMMTranspose mode, bool accumulate,
                   hipStream_t stream, EMatmulBackend = EMatmulBackend::Custom) {
    llmq_detail::check(llmq_gemm_e4m3_bf16_mode(llmq_detail::u16(c), llmq_detail::u8(a), llmq_detail::u8(b),
                                                llmq_detail::u16(bias), scale_a, scale_b, workspace, workspace_size, M, N,
                                                K, llmq_detail::mode_code(mode), 1, accumulate, stream));
}
inline void matmul(float* c, const __hip_fp8_e4m3* a, const __hip_fp8_e5m2* b, const __hip_bfloat16* bias,
                   const float* scale_a, const float* scale_b, llmqBlasHandle_t, std::byte* workspace,
                   std::size_t workspace_size, int M, int N, int K, EMMTranspose mode, bool accumulate,
                   hipStream_t stream, EMatmulBackend = EMatmulBackend::Custom) {
    llmq_detail::check(llmq_gemm_e4m3_f32_mode(c, llmq_detail::u8(a), llmq_detail::u8(b), bias, 1, scale_a, scale_b, workspace,
                                               workspace_size, M, N, K, llmq_detail::mode_code(mode), 1, accumulate, stream));
}
inline void matmul(Tensor& c, const Tensor& a, const Tensor& b, const Tensor& bias, const float* scale_a,
                   const float* scale_b, llmqBlasHandle_t handle, Tensor& workspace, int M, int N, int K,
                   EMMTranspose mode, bool accumulate, hipStream_t stream,
                   EMatmulBackend backend = EMatmulBackend::Custom) {
    std::byte* ws = workspace.Data;
    const std::size_t ws_size = workspace.empty() ? 0 : workspace.bytes();
    if (a.DType == ETensorDType::FP8_E4M3 && b.DType == ETensorDType::FP8_E5M2) {
        if (c.DType == ETensorDType::BF16)
            matmul(c.get<__hip_bfloat16>(), a.get<__hip_fp8_e4m3>(), b.get<__hip_fp8_e5m2>(),
                   bias.get_optional<__hip_bfloat16>(), scale_a, scale_b, handle, ws, ws_size, M, N, K, mode, accumulate,
                   stream, backend);
        else if (c.DType == ETensorDType::FP32)
            matmul(c.get<float>(), a.get<__hip_fp8_e4m3>(), b.get<__hip_fp8_e5m2>(), bias.get_optional<__hip_bfloat16>(),
                   scale_a, scale_b, handle, ws, ws_size, M, N, K, mode, accumulate, stream, backend);
        else llmq_detail::unsupported(__func__, c, a, b, bias, workspace);
        return;
    }
    if (a.DType != ETensorDType::FP8_E4M3 || b.DType != ETensorDType::FP8_E4M3)
        llmq_detail::unsupported(__func__, c, a, b, bias, workspace);
    if (c.DType == ETensorDType::FP32) {
        if (!bias.empty() && bias.DType == ETensorDType::BF16)
            matmul(c.get<float>(), a.get<__hip_fp8_e4m3>(), b.get<__hip_fp8_e4m3>(), bias.get<__hip_bfloat16>(), scale_a,
                   scale_b, handle, ws, ws_size, M, N, K, mode, accumulate, stream, backend);
        else
            matmul(c.get<float>(), a.get<__hip_fp8_e4m3>(), b.get<__hip_fp8_e4m3>(), bias.get_optional<float>(), scale_a,
                   scale_b, handle, ws, ws_size, M, N, K, mode, accumulate, stream, backend);
    } else if (c.DType == ETensorDType::BF16) {
        matmul(c.get<__hip_bfloat16>(), a.get<__hip_fp8_e4m3>(), b.get<__hip_fp8_e4m3>(),
               bias.get_optional<__hip_bfloat16>(), scale_a, scale_b, handle, ws, ws_size, M, N, K, mode, accumulate, stream,
               backend);
    } else {
        llmq_detail::unsupported(__func__, c, a, b, bias, workspace);
    }
}

// ---- backward_bias (reference: src/kernels/kernels.h:102-107, src/kernels/bias.cu:142-195) ---------------
// dbias[OC] += (*scale_a * *scale_b) * column sums of dout[B*T, OC]; scales both null or both non-null.
inline int get_bias_backward_scratch_size(ETensorDType dtype, int OC, const hipDeviceProp_t&) {
    // sized for any B*T (the number of row bands saturates for large row counts)
    return (int)llmq_backward_bias_scratch_bytes(1 << 30, OC, dtype == ETensorDType::BF16 ? 2 : 0);
}
inline void backward_bias(__hip_bfloat16* dbias, const __hip_fp8_e4m3* dout, const float* scale_a, const float* scale_b,
                          float* dbias_buffer, int B, int T, int OC, const hipDeviceProp_t& dp, hipStream_t stream) {
    llmq_detail::check(llmq_backward_bias_bf16(llmq_detail::u16(dbias), dout, 0, scale_a, scale_b, dbias_buffer,
                                               (std::size_t)get_bias_backward_scratch_size(ETensorDType::FP8_E4M3, OC, dp),
                                               B * T, OC, stream));
}
inline void backward_bias(__hip_bfloat16* dbias, const __hip_fp8_e5m2* dout, const float* scale_a, const float* scale_b,
                          float* dbias_buffer, int B, int T, int OC, const hipDeviceProp_t& dp, hipStream_t stream) {
    llmq_detail::check(llmq_backward_bias_bf16(llmq_detail::u16(dbias), dout, 1, scale_a, scale_b, dbias_buffer,
                                               (std::size_t)get_bias_backward_scratch_size(ETensorDType::FP8_E5M2, OC, dp),
                                               B * T, OC, stream));
}
inline void backward_bias(__hip_bfloat16* dbias, const __hip_bfloat16* dout, const float* scale_a, const float* scale_b,
                          float* dbias_buffer, int B, int T, int OC, const hipDeviceProp_t& dp, hipStream_t stream) {
    llmq_detail::check(llmq_backward_bias_bf16(llmq_detail::u16(dbias), dout, 2, scale_a, scale_b, dbias_buffer,
                                               (std::size_t)get_bias_backward_scratch_size(ETensorDType::BF16, OC, dp),
                                               B * T, OC, stream));
}
inline void backward_bias(Tensor& dbias, const Tensor& dout, const float* scale_a, const float* scale_b,
                          Tensor& dbias_buffer, int B, int T, int OC, const hipDeviceProp_t& dp, hipStream_t stream) {
    const std::size_t expected = (std::size_t)get_bias_backward_scratch_size(dout.DType, OC, dp);
    if (dbias_buffer.bytes() < expected)
        throw std::invalid_argument("scratch buffer too small: expected at least " + std::to_string(expected) +
                                    " bytes, got " + std::to_string(dbias_buffer.bytes()));
    if (dbias.DType != ETensorDType::BF16) llmq_detail::unsupported(__func__, dbias, dout, dbias_buffer);
    if (dout.DType == ETensorDType::FP8_E4M3)
        backward_bias(dbias.get<__hip_bfloat16>(), dout.get<__hip_fp8_e4m3>(), scale_a, scale_b,
                      dbias_buffer.get<float>(), B, T, OC, dp, stream);
    else if (dout.DType == ETensorDType::FP8_E5M2)
        backward_bias(dbias.get<__hip_bfloat16>(), dout.get<__hip_fp8_e5m2>(), scale_a, scale_b,
                      dbias_buffer.get<float>(), B, T, OC, dp, stream);
    else if (dout.DType == ETensorDType::BF16)
        backward_bias(dbias.get<__hip_bfloat16>(), dout.get<__hip_bfloat16>(), scale_a, scale_b,
                      dbias_buffer.get<float>(), B, T, OC, dp, stream);
    else llmq_detail::unsupported(__func__, dbias, dout, dbias_buffer);
}

// ---- swiglu (reference: src/kernels/kernels.h:155-165, src/kernels/swiglu.cu) --------------------------------
// inp[B, T, 2C] rows are [up | gate]; bf16 tensors, or fp32 throughout (the quantizing variant: bf16 input only, as in
// the reference).
inline void swiglu_forward(__hip_bfloat16* out, const __hip_bfloat16* inp, float* abs_max_ptr, int B, int T, int C,
                           hipStream_t stream) {
    llmq_detail::check(llmq_swiglu_forward_bf16(llmq_detail::u16(out), llmq_detail::u16(inp), abs_max_ptr, B, T, C, stream));
}
inline void swiglu_forward(float* out, const float* inp, float* abs_max_ptr, int B, int T, int C, hipStream_t stream) {
    llmq_detail::check(llmq_swiglu_forward_f32(out, inp, abs_max_ptr, B, T, C, stream));
}
inline void swiglu_forward(Tensor& out, const Tensor& inp, float* abs_max_ptr, int B, int T, int C, hipStream_t stream) {
    if (out.DType == ETensorDType::FP32 && inp.DType == ETensorDType::FP32)
        return swiglu_forward(out.get<float>(), inp.get<float>(), abs_max_ptr, B, T, C, stream);
    if (out.DType != ETensorDType::BF16 || inp.DType != ETensorDType::BF16) llmq_detail::unsupported(__func__, out, inp);
    swiglu_forward(out.get<__hip_bfloat16>(), inp.get<__hip_bfloat16>(), abs_max_ptr, B, T, C, stream);
}
inline void swiglu_forward_quant(__hip_fp8_e4m3* out, float* scale_ptr, const __hip_bfloat16* inp, const float* abs_max_ptr,
                                 int B, int T, int C, hipStream_t stream) {
    llmq_detail::check(llmq_swiglu_forward_quant_bf16(llmq_detail::u8(out), scale_ptr, llmq_detail::u16(inp),
                                                      abs_max_ptr, B, T, C, stream));
}
inline void swiglu_forward_quant(Tensor& out, float* scale_ptr, const Tensor& inp, const float* abs_max_ptr, int B, int T,
                                 int C, hipStream_t stream) {
    if (out.DType != ETensorDType::FP8_E4M3 || inp.DType != ETensorDType::BF16) llmq_detail::unsupported(__func__, out, inp);
    swiglu_forward_quant(out.get<__hip_fp8_e4m3>(), scale_ptr, inp.get<__hip_bfloat16>(), abs_max_ptr, B, T, C, stream);
}
inline void swiglu_backward(__hip_bfloat16* dinp, const __hip_bfloat16* dout, const __hip_bfloat16* inp, float* abs_max,
                            int B, int T, int C, hipStream_t stream) {
    llmq_detail::check(llmq_swiglu_backward_bf16(llmq_detail::u16(dinp), llmq_detail::u16(dout), llmq_detail::u16(inp),
                                                 abs_max, B, T, C, stream));
}
inline void swiglu_backward(float* dinp, const float* dout, const float* inp, float* abs_max, int B, int T, int C,
                            hipStream_t stream) {
    llmq_detail::check(llmq_swiglu_backward_f32(dinp, dout, inp, abs_max, B, T, C, stream));
}
inline void swiglu_backward(Tensor& dinp, const Tensor& dout, const Tensor& inp, float* abs_max, int B, int T, int C,
                            hipStream_t stream) {
    if (dinp.DType == ETensorDType::FP32 && dout.DType == ETensorDType::FP32 && inp.DType == ETensorDType::FP32)
        return swiglu_backward(dinp.get<float>(), dout.get<float>(), inp.get<float>(), abs_max, B, T, C, stream);
    if (dinp.DType != ETensorDType::BF16 || dout.DType != ETensorDType::BF16 || inp.DType != ETensorDType::BF16)
        llmq_detail::unsupported(__func__, dinp, dout, inp);
    swiglu_backward(dinp.get<__hip_bfloat16>(), dout.get<__hip_bfloat16>(), inp.get<__hip_bfloat16>(), abs_max, B, T, C,
                    stream);
}

// ---- rmsnorm forward (reference: src/kernels/kernels.h:45-47,57-62, src/kernels/rmsnorm.cu) ------------------------
inline void rmsnorm_forward(__hip_bfloat16* out, float* rms, const __hip_bfloat16* inp, const __hip_bfloat16* weight,
                            float* abs_max_ptr, float epsilon, int B, int T, int C, hipStream_t stream) {
    llmq_detail::check(llmq_rmsnorm_forward_bf16(llmq_detail::u16(out), rms, llmq_detail::u16(inp), llmq_detail::u16(weight),
                                                 abs_max_ptr, epsilon, B, T, C, stream));
}
inline void rmsnorm_forward(float* out, float* rms, const float* inp, const float* weight, float* abs_max_ptr, float epsilon,
                            int B, int T, int C, hipStream_t stream) {
    llmq_detail::check(llmq_rmsnorm_forward_f32(out, rms, inp, weight, abs_max_ptr, epsilon, B, T, C, stream));
}
inline void rmsnorm_forward(Tensor& out, Tensor& rms, const Tensor& inp, const Tensor& weight, float* abs_max_ptr,
                            float epsilon, int B, int T, int C, hipStream_t stream) {
    if (out.DType == ETensorDType::FP32 && inp.DType == ETensorDType::FP32 && weight.DType == ETensorDType::FP32 &&
        rms.DType == ETensorDType::FP32)
        return rmsnorm_forward(out.get<float>(), rms.get<float>(), inp.get<float>(), weight.get<float>(), abs_max_ptr, epsilon,
                               B, T, C, stream);
    if (out.DType != ETensorDType::BF16 || inp.DType != ETensorDType::BF16 || weight.DType != ETensorDType::BF16 ||
        rms.DType != ETensorDType::FP32)
        llmq_detail::unsupported(__func__, out, rms, inp, weight);
    rmsnorm_forward(out.get<__hip_bfloat16>(), rms.get<float>(), inp.get<__hip_bfloat16>(), weight.get<__hip_bfloat16>(),
                    abs_max_ptr, epsilon, B, T, C, stream);
}
inline void fused_residual_rmsnorm_forward(__hip_bfloat16* residual, __hip_bfloat16* normed, float* rrms,
                                           const __hip_bfloat16* inp1, const __hip_bfloat16* inp2,
                                           const __hip_bfloat16* weight, float* abs_max_ptr, float epsilon, int N, int C,
                                           hipStream_t stream) {
    llmq_detail::check(llmq_fused_residual_rmsnorm_forward_bf16(llmq_detail::u16(residual), llmq_detail::u16(normed), rrms,
                                                                llmq_detail::u16(inp1), llmq_detail::u16(inp2),
                                                                llmq_detail::u16(weight), abs_max_ptr, epsilon, N, C, stream));
}
inline void fused_residual_rmsnorm_forward(float* residual, float* normed, float* rrms, const float* inp1, const float* inp2,
                                           const float* weight, float* abs_max_ptr, float epsilon, int N, int C,
                                           hipStream_t stream) {
    llmq_detail::check(llmq_fused_residual_rmsnorm_forward_f32(residual, normed, rrms, inp1, inp2, weight, abs_max_ptr, epsilon,
                                                               N, C, stream));
}
inline void fused_residual_rmsnorm_forward(Tensor& residual, Tensor& normed, Tensor& rrms, const Tensor& inp1,
                                           const Tensor& inp2, const Tensor& weight, float* abs_max_ptr, float epsilon,
                                           int N, int C, hipStream_t stream) {
    if (residual.DType == ETensorDType::FP32 && normed.DType == ETensorDType::FP32 && inp1.DType == ETensorDType::FP32 &&
        inp2.DType == ETensorDType::FP32 && weight.DType == ETensorDType::FP32 && rrms.DType == ETensorDType::FP32)
        return fused_residual_rmsnorm_forward(residual.get<float>(), normed.get<float>(), rrms.get<float>(), inp1.get<float>(),
                                              inp2.get<float>(), weight.get<float>(), abs_max_ptr, epsilon, N, C, stream);
    if (residual.DType != ETensorDType::BF16 || normed.DType != ETensorDType::BF16 || inp1.DType != ETensorDType::BF16 ||
        inp2.DType != ETensorDType::BF16 || weight.DType != ETensorDType::BF16 || rrms.DType != ETensorDType::FP32)
        llmq_detail::unsupported(__func__, residual, normed, rrms, inp1, inp2, weight);
    fused_residual_rmsnorm_forward(residual.get<__hip_bfloat16>(), normed.get<__hip_bfloat16>(), rrms.get<float>(),
                                   inp1.get<__hip_bfloat16>(), inp2.get<__hip_bfloat16>(), weight.get<__hip_bfloat16>(),
                                   abs_max_ptr, epsilon, N, C, stream);
}

// ---- rmsnorm backward (reference: src/kernels/kernels.h:49-55, src/kernels/rmsnorm.cu:229-470) ----------------------
inline int get_rmsnorm_backward_scratch_size(int C, const hipDeviceProp_t&) { return (int)llmq_rmsnorm_backward_scratch_bytes(C); }
inline void rmsnorm_backward(__hip_bfloat16* dinp, __hip_bfloat16* dweight, std::byte* scratch, const __hip_bfloat16* dresidual,
                             const __hip_bfloat16* dout, const __hip_bfloat16* inp, const __hip_bfloat16* weight,
                             const float* rstd, float* abs_max_ptr, int B, int T, int C, const hipDeviceProp_t& dp,
                             hipStream_t stream) {
    llmq_detail::check(llmq_rmsnorm_backward_bf16(llmq_detail::u16(dinp), llmq_detail::u16(dweight), scratch,
                                                  (std::size_t)get_rmsnorm_backward_scratch_size(C, dp),
                                                  llmq_detail::u16(dresidual), llmq_detail::u16(dout), llmq_detail::u16(inp),
                                                  llmq_detail::u16(weight), rstd, abs_max_ptr, B, T, C, stream));
}
inline void rmsnorm_backward(float* dinp, float* dweight, std::byte* scratch, const float* dresidual, const float* dout,
                             const float* inp, const float* weight, const float* rstd, float* abs_max_ptr, int B, int T, int C,
                             const hipDeviceProp_t& dp, hipStream_t stream) {
    llmq_detail::check(llmq_rmsnorm_backward_f32(dinp, dweight, scratch, (std::size_t)get_rmsnorm_backward_scratch_size(C, dp),
                                                 dresidual, dout, inp, weight, rstd, abs_max_ptr, B, T, C, stream));
}
inline void rmsnorm_backward(Tensor& dinp, Tensor& dweight, Tensor& scratch, const Tensor& dresidual, const Tensor& dout,
                             const Tensor& inp, const Tensor& weight, const Tensor& rstd, float* abs_max_ptr, int B, int T,
                             int C, const hipDeviceProp_t& dp, hipStream_t stream) {
    if (dinp.DType == ETensorDType::FP32 && dweight.DType == ETensorDType::FP32 && dresidual.DType == ETensorDType::FP32 &&
        dout.DType == ETensorDType::FP32 && inp.DType == ETensorDType::FP32 && weight.DType == ETensorDType::FP32 &&
        rstd.DType == ETensorDType::FP32) {
        if (scratch.bytes() < (std::size_t)get_rmsnorm_backward_scratch_size(C, dp))
            throw std::invalid_argument("rmsnorm_backward: scratch buffer too small");
        llmq_detail::check(llmq_rmsnorm_backward_f32(dinp.get<float>(), dweight.get<float>(), scratch.Data, scratch.bytes(),
                                                     dresidual.get<float>(), dout.get<float>(), inp.get<float>(),
                                                     weight.get<float>(), rstd.get<float>(), abs_max_ptr, B, T, C, stream));
        return;
    }
    if (dinp.DType != ETensorDType::BF16 || dweight.DType != ETensorDType::BF16 || dresidual.DType != ETensorDType::BF16 ||
        dout.DType != ETensorDType::BF16 || inp.DType != ETensorDType::BF16 || weight.DType != ETensorDType::BF16 ||
        rstd.DType != ETensorDType::FP32)
        llmq_detail::unsupported(__func__, dinp, dweight, dresidual, dout, inp, weight, rstd);
    if (scratch.bytes() < (std::size_t)get_rmsnorm_backward_scratch_size(C, dp))
        throw std::invalid_argument("rmsnorm_backward: scratch buffer too small");
    llmq_detail::check(llmq_rmsnorm_backward_bf16(llmq_detail::u16(dinp.get<__hip_bfloat16>()),
                                                  llmq_detail::u16(dweight.get<__hip_bfloat16>()), scratch.Data, scratch.bytes(),
                                                  llmq_detail::u16(dresidual.get<__hip_bfloat16>()),
                                                  llmq_detail::u16(dout.get<__hip_bfloat16>()),
                                                  llmq_detail::u16(inp.get<__hip_bfloat16>()),
                                                  llmq_detail::u16(weight.get<__hip_bfloat16>()), rstd.get<float>(),
                                                  abs_max_ptr, B, T, C, stream));
}

// ---- rope (reference: src/kernels/kernels.h:110-117, src/kernels/rope.cu) ------------------------------------------
inline void precompute_freqs_cis(__half* freqs_cis, int dim, int end, float theta) {
    llmq_detail::check(llmq_precompute_freqs_cis_f16(reinterpret_cast<std::uint16_t*>(freqs_cis), dim, end, theta));
}
inline void rope_forward(__hip_bfloat16* out, const __hip_bfloat16* in, const __half* freqs_cis, float* abs_max_ptr, int B,
                         int T, int Nq, int Nkv, int head_dim, hipStream_t stream) {
    llmq_detail::check(llmq_rope_forward_bf16(llmq_detail::u16(out), llmq_detail::u16(in),
                                              reinterpret_cast<const std::uint16_t*>(freqs_cis), abs_max_ptr, B, T, Nq, Nkv,
                                              head_dim, stream));
}
inline void rope_backward(__hip_bfloat16* dinp, const __hip_bfloat16* dout, const __half* freqs_cis, float* abs_max_ptr, int B,
                          int T, int Nq, int Nkv, int head_dim, hipStream_t stream) {
    llmq_detail::check(llmq_rope_backward_bf16(llmq_detail::u16(dinp), llmq_detail::u16(dout),
                                               reinterpret_cast<const std::uint16_t*>(freqs_cis), abs_max_ptr, B, T, Nq, Nkv,
                                               head_dim, stream));
}

inline void precompute_freqs_cis(float* freqs_cis, int dim, int end, float theta) {
    llmq_detail::check(llmq_precompute_freqs_cis_f32(freqs_cis, dim, end, theta));
}
inline void rope_forward(float* out, const float* in, const float* freqs_cis, float* abs_max_ptr, int B, int T, int Nq, int Nkv,
                         int head_dim, hipStream_t stream) {
    llmq_detail::check(llmq_rope_forward_f32(out, in, freqs_cis, abs_max_ptr, B, T, Nq, Nkv, head_dim, stream));
}
inline void rope_backward(float* dinp, const float* dout, const float* freqs_cis, float* abs_max_ptr, int B, int T, int Nq,
                          int Nkv, int head_dim, hipStream_t stream) {
    llmq_detail::check(llmq_rope_backward_f32(dinp, dout, freqs_cis, abs_max_ptr, B, T, Nq, Nkv, head_dim, stream));
}
inline void rope_forward(Tensor& out, const Tensor& in, const Tensor& freqs_cis, float* abs_max_ptr, int B, int T, int Nq,
                         int Nkv, int head_dim, hipStream_t stream) {
    if (out.DType == ETensorDType::FP32 && in.DType == ETensorDType::FP32 && freqs_cis.DType == ETensorDType::FP32)
        return rope_forward(out.get<float>(), in.get<float>(), freqs_cis.get<float>(), abs_max_ptr, B, T, Nq, Nkv, head_dim, stream);
    if (out.DType != ETensorDType::BF16 || in.DType != ETensorDType::BF16 || freqs_cis.DType != ETensorDType::FP16)
        llmq_detail::unsupported(__func__, out, in, freqs_cis);
    rope_forward(out.get<__hip_bfloat16>(), in.get<__hip_bfloat16>(), freqs_cis.get<__half>(), abs_max_ptr, B, T, Nq, Nkv,
                 head_dim, stream);
}
inline void rope_backward(Tensor& dinp, const Tensor& dout, const Tensor& freqs_cis, float* abs_max_ptr, int B, int T, int Nq,
                          int Nkv, int head_dim, hipStream_t stream) {
    if (dinp.DType == ETensorDType::FP32 && dout.DType == ETensorDType::FP32 && freqs_cis.DType == ETensorDType::FP32)
        return rope_backward(dinp.get<float>(), dout.get<float>(), freqs_cis.get<float>(), abs_max_ptr, B, T, Nq, Nkv, head_dim,
                             stream);
    if (dinp.DType != ETensorDType::BF16 || dout.DType != ETensorDType::BF16 || freqs_cis.DType != ETensorDType::FP16)
        llmq_detail::unsupported(__func__, dinp, dout, freqs_cis);
    rope_backward(dinp.get<__hip_bfloat16>(), dout.get<__hip_bfloat16>(), freqs_cis.get<__half>(), abs_max_ptr, B, T, Nq, Nkv,
                  head_dim, stream);
}

// ---- adamw (reference: src/kernels/kernels.h:225-235, src/kernels/adamw.cu) ----------------------------------------
// bf16 parameters and gradients; moments fp32/fp32, bf16/fp32, bf16/bf16 or e4m3 (block scales)/bf16; or everything
// fp32 (no stochastic rounding).  abs_max is merged, not reset.
inline void adamw_update(float* params, const float* grads, float* m, float* v, std::size_t num_parameters, float learning_rate,
                         float beta1, float beta2, int t, float eps, float weight_decay, const float* grad_scale, float* abs_max,
                         unsigned int seed, hipStream_t stream) {
    llmq_detail::check(llmq_adamw_update_f32(params, grads, m, v, (std::int64_t)num_parameters, learning_rate, beta1, beta2, t, eps,
                                             weight_decay, grad_scale, abs_max, seed, stream));
}
inline void adamw_update(__hip_bfloat16* params, const __hip_bfloat16* grads, float* m, float* v, std::size_t num_parameters,
                         float learning_rate, float beta1, float beta2, int t, float eps, float weight_decay,
                         const float* grad_scale, float* abs_max, unsigned int seed, hipStream_t stream) {
    llmq_detail::check(llmq_adamw_update_bf16(llmq_detail::u16(params), llmq_detail::u16(grads), m, 0, v, 0,
                                              (std::int64_t)num_parameters, learning_rate, beta1, beta2, t, eps, weight_decay,
                                              grad_scale, abs_max, seed, stream));
}
inline void adamw_update(__hip_bfloat16* params, const __hip_bfloat16* grads, __hip_bfloat16* m, float* v,
                         std::size_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps,
                         float weight_decay, const float* grad_scale, float* abs_max, unsigned int seed, hipStream_t stream) {
    llmq_detail::check(llmq_adamw_update_bf16(llmq_detail::u16(params), llmq_detail::u16(grads), m, 1, v, 0,
                                              (std::int64_t)num_parameters, learning_rate, beta1, beta2, t, eps, weight_decay,
                                              grad_scale, abs_max, seed, stream));
}
inline void adamw_update(__hip_bfloat16* params, const __hip_bfloat16* grads, __hip_bfloat16* m, __hip_bfloat16* v,
                         std::size_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps,
                         float weight_decay, const float* grad_scale, float* abs_max, unsigned int seed, hipStream_t stream) {
    llmq_detail::check(llmq_adamw_update_bf16(llmq_detail::u16(params), llmq_detail::u16(grads), m, 1, v, 1,
                                              (std::int64_t)num_parameters, learning_rate, beta1, beta2, t, eps, weight_decay,
                                              grad_scale, abs_max, seed, stream));
}
// e4m3 first moment with one fp32 scale per 128 elements (m_scales), bf16 second moment (kernels.h:237-239)
inline void adamw_update(__hip_bfloat16* params, const __hip_bfloat16* grads, __hip_fp8_e4m3* m, __hip_bfloat16* v,
                         std::size_t num_parameters, float learning_rate, float beta1, float beta2, int t, float eps,
                         float weight_decay, const float* grad_scale, float* m_scales, float* abs_max, unsigned int seed,
                         hipStream_t stream) {
    llmq_detail::check(llmq_adamw_update_bf16_fp8m(llmq_detail::u16(params), llmq_detail::u16(grads),
                                                   reinterpret_cast<std::uint8_t*>(m), m_scales, llmq_detail::u16(v),
                                                   (std::int64_t)num_parameters, learning_rate, beta1, beta2, t, eps,
                                                   weight_decay, grad_scale, abs_max, seed, stream));
}

#endif  // LLMQ_KERNELS_HPP
