// RMSNorm forward (plain and with the residual add fused in) and backward for gfx950: the producers of the
// inputs of the QKV and gate+up projections and of the gradient that flows into the previous projections,
// each with the abs-max of its output computed on the way.
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
        if (valid && c < chunks) x[k] = load_nt(&inp1[base + c]);
    }
    if constexpr (RESIDUAL) {
        uint4 y[NCH];
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = lane + kWave * k;
            y[k] = make_uint4(0, 0, 0, 0);
            if (valid && c < chunks) y[k] = load_nt(&inp2[base + c]);
        }
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = lane + kWave * k;
            x[k] = make_uint4(add_pair(x[k].x, y[k].x), add_pair(x[k].y, y[k].y), add_pair(x[k].z, y[k].z),
                              add_pair(x[k].w, y[k].w));
            if (valid && c < chunks) store_nt(&residual[base + c], x[k]);
        }
    }

    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < NCH; ++k) acc = squares(squares(squares(squares(acc, x[k].x), x[k].y), x[k].z), x[k].w);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc = acc + __shfl_xor(acc, off, kWave);
    const float s = __fdiv_rn(1.0f, sqrt_rn(__fdiv_rn(acc, c_float) + epsilon));

    uint32_t fold = 0x7F807F80u;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = lane + kWave * k;
        if (c < chunks) {
            const uint4 w = weight[c];
            const uint4 o = make_uint4(norm_pair(x[k].x, w.x, s), norm_pair(x[k].y, w.y, s), norm_pair(x[k].z, w.z, s),
                                       norm_pair(x[k].w, w.w, s));
            if (valid) {
                store_nt(&normed[base + c], o);
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

// ---- backward --------------------------------------------------------------------------------------
// Semantics follow the reference (src/kernels/rmsnorm.cu:229-440, 447-470), per row bt with r = rstd[bt]:
//   g_c     = (float)weight[c] * (float)dout[bt, c]
//   k       = (sum_c g_c * inp[bt, c]) / C * r
//   dinp[bt, c]  = bf16( (float)dresidual[bt, c] + (g_c - inp[bt, c] * r * k) * r )
//   dweight[c]   = bf16( (float)dweight[c] + sum_bt inp[bt, c] * r * dout[bt, c] )        (accumulates)
//   *abs_max     = max |dinp| over the rounded outputs.
// The reference copies dresidual into dinp first and accumulates in place; here dresidual is read directly
// (it may be the same buffer as dinp).  Sums are fp32 in a fixed order (deterministic): a lane owns the same
// columns of every row it sees, so its dweight terms accumulate in registers; the waves of a workgroup add
// theirs through LDS in a fixed order, workgroup sums go to the caller's scratch [workgroups][C] and a second
// kernel adds them with a fixed tree and updates dweight.
// HBM bound: 8 bytes per element (dout, inp, dresidual read; dinp written).
// WPR waves share a row (wave `sub` of them takes the chunks sub*64 + lane + 64*WPR*k), so that a lane never
// holds more than NCH <= 4 chunks of each operand plus its 8*NCH dweight sums: enough waves stay resident to
// keep the memory system busy.  The 4 / WPR rows a workgroup works on at a time advance in lockstep (the
// row's dot product is combined through LDS, with a workgroup barrier).
template <int NCH, int WPR, bool ABSMAX>
__global__ __launch_bounds__(256) void rmsnorm_backward_kernel(uint4* dinp, float* __restrict__ partial,
                                                               const uint4* dresidual, const uint4* __restrict__ dout,
                                                               const uint4* __restrict__ inp,
                                                               const uint4* __restrict__ weight,
                                                               const float* __restrict__ rstd,
                                                               unsigned* __restrict__ absmax_out, int N, int chunks,
                                                               float c_float) {
    extern __shared__ float block_dw[];  // [8 * chunks]
    __shared__ float dot_part[2][4];
    constexpr int ROWS = 4 / WPR;  // rows in flight per workgroup
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int sub = wave % WPR, rslot = wave / WPR;
    const int c_first = sub * kWave + lane;

    float dw[NCH][8];
#pragma unroll
    for (int k = 0; k < NCH; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) dw[k][e] = 0.f;
    uint32_t fold = 0x7F807F80u;

    // Two register sets in ping-pong: the loads of the row after the current one are issued before the current
    // row is worked on, so that a wave keeps memory requests in flight through its arithmetic, the workgroup
    // barrier and its stores (one wave per SIMD pair otherwise alternates between loading and computing).
    struct RowRegs {
        uint4 d[NCH], x[NCH], old[NCH];
        float r;
        bool valid;
        int64_t base;
    };
    auto load_row = [&](RowRegs& q, int row0) {
        const int row = row0 + rslot;
        q.valid = row < N;
        q.base = (int64_t)row * chunks;
        q.r = q.valid ? rstd[row] : 0.f;
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = c_first + kWave * WPR * k;
            q.d[k] = q.x[k] = q.old[k] = make_uint4(0, 0, 0, 0);
            if (q.valid && c < chunks) {
                q.d[k] = load_nt(&dout[q.base + c]);
                q.x[k] = load_nt(&inp[q.base + c]);
                q.old[k] = load_nt(&dresidual[q.base + c]);
            }
        }
    };
    auto work_row = [&](const RowRegs& q, int parity) {
        const float r = q.r;
        float dot = 0.f;
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = c_first + kWave * WPR * k;
            if (c < chunks) {
                const uint4 w = weight[c];
                const uint32_t dv[4] = {q.d[k].x, q.d[k].y, q.d[k].z, q.d[k].w},
                               xv[4] = {q.x[k].x, q.x[k].y, q.x[k].z, q.x[k].w}, wv[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    dot = dot + (bf16_lo(wv[j]) * bf16_lo(dv[j])) * bf16_lo(xv[j]);
                    dot = dot + (bf16_hi(wv[j]) * bf16_hi(dv[j])) * bf16_hi(xv[j]);
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) dot = dot + __shfl_xor(dot, off, kWave);
        if constexpr (WPR > 1) {
            // the parts of the waves sharing the row, added in wave order (double-buffered slots: the next
            // row's writes cannot overtake this row's reads)
            if (lane == 0) dot_part[parity][wave] = dot;
            __syncthreads();
            dot = dot_part[parity][rslot * WPR];
#pragma unroll
            for (int p = 1; p < WPR; ++p) dot = dot + dot_part[parity][rslot * WPR + p];
        }
        const float kk = __fdiv_rn(dot, c_float) * r;
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int c = c_first + kWave * WPR * k;
            if (q.valid && c < chunks) {
                const uint4 w = weight[c];
                const uint32_t dv[4] = {q.d[k].x, q.d[k].y, q.d[k].z, q.d[k].w},
                               xv[4] = {q.x[k].x, q.x[k].y, q.x[k].z, q.x[k].w}, wv[4] = {w.x, w.y, w.z, w.w},
                               ov[4] = {q.old[k].x, q.old[k].y, q.old[k].z, q.old[k].w};
                uint32_t res[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float n0 = bf16_lo(xv[j]) * r, n1 = bf16_hi(xv[j]) * r;
                    dw[k][2 * j] = dw[k][2 * j] + n0 * bf16_lo(dv[j]);
                    dw[k][2 * j + 1] = dw[k][2 * j + 1] + n1 * bf16_hi(dv[j]);
                    const float v0 = (bf16_lo(wv[j]) * bf16_lo(dv[j]) - n0 * kk) * r;
                    const float v1 = (bf16_hi(wv[j]) * bf16_hi(dv[j]) - n1 * kk) * r;
                    res[j] = pack_bf16_rn(bf16_lo(ov[j]) + v0, bf16_hi(ov[j]) + v1);
                }
                const uint4 o = make_uint4(res[0], res[1], res[2], res[3]);
                store_nt(&dinp[q.base + c], o);
                if constexpr (ABSMAX) fold = fold_vec(fold, o);
            }
        }
    };
    const int step = gridDim.x * ROWS;
    RowRegs ra, rb;
    load_row(ra, blockIdx.x * ROWS);
    for (int row0 = blockIdx.x * ROWS; row0 < N; row0 += 2 * step) {  // uniform trip count
        load_row(rb, row0 + step);       // rows past the end load nothing and store nothing
        work_row(ra, 0);
        if (row0 + step < N) {           // uniform: the barrier inside is reached by all or none
            load_row(ra, row0 + 2 * step);
            work_row(rb, 1);
        }
    }

    // workgroup sum of the dweight terms: the row slots add theirs in order (the waves of one slot own
    // disjoint columns, a lane the same columns in every slot), then the whole workgroup writes the row of
    // partial sums
    for (int sl = 0; sl < ROWS; ++sl) {
        if (rslot == sl) {
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                const int c = c_first + kWave * WPR * k;
                if (c < chunks) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float* slot = &block_dw[(size_t)e * chunks + c];  // [e][chunk]: consecutive lanes, consecutive banks
                        *slot = sl == 0 ? dw[k][e] : *slot + dw[k][e];
                    }
                }
            }
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < 8 * chunks; i += 256) {
        const int e = i / chunks, c = i % chunks;
        partial[(size_t)blockIdx.x * (8 * chunks) + (size_t)c * 8 + e] = block_dw[i];
    }
    if constexpr (ABSMAX) {
        const uint32_t lo = fold & 0xFFFFu, hi = fold >> 16;
        block_min_to_atomic_max(absmax_out, lo < hi ? lo : hi, 0x7F80u, 16);
    }
}

// dweight[c] = bf16((float)dweight[c] + sum over workgroups of partial[g][c]).  A workgroup takes 32 columns as
// 8 quads x 32 lanes: lane (quad, q) adds workgroups q, q+32, ... in index order (four 16-byte loads in flight),
// the 32 lane sums are then added in lane order -- a fixed summation tree.
__global__ __launch_bounds__(256) void rmsnorm_dweight_finish_kernel(uint16_t* __restrict__ dweight,
                                                                     const float* __restrict__ partial, int groups, int C) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    __shared__ v4f red[32][8];
    const int quad = threadIdx.x % 8, q = threadIdx.x / 8;
    const int col = blockIdx.x * 32 + 4 * quad;  // C is a multiple of 8: a quad is inside or outside as a whole
    v4f s = {0.f, 0.f, 0.f, 0.f};
    if (col < C) {
        int g = q;
        for (; g + 96 < groups; g += 128) {
            const v4f p0 = *reinterpret_cast<const v4f*>(partial + (size_t)g * C + col);
            const v4f p1 = *reinterpret_cast<const v4f*>(partial + (size_t)(g + 32) * C + col);
            const v4f p2 = *reinterpret_cast<const v4f*>(partial + (size_t)(g + 64) * C + col);
            const v4f p3 = *reinterpret_cast<const v4f*>(partial + (size_t)(g + 96) * C + col);
            s = s + p0;
            s = s + p1;
            s = s + p2;
            s = s + p3;
        }
        for (; g < groups; g += 32) s = s + *reinterpret_cast<const v4f*>(partial + (size_t)g * C + col);
    }
    red[q][quad] = s;
    __syncthreads();
    if (q == 0 && col < C) {
        v4f t = red[0][quad];
#pragma unroll
        for (int k = 1; k < 32; ++k) t = t + red[k][quad];
        const uint2 old = *reinterpret_cast<const uint2*>(dweight + col);
        uint2 out;
        out.x = pack_bf16_rn(t[0] + bf16_lo(old.x), t[1] + bf16_hi(old.x));
        out.y = pack_bf16_rn(t[2] + bf16_lo(old.y), t[3] + bf16_hi(old.y));
        *reinterpret_cast<uint2*>(dweight + col) = out;
    }
}

// workgroups of the backward launch (also sizes the scratch buffer): two per compute unit
static int backward_groups() { return 2 * cu_count(); }

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

extern "C" int64_t llmq_rmsnorm_backward_scratch_bytes(int C) {
    if (C <= 0) return 0;
    return (int64_t)llmq::backward_groups() * C * (int64_t)sizeof(float);
}

extern "C" int llmq_rmsnorm_backward_bf16(uint16_t* dinp, uint16_t* dweight, void* scratch, size_t scratch_bytes,
                                          const uint16_t* dresidual, const uint16_t* dout, const uint16_t* inp,
                                          const uint16_t* weight, const float* rstd, float* abs_max_or_null, int B, int T,
                                          int C, void* stream_) {
    using namespace llmq;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t N64 = (int64_t)B * T;
    LLMQ_REQUIRE(B >= 0 && T >= 0 && C >= 0, "rmsnorm_backward: negative dimension (%d, %d, %d)", B, T, C);
    LLMQ_REQUIRE(N64 <= 0x7FFFFFFF, "rmsnorm_backward: too many rows (%lld)", (long long)N64);
    LLMQ_REQUIRE(C % 8 == 0, "rmsnorm_backward: C must be divisible by 8 (got %d)", C);
    LLMQ_REQUIRE(C <= 8192, "rmsnorm_backward: C up to 8192 is supported (got %d)", C);
    const int N = (int)N64;
    if (abs_max_or_null) {
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(abs_max_or_null));
        LLMQ_HIP_TRY(hipGetLastError());
    }
    if (N == 0 || C == 0) return LLMQ_OK;
    LLMQ_REQUIRE(dinp && dweight && dresidual && dout && inp && weight && rstd, "rmsnorm_backward: null tensor pointer");
    LLMQ_REQUIRE(aligned16(dinp) && aligned16(dresidual) && aligned16(dout) && aligned16(inp) && aligned16(weight) &&
                     aligned16(scratch),
                 "rmsnorm_backward: tensor and scratch pointers must be 16-byte aligned");
    const int chunks = C / 8;
    // waves per row so that a lane holds at most 4 chunks of each operand
    const int wpr = chunks <= 4 * kWave ? 1 : chunks <= 8 * kWave ? 2 : 4;
    const int rows_per_group = 4 / wpr;
    int groups = backward_groups();
    if (groups > (N + rows_per_group - 1) / rows_per_group) groups = (N + rows_per_group - 1) / rows_per_group;
    LLMQ_REQUIRE(scratch != nullptr && scratch_bytes >= (size_t)groups * C * sizeof(float),
                 "rmsnorm_backward: scratch of %zu bytes is too small (need %zu, see llmq_rmsnorm_backward_scratch_bytes)",
                 scratch_bytes, (size_t)groups * C * sizeof(float));
    const int per_lane = (chunks + kWave * wpr - 1) / (kWave * wpr);
    const size_t lds = (size_t)C * sizeof(float);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)groups), dim3(256), lds, stream, reinterpret_cast<uint4*>(dinp),
                           reinterpret_cast<float*>(scratch), reinterpret_cast<const uint4*>(dresidual),
                           reinterpret_cast<const uint4*>(dout), reinterpret_cast<const uint4*>(inp),
                           reinterpret_cast<const uint4*>(weight), rstd, reinterpret_cast<unsigned*>(abs_max_or_null), N,
                           chunks, (float)C);
    };
#define LLMQ_BWD(NCH, WPR)                                                   \
    do {                                                                     \
        if (abs_max_or_null) launch(rmsnorm_backward_kernel<NCH, WPR, true>); \
        else launch(rmsnorm_backward_kernel<NCH, WPR, false>);               \
    } while (0)
    if (wpr == 1) {
        if (per_lane <= 1) LLMQ_BWD(1, 1);
        else if (per_lane <= 2) LLMQ_BWD(2, 1);
        else LLMQ_BWD(4, 1);
    } else if (wpr == 2) {
        LLMQ_BWD(4, 2);
    } else {
        LLMQ_BWD(4, 4);
    }
#undef LLMQ_BWD
    LLMQ_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(rmsnorm_dweight_finish_kernel, dim3((unsigned)((C + 31) / 32)), dim3(256), 0, stream, dweight,
                       reinterpret_cast<const float*>(scratch), groups, C);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}
