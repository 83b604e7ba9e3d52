// Per-tensor abs-max reduction for gfx950.
//
// Semantics follow the reference's reduce_abs_max_kernel (src/kernels/quant.cu:11-28) and
// handle_absmax_reduction (src/kernels/kernel_utils.cuh:17-32): *result = max_i |in[i]| as fp32,
// NaNs ignored, result >= +0, slot reset before the reduction.  The result is order independent, so
// it is bit exact by construction.
//
// Design: HBM-bound streaming read (2 bytes per element).  Each lane issues UNROLL independent
// 128-bit loads per trip (grid-stride, every wave instruction covers 1 KiB contiguous), folds them
// with packed 16-bit integer ops, then wave shuffle -> LDS -> one value per workgroup.
//
// One launch per call.  The reference clears the slot with a memset and lets every block merge into it with an atomic
// max (two stream operations, and one address that all blocks hit).  Here every workgroup writes its maximum to a
// place of its own in a scratch area built into the device code and counts itself in; the workgroup that arrives last
// takes the maximum of all of them, stores it to the caller's slot (a plain store: the slot needs no clearing) and sets
// the arrival counter back to zero.  Nobody waits for anybody.  The scratch area holds kAbsmaxSlots independent
// arrival areas; a call uses the one selected by its result address ((address / 4) % kAbsmaxSlots), so calls with
// neighbouring result slots (the reference keeps [abs_max, scale] pairs in per-layer tables) use different areas.
// Calls on one stream run one after the other and can share an area; calls that overlap in time on one GPU
// (different streams without an ordering between them) must not map to the same area -- the documented limit of this
// entry point.
//
// The fold works on bit patterns: for a bf16 pattern p, a = p & 0x7FFF is |x|'s pattern and
// y = 0x7F80 - a (mod 2^16) is <= 0x7F80 for every non-NaN value and >= 0xFF81 for every NaN.
// min over y therefore ignores NaNs and finds the largest |x|; the start value 0x7F80 encodes 0.
#include "common.hpp"
#include "absmax_reduce.hpp"

namespace llmq {

// Workgroups of 16 waves: the workgroups of the first resident round finish together, find the slot still
// empty and all issue their atomic on the one address; a quarter as many workgroups means a quarter of
// that serialised tail (measured: 10 us on 2048 workgroups).
constexpr int kAbsmaxThreads = 1024;

// Every lane keeps UNROLL independent 128-bit loads in flight; out-of-range slots of the last trip are
// predicated to zero instead of falling into a serial tail loop.
// STREAM selects the cache policy of the loads; the library uses ordinary (cached) loads for every size.  The
// quantizer that follows re-reads the tensor, and what is still in the 256 MB last-level cache it gets from
// there.  For tensors beyond the cache size streaming loads make this kernel 8-10 % faster on its own (its
// allocating reads no longer push out earlier kernels' not yet written-back outputs), but those write-backs
// then fall into the quantizer and the matmul that follow: the whole bench step was 0.8 % slower with
// streaming loads above 224 MiB (alternating builds on one box: abs-max -4.3 us, quantize +2.9 us, matmul
// +8 us per launch), and slower for every tensor that fits the cache (59 MB: abs-max + quantize 35 -> 38 us).
// Arrival areas of the single-launch reduction: [kAbsmaxSlots][64 + kAbsmaxMaxBlocks] words; word 0 of an area is its
// arrival counter (zero whenever no call is using the area: zero-initialised with the module, set back by the last
// workgroup of every call), words 64.. hold one maximum per workgroup.
constexpr int kAbsmaxSlots = LLMQ_ABS_MAX_ARRIVAL_AREAS;
constexpr int kAbsmaxMaxBlocks = 8192;
constexpr int kAbsmaxAreaWords = 64 + kAbsmaxMaxBlocks;
static __device__ __align__(256) unsigned absmax_areas[kAbsmaxSlots * kAbsmaxAreaWords];

// Finish of a single-launch abs-max: `bits` is this lane's candidate (fp32 pattern of a non-negative value; patterns of
// non-negative floats order like the values).  Workgroup maximum -> own word of the area -> arrival count; the last
// workgroup to arrive reduces all words and stores the result.  Grids of one workgroup store directly.
__device__ __forceinline__ void block_max_last_arriver(unsigned* result, int area, uint32_t bits) {
    __shared__ uint32_t wave_max[16];
    __shared__ int is_last;
    auto block_max = [&](uint32_t v) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t o = __shfl_xor(v, off, kWave);
            v = o > v ? o : v;
        }
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        if (lane == 0) wave_max[wave] = v;
        __syncthreads();
        const int nw = blockDim.x / kWave;
        v = lane < nw ? wave_max[lane] : 0u;
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
            const uint32_t o = __shfl_xor(v, off, kWave);
            v = o > v ? o : v;
        }
        return v;  // valid in wave 0
    };
    const uint32_t mine = block_max(bits);
    unsigned* const words = absmax_areas + (size_t)area * kAbsmaxAreaWords;
    if (threadIdx.x == 0) {
        if (gridDim.x == 1) {
            *result = mine;
            is_last = 0;
        } else {
            __hip_atomic_store(words + 64 + blockIdx.x, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // release: the word above is visible to whoever sees this count; acquire: the last arriver sees all words
            const unsigned before = __hip_atomic_fetch_add(words, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
            is_last = before == gridDim.x - 1;
        }
    }
    __syncthreads();
    if (!is_last) return;  // uniform for the workgroup
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    uint32_t all = 0u;
    for (unsigned i = threadIdx.x; i < gridDim.x; i += blockDim.x) {
        const uint32_t w = __hip_atomic_load(words + 64 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        all = w > all ? w : all;
    }
    __syncthreads();  // wave_max is reused
    all = block_max(all);
    if (threadIdx.x == 0) {
        *result = all;
        __hip_atomic_store(words, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // the area is free again
    }
}

template <int UNROLL, bool STREAM>
__global__ __launch_bounds__(kAbsmaxThreads) void absmax_bf16_kernel(unsigned* __restrict__ result, int area,
                                                          const uint4* __restrict__ in, int64_t nvec,
                                                          const uint16_t* __restrict__ tail, int ntail) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t acc = 0x7F807F80u;
    for (int64_t i = tid; i < nvec; i += UNROLL * stride) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t idx = i + u * stride;
            v[u] = idx < nvec ? (STREAM ? load_nt(in + idx) : in[idx]) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc = fold_vec(acc, v[u]);
    }
    if (tid < ntail) acc = fold_bf16x2(acc, (uint32_t)tail[tid]);
    const uint32_t lo = acc & 0xFFFFu, hi = acc >> 16;
    block_max_last_arriver(result, area, (0x7F80u - (lo < hi ? lo : hi)) << 16);
}

template <int UNROLL>
__global__ __launch_bounds__(kAbsmaxThreads) void absmax_f32_kernel(unsigned* __restrict__ result, int area,
                                                         const uint4* __restrict__ in, int64_t nvec,
                                                         const uint32_t* __restrict__ tail, int ntail) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t acc = 0x7F800000u;
    auto fold = [&](uint32_t w) {
        uint32_t y = 0x7F800000u - (w & 0x7FFFFFFFu);  // wraps to a huge value for NaN
        acc = y < acc ? y : acc;
    };
    for (int64_t i = tid; i < nvec; i += UNROLL * stride) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t idx = i + u * stride;
            v[u] = idx < nvec ? in[idx] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) { fold(v[u].x); fold(v[u].y); fold(v[u].z); fold(v[u].w); }
    }
    if (tid < ntail) fold(tail[tid]);
    block_max_last_arriver(result, area, 0x7F800000u - acc);
}

template <typename Kernel, typename Elem>
static int launch_absmax(Kernel kernel, float* out, const Elem* in, int64_t n, int elems_per_vec, int unroll,
                         hipStream_t stream) {
    LLMQ_REQUIRE(out != nullptr, "abs_max: result pointer is null");
    LLMQ_REQUIRE(n >= 0, "abs_max: negative element count %lld", (long long)n);
    LLMQ_REQUIRE(n == 0 || in != nullptr, "abs_max: input pointer is null");
    LLMQ_REQUIRE(aligned16(in), "abs_max: input pointer must be 16-byte aligned");
    if (n == 0) {
        // the abs-max of nothing is 0: a one-lane fill kernel rather than a memset node, safe to record into a HIP graph
        hipLaunchKernelGGL(reset_slot_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<unsigned*>(out));
        LLMQ_HIP_TRY(hipGetLastError());
        return LLMQ_OK;
    }
    const int64_t nvec = n / elems_per_vec;
    const int ntail = (int)(n - nvec * elems_per_vec);
    const int64_t per_block = (int64_t)kAbsmaxThreads * unroll;
    // One trip per lane (`unroll` independent 16-byte loads each): on this chip a plain grid with many
    // short workgroups sustains more HBM bandwidth than a persistent grid-stride loop.  Tensors beyond
    // kAbsmaxMaxBlocks workgroups of that size (1 GiB of bf16) take more trips.
    int64_t blocks = (nvec + per_block - 1) / per_block;
    if (blocks > kAbsmaxMaxBlocks) blocks = kAbsmaxMaxBlocks;
    if (blocks < 1) blocks = 1;
    const int area = (int)((reinterpret_cast<uintptr_t>(out) >> 2) % kAbsmaxSlots);
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kAbsmaxThreads), 0, stream, reinterpret_cast<unsigned*>(out), area,
                       reinterpret_cast<const uint4*>(in), nvec, in + nvec * elems_per_vec, ntail);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

}  // namespace llmq

extern "C" int llmq_abs_max_bf16(float* out, const uint16_t* in, int64_t n, void* stream) {
    return llmq::launch_absmax(llmq::absmax_bf16_kernel<8, false>, out, in, n, 8, 8, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_abs_max_f32(float* out, const float* in, int64_t n, void* stream) {
    return llmq::launch_absmax(llmq::absmax_f32_kernel<8>, out, reinterpret_cast<const uint32_t*>(in), n, 4, 8,
                               static_cast<hipStream_t>(stream));
}
