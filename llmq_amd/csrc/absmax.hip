// Per-tensor abs-max reduction for gfx950.
//
// Semantics follow the reference's reduce_abs_max_kernel (src/kernels/quant.cu:11-28) and
// handle_absmax_reduction (src/kernels/kernel_utils.cuh:17-32): *result = max_i |in[i]| as fp32,
// NaNs ignored, result >= +0, slot reset before the reduction.  The result is order independent, so
// it is bit exact by construction.
//
// Design: HBM-bound streaming read (2 bytes per element).  A grid of at most four 512-lane workgroups per compute unit
// walks the tensor in chunks of 32 KiB per workgroup (chunk c of workgroup b is number b + c * grid; each lane has
// UNROLL independent 128-bit loads per chunk, every wave instruction covers 1 KiB contiguous), with the next chunk's
// loads in flight while the current one is folded with packed 16-bit integer ops; then wave shuffle -> LDS -> one
// value per workgroup.
//
// One launch per call.  The reference clears the slot with a memset and lets every block merge into it with an atomic
// max (two stream operations).  Here the workgroups meet in an arrival area built into the device code: a workgroup
// merges its maximum into a running maximum there (skipped when the value it read from there at its start is already
// as large), counts itself in, and the workgroup that arrives last stores the running maximum to the caller's slot (a
// plain store: the slot needs no clearing) and leaves the area zeroed for the next call.  Nobody waits for anybody.
// There are LLMQ_ABS_MAX_ARRIVAL_AREAS independent areas; a call uses the one selected by its result address
// ((address / 4) % areas), so calls with neighbouring result slots (the reference keeps [abs_max, scale] pairs in
// per-layer tables) use different areas.  Calls on one stream run one after the other and can share an area; calls that
// overlap in time on one GPU (different streams without an ordering between them) must not map to the same area --
// the documented limit of this entry point.
//
// The fold works on bit patterns: for a bf16 pattern p, a = p & 0x7FFF is |x|'s pattern and
// y = 0x7F80 - a (mod 2^16) is <= 0x7F80 for every non-NaN value and >= 0xFF81 for every NaN.
// min over y therefore ignores NaNs and finds the largest |x|; the start value 0x7F80 encodes 0.
#include "common.hpp"
#include "absmax_reduce.hpp"

namespace llmq {

// Measured on 310 MB tensors that no cache holds (back-to-back launches over three tensors): 1024 lanes x 8 loads, one
// chunk per workgroup 55.8 us; 512 x 4 with the pipelined walk and 4 workgroups per compute unit 53.3 us (a plain
// read-only kernel: 49.6 us); smaller workgroups without the walk lose to the arrival traffic (256 x 8: 63.6 us).
constexpr int kAbsmaxThreads = 512;
constexpr int kAbsmaxUnroll = 4;
constexpr int kAbsmaxGroupsPerCu = 4;

// Arrival areas, kAbsmaxAreaWords words each, every used word on a 128-byte line of its own: word 0 the top arrival
// counter, word 32 the top running maximum, words 64 + 32 l / 1024 + 32 l the arrival counter / running maximum of
// lane l.  Workgroup b belongs to lane b % kAbsmaxLanes (one counter for all workgroups would serialise their
// arrivals on one address); the workgroup that completes a lane's quota moves the lane's maximum to the top and counts
// the lane in; the one that completes the top counter is the last of the grid.  Every word is zero whenever no call is
// using the area: zero-initialised with the module, set back by the workgroup that completes it.
constexpr int kAbsmaxSlots = LLMQ_ABS_MAX_ARRIVAL_AREAS;
constexpr int kAbsmaxLanes = 16;
constexpr int kAbsmaxAreaWords = 2048;
static __device__ __align__(256) unsigned absmax_areas[kAbsmaxSlots * kAbsmaxAreaWords];

// Device-scope read-modify-writes whose returned value is waited for before anything else is issued.  Memory ordering
// without cache maintenance rests on that: such an operation is performed where all XCDs meet and is complete when its
// value is back, so a workgroup's maximum is in place before its arrival is counted, and whoever sees the last count
// sees every maximum.  (Release / acquire fences at device scope would do the same by writing back and invalidating
// the whole L2 of the XCD for every workgroup: measured at half the bandwidth.)  The returned value is an operand of an
// asm statement with a memory clobber: the returning form of the instruction is used and no later memory operation is
// moved in front of it.
__device__ __forceinline__ unsigned rmw_returned(unsigned v) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(v) : : "memory");
    return v;
}
__device__ __forceinline__ unsigned rmw_exchange(unsigned* p, unsigned v) {
    return rmw_returned(__hip_atomic_exchange(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ unsigned rmw_add(unsigned* p, unsigned v) {
    return rmw_returned(__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ unsigned rmw_max(unsigned* p, unsigned v) {
    return rmw_returned(__hip_atomic_fetch_max(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

// The running maximum of this workgroup's lane as it stands when the workgroup starts (lane 0 of the workgroup; the
// latency hides behind the first chunk's loads).  It only grows during a call, so a stale value is safe.
__device__ __forceinline__ unsigned arrival_seen(int area) {
    if (threadIdx.x != 0 || gridDim.x == 1) return 0u;
    return __hip_atomic_load(absmax_areas + (size_t)area * kAbsmaxAreaWords + 1024 + 32 * (blockIdx.x % kAbsmaxLanes),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Finish of a single-launch abs-max: `bits` is this lane's candidate (fp32 pattern of a non-negative value; patterns of
// non-negative floats order like the values), `seen` what arrival_seen returned.  Grids of one workgroup store directly.
__device__ __forceinline__ void block_max_last_arriver(unsigned* result, int area, uint32_t bits, unsigned seen) {
    __shared__ uint32_t wave_max[16];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = __shfl_xor(bits, off, kWave);
        bits = o > bits ? o : bits;
    }
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) wave_max[wave] = bits;
    __syncthreads();
    if (wave != 0) return;
    uint32_t v = lane < (int)blockDim.x / kWave ? wave_max[lane] : 0u;
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
        const uint32_t o = __shfl_xor(v, off, kWave);
        v = o > v ? o : v;
    }
    if (lane != 0) return;
    const unsigned grid = gridDim.x;
    if (grid == 1) {
        *result = v;
        return;
    }
    unsigned* const words = absmax_areas + (size_t)area * kAbsmaxAreaWords;
    const unsigned l = blockIdx.x % kAbsmaxLanes;
    unsigned* const lane_counter = words + 64 + 32 * l;
    unsigned* const lane_maximum = words + 1024 + 32 * l;
    if (v > seen) rmw_max(lane_maximum, v);                      // in place before the count below
    const unsigned quota = grid / kAbsmaxLanes + (l < grid % kAbsmaxLanes ? 1u : 0u);
    if (rmw_add(lane_counter, 1u) != quota - 1) return;
    // this lane is complete (nobody else touches its words now): move its maximum to the top, leave the lane zeroed
    const unsigned lane_max = rmw_exchange(lane_maximum, 0u);
    rmw_exchange(lane_counter, 0u);
    rmw_max(words + 32, lane_max);
    const unsigned lanes_in_use = grid < (unsigned)kAbsmaxLanes ? grid : (unsigned)kAbsmaxLanes;
    if (rmw_add(words, 1u) != lanes_in_use - 1) return;
    rmw_exchange(words, 0u);                                     // the area is free again
    *result = rmw_exchange(words + 32, 0u);
}

// Chunk walk shared by the two element types: fold(v) is applied to every 16-byte vector of the tensor once.  Slots
// beyond the end read as zeros (|0| never changes a maximum).
template <typename Fold>
__device__ __forceinline__ void walk_chunks(const uint4* __restrict__ in, int64_t nvec, Fold&& fold) {
    constexpr int64_t kChunk = (int64_t)kAbsmaxThreads * kAbsmaxUnroll;
    const int64_t chunks = (nvec + kChunk - 1) / kChunk;
    uint4 cur[kAbsmaxUnroll], nxt[kAbsmaxUnroll];
    auto load = [&](uint4* v, int64_t c) {
#pragma unroll
        for (int u = 0; u < kAbsmaxUnroll; ++u) {
            const int64_t idx = c * kChunk + u * kAbsmaxThreads + threadIdx.x;
            v[u] = (c < chunks && idx < nvec) ? in[idx] : make_uint4(0, 0, 0, 0);
        }
    };
    int64_t c = blockIdx.x;
    load(cur, c);
    while (c < chunks) {
        load(nxt, c + gridDim.x);
#pragma unroll
        for (int u = 0; u < kAbsmaxUnroll; ++u) fold(cur[u]);
#pragma unroll
        for (int u = 0; u < kAbsmaxUnroll; ++u) cur[u] = nxt[u];
        c += gridDim.x;
    }
}

__global__ __launch_bounds__(kAbsmaxThreads) void absmax_bf16_kernel(unsigned* __restrict__ result, int area,
                                                                     const uint4* __restrict__ in, int64_t nvec,
                                                                     const uint16_t* __restrict__ tail, int ntail) {
    const unsigned seen = arrival_seen(area);
    uint32_t acc = 0x7F807F80u;
    walk_chunks(in, nvec, [&](const uint4& v) { acc = fold_vec(acc, v); });
    if (blockIdx.x == 0 && (int)threadIdx.x < ntail) acc = fold_bf16x2(acc, (uint32_t)tail[threadIdx.x]);
    const uint32_t lo = acc & 0xFFFFu, hi = acc >> 16;
    block_max_last_arriver(result, area, (0x7F80u - (lo < hi ? lo : hi)) << 16, seen);
}

__global__ __launch_bounds__(kAbsmaxThreads) void absmax_f32_kernel(unsigned* __restrict__ result, int area,
                                                                    const uint4* __restrict__ in, int64_t nvec,
                                                                    const uint32_t* __restrict__ tail, int ntail) {
    const unsigned seen = arrival_seen(area);
    uint32_t acc = 0x7F800000u;
    auto fold = [&](uint32_t w) {
        uint32_t y = 0x7F800000u - (w & 0x7FFFFFFFu);  // wraps to a huge value for NaN
        acc = y < acc ? y : acc;
    };
    walk_chunks(in, nvec, [&](const uint4& v) { fold(v.x); fold(v.y); fold(v.z); fold(v.w); });
    if (blockIdx.x == 0 && (int)threadIdx.x < ntail) fold(tail[threadIdx.x]);
    block_max_last_arriver(result, area, 0x7F800000u - acc, seen);
}

template <typename Kernel, typename Elem>
static int launch_absmax(Kernel kernel, float* out, const Elem* in, int64_t n, int elems_per_vec, hipStream_t stream) {
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
    const int64_t per_chunk = (int64_t)kAbsmaxThreads * kAbsmaxUnroll;
    int64_t blocks = (nvec + per_chunk - 1) / per_chunk;
    const int64_t resident = (int64_t)kAbsmaxGroupsPerCu * cu_count();
    if (blocks > resident) blocks = resident;
    if (blocks < 1) blocks = 1;
    const int area = (int)((reinterpret_cast<uintptr_t>(out) >> 2) % kAbsmaxSlots);
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kAbsmaxThreads), 0, stream, reinterpret_cast<unsigned*>(out), area,
                       reinterpret_cast<const uint4*>(in), nvec, in + nvec * elems_per_vec, ntail);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

}  // namespace llmq

extern "C" int llmq_abs_max_bf16(float* out, const uint16_t* in, int64_t n, void* stream) {
    return llmq::launch_absmax(llmq::absmax_bf16_kernel, out, in, n, 8, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_abs_max_f32(float* out, const float* in, int64_t n, void* stream) {
    return llmq::launch_absmax(llmq::absmax_f32_kernel, out, reinterpret_cast<const uint32_t*>(in), n, 4,
                               static_cast<hipStream_t>(stream));
}
