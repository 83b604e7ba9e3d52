// Abs-max folding of bf16 bit patterns and the workgroup -> global slot reduction, shared by the abs-max
// kernel and by the producers that compute an abs-max of their own output on the way
// (semantics: src/kernels/kernel_utils.cuh:17-32 -- NaNs ignored, result >= +0, order independent).
//
// The fold works on bit patterns: for a bf16 pattern p, a = p & 0x7FFF is |x|'s pattern and
// y = 0x7F80 - a (mod 2^16) is <= 0x7F80 for every non-NaN value and >= 0xFF81 for every NaN.
// min over y therefore ignores NaNs and finds the largest |x|; the start value 0x7F80 encodes 0.
#pragma once

#include "common.hpp"

namespace llmq {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t fold_bf16x2(uint32_t acc, uint32_t w) {
    u16x2 a = __builtin_bit_cast(u16x2, w & 0x7FFF7FFFu);
    u16x2 y = (u16x2)(0x7F80) - a;
    u16x2 m = __builtin_elementwise_min(__builtin_bit_cast(u16x2, acc), y);
    return __builtin_bit_cast(uint32_t, m);
}

__device__ __forceinline__ uint32_t fold_vec(uint32_t acc, const uint4& v) {
    acc = fold_bf16x2(acc, v.x);
    acc = fold_bf16x2(acc, v.y);
    acc = fold_bf16x2(acc, v.z);
    acc = fold_bf16x2(acc, v.w);
    return acc;
}

// Block-level finish shared by the bf16 and fp32 kernels: `y` is "limit - |x| pattern" (smaller is
// larger |x|), `limit` the pattern of +Inf in that width, `shift` moves it to fp32 bit positions.
__device__ __forceinline__ void block_min_to_atomic_max(unsigned* result, uint32_t y, uint32_t limit, int shift) {
    __shared__ uint32_t wave_min[16];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        uint32_t o = __shfl_xor(y, off, kWave);
        y = o < y ? o : y;
    }
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) wave_min[wave] = y;
    __syncthreads();
    if (wave == 0) {
        const int nw = blockDim.x / kWave;
        y = lane < nw ? wave_min[lane] : limit;
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
            uint32_t o = __shfl_xor(y, off, kWave);
            y = o < y ? o : y;
        }
        if (lane == 0) {
            // Non-negative floats order like their bit patterns.  The slot only ever grows, so a block
            // whose maximum does not exceed the value already there skips the atomic, which would serialise
            // with those of all other blocks (reading the slot early instead, at the start of the kernel,
            // was measured: most blocks then see a stale 0 and the atomics cost a third of the bandwidth).
            uint32_t bits = (limit - y) << shift;
            if (bits > __atomic_load_n(result, __ATOMIC_RELAXED)) atomicMax(result, bits);
        }
    }
}

// Resets an abs-max slot: a one-lane fill kernel rather than a memset node, safe to record into a HIP graph.
__attribute__((unused)) static __global__ void reset_slot_kernel(unsigned* slot) { *slot = 0u; }

}  // namespace llmq
