// e4m3 x e4m3 TN GEMM for gfx950 (CDNA4) with fp32 accumulation and a scaled bf16 / fp32 epilogue.
//
// Interface semantics follow the reference's matmul for FP8 operands (src/kernels/matmul.cpp:47-153,
// 216-220; hand-written variant src/kernels/gemm_mma.cu:258-284): row-major a[M,K], b[N,K] (both K
// contiguous) produce row-major c[N,M],
//     c[n,m] = round( (sum_k b[n,k] a[m,k]) * (sa*sb) + bias[m] + (accumulate ? c[n,m] : 0) ).
//
// Kernel design (nothing here is derived from the reference's mma.sync kernel):
//   * one workgroup computes a BLK_N x BLK_M tile of c, K is walked in steps of 128 bytes;
//   * both operand tiles are staged in LDS, double buffered; with DMA == true the global->LDS copies
//     are 16-byte-per-lane direct-to-LDS loads (no VGPR staging), issued one K-step ahead;
//   * LDS rows are 128 bytes (one K-step) and the eight 16-byte chunks of a row are XOR-swizzled
//     with (row >> 1) & 7, which makes the 128-bit fragment reads of 16 consecutive rows hit all 64
//     banks exactly once; the swizzle is applied on the global side (each lane picks its source chunk)
//     because direct-to-LDS loads land linearly (lane i -> base + 16 i);
//   * the matrix instruction is v_mfma_f32_32x32x64_f8f6f4 (fp8 x fp8, K = 64 per instruction, two per
//     K-step); both operands use the same lane->K mapping, so any consistent mapping is correct;
//   * rows of the a-tile (the m / column index of c) are permuted on their way into LDS so that the NJ
//     accumulators a lane holds for one c row are NJ consecutive columns: the epilogue then stores
//     NJ packed outputs per lane and 32 lanes cover a contiguous row segment (256 B for bf16, NJ = 4);
//   * the linear workgroup id is remapped so that each of the 8 XCDs (workgroups are dealt to XCDs
//     round-robin) works on a contiguous range of tiles, walked in column-major groups of `group`
//     tile-rows for L2 reuse of both operands.
#include <type_traits>

#include "common.hpp"

namespace llmq {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kBK = 128;  // bytes (= e4m3 elements) of K per LDS stage

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename OutT> struct OutIo;
template <> struct OutIo<uint16_t> {
    static __device__ __forceinline__ float load(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }
    static __device__ __forceinline__ uint16_t cvt(float v) { return f32_to_bf16_rne(v); }
};
template <> struct OutIo<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ float cvt(float v) { return v; }
};

template <int NJ, typename OutT> struct Pack { OutT v[NJ]; } __attribute__((aligned(sizeof(OutT) * NJ)));

struct GemmArgs {
    void* c;
    const uint8_t* a;
    const uint8_t* b;
    const void* bias;
    const float* sa;
    const float* sb;
    int M, N, K;
    int bias_is_bf16;
    int accumulate;
    int group;  // tile-rows per rasterisation group
};

template <int BLK_N, int BLK_M, int WV_N, int WV_M, bool DMA, typename OutT>
__global__ __launch_bounds__(WV_N* WV_M * 64) void gemm_tn_e4m3_kernel(GemmArgs g) {
    constexpr int T = WV_N * WV_M * 64;
    constexpr int WT_N = BLK_N / WV_N, WT_M = BLK_M / WV_M;
    constexpr int NI = WT_N / 32, NJ = WT_M / 32;
    constexpr int P_BYTES = BLK_N * kBK, Q_BYTES = BLK_M * kBK, STAGE = P_BYTES + Q_BYTES;
    constexpr int P_ITERS = BLK_N * 8 / T, Q_ITERS = BLK_M * 8 / T;
    static_assert(BLK_N * 8 % T == 0 && BLK_M * 8 % T == 0, "tile chunks must divide evenly over the lanes");
    static_assert(T / 8 % 32 == 0, "row permutation assumes whole 32-row groups per load iteration");
    static_assert(NJ == 1 || NJ == 2 || NJ == 4, "packed epilogue width");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid % 64, wave = tid / 64;
    const int wn = wave / WV_M, wm = wave % WV_M;
    const int l32 = lane % 32, kg = lane / 32;

    // ---- workgroup -> tile (XCD-contiguous, grouped column-major walk) ----
    const int tiles_n = g.N / BLK_N, tiles_m = g.M / BLK_M;
    int tile_n, tile_m;
    {
        const int nwg = gridDim.x, wg = blockIdx.x;
        const int xcd = wg % 8, idx = wg / 8;
        const int q = nwg / 8, r = nwg % 8;
        const int logical = xcd * q + (xcd < r ? xcd : r) + idx;
        const int per_group = g.group * tiles_m;
        const int gid = logical / per_group;
        const int first_n = gid * g.group;
        const int gsz = (tiles_n - first_n) < g.group ? (tiles_n - first_n) : g.group;
        const int in_group = logical % per_group;
        tile_n = first_n + in_group % gsz;
        tile_m = in_group / gsz;
    }
    const int n_blk = tile_n * BLK_N, m_blk = tile_m * BLK_M;

    // ---- global -> LDS copy plan: chunk id = it*T + tid, LDS offset = 16 * chunk id (linear) ----
    const int ld_row = tid / 8;                         // + it * (T/8)
    const int ld_chunk = (tid & 7) ^ ((ld_row >> 1) & 7);  // logical 16-byte chunk this lane fetches
    const uint8_t* p_src = g.b + (int64_t)n_blk * g.K + (int64_t)ld_row * g.K + ld_chunk * 16;
    // a-tile row permutation: LDS row rho (within wave column w) holds global row NJ*(rho%32) + rho/32
    const uint8_t* q_src[Q_ITERS];
#pragma unroll
    for (int it = 0; it < Q_ITERS; ++it) {
        const int rho = it * (T / 8) + ld_row;
        const int w = rho / WT_M, rw = rho % WT_M;
        const int grow = w * WT_M + NJ * (rw % 32) + rw / 32;
        q_src[it] = g.a + (int64_t)m_blk * g.K + (int64_t)grow * g.K + ld_chunk * 16;
    }

    auto issue_loads = [&](int stage, int k0, uint4* regs) {
        uint8_t* base = lds + stage * STAGE;
#pragma unroll
        for (int it = 0; it < P_ITERS; ++it) {
            const uint8_t* src = p_src + (int64_t)it * (T / 8) * g.K + k0;
            if constexpr (DMA) {
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)src,
                    (__attribute__((address_space(3))) void*)(base + (it * T + wave * 64) * 16), 16, 0, 0);
            } else {
                regs[it] = *reinterpret_cast<const uint4*>(src);
            }
        }
#pragma unroll
        for (int it = 0; it < Q_ITERS; ++it) {
            const uint8_t* src = q_src[it] + k0;
            if constexpr (DMA) {
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)src,
                    (__attribute__((address_space(3))) void*)(base + P_BYTES + (it * T + wave * 64) * 16), 16, 0, 0);
            } else {
                regs[P_ITERS + it] = *reinterpret_cast<const uint4*>(src);
            }
        }
    };
    auto commit_loads = [&](int stage, const uint4* regs) {
        if constexpr (!DMA) {
            uint8_t* base = lds + stage * STAGE;
#pragma unroll
            for (int it = 0; it < P_ITERS; ++it)
                *reinterpret_cast<uint4*>(base + (it * T + tid) * 16) = regs[it];
#pragma unroll
            for (int it = 0; it < Q_ITERS; ++it)
                *reinterpret_cast<uint4*>(base + P_BYTES + (it * T + tid) * 16) = regs[P_ITERS + it];
        }
    };

    // ---- fragment read plan ----
    const int sw = (l32 >> 1) & 7;
    const int p_frag = (wn * WT_N + l32) * kBK;            // + ti*32*kBK
    const int q_frag = P_BYTES + (wm * WT_M + l32) * kBK;  // + tj*32*kBK

    v16f acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    uint4 regs[DMA ? 1 : (P_ITERS + Q_ITERS)];
    const int KT = g.K / kBK;

    issue_loads(0, 0, regs);
    commit_loads(0, regs);
    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) issue_loads(cur ^ 1, (kt + 1) * kBK, regs);
        const uint8_t* st = lds + cur * STAGE;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int c0 = ((4 * s + 2 * kg) ^ sw) * 16, c1 = ((4 * s + 2 * kg + 1) ^ sw) * 16;
            v8i fa[NI], fb[NJ];
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const v4i lo = *reinterpret_cast<const v4i*>(st + p_frag + i * 32 * kBK + c0);
                const v4i hi = *reinterpret_cast<const v4i*>(st + p_frag + i * 32 * kBK + c1);
                fa[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const v4i lo = *reinterpret_cast<const v4i*>(st + q_frag + j * 32 * kBK + c0);
                const v4i hi = *reinterpret_cast<const v4i*>(st + q_frag + j * 32 * kBK + c1);
                fb[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0, 0, 0, 0, 0);
        }
        if (kt + 1 < KT) commit_loads(cur ^ 1, regs);
        if constexpr (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // ---- epilogue: acc * (sa*sb) (+ bias[m]) (+ c) -> one rounding -> packed stores ----
    float scale = g.sa ? *g.sa : 1.f;
    if (g.sb) scale = scale * *g.sb;
    OutT* c = reinterpret_cast<OutT*>(g.c);
    const int m_lane = m_blk + wm * WT_M + NJ * l32;
    float bias_v[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        bias_v[j] = 0.f;
        if (g.bias) {
            bias_v[j] = g.bias_is_bf16
                            ? __uint_as_float((uint32_t) reinterpret_cast<const uint16_t*>(g.bias)[m_lane + j] << 16)
                            : reinterpret_cast<const float*>(g.bias)[m_lane + j];
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = n_blk + wn * WT_N + i * 32 + 8 * (r / 4) + 4 * kg + (r % 4);
            OutT* dst = c + (int64_t)n * g.M + m_lane;
            Pack<NJ, OutT> old, out;
            if (g.accumulate) old = *reinterpret_cast<const Pack<NJ, OutT>*>(dst);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                float t = acc[i][j][r] * scale;
                if (g.bias) t = t + bias_v[j];
                if (g.accumulate) t = t + OutIo<OutT>::load(&old.v[j]);
                out.v[j] = OutIo<OutT>::cvt(t);
            }
            *reinterpret_cast<Pack<NJ, OutT>*>(dst) = out;
        }
    }
}

// ---- software-pipelined variant ---------------------------------------------------------------------
// Same tiling, LDS layout and epilogue as above, with the K loop written as an explicit software
// pipeline over half-steps (K = 64, one matrix instruction deep).  Within a half-step the matrix
// instructions run row by row (a-fragment i against all b-fragments); as soon as row i has been
// issued its a-fragment registers are refilled from LDS for the next half-step, and the b-fragments
// of the next half-step go into a second small buffer.  LDS reads therefore stream under the matrix
// instructions with (NI + 2 NJ) fragment registers instead of a full double buffer.  The single
// workgroup barrier per K-step sits in the second half-step right after its first row has been
// queued: at that point every wave has finished reading the stage the next direct-to-LDS copies
// overwrite, and the stage fetched one step earlier has landed.
template <int MASK, int N>
__device__ __forceinline__ void sched_group() {
    if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
}

template <int BLK_N, int BLK_M, int WV_N, int WV_M, typename OutT>
__global__ __launch_bounds__(WV_N* WV_M * 64) void gemm_tn_e4m3_pipe_kernel(GemmArgs g) {
    constexpr int T = WV_N * WV_M * 64;
    constexpr int WT_N = BLK_N / WV_N, WT_M = BLK_M / WV_M;
    constexpr int NI = WT_N / 32, NJ = WT_M / 32;
    constexpr int P_BYTES = BLK_N * kBK, Q_BYTES = BLK_M * kBK, STAGE = P_BYTES + Q_BYTES;
    constexpr int P_ITERS = BLK_N * 8 / T, Q_ITERS = BLK_M * 8 / T, LOADS = P_ITERS + Q_ITERS;
    static_assert(T / 8 % 32 == 0 && (NJ == 1 || NJ == 2 || NJ == 4) && NI >= 2, "tile configuration");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wn = wave / WV_M, wm = wave % WV_M;
    const int l32 = lane % 32, kg = lane / 32;

    const int tiles_n = g.N / BLK_N, tiles_m = g.M / BLK_M;
    int tile_n, tile_m;
    {
        const int nwg = gridDim.x, wg = blockIdx.x;
        const int xcd = wg % 8, idx = wg / 8;
        const int q = nwg / 8, r = nwg % 8;
        const int logical = xcd * q + (xcd < r ? xcd : r) + idx;
        const int per_group = g.group * tiles_m;
        const int gid = logical / per_group;
        const int first_n = gid * g.group;
        const int gsz = (tiles_n - first_n) < g.group ? (tiles_n - first_n) : g.group;
        const int in_group = logical % per_group;
        tile_n = first_n + in_group % gsz;
        tile_m = in_group / gsz;
    }
    const int n_blk = tile_n * BLK_N, m_blk = tile_m * BLK_M;

    const int ld_row = tid / 8;
    const int ld_chunk = (tid & 7) ^ ((ld_row >> 1) & 7);
    const uint8_t* p_src = g.b + (int64_t)n_blk * g.K + (int64_t)ld_row * g.K + ld_chunk * 16;
    const uint8_t* q_src[Q_ITERS];
#pragma unroll
    for (int it = 0; it < Q_ITERS; ++it) {
        const int rho = it * (T / 8) + ld_row;
        const int w = rho / WT_M, rw = rho % WT_M;
        const int grow = w * WT_M + NJ * (rw % 32) + rw / 32;
        q_src[it] = g.a + (int64_t)m_blk * g.K + (int64_t)grow * g.K + ld_chunk * 16;
    }
    auto issue_loads = [&](int stage, int k0) {
        uint8_t* base = lds + stage * STAGE + wave * 1024;
#pragma unroll
        for (int it = 0; it < P_ITERS; ++it)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(p_src + (int64_t)it * (T / 8) * g.K + k0),
                (__attribute__((address_space(3))) void*)(base + it * T * 16), 16, 0, 0);
#pragma unroll
        for (int it = 0; it < Q_ITERS; ++it)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(q_src[it] + k0),
                                             (__attribute__((address_space(3))) void*)(base + P_BYTES + it * T * 16), 16,
                                             0, 0);
    };

    const int sw = (l32 >> 1) & 7;
    const int p_frag = (wn * WT_N + l32) * kBK;
    const int q_frag = P_BYTES + (wm * WT_M + l32) * kBK;
    // byte offsets of the two 16-byte chunks a lane reads in half-step 0 / 1
    const int cofs[2][2] = {{((2 * kg) ^ sw) * 16, ((2 * kg + 1) ^ sw) * 16},
                            {((4 + 2 * kg) ^ sw) * 16, ((4 + 2 * kg + 1) ^ sw) * 16}};

    auto read_frag = [&](const uint8_t* row, int h) -> v8i {
        const v4i lo = *reinterpret_cast<const v4i*>(row + cofs[h][0]);
        const v4i hi = *reinterpret_cast<const v4i*>(row + cofs[h][1]);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };

    v16f acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int KT = g.K / kBK;
    issue_loads(0, 0);
    if (KT > 1) {
        issue_loads(1, kBK);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();

    v8i fa[NI], fb[2][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i) fa[i] = read_frag(lds + p_frag + i * 32 * kBK, 0);
#pragma unroll
    for (int j = 0; j < NJ; ++j) fb[0][j] = read_frag(lds + q_frag + j * 32 * kBK, 0);

    // One half-step.  H: which half (selects the b-fragment buffer); NEXT: another half-step follows
    // and its fragments are read from `next`; SYNC: barrier after the first row (the following
    // half-step lives in the other LDS stage); REFILL: start the direct-to-LDS copies of the stage
    // after that one into the stage just released.
    auto half_step = [&](auto h_tag, auto next_tag, auto sync_tag, auto refill_tag, const uint8_t* next,
                         int refill_stage, int refill_k0) {
        constexpr int H = decltype(h_tag)::value;
        constexpr bool NEXT = decltype(next_tag)::value;
        constexpr bool SYNC = decltype(sync_tag)::value;
        constexpr bool REFILL = decltype(refill_tag)::value;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[H][j], acc[i][j], 0, 0, 0, 0, 0, 0);
            if (i == 0) {
                if constexpr (SYNC) {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                    if constexpr (REFILL) issue_loads(refill_stage, refill_k0);
                }
                if constexpr (NEXT) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) fb[H ^ 1][j] = read_frag(next + q_frag + j * 32 * kBK, H ^ 1);
                }
            }
            if constexpr (NEXT) fa[i] = read_frag(next + p_frag + i * 32 * kBK, H ^ 1);
        }
        // issue order inside the half-step: NJ matrix instructions, then the LDS reads (and a share of
        // the global->LDS loads) written after them
        if constexpr (NEXT && !SYNC) {
            sched_group<0x008, NJ>();
            sched_group<0x100, 2 * NJ + 2>();
#pragma unroll
            for (int i = 1; i < NI; ++i) {
                sched_group<0x008, NJ>();
                sched_group<0x100, 2>();
            }
        } else if constexpr (NEXT && SYNC) {
            constexpr int LD = REFILL ? LOADS : 0;
            constexpr int L0 = LD - (LD / NI) * (NI - 1);
            sched_group<0x020, L0>();
            sched_group<0x100, 2 * NJ + 2>();
#pragma unroll
            for (int i = 1; i < NI; ++i) {
                sched_group<0x008, NJ>();
                sched_group<0x100, 2>();
                sched_group<0x020, LD / NI>();
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    constexpr integral_constant<int, 0> H0{};
    constexpr integral_constant<int, 1> H1{};
    constexpr integral_constant<bool, true> Y{};
    constexpr integral_constant<bool, false> NO{};
    int kt = 0;
    for (; kt + 2 < KT; ++kt) {  // steady state: a next stage exists and one more can be fetched
        half_step(H0, Y, NO, NO, lds + (kt & 1) * STAGE, 0, 0);
        half_step(H1, Y, Y, Y, lds + ((kt + 1) & 1) * STAGE, kt & 1, (kt + 2) * kBK);
    }
    if (kt + 1 < KT) {           // second to last stage: nothing left to fetch
        half_step(H0, Y, NO, NO, lds + (kt & 1) * STAGE, 0, 0);
        half_step(H1, Y, Y, NO, lds + ((kt + 1) & 1) * STAGE, 0, 0);
        ++kt;
    }
    half_step(H0, Y, NO, NO, lds + (kt & 1) * STAGE, 0, 0);   // last stage
    half_step(H1, NO, NO, NO, lds, 0, 0);

    float scale = g.sa ? *g.sa : 1.f;
    if (g.sb) scale = scale * *g.sb;
    OutT* c = reinterpret_cast<OutT*>(g.c);
    const int m_lane = m_blk + wm * WT_M + NJ * l32;
    float bias_v[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        bias_v[j] = 0.f;
        if (g.bias) {
            bias_v[j] = g.bias_is_bf16
                            ? __uint_as_float((uint32_t) reinterpret_cast<const uint16_t*>(g.bias)[m_lane + j] << 16)
                            : reinterpret_cast<const float*>(g.bias)[m_lane + j];
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = n_blk + wn * WT_N + i * 32 + 8 * (r / 4) + 4 * kg + (r % 4);
            OutT* dst = c + (int64_t)n * g.M + m_lane;
            Pack<NJ, OutT> old, out;
            if (g.accumulate) old = *reinterpret_cast<const Pack<NJ, OutT>*>(dst);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                float t = acc[i][j][r] * scale;
                if (g.bias) t = t + bias_v[j];
                if (g.accumulate) t = t + OutIo<OutT>::load(&old.v[j]);
                out.v[j] = OutIo<OutT>::cvt(t);
            }
            *reinterpret_cast<Pack<NJ, OutT>*>(dst) = out;
        }
    }
}

template <int BLK_N, int BLK_M, int WV_N, int WV_M, typename OutT>
static int launch_pipe(const GemmArgs& g, hipStream_t stream) {
    const int tiles = (g.N / BLK_N) * (g.M / BLK_M);
    hipLaunchKernelGGL((gemm_tn_e4m3_pipe_kernel<BLK_N, BLK_M, WV_N, WV_M, OutT>), dim3((unsigned)tiles),
                       dim3(WV_N * WV_M * 64), 0, stream, g);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// ---- host side ------------------------------------------------------------------------------------
template <int BLK_N, int BLK_M, int WV_N, int WV_M, bool DMA, typename OutT>
static int launch_cfg(const GemmArgs& g, hipStream_t stream) {
    const int tiles = (g.N / BLK_N) * (g.M / BLK_M);
    hipLaunchKernelGGL((gemm_tn_e4m3_kernel<BLK_N, BLK_M, WV_N, WV_M, DMA, OutT>), dim3((unsigned)tiles),
                       dim3(WV_N * WV_M * 64), 0, stream, g);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// Variant selector: 0 = automatic.  Non-zero values pick one instantiation explicitly (used by the
// tuning harness and the tests to cover every instantiation).
int g_gemm_variant = 0;

template <typename OutT>
static int gemm_dispatch(GemmArgs g, hipStream_t stream) {
    LLMQ_REQUIRE(g.M > 0 && g.N > 0 && g.K > 0, "matmul: M, N, K must be positive (got %d, %d, %d)", g.M, g.N, g.K);
    LLMQ_REQUIRE(g.M % 128 == 0 && g.N % 128 == 0 && g.K % 128 == 0,
                 "matmul: M, N, K must be divisible by 128 (got %d, %d, %d)", g.M, g.N, g.K);
    LLMQ_REQUIRE(g.a && g.b && g.c, "matmul: null operand pointer");
    LLMQ_REQUIRE(aligned16(g.a) && aligned16(g.b) && aligned16(g.c) && aligned16(g.bias),
                 "matmul: all pointers must be 16-byte aligned");
    g.group = 8;
    int variant = g_gemm_variant;
    if (variant == 0) {
        const bool n256 = g.N % 256 == 0, m256 = g.M % 256 == 0;
        const int64_t tiles256 = (int64_t)(g.N / 256) * (g.M / 256);
        if (n256 && m256 && tiles256 >= cu_count()) variant = 6;
        else variant = 3;
    }
    switch (variant) {
        case 1: return launch_cfg<256, 256, 2, 4, true, OutT>(g, stream);
        case 2: return launch_cfg<256, 256, 2, 4, false, OutT>(g, stream);
        case 3: return launch_cfg<128, 128, 2, 2, true, OutT>(g, stream);
        case 4: return launch_cfg<128, 128, 2, 2, false, OutT>(g, stream);
        case 5: return launch_cfg<256, 256, 2, 2, true, OutT>(g, stream);
        case 6: return launch_pipe<256, 256, 2, 4, OutT>(g, stream);
        case 7: return launch_pipe<256, 256, 2, 2, OutT>(g, stream);
        case 8: return launch_pipe<128, 128, 2, 2, OutT>(g, stream);
        default: return set_error(LLMQ_ERR_INVALID_ARGUMENT, "matmul: unknown kernel variant %d", variant);
    }
}

}  // namespace llmq

extern "C" int llmq_gemm_tn_e4m3_bf16(uint16_t* c, const uint8_t* a, const uint8_t* b, const uint16_t* bias_or_null,
                                      const float* sa_or_null, const float* sb_or_null, int M, int N, int K,
                                      int accumulate, void* stream) {
    llmq::GemmArgs g{c, a, b, bias_or_null, sa_or_null, sb_or_null, M, N, K, 1, accumulate, 8};
    return llmq::gemm_dispatch<uint16_t>(g, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_gemm_tn_e4m3_f32(float* c, const uint8_t* a, const uint8_t* b, const void* bias_or_null,
                                     int bias_is_bf16, const float* sa_or_null, const float* sb_or_null, int M, int N,
                                     int K, int accumulate, void* stream) {
    llmq::GemmArgs g{c, a, b, bias_or_null, sa_or_null, sb_or_null, M, N, K, bias_is_bf16, accumulate, 8};
    return llmq::gemm_dispatch<float>(g, static_cast<hipStream_t>(stream));
}

// Tuning / test hook (not part of the drop-in surface): force a kernel instantiation, 0 = automatic.
extern "C" void llmq_debug_set_gemm_variant(int v) { llmq::g_gemm_variant = v; }
