// e4m3 x e4m3 (or x e5m2) GEMM for gfx950 (CDNA4) with fp32 accumulation and a scaled bf16 / fp32 epilogue.
//
// Interface semantics follow the reference's matmul for FP8 operands (src/kernels/matmul.cpp:47-153,
// 216-220; hand-written variant src/kernels/gemm_mma.cu:258-284): row-major a[M,K], b[N,K] (both K
// contiguous, mode TN) produce row-major c[N,M],
//     c[n,m] = round( (sum_k b[n,k] a[m,k]) * (sa*sb) + bias[m] + (accumulate ? c[n,m] : 0) ).
// For bf16 output the operands may also be stored K-major (a as [K,M], b as [K,N]: the reference's modes NN, TT, NT).
//
// Kernel design (nothing here is derived from the reference's mma.sync kernel).  Three kernels; the two tiled ones
// share the tiling, the LDS layout and the copy scheme; each has its own description further down:
//   * gemm_tn_e4m3_w4_kernel: 256 x 256 (or 256 x 224 / 192) tile, 4 waves of 128 x 128, v_mfma_f32_16x16x128_f8f6f4,
//     persistent; the default whenever M, N fit those tiles and K is a multiple of 128 from 256 up; also the K-major
//     operand modes and the K segments of a cut last round;
//   * gemm_tn_e4m3_pipe_kernel: 256 x 256 tile with 8 waves of 128 x 64 or 128 x 128 tile with 4 waves
//     of 64 x 64, v_mfma_f32_32x32x64_f8f6f4; the other shapes on the 128 lattice, and the split-K path;
//   * gemm_tn_e4m3_edge_kernel: 64 x 64 tile with predicated loads and stores: small shapes off the lattice (any M, N; K
//     a multiple of 16) and the last N % tile rows of the others; large shapes off the lattice run on RAGGED instances
//     of the four-wave kernel (last tile row / column moved back into the matrix, K tail masked in the copies).
// Common to the tiled kernels:
//   * one workgroup computes a tile of c, K is walked in steps of 128 bytes;
//   * both operand tiles are staged in LDS, double buffered, by 16-byte-per-lane direct-to-LDS loads
//     (no VGPR staging);
//   * LDS rows are 128 bytes (one K-step) and the eight 16-byte chunks of a row are XOR-swizzled with a function of
//     the row that makes the 128-bit fragment reads conflict-free for the kernel's lane -> row mapping ((row >> 1) & 7
//     for the 32x32x64 fragments, frag_swizzle() for the 16x16x128 ones); the swizzle is applied on the global side
//     (each lane picks its source chunk) because direct-to-LDS loads land linearly (lane i -> base + 16 i);
//   * both operands of the matrix instruction use the same lane->K mapping, so any consistent mapping
//     is correct;
//   * rows of the a-tile (the m / column index of c) are permuted on their way into LDS so that the
//     accumulators a lane holds for one c row are consecutive columns: the epilogue stores packed
//     groups and neighbouring lanes cover a contiguous row segment;
//   * the linear workgroup id is remapped so that each XCD (workgroups are dealt to the XCDs round-robin; their
//     number is a launch argument) works on a contiguous range of tiles, walked in column-major groups of `group`
//     tile-rows for L2 reuse of both operands.
// The 8-wave kernel's K loop is an explicit software pipeline over half-steps (K = 64, one matrix
// instruction deep).  Within a half-step the matrix instructions run row by row (b-rows fragment i
// against all a-rows fragments); as soon as row i has been issued its fragment registers are refilled
// from LDS for the next half-step, and the other operand's fragments of the next half-step go into a
// second small buffer.  LDS reads therefore stream under the matrix instructions with (NI + 2 NJ)
// fragment registers instead of a full double buffer.  The single workgroup barrier per K-step sits in
// the second half-step right after its first row has been queued: at that point every wave has
// finished reading the stage the next direct-to-LDS copies overwrite, and the stage fetched one step
// earlier has landed.  Shapes with too few output tiles to fill the chip (weight gradients of small
// layers) split K over gridDim.y: every split writes its raw fp32 accumulators to a slice of the
// caller's workspace, and a second kernel adds the slices in a fixed order and applies the epilogue, so
// the result does not depend on scheduling.
#include <atomic>
#include <type_traits>

#include "common.hpp"

namespace llmq {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int kBK = 128;  // bytes (= e4m3 elements) of K per LDS stage

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
    int group;       // tile-rows per rasterisation group
    float* partial;  // split-K only: [splits][N][M] raw accumulators (four-wave kernel: 256 x 256 tiles)
    int k_len;       // split-K only: K elements per split (multiple of 128; four-wave kernel: of 256)
    int rem_split;   // four-wave kernel: K segments per tile of an XCD's last, partial round (1 = none)
    int part_per_xcd;  // four-wave kernel: partial tiles reserved per XCD in `partial`
    int xcds;          // accelerator dies of the device (workgroup ids are dealt to them round-robin)
    int n_first;       // general-shape kernel: first c row of the region it covers (rows n_first .. N - 1)
};

// XCD x owns a contiguous range of the logical tile sequence (the first total % xcds XCDs one tile more).
__device__ __forceinline__ void xcd_tile_range(int total, int xcds, int xcd, int& first, int& count) {
    const int xq = total / xcds, xr = total % xcds;
    first = xcd * xq + (xcd < xr ? xcd : xr);
    count = xq + (xcd < xr ? 1 : 0);
}

// Logical tile number -> tile origin: groups of `group` tile-rows, column-major inside a group.
// Tiles are 256 rows (n) by BM columns (m).
// RAGGED: N and M need not be multiples of the tile: the tile counts round up and the last tile row / column is
// moved back so that it ends with the matrix (its first rows / columns then repeat those of its neighbour).
template <int BM = 256, bool RAGGED = false>
__device__ __forceinline__ void decode_tile256(const GemmArgs& g, int logical, int& n_blk, int& m_blk) {
    const int tiles_n = RAGGED ? (g.N + 255) / 256 : g.N / 256, tiles_m = RAGGED ? (g.M + BM - 1) / BM : g.M / BM;
    const int per_group = g.group * tiles_m;
    const int gid = logical / per_group;
    const int first_n = gid * g.group;
    const int gsz = (tiles_n - first_n) < g.group ? (tiles_n - first_n) : g.group;
    const int in_group = logical % per_group;
    n_blk = (first_n + in_group % gsz) * 256;
    m_blk = (in_group / gsz) * BM;
    if constexpr (RAGGED) {
        if (n_blk > g.N - 256) n_blk = g.N - 256;
        if (m_blk > g.M - BM) m_blk = g.M - BM;
    }
}

#define LLMQ_GLOBAL __attribute__((address_space(1)))

// Pair of adjacent outputs in global memory: load as fp32, store with one rounding to the output type.
template <typename OutT> struct PairIo;
template <> struct PairIo<uint16_t> {
    static __device__ __forceinline__ void load(const LLMQ_GLOBAL void* p, float& v0, float& v1) {
        const uint32_t old = *(const LLMQ_GLOBAL uint32_t*)p;
        v0 = __uint_as_float(old << 16);
        v1 = __uint_as_float(old & 0xFFFF0000u);
    }
    static __device__ __forceinline__ void store(LLMQ_GLOBAL void* p, float v0, float v1) {
        const f32x2_t v = {v0, v1};
        *(LLMQ_GLOBAL bf16x2_t*)p = __builtin_convertvector(v, bf16x2_t);  // v_cvt_pk_bf16_f32, RNE
    }
};
template <> struct PairIo<float> {
    static __device__ __forceinline__ void load(const LLMQ_GLOBAL void* p, float& v0, float& v1) {
        const f32x2_t old = *(const LLMQ_GLOBAL f32x2_t*)p;
        v0 = old[0];
        v1 = old[1];
    }
    static __device__ __forceinline__ void store(LLMQ_GLOBAL void* p, float v0, float v1) {
        const f32x2_t v = {v0, v1};
        *(LLMQ_GLOBAL f32x2_t*)p = v;
    }
};

__device__ __forceinline__ float load_bias(const void* bias, int is_bf16, int m) {
    return is_bf16 ? __uint_as_float((uint32_t) reinterpret_cast<const uint16_t*>(bias)[m] << 16)
                   : reinterpret_cast<const float*>(bias)[m];
}

// Hides a value from loop-invariant code motion: lane-derived constants that are only needed between
// tiles are recomputed from the lane id there instead of occupying registers across the K loop.
__device__ __forceinline__ int opaque(int x) {
    asm volatile("" : "+v"(x));
    return x;
}

// Pins a wave-uniform pointer in scalar registers, so that "pointer + 32-bit lane offset" selects the
// scalar-base addressing form instead of a 64-bit vector add per access.
__device__ __forceinline__ LLMQ_GLOBAL char* scalar_ptr(LLMQ_GLOBAL char* p) {
    asm volatile("" : "+s"(p));
    return p;
}

template <int MASK, int N>
__device__ __forceinline__ void sched_group() {
    if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
}

// Compile-time loop: f(integral_constant<int, B>{}), ..., f(integral_constant<int, E - 1>{}).
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// SPLIT: blockIdx.y selects a K range of g.k_len elements and the raw accumulators go to g.partial.
// B_FMT: fp8 format of the b operand (0 = e4m3, 1 = e5m2, the reference's gradient dtype option); b rows are
// the first operand of the matrix instruction, whose format field takes this value directly.
// PERSIST: the grid has one workgroup per compute unit and every workgroup walks a list of tiles.  The
// operand stream then runs across tile boundaries: the copies of the next tile's first two K-steps are
// issued during the last two K-steps of the current tile, so the epilogue of a tile overlaps with the
// fetch of the next one and no pipeline fill or workgroup launch sits between tiles.  Needs K >= 256.
// RAGGED: M, N and K need not be multiples of the tile (M a multiple of 8, K of 16).  Tile counts round up; a lane whose
// operand row lies beyond the matrix copies the matrix's last row instead (its products land in accumulators that are
// never stored), a lane whose 16-byte chunk lies beyond K copies a chunk of zeros, and the epilogue stores only what
// lies inside c.  Every lane still issues every copy, so the counters of the K loop hold as they are.
static __device__ uint4 ragged_zero_chunk;  // never written: 16 zero bytes in global memory

template <int BLK_N, int BLK_M, int WV_N, int WV_M, typename OutT, bool SPLIT, bool PERSIST, int B_FMT, bool RAGGED = false>
__global__ __launch_bounds__(WV_N* WV_M * 64) void gemm_tn_e4m3_pipe_kernel(GemmArgs g) {
    static_assert(!RAGGED || (!SPLIT && !PERSIST), "ragged shapes: one tile per workgroup, no K split");
    constexpr int T = WV_N * WV_M * 64;
    constexpr int WT_N = BLK_N / WV_N, WT_M = BLK_M / WV_M;
    constexpr int NI = WT_N / 32, NJ = WT_M / 32;
    constexpr int P_BYTES = BLK_N * kBK, Q_BYTES = BLK_M * kBK, STAGE = P_BYTES + Q_BYTES;
    constexpr int P_ITERS = BLK_N * 8 / T, Q_ITERS = BLK_M * 8 / T, LOADS = P_ITERS + Q_ITERS;
    static_assert(T / 8 % 32 == 0 && NJ == 2 && NI >= 2, "tile configuration");
    static_assert(!(SPLIT && PERSIST), "split-K tiles are not walked persistently");

    // two operand stages + 4 KiB per wave for the staged bf16 epilogue
    constexpr int EPI_BYTES = 4096;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * STAGE + WV_N * WV_M * EPI_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wn = wave / WV_M, wm = wave % WV_M;
    const int l32 = lane % 32, kg = lane / 32;

    const int tiles_n = RAGGED ? (g.N + BLK_N - 1) / BLK_N : g.N / BLK_N;
    const int tiles_m = RAGGED ? (g.M + BLK_M - 1) / BLK_M : g.M / BLK_M;
    // Tile order: XCD x (workgroups are dealt to XCDs round-robin) owns a contiguous range of the
    // "logical" tile sequence, which walks column-major groups of g.group tile-rows.
    const int total = tiles_n * tiles_m;
    const int xcd = blockIdx.x % g.xcds, slot = blockIdx.x / g.xcds;
    const int xq = (PERSIST ? total : (int)gridDim.x) / g.xcds, xr = (PERSIST ? total : (int)gridDim.x) % g.xcds;
    const int xcd_first = xcd * xq + (xcd < xr ? xcd : xr);
    auto decode = [&](int logical, int& n_blk, int& m_blk) {
        const int per_group = g.group * tiles_m;
        const int gid = logical / per_group;
        const int first_n = gid * g.group;
        const int gsz = (tiles_n - first_n) < g.group ? (tiles_n - first_n) : g.group;
        const int in_group = logical % per_group;
        n_blk = (first_n + in_group % gsz) * BLK_N;
        m_blk = (in_group / gsz) * BLK_M;
    };
    int my_tiles = 1, tile_stride = 0;
    if constexpr (PERSIST) {
        const int xcd_count = xq + (xcd < xr ? 1 : 0);
        tile_stride = gridDim.x / g.xcds;
        my_tiles = slot < xcd_count ? (xcd_count - slot + tile_stride - 1) / tile_stride : 0;
        if (my_tiles == 0) return;  // uniform for the whole workgroup, before any barrier
    }
    int logical = xcd_first + slot;
    int n_blk, m_blk;
    decode(logical, n_blk, m_blk);

    int k_begin = 0, k_count = g.K;
    if constexpr (SPLIT) {
        k_begin = blockIdx.y * g.k_len;
        k_count = (g.K - k_begin) < g.k_len ? (g.K - k_begin) : g.k_len;
    }

    // global source of every direct-to-LDS copy this lane issues for one K-step
    const uint8_t* p_src;
    const uint8_t* q_src[Q_ITERS];
    [[maybe_unused]] const uint8_t* p_rag[P_ITERS];  // RAGGED: one source per copy (rows are clamped one by one)
    [[maybe_unused]] int lane_k = 0;                 // RAGGED: offset of this lane's chunk within a K-step
    auto set_sources = [&](int nb, int mb) {
        const int t_id = PERSIST ? opaque(threadIdx.x) : tid;
        const int ld_row = t_id / 8;
        const int ld_chunk = (t_id & 7) ^ ((ld_row >> 1) & 7);
        p_src = g.b + (int64_t)nb * g.K + (int64_t)ld_row * g.K + ld_chunk * 16 + k_begin;
        if constexpr (RAGGED) {
            lane_k = ld_chunk * 16;
#pragma unroll
            for (int it = 0; it < P_ITERS; ++it) {
                int row = nb + it * (T / 8) + ld_row;
                row = row < g.N ? row : g.N - 1;
                p_rag[it] = g.b + (int64_t)row * g.K + ld_chunk * 16;
            }
        }
#pragma unroll
        for (int it = 0; it < Q_ITERS; ++it) {
            const int rho = it * (T / 8) + ld_row;
            const int w = rho / WT_M, rw = rho % WT_M;
            const int grow = w * WT_M + NJ * (rw % 32) + rw / 32;
            int row = mb + grow;
            if constexpr (RAGGED) row = row < g.M ? row : g.M - 1;
            q_src[it] = g.a + (int64_t)row * g.K + ld_chunk * 16 + k_begin;
        }
    };
    set_sources(n_blk, m_blk);
    auto issue_loads = [&](int stage_ofs, int k0) {
        uint8_t* base = lds + stage_ofs + wave * 1024;
        [[maybe_unused]] const bool beyond_k = RAGGED && k0 + lane_k >= g.K;
        [[maybe_unused]] const uint8_t* zeros = reinterpret_cast<const uint8_t*>(&ragged_zero_chunk);
#pragma unroll
        for (int it = 0; it < P_ITERS; ++it) {
            const uint8_t* src = p_src + (int64_t)it * (T / 8) * g.K + k0;
            if constexpr (RAGGED) src = beyond_k ? zeros : p_rag[it] + k0;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + it * T * 16), 16, 0, 0);
        }
#pragma unroll
        for (int it = 0; it < Q_ITERS; ++it) {
            const uint8_t* src = q_src[it] + k0;
            if constexpr (RAGGED) src = beyond_k ? zeros : src;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + P_BYTES + it * T * 16), 16,
                                             0, 0);
        }
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
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    };
    clear_acc();

    const int KT = RAGGED ? (k_count + kBK - 1) / kBK : k_count / kBK;
    issue_loads(0, 0);
    if (KT > 1) {
        issue_loads(STAGE, kBK);
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

    // One half-step.  H: which half (selects the second operand's fragment buffer); NEXT: another
    // half-step follows and its fragments are read from `next`; SYNC: barrier after the first row (the
    // following half-step lives in the other LDS stage); REFILL: start the direct-to-LDS copies of the
    // stage after that one into the stage just released.
    auto half_step = [&](auto h_tag, auto next_tag, auto sync_tag, auto refill_tag, const uint8_t* next,
                         int refill_ofs, int refill_k0) {
        constexpr int H = decltype(h_tag)::value;
        constexpr bool NEXT = decltype(next_tag)::value;
        constexpr bool SYNC = decltype(sync_tag)::value;
        constexpr bool REFILL = decltype(refill_tag)::value;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[H][j], acc[i][j], B_FMT, 0, 0, 0, 0, 0);
            if (i == 0) {
                if constexpr (SYNC) {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                    if constexpr (REFILL) issue_loads(refill_ofs, refill_k0);
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

    // Epilogue.  Accumulator register r of fragment (i, j) is c row 8*(r/4) + 4*kg + r%4 of the
    // fragment; thanks to the a-tile row permutation the lane's two j values are adjacent columns.
    // Addresses are "wave-uniform row pointer + one 32-bit lane offset", and the bias / accumulate
    // cases are separate straight-line instances, so the common case is 2 multiplies, 1 convert and
    // 1 store per output pair.
    auto epilogue_rows = [&](auto bias_tag, auto acc_tag, auto* out, float scale, int nb, int mb) {
        constexpr bool BIAS = decltype(bias_tag)::value;
        constexpr bool ACC = decltype(acc_tag)::value;
        using T = std::remove_pointer_t<decltype(out)>;
        const int e_lane = PERSIST ? opaque(threadIdx.x) % 64 : lane;
        const int el32 = e_lane % 32, ekg = e_lane / 32;
        const int m_lane = mb + wm * WT_M + NJ * el32;
        // byte offset of the lane inside a group of rows; below 2^32 (4 rows of at most 2^27 elements)
        const uint32_t lane_bytes = ((uint32_t)(4 * ekg) * (uint32_t)g.M + (uint32_t)m_lane) * (uint32_t)sizeof(T);
        // RAGGED: the lane's pair of columns lies inside c as a whole or not at all (M is even); its rows are tested one by one
        const bool col_inside = !RAGGED || m_lane < g.M;
        float bias0 = 0.f, bias1 = 0.f;
        if constexpr (BIAS) {
            if (col_inside) {
                bias0 = load_bias(g.bias, g.bias_is_bf16, m_lane);
                bias1 = load_bias(g.bias, g.bias_is_bf16, m_lane + 1);
            }
        }
        const int row0 = nb + wn * WT_N;  // wave-uniform
        auto inside = [&](int i, int r) { return !RAGGED || (col_inside && row0 + i * 32 + 8 * (r / 4) + (r % 4) + 4 * ekg < g.N); };
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            float o0[16], o1[16];
            if constexpr (ACC) {  // all 16 old values of this fragment row are requested before the first use
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    LLMQ_GLOBAL char* row = scalar_ptr((LLMQ_GLOBAL char*)(out + (int64_t)(row0 + i * 32 + 8 * (r / 4) + (r % 4)) * g.M));
                    o0[r] = o1[r] = 0.f;
                    if (inside(i, r)) PairIo<T>::load(row + lane_bytes, o0[r], o1[r]);
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if (!inside(i, r)) continue;
                LLMQ_GLOBAL char* row = scalar_ptr((LLMQ_GLOBAL char*)(out + (int64_t)(row0 + i * 32 + 8 * (r / 4) + (r % 4)) * g.M));
                float v0 = acc[i][0][r] * scale, v1 = acc[i][1][r] * scale;
                if constexpr (BIAS) {
                    v0 = v0 + bias0;
                    v1 = v1 + bias1;
                }
                if constexpr (ACC) {
                    v0 = v0 + o0[r];
                    v1 = v1 + o1[r];
                }
                PairIo<T>::store(row + lane_bytes, v0, v1);
            }
        }
    };
    // bf16 output without accumulation: every 32 x 64 fragment row of the wave tile goes through a
    // private 4 KiB LDS tile (row stride 128 B; rows 4 apart swap places pairwise so that the two lane
    // halves of a write hit different bank halves) and leaves as 16-byte pieces, eight lanes per 128-byte
    // row segment: 16 store instructions of 1 KiB per wave instead of 64 of 256 B.
    auto epilogue_staged = [&](auto bias_tag, uint16_t* out, float scale, int nb, int mb) {
        constexpr bool BIAS = decltype(bias_tag)::value;
        const int e_lane = PERSIST ? opaque(threadIdx.x) % 64 : lane;
        const int el32 = e_lane % 32, ekg = e_lane / 32;
        const int m_wave = mb + wm * WT_M;
        float bias0 = 0.f, bias1 = 0.f;
        if constexpr (BIAS) {
            if (!RAGGED || m_wave + NJ * el32 < g.M) {
                bias0 = load_bias(g.bias, g.bias_is_bf16, m_wave + NJ * el32);
                bias1 = load_bias(g.bias, g.bias_is_bf16, m_wave + NJ * el32 + 1);
            }
        }
        uint8_t* tile = lds + 2 * STAGE + wave * EPI_BYTES;
        // register r of a fragment is tile row 8*(r/4) + 4*kg + r%4, stored at row position (row ^ kg)
        uint8_t* w_even = tile + (4 * ekg) * 128 + el32 * 4 + ekg * 128;   // r % 4 even: position r%4 + kg
        uint8_t* w_odd = tile + (4 * ekg) * 128 + el32 * 4 - ekg * 128;    // r % 4 odd:  position r%4 - kg
        const int r_row = e_lane / 8, r_chunk = e_lane % 8;               // read side: position, 16-byte chunk
        const uint8_t* r_src = tile + r_row * 128 + r_chunk * 16;
        const uint32_t lane_bytes =
            ((uint32_t)(r_row ^ ekg) * (uint32_t)g.M + (uint32_t)(m_wave + r_chunk * 8)) * 2u;  // row = position ^ kg
        const int row0 = nb + wn * WT_N;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v0 = acc[i][0][r] * scale, v1 = acc[i][1][r] * scale;
                if constexpr (BIAS) {
                    v0 = v0 + bias0;
                    v1 = v1 + bias1;
                }
                const f32x2_t v = {v0, v1};
                uint8_t* dst = ((r % 4) % 2 == 0 ? w_even : w_odd) + (8 * (r / 4) + (r % 4)) * 128;
                *reinterpret_cast<bf16x2_t*>(dst) = __builtin_convertvector(v, bf16x2_t);
            }
            v4i piece[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) piece[p] = *reinterpret_cast<const v4i*>(r_src + p * 8 * 128);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                LLMQ_GLOBAL char* row = scalar_ptr((LLMQ_GLOBAL char*)(out + (int64_t)(row0 + i * 32 + p * 8) * g.M));
                // RAGGED: the lane's 8 columns lie inside c as a whole or not at all (M is a multiple of 8)
                if (RAGGED && (row0 + i * 32 + p * 8 + (r_row ^ ekg) >= g.N || m_wave + r_chunk * 8 >= g.M)) continue;
                __builtin_nontemporal_store(piece[p], (LLMQ_GLOBAL v4i*)(row + lane_bytes));
            }
        }
    };
    auto epilogue = [&](int nb, int mb) {
        constexpr std::true_type yes{};
        constexpr std::false_type no{};
        if constexpr (!SPLIT && std::is_same_v<OutT, uint16_t>) {
            if (!g.accumulate) {
                float scale = g.sa ? *g.sa : 1.f;
                if (g.sb) scale = scale * *g.sb;
                if (g.bias) epilogue_staged(yes, reinterpret_cast<uint16_t*>(g.c), scale, nb, mb);
                else epilogue_staged(no, reinterpret_cast<uint16_t*>(g.c), scale, nb, mb);
                return;
            }
        }
        if constexpr (SPLIT) {
            epilogue_rows(no, no, g.partial + (int64_t)blockIdx.y * g.N * g.M, 1.f, nb, mb);
        } else {
            float scale = g.sa ? *g.sa : 1.f;
            if (g.sb) scale = scale * *g.sb;
            OutT* c = reinterpret_cast<OutT*>(g.c);
            if (g.bias) {
                if (g.accumulate) epilogue_rows(yes, yes, c, scale, nb, mb);
                else epilogue_rows(yes, no, c, scale, nb, mb);
            } else {
                if (g.accumulate) epilogue_rows(no, yes, c, scale, nb, mb);
                else epilogue_rows(no, no, c, scale, nb, mb);
            }
        }
    };

    using std::integral_constant;
    constexpr integral_constant<int, 0> H0{};
    constexpr integral_constant<int, 1> H1{};
    constexpr integral_constant<bool, true> Y{};
    constexpr integral_constant<bool, false> NO{};
    if constexpr (!PERSIST) {
        int kt = 0;
        for (; kt + 2 < KT; ++kt) {  // steady state: a next stage exists and one more can be fetched
            half_step(H0, Y, NO, NO, lds + (kt & 1) * STAGE, 0, 0);
            half_step(H1, Y, Y, Y, lds + ((kt + 1) & 1) * STAGE, (kt & 1) * STAGE, (kt + 2) * kBK);
        }
        if (kt + 1 < KT) {           // second to last stage: nothing left to fetch
            half_step(H0, Y, NO, NO, lds + (kt & 1) * STAGE, 0, 0);
            half_step(H1, Y, Y, NO, lds + ((kt + 1) & 1) * STAGE, 0, 0);
            ++kt;
        }
        half_step(H0, Y, NO, NO, lds + (kt & 1) * STAGE, 0, 0);   // last stage
        half_step(H1, NO, NO, NO, lds, 0, 0);
        epilogue(n_blk, m_blk);
    } else {
        int cur = 0;  // byte offset of the LDS stage the current K-step lives in
        for (int t = 0; t < my_tiles; ++t) {
            for (int kt = 0; kt + 2 < KT; ++kt) {
                half_step(H0, Y, NO, NO, lds + cur, 0, 0);
                half_step(H1, Y, Y, Y, lds + (STAGE - cur), cur, (kt + 2) * kBK);
                cur = STAGE - cur;
            }
            // The copy stream moves on to the next tile (after the last tile it re-reads the first
            // K-steps of that same tile: harmless, and the loop body stays free of branches).
            const int cur_n = n_blk, cur_m = m_blk;
            if (t + 1 < my_tiles) {
                logical += tile_stride;
                decode(logical, n_blk, m_blk);
            }
            set_sources(n_blk, m_blk);
            half_step(H0, Y, NO, NO, lds + cur, 0, 0);                      // K-step KT-2
            half_step(H1, Y, Y, Y, lds + (STAGE - cur), cur, 0);
            cur = STAGE - cur;
            half_step(H0, Y, NO, NO, lds + cur, 0, 0);                      // K-step KT-1
            half_step(H1, NO, Y, Y, lds, cur, kBK);
            cur = STAGE - cur;
            epilogue(cur_n, cur_m);
            clear_acc();
            // first fragments of the next tile (its first K-step landed before the barrier above); they
            // are read only now so that the epilogue has the fragment registers to itself
#pragma unroll
            for (int i = 0; i < NI; ++i) fa[i] = read_frag(lds + cur + p_frag + i * 32 * kBK, 0);
#pragma unroll
            for (int j = 0; j < NJ; ++j) fb[0][j] = read_frag(lds + cur + q_frag + j * 32 * kBK, 0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the surplus copies of the last tile
    }
}

// Second pass of the split-K path: c = round((sum_s partial[s]) * scale + bias + old), slices added in
// index order.  One lane handles two adjacent columns; HBM-bound elementwise work.
template <typename OutT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmArgs g, int splits) {
    const int64_t pairs = (int64_t)g.N * g.M / 2;
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= pairs) return;
    const int64_t e = 2 * p;
    const int64_t slice = (int64_t)g.N * g.M;
    float v0 = 0.f, v1 = 0.f;
    for (int s = 0; s < splits; ++s) {
        float t0, t1;
        PairIo<float>::load((const LLMQ_GLOBAL float*)(g.partial + s * slice + e), t0, t1);
        v0 = v0 + t0;
        v1 = v1 + t1;
    }
    float scale = g.sa ? *g.sa : 1.f;
    if (g.sb) scale = scale * *g.sb;
    v0 = v0 * scale;
    v1 = v1 * scale;
    if (g.bias) {
        const int m = (int)(e % g.M);
        v0 = v0 + load_bias(g.bias, g.bias_is_bf16, m);
        v1 = v1 + load_bias(g.bias, g.bias_is_bf16, m + 1);
    }
    OutT* dst = reinterpret_cast<OutT*>(g.c) + e;
    if (g.accumulate) {
        float o0, o1;
        PairIo<OutT>::load((const LLMQ_GLOBAL OutT*)dst, o0, o1);
        v0 = v0 + o0;
        v1 = v1 + o1;
    }
    PairIo<OutT>::store((LLMQ_GLOBAL OutT*)dst, v0, v1);
}

// Position of 16-byte chunk c (0..7) of LDS row r (128 bytes, one K-step of one operand row) is c ^ frag_swizzle(r).
// A fragment read (ds_read_b128) has lane 16 kg + l read chunk 2 kg + h of row l.  The LDS serves such a read in four
// cycles of 16 lanes over its 64 banks, and the lanes of a cycle are not consecutive (measured with two-lane probes
// and the bank-conflict counter): {0-3, 12-15, 20-23, 24-27}, {4-11, 16-19, 28-31}, and the same plus 32.  A cycle so
// holds every row l once: rows 0-3 and 12-15 with one chunk number, rows 4-11 with that number ^ 2.  Rows of equal
// parity share banks; xor-ing the chunk with l / 2 alone would put rows 0-3, 12-15 and rows 4-11 of a cycle on the
// same banks (a two-way conflict on every read: 8 instead of 4 cycles), the extra flip of bit 1 for rows 4-11 undoes it.
__device__ __forceinline__ int frag_swizzle(int row) {
    return ((row >> 1) & 7) ^ ((((row >> 2) ^ (row >> 3)) & 1) << 1);
}

// ---- four-wave variant ----------------------------------------------------------------------------
// Same 256 x 256 x 128 workgroup tile, LDS layout, copies and tile order as above, with a different
// division of labour: 4 waves (one per SIMD, up to 512 registers each) of 128 x 128 outputs and the
// K = 128 matrix instruction v_mfma_f32_16x16x128_f8f6f4.  Against the 8-wave kernel this
//   * reads a third fewer fragment bytes from LDS (16 fragments of 16 rows per wave and K-step, 128 KiB
//     per workgroup instead of 192 KiB),
//   * moves half the accumulator registers per flop through the matrix pipe (4 per 65536 flop instead of
//     16 per 131072), which the chip turns into clock under its power limit: a register-only loop of this
//     instruction sustains about 8 % more than the 32x32x64 one on random operands,
//   * needs no LDS staging in the epilogue: the a-tile row permutation gives each lane 8 adjacent
//     columns, i.e. one 16-byte bf16 store, 16 lanes covering 256 contiguous bytes.
// With a single wave per SIMD nothing hides a stall, so the K loop is a software pipeline written out
// instruction by instruction: the 8 fragments of the second operand for step s+1 are read during rows
// 4..7 of step s into the other half of fb, the first operand's fragments rotate through 4 slots with a
// distance of 4 rows; the workgroup barrier sits after row 4, where every read of the current stage has
// been issued (and awaited) and the copies for step s+2 may overwrite it.
// The workgroup is persistent (one per compute unit, walking its XCD's tile list) and the stream of
// K-steps and copies runs across tile boundaries.  With an even number of K-steps per tile the LDS stage and the fb
// half of a step are compile-time functions of the step's parity; the ODDK instances (below) carry the stage as a
// run-time value.
//
// NJ < 8 narrows the tile along m to 2 * 16 * NJ columns (NJ second-operand fragments per wave instead of 8): a
// shape whose 256-wide tiles fill the last round of the chip badly can have a tile count that divides evenly
// (M = 3584: 14 x 32 = 448 tiles of 256 = 1.75 rounds of 256 compute units, but 16 x 32 = 512 tiles of 224 = 2
// full rounds of 7/8 the work each; M = 1536, N = 16384: 384 tiles of 256 = 1.5 rounds, 512 tiles of 192 = 2 full
// rounds of 3/4 the work).  Everything below is written for NJ fragments; NJ = 8, 7 and 6 are instantiated, the
// narrow ones for bf16 output without accumulation.
// STREAM_OUT: the bf16 stores of the full-width epilogue are non-temporal (see there).
// ODDK: the number of K-steps per tile is odd (K an odd multiple of 128, at least 384; not with SEG): the LDS stage
// and fb half of a tile's first step then alternate from tile to tile, and the tile loop carries both orders.
// KMB: the b operand is stored K-major, row-major [K, N] (the reference's mode TT: the output gradient dY[BT, OC] as
// the weight gradient's second operand, without a transposed copy).  Its tile of a K-step is then 128 rows (k) of
// 256 bytes (n) in LDS, 16-byte chunk g of row k stored at position g ^ swz(k), swz(k) = (k & 7) | ((k >> 5) & 1) << 3,
// and the fragments come out of LDS through the transposing read ds_read_b64_tr_b8: per group of 16 lanes it takes
// 8 rows x 16 bytes (lanes 2r and 2r + 1 give the addresses of the two 8-byte halves of row r) and hands lane i
// the 8 bytes of column i, i.e. 8 consecutive k of one n; four of them fill a fragment (32 k per lane, in the
// same k order as the other operand's two 16-byte reads).  The swizzle spreads the 8 rows of one read, and the
// two lane groups that share an LDS pass, over all banks.
//
// KMA: the a operand is stored K-major, row-major [K, M] (modes NN and NT: the weight W[OC, C] as the first operand of
// the dgrad, the activation X[BT, C] as that of the wgrad, without their transposed copies).  Copies and fragment reads
// are those of KMB with the operands' roles exchanged.  What does not carry over is the row permutation that gives
// a lane 8 adjacent columns of c (it is made by the copy addressing of a K-contiguous a; a transposing read hands 16
// adjacent columns to 16 adjacent lanes): a lane then owns columns 16 j + l16, and the epilogue goes through LDS --
// scale, bias and the rounding to bf16 where the accumulators are, 16 rows x 128 columns of bf16 per wave and
// fragment row into a private 4 KiB piece of LDS, read back as 16 bytes per lane and row.  That epilogue serves bf16
// output without accumulation (the old values of c would have to be fetched in the scattered layout); fp32 output and
// accumulation take the STAGE32 instances, whose epilogue hands the raw fp32 accumulators through LDS first.
// FUSE_EPI: the epilogue of full-width bf16 tiles without bias and accumulation runs under the matrix instructions of
// the tile's last and the next tile's first K-step (see k_step).
// RAGGED: M, N and K need not be multiples of the tile: edge tiles are moved back to end with the matrix, K is walked
// in whole steps with the copies of the last one masked (see masked_copy and the epilogue's ownership test).
template <typename OutT, int B_FMT, bool SEG, int NJ = 8, bool STREAM_OUT = true, bool ODDK = false, bool KMB = false,
          bool KMA = false, bool FUSE_EPI = false, bool STAGE32 = false, bool RAGGED = false>
__global__ __launch_bounds__(256) void gemm_tn_e4m3_w4_kernel(GemmArgs g) {
    static_assert(!RAGGED || (NJ == 8 && !SEG && !KMA && !KMB && !FUSE_EPI), "ragged shapes: full-width tiles of K-contiguous operands");
    static_assert(!(SEG && ODDK), "K segments are whole pairs of K-steps");
    static_assert(!STAGE32 || (KMA && !SEG && NJ == 8), "the fp32-staged epilogue belongs to the K-major first operand");
    static_assert(!FUSE_EPI || (NJ == 8 && !SEG && !KMA && std::is_same_v<OutT, uint16_t>),
                  "the epilogue under the last K-step is written for full-width bf16 tiles of K-contiguous a");
    static_assert(!((KMB || KMA) && ODDK), "the K-major operand modes are built for even K-step counts");
    static_assert(!KMA || (NJ == 8 && (SEG || STAGE32 || std::is_same_v<OutT, uint16_t>)) ||
                      (NJ < 8 && !SEG && !STAGE32 && !KMB && std::is_same_v<OutT, uint16_t>),
                  "the K-major first operand: fp32 output as K segments or through the fp32-staged epilogue; narrow tiles "
                  "for bf16 output of mode NN");
    constexpr int BLK = 256, T = 256, WT = 128, NF = 8;
    constexpr int WTM = 16 * NJ, BLKM = 2 * WTM;  // columns (first-operand rows) per wave and per tile
    constexpr int P_BYTES = BLK * kBK, STAGE = 2 * P_BYTES;
    constexpr int ITERS = BLK * 8 / T;    // 16-byte copies per lane and K-step, b rows
    constexpr int ITERS_Q = KMA ? 8 : BLKM * 8 / T;  // the same for the a rows (= NJ; a K-major a tile: 8 slabs of 16 k rows)
    static_assert(NJ == 8 || ((NJ == 7 || NJ == 6) && !SEG && std::is_same_v<OutT, uint16_t>), "unsupported tile width");
    typedef float v4f __attribute__((ext_vector_type(4)));

    constexpr int EPI_STAGE = 16 * 256;  // KMA: one fragment row of a wave's outputs as bf16, rows of 256 bytes
    constexpr int EPI32_ROW = 4 * WTM + 32;  // STAGE32: half a fragment row (8 c rows) of raw accumulators, rows padded by 32 bytes
    constexpr int EPI32_STAGE = 8 * EPI32_ROW;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * STAGE + (KMA ? 4 * (STAGE32 ? EPI32_STAGE : EPI_STAGE) : 0)];

    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wn = wave / 2, wm = wave % 2;
    const int l16 = lane % 16, kg = lane / 16;

    // Work list of this workgroup.  XCD x owns a contiguous range of the logical tile sequence and its
    // workgroups (slots) take every tile_stride-th tile of it.  With g.rem_split = S > 1 the tiles of the
    // XCD's last, partial round are left to a second launch of this kernel (SEG) that cuts each of them
    // into S segments of K (slot s: tile s / S, segment s % S) and writes raw accumulators as a 256 x 256
    // fp32 tile to g.partial for the reduction kernel below: the round then costs 1 / S of a tile.
    const int total = RAGGED ? ((g.N + BLK - 1) / BLK) * ((g.M + BLKM - 1) / BLKM) : (g.N / BLK) * (g.M / BLKM);
    const int xcd = blockIdx.x % g.xcds, slot = blockIdx.x / g.xcds;
    int xcd_first, xcd_count;
    xcd_tile_range(total, g.xcds, xcd, xcd_first, xcd_count);
    const int tile_stride = gridDim.x / g.xcds;
    // RAGGED: K is a multiple of 16 only; the stream walks K rounded up to whole steps and the copies of a tile's last
    // step leave the chunks beyond K to zeros (issue_copy)
    int my_tiles, k_first = 0, k_total = RAGGED ? (g.K + kBK - 1) / kBK * kBK : g.K;
    if constexpr (SEG) {
        const int rem = xcd_count % tile_stride;
        my_tiles = slot < rem * g.rem_split ? 1 : 0;
        xcd_first += xcd_count - rem + slot / g.rem_split - slot;  // so that tile "slot" below is the segment's tile
        k_first = (slot % g.rem_split) * g.k_len;
        k_total = k_first + g.k_len < g.K ? g.k_len : g.K - k_first;
    } else {
        my_tiles = slot < xcd_count ? (xcd_count - slot + tile_stride - 1) / tile_stride : 0;
        if (g.rem_split > 1) my_tiles = xcd_count / tile_stride;
    }
    if (my_tiles <= 0) return;  // uniform for the whole workgroup, before any barrier
    auto decode = [&](int logical, int& n_blk, int& m_blk) { decode_tile256<BLKM, RAGGED>(g, logical, n_blk, m_blk); };
    // The output factor sa * sb is read here, once, before the copy stream starts.  Read in the epilogue it would be
    // two global loads per tile, and the wait the compiler puts behind each of them (it counts only the loads it
    // knows about, so it waits for "all": vmcnt(0)) would also drain the copies of the next tile's first two K-steps
    // that are in flight at that point.
    float out_scale = 1.f;
    if constexpr (!SEG) {
        if (g.sa) out_scale = *g.sa;
        if (g.sb) out_scale = out_scale * *g.sb;
    }

    // copies: lane -> (row tid/8 of a 32-row slab, physical 16-byte chunk tid%8); every address is a
    // wave-uniform base plus a 32-bit lane offset
    const int ld_row = tid / 8;
    const int ld_chunk = (tid & 7) ^ frag_swizzle(ld_row);
    // b tile copies.  Normal layout: slab c = rows 32 c .. 32 c + 31 of the tile, lane -> (row, chunk) as above.
    // K-major layout: slab c = k rows 16 c .. 16 c + 15, lane -> (row tid / 16, physical chunk tid % 16) reading
    // global chunk (tid % 16) ^ swz(k); bit 3 of swz depends on the slab ((c >> 1) & 1), hence two lane offsets.
    const int kb_row = tid / 16, kb_chunk = (tid & 15) ^ (kb_row & 7);
    const uint32_t p_lane = KMB ? (uint32_t)kb_row * (uint32_t)g.N + (uint32_t)kb_chunk * 16u
                                : (uint32_t)ld_row * (uint32_t)g.K + (uint32_t)ld_chunk * 16u;
    const uint32_t p_lane_hi = (uint32_t)kb_row * (uint32_t)g.N + (uint32_t)(kb_chunk ^ 8) * 16u;  // KMB, slabs 2, 3, 6, 7
    const uint32_t p_step = KMB ? (uint32_t)kBK * (uint32_t)g.N : (uint32_t)kBK;  // lane offset advance per K-step
    // LDS row rho of the a-tile is row l = rho % 16 of fragment f = rho / 16 (wave half f / NJ, fragment f % NJ of
    // it) and holds global row frag_row(f) + frag_step(f) * l.  NJ = 8 and 6: fragment j of a wave half starts at
    // row j with step NJ, so that a lane of the epilogue owns NJ adjacent columns (16 or 12 bytes of bf16).  NJ = 7:
    // the first six fragments do the same with step 6 (12 bytes per lane, 4-byte aligned), the seventh takes the
    // last 16 columns of the wave half one per lane (14 adjacent columns per lane would mean 2-byte aligned
    // 12 + 2 byte stores, measured 3 us per tile slower).
    // A copy slab is two fragments, f = 2 it (lanes of its first 16 rows) and 2 it + 1: the lane offset of a slab
    // follows from the two fragments' steps and the distance of their first rows -- one value for all slabs
    // with NJ = 8 and 6, three different ones with NJ = 7 (slabs 3 and 6 hold a seventh fragment).
    auto frag_row = [](int f) {
        const int j = f % NJ;
        return WTM * (f / NJ) + ((NJ == 7 && j == 6) ? 96 : j);
    };
    auto frag_step = [](int f) { return NJ == 7 ? (f % NJ == 6 ? 1 : 6) : NJ; };
    auto slab_lane_rows = [&](int it) {  // global row of this lane's LDS row, relative to the slab's first row
        const int l = ld_row % 16;
        return ld_row < 16 ? frag_step(2 * it) * l : frag_row(2 * it + 1) - frag_row(2 * it) + frag_step(2 * it + 1) * l;
    };
    // A K-major a tile of a narrow instance is 2 NJ chunks wide: a lane whose chunk lies beyond that copies a chunk
    // 2 (8 - NJ) to the left instead (inside the tile, so inside the matrix; it lands in a place no fragment reads)
    auto inside_tile = [](int chunk) { return chunk < 2 * NJ ? chunk : chunk - 2 * (8 - NJ); };
    const uint32_t q_lane = KMA ? (uint32_t)kb_row * (uint32_t)g.M + (uint32_t)inside_tile(kb_chunk) * 16u
                                : (uint32_t)slab_lane_rows(0) * (uint32_t)g.K + (uint32_t)ld_chunk * 16u;
    const uint32_t q_lane_hi = (uint32_t)kb_row * (uint32_t)g.M + (uint32_t)inside_tile(kb_chunk ^ 8) * 16u;  // KMA, slabs 2, 3, 6, 7
    const uint32_t q_step = KMA ? (uint32_t)kBK * (uint32_t)g.M : (uint32_t)kBK;
    const uint32_t q_lane_3 = (uint32_t)slab_lane_rows(NJ == 7 ? 3 : 0) * (uint32_t)g.K + (uint32_t)ld_chunk * 16u;
    const uint32_t q_lane_6 = (uint32_t)slab_lane_rows(NJ == 7 ? 6 : 0) * (uint32_t)g.K + (uint32_t)ld_chunk * 16u;
    // The copy stream runs two K-steps ahead of the matrix instructions and has its own position: tile number
    // and K offset.  A copy's global address is "scalar base of its slab in the current tile + 32-bit lane
    // offset": the 16 slab bases change once per tile, the K offset lives in the lane offsets (one vector add
    // per K-step), so a copy costs two instructions in the K loop: the write of M0 (LDS destination) and the
    // copy itself.
    int copy_k0 = 0, copy_tile = 0;
    const uint8_t* p_base[ITERS];
    const uint8_t* q_base[ITERS_Q];
    uint32_t vp = p_lane, vp_hi = p_lane_hi, vq = q_lane, vq3 = q_lane_3, vq6 = q_lane_6;
    [[maybe_unused]] uint32_t vq_hi = q_lane_hi;
    auto tile_bases = [&](int logical) {
        int nb, mb;
        decode(logical, nb, mb);
        const uint8_t* pb = KMB ? g.b + (int64_t)k_first * g.N + nb : g.b + (int64_t)nb * g.K + k_first;
        const uint8_t* qb = KMA ? g.a + (int64_t)k_first * g.M + mb : g.a + (int64_t)mb * g.K + k_first;
        // pinned in scalar registers here, once per tile (otherwise the compiler sinks the additions to the
        // copies and repeats them in every K-step)
#pragma unroll
        for (int c = 0; c < ITERS; ++c) {
            p_base[c] = KMB ? pb + (int64_t)(16 * c) * g.N : pb + (int64_t)(32 * c) * g.K;
            asm volatile("" : "+s"(p_base[c]));
        }
#pragma unroll
        for (int it = 0; it < ITERS_Q; ++it) {
            q_base[it] = KMA ? qb + (int64_t)(16 * it) * g.M : qb + (int64_t)frag_row(2 * it) * g.K;
            asm volatile("" : "+s"(q_base[it]));
        }
    };
    tile_bases(xcd_first + slot);
    // after the copies of one K-step; past the last tile the stream re-reads that tile's first K-steps
    // (harmless, and no step needs a special case)
    // RAGGED: in a tile's last, partial K-step (K % 128 != 0) the lanes whose 16-byte chunk lies beyond K write zeros
    // instead of copying (tail_mask: lanes with a chunk inside K)
    [[maybe_unused]] const uint64_t tail_mask = __ballot(ld_chunk * 16 < (g.K % kBK == 0 ? kBK : g.K % kBK));
    [[maybe_unused]] uint64_t copy_mask = ~0ull;   // lane mask of the copies issued next
    auto advance_copy = [&]() {
        copy_k0 += kBK;
        vp += p_step;
        if constexpr (KMB) vp_hi += p_step;
        vq += q_step;
        if constexpr (KMA) vq_hi += q_step;
        if constexpr (NJ == 7) {
            vq3 += kBK;
            vq6 += kBK;
        }
        if (copy_k0 == k_total) {
            copy_k0 = 0;
            vp = p_lane;
            if constexpr (KMB) vp_hi = p_lane_hi;
            if constexpr (KMA) {
                vq = q_lane;
                vq_hi = q_lane_hi;
            } else {
                vq -= (uint32_t)k_total;
            }
            if constexpr (NJ == 7) {
                vq3 -= (uint32_t)k_total;
                vq6 -= (uint32_t)k_total;
            }
            if (copy_tile + 1 < my_tiles) ++copy_tile;
            tile_bases(xcd_first + slot + copy_tile * tile_stride);
        }
        if constexpr (RAGGED) copy_mask = copy_k0 + kBK > g.K ? tail_mask : ~0ull;
    };
    // Copy number c of a K-step, c = 0 .. COPIES-1: first the b-rows slabs, then the a-rows slabs, as two asm
    // statements.  set_m0 computes the LDS destination of the wave's part of the slab into M0 and hands it to the
    // compiler as a value living in M0; issue_copy consumes that value.  Both are modelled operands, so the compiler
    // keeps M0 intact between the two.  The hardware needs one instruction between a write of M0 and the copy that
    // uses it: the callers place a matrix instruction or an LDS read there (issue_copy_nop carries an s_nop of its
    // own for places that have none).  The compiler does not know that issue_copy is a memory instruction reading
    // scalar registers and would not keep the 5 wait states such an instruction needs after a vector instruction
    // wrote one of them (v_readlane reloading a spilled scalar): the kernel is written so that no scalar is spilled,
    // and tests/test_asm_hazards.py checks the generated code for both distances.
    const uint32_t lds_wave = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds + wave * 1024;
    // c_tag / stage_tag: integral constants (copy number, byte offset of the LDS stage): the compile-time part of
    // the destination is an immediate of the add
    // ODDK: the stage is a run-time value (stage_rt, see the tile loop) and stage_tag is 0.
    uint32_t lds_wave_stage = lds_wave;  // ODDK: lds_wave + byte offset of the stage the current K-step releases
    auto set_m0 = [&](auto c_tag, auto stage_tag) -> uint32_t {
        constexpr int C = decltype(c_tag)::value, STAGE_OFS = decltype(stage_tag)::value;
        constexpr int DST = C < ITERS ? STAGE_OFS + C * T * 16 : STAGE_OFS + P_BYTES + (C - ITERS) * T * 16;
        uint32_t tok;
        if constexpr (ODDK) asm volatile("s_add_i32 %0, %1, %2" : "={m0}"(tok) : "s"(lds_wave_stage), "n"(DST));
        else asm volatile("s_add_i32 %0, %1, %2" : "={m0}"(tok) : "s"(lds_wave), "n"(DST));
        return tok;
    };
    auto copy_src = [&](int c, const uint8_t*& src, uint32_t& lane_ofs) {
        if (c < ITERS) {
            src = p_base[c];
            lane_ofs = (KMB && ((c >> 1) & 1)) ? vp_hi : vp;
        } else {
            const int it = c - ITERS;  // slab `it` covers LDS rows 32 it .. 32 it + 31: fragments 2 it and 2 it + 1
            src = q_base[it];
            lane_ofs = KMA ? (((it >> 1) & 1) ? vq_hi : vq) : (NJ == 7 && it == 3) ? vq3 : (NJ == 7 && it == 6) ? vq6 : vq;
        }
    };
    // RAGGED: every copy runs under a lane mask -- all lanes, or in a tile's last, partial K-step the lanes whose chunk
    // lies inside K.  The other lanes neither read global memory nor write LDS; they then store 16 zero bytes to the
    // place the copy would have filled for them (M0 + 16 * lane, the destination rule of the copy instruction itself).
    // Every wave has lanes inside K (a wave covers whole rows), so the copy instruction always executes and the counter
    // bookkeeping of the K-steps holds.  One asm statement with its own branch: a branch of the compiler's between
    // the write of M0 and the copy makes it save and restore M0 right in front of the copy (too close for the
    // hardware; the hazard scan of the build rejects it).
    auto masked_copy = [&](uint32_t lane_ofs, const uint8_t* src, uint32_t tok) {
        uint32_t addr, zero;   // live inside the statement only: lane number * 16 + M0, and 0
        asm volatile(
            "s_mov_b64 exec, %4\n\t"
            "global_load_lds_dwordx4 %2, %3\n\t"
            "s_cmp_eq_u64 %4, -1\n\t"
            "s_cbranch_scc1 1f\n\t"
            "s_not_b64 exec, exec\n\t"
            "v_mbcnt_lo_u32_b32 %0, -1, 0\n\t"
            "v_mbcnt_hi_u32_b32 %0, -1, %0\n\t"
            "v_mov_b32 %1, 0\n\t"
            "v_lshl_add_u32 %0, %0, 4, m0\n\t"
            "ds_write_b32 %0, %1\n\t"
            "ds_write_b32 %0, %1 offset:4\n\t"
            "ds_write_b32 %0, %1 offset:8\n\t"
            "ds_write_b32 %0, %1 offset:12\n\t"
            "s_mov_b64 exec, -1\n"
            "1:"
            : "=&v"(addr), "=&v"(zero)
            : "v"(lane_ofs), "s"(src), "s"(copy_mask), "{m0}"(tok)
            : "memory", "scc");
    };
    auto issue_copy = [&](int c, uint32_t tok) {
        const uint8_t* src;
        uint32_t lane_ofs;
        copy_src(c, src, lane_ofs);
        if constexpr (RAGGED) masked_copy(lane_ofs, src, tok);
        else asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(lane_ofs), "s"(src), "{m0}"(tok) : "memory");
    };
    auto issue_copy_nop = [&](auto c_tag, auto stage_tag) {
        const uint8_t* src;
        uint32_t lane_ofs;
        copy_src(decltype(c_tag)::value, src, lane_ofs);
        const uint32_t tok = set_m0(c_tag, stage_tag);
        if constexpr (RAGGED) masked_copy(lane_ofs, src, tok);   // the write of exec sits between the write of M0 and the copy
        else asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_ofs), "s"(src), "{m0}"(tok) : "memory");
    };

    const int sw = frag_swizzle(l16);
    const int c0 = ((2 * kg) ^ sw) * 16, c1 = ((2 * kg + 1) ^ sw) * 16;
    const int p_frag = (wn * WT + l16) * kBK;
    const int q_frag = P_BYTES + (wm * WTM + l16) * kBK;
    auto read_frag = [&](const uint8_t* row) -> v8i {
        const v4i lo = *reinterpret_cast<const v4i*>(row + c0);
        const v4i hi = *reinterpret_cast<const v4i*>(row + c1);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    // b fragment i (rows 16 i .. 16 i + 15 of the wave's 128 rows of c) from the stage at `stage`.  K-major: this
    // lane supplies the address of half (l16 & 1) of k row 32 kg + 8 q + l16 / 2 for the q-th of four transposing
    // reads; the row's chunk 8 wn + i sits at position (8 wn + i) ^ swz(k), and with swz(k) = l16 / 2 | (kg & 1) << 3
    // for every q that is kb_base ^ (16 i) in bytes: one xor per fragment, the four reads differ by 8 rows = 2048.
    typedef int v2i_lds __attribute__((ext_vector_type(2)));
    const uint32_t kb_base = (uint32_t)((32 * kg + l16 / 2) * 256 + (l16 & 1) * 8) + (uint32_t)(((8 * wn) ^ ((kg & 1) << 3)) * 16) +
                             (uint32_t)((l16 / 2) * 16);
    auto read_frag_b = [&](const uint8_t* stage, int i) -> v8i {
        if constexpr (KMB) {
            const uint8_t* p = stage + (opaque((int)kb_base) ^ (16 * i));
            typedef __attribute__((address_space(3))) v2i_lds* lds_v2i;
            const v2i_lds r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(p));
            const v2i_lds r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(p + 2048));
            const v2i_lds r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(p + 4096));
            const v2i_lds r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(p + 6144));
            const v8i f = {r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
            return f;
        } else {
            return read_frag(stage + p_frag + i * 16 * kBK);
        }
    };
    // a fragment j (columns 16 j .. 16 j + 15 of the wave's 128 columns of c) from the stage at `stage`: the same two
    // ways, with the wave's column half wm in the place of its row half wn
    const uint32_t ka_base = (uint32_t)((32 * kg + l16 / 2) * 256 + (l16 & 1) * 8) + (uint32_t)(((8 * wm) ^ ((kg & 1) << 3)) * 16) +
                             (uint32_t)((l16 / 2) * 16);
    // Narrow tiles: the wave half wm starts at chunk NJ wm, which is no power of two, so fragment j's chunk NJ wm + j is
    // xor-ed with the lane's swizzle explicitly (one more vector instruction per fragment read)
    [[maybe_unused]] const uint32_t ka_row = (uint32_t)((32 * kg + l16 / 2) * 256 + (l16 & 1) * 8);
    [[maybe_unused]] const uint32_t ka_swz = (uint32_t)(((l16 / 2) | ((kg & 1) << 3)) * 16);
    auto frag_a_ofs = [&](int j) -> uint32_t {  // byte offset, within the a half of a stage, of the first read of fragment j
        if constexpr (NJ == 8) return (uint32_t)(opaque((int)ka_base) ^ (16 * j));
        else return (uint32_t)opaque((int)ka_row) + ((uint32_t)((NJ * wm + j) * 16) ^ (uint32_t)opaque((int)ka_swz));
    };
    typedef __attribute__((address_space(3))) v2i_lds* lds_v2i_a;
    auto read_frag_a = [&](const uint8_t* stage, int j) -> v8i {
        if constexpr (KMA) {
            const uint8_t* p = stage + P_BYTES + frag_a_ofs(j);
            const v2i_lds r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(p));
            const v2i_lds r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(p + 2048));
            const v2i_lds r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(p + 4096));
            const v2i_lds r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(p + 6144));
            const v8i f = {r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
            return f;
        } else {
            return read_frag(stage + q_frag + j * 16 * kBK);
        }
    };

    // The matrix instruction as an asm statement with the accumulator tied in place in the accumulation
    // registers: with all 256 of them holding the wave tile there is no spare for the register allocator's
    // untied form.  The memory clobber keeps every LDS read and copy in its source position relative to
    // the matrix instructions, so a K-step is issued exactly as written below.
    auto mfma = [&](v4f& c, const v8i& a, const v8i& b) {
        if constexpr (B_FMT == 0)
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b) : "memory");
        else
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1" : "+a"(c) : "v"(a), "v"(b) : "memory");
    };
    // first K-step of a tile: the accumulator input is the constant 0, so no register is initialised by an
    // instruction whose distance to the matrix instruction the compiler could not police
    auto mfma_first = [&](v4f& c, const v8i& a, const v8i& b) {
        if constexpr (B_FMT == 0)
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b) : "memory");
        else
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0 cbsz:1" : "=a"(c) : "v"(a), "v"(b) : "memory");
    };

    v4f acc[NF][NJ];  // written by the first K-step of every tile
    v8i fa[4], fb[2][NJ];

    // prologue of the stream: the first two K-steps of the first tile
    constexpr int COPIES = ITERS + ITERS_Q;  // per K-step and lane
    static_for<0, COPIES>([&](auto c) { issue_copy_nop(c, std::integral_constant<int, 0>{}); });
    advance_copy();
    static_for<0, COPIES>([&](auto c) { issue_copy_nop(c, std::integral_constant<int, STAGE>{}); });
    advance_copy();
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COPIES) : "memory");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[i] = read_frag_b(lds, i);
#pragma unroll
    for (int j = 0; j < NJ; ++j) fb[0][j] = read_frag_a(lds, j);

    // One K-step of parity PAR (LDS stage PAR, fb half PAR): rows i = 0..7 of first-operand fragments
    // against all 8 second-operand fragments.  fa rotates through 4 slots (fragment i+4 is read once row i
    // has been issued; rows 4..7 fetch the next step's first four from the other stage); the next step's
    // second-operand fragments go into the other half of fb, two per row in rows 4..7 (after the barrier).
    // The 16 copies of the step after next go into the stage this step computes from, each half as soon as it is
    // free.  The a-rows half was read into fb during the previous step: a barrier at the start of the step releases
    // it, and its copies follow every fourth matrix instruction of rows 0..3.  The b-rows half is read until row 3:
    // the barrier after row 4 releases it (and confirms that the other stage has landed); 4 copies right after that
    // barrier, the rest spread over rows 5..7.  A copy so has 5 to 13 rows of matrix instructions (256 cycles each) to
    // land before the barrier that needs it.  With a single barrier per step and all copies in rows 4..7 (4 to 8
    // rows to land) the waves spent 10 % of their cycles waiting at that barrier for data from beyond the L2; the
    // second barrier made six large shapes 6 % faster (2.90 -> 3.08 PFLOP/s, one box, alternating launches).
    // Measured against it and not kept: all eight b-rows fragments of a step in registers, so that the whole stage is
    // released at the start of the step and the landing barrier moves to row 6 (copies have 7 to 14 rows): 1-4 % slower,
    // the 32 extra live registers push address registers into scratch around the tile epilogue.  Shorter copy windows
    // (rows 0..2 for the a-rows half, rows 5..6 or row 5 for the b-rows half): 0.3-1 % slower.
    // FUSE_EPI: the epilogue of a tile runs under matrix instructions -- fragment rows 0..3 under the tile's own last
    // K-step, rows 4..7 under the first K-step of the workgroup's next tile.  Done after the K loop, the epilogue is
    // 1.5 to 2.4 us per tile in which the matrix cores idle (measured by leaving it out: 37888 x 8192 x 3584 702 ->
    // 649 us, 17920 x 16384 x 1536 316 -> 268 us).  Two resources bound how it can be hidden:
    //   * the wave's instruction issue: a slice (below) is 10 vector instructions, a matrix instruction occupies its
    //     pipe for 32 cycles -- one slice per matrix instruction (all eight rows under one K-step) was measured to
    //     stretch that K-step by as much as 60 % of what was saved; two slices per three matrix instructions fit;
    //   * the compute unit's one address unit: 16 cycles per copy or store instruction of a wave, four waves, so the
    //     16 copies of a K-step take half of its 2048 cycles and at most 16 of a tile's 32 stores per wave fit
    //     beside them (with 28 stores in one K-step: +1.3 us per tile; with 16: within the noise of none).
    // Fragment row q of a tile is final once its eight matrix instructions of the last K-step have been issued, and
    // stays intact until the next tile's first K-step reaches row q.  A slice takes four accumulators of one c row (two
    // pairs of adjacent columns): accumulation register -> vector register, times the output factor, packed rounding
    // to bf16; every second slice completes the lane's 16 bytes of a c row and stores them.  The 32 slices of rows 0..3
    // follow the matrix instructions 8 + 3k/2 (k = 0..31) of the last K-step, those of rows 4..7 the matrix
    // instructions 3k/2 of the next first K-step (each row before the step overwrites it); after a workgroup's last
    // tile rows 4..7 are written out on their own.  The slices are asm statements so that they stay where they are
    // written: the compiler would otherwise gather the read-outs behind the matrix instruction that wrote the
    // register (too close for the hardware, which needs the instruction's passes to finish first, and the values would
    // then occupy registers through the whole step).
    [[maybe_unused]] uint32_t epi_lane = 0;   // this tile: byte offset of the lane's 16 bytes within "its" c row (4 ekg rows down)
    [[maybe_unused]] int epi_row0 = 0;        // this tile: first c row of the wave tile
    [[maybe_unused]] uint32_t prev_lane = 0;  // the same two for the previous tile of this workgroup (rows 4..7 still to write)
    [[maybe_unused]] int prev_row0 = 0;
    [[maybe_unused]] uint32_t epi_pk[4];
    [[maybe_unused]] auto scaled_pair = [&](float x0, float x1) -> uint32_t {
        uint32_t out, tmp;
        asm volatile(
            "v_accvgpr_read_b32 %0, %2\n\t"
            "v_accvgpr_read_b32 %1, %3\n\t"
            "v_mul_f32 %0, %4, %0\n\t"
            "v_mul_f32 %1, %4, %1\n\t"
            "v_cvt_pk_bf16_f32 %0, %0, %1"
            : "=&v"(out), "=&v"(tmp)
            : "a"(x0), "a"(x1), "s"(out_scale));
        return out;
    };
    // slice sl (0..7) of fragment row i: c row r = sl / 2 of the row's four, column half h = sl % 2
    [[maybe_unused]] auto epi_slice = [&](auto i_tag, auto s_tag, int row0, uint32_t lane_bytes) {
        constexpr int i = decltype(i_tag)::value, sl = decltype(s_tag)::value;
        constexpr int r = sl / 2, h = sl % 2;
        epi_pk[2 * h] = scaled_pair(acc[i][4 * h][r], acc[i][4 * h + 1][r]);
        epi_pk[2 * h + 1] = scaled_pair(acc[i][4 * h + 2][r], acc[i][4 * h + 3][r]);
        if constexpr (h == 1) {
            const v4i packed = {(int)epi_pk[0], (int)epi_pk[1], (int)epi_pk[2], (int)epi_pk[3]};
            LLMQ_GLOBAL char* row_ptr =
                scalar_ptr((LLMQ_GLOBAL char*)(reinterpret_cast<uint16_t*>(g.c) + (int64_t)(row0 + 16 * i + r) * g.M));
            if constexpr (STREAM_OUT) __builtin_nontemporal_store(packed, (LLMQ_GLOBAL v4i*)(row_ptr + lane_bytes));
            else *(LLMQ_GLOBAL v4i*)(row_ptr + lane_bytes) = packed;
        }
    };
    bool pending_stores = false;  // an epilogue without accumulation has just issued its stores
    [[maybe_unused]] int stage_rt = 0;  // ODDK: byte offset of the LDS stage of the current K-step
    // par_tag: LDS stage of the step; fp_tag: the half of fb that holds its second-operand fragments (the same
    // as the stage unless ODDK, see the tile loop).
    // kYoung: copies of this step that are in flight at the step's second barrier and need not have landed (they
    // refill the a-rows half of the stage this step computes from)
    constexpr int kYoung = ITERS_Q;
    // Slice schedule of FUSE_EPI: slice k (0..31: fragment row k / 8 of a group of four, slice k % 8 of it) follows
    // the matrix instruction number 3k/2 of its window; slice_of(m) is the slice behind instruction m of the window
    // (-1: none) and stores_through(m) the number of stores issued with the slices up to instruction m.
    constexpr auto slice_of = [](int m) {
        for (int k = 0; k < 32; ++k)
            if (3 * k / 2 == m) return k;
        return -1;
    };
    constexpr auto stores_through = [](int m) {
        int n = 0;
        for (int k = 1; k < 32; k += 2)
            if (3 * k / 2 <= m) ++n;
        return n;
    };
    // last_tag: the tile's last K-step (FUSE_EPI: carries the slices of rows 0..3, window from instruction 8 on);
    // prev_tag: a first K-step that carries the slices of rows 4..7 of the workgroup's previous tile (FUSE_EPI).
    auto k_step = [&](auto par_tag, auto fp_tag, auto first_tag, auto last_tag, auto prev_tag) {
        constexpr int PAR = decltype(par_tag)::value;
        constexpr int FP = decltype(fp_tag)::value;
        constexpr bool FIRST = decltype(first_tag)::value;
        constexpr bool LAST = FUSE_EPI && decltype(last_tag)::value;
        constexpr bool PREV = FUSE_EPI && FIRST && decltype(prev_tag)::value;
        // the stage this step computes from and then releases to the copies; with ODDK a run-time value
        const uint8_t* cur = lds + (ODDK ? stage_rt : PAR * STAGE);
        const uint8_t* nxt = lds + (ODDK ? STAGE - stage_rt : (1 - PAR) * STAGE);
        constexpr std::integral_constant<int, ODDK ? 0 : PAR * STAGE> refill{};
        if constexpr (ODDK) lds_wave_stage = lds_wave + (uint32_t)stage_rt;
        // The write of M0 for a copy sits in front of the matrix instruction the copy follows.  The CU's one
        // address unit takes 16 cycles per copy instruction and the four waves issue theirs at the same time; a
        // dense burst backs up into the waves' instruction issue and stalls the matrix instructions behind it (with
        // all copies behind the second barrier: one per instruction over rows 5 and 6 was 4 % slower over six large
        // shapes than spread over rows 5..7, all sixteen right after the barrier 11 %).
        // First barrier: the a-rows half of this stage was read during the previous step; once every wave's reads
        // have returned and all waves are here it may be refilled.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __syncthreads();
        constexpr int Q_SLOTS = 4 * NJ, SPREAD = ITERS - 4, SLOTS = 3 * NJ;
        static_assert(SPREAD <= SLOTS, "not every copy of a K-step has a place in the schedule");
        static_for<0, NF>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            static_for<0, NJ>([&](auto j_tag) {
                constexpr int j = decltype(j_tag)::value;
                constexpr int p = (i - 5) * NJ + j;  // slot in rows 5..7
                constexpr int pq = i * NJ + j;  // slot in rows 0..3
                constexpr bool Q_HERE = i < 4 && ((pq + 1) * ITERS_Q / Q_SLOTS > pq * ITERS_Q / Q_SLOTS);
                constexpr bool P_HERE = i >= 5 && ((p + 1) * SPREAD / SLOTS > p * SPREAD / SLOTS);
                constexpr bool COPY_HERE = Q_HERE || P_HERE;
                constexpr int COPY_C = Q_HERE ? ITERS + pq * ITERS_Q / Q_SLOTS : P_HERE ? 4 + p * SPREAD / SLOTS : 0;
                uint32_t tok = 0;
                if constexpr (COPY_HERE) tok = set_m0(std::integral_constant<int, COPY_C>{}, refill);
                if constexpr (FIRST) mfma_first(acc[i][j], fa[i % 4], fb[FP][j]);
                else mfma(acc[i][j], fa[i % 4], fb[FP][j]);
                if constexpr (COPY_HERE) issue_copy(COPY_C, tok);
                if constexpr (i >= 5 && (j == 2 || j == 5)) {  // rows 5..7: fragments 2..7 of the next step
                    constexpr int f = 2 * (i - 4) + (j == 5 ? 1 : 0);
                    if constexpr (f < NJ) fb[1 - FP][f] = read_frag_a(nxt, f);
                }
                if constexpr (LAST && i >= 1) {
                    constexpr int k = slice_of(8 * i + j - 8);
                    if constexpr (k >= 0)
                        epi_slice(std::integral_constant<int, k / 8>{}, std::integral_constant<int, k % 8>{}, epi_row0, epi_lane);
                }
                if constexpr (PREV) {
                    constexpr int k = slice_of(8 * i + j);
                    if constexpr (k >= 0)
                        epi_slice(std::integral_constant<int, 4 + k / 8>{}, std::integral_constant<int, k % 8>{}, prev_row0, prev_lane);
                }
            });
            if constexpr (i == 4) {
                // every read of the current stage has been issued (the last one after row 3); once they
                // have returned and all waves are here the stage may be overwritten, and the next stage
                // (copied one step ago) is complete
                if constexpr (LAST) {
                    // the stores of this step's slices so far (instructions 8..39 of the step) sit behind every copy this
                    // barrier is about
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kYoung + stores_through(31)) : "memory");
                } else if constexpr (PREV) {
                    // likewise (instructions 0..39); the last copy this barrier is about went out with the last matrix
                    // instruction of the previous tile, behind all of that step's stores
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kYoung + stores_through(39)) : "memory");
                } else if constexpr (FIRST && FUSE_EPI) {
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kYoung) : "memory");
                } else if constexpr (FIRST) {
                    // Behind the copies this barrier is about (the tile's second K-step, issued before the
                    // previous tile's epilogue) sit that epilogue's stores; the counter retires in issue
                    // order, so allowing as many outstanding operations as there were stores is enough.
                    if (pending_stores) {
                        // stores of a bf16 epilogue per lane and tile: 32 (one per c row), 64 with the two-piece rows of
                        // the 224-wide tile of a K-contiguous a
                        if constexpr (sizeof(OutT) == 2 && (NJ != 7 || KMA)) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(32 + kYoung) : "memory");
                        else asm volatile("s_waitcnt vmcnt(63) lgkmcnt(0)" ::: "memory");
                    } else {
                        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kYoung) : "memory");
                    }
                } else {
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kYoung) : "memory");
                }
                __syncthreads();
                // copies 0..3, each with one of the four LDS reads of the next step's first two second-operand
                // fragments between the write of M0 and the copy
                if constexpr (KMA) {
                    // the eight transposing reads of the next step's first two a fragments, two between each write of M0
                    // and its copy
                    const uint8_t* pa0 = nxt + P_BYTES + frag_a_ofs(0);
                    const uint8_t* pa1 = nxt + P_BYTES + frag_a_ofs(1);
                    uint32_t tok = set_m0(std::integral_constant<int, 0>{}, refill);
                    const v2i_lds a00 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa0));
                    const v2i_lds a01 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa0 + 2048));
                    issue_copy(0, tok);
                    tok = set_m0(std::integral_constant<int, 1>{}, refill);
                    const v2i_lds a02 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa0 + 4096));
                    const v2i_lds a03 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa0 + 6144));
                    issue_copy(1, tok);
                    tok = set_m0(std::integral_constant<int, 2>{}, refill);
                    const v2i_lds a10 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa1));
                    const v2i_lds a11 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa1 + 2048));
                    issue_copy(2, tok);
                    tok = set_m0(std::integral_constant<int, 3>{}, refill);
                    const v2i_lds a12 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa1 + 4096));
                    const v2i_lds a13 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_a)(pa1 + 6144));
                    issue_copy(3, tok);
                    const v8i f0 = {a00[0], a00[1], a01[0], a01[1], a02[0], a02[1], a03[0], a03[1]};
                    const v8i f1 = {a10[0], a10[1], a11[0], a11[1], a12[0], a12[1], a13[0], a13[1]};
                    fb[1 - FP][0] = f0;
                    fb[1 - FP][1] = f1;
                } else {
                    const uint8_t* r0 = nxt + q_frag;
                    const uint8_t* r1 = nxt + q_frag + 16 * kBK;
                    uint32_t tok = set_m0(std::integral_constant<int, 0>{}, refill);
                    const v4i lo0 = *reinterpret_cast<const v4i*>(r0 + c0);
                    issue_copy(0, tok);
                    tok = set_m0(std::integral_constant<int, 1>{}, refill);
                    const v4i hi0 = *reinterpret_cast<const v4i*>(r0 + c1);
                    issue_copy(1, tok);
                    tok = set_m0(std::integral_constant<int, 2>{}, refill);
                    const v4i lo1 = *reinterpret_cast<const v4i*>(r1 + c0);
                    issue_copy(2, tok);
                    tok = set_m0(std::integral_constant<int, 3>{}, refill);
                    const v4i hi1 = *reinterpret_cast<const v4i*>(r1 + c1);
                    issue_copy(3, tok);
                    fb[1 - FP][0] = __builtin_shufflevector(lo0, hi0, 0, 1, 2, 3, 4, 5, 6, 7);
                    fb[1 - FP][1] = __builtin_shufflevector(lo1, hi1, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
            if constexpr (i < 4) fa[i % 4] = read_frag_b(cur, i + 4);
            else fa[i % 4] = read_frag_b(nxt, i - 4);
        });
        advance_copy();
        if constexpr (ODDK) stage_rt = STAGE - stage_rt;
    };

    using std::integral_constant;
    constexpr integral_constant<int, 0> P0{};
    constexpr integral_constant<int, 1> P1{};
    constexpr integral_constant<bool, true> Y{};
    constexpr integral_constant<bool, false> NO{};
    const int KT = k_total / kBK;  // even, or odd and at least 3 with ODDK
    int logical = xcd_first + slot;
    for (int t = 0; t < my_tiles; ++t) {
        if constexpr (FUSE_EPI) {  // where this tile's outputs go: needed by its last K-step
            int n_blk, m_blk;
            decode(logical, n_blk, m_blk);
            logical += tile_stride;
            const int e_lane = opaque(threadIdx.x) % 64;
            epi_lane = ((uint32_t)(4 * (e_lane / 16)) * (uint32_t)g.M + (uint32_t)(m_blk + wm * WTM + 8 * (e_lane % 16))) * 2u;
            epi_row0 = n_blk + wn * WT;
        }
        if constexpr (!ODDK && FUSE_EPI) {
            if (t == 0) k_step(P0, P0, Y, NO, NO);
            else k_step(P0, P0, Y, NO, Y);
            for (int kt = 1; kt + 1 < KT; kt += 2) {
                k_step(P1, P1, NO, NO, NO);
                k_step(P0, P0, NO, NO, NO);
            }
            k_step(P1, P1, NO, Y, NO);
        } else if constexpr (!ODDK) {
            k_step(P0, P0, Y, NO, NO);
            k_step(P1, P1, NO, NO, NO);
            for (int kt = 2; kt < KT; kt += 2) {
                k_step(P0, P0, NO, NO, NO);
                k_step(P1, P1, NO, NO, NO);
            }
        } else {
            // An odd number of K-steps: the LDS stage of a tile's first step alternates from tile to tile, so the
            // stage is a run-time value here (stage_rt, toggled by every step; the tags only name the fb half).  The
            // last step leaves the next tile's first second-operand fragments in fb half 1; they are moved to half
            // 0, where every tile starts.
            if (FUSE_EPI && t > 0) k_step(P0, P0, Y, NO, Y);
            else k_step(P0, P0, Y, NO, NO);
            k_step(P1, P1, NO, NO, NO);
            for (int kt = 3; kt < KT; kt += 2) {
                k_step(P0, P0, NO, NO, NO);
                k_step(P1, P1, NO, NO, NO);
            }
            k_step(P0, P0, NO, Y, NO);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < NJ; ++j) fb[0][j] = fb[1][j];
        }
        // the compiler does not know the statements above are matrix instructions: give the last ones time
        // to retire before their results are read (generously: four times the instruction's 32 cycles)
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
        if constexpr (FUSE_EPI) {
            // rows 0..3 went out under the last K-step; rows 4..7 go out under the next tile's first K-step, or here
            // after the workgroup's last tile
            prev_lane = epi_lane;
            prev_row0 = epi_row0;
            if (t + 1 == my_tiles) {
                static_for<0, 32>([&](auto k_tag) {
                    constexpr int k = decltype(k_tag)::value;
                    epi_slice(std::integral_constant<int, 4 + k / 8>{}, std::integral_constant<int, k % 8>{}, prev_row0, prev_lane);
                });
            }
            continue;
        }

        // Epilogue.  acc[i][j][r] is c row 16 i + 4 kg + r of the wave tile and, thanks to the a-tile row
        // permutation, column NJ l16 + j: a lane owns NJ adjacent columns of each of its 32 rows (8: one 16-byte
        // store per row; 6: one 12-byte store; 7: 6 adjacent columns and one of the wave half's last 16, a 12-byte
        // and a 2-byte store).  The bf16 stores
        // are non-temporal when operands and output together exceed the 256 MB last-level cache: the output (up to
        // 620 MB) is not read by this kernel again and would otherwise push the operands, which the other XCDs
        // still fetch, out of that cache (measured on one box, alternating builds: -3 to -10 % on outputs of
        // 270-620 MB).  When everything fits, ordinary stores are acknowledged sooner and the wait for them at the
        // next tile's second barrier is shorter (8192 x 8192 x 3584: 178 -> 167 us, K = 512: 48 -> 43 us).
        int n_blk, m_blk;
        decode(logical, n_blk, m_blk);
        logical += tile_stride;
        const float scale = out_scale;
        int ldc = BLK;
        OutT* c = reinterpret_cast<OutT*>(g.partial + ((int64_t)xcd * g.part_per_xcd + slot) * (BLK * BLK));
        if constexpr (SEG) {
            n_blk = m_blk = 0;  // tile-local coordinates in this slot's partial tile
        } else {
            ldc = g.M;
            c = reinterpret_cast<OutT*>(g.c);
        }
        // RAGGED: a tile moved back to end with the matrix leaves the rows / columns it shares with its neighbour to
        // that neighbour (with accumulation they must be written once)
        [[maybe_unused]] int n_own = n_blk, m_own = m_blk;
        if constexpr (RAGGED) {
            if (n_blk % BLK) n_own = (n_blk / BLK + 1) * BLK;
            if (m_blk % BLKM) m_own = (m_blk / BLKM + 1) * BLKM;
        }
        const int e_lane = opaque(threadIdx.x) % 64;
        const int el16 = e_lane % 16, ekg = e_lane / 16;
        const int m_lane = m_blk + wm * WTM + (NJ == 7 ? 6 : NJ) * el16;
        const uint32_t lane_bytes = ((uint32_t)(4 * ekg) * (uint32_t)ldc + (uint32_t)m_lane) * (uint32_t)sizeof(OutT);
        const int m_lane7 = m_blk + wm * WTM + 96 + el16;  // NJ = 7: the column of the seventh fragment
        const uint32_t lane_bytes7 = ((uint32_t)(4 * ekg) * (uint32_t)ldc + (uint32_t)m_lane7) * (uint32_t)sizeof(OutT);
        const int row0 = n_blk + wn * WT;
        auto rows = [&](auto bias_tag, auto acc_tag) {
            constexpr bool BIAS = decltype(bias_tag)::value;
            constexpr bool ACC = decltype(acc_tag)::value;
            typedef float v4fl __attribute__((ext_vector_type(4)));
            if constexpr (KMA && SEG) {
                // acc[i][j][r] is row 16 i + 4 ekg + r, column 16 j + el16 of the wave tile: the raw accumulators go to
                // the partial tile one by one (16 lanes fill 64 bytes of a row; the tile stays in the caches until
                // the reduction kernel reads it)
                LLMQ_GLOBAL float* pc = (LLMQ_GLOBAL float*)c + (row0 + 4 * ekg) * BLK + wm * WTM + el16;
#pragma unroll
                for (int i = 0; i < NF; ++i) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) pc[(16 * i + r) * BLK + 16 * j] = acc[i][j][r];
                    }
                }
            } else if constexpr (KMA && STAGE32) {
                // The general epilogue of the K-major first operand: fp32 or bf16 output, bias, accumulation.  acc[i][j][r] is
                // c row 16 i + 4 ekg + r, column 16 j + el16 of the wave tile; the old values of c and the bias belong to
                // whole row segments, so the raw accumulators change hands through LDS first: per fragment row i and
                // half hh, the wave writes the 8 c rows 4 q + 2 hh + rr (q = 0..3, rr = 0, 1) x 128 columns as fp32 into
                // its own piece of LDS (row 2 q + rr, row stride 544 bytes: the four row pairs of a write land on
                // different banks) and reads them back as 16 bytes per lane (piece p = lane + 64 t: row p / 32, columns
                // 4 (p % 32) ..+3); scale, bias, old value and the one rounding follow in the order of the other epilogues.
                // One wave's LDS operations are carried out in order, so no barrier is needed around the exchange.  Bias and
                // accumulation are run-time branches here (one copy of this code per kernel instance).
                uint8_t* es = lds + 2 * STAGE + wave * EPI32_STAGE;
                const uint32_t wr_ofs = (uint32_t)(2 * ekg) * EPI32_ROW + (uint32_t)el16 * 4u;
#pragma unroll
                for (int i = 0; i < NF; ++i) {
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
#pragma unroll
                            for (int rr = 0; rr < 2; ++rr)
                                *reinterpret_cast<float*>(es + wr_ofs + rr * EPI32_ROW + j * 64) = acc[i][j][2 * hh + rr];
                        }
#pragma unroll
                        for (int t4 = 0; t4 < 4; ++t4) {
                            const int p = e_lane + 64 * t4;
                            const int prow = p / 32, pcol = 4 * (p % 32);   // staged row 2 q + rr, first of four columns
                            const v4fl raw = *reinterpret_cast<const v4fl*>(es + prow * EPI32_ROW + pcol * 4);
                            const int crow = row0 + 16 * i + 4 * (prow / 2) + 2 * hh + (prow % 2);
                            const int ccol = m_blk + wm * WTM + pcol;
                            OutT* dst = c + (int64_t)crow * ldc + ccol;
                            float v[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                v[e] = raw[e] * scale;
                                if (g.bias) v[e] = v[e] + load_bias(g.bias, g.bias_is_bf16, ccol + e);
                            }
                            if (g.accumulate) {
                                float o0, o1, o2, o3;
                                PairIo<OutT>::load((const LLMQ_GLOBAL OutT*)dst, o0, o1);
                                PairIo<OutT>::load((const LLMQ_GLOBAL OutT*)(dst + 2), o2, o3);
                                v[0] = v[0] + o0;
                                v[1] = v[1] + o1;
                                v[2] = v[2] + o2;
                                v[3] = v[3] + o3;
                            }
                            if constexpr (std::is_same_v<OutT, uint16_t>) {
                                const f32x2_t lo2 = {v[0], v[1]}, hi2 = {v[2], v[3]};
                                typedef int v2i_g __attribute__((ext_vector_type(2)));
                                const v2i_g packed = {__builtin_bit_cast(int, __builtin_convertvector(lo2, bf16x2_t)),
                                                      __builtin_bit_cast(int, __builtin_convertvector(hi2, bf16x2_t))};
                                *(LLMQ_GLOBAL v2i_g*)dst = packed;
                            } else {
                                const v4fl out4 = {v[0], v[1], v[2], v[3]};
                                *(LLMQ_GLOBAL v4fl*)dst = out4;
                            }
                        }
                    }
                }
            } else if constexpr (KMA) {
                // acc[i][j][r] is c row 16 i + 4 ekg + r, column 16 j + el16 of the wave tile.  Per fragment row i the
                // wave writes its 16 x 128 outputs as bf16 into its own piece of LDS ([16 rows][256 bytes], the 32-byte
                // pieces of a row xor-ed with the row quad so that the four row quads of a write land on different
                // banks) and reads them back as 16 bytes per lane: row 4 q + lane / 16, columns 8 (lane % 16) ..+7.
                // One wave's LDS operations are carried out in order, so no barrier is needed around the exchange.
                uint8_t* es = lds + 2 * STAGE + wave * EPI_STAGE;
                float bias_c[NJ];
                if constexpr (BIAS) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) bias_c[j] = load_bias(g.bias, g.bias_is_bf16, m_blk + wm * WTM + 16 * j + el16);
                }
                const uint32_t wr_ofs = (uint32_t)(4 * ekg) * 256u + ((uint32_t)(el16 * 2) ^ (uint32_t)(ekg * 32));
                const uint32_t rd_ofs = (uint32_t)(e_lane / 16) * 256u + (uint32_t)(e_lane % 16) * 16u;
                const uint32_t out_bytes = ((uint32_t)(e_lane / 16) * (uint32_t)ldc + (uint32_t)(m_blk + wm * WTM + 8 * (e_lane % 16))) * 2u;
#pragma unroll
                for (int i = 0; i < NF; ++i) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
#pragma unroll
                        for (int r = 0; r < 4; r += 2) {
                            float v0 = acc[i][j][r] * scale, v1 = acc[i][j][r + 1] * scale;
                            if constexpr (BIAS) {
                                v0 = v0 + bias_c[j];
                                v1 = v1 + bias_c[j];
                            }
                            const f32x2_t pr = {v0, v1};
                            const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2_t));
                            uint8_t* w = es + (wr_ofs ^ (uint32_t)(32 * j)) + r * 256;   // column 16 j: byte 32 j of the row
                            *reinterpret_cast<uint16_t*>(w) = (uint16_t)pk;
                            *reinterpret_cast<uint16_t*>(w + 256) = (uint16_t)(pk >> 16);
                        }
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const v4i packed = *reinterpret_cast<const v4i*>(es + q * 1024 + (rd_ofs ^ (uint32_t)(32 * q)));
                        LLMQ_GLOBAL char* row_ptr = scalar_ptr((LLMQ_GLOBAL char*)(c + (int64_t)(row0 + 16 * i + 4 * q) * ldc));
                        if (NJ < 8 && e_lane % 16 >= 2 * NJ) continue;  // narrow tiles: the wave half is 16 NJ columns wide
                        if constexpr (STREAM_OUT) __builtin_nontemporal_store(packed, (LLMQ_GLOBAL v4i*)(row_ptr + out_bytes));
                        else *(LLMQ_GLOBAL v4i*)(row_ptr + out_bytes) = packed;
                    }
                }
            } else if constexpr (NJ < 8) {
                static_assert(NJ == 8 || !ACC, "the narrow tiles do not accumulate");
                float bias_n[NJ];
                if constexpr (BIAS) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        bias_n[j] = load_bias(g.bias, g.bias_is_bf16, (NJ == 7 && j == 6) ? m_lane7 : m_lane + j);
                }
                auto value = [&](int i, int j, int r) {
                    float v = acc[i][j][r] * scale;
                    if constexpr (BIAS) v = v + bias_n[j];
                    return v;
                };
                typedef int v3i_u __attribute__((ext_vector_type(3), aligned(4)));  // 12 bytes per lane
                typedef uint16_t u16_u __attribute__((aligned(2)));
#pragma unroll
                for (int i = 0; i < NF; ++i) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        LLMQ_GLOBAL char* row_ptr = scalar_ptr((LLMQ_GLOBAL char*)(c + (int64_t)(row0 + 16 * i + r) * ldc));
                        LLMQ_GLOBAL char* dst = row_ptr + lane_bytes;
                        v3i_u packed;
#pragma unroll
                        for (int j = 0; j < 3; ++j) {
                            const f32x2_t pr = {value(i, 2 * j, r), value(i, 2 * j + 1, r)};
                            packed[j] = __builtin_bit_cast(int, __builtin_convertvector(pr, bf16x2_t));
                        }
                        *(LLMQ_GLOBAL v3i_u*)dst = packed;
                        if constexpr (NJ == 7) {
                            const f32x2_t last = {value(i, NJ - 1, r), 0.f};
                            const uint32_t tail = __builtin_bit_cast(uint32_t, __builtin_convertvector(last, bf16x2_t));
                            *(LLMQ_GLOBAL u16_u*)(row_ptr + lane_bytes7) = (uint16_t)tail;
                        }
                    }
                }
            } else {
            float bias_v[8];
            static_assert(NJ >= 6 && NJ <= 8, "epilogue written for 6, 7 or 8 columns per lane");
            if constexpr (BIAS) {
#pragma unroll
                for (int j = 0; j < 8; ++j) bias_v[j] = load_bias(g.bias, g.bias_is_bf16, m_lane + j);
            }
#pragma unroll
            for (int i = 0; i < NF; ++i) {
                LLMQ_GLOBAL char* row[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    row[r] = scalar_ptr((LLMQ_GLOBAL char*)(c + (int64_t)(row0 + 16 * i + r) * ldc)) + lane_bytes;
                // RAGGED: does this lane own its 8 columns of the fragment row's c rows (see n_own / m_own)
                bool mine[4] = {true, true, true, true};
                if constexpr (RAGGED) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) mine[r] = m_lane >= m_own && row0 + 16 * i + r + 4 * ekg >= n_own;
                }
                // the old values of the fragment row's four c rows are requested together
                float old[4][8] = {};
                if constexpr (ACC) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (!mine[r]) continue;
                        if constexpr (std::is_same_v<OutT, uint16_t>) {
                            const v4i w = *(const LLMQ_GLOBAL v4i*)row[r];
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                old[r][2 * j] = __uint_as_float((uint32_t)w[j] << 16);
                                old[r][2 * j + 1] = __uint_as_float((uint32_t)w[j] & 0xFFFF0000u);
                            }
                        } else {
                            const v4fl lo = *(const LLMQ_GLOBAL v4fl*)row[r], hi = *(const LLMQ_GLOBAL v4fl*)(row[r] + 16);
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                old[r][j] = lo[j];
                                old[r][4 + j] = hi[j];
                            }
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        v[j] = acc[i][j][r] * scale;
                        if constexpr (BIAS) v[j] = v[j] + bias_v[j];
                        if constexpr (ACC) v[j] = v[j] + old[r][j];
                    }
                    if (!mine[r]) continue;
                    if constexpr (std::is_same_v<OutT, uint16_t>) {
                        v4i packed;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const f32x2_t pr = {v[2 * j], v[2 * j + 1]};
                            packed[j] = __builtin_bit_cast(int, __builtin_convertvector(pr, bf16x2_t));
                        }
                        if constexpr (STREAM_OUT) __builtin_nontemporal_store(packed, (LLMQ_GLOBAL v4i*)row[r]);
                        else *(LLMQ_GLOBAL v4i*)row[r] = packed;
                    } else {
                        const v4fl lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
                        *(LLMQ_GLOBAL v4fl*)row[r] = lo;  // two instructions interleave 16-byte pieces: left to the L2 to merge
                        *(LLMQ_GLOBAL v4fl*)(row[r] + 16) = hi;
                    }
                }
            }
            }  // NJ == 8
        };
        constexpr std::true_type yes{};
        constexpr std::false_type no{};
        if constexpr (SEG) {
            rows(no, no);
        } else if constexpr (KMA && STAGE32) {
            rows(no, no);
            pending_stores = false;  // old values may have been loaded: the next tile's first barrier waits for everything
        } else if constexpr (NJ != 8 || KMA) {
            if (g.bias) rows(yes, no);
            else rows(no, no);
            pending_stores = true;
        } else if (g.accumulate) {
            if (g.bias) rows(yes, yes);
            else rows(no, yes);
            // the loads of old values have been consumed; make the next tile's first barrier wait for
            // everything (its relaxed form counts stores only)
            pending_stores = false;
        } else {
            if (g.bias) rows(yes, no);
            else rows(no, no);
            // RAGGED: a wave may skip stores it does not own, so their number is not known to the relaxed wait
            pending_stores = !RAGGED;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the surplus copies issued during the last tile
}

// Sums the K segments of the last-round tiles that the four-wave kernel's segment launch left in
// g.partial (fixed order: the result does not depend on timing) and applies the epilogue.  One thread per
// 8 adjacent outputs; block -> (XCD, last-round tile t, 8-row band of the tile).  Must be launched with the
// same tile_stride, rem_split and part_per_xcd as the kernel that wrote the partial tiles.
template <typename OutT>
__global__ __launch_bounds__(256) void w4_segment_reduce_kernel(GemmArgs g, int tile_stride, int rem_max) {
    typedef float v4fl __attribute__((ext_vector_type(4)));
    const int band = blockIdx.x % 32, tr = blockIdx.x / 32;
    const int t = tr % rem_max, xcd = tr / rem_max;
    int xcd_first, xcd_count;
    xcd_tile_range((g.N / 256) * (g.M / 256), g.xcds, xcd, xcd_first, xcd_count);
    const int rem = xcd_count % tile_stride;
    if (t >= rem) return;
    int n_blk, m_blk;
    decode_tile256(g, xcd_first + xcd_count - rem + t, n_blk, m_blk);
    const int row = band * 8 + threadIdx.x / 32, col = (threadIdx.x % 32) * 8;
    const float* part = g.partial + ((int64_t)xcd * g.part_per_xcd + (int64_t)t * g.rem_split) * 65536 + row * 256 + col;
    v4fl lo = *reinterpret_cast<const v4fl*>(part), hi = *reinterpret_cast<const v4fl*>(part + 4);
    for (int q = 1; q < g.rem_split; ++q) {
        lo = lo + *reinterpret_cast<const v4fl*>(part + (int64_t)q * 65536);
        hi = hi + *reinterpret_cast<const v4fl*>(part + (int64_t)q * 65536 + 4);
    }
    float scale = g.sa ? *g.sa : 1.f;
    if (g.sb) scale = scale * *g.sb;
    const int m = m_blk + col;
    OutT* dst = reinterpret_cast<OutT*>(g.c) + (int64_t)(n_blk + row) * g.M + m;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        float v0 = (h < 2 ? lo[2 * h] : hi[2 * h - 4]) * scale, v1 = (h < 2 ? lo[2 * h + 1] : hi[2 * h - 3]) * scale;
        if (g.bias) {
            v0 = v0 + load_bias(g.bias, g.bias_is_bf16, m + 2 * h);
            v1 = v1 + load_bias(g.bias, g.bias_is_bf16, m + 2 * h + 1);
        }
        if (g.accumulate) {
            float o0, o1;
            PairIo<OutT>::load((const LLMQ_GLOBAL OutT*)(dst + 2 * h), o0, o1);
            v0 = v0 + o0;
            v1 = v1 + o1;
        }
        PairIo<OutT>::store((LLMQ_GLOBAL OutT*)(dst + 2 * h), v0, v1);
    }
}

// ---- general shapes ---------------------------------------------------------------------------------
// Any M, N >= 1 and any K that is a multiple of 16 (the 16-byte row alignment the reference's default backend asks
// for, src/kernels/matmul.cpp:55-57): 64 x 64 output tile per workgroup, 4 waves of 32 x 32 (one
// v_mfma_f32_32x32x64_f8f6f4 per K-step of 64), rows and K chunks beyond the operands read as zeros, every output
// element stored on its own.  It serves what the tiled kernels above cannot: an M or K off their lattice (the whole
// output) and the last N % 128 rows of an otherwise regular output (rows g.n_first .. N - 1).  Simple rather than fast:
// operands go through registers into a single LDS stage (row stride 80 bytes: the 16-byte reads of 32 consecutive
// rows spread over all banks), the next K-step's global loads are in flight while the current one is computed.
template <typename OutT, int B_FMT>
__global__ __launch_bounds__(256) void gemm_tn_e4m3_edge_kernel(GemmArgs g) {
    constexpr int TILE = 64, KS = 64, ROW = 80;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * TILE * ROW];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wn = wave / 2, wm = wave % 2, l32 = lane % 32, kg = lane / 32;
    const int n0 = g.n_first + blockIdx.y * TILE, m0 = blockIdx.x * TILE;
    // copies: thread -> (row tid / 4, 16-byte chunk tid % 4) of both operand tiles
    const int ld_row = tid / 4, ld_chunk = tid % 4;
    const bool b_ok = n0 + ld_row < g.N, a_ok = m0 + ld_row < g.M;
    const uint8_t* b_src = g.b + (int64_t)(b_ok ? n0 + ld_row : 0) * g.K + ld_chunk * 16;
    const uint8_t* a_src = g.a + (int64_t)(a_ok ? m0 + ld_row : 0) * g.K + ld_chunk * 16;
    const v4i zero = {0, 0, 0, 0};
    auto fetch = [&](int k0, v4i& vb, v4i& va) {
        const bool k_ok = k0 + ld_chunk * 16 < g.K;  // K is a multiple of 16: a chunk is inside or outside as a whole
        vb = (b_ok && k_ok) ? *reinterpret_cast<const v4i*>(b_src + k0) : zero;
        va = (a_ok && k_ok) ? *reinterpret_cast<const v4i*>(a_src + k0) : zero;
    };
    uint8_t* b_dst = lds + ld_row * ROW + ld_chunk * 16;
    uint8_t* a_dst = lds + TILE * ROW + ld_row * ROW + ld_chunk * 16;
    const uint8_t* b_frag = lds + (wn * 32 + l32) * ROW + kg * 32;
    const uint8_t* a_frag = lds + TILE * ROW + (wm * 32 + l32) * ROW + kg * 32;
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    v4i vb, va;
    fetch(0, vb, va);
    for (int k0 = 0; k0 < g.K; k0 += KS) {
        __syncthreads();  // the previous step's fragment reads are done
        *reinterpret_cast<v4i*>(b_dst) = vb;
        *reinterpret_cast<v4i*>(a_dst) = va;
        __syncthreads();
        if (k0 + KS < g.K) fetch(k0 + KS, vb, va);
        const v4i b_lo = *reinterpret_cast<const v4i*>(b_frag), b_hi = *reinterpret_cast<const v4i*>(b_frag + 16);
        const v4i a_lo = *reinterpret_cast<const v4i*>(a_frag), a_hi = *reinterpret_cast<const v4i*>(a_frag + 16);
        const v8i fb_ = __builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i fa_ = __builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7);
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb_, fa_, acc, B_FMT, 0, 0, 0, 0, 0);
    }
    // accumulator register r: c row 8 * (r / 4) + 4 * kg + r % 4 of the wave's 32 x 32 block, column l32
    float scale = g.sa ? *g.sa : 1.f;
    if (g.sb) scale = scale * *g.sb;
    const int m = m0 + wm * 32 + l32;
    if (m >= g.M) return;
    const float bias = g.bias ? load_bias(g.bias, g.bias_is_bf16, m) : 0.f;
    OutT* c = reinterpret_cast<OutT*>(g.c);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int n = n0 + wn * 32 + 8 * (r / 4) + 4 * kg + r % 4;
        if (n >= g.N) continue;
        float v = acc[r] * scale;
        if (g.bias) v = v + bias;
        OutT* dst = c + (int64_t)n * g.M + m;
        if constexpr (std::is_same_v<OutT, uint16_t>) {
            if (g.accumulate) v = v + __uint_as_float((uint32_t)*dst << 16);
            const f32x2_t pr = {v, 0.f};
            *dst = (uint16_t)(__builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2_t)) & 0xFFFFu);  // RNE
        } else {
            if (g.accumulate) v = v + *dst;
            *dst = v;
        }
    }
}

// ---- host side ------------------------------------------------------------------------------------
template <int BLK_N, int BLK_M, int WV_N, int WV_M, typename OutT, int B_FMT>
static int launch_pipe(const GemmArgs& g, int splits, int persistent_grid, hipStream_t stream) {
    const int tiles = (g.N / BLK_N) * (g.M / BLK_M);
    if (splits > 1) {
        hipLaunchKernelGGL((gemm_tn_e4m3_pipe_kernel<BLK_N, BLK_M, WV_N, WV_M, OutT, true, false, B_FMT>),
                           dim3((unsigned)tiles, (unsigned)splits), dim3(WV_N * WV_M * 64), 0, stream, g);
        LLMQ_HIP_TRY(hipGetLastError());
        const int64_t pairs = (int64_t)g.N * g.M / 2;
        hipLaunchKernelGGL((splitk_reduce_kernel<OutT>), dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream,
                           g, splits);
    } else if (persistent_grid > 0) {
        hipLaunchKernelGGL((gemm_tn_e4m3_pipe_kernel<BLK_N, BLK_M, WV_N, WV_M, OutT, false, true, B_FMT>),
                           dim3((unsigned)persistent_grid), dim3(WV_N * WV_M * 64), 0, stream, g);
    } else {
        hipLaunchKernelGGL((gemm_tn_e4m3_pipe_kernel<BLK_N, BLK_M, WV_N, WV_M, OutT, false, false, B_FMT>),
                           dim3((unsigned)tiles), dim3(WV_N * WV_M * 64), 0, stream, g);
    }
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// Kernel selection overrides, 0 / -1 = automatic.  They exist only in the test-aid build of this file
// (LLMQ_TEST_HOOKS), where the parity tests force every kernel instantiation in turn; in the product library
// they are constants and the dispatch below is a function of its arguments alone.  tile: 1 = 256 x 256 tile with
// 8 waves, 2 = 128 x 128 tile with 4 waves, 3 = four-wave kernel, 4 / 5 = its 224- / 192-wide tiles; for shapes off the
// lattice only 2 and 3 (the ragged instances of those kernels) and 6 = the 64 x 64 kernel.  splits:
// forced number of K splits (needs a workspace).  persist: -1 = automatic, 0 = never, 1 = whenever possible.
// fuse: -1 = automatic, 0 = the four-wave kernel's epilogue always after the K loop, 1 = under the last K-step wherever
// that instance exists (full-width bf16 tiles without bias and accumulation).
#ifdef LLMQ_TEST_HOOKS
static std::atomic<int> g_gemm_tile{0}, g_gemm_splits{0}, g_gemm_persist{-1}, g_gemm_fuse{-1};
#else
constexpr int g_gemm_tile = 0, g_gemm_splits = 0, g_gemm_persist = -1, g_gemm_fuse = -1;
#endif

// Launch plan of the four-wave kernel.  A persistent grid of `grid` workgroups (grid / 8 per XCD) walks
// tiles256 tiles.  When the last round of an XCD holds only a few tiles, those can be cut into rem_split K
// segments each, computed by a second launch into partial tiles in the workspace and summed by
// w4_segment_reduce_kernel: the round then takes 1 / rem_split of a tile's time, at the price of two more
// launches.  The decision uses measured figures (microseconds): a tile of depth K on an otherwise idle
// chip takes about K / 164 (twice as fast as in a full round); the operand bytes of the round stream at
// about 6 TB/s (10 TB/s when both operands fit the 256 MB last-level cache) whichever way the round is
// organised; the extra launches cost about 20, a partial tile 0.03 in the reduction.  Measured against it
// (us, whole launch, uncut / cut): 18944 x 3584 x 8192 (12 tiles left over) 388 / 362 with 4 segments;
// 3584 x 37888 x 8192 (24 left over) 758 / 742 with 3 to 5 segments; 18944 x 8192 x 3584 (64 left over, at most 2
// segments fit the workspace) 382 / 387: the first two are cut, the third is not.
struct W4Plan {
    int grid, rem_split, k_len, part_per_xcd, rem_max;
};
static W4Plan plan_w4(int tiles256, int cus, int xcds, int M, int N, int K, int forced_split, size_t workspace_bytes) {
    W4Plan p{tiles256 < cus ? (tiles256 + xcds - 1) / xcds * xcds : cus, 1, K, 0, 0};
    if (forced_split == 1 || K % (2 * kBK) != 0) return p;  // segments are whole pairs of K-steps
    const int stride = cus / xcds;
    const int xq = tiles256 / xcds, xr = tiles256 % xcds;
    // tiles in the last round of the XCDs (those with one tile more and the others)
    const int rem_hi = xr ? (xq + 1) % stride : 0, rem_lo = xq % stride;
    const int rem_max = rem_hi > rem_lo ? rem_hi : rem_lo;
    if (rem_max == 0) return p;
    const int pairs = K / (2 * kBK);  // segments are whole pairs of K-steps
    const int64_t ws_tiles = (int64_t)(workspace_bytes / (size_t)(256 * 256 * 4));
    const int rem_total = xr * rem_hi + (xcds - xr) * rem_lo;
    const double stream_us = (double)rem_total * 512.0 * K / (((double)M + N) * K <= 192e6 ? 10e6 : 6e6);
    const double tile_us = (double)K / 164.0;
    const double whole_us = tile_us > stream_us ? tile_us : stream_us;
    int best = 1;
    double best_gain = 5.0;  // what a cut must win to be worth it
    for (int s = 2; s <= stride / rem_max && s <= pairs; ++s) {
        const int seg_pairs = (pairs + s - 1) / s;
        if ((s - 1) * seg_pairs >= pairs) continue;  // would leave the last segment empty
        if ((int64_t)xcds * rem_max * s > ws_tiles) break;
        if (forced_split > 1) {
            if (s == forced_split) best = s;
            continue;
        }
        const double seg_us = tile_us * seg_pairs / pairs;
        const double cut_us = (seg_us > stream_us ? seg_us : stream_us) + 20.0 + 0.03 * rem_total * s;
        if (whole_us - cut_us > best_gain) {
            best_gain = whole_us - cut_us;
            best = s;
        }
    }
    if (best > 1) {
        p.grid = cus;
        p.rem_split = best;
        p.k_len = (pairs + best - 1) / best * 2 * kBK;
        p.part_per_xcd = rem_max * best;
        p.rem_max = rem_max;
    }
    return p;
}

// Kernel choice for outputs with less than one round of 256 x 256 tiles (weight gradients of narrow layers, small
// models), from estimated times in microseconds.  The constants come from measurements on this chip: a K-step of the
// four-wave kernel takes 0.9 us on a nearly idle chip and 1.4 us with every compute unit busy (the chip is power
// limited: the time grows with the square of the active fraction of the matrix work); a pair of co-resident
// 128 x 128 tiles advances one K-step in 0.47 to 0.85 us; a launch costs about 4-6 us, the second pass of a K split
// about 8 us plus its traffic at 4 TB/s.  Candidates: one round of 256-, 224- or 192-wide four-wave tiles, or
// 128 x 128 tiles with 1..8 K splits.  Checked against measured sweeps (7B / 1.5B / 0.5B weight-gradient shapes):
// the estimate picks the fastest or second-fastest variant, within 5 % of the fastest.
struct SmallPlan {
    int nj;      // 8, 7, 6: four-wave kernel with that many fragment columns per wave; 0: 128 x 128 tiles
    int splits;  // K splits of the 128 x 128 tiles
};
static SmallPlan plan_small(int M, int N, int K, int cus, bool ok256, bool ok224, bool ok192, int64_t ws_bytes) {
    const double kt = (double)K / kBK;
    SmallPlan best{0, 1};
    double best_us = 1e30;
    auto four_wave = [&](int nj, double penalty) {
        const int w = 32 * nj;
        const int64_t tiles = (int64_t)(N / 256) * (M / w);
        const int64_t rounds = (tiles + cus - 1) / cus;
        auto step = [&](double f) {
            const double x = f * w / 256.0;
            return (0.9 + 0.5 * x * x) * (w / 256.0) * penalty;
        };
        const double f_last = (double)(tiles - (rounds - 1) * cus) / cus;
        const double us = (rounds - 1) * (kt * step(1.0) + 6.0) + kt * step(f_last) + 6.0;
        if (us < best_us) {
            best_us = us;
            best = SmallPlan{nj, 1};
        }
    };
    if (ok256) four_wave(8, 1.0);
    if (ok224) four_wave(7, 1.05);
    if (ok192) four_wave(6, 1.08);
    const int64_t t128 = (int64_t)(N / 128) * (M / 128);
    const int64_t slice = (int64_t)N * M * 4;
    for (int sp = 1; sp <= 8; ++sp) {
        if (M % 128 != 0) break;
        if (sp > 1 && ((int64_t)sp * slice > ws_bytes || K / sp < 512)) break;
        const int64_t items = t128 * sp, slots = 2 * (int64_t)cus;
        const int64_t rounds = (items + slots - 1) / slots;
        const double f_last = (double)(items - (rounds - 1) * slots) / slots;
        double us = ((rounds - 1) * 0.85 + 0.47 + 0.38 * f_last) * (kt / sp) + 4.0 * rounds;
        if (sp > 1) us += 8.0 + (double)N * M * (4.0 * sp + 2.0) / 4e6;
        if (us < best_us) {
            best_us = us;
            best = SmallPlan{0, sp};
        }
    }
    return best;
}

// One launch of the four-wave kernel's main variant (no K segments); odd_k selects the instance for an odd number of
// K-steps.
template <typename OutT, int B_FMT, int NJ, bool STREAM_OUT, bool FUSE_EPI = false>
static void launch_w4(bool odd_k, int grid, const GemmArgs& g, hipStream_t stream) {
    if (odd_k)
        hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<OutT, B_FMT, false, NJ, STREAM_OUT, true, false, false, FUSE_EPI>),
                           dim3((unsigned)grid), dim3(256), 0, stream, g);
    else
        hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<OutT, B_FMT, false, NJ, STREAM_OUT, false, false, false, FUSE_EPI>),
                           dim3((unsigned)grid), dim3(256), 0, stream, g);
}

// Shapes off the tile lattice on the four-wave kernel (RAGGED instances): M and N from 256 up that need not be multiples
// of the tile (M a multiple of 8: the lane's 8 adjacent outputs start 16-byte aligned for bf16), K any multiple of 16
// from three K-steps up.  One persistent launch, whole 256 x 256 tiles, no cut of the last round.
template <typename OutT, int B_FMT>
static void launch_w4_ragged(const GemmArgs& g, int cus, int xcds, hipStream_t stream) {
    const int tiles = ((g.N + 255) / 256) * ((g.M + 255) / 256);
    const int grid = tiles < cus ? (tiles + xcds - 1) / xcds * xcds : cus;
    const int steps = (g.K + kBK - 1) / kBK;
    if (steps % 2)
        hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<OutT, B_FMT, false, 8, true, true, false, false, false, false, true>),
                           dim3((unsigned)grid), dim3(256), 0, stream, g);
    else
        hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<OutT, B_FMT, false, 8, true, false, false, false, false, false, true>),
                           dim3((unsigned)grid), dim3(256), 0, stream, g);
}

// Shapes off the tile lattice on 128 x 128 tiles (RAGGED instance of the 8-wave kernel family's four-wave configuration):
// any N, M a multiple of 8, K a multiple of 16.  One tile per workgroup, two workgroups per compute unit.
template <typename OutT, int B_FMT>
static int launch_pipe_ragged(const GemmArgs& g, hipStream_t stream) {
    const int64_t tiles = (int64_t)((g.N + 127) / 128) * ((g.M + 127) / 128);
    LLMQ_REQUIRE(tiles < ((int64_t)1 << 31), "matmul: too many tiles (%lld)", (long long)tiles);
    hipLaunchKernelGGL((gemm_tn_e4m3_pipe_kernel<128, 128, 2, 2, OutT, false, false, B_FMT, true>), dim3((unsigned)tiles),
                       dim3(256), 0, stream, g);
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}

// Which of the two ragged tilings is faster, from estimated times in microseconds: rounds of tiles over the chip (one
// 256 x 256 tile per compute unit, or two co-resident 128 x 128 tiles) times the K-steps of a tile at the measured cost
// of a step (1.4 / 1.0 us) plus a measured per-round cost (8 / 3 us: prologue, epilogue and the masked last step of the
// ragged four-wave instance).  Checked against a sweep of 42 shapes (M, N from 1000 to 16392, K from 400 to 8208): the
// estimate is within 10 % of the measured time and picks the faster kernel except where the two are within 5 %.
// Examples (us, 128 x 128 / four-wave): 1000 x 8192 x 3584 30 / 44, 2056 x 4100 x 3600 64 / 46, 4360 x 4100 x 656 28 / 33,
// 3584 x 8200 x 3600 131 / 90, 8200 x 8200 x 8208 649 / 448, 3000 x 16392 x 656 63 / 71.
static bool ragged_prefers_four_wave(int M, int N, int K, int cus) {
    const double steps = (double)((K + kBK - 1) / kBK);
    const int64_t t256 = (int64_t)((N + 255) / 256) * ((M + 255) / 256), t128 = (int64_t)((N + 127) / 128) * ((M + 127) / 128);
    const double r256 = (double)((t256 + cus - 1) / cus), r128 = (double)((t128 + 2 * cus - 1) / (2 * cus));
    return r256 * (1.4 * steps + 8.0) < r128 * (1.0 * steps + 3.0);
}

template <typename OutT, int B_FMT>
static int gemm_dispatch(GemmArgs g, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    LLMQ_REQUIRE(g.M > 0 && g.N > 0 && g.K > 0, "matmul: M, N, K must be positive (got %d, %d, %d)", g.M, g.N, g.K);
    const int cus = cu_count(), xcds = xcd_count();
    g.xcds = xcds;
    const int force_tile = g_gemm_tile, force_splits = g_gemm_splits, force_persist = g_gemm_persist;
    LLMQ_REQUIRE(g.K % 16 == 0, "matmul: K must be a multiple of 16 (rows of the fp8 operands are 16-byte aligned), got %d",
                 g.K);
    LLMQ_REQUIRE(g.a && g.b && g.c, "matmul: null operand pointer");
    LLMQ_REQUIRE(aligned16(g.a) && aligned16(g.b) && aligned16(g.c) && aligned16(g.bias) && aligned16(workspace),
                 "matmul: all pointers must be 16-byte aligned");
    LLMQ_REQUIRE(workspace != nullptr || workspace_bytes == 0, "matmul: workspace size given without a workspace");
    // The tiled kernels below work on a lattice: K a multiple of 128, M a multiple of 128 (or, for bf16 output
    // without accumulation, of 224 or 192) and N a multiple of 128 (256 for the narrow tiles).  Everything else goes
    // to the general-shape kernel: the whole output when M or K is off the lattice or N is below 128, otherwise the
    // last N % 128 rows while the tiled kernels take the rows before them (rows of c are independent, so the
    // split needs nothing but the row count).
    auto launch_edge = [&](int n_first) -> int {
        GemmArgs e = g;
        e.n_first = n_first;
        const dim3 grid((unsigned)((g.M + 63) / 64), (unsigned)((g.N - n_first + 63) / 64));
        hipLaunchKernelGGL((gemm_tn_e4m3_edge_kernel<OutT, B_FMT>), grid, dim3(256), 0, stream, e);
        LLMQ_HIP_TRY(hipGetLastError());
        return LLMQ_OK;
    };
    // K-step counts the four-wave kernel walks: even, or odd from 3 up
    const bool odd_k = g.K % (2 * kBK) == kBK;
    const bool w4_k = g.K % kBK == 0 && (!odd_k || g.K >= 3 * kBK);
    const bool narrow_out = std::is_same_v<OutT, uint16_t> && !g.accumulate && w4_k && cus % xcds == 0;
    const bool m_narrow = narrow_out && (g.M % 224 == 0 || g.M % 192 == 0);  // served by 256-row tiles only
    const bool on_lattice = g.K % kBK == 0 && (g.M % 128 == 0 || m_narrow) && g.N >= (g.M % 128 == 0 ? 128 : 256);
    if (!on_lattice) {
        // Three kernels serve shapes off the lattice: the four-wave kernel's ragged instances (whole 256 x 256 tiles,
        // moved back at the edges: M, N >= 256, K >= 384) and the ragged instance of the 128 x 128 tiles, whichever the
        // estimate above expects to be faster, both for M a multiple of 8 (the lane's 8 adjacent bf16 outputs start
        // 16-byte aligned); the 64 x 64 kernel for the rest (M % 8 != 0, or less than one 128 x 128 tile of outputs).
        LLMQ_REQUIRE(force_splits == 0 && (force_tile == 0 || force_tile == 2 || force_tile == 3 || force_tile == 6),
                     "matmul: M, N, K = %d, %d, %d are off the lattice of the forced kernel variant", g.M, g.N, g.K);
        const bool w4_fits = g.M >= 256 && g.N >= 256 && g.M % 8 == 0 && g.K >= 3 * kBK && cus % xcds == 0;
        const bool pipe_fits = g.M % 8 == 0;
        int pick = 6;
        if (force_tile != 0) {
            LLMQ_REQUIRE(force_tile == 6 || (force_tile == 3 ? w4_fits : pipe_fits),
                         "matmul: M, N, K = %d, %d, %d do not fit the forced ragged kernel", g.M, g.N, g.K);
            pick = force_tile;
        } else if (w4_fits && g_gemm_persist != 0 && ragged_prefers_four_wave(g.M, g.N, g.K, cus)) {
            pick = 3;
        } else if (pipe_fits && (int64_t)g.M * g.N >= 128 * 128) {
            pick = 2;
        }
        if (pick == 3) {
            g.group = 8;
            g.rem_split = 1;
            g.part_per_xcd = 0;
            launch_w4_ragged<OutT, B_FMT>(g, cus, xcds, stream);
            LLMQ_HIP_TRY(hipGetLastError());
            return LLMQ_OK;
        }
        if (pick == 2) {
            g.group = 8;
            return launch_pipe_ragged<OutT, B_FMT>(g, stream);
        }
        return launch_edge(0);
    }
    const int n_tail = g.N % (g.M % 128 == 0 ? 128 : 256);
    if (n_tail != 0) {
        LLMQ_REQUIRE(force_tile == 0 && force_splits == 0,
                     "matmul: M, N, K = %d, %d, %d are off the lattice of the forced kernel variant", g.M, g.N, g.K);
        const int rc = launch_edge(g.N - n_tail);
        if (rc != LLMQ_OK) return rc;
        g.N -= n_tail;
    }
    auto narrow_fits = [&](int width) { return narrow_out && g.N % 256 == 0 && g.M % width == 0; };
    const bool ok224 = narrow_fits(224), ok192 = narrow_fits(192);
    g.group = 8;
    int tile = force_tile;
    LLMQ_REQUIRE(tile >= 0 && tile <= 5, "matmul: unknown tile selector %d", tile);
    const bool fits256 = g.N % 256 == 0 && g.M % 256 == 0;
    LLMQ_REQUIRE((tile != 1 && tile != 3) || fits256, "matmul: the 256 x 256 tile needs M and N divisible by 256");
    const bool w4_ok = fits256 && w4_k && cus % xcds == 0;
    if (tile == 3) {
        LLMQ_REQUIRE(w4_ok, "matmul: the four-wave kernel needs K divisible by 128 and at least 256");
    }
    // The narrow tiles are taken when their whole rounds of 7/8- or 3/4-sized tiles beat the rounds of full tiles
    // by a margin, e.g. M = 3584, N = 8192: 512 tiles of 224 in 2 rounds instead of 448 in 1.75, on paper 12.5 %
    // less time.  Measured (alternating builds on one box): K = 18944 371 -> 357 us, K = 37888 860 -> 820 us, i.e.
    // 4-5 %: a narrow tile does 7/8 of the matrix work per barrier, copy and fragment-read overhead of a
    // K-step, and the 192 tiles of a three-quarter round run faster than those of a full one.  Hence the 8 %
    // (12 % for the 192-wide tile) the comparison below asks for.  The narrow tiles also serve an M that only
    // 224 or 192 divide.
    int narrow_nj = 0, small_splits = 0;
    if (tile == 4 || tile == 5) {
        LLMQ_REQUIRE(tile == 4 ? ok224 : ok192,
                     "matmul: the narrow tile (256 x %d) needs bf16 output without accumulation, N %% 256 == 0, "
                     "M %% %d == 0 and K %% 128 == 0, K >= 256", tile == 4 ? 224 : 192, tile == 4 ? 224 : 192);
        narrow_nj = tile == 4 ? 7 : 6;
    } else if (g.M % 128 != 0) {
        LLMQ_REQUIRE(tile == 0, "matmul: M = %d needs the narrow tile", g.M);
        narrow_nj = ok224 ? 7 : 6;
    } else if (tile == 0 && force_splits == 0 && (int64_t)(g.N / 256) * (g.M / 256) < cus) {
        const SmallPlan sp = plan_small(g.M, g.N, g.K, cus, w4_ok, ok224, ok192, workspace ? (int64_t)workspace_bytes : 0);
        if (sp.nj == 8) {
            tile = 3;
        } else if (sp.nj) {
            narrow_nj = sp.nj;
        } else {
            tile = 2;
            small_splits = sp.splits;
        }
    } else if (tile == 0 && w4_ok && force_splits == 0) {
        const int64_t tn = g.N / 256, t256 = tn * (g.M / 256), rem256 = t256 % cus;
        // only where the full tiles' last round would not be cut into K segments anyway (a remainder of 1-2
        // tiles per XCD), and never for less than a round of tiles
        if (t256 >= cus && (rem256 == 0 || rem256 > cus / xcds)) {
            auto rounds = [&](int64_t tiles) { return (double)((tiles + cus - 1) / cus); };
            double best = rounds(t256) * 8.0;
            if (ok224 && rounds(tn * (g.M / 224)) * 7.0 * 1.08 < best) {
                best = rounds(tn * (g.M / 224)) * 7.0 * 1.08;
                narrow_nj = 7;
            }
            if (ok192 && rounds(tn * (g.M / 192)) * 6.0 * 1.12 < best) narrow_nj = 6;
        }
    }
    if constexpr (std::is_same_v<OutT, uint16_t>) {
        if (narrow_nj) {
            const int tiles = (g.N / 256) * (g.M / (32 * narrow_nj));
            g.rem_split = 1;
            g.part_per_xcd = 0;
            const int grid = tiles < cus ? (tiles + xcds - 1) / xcds * xcds : cus;
            if (narrow_nj == 7) launch_w4<uint16_t, B_FMT, 7, true>(odd_k, grid, g, stream);
            else launch_w4<uint16_t, B_FMT, 6, true>(odd_k, grid, g, stream);
            LLMQ_HIP_TRY(hipGetLastError());
            return LLMQ_OK;
        }
    }
    if (tile == 0) {
        // Rounds of workgroups the chip needs: one 256 x 256 tile per compute unit and round (four units
        // of work), or two co-resident 128 x 128 tiles (two units, at about 0.8 of the rate per unit).
        const int64_t t256 = (int64_t)(g.N / 256) * (g.M / 256), t128 = (int64_t)(g.N / 128) * (g.M / 128);
        const double cost256 = 4.0 * (double)((t256 + cus - 1) / cus);
        const double cost128 = 2.0 * 1.25 * (double)((t128 + 2 * cus - 1) / (2 * cus));
        tile = (fits256 && t256 >= cus && cost256 <= cost128) ? 1 : 2;
    }

    // Split K when the tiles alone leave most of the chip idle: aim at about one workgroup per compute
    // unit, keep at least 512 elements of K per split, and stay inside the caller's workspace.
    const int64_t tiles = tile != 2 ? (int64_t)(g.N / 256) * (g.M / 256) : (int64_t)(g.N / 128) * (g.M / 128);
    const int64_t slice_bytes = (int64_t)g.N * g.M * 4;
    const int64_t ws_splits = (int64_t)(workspace_bytes / (size_t)slice_bytes);
    int splits = tile == 3 ? 1 : force_splits;  // for the four-wave kernel the knob cuts the last round instead
    LLMQ_REQUIRE(splits >= 0, "matmul: negative split count %d", splits);
    if (splits == 0 && small_splits > 0) {
        splits = small_splits;
    } else if (splits == 0) {
        splits = 1;
        if (2 * tiles <= cus && ws_splits >= 2) {
            int64_t want = cus / tiles;
            if (want > g.K / 512) want = g.K / 512;
            if (want > ws_splits) want = ws_splits;
            if (want > 1) splits = (int)want;
        }
    } else if (splits > 1) {
        LLMQ_REQUIRE(splits <= g.K / kBK, "matmul: %d splits for K = %d", splits, g.K);
        LLMQ_REQUIRE(ws_splits >= splits, "matmul: workspace of %zu bytes is too small for %d splits", workspace_bytes,
                     splits);
    }
    if (splits > 1) {
        const int steps = g.K / kBK;
        g.k_len = ((steps + splits - 1) / splits) * kBK;
        splits = (g.K + g.k_len - 1) / g.k_len;  // no empty split
        g.partial = reinterpret_cast<float*>(workspace);
    }
    // Persistent walk (one workgroup per compute unit) for the large tile when there is more than one
    // round of tiles; its cross-tile copy stream needs at least two K-steps.
    int persistent_grid = 0;
    const bool can_persist = tile == 1 && splits == 1 && g.K >= 2 * kBK && cus % xcds == 0;
    if (can_persist && (force_persist == 1 || (force_persist < 0 && tiles > cus))) persistent_grid = cus;
    // The four-wave kernel takes every large-tile launch it can (K a multiple of 256, no K split).
    if ((tile == 3 || (tile == 1 && force_tile == 0 && w4_ok)) && splits == 1) {
        const int tiles256 = (g.N / 256) * (g.M / 256);
        W4Plan plan = plan_w4(tiles256, cus, xcds, g.M, g.N, g.K, tile == 3 ? force_splits : 0, workspace ? workspace_bytes : 0);
        LLMQ_REQUIRE(tile != 3 || force_splits <= 1 || plan.rem_split == force_splits,
                     "matmul: cannot cut the last round into %d segments (K = %d, workspace %zu bytes)", force_splits,
                     g.K, workspace_bytes);
        g.rem_split = plan.rem_split;
        g.k_len = plan.k_len;
        g.part_per_xcd = plan.part_per_xcd;
        g.partial = reinterpret_cast<float*>(workspace);
        // operands and output together within the last-level cache: ordinary output stores (see the epilogue)
        const bool cached_out = std::is_same_v<OutT, uint16_t> &&
                                ((int64_t)g.M + g.N) * g.K + (int64_t)g.N * g.M * 2 <= ((int64_t)224 << 20);
        if constexpr (std::is_same_v<OutT, uint16_t>) {
            const int force_fuse = g_gemm_fuse;
            const bool fuse = force_fuse != 0 && g.bias == nullptr && !g.accumulate;
            if (fuse) {
                if (cached_out) launch_w4<uint16_t, B_FMT, 8, false, true>(odd_k, plan.grid, g, stream);
                else launch_w4<uint16_t, B_FMT, 8, true, true>(odd_k, plan.grid, g, stream);
            } else if (cached_out) {
                launch_w4<uint16_t, B_FMT, 8, false>(odd_k, plan.grid, g, stream);
            } else {
                launch_w4<uint16_t, B_FMT, 8, true>(odd_k, plan.grid, g, stream);
            }
        } else {
            launch_w4<OutT, B_FMT, 8, true>(odd_k, plan.grid, g, stream);
        }
        LLMQ_HIP_TRY(hipGetLastError());
        if (plan.rem_split > 1) {
            hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<float, B_FMT, true>), dim3((unsigned)plan.grid), dim3(256), 0,
                               stream, g);
            LLMQ_HIP_TRY(hipGetLastError());
            hipLaunchKernelGGL((w4_segment_reduce_kernel<OutT>), dim3((unsigned)(xcds * plan.rem_max * 32)), dim3(256), 0,
                               stream, g, plan.grid / xcds, plan.rem_max);
            LLMQ_HIP_TRY(hipGetLastError());
        }
        return LLMQ_OK;
    }
    if (tile == 1) return launch_pipe<256, 256, 2, 4, OutT, B_FMT>(g, splits, persistent_grid, stream);
    return launch_pipe<128, 128, 2, 2, OutT, B_FMT>(g, splits, 0, stream);
}

// Operands stored K-major (the reference's modes TT: b [K, N]; NN: a [K, M]; NT: both): the four-wave kernel's KMB / KMA
// instances, whole tiles only.
template <typename OutT, int B_FMT, bool KMA, bool KMB>
static int gemm_dispatch_kmajor(GemmArgs g, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    constexpr bool kBf16 = std::is_same_v<OutT, uint16_t>;
    static_assert(KMA || KMB, "mode TN goes through gemm_dispatch");
    const char* mode = KMA ? (KMB ? "NT" : "NN") : "TT";
    LLMQ_REQUIRE(g.M > 0 && g.N > 0 && g.K > 0, "matmul: M, N, K must be positive (got %d, %d, %d)", g.M, g.N, g.K);
    const int cus = cu_count(), xcds = xcd_count();
    g.xcds = xcds;
    g.group = 8;
    LLMQ_REQUIRE(g.a && g.b && g.c, "matmul: null operand pointer");
    LLMQ_REQUIRE(aligned16(g.a) && aligned16(g.b) && aligned16(g.c) && aligned16(g.bias) && aligned16(workspace),
                 "matmul: all pointers must be 16-byte aligned");
    LLMQ_REQUIRE(workspace != nullptr || workspace_bytes == 0, "matmul: workspace size given without a workspace");
    // Narrow tiles (bf16 output without accumulation): mode TT on 224-wide tiles for an M that only 224 divides; mode NN
    // on 224- or 192-wide tiles for such an M, and on 192-wide tiles for an M that 256 divides as well when whole rounds of
    // them beat the rounds of full tiles by the margin mode TN asks for (1536 x 16384 x 17920: 512 tiles of 192 in two
    // rounds instead of 384 of 256 in 1.5; measured 384 -> 343 us).  Not so the 224-wide tile: its rows of a K-major a
    // start at multiples of 224 bytes, off the 128-byte lines of the memory system three times out of four, and the
    // launch fetches 1.7 times the bytes of the full tiles (3584 x 8192 x 37888: 3.09 against 1.79 GB) for 1 % of time.
    const bool narrow_ok = kBf16 && !g.accumulate && !(KMA && KMB);
    int narrow_nj = 0;
    if (narrow_ok && g.M % 256 != 0) {
        if (g.M % 224 == 0) narrow_nj = 7;
        else if (KMA && g.M % 192 == 0) narrow_nj = 6;
    } else if (narrow_ok && KMA && g.N % 256 == 0 && g_gemm_tile == 0) {
        const int64_t tn = g.N / 256, t256 = tn * (g.M / 256), rem256 = t256 % cus;
        if (t256 >= cus && (rem256 == 0 || rem256 > cus / xcds)) {
            auto rounds = [&](int64_t tiles) { return (double)((tiles + cus - 1) / cus); };
            if (g.M % 192 == 0 && rounds(tn * (g.M / 192)) * 6.0 * 1.12 < rounds(t256) * 8.0) narrow_nj = 6;
        }
    }
    const bool m224 = narrow_nj != 0;
    LLMQ_REQUIRE(g.N % 256 == 0 && g.K % 256 == 0 && (g.M % 256 == 0 || m224) && cus % xcds == 0,
                 "matmul: a K-major operand (mode %s) needs N %% 256 == 0, K %% 256 == 0 and M %% 256 == 0 (with bf16 output and "
                 "without accumulation also M %% 224 == 0 in modes TT and NN, M %% 192 == 0 in mode NN); got M, N, K = %d, %d, %d",
                 mode, g.M, g.N, g.K);
    // the copies of a K-major operand address it as "tile base + 32-bit lane offset", and that offset walks the
    // whole K extent of the operand
    LLMQ_REQUIRE(!KMB || (int64_t)g.K * g.N < ((int64_t)1 << 31), "matmul: the K-major second operand must be smaller than 2 GiB "
                 "(K * N = %lld bytes)", (long long)((int64_t)g.K * g.N));
    LLMQ_REQUIRE(!KMA || (int64_t)g.K * g.M < ((int64_t)1 << 31), "matmul: the K-major first operand must be smaller than 2 GiB "
                 "(K * M = %lld bytes)", (long long)((int64_t)g.K * g.M));
    const int tiles = (g.N / 256) * (narrow_nj ? g.M / (32 * narrow_nj) : g.M / 256);
    const bool cached_out = ((int64_t)g.M + g.N) * g.K + (int64_t)g.N * g.M * 2 <= ((int64_t)224 << 20);
    if constexpr (kBf16 && !(KMA && KMB)) {
        if (narrow_nj) {
            const int grid = tiles < cus ? (tiles + xcds - 1) / xcds * xcds : cus;
            g.rem_split = 1;
            g.part_per_xcd = 0;
            if (narrow_nj == 7)
                hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<uint16_t, B_FMT, false, 7, true, false, KMB, KMA>), dim3((unsigned)grid),
                                   dim3(256), 0, stream, g);
            else if constexpr (KMA)
                hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<uint16_t, B_FMT, false, 6, true, false, KMB, KMA>), dim3((unsigned)grid),
                                   dim3(256), 0, stream, g);
            LLMQ_HIP_TRY(hipGetLastError());
            return LLMQ_OK;
        }
    }
    // the last, partial round of tiles cut into K segments as in mode TN (needs the caller's workspace)
    const int force_tile = g_gemm_tile, force_splits = g_gemm_splits;
    const W4Plan plan = plan_w4(tiles, cus, xcds, g.M, g.N, g.K, force_tile == 3 ? force_splits : 0, workspace ? workspace_bytes : 0);
    LLMQ_REQUIRE(force_tile != 3 || force_splits <= 1 || plan.rem_split == force_splits,
                 "matmul: cannot cut the last round into %d segments (K = %d, workspace %zu bytes)", force_splits, g.K,
                 workspace_bytes);
    g.rem_split = plan.rem_split;
    g.k_len = plan.k_len;
    g.part_per_xcd = plan.part_per_xcd;
    g.partial = reinterpret_cast<float*>(workspace);
    // The K-major first operand has two epilogues: bf16 output without accumulation goes out as packed bf16 through
    // LDS; fp32 output and accumulation take the fp32-staged one.  A K-major second operand alone changes nothing about
    // the epilogue (the lane owns adjacent columns as in mode TN).
    const bool general = KMA && (!kBf16 || g.accumulate);
    if constexpr (KMA) {
        if (general) {
            hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<OutT, B_FMT, false, 8, true, false, KMB, true, false, true>),
                               dim3((unsigned)plan.grid), dim3(256), 0, stream, g);
        }
    }
    if constexpr (kBf16) {
        if (!general) {
            if (cached_out)
                hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<uint16_t, B_FMT, false, 8, false, false, KMB, KMA>), dim3((unsigned)plan.grid),
                                   dim3(256), 0, stream, g);
            else
                hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<uint16_t, B_FMT, false, 8, true, false, KMB, KMA>), dim3((unsigned)plan.grid),
                                   dim3(256), 0, stream, g);
        }
    } else if constexpr (!KMA) {
        hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<float, B_FMT, false, 8, true, false, KMB, false>), dim3((unsigned)plan.grid),
                           dim3(256), 0, stream, g);
    }
    LLMQ_HIP_TRY(hipGetLastError());
    if (plan.rem_split > 1) {
        hipLaunchKernelGGL((gemm_tn_e4m3_w4_kernel<float, B_FMT, true, 8, true, false, KMB, KMA>), dim3((unsigned)plan.grid),
                           dim3(256), 0, stream, g);
        LLMQ_HIP_TRY(hipGetLastError());
        hipLaunchKernelGGL((w4_segment_reduce_kernel<OutT>), dim3((unsigned)(xcds * plan.rem_max * 32)), dim3(256), 0, stream,
                           g, plan.grid / xcds, plan.rem_max);
        LLMQ_HIP_TRY(hipGetLastError());
    }
    return LLMQ_OK;
}

}  // namespace llmq

namespace llmq {
// One call of the reference's matmul with an operand mode (EMMTranspose numbering: TT = 0, TN = 1, NT = 2, NN = 3).
template <typename OutT>
static int gemm_with_mode(GemmArgs g, void* workspace, size_t workspace_bytes, int mode, int b_format, hipStream_t st) {
    LLMQ_REQUIRE(b_format == 0 || b_format == 1, "matmul: unknown fp8 format %d of the second operand", b_format);
    if (mode == LLMQ_MODE_TN)
        return b_format ? gemm_dispatch<OutT, 1>(g, workspace, workspace_bytes, st) : gemm_dispatch<OutT, 0>(g, workspace, workspace_bytes, st);
    if (mode == LLMQ_MODE_TT)
        return b_format ? gemm_dispatch_kmajor<OutT, 1, false, true>(g, workspace, workspace_bytes, st)
                        : gemm_dispatch_kmajor<OutT, 0, false, true>(g, workspace, workspace_bytes, st);
    if (mode == LLMQ_MODE_NN)
        return b_format ? gemm_dispatch_kmajor<OutT, 1, true, false>(g, workspace, workspace_bytes, st)
                        : gemm_dispatch_kmajor<OutT, 0, true, false>(g, workspace, workspace_bytes, st);
    LLMQ_REQUIRE(mode == LLMQ_MODE_NT, "matmul: unknown operand mode %d (TT = 0, TN = 1, NT = 2, NN = 3)", mode);
    return b_format ? gemm_dispatch_kmajor<OutT, 1, true, true>(g, workspace, workspace_bytes, st)
                    : gemm_dispatch_kmajor<OutT, 0, true, true>(g, workspace, workspace_bytes, st);
}
}  // namespace llmq

extern "C" int llmq_gemm_e4m3_bf16_mode(uint16_t* c, const uint8_t* a, const uint8_t* b, const uint16_t* bias_or_null,
                                        const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                                        size_t workspace_bytes, int M, int N, int K, int mode, int b_format, int accumulate,
                                        void* stream) {
    llmq::GemmArgs g{c, a, b, bias_or_null, sa_or_null, sb_or_null, M, N, K, 1, accumulate, 8, nullptr, 0, 1, 0, 8, 0};
    return llmq::gemm_with_mode<uint16_t>(g, workspace_or_null, workspace_bytes, mode, b_format, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_gemm_e4m3_f32_mode(float* c, const uint8_t* a, const uint8_t* b, const void* bias_or_null, int bias_is_bf16,
                                       const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                                       size_t workspace_bytes, int M, int N, int K, int mode, int b_format, int accumulate,
                                       void* stream) {
    llmq::GemmArgs g{c, a, b, bias_or_null, sa_or_null, sb_or_null, M, N, K, bias_is_bf16, accumulate, 8, nullptr, 0, 1, 0, 8, 0};
    return llmq::gemm_with_mode<float>(g, workspace_or_null, workspace_bytes, mode, b_format, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_gemm_tn_e4m3_bf16(uint16_t* c, const uint8_t* a, const uint8_t* b, const uint16_t* bias_or_null,
                                      const float* sa_or_null, const float* sb_or_null, void* workspace_or_null,
                                      size_t workspace_bytes, int M, int N, int K, int accumulate, void* stream) {
    llmq::GemmArgs g{c, a, b, bias_or_null, sa_or_null, sb_or_null, M, N, K, 1, accumulate, 8, nullptr, 0, 1, 0, 8, 0};
    return llmq::gemm_dispatch<uint16_t, 0>(g, workspace_or_null, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_gemm_tn_e4m3_f32(float* c, const uint8_t* a, const uint8_t* b, const void* bias_or_null,
                                     int bias_is_bf16, const float* sa_or_null, const float* sb_or_null,
                                     void* workspace_or_null, size_t workspace_bytes, int M, int N, int K,
                                     int accumulate, void* stream) {
    llmq::GemmArgs g{c, a, b, bias_or_null, sa_or_null, sb_or_null, M, N, K, bias_is_bf16, accumulate, 8, nullptr, 0, 1, 0, 8, 0};
    return llmq::gemm_dispatch<float, 0>(g, workspace_or_null, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_gemm_tn_e4m3_e5m2_bf16(uint16_t* c, const uint8_t* a, const uint8_t* b_e5m2,
                                           const uint16_t* bias_or_null, const float* sa_or_null, const float* sb_or_null,
                                           void* workspace_or_null, size_t workspace_bytes, int M, int N, int K,
                                           int accumulate, void* stream) {
    llmq::GemmArgs g{c, a, b_e5m2, bias_or_null, sa_or_null, sb_or_null, M, N, K, 1, accumulate, 8, nullptr, 0, 1, 0, 8, 0};
    return llmq::gemm_dispatch<uint16_t, 1>(g, workspace_or_null, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_gemm_tn_e4m3_e5m2_f32(float* c, const uint8_t* a, const uint8_t* b_e5m2, const void* bias_or_null,
                                          int bias_is_bf16, const float* sa_or_null, const float* sb_or_null,
                                          void* workspace_or_null, size_t workspace_bytes, int M, int N, int K,
                                          int accumulate, void* stream) {
    llmq::GemmArgs g{c, a, b_e5m2, bias_or_null, sa_or_null, sb_or_null, M, N, K, bias_is_bf16, accumulate, 8, nullptr, 0, 1, 0, 8, 0};
    return llmq::gemm_dispatch<float, 1>(g, workspace_or_null, workspace_bytes, static_cast<hipStream_t>(stream));
}

#ifdef LLMQ_TEST_HOOKS
// Test-aid build only (not part of the drop-in surface, absent from the product library).
extern "C" __attribute__((visibility("default"))) void llmq_debug_set_gemm_variant(int tile, int splits) {
    llmq::g_gemm_tile = tile;
    llmq::g_gemm_splits = splits;
}
extern "C" __attribute__((visibility("default"))) void llmq_debug_set_gemm_persist(int v) { llmq::g_gemm_persist = v; }
extern "C" __attribute__((visibility("default"))) void llmq_debug_set_gemm_fuse(int v) { llmq::g_gemm_fuse = v; }
#endif
