// Byte (fp8 code) matrix transpose for gfx950: dst[c*rows + r] = src[r*cols + c].
//
// Replaces the reference's transpose_kernel for 1-byte types (src/kernels/transpose.cu:9-32,
// src/kernels/transpose_template.cuh:10-34).  Pure data movement, HBM bound (1 byte read + 1 byte
// written per element).
//
// Fast path (rows % 16 == 0 and cols % 16 == 0): a workgroup moves a [256 rows] x [128 cols] tile.
// Each lane reads 16 bytes from each of four consecutive rows (8 lanes cover a 128-byte row segment),
// transposes the four 4x4 byte blocks in registers with byte-permute instructions, writes the
// resulting dwords into an LDS tile laid out [col][row] (stride 65 dwords, see the kernel), and the tile is then
// written out as 16-byte pieces, 256 contiguous bytes per transposed row.
// Any other shape takes a simple bounds-checked 64 x 64 tile kernel.
#include "common.hpp"

namespace llmq {

constexpr int kTrRows = 256;
constexpr int kTrCols = 128;
constexpr int kTrStride = 65;

// byte k of a, b, c, d -> one dword per k (a in the lowest byte)
__device__ __forceinline__ void transpose4x4(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t out[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
    const uint32_t t1 = __builtin_amdgcn_perm(b, a, 0x07030602u);  // a2 b2 a3 b3
    const uint32_t u0 = __builtin_amdgcn_perm(d, c, 0x05010400u);  // c0 d0 c1 d1
    const uint32_t u1 = __builtin_amdgcn_perm(d, c, 0x07030602u);  // c2 d2 c3 d3
    out[0] = __builtin_amdgcn_perm(u0, t0, 0x05040100u);
    out[1] = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
    out[2] = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
    out[3] = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
}

// ROW_MAJOR_GRID: consecutive workgroups walk along the input rows (so concurrently running groups
// write neighbouring 256-byte segments of the same output rows) instead of along the input columns.
template <bool ROW_MAJOR_GRID>
__global__ __launch_bounds__(256) void transpose_u8_kernel(uint8_t* __restrict__ dst,
                                                           const uint8_t* __restrict__ src, int rows, int cols) {
    __shared__ uint32_t tile[kTrCols * kTrStride];
    const int t = threadIdx.x;
    const int r0 = (ROW_MAJOR_GRID ? blockIdx.x : blockIdx.y) * kTrRows;
    const int c0 = (ROW_MAJOR_GRID ? blockIdx.y : blockIdx.x) * kTrCols;
    const int chunk = t % 8;  // 16-column chunk
    const int q = t / 8;      // row quad within a pass (32 per pass, 2 passes)
    const int col = c0 + 16 * chunk;
    // LDS has 64 banks of 4 bytes and the row stride is 65 dwords: the dword written by lane (chunk, q) lands on bank
    // 16 chunk + q + const (mod 64), so chunks c and c + 4 would share banks (a two-way conflict on every write).
    // Flipping bit 3 of the row-quad index for the upper four chunks gives them the other half of each group of 16
    // banks; the reads below undo it.  Measured: the conflict counter goes from 0.67 to 0.50 of the LDS cycles (the
    // rest are the four-dword reads); the kernel's rate does not change, it is bound by its global access pattern.
    const int wr_flip = (chunk >> 2) * 8;

    uint4 v[2][4];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = r0 + 4 * (q + 32 * p) + j;
            if (row < rows && col < cols) {
                v[p][j] = load_nt(reinterpret_cast<const uint4*>(src + (int64_t)row * cols + col));
            } else {
                v[p][j] = make_uint4(0, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int rq = q + 32 * p;
        const uint32_t w[4][4] = {{v[p][0].x, v[p][0].y, v[p][0].z, v[p][0].w},
                                  {v[p][1].x, v[p][1].y, v[p][1].z, v[p][1].w},
                                  {v[p][2].x, v[p][2].y, v[p][2].z, v[p][2].w},
                                  {v[p][3].x, v[p][3].y, v[p][3].z, v[p][3].w}};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t o[4];
            transpose4x4(w[0][k], w[1][k], w[2][k], w[3][k], o);
#pragma unroll
            for (int b = 0; b < 4; ++b) tile[(16 * chunk + 4 * k + b) * kTrStride + (rq ^ wr_flip)] = o[b];
        }
    }
    __syncthreads();
    constexpr int ITEMS = kTrCols * (kTrRows / 16);
#pragma unroll
    for (int it = 0; it < ITEMS / 256; ++it) {
        const int item = t + 256 * it;
        const int c = item / 16, p = item % 16;
        const int r = r0 + 16 * p;
        if (c0 + c < cols && r < rows) {
            const uint32_t* s = &tile[c * kTrStride + 4 * (p ^ ((c >> 6) * 2))];
            *reinterpret_cast<uint4*>(dst + (int64_t)(c0 + c) * rows + r) = make_uint4(s[0], s[1], s[2], s[3]);
        }
    }
}

// Any shape: 64 x 64 byte tile through LDS, one byte per lane access.
__global__ __launch_bounds__(256) void transpose_u8_generic_kernel(uint8_t* __restrict__ dst,
                                                                   const uint8_t* __restrict__ src, int rows,
                                                                   int cols) {
    __shared__ uint8_t tile[64][65];
    const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    for (int j = ty; j < 64; j += 4) {
        const int r = r0 + j, c = c0 + tx;
        if (r < rows && c < cols) tile[j][tx] = src[(int64_t)r * cols + c];
    }
    __syncthreads();
    for (int j = ty; j < 64; j += 4) {
        const int c = c0 + j, r = r0 + tx;
        if (r < rows && c < cols) dst[(int64_t)c * rows + r] = tile[tx][j];
    }
}

}  // namespace llmq

extern "C" int llmq_transpose_u8(uint8_t* dst, const uint8_t* src, int rows, int cols, void* stream) {
    using namespace llmq;
    LLMQ_REQUIRE(rows >= 0 && cols >= 0, "transpose: negative shape %d x %d", rows, cols);
    if (rows == 0 || cols == 0) return LLMQ_OK;
    LLMQ_REQUIRE(dst != nullptr && src != nullptr, "transpose: null tensor pointer");
    LLMQ_REQUIRE(dst != src, "transpose: in-place transpose is not supported");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (rows % 16 == 0 && cols % 16 == 0 && aligned16(src) && aligned16(dst)) {
        const unsigned gc = (unsigned)((cols + kTrCols - 1) / kTrCols), gr = (unsigned)((rows + kTrRows - 1) / kTrRows);
        if (gc <= 65535u) {
            hipLaunchKernelGGL(transpose_u8_kernel<true>, dim3(gr, gc), dim3(256), 0, st, dst, src, rows, cols);
        } else {
            hipLaunchKernelGGL(transpose_u8_kernel<false>, dim3(gc, gr), dim3(256), 0, st, dst, src, rows, cols);
        }
    } else {
        dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
        hipLaunchKernelGGL(transpose_u8_generic_kernel, grid, dim3(256), 0, st, dst, src, rows, cols);
    }
    LLMQ_HIP_TRY(hipGetLastError());
    return LLMQ_OK;
}
