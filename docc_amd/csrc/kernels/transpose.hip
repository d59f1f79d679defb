// ml::Transpose for gfx950: Y = X with its axes permuted, any rank up to six, elements of 1, 2, 4 or 8
// bytes (the node moves bits; the reference allows integer element types too: transpose_node.h:47).
//
// Replaces the loop nest the node expands to (reference
// sdfg/src/data_flow/library_nodes/math/tensor/transpose_node.cpp: one Map per axis around a copy
// tasklet). HBM-bound: one read and one write per element. The launcher drops axes of extent one and
// merges axes that stay adjacent, then picks one of two kernels:
//   rows   the innermost axis stays innermost: rows of contiguous elements move as they are, one thread per
//          unit of up to 16 bytes (the widest that divides a row and both alignments), the outer coordinates
//          select the input row;
//   tile   the innermost input axis `a` and the innermost output axis `b` differ: a work-group moves a
//          64 x 64 tile of the (b, a) plane through LDS, reading along `a` and writing along `b`, so that
//          both sides of the copy are contiguous 64-element segments; the remaining axes number the tiles.
//          4-byte elements with everything a multiple of four elements move in 128-bit units (tile4).
#include "common.h"

namespace docc_k {

// mirrored by the launcher (csrc/rt/ops_transpose.cpp)
struct TransposeParams {
    long n;                // elements
    int rank;              // axes in `ext` (output order; for the tile kernel without a and b)
    long ext[6];
    long in_stride[6];     // input stride of each of those axes, in elements
    long out_stride[6];    // output stride (tile kernel only; the rows kernel writes linearly)
    long a_ext, b_ext;     // tile kernel: extents of the two planes' axes
    long a_out_stride;     // output stride of axis a (its input stride is 1)
    long b_in_stride;      // input stride of axis b (its output stride is 1)
    long tiles_a, tiles_b;
};

// I: unsigned when the element count fits 32 bits (the divisions are the cost of this kernel), else long
template <typename T, typename I>
__device__ __forceinline__ void transpose_rows(const T* __restrict__ X, T* __restrict__ Y, const TransposeParams& p) {
    const I n = (I) p.n, stride = (I) gridDim.x * 256;
    for (I i = (I) blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        I rem = i;
        long off = 0;
#pragma unroll
        for (int d = 5; d >= 0; d--) {
            if (d < p.rank) {
                const I e = (I) p.ext[d];
                const I q = rem / e;
                off += (long) (rem - q * e) * p.in_stride[d];
                rem = q;
            }
        }
        Y[i] = X[off];
    }
}

template <typename T>
__device__ __forceinline__ void transpose_tile(const T* __restrict__ X, T* __restrict__ Y, const TransposeParams& p) {
    __shared__ T tile[64][65];   // one element of padding: the column reads below touch 64 different banks
    long t = blockIdx.x;
    const long ta = t % p.tiles_a;
    t /= p.tiles_a;
    const long tb = t % p.tiles_b;
    long rem = t / p.tiles_b, in_base = 0, out_base = 0;
#pragma unroll
    for (int d = 5; d >= 0; d--) {
        if (d < p.rank) {
            const long e = p.ext[d], c = rem % e;
            rem /= e;
            in_base += c * p.in_stride[d];
            out_base += c * p.out_stride[d];
        }
    }
    const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
    const long a0 = ta * 64, b0 = tb * 64;
    // rows of the tile are values of b, columns values of a
#pragma unroll 4
    for (int r = part; r < 64; r += 4) {
        const long a = a0 + lane, b = b0 + r;
        if (a < p.a_ext && b < p.b_ext) tile[r][lane] = X[in_base + b * p.b_in_stride + a];
    }
    __syncthreads();
#pragma unroll 4
    for (int r = part; r < 64; r += 4) {
        const long a = a0 + r, b = b0 + lane;
        if (a < p.a_ext && b < p.b_ext) Y[out_base + a * p.a_out_stride + b] = tile[lane][r];
    }
}

// The same tile for 4-byte elements when both extents, every stride and both addresses are multiples of four
// elements: 128-bit loads along `a` (four rows of the tile per wavefront and instruction, all four of a lane's loads
// in flight) and 128-bit stores along `b`, the transposition done by four 32-bit LDS reads down a column. Row r of
// the tile starts at bank r (65 words a row), so the sixteen vectors of a row and the four rows of a wavefront fall
// on 64 different banks both ways. Plain loads and stores: with non-temporal ones this kernel took 56.5 us on
// [8192,4096] (the one-element tile 44.8, this one 42.5).
__device__ __forceinline__ void transpose_tile_v4(const float* __restrict__ X, float* __restrict__ Y, const TransposeParams& p) {
    typedef float V __attribute__((ext_vector_type(4)));
    __shared__ float tile[64][65];
    long t = blockIdx.x;
    const long ta = t % p.tiles_a;
    t /= p.tiles_a;
    const long tb = t % p.tiles_b;
    long rem = t / p.tiles_b, in_base = 0, out_base = 0;
#pragma unroll
    for (int d = 5; d >= 0; d--) {
        if (d < p.rank) {
            const long e = p.ext[d], c = rem % e;
            rem /= e;
            in_base += c * p.in_stride[d];
            out_base += c * p.out_stride[d];
        }
    }
    const int c4 = threadIdx.x & 15, row = threadIdx.x >> 4;
    const long a0 = ta * 64, b0 = tb * 64;
    V v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const long a = a0 + 4 * c4, b = b0 + row + 16 * k;
        if (a < p.a_ext && b < p.b_ext) v[k] = *reinterpret_cast<const V*>(X + in_base + b * p.b_in_stride + a);
    }
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) tile[row + 16 * k][4 * c4 + e] = v[k][e];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const long a = a0 + row + 16 * k, b = b0 + 4 * c4;
        V o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = tile[4 * c4 + e][row + 16 * k];
        if (a < p.a_ext && b < p.b_ext) *reinterpret_cast<V*>(Y + out_base + a * p.a_out_stride + b) = o;
    }
}

// The same with a tile of 128 x 128, for large tensors: rows of 512 bytes on both sides (5-13 % faster on tensors met for
// the first time, slower where it leaves fewer than four tiles per CU); p.tiles_a / p.tiles_b count tiles of 128.
// The tile is not padded (64 KB): column c of row r lives at c ^ (r & 63).
__device__ __forceinline__ void transpose_tile_v4_wide(const float* __restrict__ X, float* __restrict__ Y, const TransposeParams& p) {
    typedef float V __attribute__((ext_vector_type(4)));
    __shared__ float tile[128][128];
    long t = blockIdx.x;
    const long ta = t % p.tiles_a;
    t /= p.tiles_a;
    const long tb = t % p.tiles_b;
    long rem = t / p.tiles_b, in_base = 0, out_base = 0;
#pragma unroll
    for (int d = 5; d >= 0; d--) {
        if (d < p.rank) {
            const long e = p.ext[d], c = rem % e;
            rem /= e;
            in_base += c * p.in_stride[d];
            out_base += c * p.out_stride[d];
        }
    }
    const int c4 = threadIdx.x & 31, row = threadIdx.x >> 5;
    const long a0 = ta * 128, b0 = tb * 128;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        V v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const long a = a0 + 4 * c4, b = b0 + row + 8 * (k + 8 * half);
            if (a < p.a_ext && b < p.b_ext) v[k] = *reinterpret_cast<const V*>(X + in_base + b * p.b_in_stride + a);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int r = row + 8 * (k + 8 * half);
#pragma unroll
            for (int e = 0; e < 4; e++) tile[r][(4 * c4 + e) ^ (r & 63)] = v[k][e];
        }
    }
    __syncthreads();
#pragma unroll 4
    for (int k = 0; k < 16; k++) {
        const int ar = row + 8 * k;
        const long a = a0 + ar, b = b0 + 4 * c4;
        V o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = tile[4 * c4 + e][ar ^ ((4 * c4 + e) & 63)];
        if (a < p.a_ext && b < p.b_ext) *reinterpret_cast<V*>(Y + out_base + a * p.a_out_stride + b) = o;
    }
}

} // namespace docc_k

extern "C" __global__ __launch_bounds__(256) void docc_transpose_tile4w_b32(const float* X, float* Y, docc_k::TransposeParams p) {
    docc_k::transpose_tile_v4_wide(X, Y, p);
}

extern "C" __global__ __launch_bounds__(256) void docc_transpose_tile4_b32(const float* X, float* Y, docc_k::TransposeParams p) {
    docc_k::transpose_tile_v4(X, Y, p);
}

#define DOCC_TRANSPOSE_ROWS(BITS, T)                                                                                                  \
    extern "C" __global__ __launch_bounds__(256) void docc_transpose_rows_b##BITS##_i32(const T* X, T* Y, docc_k::TransposeParams p) { \
        docc_k::transpose_rows<T, unsigned>(X, Y, p);                                                                                 \
    }                                                                                                                                 \
    extern "C" __global__ __launch_bounds__(256) void docc_transpose_rows_b##BITS##_i64(const T* X, T* Y, docc_k::TransposeParams p) { \
        docc_k::transpose_rows<T, long>(X, Y, p);                                                                                     \
    }
// rows are moved in the widest unit (up to 128 bits) that divides them and the alignment of both tensors
DOCC_TRANSPOSE_ROWS(128, docc_k::u32x4)
#define DOCC_TRANSPOSE(BITS, T)                                                                                             \
    DOCC_TRANSPOSE_ROWS(BITS, T)                                                                                             \
    extern "C" __global__ __launch_bounds__(256) void docc_transpose_tile_b##BITS(const T* X, T* Y, docc_k::TransposeParams p) { \
        docc_k::transpose_tile<T>(X, Y, p);                                                                                  \
    }
DOCC_TRANSPOSE(8, unsigned char)
DOCC_TRANSPOSE(16, unsigned short)
DOCC_TRANSPOSE(32, unsigned int)
DOCC_TRANSPOSE(64, unsigned long)
