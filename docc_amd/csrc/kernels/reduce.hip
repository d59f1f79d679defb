// Reduce tensor nodes (ml::Sum, ml::Max, ml::Min, ml::Mean) over a block of adjacent axes, fp32
// and fp64, for gfx950.
//
// The reference expands a ReduceNode into an initialisation nest and a nest that accumulates
// through memory, left to right (sdfg/src/data_flow/library_nodes/math/tensor/reduce_node.cpp:
// 188-333; identities and combiners: sum_node.cpp:20-57 `0` and `+`, max_node.cpp:56-91
// `-INFINITY` and fmax, min_node.cpp `INFINITY` and fmin; Mean is Sum followed by a division by
// the number of reduced elements, mean_node.cpp). Here the input is seen as [outer, reduce, inner]:
//   inner == 1  one wavefront per output element: 128-bit loads strided over the wave, a tree
//               over the lanes at the end (HBM-bound: one read of X); long rows that are too few
//               to give every CU its wavefronts are cut into pieces, a wavefront each, whose
//               results a second launch reduces
//   inner  > 1  one lane per output element, walking the reduced extent with stride `inner`, so
//               that neighbouring lanes read neighbouring addresses; when there are too few
//               output elements to fill the device the reduced extent is cut into slices, one
//               work-group row per slice, whose partial results go through a buffer of the launcher in
//               device memory and are combined, in slice order, by a second launch
// Sums are therefore added in another order than the reference's loop: equal to it within the
// usual bound (reduce * epsilon * sum|x|), exactly equal for Max and Min.
#include "common.h"

namespace docc_k {

enum ReduceOp : int { kSum = 0, kMax = 1, kMin = 2, kMean = 3 };

template <int OP, typename T>
__device__ __forceinline__ T reduce_identity() {
    if (OP == kMax) return -__builtin_huge_val();
    if (OP == kMin) return __builtin_huge_val();
    return (T) 0;
}

template <int OP>
__device__ __forceinline__ float combine(float a, float b) {
    if (OP == kMax) return fmaxf(a, b);
    if (OP == kMin) return fminf(a, b);
    return a + b;
}
template <int OP>
__device__ __forceinline__ double combine(double a, double b) {
    if (OP == kMax) return fmax(a, b);
    if (OP == kMin) return fmin(a, b);
    return a + b;
}

template <int OP, typename T>
__device__ __forceinline__ T wave_combine(T v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = combine<OP>(v, __shfl_xor(v, off, kWave));
    return v;
}

// the wavefront's reduction over x[0..R), in every lane; nvec = R / VEC when x is 16-byte aligned, else 0
template <typename T, int OP, int VEC>
__device__ __forceinline__ T wave_row(const T* x, long R, long nvec) {
    typedef T V __attribute__((ext_vector_type(VEC)));
    const int lane = threadIdx.x & 63;
    {   // (a block of its own: the vector loop's index is declared again by the element loop below)
        T acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = reduce_identity<OP, T>();
        // four loads in flight per lane, combined in the order of the plain loop
        constexpr int U = 4;
        long i = lane;
        for (; i + (U - 1) * kWave < nvec; i += U * kWave) {
            V v[U];
#pragma unroll
            for (int u = 0; u < U; u++) v[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(x) + i + u * kWave);
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[e] = combine<OP>(acc[e], v[u][e]);
        }
        for (; i < nvec; i += kWave) {
            const V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(x) + i);
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] = combine<OP>(acc[e], v[e]);
        }
        T a = acc[0];
#pragma unroll
        for (int e = 1; e < VEC; e++) a = combine<OP>(a, acc[e]);
        for (long i = nvec * VEC + lane; i < R; i += kWave) a = combine<OP>(a, x[i]);
        return wave_combine<OP>(a);
    }
}

// Y[row] = reduce over X[row, 0..R); nvec = R / VEC when rows are 16-byte aligned, else 0
template <typename T, int OP, int VEC>
__device__ __forceinline__ void row_reduce(const T* X, T* Y, long rows, long R, long nvec) {
    const int lane = threadIdx.x & 63;
    const long waves = (long) gridDim.x * (256 >> 6);
    for (long row = (long) blockIdx.x * (256 >> 6) + (threadIdx.x >> 6); row < rows; row += waves) {
        const T a = wave_row<T, OP, VEC>(X + row * R, R, nvec);
        if (lane == 0) Y[row] = OP == kMean ? a / (T) R : a;
    }
}

// Short rows (at most 32 vectors, 16-byte aligned): LPR lanes a row with one vector each, 64 / LPR rows per wavefront and
// four such sets in turn, all loaded before the first is reduced; a wavefront per row would leave most lanes idle.
template <typename T, int OP, int VEC, int LPR>
__device__ __forceinline__ void row_reduce_short(const T* X, T* Y, long rows, long R) {
    typedef T V __attribute__((ext_vector_type(VEC)));
    constexpr int RPW = kWave / LPR, SETS = 4;
    const int lane = threadIdx.x & 63, l = lane % LPR, g = lane / LPR;
    const int nvec = (int) (R / VEC);
    const long first = ((long) blockIdx.x * (256 >> 6) + (threadIdx.x >> 6)) * (RPW * SETS) + g;
    const V* xv = reinterpret_cast<const V*>(X);
    V v[SETS];
    bool live[SETS];
#pragma unroll
    for (int i = 0; i < SETS; i++) {
        const long row = first + (long) i * RPW;
        live[i] = row < rows && l < nvec;
        if (live[i]) v[i] = __builtin_nontemporal_load(xv + row * nvec + l);
    }
#pragma unroll
    for (int i = 0; i < SETS; i++) {
        T a = reduce_identity<OP, T>();
        if (live[i]) {
#pragma unroll
            for (int e = 0; e < VEC; e++) a = combine<OP>(a, v[i][e]);
        }
#pragma unroll
        for (int off = LPR / 2; off >= 1; off >>= 1) a = combine<OP>(a, __shfl_xor(a, off, kWave));
        const long row = first + (long) i * RPW;
        if (l == 0 && row < rows) Y[row] = OP == kMean ? a / (T) R : a;
    }
}

// Rows too few to give every CU its wavefronts: a row is cut into `slices` pieces of `chunk` elements (a multiple of
// the vector; the last piece may be shorter), a wavefront reduces a piece into P[row, slice], and a second launch
// reduces the rows of P (Mean: adds in both, and divides by the row length at the end). `vec`: rows start on
// 16-byte boundaries.
template <typename T, int OP, int VEC>
__device__ __forceinline__ void row_reduce_pieces(void* partials, const T* X, long rows, long R, long chunk, long slices, int vec) {
    constexpr int PART = OP == kMean ? kSum : OP;
    T* P = reinterpret_cast<T*>(partials);
    const int lane = threadIdx.x & 63;
    const long waves = (long) gridDim.x * (256 >> 6), pieces = rows * slices;
    for (long piece = (long) blockIdx.x * (256 >> 6) + (threadIdx.x >> 6); piece < pieces; piece += waves) {
        const long row = piece / slices, c0 = (piece % slices) * chunk;
        const long len = c0 + chunk < R ? chunk : R - c0;
        const T a = wave_row<T, PART, VEC>(X + row * R + c0, len, vec ? len / VEC : 0);
        if (lane == 0) P[piece] = a;
    }
}

template <typename T, int OP>
__device__ __forceinline__ void row_reduce_finish(const void* partials, T* Y, long rows, long R, long slices) {
    constexpr int PART = OP == kMean ? kSum : OP;
    const T* P = reinterpret_cast<const T*>(partials);
    const int lane = threadIdx.x & 63;
    const long waves = (long) gridDim.x * (256 >> 6);
    for (long row = (long) blockIdx.x * (256 >> 6) + (threadIdx.x >> 6); row < rows; row += waves) {
        const T a = wave_row<T, PART, 1>(P + row * slices, slices, 0);
        if (lane == 0) Y[row] = OP == kMean ? a / (T) R : a;
    }
}

// Y[o, i] = reduce over r of X[o, r, i]
template <typename T, int OP>
__device__ __forceinline__ void column_reduce(const T* X, T* Y, long outer, long R, long inner) {
    const long total = outer * inner;
    const long stride = (long) gridDim.x * 256;
    for (long idx = (long) blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
        const long o = idx / inner, i = idx % inner;
        const T* x = X + o * R * inner + i;
        T a0 = reduce_identity<OP, T>(), a1 = a0, a2 = a0, a3 = a0;
        long r = 0;
        for (; r + 4 <= R; r += 4) {   // four independent chains keep the loads in flight
            a0 = combine<OP>(a0, x[(r + 0) * inner]);
            a1 = combine<OP>(a1, x[(r + 1) * inner]);
            a2 = combine<OP>(a2, x[(r + 2) * inner]);
            a3 = combine<OP>(a3, x[(r + 3) * inner]);
        }
        for (; r < R; r++) a0 = combine<OP>(a0, x[r * inner]);
        const T a = combine<OP>(combine<OP>(a0, a1), combine<OP>(a2, a3));
        Y[idx] = OP == kMean ? a / (T) R : a;
    }
}

// Partial results of the sliced column reduction live in `partials`, device memory of the launcher:
// [slice][outer * inner] elements. Every call that slices writes the part it reads back, so nothing has
// to be cleared.

// P[s, o, i] = reduce over the rows of slice s of X[o, r, i]; grid.y = number of slices. Each lane
// owns VEC neighbouring columns (inner % VEC == 0, X 16-byte aligned when VEC > 1): one 128-bit load
// per row.
template <typename T, int OP, int VEC>
__device__ __forceinline__ void column_reduce_partial(void* partials, const T* X, long outer, long R, long inner, long chunk) {
    typedef T V __attribute__((ext_vector_type(VEC)));
    T* P = reinterpret_cast<T*>(partials);
    const long total = outer * inner;
    const long idx = ((long) blockIdx.x * 256 + threadIdx.x) * VEC;
    if (idx >= total) return;
    const long r0 = (long) blockIdx.y * chunk, r1 = min(R, r0 + chunk);
    const long o = idx / inner, i = idx % inner;
    const T* x = X + o * R * inner + i;
    V a0, a1;
#pragma unroll
    for (int e = 0; e < VEC; e++) a0[e] = a1[e] = reduce_identity<OP, T>();
    long r = r0;
    for (; r + 2 <= r1; r += 2) {   // two independent chains keep the loads in flight
        const V v0 = __builtin_nontemporal_load(reinterpret_cast<const V*>(x + (r + 0) * inner));
        const V v1 = __builtin_nontemporal_load(reinterpret_cast<const V*>(x + (r + 1) * inner));
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            a0[e] = combine<OP>(a0[e], v0[e]);
            a1[e] = combine<OP>(a1[e], v1[e]);
        }
    }
    for (; r < r1; r++) {
        const V v0 = *reinterpret_cast<const V*>(x + r * inner);
#pragma unroll
        for (int e = 0; e < VEC; e++) a0[e] = combine<OP>(a0[e], v0[e]);
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) a0[e] = combine<OP>(a0[e], a1[e]);
    *reinterpret_cast<V*>(P + (long) blockIdx.y * total + idx) = a0;
}

// Y[idx] = combine over the slices of P[s, idx]. A work-group takes 16 neighbouring output
// elements; 16 lanes per element each combine every 16th slice, then one lane combines the 16
// partial values in order (the order of the additions is fixed by the launch geometry alone).
template <typename T, int OP>
__device__ __forceinline__ void column_reduce_final(const void* partials, T* Y, long total, long R, long slices) {
    __shared__ T part[16][17];
    const T* P = reinterpret_cast<const T*>(partials);
    const int col = threadIdx.x & 15, lane_s = threadIdx.x >> 4;
    const long idx = (long) blockIdx.x * 16 + col;
    T a = reduce_identity<OP, T>();
    if (idx < total) {
        // eight loads in flight, combined in slice order: one load at a time is one memory round trip per slice
        long s = lane_s;
        for (; s + 7 * 16 < slices; s += 8 * 16) {
            T v[8];
#pragma unroll
            for (int k = 0; k < 8; k++) v[k] = P[(s + 16 * k) * total + idx];
#pragma unroll
            for (int k = 0; k < 8; k++) a = combine<OP>(a, v[k]);
        }
        for (; s < slices; s += 16) a = combine<OP>(a, P[s * total + idx]);
    }
    part[lane_s][col] = a;
    __syncthreads();
    if (lane_s == 0 && idx < total) {
        T r = part[0][col];
#pragma unroll
        for (int k = 1; k < 16; k++) r = combine<OP>(r, part[k][col]);
        Y[idx] = OP == kMean ? r / (T) R : r;
    }
}

// DOT::BLAS: sum_i x[i * incx] * y[i * incy] (reference dot_node.cpp:76-165: one fma per element; the BLAS
// dispatcher prints cblas_?dot). Work-group b takes elements [b * chunk, (b + 1) * chunk) and leaves its sum in
// partials[b]; the second launch (one work-group) adds the partial sums in order and writes the result behind
// them, at partials[groups]. The split depends on n and the launch geometry alone, so the result is reproducible.
template <typename T>
__device__ __forceinline__ void dot_partial(void* partials, const T* __restrict__ x, long incx, const T* __restrict__ y, long incy, long n,
                                            long chunk) {
    __shared__ T part[4];
    const long i0 = (long) blockIdx.x * chunk, i1 = min(n, i0 + chunk);
    T a0 = (T) 0, a1 = (T) 0;
    long i = i0 + threadIdx.x;
    for (; i + 256 < i1; i += 512) {      // two independent chains
        a0 = __builtin_fma(x[i * incx], y[i * incy], a0);
        a1 = __builtin_fma(x[(i + 256) * incx], y[(i + 256) * incy], a1);
    }
    if (i < i1) a0 = __builtin_fma(x[i * incx], y[i * incy], a0);
    T a = a0 + a1;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) a += __shfl_xor(a, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) reinterpret_cast<T*>(partials)[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
}

template <typename T>
__device__ __forceinline__ void dot_final(void* partials, int groups) {
    __shared__ T part[256];
    T* P = reinterpret_cast<T*>(partials);
    T a = (T) 0;
    for (int g = threadIdx.x; g < groups; g += 256) a += P[g];
    part[threadIdx.x] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        T r = (T) 0;
        for (int k = 0; k < 256; k++) r += part[k];
        P[groups] = r;
    }
}

} // namespace docc_k

#define DOCC_DOT(SFX, T)                                                                                                       \
    extern "C" __global__ __launch_bounds__(256) void docc_dot_partial_##SFX(void* partials, const T* x, long incx, const T* y, \
                                                                             long incy, long n, long chunk) {                  \
        docc_k::dot_partial<T>(partials, x, incx, y, incy, n, chunk);                                                          \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_dot_final_##SFX(void* partials, int groups) {                          \
        docc_k::dot_final<T>(partials, groups);                                                                                \
    }
DOCC_DOT(f32, float)
DOCC_DOT(f64, double)

#define DOCC_REDUCE_SHORT(NAME, OP, LPR)                                                                                       \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_rows##LPR##_##NAME##_f32(const float* X, float* Y, long rows, long R) { \
        docc_k::row_reduce_short<float, docc_k::OP, 4, LPR>(X, Y, rows, R);                                                    \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_rows##LPR##_##NAME##_f64(const double* X, double* Y, long rows, long R) { \
        docc_k::row_reduce_short<double, docc_k::OP, 2, LPR>(X, Y, rows, R);                                                   \
    }
#define DOCC_REDUCE_SHORT_ALL(NAME, OP) \
    DOCC_REDUCE_SHORT(NAME, OP, 1) DOCC_REDUCE_SHORT(NAME, OP, 2) DOCC_REDUCE_SHORT(NAME, OP, 4) DOCC_REDUCE_SHORT(NAME, OP, 8) \
    DOCC_REDUCE_SHORT(NAME, OP, 16) DOCC_REDUCE_SHORT(NAME, OP, 32)
DOCC_REDUCE_SHORT_ALL(sum, kSum)
DOCC_REDUCE_SHORT_ALL(max, kMax)
DOCC_REDUCE_SHORT_ALL(min, kMin)
DOCC_REDUCE_SHORT_ALL(mean, kMean)

#define DOCC_REDUCE(NAME, OP)                                                                                                  \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_row_##NAME##_f32(const float* X, float* Y, long rows, long R,   \
                                                                                   long nvec) {                                \
        docc_k::row_reduce<float, docc_k::OP, 4>(X, Y, rows, R, nvec);                                                         \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_rowp_##NAME##_f32(void* P, const float* X, long rows, long R,   \
                                                                                    long chunk, long slices, int vec) {        \
        docc_k::row_reduce_pieces<float, docc_k::OP, 4>(P, X, rows, R, chunk, slices, vec);                                    \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_rowp_##NAME##_f64(void* P, const double* X, long rows, long R,  \
                                                                                    long chunk, long slices, int vec) {        \
        docc_k::row_reduce_pieces<double, docc_k::OP, 2>(P, X, rows, R, chunk, slices, vec);                                   \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_rowf_##NAME##_f32(const void* P, float* Y, long rows, long R,   \
                                                                                    long slices) {                             \
        docc_k::row_reduce_finish<float, docc_k::OP>(P, Y, rows, R, slices);                                                   \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_rowf_##NAME##_f64(const void* P, double* Y, long rows, long R,  \
                                                                                    long slices) {                             \
        docc_k::row_reduce_finish<double, docc_k::OP>(P, Y, rows, R, slices);                                                  \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_row_##NAME##_f64(const double* X, double* Y, long rows, long R, \
                                                                                   long nvec) {                                \
        docc_k::row_reduce<double, docc_k::OP, 2>(X, Y, rows, R, nvec);                                                        \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_col_##NAME##_f32(const float* X, float* Y, long outer, long R,  \
                                                                                   long inner) {                               \
        docc_k::column_reduce<float, docc_k::OP>(X, Y, outer, R, inner);                                                       \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_col_##NAME##_f64(const double* X, double* Y, long outer,        \
                                                                                   long R, long inner) {                       \
        docc_k::column_reduce<double, docc_k::OP>(X, Y, outer, R, inner);                                                      \
    }

#define DOCC_REDUCE_SLICED(NAME, OP, SFX, T)                                                                                   \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_colp_##NAME##_##SFX(void* partials, const T* X, long outer, long R, \
                                                                                      long inner, long chunk) {                \
        docc_k::column_reduce_partial<T, docc_k::OP, 1>(partials, X, outer, R, inner, chunk);                                  \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_colpv_##NAME##_##SFX(void* partials, const T* X, long outer, long R, \
                                                                                       long inner, long chunk) {               \
        docc_k::column_reduce_partial<T, docc_k::OP, 16 / sizeof(T)>(partials, X, outer, R, inner, chunk);                     \
    }                                                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_reduce_colf_##NAME##_##SFX(const void* partials, T* Y, long total, long R, \
                                                                                      long slices) {                           \
        docc_k::column_reduce_final<T, docc_k::OP>(partials, Y, total, R, slices);                                             \
    }

DOCC_REDUCE(sum, kSum)
DOCC_REDUCE(max, kMax)
DOCC_REDUCE(min, kMin)
DOCC_REDUCE(mean, kMean)
DOCC_REDUCE_SLICED(sum, kSum, f32, float)
DOCC_REDUCE_SLICED(sum, kSum, f64, double)
DOCC_REDUCE_SLICED(max, kMax, f32, float)
DOCC_REDUCE_SLICED(max, kMax, f64, double)
DOCC_REDUCE_SLICED(min, kMin, f32, float)
DOCC_REDUCE_SLICED(min, kMin, f64, double)
DOCC_REDUCE_SLICED(mean, kMean, f32, float)
DOCC_REDUCE_SLICED(mean, kMean, f64, double)
