// Matrix-vector forms of the GEMM node for gfx950: a product with one output column or one output row moves
// the matrix once and computes two flops per element, so it is HBM-bound (4 or 8 bytes per element) and the
// MFMA tiles of the GEMM kernels - built for 64 and more columns - would idle. Two kernels cover the four
// cases (C = alpha * op(A) op(B) + beta * C with n == 1 or m == 1, either operand transposed or not):
//   rows   y[i] = alpha * <M[i, :], x> + beta * y[i]      the matrix's rows are contiguous: one wavefront per row,
//          128-bit loads, the vector comes from the caches;
//   cols   y[j] = alpha * sum_p x[p] * M[p, j] + beta * y[j]   a lane owns columns (contiguous across lanes), the
//          rows are cut into slices over work-groups whose partial sums meet in a buffer of the launcher; a second
//          launch adds them in slice order, so the result does not depend on scheduling.
// fp32 sums in fp32, fp64 in fp64 (cblas_?gemm semantics, reference gemm_node.cpp:474-505), bf16 operands (raw
// 16-bit words) in fp32 with an fp32 result, like the bf16 GEMM; when beta == 0, y is not read.
#include "common.h"

#ifndef DOCC_GEMV_COL_CHAINS
#define DOCC_GEMV_COL_CHAINS 2
#endif

namespace docc_k {

template <typename T>
__device__ __forceinline__ T gemv_wave_sum(T v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// element as stored -> the type the sums run in
template <typename T, typename In> __device__ __forceinline__ T gemv_value(In v) { return (T) v; }
template <> __device__ __forceinline__ float gemv_value<float, unsigned short>(unsigned short v) { return bf16_bits_to_f32(v); }

// In: element type of the matrix and the vector, T: type of the sums and of y.
// VEC elements per load when the launcher found rows and vector aligned, else 1
template <typename In, typename T, int VEC>
__device__ __forceinline__ void gemv_rows(const In* __restrict__ M, long ld, const In* __restrict__ x, long incx, T* __restrict__ y, long incy,
                                          long rows, long k, T alpha, T beta) {
    typedef In V __attribute__((ext_vector_type(VEC)));
    const int lane = threadIdx.x & 63;
    const long row = (long) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const In* m = M + row * ld;
    T acc = (T) 0;
    if (VEC > 1) {
        const long nv = k / VEC;
        const V* mv = reinterpret_cast<const V*>(m);
        const V* xv = reinterpret_cast<const V*>(x);
        // four loads of the row in flight per lane (one at a time the wave waited out every load: 43.7 us for 8192 x 8192
        // fp32); the products are added in the order of the plain loop
        constexpr int U = 4;
        long c = lane;
        for (; c + (U - 1) * 64 < nv; c += U * 64) {
            V a[U], b[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                a[u] = __builtin_nontemporal_load(mv + c + u * 64);
                b[u] = xv[c + u * 64];
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int e = 0; e < VEC; e++) acc += gemv_value<T, In>(a[u][e]) * gemv_value<T, In>(b[u][e]);
        }
        for (; c < nv; c += 64) {
            const V a = __builtin_nontemporal_load(mv + c);
            const V b = xv[c];
#pragma unroll
            for (int e = 0; e < VEC; e++) acc += gemv_value<T, In>(a[e]) * gemv_value<T, In>(b[e]);
        }
        for (long c = nv * VEC + lane; c < k; c += 64) acc += gemv_value<T, In>(m[c]) * gemv_value<T, In>(x[c]);
    } else {
        for (long c = lane; c < k; c += 64) acc += gemv_value<T, In>(m[c]) * gemv_value<T, In>(x[c * incx]);
    }
    acc = gemv_wave_sum(acc);
    if (lane == 0) {
        T* out = y + row * incy;
        *out = beta == (T) 0 ? alpha * acc : __builtin_fma(beta, *out, alpha * acc);
    }
}

// A few vectors at once (a small batch against a weight matrix whose rows are contiguous, y = x W^T):
// y[row * sy_row + v * sy_vec] = alpha * <M[row, :], X[v, :]> + beta * y[..] for v < nv <= NV. The matrix still
// moves once; a work-group stages the vectors through LDS, 256 lane-widths at a time, for all its rows.
// RW: matrix rows per wavefront
template <typename In, typename T, int VEC, int NV, int RW>
__device__ __forceinline__ void gemv_rows_multi(const In* __restrict__ M, long ld, const In* __restrict__ X, long ldx, int nv, T* __restrict__ y,
                                                long sy_row, long sy_vec, long rows, long k, T alpha, T beta) {
    typedef In V __attribute__((ext_vector_type(VEC)));
    constexpr int STEP = 4, SPAN = STEP * 64;      // lane-widths of every vector in LDS at a time
    __shared__ V xs[NV][SPAN];
    const int lane = threadIdx.x & 63;
    const long row0 = ((long) blockIdx.x * 4 + (threadIdx.x >> 6)) * RW;
    const In* m[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) m[r] = M + (row0 + r < rows ? row0 + r : rows - 1) * ld;   // rows past the end repeat the last one
    T acc[RW][NV];
#pragma unroll
    for (int r = 0; r < RW; r++)
#pragma unroll
        for (int v = 0; v < NV; v++) acc[r][v] = (T) 0;
    const long nvec = k / VEC;
    for (long c0 = 0; c0 < nvec; c0 += SPAN) {
        __syncthreads();
        for (int i = threadIdx.x; i < NV * SPAN; i += 256) {
            const int v = i / SPAN, j = i % SPAN;
            V piece = {};
            if (v < nv && c0 + j < nvec) piece = reinterpret_cast<const V*>(X + v * ldx)[c0 + j];
            xs[v][j] = piece;
        }
        __syncthreads();
#pragma unroll
        for (int st = 0; st < STEP; st++) {
            const long c = c0 + st * 64 + lane;
            if (c0 + st * 64 < nvec) {                      // uniform over the wavefront
                const long cc = c < nvec ? c : nvec - 1;
                V a[RW];
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    a[r] = __builtin_nontemporal_load(reinterpret_cast<const V*>(m[r]) + cc);
                    if (c >= nvec) a[r] = V{};              // past the end: zero times the zero in LDS
                }
#pragma unroll
                for (int v = 0; v < NV; v++) {
                    const V b = xs[v][st * 64 + lane];
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        const T bv = gemv_value<T, In>(b[e]);
#pragma unroll
                        for (int r = 0; r < RW; r++) acc[r][v] += gemv_value<T, In>(a[r][e]) * bv;
                    }
                }
            }
        }
    }
    for (long c = nvec * VEC + lane; c < k; c += 64) {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            if (v < nv) {
                const T bv = gemv_value<T, In>(X[v * ldx + c]);
#pragma unroll
                for (int r = 0; r < RW; r++) acc[r][v] += gemv_value<T, In>(m[r][c]) * bv;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RW; r++) {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            if (v < nv) {
                const T sum = gemv_wave_sum(acc[r][v]);
                if (lane == 0 && row0 + r < rows) {
                    T* out = y + (row0 + r) * sy_row + v * sy_vec;
                    *out = beta == (T) 0 ? alpha * sum : __builtin_fma(beta, *out, alpha * sum);
                }
            }
        }
    }
}

// partial sums of rows [slice * chunk, ...) for VEC columns per lane; P[slice][col]
template <typename In, typename T, int VEC>
__device__ __forceinline__ void gemv_cols_partial(void* partials, const In* __restrict__ M, long ld, const In* __restrict__ x, long incx, long rows, long cols,
                                                  long chunk) {
    typedef In V __attribute__((ext_vector_type(VEC)));
    T* P = reinterpret_cast<T*>(partials);
    const long col = ((long) blockIdx.x * 256 + threadIdx.x) * VEC;
    if (col >= cols) return;
    const long r0 = (long) blockIdx.y * chunk;
    const long r1 = r0 + chunk < rows ? r0 + chunk : rows;
    constexpr int CH = DOCC_GEMV_COL_CHAINS;   // independent chains: that many rows' loads in flight per lane (4 and 8 are slower)
    T acc[CH][VEC];
#pragma unroll
    for (int u = 0; u < CH; u++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[u][e] = (T) 0;
    long r = r0;
    if (VEC > 1) {
        for (; r + CH <= r1; r += CH) {
            V a[CH];
            T w[CH];
#pragma unroll
            for (int u = 0; u < CH; u++) {
                a[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(M + (r + u) * ld + col));
                w[u] = gemv_value<T, In>(x[(r + u) * incx]);
            }
#pragma unroll
            for (int u = 0; u < CH; u++)
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[u][e] += w[u] * gemv_value<T, In>(a[u][e]);
        }
    }
    for (; r < r1; r++) {
        const T w = gemv_value<T, In>(x[r * incx]);
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[0][e] += w * gemv_value<T, In>(M[r * ld + col + e]);
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        T sum = acc[0][e];
#pragma unroll
        for (int u = 1; u < CH; u++) sum += acc[u][e];
        P[(long) blockIdx.y * cols + col + e] = sum;
    }
}

// The columns form for a few vectors at once (a small batch times a weight matrix stored [k][n], y = x W):
// P[slice][v][col] = sum over the slice's rows p of X[v * sx_v + p * sx_p] * M[p, col]; the matrix moves once.
template <typename In, typename T, int VEC, int NV>
__device__ __forceinline__ void gemv_cols_partial_multi(void* partials, const In* __restrict__ M, long ld, const In* __restrict__ X, long sx_v, long sx_p, int nv,
                                                        long rows, long cols, long chunk) {
    typedef In V __attribute__((ext_vector_type(VEC)));
    constexpr int STEP = 64;            // rows of the slice whose vector entries sit in LDS at a time
    __shared__ T xs[STEP][NV];
    T* P = reinterpret_cast<T*>(partials);
    const long col = ((long) blockIdx.x * 256 + threadIdx.x) * VEC;
    const bool live = col < cols;
    const long r0 = (long) blockIdx.y * chunk;
    const long r1 = r0 + chunk < rows ? r0 + chunk : rows;
    T acc[NV][VEC];
#pragma unroll
    for (int v = 0; v < NV; v++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[v][e] = (T) 0;
    for (long base = r0; base < r1; base += STEP) {
        const int cnt = r1 - base < STEP ? (int) (r1 - base) : STEP;
        __syncthreads();
        for (int i = threadIdx.x; i < STEP * NV; i += 256) {
            const int r = i / NV, v = i % NV;
            xs[r][v] = (r < cnt && v < nv) ? gemv_value<T, In>(X[v * sx_v + (base + r) * sx_p]) : (T) 0;
        }
        __syncthreads();
        if (!live) continue;
#pragma unroll 4
        for (int r = 0; r < cnt; r++) {
            T a[VEC];
            if (VEC > 1) {
                const V av = __builtin_nontemporal_load(reinterpret_cast<const V*>(M + (base + r) * ld + col));
#pragma unroll
                for (int e = 0; e < VEC; e++) a[e] = gemv_value<T, In>(av[e]);
            } else {
                a[0] = gemv_value<T, In>(M[(base + r) * ld + col]);
            }
#pragma unroll
            for (int v = 0; v < NV; v++) {
                const T w = xs[r][v];
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[v][e] += w * a[e];
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int v = 0; v < NV; v++)
        if (v < nv)
#pragma unroll
            for (int e = 0; e < VEC; e++) P[((long) blockIdx.y * nv + v) * cols + col + e] = acc[v][e];
}

// y[v * sy_vec + col * sy_col] = alpha * (sum over the slices of P[s][v][col]) + beta * y[..]; entries = nv * cols
template <typename T>
__device__ __forceinline__ void gemv_cols_final_multi(const void* partials, T* __restrict__ y, long sy_vec, long sy_col, long cols, long entries, int slices, T alpha,
                                                      T beta) {
    // 64 neighbouring entries per work-group (256-byte segments of every slice), the slices dealt to its four waves
    __shared__ T part[4][64];
    const T* P = reinterpret_cast<const T*>(partials);
    const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
    const long e = (long) blockIdx.x * 64 + c;
    T acc = (T) 0;
    if (e < entries) {
#pragma unroll 4
        for (long s = g; s < slices; s += 4) acc += P[s * entries + e];
    }
    part[g][c] = acc;
    __syncthreads();
    if (g == 0 && e < entries) {
        const T r = (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
        T* out = y + (e / cols) * sy_vec + (e % cols) * sy_col;
        *out = beta == (T) 0 ? alpha * r : __builtin_fma(beta, *out, alpha * r);
    }
}

template <typename T>
__device__ __forceinline__ void gemv_cols_final(const void* partials, T* __restrict__ y, long incy, long cols, int slices, T alpha, T beta) {
    // a work-group takes 16 neighbouring columns; 16 lanes per column each add every 16th slice, then one lane
    // adds the 16 sums in order: the order of the additions is fixed by the launch geometry alone
    __shared__ T part[16][17];
    const T* P = reinterpret_cast<const T*>(partials);
    const int c = threadIdx.x & 15, g = threadIdx.x >> 4;
    const long col = (long) blockIdx.x * 16 + c;
    T acc = (T) 0;
    if (col < cols) {
        // eight loads in flight, added in slice order
        long s = g;
        for (; s + 7 * 16 < slices; s += 8 * 16) {
            T v[8];
#pragma unroll
            for (int k = 0; k < 8; k++) v[k] = P[(s + 16 * k) * cols + col];
#pragma unroll
            for (int k = 0; k < 8; k++) acc += v[k];
        }
        for (; s < slices; s += 16) acc += P[s * cols + col];
    }
    part[g][c] = acc;
    __syncthreads();
    if (g == 0 && col < cols) {
        T r = part[0][c];
#pragma unroll
        for (int i = 1; i < 16; i++) r += part[i][c];
        T* out = y + col * incy;
        *out = beta == (T) 0 ? alpha * r : __builtin_fma(beta, *out, alpha * r);
    }
}

} // namespace docc_k

#define DOCC_GEMV(NAME, In, T, VEC)                                                                                                   \
    extern "C" __global__ __launch_bounds__(256) void docc_gemv_rows_##NAME##_v##VEC(const In* M, long ld, const In* x, long incx, T* y, \
                                                                                     long incy, long rows, long k, T alpha, T beta) { \
        docc_k::gemv_rows<In, T, VEC>(M, ld, x, incx, y, incy, rows, k, alpha, beta);                                                  \
    }                                                                                                                                 \
    extern "C" __global__ __launch_bounds__(256) void docc_gemv_colp_##NAME##_v##VEC(void* partials, const In* M, long ld, const In* x, \
                                                                                     long incx, long rows, long cols, long chunk) {   \
        docc_k::gemv_cols_partial<In, T, VEC>(partials, M, ld, x, incx, rows, cols, chunk);                                            \
    }
#define DOCC_GEMV_MULTI(NAME, In, T, VEC, NV)                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_gemv_rowsm_##NAME##_v##VEC##_n##NV(                                          \
        const In* M, long ld, const In* X, long ldx, int nv, T* y, long sy_row, long sy_vec, long rows, long k, T alpha, T beta) {     \
        docc_k::gemv_rows_multi<In, T, VEC, NV, 4>(M, ld, X, ldx, nv, y, sy_row, sy_vec, rows, k, alpha, beta);                         \
    }
// eight rows per wavefront: half the vector traffic, for matrices with enough rows to still fill the chip
#define DOCC_GEMV_MULTI_R8(NAME, In, T, VEC, NV)                                                                                       \
    extern "C" __global__ __launch_bounds__(256) void docc_gemv_rowsm_##NAME##_v##VEC##_n##NV##_r8(                                     \
        const In* M, long ld, const In* X, long ldx, int nv, T* y, long sy_row, long sy_vec, long rows, long k, T alpha, T beta) {     \
        docc_k::gemv_rows_multi<In, T, VEC, NV, 8>(M, ld, X, ldx, nv, y, sy_row, sy_vec, rows, k, alpha, beta);                         \
    }
// the columns form of the same; fp32 and fp64 only (for bf16 the MFMA tiles are as fast)
#define DOCC_GEMV_MULTI_COLS(NAME, In, T, VEC, NV)                                                                                     \
    extern "C" __global__ __launch_bounds__(256) void docc_gemv_colpm_##NAME##_v##VEC##_n##NV(                                          \
        void* partials, const In* M, long ld, const In* X, long sx_v, long sx_p, int nv, long rows, long cols, long chunk) {          \
        docc_k::gemv_cols_partial_multi<In, T, VEC, NV>(partials, M, ld, X, sx_v, sx_p, nv, rows, cols, chunk);                        \
    }
#define DOCC_GEMV_MULTI_ALL(NAME, In, T, VEC) \
    DOCC_GEMV_MULTI(NAME, In, T, VEC, 2) DOCC_GEMV_MULTI(NAME, In, T, VEC, 4) DOCC_GEMV_MULTI(NAME, In, T, VEC, 8)
#define DOCC_GEMV_MULTI_COLS_ALL(NAME, In, T, VEC) \
    DOCC_GEMV_MULTI_COLS(NAME, In, T, VEC, 2) DOCC_GEMV_MULTI_COLS(NAME, In, T, VEC, 4)
DOCC_GEMV_MULTI_ALL(f32, float, float, 4)
DOCC_GEMV_MULTI_ALL(f32, float, float, 1)
DOCC_GEMV_MULTI_ALL(f64, double, double, 2)
DOCC_GEMV_MULTI_ALL(f64, double, double, 1)
DOCC_GEMV_MULTI_R8(f32, float, float, 4, 2)
DOCC_GEMV_MULTI_R8(f32, float, float, 4, 4)
DOCC_GEMV_MULTI_R8(f64, double, double, 2, 2)
DOCC_GEMV_MULTI_R8(f64, double, double, 2, 4)
DOCC_GEMV_MULTI_COLS_ALL(f32, float, float, 4)
DOCC_GEMV_MULTI_COLS_ALL(f32, float, float, 1)
DOCC_GEMV_MULTI_COLS_ALL(f64, double, double, 2)
DOCC_GEMV_MULTI_COLS_ALL(f64, double, double, 1)
DOCC_GEMV_MULTI_ALL(bf16, unsigned short, float, 8)
DOCC_GEMV_MULTI_ALL(bf16, unsigned short, float, 1)

DOCC_GEMV(f32, float, float, 4)
DOCC_GEMV(f32, float, float, 1)
DOCC_GEMV(f64, double, double, 2)
DOCC_GEMV(f64, double, double, 1)
DOCC_GEMV(bf16, unsigned short, float, 8)
DOCC_GEMV(bf16, unsigned short, float, 1)

extern "C" __global__ __launch_bounds__(256) void docc_gemv_colf_f32(const void* partials, float* y, long incy, long cols, int slices, float alpha,
                                                                     float beta) {
    docc_k::gemv_cols_final<float>(partials, y, incy, cols, slices, alpha, beta);
}
extern "C" __global__ __launch_bounds__(256) void docc_gemv_colf_f64(const void* partials, double* y, long incy, long cols, int slices, double alpha,
                                                                     double beta) {
    docc_k::gemv_cols_final<double>(partials, y, incy, cols, slices, alpha, beta);
}
extern "C" __global__ __launch_bounds__(256) void docc_gemv_colfm_f32(const void* partials, float* y, long sy_vec, long sy_col, long cols, long entries,
                                                                      int slices, float alpha, float beta) {
    docc_k::gemv_cols_final_multi<float>(partials, y, sy_vec, sy_col, cols, entries, slices, alpha, beta);
}
extern "C" __global__ __launch_bounds__(256) void docc_gemv_colfm_f64(const void* partials, double* y, long sy_vec, long sy_col, long cols, long entries,
                                                                      int slices, double alpha, double beta) {
    docc_k::gemv_cols_final_multi<double>(partials, y, sy_vec, sy_col, cols, entries, slices, alpha, beta);
}
