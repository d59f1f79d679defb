// Softmax for gfx950: the fp32 row kernels (reduction over the last axis) and, below them, the
// general forms: fp64, and a reduction over inner axes ([outer, reduce, inner] view).
//
// Replaces the seven loop nests SoftmaxNode::expand produces (reference
// sdfg/src/data_flow/library_nodes/math/tensor/reduce_ops/softmax_node.cpp:142-252:
// Max -> Broadcast -> Sub -> Exp -> Sum -> Broadcast -> Div with six
// temporaries) by one kernel that reads X once and writes Y once.
//
// HBM-bound: algorithmic traffic is 8 bytes per element (16 in fp64). The shapes of the row kernels (one template over
// the element type; the figures are those of fp32, whose 16-byte vector holds four columns - fp64 halves the widths):
//   rows sharing a wavefront (cols <= 128, cols % 4 == 0): 1 to 32 lanes a row, 64 to 2 rows per
//       wavefront and four such sets per wavefront, butterflies inside the lanes of a row;
//   wave-per-row  (cols <= 1024, cols % 4 == 0; built up to 4096): a 64-lane wavefront
//       holds the whole row in registers (NV float4 per lane, 128-bit coalesced loads),
//       reduces max and sum with wave shuffles only - no LDS, no barrier;
//   block-per-row (cols <= 16384, cols % 4 == 0): 256 threads hold the row,
//       partial results cross the four waves through LDS; ahead of the wavefront
//       per row from 2048 columns on (more rows in flight per register); rows of
//       2049..4096 columns use 512 threads (two vectors per lane), the others 256;
//       rows of up to 65536 columns 1024 threads, where there are rows enough for half the CUs;
//   block-per-row for rows that start off a 16-byte boundary (any cols from 256 on): single
//       elements up to the first boundary and after the last, vectors between;
//   rows cut into slices (longer rows, or too few of them): two launches around one
//       (maximum, sum) pair per slice, the second reading the slice again (12 bytes per element);
//   streaming     (what is left: operands placed unequally, short ragged rows): per-lane
//       online max/sum over the row, then a second read to write the result.
#include "common.h"

using namespace docc_k;

namespace {

constexpr float kNegInf = -__builtin_huge_valf();

// element type of a row kernel: its 16-byte vector, the exponential of a non-positive argument, the maximum that drops NaNs
template <typename T> struct SoftmaxMath;
template <> struct SoftmaxMath<float> {
    static __device__ __forceinline__ float neg_inf() { return kNegInf; }
    static __device__ __forceinline__ float exp_le0(float t) { return exp_neg(t); }
    static __device__ __forceinline__ float max(float a, float b) { return fmaxf(a, b); }
};
template <> struct SoftmaxMath<double> {
    static __device__ __forceinline__ double neg_inf() { return -__builtin_huge_val(); }
    static __device__ __forceinline__ double exp_le0(double t) { return exp(t); }
    static __device__ __forceinline__ double max(double a, double b) { return fmax(a, b); }
};
template <typename T> struct RowVec;
template <> struct RowVec<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };
template <> struct RowVec<double> { typedef double type __attribute__((ext_vector_type(2))); static constexpr int N = 2; };

template <typename T> __device__ __forceinline__ typename RowVec<T>::type all_neg_inf() {
    typename RowVec<T>::type v;
#pragma unroll
    for (int e = 0; e < RowVec<T>::N; e++) v[e] = SoftmaxMath<T>::neg_inf();
    return v;
}
template <typename T> __device__ __forceinline__ T vec_max(typename RowVec<T>::type v) {
    T m = v[0];
#pragma unroll
    for (int e = 1; e < RowVec<T>::N; e++) m = SoftmaxMath<T>::max(m, v[e]);
    return m;
}
// v = exp(v - m) in place; returns the sum of the results, added in pairs
template <typename T> __device__ __forceinline__ T vec_exp(typename RowVec<T>::type& v, T m) {
#pragma unroll
    for (int e = 0; e < RowVec<T>::N; e++) v[e] = SoftmaxMath<T>::exp_le0(v[e] - m);
    if constexpr (RowVec<T>::N == 4) return (v[0] + v[1]) + (v[2] + v[3]);
    else return v[0] + v[1];
}

template <typename T, int NV>
__device__ __forceinline__ void softmax_row_wave(const T* __restrict__ x, T* __restrict__ y, int cols, int lane) {
    using V = typename RowVec<T>::type;
    const int nvec = cols / RowVec<T>::N;
    const V* xv = reinterpret_cast<const V*>(x);
    V* yv = reinterpret_cast<V*>(y);
    V v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = lane + i * kWave;
        if (c < nvec) {
            v[i] = __builtin_nontemporal_load(xv + c);
        } else {
            v[i] = all_neg_inf<T>();
        }
    }
    T m = SoftmaxMath<T>::neg_inf();
#pragma unroll
    for (int i = 0; i < NV; i++) m = SoftmaxMath<T>::max(vec_max<T>(v[i]), m);
    m = wave_max(m);
    T s = (T) 0;
#pragma unroll
    for (int i = 0; i < NV; i++) s += vec_exp<T>(v[i], m);
    s = wave_sum(s);
    // one IEEE division per row, then multiplies: within 1 ulp of the
    // element-wise division the reference's Div node performs
    const T inv = (T) 1 / s;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = lane + i * kWave;
        if (c < nvec) {
            V o = v[i] * inv;
            __builtin_nontemporal_store(o, yv + c);
        }
    }
}

template <typename T, int NV>
__device__ __forceinline__ void softmax_wave_kernel(const T* X, T* Y, long rows, int cols) {
    const int lane = threadIdx.x & (kWave - 1);
    const long row = (long) blockIdx.x * (256 / kWave) + (threadIdx.x / kWave);   // launched with 256 lanes; blockDim.x would be a load to wait for
    if (row >= rows) return;
    softmax_row_wave<T, NV>(X + row * (long) cols, Y + row * (long) cols, cols, lane);
}

// block reductions across the NW waves of a work-group
template <int NW = 4, typename T>
__device__ __forceinline__ T block_max(T v, T* lds) {
    v = wave_max(v);
    const int w = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds[w] = v;
    __syncthreads();
    T r = lds[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r = SoftmaxMath<T>::max(r, lds[i]);
    __syncthreads();
    return r;
}

template <int NW = 4, typename T>
__device__ __forceinline__ T block_sum(T v, T* lds) {
    v = wave_sum(v);
    const int w = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds[w] = v;
    __syncthreads();
    T r = lds[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r += lds[i];
    __syncthreads();
    return r;
}

template <typename T, int NV, int NW = 4>
__device__ __forceinline__ void softmax_block_kernel(const T* X, T* Y, long rows, int cols) {
    using V = typename RowVec<T>::type;
    constexpr int NT = NW * kWave;
    __shared__ T lds[NW];
    const long row = blockIdx.x;
    const int nvec = cols / RowVec<T>::N;
    const V* xv = reinterpret_cast<const V*>(X + row * (long) cols);
    V* yv = reinterpret_cast<V*>(Y + row * (long) cols);
    V v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = threadIdx.x + i * NT;
        if (c < nvec) {
            v[i] = __builtin_nontemporal_load(xv + c);
        } else {
            v[i] = all_neg_inf<T>();
        }
    }
    T m = SoftmaxMath<T>::neg_inf();
#pragma unroll
    for (int i = 0; i < NV; i++) m = SoftmaxMath<T>::max(vec_max<T>(v[i]), m);
    m = block_max<NW>(m, lds);
    T s = (T) 0;
#pragma unroll
    for (int i = 0; i < NV; i++) s += vec_exp<T>(v[i], m);
    s = block_sum<NW>(s, lds);
    const T inv = (T) 1 / s;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = threadIdx.x + i * NT;
        if (c < nvec) {
            V o = v[i] * inv;
            __builtin_nontemporal_store(o, yv + c);
        }
    }
}

// The work-group per row for rows that do not start on a 16-byte boundary (cols not a multiple of the vector, or operands
// placed off it): single elements up to the first boundary, the vectors between the first and the last boundary, single
// elements after it; a lane holds NV vectors of the middle part and at most one of the single elements. X and Y must be
// placed equally relative to 16 bytes, so that a row's boundaries are the same in both.
template <typename T, int NV, int NW>
__device__ __forceinline__ void softmax_block_any_kernel(const T* X, T* Y, long rows, int cols) {
    using V = typename RowVec<T>::type;
    using M = SoftmaxMath<T>;
    constexpr int N = RowVec<T>::N;
    constexpr int NT = NW * kWave;
    __shared__ T lds[NW];
    const long row = blockIdx.x;
    const T* x = X + row * (long) cols;
    T* y = Y + row * (long) cols;
    const int mis = (int) ((reinterpret_cast<uintptr_t>(x) / sizeof(T)) & (N - 1));
    int head = mis ? N - mis : 0;
    if (head > cols) head = cols;
    const int nvec = (cols - head) / N;
    const int tail0 = head + nvec * N;
    const int t = threadIdx.x;
    const int edge = t < head ? t : (t - head < cols - tail0 ? tail0 + t - head : -1);   // this lane's single element, if any
    T e = edge >= 0 ? x[edge] : M::neg_inf();
    const V* xv = reinterpret_cast<const V*>(x + head);
    V* yv = reinterpret_cast<V*>(y + head);
    V v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = t + i * NT;
        if (c < nvec) {
            v[i] = __builtin_nontemporal_load(xv + c);
        } else {
            v[i] = all_neg_inf<T>();
        }
    }
    T m = e;
#pragma unroll
    for (int i = 0; i < NV; i++) m = M::max(vec_max<T>(v[i]), m);
    m = block_max<NW>(m, lds);
    e = M::exp_le0(e - m);
    T s = edge >= 0 ? e : (T) 0;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const T part = vec_exp<T>(v[i], m);
        if (t + i * NT < nvec) s += part;   // a vector past the row's end is NaN when the whole row is -inf
    }
    s = block_sum<NW>(s, lds);
    const T inv = (T) 1 / s;
    if (edge >= 0) y[edge] = e * inv;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = t + i * NT;
        if (c < nvec) {
            V o = v[i] * inv;
            __builtin_nontemporal_store(o, yv + c);
        }
    }
}

// Rows of at most 32 vectors: LPR lanes of a wavefront share a row (one vector each), so a wavefront holds 64 / LPR rows
// at a time and four such sets in turn, all loaded before the first is reduced; the reductions are butterflies inside
// the LPR lanes. A wavefront per row would leave half to all but one of its lanes idle.
template <typename T, int LPR>
__device__ __forceinline__ void softmax_subwave_kernel(const T* X, T* Y, long rows, int cols) {
    using V = typename RowVec<T>::type;
    using M = SoftmaxMath<T>;
    constexpr int RPW = kWave / LPR;   // rows of a wavefront per set
    constexpr int SETS = 4;
    const int lane = threadIdx.x & (kWave - 1);
    const int l = lane % LPR, g = lane / LPR;
    const int nvec = cols / RowVec<T>::N;
    const long first = ((long) blockIdx.x * (256 / kWave) + threadIdx.x / kWave) * (RPW * SETS) + g;
    const V* xv = reinterpret_cast<const V*>(X);
    V* yv = reinterpret_cast<V*>(Y);
    V v[SETS];
    bool live[SETS];
#pragma unroll
    for (int i = 0; i < SETS; i++) {
        const long row = first + (long) i * RPW;
        live[i] = row < rows && l < nvec;
        v[i] = live[i] ? __builtin_nontemporal_load(xv + row * nvec + l) : all_neg_inf<T>();
    }
#pragma unroll
    for (int i = 0; i < SETS; i++) {
        T m = vec_max<T>(v[i]);
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) m = M::max(m, __shfl_xor(m, o));
        T s = vec_exp<T>(v[i], m);
        if (!(l < nvec)) s = (T) 0;   // a lane past the row's end holds -inf, which is NaN after the subtraction when the whole row is -inf
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
        const T inv = (T) 1 / s;
        if (live[i]) {
            V out = v[i] * inv;
            __builtin_nontemporal_store(out, yv + (first + (long) i * RPW) * nvec + l);
        }
    }
}

} // namespace

// T = float: docc_softmax_f32_<form>; T = double: docc_softmax_f64_<form>. A lane holds NV 16-byte vectors of its row.
#define DOCC_SOFTMAX_ROW_FORMS(T, SFX)                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_wave_v1(const T* X, T* Y, long rows, int cols) { softmax_wave_kernel<T, 1>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_wave_v2(const T* X, T* Y, long rows, int cols) { softmax_wave_kernel<T, 2>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_wave_v4(const T* X, T* Y, long rows, int cols) { softmax_wave_kernel<T, 4>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_wave_v8(const T* X, T* Y, long rows, int cols) { softmax_wave_kernel<T, 8>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_wave_v16(const T* X, T* Y, long rows, int cols) { softmax_wave_kernel<T, 16>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_block_v1(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 1>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_block_v2(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 2>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_block_v4(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 4>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_block_v8(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 8>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_block_v16(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 16>(X, Y, rows, cols); } \
    /* eight wavefronts per row */                                                                                                  \
    extern "C" __global__ __launch_bounds__(512) void docc_softmax_##SFX##_block8_v2(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 2, 8>(X, Y, rows, cols); } \
    /* sixteen wavefronts per row: long rows stay in registers (one read, one write), for tensors with rows enough to give every CU one */ \
    extern "C" __global__ __launch_bounds__(1024) void docc_softmax_##SFX##_block16_v8(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 8, 16>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(1024) void docc_softmax_##SFX##_block16_v16(const T* X, T* Y, long rows, int cols) { softmax_block_kernel<T, 16, 16>(X, Y, rows, cols); } \
    /* rows that start off a 16-byte boundary */                                                                                    \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_any4_v1(const T* X, T* Y, long rows, int cols) { softmax_block_any_kernel<T, 1, 4>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_any4_v4(const T* X, T* Y, long rows, int cols) { softmax_block_any_kernel<T, 4, 4>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_any4_v16(const T* X, T* Y, long rows, int cols) { softmax_block_any_kernel<T, 16, 4>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(1024) void docc_softmax_##SFX##_any16_v8(const T* X, T* Y, long rows, int cols) { softmax_block_any_kernel<T, 8, 16>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(1024) void docc_softmax_##SFX##_any16_v16(const T* X, T* Y, long rows, int cols) { softmax_block_any_kernel<T, 16, 16>(X, Y, rows, cols); } \
    /* several rows per wavefront: 1 .. 32 lanes a row */                                                                           \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_sub1(const T* X, T* Y, long rows, int cols) { softmax_subwave_kernel<T, 1>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_sub2(const T* X, T* Y, long rows, int cols) { softmax_subwave_kernel<T, 2>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_sub4(const T* X, T* Y, long rows, int cols) { softmax_subwave_kernel<T, 4>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_sub8(const T* X, T* Y, long rows, int cols) { softmax_subwave_kernel<T, 8>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_sub16(const T* X, T* Y, long rows, int cols) { softmax_subwave_kernel<T, 16>(X, Y, rows, cols); } \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SFX##_sub32(const T* X, T* Y, long rows, int cols) { softmax_subwave_kernel<T, 32>(X, Y, rows, cols); }
DOCC_SOFTMAX_ROW_FORMS(float, f32)
DOCC_SOFTMAX_ROW_FORMS(double, f64)

// Any cols, any alignment: one 256-thread block per row. Pass 1 keeps a
// per-thread running (max, sum) pair that is rescaled whenever the max moves
// (online softmax); the pairs are merged across the block; pass 2 re-reads the
// row and writes exp(x - max) / sum.
extern "C" __global__ __launch_bounds__(256) void docc_softmax_f32_stream(const float* X, float* Y, long rows,
                                                                            long cols) {
    __shared__ float lds[4];
    const long row = blockIdx.x;
    const float* x = X + row * cols;
    float* y = Y + row * cols;
    float m = kNegInf, s = 0.f;
    for (long c = threadIdx.x; c < cols; c += 256) {
        float v = x[c];
        if (v > m) {
            s = s * exp_neg(m - v) + 1.0f; // m == -inf: s is 0 and exp(-inf) is 0
            m = v;
        } else if (v != kNegInf) {   // -inf weighs nothing (and -inf - -inf must not reach the exponential); NaN poisons s
            s += exp_neg(v - m);
        }
    }
    float gm = block_max(m, lds);
    // a thread that saw no element has m = -inf, s = 0: contributes 0 (a NaN sum counts even then)
    float contrib = (m == kNegInf && s == s) ? 0.f : s * exp_neg(m - gm);
    float gs = block_sum(contrib, lds);
    gs += gm - gm;   // an infinite maximum makes every result NaN, as inf - inf does in the node's Sub step
    const float inv = 1.0f / gs;
    for (long c = threadIdx.x; c < cols; c += 256) y[c] = exp_neg(x[c] - gm) * inv;
}

// ------------------------------------------------------------------------------------------
// General forms: the reference's node reduces over any set of axes and takes its element type
// from its memlets (softmax_node.cpp:38-110). A block of adjacent axes is the middle extent of an
// [outer, reduce, inner] view of the contiguous input.

namespace {


// running (maximum, sum of exp(x - maximum)) of the elements seen so far; (-inf, 0) for none
template <typename T>
__device__ __forceinline__ void online_step(T v, T& m, T& s) {
    using M = SoftmaxMath<T>;
    if (v > m) {
        s = s * M::exp_le0(m - v) + (T) 1;   // m == -inf: s is 0 and exp(-inf) is 0
        m = v;
    } else if (v != M::neg_inf()) {   // -inf weighs nothing (and -inf - -inf must not reach the exponential); NaN poisons s
        s += M::exp_le0(v - m);
    }
}

// what a (maximum m, sum s) pair adds to a sum taken relative to g >= m: nothing when no element was seen
// (m = -inf, s = 0), but a NaN sum counts even then (a NaN element does not move the maximum)
template <typename T>
__device__ __forceinline__ T pair_weight(T m, T s, T g) {
    using M = SoftmaxMath<T>;
    return (m == M::neg_inf() && s == s) ? (T) 0 : s * M::exp_le0(m - g);
}

// merges the pairs of the NP threads that share a column; lm / ls hold one pair per thread
template <typename T>
__device__ __forceinline__ void merge_pairs(const T* lm, const T* ls, int first, int step, int count, T& gm, T& gs) {
    using M = SoftmaxMath<T>;
    gm = M::neg_inf();
    for (int i = 0; i < count; i++) gm = M::max(gm, lm[first + i * step]);
    gs = (T) 0;
    for (int i = 0; i < count; i++) gs += pair_weight(lm[first + i * step], ls[first + i * step], gm);
    gs += gm - gm;   // an infinite maximum makes every result NaN, as inf - inf does in the node's Sub step
}

// what a result is multiplied or divided by: fp32 divides once per row and multiplies, fp64 divides every element
template <typename T> __device__ __forceinline__ T softmax_scale(T gs);
template <> __device__ __forceinline__ float softmax_scale<float>(float gs) { return 1.0f / gs; }   // one division per row, then multiplies
template <> __device__ __forceinline__ double softmax_scale<double>(double gs) { return gs; }
__device__ __forceinline__ float softmax_result(float e, float scale) { return e * scale; }
__device__ __forceinline__ double softmax_result(double e, double scale) { return e / scale; }

// inner == 1, any type: one 256-thread block per row, two reads of the row.
template <typename T>
__device__ __forceinline__ void softmax_row_stream(const T* X, T* Y, long cols) {
    using M = SoftmaxMath<T>;
    __shared__ T lm[256];
    __shared__ T ls[256];
    const long row = blockIdx.x;
    const T* x = X + row * cols;
    T* y = Y + row * cols;
    T m = M::neg_inf(), s = (T) 0;
    for (long c = threadIdx.x; c < cols; c += 256) online_step(x[c], m, s);
    lm[threadIdx.x] = m;
    ls[threadIdx.x] = s;
    __syncthreads();
    // tree over the 256 pairs
    for (int half = 128; half > 0; half >>= 1) {
        if ((int) threadIdx.x < half) {
            const T m2 = lm[threadIdx.x + half], s2 = ls[threadIdx.x + half];
            const T m1 = lm[threadIdx.x], s1 = ls[threadIdx.x];
            const T g = M::max(m1, m2);
            lm[threadIdx.x] = g;
            ls[threadIdx.x] = pair_weight(m1, s1, g) + pair_weight(m2, s2, g);
        }
        __syncthreads();
    }
    const T gm = lm[0];
    const T gs = ls[0] + (gm - gm);   // an infinite maximum makes every result NaN, as inf - inf does in the node's Sub step
    for (long c = threadIdx.x; c < cols; c += 256) y[c] = M::exp_le0(x[c] - gm) / gs;
}

// inner > 1: a block owns 64 adjacent inner positions of one outer index (lane = inner position, so
// that every access of a wave is one contiguous segment) and its four waves split the reduced extent.
template <typename T>
__device__ __forceinline__ void softmax_strided_tile(const T* X, T* Y, long reduce, long inner, long tiles) {
    using M = SoftmaxMath<T>;
    __shared__ T lm[256];
    __shared__ T ls[256];
    const long o = blockIdx.x / tiles;
    const long col = (blockIdx.x % tiles) * 64 + (threadIdx.x & 63);
    const int part = threadIdx.x >> 6;
    const bool live = col < inner;
    const T* x = X + o * reduce * inner + col;
    T* y = Y + o * reduce * inner + col;
    T m = M::neg_inf(), s = (T) 0;
    if (live)
        for (long r = part; r < reduce; r += 4) online_step(x[r * inner], m, s);
    lm[threadIdx.x] = m;
    ls[threadIdx.x] = s;
    __syncthreads();
    T gm, gs;
    merge_pairs(lm, ls, (int) (threadIdx.x & 63), 64, 4, gm, gs);
    if (live)
        for (long r = part; r < reduce; r += 4) y[r * inner] = M::exp_le0(x[r * inner] - gm) / gs;
}

// The same with 16-byte vectors (inner a multiple of the vector, operands 16-byte aligned): a lane owns the VN adjacent
// columns of one vector, 256 / PARTS lanes cover the block's columns and the PARTS groups of lanes split the reduced
// extent; four rows are loaded before the first is worked in. PARTS = 16 (256 bytes of a row per block) for long
// extents, 4 (1 KB of a row) for short ones.
template <typename T, int PARTS>
__device__ __forceinline__ void softmax_strided_tile_vec(const T* X, T* Y, long reduce, long inner, long tiles) {
    using M = SoftmaxMath<T>;
    using V = typename RowVec<T>::type;
    constexpr int VN = RowVec<T>::N;
    constexpr int LANES = 256 / PARTS;       // lanes (vectors of columns) across the block
    __shared__ T lm[VN][256];
    __shared__ T ls[VN][256];
    const long o = blockIdx.x / tiles;
    const int cl = threadIdx.x % LANES, part = threadIdx.x / LANES;
    const long col = ((blockIdx.x % tiles) * LANES + cl) * VN;
    const bool live = col < inner;
    const long nv = inner / VN;                                   // vectors per row
    const V* x = reinterpret_cast<const V*>(X + o * reduce * inner + col);
    V* y = reinterpret_cast<V*>(Y + o * reduce * inner + col);
    T m[VN], s[VN];
#pragma unroll
    for (int e = 0; e < VN; e++) m[e] = M::neg_inf(), s[e] = (T) 0;
    if (live) {
        long r = part;
        for (; r + 3 * PARTS < reduce; r += 4 * PARTS) {
            V v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = x[(r + PARTS * u) * nv];
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int e = 0; e < VN; e++) online_step(v[u][e], m[e], s[e]);
        }
        for (; r < reduce; r += PARTS) {
            const V v = x[r * nv];
#pragma unroll
            for (int e = 0; e < VN; e++) online_step(v[e], m[e], s[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < VN; e++) lm[e][threadIdx.x] = m[e], ls[e][threadIdx.x] = s[e];
    __syncthreads();
    T gm[VN], scale[VN];
#pragma unroll
    for (int e = 0; e < VN; e++) {
        T gs;
        merge_pairs(lm[e], ls[e], cl, LANES, PARTS, gm[e], gs);
        scale[e] = softmax_scale<T>(gs);
    }
    if (!live) return;
    long r = part;
    for (; r + 3 * PARTS < reduce; r += 4 * PARTS) {
        V v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = __builtin_nontemporal_load(x + (r + PARTS * u) * nv);
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int e = 0; e < VN; e++) v[u][e] = softmax_result(M::exp_le0(v[u][e] - gm[e]), scale[e]);
            __builtin_nontemporal_store(v[u], y + (r + PARTS * u) * nv);
        }
    }
    for (; r < reduce; r += PARTS) {
        V v = __builtin_nontemporal_load(x + r * nv);
#pragma unroll
        for (int e = 0; e < VN; e++) v[e] = softmax_result(M::exp_le0(v[e] - gm[e]), scale[e]);
        __builtin_nontemporal_store(v, y + r * nv);
    }
}

// inner a power of two up to 32: a block owns one outer index, whose [reduce, inner] slab is contiguous;
// thread t walks the slab with stride 256 and therefore stays in column t % inner.
template <typename T>
__device__ __forceinline__ void softmax_strided_slab(const T* X, T* Y, long reduce, int inner) {
    __shared__ T lm[256];
    __shared__ T ls[256];
    using M = SoftmaxMath<T>;
    const long n = reduce * inner;
    const T* x = X + (long) blockIdx.x * n;
    T* y = Y + (long) blockIdx.x * n;
    T m = M::neg_inf(), s = (T) 0;
    for (long i = threadIdx.x; i < n; i += 256) online_step(x[i], m, s);
    lm[threadIdx.x] = m;
    ls[threadIdx.x] = s;
    __syncthreads();
    T gm, gs;
    merge_pairs(lm, ls, (int) (threadIdx.x & (inner - 1)), inner, 256 / inner, gm, gs);
    for (long i = threadIdx.x; i < n; i += 256) y[i] = M::exp_le0(x[i] - gm) / gs;
}

// Few columns and a long reduced extent leave the tile kernel with a handful of work-groups that each walk
// the whole extent twice. The sliced pair spreads the rows as well: work-group (outer index, slice of rows,
// 64-column tile) first leaves its running (maximum, sum) pairs in a buffer of the launcher, then - in a second
// launch - every work-group merges the pairs of all slices of its columns and writes the results of its own
// slice. The pairs live in `partials`, device memory of the launcher: [outer][slice][column] x (maximum, sum).

struct SlicedWork {
    long o, col, r0, r1;   // outer index, this lane's column, rows [r0, r1) of the slice
    long slice;
    bool live;
};

__device__ __forceinline__ SlicedWork sliced_work(long reduce, long inner, long tiles, int slices) {
    SlicedWork w;
    long b = blockIdx.x;
    const long tile = b % tiles;
    b /= tiles;
    w.slice = b % slices;
    w.o = b / slices;
    w.col = tile * 64 + (threadIdx.x & 63);
    const long per = (reduce + slices - 1) / slices;
    w.r0 = w.slice * per;
    w.r1 = w.r0 + per < reduce ? w.r0 + per : reduce;
    w.live = w.col < inner;
    return w;
}

template <typename T>
__device__ __forceinline__ void softmax_sliced_partial(void* partials, const T* X, long reduce, long inner, long tiles, int slices) {
    using M = SoftmaxMath<T>;
    __shared__ T lm[256];
    __shared__ T ls[256];
    const SlicedWork w = sliced_work(reduce, inner, tiles, slices);
    const int part = threadIdx.x >> 6;
    const T* x = X + w.o * reduce * inner + w.col;
    T m = M::neg_inf(), s = (T) 0;
    if (w.live)
        for (long r = w.r0 + part; r < w.r1; r += 4) online_step(x[r * inner], m, s);
    lm[threadIdx.x] = m;
    ls[threadIdx.x] = s;
    __syncthreads();
    if (part == 0 && w.live) {
        // the pair of the slice, without the NaN marker for infinite maxima: that is applied once, at the end
        T gm = M::neg_inf();
        for (int i = 0; i < 4; i++) gm = M::max(gm, lm[(threadIdx.x & 63) + 64 * i]);
        T gs = (T) 0;
        for (int i = 0; i < 4; i++) gs += pair_weight(lm[(threadIdx.x & 63) + 64 * i], ls[(threadIdx.x & 63) + 64 * i], gm);
        T* P = reinterpret_cast<T*>(partials);
        const long at = ((w.o * slices + w.slice) * inner + w.col) * 2;
        P[at] = gm;
        P[at + 1] = gs;
    }
}

template <typename T>
__device__ __forceinline__ void softmax_sliced_finish(const void* partials, const T* X, T* Y, long reduce, long inner, long tiles, int slices) {
    using M = SoftmaxMath<T>;
    __shared__ T lm[256];
    __shared__ T ls[256];
    const SlicedWork w = sliced_work(reduce, inner, tiles, slices);
    const int part = threadIdx.x >> 6;
    const T* P = reinterpret_cast<const T*>(partials);
    // the four waves share the slices of this column
    T m = M::neg_inf(), s = (T) 0;
    if (w.live)
        for (int sl = part; sl < slices; sl += 4) {
            const long at = ((w.o * slices + sl) * inner + w.col) * 2;
            const T pm = P[at], ps = P[at + 1];
            const T g = M::max(m, pm);
            s = pair_weight(m, s, g) + pair_weight(pm, ps, g);
            m = g;
        }
    lm[threadIdx.x] = m;
    ls[threadIdx.x] = s;
    __syncthreads();
    T gm, gs;
    merge_pairs(lm, ls, (int) (threadIdx.x & 63), 64, 4, gm, gs);
    if (!w.live) return;
    const T* x = X + w.o * reduce * inner + w.col;
    T* y = Y + w.o * reduce * inner + w.col;
    for (long r = w.r0 + part; r < w.r1; r += 4) y[r * inner] = M::exp_le0(x[r * inner] - gm) / gs;
}

// The sliced pair with 16-byte vectors (inner a multiple of the vector, operands 16-byte aligned): the layout of the
// vector tile kernel - a lane owns the VN columns of one vector, sixteen lanes across, sixteen row groups - over the
// rows of one slice. Same pairs in the same places of `partials` as the scalar pair.
template <typename T>
struct SlicedVecWork {
    long o, slice, col, r0, r1;
    int cl, part;
    bool live;
    __device__ __forceinline__ SlicedVecWork(long reduce, long inner, long vtiles, int slices) {
        long b = blockIdx.x;
        const long tile = b % vtiles;
        b /= vtiles;
        slice = b % slices;
        o = b / slices;
        cl = threadIdx.x & 15;
        part = threadIdx.x >> 4;
        col = (tile * 16 + cl) * RowVec<T>::N;
        const long per = (reduce + slices - 1) / slices;
        r0 = slice * per;
        r1 = r0 + per < reduce ? r0 + per : reduce;
        live = col < inner;
    }
};

template <typename T>
__device__ __forceinline__ void softmax_sliced_partial_vec(void* partials, const T* X, long reduce, long inner, long vtiles, int slices) {
    using M = SoftmaxMath<T>;
    using V = typename RowVec<T>::type;
    constexpr int VN = RowVec<T>::N;
    __shared__ T lm[VN][256];
    __shared__ T ls[VN][256];
    const SlicedVecWork<T> w(reduce, inner, vtiles, slices);
    const long nv = inner / VN;
    const V* x = reinterpret_cast<const V*>(X + w.o * reduce * inner + w.col);
    T m[VN], s[VN];
#pragma unroll
    for (int e = 0; e < VN; e++) m[e] = M::neg_inf(), s[e] = (T) 0;
    if (w.live) {
        long r = w.r0 + w.part;
        for (; r + 48 < w.r1; r += 64) {
            V v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = x[(r + 16 * u) * nv];
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int e = 0; e < VN; e++) online_step(v[u][e], m[e], s[e]);
        }
        for (; r < w.r1; r += 16) {
            const V v = x[r * nv];
#pragma unroll
            for (int e = 0; e < VN; e++) online_step(v[e], m[e], s[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < VN; e++) lm[e][threadIdx.x] = m[e], ls[e][threadIdx.x] = s[e];
    __syncthreads();
    if (w.part == 0 && w.live) {
        // the pairs of the slice, without the NaN marker for infinite maxima: that is applied once, at the end
        T* P = reinterpret_cast<T*>(partials);
#pragma unroll
        for (int e = 0; e < VN; e++) {
            T gm = M::neg_inf();
            for (int i = 0; i < 16; i++) gm = M::max(gm, lm[e][w.cl + 16 * i]);
            T gs = (T) 0;
            for (int i = 0; i < 16; i++) gs += pair_weight(lm[e][w.cl + 16 * i], ls[e][w.cl + 16 * i], gm);
            const long at = ((w.o * slices + w.slice) * inner + w.col + e) * 2;
            P[at] = gm;
            P[at + 1] = gs;
        }
    }
}

template <typename T>
__device__ __forceinline__ void softmax_sliced_finish_vec(const void* partials, const T* X, T* Y, long reduce, long inner, long vtiles, int slices) {
    using M = SoftmaxMath<T>;
    using V = typename RowVec<T>::type;
    constexpr int VN = RowVec<T>::N;
    __shared__ T lm[VN][256];
    __shared__ T ls[VN][256];
    const SlicedVecWork<T> w(reduce, inner, vtiles, slices);
    const T* P = reinterpret_cast<const T*>(partials);
    T m[VN], s[VN];
#pragma unroll
    for (int e = 0; e < VN; e++) m[e] = M::neg_inf(), s[e] = (T) 0;
    if (w.live)
        for (int sl = w.part; sl < slices; sl += 16) {
#pragma unroll
            for (int e = 0; e < VN; e++) {
                const long at = ((w.o * slices + sl) * inner + w.col + e) * 2;
                const T pm = P[at], ps = P[at + 1];
                const T g = M::max(m[e], pm);
                s[e] = pair_weight(m[e], s[e], g) + pair_weight(pm, ps, g);
                m[e] = g;
            }
        }
#pragma unroll
    for (int e = 0; e < VN; e++) lm[e][threadIdx.x] = m[e], ls[e][threadIdx.x] = s[e];
    __syncthreads();
    T gm[VN], scale[VN];
#pragma unroll
    for (int e = 0; e < VN; e++) {
        T gs;
        merge_pairs(lm[e], ls[e], w.cl, 16, 16, gm[e], gs);
        scale[e] = softmax_scale<T>(gs);
    }
    if (!w.live) return;
    const long nv = inner / VN;
    const V* x = reinterpret_cast<const V*>(X + w.o * reduce * inner + w.col);
    V* y = reinterpret_cast<V*>(Y + w.o * reduce * inner + w.col);
    long r = w.r0 + w.part;
    for (; r + 48 < w.r1; r += 64) {
        V v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = __builtin_nontemporal_load(x + (r + 16 * u) * nv);
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int e = 0; e < VN; e++) v[u][e] = softmax_result(M::exp_le0(v[u][e] - gm[e]), scale[e]);
            __builtin_nontemporal_store(v[u], y + (r + 16 * u) * nv);
        }
    }
    for (; r < w.r1; r += 16) {
        V v = __builtin_nontemporal_load(x + r * nv);
#pragma unroll
        for (int e = 0; e < VN; e++) v[e] = softmax_result(M::exp_le0(v[e] - gm[e]), scale[e]);
        __builtin_nontemporal_store(v, y + r * nv);
    }
}

// Rows cut into slices (inner == 1): rows longer than a work-group's registers hold, or too few of them to give every
// CU one. Work-group (row, slice) first leaves the (maximum, sum) pair of its `per` columns in the launcher's buffer,
// then - in a second launch - merges the pairs of its row and writes its own columns. Both launches read with 16-byte
// vectors wherever the row's address allows it: a row may start anywhere (cols need not be a multiple of the vector),
// so each slice is walked as a head of single elements up to the first 16-byte boundary, a body of vectors and a tail.
// X and Y must be equally placed relative to 16 bytes for the vector form (`vec`), else every access is one element.


// the running pair after the elements of one vector: one rescaling per vector instead of one per element
template <typename T>
__device__ __forceinline__ void online_vector(typename RowVec<T>::type v, T& m, T& s) {
    using M = SoftmaxMath<T>;
    T cm = v[0];
#pragma unroll
    for (int i = 1; i < RowVec<T>::N; i++) cm = M::max(cm, v[i]);   // NaN elements do not move the maximum
    const T nm = M::max(m, cm);
    if (nm != m) {            // m == -inf: s is 0 (or NaN) and exp(-inf) is 0
        s = s * M::exp_le0(m - nm);
        m = nm;
    }
#pragma unroll
    for (int i = 0; i < RowVec<T>::N; i++) s += (v[i] == M::neg_inf()) ? (T) 0 : M::exp_le0(v[i] - m);   // -inf weighs nothing; NaN poisons s
}

struct RowSlice {
    long c0, c1;          // columns [c0, c1) of the row
    long head, nvec;      // single elements before the vector body, vectors of the body
};

template <typename T>
__device__ __forceinline__ RowSlice row_slice(const T* x, long cols, long per, long slice, int vec) {
    RowSlice r;
    r.c0 = slice * per;
    r.c1 = r.c0 + per < cols ? r.c0 + per : cols;
    constexpr int N = RowVec<T>::N;
    if (vec) {
        const long mis = (long) ((reinterpret_cast<uintptr_t>(x + r.c0) / sizeof(T)) & (N - 1));
        r.head = mis ? N - mis : 0;
        if (r.head > r.c1 - r.c0) r.head = r.c1 - r.c0;
        r.nvec = (r.c1 - r.c0 - r.head) / N;
    } else {
        r.head = r.c1 - r.c0;
        r.nvec = 0;
    }
    return r;
}

// tree over the 256 pairs of a work-group; the result is in lm[0], ls[0]
template <typename T>
__device__ __forceinline__ void merge_block_pairs(T m, T s, T* lm, T* ls) {
    using M = SoftmaxMath<T>;
    lm[threadIdx.x] = m;
    ls[threadIdx.x] = s;
    __syncthreads();
    for (int half = 128; half > 0; half >>= 1) {
        if ((int) threadIdx.x < half) {
            const T m2 = lm[threadIdx.x + half], s2 = ls[threadIdx.x + half];
            const T m1 = lm[threadIdx.x], s1 = ls[threadIdx.x];
            const T g = M::max(m1, m2);
            lm[threadIdx.x] = g;
            ls[threadIdx.x] = pair_weight(m1, s1, g) + pair_weight(m2, s2, g);
        }
        __syncthreads();
    }
}

template <typename T>
__device__ __forceinline__ void softmax_rowslice_partial(void* partials, const T* X, long cols, long per, int slices, int vec) {
    using M = SoftmaxMath<T>;
    using V = typename RowVec<T>::type;
    constexpr int N = RowVec<T>::N;
    __shared__ T lm[256];
    __shared__ T ls[256];
    const long row = blockIdx.x / slices, slice = blockIdx.x % slices;
    const T* x = X + row * cols;
    const RowSlice r = row_slice(x, cols, per, slice, vec);
    T m = M::neg_inf(), s = (T) 0;
    // head and tail: at most N - 1 elements each in the vector form, the whole slice otherwise
    for (long c = r.c0 + threadIdx.x; c < r.c0 + r.head; c += 256) online_step(x[c], m, s);
    const V* xv = reinterpret_cast<const V*>(x + r.c0 + r.head);
    long i = threadIdx.x;
    for (; i + 768 < r.nvec; i += 1024) {   // four loads in flight per lane; ordinary loads: the second launch reads the slice again
        const V v0 = xv[i], v1 = xv[i + 256], v2 = xv[i + 512], v3 = xv[i + 768];
        online_vector<T>(v0, m, s);
        online_vector<T>(v1, m, s);
        online_vector<T>(v2, m, s);
        online_vector<T>(v3, m, s);
    }
    for (; i < r.nvec; i += 256) online_vector<T>(xv[i], m, s);
    for (long c = r.c0 + r.head + r.nvec * N + threadIdx.x; c < r.c1; c += 256) online_step(x[c], m, s);
    merge_block_pairs(m, s, lm, ls);
    if (threadIdx.x == 0) {
        T* P = reinterpret_cast<T*>(partials);
        P[blockIdx.x * 2] = lm[0];
        P[blockIdx.x * 2 + 1] = ls[0];
    }
}


template <typename T>
__device__ __forceinline__ void softmax_rowslice_finish(const void* partials, const T* X, T* Y, long cols, long per, int slices, int vec) {
    using M = SoftmaxMath<T>;
    using V = typename RowVec<T>::type;
    constexpr int N = RowVec<T>::N;
    __shared__ T lm[256];
    __shared__ T ls[256];
    const long row = blockIdx.x / slices, slice = blockIdx.x % slices;
    const T* P = reinterpret_cast<const T*>(partials) + row * slices * 2;
    T m = M::neg_inf(), s = (T) 0;
    for (int sl = threadIdx.x; sl < slices; sl += 256) {
        const T pm = P[sl * 2], ps = P[sl * 2 + 1];
        const T g = M::max(m, pm);
        s = pair_weight(m, s, g) + pair_weight(pm, ps, g);
        m = g;
    }
    merge_block_pairs(m, s, lm, ls);
    const T gm = lm[0];
    const T scale = softmax_scale<T>(ls[0] + (gm - gm));   // an infinite maximum makes every result NaN, as inf - inf does in the node's Sub step
    const T* x = X + row * cols;
    T* y = Y + row * cols;
    const RowSlice r = row_slice(x, cols, per, slice, vec);
    for (long c = r.c0 + threadIdx.x; c < r.c0 + r.head; c += 256) y[c] = softmax_result(M::exp_le0(x[c] - gm), scale);
    const V* xv = reinterpret_cast<const V*>(x + r.c0 + r.head);
    V* yv = reinterpret_cast<V*>(y + r.c0 + r.head);
    long i = threadIdx.x;
    for (; i + 768 < r.nvec; i += 1024) {
        V v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = __builtin_nontemporal_load(xv + i + 256 * j);
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int e = 0; e < N; e++) v[j][e] = softmax_result(M::exp_le0(v[j][e] - gm), scale);
            __builtin_nontemporal_store(v[j], yv + i + 256 * j);
        }
    }
    for (; i < r.nvec; i += 256) {
        V v = __builtin_nontemporal_load(xv + i);
#pragma unroll
        for (int e = 0; e < N; e++) v[e] = softmax_result(M::exp_le0(v[e] - gm), scale);
        __builtin_nontemporal_store(v, yv + i);
    }
    for (long c = r.c0 + r.head + r.nvec * N + threadIdx.x; c < r.c1; c += 256) y[c] = softmax_result(M::exp_le0(x[c] - gm), scale);
}

} // namespace

#define DOCC_SOFTMAX_ROWSLICE(T, SUFFIX)                                                                                           \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_rowslice_partial(void* partials, const T* X, long cols, \
                                                                                              long per, int slices, int vec) {      \
        softmax_rowslice_partial<T>(partials, X, cols, per, slices, vec);                                                          \
    }                                                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_rowslice_finish(const void* partials, const T* X, T* Y, \
                                                                                             long cols, long per, int slices, int vec) { \
        softmax_rowslice_finish<T>(partials, X, Y, cols, per, slices, vec);                                                        \
    }
DOCC_SOFTMAX_ROWSLICE(float, f32)
DOCC_SOFTMAX_ROWSLICE(double, f64)

#define DOCC_SOFTMAX_SLICED_VEC(T, SUFFIX)                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_slicedv_partial(void* partials, const T* X, long reduce, \
                                                                                             long inner, long tiles, int slices) { \
        softmax_sliced_partial_vec<T>(partials, X, reduce, inner, tiles, slices);                                                  \
    }                                                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_slicedv_finish(const void* partials, const T* X, T* Y, \
                                                                                            long reduce, long inner, long tiles,  \
                                                                                            int slices) {                         \
        softmax_sliced_finish_vec<T>(partials, X, Y, reduce, inner, tiles, slices);                                                \
    }
DOCC_SOFTMAX_SLICED_VEC(float, f32)
DOCC_SOFTMAX_SLICED_VEC(double, f64)

#define DOCC_SOFTMAX_SLICED(T, SUFFIX)                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_sliced_partial(void* partials, const T* X, long reduce, \
                                                                                            long inner, long tiles, int slices) { \
        softmax_sliced_partial<T>(partials, X, reduce, inner, tiles, slices);                                                 \
    }                                                                                                                         \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_sliced_finish(const void* partials, const T* X, T* Y, \
                                                                                           long reduce, long inner, long tiles, \
                                                                                           int slices) {                      \
        softmax_sliced_finish<T>(partials, X, Y, reduce, inner, tiles, slices);                                               \
    }
DOCC_SOFTMAX_SLICED(float, f32)
DOCC_SOFTMAX_SLICED(double, f64)

extern "C" __global__ __launch_bounds__(256) void docc_softmax_f64_stream(const double* X, double* Y, long rows, long cols) {
    softmax_row_stream<double>(X, Y, cols);
}
#define DOCC_SOFTMAX_STRIDED(T, SUFFIX)                                                                                     \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_tile(const T* X, T* Y, long reduce, long inner, \
                                                                                  long tiles) {                             \
        softmax_strided_tile<T>(X, Y, reduce, inner, tiles);                                                                \
    }                                                                                                                       \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_tilev16(const T* X, T* Y, long reduce, long inner, \
                                                                                     long tiles) {                          \
        softmax_strided_tile_vec<T, 16>(X, Y, reduce, inner, tiles);                                                        \
    }                                                                                                                       \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_tilev4(const T* X, T* Y, long reduce, long inner, \
                                                                                    long tiles) {                           \
        softmax_strided_tile_vec<T, 4>(X, Y, reduce, inner, tiles);                                                         \
    }                                                                                                                       \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_##SUFFIX##_slab(const T* X, T* Y, long reduce, int inner) { \
        softmax_strided_slab<T>(X, Y, reduce, inner);                                                                       \
    }
DOCC_SOFTMAX_STRIDED(float, f32)
DOCC_SOFTMAX_STRIDED(double, f64)
