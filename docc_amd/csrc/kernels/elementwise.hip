// Elementwise tensor nodes and ml::Broadcast, fp32 and fp64, for gfx950.
//
// Replace the Maps that ElementWiseUnaryNode / ElementWiseBinaryNode::expand produce (reference
// sdfg/include/sdfg/data_flow/library_nodes/math/tensor/elementwise_node.h: Y[i] = f(X[i]) or
// f(A[i], B[i]) over the linearised shape) and BroadcastNode::expand (broadcast_node.h:13-43).
// Operation semantics: elementwise_ops.h.
//
// HBM-bound: 8 (unary) or 12 (binary) bytes per fp32 element. One 128-bit access per operand
// and lane, grid-stride over the vectors, scalar tail; unaligned operands take the scalar path.
#include "elementwise_ops.h"

namespace docc_k {

template <typename T>
struct Vec128;
template <>
struct Vec128<float> {
    typedef float type __attribute__((ext_vector_type(4)));
    static constexpr int N = 4;
};
template <>
struct Vec128<double> {
    typedef double type __attribute__((ext_vector_type(2)));
    static constexpr int N = 2;
};

// Every kernel here is launched with work-groups of kGroup lanes. (blockDim.x would be a load from the hidden
// kernel arguments that each wave waits for before its first data load: waves that live for one or four vectors feel it.)
constexpr int kGroup = 256;

// nvec: number of whole 128-bit vectors to process vectorised (0 when an operand is unaligned)
template <typename T, int OP>
__device__ __forceinline__ void unary_kernel(const T* X, T* Y, long n, long nvec) {
    typedef typename Vec128<T>::type V;
    constexpr int N = Vec128<T>::N;
    const long stride = (long) gridDim.x * kGroup;
    const long tid = (long) blockIdx.x * kGroup + threadIdx.x;
    for (long i = tid; i < nvec; i += stride) {
        V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(X) + i);
#pragma unroll
        for (int e = 0; e < N; e++) v[e] = unary<OP>(v[e]);
        __builtin_nontemporal_store(v, reinterpret_cast<V*>(Y) + i);
    }
    for (long i = nvec * N + tid; i < n; i += stride) Y[i] = unary<OP>(X[i]);
}

template <typename T, int OP>
__device__ __forceinline__ void binary_kernel(const T* A, const T* B, T* Y, long n,
                                              long nvec) {
    typedef typename Vec128<T>::type V;
    constexpr int N = Vec128<T>::N;
    const long stride = (long) gridDim.x * kGroup;
    const long tid = (long) blockIdx.x * kGroup + threadIdx.x;
    for (long i = tid; i < nvec; i += stride) {
        const V a = __builtin_nontemporal_load(reinterpret_cast<const V*>(A) + i);
        const V b = __builtin_nontemporal_load(reinterpret_cast<const V*>(B) + i);
        V y;
#pragma unroll
        for (int e = 0; e < N; e++) y[e] = binary<OP>(a[e], b[e]);
        __builtin_nontemporal_store(y, reinterpret_cast<V*>(Y) + i);
    }
    for (long i = nvec * N + tid; i < n; i += stride) Y[i] = binary<OP>(A[i], B[i]);
}

// Activations with scalar operands: Y[i] = f(X[i], alpha, beta)
template <typename T, int OP>
__device__ __forceinline__ void param_unary_kernel(const T* X, T* Y, long n, long nvec, T alpha, T beta) {
    typedef typename Vec128<T>::type V;
    constexpr int N = Vec128<T>::N;
    const long stride = (long) gridDim.x * kGroup;
    const long tid = (long) blockIdx.x * kGroup + threadIdx.x;
    for (long i = tid; i < nvec; i += stride) {
        V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(X) + i);
#pragma unroll
        for (int e = 0; e < N; e++) v[e] = param_unary<OP>(v[e], alpha, beta);
        __builtin_nontemporal_store(v, reinterpret_cast<V*>(Y) + i);
    }
    for (long i = nvec * N + tid; i < n; i += stride) Y[i] = param_unary<OP>(X[i], alpha, beta);
}

// ml::Fill: every element of Y becomes one value of 1, 2, 4 or 8 bytes (fill_node.cpp:29-41: an assign
// tasklet from a scalar under the output's Maps). `pattern` holds the value repeated to 16 bytes.
__device__ __forceinline__ void fill_kernel(unsigned char* Y, long bytes, long nvec, u32x4 pattern) {
    const long stride = (long) gridDim.x * kGroup;
    const long tid = (long) blockIdx.x * kGroup + threadIdx.x;
    for (long i = tid; i < nvec; i += stride) __builtin_nontemporal_store(pattern, reinterpret_cast<u32x4*>(Y) + i);
    // the tail (and everything, when Y is not 16-byte aligned): byte b of the output is byte b % 16 of the pattern,
    // because the element size divides 16 and Y starts on an element boundary
    const unsigned char* pb = reinterpret_cast<const unsigned char*>(&pattern);
    for (long b = nvec * 16 + tid; b < bytes; b += stride) Y[b] = pb[b & 15];
}

// One operand is a scalar (the reference binds a constant or scalar container to "A" or "B",
// python/bindings/builder/py_structured_sdfg_builder.cpp:894-908): Y[i] = f(A[i], b), or
// f(b, A[i]) when LEFT.
template <typename T, int OP, bool LEFT>
__device__ __forceinline__ void binary_scalar_kernel(const T* A, T b, T* Y, long n, long nvec) {
    typedef typename Vec128<T>::type V;
    constexpr int N = Vec128<T>::N;
    const long stride = (long) gridDim.x * kGroup;
    const long tid = (long) blockIdx.x * kGroup + threadIdx.x;
    for (long i = tid; i < nvec; i += stride) {
        V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(A) + i);
#pragma unroll
        for (int e = 0; e < N; e++) v[e] = LEFT ? binary<OP>(b, v[e]) : binary<OP>(v[e], b);
        __builtin_nontemporal_store(v, reinterpret_cast<V*>(Y) + i);
    }
    for (long i = nvec * N + tid; i < n; i += stride) Y[i] = LEFT ? binary<OP>(b, A[i]) : binary<OP>(A[i], b);
}

// ml::Broadcast: Y[o] = X[offset(o)], numpy rules (an input dimension of extent 1 repeats).
// The launcher collapses the shape first (extent-1 output dimensions dropped, neighbours that
// are both repeated or both contiguous merged), so that `rank` is 1..3 for the usual cases.
// Write-bound: 4 or 8 bytes per output element; the input is re-read from cache.
struct BroadcastParams {
    int rank;
    long n;                 // elements of the output
    long out_dims[6];
    long in_strides[6];     // in elements; 0 for a repeated dimension
};

// VEC consecutive outputs of the innermost dimension per lane and step (its extent is a
// multiple of VEC), one 128-bit store; I: index type (32-bit when the output fits)
template <typename T, int VEC, typename I>
__device__ __forceinline__ void broadcast_kernel(const T* X, T* Y, const BroadcastParams& p) {
    typedef T V __attribute__((ext_vector_type(VEC)));
    const I stride = (I) gridDim.x * kGroup;
    const I nv = (I) (p.n / VEC);
    const int last = p.rank - 1;
    const I inner = (I) p.out_dims[last] / VEC;
    const bool inner_repeats = p.in_strides[last] == 0;
    // position of the lane's vector as (row, column) of the innermost dimension, advanced without divisions
    I v = (I) blockIdx.x * kGroup + threadIdx.x;
    I col = v % inner, row = v / inner;
    const I step_col = stride % inner, step_row = stride / inner;
    for (; v < nv; v += stride) {
        long off = inner_repeats ? 0 : (long) col * VEC;
        if (p.rank == 2) {
            off += (long) row * p.in_strides[0];
        } else if (p.rank > 2) {
            I rem = row;
#pragma unroll
            for (int d = 4; d >= 0; d--) {
                if (d < last) {
                    const I e = (I) p.out_dims[d];
                    off += (long) (rem % e) * p.in_strides[d];
                    rem /= e;
                }
            }
        }
        col += step_col;
        row += step_row;
        if (col >= inner) {
            col -= inner;
            row++;
        }
        V y;
        if (inner_repeats) {
            const T x = X[off];
#pragma unroll
            for (int e = 0; e < VEC; e++) y[e] = x;
        } else {
            y = *reinterpret_cast<const V*>(X + off);
        }
        __builtin_nontemporal_store(y, reinterpret_cast<V*>(Y) + v);
    }
}

// Fused chain: Y = post_k(...post_1(f(A', B'))), where A' and B' are A and B repeated to the
// output shape by numpy's rules (or a scalar), f one of the binary operations (or absent: the
// chain starts from A'), and post_i unary operations. It stands for a Broadcast node folded into
// its consumer and for unary nodes folded into their producer: one pass over memory instead of
// one per node. The operation codes are uniform over the launch, so the switches below are
// scalar branches.
struct FusedParams {
    long n;                 // elements of the output
    int rank;               // collapsed by the launcher
    long dims[6];
    long a_strides[6];      // in elements, 0 where the operand repeats
    long b_strides[6];
    int binary;             // BinaryOp or -1
    int a_scalar, b_scalar; // operand is the scalar below instead of an array
    int a_reused, b_reused; // operand repeats along some dimension: keep it in the caches
    double scalar_a, scalar_b;
    int npost;
    int post[4];            // UnaryOp codes
};

template <typename T, int VEC, typename I>
__device__ __forceinline__ void fused_kernel(const T* A, const T* B, T* Y, const FusedParams& p) {
    typedef T V __attribute__((ext_vector_type(VEC)));
    const I stride = (I) gridDim.x * kGroup;
    const I nv = (I) (p.n / VEC);
    const int last = p.rank - 1;
    const I inner = (I) p.dims[last] / VEC;
    const bool a_inner = !p.a_scalar && p.a_strides[last] != 0, b_inner = !p.b_scalar && p.b_strides[last] != 0;
    const bool has_b = p.binary >= 0;
    I v = (I) blockIdx.x * kGroup + threadIdx.x;
    I col = v % inner, row = v / inner;
    const I step_col = stride % inner, step_row = stride / inner;
    for (; v < nv; v += stride) {
        const long in = (long) col * VEC;
        long oa = a_inner ? in : 0, ob = b_inner ? in : 0;
        if (p.rank == 2) {
            oa += (long) row * p.a_strides[0];
            ob += (long) row * p.b_strides[0];
        } else if (p.rank > 2) {
            I rem = row;
#pragma unroll
            for (int d = 4; d >= 0; d--) {
                if (d < last) {
                    const I e = (I) p.dims[d];
                    const long c = (long) (rem % e);
                    rem /= e;
                    oa += c * p.a_strides[d];
                    ob += c * p.b_strides[d];
                }
            }
        }
        col += step_col;
        row += step_row;
        if (col >= inner) {
            col -= inner;
            row++;
        }
        V a, b;
        if (p.a_scalar) {
#pragma unroll
            for (int e = 0; e < VEC; e++) a[e] = (T) p.scalar_a;
        } else if (a_inner) {
            a = p.a_reused ? *reinterpret_cast<const V*>(A + oa) : __builtin_nontemporal_load(reinterpret_cast<const V*>(A + oa));
        } else {
            const T x = A[oa];
#pragma unroll
            for (int e = 0; e < VEC; e++) a[e] = x;
        }
        if (has_b) {
            if (p.b_scalar) {
#pragma unroll
                for (int e = 0; e < VEC; e++) b[e] = (T) p.scalar_b;
            } else if (b_inner) {
                b = p.b_reused ? *reinterpret_cast<const V*>(B + ob) : __builtin_nontemporal_load(reinterpret_cast<const V*>(B + ob));
            } else {
                const T x = B[ob];
#pragma unroll
                for (int e = 0; e < VEC; e++) b[e] = x;
            }
#pragma unroll
            for (int e = 0; e < VEC; e++) a[e] = apply_binary<T>(p.binary, a[e], b[e]);
        }
        for (int k = 0; k < p.npost; k++) {
#pragma unroll
            for (int e = 0; e < VEC; e++) a[e] = apply_unary<T>(p.post[k], a[e]);
        }
        __builtin_nontemporal_store(a, reinterpret_cast<V*>(Y) + v);
    }
}

// The same chain for outputs that collapse to rows x columns with both operands contiguous or repeated along
// the columns (address = base + row * s0 + column * s1, s1 0 or 1): the common cases - a bias row, a column of row
// statistics, two equal shapes, a scalar. A work-group is 2^cx_log2 column vectors wide and 256 >> cx_log2 rows
// high (narrow rows stack up in a wave, consecutive rows being consecutive memory), and a lane takes the same column
// vector of four rows, a group height apart: four loads in flight and no index arithmetic beyond an add per row; an
// operand that does not change from row to row (the bias row) is loaded once. The general kernel above recomputes
// every operand offset per vector and keeps one load in flight: 47.5 us against 41.0 here for relu(x + bias row) on
// [8192,4096] fp32. Groups are numbered along the columns first.
// What the rows kernel needs, at fixed places (a kernel argument indexed by the rank is a second, dependent load,
// and every wave waited for it before its first data load). Mirrored by the launcher.
struct FusedRowsParams {
    long rows, cols;
    long a_row_stride, b_row_stride;   // in elements; 0: the same in every row
    int a_along_cols, b_along_cols;    // operand varies along the columns (stride 1) or repeats (stride 0)
    int binary;                        // BinaryOp or -1
    int a_scalar, b_scalar;
    int a_reused, b_reused;
    int npost;
    int post[4];
    double scalar_a, scalar_b;
    int cx_log2;
    unsigned groups_x;
};

template <typename T, int VEC, bool WIDE>
__device__ __forceinline__ void fused_rows_body(const T* A, const T* B, T* Y, const FusedRowsParams& p) {
    typedef T V __attribute__((ext_vector_type(VEC)));
    constexpr int PER_LANE = 4;
    // WIDE: a group is one row high, so the row numbers (and a column operand's addresses) are the same for the whole group
    const int cx_log2 = WIDE ? 8 : p.cx_log2;
    const uint32_t groups_x = p.groups_x;
    const long rows = p.rows, cols = p.cols;
    const long sa0 = p.a_row_stride, sb0 = p.b_row_stride;
    const bool a_cols = !p.a_scalar && p.a_along_cols, b_cols = !p.b_scalar && p.b_along_cols;
    const bool has_b = p.binary >= 0;
    const int height = 256 >> cx_log2;
    const uint32_t gy = blockIdx.x / groups_x, gx = blockIdx.x - gy * groups_x;
    const long cv = ((long) gx << cx_log2) + (threadIdx.x & ((1u << cx_log2) - 1));
    if (cv * VEC >= cols) return;
    const long r0 = (long) gy * (PER_LANE * height) + (WIDE ? 0 : threadIdx.x >> cx_log2);
    auto load = [&](const T* base, bool scalar, double value, bool along_cols, long s0, bool reused, long r) {
        V v;
        if (scalar) {
#pragma unroll
            for (int e = 0; e < VEC; e++) v[e] = (T) value;
        } else if (along_cols) {
            const V* q = reinterpret_cast<const V*>(base + r * s0 + cv * VEC);
            v = reused ? *q : __builtin_nontemporal_load(q);
        } else {
            const T x = base[r * s0];
#pragma unroll
            for (int e = 0; e < VEC; e++) v[e] = x;
        }
        return v;
    };
    // an operand that is the same in every row (a scalar, a row vector) is fetched once
    const bool a_fixed = p.a_scalar || sa0 == 0, b_fixed = !has_b || p.b_scalar || sb0 == 0;
    V a0 = load(A, p.a_scalar, p.scalar_a, a_cols, 0, true, 0), b0 = a0;
    if (has_b) b0 = load(B, p.b_scalar, p.scalar_b, b_cols, 0, true, 0);
    auto finish = [&](V a, V b, long r) {
        if (has_b) {
#pragma unroll
            for (int e = 0; e < VEC; e++) a[e] = apply_binary<T>(p.binary, a[e], b[e]);
        }
        for (int k = 0; k < p.npost; k++) {
#pragma unroll
            for (int e = 0; e < VEC; e++) a[e] = apply_unary<T>(p.post[k], a[e]);
        }
        __builtin_nontemporal_store(a, reinterpret_cast<V*>(Y + r * cols) + cv);
    };
    if (r0 + (PER_LANE - 1) * height < rows) {
        V a[PER_LANE], b[PER_LANE];
#pragma unroll
        for (int u = 0; u < PER_LANE; u++) {
            a[u] = a_fixed ? a0 : load(A, false, 0, a_cols, sa0, p.a_reused, r0 + u * height);
            b[u] = b_fixed ? b0 : load(B, false, 0, b_cols, sb0, p.b_reused, r0 + u * height);
        }
#pragma unroll
        for (int u = 0; u < PER_LANE; u++) finish(a[u], b[u], r0 + u * height);
    } else {
        for (long r = r0; r < rows; r += height)
            finish(a_fixed ? a0 : load(A, false, 0, a_cols, sa0, p.a_reused, r), b_fixed ? b0 : load(B, false, 0, b_cols, sb0, p.b_reused, r), r);
    }
}

template <typename T, int VEC>
__device__ __forceinline__ void fused_rows_kernel(const T* A, const T* B, T* Y, const FusedRowsParams& p) {
    if (p.cx_log2 == 8)
        fused_rows_body<T, VEC, true>(A, B, Y, p);
    else
        fused_rows_body<T, VEC, false>(A, B, Y, p);
}

} // namespace docc_k

#define DOCC_EW_UNARY(NAME, OP)                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_f32(const float* X, float* Y, long n, long nvec) {       \
        docc_k::unary_kernel<float, docc_k::OP>(X, Y, n, nvec);                                                              \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_f64(const double* X, double* Y, long n, long nvec) {     \
        docc_k::unary_kernel<double, docc_k::OP>(X, Y, n, nvec);                                                             \
    }
#define DOCC_EW_BINARY_SCALAR(NAME, OP, SIDE, LEFT)                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_##SIDE##_f32(const float* A, float b, float* Y, long n,  \
                                                                                    long nvec) {                             \
        docc_k::binary_scalar_kernel<float, docc_k::OP, LEFT>(A, b, Y, n, nvec);                                             \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_##SIDE##_f64(const double* A, double b, double* Y,       \
                                                                                    long n, long nvec) {                     \
        docc_k::binary_scalar_kernel<double, docc_k::OP, LEFT>(A, b, Y, n, nvec);                                            \
    }
#define DOCC_EW_BINARY(NAME, OP)                                                                                             \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_f32(const float* A, const float* B, float* Y, long n,    \
                                                                           long nvec) {                                      \
        docc_k::binary_kernel<float, docc_k::OP>(A, B, Y, n, nvec);                                                          \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_f64(const double* A, const double* B, double* Y, long n, \
                                                                           long nvec) {                                      \
        docc_k::binary_kernel<double, docc_k::OP>(A, B, Y, n, nvec);                                                         \
    }                                                                                                                        \
    DOCC_EW_BINARY_SCALAR(NAME, OP, sr, false)                                                                               \
    DOCC_EW_BINARY_SCALAR(NAME, OP, sl, true)

#define DOCC_EW_PARAM_UNARY(NAME, OP)                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_f32(const float* X, float* Y, long n, long nvec, float alpha, \
                                                                           float beta) {                                     \
        docc_k::param_unary_kernel<float, docc_k::OP>(X, Y, n, nvec, alpha, beta);                                           \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_##NAME##_f64(const double* X, double* Y, long n, long nvec,       \
                                                                           double alpha, double beta) {                      \
        docc_k::param_unary_kernel<double, docc_k::OP>(X, Y, n, nvec, alpha, beta);                                          \
    }
DOCC_EW_PARAM_UNARY(elu, kElu)
DOCC_EW_PARAM_UNARY(leaky_relu, kLeakyReLU)
DOCC_EW_PARAM_UNARY(hard_sigmoid, kHardSigmoid)

extern "C" __global__ __launch_bounds__(256) void docc_fill_bytes(unsigned char* Y, long bytes, long nvec, docc_k::u32x4 pattern) {
    docc_k::fill_kernel(Y, bytes, nvec, pattern);
}

DOCC_EW_UNARY(abs, kAbs)
DOCC_EW_UNARY(exp, kExp)
DOCC_EW_UNARY(relu, kReLU)
DOCC_EW_UNARY(sigmoid, kSigmoid)
DOCC_EW_UNARY(sqrt, kSqrt)
DOCC_EW_UNARY(tanh, kTanh)
DOCC_EW_UNARY(erf, kErf)
DOCC_EW_BINARY(add, kAdd)
DOCC_EW_BINARY(sub, kSub)
DOCC_EW_BINARY(mul, kMul)
DOCC_EW_BINARY(div, kDiv)
DOCC_EW_BINARY(maximum, kMaximum)
DOCC_EW_BINARY(minimum, kMinimum)
DOCC_EW_BINARY(pow, kPow)

#define DOCC_BROADCAST(NAME, T, VEC, I)                                                                                     \
    extern "C" __global__ __launch_bounds__(256) void docc_broadcast_##NAME(const T* X, T* Y, docc_k::BroadcastParams p) {     \
        docc_k::broadcast_kernel<T, VEC, I>(X, Y, p);                                                                       \
    }
// <type>_v<lanes>_i<index bits>
DOCC_BROADCAST(f32_v4_i32, float, 4, unsigned)
DOCC_BROADCAST(f32_v1_i32, float, 1, unsigned)
DOCC_BROADCAST(f32_v4_i64, float, 4, long)
DOCC_BROADCAST(f32_v1_i64, float, 1, long)
DOCC_BROADCAST(f64_v2_i32, double, 2, unsigned)
DOCC_BROADCAST(f64_v1_i32, double, 1, unsigned)
DOCC_BROADCAST(f64_v2_i64, double, 2, long)
DOCC_BROADCAST(f64_v1_i64, double, 1, long)

#define DOCC_EW_FUSED(NAME, T, VEC, I)                                                                                      \
    extern "C" __global__ __launch_bounds__(256) void docc_ew_fused_##NAME(const T* A, const T* B, T* Y,                       \
                                                                           docc_k::FusedParams p) {                         \
        docc_k::fused_kernel<T, VEC, I>(A, B, Y, p);                                                                        \
    }
extern "C" __global__ __launch_bounds__(256) void docc_ew_fused_rows_f32_v4(const float* A, const float* B, float* Y, docc_k::FusedRowsParams p) {
    docc_k::fused_rows_kernel<float, 4>(A, B, Y, p);
}
extern "C" __global__ __launch_bounds__(256) void docc_ew_fused_rows_f64_v2(const double* A, const double* B, double* Y, docc_k::FusedRowsParams p) {
    docc_k::fused_rows_kernel<double, 2>(A, B, Y, p);
}
DOCC_EW_FUSED(f32_v4_i32, float, 4, unsigned)
DOCC_EW_FUSED(f32_v1_i32, float, 1, unsigned)
DOCC_EW_FUSED(f32_v4_i64, float, 4, long)
DOCC_EW_FUSED(f32_v1_i64, float, 1, long)
DOCC_EW_FUSED(f64_v2_i32, double, 2, unsigned)
DOCC_EW_FUSED(f64_v1_i32, double, 1, unsigned)
DOCC_EW_FUSED(f64_v2_i64, double, 2, long)
DOCC_EW_FUSED(f64_v1_i64, double, 1, long)


// ---- ml::Cast ---------------------------------------------------------------------------------
// Y[i] = (D) X[i], the conversion an assign tasklet between differently typed memlets compiles to
// (reference elementwise_ops/cast_node.cpp:39-40): round to nearest even between floating types,
// truncation towards zero from a floating type to an integer. bf16 travels as raw 16-bit words.
namespace docc_k {

struct Bf16Bits { unsigned short bits; };

template <typename S> __device__ __forceinline__ auto cast_load(const S* p, long i) { return p[i]; }
template <> __device__ __forceinline__ auto cast_load<Bf16Bits>(const Bf16Bits* p, long i) { return bf16_bits_to_f32(p[i].bits); }

template <typename D, typename V> __device__ __forceinline__ void cast_store(D* p, long i, V v) { p[i] = (D) v; }
template <> __device__ __forceinline__ void cast_store<Bf16Bits, float>(Bf16Bits* p, long i, float v) { p[i].bits = f32_to_bf16_rne(v); }

template <typename S, typename D>
__device__ __forceinline__ void cast_kernel(const S* X, D* Y, long n) {
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < n; i += stride) cast_store<D>(Y, i, cast_load<S>(X, i));
}

} // namespace docc_k

#define DOCC_CAST(SN, S, DN, D)                                                                                          \
    extern "C" __global__ __launch_bounds__(256) void docc_cast_##SN##_##DN(const S* X, D* Y, long n) {                    \
        docc_k::cast_kernel<S, D>(X, Y, n);                                                                              \
    }
DOCC_CAST(f32, float, f64, double)
DOCC_CAST(f64, double, f32, float)
DOCC_CAST(f32, float, bf16, docc_k::Bf16Bits)
DOCC_CAST(bf16, docc_k::Bf16Bits, f32, float)
DOCC_CAST(f32, float, f16, _Float16)
DOCC_CAST(f16, _Float16, f32, float)
DOCC_CAST(i32, int, f32, float)
DOCC_CAST(i32, int, f64, double)
DOCC_CAST(i64, long, f32, float)
DOCC_CAST(i64, long, f64, double)
DOCC_CAST(f32, float, i32, int)
DOCC_CAST(f64, double, i32, int)
DOCC_CAST(f32, float, i64, long)
DOCC_CAST(f64, double, i64, long)
