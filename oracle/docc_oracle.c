/*
 * docc_oracle.c - CPU restatement of what docc's `openmp` target computes for
 * the math library nodes GEMM, Softmax and Conv, plus closed-form references
 * for the two node modes the rocm target adds (bf16 GEMM, Attention).
 *
 * THIS IS TEST INFRASTRUCTURE. It is the checker that the parity tests, the
 * smoke test and the `cpu_baseline` leg of the benchmark compare against and
 * time. Nothing in the product path may call it; the product path fails when
 * its HIP library is missing instead of falling back to this file.
 *
 * Every function names the reference code it follows (paths relative to the
 * reference tree). Loop structure mirrors the reference's expansions: Maps
 * become `for` loops of which only the outermost carries
 * `#pragma omp parallel for schedule(static)`, as OMPScheduler parallelises
 * only the outermost Map (opt/src/passes/scheduler/omp_scheduler.cpp:9-20) and
 * OMPMapDispatcher prints exactly that pragma
 * (opt/src/targets/omp/codegen/omp_map_dispatcher.cpp:46-82); reductions are
 * sequential `For` loops. Build with the reference JIT's flags
 * (python/bindings/py_structured_sdfg.cpp:456,516):
 *   gcc -O3 -march=native -mtune=native -funroll-loops -fopenmp -fPIC -shared
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   gemm_*      integer-valued known-answer products (exact in every
 *               summation order), identity / permutation / rank-1 cases,
 *               numpy.matmul, long-double accumulation bound;
 *   softmax_*   scipy.special.softmax in fp64, row-sum / shift-invariance /
 *               constant-row closed forms;
 *   conv2d_f32  torch.nn.functional.conv2d in fp64, delta-kernel identity and
 *               shift, all-ones tap counts at corner/edge/interior, bias-only;
 *   attention   torch SDPA (math path) in fp64, equal-keys => mean of V,
 *               key-permutation invariance;
 *   bf16 conversion: exhaustive against torch's round-to-nearest-even;
 *   elementwise_*  numpy's ufuncs (bit-exact for the IEEE operations and the
 *               selections, <= 2 ulp for exp/tanh/erf/sigmoid), closed forms
 *               (relu of negatives is +0, sigmoid(0) = 1/2, tanh odd, x/x = 1);
 *   broadcast   numpy.broadcast_to.
 * The reference holds no numeric golden vectors for any of these nodes (its
 * tests recompute expectations with numpy/torch at run time), so the pins
 * above are the mathematics and the library cross-checks.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORACLE_API void oracle_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void) n;
#endif
}

/* ------------------------------------------------------------------ bf16 */

/* fp32 -> bf16 bits, round to nearest even; the value the reference's BFloat
 * type (`__bf16`, sdfg/src/codegen/language_extensions/cpp_language_extension.cpp:9-52)
 * takes on conversion from float. */
ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t) ((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t) (u >> 16);
}

ORACLE_API float oracle_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t) h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

ORACLE_API void oracle_f32_to_bf16_array(int64_t n, const float* src, uint16_t* dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = oracle_f32_to_bf16(src[i]);
}

ORACLE_API void oracle_bf16_to_f32_array(int64_t n, const uint16_t* src, float* dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = oracle_bf16_to_f32(src[i]);
}

/* ------------------------------------------------------------------ GEMM */

/*
 * GEMMNode::expand (sdfg/src/data_flow/library_nodes/math/blas/gemm_node.cpp:179-311),
 * NoTrans/NoTrans only, as the reference expands it:
 *   Map _i, Map _j: _sum = 0.0; For _k: _sum = A[lda*_i+_k] * B[ldb*_k+_j] + _sum;
 *   C[ldc*_i+_j] = (_sum * alpha) + (C[ldc*_i+_j] * beta)
 * The expansion reads C even when beta == 0.
 */
#define ORACLE_GEMM_EXPANDED(NAME, T)                                                                          \
    ORACLE_API void NAME(int64_t m, int64_t n, int64_t k, T alpha, const T* A, int64_t lda, const T* B,        \
                         int64_t ldb, T beta, T* C, int64_t ldc) {                                             \
        _Pragma("omp parallel for schedule(static)") for (int64_t _i = 0; _i < m; _i++) {                      \
            for (int64_t _j = 0; _j < n; _j++) {                                                               \
                T _sum = (T) 0.0;                                                                              \
                for (int64_t _k = 0; _k < k; _k++) _sum = A[lda * _i + _k] * B[ldb * _k + _j] + _sum;          \
                T scaled_sum_temp = _sum * alpha;                                                              \
                T scaled_input_temp = C[ldc * _i + _j] * beta;                                                 \
                C[ldc * _i + _j] = scaled_sum_temp + scaled_input_temp;                                        \
            }                                                                                                  \
        }                                                                                                      \
    }
ORACLE_GEMM_EXPANDED(oracle_gemm_expanded_f64, double)
ORACLE_GEMM_EXPANDED(oracle_gemm_expanded_f32, float)

/*
 * The call GEMMNodeDispatcher_BLAS prints (gemm_node.cpp:449-509):
 *   cblas_?gemm(CblasRowMajor, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)
 * restated from the BLAS definition C = alpha*op(A)*op(B) + beta*C, where C
 * is not read when beta == 0 and A, B are not referenced when alpha == 0 (the
 * BLAS definition of ?GEMM: "when ALPHA is zero then A and B are not referenced",
 * so NaNs in them do not reach C). trans codes are CBLAS's 111 (NoTrans) / 112
 * (Trans), the values the node serialises (blas_node.h:49-126). The k-loop
 * runs left to right in the element type.
 */
#define ORACLE_GEMM_BLAS(NAME, T, ACC)                                                                         \
    ORACLE_API void NAME(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, T alpha, const T* A,       \
                         int64_t lda, const T* B, int64_t ldb, T beta, T* C, int64_t ldc) {                    \
        _Pragma("omp parallel for schedule(static)") for (int64_t i = 0; i < m; i++) {                         \
            for (int64_t j = 0; j < n; j++) {                                                                  \
                ACC sum = 0;                                                                                   \
                for (int64_t p = 0; p < (alpha == (T) 0 ? 0 : k); p++) {                                       \
                    ACC a = (trans_a == 112) ? A[lda * p + i] : A[lda * i + p];                                \
                    ACC b = (trans_b == 112) ? B[ldb * j + p] : B[ldb * p + j];                                \
                    sum += a * b;                                                                              \
                }                                                                                              \
                ACC r = (ACC) alpha * sum;                                                                     \
                if (beta != (T) 0) r += (ACC) beta * (ACC) C[ldc * i + j];                                     \
                C[ldc * i + j] = (T) r;                                                                        \
            }                                                                                                  \
        }                                                                                                      \
    }
ORACLE_GEMM_BLAS(oracle_gemm_blas_f64, double, double)
ORACLE_GEMM_BLAS(oracle_gemm_blas_f32, float, float)
/* long-double accumulation: the yardstick for the 1e-12 fp64 bound */
ORACLE_GEMM_BLAS(oracle_gemm_blas_f64_ld, double, long double)
/* fp32 data, fp64 accumulation: the yardstick for the fp32 bound */
ORACLE_GEMM_BLAS(oracle_gemm_blas_f32_acc64, float, double)

/*
 * bf16 inputs (raw bits), fp32 accumulate and output. The reference has no
 * such precision (BLAS_Precision is h,s,d,c,z: blas_node.h:49-55); this is the
 * closed form C = alpha*A*B + beta*C evaluated in fp32 on the bf16 values,
 * k left to right.
 */
ORACLE_API void oracle_gemm_bf16_f32(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                                     const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, float beta,
                                     float* C, int64_t ldc) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; i++) {
        for (int64_t j = 0; j < n; j++) {
            float sum = 0.f;
            for (int64_t p = 0; p < k; p++) {
                float a = oracle_bf16_to_f32((trans_a == 112) ? A[lda * p + i] : A[lda * i + p]);
                float b = oracle_bf16_to_f32((trans_b == 112) ? B[ldb * j + p] : B[ldb * p + j]);
                sum += a * b;
            }
            float r = alpha * sum;
            if (beta != 0.f) r += beta * C[ldc * i + j];
            C[ldc * i + j] = r;
        }
    }
}

/* --------------------------------------------------------------- Softmax */

/*
 * SoftmaxNode::expand over the last axis of X[rows, cols]
 * (sdfg/src/data_flow/library_nodes/math/tensor/reduce_ops/softmax_node.cpp:112-252):
 * six malloc'd temporaries, then Max(keepdims) -> Broadcast -> Sub -> Exp ->
 * Sum(keepdims) -> Broadcast -> Div, each its own loop nest.
 * Max: identity -INFINITY, fmaxf through memory (max_node.cpp:56-91);
 * Sum: identity 0.0, left-to-right adds through memory (sum_node.cpp:20-57);
 * the reduce nests follow ReduceNode::expand (reduce_node.cpp:188-333):
 * an init nest, then Map over kept dims / For over reduced dims.
 * The reference never frees the temporaries (no Free nodes); they are freed here.
 * Returns 0, or -1 when a temporary cannot be allocated.
 */
ORACLE_API int oracle_softmax_expanded_f32(int64_t rows, int64_t cols, const float* X, float* Y) {
    size_t full = (size_t) rows * (size_t) cols;
    float* tmp_max = (float*) malloc(sizeof(float) * (size_t) (rows ? rows : 1));
    float* tmp_max_bcast = (float*) malloc(sizeof(float) * (full ? full : 1));
    float* tmp_sub = (float*) malloc(sizeof(float) * (full ? full : 1));
    float* tmp_exp = (float*) malloc(sizeof(float) * (full ? full : 1));
    float* tmp_sum = (float*) malloc(sizeof(float) * (size_t) (rows ? rows : 1));
    float* tmp_sum_bcast = (float*) malloc(sizeof(float) * (full ? full : 1));
    int rc = 0;
    if (!tmp_max || !tmp_max_bcast || !tmp_sub || !tmp_exp || !tmp_sum || !tmp_sum_bcast) {
        rc = -1;
        goto done;
    }
    /* 1. Max */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++) tmp_max[i] = -INFINITY;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t k = 0; k < cols; k++) tmp_max[i] = fmaxf(X[i * cols + k], tmp_max[i]);
    /* 1.5 Broadcast */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) tmp_max_bcast[i * cols + j] = tmp_max[i];
    /* 2. Sub */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) tmp_sub[i * cols + j] = X[i * cols + j] - tmp_max_bcast[i * cols + j];
    /* 3. Exp */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) tmp_exp[i * cols + j] = expf(tmp_sub[i * cols + j]);
    /* 4. Sum */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++) tmp_sum[i] = 0.0f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t k = 0; k < cols; k++) tmp_sum[i] = tmp_exp[i * cols + k] + tmp_sum[i];
    /* 4.5 Broadcast */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) tmp_sum_bcast[i * cols + j] = tmp_sum[i];
    /* 5. Div */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) Y[i * cols + j] = tmp_exp[i * cols + j] / tmp_sum_bcast[i * cols + j];
done:
    free(tmp_max);
    free(tmp_max_bcast);
    free(tmp_sub);
    free(tmp_exp);
    free(tmp_sum);
    free(tmp_sum_bcast);
    return rc;
}

/*
 * The same expansion for fp64 elements (the element type of the node is that of its
 * memlets, softmax_node.cpp:89-90; Max uses fmax, Exp uses exp: max_node.cpp:56-67,
 * cmath_node.h:364-365). The two broadcast temporaries are read in place of the
 * reduced ones; the arithmetic and its order are those of the seven nests above.
 * Reductions over other axes than the last are this function on the input with the
 * reduced axes moved to the end, in ascending order: the reduce nests visit the reduced
 * dimensions in that order (reduce_node.cpp:188-333).
 */
ORACLE_API int oracle_softmax_expanded_f64(int64_t rows, int64_t cols, const double* X, double* Y) {
    size_t full = (size_t) rows * (size_t) cols;
    double* tmp_max = (double*) malloc(sizeof(double) * (size_t) (rows ? rows : 1));
    double* tmp_exp = (double*) malloc(sizeof(double) * (full ? full : 1));
    double* tmp_sum = (double*) malloc(sizeof(double) * (size_t) (rows ? rows : 1));
    int rc = 0;
    if (!tmp_max || !tmp_exp || !tmp_sum) {
        rc = -1;
        goto done;
    }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++) {
        tmp_max[i] = -INFINITY;
        for (int64_t k = 0; k < cols; k++) tmp_max[i] = fmax(X[i * cols + k], tmp_max[i]);
        for (int64_t j = 0; j < cols; j++) tmp_exp[i * cols + j] = exp(X[i * cols + j] - tmp_max[i]);
        tmp_sum[i] = 0.0;
        for (int64_t k = 0; k < cols; k++) tmp_sum[i] = tmp_exp[i * cols + k] + tmp_sum[i];
        for (int64_t j = 0; j < cols; j++) Y[i * cols + j] = tmp_exp[i * cols + j] / tmp_sum[i];
    }
done:
    free(tmp_max);
    free(tmp_exp);
    free(tmp_sum);
    return rc;
}

/*
 * The decomposed numpy form the reference's own softmax benchmark compiles
 * (python/benchmarks/npbench/deep_learning/softmax/test_softmax.py:24-28):
 *   tmp_max = max(x, -1, keepdims); tmp_out = exp(x - tmp_max);
 *   tmp_sum = sum(tmp_out, -1, keepdims); return tmp_out / tmp_sum
 * i.e. a Max-reduce nest, a Sub nest, an Exp nest, a Sum-reduce nest, a Div
 * nest (broadcast operands are zero-stride views, python/docc/python/functions/numpy.py:1209-1233),
 * and the copy into the caller's return buffer (python/docc/python/ast_parser.py:1186-1210).
 * This is the form the `openmp` target can run for fp32 input and the one the
 * CPU baseline times. Returns 0 or -1 (allocation failure).
 */
ORACLE_API int oracle_softmax_numpy_f32(int64_t rows, int64_t cols, const float* X, float* ret) {
    size_t full = (size_t) rows * (size_t) cols;
    float* tmp_max = (float*) malloc(sizeof(float) * (size_t) (rows ? rows : 1));
    float* tmp_sub = (float*) malloc(sizeof(float) * (full ? full : 1));
    float* tmp_out = (float*) malloc(sizeof(float) * (full ? full : 1));
    float* tmp_sum = (float*) malloc(sizeof(float) * (size_t) (rows ? rows : 1));
    float* result = (float*) malloc(sizeof(float) * (full ? full : 1));
    int rc = 0;
    if (!tmp_max || !tmp_sub || !tmp_out || !tmp_sum || !result) {
        rc = -1;
        goto done;
    }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++) tmp_max[i] = -INFINITY;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t k = 0; k < cols; k++) tmp_max[i] = fmaxf(X[i * cols + k], tmp_max[i]);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) tmp_sub[i * cols + j] = X[i * cols + j] - tmp_max[i];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) tmp_out[i * cols + j] = expf(tmp_sub[i * cols + j]);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++) tmp_sum[i] = 0.0f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t k = 0; k < cols; k++) tmp_sum[i] = tmp_out[i * cols + k] + tmp_sum[i];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) result[i * cols + j] = tmp_out[i * cols + j] / tmp_sum[i];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) ret[i * cols + j] = result[i * cols + j];
done:
    free(tmp_max);
    free(tmp_sub);
    free(tmp_out);
    free(tmp_sum);
    free(result);
    return rc;
}

/* ------------------------------------------------------------------ Conv */

/* Output extent, ConvNode::expand (sdfg/src/data_flow/library_nodes/math/tensor/conv_node.cpp:224-233):
 * D_out = (D_in + pad_begin + pad_end - dilation*(kernel-1) - 1) / stride + 1 */
ORACLE_API int64_t oracle_conv_out_dim(int64_t d_in, int64_t pad_begin, int64_t pad_end, int64_t dilation,
                                       int64_t kernel, int64_t stride) {
    int64_t num = d_in + pad_begin + pad_end - (dilation * (kernel - 1) + 1);
    if (num < 0) return 0;
    return num / stride + 1;
}

/*
 * ConvNode::expand (conv_node.cpp:244-437), 2-d, group 1:
 *   Map n, Map oc, Map od0, Map od1: accum = 0.0;
 *     For ic, For k0, For k1:
 *       accum = X[n, ic, od0*s0 - p0 + k0*d0, od1*s1 - p1 + k1*d1] * W[oc, ic, k0, k1] + accum
 *   Y[n, oc, od0, od1] = accum + B[oc]      (or = accum without a bias edge)
 * The reference indexes X without a bounds test, so with pad > 0 it reads out
 * of bounds; the ONNX Conv definition its header cites (conv_node.h:9-22)
 * pads with zeros, which is what the guard below does.
 */
/* pads as the node carries them (conv_node.cpp:76-77, 169-176): a begin and an end per spatial axis; the begin pad
 * moves the window, the end pad only adds output positions (conv_node.cpp:224-233). */
ORACLE_API void oracle_conv2d_f32_pads(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                                       int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t pad_h_end,
                                       int64_t pad_w_end, int64_t dil_h, int64_t dil_w, const float* X, const float* Wt,
                                       const float* bias, float* Y) {
    int64_t OH = oracle_conv_out_dim(H, pad_h, pad_h_end, dil_h, KH, stride_h);
    int64_t OW = oracle_conv_out_dim(W, pad_w, pad_w_end, dil_w, KW, stride_w);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        for (int64_t oc = 0; oc < OC; oc++) {
            for (int64_t od0 = 0; od0 < OH; od0++) {
                for (int64_t od1 = 0; od1 < OW; od1++) {
                    float accum = 0.0f;
                    for (int64_t ic = 0; ic < C; ic++) {
                        for (int64_t k0 = 0; k0 < KH; k0++) {
                            for (int64_t k1 = 0; k1 < KW; k1++) {
                                int64_t ih = od0 * stride_h - pad_h + k0 * dil_h;
                                int64_t iw = od1 * stride_w - pad_w + k1 * dil_w;
                                if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                                accum = X[((n * C + ic) * H + ih) * W + iw] * Wt[((oc * C + ic) * KH + k0) * KW + k1] +
                                        accum;
                            }
                        }
                    }
                    Y[((n * OC + oc) * OH + od0) * OW + od1] = bias ? accum + bias[oc] : accum;
                }
            }
        }
    }
}

ORACLE_API void oracle_conv2d_f32(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                                  int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t dil_h,
                                  int64_t dil_w, const float* X, const float* Wt, const float* bias, float* Y) {
    oracle_conv2d_f32_pads(N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h, pad_w, dil_h, dil_w, X, Wt, bias, Y);
}

/* ------------------------------------------------------------- Attention */

/*
 * softmax(scale * Q K^T) V per (batch, head), non-causal, from bf16 inputs
 * with fp32 scores, softmax and accumulation. The reference has no attention
 * node and cannot express batched matmul (mlir/lib/Target/SDFG/LinalgToSDFGTranslator.cpp:517-523),
 * so this is the closed form, written as the reference would compose it from
 * its own pieces: MatMul (one GEMM per batch, matmul_node.cpp:366-499), scale,
 * Softmax over the last axis (softmax_node.cpp:142-252), MatMul.
 * O is fp32 [B,H,SQ,D]. Returns 0 or -1 (allocation failure).
 */
ORACLE_API int oracle_attention_bf16(int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D, float scale,
                                     const uint16_t* Q, const uint16_t* K, const uint16_t* V, float* O) {
    int64_t BH = B * H;
    int rc = 0;
#pragma omp parallel for schedule(static)
    for (int64_t bh = 0; bh < BH; bh++) {
        float* s = (float*) malloc(sizeof(float) * (size_t) (SKV ? SKV : 1));
        if (!s) {
#pragma omp atomic write
            rc = -1;
            continue;
        }
        const uint16_t* q = Q + bh * SQ * D;
        const uint16_t* kk = K + bh * SKV * D;
        const uint16_t* v = V + bh * SKV * D;
        float* o = O + bh * SQ * D;
        for (int64_t i = 0; i < SQ; i++) {
            float mx = -INFINITY;
            for (int64_t j = 0; j < SKV; j++) {
                float sum = 0.f;
                for (int64_t d = 0; d < D; d++)
                    sum = oracle_bf16_to_f32(q[i * D + d]) * oracle_bf16_to_f32(kk[j * D + d]) + sum;
                s[j] = sum * scale;
                mx = fmaxf(s[j], mx);
            }
            float den = 0.f;
            for (int64_t j = 0; j < SKV; j++) {
                s[j] = expf(s[j] - mx);
                den = s[j] + den;
            }
            for (int64_t d = 0; d < D; d++) {
                float acc = 0.f;
                for (int64_t j = 0; j < SKV; j++) acc = (s[j] / den) * oracle_bf16_to_f32(v[j * D + d]) + acc;
                o[i * D + d] = acc;
            }
        }
        free(s);
    }
    return rc;
}


/* ------------------------------------------------------------------------------------------
 * Elementwise tensor nodes: Y[i] = f(X[i]) / f(A[i], B[i]) over the linearised shape
 * (sdfg/include/sdfg/data_flow/library_nodes/math/tensor/elementwise_node.h; expansions in
 * sdfg/src/data_flow/library_nodes/math/tensor/elementwise_ops/: relu_node.cpp:40-43 fmax(x, 0.0),
 * sigmoid_node.cpp:46-70 neg -> exp -> add 1.0 -> 1.0 / x, maximum_node.cpp:64 fmax, minimum_node.cpp
 * fmin, abs/exp/sqrt/tanh/erf the libm call of the element type, add/sub/mul/div one tasklet).
 * One Map over the elements: omp parallel for. Operation codes as in include/docc_rocm_ops.h. */
#define ORACLE_UNARY_BODY(T, SUF)                                                          \
    switch (op) {                                                                          \
        case 0: y = fabs##SUF(x); break;                                                   \
        case 1: y = exp##SUF(x); break;                                                    \
        case 2: y = fmax##SUF(x, (T) 0.0); break;                                          \
        case 3: { T t = -x; t = exp##SUF(t); t = t + (T) 1.0; y = (T) 1.0 / t; break; }    \
        case 4: y = sqrt##SUF(x); break;                                                   \
        case 5: y = tanh##SUF(x); break;                                                   \
        default: y = erf##SUF(x); break;                                                   \
    }
#define ORACLE_BINARY_BODY(T, SUF)                                                         \
    switch (op) {                                                                          \
        case 0: y = a + b; break;                                                          \
        case 1: y = a - b; break;                                                          \
        case 2: y = a * b; break;                                                          \
        case 3: y = a / b; break;                                                          \
        case 4: y = fmax##SUF(a, b); break;                                                \
        case 6: y = pow##SUF(a, b); break; /* pow_node.cpp:52-54: CMathFunction::pow */     \
        default: y = fmin##SUF(a, b); break;                                               \
    }

ORACLE_API int oracle_elementwise_unary_f32(int op, int64_t n, const float* X, float* Y) {
    if (op < 0 || op > 6) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const float x = X[i];
        float y;
        ORACLE_UNARY_BODY(float, f)
        Y[i] = y;
    }
    return 0;
}

ORACLE_API int oracle_elementwise_unary_f64(int op, int64_t n, const double* X, double* Y) {
    if (op < 0 || op > 6) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const double x = X[i];
        double y;
        ORACLE_UNARY_BODY(double, )
        Y[i] = y;
    }
    return 0;
}

/* The unary nodes with scalar operands (connectors "alpha", "beta"): ml::Elu (elu_node.cpp:21-97), ml::LeakyReLU
 * (leaky_relu_node.cpp:21-68), ml::HardSigmoid (hard_sigmoid_node.cpp:21-83), operation codes 7, 8, 9. The
 * reference's expansions are unfinished - Elu computes alpha * (exp(x) - 1) for every x, LeakyReLU's multiply
 * and HardSigmoid's fma have one operand - so this restates the ONNX operators the nodes are named after,
 * keeping the steps the reference does spell out in their order (exp, minus 1.0, times alpha; a * x + b,
 * fmin with 1, fmax with 0). Parity unpinned by the reference (no test of it computes values); pinned by
 * torch's elu / leaky_relu / hardsigmoid and closed forms in tests/test_oracle.py. */
#define ORACLE_ACTIVATION_BODY(T, SUF)                                                                     \
    switch (op) {                                                                                          \
        case 7: { T t = exp##SUF(x); t = t - (T) 1.0; t = alpha * t; y = x > (T) 0.0 ? x : t; break; }     \
        case 8: y = x >= (T) 0.0 ? x : alpha * x; break;                                                   \
        default: { T t = fma##SUF(alpha, x, beta); t = fmin##SUF(t, (T) 1.0); y = fmax##SUF(t, (T) 0.0); break; } \
    }

ORACLE_API int oracle_elementwise_activation_f32(int op, int64_t n, const float* X, float* Y, float alpha, float beta) {
    if (op < 7 || op > 9) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const float x = X[i];
        float y;
        ORACLE_ACTIVATION_BODY(float, f)
        Y[i] = y;
    }
    return 0;
}

ORACLE_API int oracle_elementwise_activation_f64(int op, int64_t n, const double* X, double* Y, double alpha, double beta) {
    if (op < 7 || op > 9) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const double x = X[i];
        double y;
        ORACLE_ACTIVATION_BODY(double, )
        Y[i] = y;
    }
    return 0;
}

/* DOT::BLAS as DotNode::expand writes it (dot_node.cpp:76-165): one sequential For over i with the tasklet
 * fp_fma, res = x[i * incx] * y[i * incy] + res, printed "a * b + c" (cpp_language_extension.cpp:207-208) -
 * started from zero, as cblas_?dot, which the node's BLAS dispatcher prints, returns the plain sum. */
ORACLE_API float oracle_dot_f32(int64_t n, const float* x, int64_t incx, const float* y, int64_t incy) {
    float res = 0.0f;
    for (int64_t i = 0; i < n; i++) res = x[i * incx] * y[i * incy] + res;
    return res;
}

ORACLE_API double oracle_dot_f64(int64_t n, const double* x, int64_t incx, const double* y, int64_t incy) {
    double res = 0.0;
    for (int64_t i = 0; i < n; i++) res = x[i * incx] * y[i * incy] + res;
    return res;
}

ORACLE_API int oracle_elementwise_binary_f32(int op, int64_t n, const float* A, const float* B, float* Y) {
    if (op < 0 || op > 6) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const float a = A[i], b = B[i];
        float y;
        ORACLE_BINARY_BODY(float, f)
        Y[i] = y;
    }
    return 0;
}

ORACLE_API int oracle_elementwise_binary_f64(int op, int64_t n, const double* A, const double* B, double* Y) {
    if (op < 0 || op > 6) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const double a = A[i], b = B[i];
        double y;
        ORACLE_BINARY_BODY(double, )
        Y[i] = y;
    }
    return 0;
}

/* ml::Broadcast (sdfg/include/sdfg/data_flow/library_nodes/math/tensor/broadcast_node.h:13-43): the
 * output of shape out_shape reads the input at the same coordinates, with coordinate 0 along every
 * dimension whose input extent is 1. `esize` bytes per element, equal ranks. */
ORACLE_API int oracle_broadcast(int esize, int rank, const int64_t* in_shape, const int64_t* out_shape, const void* X, void* Y) {
    if (rank < 1 || rank > 8) return 1;
    int64_t in_stride[8], n = 1, stride = 1;
    for (int d = rank - 1; d >= 0; d--) {
        if (in_shape[d] != out_shape[d] && in_shape[d] != 1) return 2;
        in_stride[d] = in_shape[d] == 1 ? 0 : stride;
        stride *= in_shape[d];
        n *= out_shape[d];
    }
    const char* x = (const char*) X;
    char* y = (char*) Y;
#pragma omp parallel for schedule(static)
    for (int64_t o = 0; o < n; o++) {
        int64_t rem = o, off = 0;
        for (int d = rank - 1; d >= 0; d--) {
            off += (rem % out_shape[d]) * in_stride[d];
            rem /= out_shape[d];
        }
        memcpy(y + o * esize, x + off * esize, (size_t) esize);
    }
    return 0;
}

/* Reduce nodes ml::Sum / ml::Max / ml::Min / ml::Mean over a block of adjacent axes, X seen as
 * [outer, reduce, inner]. Restates ReduceNode::expand (reduce_node.cpp:188-333): Y is first set to the
 * identity (sum_node.cpp:20-57 "0", max_node.cpp:56-67 "-INFINITY", min_node.cpp "INFINITY"), then
 * accumulated through memory along the reduced extent, left to right: Y = X + Y, Y = fmax(X, Y)
 * (max_node.cpp:73-91), Y = fmin(X, Y). Mean is the Sum node followed by a Div by the number of reduced
 * elements (mean_node.cpp). op: 0 sum, 1 max, 2 min, 3 mean. */
#define ORACLE_REDUCE(NAME, T, FMAX, FMIN, NEG_INF, POS_INF)                                                  \
    ORACLE_API int NAME(int op, int64_t outer, int64_t reduce, int64_t inner, const T* X, T* Y) {              \
        if (op < 0 || op > 3) return 1;                                                                       \
        if (op == 3 && reduce == 0) return 2;                                                                 \
        _Pragma("omp parallel for schedule(static)") for (int64_t o = 0; o < outer; o++) {                    \
            for (int64_t i = 0; i < inner; i++) Y[o * inner + i] = op == 1 ? NEG_INF : op == 2 ? POS_INF : (T) 0; \
            for (int64_t r = 0; r < reduce; r++)                                                              \
                for (int64_t i = 0; i < inner; i++) {                                                         \
                    const T x = X[(o * reduce + r) * inner + i];                                              \
                    T* y = &Y[o * inner + i];                                                                 \
                    *y = op == 1 ? FMAX(x, *y) : op == 2 ? FMIN(x, *y) : x + *y;                              \
                }                                                                                             \
            if (op == 3)                                                                                      \
                for (int64_t i = 0; i < inner; i++) Y[o * inner + i] = Y[o * inner + i] / (T) reduce;         \
        }                                                                                                     \
        return 0;                                                                                             \
    }
ORACLE_REDUCE(oracle_reduce_f32, float, fmaxf, fminf, -INFINITY, INFINITY)
ORACLE_REDUCE(oracle_reduce_f64, double, fmax, fmin, -INFINITY, INFINITY)


/* ------------------------------------------------------------- Transpose */

/*
 * TransposeNode::expand (sdfg/src/data_flow/library_nodes/math/tensor/transpose_node.cpp:97-176):
 * one Map per input axis around an assign tasklet, Y[i_perm[0], i_perm[1], ...] = X[i_0, i_1, ...]
 * with Y's shape[i] = shape[perm[i]]. The node moves elements of any type (integers included,
 * transpose_node.h:47), hence bytes here. Returns 0, or 1 for a rank above 8 or an invalid perm.
 */
ORACLE_API int oracle_transpose(int element_bytes, int rank, const int64_t* shape, const int64_t* perm, const void* X, void* Y) {
    if (rank < 0 || rank > 8 || element_bytes <= 0) return 1;
    int64_t out_shape[8], out_stride[8], n = 1;
    int seen[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < rank; i++) {
        if (perm[i] < 0 || perm[i] >= rank || seen[perm[i]]) return 1;
        seen[perm[i]] = 1;
        out_shape[i] = shape[perm[i]];
        n *= shape[i];
    }
    int64_t s = 1;
    for (int i = rank - 1; i >= 0; i--) {
        out_stride[i] = s;
        s *= out_shape[i];
    }
    /* stride in Y of a step along input axis a: a sits at output position p with perm[p] == a */
    int64_t y_stride_of_input_axis[8];
    for (int p = 0; p < rank; p++) y_stride_of_input_axis[perm[p]] = out_stride[p];
    const char* x = (const char*) X;
    char* y = (char*) Y;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        int64_t rem = i, off = 0;
        for (int a = rank - 1; a >= 0; a--) {
            off += (rem % shape[a]) * y_stride_of_input_axis[a];
            rem /= shape[a];
        }
        memcpy(y + off * element_bytes, x + i * element_bytes, (size_t) element_bytes);
    }
    return 0;
}


/* ------------------------------------------------------- Map nests (tasklet bodies) */

/*
 * A perfect nest of Maps whose body is a chain of tasklets and CMath calls, as the reference's openmp target prints
 * it: the outermost Map becomes `#pragma omp parallel for schedule(static)` (opt/src/targets/omp/codegen/
 * omp_map_dispatcher.cpp:46-82), the inner ones plain `for` loops, and every tasklet a statement of its own
 *     <type> _out = <expression over the input connectors>;
 * (sdfg/src/codegen/dispatchers/block_dispatcher.cpp:219-331 with the expressions of
 * sdfg/src/codegen/language_extensions/cpp_language_extension.cpp:186-239), so every operation rounds by itself to the
 * type of its result; only fp_fma, printed as `a * b + c` in one expression, is contracted by the compiler into one
 * fused multiply-add. CMath nodes print the libm call of their stem, with the `f` suffix for float
 * (sdfg/src/data_flow/library_nodes/math/cmath/cmath_node.cpp).
 *
 * The body is handed over as a small program. Value slots: first the `n_reads` tensor elements loaded by the
 * iteration, then the `n_consts` constants (scalar operands and literals), then one slot per statement.
 *   read r:   element type (`read_f64[r]`), base pointer, one stride in elements per loop (read_strides[r * depth + l])
 *   statement s: operation name, result type (`stmt_f64[s]`), up to three argument slots (stmt_args[3 * s + k], -1: none)
 *   write w:  the slot stored, element type, base pointer, strides
 * Returns 0, or 1 for a depth outside 1..8, an unknown operation or a bad slot.
 */
enum oracle_map_op {
    MAP_ASSIGN, MAP_NEG, MAP_ADD, MAP_SUB, MAP_MUL, MAP_DIV, MAP_REM, MAP_FMA,
    MAP_SIN, MAP_COS, MAP_TAN, MAP_ASIN, MAP_ACOS, MAP_ATAN, MAP_ATAN2, MAP_SINH, MAP_COSH, MAP_TANH, MAP_ASINH, MAP_ACOSH, MAP_ATANH,
    MAP_EXP, MAP_EXP2, MAP_EXP10, MAP_EXPM1, MAP_LOG, MAP_LOG10, MAP_LOG2, MAP_LOG1P, MAP_POW, MAP_SQRT, MAP_CBRT, MAP_HYPOT,
    MAP_ERF, MAP_ERFC, MAP_TGAMMA, MAP_LGAMMA, MAP_FABS, MAP_CEIL, MAP_FLOOR, MAP_TRUNC, MAP_ROUND, MAP_NEARBYINT, MAP_RINT,
    MAP_FMOD, MAP_REMAINDER, MAP_COPYSIGN, MAP_FMAX, MAP_FMIN, MAP_FDIM, MAP_OP_COUNT
};
static const char* const oracle_map_op_names[MAP_OP_COUNT] = {
    "assign", "fp_neg", "fp_add", "fp_sub", "fp_mul", "fp_div", "fp_rem", "fp_fma",
    "sin", "cos", "tan", "asin", "acos", "atan", "atan2", "sinh", "cosh", "tanh", "asinh", "acosh", "atanh",
    "exp", "exp2", "exp10", "expm1", "log", "log10", "log2", "log1p", "pow", "sqrt", "cbrt", "hypot",
    "erf", "erfc", "tgamma", "lgamma", "fabs", "ceil", "floor", "trunc", "round", "nearbyint", "rint",
    "fmod", "remainder", "copysign", "fmax", "fmin", "fdim"};

static float oracle_map_eval_f32(int op, float a, float b, float c) {
    switch (op) {
        case MAP_ASSIGN: return a;
        case MAP_NEG: return -a;
        case MAP_ADD: { volatile float r = a + b; return r; }
        case MAP_SUB: { volatile float r = a - b; return r; }
        case MAP_MUL: { volatile float r = a * b; return r; }
        case MAP_DIV: return a / b;
        case MAP_REM: case MAP_FMOD: return fmodf(a, b);
        case MAP_FMA: return fmaf(a, b, c);
        case MAP_SIN: return sinf(a); case MAP_COS: return cosf(a); case MAP_TAN: return tanf(a);
        case MAP_ASIN: return asinf(a); case MAP_ACOS: return acosf(a); case MAP_ATAN: return atanf(a);
        case MAP_ATAN2: return atan2f(a, b);
        case MAP_SINH: return sinhf(a); case MAP_COSH: return coshf(a); case MAP_TANH: return tanhf(a);
        case MAP_ASINH: return asinhf(a); case MAP_ACOSH: return acoshf(a); case MAP_ATANH: return atanhf(a);
        case MAP_EXP: return expf(a); case MAP_EXP2: return exp2f(a); case MAP_EXP10: return powf(10.0f, a);
        case MAP_EXPM1: return expm1f(a); case MAP_LOG: return logf(a); case MAP_LOG10: return log10f(a);
        case MAP_LOG2: return log2f(a); case MAP_LOG1P: return log1pf(a); case MAP_POW: return powf(a, b);
        case MAP_SQRT: return sqrtf(a); case MAP_CBRT: return cbrtf(a); case MAP_HYPOT: return hypotf(a, b);
        case MAP_ERF: return erff(a); case MAP_ERFC: return erfcf(a); case MAP_TGAMMA: return tgammaf(a);
        case MAP_LGAMMA: return lgammaf(a); case MAP_FABS: return fabsf(a); case MAP_CEIL: return ceilf(a);
        case MAP_FLOOR: return floorf(a); case MAP_TRUNC: return truncf(a); case MAP_ROUND: return roundf(a);
        case MAP_NEARBYINT: return nearbyintf(a); case MAP_RINT: return rintf(a);
        case MAP_REMAINDER: return remainderf(a, b); case MAP_COPYSIGN: return copysignf(a, b);
        case MAP_FMAX: return fmaxf(a, b); case MAP_FMIN: return fminf(a, b); case MAP_FDIM: return fdimf(a, b);
    }
    return NAN;
}

static double oracle_map_eval_f64(int op, double a, double b, double c) {
    switch (op) {
        case MAP_ASSIGN: return a;
        case MAP_NEG: return -a;
        case MAP_ADD: { volatile double r = a + b; return r; }
        case MAP_SUB: { volatile double r = a - b; return r; }
        case MAP_MUL: { volatile double r = a * b; return r; }
        case MAP_DIV: return a / b;
        case MAP_REM: case MAP_FMOD: return fmod(a, b);
        case MAP_FMA: return fma(a, b, c);
        case MAP_SIN: return sin(a); case MAP_COS: return cos(a); case MAP_TAN: return tan(a);
        case MAP_ASIN: return asin(a); case MAP_ACOS: return acos(a); case MAP_ATAN: return atan(a);
        case MAP_ATAN2: return atan2(a, b);
        case MAP_SINH: return sinh(a); case MAP_COSH: return cosh(a); case MAP_TANH: return tanh(a);
        case MAP_ASINH: return asinh(a); case MAP_ACOSH: return acosh(a); case MAP_ATANH: return atanh(a);
        case MAP_EXP: return exp(a); case MAP_EXP2: return exp2(a); case MAP_EXP10: return pow(10.0, a);
        case MAP_EXPM1: return expm1(a); case MAP_LOG: return log(a); case MAP_LOG10: return log10(a);
        case MAP_LOG2: return log2(a); case MAP_LOG1P: return log1p(a); case MAP_POW: return pow(a, b);
        case MAP_SQRT: return sqrt(a); case MAP_CBRT: return cbrt(a); case MAP_HYPOT: return hypot(a, b);
        case MAP_ERF: return erf(a); case MAP_ERFC: return erfc(a); case MAP_TGAMMA: return tgamma(a);
        case MAP_LGAMMA: return lgamma(a); case MAP_FABS: return fabs(a); case MAP_CEIL: return ceil(a);
        case MAP_FLOOR: return floor(a); case MAP_TRUNC: return trunc(a); case MAP_ROUND: return round(a);
        case MAP_NEARBYINT: return nearbyint(a); case MAP_RINT: return rint(a);
        case MAP_REMAINDER: return remainder(a, b); case MAP_COPYSIGN: return copysign(a, b);
        case MAP_FMAX: return fmax(a, b); case MAP_FMIN: return fmin(a, b); case MAP_FDIM: return fdim(a, b);
    }
    return NAN;
}

ORACLE_API int oracle_map_nest(int depth, const int64_t* bounds,
                               int n_reads, const void* const* read_ptrs, const int64_t* read_strides, const int* read_f64,
                               int n_consts, const double* consts,
                               int n_stmts, const char* const* stmt_ops, const int* stmt_f64, const int* stmt_args,
                               int n_writes, void* const* write_ptrs, const int64_t* write_strides, const int* write_f64, const int* write_slots) {
    enum { MAX_SLOTS = 256 };
    if (depth < 1 || depth > 8 || n_reads < 0 || n_consts < 0 || n_stmts < 0 || n_writes < 1) return 1;
    const int n_slots = n_reads + n_consts + n_stmts;
    if (n_slots > MAX_SLOTS) return 1;
    int ops[MAX_SLOTS];
    for (int s = 0; s < n_stmts; s++) {
        ops[s] = -1;
        for (int k = 0; k < MAP_OP_COUNT; k++)
            if (strcmp(stmt_ops[s], oracle_map_op_names[k]) == 0) ops[s] = k;
        if (strcmp(stmt_ops[s], "fma") == 0) ops[s] = MAP_FMA;
        if (ops[s] < 0) return 1;
        for (int k = 0; k < 3; k++)
            if (stmt_args[3 * s + k] >= n_reads + n_consts + s) return 1;   /* only values computed before */
    }
    for (int w = 0; w < n_writes; w++)
        if (write_slots[w] < 0 || write_slots[w] >= n_slots) return 1;
    int64_t inner = 1;
    for (int l = 1; l < depth; l++) inner *= bounds[l];
#pragma omp parallel for schedule(static)
    for (int64_t i0 = 0; i0 < bounds[0]; i0++) {
        double slot[MAX_SLOTS];
        for (int c = 0; c < n_consts; c++) slot[n_reads + c] = consts[c];
        for (int64_t rest = 0; rest < inner; rest++) {
            int64_t idx[8];
            idx[0] = i0;
            int64_t rem = rest;
            for (int l = depth - 1; l >= 1; l--) {
                idx[l] = rem % bounds[l];
                rem /= bounds[l];
            }
            for (int r = 0; r < n_reads; r++) {
                int64_t off = 0;
                for (int l = 0; l < depth; l++) off += idx[l] * read_strides[r * depth + l];
                slot[r] = read_f64[r] ? ((const double*) read_ptrs[r])[off] : (double) ((const float*) read_ptrs[r])[off];
            }
            for (int s = 0; s < n_stmts; s++) {
                const int* a = stmt_args + 3 * s;
                const double x = a[0] >= 0 ? slot[a[0]] : 0.0, y = a[1] >= 0 ? slot[a[1]] : 0.0, z = a[2] >= 0 ? slot[a[2]] : 0.0;
                /* the inputs are converted to the type of the statement, then the operation rounds once */
                slot[n_reads + n_consts + s] = stmt_f64[s] ? oracle_map_eval_f64(ops[s], x, y, z)
                                                           : (double) oracle_map_eval_f32(ops[s], (float) x, (float) y, (float) z);
            }
            for (int w = 0; w < n_writes; w++) {
                int64_t off = 0;
                for (int l = 0; l < depth; l++) off += idx[l] * write_strides[w * depth + l];
                if (write_f64[w]) ((double*) write_ptrs[w])[off] = slot[write_slots[w]];
                else ((float*) write_ptrs[w])[off] = (float) slot[write_slots[w]];
            }
        }
    }
    return 0;
}
