/*
 * docc_rocm_ops.h - C-ABI launchers of the math library-node kernels of the
 * docc `rocm` target (GEMM, Softmax, Conv, Attention) on gfx950.
 *
 * These are the calls the rocm library-node dispatchers print into generated
 * host C++, in the place where the reference's dispatchers print
 * `cblas_dgemm(...)` (sdfg/src/data_flow/library_nodes/math/blas/gemm_node.cpp:449-509)
 * or `cublasDgemm(...)` (opt/src/targets/cuda/blas/gemm.cpp:131-185), and
 * where the reference expands Softmax and Conv into host loop nests
 * (sdfg/src/data_flow/library_nodes/math/tensor/reduce_ops/softmax_node.cpp:38-265,
 *  sdfg/src/data_flow/library_nodes/math/tensor/conv_node.cpp:85-454).
 *
 * All pointers are DEVICE pointers (the WithTransfers dispatchers copy
 * through docc_rocm_rt.h first). All matrices and tensors are dense,
 * row-major / C-order, as the reference's frontends produce them. Each call
 * enqueues its kernels on `stream` and returns without waiting. Return value:
 * 0, a hipError_t, or a negative DOCC_ROCM_ERR_* code; message in
 * docc_rocm_last_error().
 *
 * Library: libdocc_rt_rocm.so (same library as docc_rocm_rt.h).
 */
#ifndef DOCC_ROCM_OPS_H
#define DOCC_ROCM_OPS_H

#include <stddef.h>
#include <stdint.h>

#include "docc_rocm_rt.h"

#ifdef __cplusplus
extern "C" {
#endif

/* BLAS transpose codes as the reference's GEMMNode stores them
 * (sdfg/include/sdfg/data_flow/library_nodes/math/blas/blas_node.h:49-126). */
#define DOCC_ROCM_NO_TRANS 111
#define DOCC_ROCM_TRANS 112

/*
 * C[m,n] = alpha * op(A)[m,k] * op(B)[k,n] + beta * C[m,n], row-major, with
 * cblas semantics: when beta == 0, C is not read (it may hold NaNs); when alpha == 0,
 * A and B are not referenced (C = beta * C).
 * Replaces cblas_dgemm / cblas_sgemm as printed by GEMMNodeDispatcher_BLAS
 * (reference gemm_node.cpp:474-505) and cublasDgemm / cublasSgemm
 * (reference opt/src/targets/cuda/blas/gemm.cpp:131-185).
 * Zero-sized m, n: nothing is done; k == 0: C = beta * C. Products with one output
 * column or row (bf16 ones too) run as matrix-vector kernels (HBM-bound); their partial sums may pass through
 * 8 MiB of device memory that the library keeps per stream (see docc_rocm_softmax). So may the products of a
 * few rows or few output tiles with a long K extent, which are computed in parts of K and added in a fixed order
 * (the result does not depend on scheduling); parts beyond 8 MiB take a block of the device block cache for the
 * call, in stream order (up to 64 MiB).
 */
int docc_rocm_dgemm(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                    double alpha, const double* A, int64_t lda, const double* B, int64_t ldb, double beta,
                    double* C, int64_t ldc);
int docc_rocm_sgemm(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                    float alpha, const float* A, int64_t lda, const float* B, int64_t ldb, float beta, float* C,
                    int64_t ldc);

/*
 * bf16 inputs (raw bits, uint16_t, the type that crosses the reference's
 * ctypes boundary for BFloat: python/docc/compiler/compiled_sdfg.py:16-31),
 * fp32 accumulate and fp32 C. The reference's BLAS_Precision has no such
 * mode (blas_node.h:49-55); this is the rocm target's added precision.
 */
int docc_rocm_bf16gemm_f32(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                           float alpha, const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                           float beta, float* C, int64_t ldc);

/*
 * GEMM with the rest of a dense layer in its epilogue:
 *     C = act(alpha * op(A) op(B) + beta * C + bias[column])
 * `bias`: n values or NULL; `activation`: DOCC_ROCM_UNARY_RELU, DOCC_ROCM_UNARY_ABS (below) or -1
 * (the other unary operations are not built into the store: DOCC_ROCM_ERR_UNSUPPORTED). The sum is
 * rounded after each step, as the GEMM node followed by ml::Add (of the bias row, through
 * ml::Broadcast) and the unary node would round it; this is what the target's fusion pass emits
 * for that chain, so that C is written once instead of being re-read by every node. The
 * reference has no such form: its cuBLAS dispatcher calls plain gemm
 * (opt/src/targets/cuda/blas/gemm.cpp:66-96) and the epilogue stays a Map.
 */
int docc_rocm_dgemm_epilogue(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                             double alpha, const double* A, int64_t lda, const double* B, int64_t ldb, double beta,
                             double* C, int64_t ldc, const double* bias, int activation);
int docc_rocm_sgemm_epilogue(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                             float alpha, const float* A, int64_t lda, const float* B, int64_t ldb, float beta, float* C,
                             int64_t ldc, const float* bias, int activation);
int docc_rocm_bf16gemm_f32_epilogue(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                                    float alpha, const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                                    float beta, float* C, int64_t ldc, const float* bias, int activation);

/*
 * A batch of `batch` equally shaped products in one launch: entry z uses
 * A + z*stride_a, B + z*stride_b, C + z*stride_c (strides in elements; 0
 * shares an input across the batch, the C matrices must not overlap).
 * Replaces the loop of GEMM nodes that the reference's ml::MatMul expands
 * to, one per batch entry (sdfg/src/data_flow/library_nodes/math/tensor/
 * matmul_node.cpp:366-499); the reference's cuBLAS dispatcher has no batched
 * form (opt/src/targets/cuda/blas/gemm.cpp:66-96).
 */
int docc_rocm_dgemm_batched(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                            double alpha, const double* A, int64_t lda, int64_t stride_a, const double* B, int64_t ldb,
                            int64_t stride_b, double beta, double* C, int64_t ldc, int64_t stride_c, int64_t batch);
int docc_rocm_sgemm_batched(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                            float alpha, const float* A, int64_t lda, int64_t stride_a, const float* B, int64_t ldb,
                            int64_t stride_b, float beta, float* C, int64_t ldc, int64_t stride_c, int64_t batch);
int docc_rocm_bf16gemm_f32_batched(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                                   float alpha, const uint16_t* A, int64_t lda, int64_t stride_a, const uint16_t* B,
                                   int64_t ldb, int64_t stride_b, float beta, float* C, int64_t ldc, int64_t stride_c,
                                   int64_t batch);

/*
 * Y[r, :] = softmax(X[r, :]) for r in [0, rows), fp32, both [rows, cols]
 * contiguous. This is ml::Softmax over the last axis; any reduction over a
 * trailing contiguous axis of an N-d tensor is this call with
 * rows = product of the leading dims. Replaces the Max/Sub/Exp/Sum/Div
 * loop nests of SoftmaxNode::expand (reference softmax_node.cpp:142-252).
 * X == Y (in place) is allowed.
 */
int docc_rocm_softmax_f32(docc_rocm_stream_t stream, int64_t rows, int64_t cols, const float* X, float* Y);

/*
 * ml::Softmax in general: X and Y are contiguous and viewed as [outer, reduce, inner], the
 * softmax runs over the middle extent (a block of adjacent axes of the node; the product of
 * the axes before it is `outer`, of those after it `inner`); precision 32 (float) or 64
 * (double). The reference's node takes any axes and its element type from its memlets
 * (softmax_node.cpp:38-110). inner == 1 with precision 32 is docc_rocm_softmax_f32; the other
 * forms read X twice (running maximum and sum, then the results). With few columns and a long
 * reduced extent the rows are sliced over work-groups as well and the (maximum, sum) pairs of the
 * slices pass through 8 MiB of device memory that the library keeps per stream (allocated on the
 * first such call on a stream, kept until the process ends), so calls on different streams, and from
 * different threads, do not disturb each other.
 */
int docc_rocm_softmax(docc_rocm_stream_t stream, int precision, int64_t outer, int64_t reduce, int64_t inner,
                      const void* X, void* Y);

/*
 * The same with the partial results in memory of the caller: `workspace` is device memory, 256-byte
 * aligned, of at least docc_rocm_softmax_workspace_bytes(...) bytes (0 for the shapes that run as one
 * launch; at most 8 MiB); it may be reused as soon as the call's kernels have run. Same kernels and
 * launch geometry as docc_rocm_softmax, so the results are the same bits. Counterpart in the reference:
 * the temporaries SoftmaxNode::expand allocates around its loop nests (softmax_node.cpp:112-140).
 */
int64_t docc_rocm_softmax_workspace_bytes(int precision, int64_t outer, int64_t reduce, int64_t inner);
int docc_rocm_softmax_ws(docc_rocm_stream_t stream, int precision, int64_t outer, int64_t reduce, int64_t inner,
                         const void* X, void* Y, void* workspace, int64_t workspace_bytes);

/*
 * docc_rocm_softmax for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. No counterpart in the reference. The call itself allocates, loads and
 * looks up nothing: the partial results of the sliced form go through a fixed 1 MiB array of the library's own
 * device image, whose address and kernels are obtained when the device is set up, so docc_rocm_init(device)
 * must have returned before the first call (otherwise the call fails with a message that says so).
 * A shape whose partial results need more than the 1 MiB (docc_rocm_softmax_workspace_bytes(...) tells) is
 * refused with DOCC_ROCM_ERR_UNSUPPORTED and a message naming both numbers; every other shape gives the bits of
 * docc_rocm_softmax. All calls on a device share the array: it need not be cleared between calls (a call
 * writes what it reads back), but calls that overlap on one device - two streams, two threads - race.
 */
int docc_rocm_softmax_noalloc(docc_rocm_stream_t stream, int precision, int64_t outer, int64_t reduce, int64_t inner,
                              const void* X, void* Y);

/*
 * ml::Conv, 2-d, NCHW fp32, group 1 (reference conv_node.h:9-22,48-217):
 *   Y[n,oc,oh,ow] = bias[oc] + sum_{ic,kh,kw} X[n,ic,oh*sh-ph+kh*dh, ow*sw-pw+kw*dw] * W[oc,ic,kh,kw]
 * with zero padding (taps outside the image contribute 0); bias may be NULL.
 * Output size per the reference formula (conv_node.cpp:224-233):
 *   OH = (H + 2*pad_h - dil_h*(KH-1) - 1) / stride_h + 1   (same for W).
 */
int docc_rocm_conv2d_f32(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                         int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w,
                         int64_t dil_h, int64_t dil_w, const float* X, const float* Wt, const float* bias,
                         float* Y);

/*
 * The same node with device memory of the caller for a column matrix. Layers that the direct
 * kernels serve badly (small images with many channels, strides, large filters) run as an explicit
 * im2col followed by one GEMM  W[OC][C*KH*KW] x columns  over chunks of images that keep the
 * workspace under 2 GiB, and a Transpose of the result into [N][OC][OH*OW]; 1x1 stride-1 layers
 * without padding are a batched GEMM on the tensors as they lie and need no workspace. The
 * choice is made from the shape; _workspace_bytes returns 0 where a direct kernel is chosen.
 * `workspace`: 256-byte aligned, at least _workspace_bytes(...) bytes; with less (or NULL) the call
 * behaves like docc_rocm_conv2d_f32.
 */
int64_t docc_rocm_conv2d_f32_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                                             int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t dil_h,
                                             int64_t dil_w);
int docc_rocm_conv2d_f32_ws(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                            int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w,
                            int64_t dil_h, int64_t dil_w, const float* X, const float* Wt, const float* bias,
                            float* Y, void* workspace, int64_t workspace_bytes);

/*
 * The same node with the pads the reference's node carries: a begin and an end per spatial axis
 * (conv_node.cpp:76-77 `pads`: begins, then ends; :169-176 validation; :224-233 output extents)
 *   ih = oh*stride_h - pad_h + kh*dil_h,   OH = (H + pad_h + pad_h_end - dil_h*(KH-1) - 1) / stride_h + 1   (same for W).
 * `workspace` as for docc_rocm_conv2d_f32_ws (NULL: the direct kernels only).
 */
int64_t docc_rocm_conv2d_f32_pads_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                                                  int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w,
                                                  int64_t pad_h_end, int64_t pad_w_end, int64_t dil_h, int64_t dil_w);
int docc_rocm_conv2d_f32_pads(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                              int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w,
                              int64_t pad_h_end, int64_t pad_w_end, int64_t dil_h, int64_t dil_w, const float* X,
                              const float* Wt, const float* bias, float* Y, void* workspace, int64_t workspace_bytes);

/*
 * The node's `group` (reference conv_node.h / conv_node.cpp:27-40 constructor, :376-377 weights [OC][C / group][KH][KW],
 * :586 JSON field; ONNX Conv semantics: output channel oc belongs to group oc / (OC / group) and reads the C / group input
 * channels of that group). C and OC are the channels of the whole tensors; group must divide both. The direct kernels run
 * every group in one launch on that group's channels where they lie, a depthwise layer (group == C) on kernels of its own
 * (group == 1: docc_rocm_conv2d_f32_pads, `workspace` as there; it is not used for group > 1).
 */
int docc_rocm_conv2d_f32_grouped(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH,
                                 int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t pad_h_end,
                                 int64_t pad_w_end, int64_t dil_h, int64_t dil_w, int64_t group, const float* X, const float* Wt,
                                 const float* bias, float* Y, void* workspace, int64_t workspace_bytes);

/*
 * ml::Attention (a node the rocm target adds; the reference has none):
 *   O[b,h,i,:] = sum_j softmax_j(scale * <Q[b,h,i,:], K[b,h,j,:]>) * V[b,h,j,:]
 * Q [B,H,SQ,D], K and V [B,H,SKV,D], all contiguous bf16 (raw bits); fp32
 * scores, softmax and accumulation; every query attends to every key (docc_rocm_attention_bf16_causal below is the
 * causal form). O is [B,H,SQ,D], fp32 when
 * out_bf16 == 0 and bf16 (round-to-nearest-even) otherwise. D must be 32, 64 or 128
 * (docc_rocm_attention_bf16_ws takes any D).
 */
int docc_rocm_attention_bf16(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D,
                             float scale, const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O,
                             int out_bf16);

/*
 * The same node for any head dimension D, with device memory of the caller for the scores:
 * D == 32, 64 or 128 runs the kernel above and needs none; another D below 128 is widened with zero
 * columns to the next of these in the workspace (Q, K, V and the result), the kernel above runs on the
 * widened operands and the first D columns of its result are copied out; above 128 S = scale * Q K^T
 * (batched bf16 GEMM, fp32 out), a row softmax, the probabilities rounded to bf16 and O = P V run as
 * separate kernels. Either way over chunks of (batch, head) pairs that keep the workspace under 2 GiB.
 * `workspace` must be 256-byte aligned and hold what _workspace_bytes returns for the
 * same arguments (0 when no workspace is needed). Calls on one stream may share a workspace.
 */
int64_t docc_rocm_attention_bf16_workspace_bytes(int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D, int out_bf16);
int docc_rocm_attention_bf16_ws(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D,
                                float scale, const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O,
                                int out_bf16, void* workspace, int64_t workspace_bytes);

/*
 * The same with a causal mask: query i attends to the keys j <= i (torch's is_causal: the mask is aligned at the top left
 * whatever SQ and SKV are, so every query sees key 0). No counterpart in the reference (it has no attention node; a model
 * reaches it as F.scaled_dot_product_attention(..., is_causal=True) through the torch entry, mlir/docc/torch/__init__.py).
 * Head dims up to 128 (32, 64, 128 fused; others widened as in docc_rocm_attention_bf16_ws, with the workspace
 * docc_rocm_attention_bf16_workspace_bytes asks for); a work-group walks the key blocks up to its last query only.
 */
int docc_rocm_attention_bf16_causal(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D,
                                    float scale, const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O, int out_bf16,
                                    void* workspace, int64_t workspace_bytes);

/* fp32 -> bf16 (round to nearest even) and back, on the device; used by the
 * WithTransfers dispatchers when a node's inputs arrive as fp32. */
int docc_rocm_convert_f32_to_bf16(docc_rocm_stream_t stream, int64_t count, const float* src, uint16_t* dst);
int docc_rocm_convert_bf16_to_f32(docc_rocm_stream_t stream, int64_t count, const uint16_t* src, float* dst);

/* Plain device copy kernel of `bytes` bytes (multiple of 16): the known-size
 * kernel against which rocprof's FETCH_SIZE / WRITE_SIZE counters are
 * calibrated. */
int docc_rocm_copy_bytes(docc_rocm_stream_t stream, int64_t bytes, const void* src, void* dst);

/* Elementwise tensor nodes (reference sdfg/include/sdfg/data_flow/library_nodes/math/tensor/
 * elementwise_node.h: ElementWiseUnaryNode Y[i] = f(X[i]), ElementWiseBinaryNode
 * Y[i] = f(A[i], B[i]) over the linearised shape; replaces the Maps their expand()
 * emits). `precision` 32 (float) or 64 (double); `n` elements; in place (Y == X or
 * Y == A) is allowed. Operation codes: */
#define DOCC_ROCM_UNARY_ABS 0      /* ml::Abs      fabs        */
#define DOCC_ROCM_UNARY_EXP 1      /* ml::Exp      exp         */
#define DOCC_ROCM_UNARY_RELU 2     /* ml::ReLU     fmax(x, 0)  (elementwise_ops/relu_node.cpp:40-43) */
#define DOCC_ROCM_UNARY_SIGMOID 3  /* ml::Sigmoid  1/(1+exp(-x)) (sigmoid_node.cpp:46-70) */
#define DOCC_ROCM_UNARY_SQRT 4     /* ml::Sqrt     sqrt        */
#define DOCC_ROCM_UNARY_TANH 5     /* ml::Tanh     tanh        */
#define DOCC_ROCM_UNARY_ERF 6      /* ml::Erf      erf         */
#define DOCC_ROCM_UNARY_ELU 7          /* ml::Elu          x > 0 ? x : alpha * (exp(x) - 1)      (elu_node.cpp:21-97)          */
#define DOCC_ROCM_UNARY_LEAKY_RELU 8   /* ml::LeakyReLU    x >= 0 ? x : alpha * x                (leaky_relu_node.cpp:21-68)   */
#define DOCC_ROCM_UNARY_HARD_SIGMOID 9 /* ml::HardSigmoid  fmax(0, fmin(1, alpha * x + beta))    (hard_sigmoid_node.cpp:21-83) */
#define DOCC_ROCM_BINARY_ADD 0     /* ml::Add */
#define DOCC_ROCM_BINARY_SUB 1     /* ml::Sub */
#define DOCC_ROCM_BINARY_MUL 2     /* ml::Mul */
#define DOCC_ROCM_BINARY_DIV 3     /* ml::Div */
#define DOCC_ROCM_BINARY_MAXIMUM 4 /* ml::Maximum  fmax (maximum_node.cpp:64) */
#define DOCC_ROCM_BINARY_MINIMUM 5 /* ml::Minimum  fmin */
#define DOCC_ROCM_BINARY_POW 6     /* ml::Pow      pow(a, b) (pow_node.cpp:52-54) */
int docc_rocm_elementwise_unary(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* X, void* Y);
int docc_rocm_elementwise_binary(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* A, const void* B,
                                 void* Y);
/* The unary nodes with scalar operands on their "alpha" / "beta" connectors (codes 7..9 above; beta is read by
 * HardSigmoid only). The reference's expansions of these nodes are unfinished (no branch for positive inputs in
 * Elu, one-operand multiplies), so the operations are the ONNX operators of the same names; the order of the
 * steps the reference does spell out (exp, minus one, times alpha; fma, min with 1, max with 0) is kept. */
int docc_rocm_elementwise_activation(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* X, void* Y, double alpha,
                                     double beta);
/* ml::Fill (fill_node.cpp:29-41: an assign tasklet from a scalar under Maps over the output's shape): the `n`
 * elements of Y, of 1, 2, 4 or 8 bytes each, all become the element at `value` (host memory). */
int docc_rocm_fill(docc_rocm_stream_t stream, int element_bytes, int64_t n, const void* value, void* Y);
/* One operand is a scalar: the reference binds a constant or a scalar container to "A" or
 * "B" of the binary node (python/bindings/builder/py_structured_sdfg_builder.cpp:894-908).
 * Y[i] = f(A[i], scalar), or f(scalar, A[i]) when scalar_is_lhs != 0; the scalar is
 * rounded to float for precision 32. */
int docc_rocm_elementwise_binary_scalar(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* A, double scalar,
                                        int scalar_is_lhs, void* Y);

/* ml::Broadcast (reference .../tensor/broadcast_node.h:13-43): Y of shape out_shape is X
 * of shape in_shape repeated along every dimension where in_shape is 1 (numpy rules,
 * equal ranks, rank 1..6). Shapes are host arrays of `rank` extents. */
int docc_rocm_broadcast(docc_rocm_stream_t stream, int precision, int rank, const int64_t* in_shape, const int64_t* out_shape,
                        const void* X, void* Y);

/*
 * ml::Transpose: Y = X with its axes permuted, Y.shape[i] = shape[perm[i]] (the ONNX meaning the
 * reference's node has: transpose_node.h:14-60, JSON keys "shape" and "perm"); both contiguous,
 * rank <= 6, elements of 1, 2, 4 or 8 bytes (the node moves bits, integer types included), X and Y
 * distinct. Replaces the loop nest of TransposeNode::expand (transpose_node.cpp).
 */
int docc_rocm_transpose(docc_rocm_stream_t stream, int element_bytes, int rank, const int64_t* shape, const int64_t* perm,
                        const void* X, void* Y);

/*
 * ml::Cast: Y[i] = (D) X[i] for n contiguous elements, the conversion of an assign tasklet between
 * memlets of different types (reference elementwise_ops/cast_node.cpp:39-40, node keys "shape" and
 * "target_type"): round to nearest even between floating types, truncation towards zero to an
 * integer. Built: fp32 <-> fp64, bf16, fp16; int32 / int64 <-> fp32 / fp64; equal types copy.
 */
#define DOCC_ROCM_TYPE_F16 0
#define DOCC_ROCM_TYPE_BF16 1 /* raw 16-bit words */
#define DOCC_ROCM_TYPE_F32 2
#define DOCC_ROCM_TYPE_F64 3
#define DOCC_ROCM_TYPE_I32 4
#define DOCC_ROCM_TYPE_I64 5
int docc_rocm_cast(docc_rocm_stream_t stream, int src_type, int dst_type, int64_t n, const void* X, void* Y);

/* Reduce tensor nodes ml::Sum / ml::Max / ml::Min / ml::Mean over a block of adjacent axes
 * (reference sdfg/include/sdfg/data_flow/library_nodes/math/tensor/reduce_node.h and
 * reduce_ops/{sum,max,min,mean}_node.h; replaces the loop nests ReduceNode::expand emits,
 * reduce_node.cpp:188-333). X is seen as [outer, reduce, inner] (contiguous), Y as
 * [outer, inner]: Y[o, i] = op over r of X[o, r, i]; keepdims only changes the shape the caller
 * attaches to Y. Max / Min use fmax / fmin like the reference (a NaN is ignored unless the
 * whole extent is NaN); an empty extent gives the identity (0, -inf, +inf). A reduction with
 * inner > 1 and few output elements is sliced along the reduced extent; the slices' partial
 * results pass through 8 MiB of device memory that the library keeps per stream (see
 * docc_rocm_softmax): calls on different streams do not share it. */
#define DOCC_ROCM_REDUCE_SUM 0
#define DOCC_ROCM_REDUCE_MAX 1
#define DOCC_ROCM_REDUCE_MIN 2
#define DOCC_ROCM_REDUCE_MEAN 3
int docc_rocm_reduce(docc_rocm_stream_t stream, int op, int precision, int64_t outer, int64_t reduce, int64_t inner,
                     const void* X, void* Y);

/* A chain of elementwise nodes in one pass: Y = post_k(...post_1(f(A', B'))). A' and B' are
 * the operands repeated to `shape` by numpy's rules (`a_shape` / `b_shape`: `rank` extents, each
 * equal to the output's or 1), or the scalar `a_scalar` / `b_scalar` when the shape pointer is
 * NULL; `binary_op` is a DOCC_ROCM_BINARY_* code or -1 (the chain then starts from A' and B is
 * ignored); `post_ops` holds `n_post` (0..4) DOCC_ROCM_UNARY_* codes applied in order. This is
 * what the target's fusion pass emits for a Broadcast node folded into its consumer and unary
 * nodes folded into their producer (the reference reaches the same through MapFusion over the
 * expanded Maps, python/bindings/py_structured_sdfg.cpp:258-260). Each step rounds to the
 * element type as the separate nodes would. */
int docc_rocm_elementwise_fused(docc_rocm_stream_t stream, int precision, int rank, const int64_t* shape, int binary_op,
                                const int64_t* a_shape, const void* A, double a_scalar, const int64_t* b_shape, const void* B,
                                double b_scalar, int n_post, const int* post_ops, void* Y);

/* DOT::BLAS (reference dot_node.cpp:18-40 connectors __x, __y -> __out, :76-165 expansion; replaces cblas_?dot
 * of its BLAS dispatcher and cublas?dot of opt/src/targets/cuda/blas/dot.cpp:55-68): *result = sum_i
 * x[i * incx] * y[i * incy], precision 32 or 64, x and y in device memory, `result` in HOST memory; the call
 * returns when the value is there (it waits for the stream). Increments must not be negative. The sum is
 * split by n and the launch geometry alone: the same call gives the same bits. */
int docc_rocm_dot(docc_rocm_stream_t stream, int precision, int64_t n, const void* x, int64_t incx, const void* y, int64_t incy,
                  void* result);

/* Measurement aid, no counterpart in the reference: one wave watches the constant 100 MHz counter for
 * `microseconds` (1 .. 100000) and writes the shader clock it saw over that time, in MHz, to mhz[0] (device
 * memory). Launched on a stream of its own (docc_rocm_stream_create gives non-blocking ones) while a train of
 * kernels runs on another, it tells the clock the device sustains under those kernels - the figure that
 * separates "the pipe is idle" from "the power limit lowered the clock". */
int docc_rocm_clock_probe(docc_rocm_stream_t stream, int microseconds, float* mhz);

/* Measurement aid, no counterpart in the reference: `iters` rounds of 32 back-to-back
 * MFMAs per wave (precision 64: 16x16x4 fp64, 32: 32x32x2 fp32, 16: 32x32x16 bf16, 116: 16x16x32 bf16) on
 * every SIMD, `waves_per_simd` (1 or 2) waves each, operands taken from `operands`
 * (4096 floats on the device). `sink` receives 256 floats per work-group (CUs *
 * waves_per_simd groups); *flop (host, optional) the floating-point operations of
 * the launch. Timed with events it gives the matrix rate the power limit allows for
 * that operand data: the practical ceiling beside the nominal peak. */
int docc_rocm_mfma_probe(docc_rocm_stream_t stream, int precision, int waves_per_simd, int iters, const float* operands,
                         float* sink, double* flop);

#ifdef __cplusplus
}
#endif
#endif /* DOCC_ROCM_OPS_H */
