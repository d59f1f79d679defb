// Launcher for ml::Attention (see include/docc_rocm_ops.h).
#include <cmath>
#include <cstdio>
#include <cstdlib>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace {

int attention_fused(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D, float scale, const uint16_t* Q,
                    const uint16_t* K, const uint16_t* V, void* O, int out_bf16, bool causal) {
    if (B < 0 || H < 0 || SQ < 0 || SKV < 0 || D < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: negative shape");
    if (D != 32 && D != 64 && D != 128)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "attention: head dim %lld (32, 64 and 128 are built; docc_rocm_attention_bf16_ws takes any)", (long long) D);
    if (B == 0 || H == 0 || SQ == 0) return 0;
    if (SKV == 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: no keys (softmax over an empty axis)");
    if (!Q || !K || !V || !O) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: null pointer");
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: scale must be positive and finite");
    if ((((uintptr_t) Q | (uintptr_t) K | (uintptr_t) V | (uintptr_t) O) % 16) != 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: pointers must be 16-byte aligned");
    if (SQ > 0x7fffffffLL - 128 || SKV > 0x7fffffffLL - 64) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "attention: sequences must be < 2^31");
    int rc = ensure_device();
    if (rc) return rc;
    // LDS: ring of 3 stages x (K block [64][D] + V block [64][D]) bf16
    const uint32_t lds = 3 * (2 * 64 * (uint32_t) D) * 2;
    const float scale_log2e = scale * 1.4426950408889634f;
    // Two forms: 256 queries per work-group (a wavefront takes 64, so each K/V operand read from LDS serves two
    // MFMAs: fewer instructions per flop) once that still gives every CU its two resident work-groups, else 128
    // per work-group (more, smaller work-groups). DOCC_ROCM_ATTENTION_Q=128|256 forces one (tuning and tests).
    const int64_t BH = B * H, out_bytes = out_bf16 ? 2 : 4;
    // ... and only where the larger groups do not add padded queries: a wavefront multiplies its 64 queries whether they
    // exist or not (SQ = 100 would run 256 queries in the large form and 128 in the small one)
    const bool no_extra_padding = (SQ + 255) / 256 * 256 <= (SQ + 127) / 128 * 128 || SQ >= 1024;
    int per_group = ((SQ + 255) / 256) * BH >= 2 * compute_units() && no_extra_padding ? 256 : 128;
    if (const char* force = std::getenv("DOCC_ROCM_ATTENTION_Q")) {
        const int v = std::atoi(force);
        if (v == 128 || v == 256) per_group = v;
    }
    // head dim 128: the large form is eight wavefronts of 32 queries (one work-group per CU), the small one four
    if (D == 128 && !std::getenv("DOCC_ROCM_ATTENTION_Q")) per_group = ((SQ + 255) / 256) * BH >= compute_units() && no_extra_padding ? 256 : 128;
    char kernel[64];
    std::snprintf(kernel, sizeof(kernel), "docc_attention_bf16_d%d_q%d_%s%s", (int) D, per_group, out_bf16 ? "bf16out" : "f32out",
                  causal ? "_causal" : "");
    const uint32_t threads = D == 128 && per_group == 256 ? 512 : 256;
    // gridDim.y numbers the (batch, head) pairs: at most 65535 per launch
    for (int64_t h0 = 0; h0 < BH; h0 += 65535) {
        const int64_t nh = BH - h0 < 65535 ? BH - h0 : 65535;
        // causal: a work-group takes a pair of query blocks (the longest and the shortest left), see the kernel
        const int64_t query_blocks = (SQ + per_group - 1) / per_group;
        rc = launch(kernel, (uint32_t) (causal ? (query_blocks + 1) / 2 : query_blocks), (uint32_t) nh, 1, threads, lds, (hipStream_t) stream,
                    Q + h0 * SQ * D, K + h0 * SKV * D, V + h0 * SKV * D, (void*) ((char*) O + h0 * SQ * D * out_bytes), (int) SQ,
                    (int) SKV, scale_log2e);
        if (rc) return rc;
    }
    return 0;
}

} // namespace

extern "C" int docc_rocm_attention_bf16(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV,
                                        int64_t D, float scale, const uint16_t* Q, const uint16_t* K,
                                        const uint16_t* V, void* O, int out_bf16) {
    return attention_fused(stream, B, H, SQ, SKV, D, scale, Q, K, V, O, out_bf16, false);
}

// ---- any head dimension, through a caller-provided workspace -----------------------------------

namespace {

bool fused_head_dim(int64_t D) { return D == 32 || D == 64 || D == 128; }

// the head dimension of the fused kernel that a smaller one is widened to (zero columns change neither the scores
// nor the first D columns of the result); 0: none, the separate kernels run
int64_t widened_head_dim(int64_t D) { return D < 32 ? 32 : D < 64 ? 64 : D < 128 ? 128 : 0; }

// bytes of the widened Q, K, V and result per (batch, head) pair
int64_t widened_bytes_per_head(int64_t SQ, int64_t SKV, int64_t Dp, int out_bf16) {
    return (SQ + 2 * SKV) * Dp * 2 + SQ * Dp * (out_bf16 ? 2 : 4);   // Dp is a multiple of 32: every part stays 64-byte aligned
}

// bytes of scores (fp32) + probabilities (bf16) + an fp32 result per (batch, head) pair
int64_t attention_bytes_per_head(int64_t SQ, int64_t SKV, int64_t D, int out_bf16) {
    const int64_t scores = (SQ * SKV * 4 + 255) / 256 * 256, probs = (SQ * SKV * 2 + 255) / 256 * 256;
    const int64_t out32 = out_bf16 ? (SQ * D * 4 + 255) / 256 * 256 : 0;
    return scores + probs + out32;
}

constexpr int64_t kAttentionWorkspaceCap = int64_t(2) << 30;   // heads are processed in chunks that fit this

int64_t attention_heads_per_chunk(int64_t BH, int64_t per_head) {
    int64_t n = per_head > 0 ? kAttentionWorkspaceCap / per_head : BH;
    if (n < 1) n = 1;
    return n < BH ? n : BH;
}

} // namespace

extern "C" int64_t docc_rocm_attention_bf16_workspace_bytes(int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D, int out_bf16) {
    if (B <= 0 || H <= 0 || SQ <= 0 || SKV <= 0 || D <= 0) return 0;
    if (fused_head_dim(D)) return 0;   // the fused kernel keeps scores and probabilities in registers
    const int64_t per_head = widened_head_dim(D) ? widened_bytes_per_head(SQ, SKV, widened_head_dim(D), out_bf16)
                                                 : attention_bytes_per_head(SQ, SKV, D, out_bf16);
    return attention_heads_per_chunk(B * H, per_head) * per_head;
}

static int attention_any_head_dim(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D, float scale,
                                  const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O, int out_bf16, void* workspace,
                                  int64_t workspace_bytes, bool causal) {
    if (fused_head_dim(D)) return attention_fused(stream, B, H, SQ, SKV, D, scale, Q, K, V, O, out_bf16, causal);
    if (causal && !widened_head_dim(D))
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "attention: the causal form is built for head dims up to 128 (head dim %lld)", (long long) D);
    if (B < 0 || H < 0 || SQ < 0 || SKV < 0 || D < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: negative shape");
    if (B == 0 || H == 0 || SQ == 0) return 0;
    if (SKV == 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: no keys (softmax over an empty axis)");
    if (D == 0) return 0;
    if (!Q || !K || !V || !O) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: null pointer");
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: scale must be positive and finite");
    const int64_t need = docc_rocm_attention_bf16_workspace_bytes(B, H, SQ, SKV, D, out_bf16);
    if (!workspace || workspace_bytes < need || ((uintptr_t) workspace % 256) != 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: head dim %lld needs a 256-byte aligned workspace of %lld bytes",
                    (long long) D, (long long) need);
    if (const int64_t Dp = widened_head_dim(D)) {
        // a head dimension below 128 that is not built: the operands are widened with zero columns to the next one
        // that is, the fused kernel runs on them, and the first D columns of its result are the answer
        if (((uintptr_t) Q | (uintptr_t) K | (uintptr_t) V) % 2 != 0 || (uintptr_t) O % (out_bf16 ? 2 : 4) != 0)
            return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: misaligned pointer");
        if (int rc = ensure_device()) return rc;
        const int64_t BH = B * H, per_head = widened_bytes_per_head(SQ, SKV, Dp, out_bf16);
        const int64_t chunk = attention_heads_per_chunk(BH, per_head);
        hipStream_t s = (hipStream_t) stream;
        auto grid = [](int64_t items) { return (uint32_t) (items < 256 * 4096 ? (items + 255) / 256 : 4096); };
        for (int64_t h0 = 0; h0 < BH; h0 += chunk) {
            const int64_t nh = BH - h0 < chunk ? BH - h0 : chunk;
            uint16_t* Qp = (uint16_t*) workspace;
            uint16_t* Kp = Qp + nh * SQ * Dp;
            uint16_t* Vp = Kp + nh * SKV * Dp;
            void* Op = (void*) (Vp + nh * SKV * Dp);
            const struct { const uint16_t* from; uint16_t* to; int64_t rows; } parts[3] = {
                {Q + h0 * SQ * D, Qp, nh * SQ}, {K + h0 * SKV * D, Kp, nh * SKV}, {V + h0 * SKV * D, Vp, nh * SKV}};
            for (const auto& part : parts)
                if (int rc = launch("docc_pad_rows_b16", grid(part.rows * (Dp / 8)), 1, 1, 256, 0, s, part.from, part.to, (long) part.rows, (int) D, (int) Dp))
                    return rc;
            if (int rc = attention_fused(stream, 1, nh, SQ, SKV, Dp, scale, Qp, Kp, Vp, Op, out_bf16, causal)) return rc;
            const int64_t rows = nh * SQ;
            int rc = out_bf16 ? launch("docc_unpad_rows_b16", grid(rows * D), 1, 1, 256, 0, s, (const uint16_t*) Op, (uint16_t*) O + h0 * SQ * D, (long) rows,
                                       (int) D, (int) Dp)
                              : launch("docc_unpad_rows_b32", grid(rows * D), 1, 1, 256, 0, s, (const uint32_t*) Op, (uint32_t*) O + h0 * SQ * D, (long) rows,
                                       (int) D, (int) Dp);
            if (rc) return rc;
        }
        return 0;
    }
    // S = scale * Q K^T (batched bf16 GEMM, fp32 out), P = softmax rows of S, rounded to bf16, O = P V
    const int64_t BH = B * H, per_head = attention_bytes_per_head(SQ, SKV, D, out_bf16);
    const int64_t chunk = attention_heads_per_chunk(BH, per_head);
    const int64_t scores_bytes = (SQ * SKV * 4 + 255) / 256 * 256, probs_bytes = (SQ * SKV * 2 + 255) / 256 * 256;
    char* ws = (char*) workspace;
    float* S = (float*) ws;
    uint16_t* P = (uint16_t*) (ws + chunk * scores_bytes);
    float* O32 = (float*) (ws + chunk * (scores_bytes + probs_bytes));
    // inside the chunk the matrices are packed (strides in elements, not the rounded byte sizes)
    for (int64_t h0 = 0; h0 < BH; h0 += chunk) {
        const int64_t nh = BH - h0 < chunk ? BH - h0 : chunk;
        int rc = docc_rocm_bf16gemm_f32_batched(stream, DOCC_ROCM_NO_TRANS, DOCC_ROCM_TRANS, SQ, SKV, D, scale, Q + h0 * SQ * D, D,
                                                SQ * D, K + h0 * SKV * D, D, SKV * D, 0.f, S, SKV, SQ * SKV, nh);
        if (rc) return rc;
        rc = docc_rocm_softmax_f32(stream, nh * SQ, SKV, S, S);
        if (rc) return rc;
        rc = docc_rocm_convert_f32_to_bf16(stream, nh * SQ * SKV, S, P);
        if (rc) return rc;
        float* out = out_bf16 ? O32 : (float*) O + h0 * SQ * D;
        rc = docc_rocm_bf16gemm_f32_batched(stream, DOCC_ROCM_NO_TRANS, DOCC_ROCM_NO_TRANS, SQ, D, SKV, 1.f, P, SKV, SQ * SKV,
                                            V + h0 * SKV * D, D, SKV * D, 0.f, out, D, SQ * D, nh);
        if (rc) return rc;
        if (out_bf16) {
            rc = docc_rocm_convert_f32_to_bf16(stream, nh * SQ * D, O32, (uint16_t*) O + h0 * SQ * D);
            if (rc) return rc;
        }
    }
    return 0;
}

extern "C" int docc_rocm_attention_bf16_ws(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D,
                                           float scale, const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O,
                                           int out_bf16, void* workspace, int64_t workspace_bytes) {
    return attention_any_head_dim(stream, B, H, SQ, SKV, D, scale, Q, K, V, O, out_bf16, workspace, workspace_bytes, false);
}

// Query i attends to the keys j <= i (torch's is_causal: the mask is aligned at the top left). Head dims up to 128; the
// workspace is the one of docc_rocm_attention_bf16_workspace_bytes (none for 32, 64 and 128).
extern "C" int docc_rocm_attention_bf16_causal(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV, int64_t D,
                                               float scale, const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O,
                                               int out_bf16, void* workspace, int64_t workspace_bytes) {
    return attention_any_head_dim(stream, B, H, SQ, SKV, D, scale, Q, K, V, O, out_bf16, workspace, workspace_bytes, true);
}
