// Launcher for ml::Attention (see include/docc_rocm_ops.h).
#include <cmath>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

extern "C" int docc_rocm_attention_bf16(docc_rocm_stream_t stream, int64_t B, int64_t H, int64_t SQ, int64_t SKV,
                                        int64_t D, float scale, const uint16_t* Q, const uint16_t* K,
                                        const uint16_t* V, void* O, int out_bf16) {
    if (B < 0 || H < 0 || SQ < 0 || SKV < 0 || D < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: negative shape");
    if (D != 64) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "attention: head dim %lld (only 64 is built)", (long long) D);
    if (B == 0 || H == 0 || SQ == 0) return 0;
    if (SKV == 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: no keys (softmax over an empty axis)");
    if (!Q || !K || !V || !O) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: null pointer");
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: scale must be positive and finite");
    if ((((uintptr_t) Q | (uintptr_t) K | (uintptr_t) V | (uintptr_t) O) % 16) != 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "attention: pointers must be 16-byte aligned");
    if (B * H > 65535 || SQ > 0x7fffffffLL - 128 || SKV > 0x7fffffffLL - 64)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "attention: batch*heads must be <= 65535 and sequences < 2^31");
    int rc = ensure_device();
    if (rc) return rc;
    // LDS: ring of 3 stages x (K block [64][64] + V block [64][64]) bf16
    const uint32_t lds = 3 * (2 * 64 * 64) * 2;
    const float scale_log2e = scale * 1.4426950408889634f;
    return launch(out_bf16 ? "docc_attention_bf16_d64_bf16out" : "docc_attention_bf16_d64_f32out",
                  (uint32_t) ((SQ + 127) / 128), (uint32_t) (B * H), 1, 256, lds, (hipStream_t) stream, Q, K, V, O,
                  (int) SQ, (int) SKV, scale_log2e);
}
