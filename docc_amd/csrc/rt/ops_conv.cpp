// Launcher for ml::Conv (see include/docc_rocm_ops.h).
#include <cstdlib>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace {

// must match docc_k::ConvParams in csrc/kernels/conv2d.hip
struct ConvParams {
    const float* X;
    const float* Wt;
    const float* bias;
    float* Y;
    int N, C, H, W, OC, KH, KW, OH, OW;
    int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
};

int64_t out_dim(int64_t d_in, int64_t pad, int64_t dil, int64_t kernel, int64_t stride) {
    // reference conv_node.cpp:224-233 with pads_begin == pads_end
    const int64_t num = d_in + 2 * pad - (dil * (kernel - 1) + 1);
    return num < 0 ? 0 : num / stride + 1;
}

} // namespace

extern "C" int docc_rocm_conv2d_f32(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                                    int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h,
                                    int64_t pad_w, int64_t dil_h, int64_t dil_w, const float* X, const float* Wt,
                                    const float* bias, float* Y) {
    if (N < 0 || C < 0 || H < 0 || W < 0 || OC < 0 || KH <= 0 || KW <= 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: bad shape");
    if (stride_h <= 0 || stride_w <= 0 || dil_h <= 0 || dil_w <= 0 || pad_h < 0 || pad_w < 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: stride and dilation must be positive, padding non-negative");
    const int64_t OH = out_dim(H, pad_h, dil_h, KH, stride_h), OW = out_dim(W, pad_w, dil_w, KW, stride_w);
    if (N == 0 || OC == 0 || OH == 0 || OW == 0) return 0;
    if (!Y || !Wt || (C > 0 && !X)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: null pointer");
    const int64_t lim = 0x7fffffffLL;
    if (C * H * W >= lim || C * KH * KW >= lim || OH * OW >= lim || N >= lim || OC >= lim)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "conv2d: per-image extents must fit in 31 bits");
    int rc = ensure_device();
    if (rc) return rc;

    ConvParams p{X, Wt, bias, Y, (int) N, (int) C, (int) H, (int) W, (int) OC, (int) KH, (int) KW, (int) OH, (int) OW,
                 (int) stride_h, (int) stride_w, (int) pad_h, (int) pad_w, (int) dil_h, (int) dil_w};
    // Stride-1, dilation-1 3x3 and 1x1 convolutions take the LDS-halo kernel: 64 output channels x a
    // strip of TH full output rows (at most 448 pixels) per work-group, 8 input channels per chunk.
    const bool halo_shape = stride_h == 1 && stride_w == 1 && dil_h == 1 && dil_w == 1 &&
                            ((KH == 3 && KW == 3) || (KH == 1 && KW == 1)) && C % 8 == 0 && C > 0 && OW <= 448 &&
                            ((uintptr_t) Wt % 16 == 0) && ((C * KH * KW) % 4 == 0);
    if (halo_shape && !std::getenv("DOCC_ROCM_CONV_GATHER")) {
        int64_t TH = 448 / OW;
        if (TH > OH) TH = OH;
        const int64_t PS = (TH + KH - 1) * (OW + KW - 1);           // patch pixels
        const int64_t stage = 64 * (8 * KH * KW + 4) + 8 * (PS + 1);  // weights + patch + spare pixel, floats
        const int64_t strips = (OH + TH - 1) / TH;
        if (PS <= 3 * 256 && 3 * stage * 4 <= 160 * 1024 && OC * C * KH * KW < (int64_t(1) << 29) && C * H * W < (int64_t(1) << 29) && N * strips < lim && (OC + 63) / 64 <= 65535) {
            return launch(KH == 3 ? "docc_conv2d_f32_halo_3x3" : "docc_conv2d_f32_halo_1x1", (uint32_t) (N * strips),
                          (uint32_t) ((OC + 63) / 64), 1, 256, (uint32_t) (3 * stage * 4), (hipStream_t) stream, p, (int) TH);
        }
    }
    constexpr int BM = 64, BN = 128, BK = 16;
    const int64_t tiles = ((OC + BM - 1) / BM) * ((N * OH * OW + BN - 1) / BN);
    if (tiles >= lim) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "conv2d: too many tiles");
    const int64_t K = C * KH * KW;
    const bool aligned = ((uintptr_t) Wt % 16 == 0) && (K % 4 == 0);
    // LDS: 2 x (A tile [BM][BK+4] + B tile [BK][BN+8]) floats + 2 x BK table entries of 16 bytes
    const uint32_t lds = 2 * (BM * (BK + 4) + BK * (BN + 8)) * 4 + 2 * BK * 16;
    return launch(aligned ? "docc_conv2d_f32_gather_64x128_a" : "docc_conv2d_f32_gather_64x128_u", (uint32_t) tiles, 1,
                  1, 256, lds, (hipStream_t) stream, p);
}
