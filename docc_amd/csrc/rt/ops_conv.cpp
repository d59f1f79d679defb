// Launcher for ml::Conv (see include/docc_rocm_ops.h).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

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
    int XC, YC;   // channels of the tensors X and Y lie in (C and OC, or more for the groups of a grouped convolution)
    long GX, GW, GB, GY;   // grouped convolution in one launch: elements from one group's operands to the next's (grid z = groups)
};

int64_t out_dim(int64_t d_in, int64_t pad_begin, int64_t pad_end, int64_t dil, int64_t kernel, int64_t stride) {
    // reference conv_node.cpp:224-233
    const int64_t num = d_in + pad_begin + pad_end - (dil * (kernel - 1) + 1);
    return num < 0 ? 0 : num / stride + 1;
}

} // namespace

namespace {

constexpr int64_t kConvWorkspaceCap = int64_t(2) << 30;   // images are processed in chunks that fit this

// How a layer runs on the LDS-halo kernel. A work-group takes 64 output channels x a strip of TH full output rows
// and costs what its 2 x `tiles` column tiles of 32 pixels cost, filled or not; one work-group owns a CU at a time
// (the forms with 7 and 4 tiles per wave by their registers), so a launch takes rounds of work-groups x tiles per wave.
// Strips of 448 pixels (7 tiles per wave) where the images give every CU one; of 416 with the thirteenth tile shared
// by the two pixel groups (6.5 tiles per wave, or 6.25 when that tile holds at most 16 pixels and goes through the
// 16-pixel MFMA) where that saves a round's worth - the shorter strips pay about 3.5 % more for halo rows and
// per-work-group set-up (measured on 32 x 64 x 56 x 56: 7 strips of 8 rows 68.4 us, 8 strips of 7 rows 70.9 us
// with 7 tiles a wave, 67.0 us with 6.5); strips of 256 or 128 pixels (4 or 2 tiles per wave) for small images,
// whose staging of weights per chunk is spread over fewer MFMAs (taken as 8 % and 20 %).
// Images smaller than half the smallest strip go several to a work-group (`images`, the kernels with the suffix m).
// DOCC_ROCM_CONV=halo-split / halo-split-wide / halo-whole / halo-t4 / halo-t2 / halo-t4m / halo-t2m force a form (tests, tuning).
struct HaloPlan {
    int tiles = 7;        // column tiles per wave
    int64_t TH = 1;       // output rows per strip
    int64_t images = 1;   // whole images per work-group (then TH == OH): images of a few pixels share a strip
    bool split = false, narrow = false;
    double cost = 0;      // rounds x tiles per wave x overhead
};

// whether a strip of `th` rows fits: at most three patch pixels per lane and chunk, three stages in 160 KB of LDS
bool halo_strip_fits(int64_t th, int64_t OW, int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w) {
    const int64_t PS = ((th - 1) * stride_h + KH) * ((OW - 1) * stride_w + KW);
    const int64_t stage = 64 * (8 * KH * KW + 4) + 8 * (PS + 1);
    return PS <= 3 * 256 && 3 * stage * 4 <= 160 * 1024;
}

// cost 0: no form of the kernel fits the layer
HaloPlan plan_halo(int64_t N, int64_t OC, int64_t OH, int64_t OW, int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int cus) {
    const int64_t ocb = (OC + 63) / 64;
    auto fits = [&](int64_t th) { return th >= 1 && halo_strip_fits(th, OW, KH, KW, stride_h, stride_w); };
    auto rows_for = [&](int64_t pixels) {
        int64_t th = pixels / OW;
        if (th > OH) th = OH;
        if (th >= 1) th = (OH + (OH + th - 1) / th - 1) / ((OH + th - 1) / th);   // the same number of strips, evenly high
        return th;
    };
    auto rounds = [&](int64_t th) { return (double) ((N * ((OH + th - 1) / th) * ocb + cus - 1) / cus); };
    HaloPlan plan;
    plan.TH = 448 / OW < OH ? 448 / OW : OH;   // (not evened out: the strips of the whole form stay as high as they can be)
    if (plan.TH < 1) plan.TH = 1;
    plan.cost = fits(plan.TH) ? rounds(plan.TH) * 7.0 : 0.0;
    const char* force = std::getenv("DOCC_ROCM_CONV");
    const bool forced = force && std::strncmp(force, "halo-", 5) == 0;
    if (KH == 3) {
        int64_t ths = 416 / OW < OH ? 416 / OW : OH;
        if (fits(ths)) {
            const bool narrow = ths * OW <= 12 * 32 + 16;
            const double cost = rounds(ths) * (narrow ? 6.25 : 6.5) * 1.035;
            bool split = cost < plan.cost || plan.cost == 0.0;
            bool narrow_form = narrow;
            if (forced) {
                if (std::strncmp(force, "halo-split", 10) == 0) split = true;
                if (std::strcmp(force, "halo-split-wide") == 0) narrow_form = false;
                if (std::strcmp(force, "halo-whole") == 0) split = false;
            }
            if (split) {
                plan.TH = ths;
                plan.split = true;
                plan.narrow = narrow_form;
                plan.cost = cost;
            }
        }
    }
    const struct { int tiles; double overhead; const char* name; } small[2] = {{4, 1.08, "halo-t4"}, {2, 1.20, "halo-t2"}};
    for (const auto& form : small) {
        int64_t th = rows_for(64 * form.tiles);
        while (th > 1 && !fits(th)) th--;      // (a strided layer's patch grows with the rows)
        if (!fits(th)) continue;
        const double cost = rounds(th) * form.tiles * form.overhead;
        const bool take = forced && plan.cost > 0.0 ? std::strcmp(force, form.name) == 0 : cost < plan.cost || plan.cost == 0.0;
        if (take) {
            plan.tiles = form.tiles;
            plan.TH = th;
            plan.images = 1;
            plan.split = plan.narrow = false;
            plan.cost = cost;
        }
    }
    // images of a few pixels (7 x 7: 49 of the 128 pixels of the smallest strip): several whole images per work-group
    for (const auto& form : small) {
        int64_t g = 64 * form.tiles / (OH * OW);
        const int64_t patch = ((OH - 1) * stride_h + KH) * ((OW - 1) * stride_w + KW);
        while (g >= 2 && !(g * patch <= 3 * 256 && 3 * (64 * (8 * KH * KW + 4) + 8 * (g * patch + 1)) * 4 <= 160 * 1024)) g--;
        if (g < 2 || g > N) continue;
        const double cost = (double) ((((N + g - 1) / g) * ocb + cus - 1) / cus) * form.tiles * form.overhead;
        char name[16];
        std::snprintf(name, sizeof(name), "%sm", form.name);
        const bool take = forced && plan.cost > 0.0 ? std::strcmp(force, name) == 0 : cost < plan.cost || plan.cost == 0.0;
        if (take) {
            plan.tiles = form.tiles;
            plan.TH = OH;
            plan.images = g;
            plan.split = plan.narrow = false;
            plan.cost = cost;
        }
    }
    return plan;
}

// Rough times (us) of the three ways to run a layer, from what the kernels were measured to sustain: the halo kernel
// about 490 GFLOP/s per CU on the tiles it computes. The gather kernel sustains about 55 TFLOP/s when its 64 x 128
// tiles fill the CUs evenly. The GEMM on a column matrix runs at
// about 75 TFLOP/s on these shapes; the columns are written and read once at about 5 TB/s, and the extra launches
// (columns, bias, transpose) cost about 15 us.
double halo_time_us(int64_t N, int64_t OC, int64_t OH, int64_t OW, int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t K, int cus) {
    return plan_halo(N, OC, OH, OW, KH, KW, stride_h, stride_w, cus).cost * (2.0 * 64 * 64 * (double) K) / 490e3;
}

double gather_time_us(int64_t N, int64_t OC, int64_t P, int64_t K, int cus) {
    const int64_t tiles = ((OC + 63) / 64) * ((N * P + 127) / 128);
    const int64_t rounds = (tiles + cus - 1) / cus;
    // past K = 1152 (128 channels of a 3x3 kernel) a tile's share of the input no longer stays close: 35 TFLOP/s at K = 2304
    const double rate = 55e6 * (K > 1152 ? std::pow(1152.0 / (double) K, 0.65) : 1.0);
    return (double) rounds * cus * (2.0 * 64 * 128 * (double) K) / rate;
}

double gemm_time_us(int64_t N, int64_t OC, int64_t P, int64_t K, bool needs_columns) {
    const double padded_oc = (double) ((OC + 63) / 64 * 64);
    return 2.0 * padded_oc * (double) K * (double) N * (double) P / 75e6 +
           (needs_columns ? 2.0 * 4.0 * (double) N * (double) K * (double) P / 5e6 + 15.0 : 5.0);
}

// bytes of columns + GEMM result per image
int64_t conv_bytes_per_image(int64_t OC, int64_t K, int64_t P) { return (K * P * 4 + 255) / 256 * 256 + (OC * P * 4 + 255) / 256 * 256; }

enum class ConvPath { Halo, Gather, Gemm1x1, GemmColumns };

// shapes the LDS-halo kernel is built for (the launcher also wants 16-byte aligned weights)
bool halo_shape_ok(int64_t C, int64_t KH, int64_t KW, int64_t OW, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w) {
    return stride_h >= 1 && stride_h <= 2 && stride_w >= 1 && stride_w <= 2 && dil_h == 1 && dil_w == 1 && ((KH == 3 && KW == 3) || (KH == 1 && KW == 1)) &&
           C % 8 == 0 && C > 0 && OW <= 448 && (C * KH * KW) % 4 == 0 && halo_strip_fits(1, OW, KH, KW, stride_h, stride_w);
}

ConvPath choose_path(int64_t N, int64_t C, int64_t OC, int64_t KH, int64_t KW, int64_t OH, int64_t OW, int64_t stride_h, int64_t stride_w,
                     int64_t pad_h, int64_t pad_w, bool halo_ok, bool have_workspace) {
    const char* force = std::getenv("DOCC_ROCM_CONV");   // halo | gather | gemm (tuning and tests)
    const bool pointwise = KH == 1 && KW == 1 && stride_h == 1 && stride_w == 1 && pad_h == 0 && pad_w == 0;
    const ConvPath gemm = pointwise ? ConvPath::Gemm1x1 : ConvPath::GemmColumns;
    const bool gemm_ok = pointwise || have_workspace;
    if (force && force[0] == 'h' && halo_ok) return ConvPath::Halo;
    if (force && force[0] == 'g' && force[1] == 'a') return ConvPath::Gather;
    if (force && force[0] == 'g' && force[1] == 'e' && gemm_ok) return gemm;
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    const int64_t K = C * KH * KW, P = OH * OW;
    // the aligned GEMM kernels want rows of the weight and column matrices that are multiples of 16 bytes
    const bool gemm_fast = gemm_ok && K % 4 == 0 && (pointwise ? P % 4 == 0 : true);
    // 1x1 layers move more bytes than they compute, which the models above do not see: measured, the batched GEMM
    // wins from 128 input channels on (C 256 -> 64 on 56 x 56: 50 against 65 us; C 64 -> 256: 99 against 74)
    if (pointwise) return gemm_fast && C >= 128 ? gemm : halo_ok ? ConvPath::Halo : ConvPath::Gather;
    const double direct = halo_ok ? halo_time_us(N, OC, OH, OW, KH, KW, stride_h, stride_w, K, cus) : gather_time_us(N, OC, P, K, cus);
    if (gemm_fast && gemm_time_us(N, OC, P, K, true) < 0.75 * direct) return gemm;
    return halo_ok ? ConvPath::Halo : ConvPath::Gather;
}

} // namespace

extern "C" int64_t docc_rocm_conv2d_f32_pads_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                                                             int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w,
                                                             int64_t pad_h_end, int64_t pad_w_end, int64_t dil_h, int64_t dil_w) {
    if (N <= 0 || C <= 0 || OC <= 0 || KH <= 0 || KW <= 0 || stride_h <= 0 || stride_w <= 0 || dil_h <= 0 || dil_w <= 0) return 0;
    if (pad_h < 0 || pad_w < 0 || pad_h_end < 0 || pad_w_end < 0) return 0;
    const int64_t OH = out_dim(H, pad_h, pad_h_end, dil_h, KH, stride_h), OW = out_dim(W, pad_w, pad_w_end, dil_w, KW, stride_w);
    if (OH <= 0 || OW <= 0) return 0;
    // what decides between the paths is whether there is padding at all: the larger of begin and end stands for both
    pad_h = pad_h > pad_h_end ? pad_h : pad_h_end;
    pad_w = pad_w > pad_w_end ? pad_w : pad_w_end;
    if (KH == 1 && KW == 1 && stride_h == 1 && stride_w == 1 && pad_h == 0 && pad_w == 0) return 0;   // the input is the column matrix
    // nothing either when one of the direct kernels would be chosen anyway (operands assumed aligned)
    const bool halo_ok = halo_shape_ok(C, KH, KW, OW, stride_h, stride_w, dil_h, dil_w);
    if (choose_path(N, C, OC, KH, KW, OH, OW, stride_h, stride_w, pad_h, pad_w, halo_ok, true) != ConvPath::GemmColumns) return 0;
    const int64_t per_image = conv_bytes_per_image(OC, C * KH * KW, OH * OW);
    int64_t images = kConvWorkspaceCap / per_image;
    if (images < 1) images = 1;
    if (images > N) images = N;
    return images * per_image;
}

extern "C" int64_t docc_rocm_conv2d_f32_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                                                        int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t dil_h,
                                                        int64_t dil_w) {
    return docc_rocm_conv2d_f32_pads_workspace_bytes(N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h, pad_w, dil_h, dil_w);
}

// The kernels place the window with the begin pads and test every tap against the image, so the end pads only
// enter through the output extents.
static int conv2d_run(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                      int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t pad_h_end, int64_t pad_w_end, int64_t dil_h,
                      int64_t dil_w, const float* X, const float* Wt, const float* bias, float* Y, void* workspace, int64_t workspace_bytes,
                      int64_t x_channels = -1, int64_t y_channels = -1, int64_t groups = 1) {
    // x_channels, y_channels: the channels of the tensors X and Y point into, where this call is a grouped convolution (the
    // images are then that many channels apart); -1: C and OC. groups: that many convolutions of these extents in one launch
    // (grid z), group g on the channels g * C .. of X, g * OC .. of Y, filters and bias
    if (x_channels < 0) x_channels = C;
    if (y_channels < 0) y_channels = OC;
    const bool slice = x_channels != C || y_channels != OC || groups > 1;
    if (N < 0 || C < 0 || H < 0 || W < 0 || OC < 0 || KH <= 0 || KW <= 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: bad shape");
    if (stride_h <= 0 || stride_w <= 0 || dil_h <= 0 || dil_w <= 0 || pad_h < 0 || pad_w < 0 || pad_h_end < 0 || pad_w_end < 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: stride and dilation must be positive, padding non-negative");
    const int64_t OH = out_dim(H, pad_h, pad_h_end, dil_h, KH, stride_h), OW = out_dim(W, pad_w, pad_w_end, dil_w, KW, stride_w);
    const int64_t any_pad_h = pad_h > pad_h_end ? pad_h : pad_h_end, any_pad_w = pad_w > pad_w_end ? pad_w : pad_w_end;
    if (N == 0 || OC == 0 || OH == 0 || OW == 0) return 0;
    if (!Y || !Wt || (C > 0 && !X)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: null pointer");
    const int64_t lim = 0x7fffffffLL;
    if (x_channels * H * W >= lim || C * KH * KW >= lim || OH * OW >= lim || N >= lim || y_channels >= lim)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "conv2d: per-image extents must fit in 31 bits");
    int rc = ensure_device();
    if (rc) return rc;

    ConvParams p{X, Wt, bias, Y, (int) N, (int) C, (int) H, (int) W, (int) OC, (int) KH, (int) KW, (int) OH, (int) OW,
                 (int) stride_h, (int) stride_w, (int) pad_h, (int) pad_w, (int) dil_h, (int) dil_w, (int) x_channels, (int) y_channels,
                 groups > 1 ? (long) (C * H * W) : 0, groups > 1 ? (long) (OC * C * KH * KW) : 0, groups > 1 ? (long) OC : 0, groups > 1 ? (long) (OC * OH * OW) : 0};
    if (groups < 1 || groups > 65535) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "conv2d: 1 to 65535 groups");
    const uint32_t gz = (uint32_t) groups;
    // Stride-1, dilation-1 3x3 and 1x1 convolutions take the LDS-halo kernel: 64 output channels x a
    // strip of TH full output rows (at most 448 pixels) per work-group, 8 input channels per chunk.
    const bool halo_shape = halo_shape_ok(C, KH, KW, OW, stride_h, stride_w, dil_h, dil_w) && ((uintptr_t) Wt % 16 == 0);
    const int64_t need = docc_rocm_conv2d_f32_pads_workspace_bytes(N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h_end, pad_w_end,
                                                                   dil_h, dil_w);
    const bool have_workspace = workspace && workspace_bytes >= need && need > 0 && ((uintptr_t) workspace % 256) == 0;
    ConvPath path = C == 0 ? ConvPath::Gather
                           : choose_path(N, C, OC, KH, KW, OH, OW, stride_h, stride_w, any_pad_h, any_pad_w, halo_shape, have_workspace);
    // one group of a grouped convolution: the direct kernels, which take the distance between the images as it is (the
    // GEMM paths write whole [N, OC, P] tensors)
    if (slice && (path == ConvPath::Gemm1x1 || path == ConvPath::GemmColumns)) path = halo_shape ? ConvPath::Halo : ConvPath::Gather;
    if (path == ConvPath::Gemm1x1) {
        // Y[n] (OC x P) = W (OC x C) X[n] (C x P): one batched GEMM on the tensors as they lie; the bias is
        // written first and accumulated onto
        const int64_t P = OH * OW;
        if (bias) {
            const int64_t in_shape[3] = {1, OC, 1}, out_shape[3] = {N, OC, P};
            rc = docc_rocm_broadcast(stream, 32, 3, in_shape, out_shape, bias, Y);
            if (rc) return rc;
        }
        return docc_rocm_sgemm_batched(stream, DOCC_ROCM_NO_TRANS, DOCC_ROCM_NO_TRANS, OC, P, C, 1.f, Wt, C, 0, X, P, C * P, bias ? 1.f : 0.f,
                                       Y, P, OC * P, N);
    }
    if (path == ConvPath::GemmColumns) {
        const int64_t P = OH * OW, K = C * KH * KW;
        const int64_t per_image = conv_bytes_per_image(OC, K, P);
        int64_t chunk = workspace_bytes / per_image;
        if (chunk > N) chunk = N;
        float* col = (float*) workspace;
        float* result = (float*) ((char*) workspace + chunk * ((K * P * 4 + 255) / 256 * 256));
        for (int64_t n0 = 0; n0 < N; n0 += chunk) {
            const int64_t nn = N - n0 < chunk ? N - n0 : chunk;
            const int64_t cols = nn * P;
            rc = launch("docc_conv2d_im2col_f32", (uint32_t) ((cols + 255) / 256), (uint32_t) (K < 65535 ? K : 65535), 1, 256, 0,
                        (hipStream_t) stream, p, (int) n0, (int) nn, col);
            if (rc) return rc;
            // one image: the GEMM result is the output itself; more: [OC][nn][P], moved to [nn][OC][P] afterwards
            float* out = nn == 1 ? Y + n0 * OC * P : result;
            if (bias) {
                const int64_t in_shape[2] = {OC, 1}, out_shape[2] = {OC, cols};
                rc = docc_rocm_broadcast(stream, 32, 2, in_shape, out_shape, bias, out);
                if (rc) return rc;
            }
            rc = docc_rocm_sgemm(stream, DOCC_ROCM_NO_TRANS, DOCC_ROCM_NO_TRANS, OC, cols, K, 1.f, Wt, K, col, cols, bias ? 1.f : 0.f, out, cols);
            if (rc) return rc;
            if (nn > 1) {
                const int64_t shape[3] = {OC, nn, P}, perm[3] = {1, 0, 2};
                rc = docc_rocm_transpose(stream, 4, 3, shape, perm, result, Y + n0 * OC * P);
                if (rc) return rc;
            }
        }
        return 0;
    }
    if (path == ConvPath::Halo) {
        int cus = compute_units();
        if (cus <= 0) cus = 256;
        const HaloPlan plan = plan_halo(N, OC, OH, OW, KH, KW, stride_h, stride_w, cus);
        const int64_t TH = plan.TH;
        const int64_t PS = plan.images * ((TH - 1) * stride_h + KH) * ((OW - 1) * stride_w + KW);   // patch pixels
        const int64_t stage = 64 * (8 * KH * KW + 4) + 8 * (PS + 1);  // weights + patch + spare pixel, floats
        const int64_t strips = (OH + TH - 1) / TH;
        if (plan.images > 1 && plan.cost > 0.0 && PS <= 3 * 256 && 3 * stage * 4 <= 160 * 1024 && OC * C * KH * KW < (int64_t(1) << 29) &&
            plan.images * x_channels * H * W < (int64_t(1) << 29) && (OC + 63) / 64 <= 65535) {
            char name[64];
            std::snprintf(name, sizeof(name), "docc_conv2d_f32_halo_%s_t%dm%s", KH == 3 ? "3x3" : "1x1", plan.tiles, groups > 1 ? "_g" : "");
            return launch(name, (uint32_t) ((N + plan.images - 1) / plan.images), (uint32_t) ((OC + 63) / 64), gz, 256, (uint32_t) (3 * stage * 4),
                          (hipStream_t) stream, p, (int) TH, (int) plan.images);
        }
        if (plan.images == 1 && plan.cost > 0.0 && halo_strip_fits(TH, OW, KH, KW, stride_h, stride_w) && OC * C * KH * KW < (int64_t(1) << 29) && C * H * W < (int64_t(1) << 29) && N * strips < lim && (OC + 63) / 64 <= 65535) {
            char name[64];
            std::snprintf(name, sizeof(name), "docc_conv2d_f32_halo_%s%s%s", KH == 3 ? "3x3" : "1x1",
                          plan.tiles == 4 ? "_t4" : plan.tiles == 2 ? "_t2" : plan.split ? (plan.narrow ? "_split16" : "_split") : "",
                          groups > 1 ? "_g" : "");
            return launch(name, (uint32_t) (N * strips), (uint32_t) ((OC + 63) / 64), gz, 256, (uint32_t) (3 * stage * 4), (hipStream_t) stream, p, (int) TH);
        }
    }
    constexpr int BM = 64, BN = 128, BK = 16;
    const int64_t tiles = ((OC + BM - 1) / BM) * ((N * OH * OW + BN - 1) / BN);
    if (tiles >= lim) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "conv2d: too many tiles");
    const int64_t K = C * KH * KW;
    const bool aligned = ((uintptr_t) Wt % 16 == 0) && (K % 4 == 0);
    // LDS: 2 x (A tile [BM][BK+4] + B tile [BK][BN+8]) floats + 2 x BK table entries of 16 bytes
    const uint32_t lds = 2 * (BM * (BK + 4) + BK * (BN + 8)) * 4 + 2 * BK * 16;
    return launch(groups > 1 ? (aligned ? "docc_conv2d_f32_gather_64x128_a_g" : "docc_conv2d_f32_gather_64x128_u_g")
                             : (aligned ? "docc_conv2d_f32_gather_64x128_a" : "docc_conv2d_f32_gather_64x128_u"),
                  (uint32_t) tiles, 1,
                  gz, 256, lds, (hipStream_t) stream, p);
}

extern "C" int docc_rocm_conv2d_f32(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                                    int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h,
                                    int64_t pad_w, int64_t dil_h, int64_t dil_w, const float* X, const float* Wt,
                                    const float* bias, float* Y) {
    return conv2d_run(stream, N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h, pad_w, dil_h, dil_w, X, Wt, bias, Y, nullptr, 0);
}

extern "C" int docc_rocm_conv2d_f32_ws(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                                       int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h,
                                       int64_t pad_w, int64_t dil_h, int64_t dil_w, const float* X, const float* Wt,
                                       const float* bias, float* Y, void* workspace, int64_t workspace_bytes) {
    return conv2d_run(stream, N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h, pad_w, dil_h, dil_w, X, Wt, bias, Y, workspace,
                      workspace_bytes);
}

extern "C" int docc_rocm_conv2d_f32_pads(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
                                         int64_t KH, int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w,
                                         int64_t pad_h_end, int64_t pad_w_end, int64_t dil_h, int64_t dil_w, const float* X,
                                         const float* Wt, const float* bias, float* Y, void* workspace, int64_t workspace_bytes) {
    return conv2d_run(stream, N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h_end, pad_w_end, dil_h, dil_w, X, Wt, bias, Y,
                      workspace, workspace_bytes);
}

// ONNX Conv with group > 1 (reference ConvNode: W [OC][C / group][KH][KW], conv_node.cpp:376-377; output channel oc belongs
// to group oc / (OC / group) and reads that group's C / group input channels): one call of the kernels above per group, on
// the group's channels of X and Y where they lie.
extern "C" int docc_rocm_conv2d_f32_grouped(docc_rocm_stream_t stream, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int64_t KH,
                                            int64_t KW, int64_t stride_h, int64_t stride_w, int64_t pad_h, int64_t pad_w, int64_t pad_h_end,
                                            int64_t pad_w_end, int64_t dil_h, int64_t dil_w, int64_t group, const float* X, const float* Wt,
                                            const float* bias, float* Y, void* workspace, int64_t workspace_bytes) {
    if (group <= 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: group must be positive");
    if (group == 1)
        return conv2d_run(stream, N, C, H, W, OC, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h_end, pad_w_end, dil_h, dil_w, X, Wt, bias, Y,
                          workspace, workspace_bytes);
    if (C < 0 || OC < 0 || C % group != 0 || OC % group != 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: group %lld does not divide the channels (%lld in, %lld out)", (long long) group,
                    (long long) C, (long long) OC);
    if (KH <= 0 || KW <= 0 || H < 0 || W < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: bad shape");
    const int64_t cg = C / group, og = OC / group;
    const int64_t OH = out_dim(H, pad_h, pad_h_end, dil_h, KH, stride_h), OW = out_dim(W, pad_w, pad_w_end, dil_w, KW, stride_w);
    // depthwise (one input channel a group): one launch of the kernel that is bound by moving X and Y; DOCC_ROCM_CONV=gather
    // keeps the launch per group (tests)
    const char* force = std::getenv("DOCC_ROCM_CONV");
    if (cg == 1 && !(force && force[0] == 'g')) {
        if (stride_h <= 0 || stride_w <= 0 || dil_h <= 0 || dil_w <= 0 || pad_h < 0 || pad_w < 0 || pad_h_end < 0 || pad_w_end < 0 || N < 0)
            return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: stride and dilation must be positive, padding non-negative");
        if (N == 0 || OC == 0 || OH == 0 || OW == 0) return 0;
        if (!Y || !Wt || !X) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "conv2d: null pointer");
        const int64_t lim = 0x7fffffffLL, P = OH * OW;
        const int64_t blocks = N * OC * ((P + 255) / 256);
        if (C * H * W >= lim || P >= lim || N >= lim || OC >= lim || KH * KW >= lim || blocks >= lim)
            return fail(DOCC_ROCM_ERR_UNSUPPORTED, "conv2d: per-image extents must fit in 31 bits");
        if (int rc = ensure_device()) return rc;
        ConvParams p{X, Wt, bias, Y, (int) N, (int) C, (int) H, (int) W, (int) OC, (int) KH, (int) KW, (int) OH, (int) OW,
                     (int) stride_h, (int) stride_w, (int) pad_h, (int) pad_w, (int) dil_h, (int) dil_w, (int) C, (int) OC, 0, 0, 0, 0};
        // 3x3, stride 1, rows of whole aligned quads: four pixels a lane
        if (KH == 3 && KW == 3 && stride_h == 1 && stride_w == 1 && dil_h == 1 && dil_w == 1 && pad_w == 1 && OW == W && W % 4 == 0 &&
            (uintptr_t) X % 16 == 0 && (uintptr_t) Y % 16 == 0 && !(force && force[0] == 's')) {   // DOCC_ROCM_CONV=scalar: a pixel a lane (tests)
            // several output rows a lane (seven where that divides the plane's rows, as the 224 / 2^i planes of the image
            // networks, else eight, four for low planes); DOCC_ROCM_CONV=quad keeps one row a lane, DOCC_ROCM_CONV_ROWS=4|7|8
            // names the count (both for tests and measurements)
            const char* rows_env = std::getenv("DOCC_ROCM_CONV_ROWS");
            int rows = OH % 7 == 0 ? 7 : OH >= 16 ? 8 : 4;
            if (rows_env && (rows_env[0] == '4' || rows_env[0] == '7' || rows_env[0] == '8') && !rows_env[1]) rows = rows_env[0] - '0';
            const int64_t items = N * OC * (OW / 4) * ((OH + rows - 1) / rows);
            if (!(force && force[0] == 'q') && items + 255 < lim) {
                const char* name = rows == 7 ? "docc_conv2d_depthwise_f32_3x3_v4_r7" : rows == 8 ? "docc_conv2d_depthwise_f32_3x3_v4_r8" : "docc_conv2d_depthwise_f32_3x3_v4_r4";
                return launch(name, (uint32_t) ((items + 255) / 256), 1, 1, 256, 0, (hipStream_t) stream, p, (int) og);
            }
            const int64_t quads = N * OC * ((OH * (OW / 4) + 255) / 256);
            return launch("docc_conv2d_depthwise_f32_3x3_v4", (uint32_t) quads, 1, 1, 256, 0, (hipStream_t) stream, p, (int) og);
        }
        // other 3x3 layers and 5x5 ones without dilation that step by one or by two: a column and seven or four output rows a lane
        if (((KH == 3 && KW == 3) || (KH == 5 && KW == 5)) && stride_h == stride_w && (stride_h == 1 || stride_h == 2) && dil_h == 1 && dil_w == 1 &&
            !(force && (force[0] == 's' || force[0] == 'q'))) {
            const char* rows_env = std::getenv("DOCC_ROCM_CONV_ROWS");
            int rows = OH % 7 == 0 && OH >= 28 ? 7 : 4;   // measured: planes of 14 and 7 rows run faster with four
            if (rows_env && (rows_env[0] == '4' || rows_env[0] == '7') && !rows_env[1]) rows = rows_env[0] - '0';
            const int64_t items = N * OC * OW * ((OH + rows - 1) / rows);
            if (items + 255 < lim) {
                char name[64];
                std::snprintf(name, sizeof(name), "docc_conv2d_depthwise_f32_%dx%d_s%d_r%d", (int) KH, (int) KW, (int) stride_h, rows);
                return launch(name, (uint32_t) ((items + 255) / 256), 1, 1, 256, 0, (hipStream_t) stream, p, (int) og);
            }
        }
        const char* name = KH == 3 && KW == 3 ? "docc_conv2d_depthwise_f32_3x3" : KH == 5 && KW == 5 ? "docc_conv2d_depthwise_f32_5x5" : "docc_conv2d_depthwise_f32";
        return launch(name, (uint32_t) blocks, 1, 1, 256, 0, (hipStream_t) stream, p, (int) og);
    }
    // groups of at most 16 channels in, 3x3, stride 1, rows of whole aligned quads: the kernel that is bound by moving X and Y
    // (DOCC_ROCM_CONV_SMALL_GROUP=<channels> moves the limit: measurements)
    const char* sg_env = std::getenv("DOCC_ROCM_CONV_SMALL_GROUP");
    const int64_t small_group_limit = sg_env && sg_env[0] ? std::atoll(sg_env) : 16;
    // (DOCC_ROCM_CONV=gather or loop keeps the kernels of the larger groups: tests)
    if (cg <= small_group_limit && og <= 64 && KH == 3 && KW == 3 && stride_h == 1 && stride_w == 1 && dil_h == 1 && dil_w == 1 && pad_w == 1 && pad_h >= 0 &&
        pad_h_end >= 0 && pad_w_end >= 0 && OW == W && W % 4 == 0 && (uintptr_t) X % 16 == 0 && (uintptr_t) Y % 16 == 0 && X && Y && Wt && N > 0 &&
        OH > 0 && !(force && (force[0] == 'g' || force[0] == 'l'))) {
        const int ogt = og % 8 == 0 ? 8 : og % 4 == 0 ? 4 : og % 2 == 0 ? 2 : 1;
        const int64_t lim = 0x7fffffffLL;
        const int64_t blocks = N * group * (og / ogt) * ((OH * (OW / 4) + 255) / 256);
        // nine to 16 channels in: the 64 output channels of an MFMA tile are a quarter or a half real up to 32 channels out
        // (measured with 16 in and out: C512 28x28 in 32 groups 214 -> 69 us, C256 56x56 in 16 groups 352 -> 114, C64 56x56 in 4
        // groups 91 -> 40); with 64 out the tiles win (40 against 64 us), and so they do on launches that leave CUs idle
        bool pays = true;
        if (cg > 8) {
            if (int rc = ensure_device()) return rc;
            pays = og <= 32 && blocks >= (compute_units() > 0 ? compute_units() : 256);
        }
        if (pays && C * H * W < lim && OH * OW < lim && OC < lim && blocks < lim) {
            if (int rc = ensure_device()) return rc;
            ConvParams p{X, Wt, bias, Y, (int) N, (int) C, (int) H, (int) W, (int) OC, (int) KH, (int) KW, (int) OH, (int) OW,
                         (int) stride_h, (int) stride_w, (int) pad_h, (int) pad_w, (int) dil_h, (int) dil_w, (int) C, (int) OC, 0, 0, 0, 0};
            char name[64];
            // several output rows a lane, the lanes counting through the images; DOCC_ROCM_CONV=quad keeps one row a lane and
            // DOCC_ROCM_CONV_ROWS=4 takes four rows for eight output channels instead of two (tests, measurements)
            const char* rows_env = std::getenv("DOCC_ROCM_CONV_ROWS");
            const int rows = ogt == 8 ? (rows_env && rows_env[0] == '4' && !rows_env[1] ? 4 : 2) : ogt == 4 ? 4 : 8;
            const int64_t items = N * (OW / 4) * ((OH + rows - 1) / rows);
            const int64_t row_blocks = group * (og / ogt) * ((items + 255) / 256);
            // measured: the form pays once its work-groups fill the chip about three times over (768 of them on 256 CUs: C128
            // 56x56 in 32 groups 38 -> 34 us, C256 56x56 87 -> 67), and always for one or two output channels a lane, where the
            // LDS reads bound the other form (C64 56x56 19 -> 14); with fewer work-groups one row a lane has more waves to
            // hide the loads behind (C256 28x28: 24 against 29)
            const int cus = compute_units() > 0 ? compute_units() : 256;
            const bool rows_pay = row_blocks >= 3 * (int64_t) cus || ogt <= 2 || (rows_env && rows_env[0]);
            if (!(force && force[0] == 'q') && rows_pay && items + 255 < lim && row_blocks < lim) {
                std::snprintf(name, sizeof(name), "docc_conv2d_small_groups_f32_3x3_v4_o%d_r%d", ogt, rows);
                return launch(name, (uint32_t) row_blocks, 1, 1, 256, (uint32_t) (ogt * cg * 9 * 4), (hipStream_t) stream, p, (int) cg, (int) og);
            }
            std::snprintf(name, sizeof(name), "docc_conv2d_small_groups_f32_3x3_v4_o%d", ogt);
            return launch(name, (uint32_t) blocks, 1, 1, 256, (uint32_t) (ogt * cg * 9 * 4), (hipStream_t) stream, p, (int) cg, (int) og);
        }
    }
    // every group in one launch (grid z) where the groups fit it, else a launch per group
    if (group <= 65535 && !(force && force[0] == 'l'))   // DOCC_ROCM_CONV=loop: a launch per group (tests)
        return conv2d_run(stream, N, cg, H, W, og, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h_end, pad_w_end, dil_h, dil_w, X, Wt, bias, Y,
                          nullptr, 0, C, OC, group);
    for (int64_t g = 0; g < group; g++) {
        const int rc = conv2d_run(stream, N, cg, H, W, og, KH, KW, stride_h, stride_w, pad_h, pad_w, pad_h_end, pad_w_end, dil_h, dil_w,
                                  X ? X + g * cg * H * W : nullptr, Wt ? Wt + g * og * cg * KH * KW : nullptr, bias ? bias + g * og : nullptr,
                                  Y ? Y + g * og * OH * OW : nullptr, nullptr, 0, C, OC);
        if (rc) return rc;
    }
    return 0;
}
