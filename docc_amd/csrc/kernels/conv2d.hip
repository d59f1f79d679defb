// ml::Conv, 2-d NCHW fp32, as implicit GEMM on v_mfma_f32_32x32x2_f32.
//
// Replaces the 7-deep scalar loop nest ConvNode::expand produces (reference
// sdfg/src/data_flow/library_nodes/math/tensor/conv_node.cpp:244-437), with
// the zero padding of the ONNX definition the node's header cites
// (conv_node.h:9-22) - the reference's expansion has no bounds test.
//
// GEMM view:  Y[n, oc, p] = bias[oc] + sum_k W[oc, k] * Xcol[k, (n, p)]
//   M = OC, K = C*KH*KW (k = (ic*KH + kh)*KW + kw, the memory order of W),
//   N = batch * OH * OW flattened, p = oh*OW + ow.
// W is the k-contiguous A operand and is staged through LDS as in
// gemm_mfma.h. The im2col matrix is never materialised: the B tile
// [BK][BN] is gathered straight from X (consecutive threads = consecutive
// output pixels, so the loads coalesce along a row of the image; taps that
// fall into the padding read as zero). A per-k table {input offset, dh, dw}
// for the next K-step is rebuilt in LDS by BK threads per step, so no thread
// divides in the inner loop.
#include "gemm_mfma.h"
#include <type_traits>

namespace docc_k {

struct ConvParams {
    const float* X;
    const float* Wt;
    const float* bias;
    float* Y;
    int N, C, H, W, OC, KH, KW, OH, OW;
    int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
    // channels of the tensors X and Y lie in: C and OC, or more when the call is one group of a grouped convolution (the
    // images are then XC and YC channels apart)
    int XC, YC;
    // grouped convolution in one launch (the entry points with the suffix _g): blockIdx.z is the group, whose operands lie
    // these many elements further on. The kernels of a single convolution do not look at them (their registers are full).
    long GX, GW, GB, GY;
};

__device__ __forceinline__ void conv_select_group(ConvParams& p) {
    const long g = blockIdx.z;
    p.X += g * p.GX;
    p.Wt += g * p.GW;
    if (p.bias) p.bias += g * p.GB;
    p.Y += g * p.GY;
}

template <int BM, int BN, int BK, int WM, int WN, bool ALIGNED>
struct ConvGatherKernel {
    typedef Mfma<float> X;
    static constexpr int NT = 64 * WM * WN;
    static constexpr int MT = 32, VK = 4, KG = 8;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int TM = WTM / MT, TN = WTN / MT;
    static constexpr int LDA_S = BK + 4, LDB_S = BN + 8;
    static constexpr int A_ELEMS = BM * LDA_S, B_ELEMS = BK * LDB_S;
    static constexpr int NB = BK * BN / NT;  // gathered elements per thread per K-step
    static_assert(NT % BN == 0, "a thread must keep one output pixel");
    static_assert(BK * BN % NT == 0 && BK % KG == 0, "tile shape");
    static constexpr int KSTEP = NT / BN;    // k distance between a thread's consecutive elements

    typedef TileLoader<float, BM, BK, NT, ALIGNED, true> ALoader;

    static __device__ __forceinline__ void run(const ConvParams& p) {
        extern __shared__ __attribute__((aligned(16))) unsigned char docc_conv_lds[];
        float* const lds = reinterpret_cast<float*>(docc_conv_lds);
        constexpr int B_BASE = 2 * A_ELEMS;
        constexpr int T_BASE = B_BASE + 2 * B_ELEMS;  // k-table: 2 buffers x BK x {off, dh, dw, valid}
        int* const ktab = reinterpret_cast<int*>(lds + T_BASE);

        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int wm = wave / WN, wn = wave % WN;
        const long P = (long) p.OH * p.OW;
        const long ncols = (long) p.N * P;
        const int K = p.C * p.KH * p.KW;
        const int tiles_m = (p.OC + BM - 1) / BM, tiles_n = (int) ((ncols + BN - 1) / BN);
        int tm, tn;
        gemm_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        const long m0 = (long) tm * BM, n0 = (long) tn * BN;

        // this thread's output pixel for the gather
        const long gcol = n0 + tid % BN;
        const bool col_ok = gcol < ncols;
        const long gn = col_ok ? gcol / P : 0;
        const int gp = col_ok ? (int) (gcol % P) : 0;
        const int ih0 = (gp / p.OW) * p.stride_h - p.pad_h;
        const int iw0 = (gp % p.OW) * p.stride_w - p.pad_w;
        const float* xbase = p.X + (gn * p.XC * p.H + ih0) * (long) p.W + iw0;
        const int kk0 = tid / BN;  // first k row of this thread inside a K-step

        auto build_table = [&](int kt, int buf) {
            if (tid < BK) {
                const int k = kt * BK + tid;
                int4 e = {0, 0, 0, 0};
                if (k < K) {
                    const int khw = p.KH * p.KW;
                    const int ic = k / khw, r = k % khw;
                    const int dh = (r / p.KW) * p.dil_h, dw = (r % p.KW) * p.dil_w;
                    e = {(ic * p.H + dh) * p.W + dw, dh, dw, 1};
                }
                reinterpret_cast<int4*>(ktab)[buf * BK + tid] = e;
            }
        };

        f32x16 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

        ALoader la;
        float bv[NB];
        unsigned bok = 0;  // bit i: gathered element i is a real input pixel (not padding)
        la.init(p.Wt, K, m0, 0, p.OC, K, tid);
        const int full = K / BK, kleft = K - full * BK;
        auto gload = [&](int kt) {   // called for kt = 0, 1, 2, ... in order
            if (kt > 0) la.advance();
            if (kt < full) la.load_full();
            else la.load_tail(kleft, tid);
            const int4* tab = reinterpret_cast<const int4*>(ktab) + (kt & 1) * BK;
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int4 e = tab[kk0 + i * KSTEP];
                const int ih = ih0 + e.y, iw = iw0 + e.z;
                const bool ok = col_ok && e.w && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
                // branch-free: padding taps read the tensor origin and are zeroed in bstore()
                bv[i] = *(ok ? xbase + e.x : p.X);
                bok = ok ? (bok | (1u << i)) : (bok & ~(1u << i));
            }
        };
        auto bstore = [&](float* bs) {
#pragma unroll
            for (int i = 0; i < NB; i++) bs[(kk0 + i * KSTEP) * LDB_S + tid % BN] = ((bok >> i) & 1u) ? bv[i] : 0.f;
        };

        const int ktiles = (K + BK - 1) / BK;
        build_table(0, 0);
        build_table(1, 1);
        __syncthreads();
        gload(0);
        la.template store<LDA_S>(lds, tid);
        bstore(lds + B_BASE);
        __syncthreads();

        const int lrow = lane % MT, lk = (lane / MT) * VK;
        for (int kt = 0; kt < ktiles; kt++) {
            const int cur = kt & 1;
            if (kt + 1 < ktiles) gload(kt + 1);
            const float* as = lds + cur * A_ELEMS;
            const float* bs = lds + B_BASE + cur * B_ELEMS;
#pragma unroll
            for (int kg = 0; kg < BK / KG; kg++) {
                float a[TM][VK], b[TN][VK];
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    const f32x4 t = *reinterpret_cast<const f32x4*>(as + (wm * WTM + i * MT + lrow) * LDA_S + kg * KG + lk);
#pragma unroll
                    for (int s = 0; s < VK; s++) a[i][s] = t[s];
                }
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int s = 0; s < VK; s++) b[j][s] = bs[(kg * KG + lk + s) * LDB_S + wn * WTN + j * MT + lrow];
#pragma unroll
                for (int s = 0; s < VK; s++)
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) acc[i][j] = X::mfma(a[i][s], b[j][s], acc[i][j]);
            }
            // tile buffer cur^1 and table buffer cur were last read before the
            // barrier that ended the previous step, so they can be overwritten now
            if (kt + 1 < ktiles) {
                la.template store<LDA_S>(lds + (cur ^ 1) * A_ELEMS, tid);
                bstore(lds + B_BASE + (cur ^ 1) * B_ELEMS);
                build_table(kt + 2, cur);  // table buffer (kt+2)&1 == cur; its old content (step kt) is dead
            }
            __syncthreads();
        }

        // epilogue: rows = oc, columns = flattened (n, p)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const long col = n0 + wn * WTN + j * MT + lrow;
            if (col >= ncols) continue;
            const long n = col / P, pp = col % P;
            float* ybase = p.Y + n * p.YC * P + pp;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const long oc = m0 + wm * WTM + i * MT + X::acc_row(lane, r);
                    if (oc < p.OC) ybase[oc * P] = acc[i][j][r] + (p.bias ? p.bias[oc] : 0.f);
                }
            }
        }
    }
};

} // namespace docc_k

#define DOCC_CONV_GATHER(BM, BN, BK, WM, WN, AL, ALTAG)                                                         \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void docc_conv2d_f32_gather_##BM##x##BN##_##ALTAG(     \
        docc_k::ConvParams p) {                                                                                 \
        docc_k::ConvGatherKernel<BM, BN, BK, WM, WN, AL>::run(p);                                               \
    }                                                                                                           \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void docc_conv2d_f32_gather_##BM##x##BN##_##ALTAG##_g( \
        docc_k::ConvParams p) {                                                                                 \
        docc_k::conv_select_group(p);                                                                           \
        docc_k::ConvGatherKernel<BM, BN, BK, WM, WN, AL>::run(p);                                               \
    }

DOCC_CONV_GATHER(64, 128, 16, 2, 2, true, a)
DOCC_CONV_GATHER(64, 128, 16, 2, 2, false, u)

// ---------------------------------------------------------------------------------------------
// Dilation-1 convolution with LDS-staged input halos (stride 1; strides of 2 with the small strips, whose patch still fits).
//
// One work-group computes 64 output channels x a strip of TH full output rows of one image
// (TH*OW <= 448 pixels = 14 MFMA column tiles). Wave w takes output-channel tile (w & 1) and
// pixel tiles 7*(w >> 1) .. +6, so the four waves hold the whole strip in 7 accumulators each.
// TILES = 4 or 2 instead of 7 tiles per wave (strips of 256 or 128 pixels) are for layers whose images are
// too small to give every CU a strip of 448: a work-group costs what its tiles cost, filled or not.
// K = C*KH*KW is walked in chunks of 8 input channels. Per chunk the work-group stages
//   - the input patch [TH+KH-1][OW+KW-1][8] (halo rows and columns included, zeros where the
//     patch leaves the image, the eight channels of a pixel adjacent): every input pixel is read
//     from memory once per strip instead of KH*KW times, and
//   - the weight slab [64][8*KH*KW] (contiguous in memory), stored tap-major ([oc][tap][channel]),
// into one of two LDS buffers while the previous chunk is multiplied. The k-order of the MFMA
// inside a chunk is tap-major: k-group t is filter tap t, and its eight k-values are the eight
// channels (lane half g, register s -> channel 4g+s). Both operands of the four MFMAs of a tap
// are then one 128-bit LDS read per lane: the weights at [oc][t][4g..4g+3], the pixels at
// [(r+kh)*WP + (c+kw)][4g..4g+3], whose address is a wave-uniform tap term plus a per-lane pixel
// term: im2col costs one add per read.
//
// SPLIT: a strip of 13 column tiles (at most 416 pixels). The waves of a pixel group take six tiles each and
// share the thirteenth: in every chunk group 0 multiplies it over the first half of the chunk's k-slices, group 1
// over the second half (the work-group meets at a barrier per chunk, so the halves must balance inside a chunk),
// and the two partial tiles are added through LDS before the store. Both groups run the same instructions: the
// shared tile has operand registers of its own, and group 1 simply fetches them from the mirrored tap (tap 8 - t
// where group 0 reads tap t; of the middle tap each takes two of the four slices). A wave then carries 6.5 tiles instead
// of 7, which is what lets 8 strips of 7 rows (one work-group on each of 256 CUs) beat 7 strips of 8 rows on a
// 56x56 image: both are one round of work-groups, and the round is as long as its waves' MFMA count.
//
// NARROW: the shared tile holds at most 16 pixels of the strip (8 of 392 on a 56-wide image). It is then multiplied
// with the 16x16x4 MFMA - two of them for the wave's 32 output channels and four of a tap's eight channels, half the
// matrix-pipe time of the 32-pixel form - from operands read as single words: lane l holds the weight of output
// channel l % 16 and the pixel l % 16 for channel l / 16 (+ 4 for the tap's second half). The two pixel groups still
// share it by taps, the middle tap by its channel halves.
#ifndef DOCC_CONV_EARLY_STORE
#define DOCC_CONV_EARLY_STORE 1
#endif

namespace docc_k {

template <int KH, int KW, bool SPLIT = false, bool NARROW = false, int TILES = 7, bool MULTI = false>
struct ConvHaloKernel {
    static_assert(!MULTI || !SPLIT, "several images per work-group: the plain strips only");
    static_assert(!NARROW || SPLIT, "the narrow tile is the shared tile of a split strip");
    static_assert(TILES >= 2 && (!SPLIT || TILES == 7), "the last chunk goes in groups of at least two tiles; the split strip is 13 tiles");
    static constexpr int KHW = KH * KW;
    static constexpr int CI = 8;                 // input channels per chunk
    static constexpr int KC = CI * KHW;          // k per chunk
    static constexpr int TN = TILES;             // MFMA column tiles per wave (SPLIT: the seventh is the shared one)
    static constexpr int TOWN = SPLIT ? TN - 1 : TN;   // column tiles a wave has to itself
    static constexpr int LDA_S = KC + 4;
    static constexpr int A_ELEMS = 64 * LDA_S;
    static constexpr int NR = 3;                 // patch pixels per thread per chunk (upper bound)
    static constexpr int NWV = (64 * KC / 4 + 255) / 256;   // weight float4s per thread per chunk

    // MULTI: a work-group takes G whole images (TH == OH; images of a few pixels, which alone would fill a fraction of
    // the smallest strip): the patch buffer holds their G patches one after the other, pixel q of the strip is pixel
    // q % (OH * OW) of image q / (OH * OW).
    static __device__ __forceinline__ void run(const ConvParams& p, int TH, int G = 1) {
        extern __shared__ __attribute__((aligned(16))) unsigned char docc_conv_lds[];
        float* const lds = reinterpret_cast<float*>(docc_conv_lds);
        const int tid = threadIdx.x, lane = tid & 63, wave = SPLIT ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;   // SPLIT: the mirrored tap is a scalar
        const int l32 = lane & 31, g = lane >> 5;
        const int ocw = wave & 1, pg = wave >> 1;

        const int WP = (p.OW - 1) * p.stride_w + KW, PR = (TH - 1) * p.stride_h + KH, PS = PR * WP;   // the patch a strip reads
        const int PST = MULTI ? G * PS : PS;                // patch pixels of the work-group
        const int stage_elems = A_ELEMS + (PST + 1) * CI;   // [weights | patch | one spare pixel]
        const int strips = (p.OH + TH - 1) / TH;
        const int n = MULTI ? blockIdx.x * G : blockIdx.x / strips, oh0 = MULTI ? 0 : (blockIdx.x % strips) * TH;
        const int oc0 = blockIdx.y * 64;
        const int ipix = p.OH * p.OW;                  // MULTI: pixels of an image
        const int npix = MULTI ? G * ipix : TH * p.OW; // pixels of a full strip

        // per-lane patch offsets (floats) of the 7 column tiles of this wave: pixel (r, c) of the
        // strip and the channel half of this lane
        // first pixel of column tile j of this wave
        auto tile_pixel0 = [&](int j) { return j < TOWN ? (pg * TOWN + j) * 32 : 2 * TOWN * 32; };
        int boff[TN];
        // (filled in below, while the first chunk's loads are under way)
        auto pixel_offsets = [&]() {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                int q = tile_pixel0(j) + l32;
                q = q < npix ? q : 0;
                int patch0 = 0;
                if constexpr (MULTI) {
                    patch0 = (q / ipix) * PS;
                    q %= ipix;
                }
                boff[j] = (patch0 + (q / p.OW) * p.stride_h * WP + (q % p.OW) * p.stride_w) * CI + 4 * g;
            }
        };

        // patch pixels this thread moves per chunk: byte offset inside one channel plane (0 when the
        // value is a zero of the padding), validity, and the LDS pixel slot (the spare one for
        // threads beyond the patch)
        unsigned goff[NR];
        int slot[NR];
        bool inside[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const int e = tid + r * 256;
            const int img = MULTI ? e / PS : 0, pe = MULTI ? e % PS : e;      // image of the group, pixel of its patch
            const int ih = oh0 * p.stride_h - p.pad_h + pe / WP, iw = pe % WP - p.pad_w;
            inside[r] = e < PST && n + img < p.N && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            goff[r] = inside[r] ? 4u * (unsigned) (img * p.XC * p.H * p.W + ih * p.W + iw) : 0u;
            slot[r] = (e < PST ? e : PST) * CI;
        }
        const long HW = (long) p.H * p.W;
        const char* xn = reinterpret_cast<const char*>(p.X + (long) n * p.XC * HW);
        const int K = p.C * KHW;
        // weight slab: memory holds [oc][channel][tap], LDS wants [oc][tap][channel]. Each of this
        // thread's vectors is four channels of one (oc, tap): four loads KHW floats apart, one
        // 128-bit LDS write (surplus threads aim at the spare pixel).
        unsigned woff[NWV];
        int wdst[NWV];
#pragma unroll
        for (int i = 0; i < NWV; i++) {
            const int idx = tid + i * 256;
            const int row = idx / (KC / 4), rem = idx % (KC / 4);     // rem = 2*tap + channel half
            const int oc = oc0 + row < p.OC ? oc0 + row : p.OC - 1;
            woff[i] = 4u * (unsigned) (oc * K + (rem & 1) * 4 * KHW + (rem >> 1));
            wdst[i] = idx < 64 * (KC / 4) ? row * LDA_S + rem * 4 : A_ELEMS + PST * CI;
        }

        f32x16 acc[TN];
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][r] = 0.f;

        // loads of one chunk: a wave-uniform base per channel plane plus the lane's 32-bit offset
        float pv[NR][CI];
        f32x4 wv[NWV];
        // the staging work of one chunk in NSL slices: patch pixel i, or weight vector i - NR
        constexpr int NSL = NR + NWV;
        auto gload_slice = [&](int i, int ch) {
            if (i < NR) {
                const char* xc = xn + (long) ch * CI * HW * 4;
#pragma unroll
                for (int c = 0; c < CI; c++) pv[i][c] = *reinterpret_cast<const float*>(xc + (long) c * HW * 4 + goff[i]);
            } else {
                const char* wc = reinterpret_cast<const char*>(p.Wt + ch * KC);
#pragma unroll
                for (int e = 0; e < 4; e++) wv[i - NR][e] = *reinterpret_cast<const float*>(wc + woff[i - NR] + e * KHW * 4);
            }
        };
        auto gload = [&](int ch) {
#pragma unroll
            for (int i = 0; i < NSL; i++) gload_slice(i, ch);
        };
        auto stage_slice = [&](int i, int base) {
            float* as = lds + base;
            if (i < NR) {
                float* ps = as + A_ELEMS + slot[i];
                f32x4 lo, hi;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    lo[c] = inside[i] ? pv[i][c] : 0.f;
                    hi[c] = inside[i] ? pv[i][4 + c] : 0.f;
                }
                *reinterpret_cast<f32x4*>(ps) = lo;
                *reinterpret_cast<f32x4*>(ps + 4) = hi;
            } else {
                *reinterpret_cast<f32x4*>(as + wdst[i - NR]) = wv[i - NR];
            }
        };

        // The chunks form one stream of taps over a ring of three LDS buffers. While chunk ch is
        // multiplied out of buffer cur, chunk ch+1 (its loads were issued a chunk earlier) is written
        // into buffer nxt in slices spread over the taps T0..TB, each slice followed by the loads
        // that refill its registers with chunk ch+2 (a burst of all loads at once would back up the
        // address path and stall the wave), and the work-group meets at its one barrier per chunk. The last tap of the chunk already prefetches the first
        // operands of the next one, so the matrix pipe never waits for the barrier and an LDS round
        // trip in a row. Three buffers because a wave that has passed the barrier of chunk ch writes
        // buffer (ch+2)%3 while a slower wave may still read (ch)%3 and everyone reads (ch+1)%3 next.
        constexpr int T0 = 0;
        constexpr int TB = KHW > 1 ? KHW - 2 : 0;
        f32x4 a[2], b[2][TN];
        f32x4 a6[2];                                     // SPLIT: the shared tile's own weight operand (its pixels: b[.][TN - 1])
        float an6[2][2][2], bn6[2][2];                   // NARROW: weights [operand set][channel tile of 16][half of the tap], pixels [set][half]
        f32x4 accn[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};   // NARROW: the shared tile, 16 channels x 16 pixels each
        // NARROW: first pixel of the shared tile for this lane (lane % 16), as a patch offset, and the lane's channel of four
        int boffn = 0;
        auto narrow_pixel_offset = [&]() {
            if constexpr (NARROW) {
                int q = 2 * TOWN * 32 + (lane & 15);
                q = q < npix ? q : 0;
                boffn = ((q / p.OW) * p.stride_h * WP + (q % p.OW) * p.stride_w) * CI + (lane >> 4);
            }
        };
        static_assert(!SPLIT || KHW % 2 == 1, "the shared tile is halved in the middle tap");
        // slices of tap t that go into the shared tile (code order; group 1 maps them to the mirrored tap)
        auto shared_slices = [](int t) constexpr { return !SPLIT ? 4 : 4 * t + 4 <= 2 * KHW ? 4 : 4 * t < 2 * KHW ? 2 : 0; };
        // NARROW: the shared tile's operands of (code-order) tap t; group 1 reads the mirrored tap, of the middle tap each its half
        auto read_narrow = [&](int base, int t, float (&an)[2][2], float (&bn)[2]) {
            const int n6 = shared_slices(t);        // 4: both halves of the tap's channels, 2: one half
            if (n6 == 0) return;
            const int tt = pg ? KHW - 1 - t : t;                   // wave-uniform
            const int sh = (pg && n6 == 2) ? 4 : 0;                // the middle tap: group 1 takes its upper four channels
            const float* arown = lds + base + (ocw * 32 + (lane & 15)) * LDA_S + (lane >> 4) + tt * CI + sh;
            const float* bnp = lds + base + A_ELEMS + ((tt / KW) * WP + (tt % KW)) * CI + boffn + sh;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (h == 1 && n6 == 2) break;
                an[0][h] = arown[4 * h];
                an[1][h] = arown[16 * LDA_S + 4 * h];
                bn[h] = bnp[4 * h];
            }
        };
        auto fetch = [&](int base, int t, int to) {
            const float* arow = lds + base + (ocw * 32 + l32) * LDA_S + 4 * g + t * CI;
            a[to] = *reinterpret_cast<const f32x4*>(arow);
            const float* bt = lds + base + A_ELEMS + ((t / KW) * WP + (t % KW)) * CI;     // wave-uniform
#pragma unroll
            for (int j = 0; j < TOWN; j++) b[to][j] = *reinterpret_cast<const f32x4*>(bt + boff[j]);
            if constexpr (NARROW) {
                read_narrow(base, t, an6[to], bn6[to]);
            } else if constexpr (SPLIT) {
                const int n6 = shared_slices(t);
                if (n6 > 0) {
                    const int tt = pg ? KHW - 1 - t : t;                   // wave-uniform
                    const int sh = (pg && n6 == 2) ? 2 : 0;                // the middle tap: group 1 takes its upper two slices
                    const float* arow6 = lds + base + (ocw * 32 + l32) * LDA_S + 4 * g + tt * CI + sh;
                    const float* b6 = lds + base + A_ELEMS + ((tt / KW) * WP + (tt % KW)) * CI + boff[TN - 1] + sh;
                    if (n6 == 4) {
                        a6[to] = *reinterpret_cast<const f32x4*>(arow6);
                        b[to][TN - 1] = *reinterpret_cast<const f32x4*>(b6);
                    } else {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        const f32x2 av = *reinterpret_cast<const f32x2*>(arow6), bv = *reinterpret_cast<const f32x2*>(b6);
                        a6[to][0] = av[0], a6[to][1] = av[1];
                        b[to][TN - 1][0] = bv[0], b[to][TN - 1][1] = bv[1];
                    }
                }
            }
        };
        // par: parity of the chunk's first tap in the tap stream (operand registers alternate per tap).
        // Each tap is one scheduling region: its 28 MFMAs, the LDS reads of the next tap's operands,
        // and the staging slices that fall on it with their refill loads. The group barriers at the
        // end of the region lay these out as "one MFMA, then one LDS read or one LDS write and one
        // load" so that the matrix pipe is fed while the other pipes work.
        float bias_r[16];
        float biasn[2][4];                               // NARROW: bias of the shared tile's rows (channel tile, accumulator register)
        auto load_biasn = [&]() {
            if constexpr (NARROW) {
#pragma unroll
                for (int sub = 0; sub < 2; sub++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int oc = oc0 + ocw * 32 + sub * 16 + 4 * (lane >> 4) + r;
                        biasn[sub][r] = p.bias ? p.bias[oc < p.OC ? oc : p.OC - 1] : 0.f;
                    }
            }
        };
        auto step = [&](auto par_c, auto has_next_c, int cur, int nxt, int after) {
            constexpr int PAR = decltype(par_c)::value;
            constexpr bool NEXT = decltype(has_next_c)::value;
            if constexpr (!NEXT) {
                // bias of this lane's 16 accumulator rows, fetched under the last chunk
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int oc = oc0 + ocw * 32 + Mfma<float>::acc_row(lane, r);
                    bias_r[r] = p.bias ? p.bias[oc < p.OC ? oc : p.OC - 1] : 0.f;
                }
                load_biasn();
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int t = 0; t < KHW; t++) {
                const int so = (t + PAR) & 1;
                const bool reads = t + 1 < KHW || (NEXT && KHW > 1);
                if (t + 1 < KHW) fetch(cur, t + 1, so ^ 1);
                else if (NEXT && KHW > 1) fetch(nxt, 0, so ^ 1);      // the barrier of this chunk is behind us
#pragma unroll
                for (int s = 0; s < 4; s++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        if (j < TOWN) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[so][s], b[so][j][s], acc[j], 0, 0, 0);
                        else if (NARROW) {
                            // slices 0 .. 3 of the code order stand for (channel tile, half of the tap): halves first
                            if (s < shared_slices(t)) accn[s & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(an6[so][s & 1][s >> 1], bn6[so][s >> 1], accn[s & 1], 0, 0, 0);
                        } else if (s < shared_slices(t)) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a6[so][s], b[so][j][s], acc[j], 0, 0, 0);
                    }
                const int nmfma = 4 * TOWN + (SPLIT ? shared_slices(t) : 0);
                // LDS reads issued in this region: the next tap's weights, its own tiles' pixels and, if it has any, the shared tile's pair
                const int tn = t + 1 < KHW ? t + 1 : 0;
                const int nreads = 1 + TOWN + (SPLIT && shared_slices(tn) > 0 ? (NARROW ? 3 : 2) : 0);
                int writes = 0, loads = 0;
                if constexpr (NEXT) {
                    const int i0 = t < T0 ? 0 : NSL * (t - T0) / (TB + 1 - T0);
                    const int i1 = t < T0 ? 0 : (t > TB ? NSL : NSL * (t + 1 - T0) / (TB + 1 - T0));
#pragma unroll
                    for (int i = i0; i < i1; i++) {
                        stage_slice(i, nxt);
                        gload_slice(i, after);
                        writes += i < NR ? 2 : 1;
                        loads += i < NR ? CI : 4;
                    }
                }
#pragma unroll
                for (int i = 0; i < nmfma; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                // MFMA
                    if (reads && i < nreads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // LDS read
                    if (i >= nreads && i - nreads < writes) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // LDS write
                    if (i >= nreads && ((i - nreads) & 1) == 0 && (i - nreads) / 2 < loads) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);    // load
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (NEXT) {
                    if (t == TB) __syncthreads();
                }
            }
            if constexpr (NEXT && KHW == 1) fetch(nxt, 0, (PAR + 1) & 1);
        };

        // The last chunk of a wave whose own tiles lie wholly inside the output goes tile by tile instead of tap by
        // tap: all 4 * KHW MFMAs of a pair of tiles (one pixel operand read per tile and tap), and the pair's results
        // stored under the MFMAs of the pair after it. Stored at the end of the kernel, the strips of all work-groups
        // leave at once and the kernel waits for memory to take them (25.7 MB: 3.4-4.3 us of 66.5 for N32 C64 56x56;
        // 1.3 us this way, against 1.1 us that the tile-by-tile order costs). Tap 0's operands are the ones the chunk
        // before has fetched.
        const bool whole = !MULTI && oc0 + 64 <= p.OC && oh0 + TH <= p.OH && (pg + 1) * (TOWN * 32) <= npix;
        const bool early = DOCC_CONV_EARLY_STORE && KHW > 1 && whole && (long) p.OH * p.OW * 64 * 4 < (1L << 31);
        const long plane = (long) p.OH * p.OW;
        auto last_tiles = [&](auto par_c, int cur) {
            constexpr int SO = decltype(par_c)::value & 1;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int oc = oc0 + ocw * 32 + Mfma<float>::acc_row(lane, r);
                bias_r[r] = p.bias ? p.bias[oc] : 0.f;
            }
            load_biasn();
            f32x4 aw[KHW];
            const float* arow = lds + cur + (ocw * 32 + l32) * LDA_S + 4 * g;
            aw[0] = a[SO];
#pragma unroll
            for (int t = 1; t < KHW; t++) aw[t] = *reinterpret_cast<const f32x4*>(arow + t * CI);
            const float* bbase = lds + cur + A_ELEMS;
            auto bread = [&](int j, int t) { return *reinterpret_cast<const f32x4*>(bbase + ((t / KW) * WP + (t % KW)) * CI + boff[j]); };
            // full rows: pixel q of the strip is q floats behind the strip's first pixel in every channel plane. A wave-uniform
            // base and 32-bit lane offsets, one per accumulator row: a store is then an accumulator read, the bias and the store
            char* const ybase = reinterpret_cast<char*>(p.Y + ((long) n * p.YC + oc0) * plane + (long) oh0 * p.OW);
            unsigned yoff[16];
#pragma unroll
            for (int r = 0; r < 16; r++)
                yoff[r] = 4u * (unsigned) ((ocw * 32 + 4 * g + 8 * (r / 4) + r % 4) * (int) plane + pg * (TOWN * 32) + l32);
            // Stores that write through the L2 (a relaxed store of device scope, the sc1 bit): an ordinary store leaves its
            // line in the XCD's L2 until the kernel ends, and the write-back of 25.7 MB then is time nothing overlaps
            // (61.7 -> 60.8 us). Non-temporal stores do not do that: 68 us.
            auto store_row = [&](int j, int r) {
                __hip_atomic_store(reinterpret_cast<float*>(ybase + yoff[r] + j * 128), acc[j][r] + bias_r[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            };
            // The tiles go in groups of two (the first group takes a third when the count is odd): consecutive MFMAs
            // on one accumulator wait for each other (tile after tile, the chunk ran 7 % longer), two tiles alternate without.
            // Under them go the reads of the pixels a tap ahead and a share of the rows of the group before.
            constexpr int NG = TOWN / 2;
            auto group_first = [](int gi) constexpr { return gi == 0 ? 0 : TOWN - 2 * (NG - gi); };
            auto group_size = [](int gi) constexpr { return gi == 0 ? TOWN - 2 * (NG - 1) : 2; };
            // rows of group gi stored under slice s of tap t of whatever follows: taps 1 .. ntaps - 1 share them out
            auto store_part = [&](int gi, int t, int s, int ntaps) {
                const int rows = 16 * group_size(gi), per_slice = (rows + 4 * (ntaps - 1) - 1) / (4 * (ntaps - 1));
                if (t >= 1) {
                    const int k0 = ((t - 1) * 4 + s) * per_slice;
#pragma unroll
                    for (int k = k0; k < k0 + per_slice && k < rows; k++) store_row(group_first(gi) + k / 16, k % 16);
                }
            };
            f32x4 bb[3][2];
#pragma unroll
            for (int u = 0; u < group_size(0); u++) bb[u][1] = bread(u, 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int gi = 0; gi < NG; gi++) {
                const int j0 = group_first(gi), nt = group_size(gi);
#pragma unroll
                for (int t = 0; t < KHW; t++) {
                    f32x4 bv[3];
#pragma unroll
                    for (int u = 0; u < nt; u++) bv[u] = t == 0 ? b[SO][j0 + u] : bb[u][t & 1];
                    if (t > 0 && t + 1 < KHW) {
#pragma unroll
                        for (int u = 0; u < nt; u++) bb[u][(t + 1) & 1] = bread(j0 + u, t + 1);
                    }
                    if (t + 1 == KHW && gi + 1 < NG) {
#pragma unroll
                        for (int u = 0; u < group_size(gi + 1); u++) bb[u][1] = bread(group_first(gi + 1) + u, 1);
                    }
                    if constexpr (NARROW) {
                        if (gi == 1 && t == 1) {
                            // have the shared tile's bias in registers now, where the first stores wait for theirs: met for
                            // the first time at the end, its loads would be waited for together with every store before
#pragma unroll
                            for (int k = 0; k < 8; k++) asm volatile("" ::"v"(biasn[k / 4][k % 4]));
                        }
                    }
                    // a region per slice pins the order: the tiles take turns, the stores sit between their MFMAs
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = 0; s < 4; s++) {
#pragma unroll
                        for (int u = 0; u < nt; u++)
                            acc[j0 + u] = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[t][s], bv[u][s], acc[j0 + u], 0, 0, 0);
                        if (gi > 0) store_part(gi - 1, t, s, KHW);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            if constexpr (NARROW) {
                // the shared tile in its narrow form: this group's half of the chunk's taps, under them the store of the last own tiles
                float anl[2][2][2], bnl[2][2];
#pragma unroll
                for (int h = 0; h < 2; h++) anl[0][0][h] = an6[SO][0][h], anl[0][1][h] = an6[SO][1][h], bnl[0][h] = bn6[SO][h];
                constexpr int NT6 = (KHW + 1) / 2;
#pragma unroll
                for (int t = 0; t < NT6; t++) {
                    if (t + 1 < NT6) read_narrow(cur, t + 1, anl[(t + 1) & 1], bnl[(t + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        if (s < shared_slices(t))
                            accn[s & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(anl[t & 1][s & 1][s >> 1], bnl[t & 1][s >> 1], accn[s & 1], 0, 0, 0);
                        store_part(NG - 1, t, s, NT6);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            } else if constexpr (SPLIT) {
                // the shared tile: this group's half of the chunk's slices, under them the store of the last own tile
                auto read6 = [&](int t, f32x4& av, f32x4& bv) {
                    const int n6 = shared_slices(t);
                    const int tt = pg ? KHW - 1 - t : t;
                    const int sh = (pg && n6 == 2) ? 2 : 0;
                    const float* arow6 = arow + tt * CI + sh;
                    const float* b6 = bbase + ((tt / KW) * WP + (tt % KW)) * CI + boff[TN - 1] + sh;
                    if (n6 == 4) {
                        av = *reinterpret_cast<const f32x4*>(arow6);
                        bv = *reinterpret_cast<const f32x4*>(b6);
                    } else {
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        const f32x2 a2 = *reinterpret_cast<const f32x2*>(arow6), b2 = *reinterpret_cast<const f32x2*>(b6);
                        av[0] = a2[0], av[1] = a2[1];
                        bv[0] = b2[0], bv[1] = b2[1];
                    }
                };
                f32x4 a6l[2], b6l[2];
                a6l[0] = a6[SO], b6l[0] = b[SO][TN - 1];
                constexpr int NT6 = (KHW + 1) / 2;       // taps with slices of the shared tile
#pragma unroll
                for (int t = 0; t < NT6; t++) {
                    const bool rd = t + 1 < NT6;
                    if (rd) read6(t + 1, a6l[(t + 1) & 1], b6l[(t + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        if (s < shared_slices(t))
                            acc[TN - 1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a6l[t & 1][s], b6l[t & 1][s], acc[TN - 1], 0, 0, 0);
                        store_part(NG - 1, t, s, NT6);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            } else {
#pragma unroll
                for (int k = 0; k < 16 * group_size(NG - 1); k++) store_row(group_first(NG - 1) + k / 16, k % 16);
            }
        };

        const int nch = p.C / CI;
        gload(0);
        // the index arithmetic nothing needs before the first operand read goes here, under the loads' way to memory and back
        // (left to the compiler it lands behind the barrier, in front of the first MFMA)
        pixel_offsets();
        narrow_pixel_offset();
        // (an empty asm that takes the value: without it the arithmetic is moved to the first use)
#pragma unroll
        for (int j = 0; j < TN; j++) asm volatile("" : "+v"(boff[j]));
        asm volatile("" : "+v"(boffn));
        // the accumulators are cleared here as well (112 register writes that otherwise stand between the barrier and the first MFMA)
#pragma unroll
        for (int j = 0; j < TN; j++) asm volatile("" : "+a"(acc[j]));
#pragma unroll
        for (int i = 0; i < NSL; i++) stage_slice(i, 0);
        if (nch > 1) gload(1);
        __syncthreads();
        fetch(0, 0, 0);
        // ring positions as LDS float offsets
        int cur = 0, nxt = stage_elems;
        auto advance = [&]() {
            cur = nxt;
            nxt = nxt + stage_elems;
            if (nxt == 3 * stage_elems) nxt = 0;
        };
        constexpr int P1 = KHW & 1;      // parity of the second chunk of a pair
        typedef std::integral_constant<int, 0> Par0;
        typedef std::integral_constant<int, P1> Par1;
        // epilogue: rows of the accumulator = output channels, columns = pixels of the strip. A tile
        // that lies wholly inside the output (the usual case) is stored by straight-line code; one
        // branch per element costs more in instruction fetch than the stores themselves.
        auto store_tile_checked = [&](int j, bool with_bias) {
            int q = tile_pixel0(j) + l32;
            if (q >= npix) return;
            int img = 0;
            if constexpr (MULTI) {
                img = q / ipix;
                q %= ipix;
                if (n + img >= p.N) return;
            }
            const int oh = oh0 + q / p.OW, ow = q % p.OW;
            if (oh >= p.OH) return;
            float* ybase = p.Y + ((long) (n + img) * p.YC * p.OH + oh) * p.OW + ow;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int oc = oc0 + ocw * 32 + Mfma<float>::acc_row(lane, r);
                if (oc < p.OC) ybase[(long) oc * p.OH * p.OW] = with_bias ? acc[j][r] + bias_r[r] : acc[j][r];
            }
        };
        // The shared tile takes its bias here, in group 0's half, on either path to the end: read after the paths have
        // joined, the bias registers would be waited for as loads that may still be in flight, and that wait would
        // also sit out every store issued before it.
        auto bias_shared_tile = [&]() {
            if constexpr (NARROW) {
#pragma unroll
                for (int k = 0; k < 8; k++) accn[k / 4][k % 4] += pg == 0 ? biasn[k / 4][k % 4] : 0.f;
            } else if constexpr (SPLIT) {
#pragma unroll
                for (int r = 0; r < 16; r++) acc[TN - 1][r] += pg == 0 ? bias_r[r] : 0.f;
            }
        };
        auto store_own_tiles = [&]() {
            if (whole) {
#pragma unroll
                for (int j = 0; j < TOWN; j++) {
                    const int q = tile_pixel0(j) + l32;
                    float* ybase = p.Y + ((long) n * p.YC * p.OH + oh0 + q / p.OW) * p.OW + q % p.OW +
                                   (long) (oc0 + ocw * 32 + 4 * g) * p.OH * p.OW;
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        ybase[(long) (8 * (r / 4) + r % 4) * p.OH * p.OW] = acc[j][r] + bias_r[r];
                }
            } else {
#pragma unroll
                for (int j = 0; j < TOWN; j++) store_tile_checked(j, true);
            }
        };
        // the last chunk, after which only the shared tile is still to be stored (the two forms are separate paths to
        // the end of the own tiles: joined earlier, their accumulators would have to meet in the same registers)
        auto last_chunk = [&](auto par_c) {
            if (early) {
                last_tiles(par_c, cur);
                bias_shared_tile();
            } else {
                step(par_c, std::false_type{}, cur, nxt, 0);
                bias_shared_tile();
                store_own_tiles();
            }
        };
        {
            int ch = 0;
            for (; ch + 2 < nch; ch += 2) {
                step(Par0{}, std::true_type{}, cur, nxt, ch + 2);
                advance();
                step(Par1{}, std::true_type{}, cur, nxt, ch + 3 < nch ? ch + 3 : nch - 1);
                advance();
            }
            if (ch + 2 == nch) {
                step(Par0{}, std::true_type{}, cur, nxt, nch - 1);
                advance();
                last_chunk(Par1{});
            } else {
                last_chunk(Par0{});
            }
        }
        if constexpr (NARROW) {
            // The two halves of the shared tile meet in LDS, [channel tile of 32][accumulator register][lane]; group 0 stores
            // the sum. They meet in the ring's third buffer, the one after the last chunk's: what it held was read two chunks
            // ago, before the barrier every wave has passed to get here, so group 1 can write without another barrier.
            float* xch = lds + nxt + ocw * (8 * 64);
            if (pg == 1) {
#pragma unroll
                for (int k = 0; k < 8; k++) xch[k * 64 + lane] = accn[k / 4][k % 4];
            }
            __syncthreads();
            if (pg == 0) {
                const int q = 2 * TOWN * 32 + (lane & 15);
                const int oh = oh0 + q / p.OW, ow = q % p.OW;
                if (q < npix && oh < p.OH) {
                    float* ybase = p.Y + ((long) n * p.YC * p.OH + oh) * p.OW + ow;
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        const int oc = oc0 + ocw * 32 + (k / 4) * 16 + 4 * (lane >> 4) + k % 4;
                        if (oc < p.OC) ybase[(long) oc * p.OH * p.OW] = accn[k / 4][k % 4] + xch[k * 64 + lane];
                    }
                }
            }
        } else if constexpr (SPLIT) {
            // the two halves of the shared tile meet in LDS (the ring's free buffer, as above), [channel tile][accumulator register][lane]
            float* xch = lds + nxt + ocw * (16 * 64);
            if (pg == 1) {
#pragma unroll
                for (int r = 0; r < 16; r++) xch[r * 64 + lane] = acc[TN - 1][r];
            }
            __syncthreads();
            if (pg == 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) acc[TN - 1][r] += xch[r * 64 + lane];
                store_tile_checked(TN - 1, false);
            }
        }
    }
};

} // namespace docc_k

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<3, 3>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3>::run(p, TH);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<1, 1>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<1, 1>::run(p, TH);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t4(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<3, 3, false, false, 4>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t4_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3, false, false, 4>::run(p, TH);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t2(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<3, 3, false, false, 2>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t2_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3, false, false, 2>::run(p, TH);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t4(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<1, 1, false, false, 4>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t4_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<1, 1, false, false, 4>::run(p, TH);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t2(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<1, 1, false, false, 2>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t2_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<1, 1, false, false, 2>::run(p, TH);
}

// several whole images per work-group (images of a few pixels)
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t4m(docc_k::ConvParams p, int TH, int G) {
    docc_k::ConvHaloKernel<3, 3, false, false, 4, true>::run(p, TH, G);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t4m_g(docc_k::ConvParams p, int TH, int G) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3, false, false, 4, true>::run(p, TH, G);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t2m(docc_k::ConvParams p, int TH, int G) {
    docc_k::ConvHaloKernel<3, 3, false, false, 2, true>::run(p, TH, G);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_t2m_g(docc_k::ConvParams p, int TH, int G) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3, false, false, 2, true>::run(p, TH, G);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t4m(docc_k::ConvParams p, int TH, int G) {
    docc_k::ConvHaloKernel<1, 1, false, false, 4, true>::run(p, TH, G);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t4m_g(docc_k::ConvParams p, int TH, int G) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<1, 1, false, false, 4, true>::run(p, TH, G);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t2m(docc_k::ConvParams p, int TH, int G) {
    docc_k::ConvHaloKernel<1, 1, false, false, 2, true>::run(p, TH, G);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_1x1_t2m_g(docc_k::ConvParams p, int TH, int G) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<1, 1, false, false, 2, true>::run(p, TH, G);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_split(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<3, 3, true>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_split_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3, true>::run(p, TH);
}

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_split16(docc_k::ConvParams p, int TH) {
    docc_k::ConvHaloKernel<3, 3, true, true>::run(p, TH);
}
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_f32_halo_3x3_split16_g(docc_k::ConvParams p, int TH) {
    docc_k::conv_select_group(p);
    docc_k::ConvHaloKernel<3, 3, true, true>::run(p, TH);
}

// Explicit im2col for the layers the two kernels above serve badly (small images, many channels): the
// columns of images n0 .. n0+nn-1 as one row-major matrix col[K = C*KH*KW][nn * OH*OW], zero where a tap
// leaves the image, so that the convolution is one GEMM  W[OC][K] x col  into [OC][nn * OH*OW].
// Thread = one column (image, pixel), blockIdx.y walks the K rows: writes are contiguous, reads follow ow.
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_im2col_f32(docc_k::ConvParams p, int n0, int nn, float* col) {
    const int P = p.OH * p.OW, K = p.C * p.KH * p.KW;
    const long cols = (long) nn * P;
    const long j = (long) blockIdx.x * 256 + threadIdx.x;
    if (j >= cols) return;
    const int n = n0 + (int) (j / P), pix = (int) (j % P);
    const int oh = pix / p.OW, ow = pix % p.OW;
    const int ih0 = oh * p.stride_h - p.pad_h, iw0 = ow * p.stride_w - p.pad_w;
    const float* x = p.X + (long) n * p.XC * p.H * p.W;
    for (int kk = blockIdx.y; kk < K; kk += gridDim.y) {
        const int c = kk / (p.KH * p.KW), t = kk % (p.KH * p.KW);
        const int ih = ih0 + (t / p.KW) * p.dil_h, iw = iw0 + (t % p.KW) * p.dil_w;
        const bool inside = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
        col[(long) kk * cols + j] = inside ? x[((long) c * p.H + ih) * p.W + iw] : 0.f;
    }
}

// Depthwise layers (group == C: one input channel a group, `mult` output channels from it): nine or so multiply-adds per
// output element against eight bytes moved, so the layer is bound by HBM and the MFMA tiles have nothing to do.
// A work-group takes 256 consecutive pixels of one output plane (image, output channel); the plane's filter comes through
// the scalar loads (the plane is the same for the whole work-group), the taps of neighbouring pixels share cache lines.
// p.C and p.OC are the channels of the whole tensors here. Sums in the order of the taps, the bias last (as the other kernels).
namespace docc_k {
template <int KH, int KW>   // 0, 0: the filter's extents from p
__device__ __forceinline__ void conv_depthwise(const ConvParams& p, int mult) {
    const int P = p.OH * p.OW;
    const int blocks_per_plane = (P + 255) / 256;
    const long plane = blockIdx.x / blocks_per_plane;           // n * OC + oc
    const int pix = (int) (blockIdx.x % blocks_per_plane) * 256 + threadIdx.x;
    if (pix >= P) return;
    const int n = (int) (plane / p.OC), oc = (int) (plane % p.OC);
    const int c = oc / mult;
    const int kh_n = KH ? KH : p.KH, kw_n = KW ? KW : p.KW;
    const float* x = p.X + ((long) n * p.XC + c) * p.H * p.W;
    const float* w = p.Wt + (long) oc * kh_n * kw_n;
    const int oh = pix / p.OW, ow = pix % p.OW;
    const int ih0 = oh * p.stride_h - p.pad_h, iw0 = ow * p.stride_w - p.pad_w;
    float acc = 0.f;
#pragma unroll
    for (int kh = 0; kh < kh_n; kh++) {
        const int ih = ih0 + kh * p.dil_h;
        const bool row_in = (unsigned) ih < (unsigned) p.H;
#pragma unroll
        for (int kw = 0; kw < kw_n; kw++) {
            const int iw = iw0 + kw * p.dil_w;
            const float v = row_in && (unsigned) iw < (unsigned) p.W ? x[(long) ih * p.W + iw] : 0.f;
            acc = __builtin_fmaf(v, w[kh * kw_n + kw], acc);
        }
    }
    if (p.bias) acc += p.bias[oc];
    __builtin_nontemporal_store(acc, p.Y + ((long) n * p.YC + oc) * P + pix);
}
}  // namespace docc_k

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise<3, 3>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_5x5(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise<5, 5>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise<0, 0>(p, mult); }

// The common depthwise layer - 3x3, stride 1, no dilation, one column of padding on the left, rows of a multiple of four
// pixels (OW == W) - with four output pixels a lane: a row of the window is one 128-bit load and its two neighbours, shared
// by the four outputs (18 loads and 36 multiply-adds for four outputs instead of 36 loads), the store is 128 bits. The sums
// run in the order of the kernel above.
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_v4(docc_k::ConvParams p, int mult) {
    typedef float v4 __attribute__((ext_vector_type(4)));
    const int Q = p.OH * (p.OW / 4);                       // quads of an output plane
    const int blocks_per_plane = (Q + 255) / 256;
    const long plane = blockIdx.x / blocks_per_plane;     // n * OC + oc
    const int quad = (int) (blockIdx.x % blocks_per_plane) * 256 + threadIdx.x;
    if (quad >= Q) return;
    const int n = (int) (plane / p.OC), oc = (int) (plane % p.OC);
    const float* x = p.X + ((long) n * p.XC + oc / mult) * p.H * p.W;
    const float* w = p.Wt + (long) oc * 9;
    const int oh = quad / (p.OW / 4), ow = (quad % (p.OW / 4)) * 4;
    v4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kh = 0; kh < 3; kh++) {
        const int ih = oh - p.pad_h + kh;
        v4 mid = {0.f, 0.f, 0.f, 0.f};
        float left = 0.f, right = 0.f;
        if ((unsigned) ih < (unsigned) p.H) {
            const float* row = x + (long) ih * p.W;
            mid = *reinterpret_cast<const v4*>(row + ow);
            if (ow > 0) left = row[ow - 1];
            if (ow + 4 < p.W) right = row[ow + 4];
        }
        const float in[6] = {left, mid[0], mid[1], mid[2], mid[3], right};
#pragma unroll
        for (int kw = 0; kw < 3; kw++) {
            const float wt = w[kh * 3 + kw];
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] = __builtin_fmaf(in[e + kw], wt, acc[e]);
        }
    }
    if (p.bias) {
        const float b = p.bias[oc];
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] += b;
    }
    __builtin_nontemporal_store(acc, reinterpret_cast<v4*>(p.Y + ((long) n * p.YC + oc) * p.OH * p.OW + (long) oh * p.OW + ow));
}

// The same layer with R output rows of the quad a lane: the R + 2 input row segments are loaded once (3 (R + 2) loads for 4 R
// outputs instead of 9 R) and all before the first multiply-add, so a lane has that many loads in flight; the lanes count
// through (plane, block of R rows, quad of the row), so a wavefront runs over plane borders and none of its lanes idles on a
// plane that is no multiple of 256 quads (a 56 x 56 plane: 784). The filter differs between the lanes of a wavefront and
// comes through vector loads, nine for 4 R outputs. Each output sums in the order of the kernel above.
namespace docc_k {
template <int R>
__device__ __forceinline__ void conv_depthwise_3x3_v4_rows(const ConvParams& p, int mult) {
    typedef float v4 __attribute__((ext_vector_type(4)));
    const unsigned qw = (unsigned) p.OW / 4, rbs = ((unsigned) p.OH + R - 1) / R;
    const unsigned per_plane = qw * rbs;
    const unsigned item = blockIdx.x * 256u + threadIdx.x;     // the host keeps the count of items below 2^31
    const unsigned plane = item / per_plane;                   // n * OC + oc
    if (plane >= (unsigned) p.N * (unsigned) p.OC) return;
    const unsigned rest = item - plane * per_plane;
    const int ow = (int) (rest % qw) * 4, oh0 = (int) (rest / qw) * R;
    const int n = (int) (plane / (unsigned) p.OC), oc = (int) (plane % (unsigned) p.OC);
    const float* x = p.X + ((long) n * p.XC + oc / mult) * p.H * p.W;
    const float* w = p.Wt + (long) oc * 9;
    float wt[9];
#pragma unroll
    for (int t = 0; t < 9; t++) wt[t] = w[t];
    float in[R + 2][6];
#pragma unroll
    for (int j = 0; j < R + 2; j++) {
        const int ih = oh0 - p.pad_h + j;
        v4 mid = {0.f, 0.f, 0.f, 0.f};
        float left = 0.f, right = 0.f;
        if ((unsigned) ih < (unsigned) p.H) {
            const float* row = x + (long) ih * p.W;
            mid = *reinterpret_cast<const v4*>(row + ow);
            if (ow > 0) left = row[ow - 1];
            if (ow + 4 < p.W) right = row[ow + 4];
        }
        in[j][0] = left; in[j][1] = mid[0]; in[j][2] = mid[1]; in[j][3] = mid[2]; in[j][4] = mid[3]; in[j][5] = right;
    }
    const float b = p.bias ? p.bias[oc] : 0.f;
    float* y = p.Y + ((long) n * p.YC + oc) * p.OH * p.OW + ow;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (oh0 + r >= p.OH) break;
        v4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kh = 0; kh < 3; kh++)
#pragma unroll
            for (int kw = 0; kw < 3; kw++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] = __builtin_fmaf(in[r + kh][e + kw], wt[kh * 3 + kw], acc[e]);
        if (p.bias) {
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] += b;
        }
        __builtin_nontemporal_store(acc, reinterpret_cast<v4*>(y + (long) (oh0 + r) * p.OW));
    }
}
}  // namespace docc_k

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_v4_r4(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_3x3_v4_rows<4>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_v4_r7(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_3x3_v4_rows<7>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_v4_r8(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_3x3_v4_rows<8>(p, mult); }

// 3x3 depthwise layers whose rows are no whole aligned quads (14 x 14 and 7 x 7 planes) or that step by two, and 5x5 ones: a lane
// takes one output column and R output rows, loads the (R - 1) S + K input rows of its K columns once and before the first
// multiply-add, and the lanes count through (plane, block of rows, column) as above: a 7 x 7 plane fills 7 lanes instead of
// 49 of a work-group's 256, and a lane loads 27 + 9 values for seven outputs instead of 18 for one. Sums in the same order.
namespace docc_k {
template <int R, int S, int K>   // K x K filter
__device__ __forceinline__ void conv_depthwise_rows(const ConvParams& p, int mult) {
    const unsigned ow_n = (unsigned) p.OW, rbs = ((unsigned) p.OH + R - 1) / R;
    const unsigned per_plane = ow_n * rbs;
    const unsigned item = blockIdx.x * 256u + threadIdx.x;     // the host keeps the count of items below 2^31
    const unsigned plane = item / per_plane;                   // n * OC + oc
    if (plane >= (unsigned) p.N * (unsigned) p.OC) return;
    const unsigned rest = item - plane * per_plane;
    const int ow = (int) (rest % ow_n), oh0 = (int) (rest / ow_n) * R;
    const int n = (int) (plane / (unsigned) p.OC), oc = (int) (plane % (unsigned) p.OC);
    const float* x = p.X + ((long) n * p.XC + oc / mult) * p.H * p.W;
    const float* w = p.Wt + (long) oc * (K * K);
    float wt[K * K];
#pragma unroll
    for (int t = 0; t < K * K; t++) wt[t] = w[t];
    constexpr int ROWS = (R - 1) * S + K;
    float in[ROWS][K];
    const int iw0 = ow * S - p.pad_w, ih0 = oh0 * S - p.pad_h;
#pragma unroll
    for (int j = 0; j < ROWS; j++) {
        const int ih = ih0 + j;
        const bool row_in = (unsigned) ih < (unsigned) p.H;
        const float* row = x + (long) ih * p.W;
#pragma unroll
        for (int kw = 0; kw < K; kw++) in[j][kw] = row_in && (unsigned) (iw0 + kw) < (unsigned) p.W ? row[iw0 + kw] : 0.f;
    }
    const float b = p.bias ? p.bias[oc] : 0.f;
    float* y = p.Y + ((long) n * p.YC + oc) * p.OH * p.OW + ow;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (oh0 + r >= p.OH) break;
        float acc = 0.f;
#pragma unroll
        for (int kh = 0; kh < K; kh++)
#pragma unroll
            for (int kw = 0; kw < K; kw++) acc = __builtin_fmaf(in[r * S + kh][kw], wt[kh * K + kw], acc);
        if (p.bias) acc += b;
        __builtin_nontemporal_store(acc, y + (long) (oh0 + r) * p.OW);
    }
}
}  // namespace docc_k

extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_s1_r4(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<4, 1, 3>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_s1_r7(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<7, 1, 3>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_s2_r4(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<4, 2, 3>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_3x3_s2_r7(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<7, 2, 3>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_5x5_s1_r4(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<4, 1, 5>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_5x5_s1_r7(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<7, 1, 5>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_5x5_s2_r4(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<4, 2, 5>(p, mult); }
extern "C" __global__ __launch_bounds__(256) void docc_conv2d_depthwise_f32_5x5_s2_r7(docc_k::ConvParams p, int mult) { docc_k::conv_depthwise_rows<7, 2, 5>(p, mult); }

// Groups of a few channels (a ResNeXt layer: 32 groups of 4 or 8 channels in, as many out): per output element the layer does
// C/group * 9 multiply-adds against eight bytes moved, so it is bound by HBM like the depthwise one, and a 64-row MFMA tile
// would hold 4 or 8 real output channels. 3x3, stride 1, no dilation, one column of padding, rows of whole aligned quads (as
// the depthwise kernel above): a lane takes four output pixels of OGT output channels of one group, every input row segment it
// loads (one 128-bit load and its two neighbours) serves the four pixels, the three taps of the row and the OGT channels; the
// group's filters wait in LDS and are read by all lanes at once. Work-group = (image, group, OGT channels of it, 256 quads).
namespace docc_k {
template <int OGT>
__device__ __forceinline__ void conv_small_groups_3x3_v4(const ConvParams& p, int cg, int og) {
    typedef float v4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) unsigned char conv_sg_lds[];
    float* wl = reinterpret_cast<float*>(conv_sg_lds);   // [OGT][cg][9]
    const int Q = p.OH * (p.OW / 4);
    const int blocks_per_plane = (Q + 255) / 256;
    const int chunks = og / OGT;                           // OGT divides og
    long b = blockIdx.x;
    const int qblock = (int) (b % blocks_per_plane);
    b /= blocks_per_plane;
    const int chunk = (int) (b % chunks);
    b /= chunks;
    const int groups = p.OC / og;
    const int grp = (int) (b % groups), n = (int) (b / groups);
    const int oc0 = grp * og + chunk * OGT;
    for (int i = threadIdx.x; i < OGT * cg * 9; i += 256) wl[i] = p.Wt[(long) oc0 * cg * 9 + i];
    __syncthreads();
    const int quad = qblock * 256 + threadIdx.x;
    if (quad >= Q) return;
    const int oh = quad / (p.OW / 4), ow = (quad % (p.OW / 4)) * 4;
    v4 acc[OGT];
#pragma unroll
    for (int o = 0; o < OGT; o++) acc[o] = v4{0.f, 0.f, 0.f, 0.f};
    const float* x = p.X + ((long) n * p.XC + (long) grp * cg) * p.H * p.W;
    for (int ci = 0; ci < cg; ci++) {
        const float* plane = x + (long) ci * p.H * p.W;
#pragma unroll
        for (int kh = 0; kh < 3; kh++) {
            const int ih = oh - p.pad_h + kh;
            v4 mid = {0.f, 0.f, 0.f, 0.f};
            float left = 0.f, right = 0.f;
            if ((unsigned) ih < (unsigned) p.H) {
                const float* row = plane + (long) ih * p.W;
                mid = *reinterpret_cast<const v4*>(row + ow);
                if (ow > 0) left = row[ow - 1];
                if (ow + 4 < p.W) right = row[ow + 4];
            }
            const float in[6] = {left, mid[0], mid[1], mid[2], mid[3], right};
#pragma unroll
            for (int kw = 0; kw < 3; kw++)
#pragma unroll
                for (int o = 0; o < OGT; o++) {
                    const float wt = wl[(o * cg + ci) * 9 + kh * 3 + kw];
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[o][e] = __builtin_fmaf(in[e + kw], wt, acc[o][e]);
                }
        }
    }
#pragma unroll
    for (int o = 0; o < OGT; o++) {
        const int oc = oc0 + o;
        if (p.bias) {
            const float bv = p.bias[oc];
#pragma unroll
            for (int e = 0; e < 4; e++) acc[o][e] += bv;
        }
        __builtin_nontemporal_store(acc[o], reinterpret_cast<v4*>(p.Y + ((long) n * p.YC + oc) * p.OH * p.OW + (long) oh * p.OW + ow));
    }
}
}  // namespace docc_k

// The same with R output rows of the quad a lane (OGT * R = 16 accumulator quads): an input channel's R + 2 row segments are
// loaded once for the R rows, and a filter value read from LDS serves 4 R multiply-adds instead of 4 - with one row a lane the
// kernel issued an LDS read for every four multiply-adds. The lanes of a work-group count through (image, block of rows, quad)
// for one (group, OGT channels): only the last work-group of those has idle lanes (a 56 x 56 plane of 784 quads left 240 of
// 1024 idle). Each output sums over (input channel, kh, kw) in the order of the kernel above.
namespace docc_k {
template <int OGT, int R>
__device__ __forceinline__ void conv_small_groups_3x3_v4_rows(const ConvParams& p, int cg, int og) {
    typedef float v4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) unsigned char conv_sg_lds[];
    float* wl = reinterpret_cast<float*>(conv_sg_lds);   // [OGT][cg][9]
    const unsigned qw = (unsigned) p.OW / 4, rbs = ((unsigned) p.OH + R - 1) / R;
    const unsigned per_image = qw * rbs, total = (unsigned) p.N * per_image;   // the host keeps total + 255 below 2^31
    const unsigned blocks_per = (total + 255) / 256;
    const int chunks = og / OGT;                           // OGT divides og
    unsigned b = blockIdx.x;
    const unsigned iblock = b % blocks_per;
    b /= blocks_per;
    const int chunk = (int) (b % (unsigned) chunks), grp = (int) (b / (unsigned) chunks);
    const int oc0 = grp * og + chunk * OGT;
    for (int i = threadIdx.x; i < OGT * cg * 9; i += 256) wl[i] = p.Wt[(long) oc0 * cg * 9 + i];
    __syncthreads();
    const unsigned item = iblock * 256 + threadIdx.x;
    if (item >= total) return;
    const int n = (int) (item / per_image);
    const unsigned rest = item - (unsigned) n * per_image;
    const int ow = (int) (rest % qw) * 4, oh0 = (int) (rest / qw) * R;
    v4 acc[OGT][R];
#pragma unroll
    for (int o = 0; o < OGT; o++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[o][r] = v4{0.f, 0.f, 0.f, 0.f};
    const float* x = p.X + ((long) n * p.XC + (long) grp * cg) * p.H * p.W;
    for (int ci = 0; ci < cg; ci++) {
        const float* plane = x + (long) ci * p.H * p.W;
        float in[R + 2][6];
#pragma unroll
        for (int j = 0; j < R + 2; j++) {
            const int ih = oh0 - p.pad_h + j;
            v4 mid = {0.f, 0.f, 0.f, 0.f};
            float left = 0.f, right = 0.f;
            if ((unsigned) ih < (unsigned) p.H) {
                const float* row = plane + (long) ih * p.W;
                mid = *reinterpret_cast<const v4*>(row + ow);
                if (ow > 0) left = row[ow - 1];
                if (ow + 4 < p.W) right = row[ow + 4];
            }
            in[j][0] = left; in[j][1] = mid[0]; in[j][2] = mid[1]; in[j][3] = mid[2]; in[j][4] = mid[3]; in[j][5] = right;
        }
#pragma unroll
        for (int kh = 0; kh < 3; kh++)
#pragma unroll
            for (int kw = 0; kw < 3; kw++)
#pragma unroll
                for (int o = 0; o < OGT; o++) {
                    const float wt = wl[(o * cg + ci) * 9 + kh * 3 + kw];
#pragma unroll
                    for (int r = 0; r < R; r++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[o][r][e] = __builtin_fmaf(in[r + kh][e + kw], wt, acc[o][r][e]);
                }
    }
#pragma unroll
    for (int o = 0; o < OGT; o++) {
        const int oc = oc0 + o;
        const float bv = p.bias ? p.bias[oc] : 0.f;
        float* y = p.Y + ((long) n * p.YC + oc) * p.OH * p.OW + ow;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (oh0 + r >= p.OH) break;
            if (p.bias) {
#pragma unroll
                for (int e = 0; e < 4; e++) acc[o][r][e] += bv;
            }
            __builtin_nontemporal_store(acc[o][r], reinterpret_cast<v4*>(y + (long) (oh0 + r) * p.OW));
        }
    }
}
}  // namespace docc_k

#define DOCC_CONV_SMALL_GROUPS_ROWS(OGT, R)                                                                                                      \
    extern "C" __global__ __launch_bounds__(256) void docc_conv2d_small_groups_f32_3x3_v4_o##OGT##_r##R(docc_k::ConvParams p, int cg, int og) {   \
        docc_k::conv_small_groups_3x3_v4_rows<OGT, R>(p, cg, og);                                                                                \
    }
DOCC_CONV_SMALL_GROUPS_ROWS(1, 8)
DOCC_CONV_SMALL_GROUPS_ROWS(2, 8)
DOCC_CONV_SMALL_GROUPS_ROWS(4, 4)
DOCC_CONV_SMALL_GROUPS_ROWS(8, 2)
DOCC_CONV_SMALL_GROUPS_ROWS(8, 4)

#define DOCC_CONV_SMALL_GROUPS(OGT)                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void docc_conv2d_small_groups_f32_3x3_v4_o##OGT(docc_k::ConvParams p, int cg, int og) {     \
        docc_k::conv_small_groups_3x3_v4<OGT>(p, cg, og);                                                                                  \
    }
DOCC_CONV_SMALL_GROUPS(1)
DOCC_CONV_SMALL_GROUPS(2)
DOCC_CONV_SMALL_GROUPS(4)
DOCC_CONV_SMALL_GROUPS(8)
