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

namespace docc_k {

struct ConvParams {
    const float* X;
    const float* Wt;
    const float* bias;
    float* Y;
    int N, C, H, W, OC, KH, KW, OH, OW;
    int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
};

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
        const float* xbase = p.X + (gn * p.C * p.H + ih0) * (long) p.W + iw0;
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
            float* ybase = p.Y + n * p.OC * P + pp;
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
    }

DOCC_CONV_GATHER(64, 128, 16, 2, 2, true, a)
DOCC_CONV_GATHER(64, 128, 16, 2, 2, false, u)
