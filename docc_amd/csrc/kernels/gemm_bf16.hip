// bf16 x bf16 -> fp32 GEMM on gfx950 (v_mfma_f32_32x32x16_bf16):
//   C[M,N] (fp32) = alpha * op(A) * op(B) + beta * C,  A and B bf16, row-major.
//
// The reference's BLAS node has no bf16 precision
// (sdfg/include/sdfg/data_flow/library_nodes/math/blas/blas_node.h:49-55); this
// kernel backs the precision the rocm target adds. Same work decomposition as
// gemm_mfma.h (BM x BN tile per work-group, K walked through two LDS buffers,
// XCD-aware tile numbering). Operand fetch from LDS:
//   - a k-contiguous operand (A not transposed, B transposed) sits in LDS as
//     [MN][BK+8]; lane (idx = lane % 32, g = lane / 32) reads its eight
//     k-values k = 8g .. 8g+7 with one 128-bit ds_read;
//   - an mn-contiguous operand (B not transposed, A transposed) sits in LDS
//     as [BK][MN+16], the way it lies in memory; the eight k-values of a lane
//     are strided there, so they are fetched with two ds_read_b64_tr_b16: in a
//     group of 16 lanes, lane s points at 4 consecutive mn-values of k-row
//     (s / 4), columns 4 * (s % 4) .., and receives, transposed, the four
//     k-rows of column (lane % 16).
#include "gemm_mfma.h"

namespace docc_k {

typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

struct Bf16Vec {
    static constexpr int VEC = 8;
    typedef u16x8 vec_t;
};
template <>
struct Mfma<uint16_t> : Bf16Vec {};

template <int BM, int BN, int BK, int WM, int WN, bool TA, bool TB, bool ALIGNED>
struct GemmBf16Kernel {
    static constexpr int NT = 64 * WM * WN;
    static constexpr int MT = 32;
    static constexpr int KS = 16;  // k per MFMA
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int TM = WTM / MT, TN = WTN / MT;
    static constexpr bool A_KC = !TA, B_KC = TB;
    static constexpr int PADK = 8, PADM = 16;
    static constexpr int LDA_S = A_KC ? BK + PADK : BM + PADM;
    static constexpr int LDB_S = B_KC ? BK + PADK : BN + PADM;
    static constexpr int A_ELEMS = (A_KC ? BM : BK) * LDA_S;
    static constexpr int B_ELEMS = (B_KC ? BN : BK) * LDB_S;
    static_assert(BK % KS == 0, "BK must be a multiple of 16");

    typedef TileLoader<uint16_t, A_KC ? BM : BK, A_KC ? BK : BM, NT, ALIGNED, A_KC> ALoader;
    typedef TileLoader<uint16_t, B_KC ? BN : BK, B_KC ? BK : BN, NT, ALIGNED, B_KC> BLoader;

    // eight k-values (k0 .. k0+15 split over the two lane halves) of row/column `idx0 + lane % 32`
    template <bool KC, int LD>
    static __device__ __forceinline__ bf16x8 fetch(const uint16_t* tile, int idx0, int k0, int lane) {
        if (KC) {
            const u16x8 v = *reinterpret_cast<const u16x8*>(tile + (idx0 + (lane & 31)) * LD + k0 + 8 * (lane >> 5));
            return __builtin_bit_cast(bf16x8, v);
        } else {
            const int s = lane & 15, grp = lane >> 4;
            const int row = k0 + 8 * (grp >> 1) + (s >> 2);
            const int col = idx0 + 16 * (grp & 1) + 4 * (s & 3);
            typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) (tile + row * LD + col));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) (tile + (row + 4) * LD + col));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return __builtin_bit_cast(bf16x8, v);
        }
    }

    static __device__ __forceinline__ void run(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B,
                                               float* __restrict__ C, long M, long N, long K, long lda, long ldb,
                                               long ldc, float alpha, float beta, const float* bias, int act) {
        extern __shared__ __attribute__((aligned(16))) unsigned char docc_gemm_lds[];
        uint16_t* const lds = reinterpret_cast<uint16_t*>(docc_gemm_lds);
        constexpr int B_BASE = 2 * A_ELEMS;

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wm = wave / WN, wn = wave % WN;
        const int tiles_m = (int) ((M + BM - 1) / BM), tiles_n = (int) ((N + BN - 1) / BN);
        int tm, tn;
        gemm_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        const long m0 = (long) tm * BM, n0 = (long) tn * BN;

        f32x16 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

        ALoader la;
        BLoader lb;
        if (A_KC) la.init(A, lda, m0, 0, M, K, tid);
        else la.init(A, lda, 0, m0, K, M, tid);
        if (B_KC) lb.init(B, ldb, n0, 0, N, K, tid);
        else lb.init(B, ldb, 0, n0, K, N, tid);

        auto compute = [&](int cur) {
            const uint16_t* as = lds + cur * A_ELEMS;
            const uint16_t* bs = lds + B_BASE + cur * B_ELEMS;
#pragma unroll
            for (int ks = 0; ks < BK / KS; ks++) {
                bf16x8 a[TM], b[TN];
#pragma unroll
                for (int i = 0; i < TM; i++) a[i] = fetch<A_KC, LDA_S>(as, wm * WTM + i * MT, ks * KS, lane);
#pragma unroll
                for (int j = 0; j < TN; j++) b[j] = fetch<B_KC, LDB_S>(bs, wn * WTN + j * MT, ks * KS, lane);
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        };
        auto stage = [&](int buf) {
            la.template store<LDA_S>(lds + buf * A_ELEMS, tid);
            lb.template store<LDB_S>(lds + B_BASE + buf * B_ELEMS, tid);
        };

        const int full = (int) (K / BK);
        const int kleft = (int) (K - (long) full * BK);
        if (full > 0) {
            la.load_full();
            lb.load_full();
        } else {
            la.load_tail(kleft, tid);
            lb.load_tail(kleft, tid);
        }
        stage(0);
        __syncthreads();
        int kt = 0;
        for (; kt + 1 < full; kt++) {
            la.advance();
            lb.advance();
            la.load_full();
            lb.load_full();
            compute(kt & 1);
            // keep the stores of step kt+1 (which wait for its loads) behind the MFMAs of step kt:
            // without this fence the scheduler hoists them and the load latency is exposed
            __builtin_amdgcn_sched_barrier(0);
            stage((kt + 1) & 1);
            __syncthreads();
        }
        if (full > 0 && kleft > 0) {
            la.advance();
            lb.advance();
            la.load_tail(kleft, tid);
            lb.load_tail(kleft, tid);
            compute(kt & 1);
            stage((kt + 1) & 1);
            __syncthreads();
            kt++;
        }
        compute(kt & 1);

        gemm_store_wave<kGemmEpilogue, TM, TN, MT, 16>(C, ldc, M, N, m0 + wm * WTM, n0 + wn * WTN, lane & 31, alpha, beta, bias, act, acc,
                                        [&](int r) { return Mfma<float>::acc_row(lane, r); });
    }
};

} // namespace docc_k

#define DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, TA, TB, TAG, AL, ALTAG)                                                  \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void DOCC_GEMM_NAME(docc_bgemm_##BM##x##BN##x##BK##_##TAG##_##ALTAG)(      \
        const uint16_t* A, const uint16_t* B, float* C, long M, long N, long K, long lda, long ldb, long ldc,       \
        float alpha, float beta, const float* bias, int act, long batch_a, long batch_b, long batch_c) {            \
        const long z = blockIdx.y;                                                                                  \
        docc_k::GemmBf16Kernel<BM, BN, BK, WM, WN, TA, TB, AL>::run(A + z * batch_a, B + z * batch_b, C + z * batch_c, M, N, K, \
                                                                    lda, ldb, ldc, alpha, beta, bias, act);         \
    }

#define DOCC_BGEMM_CONFIG(BM, BN, BK, WM, WN)                    \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, false, false, nn, true, a)  \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, false, true, nt, true, a)   \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, true, false, tn, true, a)   \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, true, true, tt, true, a)    \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, false, false, nn, false, u) \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, false, true, nt, false, u)  \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, true, false, tn, false, u)  \
    DOCC_BGEMM_ONE(BM, BN, BK, WM, WN, true, true, tt, false, u)

DOCC_BGEMM_CONFIG(128, 128, 64, 2, 2)
DOCC_BGEMM_CONFIG(256, 256, 64, 2, 2)

#ifndef DOCC_GEMM_EPILOGUE
extern "C" __global__ __launch_bounds__(256) void docc_bgemm_scale_c(float* C, long M, long N, long ldc, float beta) {
    const long total = M * N;
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        float* p = C + (i / N) * ldc + (i % N);
        *p = (beta == 0.f) ? 0.f : beta * (*p);
    }
}
#endif
