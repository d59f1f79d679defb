// Tiled MFMA GEMM for fp32 and fp64 on gfx950:
//   C[M,N] = alpha * op(A) * op(B) + beta * C,   row-major, any M, N, K.
//
// Replaces the cblas_?gemm call the reference prints for a GEMM node
// (sdfg/src/data_flow/library_nodes/math/blas/gemm_node.cpp:474-505).
//
// Work decomposition
//   - one work-group computes a BM x BN tile of C with WM x WN wavefronts,
//     each wavefront a (BM/WM) x (BN/WN) sub-tile made of MT x MT MFMA tiles
//     (v_mfma_f32_32x32x2_f32: MT = 32; v_mfma_f64_16x16x4_f64: MT = 16);
//   - K is walked in steps of BK through two LDS buffers: while tile t is
//     multiplied from one buffer, tile t+1 travels global -> registers and is
//     stored into the other buffer, one barrier per step;
//   - the MFMA k-index is permuted so that a lane reads VK consecutive k from
//     LDS with one 128-bit load: lane group g = lane / MT owns
//     k = kg*KG + g*VK + s (s < VK), and MFMA step s consumes register s of
//     every lane. A and B use the same permutation, so the sum is unchanged;
//   - tiles are numbered so that the work-groups that land on one XCD (ids
//     congruent mod 8) cover a compact block of C and share A/B panels in
//     that XCD's L2.
#pragma once

#include "elementwise_ops.h"

// A translation unit compiled with DOCC_GEMM_EPILOGUE holds the epilogue variants of its kernels:
// same tiles, names with the suffix "_e", C = act(alpha A B + beta C + bias) in the store.
#ifdef DOCC_GEMM_EPILOGUE
#define DOCC_GEMM_NAME(base) base##_e
#else
#define DOCC_GEMM_NAME(base) base
#endif

namespace docc_k {

#ifdef DOCC_GEMM_EPILOGUE
constexpr bool kGemmEpilogue = true;
#else
constexpr bool kGemmEpilogue = false;
#endif

template <typename T>
struct Mfma;

template <>
struct Mfma<float> {
    static constexpr int MT = 32;  // MFMA tile edge
    static constexpr int G = 2;    // lane groups along k
    static constexpr int VK = 4;   // consecutive k per lane per LDS read (16 bytes)
    static constexpr int VEC = 4;  // elements per 128-bit global access
    static constexpr int NACC = 16;
    typedef f32x16 acc_t;
    typedef f32x4 vec_t;
    static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // row of accumulator register r inside the MT x MT tile (column is lane % MT)
    static __device__ __forceinline__ int acc_row(int lane, int r) { return 8 * (r / 4) + (lane / 32) * 4 + (r % 4); }
};

typedef double f64x2 __attribute__((ext_vector_type(2)));

template <>
struct Mfma<double> {
    static constexpr int MT = 16;
    static constexpr int G = 4;
    static constexpr int VK = 2;
    static constexpr int VEC = 2;
    static constexpr int NACC = 4;
    typedef f64x4 acc_t;
    typedef f64x2 vec_t;
    static __device__ __forceinline__ acc_t mfma(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int acc_row(int lane, int r) { return 4 * r + lane / 16; }
};

// Epilogue of one wave: C = alpha*acc + beta*C over its TM x TN accumulator tiles (C is not read
// when beta == 0). (row0, col0) is the wave tile's origin in C, lcol = lane % MT the lane's column,
// acc_row(r) the row of accumulator register r inside a tile for this lane. A wave tile that lies
// wholly inside C - all but the last row and column of tiles - is stored by straight-line code:
// with one bounds branch per element the instruction fetch of the cold, branchy epilogue costs
// more than the stores themselves.
// alpha * acc + beta * old with one fixed contraction (the product alpha * acc rounded, then one fused
// multiply-add), so that interior tiles, edge tiles and the fused epilogue all round alike
__device__ __forceinline__ float gemm_axpby(float alpha, float acc, float beta, float old) {
    return __builtin_fmaf(beta, old, alpha * acc);
}
__device__ __forceinline__ double gemm_axpby(double alpha, double acc, double beta, double old) {
    return __builtin_fma(beta, old, alpha * acc);
}

// Epilogue of a fused chain: C = act(alpha * A B + beta * C + bias[col]), ACT a compile-time
// UnaryOp or -1. Every step rounds as the separate nodes would (the sum is kept from contracting
// with the product before it).
template <int ACT, int TM, int TN, int MT, int NACC, typename OT, typename AccT, typename RowFn>
__device__ __forceinline__ void gemm_store_wave_epilogue(OT* C, long ldc, long M, long N, long row0, long col0, int lcol, OT alpha,
                                                         OT beta, const OT* bias, AccT (&acc)[TM][TN], RowFn acc_row) {
    const bool use_c = (beta != (OT) 0);
    const bool whole = row0 + TM * MT <= M && col0 + TN * MT <= N;
    // the bias values of this lane's columns; without a bias -0.0, whose addition changes no value
    OT b[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const long col = col0 + j * MT + lcol;
        b[j] = (bias != nullptr && (whole || col < N)) ? bias[col] : (OT) -0.0;
    }
    auto finish = [&](OT val, int j) {
        asm volatile("" : "+v"(val));   // the product is rounded before the bias is added, as by the separate nodes
        val += b[j];
        if (ACT >= 0) val = unary<ACT>(val);
        return val;
    };
    if (whole) {   // interior tile: one base address, constant offsets, no bounds tests
        OT* base = C + (row0 + acc_row(0)) * ldc + col0 + lcol;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                OT old[NACC];
                if (use_c) {
#pragma unroll
                    for (int r = 0; r < NACC; r++) old[r] = base[(long) (i * MT + acc_row(r) - acc_row(0)) * ldc + j * MT];
                }
#pragma unroll
                for (int r = 0; r < NACC; r++)
                    base[(long) (i * MT + acc_row(r) - acc_row(0)) * ldc + j * MT] =
                        finish(use_c ? gemm_axpby(alpha, (OT) acc[i][j][r], beta, old[r]) : alpha * acc[i][j][r], j);
            }
        return;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const long col = col0 + j * MT + lcol;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int r = 0; r < NACC; r++) {
                const long row = row0 + i * MT + acc_row(r);
                if (row < M && col < N) {
                    OT* p = C + row * ldc + col;
                    *p = finish(use_c ? gemm_axpby(alpha, (OT) acc[i][j][r], beta, *p) : alpha * acc[i][j][r], j);
                }
            }
    }
}

// EPI: the kernel is one of the epilogue variants (built apart from the plain kernels, whose
// register allocation must not carry the activation code); bias / act are ignored otherwise.
template <bool EPI, int TM, int TN, int MT, int NACC, typename OT, typename AccT, typename RowFn>
__device__ __forceinline__ void gemm_store_wave(OT* C, long ldc, long M, long N, long row0, long col0, int lcol,
                                                OT alpha, OT beta, const OT* bias, int act, AccT (&acc)[TM][TN], RowFn acc_row) {
    if constexpr (EPI) {
#define DOCC_EPILOGUE_CASE(ACT) \
    gemm_store_wave_epilogue<ACT, TM, TN, MT, NACC>(C, ldc, M, N, row0, col0, lcol, alpha, beta, bias, acc, acc_row)
        // only the activations that cost one instruction are built into the store: each case is a fully
        // unrolled copy of the epilogue; the others run as an elementwise kernel after the GEMM
        switch (act) {
            case kAbs: DOCC_EPILOGUE_CASE(kAbs); break;
            case kReLU: DOCC_EPILOGUE_CASE(kReLU); break;
            default: DOCC_EPILOGUE_CASE(-1); break;
        }
#undef DOCC_EPILOGUE_CASE
        return;
    }
    const bool use_c = (beta != (OT) 0);
    const bool whole = row0 + TM * MT <= M && col0 + TN * MT <= N;
    if (whole) {
        OT* base = C + (row0 + acc_row(0)) * ldc + col0 + lcol;
        if (!use_c) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int r = 0; r < NACC; r++)
                        base[(long) (i * MT + acc_row(r) - acc_row(0)) * ldc + j * MT] = alpha * acc[i][j][r];
        } else {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    OT old[NACC];
#pragma unroll
                    for (int r = 0; r < NACC; r++) old[r] = base[(long) (i * MT + acc_row(r) - acc_row(0)) * ldc + j * MT];
#pragma unroll
                    for (int r = 0; r < NACC; r++)
                        base[(long) (i * MT + acc_row(r) - acc_row(0)) * ldc + j * MT] = gemm_axpby(alpha, (OT) acc[i][j][r], beta, old[r]);
                }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const long col = col0 + j * MT + lcol;
#pragma unroll
            for (int r = 0; r < NACC; r++) {
                const long row = row0 + i * MT + acc_row(r);
                if (row < M && col < N) {
                    OT* p = C + row * ldc + col;
                    *p = use_c ? gemm_axpby(alpha, (OT) acc[i][j][r], beta, *p) : alpha * acc[i][j][r];
                }
            }
        }
    }
}

// Tile id -> tile coordinates: XCD-contiguous renumbering, then grouped
// ordering (GROUP_M rows of tiles at a time) inside each XCD's range.
__device__ __forceinline__ void gemm_tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    constexpr int kXcd = 8;
    constexpr int GROUP_M = 8;
    const int total = tiles_m * tiles_n;
    const int per = total / kXcd;
    if (pid < per * kXcd) pid = (pid % kXcd) * per + pid / kXcd;
    const int width = GROUP_M * tiles_n;
    const int group = pid / width;
    const int first_m = group * GROUP_M;
    const int gsize = min(tiles_m - first_m, GROUP_M);
    tm = first_m + (pid % width) % gsize;
    tn = (pid % width) / gsize;
}

// Global -> registers -> LDS for a ROWS x COLS tile (COLS contiguous in memory) of a row-major
// operand, walked along K. K runs along the columns for a k-contiguous operand
// (K_ALONG_COLS) and along the rows otherwise; the other coordinate is the operand's m or n
// index.
//
// Loads are unconditional in the steady state: the m/n coordinate of every vector is clamped
// into the matrix when the loader is set up (rows or columns beyond the edge hold copies of
// valid data; the outputs they feed are never stored), each vector keeps one pointer that
// advances by a constant per K-step, and only the last, partial K-step masks (to zero, because
// that data does feed valid outputs). No branch and no select stands between a load and the
// MFMAs of the current step, so the loads stay in flight while the step is multiplied.
// ALIGNED promises 16-byte aligned rows and contiguous extents that are multiples of VEC.
template <typename T, int ROWS, int COLS, int NT, bool ALIGNED, bool K_ALONG_COLS>
struct TileLoader {
    typedef typename Mfma<T>::vec_t vec_t;
    static constexpr int VEC = Mfma<T>::VEC;
    static constexpr int VPR = COLS / VEC;            // vectors per tile row
    static constexpr int NV = ROWS * VPR / NT;        // vectors per thread
    static constexpr int BK = K_ALONG_COLS ? COLS : ROWS;
    static_assert(ROWS * VPR % NT == 0, "tile does not divide among the threads");

    const T* p[NV];   // address of vector i in the current K-step
    int lim[NV];      // unaligned, K along rows: last valid element offset of the vector (may be negative)
    vec_t v[NV];
    long kstep;

    // (r0, c0): tile origin at K = 0; rmax / cmax: matrix extents
    __device__ __forceinline__ void init(const T* __restrict__ base, long ld, long r0, long c0, long rmax, long cmax,
                                         int tid) {
        kstep = K_ALONG_COLS ? (long) COLS : (long) ROWS * ld;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = tid + i * NT;
            long r = r0 + idx / VPR;
            long c = c0 + (idx % VPR) * VEC;
            lim[i] = VEC - 1;
            if (K_ALONG_COLS) {
                r = r < rmax ? r : rmax - 1;               // clamp the m/n index
            } else if (ALIGNED) {
                c = c + VEC <= cmax ? c : cmax - VEC;      // whole vectors: clamp the vector start
            } else {
                lim[i] = (int) (cmax - 1 - c);             // per element: offsets beyond lim are clamped to it
            }
            p[i] = base + r * ld + c;
        }
    }

    __device__ __forceinline__ void advance() {
#pragma unroll
        for (int i = 0; i < NV; i++) p[i] += kstep;
    }

    // a K-step that lies entirely inside [0, K)
    __device__ __forceinline__ void load_full() {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            if (ALIGNED) {
                v[i] = *reinterpret_cast<const vec_t*>(p[i]);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) v[i][e] = p[i][(!K_ALONG_COLS && e > lim[i]) ? lim[i] : e];
            }
        }
    }

    // the last K-step when only `kleft` < BK values of k remain: the rest reads as zero
    __device__ __forceinline__ void load_tail(int kleft, int tid) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = tid + i * NT;
            const int lr = idx / VPR, lc = (idx % VPR) * VEC;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const bool ok = K_ALONG_COLS ? (lc + e < kleft) : (lr < kleft);
                const int off = (!K_ALONG_COLS && !ALIGNED && e > lim[i]) ? lim[i] : e;
                // outside: read this thread's own first element of the first K-step instead (a valid address)
                const T raw = ok ? p[i][off] : (T) 0;
                v[i][e] = raw;
            }
        }
    }

    // registers -> LDS tile with row stride LDS_LD elements
    template <int LDS_LD>
    __device__ __forceinline__ void store(T* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = tid + i * NT;
            *reinterpret_cast<vec_t*>(lds + (idx / VPR) * LDS_LD + (idx % VPR) * VEC) = v[i];
        }
    }
};

// TA / TB: the operand is stored transposed in memory (A as [K,M], B as [N,K]).
// "k-contiguous" operands (A when !TA, B when TB) live in LDS as [MN][BK+PADK];
// "mn-contiguous" ones (A when TA, B when !TB) as [BK][MN+PADM].
template <typename T, int BM, int BN, int BK, int WM, int WN, bool TA, bool TB, bool ALIGNED>
struct GemmKernel {
    typedef Mfma<T> X;
    typedef typename X::acc_t acc_t;
    typedef typename X::vec_t vec_t;
    static constexpr int NT = 64 * WM * WN;
    static constexpr int MT = X::MT;
    static constexpr int VK = X::VK;
    static constexpr int KG = X::G * VK;  // k consumed per LDS read round
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int TM = WTM / MT, TN = WTN / MT;
    static constexpr int PADK = 16 / sizeof(T);
    static constexpr int PADM = 8;
    static constexpr bool A_KC = !TA, B_KC = TB;
    static constexpr int LDA_S = A_KC ? BK + PADK : BM + PADM;
    static constexpr int LDB_S = B_KC ? BK + PADK : BN + PADM;
    static constexpr int A_ELEMS = A_KC ? BM * LDA_S : BK * LDA_S;
    static constexpr int B_ELEMS = B_KC ? BN * LDB_S : BK * LDB_S;
    static constexpr int LDS_BYTES = 2 * (A_ELEMS + B_ELEMS) * (int) sizeof(T);
    static_assert(BK % KG == 0, "BK must be a multiple of the k-group");
    static_assert(WTM % MT == 0 && WTN % MT == 0, "wave tile must be a multiple of the MFMA tile");

    typedef TileLoader<T, A_KC ? BM : BK, A_KC ? BK : BM, NT, ALIGNED, A_KC> ALoader;
    typedef TileLoader<T, B_KC ? BN : BK, B_KC ? BK : BN, NT, ALIGNED, B_KC> BLoader;

    static __device__ __forceinline__ void run(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                               long M, long N, long K, long lda, long ldb, long ldc, T alpha,
                                               T beta, const T* bias, int act) {
        // all LDS addressing is derived from this one array so that the
        // compiler keeps it in the LDS address space (ds_* instructions)
        extern __shared__ __attribute__((aligned(16))) unsigned char docc_gemm_lds[];
        T* const lds = reinterpret_cast<T*>(docc_gemm_lds);
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wm = wave / WN, wn = wave % WN;
        const int tiles_m = (int) ((M + BM - 1) / BM), tiles_n = (int) ((N + BN - 1) / BN);
        int tm, tn;
        gemm_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        const long m0 = (long) tm * BM, n0 = (long) tn * BN;

        // LDS: A buffers at [0, 2*A_ELEMS), B buffers behind them
        constexpr int B_BASE = 2 * A_ELEMS;

        acc_t acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < X::NACC; r++) acc[i][j][r] = (T) 0;

        ALoader la;
        BLoader lb;
        if (A_KC) la.init(A, lda, m0, 0, M, K, tid);
        else la.init(A, lda, 0, m0, K, M, tid);
        if (B_KC) lb.init(B, ldb, n0, 0, N, K, tid);
        else lb.init(B, ldb, 0, n0, K, N, tid);

        const int lrow = lane % MT;          // row (A) / column (B) inside an MFMA tile
        const int lk = (lane / MT) * VK;     // this lane's first k inside a k-group

        auto compute = [&](int cur) {
            const T* as = lds + cur * A_ELEMS;
            const T* bs = lds + B_BASE + cur * B_ELEMS;
#pragma unroll
            for (int kg = 0; kg < BK / KG; kg++) {
                T a[TM][VK], b[TN][VK];
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    const int row = wm * WTM + i * MT + lrow;
                    if (A_KC) {
                        vec_t t = *reinterpret_cast<const vec_t*>(as + row * LDA_S + kg * KG + lk);
#pragma unroll
                        for (int s = 0; s < VK; s++) a[i][s] = t[s];
                    } else {
#pragma unroll
                        for (int s = 0; s < VK; s++) a[i][s] = as[(kg * KG + lk + s) * LDA_S + row];
                    }
                }
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int col = wn * WTN + j * MT + lrow;
                    if (B_KC) {
                        vec_t t = *reinterpret_cast<const vec_t*>(bs + col * LDB_S + kg * KG + lk);
#pragma unroll
                        for (int s = 0; s < VK; s++) b[j][s] = t[s];
                    } else {
#pragma unroll
                        for (int s = 0; s < VK; s++) b[j][s] = bs[(kg * KG + lk + s) * LDB_S + col];
                    }
                }
#pragma unroll
                for (int s = 0; s < VK; s++)
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) acc[i][j] = X::mfma(a[i][s], b[j][s], acc[i][j]);
            }
        };
        auto stage = [&](int buf) {
            la.template store<LDA_S>(lds + buf * A_ELEMS, tid);
            lb.template store<LDB_S>(lds + B_BASE + buf * B_ELEMS, tid);
        };

        // K-steps 0 .. full-1 lie inside K, an optional last one is partial
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
        for (; kt + 1 < full; kt++) {   // steady state: step kt+1 travels while step kt is multiplied
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

        gemm_store_wave<kGemmEpilogue, TM, TN, MT, X::NACC>(C, ldc, M, N, m0 + wm * WTM, n0 + wn * WTN, lrow, alpha, beta, bias, act, acc,
                                             [&](int r) { return X::acc_row(lane, r); });
    }
};

} // namespace docc_k

// Defines the four transpose variants x {aligned, unaligned} of one tile
// configuration as extern "C" kernels named
//   docc_<prefix>_<BM>x<BN>x<BK>_<nn|nt|tn|tt>_<a|u>
#define DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, TA, TB, TAG, AL, ALTAG)                                   \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void DOCC_GEMM_NAME(docc_##PREFIX##_##BM##x##BN##x##BK##_##TAG##_##ALTAG)( \
        const T* A, const T* B, T* C, long M, long N, long K, long lda, long ldb, long ldc, T alpha, T beta,    \
        const T* bias, int act, long batch_a, long batch_b, long batch_c) {                                    \
        /* blockIdx.y = entry of the batch; the strides are in elements, 0 for a shared operand */             \
        const long z = blockIdx.y;                                                                             \
        docc_k::GemmKernel<T, BM, BN, BK, WM, WN, TA, TB, AL>::run(A + z * batch_a, B + z * batch_b, C + z * batch_c, M, N, K, \
                                                                   lda, ldb, ldc, alpha, beta, bias, act);     \
    }

#define DOCC_GEMM_CONFIG(PREFIX, T, BM, BN, BK, WM, WN)                    \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, false, false, nn, true, a)  \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, false, true, nt, true, a)   \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, true, false, tn, true, a)   \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, true, true, tt, true, a)    \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, false, false, nn, false, u) \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, false, true, nt, false, u)  \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, true, false, tn, false, u)  \
    DOCC_GEMM_ONE(PREFIX, T, BM, BN, BK, WM, WN, true, true, tt, false, u)
