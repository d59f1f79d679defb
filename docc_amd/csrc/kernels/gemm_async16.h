// bf16 x bf16 -> fp32 GEMM on v_mfma_f32_16x16x32_bf16, asynchronous global -> LDS pipeline (gfx950).
//
// Why a second bf16 kernel beside gemm_async.h: on operands whose bits toggle (N(0,1) values) the product is bound
// by the board's power limit, not by the matrix pipe, and the 16x16x32 form of the instruction spends less of it: a
// loop of nothing but MFMAs on such operands sustains 2060 TFLOP/s in this form and 1800 in the 32x32x16 form (both
// 2450 on all-zero operands). The price is register traffic the other form does not have - a 128 x 128 wave tile is
// 8 x 8 instructions per 32 k, each operand piece feeds eight of them - which the schedule below is built around.
//
// Tiles in LDS and the copies are those of gemm_async.h (AsyncTile, with the placement of granules that suits these
// fragments): K-steps of 32 k, a ring of STAGES stages, every 16-byte granule travels with one global_load_lds_dwordx4. One K-step is one round of TM x TN MFMAs,
// row by row of the wave tile (slot = i * TN + j):
//   - the B pieces of the step are all resident (two sets, the other one is filled for the next step);
//   - the A pieces roll through a ring of four: piece i + 2 is read from LDS when row i begins;
//   - the copies that refill the stage read during the previous step are dealt one every SLOTS / LOADS MFMAs;
//   - one wait + barrier per step, behind the MFMA that ends row TM - 3: by then every piece of this step is in
//     registers (so the stage may be refilled during the next step) and the copies of the next step, issued two
//     steps ago, have landed; the rows after it read the next step's first pieces.
// Every read, copy and the barrier is issued behind an MFMA and fenced there, as in gemm_async.h.
// The launcher sends only products with K a multiple of 64 and at least STAGES K-steps here.
#pragma once

#include "gemm_async.h"

namespace docc_k {

template <int BM, int BN, int WM, int WN, int STAGES, bool TA, bool TB>
struct AsyncGemm16Kernel {
    typedef uint16_t T;
    static constexpr int BK = 32, MT = 16, NACC = 4;
    static constexpr int NT = 64 * WM * WN;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int TM = WTM / MT, TN = WTN / MT;
    static constexpr bool A_KC = !TA, B_KC = TB;
    typedef AsyncTile<T, A_KC ? BM : BK, A_KC ? BK : BM, NT, A_KC, 1> ATile;
    typedef AsyncTile<T, B_KC ? BN : BK, B_KC ? BK : BN, NT, B_KC, 1> BTile;
    static constexpr int STAGE_ELEMS = ATile::ELEMS + BTile::ELEMS;
    static constexpr int LDS_BYTES = STAGES * STAGE_ELEMS * (int) sizeof(T);
    static constexpr int LOADS = ATile::NV + BTile::NV;          // copies per thread and K-step
    static constexpr int SLOTS = TM * TN;                        // MFMAs per K-step
    static constexpr int RING = 4;                               // A pieces in registers
    static constexpr int BARRIER_SLOT = (TM - 2) * TN - 1;       // the MFMA the wait + barrier follow
    static constexpr int CSTRIDE = SLOTS / LOADS;                // MFMAs between two copies
    static_assert(STAGES >= 3, "the copies of a step are issued STAGES - 1 steps ahead, into the stage read one step ago");
    static_assert(TM >= 4 && TM % RING == 0 && SLOTS % LOADS == 0 && CSTRIDE >= 2,
                  "the schedule assumes rows in multiples of the A ring and fewer copies than MFMAs");
    // copy q is issued behind slot q * CSTRIDE + CSTRIDE / 2; those at or before the barrier slot are younger than what the wait is for
    static constexpr int EARLY = (BARRIER_SLOT - CSTRIDE / 2) / CSTRIDE + 1;
    static_assert((STAGES - 2) * LOADS + EARLY < 64, "vmcnt holds at most 63 outstanding loads");

    static __device__ __forceinline__ void run(const T* __restrict__ A, const T* __restrict__ B, float* __restrict__ C, long M, long N,
                                               long K, long lda, long ldb, long ldc, float alpha, float beta, const float* bias, int act) {
        extern __shared__ __attribute__((aligned(16))) unsigned char docc_gemm_lds[];
        T* const lds = reinterpret_cast<T*>(docc_gemm_lds);

        const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave / WN, wn = wave % WN;
        const int tiles_m = (int) ((M + BM - 1) / BM), tiles_n = (int) ((N + BN - 1) / BN);
        int tm, tn;
        gemm_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        const long m0 = (long) tm * BM, n0 = (long) tn * BN;

        f32x4 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < NACC; r++) acc[i][j][r] = 0;

        ATile ta;
        BTile tb;
        if (A_KC) ta.init(A, lda, m0, 0, M, K, tid);
        else ta.init(A, lda, 0, m0, K, M, tid);
        if (B_KC) tb.init(B, ldb, n0, 0, N, K, tid);
        else tb.init(B, ldb, 0, n0, K, N, tid);

        // One operand piece: 16 rows (columns) x 32 k. Lane l holds row l % 16 and k = 8 (l / 16) .. + 7 of it. Any
        // assignment of k to lanes and register halves is as good as another while A and B use the same one.
        const int lidx = lane & 15, lg = lane >> 4;
        auto piece = [&](const T* stage, bool is_a, int t) -> bf16x8 {
            const T* base = is_a ? stage : stage + ATile::ELEMS;
            const int idx0 = is_a ? wm * WTM + t * MT : wn * WTN + t * MT;
            const bool kc = is_a ? A_KC : B_KC;
            auto goff = [&](int row, int cv) { return is_a ? ATile::granule_offset(row, cv) : BTile::granule_offset(row, cv); };
            if (kc) {
                const u16x8a v = *reinterpret_cast<const u16x8a*>(base + goff(idx0 + lidx, lg));
                return __builtin_bit_cast(bf16x8, v);
            }
            // the operand lies k-major (rows of m or n): a transposing read hands each lane of a 16-lane group the
            // four k of its column out of a 4 k x 16 column block; two of them make the lane's eight k
            const int krow = 8 * lg + (lidx >> 2);
            const int col = idx0 + 4 * (lidx & 3);
            typedef __attribute__((address_space(3))) s16x4a lds_s16x4;
            const T* plo = base + goff(krow, col / 8) + (col & 7);
            const T* phi = base + goff(krow + 4, col / 8) + (col & 7);
            const s16x4a lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) plo);
            const s16x4a hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) phi);
            const s16x8a v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return __builtin_bit_cast(bf16x8, v);
        };

        bf16x8 ar[RING], bq[2][TN];

        const int ksteps = (int) (K / BK);
        auto stage_of = [&](int kt) { return lds + (kt % STAGES) * STAGE_ELEMS; };

        // ---- prologue: the first STAGES - 1 steps are copied, the first one awaited, its first pieces read
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++) {
            if (s > 0) {
                ta.advance();
                tb.advance();
            }
            T* st = stage_of(s);
            ta.issue(st, wave);
            tb.issue(st + ATile::ELEMS, wave);
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LOADS) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < TN; j++) bq[0][j] = piece(stage_of(0), false, j);
        ar[0] = piece(stage_of(0), true, 0);
        ar[1] = piece(stage_of(0), true, 1);

        // One K-step; P: which B set it multiplies with. Every step is the same straight code, so that all MFMAs sit in
        // one loop without a branch (a branch that accumulators live across makes the compiler move them): the last
        // STAGES - 1 steps, which have no step left to copy, copy the last one again into a stage that nobody reads
        // any more, and the last step reads "next" pieces that nobody uses from a stage inside the ring.
        auto kstep = [&](int kt, auto parity_c) {
            constexpr int P = decltype(parity_c)::value;
            const T* st = stage_of(kt);
            const T* nst = stage_of(kt + 1);
            T* dst = lds + ((kt + STAGES - 1) % STAGES) * STAGE_ELEMS;
            const long step = kt + STAGES - 1 < ksteps ? 1 : 0;
            ta.base += step * ta.kstep_bytes;
            tb.base += step * tb.kstep_bytes;
#pragma unroll
            for (int slot = 0; slot < SLOTS; slot++) {
                const int i = slot / TN, j = slot % TN;
                // Written out with the accumulator tied to its registers: left to itself the register allocator moves
                // the 64 four-register accumulators about at the head of the loop (1400 copies through VGPRs and
                // scratch memory in one build), since exactly as many AGPRs exist as the tile needs.
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(ar[i % RING]), "v"(bq[P][j]));
                // A piece i + 2 when row i begins: of this step, or (behind the barrier) of the next
                if (j == 0) ar[(i + 2) % RING] = i + 2 < TM ? piece(st, true, i + 2) : piece(nst, true, i + 2 - TM);
                // the next step's B pieces, one per MFMA from the row behind the barrier on
                if (slot > BARRIER_SLOT && slot - BARRIER_SLOT - 1 < TN) bq[1 - P][slot - BARRIER_SLOT - 1] = piece(nst, false, slot - BARRIER_SLOT - 1);
                if (slot % CSTRIDE == CSTRIDE / 2) {
                    const int q = slot / CSTRIDE;
                    if (q < ATile::NV) ta.issue_one(dst, q, wave);
                    else tb.issue_one(dst + ATile::ELEMS, q - ATile::NV, wave);
                }
                if (slot == BARRIER_SLOT) {
                    __builtin_amdgcn_sched_barrier(0);
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((STAGES - 3) * LOADS + EARLY) : "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // steps in pairs, so that the B set a step uses is a compile-time choice (the launcher sends an even number)
        for (int kt = 0; kt < ksteps; kt += 2) {
            kstep(kt, std::integral_constant<int, 0>{});
            kstep(kt + 1, std::integral_constant<int, 1>{});
        }

        // the last MFMAs are still in the pipe (the compiler does not see them behind the asm statements), and so are
        // the copies that nobody waits for
        asm volatile("s_nop 15\n s_nop 15\n s_waitcnt vmcnt(0)" ::: "memory");
        // 16 x 16 fp32 result tile: register r of lane l is row 4 (l / 16) + r, column l % 16
        gemm_store_wave<kGemmEpilogue, TM, TN, MT, NACC>(C, ldc, M, N, m0 + wm * WTM, n0 + wn * WTN, lidx, alpha, beta, bias, act, acc,
                                                         [&](int r) { return 4 * lg + r; });
    }
};

} // namespace docc_k

// extern "C" kernels docc_bgemma_<BM>x<BN>x32q<STAGES>_<nn|nt|tn|tt>
#define DOCC_AGEMM16_ONE(BM, BN, WM, WN, ST, TA, TB, TAG)                                                                       \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void DOCC_GEMM_NAME(docc_bgemma_##BM##x##BN##x32q##ST##_##TAG)(       \
        const uint16_t* A, const uint16_t* B, float* C, long M, long N, long K, long lda, long ldb, long ldc, float alpha,     \
        float beta, const float* bias, int act, long batch_a, long batch_b, long batch_c) {                                    \
        const long z = blockIdx.y;                                                                                             \
        docc_k::AsyncGemm16Kernel<BM, BN, WM, WN, ST, TA, TB>::run(A + z * batch_a, B + z * batch_b, C + z * batch_c, M, N, K, \
                                                                   lda, ldb, ldc, alpha, beta, bias, act);                    \
    }

#define DOCC_AGEMM16_CONFIG(BM, BN, WM, WN, ST)          \
    DOCC_AGEMM16_ONE(BM, BN, WM, WN, ST, false, false, nn) \
    DOCC_AGEMM16_ONE(BM, BN, WM, WN, ST, false, true, nt)  \
    DOCC_AGEMM16_ONE(BM, BN, WM, WN, ST, true, false, tn)  \
    DOCC_AGEMM16_ONE(BM, BN, WM, WN, ST, true, true, tt)
