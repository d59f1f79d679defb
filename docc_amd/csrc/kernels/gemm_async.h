// Tiled MFMA GEMM with an asynchronous, multi-stage global -> LDS pipeline (gfx950):
//   C[M,N] = alpha * op(A) * op(B) + beta * C,  row-major, A/B fp64, fp32 or bf16 (fp32 C for bf16).
//
// Same tiling as gemm_mfma.h; what differs is how operand tiles reach LDS:
//   - every 16-byte granule of a tile travels with one `global_load_lds_dwordx4`: the data goes
//     from memory straight into LDS, no registers and no LDS store instruction in between;
//     a wave-instruction fills 64 consecutive granules (1 KiB);
//   - S stages of LDS are kept: while step kt is multiplied, the loads of steps kt+1 .. kt+S-1
//     are in flight, so an L2 miss has S-1 steps to come back. One `s_waitcnt vmcnt(n)` and one
//     `s_barrier` per step; n leaves the newer steps' loads outstanding;
//   - because the LDS position of a granule is fixed by the lane that loads it, rows cannot be
//     padded; bank conflicts are avoided by XOR-swizzling the granule index with the row
//     (the lane simply fetches the global granule that belongs in its slot);
//   - the partial last K-step is copied the same way: the granules past K fetch the first valid k of their row
//     (column) instead, and are cleared in LDS once they have landed (one extra barrier per product).
// Requires 16-byte aligned operands with contiguous extents that are multiples of the vector
// length (the launcher sends everything else to the gemm_mfma.h kernels).
#pragma once

#include "gemm_mfma.h"
#include <type_traits>

namespace docc_k {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;
typedef uint16_t u16x8a __attribute__((ext_vector_type(8)));
typedef short s16x4a __attribute__((ext_vector_type(4)));
typedef short s16x8a __attribute__((ext_vector_type(8)));

template <typename T>
struct AsyncTraits;
template <>
struct AsyncTraits<float> {
    static constexpr int VEC = 4, MT = 32, G = 2, KG = 8, NACC = 16;   // KG: k consumed per fetch round
    typedef f32x4 vec_t;
    typedef f32x16 acc_t;
    typedef float out_t;
    static __device__ __forceinline__ int swz_mn(int k) { return ((k >> 2) & 1) << 3; }
};
template <>
struct AsyncTraits<double> {
    static constexpr int VEC = 2, MT = 16, G = 4, KG = 8, NACC = 4;
    typedef f64x2 vec_t;
    typedef f64x4 acc_t;
    typedef double out_t;
    static __device__ __forceinline__ int swz_mn(int k) { return ((k >> 1) & 1) << 3; }
};
template <>
struct AsyncTraits<uint16_t> {   // bf16 bits
    static constexpr int VEC = 8, MT = 32, G = 2, KG = 16, NACC = 16;
    typedef u16x8a vec_t;
    typedef f32x16 acc_t;
    typedef float out_t;
    static __device__ __forceinline__ int swz_mn(int k) { return (k & 3) << 2; }
};

// One operand tile of ROWS x COLS elements (COLS contiguous) in an LDS stage. LAYOUT: where a granule lies in the
// stage. 0: row after row, the granule index XORed with a function of the row - for fragments of 32 rows (columns) and
// two k-groups of lanes. 1: for the fragments of the 16x16x32 MFMA (16 rows, four k-groups, gemm_async16.h).
template <typename T, int ROWS, int COLS, int NT, bool K_ALONG_COLS, int LAYOUT = 0>
struct AsyncTile {
    typedef AsyncTraits<T> X;
    typedef typename X::vec_t vec_t;
    static constexpr int VEC = X::VEC;
    static constexpr int VPR = COLS / VEC;          // granules per row
    static constexpr int NG = ROWS * VPR;           // granules per tile
    static constexpr int NW = NT / 64;
    static constexpr int NV = NG / NT;              // granules per thread
    static constexpr int ELEMS = ROWS * COLS;
    static constexpr int BK = K_ALONG_COLS ? COLS : ROWS;
    static_assert(NG % NT == 0, "tile does not divide among the threads");
    static_assert(K_ALONG_COLS ? (VPR == 16 || VPR == 8 || VPR == 4) : (VPR >= 16), "row length not covered by the swizzles");

    static_assert(LAYOUT == 0 || (sizeof(T) == 2 && (K_ALONG_COLS ? VPR == 4 : VPR >= 16)), "layout 1: bf16 tiles 32 k deep");
    // granule-index swizzle of a row
    static __device__ __forceinline__ int swz(int row) {
        if (LAYOUT == 1) {
            // k along the columns: a fragment read is 16 rows x 4 granules (lane = 16 * granule + row); timed per
            // pattern, the reads run without bank conflicts with the granule XORed by (row >> 1) & 3.
            // k-major tile, read by transposing 64-bit reads: the lanes of half a wave read 32 bytes each of rows
            // k, k+1, k+2, k+3 and k+8 .. k+11 at once - eight shifts of 32 bytes
            return K_ALONG_COLS ? ((row >> 1) & 3) : 2 * ((row & 3) | (((row >> 3) & 1) << 2));
        }
        // 16 consecutive rows read the same k-granule at once: spread them over the 16 slots of 256 bytes
        if (K_ALONG_COLS) return VPR == 16 ? (row & 15) : VPR == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3);
        return X::swz_mn(row);
    }
    // slot (16-byte unit inside a stage) of the granule that holds columns cv*VEC .. of `row`, and the inverse
    static __device__ __forceinline__ int slot_of(int row, int cv) { return row * VPR + (cv ^ swz(row)); }
    static __device__ __forceinline__ void granule_of(int g, int& row, int& cv) {
        row = g / VPR;
        cv = (g % VPR) ^ swz(row);
    }
    // element offset (inside a stage) of that granule
    static __device__ __forceinline__ int granule_offset(int row, int cv) { return slot_of(row, cv) * VEC; }

    const char* base;      // wave-uniform: origin of the tile of the current K-step
    unsigned off[NV];      // this lane's granules: byte offsets from the origin
    long kstep_bytes;

    // The tile covers rows r0.. and columns c0.. of an rmax x cmax operand; out-of-range rows (columns
    // of a k-major tile) are clamped to the edge - their products land in rows/columns of C that are
    // never stored. The host guarantees that ROWS*ld*sizeof(T) fits the 32-bit offsets.
    __device__ __forceinline__ void init(const T* __restrict__ mat, long ld, long r0, long c0, long rmax, long cmax, int tid) {
        kstep_bytes = (K_ALONG_COLS ? (long) COLS : (long) ROWS * ld) * (long) sizeof(T);
        const int wave = tid >> 6, lane = tid & 63;
        const long cbase = K_ALONG_COLS ? c0 : (c0 + VEC <= cmax ? c0 : cmax - VEC);
        base = reinterpret_cast<const char*>(mat + r0 * ld + cbase);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int g = (i * NW + wave) * 64 + lane;   // the LDS slot this lane fills
            int row, cv;
            granule_of(g, row, cv);
            long r = r0 + row, c = c0 + (long) cv * VEC;
            if (K_ALONG_COLS) r = r < rmax ? r : rmax - 1;
            else c = c + VEC <= cmax ? c : cmax - VEC;
            off[i] = (unsigned) (((r - r0) * ld + (c - cbase)) * (long) sizeof(T));
        }
    }

    __device__ __forceinline__ void advance() { base += kstep_bytes; }

    // asynchronous copy of granule i of the current K-step into `stage` (wave: wave-uniform index)
    __device__ __forceinline__ void issue_one(T* stage, int i, int wave) const {
        __builtin_amdgcn_global_load_lds((global_ptr_t) (base + off[i]), (lds_ptr_t) (stage + (i * NW + wave) * 64 * VEC), 16, 0, 0);
    }
    __device__ __forceinline__ void issue(T* stage, int wave) const {
#pragma unroll
        for (int i = 0; i < NV; i++) issue_one(stage, i, wave);
    }

    // The partial last K-step: granule i holds k >= kleft when `past(i)` says so. Such a granule is copied from
    // k = 0 of the step (same row / column, so the address stays inside the operand) and cleared afterwards.
    __device__ __forceinline__ bool past(int i, int wave, int lane, int kleft, unsigned* back) const {
        const int g = (i * NW + wave) * 64 + lane;
        int row, cv;
        granule_of(g, row, cv);
        const bool out = K_ALONG_COLS ? (cv * VEC >= kleft) : (row >= kleft);
        // bytes from the granule's own position back to k = 0 of the step
        *back = K_ALONG_COLS ? (unsigned) (cv * VEC * (int) sizeof(T)) : (unsigned) ((long) row * (kstep_bytes / ROWS));
        return out;
    }
    __device__ __forceinline__ void issue_tail(T* stage, int kleft, int wave, int lane) const {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            unsigned back;
            const unsigned o = past(i, wave, lane, kleft, &back) ? off[i] - back : off[i];
            __builtin_amdgcn_global_load_lds((global_ptr_t) (base + o), (lds_ptr_t) (stage + (i * NW + wave) * 64 * VEC), 16, 0, 0);
        }
    }
    __device__ __forceinline__ void clear_tail(T* stage, int kleft, int wave, int lane) const {
        vec_t z;
#pragma unroll
        for (int e = 0; e < VEC; e++) z[e] = (T) 0;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            unsigned back;
            if (past(i, wave, lane, kleft, &back)) *reinterpret_cast<vec_t*>(stage + ((i * NW + wave) * 64 + lane) * VEC) = z;
        }
    }
};

template <typename T, int BM, int BN, int BK, int WM, int WN, int STAGES, bool TA, bool TB, bool SPREAD = false>
struct AsyncGemmKernel {
    typedef AsyncTraits<T> X;
    typedef typename X::acc_t acc_t;
    typedef typename X::vec_t vec_t;
    typedef typename X::out_t out_t;
    static constexpr int NT = 64 * WM * WN;
    static constexpr int MT = X::MT, VEC = X::VEC, KG = X::KG;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int TM = WTM / MT, TN = WTN / MT;
    static constexpr bool A_KC = !TA, B_KC = TB;
    typedef AsyncTile<T, A_KC ? BM : BK, A_KC ? BK : BM, NT, A_KC> ATile;
    typedef AsyncTile<T, B_KC ? BN : BK, B_KC ? BK : BN, NT, B_KC> BTile;
    static constexpr int STAGE_ELEMS = ATile::ELEMS + BTile::ELEMS;
    static constexpr int LDS_BYTES = STAGES * STAGE_ELEMS * (int) sizeof(T);
    static constexpr int LOADS_PER_STEP = ATile::NV + BTile::NV;
    static_assert(BK % KG == 0, "BK must be a multiple of the k-group");
    static_assert(STAGES >= 2 && (STAGES - 1) * LOADS_PER_STEP < 64, "vmcnt holds at most 63 outstanding loads");
    static_assert(!SPREAD || STAGES >= 3, "copies dealt over a K-step need a stage that nobody reads meanwhile");

    static __device__ __forceinline__ void run(const T* __restrict__ A, const T* __restrict__ B, out_t* __restrict__ C,
                                               long M, long N, long K, long lda, long ldb, long ldc, out_t alpha,
                                               out_t beta, const out_t* bias, int act) {
        extern __shared__ __attribute__((aligned(16))) unsigned char docc_gemm_lds[];
        T* const lds = reinterpret_cast<T*>(docc_gemm_lds);

        const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave / WN, wn = wave % WN;
        const int tiles_m = (int) ((M + BM - 1) / BM), tiles_n = (int) ((N + BN - 1) / BN);
        int tm, tn;
        gemm_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        const long m0 = (long) tm * BM, n0 = (long) tn * BN;

        acc_t acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < X::NACC; r++) acc[i][j][r] = 0;

        ATile ta;
        BTile tb;
        if (A_KC) ta.init(A, lda, m0, 0, M, K, tid);
        else ta.init(A, lda, 0, m0, K, M, tid);
        if (B_KC) tb.init(B, ldb, n0, 0, N, K, tid);
        else tb.init(B, ldb, 0, n0, K, N, tid);

        const int lidx = lane % MT;     // row of A / column of B inside an MFMA tile
        const int lg = lane / MT;       // k-group of this lane

        // ---- operands of one inner step (16 k for bf16, KG k otherwise) in two register sets --------
        constexpr int VK = VEC;
        constexpr int NKI = (sizeof(T) == 2) ? BK / 16 : BK / KG;     // inner steps per staged K-step
        static_assert(NKI % 2 == 0, "operand register sets alternate per inner step");
        bf16x8 ah[2][TM], bh[2][TN];             // bf16
        T a[2][TM][VK], b[2][TN][VK];            // fp32 / fp64
        // piece idx of a fetch: operand tile idx of A (idx < TM) or tile idx - TM of B
        constexpr int NPIECE = TM + TN;
        auto fetch_piece = [&](const T* stage, int ki, int to, int idx) {
            const bool is_a = idx < TM;
            const int t = is_a ? idx : idx - TM;
            const T* base = is_a ? stage : stage + ATile::ELEMS;
            const int idx0 = is_a ? wm * WTM + t * MT : wn * WTN + t * MT;
            const bool kc = is_a ? A_KC : B_KC;
            auto goff = [&](int row, int cv) { return is_a ? ATile::granule_offset(row, cv) : BTile::granule_offset(row, cv); };
            if constexpr (sizeof(T) == 2) {
                // bf16: one MFMA consumes 16 k; lane (idx, g) supplies k = 8g .. 8g+7
                bf16x8 r;
                if (kc) {
                    const u16x8a v = *reinterpret_cast<const u16x8a*>(base + goff(idx0 + lidx, ki * 2 + lg));
                    r = __builtin_bit_cast(bf16x8, v);
                } else {
                    // transposed read: 16-lane group = 4 k-rows x 16 columns, see gemm_bf16.hip
                    const int s = lane & 15, grp = lane >> 4;
                    const int krow = ki * 16 + 8 * (grp >> 1) + (s >> 2);
                    const int col = idx0 + 16 * (grp & 1) + 4 * (s & 3);
                    typedef __attribute__((address_space(3))) s16x4a lds_s16x4;
                    const T* plo = base + goff(krow, col / 8) + (col & 7);
                    const T* phi = base + goff(krow + 4, col / 8) + (col & 7);
                    const s16x4a lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) plo);
                    const s16x4a hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) phi);
                    const s16x8a v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    r = __builtin_bit_cast(bf16x8, v);
                }
                if (is_a) ah[to][t] = r;
                else bh[to][t] = r;
            } else {
                // fp32 / fp64: lane group g owns k = ki*KG + g*VK .. +VK-1 (VK = VEC: one granule)
                T* out = is_a ? a[to][t] : b[to][t];
                if (kc) {
                    const vec_t v = *reinterpret_cast<const vec_t*>(base + goff(idx0 + lidx, ki * X::G + lg));
#pragma unroll
                    for (int s = 0; s < VK; s++) out[s] = v[s];
                } else {
                    const int col = idx0 + lidx;
#pragma unroll
                    for (int s = 0; s < VK; s++) out[s] = base[goff(ki * KG + lg * VK + s, col / VEC) + col % VEC];
                }
            }
        };
        auto fetch = [&](const T* stage, int ki, int to) {
#pragma unroll
            for (int idx = 0; idx < NPIECE; idx++) fetch_piece(stage, ki, to, idx);
        };
        // MFMAs lo .. hi-1 of the NM of one inner step (order: k-slice, tile row, tile column)
        constexpr int NM = (sizeof(T) == 2 ? 1 : VK) * TM * TN;
        auto mma = [&](int from, int lo, int hi) {
#pragma unroll
            for (int m = lo; m < (hi < NM ? hi : NM); m++) {
                const int s = m / (TM * TN), i = (m / TN) % TM, j = m % TN;
                if constexpr (sizeof(T) == 2) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[from][i], bh[from][j], acc[i][j], 0, 0, 0);
                } else {
                    acc[i][j] = Mfma<T>::mfma(a[from][i][s], b[from][j][s], acc[i][j]);
                }
            }
        };

        // ---- pipeline --------------------------------------------------------------------------
        // The K-steps are copied STAGES ahead into a ring of LDS stages; the operands of an inner
        // step are read from LDS one inner step ahead into the other register set. The last inner
        // step of K-step kt therefore already needs K-step kt+1: that is where the wave waits for
        // its own copies of kt+1, meets the others at the barrier (after which nobody reads stage kt
        // any more: its last operands are in registers), refills stage kt with step kt+STAGES and
        // reads the first operands of kt+1. Each of these blocks is issued behind one MFMA of the
        // current inner step (fences keep them there), so the matrix pipe has work while the other
        // pipes are fed and the LDS round trip passes under the remaining MFMAs.
        const int full = (int) (K / BK);
        const int kleft = (int) (K - (long) full * BK);
        const int ksteps = full + (kleft > 0 ? 1 : 0);
        auto stage_of = [&](int kt) { return lds + (kt % STAGES) * STAGE_ELEMS; };
        auto fill = [&](int kt) {   // starts the copy of step kt (called for kt = 0, 1, 2, ... in order)
            if (kt > 0) {
                ta.advance();
                tb.advance();
            }
            T* st = stage_of(kt);
            if (kt < full) {
                ta.issue(st, wave);
                tb.issue(st + ATile::ELEMS, wave);
            } else {
                ta.issue_tail(st, kleft, wave, lane);
                tb.issue_tail(st + ATile::ELEMS, kleft, wave, lane);
            }
        };
        // step kt has landed once at most the loads of the STAGES-2 newer full steps are outstanding;
        // near the end fewer newer steps exist, so everything is awaited
        // after the barrier that puts step kt into every wave's view: the partial last step has what lies past K
        // cleared (every lane clears the granules it copied itself, which its own wait has seen land)
        auto clear_if_tail = [&](int kt) {
            if (kleft > 0 && kt == full) {
                T* st = stage_of(kt);
                ta.clear_tail(st, kleft, wave, lane);
                tb.clear_tail(st + ATile::ELEMS, kleft, wave, lane);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
        };
        auto arrive = [&](int kt) {
            if (kt + STAGES - 2 < full) {
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((STAGES - 2) * LOADS_PER_STEP) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            }
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            clear_if_tail(kt);
        };
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++)
            if (s < ksteps) fill(s);
        arrive(0);
        if (!SPREAD && STAGES - 1 < ksteps) fill(STAGES - 1);
        fetch(stage_of(0), 0, 0);

        // the last K-step has no successor: it is peeled so that the loop body is free of branches
        // around MFMAs (they would make the compiler copy accumulators between the paths)
        // One inner step: its NM MFMAs, each followed (and fenced, so that it stays there) by its
        // share of the other pipes' work - a lump of LDS reads or copies between two MFMAs would
        // leave the matrix pipe idle while the lump is issued.
        //   inner steps but the last: the LDS reads of the next inner step's operands;
        //   last inner step, after its first MFMA: wait + barrier (see above), then the copies that
        //   refill stage kt and the LDS reads of step kt+1's first operands.
        // mode 0: steady state (the refill is a full asynchronous step, nothing in the body branches);
        // mode 1: near the end (the refill may be the K tail or absent); mode 2: the last step
        // shares per MFMA slot. The LDS reads are dealt over the first half of an inner step's slots only, so that
        // the last of them is issued at least half an inner step before its operand is needed (with the four
        // MFMAs of an fp64 inner step, one read per MFMA left the last read 64 cycles: the next step waited for it)
        constexpr int PSLOTS = NM / 2 > 0 ? NM / 2 : 1, PSLOTS_LAST = NM / 2 > 0 ? NM / 2 : 1;
        constexpr int PPM = (NPIECE + PSLOTS - 1) / PSLOTS;           // pieces per MFMA, inner steps but the last
        constexpr int PPL = (NPIECE + PSLOTS_LAST - 1) / PSLOTS_LAST; // pieces per MFMA, last inner step
        constexpr int LPM = (LOADS_PER_STEP + NM - 2) / (NM - 1);     // copies per MFMA, last inner step
        auto kstep_burst = [&](int kt, auto mode_c) {
            constexpr int MODE = decltype(mode_c)::value;
            constexpr bool NEXT = MODE != 2;
            const T* st = stage_of(kt);
#pragma unroll
            for (int ki = 0; ki < NKI; ki++) {
                if (ki + 1 < NKI) {
#pragma unroll
                    for (int n = 0; n < NM; n++) {
                        mma(ki & 1, n, n + 1);
#pragma unroll
                        for (int q = n * PPM; q < (n + 1) * PPM && q < NPIECE; q++) fetch_piece(st, ki + 1, (ki + 1) & 1, q);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else if (NEXT) {
                    mma(ki & 1, 0, 1);
                    __builtin_amdgcn_sched_barrier(0);
                    T* dst = lds + (kt % STAGES) * STAGE_ELEMS;     // stage kt, free after the barrier
                    if (MODE == 0) {
                        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((STAGES - 2) * LOADS_PER_STEP) : "memory");
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                        ta.advance();
                        tb.advance();
                    } else {
                        arrive(kt + 1);
                        if (kt + STAGES < ksteps) fill(kt + STAGES);
                    }
                    const T* nst = stage_of(kt + 1);
#pragma unroll
                    for (int n = 1; n < NM; n++) {
                        mma(ki & 1, n, n + 1);
                        if (MODE == 0) {
#pragma unroll
                            for (int q = (n - 1) * LPM; q < n * LPM && q < LOADS_PER_STEP; q++) {
                                if (q < ATile::NV) ta.issue_one(dst, q, wave);
                                else tb.issue_one(dst + ATile::ELEMS, q - ATile::NV, wave);
                            }
                        }
#pragma unroll
                        for (int q = (n - 1) * PPL; q < n * PPL && q < NPIECE; q++) fetch_piece(nst, 0, 0, q);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    mma(ki & 1, 0, NM);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // The same with the copies dealt out (SPREAD). All four waves leave the barrier together, and a run of
        // copies from each of them at that moment queues up in the one vector-memory pipe of the CU; the waves
        // then sit behind their own copies while the matrix pipe idles. Here K-step kt issues the copies of step
        // kt+STAGES-1, one every LSTRIDE MFMAs over the whole step, into the stage that the barrier at the end
        // of step kt-1 freed; nobody reads that stage before step kt+STAGES-1. At the wait in the last inner
        // step the copies of step kt+1 are older than those of STAGES-3 whole steps and the EARLY copies this
        // step has issued so far.
        constexpr int SLOTS = NKI * NM;                                                        // MFMAs of a K-step
        constexpr int LSTRIDE = SLOTS / LOADS_PER_STEP > 0 ? SLOTS / LOADS_PER_STEP : 1;       // MFMAs between two copies
        constexpr int LPS = (LOADS_PER_STEP + SLOTS - 1) / SLOTS;                              // copies per slot when there are more copies than MFMAs
        // copies issued behind MFMA `slot` (0-based over the K-step): indices [lo, hi)
        auto copies_lo = [](int slot) constexpr { return SLOTS >= LOADS_PER_STEP ? (slot + 1) / LSTRIDE : slot * LPS; };
        constexpr int WAIT_SLOT = (NKI - 1) * NM;                                              // the MFMA the wait follows
        constexpr int EARLY_RAW = SLOTS >= LOADS_PER_STEP ? (WAIT_SLOT + 2) / LSTRIDE : (WAIT_SLOT + 1) * LPS;    // = copies_lo(WAIT_SLOT + 1)
        constexpr int EARLY = EARLY_RAW < LOADS_PER_STEP ? EARLY_RAW : LOADS_PER_STEP;
        auto kstep_spread = [&](int kt, auto mode_c) {
            constexpr int MODE = decltype(mode_c)::value;
            constexpr bool NEXT = MODE != 2;
            const T* st = stage_of(kt);
            T* dst = lds + ((kt + STAGES - 1) % STAGES) * STAGE_ELEMS;
            if (MODE == 0) {
                ta.advance();
                tb.advance();
            } else if (MODE == 1) {
                if (kt + STAGES - 1 < ksteps) fill(kt + STAGES - 1);    // the K tail
            }
            auto copies = [&](int slot) {
                if (MODE != 0) return;
                int lo = copies_lo(slot), hi = copies_lo(slot + 1);
                if (slot == SLOTS - 1) hi = LOADS_PER_STEP;
#pragma unroll
                for (int q = lo; q < hi && q < LOADS_PER_STEP; q++) {
                    if (q < ATile::NV) ta.issue_one(dst, q, wave);
                    else tb.issue_one(dst + ATile::ELEMS, q - ATile::NV, wave);
                }
            };
#pragma unroll
            for (int ki = 0; ki < NKI; ki++) {
                if (ki + 1 < NKI) {
#pragma unroll
                    for (int n = 0; n < NM; n++) {
                        mma(ki & 1, n, n + 1);
#pragma unroll
                        for (int q = n * PPM; q < (n + 1) * PPM && q < NPIECE; q++) fetch_piece(st, ki + 1, (ki + 1) & 1, q);
                        copies(ki * NM + n);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else if (NEXT) {
                    mma(ki & 1, 0, 1);
                    copies(ki * NM);
                    __builtin_amdgcn_sched_barrier(0);
                    if (MODE == 0) {
                        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((STAGES - 3) * LOADS_PER_STEP + EARLY) : "memory");
                    } else {
                        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    }
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    if (MODE != 0) clear_if_tail(kt + 1);
                    const T* nst = stage_of(kt + 1);
#pragma unroll
                    for (int n = 1; n < NM; n++) {
                        mma(ki & 1, n, n + 1);
#pragma unroll
                        for (int q = (n - 1) * PPL; q < n * PPL && q < NPIECE; q++) fetch_piece(nst, 0, 0, q);
                        copies(ki * NM + n);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    mma(ki & 1, 0, NM);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto kstep = [&](int kt, auto mode_c) {
            if constexpr (SPREAD) kstep_spread(kt, mode_c);
            else kstep_burst(kt, mode_c);
        };
        int kt = 0;
        for (; kt + STAGES - (SPREAD ? 1 : 0) < full; kt++) kstep(kt, std::integral_constant<int, 0>{});
        for (; kt + 1 < ksteps; kt++) kstep(kt, std::integral_constant<int, 1>{});
        kstep(kt, std::integral_constant<int, 2>{});

        // ---- epilogue ------------------------------------------------------------------------------
        gemm_store_wave<kGemmEpilogue, TM, TN, MT, X::NACC>(C, ldc, M, N, m0 + wm * WTM, n0 + wn * WTN, lidx, alpha, beta, bias, act, acc, [&](int r) {
            return (sizeof(T) == 8) ? Mfma<double>::acc_row(lane, r) : Mfma<float>::acc_row(lane, r);
        });
    }
};

} // namespace docc_k

// extern "C" kernels docc_<prefix>a_<BM>x<BN>x<BK>s<STAGES>_<nn|nt|tn|tt>
#define DOCC_AGEMM_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, TA, TB, TAG)                                          \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void DOCC_GEMM_NAME(docc_##PREFIX##a_##BM##x##BN##x##BK##s##ST##_##TAG)(  \
        const T* A, const T* B, OT* C, long M, long N, long K, long lda, long ldb, long ldc, OT alpha, OT beta,    \
        const OT* bias, int act, long batch_a, long batch_b, long batch_c) {                                       \
        const long z = blockIdx.y;                                                                                 \
        docc_k::AsyncGemmKernel<T, BM, BN, BK, WM, WN, ST, TA, TB>::run(A + z * batch_a, B + z * batch_b, C + z * batch_c, M, N, \
                                                                        K, lda, ldb, ldc, alpha, beta, bias, act); \
    }

// the same with the copies dealt over the K-step: docc_<prefix>a_<BM>x<BN>x<BK>p<STAGES>_<nn|nt|tn|tt>
#define DOCC_AGEMM_SPREAD_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, TA, TB, TAG)                                   \
    extern "C" __global__ __launch_bounds__(64 * WM * WN) void DOCC_GEMM_NAME(docc_##PREFIX##a_##BM##x##BN##x##BK##p##ST##_##TAG)(  \
        const T* A, const T* B, OT* C, long M, long N, long K, long lda, long ldb, long ldc, OT alpha, OT beta,    \
        const OT* bias, int act, long batch_a, long batch_b, long batch_c) {                                       \
        const long z = blockIdx.y;                                                                                 \
        docc_k::AsyncGemmKernel<T, BM, BN, BK, WM, WN, ST, TA, TB, true>::run(A + z * batch_a, B + z * batch_b, C + z * batch_c, \
                                                                              M, N, K, lda, ldb, ldc, alpha, beta, bias, act);  \
    }

#define DOCC_AGEMM_SPREAD_CONFIG(PREFIX, T, OT, BM, BN, BK, WM, WN, ST)            \
    DOCC_AGEMM_SPREAD_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, false, false, nn)   \
    DOCC_AGEMM_SPREAD_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, false, true, nt)    \
    DOCC_AGEMM_SPREAD_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, true, false, tn)    \
    DOCC_AGEMM_SPREAD_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, true, true, tt)

#define DOCC_AGEMM_CONFIG(PREFIX, T, OT, BM, BN, BK, WM, WN, ST)            \
    DOCC_AGEMM_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, false, false, nn)   \
    DOCC_AGEMM_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, false, true, nt)    \
    DOCC_AGEMM_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, true, false, tn)    \
    DOCC_AGEMM_ONE(PREFIX, T, OT, BM, BN, BK, WM, WN, ST, true, true, tt)
