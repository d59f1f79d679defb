// ml::Attention forward (all keys, or causal), bf16 inputs, head dim 32, 64 or 128, for gfx950:
//   O[b,h,i,:] = sum_j softmax_j(scale * <Q[b,h,i,:], K[b,h,j,:]>) V[b,h,j,:]
// with fp32 scores, softmax statistics and accumulation.
//
// The reference has no attention node and its MatMul node cannot take batched
// operands from the torch path (mlir/lib/Target/SDFG/LinalgToSDFGTranslator.cpp:517-523);
// composed from its own nodes this would be MatMul -> scale -> Softmax
// (softmax_node.cpp:142-252) -> MatMul with an [S,S] fp32 score matrix per
// head in memory. This kernel never stores scores: it walks the keys in
// blocks of 64 with an online max/sum (flash-attention style).
//
// Layout of the computation (one work-group = four wavefronts of one head - eight at head dim 128 -, each with QT
// tiles of 32 queries: 256 queries per work-group with QT = 2, 128 with QT = 1; K and V blocks are shared through LDS;
// the figures below are those of head dim 64, the case the kernel was tuned on):
//   S^T[key, q]  = K_blk[key, d] * Q^T[d, q]     v_mfma_f32_32x32x16_bf16, A = K (d-contiguous
//                                                128-bit LDS reads), B = Q (kept in registers)
//   the transposed product puts one query per lane (column = lane % 32) and 32 of
//   the block's 64 keys in that lane's registers, so max and sum over keys are
//   register reductions plus one exchange between lane and lane^32, and the
//   per-query rescale of the output is a per-lane scalar;
//   O^T[d, q]   += V^T[d, key] * P^T[key, q]     A = V read transposed from its [key][d] LDS
//                                                tile with ds_read_b64_tr_b16, B = P^T taken
//                                                from the S^T accumulator registers as they
//                                                are (the k-order of the MFMA is permuted to
//                                                the accumulator's row order on both operands).
//
// What bounds it on this device: the vector ALU next to the matrix pipe. Per 64-key block and 64 queries a wave issues
// 32 MFMAs (1024 cycles of the matrix pipe) and 64 exp2, 64 fma, 32 cvt_pk, 32 dot2 (about as many cycles of the vector
// pipe), and the two hardly overlap: with pieces of the block loop taken out one at a time the time falls by the share
// of the instructions removed, whatever pipe they ran on (16 MFMAs 56 %, the eight 128-bit K reads 10 %, the sixteen
// transposed V reads 6 %, the copies 9 %, 16 dot2 7.6 %, 32 exp 17 %, 32 fma 7 %), and a wave that streams MFMAs
// leaves the other wave of its SIMD about 55 % of the vector pipe's rate (measured with two-wave probes: 24 such vector
// instructions take 71 ns alone and 128 ns beside a wave issuing MFMAs back to back, which itself is not slowed).
// Issuing the score MFMAs of the next block between the exponentials changes nothing. The power limit adds about 8 %
// on N(0,1) operands (the same launch on zeros). So the design goal is the fewest instructions per flop:
//   - QT = 2: a wavefront takes 64 queries, so every K and V operand read from LDS, and every block copied
//     into LDS, serves twice the MFMAs (LDS reads and copies per flop halve);
//   - p = exp2(s * c - m) with c = scale * log2(e) applied to the fp32 score by one fma: Q and K enter
//     the MFMA as they are (folding c into a re-rounded bf16 Q costs 2^-9 of every product, which at
//     logits of +-60 is an error of 1.6e-2 in the result);
//   - m does not have to be the exact running maximum: softmax is shift invariant and fp32/bf16
//     keep their relative precision at any magnitude, so m stays what the first block set until a
//     block's row sum shows growth beyond 2^40 (or inf, or NaN) - only then the block takes the slow
//     path (scores recomputed, true block maximum, rescale of the output and the sum, p again). The usual
//     block has no max pass and no rescale. A lane that has seen nothing but -inf scores so far keeps
//     m = -inf, which makes its next block's sum inf or NaN and so leads it through the slow path until a
//     finite score turns up;
//   - p is packed to bf16 with v_cvt_pk_bf16_f32 and the row sum is taken from the packed values with
//     v_dot2c_f32_bf16: it sums exactly what the second product multiplies.
// K/V blocks arrive in a ring of three LDS stages by asynchronous global->LDS copies, two blocks ahead.
#include "gemm_mfma.h"
#include <type_traits>

namespace docc_k {

typedef uint16_t u16x8_t __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* attn_lds_ptr_t;
typedef const __attribute__((address_space(1))) void* attn_global_ptr_t;

template <>
struct Mfma<uint16_t> {
    static constexpr int VEC = 8;
    typedef u16x8_t vec_t;
};

constexpr int kBlockKV = 64;     // keys per step
constexpr int kAttnStages = 3;   // LDS ring depth: blocks kb+1 and kb+2 are in flight while block kb is worked on

// granule (8 bf16) index inside a row of HD / 8 granules, swizzled so that the reads below are conflict-free:
// K: sixteen lanes of a 128-bit read touch 16 consecutive rows at one granule column; V: half a wavefront of a
// transposed 64-bit read touches 4 consecutive rows x 4 granule columns. The LDS moves 256 bytes a cycle, which is
// four rows at head dim 32, two at 64 and one at 128: the swizzle spreads the rows that would meet in the same banks.
template <int HD> __device__ __forceinline__ int attn_k_swz(int row);
template <> __device__ __forceinline__ int attn_k_swz<32>(int row) { return (row >> 2) & 3; }
template <> __device__ __forceinline__ int attn_k_swz<64>(int row) { return (row >> 1) & 7; }
template <> __device__ __forceinline__ int attn_k_swz<128>(int row) { return row & 15; }
template <int HD> __device__ __forceinline__ int attn_v_swz(int row);
template <> __device__ __forceinline__ int attn_v_swz<32>(int) { return 0; }
template <> __device__ __forceinline__ int attn_v_swz<64>(int row) { return ((row >> 1) & 1) << 2; }
template <> __device__ __forceinline__ int attn_v_swz<128>(int row) { return (row & 3) << 2; }
template <int HD> __device__ __forceinline__ int attn_k_off(int row, int cv) { return (row * (HD / 8) + (cv ^ attn_k_swz<HD>(row))) * 8; }
template <int HD> __device__ __forceinline__ int attn_v_off(int row, int cv) { return (row * (HD / 8) + (cv ^ attn_v_swz<HD>(row))) * 8; }

// x of lanes 0..31 (which = 0) or of lanes 32..63 (which = 1), seen from both halves of the wave:
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second.
// The second operand goes through an empty asm so that the compiler cannot treat the two results
// of a swap of equal inputs as equal.
__device__ __forceinline__ float half_swap(float x, int which) {
    unsigned a = __builtin_bit_cast(unsigned, x), b = a;
    asm volatile("" : "+v"(b));
    const auto sw = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    return __builtin_bit_cast(float, which ? sw[1] : sw[0]);
}

// CAUSAL: query i sees the keys j <= i (torch's is_causal: the mask is aligned at the top left whatever SQ and SKV are, so
// every query sees key 0 and no row is empty). A work-group then walks the blocks up to its last query's only, and the
// blocks that reach past a wavefront's first query have the scores of the later keys set to -inf.
template <bool OUT_BF16, int QT, int HD, int NW, bool CAUSAL = false>
__device__ __forceinline__ void attention_fwd(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                                              const uint16_t* __restrict__ V, void* __restrict__ O, int SQ,
                                              int SKV, float scale_log2e) {
    extern __shared__ __attribute__((aligned(16))) unsigned char docc_attn_lds[];
    uint16_t* const lds = reinterpret_cast<uint16_t*>(docc_attn_lds);
    constexpr int kHeadDim = HD;
    constexpr int kBlockQ = NW * 32 * QT;                    // queries per work-group
    constexpr int kTileElems = kBlockKV * kHeadDim;          // one K or V block, unpadded, 16-byte granules swizzled
    constexpr int kStageElems = 2 * kTileElems;              // [K | V]
    constexpr int GR = HD / 8;                               // granules per row of a block
    constexpr int RP = NW * 64 / GR;                         // rows of a block that the work-group copies at a time
    constexpr int PASSES = kBlockKV / RP;
    constexpr int KS = HD / 16, DT = HD / 32;                // MFMA steps over d of the score product, 32-row tiles of O^T
    static_assert(PASSES >= 1 && PASSES * RP == kBlockKV, "the work-group's lanes must tile a block");

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qj = lane & 31, g = lane >> 5;
    // work-group -> (head, query block): consecutive work-group ids go round the 8 XCDs, so the id is
    // renumbered to give each XCD whole heads - the query blocks of a head then share one L2
    const int nqb = gridDim.x, total = gridDim.x * gridDim.y;
    int lid = blockIdx.y * gridDim.x + blockIdx.x;
    if (total % 8 == 0) lid = (lid % 8) * (total / 8) + lid / 8;
    const long bh = lid / nqb;
    // Causal: a work-group takes a pair of query blocks, the one with the most keys and the one with the fewest of what is
    // left (blocks t and T - 1 - t of the T = ceil(SQ / kBlockQ) of a head), one after the other: every work-group then has
    // the same number of key blocks to walk, and the launch does not end on a few long ones (the grid's x extent is the
    // number of pairs; the middle block of an odd T is a pair of one)
    const int tiles_q = (SQ + kBlockQ - 1) / kBlockQ;
    const int first_of_pair = lid % nqb;
    // one query block of the head, start to finish
    auto run_block = [&](const int qblk) {
    const uint16_t* Qh = Q + bh * (long) SQ * kHeadDim;
    const char* Kh = reinterpret_cast<const char*>(K + bh * (long) SKV * kHeadDim);
    const char* Vh = reinterpret_cast<const char*>(V + bh * (long) SKV * kHeadDim);
    const int q0 = qblk * kBlockQ + wave * (32 * QT) + qj;   // this lane's queries: q0 + 32 * qt
    const float c = scale_log2e;
    const float ninf = -__builtin_huge_valf();

    // Q^T as the B operand of the score product: d = 16*ks + 8*g .. +7 of query q0 + 32*qt
    bf16x8 bq[QT][KS];
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            u16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (q0 + 32 * qt < SQ) v = *reinterpret_cast<const u16x8_t*>(Qh + (long) (q0 + 32 * qt) * kHeadDim + 16 * ks + 8 * g);
            bq[qt][ks] = __builtin_bit_cast(bf16x8, v);
        }

    const int all_blocks = (SKV + kBlockKV - 1) / kBlockKV;
    const int wg_last_query = qblk * kBlockQ + kBlockQ - 1 < SQ - 1 ? qblk * kBlockQ + kBlockQ - 1 : SQ - 1;
    const int nblocks = CAUSAL && wg_last_query / kBlockKV + 1 < all_blocks ? wg_last_query / kBlockKV + 1 : all_blocks;
    const int wave_first_query = qblk * kBlockQ + wave * (32 * QT);
    const int full_blocks = SKV / kBlockKV, keys_left = SKV - full_blocks * kBlockKV;

    // K/V copies: a block is 64 * GR granules of 16 bytes per tensor, PASSES per thread. LDS slot s (in copy
    // order: lane-contiguous) holds row s / GR, granule column (s % GR) ^ swizzle(row). The later granules of a
    // lane lie RP rows below the first, where both swizzles repeat: one offset per tensor serves all.
    const int copy_row = wave * (64 / GR) + lane / GR;
    const unsigned koff = (unsigned) ((copy_row * GR + ((lane % GR) ^ attn_k_swz<HD>(copy_row))) * 16);
    const unsigned voff = (unsigned) ((copy_row * GR + ((lane % GR) ^ attn_v_swz<HD>(copy_row))) * 16);
    constexpr unsigned kPassBytes = RP * HD * 2;
    auto issue = [&](int kb) {   // starts the copy of block kb into its stage
        uint16_t* st = lds + (kb % kAttnStages) * kStageElems;
        const char* kp = Kh + (long) kb * (kTileElems * 2);
        const char* vp = Vh + (long) kb * (kTileElems * 2);
        if (kb < full_blocks) {
            // scalar base + 32-bit lane offset: the empty asm keeps the compiler from adding the head's base to
            // the offsets once, outside the loop, which would cost 64-bit addresses per lane
            unsigned ko = koff, vo = voff;
            asm volatile("" : "+v"(ko), "+v"(vo));
#pragma unroll
            for (int i = 0; i < PASSES; i++) {
                __builtin_amdgcn_global_load_lds((attn_global_ptr_t) (kp + kPassBytes * i + ko), (attn_lds_ptr_t) (st + (i * NW + wave) * 512), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((attn_global_ptr_t) (vp + kPassBytes * i + vo), (attn_lds_ptr_t) (st + kTileElems + (i * NW + wave) * 512), 16, 0, 0);
            }
        } else {
            // the partial last block: rows past the end copy the last key (their scores are masked, their V rows zeroed)
#pragma unroll
            for (int i = 0; i < PASSES; i++) {
                const int row = copy_row + RP * i;
                const unsigned back = row >= keys_left ? (unsigned) ((row - (keys_left - 1)) * (HD * 2)) : 0u;
                __builtin_amdgcn_global_load_lds((attn_global_ptr_t) (kp + (koff + kPassBytes * i - back)), (attn_lds_ptr_t) (st + (i * NW + wave) * 512), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((attn_global_ptr_t) (vp + (voff + kPassBytes * i - back)), (attn_lds_ptr_t) (st + kTileElems + (i * NW + wave) * 512), 16, 0, 0);
            }
        }
    };
    // block kb has landed in every wave's view and every wave is done with block kb-1; rows of a partial
    // last V block are cleared so that 0 * (copied value) cannot produce a NaN
    auto arrive = [&](int kb) {
        // each block is 2 * PASSES copies per lane; one newer block may still be in flight
        if (kb + 1 < nblocks) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * PASSES) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (kb >= full_blocks) {
            uint16_t* vt = lds + (kb % kAttnStages) * kStageElems + kTileElems;
            const u16x8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int s = keys_left * GR + tid; s < kBlockKV * GR; s += 64 * NW) *reinterpret_cast<u16x8_t*>(vt + s * 8) = z;
            __syncthreads();
        }
    };

    f32x16 ot[QT][DT];  // O^T tiles: d = 32*dt + acc_row(lane, r), column = this lane's query of tile qt
    float m_run[QT];    // reference point of the exponentials (log2 domain); -inf: nothing finite seen yet
    float l_part[QT];   // this lane's part of the running sum (its 32 keys per block)
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        m_run[qt] = ninf;
        l_part[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) ot[qt][dt][r] = 0.f;
    }

    // lane roles for the transposed V reads (see gemm_bf16.hip)
    const int ts = lane & 15, tgrp = lane >> 4;
    const int tr_row = 4 * (tgrp >> 1) + (ts >> 2);            // + 16*(u%2) + 32*t (+8 for the high half)
    const int tr_col = 16 * (tgrp & 1) + 4 * (ts & 3);         // + 32*dt
    typedef __attribute__((address_space(3))) s16x4_t lds_s16x4;

    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // raw scores, transposed: s[qt][t][r] = <K[32t + acc_row(r)], Q[q0 + 32 qt]>; keys past the end score -inf.
    // All K operands are requested before the first MFMA: one LDS round trip, not eight; each serves QT MFMAs.
    auto scores = [&](int kb, f32x16 (&s)[QT][2]) {
        const uint16_t* ks_ = lds + (kb % kAttnStages) * kStageElems;
        u16x8_t kv[2][KS];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) kv[t][ks] = *reinterpret_cast<const u16x8_t*>(ks_ + attn_k_off<HD>(32 * t + qj, 2 * ks + g));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
                    s[qt][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kv[t][ks]), bq[qt][ks],
                                                                      ks == 0 ? zero16 : s[qt][t], 0, 0, 0);
        if ((kb + 1) * kBlockKV > SKV) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (kb * kBlockKV + 32 * t + Mfma<float>::acc_row(lane, r) >= SKV) {
#pragma unroll
                        for (int qt = 0; qt < QT; qt++) s[qt][t][r] = ninf;
                    }
        }
        if (CAUSAL && (kb + 1) * kBlockKV - 1 > wave_first_query) {   // the block holds keys past this wavefront's first query
            // key = 64 kb + 32 t + 8 (r / 4) + 4 g + r % 4 > query  <=>  32 t + 8 (r / 4) + r % 4 > query - 64 kb - 4 g: a constant of
            // the instruction against one value per lane and query tile, no table of key numbers in registers
#pragma unroll
            for (int qt = 0; qt < QT; qt++) {
                const int lim = q0 + 32 * qt - kb * kBlockKV - 4 * g;
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        s[qt][t][r] = 32 * t + 8 * (r / 4) + (r % 4) > lim ? ninf : s[qt][t][r];
            }
        }
    };

    bf16x2_t pk[QT][2][8];
    bf16x2_t ones;
    ones[0] = (__bf16) 1.0f;
    ones[1] = (__bf16) 1.0f;
    // p = exp2(s*c - mc), packed to bf16 pairs in accumulator order; returns the lane's row sum of the packed values
    auto exponentials = [&](const f32x16 (&s)[2], bf16x2_t (&pq)[2][8], float mc) {
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                bf16x2_t pp;
                pp[0] = (__bf16) __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], c, -mc));
                pp[1] = (__bf16) __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r + 1], c, -mc));
                pq[t][r / 2] = pp;
                psum = __builtin_amdgcn_fdot2_f32_bf16(pp, ones, psum, false);
            }
        return psum;
    };
    // reference point a lane subtracts: 0 while it has seen no finite score (its scores are all -inf then, p = 0)
    auto base_of = [&](float m) { return m == ninf ? 0.f : m; };
    // the maximum of the scaled scores of the lane pair's query (c > 0)
    auto scaled_max = [&](const f32x16 (&s)[2]) {
        float mx = s[0][0];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[t][r]);
        return fmaxf(half_swap(mx, 0), half_swap(mx, 1)) * c;
    };

    f32x16 st[QT][2];
    // one block: scores -> exponentials -> O^T += V^T P^T
    auto block = [&](int kb, auto first_c) {
        constexpr bool FIRST = decltype(first_c)::value;
        // block kb must have landed; after the barrier every wave is done with block kb-1, whose
        // stage takes block kb+2
        arrive(kb);
        if (kb + 2 < nblocks) issue(kb + 2);
        scores(kb, st);
        if (FIRST) {
            // the first block sets the reference point
#pragma unroll
            for (int qt = 0; qt < QT; qt++) m_run[qt] = scaled_max(st[qt]);
        }
        float psum[QT];
        bool slow = false;
#pragma unroll
        for (int qt = 0; qt < QT; qt++) {
            psum[qt] = exponentials(st[qt], pk[qt], base_of(m_run[qt]));
            // growth of the maximum beyond 2^40 over the reference point (or an overflow, or a NaN) shows in the sum
            slow = slow || !(psum[qt] < 0x1p40f);
        }
        if (__builtin_amdgcn_ballot_w64(slow) != 0) {
            // the slow path: the reference point moves to the maximum of what the lane pair has seen. The raw
            // scores were consumed by the packing, so they are computed again (K of block kb is still in LDS).
            scores(kb, st);
#pragma unroll
            for (int qt = 0; qt < QT; qt++) {
                const float m_new = fmaxf(m_run[qt], scaled_max(st[qt]));     // fmaxf drops a NaN: it shows up in p instead
                // exp2(-inf - -inf) would be NaN: a lane that still has nothing finite has nothing to rescale either
                const float alpha = m_new == ninf ? 1.f : __builtin_amdgcn_exp2f(m_run[qt] - m_new);
                m_run[qt] = m_new;
                l_part[qt] *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int r = 0; r < 16; r++) ot[qt][dt][r] *= alpha;
                psum[qt] = exponentials(st[qt], pk[qt], base_of(m_new));
            }
        }
#pragma unroll
        for (int qt = 0; qt < QT; qt++) l_part[qt] += psum[qt];

        // O^T += V^T P^T, 16 keys per MFMA; key order inside a step follows the accumulator rows.
        // The V operands of two steps are requested together (they do not depend on P); each serves QT MFMAs.
        const uint16_t* vs_ = lds + (kb % kAttnStages) * kStageElems + kTileElems;
        auto pv_half = [&](int h) {
            s16x8_t va[2][DT];
#pragma unroll
            for (int uu = 0; uu < 2; uu++) {
                const int u = 2 * h + uu;
                const int row = 32 * (u >> 1) + 16 * (u & 1) + tr_row;
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const int col = 32 * dt + tr_col;
                    const uint16_t* plo = vs_ + attn_v_off<HD>(row, col >> 3) + (col & 7);
                    const uint16_t* phi = vs_ + attn_v_off<HD>(row + 8, col >> 3) + (col & 7);
                    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) plo);
                    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) phi);
                    va[uu][dt] = s16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int uu = 0; uu < 2; uu++) {
                const int u = 2 * h + uu;
#pragma unroll
                for (int qt = 0; qt < QT; qt++) {
                    struct Pack { bf16x2_t v[4]; } pack = {{pk[qt][u >> 1][4 * (u & 1)], pk[qt][u >> 1][4 * (u & 1) + 1],
                                                            pk[qt][u >> 1][4 * (u & 1) + 2], pk[qt][u >> 1][4 * (u & 1) + 3]}};
                    const bf16x8 pb = __builtin_bit_cast(bf16x8, pack);
#pragma unroll
                    for (int dt = 0; dt < DT; dt++)
                        ot[qt][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, va[uu][dt]), pb, ot[qt][dt], 0, 0, 0);
                }
            }
        };
        pv_half(0);
        pv_half(1);
    };

    issue(0);
    if (nblocks > 1) issue(1);
    block(0, std::true_type{});
    for (int kb = 1; kb < nblocks; kb++) block(kb, std::false_type{});

#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        const int q = q0 + 32 * qt;
        const float l = half_swap(l_part[qt], 0) + half_swap(l_part[qt], 1);
        const float inv = 1.0f / l;
        if (q < SQ) {
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int d = 32 * dt + 8 * rq + 4 * g;   // registers 4*rq .. 4*rq+3 hold d .. d+3
                    const long off = (bh * (long) SQ + q) * kHeadDim + d;
                    if (OUT_BF16) {
                        u16x4_t o;
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = f32_to_bf16_rne(ot[qt][dt][4 * rq + e] * inv);
                        *reinterpret_cast<u16x4_t*>(reinterpret_cast<uint16_t*>(O) + off) = o;
                    } else {
                        f32x4 o;
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = ot[qt][dt][4 * rq + e] * inv;
                        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(O) + off) = o;
                    }
                }
            }
        }
    }
    };
    if constexpr (!CAUSAL) {
        run_block(first_of_pair);
    } else {
#pragma unroll 1
        for (int pass = 0; pass < 2; pass++) {
            if (pass == 1 && first_of_pair == tiles_q - 1 - first_of_pair) break;
            run_block(pass == 0 ? tiles_q - 1 - first_of_pair : first_of_pair);
            __syncthreads();   // every wave is done with the LDS ring before the next query block's copies land in it
        }
    }
}

} // namespace docc_k

#define DOCC_ATTENTION_KERNEL_D(name, out_bf16, qt, waves, hd, nw)                                                                \
    extern "C" __global__ __launch_bounds__(64 * nw) __attribute__((amdgpu_waves_per_eu(waves))) void name(                       \
        const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O, int SQ, int SKV, float scale_log2e) {                   \
        docc_k::attention_fwd<out_bf16, qt, hd, nw>(Q, K, V, O, SQ, SKV, scale_log2e);                                            \
    }                                                                                                                             \
    extern "C" __global__ __launch_bounds__(64 * nw) __attribute__((amdgpu_waves_per_eu(waves))) void name##_causal(              \
        const uint16_t* Q, const uint16_t* K, const uint16_t* V, void* O, int SQ, int SKV, float scale_log2e) {                   \
        docc_k::attention_fwd<out_bf16, qt, hd, nw, true>(Q, K, V, O, SQ, SKV, scale_log2e);                                      \
    }
#define DOCC_ATTENTION_KERNEL(name, out_bf16, qt, waves) DOCC_ATTENTION_KERNEL_D(name, out_bf16, qt, waves, 64, 4)

// 64 queries per wavefront (256 per work-group): the form for long query axes
DOCC_ATTENTION_KERNEL(docc_attention_bf16_d64_q256_f32out, false, 2, 2)
DOCC_ATTENTION_KERNEL(docc_attention_bf16_d64_q256_bf16out, true, 2, 2)
// 32 queries per wavefront (128 per work-group): more work-groups where there are few queries
DOCC_ATTENTION_KERNEL(docc_attention_bf16_d64_q128_f32out, false, 1, 3)
DOCC_ATTENTION_KERNEL(docc_attention_bf16_d64_q128_bf16out, true, 1, 3)
// head dim 32: the same two forms (half the MFMAs per block, the vector work of the softmax unchanged)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d32_q256_f32out, false, 2, 2, 32, 4)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d32_q256_bf16out, true, 2, 2, 32, 4)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d32_q128_f32out, false, 1, 3, 32, 4)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d32_q128_bf16out, true, 1, 3, 32, 4)
// head dim 128: 32 queries per wavefront (the registers hold one tile of queries: 64 of O^T, 32 of Q, 64 of K operands),
// eight wavefronts share the K and V blocks of a work-group (96 KB of LDS: one work-group per CU, two wavefronts per SIMD);
// the four-wavefront form is for short query axes
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d128_q256_f32out, false, 1, 2, 128, 8)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d128_q256_bf16out, true, 1, 2, 128, 8)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d128_q128_f32out, false, 1, 1, 128, 4)
DOCC_ATTENTION_KERNEL_D(docc_attention_bf16_d128_q128_bf16out, true, 1, 1, 128, 4)
