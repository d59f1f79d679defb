// ml::Attention forward (non-causal), bf16 inputs, head dim 64, for gfx950:
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
// Layout of the computation (one work-group = 128 queries of one head, four
// wavefronts of 32 queries each; K and V blocks are shared through LDS):
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
#include "gemm_mfma.h"

namespace docc_k {

typedef uint16_t u16x8_t __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));

template <>
struct Mfma<uint16_t> {
    static constexpr int VEC = 8;
    typedef u16x8_t vec_t;
};

constexpr int kHeadDim = 64;
constexpr int kBlockQ = 128;   // queries per work-group
constexpr int kBlockKV = 64;   // keys per step
constexpr int kLdK = kHeadDim + 8;    // K tile [key][d], padded
constexpr int kLdV = kHeadDim + 16;   // V tile [key][d], padded for the transposed reads
constexpr int kKElems = kBlockKV * kLdK, kVElems = kBlockKV * kLdV;

template <bool OUT_BF16>
__device__ __forceinline__ void attention_fwd_d64(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                                                  const uint16_t* __restrict__ V, void* __restrict__ O, int SQ,
                                                  int SKV, float scale_log2e) {
    extern __shared__ __attribute__((aligned(16))) unsigned char docc_attn_lds[];
    uint16_t* const lds = reinterpret_cast<uint16_t*>(docc_attn_lds);
    constexpr int V_BASE = 2 * kKElems;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qj = lane & 31, g = lane >> 5;
    const long bh = blockIdx.y;
    const uint16_t* Qh = Q + bh * (long) SQ * kHeadDim;
    const uint16_t* Kh = K + bh * (long) SKV * kHeadDim;
    const uint16_t* Vh = V + bh * (long) SKV * kHeadDim;
    const int q = blockIdx.x * kBlockQ + wave * 32 + qj;   // this lane's query

    // Q^T as the B operand of the score product: d = 16*ks + 8*g .. +7 of query q
    bf16x8 bq[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        u16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (q < SQ) v = *reinterpret_cast<const u16x8_t*>(Qh + (long) q * kHeadDim + 16 * ks + 8 * g);
        bq[ks] = __builtin_bit_cast(bf16x8, v);
    }

    f32x16 ot[2];   // O^T tiles: d = 32*dt + acc_row(lane, r), column = this lane's query
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) ot[dt][r] = 0.f;
    float m_run = -__builtin_huge_valf();   // running max of scale*log2e*score
    float l_part = 0.f;                     // this lane's part of the running sum (its 32 keys per block)

    // K and V blocks: 64 keys x 64 d, walked along the keys; keys past the end read as zero
    typedef TileLoader<uint16_t, kBlockKV, kHeadDim, 256, true, false> KVLoader;
    KVLoader lk, lv;
    const int nblocks = (SKV + kBlockKV - 1) / kBlockKV;
    const int full_blocks = SKV / kBlockKV, keys_left = SKV - full_blocks * kBlockKV;
    lk.init(Kh, kHeadDim, 0, 0, SKV, kHeadDim, tid);
    lv.init(Vh, kHeadDim, 0, 0, SKV, kHeadDim, tid);
    if (full_blocks > 0) {
        lk.load_full();
        lv.load_full();
    } else {
        lk.load_tail(keys_left, tid);
        lv.load_tail(keys_left, tid);
    }
    lk.template store<kLdK>(lds, tid);
    lv.template store<kLdV>(lds + V_BASE, tid);
    __syncthreads();

    // lane roles for the transposed V reads (see gemm_bf16.hip)
    const int ts = lane & 15, tgrp = lane >> 4;
    const int tr_row = 4 * (tgrp >> 1) + (ts >> 2);            // + 16*(u%2) + 32*t (+8 for the high half)
    const int tr_col = 16 * (tgrp & 1) + 4 * (ts & 3);         // + 32*dt
    typedef __attribute__((address_space(3))) s16x4_t lds_s16x4;

    for (int kb = 0; kb < nblocks; kb++) {
        const int cur = kb & 1;
        if (kb + 1 < full_blocks) {
            lk.advance();
            lv.advance();
            lk.load_full();
            lv.load_full();
        } else if (kb + 1 < nblocks) {
            lk.advance();
            lv.advance();
            lk.load_tail(keys_left, tid);
            lv.load_tail(keys_left, tid);
        }
        const uint16_t* ks_ = lds + cur * kKElems;
        const uint16_t* vs_ = lds + V_BASE + cur * kVElems;

        // scores, transposed: st[t][r] = <K[32t + acc_row(r)], Q[q]>
        f32x16 st[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int r = 0; r < 16; r++) st[t][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const u16x8_t kv = *reinterpret_cast<const u16x8_t*>(ks_ + (32 * t + qj) * kLdK + 16 * ks + 8 * g);
                st[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kv), bq[ks], st[t], 0, 0, 0);
            }
        }
        // keys past the end (last block only) score -inf
        if ((kb + 1) * kBlockKV > SKV) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = kb * kBlockKV + 32 * t + Mfma<float>::acc_row(lane, r);
                    if (key >= SKV) st[t][r] = -__builtin_huge_valf();
                }
        }
        // online softmax over this lane's 32 keys and its partner's (lane ^ 32) 32 keys
        float mx = st[0][0];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[t][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx * scale_log2e);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);   // first block: exp2(-inf) = 0
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[t][r], scale_log2e, -m_new));
                st[t][r] = p;
                psum += p;
            }
        l_part = __builtin_fmaf(l_part, alpha, psum);
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) ot[dt][r] *= alpha;

        // O^T += V^T P^T, 16 keys per MFMA; key order inside a step follows the accumulator rows
#pragma unroll
        for (int u = 0; u < 4; u++) {
            bf16x8 pb;
#pragma unroll
            for (int e = 0; e < 8; e++) pb[e] = (__bf16) st[u >> 1][8 * (u & 1) + e];
            const int row = 32 * (u >> 1) + 16 * (u & 1) + tr_row;
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                const uint16_t* vp = vs_ + row * kLdV + 32 * dt + tr_col;
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) vp);
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*) (vp + 8 * kLdV));
                const s16x8_t va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                ot[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, va), pb, ot[dt], 0, 0, 0);
            }
        }

        if (kb + 1 < nblocks) {
            lk.template store<kLdK>(lds + (cur ^ 1) * kKElems, tid);
            lv.template store<kLdV>(lds + V_BASE + (cur ^ 1) * kVElems, tid);
        }
        __syncthreads();
    }

    const float l = l_part + __shfl_xor(l_part, 32, 64);
    const float inv = 1.0f / l;
    if (q < SQ) {
#pragma unroll
        for (int dt = 0; dt < 2; dt++) {
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                const int d = 32 * dt + 8 * rq + 4 * g;   // registers 4*rq .. 4*rq+3 hold d .. d+3
                const long off = (bh * (long) SQ + q) * kHeadDim + d;
                if (OUT_BF16) {
                    u16x4_t o;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = f32_to_bf16_rne(ot[dt][4 * rq + e] * inv);
                    *reinterpret_cast<u16x4_t*>(reinterpret_cast<uint16_t*>(O) + off) = o;
                } else {
                    f32x4 o;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = ot[dt][4 * rq + e] * inv;
                    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(O) + off) = o;
                }
            }
        }
    }
}

} // namespace docc_k

extern "C" __global__ __launch_bounds__(256) void docc_attention_bf16_d64_f32out(const uint16_t* Q, const uint16_t* K,
                                                                                 const uint16_t* V, void* O, int SQ,
                                                                                 int SKV, float scale_log2e) {
    docc_k::attention_fwd_d64<false>(Q, K, V, O, SQ, SKV, scale_log2e);
}

extern "C" __global__ __launch_bounds__(256) void docc_attention_bf16_d64_bf16out(const uint16_t* Q, const uint16_t* K,
                                                                                  const uint16_t* V, void* O, int SQ,
                                                                                  int SKV, float scale_log2e) {
    docc_k::attention_fwd_d64<true>(Q, K, V, O, SQ, SKV, scale_log2e);
}
