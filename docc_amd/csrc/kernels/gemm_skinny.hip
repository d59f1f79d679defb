// A few rows times a wide matrix for gfx950: C[m, n] = alpha * A[m, k] * op(B) + beta * C with m up to 32 and n, k in the
// thousands (a batch of vectors through a layer); fp32 first, bf16 with B stored [n][k] further down. The product reads B once (4 k n bytes) for 2 m k n flops, so it is bound by
// HBM as long as the MFMA work stays small: the 32 x 32 x 2 instruction allows 9.8 TB/s of B at the device's fp32 rate, the
// 16 x 16 x 4 one (m <= 16) twice that. The tiles of the GEMM kernels stage both operands through LDS in steps a work-group
// waits out and pad m to 64; here B goes from global memory straight into the MFMA operand registers:
//   * a work-group owns 128 columns of one part of K; its NW wavefronts cut that part among themselves, every wavefront
//     keeps an MT x 128 block of sums in registers (MT = 16 or 32 rows);
//   * K advances in chunks of CH: a lane holds CH / G consecutive k of its row of A (G = 64 / MT lane groups along k) and
//     loads, for each of those k, the columns (B stored [k][n]: 128-bit loads along n) or, for its rows of B (B stored
//     [n][k]), 128-bit loads along k that it feeds to the MFMA; the loads of the next chunks are issued before the products
//     of this one;
//   * the wavefronts' blocks are added pairwise through LDS (wave w + NW/2 into wave w, then halves again), and wave 0
//     stores the part's product; the launcher adds the parts in order with docc_splitk_combine_f32, so the result does
//     not depend on scheduling. With one part the store applies alpha and beta itself.
// Sums run in fp32 (cblas_sgemm semantics, reference gemm_node.cpp:474-505).
#include "common.h"

namespace docc_k {

typedef float skinny_f32x4 __attribute__((ext_vector_type(4)));
typedef float skinny_f32x16 __attribute__((ext_vector_type(16)));

template <int MT> struct SkinnyMfma;
template <> struct SkinnyMfma<32> {
    typedef skinny_f32x16 acc_t;
    static constexpr int NACC = 16;
    static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
    // row of register r of the block of sums for lane group g (the column is the lane's index within its group)
    static __device__ __forceinline__ int row(int g, int r) { return 8 * (r / 4) + 4 * g + (r % 4); }
};
template <> struct SkinnyMfma<16> {
    typedef skinny_f32x4 acc_t;
    static constexpr int NACC = 4;
    static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row(int g, int r) { return 4 * g + r; }
};

// MT: rows of the MFMA (m <= MT). TB: B stored [n][k] (C = A B^T). NW: wavefronts per work-group. CH: k per chunk. NBUF: sets
// of operand registers, NBUF - 1 chunks' loads are in flight during a chunk's products.
// P: the part's product, [parts][m][ldp] when direct == 0, else C itself (one part).
template <int MT, bool TB, int NW, int CH, int NBUF>
__device__ __forceinline__ void gemm_skinny(const float* __restrict__ A, long lda, const float* __restrict__ B, long ldb, float* __restrict__ P,
                                            long ldp, long m, long n, long k, long kpart, float alpha, float beta, int direct) {
    typedef SkinnyMfma<MT> M;
    typedef typename M::acc_t acc_t;
    constexpr int G = 64 / MT;       // lane groups along k
    constexpr int KL = CH / G;       // consecutive k of a lane in a chunk
    constexpr int NJ = 128 / MT;     // MFMA blocks of sums across the 128 columns
    constexpr int SETS = NJ / 4;     // NN: 128-bit loads of a lane per k (4 MT columns each over the wavefront)
    constexpr int NLOAD = TB ? NJ * KL / 4 : KL * SETS;   // 128-bit loads of B per lane and chunk
    constexpr int SLOT = NJ * M::NACC / 4 * 64;           // 128-bit words of a wavefront's block of sums
    extern __shared__ __attribute__((aligned(16))) unsigned char skinny_lds[];
    skinny_f32x4* lds = reinterpret_cast<skinny_f32x4*>(skinny_lds);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave: uniform, in a scalar register
    const int c = lane % MT, g = lane / MT;
    const long n0 = (long) blockIdx.x * 128;
    const long part = blockIdx.y;
    const long kw = kpart / NW;                       // a multiple of CH
    const long k_begin = part * kpart + wave * kw;
    long k_end = k_begin + kw;
    if (k_end > k) k_end = k;

    acc_t acc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int r = 0; r < M::NACC; r++) acc[j][r] = 0.0f;

    // Addresses are a base every lane shares (the chunk's first k; the compiler keeps it in scalar registers) plus a 32-bit
    // offset of the lane. NN: the lane's columns n0 + 4 MT s + 4c .. + 3 (s < SETS) at k + KL g; NT: its rows of B
    // n0 + MT j + c at k + KL g
    const unsigned b_lane = TB ? (unsigned) (c * ldb + KL * g) : (unsigned) (KL * g * ldb + 4 * c);
    const unsigned a_lane = (unsigned) (c * lda + KL * g);
    const skinny_f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};

    auto load_b = [&](long kb, skinny_f32x4 (&bv)[NLOAD]) {
        const long kl = kb + KL * g;   // the lane's k of this chunk
        const bool whole = kb + CH <= k_end;
        if (TB) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const bool ok = n0 + MT * j + c < n;
                const float* base = B + (n0 + MT * j) * ldb + kb;
#pragma unroll
                for (int q = 0; q < KL / 4; q++)
                    bv[j * (KL / 4) + q] = ok && (whole || kl + 4 * q < k_end) ? *reinterpret_cast<const skinny_f32x4*>(base + b_lane + 4 * q) : zero4;
            }
        } else {
#pragma unroll
            for (int i = 0; i < KL; i++)
#pragma unroll
                for (int s = 0; s < SETS; s++) {
                    const bool ok = n0 + 4 * MT * s + 4 * c < n;
                    const float* base = B + (kb + i) * ldb + n0 + 4 * MT * s;
                    bv[i * SETS + s] =
                        ok && (whole || kl + i < k_end) ? __builtin_nontemporal_load(reinterpret_cast<const skinny_f32x4*>(base + b_lane)) : zero4;
                }
        }
    };
    auto load_a = [&](long kb, skinny_f32x4 (&av)[KL / 4]) {
        const long kl = kb + KL * g;
        const bool whole = kb + CH <= k_end;
        const float* base = A + kb;
#pragma unroll
        for (int q = 0; q < KL / 4; q++)
            av[q] = c < m && (whole || kl + 4 * q < k_end) ? *reinterpret_cast<const skinny_f32x4*>(base + a_lane + 4 * q) : zero4;
    };
    auto products = [&](const skinny_f32x4 (&av)[KL / 4], const skinny_f32x4 (&bv)[NLOAD]) {
#pragma unroll
        for (int i = 0; i < KL; i++)
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const float a = av[i / 4][i % 4];
                const float b = TB ? bv[j * (KL / 4) + i / 4][i % 4] : bv[i * SETS + j / 4][j % 4];
                acc[j] = M::mfma(a, b, acc[j]);
            }
    };

    {
        skinny_f32x4 bq[NBUF][NLOAD], aq[NBUF][KL / 4];
#pragma unroll
        for (int u = 0; u < NBUF - 1; u++) {
            load_b(k_begin + u * CH, bq[u]);   // past k_end: zeros, no access
            load_a(k_begin + u * CH, aq[u]);
        }
        // NBUF chunks a turn, so that the sets of operand registers rotate by name
        for (long kb = k_begin; kb < k_end; kb += NBUF * CH) {
#pragma unroll
            for (int u = 0; u < NBUF; u++) {
                const long kc = kb + u * CH;
                if (kc < k_end) {
                    load_b(kc + (NBUF - 1) * CH, bq[(u + NBUF - 1) % NBUF]);
                    load_a(kc + (NBUF - 1) * CH, aq[(u + NBUF - 1) % NBUF]);
                    products(aq[u], bq[u]);
                }
            }
        }
    }

    // The wavefronts' blocks meet in LDS, NW/2 places of SLOT words. Word (j / 4, r) of a lane holds register r of its blocks
    // 4 (j / 4) .. + 3: for NN the four columns of one 128-bit store.
#pragma unroll
    for (int half = NW / 2; half >= 1; half /= 2) {
        if (wave >= half && wave < 2 * half) {
            skinny_f32x4* slot = lds + (long) (wave - half) * SLOT;
#pragma unroll
            for (int s = 0; s < NJ / 4; s++)
#pragma unroll
                for (int r = 0; r < M::NACC; r++) {
                    skinny_f32x4 v = {acc[4 * s][r], acc[4 * s + 1][r], acc[4 * s + 2][r], acc[4 * s + 3][r]};
                    slot[(s * M::NACC + r) * 64 + lane] = v;
                }
        }
        __syncthreads();
        if (wave < half) {
            const skinny_f32x4* slot = lds + (long) wave * SLOT;
#pragma unroll
            for (int s = 0; s < NJ / 4; s++)
#pragma unroll
                for (int r = 0; r < M::NACC; r++) {
                    const skinny_f32x4 v = slot[(s * M::NACC + r) * 64 + lane];
                    acc[4 * s][r] += v[0];
                    acc[4 * s + 1][r] += v[1];
                    acc[4 * s + 2][r] += v[2];
                    acc[4 * s + 3][r] += v[3];
                }
        }
        __syncthreads();
    }
    if (wave != 0) return;
    float* out = direct ? P : P + part * m * ldp;
#pragma unroll
    for (int r = 0; r < M::NACC; r++) {
        const long row = M::row(g, r);
        if (row >= m) continue;
        if (TB) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const long col = n0 + MT * j + c;
                if (col >= n) continue;
                float* o = out + row * ldp + col;
                const float v = acc[j][r];
                *o = direct ? (beta == 0.0f ? alpha * v : alpha * v + beta * *o) : v;
            }
        } else {
#pragma unroll
            for (int s = 0; s < SETS; s++) {
                const long col = n0 + 4 * MT * s + 4 * c;
                if (col >= n) continue;
                skinny_f32x4* o = reinterpret_cast<skinny_f32x4*>(out + row * ldp + col);
                skinny_f32x4 v = {acc[4 * s][r], acc[4 * s + 1][r], acc[4 * s + 2][r], acc[4 * s + 3][r]};
                if (direct) {
                    if (beta == 0.0f) {
                        v = alpha * v;
                    } else {
                        const skinny_f32x4 old = *o;
                        v = alpha * v + beta * old;
                    }
                }
                *o = v;
            }
        }
    }
}

// bf16 operands, B stored [n][k] (the layout of a layer's weights), fp32 sums and result: v_mfma_f32_16x16x32_bf16 takes eight
// consecutive k of a row of B per lane - exactly a 128-bit load from that row, so B goes from global memory into the
// instruction as it is. A work-group owns 64 columns of one part of K; K advances in chunks of 64 (two loads per lane and
// group of 16 columns: a row's 128-byte line is used up within the chunk). RT blocks of 16 rows of A share the loads of B; the
// matrix pipe is idle most of the time (a kilobyte of B per 16 cycles), the product is bound by reading B. Four blocks of rows
// (230 registers) ran slower than the tiles.
template <int RT, int NW, int NBUF>
__device__ __forceinline__ void gemm_skinny_bf16_nt(const uint16_t* __restrict__ A, long lda, const uint16_t* __restrict__ B, long ldb,
                                                    float* __restrict__ P, long ldp, long m, long n, long k, long kpart, float alpha, float beta,
                                                    int direct) {
    constexpr int CH = 64, NJ = 4;
    constexpr int SLOT = RT * NJ * 64;   // 128-bit words of a wavefront's block of sums
    extern __shared__ __attribute__((aligned(16))) unsigned char skinny_lds[];
    f32x4* lds = reinterpret_cast<f32x4*>(skinny_lds);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const long n0 = (long) blockIdx.x * (16 * NJ);
    const long part = blockIdx.y;
    const long kw = kpart / NW;   // a multiple of CH
    const long k_begin = part * kpart + wave * kw;
    long k_end = k_begin + kw;
    if (k_end > k) k_end = k;

    f32x4 acc[RT][NJ];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[rt][j][r] = 0.0f;

    const unsigned b_lane = (unsigned) (c * ldb + 8 * g), a_lane = (unsigned) (c * lda + 8 * g);
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // half h of a chunk: the lane's k are kb + 32 h + 8 g .. + 7
    auto load_b = [&](long kb, bf16x8 (&bv)[2 * NJ]) {
        const bool whole = kb + CH <= k_end;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const bool ok = n0 + 16 * j + c < n;
            const uint16_t* base = B + (n0 + 16 * j) * ldb + kb;
#pragma unroll
            for (int h = 0; h < 2; h++)
                bv[2 * j + h] = ok && (whole || kb + 32 * h + 8 * g < k_end) ? *reinterpret_cast<const bf16x8*>(base + b_lane + 32 * h) : zero8;
        }
    };
    auto load_a = [&](long kb, bf16x8 (&av)[2 * RT]) {
        const bool whole = kb + CH <= k_end;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const uint16_t* base = A + (long) (16 * rt) * lda + kb;
#pragma unroll
            for (int h = 0; h < 2; h++)
                av[2 * rt + h] = 16 * rt + c < m && (whole || kb + 32 * h + 8 * g < k_end) ? *reinterpret_cast<const bf16x8*>(base + a_lane + 32 * h) : zero8;
        }
    };
    auto products = [&](const bf16x8 (&av)[2 * RT], const bf16x8 (&bv)[2 * NJ]) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int rt = 0; rt < RT; rt++) acc[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[2 * rt + h], bv[2 * j + h], acc[rt][j], 0, 0, 0);
    };

    {
        bf16x8 bq[NBUF][2 * NJ], aq[NBUF][2 * RT];
#pragma unroll
        for (int u = 0; u < NBUF - 1; u++) {
            load_b(k_begin + u * CH, bq[u]);   // past k_end: zeros, no access
            load_a(k_begin + u * CH, aq[u]);
        }
        for (long kb = k_begin; kb < k_end; kb += NBUF * CH) {
#pragma unroll
            for (int u = 0; u < NBUF; u++) {
                const long kc = kb + u * CH;
                if (kc < k_end) {
                    load_b(kc + (NBUF - 1) * CH, bq[(u + NBUF - 1) % NBUF]);
                    load_a(kc + (NBUF - 1) * CH, aq[(u + NBUF - 1) % NBUF]);
                    products(aq[u], bq[u]);
                }
            }
        }
    }

    // the wavefronts' blocks meet in LDS as above; a word is one block's four registers of a lane
#pragma unroll
    for (int half = NW / 2; half >= 1; half /= 2) {
        if (wave >= half && wave < 2 * half) {
            f32x4* slot = lds + (long) (wave - half) * SLOT;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int j = 0; j < NJ; j++) slot[(rt * NJ + j) * 64 + lane] = acc[rt][j];
        }
        __syncthreads();
        if (wave < half) {
            const f32x4* slot = lds + (long) wave * SLOT;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int j = 0; j < NJ; j++) acc[rt][j] += slot[(rt * NJ + j) * 64 + lane];
        }
        __syncthreads();
    }
    if (wave != 0) return;
    float* out = direct ? P : P + part * m * ldp;
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            // register r of a 16 x 16 block of sums: row 4 (lane / 16) + r, column lane % 16
            const long row = 16 * rt + 4 * g + r;
            if (row >= m) continue;
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const long col = n0 + 16 * j + c;
                if (col >= n) continue;
                float* o = out + row * ldp + col;
                const float v = acc[rt][j][r];
                *o = direct ? (beta == 0.0f ? alpha * v : alpha * v + beta * *o) : v;
            }
        }
}

// fp64, B stored [k][n], up to 16 rows: the same scheme on v_mfma_f64_16x16x4_f64 (a lane holds one k of its row of A and of
// its column of B; 512 bytes of B per instruction and 64 cycles: 19.6 TB/s at the device's fp64 rate, so the product is bound by
// reading B). A work-group owns 64 columns of one part of K; a lane's 128-bit load of B is two adjacent columns, K advances in
// chunks of 16 (four consecutive k per lane group).
template <int NW, int NBUF>
__device__ __forceinline__ void gemm_skinny_f64_nn(const double* __restrict__ A, long lda, const double* __restrict__ B, long ldb,
                                                   double* __restrict__ P, long ldp, long m, long n, long k, long kpart, double alpha,
                                                   double beta, int direct) {
    typedef double d2 __attribute__((ext_vector_type(2)));
    constexpr int CH = 16, KL = 4, SETS = 2, NJ = 4;   // 64 columns: two loads of two columns a lane and k
    constexpr int SLOT = NJ / 2 * 4 * 64;              // 128-bit words of a wavefront's block of sums
    extern __shared__ __attribute__((aligned(16))) unsigned char skinny_lds[];
    d2* lds = reinterpret_cast<d2*>(skinny_lds);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const long n0 = (long) blockIdx.x * 64;
    const long part = blockIdx.y;
    const long kw = kpart / NW;   // a multiple of CH
    const long k_begin = part * kpart + wave * kw;
    long k_end = k_begin + kw;
    if (k_end > k) k_end = k;

    f64x4 acc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[j][r] = 0.0;

    const unsigned b_lane = (unsigned) (KL * g * ldb + 2 * c), a_lane = (unsigned) (c * lda + KL * g);
    const d2 zero2 = {0.0, 0.0};
    auto load_b = [&](long kb, d2 (&bv)[KL * SETS]) {
        const long kl = kb + KL * g;
        const bool whole = kb + CH <= k_end;
#pragma unroll
        for (int i = 0; i < KL; i++)
#pragma unroll
            for (int s = 0; s < SETS; s++) {
                const bool ok = n0 + 32 * s + 2 * c < n;
                const double* base = B + (kb + i) * ldb + n0 + 32 * s;
                bv[i * SETS + s] = ok && (whole || kl + i < k_end) ? __builtin_nontemporal_load(reinterpret_cast<const d2*>(base + b_lane)) : zero2;
            }
    };
    auto load_a = [&](long kb, d2 (&av)[KL / 2]) {
        const long kl = kb + KL * g;
        const bool whole = kb + CH <= k_end;
#pragma unroll
        for (int q = 0; q < KL / 2; q++)
            av[q] = c < m && (whole || kl + 2 * q < k_end) ? *reinterpret_cast<const d2*>(A + kb + a_lane + 2 * q) : zero2;
    };
    auto products = [&](const d2 (&av)[KL / 2], const d2 (&bv)[KL * SETS]) {
#pragma unroll
        for (int i = 0; i < KL; i++)
#pragma unroll
            for (int j = 0; j < NJ; j++)
                acc[j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i / 2][i % 2], bv[i * SETS + j / 2][j % 2], acc[j], 0, 0, 0);
    };
    {
        d2 bq[NBUF][KL * SETS], aq[NBUF][KL / 2];
#pragma unroll
        for (int u = 0; u < NBUF - 1; u++) {
            load_b(k_begin + u * CH, bq[u]);   // past k_end: zeros, no access
            load_a(k_begin + u * CH, aq[u]);
        }
        for (long kb = k_begin; kb < k_end; kb += NBUF * CH) {
#pragma unroll
            for (int u = 0; u < NBUF; u++) {
                const long kc = kb + u * CH;
                if (kc < k_end) {
                    load_b(kc + (NBUF - 1) * CH, bq[(u + NBUF - 1) % NBUF]);
                    load_a(kc + (NBUF - 1) * CH, aq[(u + NBUF - 1) % NBUF]);
                    products(aq[u], bq[u]);
                }
            }
        }
    }
    // the wavefronts' blocks meet in LDS; a word holds register r of the blocks 2 s and 2 s + 1: two adjacent columns
#pragma unroll
    for (int half = NW / 2; half >= 1; half /= 2) {
        if (wave >= half && wave < 2 * half) {
            d2* slot = lds + (long) (wave - half) * SLOT;
#pragma unroll
            for (int s = 0; s < SETS; s++)
#pragma unroll
                for (int r = 0; r < 4; r++) slot[(s * 4 + r) * 64 + lane] = d2{acc[2 * s][r], acc[2 * s + 1][r]};
        }
        __syncthreads();
        if (wave < half) {
            const d2* slot = lds + (long) wave * SLOT;
#pragma unroll
            for (int s = 0; s < SETS; s++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const d2 v = slot[(s * 4 + r) * 64 + lane];
                    acc[2 * s][r] += v[0];
                    acc[2 * s + 1][r] += v[1];
                }
        }
        __syncthreads();
    }
    if (wave != 0) return;
    double* out = direct ? P : P + part * m * ldp;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const long row = 4 * r + g;   // register r of a 16 x 16 block of fp64 sums: row 4 r + lane / 16, column lane % 16
        if (row >= m) continue;
#pragma unroll
        for (int s = 0; s < SETS; s++) {
            const long col = n0 + 32 * s + 2 * c;
            if (col >= n) continue;
            d2* o = reinterpret_cast<d2*>(out + row * ldp + col);
            d2 v = {acc[2 * s][r], acc[2 * s + 1][r]};
            if (direct) {
                if (beta == 0.0) {
                    v = alpha * v;
                } else {
                    const d2 old = *o;
                    v = alpha * v + beta * old;
                }
            }
            *o = v;
        }
    }
}

}  // namespace docc_k

#define DOCC_GEMM_SKINNY(MT, TB, TBN, NW, CH, NBUF)                                                                                             \
    extern "C" __global__ __launch_bounds__(64 * NW) void docc_sgemm_skinny##MT##_n##TBN##_w##NW##_c##CH##_b##NBUF(                             \
        const float* A, long lda, const float* B, long ldb, float* P, long ldp, long m, long n, long k, long kpart, float alpha, float beta,      \
        int direct) {                                                                                                                            \
        docc_k::gemm_skinny<MT, TB, NW, CH, NBUF>(A, lda, B, ldb, P, ldp, m, n, k, kpart, alpha, beta, direct);                                  \
    }

// B stored [k][n]: 16 k per chunk, one spare set of operands (more sets cost wavefronts per SIMD and ran slower). B stored [n][k]:
// 32 k per chunk, so that a row's 128-byte line is used up within the chunk; up to 16 rows of A.
DOCC_GEMM_SKINNY(16, false, n, 4, 16, 2)
DOCC_GEMM_SKINNY(32, false, n, 4, 16, 2)
DOCC_GEMM_SKINNY(16, true, t, 4, 32, 2)

#define DOCC_GEMM_SKINNY_BF16(RT, NW, NBUF)                                                                                                     \
    extern "C" __global__ __launch_bounds__(64 * NW) void docc_bgemm_skinny##RT##_nt_w##NW##_b##NBUF(                                           \
        const uint16_t* A, long lda, const uint16_t* B, long ldb, float* P, long ldp, long m, long n, long k, long kpart, float alpha,           \
        float beta, int direct) {                                                                                                                \
        docc_k::gemm_skinny_bf16_nt<RT, NW, NBUF>(A, lda, B, ldb, P, ldp, m, n, k, kpart, alpha, beta, direct);                                  \
    }

DOCC_GEMM_SKINNY_BF16(1, 4, 2)
DOCC_GEMM_SKINNY_BF16(2, 4, 2)

extern "C" __global__ __launch_bounds__(256) void docc_dgemm_skinny16_nn_w4_b2(const double* A, long lda, const double* B, long ldb, double* P,
                                                                              long ldp, long m, long n, long k, long kpart, double alpha,
                                                                              double beta, int direct) {
    docc_k::gemm_skinny_f64_nn<4, 2>(A, lda, B, ldb, P, ldp, m, n, k, kpart, alpha, beta, direct);
}
