// Launchers for the GEMM node kernels (see include/docc_rocm_ops.h).
#include <cstdio>
#include <type_traits>
#include <cstdlib>
#include <cstring>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace {

struct TileConfig {
    int bm, bn, bk, waves;
    int stages;  // > 0: asynchronous multi-stage kernel (gemm_async.h), aligned operands only
    bool spread = false;  // asynchronous kernels: the variant that deals a stage's copies over the whole K-step (3 stages or more)
    bool small = false;   // asynchronous bf16 kernels: the variant built on the 16x16x32 MFMA
};

// LDS bytes of GemmKernel<T, BM, BN, BK, ...> (csrc/kernels/gemm_mfma.h)
size_t gemm_lds_bytes(const TileConfig& c, bool ta, bool tb, size_t elem) {
    // fp32/fp64 pad mn-contiguous rows by 8 elements, bf16 (GemmBf16Kernel) by 16
    const int padk = (int) (16 / elem), padm = elem == 2 ? 16 : 8;
    const bool a_kc = !ta, b_kc = tb;
    const int lda_s = a_kc ? c.bk + padk : c.bm + padm;
    const int ldb_s = b_kc ? c.bk + padk : c.bn + padm;
    const size_t a_elems = (size_t) (a_kc ? c.bm : c.bk) * lda_s;
    const size_t b_elems = (size_t) (b_kc ? c.bn : c.bk) * ldb_s;
    return 2 * (a_elems + b_elems) * elem;
}

// One output column or one output row: the matrix-vector kernels (csrc/kernels/gemv.hip). Returns 1 when the
// shape is not one of theirs (the caller goes on to the tiled kernels), 0 or an error code otherwise.
template <typename T, typename S>
int gemv_launch(const char* prefix, hipStream_t s, bool ta, bool tb, int64_t m, int64_t n, int64_t k, S alpha, const T* A, int64_t lda,
                const T* B, int64_t ldb, S beta, S* C, int64_t ldc) {
    if (std::getenv("DOCC_ROCM_GEMV_OFF")) return 1;   // tuning and tests: always the tiled kernels
    const T *M, *x;
    int64_t ld, incx, incy, rows, cols;
    bool by_rows;
    if (m > 1 && n > 1) {
        // two to eight rows or columns of output with both operands stored row by row along k (op(A) = A, op(B) = B^T,
        // the product of a small batch with a weight matrix): the larger operand moves once
        if (m > 8 && n > 8) return 1;
        int cusm = compute_units();
        if (cusm <= 0) cusm = 256;
        // five to eight vectors would be two passes over the matrix: the tiles with K in parts are faster (fp32 8 x 4096 x 4096:
        // 39 us here, 26 there; 8 x 8192 x 8192: 95 against 81; fp64 8 x 8192 x 8192: 296 against 172)
        const int64_t max_vectors = 4;
        if (sizeof(T) != 2 && ((m <= max_vectors && !ta && !tb) || (n <= max_vectors && ta && !tb && m > 8))) {
            // the large operand is stored [k][columns] (y = x W with W as numpy holds it): columns form, sliced over k
            const bool small_a = m <= max_vectors && !ta;
            const int64_t nv = small_a ? m : n, cols = small_a ? n : m;
            const T* mat = small_a ? B : A;
            const T* vecs = small_a ? A : B;
            const int64_t ldm = small_a ? ldb : lda;
            const int64_t sx_v = small_a ? lda : 1, sx_p = small_a ? 1 : ldb;          // A[v][p] or B[p][v]
            const int64_t sy_vec = small_a ? ldc : 1, sy_col = small_a ? 1 : ldc;
            if (cols < 1024 || k < 64) return 1;
            const int vecw = 16 / (int) sizeof(T);
            const bool aligned = (uintptr_t) mat % 16 == 0 && ldm % vecw == 0 && cols % vecw == 0;
            const int lanes = aligned ? vecw : 1;
            const int64_t col_blocks = (cols / lanes + 255) / 256;
            // 1.75 work-groups per CU (measured against 0.75 .. 6 per CU on five shapes: 4 x 8192 x 8192 in 46.9 us against
            // 51.7 with two, 8 x 8192 x 8192 in 93.9 against 102.3, 4 x 4096 x 11008 in 32.9 against 35.3)
            int64_t slices = (7 * (int64_t) cusm / 4 + col_blocks - 1) / col_blocks;
            if (slices > k / 16) slices = k / 16;
            // the partial sums are written and read back: keep them under a sixteenth of the matrix's bytes
            const int64_t group = nv < 4 ? nv : 4;                                     // vectors per pass
            int64_t cheap = k * (int64_t) sizeof(T) / (16 * (int64_t) sizeof(S) * group);
            if (cheap * col_blocks < 4 * (int64_t) cusm) cheap *= 2;      // ... unless that leaves the chip short of work-groups
            if (slices > cheap) slices = cheap;
            const int64_t fit = (int64_t) kPartialsBytes / ((int64_t) sizeof(S) * cols * group);
            if (slices > fit) slices = fit;
            if (slices > 256) slices = 256;
            if (const char* e = std::getenv("DOCC_ROCM_GEMV_SLICES")) {   // tuning: a cap on the slices
                const int64_t cap = std::atoi(e);
                if (cap >= 1 && cap < slices) slices = cap;
            }
            if (slices < 1 || col_blocks > 0x7fffffffLL) return 1;
            const int64_t chunk = (k + slices - 1) / slices;
            slices = (k + chunk - 1) / chunk;
            // five to eight vectors go as two passes of at most four: two reads of the matrix beat one with eight sums a lane
            char kname[64], fname[64];
            std::snprintf(fname, sizeof(fname), "docc_gemv_colfm_f%d", (int) sizeof(S) * 8);
            PartialsLease partials;
            if (int rcp = partials_for(s, &partials)) return rcp;
            for (int64_t v0 = 0; v0 < nv; v0 += 4) {
                const int64_t gv = nv - v0 < 4 ? nv - v0 : 4;
                std::snprintf(kname, sizeof(kname), "docc_gemv_colpm_%s_v%d_n%d", sizeof(T) == 4 ? "f32" : "f64", lanes, gv <= 2 ? 2 : 4);
                int rcm = launch(kname, (uint32_t) col_blocks, (uint32_t) slices, 1, 256, 0, s, partials.ptr, mat, (long) ldm, vecs + v0 * sx_v,
                                 (long) sx_v, (long) sx_p, (int) gv, (long) k, (long) cols, (long) chunk);
                if (rcm) return rcm;
                const int64_t entries = gv * cols;
                rcm = launch(fname, (uint32_t) ((entries + 63) / 64), 1, 1, 256, 0, s, (const void*) partials.ptr, C + v0 * sy_vec, (long) sy_vec,
                             (long) sy_col, (long) cols, (long) entries, (int) slices, alpha, beta);
                if (rcm) return rcm;
            }
            return 0;
        }
        if (ta || !tb) return 1;
        const bool small_a = m <= n;                  // the vectors: A's rows (m of them) or B's rows (n of them)
        const int64_t nv = small_a ? m : n, big = small_a ? n : m;
        int cus0 = compute_units();
        if (cus0 <= 0) cus0 = 256;
        // five to eight vectors: fp64 is faster through the MFMA tiles (8 x 8192 x 8192: 166 us against 218 here), bf16 too
        // once the matrix is large (8 x 28672 x 8192: 111 us against 137; 8 x 8192 x 8192: 56 against 46 here)
        const int64_t max_nv = sizeof(T) == 8 || (sizeof(T) == 2 && big * k > (int64_t(1) << 27)) ? 4 : 8;
        const int vecw = 16 / (int) sizeof(T);
        const bool aligned = ((uintptr_t) (small_a ? B : A) | (uintptr_t) (small_a ? A : B)) % 16 == 0 && (small_a ? ldb : lda) % vecw == 0 &&
                             (small_a ? lda : ldb) % vecw == 0;
        // a wavefront takes four matrix rows, or eight where that still leaves a work-group per CU (fp32 4 x 8192 x 8192:
        // 79 -> 68 us; bf16 gains nothing from it)
        const bool eight = nv <= 4 && aligned && sizeof(T) != 2 && big >= 32 * (int64_t) cus0;
        const int64_t wg_rows = eight ? 32 : 16;
        if (nv > max_nv || big < 16 * (int64_t) cus0 || (big + wg_rows - 1) / wg_rows > 0x7fffffffLL) return 1;
        const T* mat = small_a ? B : A;
        const T* vecs = small_a ? A : B;
        const int64_t ldm = small_a ? ldb : lda, ldx = small_a ? lda : ldb;
        const int64_t sy_row = small_a ? 1 : ldc, sy_vec = small_a ? ldc : 1;
        char kname[64];
        std::snprintf(kname, sizeof(kname), "docc_gemv_rowsm_%s_v%d_n%d%s", sizeof(T) == 2 ? "bf16" : sizeof(T) == 4 ? "f32" : "f64",
                      aligned ? vecw : 1, nv <= 2 ? 2 : nv <= 4 ? 4 : 8, eight ? "_r8" : "");
        return launch(kname, (uint32_t) ((big + wg_rows - 1) / wg_rows), 1, 1, 256, 0, s, mat, (long) ldm, vecs, (long) ldx, (int) nv, C, (long) sy_row,
                      (long) sy_vec, (long) big, (long) k, alpha, beta);
    }
    if (n == 1) {          // y = op(A) b: A as stored is [m][k] (rows form) or [k][m] (columns form)
        M = A, ld = lda, x = B, incx = tb ? 1 : ldb, incy = ldc;
        by_rows = !ta;
        rows = ta ? k : m, cols = ta ? m : k;
    } else if (m == 1) {   // y = a op(B): B as stored is [n][k] (rows form) or [k][n] (columns form)
        M = B, ld = ldb, x = A, incx = ta ? lda : 1, incy = 1;
        by_rows = tb;
        rows = tb ? n : k, cols = tb ? k : n;
    } else {
        return 1;
    }
    const int vec = 16 / (int) sizeof(T);
    const char* type = sizeof(T) == 2 ? "bf16" : sizeof(T) == 4 ? "f32" : "f64";   // elements of the matrix
    const int bits = (int) sizeof(S) * 8;                                        // of the sums and of y
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    char name[64];
    if (by_rows) {
        // one wavefront per row: worth it from a few rows per SIMD on
        if (rows < 4 * (int64_t) cus) return 1;
        if ((rows + 3) / 4 > 0x7fffffffLL) return 1;
        const bool aligned = incx == 1 && ((uintptr_t) M | (uintptr_t) x) % 16 == 0 && ld % vec == 0;
        std::snprintf(name, sizeof(name), "docc_gemv_rows_%s_v%d", type, aligned ? vec : 1);
        return launch(name, (uint32_t) ((rows + 3) / 4), 1, 1, 256, 0, s, M, (long) ld, x, (long) incx, C, (long) incy, (long) rows,
                      (long) cols, alpha, beta);
    }
    // columns form: lanes own columns, the rows are sliced so that 2.6 work-groups per CU share the matrix (measured
    // on eight shapes from 4096 x 4096 to 28672 x 8192 against 1.5, 2, 3, 4, 6 and 8 per CU: the fastest on every one,
    // 8192 x 8192 fp32 in 42 us against 50 with eight - fewer slices also leave less for the second launch to add);
    // the slices' sums meet in the stream's partial-results buffer
    if (cols < 256 || rows < 64) return 1;
    const bool aligned = (uintptr_t) M % 16 == 0 && ld % vec == 0 && cols % vec == 0;
    const int lanes = aligned ? vec : 1;
    const int64_t col_blocks = (cols / lanes + 255) / 256;
    int64_t slices = (21 * (int64_t) cus / 8 + col_blocks - 1) / col_blocks;
    if (slices > rows / 16) slices = rows / 16;
    const int64_t fit = (int64_t) kPartialsBytes / ((int64_t) sizeof(S) * cols);
    if (slices > fit) slices = fit;
    if (slices > 256) slices = 256;
    if (const char* e = std::getenv("DOCC_ROCM_GEMV_SLICES")) {   // tuning: a cap on the slices
        const int64_t cap = std::atoi(e);
        if (cap >= 1 && cap < slices) slices = cap;
    }
    if (slices < 1) return 1;
    const int64_t chunk = (rows + slices - 1) / slices;
    slices = (rows + chunk - 1) / chunk;
    if (col_blocks > 0x7fffffffLL || slices > 65535) return 1;
    PartialsLease partials;
    if (int rcp = partials_for(s, &partials)) return rcp;
    std::snprintf(name, sizeof(name), "docc_gemv_colp_%s_v%d", type, lanes);
    int rc = launch(name, (uint32_t) col_blocks, (uint32_t) slices, 1, 256, 0, s, partials.ptr, M, (long) ld, x, (long) incx, (long) rows,
                    (long) cols, (long) chunk);
    if (rc) return rc;
    std::snprintf(name, sizeof(name), "docc_gemv_colf_f%d", bits);
    return launch(name, (uint32_t) ((cols + 15) / 16), 1, 1, 256, 0, s, (const void*) partials.ptr, C, (long) incy, (long) cols, (int) slices,
                  alpha, beta);
}

// T: element type of A and B; S: type of C, alpha and beta
template <typename T, typename S = T>
int gemm_launch(const char* prefix, docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n,
                int64_t k, S alpha, const T* A, int64_t lda, const T* B, int64_t ldb, S beta, S* C, int64_t ldc,
                TileConfig (*pick)(int64_t m, int64_t n, int64_t batch, bool aligned, int force), const S* bias = nullptr,
                int activation = -1, int64_t batch = 1, int64_t batch_a = 0, int64_t batch_b = 0, int64_t batch_c = 0) {
    if ((trans_a != DOCC_ROCM_NO_TRANS && trans_a != DOCC_ROCM_TRANS) ||
        (trans_b != DOCC_ROCM_NO_TRANS && trans_b != DOCC_ROCM_TRANS))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: transpose code must be 111 or 112", prefix);
    if (m < 0 || n < 0 || k < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: negative dimension", prefix);
    const bool ta = trans_a == DOCC_ROCM_TRANS, tb = trans_b == DOCC_ROCM_TRANS;
    const int64_t a_cols = ta ? m : k, b_cols = tb ? k : n;
    if (lda < (a_cols > 1 ? a_cols : 1) || ldb < (b_cols > 1 ? b_cols : 1) || ldc < (n > 1 ? n : 1))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: leading dimension too small (lda=%lld ldb=%lld ldc=%lld)",
                    prefix, (long long) lda, (long long) ldb, (long long) ldc);
    if (activation < -1 || activation > DOCC_ROCM_UNARY_ERF)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: unknown activation %d", prefix, activation);
    if (activation >= 0 && activation != DOCC_ROCM_UNARY_RELU && activation != DOCC_ROCM_UNARY_ABS)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: only ReLU and Abs are built into the GEMM store (activation %d)", prefix, activation);
    if (batch < 0 || batch > 65535) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: batch must be 0..65535", prefix);
    if (batch_a < 0 || batch_b < 0 || batch_c < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: negative batch stride", prefix);
    if (m == 0 || n == 0 || batch == 0) return 0;
    if (batch > 1 && batch_c < (m - 1) * ldc + n) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: the C matrices of the batch overlap", prefix);
    if (!C || (k > 0 && (!A || !B))) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: null pointer", prefix);
    int rc = ensure_device();
    if (rc) return rc;
    hipStream_t s = (hipStream_t) stream;
    char name[96];
    if (k == 0 || alpha == (S) 0) {   // an empty product, or one BLAS does not reference ("when ALPHA is zero ...")
        std::snprintf(name, sizeof(name), "docc_%s_scale_c", prefix);
        int64_t blocks = (m * n + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        for (int64_t z = 0; z < batch && rc == 0; z++)   // an empty product: one small launch per entry
            rc = launch(name, (uint32_t) blocks, 1, 1, 256, 0, s, C + z * batch_c, (long) m, (long) n, (long) ldc, beta);
        if (rc || (!bias && activation < 0)) return rc;
        if (batch > 1) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: k == 0 or alpha == 0 with an epilogue and a batch", prefix);
        // the epilogue of an empty product: C = act(beta * C + bias), through the elementwise kernel
        if (ldc != n) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: k == 0 or alpha == 0 with an epilogue needs ldc == n", prefix);
        const int64_t shape[2] = {m, n}, row[2] = {1, n};
        const int post[1] = {activation};
        return docc_rocm_elementwise_fused(stream, sizeof(S) == 8 ? 64 : 32, 2, shape, bias ? DOCC_ROCM_BINARY_ADD : -1, shape, C, 0.0,
                                           bias ? row : nullptr, bias, 0.0, activation >= 0 ? 1 : 0, post, C);
    }
    const bool epilogue = bias || activation >= 0;
    // A tall matrix times a few columns held as numpy holds them (B [k][n], n small): rows of B are a few elements long, so
    // the kernels that read whole vectors along n do not apply (n = 2, 5, 9 ... went through the element-wise tiles at a
    // ninth of the rate) and the matrix-vector kernels want the vectors contiguous along k. B is small: it is transposed
    // into a block of the device block cache first (k x n elements), and the product runs as A B'^T.
    if (!tb && batch == 1 && n >= 2 && n <= 64 && ldb == n && m >= 1024 && k >= 256 && k % (16 / (int64_t) sizeof(T)) == 0 &&
        (n <= 4 || n % (16 / (int64_t) sizeof(T)) != 0) && !std::getenv("DOCC_ROCM_GEMV_OFF")) {
        void* bt = nullptr;
        if ((rc = docc_rocm_malloc_async(&bt, (size_t) (n * k) * sizeof(T), stream))) return rc;
        const int64_t shape[2] = {k, n}, perm[2] = {1, 0};
        rc = docc_rocm_transpose(stream, (int) sizeof(T), 2, shape, perm, B, bt);
        if (!rc)
            rc = gemm_launch<T, S>(prefix, stream, trans_a, DOCC_ROCM_TRANS, m, n, k, alpha, A, lda, (const T*) bt, k, beta, C, ldc, pick, bias, activation);
        const int rc2 = docc_rocm_free_async(bt, stream);
        return rc ? rc : rc2;
    }
    // Five to 32 rows of fp32 against a wide matrix go to the kernels of csrc/kernels/gemm_skinny.hip (below); measured against
    // the tiles with K in parts and the matrix-vector forms, they pay from 8 M elements of B (16 M above 16 rows).
    // DOCC_ROCM_GEMM_SKINNY=1 takes them for smaller ones too (tests).
    const char* skinny_env = std::getenv("DOCC_ROCM_GEMM_SKINNY");
    const bool skinny_on = !(skinny_env && skinny_env[0] == '0'), skinny_any_size = skinny_env && skinny_env[0] == '1';
    // (a lane's offset from the chunk's base, up to 31 rows of either operand, is held in 32 bits)
    const bool skinny_base = batch == 1 && !ta && (!epilogue || ldc == n) && n >= 512 && k >= 512 && skinny_on && (uintptr_t) A % 16 == 0 &&
                             (uintptr_t) B % 16 == 0 && lda < (int64_t(1) << 26) && ldb < (int64_t(1) << 26);
    // (B stored [n][k]: from 3 rows, where the matrix-vector form for several vectors falls behind - 4 x 8192 x 8192 67 -> 57 us,
    // 4 x 4096 x 11008 62 -> 48 - but up to 8 rows not above 128 M elements, where that form is the faster one again)
    const bool skinny_f32 = sizeof(T) == 4 && skinny_base && m >= (skinny_any_size ? 2 : tb ? 3 : 5) && m <= (tb ? 16 : 32) &&
                            !(tb && m <= 8 && n * k > (int64_t(1) << 27)) &&
                            (n * k >= (m <= 16 ? int64_t(8) << 20 : int64_t(16) << 20) || skinny_any_size) && lda % 4 == 0 && ldb % 4 == 0 &&
                            k % 4 == 0 && (tb || n % 4 == 0);
    // bf16 with B stored [n][k] (a layer's weights): 3 to 32 rows (two rows are faster as matrix-vector products, 64 on the tiles)
    const bool skinny_bf16 = sizeof(T) == 2 && skinny_base && tb && m >= 3 && m <= 32 && (n * k >= (int64_t(8) << 20) || skinny_any_size) &&
                             lda % 8 == 0 && ldb % 8 == 0 && k % 8 == 0;
    // fp64 with B stored [k][n]: 5 to 16 rows (up to four are matrix-vector products, above 16 the tiles)
    const bool skinny_f64 = sizeof(T) == 8 && skinny_base && !tb && m >= 5 && m <= 16 && (n * k >= (int64_t(4) << 20) || skinny_any_size) &&
                            lda % 2 == 0 && ldb % 2 == 0 && k % 2 == 0 && n % 2 == 0;
    const bool skinny = skinny_f32 || skinny_bf16 || skinny_f64;
    if ((m <= 8 || n <= 8) && !skinny && batch == 1 && (!epilogue || ldc == n)) {
        rc = gemv_launch<T, S>(prefix, s, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
        if (rc == 0 && epilogue) {
            // the few rows or columns of output are a small tensor: bias and activation as one elementwise pass over it,
            // the same roundings as the fused store
            const int64_t shape[2] = {m, n}, row[2] = {1, n};
            const int post[1] = {activation};
            return docc_rocm_elementwise_fused(stream, sizeof(S) == 8 ? 64 : 32, 2, shape, bias ? DOCC_ROCM_BINARY_ADD : -1, shape, C, 0.0,
                                               bias ? row : nullptr, bias, 0.0, activation >= 0 ? 1 : 0, post, C);
        }
        if (rc != 1) return rc;
    }
    const size_t vec = 16 / sizeof(T);
    // the aligned kernels read whole 128-bit vectors: pointers, leading dimensions and the
    // contiguous extents of both operands must be multiples of the vector length
    const int64_t a_contig = ta ? m : k, b_contig = tb ? k : n;
    const bool aligned = ((uintptr_t) A % 16 == 0) && ((uintptr_t) B % 16 == 0) && (lda % vec == 0) && (ldb % vec == 0) &&
                         (a_contig % (int64_t) vec == 0) && (b_contig % (int64_t) vec == 0) &&
                         (batch == 1 || (batch_a % (int64_t) vec == 0 && batch_b % (int64_t) vec == 0));
    // A few rows against a wide fp32 matrix: B goes from global memory straight into the MFMA operands, 128 columns of one part
    // of K per work-group, the parts added in order by a second launch. With B stored [n][k] the lanes of a load walk different
    // rows, which pays up to 16 rows only. DOCC_ROCM_GEMM_SKINNY=0 switches it off, DOCC_ROCM_GEMM_SPLITK forces the number of
    // parts (tests, tuning).
    if (skinny) {
        {
            int cus = compute_units();
            if (cus <= 0) cus = 256;
            // fp32: 16 or 32 rows per MFMA, 128 columns per work-group; bf16: 1, 2 or 4 blocks of 16 rows, 64 columns
            const int nw = 4, nbuf = 2;
            const int ch = skinny_bf16 ? 64 : tb ? 32 : 16, mt = skinny_bf16 ? (m <= 16 ? 1 : 2) : m <= 16 ? 16 : 32;
            const int64_t col_blocks = skinny_bf16 || skinny_f64 ? (n + 63) / 64 : (n + 127) / 128;
            const int64_t unit = (int64_t) nw * ch;
            auto part_length = [&](int64_t parts) { return ((k + parts - 1) / parts + unit - 1) / unit * unit; };
            // The number of parts: measured on 4096 x 4096, 8192 x 8192, 11008 x 4096 and 4096 x 11008, what counts is that
            // the work-groups come out as whole rounds over the CUs (8192 x 8192: 4, 8 and 12 parts 48-51 us, 6 parts 56 us),
            // then few parts (their products are written and read again) and 128 and more k per wavefront.
            int64_t parts = 1;
            double best = -1.0;
            for (int64_t p = 1; p <= 64 && part_length(p) >= nw * 64 && p * 16 * m <= k; p++) {
                const int64_t kp = part_length(p);
                if ((k + kp - 1) / kp != p) continue;   // rounding to whole chunks made it fewer parts
                // B stored [n][k]: a lane walks its row of B, and parts longer than 4096 ran a quarter slower (bf16 16384 x 16384
                // in 1 or 2 parts 127 us, in 4 parts 97)
                if (tb && kp > 4096 && part_length(p + 1) >= nw * 64) continue;
                const double per_cu = (double) (col_blocks * p) / cus;
                const double score = per_cu / (double) (int64_t) (per_cu + 0.999999) - 0.01 * (double) p - (kp < nw * 128 ? 0.15 : 0.0);
                if (score > best) {
                    best = score;
                    parts = p;
                }
            }
            if (const char* e = std::getenv("DOCC_ROCM_GEMM_SPLITK"))
                if (std::atoll(e) > 0 && part_length(std::atoll(e)) >= unit) parts = std::atoll(e);
            const int64_t kpart = part_length(parts);
            parts = (k + kpart - 1) / kpart;
            const int64_t bytes = parts * m * n * (int64_t) sizeof(S);
            const bool direct = parts == 1 && (tb || ((uintptr_t) C % 16 == 0 && ldc % (skinny_f64 ? 2 : 4) == 0));
            if (direct || bytes <= (int64_t(64) << 20)) {
                PartialsLease lease;
                void* buf = nullptr;
                const bool own_block = !direct && bytes > (int64_t) kPartialsBytes;
                if (own_block) {
                    if ((rc = docc_rocm_malloc_async(&buf, (size_t) bytes, stream))) return rc;
                } else if (!direct) {
                    if ((rc = partials_for(s, &lease))) return rc;
                    buf = lease.ptr;
                }
                if (skinny_f64)
                    std::snprintf(name, sizeof(name), "docc_dgemm_skinny16_nn_w%d_b%d", nw, nbuf);
                else if (skinny_bf16)
                    std::snprintf(name, sizeof(name), "docc_bgemm_skinny%d_nt_w%d_b%d", mt, nw, nbuf);
                else
                    std::snprintf(name, sizeof(name), "docc_sgemm_skinny%d_n%c_w%d_c%d_b%d", mt, tb ? 't' : 'n', nw, ch, nbuf);
                const uint32_t slot_bytes = skinny_bf16 ? 4096u * mt : mt == 32 && !skinny_f64 ? 16384u : 8192u;   // a wavefront's block of sums
                rc = launch(name, (uint32_t) col_blocks, (uint32_t) parts, 1, 64 * nw, (uint32_t) (nw / 2) * slot_bytes, s, A, (long) lda, B, (long) ldb,
                            direct ? (void*) C : buf, (long) (direct ? ldc : n), (long) m, (long) n, (long) k, (long) kpart, alpha, beta,
                            direct ? 1 : 0);
                if (!rc && !direct) {
                    int64_t blocks = (m * n + 255) / 256;
                    if (blocks > 4096) blocks = 4096;
                    rc = launch(sizeof(S) == 8 ? "docc_splitk_combine_f64" : "docc_splitk_combine_f32", (uint32_t) blocks, 1, 1, 256, 0, s, (const S*) buf, C,
                                (long) m, (long) n, (long) ldc, (int) parts, alpha, beta);
                }
                if (own_block) {
                    const int rc2 = docc_rocm_free_async(buf, stream);
                    if (!rc) rc = rc2;
                }
                if (rc || !epilogue) return rc;
                // the few rows of output are a small tensor: bias and activation as one elementwise pass over it, the same
                // roundings as the fused store
                const int64_t shape[2] = {m, n}, row[2] = {1, n};
                const int post[1] = {activation};
                return docc_rocm_elementwise_fused(stream, sizeof(S) == 8 ? 64 : 32, 2, shape, bias ? DOCC_ROCM_BINARY_ADD : -1, shape, C, 0.0,
                                                   bias ? row : nullptr, bias, 0.0, activation >= 0 ? 1 : 0, post, C);
            }
        }
    }
    // DOCC_ROCM_GEMM_TILE=big|small overrides the size heuristic (tests, tuning)
    const char* force = std::getenv("DOCC_ROCM_GEMM_TILE");
    TileConfig cfg = pick(m, n, batch, aligned, force && force[0] == 'b' ? 1 : force && force[0] == 's' ? -1 : 0);
    // DOCC_ROCM_GEMM_CFG=BMxBNxBKxWAVES[xSTAGES[p|q]] selects a built configuration directly (tuning)
    if (const char* c = std::getenv("DOCC_ROCM_GEMM_CFG")) {
        TileConfig t{};
        char tag = 0;
        const int got = std::sscanf(c, "%dx%dx%dx%dx%d%c", &t.bm, &t.bn, &t.bk, &t.waves, &t.stages, &tag);
        t.spread = got == 6 && tag == 'p';
        t.small = got == 6 && tag == 'q';
        if (got >= 4 && t.bm > 0 && t.bn > 0 && t.bk > 0 && t.waves > 0) cfg = t;
    }
    // the 16x16x32 kernels (gemm_async16.h) take whole pairs of K-steps, at least a ring of them
    if (cfg.small && !(k % (2 * cfg.bk) == 0 && k >= (int64_t) cfg.stages * cfg.bk)) cfg.small = false;
    // the asynchronous kernels need aligned operands and address a tile with 32-bit byte offsets
    const int64_t max_edge = cfg.bm > cfg.bn ? (cfg.bm > cfg.bk ? cfg.bm : cfg.bk) : (cfg.bn > cfg.bk ? cfg.bn : cfg.bk);
    const bool offsets_fit = max_edge * (lda > ldb ? lda : ldb) * (int64_t) sizeof(T) < (int64_t(1) << 32);
    if (cfg.stages > 0 && !(aligned && offsets_fit)) cfg = pick(m, n, batch, false, 0);
    const int64_t tiles = ((m + cfg.bm - 1) / cfg.bm) * ((n + cfg.bn - 1) / cfg.bn);
    if (tiles > 0x7fffffffLL) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: too many tiles", prefix);
    // Few output tiles and a long K extent (a handful of rows against a wide matrix: the product is bound by reading
    // that matrix, and a work-group per tile reads it on a few CUs only): K is cut into parts, each part's product is
    // one entry of a batched launch into the stream's buffer of partial results, and a second launch adds the parts
    // (in order: the result does not depend on the device's scheduling). DOCC_ROCM_GEMM_SPLITK=0 switches it off,
    // another number forces that many parts where K allows it (tests, tuning).
    if (batch == 1 && (!epilogue || ldc == n) && aligned && k >= 1024) {
        int cus = compute_units();
        if (cus <= 0) cus = 256;
        const char* env = std::getenv("DOCC_ROCM_GEMM_SPLITK");
        // the parts' products: in the stream's buffer of partial results where they fit, else in a block of the device
        // block cache (taken and returned in stream order), up to 64 MiB
        constexpr int64_t kMaxPartBytes = int64_t(64) << 20;
        auto allowed = [&](int64_t parts) {
            return parts <= 64 && k % parts == 0 && (k / parts) % 64 == 0 && k / parts >= 256 && parts * m * n * (int64_t) sizeof(S) <= kMaxPartBytes;
        };
        // Estimated seconds of the product in `parts` parts on the tile the picker gives that many matrices: the work of
        // the padded tiles at what the tile sustains (relative to the 128 x 256 one) on the share of the CUs that get a
        // work-group, plus writing and reading the parts at 5 TB/s and a second launch.
        auto seconds = [&](const TileConfig& c, int64_t parts) {
            const double tm = (double) ((m + c.bm - 1) / c.bm), tn = (double) ((n + c.bn - 1) / c.bn);
            const double area = (double) c.bm * c.bn;
            const double rel = area >= 65536 ? 1.03 : area >= 32768 ? 1.0 : area >= 16384 ? 0.97 : 0.75;
            // the share of the CUs' time that does work: below one work-group per CU the CUs that get one, above it the
            // whole rounds (344 work-groups on 256 CUs take as long as 512)
            const double per_cu = tm * tn * (double) parts / cus;
            const double fill = per_cu < 1.0 ? per_cu : per_cu / (double) (int64_t) (per_cu + 0.999999);
            const double rate = sizeof(T) == 8 ? 68e12 : sizeof(T) == 4 ? 141e12 : 1.25e15;
            double t = 2.0 * tm * c.bm * tn * c.bn * (double) k / (rate * rel * fill);
            if (parts > 1) t += 2.0 * (double) parts * (double) m * (double) n * sizeof(S) / 5e12 + 3e-6;
            return t;
        };
        int64_t splits = 1;
        if (env) {
            const int64_t wanted = std::atoll(env);
            while (splits * 2 <= wanted && allowed(splits * 2)) splits *= 2;
        } else if (tiles < cus) {   // CUs without a work-group: the case parts are for
            double best = seconds(cfg, 1);
            for (int64_t parts = 2; allowed(parts); parts *= 2) {
                const TileConfig c = pick(m, n, parts, true, 0);
                if (c.stages == 0) break;
                const double t = seconds(c, parts);
                if (t < 0.9 * best) {   // only for a clear gain: the estimate is rough
                    best = t;
                    splits = parts;
                }
            }
        }
        if (splits >= 2) {
            const int64_t bytes = splits * m * n * (int64_t) sizeof(S);
            PartialsLease lease;
            void* parts = nullptr;
            const bool own_block = bytes > (int64_t) kPartialsBytes;
            if (own_block) {
                if ((rc = docc_rocm_malloc_async(&parts, (size_t) bytes, stream))) return rc;
            } else {
                if ((rc = partials_for(s, &lease))) return rc;
                parts = lease.ptr;
            }
            const int64_t part = k / splits;
            rc = gemm_launch<T, S>(prefix, stream, trans_a, trans_b, m, n, part, (S) 1, A, lda, B, ldb, (S) 0, (S*) parts, n, pick, nullptr, -1, splits,
                                   ta ? part * lda : part, tb ? part : part * ldb, m * n);
            if (!rc) {
                int64_t blocks = (m * n + 255) / 256;
                if (blocks > 4096) blocks = 4096;
                rc = launch(sizeof(S) == 8 ? "docc_splitk_combine_f64" : "docc_splitk_combine_f32", (uint32_t) blocks, 1, 1, 256, 0, s, (const S*) parts, C,
                            (long) m, (long) n, (long) ldc, (int) splits, alpha, beta);
            }
            if (own_block) {
                const int rc2 = docc_rocm_free_async(parts, stream);
                if (!rc) rc = rc2;
            }
            if (rc || !epilogue) return rc;
            // bias and activation as one elementwise pass over the output, the same roundings as the fused store
            const int64_t shape[2] = {m, n}, row[2] = {1, n};
            const int post[1] = {activation};
            return docc_rocm_elementwise_fused(stream, sizeof(S) == 8 ? 64 : 32, 2, shape, bias ? DOCC_ROCM_BINARY_ADD : -1, shape, C, 0.0,
                                               bias ? row : nullptr, bias, 0.0, activation >= 0 ? 1 : 0, post, C);
        }
    }
    size_t lds;
    if (cfg.stages > 0) {
        std::snprintf(name, sizeof(name), "docc_%sa_%dx%dx%d%c%d_%c%c", prefix, cfg.bm, cfg.bn, cfg.bk, cfg.small ? 'q' : cfg.spread ? 'p' : 's', cfg.stages,
                      ta ? 't' : 'n', tb ? 't' : 'n');
        lds = (size_t) cfg.stages * ((size_t) cfg.bm * cfg.bk + (size_t) cfg.bk * cfg.bn) * sizeof(T);
    } else {
        std::snprintf(name, sizeof(name), "docc_%s_%dx%dx%d_%c%c_%c", prefix, cfg.bm, cfg.bn, cfg.bk, ta ? 't' : 'n',
                      tb ? 't' : 'n', aligned ? 'a' : 'u');
        lds = gemm_lds_bytes(cfg, ta, tb, sizeof(T));
    }
    // the variants with bias / activation in the store carry the suffix "_e"
    if (bias || activation >= 0) std::strncat(name, "_e", sizeof(name) - std::strlen(name) - 1);
    return launch(name, (uint32_t) tiles, (uint32_t) batch, 1, 64 * cfg.waves, (uint32_t) lds, s, A, B, C, (long) m, (long) n,
                  (long) k, (long) lda, (long) ldb, (long) ldc, alpha, beta, bias, activation, (long) batch_a, (long) batch_b,
                  (long) batch_c);
}

} // namespace

// A batch of equally shaped products in launches of at most 65535 entries (the limit of gridDim.y).
template <typename T, typename S>
static int gemm_batched(const char* prefix, docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                        S alpha, const T* A, int64_t lda, int64_t stride_a, const T* B, int64_t ldb, int64_t stride_b, S beta, S* C,
                        int64_t ldc, int64_t stride_c, int64_t batch,
                        TileConfig (*pick)(int64_t m, int64_t n, int64_t batch, bool aligned, int force)) {
    if (batch < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: negative batch", prefix);
    const int64_t kMaxGridY = 65535;
    for (int64_t b0 = 0; b0 < batch; b0 += kMaxGridY) {
        const int64_t nb = batch - b0 < kMaxGridY ? batch - b0 : kMaxGridY;
        const int rc = gemm_launch<T, S>(prefix, stream, trans_a, trans_b, m, n, k, alpha, A ? A + b0 * stride_a : A, lda,
                                         B ? B + b0 * stride_b : B, ldb, beta, C ? C + b0 * stride_c : C, ldc, pick, nullptr, -1, nb,
                                         stride_a, stride_b, stride_c);
        if (rc) return rc;
    }
    return 0;
}

extern "C" {

// Tile selection. `force`: +1 largest tile, -1 smallest tile, 0 by problem size. Asynchronous
// (staged) configurations need aligned operands; the others handle everything.
// tiles of one matrix times the number of matrices: what there is to spread over the compute units
static int64_t tiles_of(int64_t m, int64_t n, int bm, int bn, int64_t batch = 1) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn) * batch; }

static TileConfig pick_sgemm(int64_t m, int64_t n, int64_t batch, bool aligned, int force) {
    const TileConfig huge{256, 256, 32, 4, 2}, wide{128, 256, 32, 4, 2}, big{128, 128, 32, 4, 3}, small{64, 64, 16, 4, 4};
    const TileConfig plain_big{128, 128, 16, 4, 0}, plain_small{64, 64, 16, 4, 0};
    if (!aligned) return force > 0 ? plain_big : force < 0 ? plain_small : (tiles_of(m, n, 128, 128, batch) >= 256 ? plain_big : plain_small);
    if (force) return force > 0 ? huge : small;
    // Score = share of a tile's area that is real output x share of the CUs that get a work-group x what the
    // tile sustains relative to the 128x256 one (146 / 141 / 138 / about 105 TFLOP/s on large problems): a 64-row
    // product wastes half of a 128-row tile, a 1000^2 one leaves most CUs idle with the large tiles.
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    auto score = [&](const TileConfig& c, double rel) {
        const double padded = (double) ((m + c.bm - 1) / c.bm * c.bm) * (double) ((n + c.bn - 1) / c.bn * c.bn);
        const double fill = (double) tiles_of(m, n, c.bm, c.bn, batch) / cus;
        return rel * ((double) m * (double) n / padded) * (fill < 1.0 ? fill : 1.0);
    };
    const double sh = score(huge, 1.03), sw = score(wide, 1.0), sb = score(big, 0.97), ss = score(small, 0.75);
    // one work-group of the two largest tiles owns a CU, so their work-groups run in rounds: the 256x256 tile only
    // where its rounds take no longer than those of the 128x256 one
    auto rounds = [&](const TileConfig& c) { return (double) ((tiles_of(m, n, c.bm, c.bn, batch) + cus - 1) / cus) * c.bm * c.bn; };
    if (sh >= sw && sh >= sb && sh >= ss && rounds(huge) / 1.03 <= rounds(wide)) return huge;
    return sw >= sb && sw >= ss ? wide : sb >= ss ? big : small;
}

static TileConfig pick_dgemm(int64_t m, int64_t n, int64_t batch, bool aligned, int force) {
    const TileConfig big{128, 128, 16, 4, 3}, mid{64, 64, 16, 4, 4}, small{64, 32, 16, 4, 4};
    const TileConfig plain_big{128, 128, 16, 4, 0}, plain_small{64, 64, 16, 4, 0};
    if (!aligned) return force > 0 ? plain_big : plain_small;
    if (force) return force > 0 ? big : small;
    const int64_t t = tiles_of(m, n, 64, 64, batch);
    return t >= 2048 ? big : t > 512 ? mid : small;   // few tiles: halve them so that two work-groups share a CU
}

static TileConfig pick_bgemm(int64_t m, int64_t n, int64_t batch, bool aligned, int force) {
    // big: on the 16x16x32 MFMA where K allows it (see gemm_launch), else on the 32x32x16 one with the copies dealt out
    const TileConfig big{256, 256, 32, 4, 4, true, true}, small{128, 128, 32, 4, 4};
    const TileConfig plain_big{256, 256, 64, 4, 0}, plain_small{128, 128, 64, 4, 0};
    if (!aligned) return force > 0 ? plain_big : force < 0 ? plain_small : (tiles_of(m, n, 256, 256, batch) >= 256 ? plain_big : plain_small);
    if (force) return force > 0 ? big : small;
    return tiles_of(m, n, 256, 256, batch) >= 192 ? big : small;
}

int docc_rocm_sgemm(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                    const float* A, int64_t lda, const float* B, int64_t ldb, float beta, float* C, int64_t ldc) {
    return gemm_launch<float>("sgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, pick_sgemm);
}

int docc_rocm_dgemm(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                    double alpha, const double* A, int64_t lda, const double* B, int64_t ldb, double beta, double* C,
                    int64_t ldc) {
    return gemm_launch<double>("dgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, pick_dgemm);
}

int docc_rocm_bf16gemm_f32(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                           float alpha, const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, float beta,
                           float* C, int64_t ldc) {
    return gemm_launch<uint16_t, float>("bgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
                                        pick_bgemm);
}

int docc_rocm_sgemm_epilogue(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                             const float* A, int64_t lda, const float* B, int64_t ldb, float beta, float* C, int64_t ldc,
                             const float* bias, int activation) {
    return gemm_launch<float>("sgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, pick_sgemm, bias,
                              activation);
}

int docc_rocm_dgemm_epilogue(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                             double alpha, const double* A, int64_t lda, const double* B, int64_t ldb, double beta, double* C,
                             int64_t ldc, const double* bias, int activation) {
    return gemm_launch<double>("dgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, pick_dgemm, bias,
                               activation);
}

int docc_rocm_bf16gemm_f32_epilogue(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                                    float alpha, const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, float beta,
                                    float* C, int64_t ldc, const float* bias, int activation) {
    return gemm_launch<uint16_t, float>("bgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
                                        pick_bgemm, bias, activation);
}

int docc_rocm_sgemm_batched(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                            const float* A, int64_t lda, int64_t stride_a, const float* B, int64_t ldb, int64_t stride_b, float beta,
                            float* C, int64_t ldc, int64_t stride_c, int64_t batch) {
    return gemm_batched<float, float>("sgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, stride_a, B, ldb, stride_b, beta, C,
                                      ldc, stride_c, batch, pick_sgemm);
}

int docc_rocm_dgemm_batched(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, double alpha,
                            const double* A, int64_t lda, int64_t stride_a, const double* B, int64_t ldb, int64_t stride_b,
                            double beta, double* C, int64_t ldc, int64_t stride_c, int64_t batch) {
    return gemm_batched<double, double>("dgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, stride_a, B, ldb, stride_b, beta,
                                        C, ldc, stride_c, batch, pick_dgemm);
}

int docc_rocm_bf16gemm_f32_batched(docc_rocm_stream_t stream, int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                                   const uint16_t* A, int64_t lda, int64_t stride_a, const uint16_t* B, int64_t ldb,
                                   int64_t stride_b, float beta, float* C, int64_t ldc, int64_t stride_c, int64_t batch) {
    return gemm_batched<uint16_t, float>("bgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, stride_a, B, ldb, stride_b, beta,
                                         C, ldc, stride_c, batch, pick_bgemm);
}

} // extern "C"
