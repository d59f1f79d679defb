// Launchers for the elementwise tensor nodes and ml::Broadcast (see include/docc_rocm_ops.h).
#include <cstdio>
#include <cstdlib>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace {

const char* const kUnaryNames[] = {"abs", "exp", "relu", "sigmoid", "sqrt", "tanh", "erf"};
const char* const kBinaryNames[] = {"add", "sub", "mul", "div", "maximum", "minimum", "pow"};

// Work-groups for `items` lane-items, at most `per_cu` per compute unit (the kernels stride over the
// rest). Measured on [8192, 4096] fp32: kernels that only move data are fastest with one vector per lane
// and no striding (128 per CU: add 6.7, relu 6.5, broadcast 6.4 TB/s against 6.1 / 6.0 / 5.6 at 16 per CU);
// the transcendental ones want 64 per CU, the fused chain with its per-lane index set-up 32.
// DOCC_ROCM_EW_GRID overrides all three (tuning).
constexpr int kGridStreaming = 128, kGridTranscendental = 64, kGridFused = 32;

uint32_t grid_for(int64_t items, int per_cu) {
    static const int forced = [] { const char* e = std::getenv("DOCC_ROCM_EW_GRID"); return e ? std::atoi(e) : 0; }();
    if (forced > 0) per_cu = forced;
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    int64_t blocks = (items + 255) / 256;
    const int64_t cap = (int64_t) cus * per_cu;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (uint32_t) blocks;
}

bool is_transcendental(int unary_op) {
    return unary_op == DOCC_ROCM_UNARY_EXP || unary_op == DOCC_ROCM_UNARY_SIGMOID || unary_op == DOCC_ROCM_UNARY_TANH ||
           unary_op == DOCC_ROCM_UNARY_ERF;
}

// mirrors docc_k::BroadcastParams (csrc/kernels/elementwise.hip)
struct BroadcastParams {
    int rank;
    long n;
    long out_dims[6];
    long in_strides[6];
};

// mirrors docc_k::FusedParams (csrc/kernels/elementwise.hip)
struct FusedParams {
    long n;
    int rank;
    long dims[6];
    long a_strides[6];
    long b_strides[6];
    int binary;
    int a_scalar, b_scalar;
    int a_reused, b_reused;
    double scalar_a, scalar_b;
    int npost;
    int post[4];
};

// mirrors docc_k::FusedRowsParams
struct FusedRowsParams {
    long rows, cols;
    long a_row_stride, b_row_stride;
    int a_along_cols, b_along_cols;
    int binary;
    int a_scalar, b_scalar;
    int a_reused, b_reused;
    int npost;
    int post[4];
    double scalar_a, scalar_b;
    int cx_log2;
    unsigned groups_x;
};

// element strides of an operand of shape `in` (extent 1 repeats) inside the output shape
int operand_strides(const char* what, int rank, const int64_t* in, const int64_t* out, long* strides) {
    long stride = 1;
    for (int d = rank - 1; d >= 0; d--) {
        if (in[d] != out[d] && in[d] != 1)
            return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: dimension %d has extent %lld, cannot become %lld", what, d,
                        (long long) in[d], (long long) out[d]);
        strides[d] = in[d] == 1 ? 0 : stride;
        stride *= (long) in[d];
    }
    return 0;
}

int check_precision(const char* what, int precision) {
    if (precision != 32 && precision != 64) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: precision must be 32 or 64", what);
    return 0;
}

} // namespace

extern "C" int docc_rocm_elementwise_unary(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* X, void* Y) {
    if (op < 0 || op >= (int) (sizeof(kUnaryNames) / sizeof(kUnaryNames[0])))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_unary: unknown operation %d", op);
    if (int rc = check_precision("elementwise_unary", precision)) return rc;
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_unary: negative count");
    if (n == 0) return 0;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_unary: null pointer");
    if (int rc = ensure_device()) return rc;
    const int per_vec = precision == 32 ? 4 : 2;
    const bool aligned = (((uintptr_t) X | (uintptr_t) Y) % 16) == 0;
    const long nvec = aligned ? (long) (n / per_vec) : 0;
    char name[64];
    std::snprintf(name, sizeof(name), "docc_ew_%s_f%d", kUnaryNames[op], precision);
    return launch(name, grid_for(aligned ? (n + per_vec - 1) / per_vec : n, is_transcendental(op) ? kGridTranscendental : kGridStreaming), 1, 1,
                  256, 0, (hipStream_t) stream, X, Y, (long) n, nvec);
}

extern "C" int docc_rocm_elementwise_activation(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* X, void* Y,
                                                double alpha, double beta) {
    static const char* const names[] = {"elu", "leaky_relu", "hard_sigmoid"};
    if (op < DOCC_ROCM_UNARY_ELU || op > DOCC_ROCM_UNARY_HARD_SIGMOID)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_activation: unknown operation %d", op);
    if (int rc = check_precision("elementwise_activation", precision)) return rc;
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_activation: negative count");
    if (n == 0) return 0;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_activation: null pointer");
    if (int rc = ensure_device()) return rc;
    const int per_vec = precision == 32 ? 4 : 2;
    const bool aligned = (((uintptr_t) X | (uintptr_t) Y) % 16) == 0;
    const long nvec = aligned ? (long) (n / per_vec) : 0;
    char name[64];
    std::snprintf(name, sizeof(name), "docc_ew_%s_f%d", names[op - DOCC_ROCM_UNARY_ELU], precision);
    const uint32_t grid = grid_for(aligned ? (n + per_vec - 1) / per_vec : n, op == DOCC_ROCM_UNARY_ELU ? kGridTranscendental : kGridStreaming);
    if (precision == 32) return launch(name, grid, 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) n, nvec, (float) alpha, (float) beta);
    return launch(name, grid, 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) n, nvec, alpha, beta);
}

extern "C" int docc_rocm_fill(docc_rocm_stream_t stream, int element_bytes, int64_t n, const void* value, void* Y) {
    if (element_bytes != 1 && element_bytes != 2 && element_bytes != 4 && element_bytes != 8)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "fill: element size must be 1, 2, 4 or 8 bytes");
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "fill: negative count");
    if (n == 0) return 0;
    if (!value || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "fill: null pointer");
    if ((uintptr_t) Y % (uintptr_t) element_bytes) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "fill: the output is not aligned to its element size");
    if (int rc = ensure_device()) return rc;
    struct alignas(16) Pattern { unsigned char b[16]; } pattern;      // passed by value, like the kernel's uint4
    for (int i = 0; i < 16; i++) pattern.b[i] = ((const unsigned char*) value)[i % element_bytes];
    const long bytes = (long) n * element_bytes;
    const long nvec = (uintptr_t) Y % 16 == 0 ? bytes / 16 : 0;
    return launch("docc_fill_bytes", grid_for(nvec > 0 ? nvec : bytes, kGridStreaming), 1, 1, 256, 0, (hipStream_t) stream, Y, bytes, nvec, pattern);
}

extern "C" int docc_rocm_elementwise_binary(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* A,
                                            const void* B, void* Y) {
    if (op < 0 || op >= (int) (sizeof(kBinaryNames) / sizeof(kBinaryNames[0])))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_binary: unknown operation %d", op);
    if (int rc = check_precision("elementwise_binary", precision)) return rc;
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_binary: negative count");
    if (n == 0) return 0;
    if (!A || !B || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_binary: null pointer");
    if (int rc = ensure_device()) return rc;
    const int per_vec = precision == 32 ? 4 : 2;
    const bool aligned = (((uintptr_t) A | (uintptr_t) B | (uintptr_t) Y) % 16) == 0;
    const long nvec = aligned ? (long) (n / per_vec) : 0;
    char name[64];
    std::snprintf(name, sizeof(name), "docc_ew_%s_f%d", kBinaryNames[op], precision);
    return launch(name, grid_for(aligned ? (n + per_vec - 1) / per_vec : n, op == DOCC_ROCM_BINARY_POW ? kGridTranscendental : kGridStreaming), 1, 1, 256, 0, (hipStream_t) stream, A, B, Y, (long) n,
                  nvec);
}

extern "C" int docc_rocm_elementwise_binary_scalar(docc_rocm_stream_t stream, int op, int precision, int64_t n, const void* A,
                                                   double scalar, int scalar_is_lhs, void* Y) {
    if (op < 0 || op >= (int) (sizeof(kBinaryNames) / sizeof(kBinaryNames[0])))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_binary_scalar: unknown operation %d", op);
    if (int rc = check_precision("elementwise_binary_scalar", precision)) return rc;
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_binary_scalar: negative count");
    if (n == 0) return 0;
    if (!A || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "elementwise_binary_scalar: null pointer");
    if (int rc = ensure_device()) return rc;
    const int per_vec = precision == 32 ? 4 : 2;
    const bool aligned = (((uintptr_t) A | (uintptr_t) Y) % 16) == 0;
    const long nvec = aligned ? (long) (n / per_vec) : 0;
    char name[64];
    std::snprintf(name, sizeof(name), "docc_ew_%s_%s_f%d", kBinaryNames[op], scalar_is_lhs ? "sl" : "sr", precision);
    const uint32_t grid = grid_for(aligned ? (n + per_vec - 1) / per_vec : n, op == DOCC_ROCM_BINARY_POW ? kGridTranscendental : kGridStreaming);
    if (precision == 32) return launch(name, grid, 1, 1, 256, 0, (hipStream_t) stream, A, (float) scalar, Y, (long) n, nvec);
    return launch(name, grid, 1, 1, 256, 0, (hipStream_t) stream, A, scalar, Y, (long) n, nvec);
}

extern "C" int docc_rocm_broadcast(docc_rocm_stream_t stream, int precision, int rank, const int64_t* in_shape,
                                   const int64_t* out_shape, const void* X, void* Y) {
    if (int rc = check_precision("broadcast", precision)) return rc;
    if (rank < 1 || rank > 6) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "broadcast: rank %d (1..6 are built)", rank);
    if (!in_shape || !out_shape) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "broadcast: null shape");
    long dims[6], strides[6];
    long n = 1, stride = 1;
    for (int d = rank - 1; d >= 0; d--) {
        if (in_shape[d] < 0 || out_shape[d] < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "broadcast: negative extent");
        if (in_shape[d] != out_shape[d] && in_shape[d] != 1)
            return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "broadcast: dimension %d has extent %lld, cannot become %lld", d,
                        (long long) in_shape[d], (long long) out_shape[d]);
        dims[d] = (long) out_shape[d];
        strides[d] = in_shape[d] == 1 ? 0 : stride;
        stride *= (long) in_shape[d];
        n *= (long) out_shape[d];
    }
    if (n == 0) return 0;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "broadcast: null pointer");
    if (int rc = ensure_device()) return rc;
    // collapse: drop extent-1 dimensions, merge neighbours that are both repeated or contiguous
    BroadcastParams p{};
    p.n = n;
    int r = 0;
    for (int d = 0; d < rank; d++) {
        if (dims[d] == 1) continue;
        if (r > 0 && ((p.in_strides[r - 1] == 0 && strides[d] == 0) ||
                      (strides[d] != 0 && p.in_strides[r - 1] == strides[d] * dims[d]))) {
            p.out_dims[r - 1] *= dims[d];
            p.in_strides[r - 1] = strides[d];
        } else {
            p.out_dims[r] = dims[d];
            p.in_strides[r] = strides[d];
            r++;
        }
    }
    if (r == 0) {  // a single element
        p.out_dims[0] = 1;
        p.in_strides[0] = 0;
        r = 1;
    }
    p.rank = r;
    const int per_vec = precision == 32 ? 4 : 2;
    const bool vec = p.out_dims[r - 1] % per_vec == 0 && (uintptr_t) Y % 16 == 0 &&
                     (p.in_strides[r - 1] == 0 || (uintptr_t) X % 16 == 0);
    const int lanes = vec ? per_vec : 1;
    char name[64];
    std::snprintf(name, sizeof(name), "docc_broadcast_f%d_v%d_i%d", precision, lanes, n < (1L << 31) ? 32 : 64);
    return launch(name, grid_for(n / lanes, kGridStreaming), 1, 1, 256, 0, (hipStream_t) stream, X, Y, p);
}

extern "C" int docc_rocm_elementwise_fused(docc_rocm_stream_t stream, int precision, int rank, const int64_t* shape, int binary_op,
                                           const int64_t* a_shape, const void* A, double a_scalar, const int64_t* b_shape,
                                           const void* B, double b_scalar, int n_post, const int* post_ops, void* Y) {
    const char* what = "elementwise_fused";
    if (int rc = check_precision(what, precision)) return rc;
    if (rank < 1 || rank > 6) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: rank %d (1..6 are built)", what, rank);
    if (!shape) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: null shape", what);
    const int n_binary = (int) (sizeof(kBinaryNames) / sizeof(kBinaryNames[0])), n_unary = (int) (sizeof(kUnaryNames) / sizeof(kUnaryNames[0]));
    if (binary_op < -1 || binary_op >= n_binary) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: unknown binary operation %d", what, binary_op);
    if (n_post < 0 || n_post > 4) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "%s: %d unary operations (up to 4)", what, n_post);
    if (n_post > 0 && !post_ops) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: null operation list", what);
    FusedParams p{};
    for (int k = 0; k < n_post; k++) {
        if (post_ops[k] < 0 || post_ops[k] >= n_unary) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: unknown unary operation %d", what, post_ops[k]);
        p.post[k] = post_ops[k];
    }
    p.npost = n_post;
    p.binary = binary_op;
    const bool has_b = binary_op >= 0;
    p.a_scalar = a_shape == nullptr;
    p.b_scalar = has_b && b_shape == nullptr;
    p.scalar_a = a_scalar;
    p.scalar_b = b_scalar;
    if (p.a_scalar && (!has_b || p.b_scalar)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: no array operand", what);
    long dims[6], sa[6] = {0}, sb[6] = {0};
    long n = 1;
    for (int d = 0; d < rank; d++) {
        if (shape[d] < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: negative extent", what);
        dims[d] = (long) shape[d];
        n *= dims[d];
    }
    if (!p.a_scalar)
        if (int rc = operand_strides(what, rank, a_shape, shape, sa)) return rc;
    if (has_b && !p.b_scalar)
        if (int rc = operand_strides(what, rank, b_shape, shape, sb)) return rc;
    if (n == 0) return 0;
    if (!Y || (!p.a_scalar && !A) || (has_b && !p.b_scalar && !B)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
    if (int rc = ensure_device()) return rc;
    // collapse: drop extent-1 dimensions; merge neighbours that are contiguous (or repeated) in both operands
    int r = 0;
    for (int d = 0; d < rank; d++) {
        if (dims[d] == 1) continue;
        if (r > 0 && p.a_strides[r - 1] == sa[d] * dims[d] && p.b_strides[r - 1] == sb[d] * dims[d]) {
            p.dims[r - 1] *= dims[d];
            p.a_strides[r - 1] = sa[d];
            p.b_strides[r - 1] = sb[d];
        } else {
            p.dims[r] = dims[d];
            p.a_strides[r] = sa[d];
            p.b_strides[r] = sb[d];
            r++;
        }
    }
    if (r == 0) {
        p.dims[0] = 1;
        r = 1;
    }
    p.rank = r;
    p.n = n;
    for (int d = 0; d < r; d++) {
        if (p.a_strides[d] == 0) p.a_reused = 1;
        if (p.b_strides[d] == 0) p.b_reused = 1;
    }
    const int per_vec = precision == 32 ? 4 : 2;
    auto vector_ok = [&](bool scalar, const void* ptr, long inner_stride) {
        return scalar || inner_stride == 0 || (inner_stride == 1 && (uintptr_t) ptr % 16 == 0);
    };
    const bool vec = p.dims[r - 1] % per_vec == 0 && (uintptr_t) Y % 16 == 0 && vector_ok(p.a_scalar, A, p.a_strides[r - 1]) &&
                     (!has_b || vector_ok(p.b_scalar, B, p.b_strides[r - 1]));
    const int lanes = vec ? per_vec : 1;
    char name[64];
    // rows x columns with every operand contiguous or repeated along the columns: the kernel that walks rows
    // one long run of full and scalar operands is cut into rows of 256 vectors for it
    const long run_vecs = r == 1 ? p.dims[0] / per_vec : 0;
    const bool general_only = std::getenv("DOCC_ROCM_EW_FUSED_GENERAL") != nullptr;
    if (vec && !general_only && run_vecs > 256 && run_vecs % 256 == 0) {
        p.rank = 2;
        p.dims[0] = run_vecs / 256, p.dims[1] = 256 * per_vec;
        p.a_strides[1] = p.a_strides[0], p.a_strides[0] *= p.dims[1];
        p.b_strides[1] = p.b_strides[0], p.b_strides[0] *= p.dims[1];
    }
    if (vec && p.rank <= 2 && !general_only) {
        const long rows = p.rank == 2 ? p.dims[0] : 1, cvecs = p.dims[p.rank - 1] / per_vec;
        // a group: 2^cx_log2 column vectors by 256 >> cx_log2 rows, four rows a lane
        int cx_log2 = 0;
        while (cx_log2 < 8 && (1L << cx_log2) < cvecs) cx_log2++;
        const long groups_x = (cvecs + (1L << cx_log2) - 1) >> cx_log2, rows_per_group = 4L * (256 >> cx_log2);
        const long groups = groups_x * ((rows + rows_per_group - 1) / rows_per_group);
        // not for widths that leave more than a quarter of the lanes without a column
        if (groups <= 0x7fffffffL && cvecs * 4 >= (groups_x << cx_log2) * 3) {
            FusedRowsParams q{};
            const int last = p.rank - 1;
            q.rows = rows, q.cols = p.dims[last];
            q.a_row_stride = p.rank == 2 ? p.a_strides[0] : 0, q.b_row_stride = p.rank == 2 ? p.b_strides[0] : 0;
            q.a_along_cols = p.a_strides[last] != 0, q.b_along_cols = p.b_strides[last] != 0;
            q.binary = p.binary, q.a_scalar = p.a_scalar, q.b_scalar = p.b_scalar, q.a_reused = p.a_reused, q.b_reused = p.b_reused;
            q.npost = p.npost;
            for (int k = 0; k < 4; k++) q.post[k] = p.post[k];
            q.scalar_a = p.scalar_a, q.scalar_b = p.scalar_b;
            q.cx_log2 = cx_log2, q.groups_x = (unsigned) groups_x;
            std::snprintf(name, sizeof(name), "docc_ew_fused_rows_f%d_v%d", precision, per_vec);
            return launch(name, (uint32_t) groups, 1, 1, 256, 0, (hipStream_t) stream, A, B, Y, q);
        }
    }
    std::snprintf(name, sizeof(name), "docc_ew_fused_f%d_v%d_i%d", precision, lanes, n < (1L << 31) ? 32 : 64);
    return launch(name, grid_for(n / lanes, kGridFused), 1, 1, 256, 0, (hipStream_t) stream, A, B, Y, p);
}

extern "C" int docc_rocm_cast(docc_rocm_stream_t stream, int src_type, int dst_type, int64_t n, const void* X, void* Y) {
    static const char* const kTypeNames[] = {"f16", "bf16", "f32", "f64", "i32", "i64"};
    static const int kSize[] = {2, 2, 4, 8, 4, 8};
    if (src_type < 0 || src_type > DOCC_ROCM_TYPE_I64 || dst_type < 0 || dst_type > DOCC_ROCM_TYPE_I64)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "cast: unknown type code");
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "cast: negative count");
    if (n == 0) return 0;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "cast: null pointer");
    if (src_type == dst_type) {
        if (X == Y) return 0;
        return check(hipMemcpyAsync(Y, X, (size_t) n * kSize[src_type], hipMemcpyDeviceToDevice, resolve_stream((hipStream_t) stream)), "hipMemcpyAsync");
    }
    // built: fp32 <-> fp64 / bf16 / fp16, int32 / int64 <-> fp32 / fp64
    const bool f = src_type == DOCC_ROCM_TYPE_F32 || src_type == DOCC_ROCM_TYPE_F64, g = dst_type == DOCC_ROCM_TYPE_F32 || dst_type == DOCC_ROCM_TYPE_F64;
    const bool s16 = src_type <= DOCC_ROCM_TYPE_BF16, d16 = dst_type <= DOCC_ROCM_TYPE_BF16;
    const bool si = src_type >= DOCC_ROCM_TYPE_I32, di = dst_type >= DOCC_ROCM_TYPE_I32;
    const bool built = (f && g) || (s16 && dst_type == DOCC_ROCM_TYPE_F32) || (d16 && src_type == DOCC_ROCM_TYPE_F32) || (si && g) || (f && di);
    if (!built)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "cast: %s -> %s is not built (16-bit types convert through f32, integers to and from f32 / f64)",
                    kTypeNames[src_type], kTypeNames[dst_type]);
    int rc = ensure_device();
    if (rc) return rc;
    char name[48];
    std::snprintf(name, sizeof(name), "docc_cast_%s_%s", kTypeNames[src_type], kTypeNames[dst_type]);
    return launch(name, grid_for(n, kGridStreaming), 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) n);
}
