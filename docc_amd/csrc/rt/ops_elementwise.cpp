// Launchers for the elementwise tensor nodes and ml::Broadcast (see include/docc_rocm_ops.h).
#include <cstdio>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace {

const char* const kUnaryNames[] = {"abs", "exp", "relu", "sigmoid", "sqrt", "tanh", "erf"};
const char* const kBinaryNames[] = {"add", "sub", "mul", "div", "maximum", "minimum"};

uint32_t grid_for(int64_t items) {
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    int64_t blocks = (items + 255) / 256;
    const int64_t cap = (int64_t) cus * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (uint32_t) blocks;
}

// mirrors docc_k::BroadcastParams (csrc/kernels/elementwise.hip)
struct BroadcastParams {
    int rank;
    long n;
    long out_dims[6];
    long in_strides[6];
};

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
    return launch(name, grid_for(aligned ? (n + per_vec - 1) / per_vec : n), 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) n, nvec);
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
    return launch(name, grid_for(aligned ? (n + per_vec - 1) / per_vec : n), 1, 1, 256, 0, (hipStream_t) stream, A, B, Y, (long) n,
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
    const uint32_t grid = grid_for(aligned ? (n + per_vec - 1) / per_vec : n);
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
    return launch(name, grid_for(n / lanes), 1, 1, 256, 0, (hipStream_t) stream, X, Y, p);
}
