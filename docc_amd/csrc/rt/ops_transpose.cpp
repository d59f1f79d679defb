// Launcher for ml::Transpose (see include/docc_rocm_ops.h).
#include <cstdio>
#include <cstdlib>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace {

// mirrors docc_k::TransposeParams (csrc/kernels/transpose.hip)
struct TransposeParams {
    long n;
    int rank;
    long ext[6];
    long in_stride[6];
    long out_stride[6];
    long a_ext, b_ext;
    long a_out_stride;
    long b_in_stride;
    long tiles_a, tiles_b;
};

} // namespace

extern "C" int docc_rocm_transpose(docc_rocm_stream_t stream, int element_bytes, int rank, const int64_t* shape, const int64_t* perm,
                                   const void* X, void* Y) {
    if (element_bytes != 1 && element_bytes != 2 && element_bytes != 4 && element_bytes != 8)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: element size must be 1, 2, 4 or 8 bytes");
    if (rank < 0 || rank > 6) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "transpose: rank must be 0..6");
    if (rank > 0 && (!shape || !perm)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: null shape or permutation");
    bool seen[6] = {false, false, false, false, false, false};
    int64_t n = 1;
    for (int i = 0; i < rank; i++) {
        if (shape[i] < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: negative extent");
        if (perm[i] < 0 || perm[i] >= rank || seen[perm[i]]) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: not a permutation");
        seen[perm[i]] = true;
        n *= shape[i];
    }
    if (n == 0) return 0;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: null pointer");
    if (X == Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: in place is not supported");
    int rc = ensure_device();
    if (rc) return rc;

    // input strides, then the axes in output order without those of extent one
    int64_t in_stride[6];
    int64_t s = 1;
    for (int i = rank - 1; i >= 0; i--) {
        in_stride[i] = s;
        s *= shape[i];
    }
    int64_t ext[6], ist[6];
    int src_axis[6];
    int r = 0;
    for (int i = 0; i < rank; i++) {
        if (shape[perm[i]] == 1) continue;
        ext[r] = shape[perm[i]];
        ist[r] = in_stride[perm[i]];
        src_axis[r] = (int) perm[i];
        r++;
    }
    // merge output axes that are adjacent in the input as well: (i, i+1) with stride[i] == ext[i+1] * stride[i+1]
    int m = 0;
    for (int i = 0; i < r; i++) {
        if (m > 0 && ist[m - 1] == ext[i] * ist[i]) {
            ext[m - 1] *= ext[i];
            ist[m - 1] = ist[i];
            src_axis[m - 1] = src_axis[i];
        } else {
            ext[m] = ext[i];
            ist[m] = ist[i];
            src_axis[m] = src_axis[i];
            m++;
        }
    }
    r = m;
    hipStream_t st = resolve_stream((hipStream_t) stream);
    if (r <= 1)   // nothing moves
        return check(hipMemcpyAsync(Y, X, (size_t) n * element_bytes, hipMemcpyDeviceToDevice, st), "hipMemcpyAsync");

    int64_t ost[6];
    s = 1;
    for (int i = r - 1; i >= 0; i--) {
        ost[i] = s;
        s *= ext[i];
    }
    TransposeParams p{};
    p.n = n;
    char name[48];
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    if (ist[r - 1] == 1) {
        // the innermost axis stays: rows of ext[r-1] contiguous elements move as they are, in units of up to
        // 16 bytes (every other stride is a multiple of the row length, so it scales with the unit)
        int unit = element_bytes;
        const int64_t row_bytes = ext[r - 1] * element_bytes;
        while (unit < 16 && row_bytes % (unit * 2) == 0 && ((uintptr_t) X | (uintptr_t) Y) % (unit * 2) == 0) unit *= 2;
        const int64_t scale = unit / element_bytes;
        p.rank = r;
        for (int i = 0; i < r; i++) {
            p.ext[i] = i == r - 1 ? ext[i] / scale : ext[i];
            p.in_stride[i] = i == r - 1 ? 1 : ist[i] / scale;
        }
        p.n = n / scale;
        std::snprintf(name, sizeof(name), "docc_transpose_rows_b%d_%s", unit * 8, p.n < (int64_t(1) << 31) ? "i32" : "i64");
        int64_t blocks = (p.n + 255) / 256;
        if (blocks > (int64_t) cus * 128) blocks = (int64_t) cus * 128;
        return launch(name, (uint32_t) blocks, 1, 1, 256, 0, st, X, Y, p);
    }
    // the input's innermost axis (stride 1) sits at output position `pa`; the plane (b = output's innermost
    // axis, a) is moved in 64 x 64 tiles, the other axes number the planes
    int pa = -1;
    for (int i = 0; i < r; i++)
        if (ist[i] == 1) pa = i;
    if (pa < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "transpose: internal error (no unit-stride axis)");
    p.a_ext = ext[pa];
    p.a_out_stride = ost[pa];
    p.b_ext = ext[r - 1];
    p.b_in_stride = ist[r - 1];
    p.tiles_a = (p.a_ext + 63) / 64;
    p.tiles_b = (p.b_ext + 63) / 64;
    int k = 0;
    int64_t planes = 1;
    for (int i = 0; i < r - 1; i++) {
        if (i == pa) continue;
        p.ext[k] = ext[i];
        p.in_stride[k] = ist[i];
        p.out_stride[k] = ost[i];
        planes *= ext[i];
        k++;
    }
    p.rank = k;
    const int64_t blocks = planes * p.tiles_a * p.tiles_b;
    if (blocks > 0x7fffffffLL) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "transpose: more than 2^31-1 tiles");
    // 4-byte elements, every extent, stride and address a multiple of four elements: the tile in 128-bit units
    bool quads = element_bytes == 4 && p.a_ext % 4 == 0 && p.b_ext % 4 == 0 && p.b_in_stride % 4 == 0 && p.a_out_stride % 4 == 0 &&
                 ((uintptr_t) X | (uintptr_t) Y) % 16 == 0 && !std::getenv("DOCC_ROCM_TRANSPOSE_SCALAR");
    for (int i = 0; i < p.rank; i++) quads = quads && p.in_stride[i] % 4 == 0 && p.out_stride[i] % 4 == 0;
    if (quads) {
        // tiles of 128 x 128 (rows of 512 bytes on both sides) where they still number four per CU: on tensors met for the
        // first time [8192, 4096] takes 53.5 us against 56.5, [16384, 16384] 427 against 465, [2048, 2048] 9.6 against 7.9.
        // DOCC_ROCM_TRANSPOSE_WIDE=1|0 forces the choice (tests, tuning).
        TransposeParams w = p;
        w.tiles_a = (p.a_ext + 127) / 128;
        w.tiles_b = (p.b_ext + 127) / 128;
        const int64_t wide_blocks = planes * w.tiles_a * w.tiles_b;
        int cus = compute_units();
        if (cus <= 0) cus = 256;
        const char* force = std::getenv("DOCC_ROCM_TRANSPOSE_WIDE");
        if (force ? force[0] == '1' : wide_blocks >= 4 * (int64_t) cus)
            return launch("docc_transpose_tile4w_b32", (uint32_t) wide_blocks, 1, 1, 256, 0, st, X, Y, w);
    }
    if (quads) return launch("docc_transpose_tile4_b32", (uint32_t) blocks, 1, 1, 256, 0, st, X, Y, p);
    std::snprintf(name, sizeof(name), "docc_transpose_tile_b%d", element_bytes * 8);
    return launch(name, (uint32_t) blocks, 1, 1, 256, 0, st, X, Y, p);
}
