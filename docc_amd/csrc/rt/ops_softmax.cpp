// Launchers for ml::Softmax and the utility kernels (see include/docc_rocm_ops.h).
#include <cstdio>
#include <cstdlib>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

namespace docc::rt::rocm {

// Slices of the row-sliced form of a softmax over the rows of [rows, cols] (two launches around (maximum, sum) pairs,
// rows * slices * 2 elements of them), 0 where a one-launch kernel serves; *per = columns of a slice. Rows that a
// work-group's registers hold (4096 16-byte vectors; 16384 with sixteen wavefronts, `in_registers`, where there are rows
// enough to occupy half the CUs that way) stay with the one-launch kernels; longer rows, or rows too few to fill the
// device one work-group each, are cut so that about eight work-groups per CU share the tensor, no slice shorter
// than 4096 columns.
int64_t softmax_row_slices(int precision, int64_t rows, int64_t cols, bool in_registers, int cus, int64_t capacity, int64_t* per) {
    const int64_t per_vec = 128 / precision;
    if (cols <= 4096 * per_vec) return 0;
    if (in_registers && cols <= 16384 * per_vec && rows >= cus / 2) return 0;
    int64_t slices = (8 * (int64_t) cus + rows - 1) / rows;
    if (slices > cols / 4096) slices = cols / 4096;
    if (slices > 1024) slices = 1024;
    if (slices < 1) slices = 1;
    const int64_t width = ((cols + slices - 1) / slices + 1023) / 1024 * 1024;
    slices = (cols + width - 1) / width;
    if (rows > 0x7fffffffLL / slices) return 0;
    if (rows * slices * 2 * (precision / 8) > capacity) return 0;
    if (per) *per = width;
    return slices;
}

namespace {
int softmax_rowsliced(hipStream_t s, int precision, int64_t rows, int64_t cols, int64_t slices, int64_t per, const void* X, void* Y, void* partials) {
    PartialsLease lease;
    if (!partials) {
        if (int rc = partials_for(s, &lease)) return rc;
        partials = lease.ptr;
    }
    const size_t elem = (size_t) precision / 8;
    const int vec = ((uintptr_t) X % elem == 0) && ((uintptr_t) Y % elem == 0) && ((uintptr_t) X % 16 == (uintptr_t) Y % 16);
    const char* t = precision == 32 ? "f32" : "f64";
    char name[64];
    std::snprintf(name, sizeof(name), "docc_softmax_%s_rowslice_partial", t);
    if (int rc = launch(name, (uint32_t) (rows * slices), 1, 1, 256, 0, s, partials, X, (long) cols, (long) per, (int) slices, vec)) return rc;
    std::snprintf(name, sizeof(name), "docc_softmax_%s_rowslice_finish", t);
    return launch(name, (uint32_t) (rows * slices), 1, 1, 256, 0, s, (const void*) partials, X, Y, (long) cols, (long) per, (int) slices, vec);
}
} // namespace

// The row softmax (inner == 1) in either precision; `partials` as for softmax_general. The forms are chosen by the
// number of 16-byte vectors in a row (four floats or two doubles each), which is what a lane holds.
int softmax_rows(hipStream_t s, int precision, int64_t rows, int64_t cols, const void* X, void* Y, void* partials) {
    if (rows > 0x7fffffffLL) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "softmax: more than 2^31-1 rows");
    const int64_t per_vec = 128 / precision, elem = precision / 8;
    const char* t = precision == 32 ? "f32" : "f64";
    char name[64];
    auto run = [&](const char* form, uint32_t groups, uint32_t threads) {
        std::snprintf(name, sizeof(name), "docc_softmax_%s_%s", t, form);
        return launch(name, groups, 1, 1, threads, 0, s, X, Y, (long) rows, (int) cols);
    };
    auto stream_kernel = [&]() {
        std::snprintf(name, sizeof(name), "docc_softmax_%s_stream", t);
        return launch(name, (uint32_t) rows, 1, 1, 256, 0, s, X, Y, (long) rows, (long) cols);
    };
    const bool vec_ok = (cols % per_vec == 0) && (((uintptr_t) X | (uintptr_t) Y) % 16 == 0);
    // rows that start off a 16-byte boundary are still read in vectors when they start equally far off it in X and Y
    const bool same_place = (((uintptr_t) X | (uintptr_t) Y) % elem == 0) && ((uintptr_t) X % 16 == (uintptr_t) Y % 16);
    const int64_t nvec = (cols + per_vec - 1) / per_vec;
    if (nvec > 4096) {
        int cus = compute_units();
        if (cus <= 0) cus = 256;
        int64_t per = 0;
        const int64_t slices = softmax_row_slices(precision, rows, cols, vec_ok || same_place, cus, (int64_t) kPartialsBytes, &per);
        if (slices > 0) return softmax_rowsliced(s, precision, rows, cols, slices, per, X, Y, partials);
        if (vec_ok && nvec <= 16384) return run(nvec <= 8192 ? "block16_v8" : "block16_v16", (uint32_t) rows, 1024);
        if (same_place && nvec <= 16384) return run(nvec <= 8192 ? "any16_v8" : "any16_v16", (uint32_t) rows, 1024);
        return stream_kernel();
    }
    // Up to 256 vectors (1024 floats) one wavefront per row moves the most bytes (6.1-6.4 TB/s measured against 2.6-5.6
    // for a work-group per row); from 512 vectors on the work-group per row is ahead (6.1-6.3 against
    // 5.8-6.0 TB/s). DOCC_ROCM_SOFTMAX=wave|block overrides the choice (tuning; block = four wavefronts per row).
    const char* force = std::getenv("DOCC_ROCM_SOFTMAX");
    const bool wave = force && force[0] == 'w' ? true : force && force[0] == 'b' ? false : nvec <= 256;
    if (vec_ok && nvec <= 32 && !force) {
        // several rows per wavefront: LPR lanes a row, four sets of 64 / LPR rows per wavefront, four wavefronts
        int lpr = 1;
        while (lpr < nvec) lpr *= 2;
        char form[16];
        std::snprintf(form, sizeof(form), "sub%d", lpr);
        const int64_t rows_per_group = 4 * 4 * (64 / lpr);
        return run(form, (uint32_t) ((rows + rows_per_group - 1) / rows_per_group), 256);
    }
    if (vec_ok && nvec <= 1024 && wave)   // one wavefront per row, 4 rows per 256-thread block
        return run(nvec <= 64 ? "wave_v1" : nvec <= 128 ? "wave_v2" : nvec <= 256 ? "wave_v4" : nvec <= 512 ? "wave_v8" : "wave_v16",
                   (uint32_t) ((rows + 3) / 4), 256);
    if (vec_ok && nvec > 512 && nvec <= 1024 && !(force && force[0] == 'b'))
        // eight wavefronts per row, two vectors per lane: 6.24 TB/s against 6.09 with four wavefronts at 4096 floats
        return run("block8_v2", (uint32_t) rows, 512);
    if (vec_ok)
        return run(nvec <= 256 ? "block_v1" : nvec <= 512 ? "block_v2" : nvec <= 1024 ? "block_v4" : nvec <= 2048 ? "block_v8" : "block_v16",
                   (uint32_t) rows, 256);
    if (same_place && nvec >= 64 && !force) return run(nvec <= 256 ? "any4_v1" : nvec <= 1024 ? "any4_v4" : "any4_v16", (uint32_t) rows, 256);
    return stream_kernel();
}

} // namespace docc::rt::rocm

extern "C" {

int docc_rocm_softmax_f32(docc_rocm_stream_t stream, int64_t rows, int64_t cols, const float* X, float* Y) {
    if (rows < 0 || cols < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "softmax: negative shape");
    if (rows == 0 || cols == 0) return 0;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "softmax: null pointer");
    if (int rc = ensure_device()) return rc;
    return softmax_rows((hipStream_t) stream, 32, rows, cols, X, Y, nullptr);
}

} // extern "C"

namespace docc::rt::rocm {

// Number of row slices of the sliced form for softmax over the middle extent of an [outer, reduce, inner] view
// (inner > 32 or not a power of two), 0 when the one-launch tile kernel is used. Few (outer index, column
// tile) pairs and many rows: the rows are sliced as well, so that about four work-groups per CU share the
// tensor; the (maximum, sum) pairs of the slices need outer * slices * inner * 2 elements of `capacity` bytes.
int64_t softmax_slices(int precision, int64_t outer, int64_t reduce, int64_t inner, int cus, int64_t capacity) {
    const int64_t tiles = (inner + 63) / 64, groups = outer * tiles;
    if (groups >= 2 * (int64_t) cus || reduce < 256) return 0;
    int64_t slices = (4 * (int64_t) cus + groups - 1) / groups;
    if (slices > reduce / 64) slices = reduce / 64;
    const int64_t pair_bytes = 2 * (precision / 8);
    const int64_t fit = capacity / (outer * inner * pair_bytes);
    if (slices > fit) slices = fit;
    return slices >= 2 ? slices : 0;
}

// The general softmax. `partials` = nullptr: the sliced form takes the stream's partial-results buffer;
// otherwise `partials` (at least softmax_slices(.., kPartialsBytes) slices' worth of pairs) is used.
int softmax_general(hipStream_t s, int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X, void* Y, void* partials) {
    const char* t = precision == 32 ? "f32" : "f64";
    char name[64];
    if (inner == 1) return softmax_rows(s, precision, outer, reduce, X, Y, partials);
    if (inner <= 32 && (inner & (inner - 1)) == 0) {
        // a few inner positions: one work-group per outer index walks its contiguous slab
        if (outer > 0x7fffffffLL) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "softmax: more than 2^31-1 outer indices");
        std::snprintf(name, sizeof(name), "docc_softmax_%s_slab", t);
        return launch(name, (uint32_t) outer, 1, 1, 256, 0, s, X, Y, (long) reduce, (int) inner);
    }
    const int64_t tiles = (inner + 63) / 64;
    if (tiles > 0x7fffffffLL / outer) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "softmax: more than 2^31-1 work-groups");
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    const int64_t groups = outer * tiles;
    const int64_t slices = softmax_slices(precision, outer, reduce, inner, cus, (int64_t) kPartialsBytes);
    if (slices >= 2) {
        PartialsLease lease;
        if (!partials) {
            if (int rc = partials_for(s, &lease)) return rc;
            partials = lease.ptr;
        }
        const int64_t vec = 128 / precision;
        const char* form = std::getenv("DOCC_ROCM_SOFTMAX_TILE");
        const int64_t vtiles = (inner / vec + 15) / 16;
        // columns in 16-byte vectors where the tensor allows it: 16 vectors of columns per work-group
        const bool vectors = inner % vec == 0 && (((uintptr_t) X | (uintptr_t) Y) % 16) == 0 && !(form && form[0] == 's') &&
                             outer * vtiles <= 0x7fffffffLL / slices;
        const int64_t launch_tiles = vectors ? vtiles : tiles;
        std::snprintf(name, sizeof(name), "docc_softmax_%s_sliced%s_partial", t, vectors ? "v" : "");
        int rc = launch(name, (uint32_t) (outer * launch_tiles * slices), 1, 1, 256, 0, s, partials, X, (long) reduce, (long) inner, (long) launch_tiles,
                        (int) slices);
        if (rc) return rc;
        std::snprintf(name, sizeof(name), "docc_softmax_%s_sliced%s_finish", t, vectors ? "v" : "");
        return launch(name, (uint32_t) (outer * launch_tiles * slices), 1, 1, 256, 0, s, (const void*) partials, X, Y, (long) reduce, (long) inner,
                      (long) launch_tiles, (int) slices);
    }
    const int64_t per_vec = 128 / precision;
    const char* tile_form = std::getenv("DOCC_ROCM_SOFTMAX_TILE");   // scalar | v16 | v4 (tests, tuning)
    if (inner % per_vec == 0 && (((uintptr_t) X | (uintptr_t) Y) % 16) == 0 && !(tile_form && tile_form[0] == 's')) {
        // 16-byte vectors: a work-group owns 16 vectors of columns and splits the extent sixteen ways, or 64 and four ways
        // measured (us, sixteen / four ways / the scalar kernel): [64, 1024, 1024] fp32 124 / 189 / 343, [1024, 64, 1024] 144 / 127 / 198,
        // [16, 21, 262144] 443 / 139 / 283, [256, 300, 256] 39 / 59 / 65, [4096, 128, 64] 62 / 115 / 68 (fp64: 179 / 202 / 159)
        const int64_t row_vectors = inner / per_vec;
        int parts = reduce >= 200 ? 16 : row_vectors >= 64 ? 4 : 0;
        if (tile_form && tile_form[0] == 'v') parts = tile_form[1] == '4' ? 4 : 16;
        const int64_t lanes = parts ? 256 / parts : 1;
        const int64_t vtiles = (row_vectors + lanes - 1) / lanes;
        if (parts && vtiles <= 0x7fffffffLL / outer) {
            std::snprintf(name, sizeof(name), "docc_softmax_%s_tilev%d", t, parts);
            return launch(name, (uint32_t) (outer * vtiles), 1, 1, 256, 0, s, X, Y, (long) reduce, (long) inner, (long) vtiles);
        }
    }
    std::snprintf(name, sizeof(name), "docc_softmax_%s_tile", t);
    return launch(name, (uint32_t) (outer * tiles), 1, 1, 256, 0, s, X, Y, (long) reduce, (long) inner, (long) tiles);
}

// argument checks shared by the entry points of the general softmax; 1 = nothing to do
int softmax_check(int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X, const void* Y) {
    if (precision != 32 && precision != 64) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "softmax: precision must be 32 or 64");
    if (outer < 0 || reduce < 0 || inner < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "softmax: negative shape");
    if (outer == 0 || reduce == 0 || inner == 0) return 1;
    if (!X || !Y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "softmax: null pointer");
    return 0;
}

} // namespace docc::rt::rocm

extern "C" {

int docc_rocm_softmax(docc_rocm_stream_t stream, int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X, void* Y) {
    if (int rc = softmax_check(precision, outer, reduce, inner, X, Y)) return rc == 1 ? 0 : rc;
    if (int rc = ensure_device()) return rc;
    return softmax_general((hipStream_t) stream, precision, outer, reduce, inner, X, Y, nullptr);
}

int64_t docc_rocm_softmax_workspace_bytes(int precision, int64_t outer, int64_t reduce, int64_t inner) {
    if ((precision != 32 && precision != 64) || outer <= 0 || reduce <= 0 || inner <= 0) return 0;
    if (inner != 1 && inner <= 32 && (inner & (inner - 1)) == 0) return 0;
    if (ensure_device()) return 0;
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    if (inner == 1)   // for any placement of the operands: rows that could stay in registers are cut when a pointer is not 16-byte aligned
        return (softmax_row_slices(precision, outer, reduce, false, cus, (int64_t) kPartialsBytes, nullptr) * outer * 2 * (precision / 8) + 255) / 256 * 256;
    const int64_t slices = softmax_slices(precision, outer, reduce, inner, cus, (int64_t) kPartialsBytes);
    return (slices * outer * inner * 2 * (precision / 8) + 255) / 256 * 256;
}

int docc_rocm_softmax_ws(docc_rocm_stream_t stream, int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X, void* Y,
                         void* workspace, int64_t workspace_bytes) {
    if (int rc = softmax_check(precision, outer, reduce, inner, X, Y)) return rc == 1 ? 0 : rc;
    if (int rc = ensure_device()) return rc;
    const int64_t need = docc_rocm_softmax_workspace_bytes(precision, outer, reduce, inner);
    if (need > 0 && (!workspace || workspace_bytes < need || ((uintptr_t) workspace % 256) != 0))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "softmax: this shape needs a 256-byte aligned workspace of %lld bytes", (long long) need);
    // need == 0: the shape runs as one launch and no partial results exist
    return softmax_general((hipStream_t) stream, precision, outer, reduce, inner, X, Y, need > 0 ? workspace : nullptr);
}

static uint32_t grid_for(int64_t items) {
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    int64_t blocks = (items + 255) / 256;
    int64_t cap = (int64_t) cus * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (uint32_t) blocks;
}

int docc_rocm_copy_bytes(docc_rocm_stream_t stream, int64_t bytes, const void* src, void* dst) {
    if (bytes < 0 || bytes % 16 != 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "copy_bytes: size must be a multiple of 16");
    if (bytes == 0) return 0;
    if (!src || !dst || (((uintptr_t) src | (uintptr_t) dst) % 16) != 0)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "copy_bytes: pointers must be 16-byte aligned");
    int rc = ensure_device();
    if (rc) return rc;
    long n16 = bytes / 16;
    // a work-group per 1024 vectors; more than 2^31 - 1 work-groups (32 TiB) in launches of that many
    const long per_launch = 0x7fffffffL;
    for (long done = 0; done < n16;) {
        long groups = (n16 - done + 1023) / 1024;
        if (groups > per_launch) groups = per_launch;
        const long count = groups * 1024 < n16 - done ? groups * 1024 : n16 - done;
        rc = launch("docc_copy_b128", (uint32_t) groups, 1, 1, 256, 0, (hipStream_t) stream, (const char*) src + done * 16, (char*) dst + done * 16, count);
        if (rc) return rc;
        done += count;
    }
    return 0;
}

int docc_rocm_mfma_probe(docc_rocm_stream_t stream, int precision, int waves_per_simd, int iters, const float* operands,
                         float* sink, double* flop) {
    if (precision != 64 && precision != 32 && precision != 16 && precision != 116)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "mfma_probe: precision must be 64, 32, 16 or 116");
    if (waves_per_simd < 1 || waves_per_simd > 2 || iters < 1) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "mfma_probe: waves_per_simd in 1..2, iters >= 1");
    if (!operands || !sink) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "mfma_probe: null pointer");
    int rc = ensure_device();
    if (rc) return rc;
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    const uint32_t groups = (uint32_t) (cus * waves_per_simd);
    // flop per MFMA: 16x16x4 fp64 = 2048, 32x32x2 fp32 = 4096, 32x32x16 bf16 = 32768, 16x16x32 bf16 = 16384; 32 MFMAs per round, 4 waves per group
    const double per_mfma = precision == 64 ? 2048.0 : precision == 32 ? 4096.0 : precision == 16 ? 32768.0 : 16384.0;
    if (flop) *flop = per_mfma * 32.0 * iters * 4.0 * groups;
    return launch(precision == 64 ? "docc_mfma_probe_f64" : precision == 32 ? "docc_mfma_probe_f32" : precision == 16 ? "docc_mfma_probe_bf16" : "docc_mfma_probe_bf16_16x16x32", groups, 1, 1,
                  256, 0, (hipStream_t) stream, operands, sink, iters);
}

int docc_rocm_clock_probe(docc_rocm_stream_t stream, int microseconds, float* mhz) {
    if (microseconds < 1 || microseconds > 100000) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "clock_probe: 1 .. 100000 microseconds");
    if (!mhz) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "clock_probe: null pointer");
    int rc = ensure_device();
    if (rc) return rc;
    return launch("docc_clock_probe", 1, 1, 1, 64, 0, (hipStream_t) stream, mhz, (long) microseconds * 100);
}

int docc_rocm_convert_f32_to_bf16(docc_rocm_stream_t stream, int64_t count, const float* src, uint16_t* dst) {
    if (count < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "convert: negative count");
    if (count == 0) return 0;
    if (!src || !dst) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "convert: null pointer");
    int rc = ensure_device();
    if (rc) return rc;
    return launch("docc_f32_to_bf16", grid_for(count), 1, 1, 256, 0, (hipStream_t) stream, src, dst, (long) count);
}

int docc_rocm_convert_bf16_to_f32(docc_rocm_stream_t stream, int64_t count, const uint16_t* src, float* dst) {
    if (count < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "convert: negative count");
    if (count == 0) return 0;
    if (!src || !dst) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "convert: null pointer");
    int rc = ensure_device();
    if (rc) return rc;
    return launch("docc_bf16_to_f32", grid_for(count), 1, 1, 256, 0, (hipStream_t) stream, src, dst, (long) count);
}

} // extern "C"
