// Launcher for the reduce tensor nodes (see include/docc_rocm_ops.h).
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "docc_rocm_ops.h"
#include "rt_state.h"

using namespace docc::rt::rocm;

extern "C" int docc_rocm_reduce(docc_rocm_stream_t stream, int op, int precision, int64_t outer, int64_t reduce, int64_t inner,
                                const void* X, void* Y) {
    static const char* const names[] = {"sum", "max", "min", "mean"};
    if (op < 0 || op > DOCC_ROCM_REDUCE_MEAN) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "reduce: unknown operation %d", op);
    if (precision != 32 && precision != 64) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "reduce: precision must be 32 or 64");
    if (outer < 0 || reduce < 0 || inner < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "reduce: negative extent");
    if (outer == 0 || inner == 0) return 0;
    if (reduce == 0 && (op == DOCC_ROCM_REDUCE_MEAN))
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "reduce: mean over an empty extent");
    if (!Y || (reduce > 0 && !X)) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "reduce: null pointer");
    if (int rc = ensure_device()) return rc;
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    char name[64];
    if (inner == 1) {
        const int per_vec = precision == 32 ? 4 : 2;
        const size_t elem = precision / 8;
        // every row starts on a 16-byte boundary
        const bool aligned = (uintptr_t) X % 16 == 0 && (reduce * elem) % 16 == 0;
        const long nvec = aligned ? (long) (reduce / per_vec) : 0;
        // short rows: several share a wavefront (1 to 32 lanes a row, four sets of rows per wavefront, four wavefronts)
        if (aligned && nvec >= 1 && nvec <= 32 && outer >= 64) {
            int lpr = 1;
            while (lpr < nvec) lpr *= 2;
            const int64_t per_group = 4 * 4 * (64 / lpr);
            std::snprintf(name, sizeof(name), "docc_reduce_rows%d_%s_f%d", lpr, names[op], precision);
            return launch(name, (uint32_t) ((outer + per_group - 1) / per_group), 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) outer, (long) reduce);
        }
        // Long rows, and too few of them for eight wavefronts per CU: each row in pieces of at least 4096 elements, one
        // wavefront a piece, the pieces' results through the stream's buffer of partial results and a second launch
        if (outer < (int64_t) cus * 8 && reduce >= 8192) {
            int64_t pieces_wanted = (int64_t) cus * 8;
            if (const char* e = std::getenv("DOCC_ROCM_REDUCE_PIECES")) pieces_wanted = std::atoll(e) > 0 ? std::atoll(e) : pieces_wanted;   // tuning
            int64_t slices = (pieces_wanted + outer - 1) / outer;
            if (slices > reduce / 4096) slices = reduce / 4096;
            if (slices > 4096) slices = 4096;
            const int64_t chunk = ((reduce + slices - 1) / slices + 1023) / 1024 * 1024;
            slices = (reduce + chunk - 1) / chunk;
            if (slices > 1 && outer * slices * (int64_t) elem <= (int64_t) kPartialsBytes) {
                PartialsLease partials;
                if (int rc = partials_for((hipStream_t) stream, &partials)) return rc;
                const int64_t pieces = outer * slices;
                int64_t groups = (pieces + 3) / 4;
                if (groups > (int64_t) cus * 16) groups = (int64_t) cus * 16;
                std::snprintf(name, sizeof(name), "docc_reduce_rowp_%s_f%d", names[op], precision);
                if (int rc = launch(name, (uint32_t) groups, 1, 1, 256, 0, (hipStream_t) stream, partials.ptr, X, (long) outer, (long) reduce, (long) chunk,
                                    (long) slices, aligned ? 1 : 0))
                    return rc;
                groups = (outer + 3) / 4;
                std::snprintf(name, sizeof(name), "docc_reduce_rowf_%s_f%d", names[op], precision);
                return launch(name, (uint32_t) groups, 1, 1, 256, 0, (hipStream_t) stream, (const void*) partials.ptr, Y, (long) outer, (long) reduce,
                              (long) slices);
            }
        }
        int64_t blocks = (outer + 3) / 4;   // four wavefronts per work-group, one row each
        if (blocks > (int64_t) cus * 16) blocks = (int64_t) cus * 16;
        std::snprintf(name, sizeof(name), "docc_reduce_row_%s_f%d", names[op], precision);
        return launch(name, (uint32_t) blocks, 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) outer, (long) reduce, nvec);
    }
    const int64_t total = outer * inner;
    int64_t blocks = (total + 255) / 256;
    // Too few output elements to fill the device: cut the reduced extent into slices. Their partial
    // results go through the stream's partial-results buffer.
    if (blocks < (int64_t) cus * 2 && reduce >= 64) {
        const int per_vec = 128 / precision;
        const bool vec = inner % per_vec == 0 && (uintptr_t) X % 16 == 0;
        const int64_t pblocks = vec ? (total / per_vec + 255) / 256 : blocks;
        const int64_t scratch_elems = (int64_t) kPartialsBytes / (precision / 8);
        // about three work-groups per CU: measured on [64, 1024, 512], [512, 512, 128], [8, 4096, 2048] and [1, 8192, 4096], twice as
        // many slices cost 5-30 % (the second launch reads them all), half as many leave CUs without work
        int64_t slices = ((int64_t) cus * 3 + pblocks - 1) / pblocks;
        if (slices > reduce / 16) slices = reduce / 16;
        if (slices > scratch_elems / total) slices = scratch_elems / total;
        int64_t cap = 1024;
        if (const char* e = std::getenv("DOCC_ROCM_REDUCE_SLICES")) cap = std::atoll(e) > 0 ? std::atoll(e) : cap;   // tuning
        if (slices > cap) slices = cap;
        if (slices > 1) {
            const int64_t chunk = (reduce + slices - 1) / slices;
            slices = (reduce + chunk - 1) / chunk;
            PartialsLease partials;
            if (int rc = partials_for((hipStream_t) stream, &partials)) return rc;
            std::snprintf(name, sizeof(name), "docc_reduce_colp%s_%s_f%d", vec ? "v" : "", names[op], precision);
            // the partial pass of a mean adds; the division happens once, in the final pass
            if (int rc = launch(name, (uint32_t) pblocks, (uint32_t) slices, 1, 256, 0, (hipStream_t) stream, partials.ptr, X, (long) outer,
                                (long) reduce, (long) inner, (long) chunk))
                return rc;
            std::snprintf(name, sizeof(name), "docc_reduce_colf_%s_f%d", names[op], precision);
            return launch(name, (uint32_t) ((total + 15) / 16), 1, 1, 256, 0, (hipStream_t) stream, (const void*) partials.ptr, Y, (long) total,
                          (long) reduce, (long) slices);
        }
    }
    if (blocks > (int64_t) cus * 16) blocks = (int64_t) cus * 16;
    std::snprintf(name, sizeof(name), "docc_reduce_col_%s_f%d", names[op], precision);
    return launch(name, (uint32_t) blocks, 1, 1, 256, 0, (hipStream_t) stream, X, Y, (long) outer, (long) reduce, (long) inner);
}

// DOT::BLAS. Like cblas_?dot / cublas?dot with the result in host memory (reference dot_node.cpp dispatcher,
// opt/src/targets/cuda/blas/dot.cpp:55-68): the call returns when the value is there.
extern "C" int docc_rocm_dot(docc_rocm_stream_t stream, int precision, int64_t n, const void* x, int64_t incx, const void* y, int64_t incy,
                             void* result) {
    if (precision != 32 && precision != 64) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "dot: precision must be 32 or 64");
    if (n < 0) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "dot: negative length");
    if (!result) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "dot: null result");
    const size_t elem = precision / 8;
    if (n == 0) {
        std::memset(result, 0, elem);
        return 0;
    }
    if (!x || !y) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "dot: null pointer");
    if (incx < 0 || incy < 0) return fail(DOCC_ROCM_ERR_UNSUPPORTED, "dot: negative increments are not supported");
    if (int rc = ensure_device()) return rc;
    int cus = compute_units();
    if (cus <= 0) cus = 256;
    // about four work-groups per CU, at least 2048 elements each
    int64_t groups = (n + 2047) / 2048;
    if (groups > 4 * (int64_t) cus) groups = 4 * (int64_t) cus;
    const int64_t chunk = (n + groups - 1) / groups;
    groups = (n + chunk - 1) / chunk;
    if (capturing()) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "dot: returns its result to the host and cannot be captured into a graph");
    hipStream_t s = resolve_stream((hipStream_t) stream);
    PartialsLease partials;
    if (int rc = partials_for(s, &partials)) return rc;
    const char* t = precision == 32 ? "f32" : "f64";
    char name[64];
    std::snprintf(name, sizeof(name), "docc_dot_partial_%s", t);
    if (int rc = launch(name, (uint32_t) groups, 1, 1, 256, 0, s, partials.ptr, x, (long) incx, y, (long) incy, (long) n, (long) chunk)) return rc;
    std::snprintf(name, sizeof(name), "docc_dot_final_%s", t);
    if (int rc = launch(name, 1, 1, 1, 256, 0, s, partials.ptr, (int) groups)) return rc;
    if (int rc = check(hipMemcpyAsync(result, (const char*) partials.ptr + (size_t) groups * elem, elem, hipMemcpyDeviceToHost, s), "hipMemcpyAsync (dot)"))
        return rc;
    return check(hipStreamSynchronize(s), "hipStreamSynchronize (dot)");
}
