// docc_rocm_softmax_noalloc (see include/docc_rocm_ops.h): the general softmax for callers that cannot
// allocate. The partial results of the sliced form live in a fixed array of the device image below instead of
// memory obtained at run time; everything else - the kernels, their geometry, the results - is
// docc_rocm_softmax.
//
// This is the only source file of the runtime that is compiled as HIP (host and device): the array has to be
// a symbol of a device image that the HIP runtime registers with the library, so that its address on each
// device can be asked for once, at set-up. Its name stands for the symbol, not for a device address: host
// code uses the address hipGetSymbolAddress returned, nothing else.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>

#include "docc_rocm_ops.h"
#include "rt_state.h"

namespace {

constexpr size_t kScratchBytes = size_t(1) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_setup_mutex;
void* g_scratch_ptr[kMaxDevices] = {};   // address of `scratch` on each device that has been set up

} // namespace

namespace docc::rt::rocm {

int64_t softmax_slices(int precision, int64_t outer, int64_t reduce, int64_t inner, int cus, int64_t capacity);
int softmax_general(hipStream_t s, int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X, void* Y, void* partials);
int softmax_check(int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X, const void* Y);
int64_t softmax_row_slices(int precision, int64_t rows, int64_t cols, bool in_registers, int cus, int64_t capacity, int64_t* per);

// Part of a device's set-up (docc_rocm_init, or the first launcher call on the device), with that device
// current: asks for the address of the array on this device and resolves the kernels the entry point
// launches, so that the entry point itself looks nothing up.
int noalloc_setup_device(int dev) {
    if (dev < 0 || dev >= kMaxDevices) return 0;   // the entry point refuses such a device
    std::lock_guard<std::mutex> lock(g_setup_mutex);
    if (g_scratch_ptr[dev]) return 0;
    void* ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress((void**) &ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr)
        return fail(err != hipSuccess ? (int) err : DOCC_ROCM_ERR_KERNEL_IMAGE, "address of the no-allocation scratch array on device %d: %s", dev,
                    hipGetErrorString(err));
    // every kernel docc_rocm_softmax may launch, in both precisions
    static const char* const forms[] = {
        "stream",     "slab",      "tile",      "tilev16",   "tilev4",    "sliced_partial", "sliced_finish", "slicedv_partial", "slicedv_finish", "rowslice_partial", "rowslice_finish",
        "wave_v1",    "wave_v2",   "wave_v4",   "wave_v8",        "wave_v16",      "block8_v2",        "block_v1",
        "block_v2",   "block_v4",  "block_v8",  "block_v16",      "block16_v8",    "block16_v16",      "any4_v1",
        "any4_v4",    "any4_v16",  "any16_v8",  "any16_v16",      "sub1",          "sub2",             "sub4",
        "sub8",       "sub16",     "sub32",
    };
    for (const char* form : forms)
        for (const char* type : {"f32", "f64"}) {
            char name[64];
            std::snprintf(name, sizeof(name), "docc_softmax_%s_%s", type, form);
            hipFunction_t fn;
            if (int rc = kernel(name, &fn)) return rc;
        }
    g_scratch_ptr[dev] = ptr;
    return 0;
}

} // namespace docc::rt::rocm

using namespace docc::rt::rocm;

extern "C" int docc_rocm_softmax_noalloc(docc_rocm_stream_t stream, int precision, int64_t outer, int64_t reduce, int64_t inner, const void* X,
                                         void* Y) {
    if (int rc = softmax_check(precision, outer, reduce, inner, X, Y)) return rc == 1 ? 0 : rc;
    int dev = -1;
    if (int rc = check(hipGetDevice(&dev), "hipGetDevice")) return rc;
    void* const partials = dev >= 0 && dev < kMaxDevices ? g_scratch_ptr[dev] : nullptr;
    if (!partials)
        return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT,
                    "softmax_noalloc: device %d has not been set up; call docc_rocm_init(%d) first (this entry point loads and allocates nothing)",
                    dev, dev);
    if (inner == 1) {
        int cus = compute_units();
        if (cus <= 0) cus = 256;
        // rows cut into slices leave one (maximum, sum) pair per row and slice
        const int64_t need = softmax_row_slices(precision, outer, reduce, false, cus, (int64_t) kPartialsBytes, nullptr) * outer * 2 * (precision / 8);
        if (need > (int64_t) kScratchBytes)
            return fail(DOCC_ROCM_ERR_UNSUPPORTED,
                        "softmax_noalloc: this shape needs %lld bytes of partial results, the entry point holds %lld; use docc_rocm_softmax or "
                        "docc_rocm_softmax_ws",
                        (long long) need, (long long) kScratchBytes);
    } else if (!(inner <= 32 && (inner & (inner - 1)) == 0)) {
        int cus = compute_units();
        if (cus <= 0) cus = 256;
        // the slices docc_rocm_softmax would cut the rows into, and the bytes their (maximum, sum) pairs take
        const int64_t slices = softmax_slices(precision, outer, reduce, inner, cus, (int64_t) kPartialsBytes);
        const int64_t need = slices * outer * inner * 2 * (precision / 8);
        if (need > (int64_t) kScratchBytes)
            return fail(DOCC_ROCM_ERR_UNSUPPORTED,
                        "softmax_noalloc: this shape needs %lld bytes of partial results, the entry point holds %lld; use docc_rocm_softmax or "
                        "docc_rocm_softmax_ws",
                        (long long) need, (long long) kScratchBytes);
    }
    // calls on one device share the array: a call overwrites what the last one left before it reads it back,
    // so nothing has to be cleared, and calls that overlap (two streams, two threads) race
    return softmax_general((hipStream_t) stream, precision, outer, reduce, inner, X, Y, partials);
}
