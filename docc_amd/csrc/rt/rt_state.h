// Internal state of the thin HIP runtime: per-device code object with the
// math kernels, a function cache, and the thread-local error string.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdint>
#include <mutex>
#include <string>

#include "docc_rocm_rt.h"

namespace docc::rt::rocm {

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Maps a hipError_t to the return convention (0 or the code, message recorded).
int check(hipError_t err, const char* what);

// Makes sure the current device has its state (module loaded). 0 or error.
int ensure_device();

// Looks up a kernel of the math code object on the current device.
int kernel(const char* name, hipFunction_t* fn);

// Number of compute units of the current device (after ensure_device()).
int compute_units();

// Partial results of the launchers that run as a pair of launches (sliced softmax, column reductions, column
// matrix-vector products): kPartialsBytes of device memory per (device, stream), created on the first such call
// on that stream and kept until the process ends. Two calls on different streams so never share a buffer; the
// lease also holds the stream's lock, so that two host threads feeding one stream enqueue their pairs one after
// the other. Keep the lease alive until the second launch of the pair has been issued.
constexpr size_t kPartialsBytes = size_t(8) << 20;
struct PartialsLease {
    void* ptr = nullptr;
    std::unique_lock<std::mutex> lock;
};
int partials_for(hipStream_t stream, PartialsLease* lease);

// The stream work is enqueued on: `stream` itself, or - where generated code and callers pass the null stream -
// the stream the calling thread has named with docc_rocm_set_default_stream (the null stream if none).
hipStream_t resolve_stream(hipStream_t stream);
// True while the calling thread has a graph capture open: calls that must wait for the device refuse then.
bool capturing();

// Launch helper: packs the addresses of `args` for hipModuleLaunchKernel.
template <typename... Args>
int launch(const char* name, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t block, uint32_t shared_bytes,
           hipStream_t stream, Args... args) {
    hipFunction_t fn;
    int rc = kernel(name, &fn);
    if (rc) return rc;
    stream = resolve_stream(stream);
    void* ptrs[] = {(void*) &args...};
    if (gx == 0 || gy == 0 || gz == 0) return 0;
    if (gy > 65535u || gz > 65535u) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "%s: grid y/z too large", name);
    return check(hipModuleLaunchKernel(fn, gx, gy, gz, block, 1, 1, shared_bytes, stream, ptrs, nullptr), name);
}

} // namespace docc::rt::rocm
