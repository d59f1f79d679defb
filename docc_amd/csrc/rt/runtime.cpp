// Thin C-ABI HIP runtime of the docc `rocm` target (see include/docc_rocm_rt.h).
//
// Structural counterpart of docc::rt::et::EtRuntimeWrapper (reference
// targets/et/rt/src/runtime.cpp:55-176): a process-wide singleton per device
// that owns the loaded kernel image, with the image located next to the
// library unless an environment variable points elsewhere
// (reference runtime.cpp:129-143).
#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <condition_variable>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

#include "rt_state.h"

namespace docc::rt::rocm {

namespace {

thread_local std::string g_last_error;

// One gfx950 code object per kernel family; all of them must be present.
const char* const kKernelImages[] = {
    "docc_rocm_util.hsaco",
    "docc_rocm_softmax.hsaco",
    "docc_rocm_gemm_f32.hsaco",
    "docc_rocm_gemm_f64.hsaco",
    "docc_rocm_gemm_bf16.hsaco",
    "docc_rocm_gemm_bf16_async.hsaco",
    "docc_rocm_gemm_bf16_async_big.hsaco",
    "docc_rocm_gemm_f32_epilogue.hsaco",
    "docc_rocm_gemm_f64_epilogue.hsaco",
    "docc_rocm_gemm_bf16_epilogue.hsaco",
    "docc_rocm_gemm_bf16_async_epilogue.hsaco",
    "docc_rocm_gemm_bf16_async_big_epilogue.hsaco",
    "docc_rocm_gemm_f32_big.hsaco",
    "docc_rocm_gemm_f32_big_epilogue.hsaco",
    "docc_rocm_conv2d.hsaco",
    "docc_rocm_attention.hsaco",
    "docc_rocm_elementwise.hsaco",
    "docc_rocm_reduce.hsaco",
    "docc_rocm_transpose.hsaco",
    "docc_rocm_gemv.hsaco",
    "docc_rocm_gemm_skinny.hsaco",
};

struct DeviceState {
    bool ready = false;          // kernel images loaded
    bool noalloc_ready = false;  // set-up of docc_rocm_softmax_noalloc done
    std::vector<hipModule_t> modules;
    int compute_units = 0;
    std::unordered_map<std::string, hipFunction_t> functions;
};

std::mutex g_mutex;
std::vector<DeviceState> g_devices;

// Device blocks that docc_rocm_free keeps for the next docc_rocm_malloc of the same (rounded) size: generated
// code allocates and frees the same buffers on every call of a compiled function, and hipMalloc / hipFree
// cost more than a small kernel. Keyed by (device, bytes); `live` remembers the size of what is handed out.
//
// A cached block carries the point in a stream behind which its last owner's work is over: docc_rocm_free_async
// records an event on the stream the owner worked on instead of waiting for the device, and the next owner either
// continues on that same stream (stream order keeps it behind the old work), makes its own stream wait for the event
// (docc_rocm_malloc_async), or waits for it on the host (docc_rocm_malloc). docc_rocm_free has waited for the whole
// device and leaves `pending` false.
struct CachedBlock {
    void* ptr = nullptr;
    hipEvent_t released = nullptr;   // created the first time the block is freed on a stream, reused afterwards
    hipStream_t stream = nullptr;    // the stream `released` was recorded on
    bool pending = false;            // `released` may not have happened yet
};

struct BlockCache {
    std::mutex mutex;
    std::multimap<std::pair<int, size_t>, CachedBlock> free_blocks;
    struct Live {
        int device;
        size_t bytes;
        hipEvent_t released;         // travels with the block so that it is created once
    };
    std::unordered_map<void*, Live> live;
    size_t cached_bytes = 0;
    size_t limit = 0;   // bytes the cache may hold; 0 switches it off
};

BlockCache& block_cache() {
    static BlockCache* cache = [] {
        auto* c = new BlockCache();   // never destroyed: blocks may be freed during process exit
        c->limit = size_t(4) << 30;
        if (const char* e = std::getenv("DOCC_ROCM_POOL_BYTES")) c->limit = (size_t) std::strtoull(e, nullptr, 10);
        return c;
    }();
    return *cache;
}

// A graph capture in progress on the calling thread. Device memory that the captured code takes from the block cache
// belongs to the graph from then on (every replay writes to those addresses): blocks "freed" during the capture go to
// a list of the capture's own, from which later allocations of the same capture are served (the captured work is one
// chain in stream order, so a block's next user starts after its last one), and all of them return to the cache when
// the graph is destroyed.
struct Capture {
    hipStream_t stream = nullptr;
    hipStream_t previous_default = nullptr;
    std::vector<std::pair<void*, size_t>> blocks;          // every block the capture holds
    std::multimap<size_t, void*> free_blocks;              // those not in use at this point of the capture
};

struct Graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<std::pair<void*, size_t>> blocks;
};

std::mutex g_failure_mutex;
int g_failure_code = 0;
std::string g_failure_message;

std::string kernel_image_dir() {
    const char* env = std::getenv("DOCC_ROCM_KERNEL_PATH");
    std::string dir;
    if (env && *env) {
        dir = env;
    } else {
        Dl_info info;
        if (dladdr((void*) &kernel_image_dir, &info) && info.dli_fname) {
            dir = info.dli_fname;
            auto pos = dir.find_last_of('/');
            dir = (pos == std::string::npos) ? "." : dir.substr(0, pos);
        } else {
            dir = ".";
        }
    }
    return dir;
}

} // namespace

namespace {
// What the calling thread has set with docc_rocm_set_default_stream, and the capture it has open (if any).
thread_local hipStream_t t_default_stream = nullptr;
thread_local Capture* t_capture = nullptr;
} // namespace

hipStream_t resolve_stream(hipStream_t stream) { return stream ? stream : t_default_stream; }

bool capturing() { return t_capture != nullptr; }

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int check(hipError_t err, const char* what) {
    if (err == hipSuccess) return 0;
    return fail((int) err, "%s: %s (%s)", what, hipGetErrorString(err), hipGetErrorName(err));
}

int noalloc_setup_device(int dev);   // noalloc.hip

namespace {
int load_device_images(int dev);
}

int ensure_device() {
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return fail(DOCC_ROCM_ERR_NO_DEVICE, "no HIP device: %s", hipGetErrorString(err));
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if ((size_t) dev < g_devices.size() && g_devices[dev].ready && g_devices[dev].noalloc_ready) return 0;
    }
    if (int rc = load_device_images(dev)) return rc;
    // the entry point that allocates nothing gets its array's address and its kernels now (outside the lock:
    // the kernel lookups take it)
    if (int rc = noalloc_setup_device(dev)) return rc;
    std::lock_guard<std::mutex> lock(g_mutex);
    g_devices[dev].noalloc_ready = true;
    return 0;
}

namespace {
int load_device_images(int dev) {
    hipError_t err;
    std::lock_guard<std::mutex> lock(g_mutex);
    if ((size_t) dev >= g_devices.size()) g_devices.resize(dev + 1);
    DeviceState& st = g_devices[dev];
    if (st.ready) return 0;
    hipDeviceProp_t prop;
    int rc = check(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties");
    if (rc) return rc;
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(DOCC_ROCM_ERR_UNSUPPORTED, "device %d is %s; the rocm target is built for gfx950 only", dev,
                    prop.gcnArchName);
    st.compute_units = prop.multiProcessorCount;
    std::string dir = kernel_image_dir();
    std::vector<hipModule_t> modules;
    for (const char* image : kKernelImages) {
        std::string path = dir + "/" + image;
        hipModule_t m;
        err = hipModuleLoad(&m, path.c_str());
        if (err != hipSuccess) {
            for (hipModule_t loaded : modules) (void) hipModuleUnload(loaded);
            return fail(DOCC_ROCM_ERR_KERNEL_IMAGE, "cannot load kernel image %s: %s", path.c_str(),
                        hipGetErrorString(err));
        }
        modules.push_back(m);
    }
    st.modules = std::move(modules);
    st.ready = true;
    return 0;
}
} // namespace

int kernel(const char* name, hipFunction_t* fn) {
    int dev = 0;
    (void) hipGetDevice(&dev);
    {
        // not ensure_device(): the device's own set-up looks kernels up before it is complete
        std::lock_guard<std::mutex> lock(g_mutex);
        if ((size_t) dev >= g_devices.size() || !g_devices[dev].ready) dev = -1;
    }
    if (dev < 0) {
        int rc = ensure_device();
        if (rc) return rc;
        (void) hipGetDevice(&dev);
    }
    std::lock_guard<std::mutex> lock(g_mutex);
    DeviceState& st = g_devices[dev];
    auto it = st.functions.find(name);
    if (it != st.functions.end()) {
        *fn = it->second;
        return 0;
    }
    hipFunction_t f = nullptr;
    hipError_t err = hipErrorNotFound;
    for (hipModule_t m : st.modules) {
        err = hipModuleGetFunction(&f, m, name);
        if (err == hipSuccess) break;
    }
    // a miss in one image leaves HIP's per-thread "last error" set; clear it so
    // that other users of the HIP runtime in this process do not pick it up
    (void) hipGetLastError();
    if (err != hipSuccess)
        return fail(DOCC_ROCM_ERR_KERNEL_IMAGE, "kernel %s not in any kernel image: %s", name, hipGetErrorString(err));
    st.functions.emplace(name, f);
    *fn = f;
    return 0;
}

namespace {
struct PartialsSlot {
    void* ptr = nullptr;
    std::mutex busy;
};
std::mutex g_partials_mutex;
// never destroyed: the slots' mutexes may be held while the process exits
std::map<std::pair<int, hipStream_t>, PartialsSlot*>& partials_slots() {
    static auto* slots = new std::map<std::pair<int, hipStream_t>, PartialsSlot*>();
    return *slots;
}
} // namespace

int partials_for(hipStream_t stream, PartialsLease* lease) {
    stream = resolve_stream(stream);
    int dev = 0;
    int rc = check(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    PartialsSlot* slot = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_partials_mutex);
        auto& slots = partials_slots();
        auto it = slots.find({dev, stream});
        if (it == slots.end()) it = slots.emplace(std::make_pair(dev, stream), new PartialsSlot()).first;
        slot = it->second;
    }
    std::unique_lock<std::mutex> busy(slot->busy);
    if (!slot->ptr) {
        rc = check(hipMalloc(&slot->ptr, kPartialsBytes), "hipMalloc (partial results)");
        if (rc) {
            slot->ptr = nullptr;
            return rc;
        }
    }
    lease->ptr = slot->ptr;
    lease->lock = std::move(busy);
    return 0;
}

// The stream goes away: its partial-results buffers (one per device it was used on) go with it. A launcher still
// running on the stream from another thread would be the caller's error, as with hipStreamDestroy itself.
void release_partials(hipStream_t stream) {
    std::vector<PartialsSlot*> gone;
    {
        std::lock_guard<std::mutex> lock(g_partials_mutex);
        auto& slots = partials_slots();
        for (auto it = slots.begin(); it != slots.end();)
            if (it->first.second == stream) {
                gone.push_back(it->second);
                it = slots.erase(it);
            } else {
                ++it;
            }
    }
    for (PartialsSlot* slot : gone) {
        {
            std::lock_guard<std::mutex> busy(slot->busy);
            if (slot->ptr) (void) hipFree(slot->ptr);   // waits for the kernels that still use it
            slot->ptr = nullptr;
        }
        delete slot;
    }
}

int compute_units() {
    int dev = 0;
    (void) hipGetDevice(&dev);
    std::lock_guard<std::mutex> lock(g_mutex);
    if ((size_t) dev >= g_devices.size()) return 0;
    return g_devices[dev].compute_units;
}

} // namespace docc::rt::rocm

using namespace docc::rt::rocm;

// ---- uploads from pageable memory ---------------------------------------------------------------------------
// hipMemcpyAsync from memory the driver has not pinned goes through the driver's own staging at about 30 GB/s on
// these machines; from pinned memory the same bytes move at 57 GB/s. The caller's arrays (numpy's) are pageable, so a
// large upload is staged here instead: helper threads copy the source into a ring of pinned chunks while the chunks
// already filled travel over PCIe. The call returns when the last chunk has been handed to the stream, i.e. after the
// source has been read completely (what hipMemcpyAsync guarantees for pageable memory as well).
// DOCC_ROCM_H2D_THREADS=<n> sets the number of copying threads (default 4; 0 switches the staging off).
namespace {

constexpr size_t kStageMin = size_t(16) << 20;     // smaller uploads go straight to the driver (no gain measured below)
constexpr size_t kStageChunk = size_t(8) << 20;
constexpr int kStageBuffers = 4;

std::mutex g_pinned_mutex;
std::map<uintptr_t, size_t> g_pinned;   // blocks from docc_rocm_host_malloc: start -> bytes

void note_pinned(void* p, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    g_pinned[(uintptr_t) p] = bytes;
}

void forget_pinned(void* p) {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    g_pinned.erase((uintptr_t) p);
}

bool is_pinned(const void* p, size_t bytes) {
    {
        std::lock_guard<std::mutex> lock(g_pinned_mutex);
        auto it = g_pinned.upper_bound((uintptr_t) p);
        if (it != g_pinned.begin()) {
            --it;
            if ((uintptr_t) p + bytes <= it->first + it->second) return true;
        }
    }
    // memory the caller pinned itself (hipHostMalloc, torch's pin_memory): the driver knows it. A pointer it has
    // never seen makes the query fail, which is the answer "pageable"; the error it leaves is cleared.
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void) hipGetLastError();
        return false;
    }
    return attr.type == hipMemoryTypeHost;
}

// A fixed pool of threads that copy slices of one chunk; never torn down (the threads sleep on a condition variable
// until the process ends).
class CopyPool {
public:
    explicit CopyPool(int threads) {
        for (int i = 0; i < threads; i++) std::thread([this] { work(); }).detach();
    }
    // copies `bytes` from src to dst with every thread of the pool and the caller
    void copy(char* dst, const char* src, size_t bytes, int parts) {
        const size_t slice = ((bytes + (size_t) parts - 1) / (size_t) parts + 4095) & ~size_t(4095);
        size_t first = slice < bytes ? slice : bytes;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            for (size_t off = first; off < bytes; off += slice) {
                jobs_.push_back({dst + off, src + off, off + slice <= bytes ? slice : bytes - off});
                pending_++;
            }
        }
        wake_.notify_all();
        std::memcpy(dst, src, first);
        std::unique_lock<std::mutex> lock(mutex_);
        done_.wait(lock, [this] { return pending_ == 0; });
    }

private:
    struct Job {
        char* dst;
        const char* src;
        size_t bytes;
    };
    void work() {
        for (;;) {
            Job job;
            {
                std::unique_lock<std::mutex> lock(mutex_);
                wake_.wait(lock, [this] { return !jobs_.empty(); });
                job = jobs_.back();
                jobs_.pop_back();
            }
            std::memcpy(job.dst, job.src, job.bytes);
            {
                std::lock_guard<std::mutex> lock(mutex_);
                pending_--;
            }
            done_.notify_all();
        }
    }
    std::mutex mutex_;
    std::condition_variable wake_, done_;
    std::vector<Job> jobs_;
    size_t pending_ = 0;
};

struct Stager {
    std::mutex mutex;              // one staged upload at a time
    bool tried = false, ready = false;
    int threads = 0;
    char* buffer[kStageBuffers] = {};
    hipEvent_t sent[kStageBuffers] = {};
    bool in_flight[kStageBuffers] = {};
    CopyPool* pool = nullptr;
};
Stager g_stager;

// 0: done, 1: not staged (the caller falls back to the plain copy), other: error
int staged_h2d(void* dst_dev, const void* src_host, size_t bytes, hipStream_t stream) {
    Stager& st = g_stager;
    std::lock_guard<std::mutex> lock(st.mutex);
    if (!st.tried) {
        st.tried = true;
        int threads = 4;
        if (const char* e = std::getenv("DOCC_ROCM_H2D_THREADS")) threads = std::atoi(e);
        if (threads > 64) threads = 64;
        if (threads >= 1) {
            bool ok = true;
            for (int i = 0; i < kStageBuffers && ok; i++)
                ok = hipHostMalloc((void**) &st.buffer[i], kStageChunk, hipHostMallocDefault) == hipSuccess &&
                     hipEventCreateWithFlags(&st.sent[i], hipEventDisableTiming) == hipSuccess;
            if (ok) {
                st.threads = threads;
                st.pool = new CopyPool(threads - 1);
                st.ready = true;
            } else {
                (void) hipGetLastError();
            }
        }
    }
    if (!st.ready) return 1;
    const char* src = (const char*) src_host;
    char* dst = (char*) dst_dev;
    int slot = 0;
    for (size_t off = 0; off < bytes; off += kStageChunk, slot = (slot + 1) % kStageBuffers) {
        const size_t n = bytes - off < kStageChunk ? bytes - off : kStageChunk;
        if (st.in_flight[slot]) {
            int rc = check(hipEventSynchronize(st.sent[slot]), "hipEventSynchronize(H2D staging)");
            if (rc) return rc;
            st.in_flight[slot] = false;
        }
        st.pool->copy(st.buffer[slot], src + off, n, st.threads);
        int rc = check(hipMemcpyAsync(dst + off, st.buffer[slot], n, hipMemcpyHostToDevice, stream), "hipMemcpyAsync(H2D, staged)");
        if (rc) return rc;
        rc = check(hipEventRecord(st.sent[slot], stream), "hipEventRecord(H2D staging)");
        if (rc) return rc;
        st.in_flight[slot] = true;
    }
    return 0;
}

} // namespace

extern "C" {

int docc_rocm_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int docc_rocm_init(int device) {
    int n = docc_rocm_device_count();
    if (n <= 0) return fail(DOCC_ROCM_ERR_NO_DEVICE, "no HIP device visible");
    if (device < 0 || device >= n) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "device %d out of range [0,%d)", device, n);
    int rc = check(hipSetDevice(device), "hipSetDevice");
    if (rc) return rc;
    return ensure_device();
}

int docc_rocm_device_info(char* arch, size_t arch_len, int* compute_units_out, int* clock_khz) {
    int dev = 0;
    int rc = check(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    hipDeviceProp_t prop;
    rc = check(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties");
    if (rc) return rc;
    if (arch && arch_len) {
        std::strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (compute_units_out) *compute_units_out = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    return 0;
}

int docc_rocm_module_load(const char* path, docc_rocm_module_t* module) {
    if (!path || !module) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "module_load: null argument");
    hipModule_t m;
    hipError_t err = hipModuleLoad(&m, path);
    if (err != hipSuccess) {
        (void) hipGetLastError();   // reported here; other users of the HIP runtime in this process must not pick it up
        return fail(DOCC_ROCM_ERR_KERNEL_IMAGE, "cannot load %s: %s", path, hipGetErrorString(err));
    }
    *module = m;
    return 0;
}

int docc_rocm_module_unload(docc_rocm_module_t module) {
    return check(hipModuleUnload((hipModule_t) module), "hipModuleUnload");
}

int docc_rocm_module_get_function(docc_rocm_module_t module, const char* name, docc_rocm_function_t* function) {
    if (!module || !name || !function) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "get_function: null argument");
    hipFunction_t f;
    hipError_t err = hipModuleGetFunction(&f, (hipModule_t) module, name);
    if (err != hipSuccess) {
        (void) hipGetLastError();
        return fail(DOCC_ROCM_ERR_KERNEL_IMAGE, "kernel %s not found: %s", name, hipGetErrorString(err));
    }
    *function = f;
    return 0;
}

namespace {

// `stream` matters only if `ordered`: then a block whose release is still pending is handed out behind that release
// in `stream`'s own order; otherwise the host waits for the release.
int pool_malloc(void** dev_ptr, size_t bytes, bool ordered, hipStream_t stream) {
    if (!dev_ptr) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "malloc: null argument");
    *dev_ptr = nullptr;
    if (bytes == 0) return 0;
    BlockCache& c = block_cache();
    if (c.limit == 0) return check(hipMalloc(dev_ptr, bytes), "hipMalloc");
    const size_t rounded = (bytes + 255) & ~size_t(255);
    int dev = 0;
    int rc = check(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    stream = resolve_stream(stream);
    Capture* capture = t_capture;
    if (capture) {
        // a block of the capture's own first; from the cache only one that needs no wait (no event may be waited for
        // or recorded while the stream is being captured)
        auto mine = capture->free_blocks.find(rounded);
        if (mine != capture->free_blocks.end()) {
            *dev_ptr = mine->second;
            capture->free_blocks.erase(mine);
            return 0;
        }
        ordered = true;
        stream = capture->stream;
    }
    CachedBlock got;
    {
        std::lock_guard<std::mutex> lock(c.mutex);
        auto range = c.free_blocks.equal_range({dev, rounded});
        auto pick = capture ? range.second : range.first;
        // prefer a block that needs no wait: released on this very stream, or not pending at all
        for (auto it = range.first; it != range.second; ++it)
            if (!it->second.pending || (!capture && ordered && it->second.stream == stream)) {
                pick = it;
                break;
            }
        if (pick != range.second) {
            got = pick->second;
            c.cached_bytes -= rounded;
            c.free_blocks.erase(pick);
            c.live[got.ptr] = {dev, rounded, got.released};
        }
    }
    if (got.ptr) {
        if (got.pending && !(ordered && got.stream == stream)) {
            rc = ordered ? check(hipStreamWaitEvent(stream, got.released, 0), "hipStreamWaitEvent(block release)")
                         : check(hipEventSynchronize(got.released), "hipEventSynchronize(block release)");
            if (rc) return rc;   // the block stays in `live`; its owner-to-be never sees it
        }
        *dev_ptr = got.ptr;
        if (capture) capture->blocks.push_back({got.ptr, rounded});
        return 0;
    }
    hipError_t e = hipMalloc(dev_ptr, rounded);
    if (e == hipErrorOutOfMemory) {   // give the cached blocks back and try once more
        (void) hipGetLastError();
        docc_rocm_pool_trim();
        e = hipMalloc(dev_ptr, rounded);
    }
    rc = check(e, "hipMalloc");
    if (rc) return rc;
    std::lock_guard<std::mutex> lock(c.mutex);
    c.live[*dev_ptr] = {dev, rounded, nullptr};
    if (capture) capture->blocks.push_back({*dev_ptr, rounded});
    return 0;
}

int pool_free(void* dev_ptr, bool ordered, hipStream_t stream) {
    if (!dev_ptr) return 0;
    BlockCache& c = block_cache();
    stream = resolve_stream(stream);
    if (Capture* capture = t_capture) {
        // the block stays with the capture (and later with its graph); a block from before the capture joins it
        size_t bytes = 0;
        for (auto& b : capture->blocks)
            if (b.first == dev_ptr) bytes = b.second;
        if (bytes == 0) {
            std::lock_guard<std::mutex> lock(c.mutex);
            auto it = c.live.find(dev_ptr);
            if (it == c.live.end()) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "free during a graph capture: not a block of this runtime");
            bytes = it->second.bytes;
            capture->blocks.push_back({dev_ptr, bytes});
        }
        capture->free_blocks.insert({bytes, dev_ptr});
        return 0;
    }
    BlockCache::Live info{0, 0, nullptr};
    bool keep = false;
    {
        std::lock_guard<std::mutex> lock(c.mutex);
        auto it = c.live.find(dev_ptr);
        if (it != c.live.end()) {
            info = it->second;
            c.live.erase(it);
            keep = c.limit > 0 && info.bytes <= c.limit - (c.cached_bytes < c.limit ? c.cached_bytes : c.limit);
        }
    }
    if (!keep) {
        if (info.released) (void) hipEventDestroy(info.released);
        return check(hipFree(dev_ptr), "hipFree");   // waits for the device itself
    }
    CachedBlock blk;
    blk.ptr = dev_ptr;
    blk.released = info.released;
    int rc = 0;
    if (ordered) {
        if (!blk.released) rc = check(hipEventCreateWithFlags(&blk.released, hipEventDisableTiming), "hipEventCreate(block release)");
        if (!rc) rc = check(hipEventRecord(blk.released, stream), "hipEventRecord(block release)");
        blk.stream = stream;
        blk.pending = true;
    } else {
        // hipFree waits for the device before it releases memory; a block that stays allocated must do the same
        // before another caller can get it
        rc = check(hipDeviceSynchronize(), "hipDeviceSynchronize");
    }
    if (rc) {
        if (blk.released) (void) hipEventDestroy(blk.released);
        (void) hipFree(dev_ptr);
        return rc;
    }
    std::lock_guard<std::mutex> lock(c.mutex);
    c.free_blocks.insert({{info.device, info.bytes}, blk});
    c.cached_bytes += info.bytes;
    return 0;
}

} // namespace

int docc_rocm_malloc(void** dev_ptr, size_t bytes) { return pool_malloc(dev_ptr, bytes, false, nullptr); }

int docc_rocm_malloc_async(void** dev_ptr, size_t bytes, docc_rocm_stream_t stream) {
    return pool_malloc(dev_ptr, bytes, true, (hipStream_t) stream);
}

int docc_rocm_free(void* dev_ptr) { return pool_free(dev_ptr, false, nullptr); }

int docc_rocm_free_async(void* dev_ptr, docc_rocm_stream_t stream) { return pool_free(dev_ptr, true, (hipStream_t) stream); }

int docc_rocm_pool_trim(void) {
    BlockCache& c = block_cache();
    std::multimap<std::pair<int, size_t>, CachedBlock> blocks;
    {
        std::lock_guard<std::mutex> lock(c.mutex);
        blocks.swap(c.free_blocks);
        c.cached_bytes = 0;
    }
    int rc = 0;
    for (auto& b : blocks) {
        // hipFree waits for the device, which covers a release that is still pending
        const int r = check(hipFree(b.second.ptr), "hipFree");
        if (b.second.released) (void) hipEventDestroy(b.second.released);
        if (r && !rc) rc = r;
    }
    return rc;
}

int docc_rocm_pool_stats(size_t* cached_bytes, size_t* cached_blocks, size_t* limit_bytes) {
    BlockCache& c = block_cache();
    std::lock_guard<std::mutex> lock(c.mutex);
    if (cached_bytes) *cached_bytes = c.cached_bytes;
    if (cached_blocks) *cached_blocks = c.free_blocks.size();
    if (limit_bytes) *limit_bytes = c.limit;
    return 0;
}

int docc_rocm_pool_set_limit(size_t limit_bytes) {
    BlockCache& c = block_cache();
    {
        std::lock_guard<std::mutex> lock(c.mutex);
        c.limit = limit_bytes;
    }
    size_t cached = 0;
    docc_rocm_pool_stats(&cached, nullptr, nullptr);
    return cached > limit_bytes ? docc_rocm_pool_trim() : 0;
}

int docc_rocm_memset_async(void* dev_ptr, int value, size_t bytes, docc_rocm_stream_t stream) {
    if (bytes == 0) return 0;
    if (capturing()) {
        // a kernel instead of a memset node in the graph
        long groups = (long) ((bytes / 16 + 1023) / 1024);
        if (groups < 1) groups = 1;
        if (groups > 4096) groups = 4096;
        return launch("docc_fill_b8", (uint32_t) groups, 1, 1, 256, 0, (hipStream_t) stream, dev_ptr, value, (long) bytes);
    }
    return check(hipMemsetAsync(dev_ptr, value, bytes, resolve_stream((hipStream_t) stream)), "hipMemsetAsync");
}

int docc_rocm_host_malloc(void** host_ptr, size_t bytes) {
    if (!host_ptr) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "host_malloc: null argument");
    *host_ptr = nullptr;
    if (bytes == 0) return 0;
    const int rc = check(hipHostMalloc(host_ptr, bytes, hipHostMallocDefault), "hipHostMalloc");
    if (rc == 0) note_pinned(*host_ptr, bytes);
    return rc;
}

int docc_rocm_host_free(void* host_ptr) {
    if (!host_ptr) return 0;
    forget_pinned(host_ptr);
    return check(hipHostFree(host_ptr), "hipHostFree");
}

int docc_rocm_memcpy_h2d_async(void* dst_dev, const void* src_host, size_t bytes, docc_rocm_stream_t stream) {
    if (bytes == 0) return 0;
    if (bytes >= kStageMin && !capturing() && !is_pinned(src_host, bytes)) {
        const int rc = staged_h2d(dst_dev, src_host, bytes, resolve_stream((hipStream_t) stream));
        if (rc != 1) return rc;     // 1: staging is switched off or could not be set up
    }
    return check(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, resolve_stream((hipStream_t) stream)), "hipMemcpyAsync(H2D)");
}

int docc_rocm_memcpy_d2h_async(void* dst_host, const void* src_dev, size_t bytes, docc_rocm_stream_t stream) {
    if (bytes == 0) return 0;
    return check(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, resolve_stream((hipStream_t) stream)), "hipMemcpyAsync(D2H)");
}

int docc_rocm_memcpy_d2d_async(void* dst_dev, const void* src_dev, size_t bytes, docc_rocm_stream_t stream) {
    if (bytes == 0) return 0;
    return check(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, resolve_stream((hipStream_t) stream)), "hipMemcpyAsync(D2D)");
}

int docc_rocm_stream_create(docc_rocm_stream_t* stream) {
    if (!stream) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "stream_create: null argument");
    hipStream_t s;
    int rc = check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
    if (rc) return rc;
    *stream = s;
    return 0;
}

int docc_rocm_stream_destroy(docc_rocm_stream_t stream) {
    if (!stream) return 0;
    if (t_default_stream == (hipStream_t) stream) t_default_stream = nullptr;
    release_partials((hipStream_t) stream);
    return check(hipStreamDestroy((hipStream_t) stream), "hipStreamDestroy");
}

int docc_rocm_stream_sync(docc_rocm_stream_t stream) {
    return check(hipStreamSynchronize(resolve_stream((hipStream_t) stream)), "hipStreamSynchronize");
}

int docc_rocm_device_sync(void) { return check(hipDeviceSynchronize(), "hipDeviceSynchronize"); }

int docc_rocm_launch(docc_rocm_function_t function, const uint32_t grid[3], const uint32_t block[3],
                     uint32_t shared_bytes, docc_rocm_stream_t stream, void** args) {
    if (!function || !grid || !block) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "launch: null argument");
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return 0;
    uint64_t threads = (uint64_t) block[0] * block[1] * block[2];
    if (threads == 0 || threads > 1024) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "launch: block of %llu threads", (unsigned long long) threads);
    return check(hipModuleLaunchKernel((hipFunction_t) function, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                       shared_bytes, resolve_stream((hipStream_t) stream), args, nullptr),
                 "hipModuleLaunchKernel");
}

int docc_rocm_event_create(docc_rocm_event_t* event) {
    if (!event) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "event_create: null argument");
    hipEvent_t e;
    int rc = check(hipEventCreate(&e), "hipEventCreate");
    if (rc) return rc;
    *event = e;
    return 0;
}

int docc_rocm_event_destroy(docc_rocm_event_t event) {
    if (!event) return 0;
    return check(hipEventDestroy((hipEvent_t) event), "hipEventDestroy");
}

int docc_rocm_event_record(docc_rocm_event_t event, docc_rocm_stream_t stream) {
    return check(hipEventRecord((hipEvent_t) event, resolve_stream((hipStream_t) stream)), "hipEventRecord");
}

int docc_rocm_event_elapsed_ms(docc_rocm_event_t start, docc_rocm_event_t stop, float* ms) {
    if (!ms) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "event_elapsed: null argument");
    int rc = check(hipEventSynchronize((hipEvent_t) stop), "hipEventSynchronize");
    if (rc) return rc;
    return check(hipEventElapsedTime(ms, (hipEvent_t) start, (hipEvent_t) stop), "hipEventElapsedTime");
}

int docc_rocm_set_default_stream(docc_rocm_stream_t stream) {
    if (t_capture) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "set_default_stream: a graph capture is open on this thread");
    t_default_stream = (hipStream_t) stream;
    return 0;
}

int docc_rocm_graph_capture_begin(docc_rocm_stream_t stream) {
    if (!stream) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "graph_capture_begin: the null stream cannot be captured; create one");
    if (t_capture) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "graph_capture_begin: a capture is already open on this thread");
    int rc = ensure_device();
    if (rc) return rc;
    // Everything released so far is over once the device has been waited for, so every cached block can be handed
    // out during the capture without a wait (which a capturing stream could not record).
    rc = check(hipDeviceSynchronize(), "hipDeviceSynchronize");
    if (rc) return rc;
    {
        BlockCache& c = block_cache();
        std::lock_guard<std::mutex> lock(c.mutex);
        for (auto& b : c.free_blocks) b.second.pending = false;
    }
    // relaxed: the block cache may still have to call hipMalloc for a size it has not seen
    rc = check(hipStreamBeginCapture((hipStream_t) stream, hipStreamCaptureModeRelaxed), "hipStreamBeginCapture");
    if (rc) return rc;
    auto* capture = new Capture();
    capture->stream = (hipStream_t) stream;
    capture->previous_default = t_default_stream;
    t_default_stream = (hipStream_t) stream;
    t_capture = capture;
    return 0;
}

namespace {
// the blocks go back to the cache, free for anybody: the device has finished with them
void return_blocks(const std::vector<std::pair<void*, size_t>>& blocks) {
    if (blocks.empty()) return;
    (void) hipDeviceSynchronize();
    BlockCache& c = block_cache();
    int dev = 0;
    (void) hipGetDevice(&dev);
    for (auto& b : blocks) {
        hipEvent_t released = nullptr;
        bool keep = false;
        {
            std::lock_guard<std::mutex> lock(c.mutex);
            auto it = c.live.find(b.first);
            if (it != c.live.end()) {
                released = it->second.released;
                dev = it->second.device;
                c.live.erase(it);
            }
            keep = c.limit > 0 && b.second <= c.limit - (c.cached_bytes < c.limit ? c.cached_bytes : c.limit);
            if (keep) {
                CachedBlock blk;
                blk.ptr = b.first;
                blk.released = released;
                c.free_blocks.insert({{dev, b.second}, blk});
                c.cached_bytes += b.second;
            }
        }
        if (!keep) {
            if (released) (void) hipEventDestroy(released);
            (void) hipFree(b.first);
        }
    }
}
} // namespace

int docc_rocm_graph_capture_end(docc_rocm_graph_t* graph) {
    Capture* capture = t_capture;
    if (!capture) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "graph_capture_end: no capture is open on this thread");
    t_capture = nullptr;
    t_default_stream = capture->previous_default;
    auto* g = new Graph();
    g->blocks = std::move(capture->blocks);
    int rc = check(hipStreamEndCapture(capture->stream, &g->graph), "hipStreamEndCapture");
    delete capture;
    if (!rc && !graph) rc = fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "graph_capture_end: null argument");
    if (!rc) rc = check(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    if (rc) {
        if (g->graph) (void) hipGraphDestroy(g->graph);
        return_blocks(g->blocks);
        delete g;
        return rc;
    }
    *graph = g;
    return 0;
}

int docc_rocm_graph_launch(docc_rocm_graph_t graph, docc_rocm_stream_t stream) {
    if (!graph) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "graph_launch: null graph");
    if (t_capture) return fail(DOCC_ROCM_ERR_INVALID_ARGUMENT, "graph_launch: a capture is open on this thread");
    return check(hipGraphLaunch(((Graph*) graph)->exec, resolve_stream((hipStream_t) stream)), "hipGraphLaunch");
}

int docc_rocm_graph_destroy(docc_rocm_graph_t graph) {
    if (!graph) return 0;
    auto* g = (Graph*) graph;
    return_blocks(g->blocks);          // waits for the device first: a replay may still be running
    int rc = check(hipGraphExecDestroy(g->exec), "hipGraphExecDestroy");
    const int rc2 = check(hipGraphDestroy(g->graph), "hipGraphDestroy");
    delete g;
    return rc ? rc : rc2;
}

void docc_rocm_report_failure(const char* function, const char* call, int code) {
    char buf[1024];
    std::snprintf(buf, sizeof(buf), "%s: %s failed with code %d: %s", function ? function : "?", call ? call : "?", code,
                  g_last_error.c_str());
    if (std::getenv("DOCC_ROCM_DEBUG")) {
        std::fprintf(stderr, "docc rocm: %s\n", buf);
        std::exit(EXIT_FAILURE);
    }
    std::lock_guard<std::mutex> lock(g_failure_mutex);
    if (g_failure_code == 0) {  // keep the first failure: later ones are usually consequences
        g_failure_code = code;
        g_failure_message = buf;
    }
}

int docc_rocm_take_failure(char* message, size_t message_len) {
    std::lock_guard<std::mutex> lock(g_failure_mutex);
    const int code = g_failure_code;
    if (message && message_len) {
        std::strncpy(message, g_failure_message.c_str(), message_len - 1);
        message[message_len - 1] = 0;
    }
    g_failure_code = 0;
    g_failure_message.clear();
    return code;
}

const char* docc_rocm_last_error(void) { return g_last_error.c_str(); }

const char* docc_rocm_version(void) { return "docc-rocm 0.1 (gfx950)"; }

} // extern "C"
