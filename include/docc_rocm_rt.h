/*
 * docc_rocm_rt.h - thin C-ABI HIP runtime of the docc `rocm` target.
 *
 * This is the only door through which generated host C++ reaches the GPU:
 * module load, device memory, asynchronous copies, kernel launch, stream
 * synchronisation and an error string. It plays the role that
 * docc::rt::et::EtRuntimeWrapper plays for the ET-SoC target
 * (reference targets/et/rt/include/docc/rt/et/et.h:9-30, used by the
 * dispatcher at targets/et/src/et/blas/gemm.cpp:137-204) and that the raw
 * cudaMalloc/cudaMemcpy/cudaFree calls play for the CUDA target
 * (reference opt/src/targets/cuda/cuda_data_offloading_node.cpp:139-173,
 * opt/src/targets/cuda/blas/gemm.cpp:66-96).
 *
 * Conventions
 *   - every function returns 0 on success and a non-zero HIP error code (or
 *     a negative docc code, see below) on failure; the message is available
 *     from docc_rocm_last_error() on the calling thread;
 *   - plain pointers and sizes only; `stream` is a hipStream_t passed as
 *     void* (NULL = the device's default stream);
 *   - one process-wide state per device, created by docc_rocm_init() or
 *     lazily by the first call; thread-safe.
 *
 * Library: libdocc_rt_rocm.so. The gfx950 code objects that hold the math
 * kernels (docc_rocm_<family>.hsaco, one per kernel family) are looked up next
 * to the library; the
 * environment variable DOCC_ROCM_KERNEL_PATH overrides the directory, in the
 * way DOCC_ET_KERNEL_PATH does for the ET target
 * (reference targets/et/rt/src/runtime.cpp:129-143).
 */
#ifndef DOCC_ROCM_RT_H
#define DOCC_ROCM_RT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* negative codes are docc's own, positive ones are hipError_t values */
#define DOCC_ROCM_OK 0
#define DOCC_ROCM_ERR_INVALID_ARGUMENT (-1)
#define DOCC_ROCM_ERR_UNSUPPORTED (-2)
#define DOCC_ROCM_ERR_KERNEL_IMAGE (-3) /* code object missing or not loadable */
#define DOCC_ROCM_ERR_NO_DEVICE (-4)

typedef void* docc_rocm_module_t;   /* hipModule_t   */
typedef void* docc_rocm_function_t; /* hipFunction_t */
typedef void* docc_rocm_stream_t;   /* hipStream_t   */

/* Selects `device` for the calling thread, creates its state and loads the
 * math-kernel code object. Replaces EtRuntimeWrapper::get_instance() +
 * get_device(idx) (reference et.h:16-20). Idempotent. */
int docc_rocm_init(int device);

/* Number of visible HIP devices, or 0. Does not create any state. */
int docc_rocm_device_count(void);

/* Name (gcnArchName) and compute-unit count of the current device. */
int docc_rocm_device_info(char* arch, size_t arch_len, int* compute_units, int* clock_khz);

/* Loads a gfx950 code object from a file. Replaces
 * EtRuntimeWrapper::load_kernel_binary_blocking (reference et.h:22-23). */
int docc_rocm_module_load(const char* path, docc_rocm_module_t* module);
int docc_rocm_module_unload(docc_rocm_module_t module);
int docc_rocm_module_get_function(docc_rocm_module_t module, const char* name, docc_rocm_function_t* function);

/* Device memory. Replace cudaMalloc / cudaFree of the CUDA offloading node
 * (reference cuda_data_offloading_node.cpp:150-170). */
int docc_rocm_malloc(void** dev_ptr, size_t bytes);
int docc_rocm_free(void* dev_ptr);
/* docc_rocm_free waits for the device (as hipFree does) and keeps the block for the next
 * docc_rocm_malloc of the same size, rounded up to 256 bytes: a compiled function allocates the
 * same buffers on every call. The cache holds at most DOCC_ROCM_POOL_BYTES bytes (default 4 GiB,
 * 0 = every call goes to hipMalloc / hipFree) and is emptied when hipMalloc runs out of memory.
 * No counterpart in the reference, whose CUDA nodes call cudaMalloc / cudaFree each time. */
/* Stream-ordered forms, what generated code calls: docc_rocm_free_async does not wait; it records, on `stream`,
 * the point behind which the block's last use lies (the caller must have issued every use of the block on
 * `stream`, or have ordered `stream` behind them), and the block goes to the cache at once. The next
 * docc_rocm_malloc_async on the same stream gets it without any wait, on another stream after that stream has
 * been made to wait for the recorded point (hipStreamWaitEvent; the new owner must then start using the
 * block on the stream it named), and a plain docc_rocm_malloc after the host has waited for it. A compiled
 * function that frees its buffers and is called again therefore never waits for the device on their account.
 * The counterpart in CUDA terms is cudaMallocAsync / cudaFreeAsync; the reference's nodes use the blocking pair. */
int docc_rocm_malloc_async(void** dev_ptr, size_t bytes, docc_rocm_stream_t stream);
int docc_rocm_free_async(void* dev_ptr, docc_rocm_stream_t stream);
int docc_rocm_pool_trim(void);
int docc_rocm_pool_stats(size_t* cached_bytes, size_t* cached_blocks, size_t* limit_bytes);
int docc_rocm_pool_set_limit(size_t limit_bytes);
int docc_rocm_memset_async(void* dev_ptr, int value, size_t bytes, docc_rocm_stream_t stream);

/* Pinned host memory (hipHostMalloc) for callers that want truly
 * asynchronous copies. */
int docc_rocm_host_malloc(void** host_ptr, size_t bytes);
int docc_rocm_host_free(void* host_ptr);

/* Copies on a stream. Replace the blocking cudaMemcpy H2D/D2H of the CUDA
 * offloading node (reference cuda_data_offloading_node.cpp:153-166); the
 * caller orders them with docc_rocm_stream_sync. An upload of 16 MiB or more
 * from memory that docc_rocm_host_malloc did not return is staged through
 * pinned chunks of the runtime (helper threads, DOCC_ROCM_H2D_THREADS): the
 * source has been read when the call returns, as with hipMemcpyAsync from
 * pageable memory. */
int docc_rocm_memcpy_h2d_async(void* dst_dev, const void* src_host, size_t bytes, docc_rocm_stream_t stream);
int docc_rocm_memcpy_d2h_async(void* dst_host, const void* src_dev, size_t bytes, docc_rocm_stream_t stream);
int docc_rocm_memcpy_d2d_async(void* dst_dev, const void* src_dev, size_t bytes, docc_rocm_stream_t stream);

/* Streams (default priority only). docc_rocm_stream_destroy also releases the 8 MiB of partial results that
 * the two-launch kernels (sliced softmax, column reductions, column matrix-vector products, dot) keep per
 * stream; they allocate it with hipMalloc on their first call on a stream, so that first call waits for the
 * device: run a function once on a stream before capturing it there. */
int docc_rocm_stream_create(docc_rocm_stream_t* stream);
int docc_rocm_stream_destroy(docc_rocm_stream_t stream);
int docc_rocm_stream_sync(docc_rocm_stream_t stream);
int docc_rocm_device_sync(void);

/* Launches `function` with an array of pointers to its arguments, as
 * hipModuleLaunchKernel takes them. Replaces the `<<<grid, block>>>` launch
 * the CUDA map dispatcher prints (reference
 * opt/src/targets/cuda/codegen/cuda_map_dispatcher.cpp:236-262). */
int docc_rocm_launch(docc_rocm_function_t function, const uint32_t grid[3], const uint32_t block[3],
                     uint32_t shared_bytes, docc_rocm_stream_t stream, void** args);

/* Events, for timing on the stream the kernels run on. */
typedef void* docc_rocm_event_t;
int docc_rocm_event_create(docc_rocm_event_t* event);
int docc_rocm_event_destroy(docc_rocm_event_t event);
int docc_rocm_event_record(docc_rocm_event_t event, docc_rocm_stream_t stream);
int docc_rocm_event_elapsed_ms(docc_rocm_event_t start, docc_rocm_event_t stop, float* ms);

/*
 * Graph capture of generated code. A compiled function is a fixed chain of launches, copies and (cached)
 * allocations on the null stream; a caller that runs it many times on the same buffers records it once and replays
 * the record, which costs one submission instead of one per kernel. No counterpart in the reference: its CUDA
 * target launches kernel by kernel and synchronizes after each (reference
 * opt/src/targets/cuda/codegen/cuda_map_dispatcher.cpp:236-262).
 *
 * docc_rocm_set_default_stream names, for the calling thread, the stream that stands in wherever generated code or
 * a caller passes the null stream to this library (kernels, copies, allocations, docc_rocm_stream_sync); null
 * restores the null stream. docc_rocm_graph_capture_begin waits for the device, starts a relaxed-mode capture on
 * `stream` (not null) and makes it the thread's default stream; every call of this library on that thread up to
 * docc_rocm_graph_capture_end is recorded instead of run. During a capture
 *   - docc_rocm_malloc[_async] hands out blocks that then belong to the graph (every replay uses those addresses);
 *     docc_rocm_free[_async] returns them to the capture, which serves its own later allocations from them, and
 *     neither waits for anything. The blocks go back to the block cache in docc_rocm_graph_destroy;
 *   - calls that hand a result to the host refuse (docc_rocm_dot) or end the capture with an error from HIP
 *     (docc_rocm_stream_sync, docc_rocm_device_sync, docc_rocm_event_elapsed_ms): a function that copies results
 *     to host memory and waits for them is captured up to that wait at most. Capture functions whose arguments
 *     stay on the device;
 *   - copies from or to host memory need pinned memory (docc_rocm_host_malloc) and are replayed from / to the
 *     same addresses.
 * Run the function once on `stream` (docc_rocm_set_default_stream) before capturing it, so that kernel images
 * are loaded and the per-stream partial results exist. Kernels that keep partial results (see Streams above)
 * record the capture stream's buffer: replay on that stream, or keep it idle while a replay runs elsewhere.
 * docc_rocm_graph_launch enqueues one replay on `stream` (null: the thread's default). docc_rocm_graph_destroy
 * waits for the device. The library records no memset nodes.
 */
typedef void* docc_rocm_graph_t;
int docc_rocm_set_default_stream(docc_rocm_stream_t stream);
int docc_rocm_graph_capture_begin(docc_rocm_stream_t stream);
int docc_rocm_graph_capture_end(docc_rocm_graph_t* graph);
int docc_rocm_graph_launch(docc_rocm_graph_t graph, docc_rocm_stream_t stream);
int docc_rocm_graph_destroy(docc_rocm_graph_t graph);

/*
 * Failure channel of generated code. The generated `extern "C"` functions have
 * no error return (reference calling convention: sdfg/src/codegen/code_generators/cpp_code_generator.cpp:8-24),
 * so a failing runtime call is reported here and the generated function
 * returns early. With DOCC_ROCM_DEBUG set in the environment the report is
 * printed and the process exits, which is what the reference's CUDA target
 * does under DOCC_CUDA_DEBUG (opt/src/targets/cuda/cuda.cpp:62-91); otherwise
 * the failure is kept until the caller collects it with
 * docc_rocm_take_failure (returns the code, 0 if none, and clears it).
 */
void docc_rocm_report_failure(const char* function, const char* call, int code);
int docc_rocm_take_failure(char* message, size_t message_len);

/* Message of the last failure on this thread ("" if none). */
const char* docc_rocm_last_error(void);

/* Library version string, e.g. "docc-rocm 0.1 (gfx950)". */
const char* docc_rocm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* DOCC_ROCM_RT_H */
