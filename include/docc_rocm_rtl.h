/*
 * docc_rocm_rtl.h - the instrumentation protocol of docc's generated code, with a ROCm
 * event set.
 *
 * Generated code brackets a region with
 *     __daisy_metadata_t md; md.<field> = ...;
 *     long long id = __daisy_instrumentation_init(&md, <event set>);
 *     __daisy_instrumentation_enter(id);  ...region...  __daisy_instrumentation_exit(id);
 *     __daisy_instrumentation_metric(id, "flop", <value>);   (one per metric)
 *     __daisy_instrumentation_finalize(id);
 * (reference sdfg/src/codegen/instrumentation/instrumentation_plan.cpp:22-141). The types and
 * functions below are those of the reference's rtl/include/daisy_rtl/daisy_rtl.h:11-75 - same
 * names, fields and order - plus the event set __DAISY_EVENT_SET_ROCM. The argument-capture
 * half of that header (`__daisy_capture_*`) is not part of the rocm target.
 *
 * Library: libdocc_rtl_rocm.so (docc_amd/csrc/rtl/instrumentation.cpp). What it does per
 * event set:
 *   CPU, CUDA  wall-clock time of the region (no PAPI counters here)
 *   ROCM       the region is bracketed on the device's null stream: enter and exit record a
 *              HIP event each and return; the duration is the time between the two events,
 *              read when the trace is written (no host wait inside instrumented code: the
 *              stream runs on as it does without instrumentation); without a GPU it degrades
 *              to wall-clock time. While a region is
 *              open a roctx range named after its region_uuid is pushed (when
 *              librocprofiler-sdk-roctx.so or libroctx64.so can be loaded), so that rocprofv3 --marker-trace shows the regions.
 *   NONE       metrics only
 * At process exit the regions are written as a Chrome trace ({"traceEvents":[...]}) in the
 * layout of the reference's runtime (rtl/src/instrumentation.cpp:173-456), to the file named by
 * __DAISY_INSTRUMENTATION_FILE (default daisy_trace.json); __DAISY_INSTRUMENTATION_MODE=aggregate
 * writes one event per region with mean / variance / count / min / max instead of one per
 * execution. Metrics appear with the "static:::" prefix.
 */
#ifndef DOCC_ROCM_RTL_H
#define DOCC_ROCM_RTL_H

#include <stdbool.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum __daisy_event_set {
    __DAISY_EVENT_SET_CPU = 0,
    __DAISY_EVENT_SET_CUDA = 1,
    __DAISY_EVENT_SET_NONE = 2,
    __DAISY_EVENT_SET_ROCM = 3, /* added by the rocm target */
};

typedef struct __daisy_metadata {
    /* source location */
    const char* file_name;
    const char* function_name;
    long line_begin;
    long line_end;
    long column_begin;
    long column_end;

    /* SDFG scope */
    const char* sdfg_name;
    const char* sdfg_file;
    const char* arg_capture_path;
    const char* features_file;
    const char* opt_report_file;

    /* element scope */
    size_t element_id;
    const char* element_type;
    const char* target_type;

    /* loop information */
    int loopnest_index;
    size_t num_loops;
    size_t num_maps;
    size_t num_fors;
    size_t num_whiles;
    size_t max_depth;
    bool is_perfectly_nested;
    bool is_perfectly_parallel;
    bool is_elementwise;
    bool has_side_effects;

    const char* region_uuid;
} __daisy_metadata_t;

/* Registers a region (or finds the one with the same region_uuid) and returns its id. The
 * strings are copied: the metadata may live on the caller's stack. */
size_t __daisy_instrumentation_init(__daisy_metadata_t* metadata, enum __daisy_event_set event_set);
void __daisy_instrumentation_finalize(size_t region_id);
void __daisy_instrumentation_enter(size_t region_id);
void __daisy_instrumentation_exit(size_t region_id);
/* Named per-region values, aggregated over the executions of the region. */
void __daisy_instrumentation_increment(size_t region_id, const char* name, long long value);
void __daisy_instrumentation_metric(size_t region_id, const char* name, double value);

/* Writes the trace file now (it is also written at process exit). No counterpart in the
 * reference: for hosts that unload the library or never exit normally. Returns 0 or -1. */
int docc_rocm_rtl_flush(void);

#ifdef __cplusplus
}
#endif
#endif /* DOCC_ROCM_RTL_H */
