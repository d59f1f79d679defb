/*
 * docc_rocm_target.h - C ABI of the `rocm` target library (libdocc_rocm_target.so):
 * SDFG (de)serialisation, scheduling for the rocm target, host-code generation
 * and the compile/link driver.
 *
 * It exposes, over plain strings, the steps the reference's Python driver
 * performs on a `StructuredSDFG` through its pybind11 module
 * (python/bindings/py_structured_sdfg.cpp:124-560: validate, schedule(target),
 * _compile; python/bindings/bindings.cpp:136-160,483-487) and is what a
 * `register_target_overrides("rocm", schedule_fn, compile_fn)` hook
 * (python/docc/python/target_registry.py:4-42) calls into.
 *
 * SDFGs travel as JSON text. Functions returning `char*` return a
 * malloc'ed NUL-terminated string that the caller releases with
 * docc_rocm_target_free, or NULL on failure with the message available from
 * docc_rocm_target_last_error() on the calling thread.
 */
#ifndef DOCC_ROCM_TARGET_H
#define DOCC_ROCM_TARGET_H

#ifdef __cplusplus
extern "C" {
#endif

/* Registers the rocm plugin's serializers and dispatchers (idempotent). Counterpart of
 * register_cuda_plugin() (reference opt/include/sdfg/targets/cuda/plugin.h:20-105) being called
 * from the module initialiser (python/bindings/bindings.cpp:51-60). Returns 0. */
int docc_rocm_target_register(void);

/* JSON array of the registered "<code>::<implementation type>" dispatcher keys. */
char* docc_rocm_target_dispatcher_keys(void);

/* JSON array of the target mapper factories in plugins::TargetMapperRegistry, highest priority first:
 * [{"target": "rocm", "priority": 100}, ...] (reference sdfg/include/sdfg/plugins/target_mapping.h:24-37). */
char* docc_rocm_target_mappers(void);

/* Parses and validates an SDFG; returns its canonical JSON. Counterpart of
 * StructuredSDFG.parse + validate (reference bindings.cpp:136-160). */
char* docc_rocm_target_validate(const char* sdfg_json);

/* Reads an SDFG in docc's own JSON format - what StructuredSDFG.dump / JSONSerializer::serialize
 * write (reference sdfg/src/serializer/json_serializer.cpp:56-353, python/bindings/py_structured_sdfg.cpp:263-292) -
 * and returns it in this library's format. Accepted: a root sequence of blocks with one library node
 * each (GEMM and the ml:: nodes of this target, with their access and constant nodes), Malloc / Free
 * nodes and managed storage for temporaries, a final return. Anything else (loop nests, tasklets,
 * branches, views) is an error that names the element. Every other entry point of this header accepts
 * both formats. */
char* docc_rocm_target_import(const char* docc_json);

/* The reverse: an SDFG of this library in docc's JSON format (blocks with library / access /
 * constant nodes and edges, transitions, a closing return node, element ids renumbered). */
char* docc_rocm_target_export(const char* sdfg_json);

/* Runs the rocm scheduling passes (node mapping, offloading, transfer minimisation) and
 * returns the scheduled SDFG. `options_json` may be NULL or an object with
 * "offload": "function" | "node" | "none", "require_all_mapped": bool, "fuse": bool (fold
 * Broadcast and unary elementwise nodes into their neighbours, default true) and "match_softmax": bool
 * (replace softmax written out as Max, Sub, Exp, Sum, Div nodes by one ml::Softmax, default true).
 * Counterpart of PyStructuredSDFG::schedule (reference py_structured_sdfg.cpp:320-347). */
char* docc_rocm_target_schedule(const char* sdfg_json, const char* category, const char* options_json);

/* Generates <output_dir>/<name>.h and <name>.cpp and returns a JSON report:
 * {"header": path, "source": path, "function": definition, "instrumentation": [...]}.
 * `instrumentation_mode`: NULL or "" for none, "ols" to bracket every rocm node and transfer with
 * the `__daisy_instrumentation_*` calls (include/docc_rocm_rtl.h); any other value is the error
 * "Unsupported instrumentation plan: <mode>".
 * Counterpart of CPPCodeGenerator::generate + as_source (reference py_structured_sdfg.cpp:355-420). */
char* docc_rocm_target_generate(const char* sdfg_json, const char* output_dir, const char* instrumentation_mode);

/* generate + compile + link into <output_dir>/lib<name>.so against `runtime_lib_dir`/libdocc_rt_rocm.so
 * with headers from `include_dir`; returns the library path. The compiler is
 * $DOCC_CXX, else ROCm's clang++, invoked through std::system like the reference's JIT step
 * (py_structured_sdfg.cpp:456,485,516-551: -c -fPIC -O3 -march=native -mtune=native -funroll-loops, then -shared).
 * An instrumented library also links `runtime_lib_dir`/libdocc_rtl_rocm.so. */
char* docc_rocm_target_compile(const char* sdfg_json, const char* output_dir, const char* include_dir,
                               const char* runtime_lib_dir, const char* instrumentation_mode);

/* JSON object counting the library nodes per "<code>::<implementation type>" plus transfers,
 * the analogue of loop_report() (reference py_structured_sdfg.cpp:570-583). */
char* docc_rocm_target_report(const char* sdfg_json);

void docc_rocm_target_free(char* text);
const char* docc_rocm_target_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* DOCC_ROCM_TARGET_H */
