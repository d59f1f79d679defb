// C ABI of the rocm target library (include/docc_rocm_target.h).
#include "docc_rocm_target.h"

#include <cstdlib>
#include <cstring>
#include <filesystem>
#include <fstream>

#include "rocm_target.h"

using namespace sdfg;

namespace {

thread_local std::string g_error;

char* dup(const std::string& s) {
    char* out = (char*) std::malloc(s.size() + 1);
    if (out) std::memcpy(out, s.c_str(), s.size() + 1);
    return out;
}

template <typename F>
char* guarded(F&& fn) {
    try {
        g_error.clear();
        return dup(fn());
    } catch (const std::exception& e) {
        g_error = e.what();
        return nullptr;
    }
}

std::unique_ptr<StructuredSDFG> parse(const char* text) {
    if (!text) throw std::invalid_argument("null SDFG text");
    rocm::register_rocm_plugin();
    json::Value j = json::Value::parse(text);
    // SDFGs written by the reference's own serializer are accepted wherever an SDFG is
    if (serializer::is_reference_format(j)) j = serializer::import_reference_json(j);
    auto sdfg = StructuredSDFG::from_json(j);
    sdfg->validate();
    return sdfg;
}

std::string host_compiler() {
    if (const char* cxx = std::getenv("DOCC_CXX"))
        if (*cxx) return cxx;
    const char* rocm = std::getenv("ROCM_PATH");
    std::filesystem::path p = std::filesystem::path(rocm && *rocm ? rocm : "/opt/rocm") / "lib" / "llvm" / "bin" / "clang++";
    if (std::filesystem::exists(p)) return p.string();
    return "c++";
}

struct Generated {
    std::filesystem::path header, source;
    std::string function;
    std::vector<codegen::InstrumentationInfo> instrumentation;
    std::vector<std::filesystem::path> snippet_files;
};

Generated generate(StructuredSDFG& sdfg, const char* output_dir, const char* instrumentation_mode, bool* instrumented = nullptr) {
    if (!output_dir || !*output_dir) throw std::invalid_argument("no output directory");
    std::filesystem::path dir(output_dir);
    std::filesystem::create_directories(dir);
    auto snippets = std::make_shared<codegen::CodeSnippetFactory>(dir);
    auto plan = codegen::InstrumentationPlan::from_mode(sdfg, instrumentation_mode ? instrumentation_mode : "");
    if (instrumented) *instrumented = !plan->empty();
    codegen::CPPCodeGenerator gen(sdfg, snippets, "", plan.get());
    gen.generate();
    Generated g;
    g.header = dir / (sdfg.name() + ".h");
    g.source = dir / (sdfg.name() + ".cpp");
    if (!gen.as_source(g.header, g.source)) throw std::runtime_error("cannot write generated code into " + dir.string());
    for (auto& kv : snippets->snippets()) {
        if (!kv.second.is_as_file()) continue;
        std::filesystem::path p = dir / (kv.first + "." + kv.second.extension());
        std::ofstream f(p, std::ofstream::out | std::ofstream::trunc);
        f << kv.second.stream().str();
        g.snippet_files.push_back(p);
    }
    g.function = gen.function_definition();
    g.instrumentation = gen.instrumentation();
    return g;
}

std::string quote(const std::string& s) { return "'" + s + "'"; }

std::string device_compiler() {
    if (const char* hipcc = std::getenv("DOCC_HIPCC"))
        if (*hipcc) return hipcc;
    const char* rocm = std::getenv("ROCM_PATH");
    return (std::filesystem::path(rocm && *rocm ? rocm : "/opt/rocm") / "bin" / "hipcc").string();
}

// The kernels the map dispatcher wrote ("<kernel>.hip") become code objects next to the library ("<kernel>.hsaco"),
// one compiler process per file, as the reference's driver compiles its ".cu" snippets
// (python/bindings/py_structured_sdfg.cpp:445-466). No contraction of separate statements into fused multiply-adds:
// every tasklet rounds by itself, as in the host code the reference generates. Packed fp32 instructions are switched
// off as for every kernel of this target.
void compile_device_snippets(const Generated& g, const std::filesystem::path& log) {
    for (auto& file : g.snippet_files) {
        if (file.extension() != ".hip") continue;
        std::filesystem::path object = file;
        object.replace_extension(".hsaco");
        const std::string cmd = device_compiler() + " --genco --offload-arch=gfx950 -O3 -std=c++17 -ffp-contract=off "
                                "-Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-command-line-argument " +
                                quote(file.string()) + " -o " + quote(object.string()) + " >> " + quote(log.string()) + " 2>&1";
        if (std::system(cmd.c_str()) != 0) throw std::runtime_error("Compilation failed: " + cmd);
    }
}

} // namespace

extern "C" {

int docc_rocm_target_register(void) {
    rocm::register_rocm_plugin();
    return 0;
}

char* docc_rocm_target_dispatcher_keys(void) {
    return guarded([] {
        rocm::register_rocm_plugin();
        json::Array a;
        for (auto& k : codegen::LibraryNodeDispatcherRegistry::instance().keys()) a.emplace_back(k);
        return json::Value(std::move(a)).dump();
    });
}

char* docc_rocm_target_mappers(void) {
    return guarded([] {
        rocm::register_rocm_plugin();
        json::Array a;
        for (auto& f : plugins::TargetMapperRegistry::instance().get_all_mappers()) {
            json::Value e;
            e.set("target", f->for_target());
            e.set("priority", (int64_t) f->priority());
            a.push_back(std::move(e));
        }
        return json::Value(std::move(a)).dump();
    });
}

char* docc_rocm_target_validate(const char* sdfg_json) {
    return guarded([&] { return parse(sdfg_json)->to_json().dump(2); });
}

char* docc_rocm_target_import(const char* docc_json) {
    return guarded([&] {
        if (!docc_json) throw std::invalid_argument("null SDFG text");
        rocm::register_rocm_plugin();
        json::Value j = json::Value::parse(docc_json);
        if (!serializer::is_reference_format(j)) throw InvalidSDFGException("not in docc's SDFG JSON format (no \"element_counter\")");
        auto sdfg = StructuredSDFG::from_json(serializer::import_reference_json(j));
        sdfg->validate();
        return sdfg->to_json().dump(2);
    });
}

char* docc_rocm_target_export(const char* sdfg_json) {
    return guarded([&] { return serializer::export_reference_json(*parse(sdfg_json)).dump(2); });
}

char* docc_rocm_target_schedule(const char* sdfg_json, const char* category, const char* options_json) {
    return guarded([&] {
        auto sdfg = parse(sdfg_json);
        rocm::ScheduleOptions options;
        if (options_json && *options_json) {
            json::Value o = json::Value::parse(options_json);
            if (const json::Value* v = o.find("offload")) options.offload = v->as_string();
            if (const json::Value* v = o.find("require_all_mapped")) options.require_all_mapped = v->as_bool();
            if (const json::Value* v = o.find("fuse")) options.fuse_elementwise = v->as_bool();
            if (const json::Value* v = o.find("match_softmax")) options.match_softmax = v->as_bool();
            if (const json::Value* v = o.find("fuse_maps")) options.fuse_maps = v->as_bool();
        }
        // merged chains are kernels this machine has to compile: without a device compiler the nodes keep their
        // prebuilt kernels (a program that holds map nests of its own still needs one, and says so when compiled)
        if (options.fuse_maps && device_compiler().find('/') != std::string::npos && !std::filesystem::exists(device_compiler()))
            options.fuse_maps = false;
        builder::StructuredSDFGBuilder builder(*sdfg);
        analysis::AnalysisManager analysis_manager(*sdfg);
        rocm::rocm_scheduling_passes(builder, analysis_manager, category ? category : "server", options);
        sdfg->validate();
        return sdfg->to_json().dump(2);
    });
}

char* docc_rocm_target_generate(const char* sdfg_json, const char* output_dir, const char* instrumentation_mode) {
    return guarded([&] {
        auto sdfg = parse(sdfg_json);
        Generated g = generate(*sdfg, output_dir, instrumentation_mode);
        json::Value report;
        report.set("header", g.header.string());
        report.set("source", g.source.string());
        report.set("function", g.function);
        json::Array regions;
        for (auto& info : g.instrumentation) {
            json::Value r;
            r.set("region", info.region_name);
            r.set("element_id", info.element_id);
            r.set("element_type", info.element_type);
            r.set("target_type", info.target_type);
            json::Value metrics{json::Object{}};
            for (auto& kv : info.metrics) metrics.set(kv.first, kv.second);
            r.set("metrics", std::move(metrics));
            regions.push_back(std::move(r));
        }
        report.set("instrumentation", json::Value(std::move(regions)));
        return report.dump(2);
    });
}

char* docc_rocm_target_compile(const char* sdfg_json, const char* output_dir, const char* include_dir,
                               const char* runtime_lib_dir, const char* instrumentation_mode) {
    return guarded([&] {
        if (!include_dir || !runtime_lib_dir) throw std::invalid_argument("include and runtime library directories are required");
        auto sdfg = parse(sdfg_json);
        bool instrumented = false;
        Generated g = generate(*sdfg, output_dir, instrumentation_mode, &instrumented);
        const std::filesystem::path dir(output_dir);
        const std::string cxx = host_compiler();
        // compile, then link: two compiler processes, as the reference's JIT does
        const std::filesystem::path object = dir / (sdfg->name() + ".o");
        const std::filesystem::path log = dir / "compile.log";
        std::string compile = cxx + " -c -fPIC -O3 -march=native -mtune=native -funroll-loops -std=c++17 -I" + quote(include_dir) +
                              " " + quote(g.source.string()) + " -o " + quote(object.string()) + " > " + quote(log.string()) + " 2>&1";
        if (std::system(compile.c_str()) != 0) throw std::runtime_error("Compilation failed: " + compile);
        compile_device_snippets(g, log);
        const std::filesystem::path lib = dir / ("lib" + sdfg->name() + ".so");
        std::string link = cxx + " -shared " + quote(object.string()) + " -o " + quote(lib.string()) + " -L" + quote(runtime_lib_dir) +
                           (instrumented ? " -ldocc_rtl_rocm" : "") + " -ldocc_rt_rocm -Wl,-rpath," + quote(runtime_lib_dir) + " -lm -lstdc++ >> " + quote(log.string()) + " 2>&1";
        if (std::system(link.c_str()) != 0) throw std::runtime_error("Linking failed: " + link);
        return lib.string();
    });
}

char* docc_rocm_target_report(const char* sdfg_json) {
    return guarded([&] {
        auto sdfg = parse(sdfg_json);
        std::map<std::string, int64_t> counts;
        int64_t h2d = 0, d2h = 0;
        for (auto& blk : sdfg->blocks()) {
            counts[blk.node->code() + "::" + blk.node->implementation_type()]++;
            counts[blk.node->code()]++;
            if (blk.node->code() == rocm::LibraryNodeType_ROCM_Offloading) {
                auto& n = static_cast<const rocm::ROCMDataOffloadingNode&>(*blk.node);
                h2d += n.is_h2d();
                d2h += n.is_d2h();
            }
        }
        json::Value r{json::Object{}};
        for (auto& kv : counts) r.set(kv.first, kv.second);
        r.set("H2D", h2d);
        r.set("D2H", d2h);
        return r.dump();
    });
}

void docc_rocm_target_free(char* text) { std::free(text); }

const char* docc_rocm_target_last_error(void) { return g_error.c_str(); }

} // extern "C"
