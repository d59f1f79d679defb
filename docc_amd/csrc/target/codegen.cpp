#include "codegen.h"

#include <map>

#include <algorithm>
#include <fstream>

namespace sdfg::codegen {

void PrettyPrinter::write(const std::string& s) {
    for (char c : s) {
        if (c == '\n') {
            out_ << '\n';
            at_line_start_ = true;
            continue;
        }
        if (at_line_start_) {
            out_ << std::string((size_t) indent_, ' ');
            at_line_start_ = false;
        }
        out_ << c;
    }
}

std::string CPPLanguageExtension::primitive_type(types::PrimitiveType t) const {
    using P = types::PrimitiveType;
    switch (t) {
        case P::Void: return "void";
        case P::Bool: return "bool";
        case P::Int8: return "int8_t";
        case P::Int16: return "int16_t";
        case P::Int32: return "int32_t";
        case P::Int64: return "int64_t";
        case P::UInt8: return "uint8_t";
        case P::UInt16: return "uint16_t";
        case P::UInt32: return "uint32_t";
        case P::UInt64: return "uint64_t";
        case P::Half: return "_Float16";
        case P::BFloat: return "__bf16";
        case P::Float: return "float";
        case P::Double: return "double";
    }
    return "void";
}

std::string CPPLanguageExtension::declaration(const std::string& name, const Container& c) const {
    std::string s = primitive_type(c.element);
    s += c.is_pointer ? " *" : " ";
    return s + name;
}

CodeSnippet& CodeSnippetFactory::require(const std::string& name, const std::string& extension, bool as_file) {
    auto it = snippets_.find(name);
    if (it != snippets_.end()) {
        if (it->second.extension() != extension)
            throw std::runtime_error("Code snippet " + name + " already exists with extension " + it->second.extension());
        return it->second;
    }
    return snippets_.emplace(name, CodeSnippet(extension, as_file)).first->second;
}

void LibraryNodeDispatcher::dispatch(PrettyPrinter& stream, PrettyPrinter& globals_stream,
                                     CodeSnippetFactory& library_snippet_factory) {
    // A connector's local hides a container of the same name for the rest of the scope (and `T *X = X;` reads the
    // local itself). The reference's connectors are spelled `__A`, `_in`, ... and never meet a container; the tensor
    // nodes' are `X`, `Y`, `A`, `B`, `C`, which a user's arrays may be called too. Where a connector of this node and
    // a container bound to it share a name, the containers are first copied under names nothing else uses.
    bool clash = false;
    auto bound = [&](const std::string& name) {
        for (auto& in : data_flow_graph_.inputs)
            if (!in.is_constant && in.data == name) return true;
        for (auto& out : data_flow_graph_.outputs)
            if (out.data == name) return true;
        return false;
    };
    for (auto& in : data_flow_graph_.inputs) clash = clash || bound(in.connector);
    for (auto& out : data_flow_graph_.outputs) clash = clash || bound(out.connector);

    stream << "{" << std::endl;
    stream.setIndent(stream.indent() + 4);
    std::map<std::string, std::string> alias;   // connector -> the name its container's value is read from / written to
    if (clash) {
        size_t k = 0;
        auto capture = [&](const std::string& connector, const std::string& data) {
            const std::string name = "__docc_bound_" + std::to_string(k++);
            stream << language_extension_.declaration(name, function_.container(data)) << " = " << data << ";" << std::endl;
            alias[connector] = name;
        };
        for (auto& in : data_flow_graph_.inputs)
            if (!in.is_constant) capture(in.connector, in.data);
        for (auto& out : data_flow_graph_.outputs)
            if (!data_flow_graph_.input(out.connector)) capture(out.connector, out.data);
        stream << "{" << std::endl;
        stream.setIndent(stream.indent() + 4);
    }
    auto source_of = [&](const std::string& connector, const std::string& data) {
        auto it = alias.find(connector);
        return it == alias.end() ? data : it->second;
    };

    // one local per input connector: container value or constant literal
    for (auto& in : data_flow_graph_.inputs) {
        if (in.is_constant) {
            stream << language_extension_.primitive_type(in.type) << " " << in.connector << " = " << in.data << ";" << std::endl;
        } else {
            const Container& c = function_.container(in.data);
            stream << language_extension_.declaration(in.connector, c) << " = " << source_of(in.connector, in.data) << ";" << std::endl;
        }
    }
    // outputs that are not inputs as well get a local too
    for (auto& out : data_flow_graph_.outputs) {
        if (data_flow_graph_.input(out.connector)) continue;
        const Container& c = function_.container(out.data);
        stream << language_extension_.declaration(out.connector, c) << " = " << source_of(out.connector, out.data) << ";" << std::endl;
    }
    stream << std::endl;

    this->dispatch_code(stream, globals_stream, library_snippet_factory);

    stream << std::endl;
    if (clash) {
        // out of the connectors' scope first, then into the containers
        for (auto& out : data_flow_graph_.outputs)
            if (alias.count(out.connector)) stream << alias[out.connector] << " = " << out.connector << ";" << std::endl;
        stream.setIndent(stream.indent() - 4);
        stream << "}" << std::endl;
        for (auto& out : data_flow_graph_.outputs)
            if (alias.count(out.connector)) stream << out.data << " = " << alias[out.connector] << ";" << std::endl;
    } else {
        for (auto& out : data_flow_graph_.outputs) stream << out.data << " = " << out.connector << ";" << std::endl;
    }

    stream.setIndent(stream.indent() - 4);
    stream << "}" << std::endl;
}

InstrumentationInfo LibraryNodeDispatcher::instrumentation_info() const {
    // reference block_dispatcher.cpp:440-442: element id, "unknown", SEQUENTIAL
    InstrumentationInfo info;
    info.element_id = node_.element_id();
    info.region_name = node_.code();
    const Expression flop = node_.flop();
    if (!flop.empty()) info.metrics["flop"] = flop;
    return info;
}

// ------------------------------------------------------------------ instrumentation plan

namespace {
std::string c_string(const std::string& s) {
    std::string out = "\"";
    for (char c : s) {
        if (c == '"' || c == '\\') out += '\\';
        if (c == '\n') {
            out += "\\n";
            continue;
        }
        out += c;
    }
    return out + "\"";
}

std::string metadata_or_empty(const StructuredSDFG& sdfg, const char* key) {
    auto it = sdfg.metadata().find(key);
    return it == sdfg.metadata().end() ? "" : it->second;
}
} // namespace

void InstrumentationPlan::begin_instrumentation(const structured_control_flow::Block& block, PrettyPrinter& stream,
                                                const InstrumentationInfo& info) const {
    const std::string stem = sdfg_.name() + "_" + std::to_string(block.node->element_id());
    const std::string md = stem + "_md", id = stem + "_id";
    const auto& dbg = block.debug_info;
    stream << "__daisy_metadata_t " << md << ";" << std::endl;
    stream << md << ".file_name = " << c_string(dbg.filename) << ";" << std::endl;
    stream << md << ".function_name = " << c_string(dbg.function) << ";" << std::endl;
    stream << md << ".line_begin = " << dbg.start_line << ";" << std::endl;
    stream << md << ".line_end = " << dbg.end_line << ";" << std::endl;
    stream << md << ".column_begin = " << dbg.start_column << ";" << std::endl;
    stream << md << ".column_end = " << dbg.end_column << ";" << std::endl;
    stream << md << ".sdfg_name = " << c_string(sdfg_.name()) << ";" << std::endl;
    stream << md << ".sdfg_file = " << c_string(metadata_or_empty(sdfg_, "sdfg_file")) << ";" << std::endl;
    stream << md << ".arg_capture_path = " << c_string(metadata_or_empty(sdfg_, "arg_capture_path")) << ";" << std::endl;
    stream << md << ".features_file = " << c_string(metadata_or_empty(sdfg_, "features_file")) << ";" << std::endl;
    stream << md << ".opt_report_file = " << c_string(metadata_or_empty(sdfg_, "opt_report_file")) << ";" << std::endl;
    stream << md << ".element_id = " << info.element_id << ";" << std::endl;
    stream << md << ".element_type = " << c_string(info.element_type) << ";" << std::endl;
    stream << md << ".target_type = " << c_string(info.target_type) << ";" << std::endl;
    const LoopInfo& li = info.loop_info;
    stream << md << ".loopnest_index = " << li.loopnest_index << ";" << std::endl;
    stream << md << ".num_loops = " << li.num_loops << ";" << std::endl;
    stream << md << ".num_maps = " << li.num_maps << ";" << std::endl;
    stream << md << ".num_fors = " << li.num_fors << ";" << std::endl;
    stream << md << ".num_whiles = " << li.num_whiles << ";" << std::endl;
    stream << md << ".max_depth = " << li.max_depth << ";" << std::endl;
    stream << md << ".is_perfectly_nested = " << (li.is_perfectly_nested ? "1" : "0") << ";" << std::endl;
    stream << md << ".is_perfectly_parallel = " << (li.is_perfectly_parallel ? "1" : "0") << ";" << std::endl;
    stream << md << ".is_elementwise = " << (li.is_elementwise ? "1" : "0") << ";" << std::endl;
    stream << md << ".has_side_effects = " << (li.has_side_effects ? "1" : "0") << ";" << std::endl;
    stream << md << ".region_uuid = " << c_string(stem) << ";" << std::endl;
    const char* set = "__DAISY_EVENT_SET_NONE";
    switch (nodes_.at(block.node->element_id())) {
        case InstrumentationEventType::CPU: set = "__DAISY_EVENT_SET_CPU"; break;
        case InstrumentationEventType::ROCM: set = "__DAISY_EVENT_SET_ROCM"; break;
        case InstrumentationEventType::NONE: break;
    }
    stream << "long long " << id << " = __daisy_instrumentation_init(&" << md << ", " << set << ");" << std::endl;
    stream << "__daisy_instrumentation_enter(" << id << ");" << std::endl;
}

void InstrumentationPlan::end_instrumentation(const structured_control_flow::Block& block, PrettyPrinter& stream,
                                              const InstrumentationInfo& info) const {
    const std::string id = sdfg_.name() + "_" + std::to_string(block.node->element_id()) + "_id";
    stream << "__daisy_instrumentation_exit(" << id << ");" << std::endl;
    for (auto& entry : info.metrics)
        stream << "__daisy_instrumentation_metric(" << id << ", \"" << entry.first << "\", " << entry.second << ");" << std::endl;
    stream << "__daisy_instrumentation_finalize(" << id << ");" << std::endl;
}

std::unique_ptr<InstrumentationPlan> InstrumentationPlan::none(const StructuredSDFG& sdfg) {
    return std::make_unique<InstrumentationPlan>(sdfg, std::map<size_t, InstrumentationEventType>{});
}

std::unique_ptr<InstrumentationPlan> InstrumentationPlan::outermost_loops_plan(const StructuredSDFG& sdfg) {
    std::map<size_t, InstrumentationEventType> nodes;
    for (auto& blk : sdfg.blocks()) {
        const std::string& impl = blk.node->implementation_type();
        const auto* offloading = dynamic_cast<const rocm::ROCMDataOffloadingNode*>(blk.node.get());
        const bool transfer = offloading && (offloading->is_h2d() || offloading->is_d2h());
        if ((!offloading && impl.rfind("ROCM", 0) == 0) || transfer) nodes[blk.node->element_id()] = InstrumentationEventType::ROCM;
    }
    return std::make_unique<InstrumentationPlan>(sdfg, std::move(nodes));
}

std::unique_ptr<InstrumentationPlan> InstrumentationPlan::from_mode(const StructuredSDFG& sdfg, const std::string& mode) {
    if (mode.empty()) return none(sdfg);
    if (mode == "ols") return outermost_loops_plan(sdfg);
    throw std::runtime_error("Unsupported instrumentation plan: " + mode);
}

LibraryNodeDispatcherRegistry& LibraryNodeDispatcherRegistry::instance() {
    static LibraryNodeDispatcherRegistry registry;
    return registry;
}

void LibraryNodeDispatcherRegistry::register_library_node_dispatcher(const std::string& key, LibraryNodeDispatcherFn fn) {
    std::lock_guard<std::mutex> lock(mutex_);
    factories_.emplace(key, std::move(fn));
}

LibraryNodeDispatcherFn LibraryNodeDispatcherRegistry::get_library_node_dispatcher(const std::string& key) const {
    auto it = factories_.find(key);
    return it == factories_.end() ? nullptr : it->second;
}

std::vector<std::string> LibraryNodeDispatcherRegistry::keys() const {
    std::lock_guard<std::mutex> lock(mutex_);
    std::vector<std::string> out;
    for (auto& kv : factories_) out.push_back(kv.first);
    std::sort(out.begin(), out.end());
    return out;
}

CPPCodeGenerator::CPPCodeGenerator(StructuredSDFG& sdfg, std::shared_ptr<CodeSnippetFactory> library_snippet_factory,
                                   std::string externals_prefix, const InstrumentationPlan* instrumentation_plan)
    : sdfg_(sdfg), library_snippet_factory_(library_snippet_factory ? std::move(library_snippet_factory)
                                                                     : std::make_shared<CodeSnippetFactory>()),
      externals_prefix_(std::move(externals_prefix)), instrumentation_plan_(instrumentation_plan) {}

std::string CPPCodeGenerator::function_definition() {
    std::vector<std::string> args;
    for (auto& name : sdfg_.arguments()) args.push_back(language_extension_.declaration(name, sdfg_.container(name)));
    std::string arglist;
    for (size_t i = 0; i < args.size(); i++) arglist += (i ? ", " : "") + args[i];
    if (arglist.empty()) arglist = "void";
    std::string ret = "void ";
    if (!sdfg_.return_container().empty()) ret = language_extension_.declaration("", sdfg_.container(sdfg_.return_container()));
    return "extern \"C\" " + ret + externals_prefix_ + sdfg_.name() + "(" + arglist + ")";
}

void CPPCodeGenerator::dispatch_includes() {
    includes_stream_ << "#include <cmath>" << std::endl;
    includes_stream_ << "#include <cstdio>" << std::endl;
    includes_stream_ << "#include <cstdlib>" << std::endl;
    includes_stream_ << "#include <cstring>" << std::endl;
    includes_stream_ << "#include <cstdint>" << std::endl;
    // the reference includes <daisy_rtl/daisy_rtl.h> here; this header declares the same protocol
    if (instrumentation_plan_ && !instrumentation_plan_->empty()) includes_stream_ << "#include \"docc_rocm_rtl.h\"" << std::endl;
}

void CPPCodeGenerator::dispatch_schedule() {
    main_stream_.setIndent(4);
    // transients are declared at the top of the function (reference cpp_code_generator.cpp:156-224)
    for (auto& kv : sdfg_.containers()) {
        const Container& c = kv.second;
        if (c.is_argument) continue;
        main_stream_ << language_extension_.declaration(c.name, c);
        if (c.is_pointer) main_stream_ << " = nullptr";
        main_stream_ << ";" << std::endl;
    }
    // host transients are managed allocations of the function
    for (auto& kv : sdfg_.containers()) {
        const Container& c = kv.second;
        if (c.is_argument || !c.transient || !c.is_pointer || c.storage != "CPU" || c.size_bytes.empty()) continue;
        main_stream_ << c.name << " = (" << language_extension_.primitive_type(c.element) << " *) malloc(" << c.size_bytes
                     << ");" << std::endl;
    }
    auto& registry = LibraryNodeDispatcherRegistry::instance();
    for (auto& blk : sdfg_.blocks()) {
        const std::string key = blk.node->code() + "::" + blk.node->implementation_type();
        auto factory = registry.get_library_node_dispatcher(key);
        if (!factory) throw std::runtime_error("No library node dispatcher found for library node code: " + key);
        auto dispatcher = factory(language_extension_, sdfg_, blk, *blk.node);
        // brackets as in the reference's DataFlowDispatcher::dispatch_library_node (block_dispatcher.cpp:305-319)
        const bool instrument = instrumentation_plan_ && instrumentation_plan_->should_instrument(*blk.node);
        const InstrumentationInfo info = dispatcher->instrumentation_info();
        if (instrument) instrumentation_plan_->begin_instrumentation(blk, main_stream_, info);
        dispatcher->dispatch(main_stream_, globals_stream_, *library_snippet_factory_);
        if (instrument) instrumentation_plan_->end_instrumentation(blk, main_stream_, info);
        instrumentation_.push_back(info);
    }
    for (auto& kv : sdfg_.containers()) {
        const Container& c = kv.second;
        if (c.is_argument || !c.transient || !c.is_pointer || c.storage != "CPU" || c.size_bytes.empty()) continue;
        if (c.name == sdfg_.return_container()) continue;  // ownership passes to the caller
        main_stream_ << "free(" << c.name << ");" << std::endl;
    }
    if (!sdfg_.return_container().empty()) main_stream_ << "return " << sdfg_.return_container() << ";" << std::endl;
}

bool CPPCodeGenerator::generate() {
    dispatch_includes();
    dispatch_schedule();
    return true;
}

std::string CPPCodeGenerator::header_text() const {
    return "#pragma once\n" + includes_stream_.str() + "\n" + classes_stream_.str() + "\n";
}

std::string CPPCodeGenerator::source_text(const std::string& header_name) {
    std::ostringstream src;
    src << "#include \"" << header_name << "\"\n";
    // the same include may be requested by several dispatchers: keep the first of each line
    {
        std::istringstream lines(globals_stream_.str());
        std::vector<std::string> seen;
        std::string line;
        while (std::getline(lines, line)) {
            if (line.rfind("#include", 0) == 0) {
                if (std::find(seen.begin(), seen.end(), line) != seen.end()) continue;
                seen.push_back(line);
            }
            src << line << "\n";
        }
    }
    src << "\n" << function_definition() << "\n{\n";
    auto init_once = library_snippet_factory_->find(CODE_SNIPPET_INIT_ONCE);
    if (init_once != library_snippet_factory_->snippets().end()) src << init_once->second.stream().str() << "\n";
    src << main_stream_.str() << "\n";
    auto deinit_once = library_snippet_factory_->find(CODE_SNIPPET_DEINIT_ONCE);
    if (deinit_once != library_snippet_factory_->snippets().end()) src << deinit_once->second.stream().str() << "\n";
    src << "}\n";
    return src.str();
}

bool CPPCodeGenerator::as_source(const std::filesystem::path& header_path, const std::filesystem::path& source_path) {
    std::ofstream header(header_path, std::ofstream::out | std::ofstream::trunc);
    if (!header.is_open()) return false;
    std::ofstream source(source_path, std::ofstream::out | std::ofstream::trunc);
    if (!source.is_open()) return false;
    header << header_text();
    source << source_text(header_path.filename().string());
    return true;
}

} // namespace sdfg::codegen

namespace sdfg::plugins {

TargetMapperRegistry& TargetMapperRegistry::instance() {
    static TargetMapperRegistry registry;
    return registry;
}

const std::vector<std::shared_ptr<TargetMapperFactory>> TargetMapperRegistry::get_all_mappers() {
    std::lock_guard<std::mutex> lock(mutex_);
    return factories_;
}

void TargetMapperRegistry::register_target_mapper(std::shared_ptr<TargetMapperFactory> factory) {
    if (!factory) return;
    std::lock_guard<std::mutex> lock(mutex_);
    // highest priority first; equal priorities in the order they were registered
    const int p = factory->priority();
    auto it = factories_.begin();
    while (it != factories_.end() && (*it)->priority() >= p) ++it;
    factories_.insert(it, std::move(factory));
}

std::vector<std::shared_ptr<TargetMapper>> TargetMapperRegistry::create_for_target(const std::string& target) {
    std::vector<std::shared_ptr<TargetMapper>> mappers;
    for (auto& f : get_all_mappers())
        if (f->for_target() == target) mappers.push_back(f->create());
    return mappers;
}

} // namespace sdfg::plugins

namespace sdfg::passes {

bool TargetMappingPass::run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager) {
    bool applied = false;
    for (auto& blk : builder.subject().blocks()) {
        for (const auto& mapper : target_mappers_) {
            if (mapper->try_map(builder, analysis_manager, *blk.node)) {
                applied = true;
                break;  // the first mapper that accepts the node wins
            }
        }
    }
    return applied;
}

} // namespace sdfg::passes
