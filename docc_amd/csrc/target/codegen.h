// Host-code generation for SDFGs whose blocks hold library nodes: pretty
// printer, C++ language extension, code-snippet factory, the library-node
// dispatcher interface with its "<code>::<implementation type>" registry, and
// the generator that prints `extern "C" <ret> <name>(<arguments>)`.
//
// Interfaces follow the reference's codegen layer:
//   LibraryNodeDispatcher           sdfg/include/sdfg/codegen/dispatchers/block_dispatcher.h:105-172
//   LibraryNodeDispatcherRegistry   sdfg/include/sdfg/codegen/dispatchers/node_dispatcher_registry.h:140-205
//   CodeSnippetFactory              sdfg/include/sdfg/codegen/code_snippet_factory.h:9-53
//   CPPCodeGenerator                sdfg/src/codegen/code_generators/cpp_code_generator.cpp:8-57
//   CStyleBaseCodeGenerator         sdfg/src/codegen/code_generators/c_style_base_code_generator.cpp:28-84
#pragma once

#include <filesystem>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "sdfg_lite.h"

namespace sdfg::codegen {

// An ostream-like printer that indents every new line.
class PrettyPrinter {
public:
    explicit PrettyPrinter(int indent = 0) : indent_(indent) {}
    int indent() const { return indent_; }
    void setIndent(int indent) { indent_ = indent < 0 ? 0 : indent; }
    std::string str() const { return out_.str(); }
    void clear() {
        out_.str("");
        at_line_start_ = true;
    }

    template <typename T>
    PrettyPrinter& operator<<(const T& value) {
        std::ostringstream tmp;
        tmp << value;
        write(tmp.str());
        return *this;
    }
    PrettyPrinter& operator<<(std::ostream& (*manip)(std::ostream&) ) {
        (void) manip;  // std::endl
        out_ << '\n';
        at_line_start_ = true;
        return *this;
    }

private:
    void write(const std::string& s);
    std::ostringstream out_;
    int indent_;
    bool at_line_start_ = true;
};

// reference: sdfg/src/codegen/language_extensions/cpp_language_extension.cpp:9-52
class LanguageExtension {
public:
    virtual ~LanguageExtension() = default;
    virtual std::string language() const = 0;
    virtual std::string primitive_type(types::PrimitiveType t) const = 0;
    virtual std::string declaration(const std::string& name, const Container& c) const = 0;
    virtual std::string expression(const Expression& e) const { return e; }
};

class CPPLanguageExtension : public LanguageExtension {
public:
    std::string language() const override { return "C++"; }
    std::string primitive_type(types::PrimitiveType t) const override;
    std::string declaration(const std::string& name, const Container& c) const override;
};

inline const std::string CODE_SNIPPET_INIT_ONCE = "init_once";
inline const std::string CODE_SNIPPET_DEINIT_ONCE = "deinit_once";

class CodeSnippet {
public:
    CodeSnippet(std::string extension, bool as_file) : extension_(std::move(extension)), as_file_(as_file) {}
    PrettyPrinter& stream() { return stream_; }
    const PrettyPrinter& stream() const { return stream_; }
    const std::string& extension() const { return extension_; }
    bool is_as_file() const { return as_file_; }

private:
    PrettyPrinter stream_;
    std::string extension_;
    bool as_file_;
};

class CodeSnippetFactory {
public:
    explicit CodeSnippetFactory(std::filesystem::path output_path = {}) : output_path_(std::move(output_path)) {}
    // returns the snippet called `name`, creating it on first use
    CodeSnippet& require(const std::string& name, const std::string& extension, bool as_file = true);
    std::map<std::string, CodeSnippet>::iterator find(const std::string& name) { return snippets_.find(name); }
    const std::map<std::string, CodeSnippet>& snippets() const { return snippets_; }
    std::map<std::string, CodeSnippet>& snippets() { return snippets_; }
    const std::filesystem::path& output_path() const { return output_path_; }

private:
    std::filesystem::path output_path_;
    std::map<std::string, CodeSnippet> snippets_;
};

// reference: sdfg/include/sdfg/analysis/loop_analysis.h:25-42 (defaults of a non-loop element)
struct LoopInfo {
    int loopnest_index = -1;
    size_t num_loops = 0, num_maps = 0, num_fors = 0, num_whiles = 0, max_depth = 0;
    bool is_perfectly_nested = false, is_perfectly_parallel = false, is_elementwise = false, has_side_effects = false;
};

// reference: sdfg/include/sdfg/codegen/instrumentation/instrumentation_info.h:15-59
inline const std::string ElementType_H2DTransfer = "h2d_transfer";
inline const std::string ElementType_D2HTransfer = "d2h_transfer";
inline const std::string ElementType_Math = "math";
inline const std::string ElementType_Unknown = "unknown";
inline const std::string TargetType_SEQUENTIAL = "SEQUENTIAL";
inline const std::string TargetType_ROCM = "ROCM";

struct InstrumentationInfo {
    size_t element_id = 0;
    std::string element_type = ElementType_Unknown;
    std::string target_type = TargetType_SEQUENTIAL;
    LoopInfo loop_info;
    std::map<std::string, Expression> metrics;      // e.g. "flop", "pcie_bytes"
    std::string region_name;                        // the node's code, for the generator's report
};

enum class InstrumentationEventType { CPU, ROCM, NONE };

// Which elements are bracketed by the `__daisy_instrumentation_*` calls, and the text of the
// brackets (reference sdfg/src/codegen/instrumentation/instrumentation_plan.cpp:22-141: one
// `__daisy_metadata_t <sdfg>_<id>_md`, `long long <sdfg>_<id>_id = __daisy_instrumentation_init`,
// enter / exit, one `__daisy_instrumentation_metric` per metric, finalize).
class InstrumentationPlan {
public:
    InstrumentationPlan(const StructuredSDFG& sdfg, std::map<size_t, InstrumentationEventType> nodes)
        : sdfg_(sdfg), nodes_(std::move(nodes)) {}

    bool should_instrument(const data_flow::LibraryNode& node) const { return nodes_.count(node.element_id()) != 0; }
    bool empty() const { return nodes_.empty(); }
    size_t size() const { return nodes_.size(); }
    void begin_instrumentation(const structured_control_flow::Block& block, PrettyPrinter& stream, const InstrumentationInfo& info) const;
    void end_instrumentation(const structured_control_flow::Block& block, PrettyPrinter& stream, const InstrumentationInfo& info) const;

    static std::unique_ptr<InstrumentationPlan> none(const StructuredSDFG& sdfg);
    // The reference's "ols" mode brackets the outermost loops. The rocm target's library nodes
    // stand where the outermost loop of their expansion would be, so they are the regions here:
    // every node whose implementation type is a rocm one, and every transfer.
    static std::unique_ptr<InstrumentationPlan> outermost_loops_plan(const StructuredSDFG& sdfg);
    // "" -> none, "ols" -> outermost_loops_plan, anything else throws
    // "Unsupported instrumentation plan: <mode>" (reference python/bindings/py_structured_sdfg.cpp:376-383)
    static std::unique_ptr<InstrumentationPlan> from_mode(const StructuredSDFG& sdfg, const std::string& mode);

private:
    const StructuredSDFG& sdfg_;
    std::map<size_t, InstrumentationEventType> nodes_;
};

class LibraryNodeDispatcher {
public:
    LibraryNodeDispatcher(LanguageExtension& language_extension, const Function& function,
                          const data_flow::DataFlowGraph& data_flow_graph, const data_flow::LibraryNode& node)
        : language_extension_(language_extension), function_(function), data_flow_graph_(data_flow_graph), node_(node) {}
    virtual ~LibraryNodeDispatcher() = default;

    virtual bool begin_node(PrettyPrinter&) { return false; }
    virtual void end_node(PrettyPrinter&, bool) {}
    // Prints the node: a scope with one local per connector, dispatch_code(), write-back of
    // the outputs (reference block_dispatcher.cpp:333-438).
    virtual void dispatch(PrettyPrinter& stream, PrettyPrinter& globals_stream, CodeSnippetFactory& library_snippet_factory);
    virtual void dispatch_code(PrettyPrinter&, PrettyPrinter&, CodeSnippetFactory&) {}
    virtual InstrumentationInfo instrumentation_info() const;

protected:
    LanguageExtension& language_extension_;
    const Function& function_;
    const data_flow::DataFlowGraph& data_flow_graph_;
    const data_flow::LibraryNode& node_;
};

// the reference's parameter list (codegen/dispatchers/node_dispatcher_registry.h:140-141)
using LibraryNodeDispatcherFn = std::function<std::unique_ptr<LibraryNodeDispatcher>(
    LanguageExtension&, const Function&, const data_flow::DataFlowGraph&, const data_flow::LibraryNode&)>;

class LibraryNodeDispatcherRegistry {
public:
    static LibraryNodeDispatcherRegistry& instance();
    // key = "<code>::<implementation type>"; a key that is already taken is left as it is
    void register_library_node_dispatcher(const std::string& key, LibraryNodeDispatcherFn fn);
    LibraryNodeDispatcherFn get_library_node_dispatcher(const std::string& key) const;
    std::vector<std::string> keys() const;
    size_t size() const { return factories_.size(); }

private:
    mutable std::mutex mutex_;
    std::unordered_map<std::string, LibraryNodeDispatcherFn> factories_;
};

class CPPCodeGenerator {
public:
    CPPCodeGenerator(StructuredSDFG& sdfg, std::shared_ptr<CodeSnippetFactory> library_snippet_factory = nullptr,
                     std::string externals_prefix = "", const InstrumentationPlan* instrumentation_plan = nullptr);

    // Walks the root sequence and fills the streams. Throws std::runtime_error
    // "No library node dispatcher found for library node code: <key>" when a key is missing
    // (reference block_dispatcher.cpp:321).
    bool generate();
    std::string function_definition();
    // Writes <name>.h / <name>.cpp as the reference's as_source does.
    bool as_source(const std::filesystem::path& header_path, const std::filesystem::path& source_path);
    std::string header_text() const;
    std::string source_text(const std::string& header_name);
    CodeSnippetFactory& library_snippet_factory() { return *library_snippet_factory_; }
    LanguageExtension& language_extension() { return language_extension_; }
    const std::vector<InstrumentationInfo>& instrumentation() const { return instrumentation_; }

private:
    void dispatch_includes();
    void dispatch_schedule();

    StructuredSDFG& sdfg_;
    CPPLanguageExtension language_extension_;
    std::shared_ptr<CodeSnippetFactory> library_snippet_factory_;
    std::string externals_prefix_;
    const InstrumentationPlan* instrumentation_plan_;
    PrettyPrinter includes_stream_, classes_stream_, globals_stream_, main_stream_;
    std::vector<InstrumentationInfo> instrumentation_;
};

} // namespace sdfg::codegen

namespace sdfg::plugins {

// reference: sdfg/include/sdfg/plugins/plugins.h:16-49
struct Context {
    serializer::LibraryNodeSerializerRegistry& library_node_serializer_registry;
    codegen::LibraryNodeDispatcherRegistry& library_node_dispatcher_registry;

    static Context global_context() {
        return Context{serializer::LibraryNodeSerializerRegistry::instance(), codegen::LibraryNodeDispatcherRegistry::instance()};
    }
};

struct Plugin {
    const char* name;
    const char* version;
    const char* description;
    void (*register_plugin_callback)(Context& context);
};

// reference: sdfg/include/sdfg/plugins/target_mapping.h:11-37
class TargetMapper {
public:
    virtual ~TargetMapper() = default;
    virtual bool try_map(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager,
                         data_flow::LibraryNode& node) const = 0;
};

// reference: sdfg/include/sdfg/plugins/target_mapping.h:24-37 (declared there, with no definition in the tree; the
// registry here keeps the factories ordered by priority, highest first, and by registration within one priority)
class TargetMapperFactory {
public:
    virtual ~TargetMapperFactory() = default;
    virtual std::unique_ptr<TargetMapper> create() const = 0;
    virtual int priority() = 0;
    virtual const std::string& for_target() const = 0;
};

class TargetMapperRegistry {
public:
    static TargetMapperRegistry& instance();
    const std::vector<std::shared_ptr<TargetMapperFactory>> get_all_mappers();
    void register_target_mapper(std::shared_ptr<TargetMapperFactory> factory);
    // the mappers of one target, in the order get_all_mappers() gives
    std::vector<std::shared_ptr<TargetMapper>> create_for_target(const std::string& target);

private:
    std::mutex mutex_;
    std::vector<std::shared_ptr<TargetMapperFactory>> factories_;
};

} // namespace sdfg::plugins

namespace sdfg::passes {

// reference: opt/src/passes/targets/target_mapping_pass.cpp:12-38
class TargetMappingPass {
public:
    explicit TargetMappingPass(std::vector<std::shared_ptr<plugins::TargetMapper>> target_mappers)
        : target_mappers_(std::move(target_mappers)) {}
    std::string name() { return "TargetMapper"; }
    bool run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager);

private:
    std::vector<std::shared_ptr<plugins::TargetMapper>> target_mappers_;
};

} // namespace sdfg::passes
