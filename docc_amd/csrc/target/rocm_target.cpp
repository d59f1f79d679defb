#include "rocm_target.h"

#include <algorithm>
#include <mutex>
#include <set>
#include <sstream>

namespace sdfg::rocm {

using codegen::CodeSnippetFactory;
using codegen::InstrumentationInfo;
using codegen::LanguageExtension;
using codegen::LibraryNodeDispatcher;
using codegen::PrettyPrinter;
using data_flow::ConnectorBinding;
using data_flow::DataFlowGraph;
using data_flow::LibraryNode;
using structured_control_flow::Block;
namespace blas = math::blas;
namespace tensor = math::tensor;

namespace {

bool is_rocm_impl(const std::string& impl) {
    return impl == ImplementationType_ROCMWithTransfers || impl == ImplementationType_ROCMWithoutTransfers;
}

bool is_elementwise_code(const std::string& c) {
    for (auto& u : tensor::UnaryNodeCodes)
        if (u == c) return true;
    for (auto& b : tensor::BinaryNodeCodes)
        if (b == c) return true;
    return false;
}

bool is_math_node(const LibraryNode& node) {
    const std::string& c = node.code();
    return c == blas::LibraryNodeType_GEMM || c == tensor::LibraryNodeType_Softmax || c == tensor::LibraryNodeType_Conv ||
           c == tensor::LibraryNodeType_MatMul || c == tensor::LibraryNodeType_Attention || c == tensor::LibraryNodeType_Broadcast ||
           c == tensor::LibraryNodeType_Transpose || c == tensor::LibraryNodeType_Cast || c == tensor::LibraryNodeType_Fill ||
           c == blas::LibraryNodeType_DOT || c == LibraryNodeType_ROCM_Map ||
           std::find(tensor::ActivationNodeCodes.begin(), tensor::ActivationNodeCodes.end(), c) != tensor::ActivationNodeCodes.end() ||
           is_elementwise_code(c) || std::find(tensor::ReduceNodeCodes.begin(), tensor::ReduceNodeCodes.end(), c) != tensor::ReduceNodeCodes.end();
}

// Preamble every rocm dispatcher puts into the globals stream (duplicates are folded by the generator).
void emit_runtime_preamble(PrettyPrinter& globals, const Function& function) {
    if (globals.str().find("#define DOCC_ROCM_CHECK") != std::string::npos) return;  // once per file
    globals << "#include \"docc_rocm_rt.h\"" << std::endl;
    globals << "#include \"docc_rocm_ops.h\"" << std::endl;
    globals << "#ifndef DOCC_ROCM_CHECK" << std::endl;
    globals << "#define DOCC_ROCM_ON_FAILURE " << (function.return_container().empty() ? "return" : "return nullptr") << std::endl;
    globals << "#define DOCC_ROCM_CHECK(call) do { int __docc_rc = (call); if (__docc_rc != 0) { "
               "docc_rocm_report_failure(__func__, #call, __docc_rc); DOCC_ROCM_ON_FAILURE; } } while (0)"
            << std::endl;
    globals << "#endif" << std::endl;
}

// ---- with-transfers scaffolding ---------------------------------------------------------

struct DeviceOperand {
    std::string connector;  // host-side local, e.g. "__A"
    std::string device;     // device-side local, e.g. "d___A"
    Expression bytes;
    bool copy_in;
    bool copy_out;
};

void emit_transfers_begin(PrettyPrinter& s, const std::vector<DeviceOperand>& ops) {
    for (auto& op : ops) {
        s << "void *" << op.device << " = nullptr;" << std::endl;
        s << "const size_t " << op.device << "_bytes = (size_t) (" << op.bytes << ");" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_malloc_async(&" << op.device << ", " << op.device << "_bytes, nullptr));" << std::endl;
    }
    for (auto& op : ops)
        if (op.copy_in)
            s << "DOCC_ROCM_CHECK(docc_rocm_memcpy_h2d_async(" << op.device << ", " << op.connector << ", " << op.device
              << "_bytes, nullptr));" << std::endl;
}

void emit_transfers_end(PrettyPrinter& s, const std::vector<DeviceOperand>& ops) {
    for (auto& op : ops)
        if (op.copy_out)
            s << "DOCC_ROCM_CHECK(docc_rocm_memcpy_d2h_async(" << op.connector << ", " << op.device << ", " << op.device
              << "_bytes, nullptr));" << std::endl;
    s << "DOCC_ROCM_CHECK(docc_rocm_stream_sync(nullptr));" << std::endl;
    for (auto& op : ops) s << "DOCC_ROCM_CHECK(docc_rocm_free_async(" << op.device << ", nullptr));" << std::endl;
}

Expression sum_bytes(const std::vector<DeviceOperand>& ops) {
    Expression e;
    for (auto& op : ops) {
        if (op.copy_in) e += (e.empty() ? "" : " + ") + ("(" + op.bytes + ")");
        if (op.copy_out) e += (e.empty() ? "" : " + ") + ("(" + op.bytes + ")");
    }
    return e.empty() ? "0" : e;
}

// Base for the math-node dispatchers: prints the launcher call on `args` (device pointers),
// with or without the surrounding transfers.
class RocmMathDispatcher : public LibraryNodeDispatcher {
public:
    RocmMathDispatcher(LanguageExtension& le, const Function& f, const DataFlowGraph& b, const LibraryNode& n, bool with_transfers)
        : LibraryNodeDispatcher(le, f, b, n), with_transfers_(with_transfers) {}

    void dispatch_code(PrettyPrinter& stream, PrettyPrinter& globals, CodeSnippetFactory&) override {
        emit_runtime_preamble(globals, function_);
        const std::string guard = guard_condition();
        if (!guard.empty()) {
            stream << "if (" << guard << ") {" << std::endl;
            stream.setIndent(stream.indent() + 4);
        }
        std::vector<DeviceOperand> ops;
        if (with_transfers_) {
            ops = operands();
            emit_transfers_begin(stream, ops);
        }
        // the pointer a launcher receives: the connector's local as it is (a device pointer already), or the
        // device copy this dispatcher made. A connector that is not among the copied operands would hand a
        // host pointer to a kernel, so it is an error here rather than a fault on the device.
        auto name_of = [&](const std::string& connector) -> std::string {
            if (!with_transfers_) return connector;
            for (auto& op : ops)
                if (op.connector == connector) return op.device;
            throw std::runtime_error("rocm dispatcher of " + node_.code() + ": connector '" + connector +
                                     "' is passed to the launcher but is not one of the node's device operands");
        };
        emit_launch(stream, name_of);
        if (with_transfers_) emit_transfers_end(stream, ops);
        if (!guard.empty()) {
            stream.setIndent(stream.indent() - 4);
            stream << "}" << std::endl;
        }
    }

    InstrumentationInfo instrumentation_info() const override {
        InstrumentationInfo info = LibraryNodeDispatcher::instrumentation_info();
        info.element_type = codegen::ElementType_Math;
        info.target_type = codegen::TargetType_ROCM;
        if (with_transfers_) info.metrics["pcie_bytes"] = sum_bytes(operands());
        return info;
    }

protected:
    virtual std::vector<DeviceOperand> operands() const = 0;
    virtual void emit_launch(PrettyPrinter& stream, const std::function<std::string(const std::string&)>& name_of) = 0;
    virtual std::string guard_condition() const { return ""; }

    DeviceOperand operand(const std::string& connector, bool in, bool out) const {
        const auto& names = out ? node_.outputs() : node_.inputs();
        if (std::find(names.begin(), names.end(), connector) == names.end() && data_flow_graph_.input(connector) == nullptr &&
            data_flow_graph_.output(connector) == nullptr)
            throw std::runtime_error("rocm dispatcher of " + node_.code() + ": the node has no connector '" + connector + "'");
        return DeviceOperand{connector, "d_" + connector, node_.connector_bytes(connector), in, out};
    }

    bool with_transfers_;
};

// ---- GEMM ---------------------------------------------------------------------------------

class GEMMNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    const blas::GEMMNode& gemm() const { return static_cast<const blas::GEMMNode&>(node_); }

    std::vector<DeviceOperand> operands() const override {
        // C travels to the device only when the node reads it (beta != 0)
        const bool read_c = node_.reads("__C", data_flow_graph_.inputs);
        std::vector<DeviceOperand> ops{operand("__A", true, false), operand("__B", true, false)};
        if (gemm().epilogue_bias()) ops.push_back(operand("__bias", true, false));
        ops.push_back(operand("__C", read_c, true));
        return ops;
    }

    std::string guard_condition() const override {
        // same guard as the cuBLAS dispatcher (reference opt/src/targets/cuda/blas/gemm.cpp:17-26)
        return "(" + gemm().m() + ") != 0 && (" + gemm().n() + ") != 0";
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& g = gemm();
        std::string fn, in_t, out_t;
        switch (g.precision()) {
            case blas::d: fn = "docc_rocm_dgemm"; in_t = out_t = "double"; break;
            case blas::s: fn = "docc_rocm_sgemm"; in_t = out_t = "float"; break;
            case blas::b: fn = "docc_rocm_bf16gemm_f32"; in_t = "uint16_t"; out_t = "float"; break;
            default: throw std::runtime_error("Invalid precision for ROCM GEMM node");
        }
        if (g.has_epilogue()) fn += "_epilogue";
        s << "DOCC_ROCM_CHECK(" << fn << "(nullptr, " << (int) g.trans_a() << ", " << (int) g.trans_b() << ", "
          << language_extension_.expression(g.m()) << ", " << language_extension_.expression(g.n()) << ", "
          << language_extension_.expression(g.k()) << ", __alpha, (const " << in_t << " *) " << name_of("__A") << ", "
          << language_extension_.expression(g.lda()) << ", (const " << in_t << " *) " << name_of("__B") << ", "
          << language_extension_.expression(g.ldb()) << ", __beta, (" << out_t << " *) " << name_of("__C") << ", "
          << language_extension_.expression(g.ldc());
        if (g.has_epilogue()) {
            // C = act(alpha A B + beta C + bias[column]) in the store of the GEMM
            int act = -1;
            for (size_t i = 0; i < tensor::UnaryNodeCodes.size(); i++)
                if (tensor::UnaryNodeCodes[i] == g.epilogue_activation()) act = (int) i;
            if (g.epilogue_bias())
                s << ", (const " << out_t << " *) " << name_of("__bias");
            else
                s << ", nullptr";
            s << ", " << act;
            if (act >= 0) s << " /* " << g.epilogue_activation() << " */";
        }
        s << "));" << std::endl;
    }
};

// ---- MatMul (batched) -----------------------------------------------------------------------

class MatMulNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    const tensor::MatMulNode& mm() const { return static_cast<const tensor::MatMulNode&>(node_); }

    std::vector<DeviceOperand> operands() const override {
        return {operand("A", true, false), operand("B", true, false), operand("Y", false, true)};
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        // the batch of GEMMs (alpha 1, beta 0) that the reference's expansion loops over
        // (matmul_node.cpp:366-499), as one launch
        const auto& n = mm();
        std::string fn, in_t, out_t, one, zero;
        switch (n.element()) {
            case types::PrimitiveType::Double: fn = "docc_rocm_dgemm"; in_t = out_t = "double"; one = "1.0"; zero = "0.0"; break;
            case types::PrimitiveType::Float: fn = "docc_rocm_sgemm"; in_t = out_t = "float"; one = "1.0f"; zero = "0.0f"; break;
            case types::PrimitiveType::BFloat: fn = "docc_rocm_bf16gemm_f32"; in_t = "uint16_t"; out_t = "float"; one = "1.0f"; zero = "0.0f"; break;
            default: throw std::runtime_error("Invalid element type for ROCM MatMul node");
        }
        const Expression stride_b = n.b_is_batched() ? symbolic::mul(n.k(), n.n()) : Expression("0");
        s << "DOCC_ROCM_CHECK(" << fn << "_batched(nullptr, 111, 111, " << n.m() << ", " << n.n() << ", " << n.k() << ", " << one
          << ", (const " << in_t << " *) " << name_of("A") << ", " << n.k() << ", (int64_t) (" << symbolic::mul(n.m(), n.k())
          << "), (const " << in_t << " *) " << name_of("B") << ", " << n.n() << ", (int64_t) (" << stride_b << "), " << zero
          << ", (" << out_t << " *) " << name_of("Y") << ", " << n.n() << ", (int64_t) (" << symbolic::mul(n.m(), n.n())
          << "), (int64_t) (" << n.batch() << ")));" << std::endl;
    }
};

// ---- Softmax ------------------------------------------------------------------------------

class SoftmaxNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("X", true, false), operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::SoftmaxNode&>(node_);
        if (n.last_axis_only() && n.element() == types::PrimitiveType::Float) {
            s << "DOCC_ROCM_CHECK(docc_rocm_softmax_f32(nullptr, " << n.rows() << ", " << n.cols() << ", (const float *) "
              << name_of("X") << ", (float *) " << name_of("Y") << "));" << std::endl;
            return;
        }
        // a block of adjacent axes: the middle extent of an [outer, extent, inner] view
        s << "DOCC_ROCM_CHECK(docc_rocm_softmax(nullptr, " << (n.element() == types::PrimitiveType::Double ? 64 : 32) << ", "
          << n.outer() << ", " << n.extent() << ", " << n.inner() << ", (const void *) " << name_of("X") << ", (void *) "
          << name_of("Y") << "));" << std::endl;
    }
};

// ---- Conv ---------------------------------------------------------------------------------

class ConvNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    const tensor::ConvNode& conv() const { return static_cast<const tensor::ConvNode&>(node_); }

    std::vector<DeviceOperand> operands() const override {
        std::vector<DeviceOperand> ops{operand("X", true, false), operand("W", true, false)};
        if (conv().has_bias()) ops.push_back(operand("B", true, false));
        ops.push_back(operand("Y", false, true));
        return ops;
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& c = conv();
        auto get = [](const std::vector<Expression>& v, size_t i, const char* dflt) { return v.empty() ? Expression(dflt) : v[i]; };
        std::ostringstream dims;
        dims << c.shape()[0] << ", " << c.shape()[1] << ", " << c.shape()[2] << ", " << c.shape()[3] << ", " << c.output_channels() << ", "
             << c.kernel_shape()[0] << ", " << c.kernel_shape()[1] << ", " << get(c.strides(), 0, "1") << ", " << get(c.strides(), 1, "1")
             << ", " << get(c.pads(), 0, "0") << ", " << get(c.pads(), 1, "0") << ", " << get(c.pads(), 2, "0") << ", " << get(c.pads(), 3, "0")
             << ", " << get(c.dilations(), 0, "1") << ", " << get(c.dilations(), 1, "1");   // pads: begins, then ends
        // layers that run as im2col + GEMM take their column matrix from a workspace that lives around the node;
        // for the others the size is 0 and nothing is allocated
        int64_t group = 1;
        if (!symbolic::is_integer(c.group(), &group) || group != 1) {
            // the node's group (weights [C_out][C_in / group][kh][kw]): the direct kernels, once per group
            s << "DOCC_ROCM_CHECK(docc_rocm_conv2d_f32_grouped(nullptr, " << dims.str() << ", (int64_t) (" << c.group() << "), (const float *) "
              << name_of("X") << ", (const float *) " << name_of("W") << ", "
              << (c.has_bias() ? "(const float *) " + name_of("B") : std::string("nullptr")) << ", (float *) " << name_of("Y")
              << ", nullptr, 0));" << std::endl;
            return;
        }
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        s << "const int64_t __ws_bytes = docc_rocm_conv2d_f32_pads_workspace_bytes(" << dims.str() << ");" << std::endl;
        s << "void *__ws = nullptr;" << std::endl;
        s << "if (__ws_bytes > 0) DOCC_ROCM_CHECK(docc_rocm_malloc_async(&__ws, (size_t) __ws_bytes, nullptr));" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_conv2d_f32_pads(nullptr, " << dims.str() << ", (const float *) " << name_of("X")
          << ", (const float *) " << name_of("W") << ", "
          << (c.has_bias() ? "(const float *) " + name_of("B") : std::string("nullptr")) << ", (float *) " << name_of("Y")
          << ", __ws, __ws_bytes));" << std::endl;
        s << "if (__ws) DOCC_ROCM_CHECK(docc_rocm_free_async(__ws, nullptr));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// ---- Attention ----------------------------------------------------------------------------

class AttentionNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override {
        return {operand("Q", true, false), operand("K", true, false), operand("V", true, false), operand("O", false, true)};
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& a = static_cast<const tensor::AttentionNode&>(node_);
        const auto& q = a.shape_q();
        const int out_bf16 = a.output_element() == types::PrimitiveType::BFloat ? 1 : 0;
        int64_t d = 0;
        if (a.causal()) {
            // query i attends to the keys j <= i: the entry point for every head dimension it is built for (a workspace for
            // those that are widened, none for 32, 64 and 128)
            std::ostringstream cd;
            cd << q[0] << ", " << q[1] << ", " << q[2] << ", " << a.seq_kv() << ", " << q[3];
            s << "{" << std::endl;
            s.setIndent(s.indent() + 4);
            s << "const int64_t __ws_bytes = docc_rocm_attention_bf16_workspace_bytes(" << cd.str() << ", " << out_bf16 << ");" << std::endl;
            s << "void *__ws = nullptr;" << std::endl;
            s << "if (__ws_bytes > 0) DOCC_ROCM_CHECK(docc_rocm_malloc_async(&__ws, (size_t) __ws_bytes, nullptr));" << std::endl;
            s << "DOCC_ROCM_CHECK(docc_rocm_attention_bf16_causal(nullptr, " << cd.str() << ", (float) (" << a.scale()
              << "), (const uint16_t *) " << name_of("Q") << ", (const uint16_t *) " << name_of("K") << ", (const uint16_t *) "
              << name_of("V") << ", (void *) " << name_of("O") << ", " << out_bf16 << ", __ws, __ws_bytes));" << std::endl;
            s << "if (__ws) DOCC_ROCM_CHECK(docc_rocm_free_async(__ws, nullptr));" << std::endl;
            s.setIndent(s.indent() - 4);
            s << "}" << std::endl;
            return;
        }
        if (symbolic::is_integer(q[3], &d) && (d == 32 || d == 64 || d == 128)) {   // the head dimensions of the fused kernel
            s << "DOCC_ROCM_CHECK(docc_rocm_attention_bf16(nullptr, " << q[0] << ", " << q[1] << ", " << q[2] << ", " << a.seq_kv()
              << ", " << q[3] << ", (float) (" << a.scale() << "), (const uint16_t *) " << name_of("Q") << ", (const uint16_t *) "
              << name_of("K") << ", (const uint16_t *) " << name_of("V") << ", (void *) " << name_of("O") << ", " << out_bf16
              << "));" << std::endl;
            return;
        }
        // another head dimension (or one known at run time only): scores and probabilities live in a
        // workspace that this node allocates around its launches
        std::ostringstream dims;
        dims << q[0] << ", " << q[1] << ", " << q[2] << ", " << a.seq_kv() << ", " << q[3];
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        s << "const int64_t __ws_bytes = docc_rocm_attention_bf16_workspace_bytes(" << dims.str() << ", " << out_bf16 << ");" << std::endl;
        s << "void *__ws = nullptr;" << std::endl;
        s << "if (__ws_bytes > 0) DOCC_ROCM_CHECK(docc_rocm_malloc_async(&__ws, (size_t) __ws_bytes, nullptr));" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_attention_bf16_ws(nullptr, " << dims.str() << ", (float) (" << a.scale()
          << "), (const uint16_t *) " << name_of("Q") << ", (const uint16_t *) " << name_of("K") << ", (const uint16_t *) "
          << name_of("V") << ", (void *) " << name_of("O") << ", " << out_bf16 << ", __ws, __ws_bytes));" << std::endl;
        s << "if (__ws) DOCC_ROCM_CHECK(docc_rocm_free_async(__ws, nullptr));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// ---- offloading node ------------------------------------------------------------------------

class ROCMDataOffloadingNodeDispatcher : public LibraryNodeDispatcher {
public:
    using LibraryNodeDispatcher::LibraryNodeDispatcher;

    void dispatch_code(PrettyPrinter& s, PrettyPrinter& globals, CodeSnippetFactory&) override {
        emit_runtime_preamble(globals, function_);
        const auto& n = static_cast<const ROCMDataOffloadingNode&>(node_);
        const std::string size = language_extension_.expression(n.size());
        // order as in the CUDA offloading dispatcher (reference cuda_data_offloading_node.cpp:139-173):
        // allocate, copy, free; copies are followed by a stream wait because the node is blocking
        if (n.is_alloc()) {
            const std::string dst = n.is_h2d() ? "_dst" : "_ret";
            s << "DOCC_ROCM_CHECK(docc_rocm_malloc_async((void **) &" << dst << ", (size_t) (" << size << "), nullptr));" << std::endl;
        }
        if (n.is_h2d()) {
            s << "DOCC_ROCM_CHECK(docc_rocm_memcpy_h2d_async(_dst, _src, (size_t) (" << size << "), nullptr));" << std::endl;
        } else if (n.is_d2h()) {
            s << "DOCC_ROCM_CHECK(docc_rocm_memcpy_d2h_async(_dst, _src, (size_t) (" << size << "), nullptr));" << std::endl;
            s << "DOCC_ROCM_CHECK(docc_rocm_stream_sync(nullptr));" << std::endl;
        }
        if (n.is_free()) {
            const std::string ptr = n.is_d2h() ? "_src" : "_ptr";
            s << "DOCC_ROCM_CHECK(docc_rocm_free_async(" << ptr << ", nullptr));" << std::endl;
        }
    }

    InstrumentationInfo instrumentation_info() const override {
        const auto& n = static_cast<const ROCMDataOffloadingNode&>(node_);
        // as the CUDA transfer node reports itself (reference cuda_data_offloading_node.cpp:175-196)
        InstrumentationInfo info = LibraryNodeDispatcher::instrumentation_info();
        info.region_name = n.toStr();
        info.target_type = codegen::TargetType_ROCM;
        if (n.is_h2d() || n.is_d2h()) {
            info.element_type = n.is_h2d() ? codegen::ElementType_H2DTransfer : codegen::ElementType_D2HTransfer;
            info.metrics["pcie_bytes"] = n.size();
        }
        return info;
    }
};

// ---- Elementwise / Broadcast ----------------------------------------------------------------
// Counterpart of what CUDAMapDispatcher prints for the Maps these nodes expand to (reference
// opt/src/targets/cuda/...): here one launcher call per node.

class ElementWiseNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    // a constant or a scalar container bound to "A" or "B" (the reference's builder binds
    // either, python/bindings/builder/py_structured_sdfg_builder.cpp:894-908)
    bool is_scalar(const std::string& connector) const {
        const auto* in = data_flow_graph_.input(connector);
        return in && (in->is_constant || !function_.container(in->data).is_pointer);
    }

    std::vector<DeviceOperand> operands() const override {
        const auto& n = static_cast<const tensor::ElementWiseNode&>(node_);
        if (!n.is_binary()) return {operand("X", true, false), operand("Y", false, true)};
        std::vector<DeviceOperand> ops;
        if (!is_scalar("A")) ops.push_back(operand("A", true, false));
        if (!is_scalar("B")) ops.push_back(operand("B", true, false));
        ops.push_back(operand("C", false, true));
        return ops;
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::ElementWiseNode&>(node_);
        const int precision = n.element() == types::PrimitiveType::Double ? 64 : 32;
        if (!n.is_binary()) {
            s << "DOCC_ROCM_CHECK(docc_rocm_elementwise_unary(nullptr, " << n.operation() << " /* " << n.code() << " */, " << precision
              << ", " << n.count() << ", " << name_of("X") << ", " << name_of("Y") << "));" << std::endl;
            return;
        }
        const bool sa = is_scalar("A"), sb = is_scalar("B");
        if (sa && sb) throw InvalidSDFGException(n.code() + ": both operands are scalars");
        if (sa || sb)
            s << "DOCC_ROCM_CHECK(docc_rocm_elementwise_binary_scalar(nullptr, " << n.operation() << " /* " << n.code() << " */, "
              << precision << ", " << n.count() << ", " << name_of(sa ? "B" : "A") << ", (double) " << (sa ? "A" : "B") << ", "
              << (sa ? 1 : 0) << ", " << name_of("C") << "));" << std::endl;
        else
            s << "DOCC_ROCM_CHECK(docc_rocm_elementwise_binary(nullptr, " << n.operation() << " /* " << n.code() << " */, " << precision
              << ", " << n.count() << ", " << name_of("A") << ", " << name_of("B") << ", " << name_of("C") << "));" << std::endl;
    }
};

// ml::Elu / ml::LeakyReLU / ml::HardSigmoid: "alpha" and "beta" are scalars (constants or scalar containers) and
// travel by value; an operand the graph leaves unbound takes its operator's default.
class ActivationNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("X", true, false), operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::ActivationNode&>(node_);
        const int precision = n.element() == types::PrimitiveType::Double ? 64 : 32;
        auto scalar = [&](const std::string& connector) -> std::string {
            const auto* in = data_flow_graph_.input(connector);
            if (!in) return connector == "beta" && n.code() != "ml::HardSigmoid" ? "0.0" : n.default_operand(connector);
            if (!in->is_constant && function_.container(in->data).is_pointer)
                throw InvalidSDFGException(n.code() + ": operand '" + connector + "' must be a scalar");
            return "(double) " + connector;
        };
        s << "DOCC_ROCM_CHECK(docc_rocm_elementwise_activation(nullptr, " << n.operation() << " /* " << n.code() << " */, " << precision << ", "
          << n.count() << ", " << name_of("X") << ", " << name_of("Y") << ", " << scalar("alpha") << ", " << scalar("beta") << "));" << std::endl;
    }
};

// ml::Fill: the value is the scalar (or constant) on "X", handed over through host memory
class FillNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::FillNode&>(node_);
        const auto* in = data_flow_graph_.input("X");
        if (!in) throw InvalidSDFGException("ml::Fill: no value on connector 'X'");
        if (!in->is_constant && function_.container(in->data).is_pointer) throw InvalidSDFGException("ml::Fill: the value on 'X' must be a scalar");
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        s << "const " << language_extension_.primitive_type(n.element()) << " __docc_value = (" << language_extension_.primitive_type(n.element())
          << ") X;" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_fill(nullptr, (int) sizeof(__docc_value), " << n.count() << ", &__docc_value, " << name_of("Y") << "));"
          << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// DOT::BLAS: the vectors are device operands, the result a scalar of the host function (reference cuBLAS form
// opt/src/targets/cuda/blas/dot.cpp:55-68 passes &__out the same way); the launcher returns with the value.
class DotNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("__x", true, false), operand("__y", true, false)}; }

    std::string guard_condition() const override { return ""; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const blas::DotNode&>(node_);
        const auto* out = data_flow_graph_.output("__out");
        if (!out || function_.container(out->data).is_pointer) throw InvalidSDFGException("DOT: the result on '__out' must be a scalar container");
        s << "DOCC_ROCM_CHECK(docc_rocm_dot(nullptr, " << (n.precision() == blas::d ? 64 : 32) << ", " << language_extension_.expression(n.n()) << ", "
          << name_of("__x") << ", " << language_extension_.expression(n.incx()) << ", " << name_of("__y") << ", "
          << language_extension_.expression(n.incy()) << ", &__out));" << std::endl;
    }
};

class BroadcastNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("X", true, false), operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::BroadcastNode&>(node_);
        const int precision = n.element() == types::PrimitiveType::Double ? 64 : 32;
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        auto list = [&](const char* name, const std::vector<Expression>& shape) {
            s << "const int64_t " << name << "[] = {";
            for (size_t i = 0; i < shape.size(); i++) s << (i ? ", " : "") << "(int64_t) (" << shape[i] << ")";
            s << "};" << std::endl;
        };
        list("__docc_in_shape", n.input_shape());
        list("__docc_out_shape", n.output_shape());
        s << "DOCC_ROCM_CHECK(docc_rocm_broadcast(nullptr, " << precision << ", " << n.output_shape().size()
          << ", __docc_in_shape, __docc_out_shape, " << name_of("X") << ", " << name_of("Y") << "));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// ---- Cast ----------------------------------------------------------------------------------

// runtime type code (DOCC_ROCM_TYPE_*) of an element type, or -1
int cast_type_code(types::PrimitiveType t) {
    switch (t) {
        case types::PrimitiveType::Half: return 0;
        case types::PrimitiveType::BFloat: return 1;
        case types::PrimitiveType::Float: return 2;
        case types::PrimitiveType::Double: return 3;
        case types::PrimitiveType::Int32: return 4;
        case types::PrimitiveType::Int64: return 5;
        default: return -1;
    }
}

bool cast_is_built(int s, int d) {
    if (s < 0 || d < 0) return false;
    if (s == d) return true;
    const bool f = s == 2 || s == 3, g = d == 2 || d == 3;
    return (f && g) || (s <= 1 && d == 2) || (d <= 1 && s == 2) || (s >= 4 && g) || (f && d >= 4);
}

class CastNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("X", true, false), operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::CastNode&>(node_);
        s << "DOCC_ROCM_CHECK(docc_rocm_cast(nullptr, " << cast_type_code(n.element()) << " /* " << types::primitive_type_to_string(n.element())
          << " */, " << cast_type_code(n.target_type()) << " /* " << types::primitive_type_to_string(n.target_type()) << " */, " << n.count()
          << ", " << name_of("X") << ", " << name_of("Y") << "));" << std::endl;
    }
};

// ---- Transpose -----------------------------------------------------------------------------

class TransposeNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("X", true, false), operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::TransposeNode&>(node_);
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        s << "const int64_t __docc_shape[] = {";
        for (size_t i = 0; i < n.shape().size(); i++) s << (i ? ", " : "") << "(int64_t) (" << n.shape()[i] << ")";
        s << "};" << std::endl;
        s << "const int64_t __docc_perm[] = {";
        for (size_t i = 0; i < n.perm().size(); i++) s << (i ? ", " : "") << n.perm()[i];
        s << "};" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_transpose(nullptr, " << types::primitive_type_size(n.element()) << ", " << n.shape().size()
          << ", __docc_shape, __docc_perm, " << name_of("X") << ", " << name_of("Y") << "));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// ---- Reduce --------------------------------------------------------------------------------

class ReduceNodeDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    std::vector<DeviceOperand> operands() const override { return {operand("X", true, false), operand("Y", false, true)}; }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = static_cast<const tensor::ReduceNode&>(node_);
        const int precision = n.element() == types::PrimitiveType::Double ? 64 : 32;
        auto call = [&](const Expression& outer, const Expression& extent, const Expression& inner, const std::string& x, const std::string& y) {
            s << "DOCC_ROCM_CHECK(docc_rocm_reduce(nullptr, " << n.operation() << " /* " << n.code() << " */, " << precision << ", "
              << outer << ", " << extent << ", " << inner << ", " << x << ", " << y << "));" << std::endl;
        };
        if (n.adjacent_axes()) {
            call(n.outer(), n.extent(), n.inner(), name_of("X"), name_of("Y"));
            return;
        }
        // Axes in several blocks: one reduction per block of adjacent axes, the innermost block first, through device
        // temporaries (a sum of sums, a maximum of maxima, and - the blocks being full extents - a mean of means).
        // The reference's expansion is one loop nest over all the axes (reduce_node.cpp:188-333); for Sum and Mean the
        // order of the additions differs from it, as it does inside one block.
        const auto axes = n.sorted_axes();
        std::vector<std::pair<size_t, size_t>> runs;   // [first, last] positions in the current shape
        for (size_t i = 0; i < axes.size();) {
            size_t j = i;
            while (j + 1 < axes.size() && axes[j + 1] == axes[j] + 1) j++;
            runs.emplace_back((size_t) axes[i], (size_t) axes[j]);
            i = j + 1;
        }
        const Expression elem = symbolic::integer(precision / 8);
        std::vector<Expression> shape = n.shape();
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        s << "void *__docc_part[2] = {nullptr, nullptr};" << std::endl;
        std::string from = name_of("X");
        for (size_t k = runs.size(); k-- > 0;) {
            const auto [lo, hi] = runs[k];
            const Expression outer = symbolic::product(shape, 0, lo), extent = symbolic::product(shape, lo, hi + 1),
                             inner = symbolic::product(shape, hi + 1, shape.size());
            std::string to = name_of("Y");
            if (k > 0) {
                const int slot = (int) ((runs.size() - 1 - k) & 1);
                to = "__docc_part[" + std::to_string(slot) + "]";
                if (runs.size() - 1 - k < 2)   // a later step reuses the slot: its result is never larger
                    s << "DOCC_ROCM_CHECK(docc_rocm_malloc_async(&" << to << ", (size_t) (" << symbolic::mul(symbolic::mul(outer, inner), elem) << "), nullptr));" << std::endl;
            }
            call(outer, extent, inner, from, to);
            shape.erase(shape.begin() + (long) lo, shape.begin() + (long) hi + 1);
            from = to;
        }
        s << "if (__docc_part[0]) DOCC_ROCM_CHECK(docc_rocm_free_async(__docc_part[0], nullptr));" << std::endl;
        s << "if (__docc_part[1]) DOCC_ROCM_CHECK(docc_rocm_free_async(__docc_part[1], nullptr));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// ---- fused elementwise chain ---------------------------------------------------------------

class FusedElementWiseDispatcher_ROCM : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

protected:
    const ROCMFusedElementWiseNode& fused() const { return static_cast<const ROCMFusedElementWiseNode&>(node_); }

    std::vector<DeviceOperand> operands() const override {
        std::vector<DeviceOperand> ops;
        if (!fused().a_shape().empty()) ops.push_back(operand("A", true, false));
        if (fused().has_b() && !fused().b_shape().empty()) ops.push_back(operand("B", true, false));
        ops.push_back(operand("Y", false, true));
        return ops;
    }

    static int index_of(const std::vector<std::string>& codes, const std::string& code) {
        for (size_t i = 0; i < codes.size(); i++)
            if (codes[i] == code) return (int) i;
        return -1;
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = fused();
        const int precision = n.element() == types::PrimitiveType::Double ? 64 : 32;
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        auto list = [&](const char* name, const std::vector<Expression>& shape) {
            s << "const int64_t " << name << "[] = {";
            for (size_t i = 0; i < shape.size(); i++) s << (i ? ", " : "") << "(int64_t) (" << shape[i] << ")";
            s << "};" << std::endl;
        };
        list("__docc_shape", n.shape());
        const bool a_array = !n.a_shape().empty(), b_array = n.has_b() && !n.b_shape().empty();
        if (a_array) list("__docc_a_shape", n.a_shape());
        if (b_array) list("__docc_b_shape", n.b_shape());
        s << "const int __docc_post[] = {";
        for (size_t i = 0; i < n.post().size(); i++)
            s << (i ? ", " : "") << index_of(tensor::UnaryNodeCodes, n.post()[i]) << " /* " << n.post()[i] << " */";
        if (n.post().empty()) s << "0";
        s << "};" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_elementwise_fused(nullptr, " << precision << ", " << n.shape().size() << ", __docc_shape, ";
        if (n.has_b())
            s << index_of(tensor::BinaryNodeCodes, n.binary()) << " /* " << n.binary() << " */, ";
        else
            s << "-1, ";
        if (a_array)
            s << "__docc_a_shape, " << name_of("A") << ", 0.0, ";
        else
            s << "nullptr, nullptr, (double) A, ";
        if (b_array)
            s << "__docc_b_shape, " << name_of("B") << ", 0.0, ";
        else if (n.has_b())
            s << "nullptr, nullptr, (double) B, ";
        else
            s << "nullptr, nullptr, 0.0, ";
        s << n.post().size() << ", __docc_post, " << name_of("Y") << "));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }
};

// ---- Map nests -------------------------------------------------------------------------------
// Counterpart of CUDAMapDispatcher (reference opt/src/targets/cuda/cuda_map_dispatcher.cpp:42-262): the kernel goes
// into a snippet file of its own (there "<kernel>.cu", compiled with nvcc by the driver and linked in,
// py_structured_sdfg.cpp:445-466; here "<kernel>.hip", compiled to the code object "<kernel>.hsaco" that lies next
// to the generated library), and the host side launches it - there `kernel<<<grid, block>>>(args)`, here the
// runtime's module_load / module_get_function / launch, since the host code is compiled by a plain C++ compiler.

class ROCMMapDispatcher : public RocmMathDispatcher {
public:
    using RocmMathDispatcher::RocmMathDispatcher;

    void dispatch_code(PrettyPrinter& stream, PrettyPrinter& globals, CodeSnippetFactory& snippets) override {
        globals_ = &globals;
        snippets_ = &snippets;
        RocmMathDispatcher::dispatch_code(stream, globals, snippets);
    }

protected:
    const ROCMMapNode& map() const { return static_cast<const ROCMMapNode&>(node_); }

    std::vector<DeviceOperand> operands() const override {
        std::vector<DeviceOperand> ops;
        for (auto& r : map().reads()) ops.push_back(operand(r.connector, true, false));
        for (auto& w : map().writes()) ops.push_back(operand(w.connector, false, true));
        return ops;
    }

    static void emit_loader(PrettyPrinter& globals) {
        if (globals.str().find("__docc_rocm_map_kernel(") != std::string::npos) return;   // once per file
        globals << "#include <dlfcn.h>" << std::endl;
        globals << "#include <mutex>" << std::endl;
        globals << "#include <string>" << std::endl;
        globals << "namespace {" << std::endl;
        globals << "// a generated kernel image and its entry points; the image lies next to this library" << std::endl;
        globals << "struct __docc_rocm_map_image {" << std::endl;
        globals << "    std::mutex mutex;" << std::endl;
        globals << "    docc_rocm_module_t module = nullptr;" << std::endl;
        globals << "    docc_rocm_function_t functions[4] = {nullptr, nullptr, nullptr, nullptr};" << std::endl;
        globals << "};" << std::endl;
        globals << "int __docc_rocm_map_kernel(__docc_rocm_map_image &image, const char *file, const char *name, int slot, docc_rocm_function_t *function) {" << std::endl;
        globals << "    std::lock_guard<std::mutex> lock(image.mutex);" << std::endl;
        globals << "    if (!image.module) {" << std::endl;
        globals << "        std::string path = file;" << std::endl;
        globals << "        Dl_info info;" << std::endl;
        globals << "        if (dladdr((const void *) &__docc_rocm_map_kernel, &info) && info.dli_fname) {" << std::endl;
        globals << "            const std::string lib = info.dli_fname;" << std::endl;
        globals << "            const size_t slash = lib.find_last_of('/');" << std::endl;
        globals << "            if (slash != std::string::npos) path = lib.substr(0, slash + 1) + file;" << std::endl;
        globals << "        }" << std::endl;
        globals << "        const int rc = docc_rocm_module_load(path.c_str(), &image.module);" << std::endl;
        globals << "        if (rc != 0) return rc;" << std::endl;
        globals << "    }" << std::endl;
        globals << "    if (!image.functions[slot]) {" << std::endl;
        globals << "        const int rc = docc_rocm_module_get_function(image.module, name, &image.functions[slot]);" << std::endl;
        globals << "        if (rc != 0) return rc;" << std::endl;
        globals << "    }" << std::endl;
        globals << "    *function = image.functions[slot];" << std::endl;
        globals << "    return 0;" << std::endl;
        globals << "}" << std::endl;
        globals << "} // namespace" << std::endl;
    }

    void emit_launch(PrettyPrinter& s, const std::function<std::string(const std::string&)>& name_of) override {
        const auto& n = map();
        for (auto& sym : n.symbols())
            if (!function_.exists(sym) || function_.container(sym).is_pointer)
                throw std::runtime_error("ROCMMap: '" + sym + "' in a bound or a stride is not a scalar of the function");
        // the reference's kernel name (cuda_map_dispatcher.cpp:135)
        const std::string kernel = "kernel_" + function_.name() + "_" + std::to_string(node_.element_id());
        const RocmMapKernelPlan plan = plan_rocm_map_kernel(n, kernel);
        auto& snippet = snippets_->require(kernel, "hip", true).stream();
        if (snippet.str().empty()) snippet << plan.source;
        emit_loader(*globals_);
        *globals_ << "static __docc_rocm_map_image __docc_image_" << kernel << ";" << std::endl;

        const size_t depth = plan.bounds.size();
        const int V = plan.vector_width;
        s << "{" << std::endl;
        s.setIndent(s.indent() + 4);
        for (size_t l = 0; l < depth; l++) s << "long long __docc_b" << l << " = (long long) (" << plan.bounds[l] << ");" << std::endl;
        s << "bool __docc_empty = false, __docc_wide = false;" << std::endl;
        for (size_t l = 0; l < depth; l++) s << "__docc_empty = __docc_empty || __docc_b" << l << " <= 0;" << std::endl;
        // 32-bit indices when every operand and the iteration count stay below 2^31
        for (auto& op : plan.operands) s << "__docc_wide = __docc_wide || (long long) (" << op.extent << ") > 0x7fffffffLL;" << std::endl;
        s << "if (!__docc_empty) {" << std::endl;
        s.setIndent(s.indent() + 4);
        for (auto& op : plan.operands)
            s << (op.write ? "" : "const ") << (op.element == types::PrimitiveType::Double ? "double" : "float") << " *__docc_p_" << op.connector
              << " = (" << (op.write ? "" : "const ") << (op.element == types::PrimitiveType::Double ? "double" : "float") << " *) " << name_of(op.connector) << ";" << std::endl;
        for (auto& op : plan.operands)
            for (size_t l = 0; l < depth; l++)
                if (op.strides[l] != "0" && op.strides[l] != "1")
                    s << "long long __docc_st_" << op.connector << "_" << l << " = (long long) (" << op.strides[l] << ");" << std::endl;
        if (V > 1) {
            s << "bool __docc_vector = __docc_b" << depth - 1 << " % " << V << " == 0;" << std::endl;
            for (auto& op : plan.operands)
                if (op.vector)
                    s << "__docc_vector = __docc_vector && ((uintptr_t) __docc_p_" << op.connector << ") % "
                      << V * (op.element == types::PrimitiveType::Double ? 8 : 4) << " == 0;" << std::endl;
        } else {
            s << "const bool __docc_vector = false;" << std::endl;
        }
        s << "unsigned long long __docc_threads = (unsigned long long) (__docc_vector ? __docc_b" << depth - 1 << " / " << V << " : __docc_b" << depth - 1 << ");" << std::endl;
        for (size_t l = 0; l + 1 < depth; l++) s << "__docc_threads *= (unsigned long long) __docc_b" << l << ";" << std::endl;
        s << "__docc_wide = __docc_wide || __docc_threads > 0x7fffffffULL;" << std::endl;
        s << "const unsigned long long __docc_groups = (__docc_threads + 255) / 256;" << std::endl;
        s << "if (__docc_groups > 0x7fffffffULL) {" << std::endl;
        s << "    docc_rocm_report_failure(__func__, \"" << kernel << ": more than 2^31 work-groups\", DOCC_ROCM_ERR_UNSUPPORTED);" << std::endl;
        s << "    DOCC_ROCM_ON_FAILURE;" << std::endl;
        s << "}" << std::endl;
        s << "static const char *const __docc_names[4] = {\"" << kernel << "_s32\", \"" << kernel << "_s64\", \"" << kernel << "_v32\", \"" << kernel << "_v64\"};" << std::endl;
        s << "const int __docc_slot = (__docc_vector ? 2 : 0) + (__docc_wide ? 1 : 0);" << std::endl;
        s << "docc_rocm_function_t __docc_fn = nullptr;" << std::endl;
        s << "DOCC_ROCM_CHECK(__docc_rocm_map_kernel(__docc_image_" << kernel << ", \"" << kernel << ".hsaco\", __docc_names[__docc_slot], __docc_slot, &__docc_fn));" << std::endl;
        s << "void *__docc_args[] = {";
        bool first = true;
        auto arg = [&](const std::string& name) {
            s << (first ? "" : ", ") << "(void *) &" << name;
            first = false;
        };
        for (auto& op : plan.operands) arg("__docc_p_" + op.connector);
        for (auto& sc : n.scalars()) arg(sc.connector);
        for (size_t l = 0; l < depth; l++) arg("__docc_b" + std::to_string(l));
        for (auto& op : plan.operands)
            for (size_t l = 0; l < depth; l++)
                if (op.strides[l] != "0" && op.strides[l] != "1") arg("__docc_st_" + op.connector + "_" + std::to_string(l));
        s << "};" << std::endl;
        s << "const uint32_t __docc_grid[3] = {(uint32_t) __docc_groups, 1, 1}, __docc_block[3] = {256, 1, 1};" << std::endl;
        s << "DOCC_ROCM_CHECK(docc_rocm_launch(__docc_fn, __docc_grid, __docc_block, 0, nullptr, __docc_args));" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
        s.setIndent(s.indent() - 4);
        s << "}" << std::endl;
    }

private:
    PrettyPrinter* globals_ = nullptr;
    CodeSnippetFactory* snippets_ = nullptr;
};

template <typename D>
void register_math(codegen::LibraryNodeDispatcherRegistry& reg, const std::string& code) {
    for (bool with : {true, false}) {
        reg.register_library_node_dispatcher(
            code + "::" + (with ? ImplementationType_ROCMWithTransfers : ImplementationType_ROCMWithoutTransfers),
            [with](LanguageExtension& le, const Function& f, const DataFlowGraph& b, const LibraryNode& n) {
                return std::make_unique<D>(le, f, b, n, with);
            });
    }
}

std::unique_ptr<LibraryNode> deserialize_attention(const json::Value& j) { return tensor::AttentionNode::from_json(j); }
std::unique_ptr<LibraryNode> deserialize_offloading(const json::Value& j) { return ROCMDataOffloadingNode::from_json(j); }

} // namespace

void register_plugin(plugins::Context& context) {
    auto& ser = context.library_node_serializer_registry;
    ser.register_library_node_serializer(tensor::LibraryNodeType_Attention, &deserialize_attention);
    ser.register_library_node_serializer(LibraryNodeType_ROCM_Offloading, &deserialize_offloading);

    auto& reg = context.library_node_dispatcher_registry;
    register_math<GEMMNodeDispatcher_ROCM>(reg, blas::LibraryNodeType_GEMM);
    register_math<MatMulNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_MatMul);
    register_math<SoftmaxNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Softmax);
    register_math<ConvNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Conv);
    register_math<AttentionNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Attention);
    for (auto& code : tensor::UnaryNodeCodes) register_math<ElementWiseNodeDispatcher_ROCM>(reg, code);
    for (auto& code : tensor::BinaryNodeCodes) register_math<ElementWiseNodeDispatcher_ROCM>(reg, code);
    for (auto& code : tensor::ActivationNodeCodes) register_math<ActivationNodeDispatcher_ROCM>(reg, code);
    register_math<FillNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Fill);
    register_math<DotNodeDispatcher_ROCM>(reg, blas::LibraryNodeType_DOT);
    register_math<BroadcastNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Broadcast);
    register_math<TransposeNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Transpose);
    register_math<CastNodeDispatcher_ROCM>(reg, tensor::LibraryNodeType_Cast);
    for (auto& code : tensor::ReduceNodeCodes) register_math<ReduceNodeDispatcher_ROCM>(reg, code);
    register_math<FusedElementWiseDispatcher_ROCM>(reg, LibraryNodeType_ROCM_FusedElementWise);
    register_math<ROCMMapDispatcher>(reg, LibraryNodeType_ROCM_Map);
    reg.register_library_node_dispatcher(
        LibraryNodeType_ROCM_Offloading + "::" + ImplementationType_NONE,
        [](LanguageExtension& le, const Function& f, const DataFlowGraph& b, const LibraryNode& n) {
            return std::make_unique<ROCMDataOffloadingNodeDispatcher>(le, f, b, n);
        });
}

void register_rocm_plugin() {
    auto context = plugins::Context::global_context();
    register_plugin(context);
    // the mapper's factory, once (the dispatcher registry ignores a second registration by itself)
    static std::once_flag once;
    std::call_once(once, [] { plugins::TargetMapperRegistry::instance().register_target_mapper(std::make_shared<RocmLibNodeMapperFactory>()); });
}

const std::string& RocmLibNodeMapperFactory::for_target() const {
    static const std::string target = "rocm";
    return target;
}

const plugins::Plugin rocm_plugin = {"rocm", "0.1", "MI355X (gfx950) target for the math library nodes", &register_plugin};

// ---------------------------------------------------------------------------------- mapper

bool RocmLibNodeMapper::try_map(builder::StructuredSDFGBuilder&, analysis::AnalysisManager&, LibraryNode& node) const {
    reason_.clear();
    auto decline = [&](const std::string& why) {
        reason_ = node.code() + ": " + why;
        return false;
    };
    using P = types::PrimitiveType;
    if (node.code() == blas::LibraryNodeType_GEMM) {
        auto* g = dynamic_cast<blas::GEMMNode*>(&node);
        if (!g) return decline("not a GEMM node object");
        if (g->layout() != blas::RowMajor) return decline("only row-major layout is supported");
        if (g->trans_a() == blas::ConjTrans || g->trans_b() == blas::ConjTrans) return decline("conjugate transpose is not supported");
        if (g->precision() != blas::s && g->precision() != blas::d && g->precision() != blas::b)
            return decline("precision must be s, d or b (bf16 with fp32 accumulate)");
    } else if (node.code() == tensor::LibraryNodeType_MatMul) {
        auto* m = dynamic_cast<tensor::MatMulNode*>(&node);
        if (!m) return decline("not a MatMul node object");
        if (m->element() != P::Float && m->element() != P::Double && m->element() != P::BFloat)
            return decline("element type must be Float, Double or BFloat");
    } else if (node.code() == tensor::LibraryNodeType_Softmax) {
        auto* s = dynamic_cast<tensor::SoftmaxNode*>(&node);
        if (!s) return decline("not a Softmax node object");
        if (s->element() != P::Float && s->element() != P::Double) return decline("element type must be Float or Double");
        if (!s->adjacent_axes()) return decline("the reduced axes must be adjacent (one block)");
    } else if (node.code() == tensor::LibraryNodeType_Conv) {
        auto* c = dynamic_cast<tensor::ConvNode*>(&node);
        if (!c) return decline("not a Conv node object");
        if (c->element() != P::Float) return decline("only Float is supported");
        if (c->kernel_shape().size() != 2) return decline("only 2-d convolution is supported");
        int64_t group = 1;
        if (symbolic::is_integer(c->group(), &group) && group < 1) return decline("group must be positive");
    } else if (node.code() == tensor::LibraryNodeType_Attention) {
        auto* a = dynamic_cast<tensor::AttentionNode*>(&node);
        if (!a) return decline("not an Attention node object");
        if (a->element() != P::BFloat) return decline("inputs must be BFloat");
        if (a->output_element() != P::BFloat && a->output_element() != P::Float) return decline("output must be BFloat or Float");
        int64_t head_dim = 0;
        if (a->causal() && symbolic::is_integer(a->shape_q()[3], &head_dim) && head_dim > 128)
            return decline("the causal form is built for head dimensions up to 128");
        // head dimensions 32, 64 and 128 run the fused kernel, any other the GEMM / softmax / GEMM sequence
    } else if (auto* act = dynamic_cast<tensor::ActivationNode*>(&node)) {
        if (act->element() != P::Float && act->element() != P::Double) return decline("element type must be Float or Double");
    } else if (auto* fill = dynamic_cast<tensor::FillNode*>(&node)) {
        const size_t size = types::primitive_type_size(fill->element());
        if (size != 1 && size != 2 && size != 4 && size != 8) return decline("elements must be 1, 2, 4 or 8 bytes");
    } else if (auto* dot = dynamic_cast<blas::DotNode*>(&node)) {
        if (dot->precision() != blas::s && dot->precision() != blas::d) return decline("precision must be s or d");
    } else if (is_elementwise_code(node.code())) {
        auto* e = dynamic_cast<tensor::ElementWiseNode*>(&node);
        if (!e) return decline("not an elementwise node object");
        if (e->element() != P::Float && e->element() != P::Double) return decline("element type must be Float or Double");
    } else if (auto* r = dynamic_cast<tensor::ReduceNode*>(&node)) {
        if (r->element() != P::Float && r->element() != P::Double) return decline("element type must be Float or Double");
    } else if (node.code() == tensor::LibraryNodeType_Broadcast) {
        auto* b = dynamic_cast<tensor::BroadcastNode*>(&node);
        if (!b) return decline("not a Broadcast node object");
        if (b->element() != P::Float && b->element() != P::Double) return decline("element type must be Float or Double");
        if (b->output_shape().size() > 6) return decline("rank above 6 is not supported");
    } else if (node.code() == tensor::LibraryNodeType_Cast) {
        auto* c = dynamic_cast<tensor::CastNode*>(&node);
        if (!c) return decline("not a Cast node object");
        if (!cast_is_built(cast_type_code(c->element()), cast_type_code(c->target_type())))
            return decline(std::string("conversion ") + types::primitive_type_to_string(c->element()) + " -> " +
                           types::primitive_type_to_string(c->target_type()) + " is not built");
    } else if (node.code() == LibraryNodeType_ROCM_Map) {
        // a nest of maps over dense tensors: always has a kernel, it is generated for the node
        if (!dynamic_cast<ROCMMapNode*>(&node)) return decline("not a ROCMMap node object");
    } else if (node.code() == tensor::LibraryNodeType_Transpose) {
        auto* t = dynamic_cast<tensor::TransposeNode*>(&node);
        if (!t) return decline("not a Transpose node object");
        const size_t bytes = types::primitive_type_size(t->element());
        if (bytes != 1 && bytes != 2 && bytes != 4 && bytes != 8) return decline("element size must be 1, 2, 4 or 8 bytes");
        if (t->shape().size() > 6 || t->shape().empty()) return decline("rank must be 1..6");
    } else {
        return false;  // not a node of this target
    }
    node.implementation_type() = implementation_type_;
    return true;
}

// ---------------------------------------------------------------------------------- fusion

namespace {

ConnectorBinding make_binding(const std::string& connector, const std::string& data) {
    ConnectorBinding b;
    b.connector = connector;
    b.data = data;
    return b;
}

bool is_rocm_type(const std::string& impl) {
    return impl == ImplementationType_ROCMWithTransfers || impl == ImplementationType_ROCMWithoutTransfers;
}

struct Uses {
    std::vector<size_t> readers, writers;
};

Uses uses_of(const StructuredSDFG& sdfg, const std::string& name) {
    Uses u;
    for (size_t i = 0; i < sdfg.blocks().size(); i++) {
        const Block& b = sdfg.blocks()[i];
        for (auto& in : b.inputs)
            if (!in.is_constant && in.data == name) u.readers.push_back(i);
        for (auto& out : b.outputs)
            if (out.data == name) u.writers.push_back(i);
    }
    return u;
}

// an intermediate that exists only to carry a value from block `producer` to block `consumer`
bool is_private_link(const StructuredSDFG& sdfg, const std::string& name, size_t producer, size_t consumer) {
    const Container& c = sdfg.container(name);
    if (c.is_argument || !c.transient || name == sdfg.return_container()) return false;
    const Uses u = uses_of(sdfg, name);
    return u.writers.size() == 1 && u.writers[0] == producer && u.readers.size() == 1 && u.readers[0] == consumer && producer < consumer;
}

// nothing between the two blocks (exclusive) writes `name`
bool unwritten_between(const StructuredSDFG& sdfg, const std::string& name, size_t from, size_t to) {
    for (size_t i = from + 1; i < to; i++)
        for (auto& out : sdfg.blocks()[i].outputs)
            if (out.data == name) return false;
    return true;
}

// nothing between the two blocks (exclusive) reads or writes `name`
bool untouched_between(const StructuredSDFG& sdfg, const std::string& name, size_t from, size_t to) {
    for (size_t i = from + 1; i < to; i++) {
        for (auto& in : sdfg.blocks()[i].inputs)
            if (!in.is_constant && in.data == name) return false;
        for (auto& out : sdfg.blocks()[i].outputs)
            if (out.data == name) return false;
    }
    return true;
}

// Rewrites an elementwise node as the equivalent fused node (no-op for one that already is).
void make_fused(StructuredSDFG& sdfg, size_t i) {
    Block& blk = sdfg.blocks()[i];
    auto* e = dynamic_cast<tensor::ElementWiseNode*>(blk.node.get());
    if (!e) return;
    const bool binary = e->is_binary();
    auto shape_of = [&](const char* connector) -> std::vector<Expression> {
        const ConnectorBinding* in = blk.input(connector);
        const bool scalar = in->is_constant || !sdfg.container(in->data).is_pointer;
        return scalar ? std::vector<Expression>{} : e->shape();
    };
    auto node = std::make_unique<ROCMFusedElementWiseNode>(
        e->implementation_type(), e->shape(), e->element(), binary ? e->code() : "", shape_of(binary ? "A" : "X"),
        binary ? shape_of("B") : std::vector<Expression>{}, binary ? std::vector<std::string>{} : std::vector<std::string>{e->code()});
    node->set_element_id(e->element_id());
    for (auto& in : blk.inputs)
        if (in.connector == "X") in.connector = "A";
    for (auto& out : blk.outputs) out.connector = "Y";
    blk.node = std::move(node);
}

} // namespace

bool RocmSoftmaxPatternPass::run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager&) {
    StructuredSDFG& sdfg = builder.subject();
    auto& blocks = sdfg.blocks();
    bool applied = false;
    // the single block that writes `name`, or -1
    auto writer_of = [&](const std::string& name) -> long {
        const Uses u = uses_of(sdfg, name);
        return u.writers.size() == 1 ? (long) u.writers[0] : -1;
    };
    auto private_value = [&](const std::string& name, std::vector<size_t> readers) {
        const Container& c = sdfg.container(name);
        if (c.is_argument || !c.transient || name == sdfg.return_container()) return false;
        Uses u = uses_of(sdfg, name);
        std::sort(readers.begin(), readers.end());
        std::sort(u.readers.begin(), u.readers.end());
        return u.writers.size() == 1 && u.readers == readers;
    };
    auto elementwise = [&](long i, const char* code, bool binary) -> tensor::ElementWiseNode* {
        if (i < 0) return nullptr;
        auto* e = dynamic_cast<tensor::ElementWiseNode*>(blocks[(size_t) i].node.get());
        return e && e->code() == code && e->is_binary() == binary && e->implementation_type() == ImplementationType_NONE ? e : nullptr;
    };
    auto data_of = [&](size_t i, const char* connector) -> std::string {
        const ConnectorBinding* b = blocks[i].input(connector);
        return b && !b->is_constant ? b->data : std::string();
    };
    // Broadcast of a keepdims reduction `code` of `source` over `axes`: fills the two block indices
    auto reduced_and_repeated = [&](const std::string& repeated, const char* code, const std::vector<Expression>& shape, long* bc_at, long* red_at,
                                    std::vector<int64_t>* axes, std::string* source) {
        *bc_at = repeated.empty() ? -1 : writer_of(repeated);
        if (*bc_at < 0) return false;
        auto* bc = dynamic_cast<tensor::BroadcastNode*>(blocks[(size_t) *bc_at].node.get());
        if (!bc || bc->implementation_type() != ImplementationType_NONE || bc->output_shape() != shape) return false;
        const std::string small = data_of((size_t) *bc_at, "X");
        *red_at = small.empty() ? -1 : writer_of(small);
        if (*red_at < 0) return false;
        auto* red = dynamic_cast<tensor::ReduceNode*>(blocks[(size_t) *red_at].node.get());
        if (!red || red->code() != code || red->implementation_type() != ImplementationType_NONE || !red->keepdims() || red->shape() != shape) return false;
        // the broadcast repeats exactly the reduced axes
        const auto ax = red->sorted_axes();
        if (bc->input_shape().size() != shape.size()) return false;
        for (size_t d = 0; d < shape.size(); d++) {
            const bool reduced = std::find(ax.begin(), ax.end(), (int64_t) d) != ax.end();
            if (bc->input_shape()[d] != (reduced ? Expression("1") : shape[d])) return false;
        }
        *axes = ax;
        *source = data_of((size_t) *red_at, "X");
        return !source->empty();
    };
    bool changed = true;
    while (changed) {
        changed = false;
        for (size_t at = 0; at < blocks.size() && !changed; at++) {
            auto* div = elementwise((long) at, "ml::Div", true);
            if (!div) continue;
            const std::vector<Expression> shape = div->shape();
            const std::string e_name = data_of(at, "A"), den = data_of(at, "B");
            long bc2, sum_at, bc1, max_at;
            std::vector<int64_t> axes_sum, axes_max;
            std::string sum_src, max_src;
            if (e_name.empty() || !reduced_and_repeated(den, "ml::Sum", shape, &bc2, &sum_at, &axes_sum, &sum_src) || sum_src != e_name) continue;
            const long exp_at = writer_of(e_name);
            auto* ex = elementwise(exp_at, "ml::Exp", false);
            if (!ex || ex->shape() != shape || ex->element() != div->element()) continue;
            const std::string d_name = data_of((size_t) exp_at, "X");
            const long sub_at = d_name.empty() ? -1 : writer_of(d_name);
            auto* sub = elementwise(sub_at, "ml::Sub", true);
            if (!sub || sub->shape() != shape) continue;
            const std::string x_name = data_of((size_t) sub_at, "A"), shift = data_of((size_t) sub_at, "B");
            if (x_name.empty() || !reduced_and_repeated(shift, "ml::Max", shape, &bc1, &max_at, &axes_max, &max_src)) continue;
            if (max_src != x_name || axes_max != axes_sum) continue;
            // program order, and every value in between private to the pattern
            const size_t i_max = (size_t) max_at, i_bc1 = (size_t) bc1, i_sub = (size_t) sub_at, i_exp = (size_t) exp_at, i_sum = (size_t) sum_at, i_bc2 = (size_t) bc2;
            if (!(i_max < i_bc1 && i_bc1 < i_sub && i_sub < i_exp && i_exp < i_sum && i_sum < i_bc2 && i_bc2 < at)) continue;
            const std::string m_name = blocks[i_max].outputs[0].data, s_name = blocks[i_sum].outputs[0].data, y_name = blocks[at].outputs[0].data;
            if (!private_value(m_name, {i_bc1}) || !private_value(shift, {i_sub}) || !private_value(d_name, {i_exp}) ||
                !private_value(e_name, {i_sum, at}) || !private_value(s_name, {i_bc2}) || !private_value(den, {at}))
                continue;
            // X as the Max saw it must be what the Sub sees, and the result must not be looked at before the Div stood
            if (!unwritten_between(sdfg, x_name, i_max, at) || (y_name != x_name && !untouched_between(sdfg, y_name, i_max, at))) continue;
            if (y_name == x_name) continue;   // in place: the softmax kernels allow it, the pattern's readers of X in between do not
            auto node = std::make_unique<tensor::SoftmaxNode>(ImplementationType_NONE, shape, axes_sum, div->element());
            // only a node the mapper takes (RocmLibNodeMapper::try_map): otherwise the seven nodes, which it maps
            // one by one, would become one that it declines
            if ((div->element() != types::PrimitiveType::Float && div->element() != types::PrimitiveType::Double) || !node->adjacent_axes()) continue;
            node->set_element_id(div->element_id());
            Block& last = blocks[at];
            last.node = std::move(node);
            last.inputs.clear();
            ConnectorBinding in;
            in.connector = "X";
            in.data = x_name;
            last.inputs.push_back(in);
            last.outputs[0].connector = "Y";
            // the other six blocks go, highest index first, and their values with them
            for (size_t i : {i_bc2, i_sum, i_exp, i_sub, i_bc1, i_max}) blocks.erase(blocks.begin() + (long) i);
            for (auto& name : {m_name, shift, d_name, e_name, s_name, den}) sdfg.remove_container(name);
            changed = applied = true;
        }
    }
    return applied;
}

bool RocmElementwiseFusionPass::run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager&) {
    StructuredSDFG& sdfg = builder.subject();
    auto& blocks = sdfg.blocks();
    bool applied = false;
    bool changed = true;
    while (changed) {
        changed = false;
        // (1) a Broadcast whose result feeds exactly one operand of one later binary node: the node
        //     reads the small operand itself
        for (size_t i = 0; i < blocks.size() && !changed; i++) {
            auto* bc = dynamic_cast<tensor::BroadcastNode*>(blocks[i].node.get());
            if (!bc || !is_rocm_type(bc->implementation_type())) continue;
            const std::string link = blocks[i].outputs[0].data, source = blocks[i].inputs[0].data;
            const Uses u = uses_of(sdfg, link);
            if (u.readers.size() != 1) continue;
            const size_t j = u.readers[0];
            if (!is_private_link(sdfg, link, i, j) || !unwritten_between(sdfg, source, i, j)) continue;
            auto* consumer = blocks[j].node.get();
            const bool plain = dynamic_cast<tensor::ElementWiseNode*>(consumer) && static_cast<tensor::ElementWiseNode*>(consumer)->is_binary();
            auto* fused = dynamic_cast<ROCMFusedElementWiseNode*>(consumer);
            if (!(plain || (fused && fused->has_b())) || consumer->implementation_type() != bc->implementation_type()) continue;
            // the consumer must not write the small operand it is about to read in a different order
            if (blocks[j].outputs[0].data == source) continue;
            if (plain) make_fused(sdfg, j);
            auto* f = static_cast<ROCMFusedElementWiseNode*>(blocks[j].node.get());
            if (f->shape() != bc->output_shape()) continue;
            const char* connector = blocks[j].input("A")->data == link && !blocks[j].input("A")->is_constant ? "A" : "B";
            auto node = std::make_unique<ROCMFusedElementWiseNode>(
                f->implementation_type(), f->shape(), f->element(), f->binary(),
                std::string(connector) == "A" ? bc->input_shape() : f->a_shape(),
                std::string(connector) == "B" ? bc->input_shape() : f->b_shape(), f->post());
            node->set_element_id(f->element_id());
            blocks[j].node = std::move(node);
            for (auto& in : blocks[j].inputs)
                if (in.connector == connector) in.data = source;
            blocks.erase(blocks.begin() + (long) i);
            sdfg.remove_container(link);
            changed = applied = true;
        }
        // (2) a unary node on a value that only it reads: an epilogue of the elementwise node that made the value
        for (size_t j = 0; j < blocks.size() && !changed; j++) {
            auto* un = dynamic_cast<tensor::ElementWiseNode*>(blocks[j].node.get());
            if (!un || un->is_binary() || !is_rocm_type(un->implementation_type())) continue;
            const ConnectorBinding* x = blocks[j].input("X");
            if (!x || x->is_constant) continue;
            const std::string link = x->data, result = blocks[j].outputs[0].data;
            const Uses u = uses_of(sdfg, link);
            if (u.writers.size() != 1) continue;
            const size_t i = u.writers[0];
            if (!is_private_link(sdfg, link, i, j)) continue;
            auto* producer = blocks[i].node.get();
            const bool plain = dynamic_cast<tensor::ElementWiseNode*>(producer) != nullptr;
            auto* fused = dynamic_cast<ROCMFusedElementWiseNode*>(producer);
            if (!(plain || fused) || producer->implementation_type() != un->implementation_type()) continue;
            // the result is now written where the producer stands: nothing in between may look at it,
            // and the producer must not read it through a repeated (out-of-order) operand
            if (!untouched_between(sdfg, result, i, j)) continue;
            if (plain) make_fused(sdfg, i);
            auto* f = static_cast<ROCMFusedElementWiseNode*>(blocks[i].node.get());
            if (f->post().size() >= 4 || f->shape() != un->shape()) continue;
            bool aliased_repeat = false;
            for (auto& in : blocks[i].inputs)
                if (!in.is_constant && in.data == result) {
                    const auto& s = in.connector == "A" ? f->a_shape() : f->b_shape();
                    if (s != f->shape()) aliased_repeat = true;
                }
            if (aliased_repeat) continue;
            f->post().push_back(un->code());
            blocks[i].outputs[0].data = result;
            blocks.erase(blocks.begin() + (long) j);
            sdfg.remove_container(link);
            changed = applied = true;
        }
        // (3) the elementwise node behind a GEMM: the bias row and a one-instruction activation move into
        //     the GEMM's store; what is left of the chain (other activations) stays an elementwise node
        for (size_t i = 0; i < blocks.size() && !changed; i++) {
            auto* gemm = dynamic_cast<blas::GEMMNode*>(blocks[i].node.get());
            if (!gemm || !is_rocm_type(gemm->implementation_type()) || gemm->has_epilogue()) continue;
            if (gemm->ldc() != gemm->n()) continue;   // the chain sees C as a dense [m, n] array
            const std::string link = blocks[i].outputs[0].data;
            const Container& lc = sdfg.container(link);
            if (lc.is_argument || !lc.transient || link == sdfg.return_container()) continue;
            const Uses u = uses_of(sdfg, link);
            // the GEMM's own "__C" binding counts as a reader only if beta may be non-zero
            const bool reads_c = gemm->reads("__C", blocks[i].inputs);
            std::vector<size_t> readers;
            for (size_t r : u.readers)
                if (r != i || reads_c) readers.push_back(r);
            if (u.writers.size() != 1 || readers.size() != 1 || readers[0] <= i) continue;
            const size_t j = readers[0];
            if (dynamic_cast<tensor::ElementWiseNode*>(blocks[j].node.get())) {
                if (blocks[j].node->implementation_type() != gemm->implementation_type()) continue;
                make_fused(sdfg, j);
            }
            auto* f = dynamic_cast<ROCMFusedElementWiseNode*>(blocks[j].node.get());
            if (!f || f->implementation_type() != gemm->implementation_type()) continue;
            if (f->element() != blas::precision_output_type(gemm->precision())) continue;
            // [.., n] with the leading extents multiplying to m
            const auto& shape = f->shape();
            if (shape.empty() || shape.back() != gemm->n()) continue;
            Expression lead = "1";
            for (size_t d = 0; d + 1 < shape.size(); d++) lead = symbolic::mul(lead, shape[d]);
            if (lead != gemm->m()) continue;
            auto is_row = [&](const std::vector<Expression>& s) {
                if (s.size() != shape.size() || s.back() != gemm->n()) return false;
                for (size_t d = 0; d + 1 < s.size(); d++)
                    if (s[d] != "1") return false;
                return true;
            };
            const ConnectorBinding* a = blocks[j].input("A");
            const ConnectorBinding* b = f->has_b() ? blocks[j].input("B") : nullptr;
            const bool a_is_link = a && !a->is_constant && a->data == link && f->a_shape() == shape;
            const bool b_is_link = b && !b->is_constant && b->data == link && f->b_shape() == shape;
            std::string bias;
            if (f->has_b()) {
                if (f->binary() != "ml::Add" || a_is_link == b_is_link) continue;
                const ConnectorBinding* other = a_is_link ? b : a;
                if (other->is_constant || !sdfg.container(other->data).is_pointer || !is_row(a_is_link ? f->b_shape() : f->a_shape())) continue;
                if (shape.size() > 1 && gemm->m() == "1") continue;   // a [1, n] operand is ambiguous with the full shape
                bias = other->data;
                if (!unwritten_between(sdfg, bias, i, j)) continue;
            } else if (!a_is_link) {
                continue;
            }
            std::vector<std::string> post = f->post();
            std::string activation;
            if (!post.empty() && (post[0] == "ml::ReLU" || post[0] == "ml::Abs")) {
                activation = post[0];
                post.erase(post.begin());
            }
            if (bias.empty() && activation.empty()) continue;
            const std::string result = blocks[j].outputs[0].data;
            if (post.empty()) {
                // the whole chain is in the store: the GEMM writes the chain's result
                if (!untouched_between(sdfg, result, i, j) || result == bias) continue;
                bool operand_is_result = false;
                for (auto& in : blocks[i].inputs)
                    if (!in.is_constant && in.data == result) operand_is_result = true;
                if (operand_is_result) continue;   // A or B would be overwritten while it is read
                gemm->set_epilogue(!bias.empty(), activation);
                for (auto& in : blocks[i].inputs)
                    if (in.connector == "__C") in.data = result;
                blocks[i].outputs[0].data = result;
                if (!bias.empty()) blocks[i].inputs.push_back(make_binding("__bias", bias));
                blocks.erase(blocks.begin() + (long) j);
                sdfg.remove_container(link);
            } else {
                gemm->set_epilogue(!bias.empty(), activation);
                if (!bias.empty()) blocks[i].inputs.push_back(make_binding("__bias", bias));
                auto rest = std::make_unique<ROCMFusedElementWiseNode>(f->implementation_type(), shape, f->element(), "", shape,
                                                                       std::vector<Expression>{}, post);
                rest->set_element_id(f->element_id());
                std::vector<ConnectorBinding> inputs{make_binding("A", link)};
                blocks[j].inputs = std::move(inputs);
                blocks[j].node = std::move(rest);
            }
            changed = applied = true;
        }
    }
    return applied;
}

// ------------------------------------------------------------------------------ offloading

namespace {

bool is_offloading(const Block& b) { return b.node->code() == LibraryNodeType_ROCM_Offloading; }

const ROCMDataOffloadingNode& offloading(const Block& b) { return static_cast<const ROCMDataOffloadingNode&>(*b.node); }

} // namespace

bool RocmOffloadTransform::run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager&) {
    StructuredSDFG& sdfg = builder.subject();
    bool applied = false;
    // indices move while blocks are inserted: walk by position
    for (size_t i = 0; i < sdfg.blocks().size(); i++) {
        if (sdfg.blocks()[i].node->implementation_type() != ImplementationType_ROCMWithoutTransfers) continue;
        if (is_offloading(sdfg.blocks()[i])) continue;
        // already surrounded? (a device container is bound)
        bool on_host = false;
        for (auto& in : sdfg.blocks()[i].inputs)
            if (!in.is_constant && sdfg.container(in.data).storage == "CPU" && sdfg.container(in.data).is_pointer) on_host = true;
        for (auto& out : sdfg.blocks()[i].outputs)
            if (sdfg.container(out.data).storage == "CPU" && sdfg.container(out.data).is_pointer) on_host = true;
        if (!on_host) continue;

        struct Plan {
            std::string host, device;
            Expression bytes;
            bool read = false, written = false;
        };
        std::vector<Plan> plans;
        auto plan_for = [&](const std::string& host) -> Plan& {
            for (auto& p : plans)
                if (p.host == host) return p;
            plans.push_back(Plan{host, "__daisy_rocm_" + std::to_string(sdfg.blocks()[i].node->element_id()) + "_" + host, "", false, false});
            return plans.back();
        };
        {
            const Block& blk = sdfg.blocks()[i];
            for (auto& in : blk.inputs) {
                if (in.is_constant || !sdfg.container(in.data).is_pointer) continue;
                Plan& p = plan_for(in.data);
                p.bytes = blk.node->connector_bytes(in.connector);
                if (blk.node->reads(in.connector, blk.inputs)) p.read = true;
            }
            for (auto& out : blk.outputs) {
                if (!sdfg.container(out.data).is_pointer) continue;   // a scalar result (DOT's __out) stays a host scalar
                Plan& p = plan_for(out.data);
                p.bytes = blk.node->connector_bytes(out.connector);
                p.written = true;
            }
        }
        for (auto& p : plans) {
            Container dev;
            dev.name = p.device;
            dev.is_pointer = true;
            dev.element = sdfg.container(p.host).element;
            dev.transient = true;
            dev.storage = "ROCM_Generic";
            sdfg.add_container(dev, false);
        }
        // rebind the node to the device containers
        for (auto& in : sdfg.blocks()[i].inputs)
            for (auto& p : plans)
                if (!in.is_constant && in.data == p.host) in.data = p.device;
        for (auto& out : sdfg.blocks()[i].outputs)
            for (auto& p : plans)
                if (out.data == p.host) out.data = p.device;
        // the transfers of a node carry its source position
        const structured_control_flow::DebugInfo dbg = sdfg.blocks()[i].debug_info;
        // before: ALLOC (+H2D when the node reads the operand)
        size_t pos = i;
        for (auto& p : plans) {
            if (p.read) {
                sdfg.add_block(std::make_unique<ROCMDataOffloadingNode>(p.bytes, 0, DataTransferDirection::H2D, BufferLifecycle::ALLOC),
                               {make_binding("_src", p.host)}, {make_binding("_dst", p.device)}, pos++).debug_info = dbg;
            } else {
                sdfg.add_block(std::make_unique<ROCMDataOffloadingNode>(p.bytes, 0, DataTransferDirection::NONE, BufferLifecycle::ALLOC),
                               {}, {make_binding("_ret", p.device)}, pos++).debug_info = dbg;
            }
        }
        // the node now sits at `pos`; after it: D2H+FREE for what it wrote, FREE for the rest
        size_t after = pos + 1;
        for (auto& p : plans) {
            if (p.written) {
                sdfg.add_block(std::make_unique<ROCMDataOffloadingNode>(p.bytes, 0, DataTransferDirection::D2H, BufferLifecycle::FREE),
                               {make_binding("_src", p.device)}, {make_binding("_dst", p.host)}, after++).debug_info = dbg;
            }
        }
        for (auto& p : plans) {
            if (!p.written) {
                sdfg.add_block(std::make_unique<ROCMDataOffloadingNode>(p.bytes, 0, DataTransferDirection::NONE, BufferLifecycle::FREE),
                               {make_binding("_ptr", p.device)}, {}, after++).debug_info = dbg;
            }
        }
        i = after - 1;
        applied = true;
    }
    return applied;
}

bool RocmDataTransferMinimizationPass::run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager&) {
    // The root sequence is straight-line code, so the device copy of every host container can be
    // tracked exactly: one forward walk keeps, per host container, the device buffer that holds its
    // current value. An upload from a container whose value already sits in a buffer of the same
    // extent is dropped and its buffer renamed to the first one (however many nodes read it, and
    // whatever lies between them); a node that rewrites a container takes over the buffer the old
    // value lived in; a download is kept only where the host looks at the data before the device
    // writes it again; every buffer is freed once, behind its last use.
    StructuredSDFG& sdfg = builder.subject();
    std::vector<Block> old = std::move(sdfg.blocks());
    std::vector<Block>& out = sdfg.blocks();
    out.clear();
    bool applied = false;

    struct Resident {
        std::string device;
        Expression bytes;
        int device_id = 0;
    };
    std::map<std::string, Resident> current;          // host container -> buffer holding its value
    std::map<std::string, std::string> stale;         // host container whose own memory is out of date -> that buffer
    std::map<std::string, std::string> renamed;       // dropped device container -> the one used instead
    std::map<std::string, Resident> allocated;        // device buffers of the function, in need of a FREE
    std::vector<std::string> allocation_order;

    auto host_side = [&](const Block& b) { return !is_offloading(b) && !is_rocm_impl(b.node->implementation_type()); };
    auto reads_container = [&](const Block& b, const std::string& name) {
        for (auto& in : b.inputs)
            if (!in.is_constant && in.data == name) return true;
        return false;
    };
    auto writes_container = [&](const Block& b, const std::string& name) {
        for (auto& o : b.outputs)
            if (o.data == name) return true;
        return false;
    };
    // does host code look at `host` after position `from` of the old sequence, before the device
    // replaces all of it again?
    auto host_needs = [&](const std::string& host, const Expression& bytes, size_t from) {
        for (size_t j = from; j < old.size(); j++) {
            const Block& b = old[j];
            if (!b.node) continue;
            if (is_offloading(b)) {
                const auto& node = offloading(b);
                if (node.is_d2h() && b.outputs[0].data == host && symbolic::equal(node.size(), bytes)) return false;
                if (node.is_h2d() && b.inputs[0].data == host) {
                    const auto it = current.find(host);
                    // an upload that will not be dropped reads the host memory
                    if (it == current.end() || !symbolic::equal(it->second.bytes, node.size()) || it->second.device_id != node.device_id()) return true;
                }
                continue;
            }
            if (host_side(b) && (reads_container(b, host) || writes_container(b, host))) return true;
        }
        const Container& c = sdfg.container(host);
        return c.is_argument || host == sdfg.return_container();
    };
    auto emit_download = [&](const std::string& host, const Resident& from, const structured_control_flow::DebugInfo& dbg) {
        Block blk;
        blk.element_id = sdfg.next_element_id();
        blk.debug_info = dbg;
        blk.node = std::make_unique<ROCMDataOffloadingNode>(from.bytes, from.device_id, DataTransferDirection::D2H, BufferLifecycle::NO_CHANGE);
        blk.node->set_element_id(sdfg.next_element_id());
        blk.inputs = {make_binding("_src", from.device)};
        blk.outputs = {make_binding("_dst", host)};
        out.push_back(std::move(blk));
    };

    for (size_t i = 0; i < old.size(); i++) {
        Block b = std::move(old[i]);
        old[i].node.reset();
        for (auto& in : b.inputs)
            if (!in.is_constant && renamed.count(in.data)) in.data = renamed[in.data];
        for (auto& o : b.outputs)
            if (renamed.count(o.data)) o.data = renamed[o.data];

        if (!is_offloading(b)) {
            if (host_side(b)) {
                // host code: bring in what it reads, forget device copies of what it writes
                for (auto& in : b.inputs)
                    if (!in.is_constant && stale.count(in.data)) {
                        emit_download(in.data, current.at(in.data), b.debug_info);
                        stale.erase(in.data);
                    }
                for (auto& o : b.outputs) {
                    current.erase(o.data);
                    stale.erase(o.data);
                }
            }
            out.push_back(std::move(b));
            continue;
        }

        const auto& node = offloading(b);
        if (node.is_h2d()) {
            const std::string host = b.inputs[0].data, device = b.outputs[0].data;
            const auto it = current.find(host);
            if (node.is_alloc() && it != current.end() && symbolic::equal(it->second.bytes, node.size()) && it->second.device_id == node.device_id()) {
                renamed[device] = it->second.device;      // the value is on the device already
                applied = true;
                continue;
            }
            if (stale.count(host)) {                      // an upload of another extent: the host memory must be current first
                emit_download(host, current.at(host), b.debug_info);
                stale.erase(host);
            }
            current[host] = Resident{device, node.size(), node.device_id()};
            if (node.is_alloc() && !allocated.count(device)) {
                allocated[device] = current[host];
                allocation_order.push_back(device);
            }
            out.push_back(std::move(b));
            continue;
        }
        if (node.is_d2h()) {
            const std::string device = b.inputs[0].data, host = b.outputs[0].data;
            const Resident here{device, node.size(), node.device_id()};
            current[host] = here;
            if (host_needs(host, node.size(), i + 1)) {
                stale.erase(host);
                emit_download(host, here, b.debug_info);
                out.back().node->set_element_id(b.node->element_id());
                out.back().element_id = b.element_id;
            } else {
                stale[host] = device;
                applied = true;
            }
            continue;                                     // a FREE comes behind the buffer's last use
        }
        if (node.is_alloc()) {
            // a buffer some node is about to fill: the download that follows names the host container
            const std::string device = b.outputs[0].data;
            std::string host;
            for (size_t j = i + 1; j < old.size() && host.empty(); j++) {
                if (!old[j].node || !is_offloading(old[j])) continue;
                if (offloading(old[j]).is_d2h() && old[j].inputs[0].data == device) host = old[j].outputs[0].data;
                else if (offloading(old[j]).is_free() && old[j].inputs[0].data == device) break;
            }
            const auto it = host.empty() ? current.end() : current.find(host);
            if (it != current.end() && symbolic::equal(it->second.bytes, node.size()) && it->second.device_id == node.device_id()) {
                renamed[device] = it->second.device;      // the old value's buffer is overwritten in place
                applied = true;
                continue;
            }
            if (!allocated.count(device)) {
                allocated[device] = Resident{device, node.size(), node.device_id()};
                allocation_order.push_back(device);
            }
            out.push_back(std::move(b));
            continue;
        }
        // a bare FREE: dropped here, placed behind the last use below
        if (node.is_free()) continue;
        out.push_back(std::move(b));
    }

    // one FREE per buffer, behind its last use; a download that is the last use frees as well
    for (auto rit = allocation_order.rbegin(); rit != allocation_order.rend(); ++rit) {
        const Resident& r = allocated.at(*rit);
        size_t last = out.size();
        for (size_t j = out.size(); j-- > 0;) {
            if (reads_container(out[j], r.device) || writes_container(out[j], r.device)) {
                last = j;
                break;
            }
        }
        if (last == out.size()) continue;
        Block& user = out[last];
        if (is_offloading(user) && offloading(user).is_d2h() && !offloading(user).is_free() && user.inputs[0].data == r.device) {
            auto both = std::make_unique<ROCMDataOffloadingNode>(r.bytes, r.device_id, DataTransferDirection::D2H, BufferLifecycle::FREE);
            both->set_element_id(user.node->element_id());
            user.node = std::move(both);
            continue;
        }
        Block blk;
        blk.element_id = sdfg.next_element_id();
        blk.debug_info = user.debug_info;
        blk.node = std::make_unique<ROCMDataOffloadingNode>(r.bytes, r.device_id, DataTransferDirection::NONE, BufferLifecycle::FREE);
        blk.node->set_element_id(sdfg.next_element_id());
        blk.inputs = {make_binding("_ptr", r.device)};
        // behind the other FREEs that already follow this position
        size_t pos = last + 1;
        while (pos < out.size() && is_offloading(out[pos]) && offloading(out[pos]).transfer_direction() == DataTransferDirection::NONE &&
               offloading(out[pos]).is_free())
            pos++;
        out.insert(out.begin() + (long) pos, std::move(blk));
    }

    // device containers that were renamed away, and host memory of transients nobody touches any more
    for (auto& kv : renamed) {
        bool used = false;
        for (auto& b : out)
            if (reads_container(b, kv.first) || writes_container(b, kv.first)) used = true;
        if (!used && sdfg.exists(kv.first)) sdfg.remove_container(kv.first);
    }
    std::vector<std::string> names;
    for (auto& kv : sdfg.containers()) names.push_back(kv.first);
    for (auto& name : names) {
        Container& c = sdfg.container(name);
        if (!c.transient || c.is_argument || c.storage != "CPU" || c.size_bytes.empty() || name == sdfg.return_container()) continue;
        bool used = false;
        for (auto& b : out)
            if (reads_container(b, name) || writes_container(b, name)) used = true;
        if (!used) c.size_bytes.clear();
    }
    return applied;
}

void rocm_scheduling_passes(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager,
                            const std::string& category, const ScheduleOptions& options) {
    (void) category;  // "desktop" / "server": one code path, kept for the interface
    register_rocm_plugin();
    if (options.offload != "function" && options.offload != "node" && options.offload != "none")
        throw std::invalid_argument("rocm: option offload must be 'function', 'node' or 'none'");
    const std::string impl = options.offload == "node" ? ImplementationType_ROCMWithTransfers : ImplementationType_ROCMWithoutTransfers;
    if (options.match_softmax) {
        RocmSoftmaxPatternPass pattern;
        pattern.run_pass(builder, analysis_manager);
    }
    auto mapper = std::make_shared<RocmLibNodeMapper>(impl);
    for (auto& blk : builder.subject().blocks()) {
        if (!is_math_node(*blk.node) || is_rocm_impl(blk.node->implementation_type())) continue;
        if (!mapper->try_map(builder, analysis_manager, *blk.node) && options.require_all_mapped)
            throw InvalidSDFGException("rocm target cannot map node " + mapper->last_decline_reason() +
                                       " (this target has no CPU lowering)");
    }
    if (options.fuse_elementwise) {
        RocmElementwiseFusionPass fusion;
        fusion.run_pass(builder, analysis_manager);
    }
    if (options.fuse_elementwise && options.fuse_maps) {
        RocmMapFusionPass maps;
        maps.run_pass(builder, analysis_manager);
    }
    if (options.offload == "none") {
        // the caller's pointers are device pointers, so every array the nodes touch lives in HBM:
        // arguments are relabelled, transients are allocated and freed on the device around their uses
        // (a host malloc'ed transient handed to a kernel would fault)
        StructuredSDFG& sdfg = builder.subject();
        std::vector<std::string> transients;
        for (auto& kv : sdfg.containers()) {
            if (!kv.second.is_pointer) continue;
            Container& c = sdfg.container(kv.first);
            c.storage = "ROCM_Generic";
            if (c.transient && !c.is_argument && !c.size_bytes.empty()) transients.push_back(kv.first);
        }
        for (auto& name : transients) {
            auto touches = [&](const Block& b) {
                for (auto& in : b.inputs)
                    if (!in.is_constant && in.data == name) return true;
                for (auto& out : b.outputs)
                    if (out.data == name) return true;
                return false;
            };
            size_t first = (size_t) -1, last = 0;
            for (size_t i = 0; i < sdfg.blocks().size(); i++)
                if (touches(sdfg.blocks()[i])) {
                    if (first == (size_t) -1) first = i;
                    last = i;
                }
            Container& c = sdfg.container(name);
            const Expression bytes = c.size_bytes;
            c.size_bytes.clear();  // no host allocation
            if (first == (size_t) -1) continue;
            sdfg.add_block(std::make_unique<ROCMDataOffloadingNode>(bytes, 0, DataTransferDirection::NONE, BufferLifecycle::FREE),
                           {make_binding("_ptr", name)}, {}, last + 1);
            sdfg.add_block(std::make_unique<ROCMDataOffloadingNode>(bytes, 0, DataTransferDirection::NONE, BufferLifecycle::ALLOC),
                           {}, {make_binding("_ret", name)}, first);
        }
    }
    if (options.offload == "function") {
        RocmOffloadTransform offload;
        offload.run_pass(builder, analysis_manager);
        RocmDataTransferMinimizationPass minimize;
        minimize.run_pass(builder, analysis_manager);
    }
    analysis_manager.invalidate_all();
}

} // namespace sdfg::rocm
