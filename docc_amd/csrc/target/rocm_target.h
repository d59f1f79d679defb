// The `rocm` target: plugin registration, the library-node mapper, the
// offloading transform with transfer minimisation, and the dispatchers that
// print host C++ against the thin HIP runtime (include/docc_rocm_rt.h) and the
// kernel launchers (include/docc_rocm_ops.h).
//
// Structure follows the two device targets of the reference:
//   ET-SoC  targets/et/src/et/target.cpp:21-47 (register_plugin, scheduling passes),
//           targets/et/src/et/et_lib_node_mapper.cpp:10-25 (TargetMapper::try_map),
//           targets/et/src/et/blas/gemm.cpp:132-205 (WithTransfers dispatcher);
//   CUDA    opt/include/sdfg/targets/cuda/plugin.h:20-105 (register_cuda_plugin),
//           opt/src/targets/cuda/blas/gemm.cpp:33-185 (With/WithoutTransfers dispatchers),
//           opt/src/targets/cuda/cuda_data_offloading_node.cpp:139-173 (transfer node dispatcher),
//           opt/src/transformations/offloading/offload_transform.cpp:86-140 and
//           opt/src/passes/offloading/data_transfer_minimization_pass.cpp (transfer elimination).
#pragma once

#include "codegen.h"

namespace sdfg::rocm {

// Registers (idempotently) the rocm serializers and dispatchers in the global registries.
void register_rocm_plugin();
void register_plugin(plugins::Context& context);
extern const plugins::Plugin rocm_plugin;

// Maps GEMM / ml::MatMul / ml::Softmax / ml::Conv / ml::Attention nodes whose dtype and layout the
// kernels support to `implementation_type` (ROCMWithTransfers or ROCMWithoutTransfers);
// declines (returns false, node untouched) otherwise and records why.
class RocmLibNodeMapper : public plugins::TargetMapper {
public:
    explicit RocmLibNodeMapper(std::string implementation_type = ImplementationType_ROCMWithTransfers)
        : implementation_type_(std::move(implementation_type)) {}
    bool try_map(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager,
                 data_flow::LibraryNode& node) const override;
    // why the last declined node was declined ("" if none)
    const std::string& last_decline_reason() const { return reason_; }

private:
    std::string implementation_type_;
    mutable std::string reason_;
};

// The mapper's factory as a docc plugin hands it over (plugins::TargetMapperFactory, reference
// sdfg/include/sdfg/plugins/target_mapping.h:24-30): target "rocm", one factory per implementation type.
// register_plugin() puts the ROCMWithoutTransfers one (the default schedule) into plugins::TargetMapperRegistry.
class RocmLibNodeMapperFactory : public plugins::TargetMapperFactory {
public:
    explicit RocmLibNodeMapperFactory(std::string implementation_type = ImplementationType_ROCMWithoutTransfers, int priority = 100)
        : implementation_type_(std::move(implementation_type)), priority_(priority) {}
    std::unique_ptr<plugins::TargetMapper> create() const override { return std::make_unique<RocmLibNodeMapper>(implementation_type_); }
    int priority() override { return priority_; }
    const std::string& for_target() const override;

private:
    std::string implementation_type_;
    int priority_;
};

// Surrounds every ROCMWithoutTransfers node with offloading blocks (ALLOC[+H2D] before,
// [D2H+]FREE after) on device containers `__daisy_rocm_<element id>_<container>`.
class RocmOffloadTransform {
public:
    std::string name() { return "RocmOffloadTransform"; }
    bool run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager);
};

// Removes D2H(+FREE) / H2D(+ALLOC) pairs on the same host container between consecutive
// device nodes so that intermediates stay in HBM; drops the D2H altogether when the host
// never looks at the container, and the host allocation of such transients with it.
class RocmDataTransferMinimizationPass {
public:
    std::string name() { return "RocmDataTransferMinimization"; }
    bool run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager);
};

// Folds a Broadcast node into the binary elementwise node that consumes it and unary elementwise
// nodes into the elementwise node that produces their operand (ROCMFusedElementWise, one kernel
// per chain), when the value in between is a transient nothing else looks at. Counterpart of
// the reference's MapFusion over the expanded Maps (python/bindings/py_structured_sdfg.cpp:258-260).
class RocmElementwiseFusionPass {
public:
    std::string name() { return "RocmElementwiseFusion"; }
    bool run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager);
};

// Merges blocks of elementwise kind (tensor elementwise nodes, ROCMFusedElementWise, ml::Broadcast, ROCMMap with one
// result) that the fusion pass above left as separate launches into one ROCMMap node, when the value in between is
// a transient that only the later block reads: one generated kernel per chain, whatever its length and however many
// of its operands are repeated rows or scalars. The merged block stands where the later one stood. Runs after
// RocmElementwiseFusionPass, so a chain the prebuilt fused kernel takes whole needs no device compiler.
class RocmMapFusionPass {
public:
    std::string name() { return "RocmMapFusion"; }
    bool run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager);
};

// Recognises softmax written out in its pieces - the form numpy code takes, and what the reference's SoftmaxNode
// expands to (softmax_node.cpp:142-252): m = Max(X, axes, keepdims); e = Exp(X - broadcast(m)); Y = e / broadcast(Sum(e,
// axes, keepdims)) - and replaces the seven nodes by one ml::Softmax when every value in between is a transient that
// nothing else looks at. Runs before the mapping (on nodes without an implementation type).
class RocmSoftmaxPatternPass {
public:
    std::string name() { return "RocmSoftmaxPattern"; }
    bool run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager);
};

// The kernel a ROCMMap node becomes (map_kernel.cpp) and what the host side needs to launch it: the loops as the
// kernel sees them (adjacent loops that every operand walks as one are merged), the operands in parameter order,
// and the source text. Kernel parameters: one pointer per operand, the scalar operands by value, one `long long` per
// bound, then one `long long` per stride that is neither 0 nor 1 (operand by operand, loop by loop). The text defines
// `<kernel_name>_s32` / `_s64` (one iteration per thread, indices in 32 / 64 bits) and, when some operand is contiguous
// along the innermost loop, `_v32` / `_v64` (`vector_width` iterations per thread, 128-bit accesses).
struct RocmMapKernelPlan {
    struct Operand {
        std::string connector;
        bool write;
        types::PrimitiveType element;
        std::vector<Expression> strides;   // per merged loop
        Expression extent;
        bool vector;                       // contiguous along the innermost loop
        bool streamed;                     // no loop repeats it
    };
    std::string kernel_name;
    std::vector<Expression> bounds;
    std::vector<Operand> operands;
    int vector_width = 1;
    std::string source;
};
RocmMapKernelPlan plan_rocm_map_kernel(const ROCMMapNode& node, const std::string& kernel_name);

struct ScheduleOptions {
    // "function": nodes run WithoutTransfers between hoisted, minimised transfers (default)
    // "node":     every node copies its operands itself (ROCMWithTransfers)
    // "none":     the caller passes device pointers; no transfers are generated
    std::string offload = "function";
    // refuse to leave a math node unmapped (there is no CPU lowering in this target)
    bool require_all_mapped = true;
    // run RocmElementwiseFusionPass after the mapping
    bool fuse_elementwise = true;
    // run RocmSoftmaxPatternPass before the mapping
    bool match_softmax = true;
    // run RocmMapFusionPass after the elementwise fusion, if that runs (its kernels are compiled by hipcc when the
    // program is)
    bool fuse_maps = true;
};

// The scheduling entry of the target: mapping pass (+ offloading passes).
void rocm_scheduling_passes(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager& analysis_manager,
                            const std::string& category, const ScheduleOptions& options);

} // namespace sdfg::rocm
