// Kernel text for a ROCMMap node: the counterpart of the snippet the reference's CUDAMapDispatcher writes for an
// offloaded Map nest (opt/src/targets/cuda/cuda_map_dispatcher.cpp:42-168 kernel preamble and body, :180-213 the
// `if (indvar < bound)` guard). There the body is printed by the generic sequence dispatcher and the nest maps onto
// the x / y / z block dimensions; here the nest is flattened onto one grid dimension, one thread takes a short run of
// the innermost loop, and operands that are contiguous along that loop move as 128-bit vectors.
#include <sstream>

#include "rocm_target.h"

namespace sdfg::rocm {

namespace {

// bf16 tensors are loaded, converted by an assignment (the compiler's conversions: exact to float, to nearest even back) and stored
const char* c_type(types::PrimitiveType t) {
    return t == types::PrimitiveType::Double ? "double" : t == types::PrimitiveType::BFloat ? "__bf16" : "float";
}

bool is_literal_stride(const Expression& s) { return s == "0" || s == "1"; }

// `stride of the outer loop` == `extent of the inner loop` * `stride of the inner loop`, in the spelling the importer
// composes strides with (interchange.cpp, layout_of): the two loops are then one walk through the operand
bool walks_as_one(const Expression& outer, const Expression& inner, const Expression& inner_extent) {
    if (outer == "0" && inner == "0") return true;
    if (inner == "0" || outer == "0") return false;
    return outer == (inner == "1" ? inner_extent : "(" + inner_extent + ")*" + inner);
}

std::string spell(const ROCMMapNode::Statement& st) {
    const bool f32 = st.type != types::PrimitiveType::Double;
    const std::string T = c_type(st.type);
    auto arg = [&](size_t i) {
        const std::string& a = st.args[i];
        return "(" + T + ") (" + (a[0] == '#' ? a.substr(1) : a) + ")";
    };
    if (st.op == "assign") return arg(0);
    if (st.op == "fp_neg") return "-" + arg(0);
    if (st.op == "fp_add") return arg(0) + " + " + arg(1);
    if (st.op == "fp_sub") return arg(0) + " - " + arg(1);
    if (st.op == "fp_mul") return arg(0) + " * " + arg(1);
    if (st.op == "fp_div") return arg(0) + " / " + arg(1);
    if (st.op == "fp_rem") return std::string(f32 ? "fmodf(" : "fmod(") + arg(0) + ", " + arg(1) + ")";
    // the reference prints `a * b + c` in one expression, which its compiler contracts (-ffp-contract=on is clang's
    // default); the kernels are compiled without contraction so that separate tasklets stay separate roundings,
    // and the one fused operation is asked for by name
    if (st.op == "fp_fma" || st.op == "fma") return std::string(f32 ? "__builtin_fmaf(" : "__builtin_fma(") + arg(0) + ", " + arg(1) + ", " + arg(2) + ")";
    std::string call = st.op + (f32 ? "f(" : "(");
    for (size_t i = 0; i < st.args.size(); i++) call += (i ? ", " : "") + arg(i);
    return call + ")";
}

} // namespace

RocmMapKernelPlan plan_rocm_map_kernel(const ROCMMapNode& node, const std::string& kernel_name) {
    RocmMapKernelPlan plan;
    plan.kernel_name = kernel_name;
    for (auto& r : node.reads()) plan.operands.push_back({r.connector, false, r.element, r.strides, r.extent, false, true});
    for (auto& w : node.writes()) plan.operands.push_back({w.connector, true, w.element, w.strides, w.extent, false, true});
    plan.bounds = node.bounds();

    // adjacent loops that every operand walks as one become one loop (a nest over dense operands of one shape
    // collapses to a single loop and the kernel divides nothing)
    for (size_t l = plan.bounds.size(); l-- > 1;) {
        bool all = true;
        for (auto& op : plan.operands) all = all && walks_as_one(op.strides[l - 1], op.strides[l], plan.bounds[l]);
        if (!all) continue;
        plan.bounds[l - 1] = "(" + plan.bounds[l - 1] + ")*(" + plan.bounds[l] + ")";
        plan.bounds.erase(plan.bounds.begin() + (long) l);
        for (auto& op : plan.operands) {
            op.strides[l - 1] = op.strides[l];
            op.strides.erase(op.strides.begin() + (long) l);
        }
    }
    const size_t depth = plan.bounds.size();
    bool any_double = false, any_vector = false;
    for (auto& op : plan.operands) {
        any_double = any_double || op.element == types::PrimitiveType::Double;
        op.vector = op.strides[depth - 1] == "1";
        any_vector = any_vector || op.vector;
        for (auto& s : op.strides) op.streamed = op.streamed && s != "0";
    }
    plan.vector_width = any_vector ? (any_double ? 2 : 4) : 1;

    // ---- parameters: operand pointers, scalars, bounds, the strides that are not 0 or 1
    std::ostringstream params, args;
    for (size_t i = 0; i < plan.operands.size(); i++) {
        auto& op = plan.operands[i];
        params << (i ? ", " : "") << (op.write ? "" : "const ") << c_type(op.element) << "* p_" << op.connector;
        args << (i ? ", " : "") << "p_" << op.connector;
    }
    for (auto& s : node.scalars()) {
        params << ", " << c_type(s.element) << " " << s.connector;
        args << ", " << s.connector;
    }
    for (size_t l = 0; l < depth; l++) {
        params << ", long long b" << l;
        args << ", b" << l;
    }
    for (auto& op : plan.operands)
        for (size_t l = 0; l < depth; l++)
            if (!is_literal_stride(op.strides[l])) {
                params << ", long long st_" << op.connector << "_" << l;
                args << ", st_" << op.connector << "_" << l;
            }

    std::ostringstream s;
    s << "// generated by the docc rocm target for gfx950: " << kernel_name << std::endl;
    s << "#include <hip/hip_runtime.h>" << std::endl << std::endl;
    s << "namespace {" << std::endl << std::endl;
    s << "template <typename T, int N> struct docc_vec { typedef T type __attribute__((ext_vector_type(N))); };" << std::endl;
    s << "template <typename T> struct docc_vec<T, 1> { typedef T type; };" << std::endl << std::endl;
    s << "// N consecutive elements; `streamed`: met once by the whole grid, so the caches need not keep them" << std::endl;
    s << "template <typename T, int N, bool streamed>" << std::endl;
    s << "__device__ __forceinline__ void docc_load(const T* p, T (&v)[N]) {" << std::endl;
    s << "    typedef typename docc_vec<T, N>::type V;" << std::endl;
    s << "    const V x = streamed ? __builtin_nontemporal_load((const V*) p) : *(const V*) p;" << std::endl;
    s << "    if constexpr (N == 1) v[0] = x;" << std::endl;
    s << "    else" << std::endl;
    s << "        for (int i = 0; i < N; i++) v[i] = x[i];" << std::endl;
    s << "}" << std::endl << std::endl;
    s << "template <typename T, int N>" << std::endl;
    s << "__device__ __forceinline__ void docc_store(T* p, const T (&v)[N]) {" << std::endl;
    s << "    typedef typename docc_vec<T, N>::type V;" << std::endl;
    s << "    V x;" << std::endl;
    s << "    if constexpr (N == 1) x = v[0];" << std::endl;
    s << "    else" << std::endl;
    s << "        for (int i = 0; i < N; i++) x[i] = v[i];" << std::endl;
    s << "    __builtin_nontemporal_store(x, (V*) p);" << std::endl;
    s << "}" << std::endl << std::endl;

    s << "// one thread: V consecutive iterations of the innermost loop; I: the type indices are computed in" << std::endl;
    s << "template <typename I, int V>" << std::endl;
    s << "__device__ __forceinline__ void docc_nest(" << params.str() << ") {" << std::endl;
    s << "    const I inner = (I) b" << depth - 1 << " / V;" << std::endl;
    s << "    I total = inner;" << std::endl;
    for (size_t l = 0; l + 1 < depth; l++) s << "    total *= (I) b" << l << ";" << std::endl;
    s << "    const I gid = (I) blockIdx.x * (I) 256 + (I) threadIdx.x;" << std::endl;
    s << "    if (gid < total) {" << std::endl;   // the guard of the reference's kernels (cuda_map_dispatcher.cpp:208-213)
    if (depth == 1) {
        s << "        const I i0 = gid * V;" << std::endl;
    } else {
        s << "        I rest = gid;" << std::endl;
        s << "        const I i" << depth - 1 << " = (rest % inner) * V;" << std::endl;
        s << "        rest /= inner;" << std::endl;
        for (size_t l = depth - 1; l-- > 1;) {
            s << "        const I i" << l << " = rest % (I) b" << l << ";" << std::endl;
            s << "        rest /= (I) b" << l << ";" << std::endl;
        }
        s << "        const I i0 = rest;" << std::endl;
    }
    for (auto& op : plan.operands) {
        s << "        const I o_" << op.connector << " = (I) 0";
        for (size_t l = 0; l < depth; l++) {
            if (op.strides[l] == "0") continue;
            s << " + i" << l;
            if (op.strides[l] != "1") s << " * (I) st_" << op.connector << "_" << l;
        }
        s << ";" << std::endl;
    }
    for (auto& op : plan.operands) {
        const std::string T = c_type(op.element), c = op.connector;
        s << "        " << T << " e_" << c << "[V];" << std::endl;
        if (op.write) continue;
        const Expression& in = op.strides[depth - 1];
        if (in == "1") {
            s << "        docc_load<" << T << ", V, " << (op.streamed ? "true" : "false") << ">(p_" << c << " + o_" << c << ", e_" << c << ");" << std::endl;
        } else if (in == "0") {
            s << "        for (int v = 0; v < V; v++) e_" << c << "[v] = p_" << c << "[o_" << c << "];" << std::endl;
        } else {
            s << "        for (int v = 0; v < V; v++) e_" << c << "[v] = p_" << c << "[o_" << c << " + (I) v * (I) st_" << c << "_" << depth - 1 << "];" << std::endl;
        }
    }
    s << "#pragma unroll" << std::endl;
    s << "        for (int v = 0; v < V; v++) {" << std::endl;
    for (auto& r : node.reads()) s << "            const " << c_type(r.element) << " " << r.connector << " = e_" << r.connector << "[v];" << std::endl;
    for (auto& st : node.statements()) s << "            const " << c_type(st.type) << " " << st.out << " = " << spell(st) << ";" << std::endl;
    for (auto& w : node.writes())
        s << "            e_" << w.connector << "[v] = (" << c_type(w.element) << ") (" << (w.value[0] == '#' ? w.value.substr(1) : w.value) << ");" << std::endl;
    s << "        }" << std::endl;
    for (auto& op : plan.operands) {
        if (!op.write) continue;
        const std::string T = c_type(op.element), c = op.connector;
        const Expression& in = op.strides[depth - 1];
        if (in == "1")
            s << "        docc_store<" << T << ", V>(p_" << c << " + o_" << c << ", e_" << c << ");" << std::endl;
        else
            s << "        for (int v = 0; v < V; v++) p_" << c << "[o_" << c << " + (I) v * (I) st_" << c << "_" << depth - 1 << "] = e_" << c << "[v];" << std::endl;
    }
    s << "    }" << std::endl;
    s << "}" << std::endl << std::endl;
    s << "} // namespace" << std::endl << std::endl;

    // variants: s / v = one or `vector_width` iterations per thread, 32 / 64 = the index type
    struct Variant {
        const char* suffix;
        const char* index;
        bool vector;
    };
    const Variant variants[] = {{"_s32", "unsigned int", false}, {"_s64", "unsigned long long", false}, {"_v32", "unsigned int", true},
                                {"_v64", "unsigned long long", true}};
    for (auto& v : variants) {
        if (v.vector && plan.vector_width == 1) continue;
        s << "extern \"C\" __global__ void __launch_bounds__(256) " << kernel_name << v.suffix << "(" << params.str() << ") {" << std::endl;
        s << "    docc_nest<" << v.index << ", " << (v.vector ? plan.vector_width : 1) << ">(" << args.str() << ");" << std::endl;
        s << "}" << std::endl << std::endl;
    }
    plan.source = s.str();
    return plan;
}

} // namespace sdfg::rocm
