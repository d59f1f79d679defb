#include "sdfg_lite.h"

#include <algorithm>
#include <cstdlib>
#include <mutex>

namespace sdfg {

// ------------------------------------------------------------------ types

namespace types {

namespace {
struct Entry {
    PrimitiveType t;
    const char* name;
    size_t size;
};
const Entry kTypes[] = {
    {PrimitiveType::Void, "Void", 0},     {PrimitiveType::Bool, "Bool", 1},     {PrimitiveType::Int8, "Int8", 1},
    {PrimitiveType::Int16, "Int16", 2},   {PrimitiveType::Int32, "Int32", 4},   {PrimitiveType::Int64, "Int64", 8},
    {PrimitiveType::UInt8, "UInt8", 1},   {PrimitiveType::UInt16, "UInt16", 2}, {PrimitiveType::UInt32, "UInt32", 4},
    {PrimitiveType::UInt64, "UInt64", 8}, {PrimitiveType::Half, "Half", 2},     {PrimitiveType::BFloat, "BFloat", 2},
    {PrimitiveType::Float, "Float", 4},   {PrimitiveType::Double, "Double", 8},
};
} // namespace

const char* primitive_type_to_string(PrimitiveType t) {
    for (auto& e : kTypes)
        if (e.t == t) return e.name;
    return "Void";
}

PrimitiveType primitive_type_from_string(const std::string& s) {
    for (auto& e : kTypes)
        if (s == e.name) return e.t;
    throw InvalidSDFGException("unknown primitive type '" + s + "'");
}

size_t primitive_type_size(PrimitiveType t) {
    for (auto& e : kTypes)
        if (e.t == t) return e.size;
    return 0;
}

bool is_floating_point(PrimitiveType t) {
    return t == PrimitiveType::Half || t == PrimitiveType::BFloat || t == PrimitiveType::Float || t == PrimitiveType::Double;
}

} // namespace types

// --------------------------------------------------------------- symbolic

namespace symbolic {

bool is_integer(const Expression& e, int64_t* value) {
    if (e.empty()) return false;
    char* end = nullptr;
    long long v = std::strtoll(e.c_str(), &end, 10);
    if (end == e.c_str() || *end != 0) return false;
    if (value) *value = v;
    return true;
}

Expression integer(int64_t v) { return std::to_string(v); }

static bool is_atom(const Expression& e) {
    for (char c : e)
        if (!(std::isalnum((unsigned char) c) || c == '_')) return false;
    return !e.empty();
}

Expression mul(const Expression& a, const Expression& b) {
    int64_t x, y;
    const bool ia = is_integer(a, &x), ib = is_integer(b, &y);
    if (ia && ib) return integer(x * y);
    if (ia && x == 1) return b;
    if (ib && y == 1) return a;
    if ((ia && x == 0) || (ib && y == 0)) return "0";
    return (is_atom(a) ? a : "(" + a + ")") + "*" + (is_atom(b) ? b : "(" + b + ")");
}

Expression product(const std::vector<Expression>& v, size_t begin, size_t end) {
    Expression p = "1";
    for (size_t i = begin; i < end; i++) p = mul(p, v[i]);
    return p;
}

namespace {

// integer polynomials over the symbols: sorted symbol list -> coefficient
using Polynomial = std::map<std::vector<std::string>, int64_t>;

struct PolynomialParser {
    const std::string& text;
    size_t at = 0;
    bool ok = true;

    void skip() {
        while (at < text.size() && std::isspace((unsigned char) text[at])) at++;
    }
    static Polynomial times(const Polynomial& a, const Polynomial& b) {
        Polynomial out;
        for (auto& x : a)
            for (auto& y : b) {
                std::vector<std::string> symbols = x.first;
                symbols.insert(symbols.end(), y.first.begin(), y.first.end());
                std::sort(symbols.begin(), symbols.end());
                out[symbols] += x.second * y.second;
            }
        return out;
    }
    Polynomial factor() {
        skip();
        Polynomial p;
        if (at >= text.size()) {
            ok = false;
        } else if (text[at] == '(') {
            at++;
            p = sum();
            skip();
            if (at < text.size() && text[at] == ')') at++;
            else ok = false;
        } else if (text[at] == '-') {
            at++;
            p = times(Polynomial{{{}, -1}}, factor());
        } else if (std::isdigit((unsigned char) text[at])) {
            int64_t v = 0;
            while (at < text.size() && std::isdigit((unsigned char) text[at])) v = v * 10 + (text[at++] - '0');
            p[{}] = v;
        } else if (std::isalpha((unsigned char) text[at]) || text[at] == '_') {
            std::string name;
            while (at < text.size() && (std::isalnum((unsigned char) text[at]) || text[at] == '_')) name += text[at++];
            skip();
            if (at < text.size() && text[at] == '(') ok = false;   // a call
            p[{name}] = 1;
        } else {
            ok = false;
        }
        return p;
    }
    Polynomial product() {
        Polynomial p = factor();
        for (skip(); ok && at < text.size() && text[at] == '*'; skip()) {
            at++;
            p = times(p, factor());
        }
        return p;
    }
    Polynomial sum() {
        Polynomial p = product();
        for (skip(); ok && at < text.size() && (text[at] == '+' || text[at] == '-'); skip()) {
            const int64_t sign = text[at++] == '+' ? 1 : -1;
            for (auto& term : product()) p[term.first] += sign * term.second;
        }
        return p;
    }
    bool parse(Polynomial* out) {
        Polynomial p = sum();
        skip();
        if (!ok || at != text.size()) return false;
        for (auto it = p.begin(); it != p.end();) it = it->second == 0 ? p.erase(it) : std::next(it);
        *out = std::move(p);
        return true;
    }
};

} // namespace

bool equal(const Expression& a, const Expression& b) {
    if (a == b) return true;
    Polynomial pa, pb;
    PolynomialParser parse_a{a}, parse_b{b};
    return parse_a.parse(&pa) && parse_b.parse(&pb) && pa == pb;
}

} // namespace symbolic

namespace {

using json::Array;
using json::Object;
using json::Value;

Value exprs_to_json(const std::vector<Expression>& v) {
    Array a;
    for (auto& e : v) a.emplace_back(e);
    return Value(std::move(a));
}

std::vector<Expression> exprs_from_json(const Value& v) {
    std::vector<Expression> out;
    for (auto& e : v.as_array()) out.push_back(e.as_expression());
    return out;
}

Expression product(const std::vector<Expression>& v, size_t begin, size_t end) { return symbolic::product(v, begin, end); }

Expression bytes_of(const Expression& elems, types::PrimitiveType t) {
    return symbolic::mul(elems, symbolic::integer((int64_t) types::primitive_type_size(t)));
}

std::string impl_of(const Value& j) {
    const Value* v = j.find("implementation_type");
    return v ? v->as_string() : ImplementationType_NONE;
}

} // namespace

// ------------------------------------------------------------------- GEMM

namespace math::blas {

types::PrimitiveType precision_input_type(BLAS_Precision p) {
    switch (p) {
        case h: return types::PrimitiveType::Half;
        case s: return types::PrimitiveType::Float;
        case d: return types::PrimitiveType::Double;
        case b: return types::PrimitiveType::BFloat;
        default: throw InvalidSDFGException("GEMM: complex precisions are not supported");
    }
}

types::PrimitiveType precision_output_type(BLAS_Precision p) {
    return p == b ? types::PrimitiveType::Float : precision_input_type(p);
}

GEMMNode::GEMMNode(std::string implementation_type, BLAS_Precision precision, BLAS_Layout layout, BLAS_Transpose trans_a,
                   BLAS_Transpose trans_b, Expression m, Expression n, Expression k, Expression lda, Expression ldb,
                   Expression ldc)
    // connectors as in the reference (gemm_node.cpp:29-40)
    : LibraryNode(LibraryNodeType_GEMM, {"__C"}, {"__A", "__B", "__C", "__alpha", "__beta"}, false,
                  std::move(implementation_type)),
      precision_(precision), layout_(layout), trans_a_(trans_a), trans_b_(trans_b), m_(std::move(m)), n_(std::move(n)),
      k_(std::move(k)), lda_(std::move(lda)), ldb_(std::move(ldb)), ldc_(std::move(ldc)) {}

void GEMMNode::set_epilogue(bool bias, std::string activation) {
    if (bias && !epilogue_bias_) inputs_.push_back("__bias");
    if (!bias && epilogue_bias_) inputs_.erase(std::remove(inputs_.begin(), inputs_.end(), std::string("__bias")), inputs_.end());
    epilogue_bias_ = bias;
    epilogue_activation_ = std::move(activation);
}

void GEMMNode::validate() const {
    if (precision_ != h && precision_ != s && precision_ != d && precision_ != b)
        throw InvalidSDFGException("GEMM: unsupported precision");
    if (layout_ != RowMajor && layout_ != ColMajor) throw InvalidSDFGException("GEMM: bad layout code");
    for (auto t : {trans_a_, trans_b_})
        if (t != No && t != Trans && t != ConjTrans) throw InvalidSDFGException("GEMM: bad transpose code");
    for (auto* e : {&m_, &n_, &k_, &lda_, &ldb_, &ldc_})
        if (e->empty()) throw InvalidSDFGException("GEMM: empty dimension expression");
    if (!epilogue_activation_.empty() && epilogue_activation_ != "ml::ReLU" && epilogue_activation_ != "ml::Abs")
        throw InvalidSDFGException("GEMM: only ml::ReLU and ml::Abs can be part of the store, not " + epilogue_activation_);
}

Expression GEMMNode::flop() const {
    // 2*m*n*k multiply-adds plus the alpha/beta epilogue (reference gemm_node.cpp:337-356)
    return "2*" + symbolic::mul(symbolic::mul(m_, n_), k_) + " + 2*" + symbolic::mul(m_, n_);
}

void GEMMNode::to_json(Value& j) const {
    // keys as in GEMMNodeSerializer (reference gemm_node.cpp:387-405)
    j.set("precision", (int64_t) precision_);
    j.set("layout", (int64_t) layout_);
    j.set("trans_a", (int64_t) trans_a_);
    j.set("trans_b", (int64_t) trans_b_);
    j.set("m", m_);
    j.set("n", n_);
    j.set("k", k_);
    j.set("lda", lda_);
    j.set("ldb", ldb_);
    j.set("ldc", ldc_);
    if (has_epilogue()) {
        j.set("epilogue_bias", epilogue_bias_);
        j.set("epilogue_activation", epilogue_activation_);
    }
}

std::unique_ptr<GEMMNode> GEMMNode::from_json(const Value& j) {
    auto node = std::make_unique<GEMMNode>(impl_of(j), (BLAS_Precision) j.at("precision").as_int(),
                                           (BLAS_Layout) j.at("layout").as_int(), (BLAS_Transpose) j.at("trans_a").as_int(),
                                           (BLAS_Transpose) j.at("trans_b").as_int(), j.at("m").as_expression(),
                                           j.at("n").as_expression(), j.at("k").as_expression(), j.at("lda").as_expression(),
                                           j.at("ldb").as_expression(), j.at("ldc").as_expression());
    const Value* eb = j.find("epilogue_bias");
    const Value* ea = j.find("epilogue_activation");
    if (eb || ea) node->set_epilogue(eb && eb->as_bool(), ea ? ea->as_string() : "");
    return node;
}

Expression GEMMNode::connector_bytes(const std::string& connector) const {
    // row-major storage: rows x leading dimension
    if (connector == "__A") return bytes_of(symbolic::mul(trans_a_ == No ? m_ : k_, lda_), precision_input_type(precision_));
    if (connector == "__B") return bytes_of(symbolic::mul(trans_b_ == No ? k_ : n_, ldb_), precision_input_type(precision_));
    if (connector == "__C") return bytes_of(symbolic::mul(m_, ldc_), precision_output_type(precision_));
    if (connector == "__bias") return bytes_of(n_, precision_output_type(precision_));
    return "0";
}

bool GEMMNode::reads(const std::string& connector, const std::vector<data_flow::ConnectorBinding>& inputs) const {
    if (connector != "__C") return true;
    for (auto& b : inputs)
        if (b.connector == "__beta" && b.is_constant) return std::strtod(b.data.c_str(), nullptr) != 0.0;
    return true;
}

} // namespace math::blas

// ----------------------------------------------------------- tensor nodes

namespace math::blas {

DotNode::DotNode(std::string implementation_type, BLAS_Precision precision, Expression n, Expression incx, Expression incy)
    : LibraryNode(LibraryNodeType_DOT, {"__out"}, {"__x", "__y"}, false, std::move(implementation_type)), precision_(precision),
      n_(std::move(n)), incx_(std::move(incx)), incy_(std::move(incy)) {}

void DotNode::validate() const {
    if (precision_ != s && precision_ != d) throw InvalidSDFGException("DOT: precision must be s or d");
    if (n_.empty() || incx_.empty() || incy_.empty()) throw InvalidSDFGException("DOT: n, incx and incy are required");
}

Expression DotNode::flop() const { return "((" + n_ + ") + ((" + n_ + ") - 1))"; }

void DotNode::to_json(json::Value& j) const {
    j.set("precision", (int64_t) precision_);
    j.set("n", n_);
    j.set("incx", incx_);
    j.set("incy", incy_);
}

std::unique_ptr<DotNode> DotNode::from_json(const json::Value& j) {
    return std::make_unique<DotNode>(impl_of(j), (BLAS_Precision) j.at("precision").as_int(), j.at("n").as_expression(),
                                     j.at("incx").as_expression(), j.at("incy").as_expression());
}

Expression DotNode::connector_bytes(const std::string& connector) const {
    const types::PrimitiveType t = precision_input_type(precision_);
    if (connector == "__out") return bytes_of("1", t);
    const Expression& inc = connector == "__x" ? incx_ : incy_;
    // the span of the n strided elements: (n - 1) * inc + 1
    int64_t n = 0, step = 0;
    if (symbolic::is_integer(inc, &step) && step == 1) return bytes_of(n_, t);
    if (symbolic::is_integer(n_, &n) && symbolic::is_integer(inc, &step)) return bytes_of(symbolic::integer(n > 0 ? (n - 1) * step + 1 : 0), t);
    return bytes_of("(((" + n_ + ") - 1) * (" + inc + ") + 1)", t);
}

} // namespace math::blas

namespace math::tensor {

SoftmaxNode::SoftmaxNode(std::string implementation_type, std::vector<Expression> shape, std::vector<int64_t> axes,
                         types::PrimitiveType element)
    : LibraryNode(LibraryNodeType_Softmax, {"Y"}, {"X"}, false, std::move(implementation_type)), shape_(std::move(shape)),
      axes_(std::move(axes)), element_(element) {}

Expression SoftmaxNode::rows() const { return product(shape_, 0, shape_.empty() ? 0 : shape_.size() - 1); }
Expression SoftmaxNode::cols() const { return shape_.empty() ? "1" : shape_.back(); }

bool SoftmaxNode::last_axis_only() const {
    if (axes_.size() != 1) return false;
    const int64_t rank = (int64_t) shape_.size();
    return axes_[0] == -1 || axes_[0] == rank - 1;
}

std::vector<int64_t> SoftmaxNode::sorted_axes() const {
    std::vector<int64_t> a = axes_;
    const int64_t rank = (int64_t) shape_.size();
    for (auto& v : a)
        if (v < 0) v += rank;
    std::sort(a.begin(), a.end());
    a.erase(std::unique(a.begin(), a.end()), a.end());
    return a;
}

bool SoftmaxNode::adjacent_axes() const {
    const auto a = sorted_axes();
    return !a.empty() && a.back() - a.front() + 1 == (int64_t) a.size();
}

Expression SoftmaxNode::outer() const { return product(shape_, 0, (size_t) sorted_axes().front()); }
Expression SoftmaxNode::extent() const { return product(shape_, (size_t) sorted_axes().front(), (size_t) sorted_axes().back() + 1); }
Expression SoftmaxNode::inner() const { return product(shape_, (size_t) sorted_axes().back() + 1, shape_.size()); }

void SoftmaxNode::validate() const {
    if (shape_.empty()) throw InvalidSDFGException("Softmax: empty shape");
    if (axes_.empty()) throw InvalidSDFGException("Softmax: no reduction axis");
    const int64_t rank = (int64_t) shape_.size();
    for (auto a : axes_)
        if (a < -rank || a >= rank) throw InvalidSDFGException("Softmax: axis out of range");
}

void SoftmaxNode::to_json(Value& j) const {
    // keys as in the reduce-node serializer (reference reduce_node.h:194-245); keepdims is
    // always false for Softmax (softmax_node.cpp:31-33)
    j.set("shape", exprs_to_json(shape_));
    Array ax;
    for (auto a : axes_) ax.emplace_back(a);
    j.set("axes", Value(std::move(ax)));
    j.set("keepdims", false);
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<SoftmaxNode> SoftmaxNode::from_json(const Value& j) {
    std::vector<int64_t> axes;
    for (auto& a : j.at("axes").as_array()) axes.push_back(a.as_int());
    if (const Value* kd = j.find("keepdims"))
        if (kd->is_bool() && kd->as_bool()) throw InvalidSDFGException("Unsupported attribute on library node: softmax");
    const Value* et = j.find("element_type");
    return std::make_unique<SoftmaxNode>(impl_of(j), exprs_from_json(j.at("shape")), std::move(axes),
                                         et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression SoftmaxNode::connector_bytes(const std::string&) const { return bytes_of(product(shape_, 0, shape_.size()), element_); }

ConvNode::ConvNode(std::string implementation_type, std::vector<Expression> shape, std::vector<Expression> kernel_shape,
                   std::vector<Expression> strides, std::vector<Expression> pads, std::vector<Expression> dilations,
                   Expression output_channels, Expression group, bool has_bias, types::PrimitiveType element)
    : LibraryNode(LibraryNodeType_Conv, {"Y"}, has_bias ? std::vector<std::string>{"X", "W", "B"} : std::vector<std::string>{"X", "W"},
                  false, std::move(implementation_type)),
      shape_(std::move(shape)), kernel_shape_(std::move(kernel_shape)), strides_(std::move(strides)), pads_(std::move(pads)),
      dilations_(std::move(dilations)), output_channels_(std::move(output_channels)), group_(std::move(group)),
      has_bias_(has_bias), element_(element) {}

void ConvNode::validate() const {
    const size_t spatial = kernel_shape_.size();
    if (spatial == 0) throw InvalidSDFGException("Conv: kernel_shape is empty");
    if (shape_.size() != spatial + 2) throw InvalidSDFGException("Conv: input shape must be [N, C, spatial...]");
    if (!strides_.empty() && strides_.size() != spatial) throw InvalidSDFGException("Conv: strides rank mismatch");
    if (!pads_.empty() && pads_.size() != 2 * spatial) throw InvalidSDFGException("Conv: pads must hold begins and ends");
    if (!dilations_.empty() && dilations_.size() != spatial) throw InvalidSDFGException("Conv: dilations rank mismatch");
}

Expression ConvNode::output_dim(size_t i) const {
    const size_t spatial = kernel_shape_.size();
    const Expression stride = strides_.empty() ? "1" : strides_[i];
    const Expression pb = pads_.empty() ? "0" : pads_[i], pe = pads_.empty() ? "0" : pads_[spatial + i];
    const Expression dil = dilations_.empty() ? "1" : dilations_[i];
    int64_t d, b, e, l, k, s;
    if (symbolic::is_integer(shape_[2 + i], &d) && symbolic::is_integer(pb, &b) && symbolic::is_integer(pe, &e) &&
        symbolic::is_integer(dil, &l) && symbolic::is_integer(kernel_shape_[i], &k) && symbolic::is_integer(stride, &s) && s > 0) {
        const int64_t num = d + b + e - (l * (k - 1) + 1);
        return symbolic::integer(num < 0 ? 0 : num / s + 1);
    }
    return "((" + shape_[2 + i] + " + " + pb + " + " + pe + " - (" + dil + "*(" + kernel_shape_[i] + " - 1) + 1)) / " + stride + " + 1)";
}

Expression ConvNode::flop() const {
    Expression out = symbolic::mul(shape_[0], output_channels_);
    Expression taps = shape_[1];
    for (size_t i = 0; i < kernel_shape_.size(); i++) {
        out = symbolic::mul(out, output_dim(i));
        taps = symbolic::mul(taps, kernel_shape_[i]);
    }
    int64_t g = 1;
    if (!symbolic::is_integer(group_, &g)) return "2*(" + symbolic::mul(out, taps) + ") / (" + group_ + ")";
    if (g > 1) return "2*(" + symbolic::mul(out, taps) + ") / " + std::to_string(g);
    return "2*" + symbolic::mul(out, taps);
}

void ConvNode::to_json(Value& j) const {
    // keys as in ConvNodeSerializer (reference conv_node.cpp:552-589)
    j.set("shape", exprs_to_json(shape_));
    j.set("kernel_shape", exprs_to_json(kernel_shape_));
    j.set("strides", exprs_to_json(strides_));
    j.set("pads", exprs_to_json(pads_));
    j.set("dilations", exprs_to_json(dilations_));
    j.set("output_channels", output_channels_);
    j.set("group", group_);
    j.set("has_bias", has_bias_);
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<ConvNode> ConvNode::from_json(const Value& j) {
    const Value* hb = j.find("has_bias");
    const Value* et = j.find("element_type");
    return std::make_unique<ConvNode>(impl_of(j), exprs_from_json(j.at("shape")), exprs_from_json(j.at("kernel_shape")),
                                      exprs_from_json(j.at("strides")), exprs_from_json(j.at("pads")),
                                      exprs_from_json(j.at("dilations")), j.at("output_channels").as_expression(),
                                      j.at("group").as_expression(), hb ? hb->as_bool() : false,
                                      et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression ConvNode::connector_bytes(const std::string& connector) const {
    if (connector == "X") return bytes_of(product(shape_, 0, shape_.size()), element_);
    if (connector == "W") {   // [C_out][C_in / group][k0][k1] (reference conv_node.cpp:376-377)
        Expression e = symbolic::mul(output_channels_, shape_[1]);
        for (auto& k : kernel_shape_) e = symbolic::mul(e, k);
        int64_t g = 1;
        if (!symbolic::is_integer(group_, &g)) e = "(" + e + ") / (" + group_ + ")";
        else if (g > 1) e = "(" + e + ") / " + std::to_string(g);
        return bytes_of(e, element_);
    }
    if (connector == "B") return bytes_of(output_channels_, element_);
    Expression e = symbolic::mul(shape_[0], output_channels_);
    for (size_t i = 0; i < kernel_shape_.size(); i++) e = symbolic::mul(e, output_dim(i));
    return bytes_of(e, element_);
}

MatMulNode::MatMulNode(std::string implementation_type, std::vector<Expression> shape_a, std::vector<Expression> shape_b,
                       types::PrimitiveType element)
    : LibraryNode(LibraryNodeType_MatMul, {"Y"}, {"A", "B"}, false, std::move(implementation_type)),
      shape_a_(std::move(shape_a)), shape_b_(std::move(shape_b)), element_(element) {}

Expression MatMulNode::batch() const { return product(shape_a_, 0, shape_a_.size() - 2); }

void MatMulNode::validate() const {
    if (shape_a_.size() < 2 || shape_b_.size() < 2) throw InvalidSDFGException("MatMul: operands must be at least 2-d");
    if (shape_b_.size() > 2 && shape_b_.size() != shape_a_.size())
        throw InvalidSDFGException("MatMul: B must be 2-d or have A's rank");
    // integer element types are rejected by the reference as well (matmul_node.cpp:338-341)
    if (!types::is_floating_point(element_)) throw InvalidSDFGException("MatMul: floating point elements only");
}

Expression MatMulNode::flop() const { return "2*" + symbolic::mul(symbolic::mul(batch(), symbolic::mul(m(), n())), k()); }

void MatMulNode::to_json(Value& j) const {
    // keys as in the reference's serializer (matmul_node.cpp:546-628); operands are contiguous,
    // so strides and offsets are implied by the shapes
    j.set("shape_a", exprs_to_json(shape_a_));
    j.set("shape_b", exprs_to_json(shape_b_));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<MatMulNode> MatMulNode::from_json(const Value& j) {
    const Value* et = j.find("element_type");
    return std::make_unique<MatMulNode>(impl_of(j), exprs_from_json(j.at("shape_a")), exprs_from_json(j.at("shape_b")),
                                        et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression MatMulNode::connector_bytes(const std::string& connector) const {
    const types::PrimitiveType out = element_ == types::PrimitiveType::BFloat ? types::PrimitiveType::Float : element_;
    if (connector == "A") return bytes_of(product(shape_a_, 0, shape_a_.size()), element_);
    if (connector == "B") return bytes_of(product(shape_b_, 0, shape_b_.size()), element_);
    return bytes_of(symbolic::mul(batch(), symbolic::mul(m(), n())), out);
}

AttentionNode::AttentionNode(std::string implementation_type, std::vector<Expression> shape_q, Expression seq_kv,
                             std::string scale, types::PrimitiveType element, types::PrimitiveType output_element, bool causal)
    : LibraryNode(LibraryNodeType_Attention, {"O"}, {"Q", "K", "V"}, false, std::move(implementation_type)),
      shape_q_(std::move(shape_q)), seq_kv_(std::move(seq_kv)), scale_(std::move(scale)), element_(element),
      output_element_(output_element), causal_(causal) {}

void AttentionNode::validate() const {
    if (shape_q_.size() != 4) throw InvalidSDFGException("Attention: Q must be [B, H, S, D]");
    if (seq_kv_.empty() || scale_.empty()) throw InvalidSDFGException("Attention: missing seq_kv or scale");
}

Expression AttentionNode::flop() const {
    // Q K^T and P V: 4 * B * H * SQ * SKV * D
    return "4*" + symbolic::mul(symbolic::mul(product(shape_q_, 0, 3), seq_kv_), shape_q_[3]);
}

void AttentionNode::to_json(Value& j) const {
    j.set("shape_q", exprs_to_json(shape_q_));
    j.set("seq_kv", seq_kv_);
    j.set("scale", scale_);
    j.set("element_type", types::primitive_type_to_string(element_));
    j.set("output_type", types::primitive_type_to_string(output_element_));
    if (causal_) j.set("causal", true);
}

std::unique_ptr<AttentionNode> AttentionNode::from_json(const Value& j) {
    const Value* causal = j.find("causal");
    return std::make_unique<AttentionNode>(impl_of(j), exprs_from_json(j.at("shape_q")), j.at("seq_kv").as_expression(),
                                           j.at("scale").as_expression(),
                                           types::primitive_type_from_string(j.at("element_type").as_string()),
                                           types::primitive_type_from_string(j.at("output_type").as_string()),
                                           causal ? causal->as_bool() : false);
}

Expression AttentionNode::connector_bytes(const std::string& connector) const {
    const Expression bh = product(shape_q_, 0, 2);
    if (connector == "Q") return bytes_of(product(shape_q_, 0, 4), element_);
    if (connector == "O") return bytes_of(product(shape_q_, 0, 4), output_element_);
    return bytes_of(symbolic::mul(symbolic::mul(bh, seq_kv_), shape_q_[3]), element_);
}

// ---- elementwise / broadcast ----

ReduceNode::ReduceNode(std::string code, std::string implementation_type, std::vector<Expression> shape, std::vector<int64_t> axes,
                       bool keepdims, types::PrimitiveType element)
    : LibraryNode(std::move(code), {"Y"}, {"X"}, false, std::move(implementation_type)), shape_(std::move(shape)),
      axes_(std::move(axes)), keepdims_(keepdims), element_(element) {}

int ReduceNode::operation() const {
    for (size_t i = 0; i < ReduceNodeCodes.size(); i++)
        if (ReduceNodeCodes[i] == code_) return (int) i;
    return -1;
}

std::vector<int64_t> ReduceNode::sorted_axes() const {
    std::vector<int64_t> a = axes_;
    const int64_t rank = (int64_t) shape_.size();
    for (auto& v : a)
        if (v < 0) v += rank;
    std::sort(a.begin(), a.end());
    a.erase(std::unique(a.begin(), a.end()), a.end());
    return a;
}

bool ReduceNode::adjacent_axes() const {
    const auto a = sorted_axes();
    return !a.empty() && a.back() - a.front() + 1 == (int64_t) a.size();
}

Expression ReduceNode::outer() const { return product(shape_, 0, (size_t) sorted_axes().front()); }
Expression ReduceNode::extent() const { return product(shape_, (size_t) sorted_axes().front(), (size_t) sorted_axes().back() + 1); }
Expression ReduceNode::inner() const { return product(shape_, (size_t) sorted_axes().back() + 1, shape_.size()); }
Expression ReduceNode::product_all() const { return product(shape_, 0, shape_.size()); }

void ReduceNode::validate() const {
    if (operation() < 0) throw InvalidSDFGException(code_ + ": not a reduce node code");
    if (shape_.empty()) throw InvalidSDFGException(code_ + ": empty shape");
    if (axes_.empty()) throw InvalidSDFGException(code_ + ": no reduction axis");
    const int64_t rank = (int64_t) shape_.size();
    for (auto a : axes_)
        if (a < -rank || a >= rank)   // message of the reference's expansion (mean_node.cpp)
            throw InvalidSDFGException("Library Node: Axis value out of bounds. Axis: " + std::to_string(a) +
                                       " Shape size: " + std::to_string(rank));
}

void ReduceNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    Array ax;
    for (auto a : axes_) ax.emplace_back(a);
    j.set("axes", Value(std::move(ax)));
    j.set("keepdims", keepdims_);
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<ReduceNode> ReduceNode::from_json(const Value& j) {
    std::vector<int64_t> axes;
    for (auto& a : j.at("axes").as_array()) axes.push_back(a.as_int());
    const Value* kd = j.find("keepdims");
    const Value* et = j.find("element_type");
    return std::make_unique<ReduceNode>(j.at("code").as_string(), impl_of(j), exprs_from_json(j.at("shape")), std::move(axes),
                                        kd && kd->is_bool() && kd->as_bool(),
                                        et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression ReduceNode::connector_bytes(const std::string& connector) const {
    if (connector == "X") return bytes_of(product_all(), element_);
    // the output holds every extent that is not reduced
    Expression kept = "1";
    const auto axes = sorted_axes();
    for (size_t d = 0; d < shape_.size(); d++)
        if (std::find(axes.begin(), axes.end(), (int64_t) d) == axes.end()) kept = symbolic::mul(kept, shape_[d]);
    return bytes_of(kept, element_);
}

static bool is_in(const std::vector<std::string>& v, const std::string& s) {
    for (auto& e : v)
        if (e == s) return true;
    return false;
}

ElementWiseNode::ElementWiseNode(std::string code, std::string implementation_type, std::vector<Expression> shape,
                                 types::PrimitiveType element)
    : LibraryNode(code, is_in(BinaryNodeCodes, code) ? std::vector<std::string>{"C"} : std::vector<std::string>{"Y"},
                  is_in(BinaryNodeCodes, code) ? std::vector<std::string>{"A", "B"} : std::vector<std::string>{"X"}, false,
                  std::move(implementation_type)),
      shape_(std::move(shape)), element_(element) {}

int ElementWiseNode::operation() const {
    const auto& codes = is_binary() ? BinaryNodeCodes : UnaryNodeCodes;
    for (size_t i = 0; i < codes.size(); i++)
        if (codes[i] == code_) return (int) i;
    return -1;
}

Expression ElementWiseNode::count() const { return product(shape_, 0, shape_.size()); }

void ElementWiseNode::validate() const {
    if (operation() < 0) throw InvalidSDFGException(code_ + ": not an elementwise node code");
    if (shape_.empty()) throw InvalidSDFGException(code_ + ": empty shape");
}

void ElementWiseNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<ElementWiseNode> ElementWiseNode::from_json(const Value& j) {
    const Value* et = j.find("element_type");
    return std::make_unique<ElementWiseNode>(j.at("code").as_string(), impl_of(j), exprs_from_json(j.at("shape")),
                                             et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression ElementWiseNode::connector_bytes(const std::string&) const { return bytes_of(count(), element_); }

BroadcastNode::BroadcastNode(std::string implementation_type, std::vector<Expression> input_shape,
                             std::vector<Expression> output_shape, types::PrimitiveType element)
    : LibraryNode(LibraryNodeType_Broadcast, {"Y"}, {"X"}, false, std::move(implementation_type)),
      input_shape_(std::move(input_shape)), output_shape_(std::move(output_shape)), element_(element) {}

void BroadcastNode::validate() const {
    if (output_shape_.empty()) throw InvalidSDFGException("Broadcast: empty output shape");
    if (input_shape_.size() != output_shape_.size()) throw InvalidSDFGException("Broadcast: input and output ranks differ");
    for (size_t d = 0; d < input_shape_.size(); d++) {
        int64_t a = 0, b = 0;
        if (symbolic::is_integer(input_shape_[d], &a) && symbolic::is_integer(output_shape_[d], &b) && a != b && a != 1)
            throw InvalidSDFGException("Broadcast: dimension " + std::to_string(d) + " cannot be broadcast");
    }
}

void BroadcastNode::to_json(Value& j) const {
    j.set("input_shape", exprs_to_json(input_shape_));
    j.set("output_shape", exprs_to_json(output_shape_));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<BroadcastNode> BroadcastNode::from_json(const Value& j) {
    const Value* et = j.find("element_type");
    return std::make_unique<BroadcastNode>(impl_of(j), exprs_from_json(j.at("input_shape")), exprs_from_json(j.at("output_shape")),
                                           et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression BroadcastNode::connector_bytes(const std::string& connector) const {
    const auto& shape = connector == "X" ? input_shape_ : output_shape_;
    return bytes_of(product(shape, 0, shape.size()), element_);
}

ActivationNode::ActivationNode(std::string code, std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element)
    // "alpha" (and "beta" of HardSigmoid) are connectors a graph may leave unbound, so they are not among the
    // inputs whose binding validate() insists on
    : LibraryNode(code, {"Y"}, {"X"}, false, std::move(implementation_type)), shape_(std::move(shape)), element_(element) {}

int ActivationNode::operation() const {
    for (size_t i = 0; i < ActivationNodeCodes.size(); i++)
        if (ActivationNodeCodes[i] == code_) return 7 + (int) i;
    return -1;
}

Expression ActivationNode::count() const { return product(shape_, 0, shape_.size()); }

std::string ActivationNode::default_operand(const std::string& connector) const {
    if (code_ == "ml::Elu") return "1.0";
    if (code_ == "ml::LeakyReLU") return "0.01";
    return connector == "alpha" ? "0.2" : "0.5";
}

void ActivationNode::validate() const {
    if (operation() < 0) throw InvalidSDFGException(code_ + ": not an activation node code");
    if (shape_.empty()) throw InvalidSDFGException(code_ + ": empty shape");
}

void ActivationNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<ActivationNode> ActivationNode::from_json(const Value& j) {
    const Value* et = j.find("element_type");
    return std::make_unique<ActivationNode>(j.at("code").as_string(), impl_of(j), exprs_from_json(j.at("shape")),
                                            et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression ActivationNode::connector_bytes(const std::string& connector) const {
    if (connector == "alpha" || connector == "beta") return bytes_of("1", element_);
    return bytes_of(count(), element_);
}

FillNode::FillNode(std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element)
    : LibraryNode(LibraryNodeType_Fill, {"Y"}, {"X"}, false, std::move(implementation_type)), shape_(std::move(shape)), element_(element) {}

Expression FillNode::count() const { return shape_.empty() ? Expression("1") : product(shape_, 0, shape_.size()); }

void FillNode::validate() const {
    if (element_ == types::PrimitiveType::Void) throw InvalidSDFGException("Fill: void element type");
}

void FillNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<FillNode> FillNode::from_json(const Value& j) {
    const Value* et = j.find("element_type");
    return std::make_unique<FillNode>(impl_of(j), exprs_from_json(j.at("shape")),
                                      et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression FillNode::connector_bytes(const std::string& connector) const {
    return connector == "X" ? bytes_of("1", element_) : bytes_of(count(), element_);
}

CastNode::CastNode(std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element, types::PrimitiveType target)
    : LibraryNode(LibraryNodeType_Cast, {"Y"}, {"X"}, false, std::move(implementation_type)), shape_(std::move(shape)), element_(element),
      target_(target) {}

Expression CastNode::count() const { return shape_.empty() ? Expression("1") : product(shape_, 0, shape_.size()); }

void CastNode::validate() const {
    if (element_ == types::PrimitiveType::Void || target_ == types::PrimitiveType::Void) throw InvalidSDFGException("Cast: void element type");
}

void CastNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    j.set("target_type", types::primitive_type_to_string(target_));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<CastNode> CastNode::from_json(const Value& j) {
    const Value* et = j.find("element_type");
    return std::make_unique<CastNode>(impl_of(j), exprs_from_json(j.at("shape")),
                                      et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float,
                                      types::primitive_type_from_string(j.at("target_type").as_string()));
}

Expression CastNode::connector_bytes(const std::string& connector) const { return bytes_of(count(), connector == "X" ? element_ : target_); }

TransposeNode::TransposeNode(std::string implementation_type, std::vector<Expression> shape, std::vector<int64_t> perm,
                             types::PrimitiveType element)
    : LibraryNode(LibraryNodeType_Transpose, {"Y"}, {"X"}, false, std::move(implementation_type)), shape_(std::move(shape)),
      perm_(std::move(perm)), element_(element) {
    if (perm_.empty())   // default permutation: reverse (transpose_node.cpp:27-31)
        for (size_t i = 0; i < shape_.size(); i++) perm_.push_back((int64_t) (shape_.size() - 1 - i));
}

void TransposeNode::validate() const {
    if (perm_.size() != shape_.size()) throw InvalidSDFGException("Permutation rank must match shape rank");
    std::vector<bool> seen(shape_.size(), false);
    for (auto p : perm_) {
        if (p < 0 || p >= (int64_t) shape_.size() || seen[(size_t) p]) throw InvalidSDFGException("Transpose: perm is not a permutation of the axes");
        seen[(size_t) p] = true;
    }
}

void TransposeNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    Array pm;
    for (auto p : perm_) pm.emplace_back(p);
    j.set("perm", Value(std::move(pm)));
    j.set("element_type", types::primitive_type_to_string(element_));
}

std::unique_ptr<TransposeNode> TransposeNode::from_json(const Value& j) {
    std::vector<int64_t> perm;
    if (const Value* pm = j.find("perm"))
        for (auto& p : pm->as_array()) perm.push_back(p.as_int());
    const Value* et = j.find("element_type");
    return std::make_unique<TransposeNode>(impl_of(j), exprs_from_json(j.at("shape")), std::move(perm),
                                           et ? types::primitive_type_from_string(et->as_string()) : types::PrimitiveType::Float);
}

Expression TransposeNode::connector_bytes(const std::string&) const { return bytes_of(product(shape_, 0, shape_.size()), element_); }

} // namespace math::tensor

// ------------------------------------------------------------- offloading

namespace rocm {

namespace {
std::vector<std::string> offload_inputs(DataTransferDirection d, BufferLifecycle l) {
    if (d != DataTransferDirection::NONE) return {"_src"};
    if (l == BufferLifecycle::FREE) return {"_ptr"};
    return {};
}
std::vector<std::string> offload_outputs(DataTransferDirection d, BufferLifecycle l) {
    if (d != DataTransferDirection::NONE) return {"_dst"};
    if (l == BufferLifecycle::ALLOC) return {"_ret"};
    return {};
}
} // namespace

ROCMFusedElementWiseNode::ROCMFusedElementWiseNode(std::string implementation_type, std::vector<Expression> shape,
                                                   types::PrimitiveType element, std::string binary, std::vector<Expression> a_shape,
                                                   std::vector<Expression> b_shape, std::vector<std::string> post)
    : LibraryNode(LibraryNodeType_ROCM_FusedElementWise, {"Y"},
                  binary.empty() ? std::vector<std::string>{"A"} : std::vector<std::string>{"A", "B"}, false, std::move(implementation_type)),
      shape_(std::move(shape)), element_(element), binary_(std::move(binary)), a_shape_(std::move(a_shape)),
      b_shape_(std::move(b_shape)), post_(std::move(post)) {}

void ROCMFusedElementWiseNode::validate() const {
    using namespace math::tensor;
    auto known = [](const std::vector<std::string>& codes, const std::string& c) { return std::find(codes.begin(), codes.end(), c) != codes.end(); };
    if (shape_.empty() || shape_.size() > 6) throw InvalidSDFGException(code_ + ": rank must be 1..6");
    if (!binary_.empty() && !known(BinaryNodeCodes, binary_)) throw InvalidSDFGException(code_ + ": unknown binary operation " + binary_);
    if (post_.size() > 4) throw InvalidSDFGException(code_ + ": more than four unary operations");
    for (auto& p : post_)
        if (!known(UnaryNodeCodes, p)) throw InvalidSDFGException(code_ + ": unknown unary operation " + p);
    for (auto* operand : {&a_shape_, &b_shape_}) {
        if (operand->empty()) continue;   // scalar
        if (operand->size() != shape_.size()) throw InvalidSDFGException(code_ + ": operand rank differs from the output rank");
        for (size_t d = 0; d < shape_.size(); d++)
            if ((*operand)[d] != shape_[d] && (*operand)[d] != "1")
                throw InvalidSDFGException(code_ + ": dimension " + std::to_string(d) + " cannot be broadcast");
    }
    if (a_shape_.empty() && (binary_.empty() || b_shape_.empty())) throw InvalidSDFGException(code_ + ": no array operand");
}

Expression ROCMFusedElementWiseNode::flop() const {
    const size_t ops = (binary_.empty() ? 0 : 1) + post_.size();
    return symbolic::mul(std::to_string(ops ? ops : 1), product(shape_, 0, shape_.size()));
}

void ROCMFusedElementWiseNode::to_json(Value& j) const {
    j.set("shape", exprs_to_json(shape_));
    j.set("element_type", types::primitive_type_to_string(element_));
    j.set("binary", binary_);
    j.set("a_shape", exprs_to_json(a_shape_));
    j.set("b_shape", exprs_to_json(b_shape_));
    Array post;
    for (auto& p : post_) post.emplace_back(p);
    j.set("post", Value(std::move(post)));
}

std::unique_ptr<ROCMFusedElementWiseNode> ROCMFusedElementWiseNode::from_json(const Value& j) {
    std::vector<std::string> post;
    for (auto& p : j.at("post").as_array()) post.push_back(p.as_string());
    return std::make_unique<ROCMFusedElementWiseNode>(impl_of(j), exprs_from_json(j.at("shape")),
                                                      types::primitive_type_from_string(j.at("element_type").as_string()),
                                                      j.at("binary").as_string(), exprs_from_json(j.at("a_shape")),
                                                      exprs_from_json(j.at("b_shape")), std::move(post));
}

Expression ROCMFusedElementWiseNode::connector_bytes(const std::string& connector) const {
    const std::vector<Expression>& s = connector == "A" ? a_shape_ : connector == "B" ? b_shape_ : shape_;
    return bytes_of(s.empty() ? Expression("1") : product(s, 0, s.size()), element_);
}

// ---- ROCMMap

namespace {
std::vector<std::string> map_inputs(const std::vector<ROCMMapNode::Access>& reads, const std::vector<ROCMMapNode::ScalarOperand>& scalars) {
    std::vector<std::string> names;
    for (auto& r : reads) names.push_back(r.connector);
    for (auto& s : scalars) names.push_back(s.connector);
    return names;
}
std::vector<std::string> map_outputs(const std::vector<ROCMMapNode::Access>& writes) {
    std::vector<std::string> names;
    for (auto& w : writes) names.push_back(w.connector);
    return names;
}
const std::map<std::string, int>& map_operations() {
    static const std::map<std::string, int> ops = {
        {"assign", 1}, {"fp_neg", 1}, {"fp_add", 2}, {"fp_sub", 2}, {"fp_mul", 2}, {"fp_div", 2}, {"fp_rem", 2}, {"fp_fma", 3},
        // CMath stems (reference cmath_node.h:21-96) that take and return the element type
        {"sin", 1}, {"cos", 1}, {"tan", 1}, {"asin", 1}, {"acos", 1}, {"atan", 1}, {"atan2", 2}, {"sinh", 1}, {"cosh", 1}, {"tanh", 1},
        {"asinh", 1}, {"acosh", 1}, {"atanh", 1}, {"exp", 1}, {"exp2", 1}, {"exp10", 1}, {"expm1", 1}, {"log", 1}, {"log10", 1},
        {"log2", 1}, {"log1p", 1}, {"pow", 2}, {"sqrt", 1}, {"cbrt", 1}, {"hypot", 2}, {"erf", 1}, {"erfc", 1}, {"tgamma", 1},
        {"lgamma", 1}, {"fabs", 1}, {"ceil", 1}, {"floor", 1}, {"trunc", 1}, {"round", 1}, {"nearbyint", 1}, {"rint", 1},
        {"fmod", 2}, {"remainder", 2}, {"copysign", 2}, {"fmax", 2}, {"fmin", 2}, {"fdim", 2}, {"fma", 3}};
    return ops;
}
} // namespace

ROCMMapNode::ROCMMapNode(std::string implementation_type, std::vector<std::string> indvars, std::vector<Expression> bounds,
                         std::vector<std::string> symbols, std::vector<Access> reads, std::vector<Access> writes,
                         std::vector<ScalarOperand> scalars, std::vector<Statement> statements)
    : LibraryNode(LibraryNodeType_ROCM_Map, map_outputs(writes), map_inputs(reads, scalars), false, std::move(implementation_type)),
      indvars_(std::move(indvars)), bounds_(std::move(bounds)), symbols_(std::move(symbols)), reads_(std::move(reads)),
      writes_(std::move(writes)), scalars_(std::move(scalars)), statements_(std::move(statements)) {}

int ROCMMapNode::arity(const std::string& op) {
    auto it = map_operations().find(op);
    return it == map_operations().end() ? -1 : it->second;
}

bool ROCMMapNode::is_cmath(const std::string& op) { return arity(op) >= 0 && op != "assign" && op.rfind("fp_", 0) != 0; }

void ROCMMapNode::validate() const {
    using P = types::PrimitiveType;
    auto floating = [](P t) { return t == P::Float || t == P::Double; };
    if (indvars_.empty() || indvars_.size() > 6 || indvars_.size() != bounds_.size())
        throw InvalidSDFGException(code_ + ": one bound per induction variable, 1..6 of them");
    if (writes_.empty()) throw InvalidSDFGException(code_ + ": a nest that stores nothing");
    std::vector<std::string> defined;
    auto define = [&](const std::string& name) {
        if (name.empty() || name[0] == '#' || std::find(defined.begin(), defined.end(), name) != defined.end())
            throw InvalidSDFGException(code_ + ": name '" + name + "' is empty, a literal, or defined twice");
        defined.push_back(name);
    };
    for (auto* list : {&reads_, &writes_})
        for (auto& a : *list) {
            if (a.strides.size() != indvars_.size()) throw InvalidSDFGException(code_ + ": operand " + a.connector + " needs one stride per induction variable");
            // bf16 tensors are loaded and stored (converted by the assignments next to them), never computed on
            if (!floating(a.element) && a.element != types::PrimitiveType::BFloat)
                throw InvalidSDFGException(code_ + ": operand " + a.connector + " must be Float, Double or BFloat");
        }
    for (auto& r : reads_) define(r.connector);
    for (auto& s : scalars_) {
        if (!floating(s.element)) throw InvalidSDFGException(code_ + ": scalar " + s.connector + " must be Float or Double");
        define(s.connector);
    }
    auto known = [&](const std::string& name) {
        return (name.size() > 1 && name[0] == '#') || std::find(defined.begin(), defined.end(), name) != defined.end();
    };
    for (auto& st : statements_) {
        const int n = arity(st.op);
        if (n < 0) throw InvalidSDFGException(code_ + ": unknown operation '" + st.op + "'");
        if ((int) st.args.size() != n) throw InvalidSDFGException(code_ + ": operation " + st.op + " takes " + std::to_string(n) + " arguments");
        if (!floating(st.type) && !(st.type == types::PrimitiveType::BFloat && st.op == "assign"))
            throw InvalidSDFGException(code_ + ": statement " + st.out + " must be Float or Double (BFloat for an assignment)");
        for (auto& a : st.args)
            if (!known(a)) throw InvalidSDFGException(code_ + ": statement " + st.out + " uses '" + a + "' before it is defined");
        define(st.out);
    }
    for (auto& w : writes_) {
        if (!known(w.value)) throw InvalidSDFGException(code_ + ": " + w.connector + " stores '" + w.value + "', which nothing defines");
        for (auto& other : writes_)
            if (&other != &w && other.connector == w.connector) throw InvalidSDFGException(code_ + ": connector " + w.connector + " written twice");
    }
}

Expression ROCMMapNode::flop() const {
    size_t ops = 0;
    for (auto& st : statements_) ops += st.op == "assign" ? 0 : st.op == "fp_fma" || st.op == "fma" ? 2 : 1;
    return symbolic::mul(std::to_string(ops), product(bounds_, 0, bounds_.size()));
}

void ROCMMapNode::to_json(Value& j) const {
    auto names = [](const std::vector<std::string>& v) {
        Array a;
        for (auto& n : v) a.emplace_back(n);
        return Value(std::move(a));
    };
    auto accesses = [&](const std::vector<Access>& list, bool with_value) {
        Array out;
        for (auto& a : list) {
            Value v;
            v.set("connector", a.connector);
            v.set("strides", exprs_to_json(a.strides));
            v.set("extent", a.extent);
            v.set("element_type", types::primitive_type_to_string(a.element));
            if (with_value) v.set("value", a.value);
            out.push_back(std::move(v));
        }
        return Value(std::move(out));
    };
    j.set("indvars", names(indvars_));
    j.set("bounds", exprs_to_json(bounds_));
    j.set("symbols", names(symbols_));
    j.set("reads", accesses(reads_, false));
    j.set("writes", accesses(writes_, true));
    Array scalars;
    for (auto& s : scalars_) {
        Value v;
        v.set("connector", s.connector);
        v.set("element_type", types::primitive_type_to_string(s.element));
        scalars.push_back(std::move(v));
    }
    j.set("scalars", Value(std::move(scalars)));
    Array statements;
    for (auto& st : statements_) {
        Value v;
        v.set("out", st.out);
        v.set("type", types::primitive_type_to_string(st.type));
        v.set("op", st.op);
        v.set("args", names(st.args));
        statements.push_back(std::move(v));
    }
    j.set("statements", Value(std::move(statements)));
}

std::unique_ptr<ROCMMapNode> ROCMMapNode::from_json(const Value& j) {
    auto names = [](const Value& v) {
        std::vector<std::string> out;
        for (auto& n : v.as_array()) out.push_back(n.as_string());
        return out;
    };
    auto accesses = [&](const Value& v, bool with_value) {
        std::vector<Access> out;
        for (auto& a : v.as_array()) {
            Access acc;
            acc.connector = a.at("connector").as_string();
            acc.strides = exprs_from_json(a.at("strides"));
            acc.extent = a.at("extent").as_expression();
            acc.element = types::primitive_type_from_string(a.at("element_type").as_string());
            if (with_value) acc.value = a.at("value").as_string();
            out.push_back(std::move(acc));
        }
        return out;
    };
    std::vector<ScalarOperand> scalars;
    for (auto& s : j.at("scalars").as_array())
        scalars.push_back({s.at("connector").as_string(), types::primitive_type_from_string(s.at("element_type").as_string())});
    std::vector<Statement> statements;
    for (auto& s : j.at("statements").as_array())
        statements.push_back({s.at("out").as_string(), types::primitive_type_from_string(s.at("type").as_string()), s.at("op").as_string(),
                              names(s.at("args"))});
    return std::make_unique<ROCMMapNode>(impl_of(j), names(j.at("indvars")), exprs_from_json(j.at("bounds")), names(j.at("symbols")),
                                         accesses(j.at("reads"), false), accesses(j.at("writes"), true), std::move(scalars),
                                         std::move(statements));
}

Expression ROCMMapNode::connector_bytes(const std::string& connector) const {
    for (auto* list : {&reads_, &writes_})
        for (auto& a : *list)
            if (a.connector == connector) return bytes_of(a.extent, a.element);
    for (auto& s : scalars_)
        if (s.connector == connector) return bytes_of("1", s.element);
    throw InvalidSDFGException(code_ + ": no connector '" + connector + "'");
}

ROCMDataOffloadingNode::ROCMDataOffloadingNode(Expression size, int device_id, DataTransferDirection direction,
                                               BufferLifecycle lifecycle)
    : LibraryNode(LibraryNodeType_ROCM_Offloading, offload_outputs(direction, lifecycle), offload_inputs(direction, lifecycle),
                  true, ImplementationType_NONE),
      size_(std::move(size)), device_id_(device_id), direction_(direction), lifecycle_(lifecycle) {
    if (direction == DataTransferDirection::NONE && lifecycle == BufferLifecycle::NO_CHANGE)
        throw InvalidSDFGException("ROCMOffloading: node neither transfers nor changes a buffer");
}

bool ROCMDataOffloadingNode::equal_with(const ROCMDataOffloadingNode& other) const {
    return size_ == other.size_ && device_id_ == other.device_id_ && direction_ == other.direction_ &&
           lifecycle_ == other.lifecycle_;
}

bool ROCMDataOffloadingNode::redundant_with(const ROCMDataOffloadingNode& other) const {
    // a D2H(+FREE) directly followed by an H2D(+ALLOC) of the same size on the same device
    // (reference data_offloading_node.cpp:85-118)
    if (size_ != other.size_ || device_id_ != other.device_id_) return false;
    const bool opposite_dir = (int) direction_ == -(int) other.direction_ && direction_ != DataTransferDirection::NONE;
    const bool opposite_life = (int) lifecycle_ == -(int) other.lifecycle_;
    return opposite_dir && opposite_life;
}

std::string ROCMDataOffloadingNode::toStr() const {
    std::string s = "ROCM";
    if (is_alloc()) s += " ALLOC";
    if (is_h2d()) s += " H2D";
    if (is_d2h()) s += " D2H";
    if (is_free()) s += " FREE";
    return s;
}

void ROCMDataOffloadingNode::to_json(Value& j) const {
    // keys as in the CUDA offloading node's serializer (reference cuda_data_offloading_node.cpp:198-256)
    j.set("size", size_);
    j.set("device_id", (int64_t) device_id_);
    j.set("transfer_direction", (int64_t) direction_);
    j.set("buffer_lifecycle", (int64_t) lifecycle_);
}

std::unique_ptr<ROCMDataOffloadingNode> ROCMDataOffloadingNode::from_json(const Value& j) {
    return std::make_unique<ROCMDataOffloadingNode>(j.at("size").is_null() ? "0" : j.at("size").as_expression(),
                                                    (int) j.at("device_id").as_int(),
                                                    (DataTransferDirection) j.at("transfer_direction").as_int(),
                                                    (BufferLifecycle) j.at("buffer_lifecycle").as_int());
}

} // namespace rocm

// ------------------------------------------------------------------- SDFG

namespace data_flow {

const data_flow::ConnectorBinding* DataFlowGraph::input(const std::string& connector) const {
    for (auto& b : inputs)
        if (b.connector == connector) return &b;
    return nullptr;
}

const data_flow::ConnectorBinding* DataFlowGraph::output(const std::string& connector) const {
    for (auto& b : outputs)
        if (b.connector == connector) return &b;
    return nullptr;
}

} // namespace data_flow

const Container& StructuredSDFG::container(const std::string& name) const {
    auto it = containers_.find(name);
    if (it == containers_.end()) throw InvalidSDFGException("container '" + name + "' does not exist");
    return it->second;
}

Container& StructuredSDFG::container(const std::string& name) {
    auto it = containers_.find(name);
    if (it == containers_.end()) throw InvalidSDFGException("container '" + name + "' does not exist");
    return it->second;
}

void StructuredSDFG::add_container(Container c, bool is_argument) {
    if (c.name.empty()) throw InvalidSDFGException("container without a name");
    if (containers_.count(c.name)) throw InvalidSDFGException("container '" + c.name + "' already exists");
    c.is_argument = is_argument;
    if (is_argument) arguments_.push_back(c.name);
    containers_.emplace(c.name, std::move(c));
}

void StructuredSDFG::remove_container(const std::string& name) {
    const Container& c = container(name);
    if (c.is_argument || name == return_container_) throw InvalidSDFGException("container '" + name + "' is part of the signature");
    for (auto& blk : blocks_) {
        for (auto& in : blk.inputs)
            if (!in.is_constant && in.data == name) throw InvalidSDFGException("container '" + name + "' is still in use");
        for (auto& out : blk.outputs)
            if (out.data == name) throw InvalidSDFGException("container '" + name + "' is still in use");
    }
    containers_.erase(name);
}

structured_control_flow::Block& StructuredSDFG::add_block(std::unique_ptr<data_flow::LibraryNode> node,
                                                          std::vector<data_flow::ConnectorBinding> inputs,
                                                          std::vector<data_flow::ConnectorBinding> outputs,
                                                          size_t position) {
    structured_control_flow::Block blk;
    blk.element_id = next_element_id();
    node->set_element_id(next_element_id());
    blk.node = std::move(node);
    blk.inputs = std::move(inputs);
    blk.outputs = std::move(outputs);
    if (position == (size_t) -1 || position >= blocks_.size()) {
        blocks_.push_back(std::move(blk));
        return blocks_.back();
    }
    auto it = blocks_.insert(blocks_.begin() + (long) position, std::move(blk));
    return *it;
}

const std::string& StructuredSDFG::metadata(const std::string& key) const {
    auto it = metadata_.find(key);
    if (it == metadata_.end()) throw std::out_of_range("metadata key '" + key + "' not found");
    return it->second;
}

void StructuredSDFG::validate() const {
    if (name_.empty()) throw InvalidSDFGException("SDFG without a name");
    for (auto& a : arguments_)
        if (!containers_.count(a)) throw InvalidSDFGException("argument '" + a + "' has no container");
    if (!return_container_.empty() && !containers_.count(return_container_))
        throw InvalidSDFGException("return container '" + return_container_ + "' does not exist");
    for (auto& blk : blocks_) {
        if (!blk.node) throw InvalidSDFGException("block without a library node");
        blk.node->validate();
        auto check = [&](const std::vector<std::string>& connectors, const std::vector<data_flow::ConnectorBinding>& bound,
                         const char* what) {
            for (auto& c : connectors) {
                const data_flow::ConnectorBinding* hit = nullptr;
                for (auto& b : bound)
                    if (b.connector == c) hit = &b;
                if (!hit)
                    throw InvalidSDFGException(blk.node->code() + ": " + what + " connector '" + c + "' is not connected");
                if (!hit->is_constant && !containers_.count(hit->data))
                    throw InvalidSDFGException(blk.node->code() + ": connector '" + c + "' refers to unknown container '" +
                                               hit->data + "'");
            }
        };
        check(blk.node->inputs(), blk.inputs, "input");
        check(blk.node->outputs(), blk.outputs, "output");
        // all tensor operands of a node share one element type unless the node says otherwise
        // (reference tensor_node.cpp:56-101); GEMM precision 'b' and Attention carry their own output type
    }
}

json::Value StructuredSDFG::to_json() const {
    Value j;
    j.set("type", "structured_sdfg");
    j.set("name", name_);
    Array args;
    for (auto& a : arguments_) args.emplace_back(a);
    j.set("arguments", Value(std::move(args)));
    Value conts{Object{}};
    for (auto& kv : containers_) {
        Value c;
        c.set("type", kv.second.is_pointer ? "pointer" : "scalar");
        c.set("element", types::primitive_type_to_string(kv.second.element));
        c.set("transient", kv.second.transient);
        c.set("storage", kv.second.storage);
        if (!kv.second.size_bytes.empty()) c.set("size", kv.second.size_bytes);
        conts.set(kv.first, std::move(c));
    }
    j.set("containers", std::move(conts));
    j.set("return", return_container_);
    Value meta{Object{}};
    for (auto& kv : metadata_) meta.set(kv.first, kv.second);
    j.set("metadata", std::move(meta));
    Array children;
    for (auto& blk : blocks_) {
        Value node;
        // envelope as written by the reference's serializer (json_serializer.cpp:132-142)
        node.set("type", "library_node");
        node.set("element_id", blk.node->element_id());
        node.set("code", blk.node->code());
        node.set("implementation_type", blk.node->implementation_type());
        node.set("side_effect", blk.node->side_effect());
        blk.node->to_json(node);
        auto bindings = [](const std::vector<data_flow::ConnectorBinding>& v) {
            Array a;
            for (auto& b : v) {
                Value e;
                e.set("connector", b.connector);
                if (b.is_constant) {
                    e.set("constant", b.data);
                    e.set("type", types::primitive_type_to_string(b.type));
                } else {
                    e.set("data", b.data);
                }
                a.push_back(std::move(e));
            }
            return Value(std::move(a));
        };
        Value df;
        df.set("library_node", std::move(node));
        df.set("inputs", bindings(blk.inputs));
        df.set("outputs", bindings(blk.outputs));
        Value b;
        b.set("type", "block");
        b.set("element_id", blk.element_id);
        if (blk.debug_info.has) {
            Value d;
            d.set("has", true);
            d.set("filename", blk.debug_info.filename);
            d.set("function", blk.debug_info.function);
            d.set("start_line", (int64_t) blk.debug_info.start_line);
            d.set("start_column", (int64_t) blk.debug_info.start_column);
            d.set("end_line", (int64_t) blk.debug_info.end_line);
            d.set("end_column", (int64_t) blk.debug_info.end_column);
            b.set("debug_info", std::move(d));
        }
        b.set("dataflow", std::move(df));
        children.push_back(std::move(b));
    }
    Value root;
    root.set("type", "sequence");
    root.set("children", Value(std::move(children)));
    j.set("root", std::move(root));
    return j;
}

std::unique_ptr<StructuredSDFG> StructuredSDFG::from_json(const json::Value& j) {
    auto sdfg = std::make_unique<StructuredSDFG>(j.at("name").as_string());
    const Value& conts = j.at("containers");
    auto make = [&](const std::string& name) {
        const Value& c = conts.at(name);
        Container out;
        out.name = name;
        out.is_pointer = c.at("type").as_string() == "pointer";
        out.element = types::primitive_type_from_string(c.at("element").as_string());
        if (const Value* t = c.find("transient")) out.transient = t->as_bool();
        if (const Value* s = c.find("storage")) out.storage = s->as_string();
        if (const Value* s = c.find("size"))
            if (!s->is_null()) out.size_bytes = s->as_expression();
        return out;
    };
    for (auto& a : j.at("arguments").as_array()) sdfg->add_container(make(a.as_string()), true);
    for (auto& kv : conts.as_object())
        if (!sdfg->exists(kv.first)) sdfg->add_container(make(kv.first), false);
    if (const Value* r = j.find("return"))
        if (r->is_string()) sdfg->set_return_container(r->as_string());
    if (const Value* m = j.find("metadata"))
        for (auto& kv : m->as_object()) sdfg->add_metadata(kv.first, kv.second.as_string());
    auto& registry = serializer::LibraryNodeSerializerRegistry::instance();
    for (auto& child : j.at("root").at("children").as_array()) {
        if (child.at("type").as_string() != "block") throw InvalidSDFGException("only blocks are supported in the root sequence");
        const Value& df = child.at("dataflow");
        const Value& nj = df.at("library_node");
        const std::string code = nj.at("code").as_string();
        auto fn = registry.get_library_node_serializer(code);
        if (!fn) throw std::runtime_error("No library node serializer found for " + code);
        auto node = fn(nj);
        auto bindings = [](const Value& arr) {
            std::vector<data_flow::ConnectorBinding> out;
            for (auto& e : arr.as_array()) {
                data_flow::ConnectorBinding b;
                b.connector = e.at("connector").as_string();
                if (const Value* c = e.find("constant")) {
                    b.is_constant = true;
                    b.data = c->as_expression();
                    b.type = types::primitive_type_from_string(e.at("type").as_string());
                } else {
                    b.data = e.at("data").as_string();
                }
                out.push_back(std::move(b));
            }
            return out;
        };
        auto& blk = sdfg->add_block(std::move(node), bindings(df.at("inputs")), bindings(df.at("outputs")));
        if (const Value* d = child.find("debug_info")) {
            const Value* has = d->find("has");
            if (has && has->as_bool()) {
                blk.debug_info.has = true;
                blk.debug_info.filename = d->at("filename").as_string();
                blk.debug_info.function = d->at("function").as_string();
                blk.debug_info.start_line = (long) d->at("start_line").as_int();
                blk.debug_info.start_column = (long) d->at("start_column").as_int();
                blk.debug_info.end_line = (long) d->at("end_line").as_int();
                blk.debug_info.end_column = (long) d->at("end_column").as_int();
            }
        }
    }
    return sdfg;
}

// ------------------------------------------------------------- serializers

namespace serializer {

namespace {
std::mutex g_serializer_mutex;

template <typename T>
std::unique_ptr<data_flow::LibraryNode> deserialize(const json::Value& j) {
    return T::from_json(j);
}
} // namespace

LibraryNodeSerializerRegistry::LibraryNodeSerializerRegistry() {
    fns_[math::blas::LibraryNodeType_GEMM] = &deserialize<math::blas::GEMMNode>;
    fns_[math::tensor::LibraryNodeType_Softmax] = &deserialize<math::tensor::SoftmaxNode>;
    fns_[math::tensor::LibraryNodeType_Conv] = &deserialize<math::tensor::ConvNode>;
    fns_[math::tensor::LibraryNodeType_MatMul] = &deserialize<math::tensor::MatMulNode>;
    for (auto& code : math::tensor::UnaryNodeCodes) fns_[code] = &deserialize<math::tensor::ElementWiseNode>;
    for (auto& code : math::tensor::BinaryNodeCodes) fns_[code] = &deserialize<math::tensor::ElementWiseNode>;
    fns_[math::tensor::LibraryNodeType_Broadcast] = &deserialize<math::tensor::BroadcastNode>;
    fns_[math::tensor::LibraryNodeType_Transpose] = &deserialize<math::tensor::TransposeNode>;
    fns_[math::tensor::LibraryNodeType_Cast] = &deserialize<math::tensor::CastNode>;
    for (auto& code : math::tensor::ActivationNodeCodes) fns_[code] = &deserialize<math::tensor::ActivationNode>;
    fns_[math::tensor::LibraryNodeType_Fill] = &deserialize<math::tensor::FillNode>;
    fns_[math::blas::LibraryNodeType_DOT] = &deserialize<math::blas::DotNode>;
    for (auto& code : math::tensor::ReduceNodeCodes) fns_[code] = &deserialize<math::tensor::ReduceNode>;
    fns_[rocm::LibraryNodeType_ROCM_FusedElementWise] = &deserialize<rocm::ROCMFusedElementWiseNode>;
    fns_[rocm::LibraryNodeType_ROCM_Map] = &deserialize<rocm::ROCMMapNode>;
}

LibraryNodeSerializerRegistry& LibraryNodeSerializerRegistry::instance() {
    static LibraryNodeSerializerRegistry registry;
    return registry;
}

void LibraryNodeSerializerRegistry::register_library_node_serializer(const std::string& code, LibraryNodeDeserializeFn fn) {
    std::lock_guard<std::mutex> lock(g_serializer_mutex);
    fns_.emplace(code, fn);  // duplicates are ignored
}

LibraryNodeDeserializeFn LibraryNodeSerializerRegistry::get_library_node_serializer(const std::string& code) const {
    auto it = fns_.find(code);
    return it == fns_.end() ? nullptr : it->second;
}

size_t LibraryNodeSerializerRegistry::size() const { return fns_.size(); }

} // namespace serializer

} // namespace sdfg
