// A descriptor-level carrier for the parts of docc's SDFG that the rocm target
// needs: typed containers, an ordered argument list, a root sequence of
// blocks each holding one library node with its connector bindings, and the
// math library nodes GEMM / ml::MatMul / ml::Softmax / ml::Conv (fields, connector names
// and JSON keys as in the reference) plus the ml::Attention node and the
// ROCMOffloading transfer node that the rocm target adds.
//
// The reference's own IR (sdfg/include/sdfg/structured_sdfg.h, data_flow/*.h)
// is a general graph with symbolic expressions (SymEngine); here symbolic
// expressions are kept as C-expression strings over the function's integer
// arguments, which is what they are printed as in generated code anyway.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "json.h"

namespace sdfg {

class InvalidSDFGException : public std::runtime_error {
public:
    using std::runtime_error::runtime_error;
};

namespace types {

// reference: sdfg/include/sdfg/types/type.h (PrimitiveType)
enum class PrimitiveType { Void, Bool, Int8, Int16, Int32, Int64, UInt8, UInt16, UInt32, UInt64, Half, BFloat, Float, Double };

const char* primitive_type_to_string(PrimitiveType t);
PrimitiveType primitive_type_from_string(const std::string& s);
size_t primitive_type_size(PrimitiveType t);
bool is_floating_point(PrimitiveType t);

} // namespace types

using Expression = std::string;  // C expression over int64 symbols, e.g. "_s0*_s1"

namespace symbolic {
Expression mul(const Expression& a, const Expression& b);
Expression integer(int64_t v);
bool is_integer(const Expression& e, int64_t* value = nullptr);
// v[begin] * ... * v[end - 1] ("1" for an empty range)
Expression product(const std::vector<Expression>& v, size_t begin, size_t end);
// Whether the two expressions denote the same value for every value of their symbols, as far as sums and products of
// integers and symbols go ("(32)*16" and "512", "(n)*m" and "m*n"); anything else (quotients, calls) compares as text.
bool equal(const Expression& a, const Expression& b);
} // namespace symbolic

// Implementation types, following the "<LIB>With[out]Transfers" naming of the
// reference (opt/include/sdfg/targets/cuda/cuda.h:20-26, targets/et/include/docc/target/et/target.h:10-11)
inline const std::string ImplementationType_NONE = "NONE";
inline const std::string ImplementationType_BLAS = "BLAS";
inline const std::string ImplementationType_ROCMWithTransfers = "ROCMWithTransfers";
inline const std::string ImplementationType_ROCMWithoutTransfers = "ROCMWithoutTransfers";

struct Container {
    std::string name;
    bool is_pointer = false;
    types::PrimitiveType element = types::PrimitiveType::Void;
    bool is_argument = false;
    bool transient = false;      // allocated and freed by the generated function
    Expression size_bytes;       // transients: byte size
    std::string storage = "CPU"; // "CPU" | "ROCM_Generic" (device memory, cf. NV_Generic in cuda_transform.h:21-37)
};

namespace data_flow {

struct ConnectorBinding {
    std::string connector;
    bool is_constant = false;    // ConstantNode: `data` is the literal, printed verbatim
    std::string data;            // container name or literal
    types::PrimitiveType type = types::PrimitiveType::Void;  // constants only
};

// reference: sdfg/include/sdfg/data_flow/library_node.h:98-179
class LibraryNode {
public:
    LibraryNode(std::string code, std::vector<std::string> outputs, std::vector<std::string> inputs, bool side_effect,
                std::string implementation_type)
        : code_(std::move(code)), outputs_(std::move(outputs)), inputs_(std::move(inputs)), side_effect_(side_effect),
          implementation_type_(std::move(implementation_type)) {}
    virtual ~LibraryNode() = default;

    const std::string& code() const { return code_; }
    const std::string& implementation_type() const { return implementation_type_; }
    std::string& implementation_type() { return implementation_type_; }
    bool side_effect() const { return side_effect_; }
    const std::vector<std::string>& inputs() const { return inputs_; }
    const std::vector<std::string>& outputs() const { return outputs_; }
    size_t element_id() const { return element_id_; }
    void set_element_id(size_t id) { element_id_ = id; }

    virtual std::string toStr() const { return code_; }
    virtual void validate() const {}
    // floating point operations, as an expression, or "" when unknown
    virtual Expression flop() const { return ""; }
    // node payload (everything except the envelope keys)
    virtual void to_json(json::Value& j) const = 0;

    // Offloading support: byte extent of the memory behind a connector, and
    // whether the node reads what is behind an input connector (GEMM does not
    // read __C when beta is the constant 0).
    virtual Expression connector_bytes(const std::string& connector) const = 0;
    virtual bool reads(const std::string& connector, const std::vector<ConnectorBinding>& inputs) const { return true; }

protected:
    std::string code_;
    std::vector<std::string> outputs_;
    std::vector<std::string> inputs_;
    bool side_effect_;
    std::string implementation_type_;
    size_t element_id_ = 0;
};

} // namespace data_flow

namespace math::blas {

// reference: sdfg/include/sdfg/data_flow/library_nodes/math/blas/blas_node.h:49-126
enum BLAS_Precision : int { h = 'h', s = 's', d = 'd', c = 'c', z = 'z', b = 'b' /* bf16 in, fp32 accumulate/out: added by the rocm target */ };
enum BLAS_Layout : int { RowMajor = 101, ColMajor = 102 };
enum BLAS_Transpose : int { No = 111, Trans = 112, ConjTrans = 113 };

types::PrimitiveType precision_input_type(BLAS_Precision p);
types::PrimitiveType precision_output_type(BLAS_Precision p);

inline const std::string LibraryNodeType_GEMM = "GEMM";

// reference: sdfg/include/sdfg/data_flow/library_nodes/math/blas/gemm_node.h:14-112
class GEMMNode : public data_flow::LibraryNode {
public:
    GEMMNode(std::string implementation_type, BLAS_Precision precision, BLAS_Layout layout, BLAS_Transpose trans_a,
             BLAS_Transpose trans_b, Expression m, Expression n, Expression k, Expression lda, Expression ldb,
             Expression ldc);

    BLAS_Precision precision() const { return precision_; }
    BLAS_Layout layout() const { return layout_; }
    BLAS_Transpose trans_a() const { return trans_a_; }
    BLAS_Transpose trans_b() const { return trans_b_; }
    const Expression& m() const { return m_; }
    const Expression& n() const { return n_; }
    const Expression& k() const { return k_; }
    const Expression& lda() const { return lda_; }
    const Expression& ldb() const { return ldb_; }
    const Expression& ldc() const { return ldc_; }
    types::PrimitiveType scalar_primitive() const { return precision_input_type(precision_); }

    // Set by the rocm target's fusion pass only (the reference's node has neither): the rest of a dense
    // layer in the store, C = act(alpha A B + beta C + bias[column]). `bias` adds the input connector
    // "__bias" (n values of C's type); `activation` is an elementwise node code or "". JSON keys
    // "epilogue_bias" / "epilogue_activation", written only when set.
    void set_epilogue(bool bias, std::string activation);
    bool epilogue_bias() const { return epilogue_bias_; }
    const std::string& epilogue_activation() const { return epilogue_activation_; }
    bool has_epilogue() const { return epilogue_bias_ || !epilogue_activation_.empty(); }

    void validate() const override;
    Expression flop() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    bool reads(const std::string& connector, const std::vector<data_flow::ConnectorBinding>& inputs) const override;
    static std::unique_ptr<GEMMNode> from_json(const json::Value& j);

private:
    BLAS_Precision precision_;
    BLAS_Layout layout_;
    BLAS_Transpose trans_a_, trans_b_;
    Expression m_, n_, k_, lda_, ldb_, ldc_;
    bool epilogue_bias_ = false;
    std::string epilogue_activation_;
};

// reference: sdfg/include/sdfg/data_flow/library_nodes/math/blas/dot_node.h, dot_node.cpp:18-40 (connectors
// "__x", "__y" -> "__out", a scalar), JSON keys code, precision, n, incx, incy (dot_node.cpp:189-202)
inline const std::string LibraryNodeType_DOT = "DOT";

class DotNode : public data_flow::LibraryNode {
public:
    DotNode(std::string implementation_type, BLAS_Precision precision, Expression n, Expression incx, Expression incy);
    BLAS_Precision precision() const { return precision_; }
    const Expression& n() const { return n_; }
    const Expression& incx() const { return incx_; }
    const Expression& incy() const { return incy_; }

    void validate() const override;
    Expression flop() const override;   // n multiplications + n - 1 additions (dot_node.cpp:167-171)
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<DotNode> from_json(const json::Value& j);

private:
    BLAS_Precision precision_;
    Expression n_, incx_, incy_;
};

} // namespace math::blas

namespace math::tensor {

inline const std::string LibraryNodeType_Softmax = "ml::Softmax";
inline const std::string LibraryNodeType_Conv = "ml::Conv";
inline const std::string LibraryNodeType_MatMul = "ml::MatMul";
inline const std::string LibraryNodeType_Attention = "ml::Attention";

// reference: .../tensor/reduce_ops/softmax_node.h:9-49, reduce_node.h:194-245
class SoftmaxNode : public data_flow::LibraryNode {
public:
    SoftmaxNode(std::string implementation_type, std::vector<Expression> shape, std::vector<int64_t> axes,
                types::PrimitiveType element = types::PrimitiveType::Float);
    const std::vector<Expression>& shape() const { return shape_; }
    const std::vector<int64_t>& axes() const { return axes_; }
    types::PrimitiveType element() const { return element_; }
    Expression rows() const;  // product of all dims but the last
    Expression cols() const;  // the last dim
    bool last_axis_only() const;
    // the axes, normalised and sorted; `adjacent` tells whether they form one block, which is the
    // middle extent of an [outer, extent, inner] view of the input
    std::vector<int64_t> sorted_axes() const;
    bool adjacent_axes() const;
    Expression outer() const;
    Expression extent() const;
    Expression inner() const;

    void validate() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<SoftmaxNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    std::vector<int64_t> axes_;
    types::PrimitiveType element_;
};

// reference: .../tensor/conv_node.h:48-217, conv_node.cpp:552-647
class ConvNode : public data_flow::LibraryNode {
public:
    ConvNode(std::string implementation_type, std::vector<Expression> shape, std::vector<Expression> kernel_shape,
             std::vector<Expression> strides, std::vector<Expression> pads, std::vector<Expression> dilations,
             Expression output_channels, Expression group, bool has_bias,
             types::PrimitiveType element = types::PrimitiveType::Float);
    const std::vector<Expression>& shape() const { return shape_; }              // N, C, spatial...
    const std::vector<Expression>& kernel_shape() const { return kernel_shape_; }
    const std::vector<Expression>& strides() const { return strides_; }
    const std::vector<Expression>& pads() const { return pads_; }                // begins..., ends...
    const std::vector<Expression>& dilations() const { return dilations_; }
    const Expression& output_channels() const { return output_channels_; }
    const Expression& group() const { return group_; }
    bool has_bias() const { return has_bias_; }
    types::PrimitiveType element() const { return element_; }
    // D_out per spatial dim (conv_node.cpp:224-233)
    Expression output_dim(size_t i) const;

    void validate() const override;
    Expression flop() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<ConvNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_, kernel_shape_, strides_, pads_, dilations_;
    Expression output_channels_, group_;
    bool has_bias_;
    types::PrimitiveType element_;
};

// reference: .../tensor/matmul_node.h:49-193 (ONNX MatMul [...,M,K] @ [...,K,N]); contiguous operands only
class MatMulNode : public data_flow::LibraryNode {
public:
    MatMulNode(std::string implementation_type, std::vector<Expression> shape_a, std::vector<Expression> shape_b,
               types::PrimitiveType element);
    const std::vector<Expression>& shape_a() const { return shape_a_; }
    const std::vector<Expression>& shape_b() const { return shape_b_; }
    types::PrimitiveType element() const { return element_; }
    Expression batch() const;   // product of the leading dims of A ("1" when none); B must match or be 2-d
    bool b_is_batched() const { return shape_b_.size() > 2; }
    Expression m() const { return shape_a_[shape_a_.size() - 2]; }
    Expression k() const { return shape_a_.back(); }
    Expression n() const { return shape_b_.back(); }

    void validate() const override;
    Expression flop() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<MatMulNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_a_, shape_b_;
    types::PrimitiveType element_;
};

// Added by the rocm target; the reference's node set has no attention
// (sdfg/include/sdfg/data_flow/library_nodes/math/math.h:5-42).
// O = softmax(scale * Q K^T) V, Q [B,H,SQ,D], K/V [B,H,SKV,D]; with the `causal` flag query i attends to the keys j <= i.
class AttentionNode : public data_flow::LibraryNode {
public:
    AttentionNode(std::string implementation_type, std::vector<Expression> shape_q, Expression seq_kv, std::string scale,
                  types::PrimitiveType element, types::PrimitiveType output_element, bool causal = false);
    const std::vector<Expression>& shape_q() const { return shape_q_; }
    const Expression& seq_kv() const { return seq_kv_; }
    const std::string& scale() const { return scale_; }
    types::PrimitiveType element() const { return element_; }
    types::PrimitiveType output_element() const { return output_element_; }
    // query i attends to the keys j <= i (torch's is_causal)
    bool causal() const { return causal_; }

    void validate() const override;
    Expression flop() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<AttentionNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_q_;
    Expression seq_kv_;
    std::string scale_;
    types::PrimitiveType element_, output_element_;
    bool causal_ = false;
};

// Reduce nodes over a set of axes, "X" -> "Y" (reference .../tensor/reduce_node.h, reduce_ops/
// {sum,max,min,mean}_node.h; JSON keys shape, axes, keepdims as in reduce_node.h:194-245). Y has
// the reduced axes removed, or kept with extent 1 when keepdims is set.
inline const std::vector<std::string> ReduceNodeCodes = {"ml::Sum", "ml::Max", "ml::Min", "ml::Mean"};

class ReduceNode : public data_flow::LibraryNode {
public:
    ReduceNode(std::string code, std::string implementation_type, std::vector<Expression> shape, std::vector<int64_t> axes,
               bool keepdims, types::PrimitiveType element);
    const std::vector<Expression>& shape() const { return shape_; }
    const std::vector<int64_t>& axes() const { return axes_; }
    bool keepdims() const { return keepdims_; }
    types::PrimitiveType element() const { return element_; }
    // position of the code in ReduceNodeCodes = the runtime's operation code
    int operation() const;
    // the axes, normalised and sorted; `adjacent` tells whether they form one block
    std::vector<int64_t> sorted_axes() const;
    bool adjacent_axes() const;
    // [outer, reduce, inner] view of the input for a block of adjacent axes
    Expression outer() const;
    Expression extent() const;
    Expression inner() const;

    void validate() const override;
    Expression flop() const override { return product_all(); }
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<ReduceNode> from_json(const json::Value& j);

private:
    Expression product_all() const;
    std::vector<Expression> shape_;
    std::vector<int64_t> axes_;
    bool keepdims_;
    types::PrimitiveType element_;
};

// Elementwise tensor nodes: Y[i] = f(X[i]) or f(A[i], B[i]) over the linearised shape.
// reference: .../tensor/elementwise_node.cpp:20 (ElementWiseUnaryNode "X" -> "Y"), :176
// (ElementWiseBinaryNode "A","B" -> "C"), JSON keys code + shape; elementwise_ops/*.h for the codes.
inline const std::vector<std::string> UnaryNodeCodes = {"ml::Abs", "ml::Exp", "ml::ReLU", "ml::Sigmoid", "ml::Sqrt", "ml::Tanh", "ml::Erf"};
inline const std::vector<std::string> BinaryNodeCodes = {"ml::Add", "ml::Sub", "ml::Mul", "ml::Div", "ml::Maximum", "ml::Minimum", "ml::Pow"};
inline const std::string LibraryNodeType_Broadcast = "ml::Broadcast";
inline const std::string LibraryNodeType_Transpose = "ml::Transpose";
inline const std::string LibraryNodeType_Cast = "ml::Cast";

class ElementWiseNode : public data_flow::LibraryNode {
public:
    ElementWiseNode(std::string code, std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element);
    const std::vector<Expression>& shape() const { return shape_; }
    types::PrimitiveType element() const { return element_; }
    bool is_binary() const { return inputs_.size() == 2; }
    // position of the code in UnaryNodeCodes / BinaryNodeCodes = the runtime's operation code
    int operation() const;
    Expression count() const;

    void validate() const override;
    Expression flop() const override { return count(); }
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<ElementWiseNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    types::PrimitiveType element_;
};

// reference: .../tensor/broadcast_node.h:13-80 ("X" -> "Y", JSON keys input_shape, output_shape)
class BroadcastNode : public data_flow::LibraryNode {
public:
    BroadcastNode(std::string implementation_type, std::vector<Expression> input_shape, std::vector<Expression> output_shape,
                  types::PrimitiveType element);
    const std::vector<Expression>& input_shape() const { return input_shape_; }
    const std::vector<Expression>& output_shape() const { return output_shape_; }
    types::PrimitiveType element() const { return element_; }

    void validate() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<BroadcastNode> from_json(const json::Value& j);

private:
    std::vector<Expression> input_shape_, output_shape_;
    types::PrimitiveType element_;
};

// reference: .../tensor/elementwise_ops/cast_node.h:13-60 (connectors "X" -> "Y", JSON keys "shape" and
// "target_type"; the input's element type comes from its memlet there and is kept on the node here)
class CastNode : public data_flow::LibraryNode {
public:
    CastNode(std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element, types::PrimitiveType target);
    const std::vector<Expression>& shape() const { return shape_; }
    types::PrimitiveType element() const { return element_; }
    types::PrimitiveType target_type() const { return target_; }
    Expression count() const;

    void validate() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<CastNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    types::PrimitiveType element_, target_;
};

// The unary nodes with scalar operands. reference: .../elementwise_ops/elu_node.cpp:21 ("X", "alpha" -> "Y"),
// leaky_relu_node.cpp:21 (the same), hard_sigmoid_node.cpp:21-22 ("X", "alpha", "beta" -> "Y"); JSON keys code +
// shape (ElementWiseUnaryNodeSerializer). "alpha" / "beta" are bound to constants or scalar containers; an
// operand that is left unbound takes the ONNX default of its operator (Elu 1, LeakyReLU 0.01, HardSigmoid 0.2 / 0.5).
inline const std::vector<std::string> ActivationNodeCodes = {"ml::Elu", "ml::LeakyReLU", "ml::HardSigmoid"};

class ActivationNode : public data_flow::LibraryNode {
public:
    ActivationNode(std::string code, std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element);
    const std::vector<Expression>& shape() const { return shape_; }
    types::PrimitiveType element() const { return element_; }
    // the runtime's operation code (DOCC_ROCM_UNARY_ELU ...)
    int operation() const;
    Expression count() const;
    // the literal an unbound "alpha" / "beta" stands for
    std::string default_operand(const std::string& connector) const;

    void validate() const override;
    Expression flop() const override { return count(); }
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<ActivationNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    types::PrimitiveType element_;
};

// reference: .../elementwise_ops/fill_node.cpp:17-41 ("X" -> "Y" with X a scalar or a constant: every element
// of Y becomes X; JSON keys code + shape)
inline const std::string LibraryNodeType_Fill = "ml::Fill";

class FillNode : public data_flow::LibraryNode {
public:
    FillNode(std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element);
    const std::vector<Expression>& shape() const { return shape_; }
    types::PrimitiveType element() const { return element_; }
    Expression count() const;

    void validate() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    bool reads(const std::string& connector, const std::vector<data_flow::ConnectorBinding>&) const override { return connector == "X"; }
    static std::unique_ptr<FillNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    types::PrimitiveType element_;
};

// reference: .../tensor/transpose_node.h:14-60 (connectors "X" -> "Y", JSON keys "shape" and "perm";
// an empty permutation reverses the axes, transpose_node.cpp:27-31)
class TransposeNode : public data_flow::LibraryNode {
public:
    TransposeNode(std::string implementation_type, std::vector<Expression> shape, std::vector<int64_t> perm, types::PrimitiveType element);
    const std::vector<Expression>& shape() const { return shape_; }   // of the input
    const std::vector<int64_t>& perm() const { return perm_; }        // output axis i is input axis perm[i]
    types::PrimitiveType element() const { return element_; }

    void validate() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<TransposeNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    std::vector<int64_t> perm_;
    types::PrimitiveType element_;
};

} // namespace math::tensor

namespace rocm {

inline const std::string LibraryNodeType_ROCM_Offloading = "ROCMOffloading";

// reference: opt/include/sdfg/targets/offloading/data_offloading_node.h:16-97
enum class DataTransferDirection : int { D2H = -1, NONE = 0, H2D = 1 };
enum class BufferLifecycle : int { FREE = -1, NO_CHANGE = 0, ALLOC = 1 };

// Counterpart of CUDADataOffloadingNode (opt/src/targets/cuda/cuda_data_offloading_node.cpp:26-256):
// connectors: H2D  in "_src" (host)   out "_dst" (device)
//             D2H  in "_src" (device) out "_dst" (host)
//             ALLOC only: out "_ret" (device);  FREE only: in "_ptr" (device)
class ROCMDataOffloadingNode : public data_flow::LibraryNode {
public:
    ROCMDataOffloadingNode(Expression size, int device_id, DataTransferDirection direction, BufferLifecycle lifecycle);
    const Expression& size() const { return size_; }
    int device_id() const { return device_id_; }
    DataTransferDirection transfer_direction() const { return direction_; }
    BufferLifecycle buffer_lifecycle() const { return lifecycle_; }
    bool is_h2d() const { return direction_ == DataTransferDirection::H2D; }
    bool is_d2h() const { return direction_ == DataTransferDirection::D2H; }
    bool is_alloc() const { return lifecycle_ == BufferLifecycle::ALLOC; }
    bool is_free() const { return lifecycle_ == BufferLifecycle::FREE; }
    bool blocking() const { return true; }
    // true when `other` undoes or repeats this node on the same buffers (D2H followed by H2D ...)
    bool redundant_with(const ROCMDataOffloadingNode& other) const;
    bool equal_with(const ROCMDataOffloadingNode& other) const;

    std::string toStr() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string&) const override { return size_; }
    static std::unique_ptr<ROCMDataOffloadingNode> from_json(const json::Value& j);

private:
    Expression size_;
    int device_id_;
    DataTransferDirection direction_;
    BufferLifecycle lifecycle_;
};

// A chain of elementwise nodes run as one kernel: Y = post_k(...post_1(binary(A', B'))), A' and
// B' the operands repeated to `shape` (or scalars). Written only by the target's fusion pass, in
// place of a Broadcast node folded into its consumer and of unary nodes folded into their
// producer; the reference fuses the expanded Maps instead (py_structured_sdfg.cpp:258-260).
// connectors: in "A" [, "B"], out "Y". JSON keys: shape, element_type, binary ("" = none),
// a_shape / b_shape ([] = scalar operand), post.
inline const std::string LibraryNodeType_ROCM_FusedElementWise = "ROCMFusedElementWise";

class ROCMFusedElementWiseNode : public data_flow::LibraryNode {
public:
    ROCMFusedElementWiseNode(std::string implementation_type, std::vector<Expression> shape, types::PrimitiveType element,
                             std::string binary, std::vector<Expression> a_shape, std::vector<Expression> b_shape,
                             std::vector<std::string> post);
    const std::vector<Expression>& shape() const { return shape_; }
    types::PrimitiveType element() const { return element_; }
    const std::string& binary() const { return binary_; }
    const std::vector<Expression>& a_shape() const { return a_shape_; }
    const std::vector<Expression>& b_shape() const { return b_shape_; }
    const std::vector<std::string>& post() const { return post_; }
    std::vector<std::string>& post() { return post_; }
    bool has_b() const { return !binary_.empty(); }

    void validate() const override;
    Expression flop() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<ROCMFusedElementWiseNode> from_json(const json::Value& j);

private:
    std::vector<Expression> shape_;
    types::PrimitiveType element_;
    std::string binary_;
    std::vector<Expression> a_shape_, b_shape_;
    std::vector<std::string> post_;
};

// A perfect nest of Maps (from 0, step 1, `indvar < bound`) whose body is a chain of tasklets and CMath calls over
// dense tensors: what the reference hands to its CUDAMapDispatcher (opt/src/targets/cuda/cuda_map_dispatcher.cpp:42-262)
// as a Map element with a body sequence. The block list has no nested control flow, so the nest travels as one node
// that spells the body out:
//   reads   - tensor elements loaded once per iteration: connector, one stride per induction variable ("0": the
//             variable does not index the operand, i.e. it is repeated along that loop), element count, element type;
//   scalars - values passed to the kernel by value (scalar containers, constants bound to a connector);
//   statements - in order: `out = op(args)`; an argument names a read or scalar connector, the `out` of an earlier
//             statement, or a literal spelled "#<text>"; `op` is a tasklet code by name (assign, fp_neg, fp_add, fp_sub,
//             fp_mul, fp_div, fp_rem, fp_fma: reference sdfg/include/sdfg/data_flow/tasklet.h:94-153) or the stem of
//             a CMath function (cmath_node.h:21-96);
//   writes  - tensor elements stored once per iteration, each naming the value it stores;
//   symbols - the integer scalar containers that bounds and strides mention.
// Written by the importer of docc's JSON for nests that are not one of the prebuilt kernels
// (serializer::import_reference_json); dispatched by ROCMMapDispatcher as a generated gfx950 kernel.
inline const std::string LibraryNodeType_ROCM_Map = "ROCMMap";

class ROCMMapNode : public data_flow::LibraryNode {
public:
    struct Access {
        std::string connector;
        std::vector<Expression> strides;   // elements, one per induction variable
        Expression extent;                 // elements the operand spans
        types::PrimitiveType element;
        std::string value;                 // writes: the statement result (or read / scalar) stored
    };
    struct ScalarOperand {
        std::string connector;
        types::PrimitiveType element;
    };
    struct Statement {
        std::string out;
        types::PrimitiveType type;
        std::string op;
        std::vector<std::string> args;
    };

    ROCMMapNode(std::string implementation_type, std::vector<std::string> indvars, std::vector<Expression> bounds,
                std::vector<std::string> symbols, std::vector<Access> reads, std::vector<Access> writes,
                std::vector<ScalarOperand> scalars, std::vector<Statement> statements);

    const std::vector<std::string>& indvars() const { return indvars_; }
    const std::vector<Expression>& bounds() const { return bounds_; }
    const std::vector<std::string>& symbols() const { return symbols_; }
    const std::vector<Access>& reads() const { return reads_; }
    const std::vector<Access>& writes() const { return writes_; }
    const std::vector<ScalarOperand>& scalars() const { return scalars_; }
    const std::vector<Statement>& statements() const { return statements_; }

    // number of arguments of a body operation, or -1 for one the kernels cannot spell
    static int arity(const std::string& op);
    static bool is_cmath(const std::string& op);

    void validate() const override;
    Expression flop() const override;
    void to_json(json::Value& j) const override;
    Expression connector_bytes(const std::string& connector) const override;
    static std::unique_ptr<ROCMMapNode> from_json(const json::Value& j);

private:
    std::vector<std::string> indvars_;
    std::vector<Expression> bounds_;
    std::vector<std::string> symbols_;
    std::vector<Access> reads_, writes_;
    std::vector<ScalarOperand> scalars_;
    std::vector<Statement> statements_;
};

} // namespace rocm

namespace data_flow {

// The dataflow of a block as this target needs it: the one library node and what its connectors are bound to.
// It stands where the reference's data_flow::DataFlowGraph stands in the dispatcher interfaces
// (codegen/dispatchers/node_dispatcher_registry.h:140-141); there a dispatcher reaches the same facts through
// in_edges(node) / out_edges(node) and the access or constant node at the other end of each memlet.
struct DataFlowGraph {
    std::unique_ptr<LibraryNode> node;
    std::vector<ConnectorBinding> inputs;
    std::vector<ConnectorBinding> outputs;

    const ConnectorBinding* input(const std::string& connector) const;
    const ConnectorBinding* output(const std::string& connector) const;
};

} // namespace data_flow

namespace structured_control_flow {

// Source position of an element (reference sdfg/include/sdfg/element.h DebugInfo; JSON keys of
// json_serializer.cpp debug_info_to_json: has, filename, function, start_line, start_column,
// end_line, end_column).
struct DebugInfo {
    bool has = false;
    std::string filename, function;
    long start_line = 0, start_column = 0, end_line = 0, end_column = 0;
};

// One block of the root sequence: a dataflow graph with exactly one library node
// (reference structured_control_flow/block.h: Block::dataflow()).
struct Block : public data_flow::DataFlowGraph {
    size_t element_id = 0;
    DebugInfo debug_info;

    const data_flow::DataFlowGraph& dataflow() const { return *this; }
    data_flow::DataFlowGraph& dataflow() { return *this; }
};

} // namespace structured_control_flow

// reference: sdfg/include/sdfg/function.h + structured_sdfg.h
class StructuredSDFG {
public:
    explicit StructuredSDFG(std::string name) : name_(std::move(name)) {}

    const std::string& name() const { return name_; }
    const std::vector<std::string>& arguments() const { return arguments_; }
    const std::map<std::string, Container>& containers() const { return containers_; }
    std::vector<structured_control_flow::Block>& blocks() { return blocks_; }
    const std::vector<structured_control_flow::Block>& blocks() const { return blocks_; }
    bool exists(const std::string& name) const { return containers_.count(name) != 0; }
    const Container& container(const std::string& name) const;
    Container& container(const std::string& name);
    // "" = void function; otherwise the function returns this pointer container (torch entry)
    const std::string& return_container() const { return return_container_; }
    void set_return_container(const std::string& name) { return_container_ = name; }

    void add_container(Container c, bool is_argument);
    // a transient that no block refers to any more
    void remove_container(const std::string& name);
    structured_control_flow::Block& add_block(std::unique_ptr<data_flow::LibraryNode> node,
                                              std::vector<data_flow::ConnectorBinding> inputs,
                                              std::vector<data_flow::ConnectorBinding> outputs, size_t position = (size_t) -1);
    size_t next_element_id() { return ++element_counter_; }

    void add_metadata(const std::string& key, const std::string& value) { metadata_[key] = value; }
    const std::string& metadata(const std::string& key) const;
    const std::map<std::string, std::string>& metadata() const { return metadata_; }

    // structure checks: containers exist, connectors complete, element types agree
    void validate() const;

    json::Value to_json() const;
    static std::unique_ptr<StructuredSDFG> from_json(const json::Value& j);

private:
    std::string name_;
    std::vector<std::string> arguments_;
    std::map<std::string, Container> containers_;
    std::vector<structured_control_flow::Block> blocks_;
    std::map<std::string, std::string> metadata_;
    std::string return_container_;
    size_t element_counter_ = 0;
};

using Function = StructuredSDFG;

namespace serializer {

// The reference's own wire format (sdfg/src/serializer/json_serializer.cpp:56-353), see interchange.cpp.
bool is_reference_format(const json::Value& j);
// -> the block-list JSON that StructuredSDFG::from_json reads; throws InvalidSDFGException naming the
// element that has no lowering on the rocm target
json::Value import_reference_json(const json::Value& j);
json::Value export_reference_json(const StructuredSDFG& sdfg);

// reference: sdfg/include/sdfg/serializer/json_serializer.h (LibraryNodeSerializerRegistry)
using LibraryNodeDeserializeFn = std::unique_ptr<data_flow::LibraryNode> (*)(const json::Value&);

class LibraryNodeSerializerRegistry {
public:
    static LibraryNodeSerializerRegistry& instance();
    // first registration wins, as in the reference's registries
    void register_library_node_serializer(const std::string& code, LibraryNodeDeserializeFn fn);
    LibraryNodeDeserializeFn get_library_node_serializer(const std::string& code) const;
    size_t size() const;

private:
    LibraryNodeSerializerRegistry();
    std::map<std::string, LibraryNodeDeserializeFn> fns_;
};

} // namespace serializer

namespace builder {
// Thin stand-in for builder::StructuredSDFGBuilder: the object passes mutate an SDFG through.
class StructuredSDFGBuilder {
public:
    explicit StructuredSDFGBuilder(StructuredSDFG& sdfg) : sdfg_(sdfg) {}
    StructuredSDFG& subject() { return sdfg_; }

private:
    StructuredSDFG& sdfg_;
};
} // namespace builder

namespace analysis {
class AnalysisManager {
public:
    explicit AnalysisManager(StructuredSDFG& sdfg) : sdfg_(sdfg) {}
    StructuredSDFG& sdfg() { return sdfg_; }
    void invalidate_all() {}

private:
    StructuredSDFG& sdfg_;
};
} // namespace analysis

} // namespace sdfg
