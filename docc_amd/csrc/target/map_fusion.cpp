// RocmMapFusionPass: chains of elementwise work that the prebuilt fused kernel cannot take in one launch (more than
// one two-operand operation, several repeated operands) become one ROCMMap node, i.e. one generated kernel that
// reads every input once and writes only the chain's result. Counterpart of the reference's MapFusion, which merges
// the expanded Maps of consecutive tensor nodes before its CUDA target turns each remaining Map into a kernel
// (python/bindings/py_structured_sdfg.cpp:258-260; opt/src/targets/cuda/cuda_map_dispatcher.cpp:42-262).
#include <algorithm>
#include <cctype>
#include <map>
#include <optional>
#include <set>

#include "rocm_target.h"

namespace sdfg::rocm {

using data_flow::ConnectorBinding;
using structured_control_flow::Block;
namespace tensor = math::tensor;

namespace {

using Statement = ROCMMapNode::Statement;
using P = types::PrimitiveType;

bool is_rocm_type(const std::string& impl) {
    return impl == ImplementationType_ROCMWithTransfers || impl == ImplementationType_ROCMWithoutTransfers;
}

// A block of elementwise kind written as loops over a shape: loads, statements on values, one store. Values carry
// names that are unique within the pass; the node built from the form renames them.
struct MapForm {
    struct Read {
        std::string data;
        std::vector<Expression> strides;
        Expression extent;
        P element;
        std::string value;
    };
    struct Scalar {
        ConnectorBinding source;   // a scalar container or a constant
        P element;
        std::string value;
    };
    std::vector<Expression> bounds;
    std::vector<Read> reads;
    std::vector<Scalar> scalars;
    struct Result {
        std::string value, data;
        std::vector<Expression> strides;
        Expression extent;
        P element;
    };
    std::vector<Statement> statements;
    std::vector<Result> results;   // the tensor nodes have one; a nest that was imported, or merged, may store several
    P element = P::Float;          // of the statements a tensor node becomes
};

class Converter {
public:
    explicit Converter(const StructuredSDFG& sdfg) : sdfg_(sdfg) {}

    // nullopt: the block is not of elementwise kind (or uses an operation the statements cannot spell)
    std::optional<MapForm> form_of(const Block& blk) {
        if (!is_rocm_type(blk.node->implementation_type()) || blk.outputs.empty()) return std::nullopt;
        std::optional<MapForm> f;
        if (auto* m = dynamic_cast<const ROCMMapNode*>(blk.node.get())) f = from_map(blk, *m);
        else if (auto* e = dynamic_cast<const tensor::ElementWiseNode*>(blk.node.get())) f = from_elementwise(blk, *e);
        else if (auto* fe = dynamic_cast<const ROCMFusedElementWiseNode*>(blk.node.get())) f = from_fused(blk, *fe);
        else if (auto* b = dynamic_cast<const tensor::BroadcastNode*>(blk.node.get())) f = from_broadcast(blk, *b);
        else if (auto* c = dynamic_cast<const tensor::CastNode*>(blk.node.get())) f = from_cast(blk, *c);
        if (f && f->bounds.size() > 6) return std::nullopt;   // a ROCMMap node holds at most six loops
        return f;
    }

    std::string fresh(const char* kind) { return std::string(kind) + std::to_string(counter_++); }

private:
    // loops: the dimensions of `shape` that are not literally 1 (a single loop of one iteration if none is left)
    static std::vector<size_t> kept_dims(const std::vector<Expression>& shape) {
        std::vector<size_t> kept;
        for (size_t d = 0; d < shape.size(); d++)
            if (shape[d] != "1") kept.push_back(d);
        return kept;
    }

    // Strides of a dense row-major operand of shape `own` (same rank as `shape` after right alignment; an extent of 1
    // where `shape` has more repeats the operand) along the loops, in the spelling the kernel planner merges loops by.
    static bool layout(const std::vector<Expression>& shape, std::vector<Expression> own, std::vector<Expression>* strides, Expression* extent) {
        if (own.size() > shape.size()) return false;
        own.insert(own.begin(), shape.size() - own.size(), "1");
        const std::vector<size_t> kept = kept_dims(shape);
        std::vector<Expression> per(kept.empty() ? 1 : kept.size(), "0");
        Expression run = "1";
        for (size_t k = kept.size(); k-- > 0;) {
            const size_t d = kept[k];
            if (own[d] == "1") continue;          // repeated along this loop
            if (own[d] != shape[d]) return false;
            per[k] = run;
            run = run == "1" ? own[d] : "(" + own[d] + ")*" + run;
        }
        *strides = per;
        *extent = run;
        return true;
    }

    static std::vector<Expression> bounds_of(const std::vector<Expression>& shape) {
        std::vector<Expression> b;
        for (size_t d : kept_dims(shape)) b.push_back(shape[d]);
        if (b.empty()) b.push_back("1");
        return b;
    }

    // a connector's value: a load (array), a kernel argument (scalar container or constant)
    bool operand(MapForm& f, const Block& blk, const std::string& connector, const std::vector<Expression>& shape,
                 const std::vector<Expression>& own_shape, std::string* value, std::optional<P> loaded_as = std::nullopt) {
        const ConnectorBinding* in = blk.input(connector);
        if (!in) return false;
        if (in->is_constant || !sdfg_.container(in->data).is_pointer) {
            // passed by value as the host code holds it: the local of the connector has the constant's or the container's type
            const P held = in->is_constant ? in->type : sdfg_.container(in->data).element;
            if (!floating(held)) return false;
            MapForm::Scalar s{*in, held, fresh("s")};
            *value = s.value;
            f.scalars.push_back(std::move(s));
            return true;
        }
        MapForm::Read r;
        r.data = in->data;
        r.element = loaded_as.value_or(f.element);
        if (!layout(shape, own_shape, &r.strides, &r.extent)) return false;
        r.value = fresh("r");
        *value = r.value;
        f.reads.push_back(std::move(r));
        return true;
    }

    bool result(MapForm& f, const Block& blk, const std::vector<Expression>& shape, const std::string& value) {
        MapForm::Result r;
        r.data = blk.outputs[0].data;
        r.value = value;
        r.element = f.element;
        if (!layout(shape, shape, &r.strides, &r.extent)) return false;
        f.results.push_back(std::move(r));
        return true;
    }

    std::string emit(MapForm& f, const std::string& op, std::vector<std::string> args) {
        Statement st{fresh("t"), f.element, op, std::move(args)};
        f.statements.push_back(st);
        return st.out;
    }

    // the operations of elementwise_ops.h as statements; empty: not spelled here
    std::string unary(MapForm& f, const std::string& code, const std::string& x) {
        static const std::map<std::string, std::string> calls = {{"ml::Abs", "fabs"}, {"ml::Exp", "exp"}, {"ml::Sqrt", "sqrt"},
                                                                 {"ml::Tanh", "tanh"}, {"ml::Erf", "erf"}};
        auto c = calls.find(code);
        if (c != calls.end()) return emit(f, c->second, {x});
        if (code == "ml::ReLU") return emit(f, "fmax", {x, "#0.0"});
        if (code == "ml::Sigmoid") {
            const std::string e = emit(f, "exp", {emit(f, "fp_neg", {x})});
            return emit(f, "fp_div", {"#1.0", emit(f, "fp_add", {"#1.0", e})});
        }
        return "";
    }

    std::string binary(MapForm& f, const std::string& code, const std::string& a, const std::string& b) {
        static const std::map<std::string, std::string> ops = {{"ml::Add", "fp_add"}, {"ml::Sub", "fp_sub"}, {"ml::Mul", "fp_mul"},
                                                               {"ml::Div", "fp_div"}, {"ml::Maximum", "fmax"}, {"ml::Minimum", "fmin"},
                                                               {"ml::Pow", "pow"}};
        auto o = ops.find(code);
        return o == ops.end() ? "" : emit(f, o->second, {a, b});
    }

    static bool floating(P t) { return t == P::Float || t == P::Double; }

    std::optional<MapForm> from_elementwise(const Block& blk, const tensor::ElementWiseNode& e) {
        if (!floating(e.element()) || e.shape().empty()) return std::nullopt;
        MapForm f;
        f.element = e.element();
        f.bounds = bounds_of(e.shape());
        std::string y;
        if (e.is_binary()) {
            std::string a, b;
            if (!operand(f, blk, "A", e.shape(), e.shape(), &a) || !operand(f, blk, "B", e.shape(), e.shape(), &b)) return std::nullopt;
            y = binary(f, e.code(), a, b);
        } else {
            std::string x;
            if (!operand(f, blk, "X", e.shape(), e.shape(), &x)) return std::nullopt;
            y = unary(f, e.code(), x);
        }
        if (y.empty() || !result(f, blk, e.shape(), y)) return std::nullopt;
        return f;
    }

    std::optional<MapForm> from_fused(const Block& blk, const ROCMFusedElementWiseNode& n) {
        if (!floating(n.element()) || n.shape().empty()) return std::nullopt;
        MapForm f;
        f.element = n.element();
        f.bounds = bounds_of(n.shape());
        std::string y;
        if (!operand(f, blk, "A", n.shape(), n.a_shape(), &y)) return std::nullopt;
        if (n.has_b()) {
            std::string b;
            if (!operand(f, blk, "B", n.shape(), n.b_shape(), &b)) return std::nullopt;
            y = binary(f, n.binary(), y, b);
            if (y.empty()) return std::nullopt;
        }
        for (auto& code : n.post()) {
            y = unary(f, code, y);
            if (y.empty()) return std::nullopt;
        }
        if (f.statements.empty()) y = emit(f, "assign", {y});
        if (!result(f, blk, n.shape(), y)) return std::nullopt;
        return f;
    }

    std::optional<MapForm> from_broadcast(const Block& blk, const tensor::BroadcastNode& b) {
        if (!floating(b.element()) || b.output_shape().empty()) return std::nullopt;
        MapForm f;
        f.element = b.element();
        f.bounds = bounds_of(b.output_shape());
        std::string x;
        if (!operand(f, blk, "X", b.output_shape(), b.input_shape(), &x)) return std::nullopt;
        if (!result(f, blk, b.output_shape(), emit(f, "assign", {x}))) return std::nullopt;
        return f;
    }

    // between float, double and bf16 (a bf16 tensor widened for the float32 nodes, their result rounded to bf16: the
    // compiler's conversions, to nearest even): the conversion is the assignment's
    std::optional<MapForm> from_cast(const Block& blk, const tensor::CastNode& c) {
        auto convertible = [](P t) { return floating(t) || t == P::BFloat; };
        if (!convertible(c.element()) || !convertible(c.target_type()) || c.shape().empty()) return std::nullopt;
        if (c.element() == P::BFloat && c.target_type() == P::BFloat) return std::nullopt;
        MapForm f;
        f.element = c.target_type();
        f.bounds = bounds_of(c.shape());
        std::string x;
        const ConnectorBinding* in = blk.input("X");
        if (!in || in->is_constant || !sdfg_.container(in->data).is_pointer) return std::nullopt;
        if (!operand(f, blk, "X", c.shape(), c.shape(), &x, c.element())) return std::nullopt;
        if (!result(f, blk, c.shape(), emit(f, "assign", {x}))) return std::nullopt;
        return f;
    }

    std::optional<MapForm> from_map(const Block& blk, const ROCMMapNode& m) {
        MapForm f;
        f.bounds = m.bounds();
        f.element = m.writes()[0].element;
        std::map<std::string, std::string> names;   // the node's names -> values of the pass
        for (auto& r : m.reads()) {
            const ConnectorBinding* in = blk.input(r.connector);
            if (!in || in->is_constant) return std::nullopt;
            names[r.connector] = fresh("r");
            f.reads.push_back({in->data, r.strides, r.extent, r.element, names[r.connector]});
        }
        for (auto& s : m.scalars()) {
            const ConnectorBinding* in = blk.input(s.connector);
            if (!in) return std::nullopt;
            names[s.connector] = fresh("s");
            f.scalars.push_back({*in, s.element, names[s.connector]});
        }
        auto renamed = [&](const std::string& name) { return name[0] == '#' ? name : names.at(name); };
        for (auto& st : m.statements()) {
            Statement out{fresh("t"), st.type, st.op, {}};
            for (auto& a : st.args) out.args.push_back(renamed(a));
            names[st.out] = out.out;
            f.statements.push_back(std::move(out));
        }
        for (auto& w : m.writes()) {
            const ConnectorBinding* out = blk.output(w.connector);
            if (!out) return std::nullopt;
            f.results.push_back({renamed(w.value), out->data, w.strides, w.extent, w.element});
        }
        return f;
    }

    const StructuredSDFG& sdfg_;
    size_t counter_ = 0;
};

// the scalar containers that `text` mentions
void scan_symbols(const StructuredSDFG& sdfg, const Expression& text, std::vector<std::string>& symbols) {
    std::string word;
    auto flush = [&]() {
        if (!word.empty() && !std::isdigit((unsigned char) word[0]) && sdfg.exists(word) && !sdfg.container(word).is_pointer &&
            std::find(symbols.begin(), symbols.end(), word) == symbols.end())
            symbols.push_back(word);
        word.clear();
    };
    for (char ch : text) {
        if (std::isalnum((unsigned char) ch) || ch == '_') word += ch;
        else flush();
    }
    flush();
}

// The form as a node and its bindings, in place of the node of `blk`.
void install(const StructuredSDFG& sdfg, Block& blk, const MapForm& f) {
    std::map<std::string, std::string> names;
    std::vector<ROCMMapNode::Access> reads, writes;
    std::vector<ROCMMapNode::ScalarOperand> scalars;
    std::vector<ConnectorBinding> inputs;
    for (auto& r : f.reads) {
        // one load per (container, index form)
        std::string connector;
        for (size_t k = 0; k < reads.size(); k++)
            if (inputs[k].data == r.data && reads[k].strides == r.strides && reads[k].element == r.element) connector = reads[k].connector;
        if (connector.empty()) {
            connector = "_in" + std::to_string(reads.size());
            reads.push_back({connector, r.strides, r.extent, r.element, ""});
            ConnectorBinding b;
            b.connector = connector;
            b.data = r.data;
            inputs.push_back(b);
        }
        names[r.value] = connector;
    }
    std::vector<ConnectorBinding> scalar_inputs;
    for (auto& s : f.scalars) {
        std::string connector;
        for (size_t k = 0; k < scalars.size(); k++)
            if (scalar_inputs[k].is_constant == s.source.is_constant && scalar_inputs[k].data == s.source.data &&
                scalar_inputs[k].type == s.source.type && scalars[k].element == s.element)
                connector = scalars[k].connector;
        if (connector.empty()) {
            connector = "_c" + std::to_string(scalars.size());
            scalars.push_back({connector, s.element});
            ConnectorBinding b = s.source;
            b.connector = connector;
            scalar_inputs.push_back(b);
        }
        names[s.value] = connector;
    }
    inputs.insert(inputs.end(), scalar_inputs.begin(), scalar_inputs.end());
    std::vector<Statement> statements;
    auto renamed = [&](const std::string& name) { return name[0] == '#' ? name : names.at(name); };
    for (auto& st : f.statements) {
        Statement out{"_v" + std::to_string(statements.size()), st.type, st.op, {}};
        for (auto& a : st.args) out.args.push_back(renamed(a));
        names[st.out] = out.out;
        statements.push_back(std::move(out));
    }
    std::vector<ConnectorBinding> outputs;
    for (auto& r : f.results) {
        ConnectorBinding b;
        b.connector = "_out" + std::to_string(writes.size());
        b.data = r.data;
        writes.push_back({b.connector, r.strides, r.extent, r.element, renamed(r.value)});
        outputs.push_back(b);
    }
    std::vector<std::string> indvars, symbols;
    for (size_t l = 0; l < f.bounds.size(); l++) {
        indvars.push_back("_i" + std::to_string(l));
        scan_symbols(sdfg, f.bounds[l], symbols);
    }
    for (auto* list : {&reads, &writes})
        for (auto& a : *list)
            for (auto& st : a.strides) scan_symbols(sdfg, st, symbols);
    auto node = std::make_unique<ROCMMapNode>(blk.node->implementation_type(), indvars, f.bounds, symbols, reads, writes, scalars, statements);
    node->set_element_id(blk.node->element_id());
    blk.node = std::move(node);
    blk.inputs = std::move(inputs);
    blk.outputs = std::move(outputs);
}

bool written_between(const StructuredSDFG& sdfg, const std::string& name, size_t from, size_t to) {
    for (size_t i = from + 1; i < to; i++)
        for (auto& out : sdfg.blocks()[i].outputs)
            if (out.data == name) return true;
    return false;
}

bool touched_between(const StructuredSDFG& sdfg, const std::string& name, size_t from, size_t to) {
    for (size_t i = from + 1; i < to; i++) {
        for (auto& in : sdfg.blocks()[i].inputs)
            if (!in.is_constant && in.data == name) return true;
        for (auto& out : sdfg.blocks()[i].outputs)
            if (out.data == name) return true;
    }
    return false;
}

// a value that only block `reader` reads and only block `writer` writes, and that nobody outside the function sees
bool private_to(const StructuredSDFG& sdfg, const std::string& name, size_t writer, size_t reader) {
    const Container& c = sdfg.container(name);
    if (c.is_argument || !c.transient || name == sdfg.return_container()) return false;
    for (size_t b = 0; b < sdfg.blocks().size(); b++) {
        for (auto& in : sdfg.blocks()[b].inputs)
            if (!in.is_constant && in.data == name && b != reader) return false;
        for (auto& out : sdfg.blocks()[b].outputs)
            if (out.data == name && b != writer) return false;
    }
    return true;
}

} // namespace

bool RocmMapFusionPass::run_pass(builder::StructuredSDFGBuilder& builder, analysis::AnalysisManager&) {
    StructuredSDFG& sdfg = builder.subject();
    auto& blocks = sdfg.blocks();
    Converter convert(sdfg);
    bool applied = false;
    bool changed = true;
    while (changed) {
        changed = false;
        for (size_t j = 0; j < blocks.size() && !changed; j++) {
            std::optional<MapForm> consumer = convert.form_of(blocks[j]);
            if (!consumer) continue;
            for (size_t k = 0; k < consumer->reads.size() && !changed; k++) {
                // the block that wrote what this load reads: the last writer before j, and the only one
                const std::string link = consumer->reads[k].data;
                long writer = -1;
                size_t writers = 0;
                for (size_t b = 0; b < blocks.size(); b++)
                    for (auto& out : blocks[b].outputs)
                        if (out.data == link) {
                            writers++;
                            if (b < j) writer = (long) b;
                        }
                if (writer < 0 || writers != 1) continue;
                const size_t i = (size_t) writer;
                if (blocks[i].node->implementation_type() != blocks[j].node->implementation_type()) continue;
                std::optional<MapForm> producer = convert.form_of(blocks[i]);
                if (!producer) continue;

                // The producer's loops among the consumer's. Equal bounds: loop for loop. Fewer loops (a value per row
                // that the consumer repeats along the others): the consumer's loops along which the link is indexed,
                // in order; the producer's work is then done again for every iteration of the other loops, which is
                // cheaper than a launch and a round trip through memory for values this small.
                std::vector<long> at(consumer->bounds.size(), -1);     // consumer loop -> producer loop
                const MapForm::Result* linked = nullptr;
                for (auto& r : producer->results)
                    if (r.data == link) linked = &r;
                if (!linked) continue;
                const bool same_loops = producer->bounds == consumer->bounds;
                if (same_loops) {
                    for (size_t l = 0; l < at.size(); l++) at[l] = (long) l;
                } else {
                    size_t next = 0;
                    bool fits = true;
                    for (size_t l = 0; l < at.size(); l++) {
                        if (consumer->reads[k].strides[l] == "0") continue;
                        if (next >= producer->bounds.size() || producer->bounds[next] != consumer->bounds[l]) fits = false;
                        else at[l] = (long) next++;
                    }
                    // (a short chain only: it is repeated for every element of the consumer)
                    if (!fits || next != producer->bounds.size() || producer->statements.size() > 8) continue;
                }
                auto along_consumer = [&](const std::vector<Expression>& strides) {
                    std::vector<Expression> out(at.size(), "0");
                    for (size_t l = 0; l < at.size(); l++)
                        if (at[l] >= 0) out[l] = strides[(size_t) at[l]];
                    return out;
                };
                // every load of a producer result takes the element the producer's iteration stores
                bool same_elements = true;
                for (auto& r : consumer->reads)
                    for (auto& pr : producer->results)
                        if (r.data == pr.data && (r.strides != along_consumer(pr.strides) || r.element != pr.element)) same_elements = false;
                if (!same_elements) continue;
                // Which producer results are still stored: those somebody else looks at. They are stored where the
                // consumer stands, so nobody may look at them in between; with fewer loops than the consumer they
                // would be stored over and over, so there all of them must be private to the two blocks.
                std::vector<MapForm::Result> kept;
                bool ok = true;
                for (auto& pr : producer->results) {
                    if (private_to(sdfg, pr.data, i, j)) continue;
                    if (!same_loops || touched_between(sdfg, pr.data, i, j)) ok = false;
                    for (auto& cr : consumer->results)
                        if (cr.data == pr.data) ok = false;
                    kept.push_back(pr);
                }
                // the producer's work moves to where the consumer stands: what it reads must still hold the same
                // values there, and a consumer result may alias a producer operand only element by element
                for (auto& r : producer->reads) {
                    if (written_between(sdfg, r.data, i, j)) ok = false;
                    for (auto& cr : consumer->results)
                        if (r.data == cr.data && along_consumer(r.strides) != cr.strides) ok = false;
                }
                for (auto& sc : producer->scalars)
                    if (!sc.source.is_constant && written_between(sdfg, sc.source.data, i, j)) ok = false;
                if (!ok) continue;

                MapForm merged;
                merged.bounds = consumer->bounds;
                merged.element = consumer->element;
                for (auto r : producer->reads) {
                    r.strides = along_consumer(r.strides);
                    merged.reads.push_back(std::move(r));
                }
                merged.scalars = producer->scalars;
                merged.statements = producer->statements;
                std::map<std::string, std::string> forwarded;   // consumer loads of producer results -> the producer's values
                for (auto& r : consumer->reads) {
                    const MapForm::Result* from = nullptr;
                    for (auto& pr : producer->results)
                        if (pr.data == r.data) from = &pr;
                    if (from) forwarded[r.value] = from->value;
                    else merged.reads.push_back(r);
                }
                merged.scalars.insert(merged.scalars.end(), consumer->scalars.begin(), consumer->scalars.end());
                auto through = [&](const std::string& name) {
                    auto it = forwarded.find(name);
                    return it == forwarded.end() ? name : it->second;
                };
                for (auto st : consumer->statements) {
                    for (auto& a : st.args) a = through(a);
                    merged.statements.push_back(std::move(st));
                }
                merged.results = kept;
                for (auto r : consumer->results) {
                    r.value = through(r.value);
                    merged.results.push_back(std::move(r));
                }
                // a result that is a loaded value or a literal as it stands needs a statement of its own
                for (auto& r : merged.results) {
                    bool is_statement = false;
                    for (auto& st : merged.statements) is_statement = is_statement || st.out == r.value;
                    if (!is_statement) {
                        Statement copy{convert.fresh("t"), r.element, "assign", {r.value}};
                        r.value = copy.out;
                        merged.statements.push_back(std::move(copy));
                    }
                }
                std::vector<std::string> dropped;
                for (auto& pr : producer->results)
                    if (private_to(sdfg, pr.data, i, j)) dropped.push_back(pr.data);
                install(sdfg, blocks[j], merged);
                blocks.erase(blocks.begin() + (long) i);
                for (auto& name : dropped) sdfg.remove_container(name);
                changed = applied = true;
            }
        }
    }
    return applied;
}

} // namespace sdfg::rocm
