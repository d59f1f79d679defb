// Conversion between the reference's SDFG wire format and the block list of this target.
//
// The reference writes an SDFG as (sdfg/src/serializer/json_serializer.cpp:56-353)
//   { name, element_counter, type, return_type, structures[], containers{name: <type>}, arguments[],
//     externals[], metadata{}, root: <sequence> }
//   <sequence> = { type "sequence", children[], transitions[] }, children: block | for | map | while |
//                if_else | return | break | continue | sequence
//   block.dataflow = { nodes[], edges[] }; nodes: access_node {data} | constant_node {data, data_type} |
//                    tasklet | library_node {code, implementation_type, ...payload};
//                    edges: {src, dst, src_conn, dst_conn, subset[], base_type}
//   <type> = { type: scalar | pointer | array | structure | function | tensor | reference,
//              primitive_type (enum value), pointee_type / element_type, storage_type {value, allocation,
//              deallocation, allocation_size?}, ... }
// What the rocm target can take from it is a root sequence of blocks that hold one library node
// each (with its access and constant nodes), allocation and release of temporaries (Malloc / Free
// nodes, managed storage), a final return, and the loop nests that are elementwise work in disguise:
// a perfect nest of Maps (or of the Fors the front end writes before its For2Map pass) over one block
// with one tasklet or CMath node whose operands are dense tensors indexed by the loop variables. That is
// the form the elementwise tensor nodes expand to (elementwise_node.cpp:86-240) and the form of the copy
// into the return buffer (python/docc/python/ast_parser.py:1186-1210, :2102-2270); it is folded back into
// the node the target has a kernel for (ml::Transpose for a copy, ml::Fill, the elementwise nodes). The
// reference's CUDA target instead prints a kernel per Map nest (opt/src/targets/cuda/codegen/
// cuda_map_dispatcher.cpp:42-168); here the kernels exist already, so the nest is matched, not compiled.
// A scalar stored through an assign tasklet (the scalar form of the return copy) becomes an ml::Fill of one
// element. The expansion of a reduce node (reduce_node.cpp:186-330: a nest that stores the identity, then maps
// around fors whose body accumulates onto the result) is folded back into ml::Sum / ml::Max / ml::Min, and a copy
// whose source some loops do not index (broadcast_node.cpp:110-187) into ml::Broadcast, so that an expanded softmax
// arrives as the seven nodes the softmax pattern pass knows. Other loops, tasklets and branches have no lowering
// and are refused with the element named.
#include <algorithm>
#include <cctype>
#include <map>
#include <set>

#include "rocm_target.h"
#include "sdfg_lite.h"

namespace sdfg::serializer {

using json::Array;
using json::Object;
using json::Value;

namespace {

// enum PrimitiveType of the reference (sdfg/include/sdfg/types/type.h:35-55), by value
const char* const kReferencePrimitive[] = {"Void",  "Bool",   "Int8",   "Int16",   "Int32", "Int64",  "Int128", "UInt8",
                                           "UInt16", "UInt32", "UInt64", "UInt128", "Half",  "BFloat", "Float",  "Double"};

types::PrimitiveType primitive_of(const Value& v, const std::string& where) {
    const int64_t i = v.as_int();
    if (i < 0 || i >= (int64_t) (sizeof(kReferencePrimitive) / sizeof(kReferencePrimitive[0])) || i == 6 || i == 11)
        throw InvalidSDFGException(where + ": primitive type " + std::to_string(i) + " is not supported");
    return types::primitive_type_from_string(kReferencePrimitive[i]);
}

int64_t reference_primitive(types::PrimitiveType t) {
    const std::string name = types::primitive_type_to_string(t);
    for (size_t i = 0; i < sizeof(kReferencePrimitive) / sizeof(kReferencePrimitive[0]); i++)
        if (name == kReferencePrimitive[i]) return (int64_t) i;
    return 0;
}

// element type behind a scalar, pointer, array or tensor type
types::PrimitiveType element_of(const Value& type, const std::string& where) {
    const std::string kind = type.at("type").as_string();
    if (kind == "scalar") return primitive_of(type.at("primitive_type"), where);
    if (kind == "pointer") {
        const Value* pointee = type.find("pointee_type");
        if (!pointee) throw InvalidSDFGException(where + ": opaque pointer");
        return element_of(*pointee, where);
    }
    if (kind == "array" || kind == "tensor") return element_of(type.at("element_type"), where);
    throw InvalidSDFGException(where + ": " + kind + " types are not supported by the rocm target");
}

// Expressions arrive in SymEngine's spelling; the only construct of it that is not C is the power
// operator. `base**n` (n a small non-negative integer) becomes a product.
std::string c_expression(std::string e) {
    for (size_t at = e.find("**"); at != std::string::npos; at = e.find("**")) {
        size_t begin = at;
        if (begin > 0 && e[begin - 1] == ')') {
            int depth = 0;
            while (begin > 0) {
                begin--;
                if (e[begin] == ')') depth++;
                if (e[begin] == '(' && --depth == 0) break;
            }
            if (depth != 0) throw InvalidSDFGException("unbalanced expression '" + e + "'");
        } else {
            while (begin > 0 && (std::isalnum((unsigned char) e[begin - 1]) || e[begin - 1] == '_' || e[begin - 1] == '.')) begin--;
        }
        size_t end = at + 2;
        while (end < e.size() && std::isdigit((unsigned char) e[end])) end++;
        if (begin == at || end == at + 2 || end - (at + 2) > 2)
            throw InvalidSDFGException("power in '" + e + "' is not a small integer power of a term");
        const std::string base = e.substr(begin, at - begin);
        const int n = std::stoi(e.substr(at + 2, end - (at + 2)));
        std::string product = n == 0 ? "1" : "(" + base;
        for (int i = 1; i < n; i++) product += "*" + base;
        if (n > 0) product += ")";
        e = e.substr(0, begin) + product + e.substr(end);
    }
    return e;
}

// the same rewrite on every string inside a node payload
Value c_expressions(const Value& v) {
    if (v.is_string()) return Value(c_expression(v.as_string()));
    if (v.is_array()) {
        Array a;
        for (auto& e : v.as_array()) a.push_back(c_expressions(e));
        return Value(std::move(a));
    }
    if (v.is_object()) {
        Object o;
        for (auto& kv : v.as_object()) o.emplace_back(kv.first, c_expressions(kv.second));
        return Value(std::move(o));
    }
    return v;
}

std::string describe(const Value& element) {
    std::string s = element.at("type").as_string();
    if (const Value* id = element.find("element_id")) s += " (element " + std::to_string(id->as_int()) + ")";
    return s;
}

Value debug_info_of(const Value& element) {
    const Value* d = element.find("debug_info");
    if (d && d->is_object()) {
        const Value* has = d->find("has");
        if (has && has->is_bool() && has->as_bool()) return *d;
    }
    return Value();
}


// ---- expressions of loop nests ---------------------------------------------------------------
// Index arithmetic arrives as SymEngine prints it ("_i0", "_s1*_i0 + _i1", "1 + _i0", "_i0 < _s0"). The
// matcher needs sums of products only: a term is an integer coefficient times a sorted list of symbols.

std::string strip(const std::string& e) {
    std::string s;
    for (char c : e)
        if (!std::isspace((unsigned char) c)) s += c;
    // outer parentheses that span the whole expression
    for (bool again = true; again && s.size() >= 2 && s.front() == '(' && s.back() == ')';) {
        int depth = 0;
        again = true;
        for (size_t i = 0; i + 1 < s.size(); i++) {
            if (s[i] == '(') depth++;
            if (s[i] == ')') depth--;
            if (depth == 0) {
                again = false;
                break;
            }
        }
        if (again) s = s.substr(1, s.size() - 2);
    }
    return s;
}

std::vector<std::string> split_top(const std::string& e, char sep) {
    std::vector<std::string> parts;
    int depth = 0;
    std::string cur;
    for (char c : e) {
        if (c == '(') depth++;
        if (c == ')') depth--;
        if (c == sep && depth == 0) {
            parts.push_back(cur);
            cur.clear();
        } else {
            cur += c;
        }
    }
    parts.push_back(cur);
    return parts;
}

struct Term {
    int64_t coefficient = 1;
    std::vector<std::string> symbols;   // sorted
    bool operator==(const Term& o) const { return coefficient == o.coefficient && symbols == o.symbols; }
};

// a product of integers and symbols; false for anything else (sums inside, divisions, calls)
bool parse_term(const std::string& text, Term* out) {
    Term t;
    for (auto& f : split_top(strip(text), '*')) {
        const std::string factor = strip(f);
        if (factor.empty()) return false;
        int64_t v = 0;
        if (symbolic::is_integer(factor, &v)) {
            t.coefficient *= v;
            continue;
        }
        for (char c : factor)
            if (!(std::isalnum((unsigned char) c) || c == '_')) return false;
        if (std::isdigit((unsigned char) factor[0])) return false;
        t.symbols.push_back(factor);
    }
    std::sort(t.symbols.begin(), t.symbols.end());
    *out = t;
    return true;
}

Term term_product(const Term& a, const Term& b) {
    Term t;
    t.coefficient = a.coefficient * b.coefficient;
    t.symbols = a.symbols;
    t.symbols.insert(t.symbols.end(), b.symbols.begin(), b.symbols.end());
    std::sort(t.symbols.begin(), t.symbols.end());
    return t;
}

// One loop of a nest in the only form matched: for (var = 0; var < extent; var = var + 1)
struct NestLoop {
    std::string var;
    Expression extent;
    Term extent_term;
};

// How an operand walks memory: a stride (in elements) per loop of the nest; `dense` tells in which order of
// the loops the strides are those of a C-contiguous tensor over the loops' extents (outermost first).
struct OperandWalk {
    bool scalar = false;               // a constant or a scalar container
    Value binding;                     // {"data": ...} or {"constant": ..., "type": ...}
    std::vector<int> order;            // loop indices, outermost dimension first
    std::vector<int> missing;          // loops of the nest that do not index the operand (a reduced or a repeated extent)
    int units = 0;                     // dimensions indexed by the constant 0 (extent 1: a kept or a repeated dimension)
    bool partial() const { return !missing.empty() || units > 0; }
    bool uses(int loop) const { return std::find(order.begin(), order.end(), loop) != order.end(); }
};

struct Import {
    const Value& src;
    Value out;
    Object containers;   // lite container entries, by name
    std::set<std::string> transient_done;

    explicit Import(const Value& j) : src(j) {}

    Value& container(const std::string& name) {
        for (auto& kv : containers)
            if (kv.first == name) return kv.second;
        throw InvalidSDFGException("container '" + name + "' does not exist");
    }

    void import_containers() {
        for (auto& kv : src.at("containers").as_object()) {
            const Value& t = kv.second;
            const std::string kind = t.at("type").as_string();
            const std::string where = "container '" + kv.first + "'";
            Value c;
            if (kind == "scalar") {
                c.set("type", "scalar");
            } else if (kind == "pointer") {
                c.set("type", "pointer");
            } else {
                throw InvalidSDFGException(where + ": " + kind + " types are not supported by the rocm target");
            }
            c.set("element", types::primitive_type_to_string(element_of(t, where)));
            bool transient = false;
            std::string storage = "CPU";
            if (const Value* st = t.find("storage_type")) {
                const std::string v = st->at("value").as_string();
                if (v == "ROCM_Generic")
                    storage = v;
                else if (v.rfind("CPU", 0) != 0)
                    throw InvalidSDFGException(where + ": storage " + v + " belongs to another target");
                // managed allocation: the generated function owns the buffer (reference type.h:67-79)
                const Value* alloc = st->find("allocation");
                const Value* size = st->find("allocation_size");
                if (alloc && alloc->as_int() == 1 && size) {
                    transient = true;
                    c.set("size", c_expression(size->as_expression()));
                }
            }
            c.set("transient", transient);
            c.set("storage", storage);
            containers.emplace_back(kv.first, std::move(c));
        }
    }

    // a block of the reference -> nullopt (nothing to do) or one lite block
    bool import_block(const Value& block, Array& children) {
        const Value& df = block.at("dataflow");
        const Array& nodes = df.at("nodes").as_array();
        if (nodes.empty()) return false;   // e.g. the empty view block add_gemm leaves behind
        std::map<int64_t, const Value*> by_id;
        const Value* lib = nullptr;
        for (auto& n : nodes) {
            by_id[n.at("element_id").as_int()] = &n;
            const std::string kind = n.at("type").as_string();
            if (kind == "tasklet" || (kind == "library_node" && n.at("code").as_string() == "CMath")) {
                // a statement outside any loop: the scalar forms (a scalar stored into a buffer)
                lower_tasklet_block(block, {}, children);
                return true;
            }
            if (kind == "library_node") {
                if (lib) throw InvalidSDFGException(describe(block) + ": more than one library node in a block");
                lib = &n;
            }
        }
        if (!lib) return false;   // access nodes only: no computation
        const int64_t lib_id = lib->at("element_id").as_int();
        const std::string code = lib->at("code").as_string();

        auto node_of = [&](const Value& edge, const char* end) -> const Value& {
            auto it = by_id.find(edge.at(end).as_int());
            if (it == by_id.end()) throw InvalidSDFGException(describe(block) + ": edge refers to an unknown node");
            return *it->second;
        };

        Array inputs, outputs;
        const Value* out_type = nullptr;
        const Value* in_type = nullptr;
        bool has_bias_edge = false;
        for (auto& e : df.at("edges").as_array()) {
            const bool into = e.at("dst").as_int() == lib_id, from = e.at("src").as_int() == lib_id;
            if (!into && !from) throw InvalidSDFGException(describe(block) + ": data movement beside the library node");
            for (auto& s : e.at("subset").as_array())
                if (s.as_expression() != "0")
                    throw InvalidSDFGException(describe(block) + ": a subset on an operand of " + code + " (views are not supported)");
            Value b;
            if (into) {
                const Value& n = node_of(e, "src");
                b.set("connector", e.at("dst_conn").as_string());
                if (n.at("type").as_string() == "constant_node") {
                    b.set("constant", c_expression(n.at("data").as_expression()));
                    b.set("type", types::primitive_type_to_string(element_of(n.at("data_type"), describe(n))));
                } else {
                    b.set("data", n.at("data").as_string());
                }
                if (!in_type) in_type = &e.at("base_type");
                if (e.at("dst_conn").as_string() == "B") has_bias_edge = true;
                inputs.push_back(std::move(b));
            } else {
                const Value& n = node_of(e, "dst");
                b.set("connector", e.at("src_conn").as_string());
                b.set("data", n.at("data").as_string());
                out_type = &e.at("base_type");
                outputs.push_back(std::move(b));
            }
        }

        // allocation and release of a temporary: the container becomes a transient of the function
        if (code == "Malloc") {
            if (outputs.size() != 1) throw InvalidSDFGException(describe(*lib) + ": Malloc without a target");
            Value& c = container(outputs[0].at("data").as_string());
            c.set("transient", true);
            c.set("size", c_expression(lib->at("size").as_expression()));
            return false;
        }
        if (code == "Free") return false;

        Value node{Object{}};
        for (auto& kv : lib->as_object())
            if (kv.first != "debug_info") node.set(kv.first, c_expressions(kv.second));
        node.set("side_effect", false);
        // what the reference keeps in the memlet types, the block list keeps on the node
        if (code == "ml::Cast") {   // "target_type" is the enum value there, the name here; the element type is the input's
            if (!in_type) throw InvalidSDFGException(describe(*lib) + ": no input edge");
            const Value* tt = node.find("target_type");
            if (tt && tt->is_number()) node.set("target_type", types::primitive_type_to_string(primitive_of(*tt, describe(*lib))));
            if (!node.contains("element_type")) node.set("element_type", types::primitive_type_to_string(element_of(*in_type, describe(*lib))));
        }
        if (code != "GEMM" && !node.contains("element_type")) {
            if (!out_type) throw InvalidSDFGException(describe(*lib) + ": no output edge");
            node.set("element_type", types::primitive_type_to_string(element_of(*out_type, describe(*lib))));
        }
        if (code == "ml::Conv" && !node.contains("has_bias")) node.set("has_bias", has_bias_edge);
        if (code == "ml::MatMul") {
            for (const char* key : {"offset_a", "offset_b"})
                if (const Value* o = node.find(key))
                    if (o->as_expression() != "0") throw InvalidSDFGException(describe(*lib) + ": ml::MatMul with an operand offset");
            for (const char* key : {"strides_a", "strides_b"})
                if (const Value* s = node.find(key))
                    if (!s->as_array().empty() && s->as_array().back().as_expression() != "1")
                        throw InvalidSDFGException(describe(*lib) + ": ml::MatMul on a non-contiguous operand");
        }

        Value flow;
        flow.set("library_node", std::move(node));
        flow.set("inputs", Value(std::move(inputs)));
        flow.set("outputs", Value(std::move(outputs)));
        Value b;
        b.set("type", "block");
        b.set("element_id", block.at("element_id").as_int());
        Value dbg = debug_info_of(*lib);
        if (dbg.is_null()) dbg = debug_info_of(block);
        if (!dbg.is_null()) b.set("debug_info", std::move(dbg));
        b.set("dataflow", std::move(flow));
        children.push_back(std::move(b));
        return true;
    }


    [[noreturn]] void refuse(const Value& element, const std::string& why) {
        throw InvalidSDFGException(describe(element) + ": " + why + " (the rocm target lowers library nodes and the elementwise loop nests "
                                   "that match one of its kernels)");
    }

    // strides of `edge`'s operand per loop of the nest -> order of the loops in which it is dense
    bool walk_of(const Value& block, const Value& edge, const Value& node, const std::vector<NestLoop>& loops, OperandWalk* walk) {
        const std::string kind = node.at("type").as_string();
        if (kind == "constant_node") {
            walk->scalar = true;
            walk->binding.set("constant", c_expression(node.at("data").as_expression()));
            walk->binding.set("type", types::primitive_type_to_string(element_of(node.at("data_type"), describe(node))));
            return true;
        }
        const std::string data = node.at("data").as_string();
        walk->binding.set("data", data);
        const Value& c = container(data);
        if (c.at("type").as_string() == "scalar") {
            walk->scalar = true;
            auto known = assigned.find(data);
            if (known != assigned.end()) {
                // converted to the element type of the operation that reads it, as the generated C of the reference would
                Value b{Object{}};
                b.set("constant", "(" + c_expression(known->second) + ")");
                b.set("type", types::primitive_type_to_string(element_of(edge.at("base_type"), describe(node))));
                walk->binding = std::move(b);
            }
            return true;
        }
        const Value& type = edge.at("base_type");
        const std::string tkind = type.at("type").as_string();
        const Array& subset = edge.at("subset").as_array();
        if (loops.empty()) {
            // a statement outside any loop touches one element of a buffer: only the first one has a form here
            // (the caller allows it as the place a scalar is stored to)
            for (auto& sub : subset)
                if (strip(sub.as_expression()) != "0") return false;
            walk->scalar = true;
            return true;
        }
        std::vector<Term> strides(loops.size());
        std::vector<bool> seen(loops.size(), false);
        auto loop_of = [&](const std::string& name) {
            for (size_t l = 0; l < loops.size(); l++)
                if (loops[l].var == name) return (int) l;
            return -1;
        };
        if (tkind == "tensor") {
            // one index per dimension, each a loop variable; the strides are the type's
            const Array& tstrides = type.at("strides").as_array();
            if (subset.size() != tstrides.size()) return false;
            if (const Value* off = type.find("offset"))
                if (strip(off->as_expression()) != "0") return false;
            for (size_t d = 0; d < subset.size(); d++) {
                const std::string index = strip(subset[d].as_expression());
                if (index == "0") {   // a dimension of extent 1 (a reduced dimension that was kept, or one that is repeated)
                    walk->units++;
                    continue;
                }
                const int l = loop_of(index);
                Term st;
                if (l < 0 || seen[l] || !parse_term(tstrides[d].as_expression(), &st)) return false;
                if (st.coefficient == 0) {   // a repeated dimension of a view (the front end's broadcasting, numpy.py:2679-2705)
                    walk->units++;
                    continue;                // the loop stays unseen: it does not index the operand's memory
                }
                seen[l] = true;
                strides[l] = st;
            }
        } else if (tkind == "pointer" || tkind == "array") {
            // one linearised index: a sum of (stride * loop variable) terms
            if (subset.size() != 1) return false;
            for (auto& part : split_top(strip(subset[0].as_expression()), '+')) {
                Term t;
                if (!parse_term(part, &t)) return false;
                int l = -1;
                for (size_t k = 0; k < t.symbols.size(); k++) {
                    const int hit = loop_of(t.symbols[k]);
                    if (hit >= 0) {
                        if (l >= 0) return false;   // a product of two loop variables
                        l = hit;
                        t.symbols.erase(t.symbols.begin() + (long) k);
                        k--;
                    }
                }
                if (l < 0 || seen[l]) return false;   // a constant offset, or a variable twice
                seen[l] = true;
                strides[l] = t;
            }
        } else {
            return false;
        }
        // loops that do not index the operand: the callers that know reductions and broadcasts look at `missing`
        std::vector<bool> used(loops.size(), false);
        for (size_t l = 0; l < loops.size(); l++)
            if (!seen[l]) {
                walk->missing.push_back((int) l);
                used[l] = true;
            }
        // innermost: stride 1; then the loop whose stride is the product of the extents found so far; ...
        std::vector<int> inner_first;
        Term expect;
        for (size_t n = 0; n < loops.size(); n++) {
            int found = -1;
            for (size_t l = 0; l < loops.size(); l++)
                if (!used[l] && strides[l] == expect) found = (int) l;
            if (found < 0) {
                // extents of 1 have any stride; nothing else may be left
                for (size_t l = 0; l < loops.size(); l++)
                    if (!used[l] && !(loops[l].extent_term == Term{})) return false;
                for (size_t l = 0; l < loops.size(); l++)
                    if (!used[l]) inner_first.push_back((int) l);
                break;
            }
            used[found] = true;
            inner_first.push_back(found);
            expect = term_product(expect, loops[found].extent_term);
        }
        walk->order.assign(inner_first.rbegin(), inner_first.rend());
        (void) block;
        return true;
    }

    // `element` is a for or a map: the nest below it. A body of one operation is matched against the prebuilt kernels
    // first (elementwise nodes, copies, fills, reductions, repeated operands); what they do not cover - several
    // operations, operands that walk memory in different orders, operations without a node - becomes one generated
    // kernel (ROCMMap) if every loop of the nest is a map, i.e. its iterations are independent by construction.
    void import_loop_nest(const Value& element, Array& children) {
        std::vector<NestLoop> loops;
        std::vector<const Value*> body;
        bool all_maps = true;
        const Value* at = &element;
        while (body.empty()) {
            const std::string kind = at->at("type").as_string();
            const Value* seq = nullptr;
            if (kind == "for" || kind == "map") {
                NestLoop loop;
                loop.var = strip(at->at("indvar").as_expression());
                if (strip(at->at("init").as_expression()) != "0") refuse(*at, "the loop does not start at 0");
                const std::string update = strip(at->at("update").as_expression());
                if (update != "1+" + loop.var && update != loop.var + "+1") refuse(*at, "the loop's step is not 1");
                const std::string cond = strip(at->at("condition").as_expression());
                if (cond.rfind(loop.var + "<", 0) != 0 || cond.find("<=") != std::string::npos) refuse(*at, "the loop's condition is not 'variable < bound'");
                loop.extent = c_expression(strip(cond.substr(loop.var.size() + 1)));
                if (!parse_term(loop.extent, &loop.extent_term)) refuse(*at, "the loop's bound is not a product of symbols and integers");
                loops.push_back(loop);
                all_maps = all_maps && kind == "map";
                seq = &at->at("root");
            } else if (kind == "sequence") {
                seq = at;
            } else if (kind == "block") {
                body.push_back(at);
                break;
            } else {
                refuse(*at, "control flow inside a loop nest");
            }
            if (const Value* transitions = seq->find("transitions"))
                for (auto& t : transitions->as_array())
                    if (!t.at("assignments").as_array().empty()) refuse(t, "symbol assignments inside a loop nest");
            std::vector<const Value*> kids;
            for (auto& child : seq->at("children").as_array()) {
                if (child.at("type").as_string() == "block" && child.at("dataflow").at("nodes").as_array().empty()) continue;
                kids.push_back(&child);
            }
            if (kids.empty()) return;   // an empty nest does nothing
            if (kids.size() == 1) {
                at = kids[0];
                continue;
            }
            // several statements: the body of the innermost loop, a run of blocks
            for (const Value* k : kids)
                if (k->at("type").as_string() != "block") refuse(*at, "more than one statement in a loop body, one of them control flow");
            if (!all_maps) refuse(*at, "more than one statement in a loop body (several statements are lowered under maps only)");
            body = kids;
        }
        if (loops.size() > 6) refuse(element, "a loop nest deeper than 6");
        size_t operations = 0;
        for (const Value* b : body)
            for (auto& n : b->at("dataflow").at("nodes").as_array()) {
                const std::string kind = n.at("type").as_string();
                operations += kind == "tasklet" || kind == "library_node";
            }
        if (body.size() == 1 && operations <= 1) {
            if (!all_maps) {
                lower_tasklet_block(*body[0], loops, children);
                return;
            }
            // what the attempt adds before it gives up (a repeated operand's temporary and its Broadcast) goes again
            const size_t n_children = children.size(), n_containers = containers.size();
            try {
                lower_tasklet_block(*body[0], loops, children);
                return;
            } catch (const InvalidSDFGException&) {
                children.resize(n_children);
                containers.resize(n_containers);
            }
        }
        lower_map_nest(element, body, loops, children);
    }

    // The body blocks of a nest of maps as one ROCMMap node (see sdfg_lite.h): loads, a list of statements, stores.
    void lower_map_nest(const Value& element, const std::vector<const Value*>& body, const std::vector<NestLoop>& loops, Array& children) {
        static const std::map<int64_t, std::string> tasklet_names = {{0, "assign"}, {1, "fp_neg"}, {2, "fp_add"}, {3, "fp_sub"},
                                                                     {4, "fp_mul"}, {5, "fp_div"}, {6, "fp_rem"}, {7, "fp_fma"}};
        using P = types::PrimitiveType;
        Array reads, writes, scalars, statements, inputs, outputs;
        std::map<std::string, std::string> current;      // scalar container written in the body -> the value it holds now
        std::map<std::string, std::string> stored;       // container|strides -> the value this nest stores there
        std::map<std::string, size_t> write_at;          // container|strides -> index in `writes`
        std::map<std::string, std::string> read_conn;    // container|strides -> connector of the load
        std::map<std::string, std::string> scalar_conn;  // scalar container -> connector
        std::map<std::string, std::set<std::string>> read_keys, write_keys;   // per container: how it is indexed
        size_t n_values = 0;

        auto is_argument = [&](const std::string& name) {
            for (auto& arg : src.at("arguments").as_array())
                if (arg.as_string() == name) return true;
            return false;
        };
        auto floating = [&](P t, const Value& where) {
            if (t != P::Float && t != P::Double) refuse(where, std::string("a value of type ") + types::primitive_type_to_string(t) + " in a loop body (Float and Double only)");
            return t;
        };
        // strides (elements) per loop and the element count of a dense operand
        auto layout_of = [&](const OperandWalk& w, Array* strides, std::string* extent, std::string* key) {
            std::vector<std::string> per_loop(loops.size(), "0");
            std::string run = "1";
            for (size_t k = w.order.size(); k-- > 0;) {
                per_loop[(size_t) w.order[k]] = run;
                run = run == "1" ? loops[(size_t) w.order[k]].extent : "(" + loops[(size_t) w.order[k]].extent + ")*" + run;
            }
            *extent = run;
            for (auto& st : per_loop) {
                strides->emplace_back(st);
                *key += "|" + st;
            }
        };

        for (const Value* block : body) {
            const Value& df = block->at("dataflow");
            std::map<int64_t, const Value*> by_id;
            std::vector<const Value*> ops;
            for (auto& n : df.at("nodes").as_array()) {
                by_id[n.at("element_id").as_int()] = &n;
                const std::string kind = n.at("type").as_string();
                if (kind == "tasklet") ops.push_back(&n);
                else if (kind == "library_node") {
                    if (n.at("code").as_string() != "CMath") refuse(n, "a library node inside a loop nest");
                    ops.push_back(&n);
                }
            }
            std::map<int64_t, std::map<std::string, const Value*>> in_edges;   // op -> connector -> edge
            std::map<int64_t, std::vector<const Value*>> out_edges;            // op -> edges
            std::map<int64_t, int64_t> producer;                                // access node -> op that writes it here
            auto is_op = [&](int64_t id) {
                for (const Value* o : ops)
                    if (o->at("element_id").as_int() == id) return true;
                return false;
            };
            for (auto& e : df.at("edges").as_array()) {
                const int64_t from = e.at("src").as_int(), to = e.at("dst").as_int();
                if (!by_id.count(from) || !by_id.count(to)) refuse(*block, "an edge refers to an unknown node");
                if (is_op(to) && !is_op(from)) in_edges[to][e.at("dst_conn").as_string()] = &e;
                else if (is_op(from) && !is_op(to)) {
                    out_edges[from].push_back(&e);
                    producer[to] = from;
                } else
                    refuse(*block, "data movement beside the operations");
            }
            // the operations in an order in which every value is computed before it is used
            std::vector<const Value*> order;
            std::set<int64_t> done;
            while (order.size() < ops.size()) {
                bool progress = false;
                for (const Value* op : ops) {
                    const int64_t id = op->at("element_id").as_int();
                    if (done.count(id)) continue;
                    bool ready = true;
                    for (auto& kv : in_edges[id]) {
                        auto p = producer.find(kv.second->at("src").as_int());
                        ready = ready && (p == producer.end() || done.count(p->second));
                    }
                    if (!ready) continue;
                    order.push_back(op);
                    done.insert(id);
                    progress = true;
                }
                if (!progress) refuse(*block, "operations that depend on each other in a cycle");
            }

            for (const Value* op : order) {
                const int64_t id = op->at("element_id").as_int();
                std::string name;
                std::vector<std::string> connectors;
                if (op->at("type").as_string() == "tasklet") {
                    auto it = tasklet_names.find(op->at("code").as_int());
                    if (it == tasklet_names.end()) refuse(*op, "tasklet code " + std::to_string(op->at("code").as_int()) + " has no kernel");
                    name = it->second;
                    for (auto& i : op->at("inputs").as_array()) connectors.push_back(i.as_string());
                } else {
                    name = op->at("function_stem").as_string();
                    if (!rocm::ROCMMapNode::is_cmath(name)) refuse(*op, "CMath function '" + name + "' has no kernel");
                    for (int k = 1; k <= rocm::ROCMMapNode::arity(name); k++) connectors.push_back("_in" + std::to_string(k));
                }
                if ((int) connectors.size() != rocm::ROCMMapNode::arity(name)) refuse(*op, "operation " + name + " with " + std::to_string(connectors.size()) + " inputs");
                Array args;
                for (auto& conn : connectors) {
                    auto hit = in_edges[id].find(conn);
                    if (hit == in_edges[id].end()) refuse(*op, "input '" + conn + "' is not connected");
                    const Value& e = *hit->second;
                    const Value& node = *by_id.at(e.at("src").as_int());
                    if (node.at("type").as_string() == "constant_node") {
                        floating(element_of(node.at("data_type"), describe(node)), node);
                        args.emplace_back("#" + c_expression(node.at("data").as_expression()));
                        continue;
                    }
                    const std::string data = node.at("data").as_string();
                    const Value& c = container(data);
                    const P element = types::primitive_type_from_string(c.at("element").as_string());
                    if (c.at("type").as_string() == "scalar") {
                        auto cur = current.find(data);
                        auto known = assigned.find(data);
                        if (cur != current.end()) {
                            args.emplace_back(cur->second);
                        } else if (known != assigned.end()) {
                            args.emplace_back("#(" + c_expression(known->second) + ")");
                        } else {
                            floating(element, node);
                            auto sc = scalar_conn.find(data);
                            if (sc == scalar_conn.end()) {
                                sc = scalar_conn.emplace(data, "_c" + std::to_string(scalar_conn.size())).first;
                                Value s;
                                s.set("connector", sc->second);
                                s.set("element_type", types::primitive_type_to_string(element));
                                scalars.push_back(std::move(s));
                                Value b;
                                b.set("data", data);
                                b.set("connector", sc->second);
                                inputs.push_back(std::move(b));
                            }
                            args.emplace_back(sc->second);
                        }
                        continue;
                    }
                    floating(element, node);
                    OperandWalk w;
                    if (loops.empty() || !walk_of(*block, e, node, loops, &w) || w.scalar)
                        refuse(*block, "operand '" + data + "' is not a dense tensor indexed by the loop variables");
                    Array strides;
                    std::string extent, key = data;
                    layout_of(w, &strides, &extent, &key);
                    auto st = stored.find(key);
                    if (st != stored.end()) {   // the element this iteration has just computed
                        args.emplace_back(st->second);
                        continue;
                    }
                    read_keys[data].insert(key);
                    auto rc = read_conn.find(key);
                    if (rc == read_conn.end()) {
                        rc = read_conn.emplace(key, "_in" + std::to_string(read_conn.size())).first;
                        Value r;
                        r.set("connector", rc->second);
                        r.set("strides", Value(std::move(strides)));
                        r.set("extent", extent);
                        r.set("element_type", types::primitive_type_to_string(element));
                        reads.push_back(std::move(r));
                        Value b;
                        b.set("data", data);
                        b.set("connector", rc->second);
                        inputs.push_back(std::move(b));
                    }
                    args.emplace_back(rc->second);
                }
                auto outs = out_edges.find(id);
                if (outs == out_edges.end() || outs->second.empty()) refuse(*op, "an operation without a result");
                const std::string value = "_v" + std::to_string(n_values++);
                P type = P::Void;
                if (op->at("type").as_string() != "tasklet" && op->contains("primitive_type")) type = primitive_of(op->at("primitive_type"), describe(*op));
                if (type == P::Void) type = element_of(outs->second[0]->at("base_type"), describe(*block));
                floating(type, *op);
                Value stmt;
                stmt.set("out", value);
                stmt.set("type", types::primitive_type_to_string(type));
                stmt.set("op", name);
                stmt.set("args", Value(std::move(args)));
                statements.push_back(std::move(stmt));
                for (const Value* e : outs->second) {
                    const Value& node = *by_id.at(e->at("dst").as_int());
                    if (node.at("type").as_string() != "access_node") refuse(*block, "a result that does not go to a container");
                    const std::string data = node.at("data").as_string();
                    const Value& c = container(data);
                    const P element = floating(types::primitive_type_from_string(c.at("element").as_string()), node);
                    if (c.at("type").as_string() == "scalar") {
                        if (is_argument(data)) refuse(*block, "a scalar argument ('" + data + "') written inside a loop nest");
                        current[data] = value;
                        continue;
                    }
                    OperandWalk w;
                    if (loops.empty() || !walk_of(*block, *e, node, loops, &w) || w.scalar)
                        refuse(*block, "operand '" + data + "' is not a dense tensor indexed by the loop variables");
                    if (w.partial()) refuse(*block, "a result that some loops of the nest do not index");
                    Array strides;
                    std::string extent, key = data;
                    layout_of(w, &strides, &extent, &key);
                    write_keys[data].insert(key);
                    auto at = write_at.find(key);
                    if (at != write_at.end()) {
                        writes[at->second].set("value", value);   // stored again: the later value stays
                    } else {
                        write_at[key] = writes.size();
                        Value wv;
                        const std::string connector = "_out" + std::to_string(writes.size());
                        wv.set("connector", connector);
                        wv.set("strides", Value(std::move(strides)));
                        wv.set("extent", extent);
                        wv.set("element_type", types::primitive_type_to_string(element));
                        wv.set("value", value);
                        writes.push_back(std::move(wv));
                        Value b;
                        b.set("data", data);
                        b.set("connector", connector);
                        outputs.push_back(std::move(b));
                    }
                    stored[key] = value;
                }
            }
        }
        if (writes.empty()) refuse(element, "a loop nest that stores nothing to a tensor");
        // iterations are independent only if nobody reads or writes an element that another iteration writes
        for (auto& kv : write_keys) {
            if (kv.second.size() > 1) refuse(element, "'" + kv.first + "' is written through two different index forms in one nest");
            auto r = read_keys.find(kv.first);
            if (r != read_keys.end() && (r->second.size() > 1 || *r->second.begin() != *kv.second.begin()))
                refuse(element, "'" + kv.first + "' is read at other elements than the one the iteration writes");
        }
        // the integer scalars that bounds and strides mention
        Array symbols, indvars, bounds;
        std::set<std::string> seen;
        auto scan = [&](const std::string& text) {
            std::string word;
            auto flush = [&]() {
                if (!word.empty() && !std::isdigit((unsigned char) word[0]) && !seen.count(word)) {
                    bool is_var = false;
                    for (auto& l : loops) is_var = is_var || l.var == word;
                    if (!is_var) {
                        bool exists = false;
                        for (auto& kv : containers) exists = exists || kv.first == word;
                        if (!exists || container(word).at("type").as_string() != "scalar")
                            refuse(element, "'" + word + "' in a bound or an index is not a scalar of the function");
                        seen.insert(word);
                        symbols.emplace_back(word);
                    }
                }
                word.clear();
            };
            for (char ch : text) {
                if (std::isalnum((unsigned char) ch) || ch == '_') word += ch;
                else flush();
            }
            flush();
        };
        for (auto& l : loops) {
            indvars.emplace_back(l.var);
            bounds.emplace_back(l.extent);
            scan(l.extent);
        }
        for (auto* list : {&reads, &writes})
            for (auto& a : *list)
                for (auto& st : a.at("strides").as_array()) scan(st.as_string());
        Value node{Object{}};
        node.set("type", "library_node");
        node.set("element_id", element.at("element_id").as_int());
        node.set("code", rocm::LibraryNodeType_ROCM_Map);
        node.set("implementation_type", "NONE");
        node.set("side_effect", false);
        node.set("indvars", Value(std::move(indvars)));
        node.set("bounds", Value(std::move(bounds)));
        node.set("symbols", Value(std::move(symbols)));
        node.set("reads", Value(std::move(reads)));
        node.set("writes", Value(std::move(writes)));
        node.set("scalars", Value(std::move(scalars)));
        node.set("statements", Value(std::move(statements)));
        Value flow;
        flow.set("library_node", std::move(node));
        flow.set("inputs", Value(std::move(inputs)));
        flow.set("outputs", Value(std::move(outputs)));
        Value b;
        b.set("type", "block");
        b.set("element_id", body[0]->at("element_id").as_int());
        Value dbg = debug_info_of(element);
        if (!dbg.is_null()) b.set("debug_info", std::move(dbg));
        b.set("dataflow", std::move(flow));
        children.push_back(std::move(b));
    }

    // One block with one tasklet (or CMath node) under `loops` (none: a scalar statement).
    void lower_tasklet_block(const Value& block, const std::vector<NestLoop>& loops, Array& children) {
        const Value& df = block.at("dataflow");
        std::map<int64_t, const Value*> by_id;
        const Value* op = nullptr;
        for (auto& n : df.at("nodes").as_array()) {
            by_id[n.at("element_id").as_int()] = &n;
            const std::string kind = n.at("type").as_string();
            if (kind == "tasklet" || kind == "library_node") {
                if (op) refuse(block, "more than one operation in a loop body");
                op = &n;
            }
        }
        if (!op) return;
        const int64_t op_id = op->at("element_id").as_int();
        std::map<std::string, OperandWalk> in;
        OperandWalk out;
        const Value* out_type = nullptr;
        bool out_is_pointer = false;
        for (auto& e : df.at("edges").as_array()) {
            const bool into = e.at("dst").as_int() == op_id, from = e.at("src").as_int() == op_id;
            if (!into && !from) refuse(block, "data movement beside the operation");
            const Value& other = *by_id.at(e.at(into ? "src" : "dst").as_int());
            OperandWalk w;
            if (!walk_of(block, e, other, loops, &w))
                refuse(block, "operand '" + (other.contains("data") ? other.at("data").as_expression() : std::string("?")) +
                                  "' is not a dense tensor indexed by the loop variables");
            if (into) {
                if (w.scalar && other.at("type").as_string() == "access_node" && container(other.at("data").as_string()).at("type").as_string() != "scalar")
                    refuse(block, "one element of '" + other.at("data").as_string() + "' read outside a loop");
                in[e.at("dst_conn").as_string()] = w;
            } else {
                if (out_type) refuse(block, "an operation with two results");
                out = w;
                out_type = &e.at("base_type");
                out_is_pointer = other.at("type").as_string() == "access_node" && container(other.at("data").as_string()).at("type").as_string() == "pointer";
                if (out.scalar && out_is_pointer) {
                    // a scalar stored to element 0 of a buffer (the scalar form of the return copy)
                    for (auto& sub : e.at("subset").as_array())
                        if (strip(sub.as_expression()) != "0") refuse(block, "a store to one element other than the first");
                }
            }
        }
        if (!out_type) refuse(block, "an operation without a result");
        const types::PrimitiveType element = element_of(*out_type, describe(block));

        // what the operation is
        std::string code;      // node code of the target
        std::vector<std::string> operands;   // the operation's input connectors in order
        if (op->at("type").as_string() == "tasklet") {
            const int64_t tc = op->at("code").as_int();
            for (auto& i : op->at("inputs").as_array()) operands.push_back(i.as_string());
            // enum TaskletCode (reference sdfg/include/sdfg/data_flow/tasklet.h:94-153)
            switch (tc) {
                case 0: code = "assign"; break;
                case 2: code = "ml::Add"; break;
                case 3: code = "ml::Sub"; break;
                case 4: code = "ml::Mul"; break;
                case 5: code = "ml::Div"; break;
                default: refuse(*op, "tasklet code " + std::to_string(tc) + " has no kernel");
            }
        } else {
            if (op->at("code").as_string() != "CMath") refuse(*op, "a library node inside a loop nest");
            const std::string stem = op->at("function_stem").as_string();
            static const std::map<std::string, std::string> functions = {
                {"exp", "ml::Exp"}, {"sqrt", "ml::Sqrt"}, {"tanh", "ml::Tanh"}, {"erf", "ml::Erf"}, {"fabs", "ml::Abs"},
                {"fmax", "ml::Maximum"}, {"fmin", "ml::Minimum"}, {"pow", "ml::Pow"}};
            auto it = functions.find(stem);
            if (it == functions.end()) refuse(*op, "CMath function '" + stem + "' has no kernel");
            code = it->second;
            operands = {"_in1", "_in2"};
            if (code == "ml::Exp" || code == "ml::Sqrt" || code == "ml::Tanh" || code == "ml::Erf" || code == "ml::Abs") operands = {"_in1"};
        }
        for (auto& name : operands)
            if (!in.count(name)) refuse(*op, "input '" + name + "' is not connected");

        auto shape_in = [&](const std::vector<int>& order) {
            Array shape;
            for (int l : order) shape.emplace_back(loops[(size_t) l].extent);
            if (shape.empty()) shape.emplace_back("1");
            return Value(std::move(shape));
        };
        auto bind = [&](const char* connector, const OperandWalk& w) {
            Value b = w.binding;
            b.set("connector", connector);
            return b;
        };
        if (out.scalar && !out_is_pointer) refuse(block, "a scalar computed by a tasklet");

        // ---- reductions and repeated operands (ReduceNode::expand, reduce_node.cpp:122-345; BroadcastNode::expand,
        // broadcast_node.cpp:110-187). A reduction is a binary operation whose second operand is its own result,
        // in a nest some of whose loops do not index the result; the nest before it sets the result to the
        // operation's identity.
        auto extents_of = [&](const std::vector<int>& order) {
            Array shape;
            for (int l : order) shape.emplace_back(loops[(size_t) l].extent);
            return shape;
        };
        auto subsequence = [](const std::vector<int>& part, const std::vector<int>& whole) {
            size_t at = 0;
            for (int l : whole)
                if (at < part.size() && part[at] == l) at++;
            return at == part.size();
        };
        auto emit = [&](Value node, Array inputs, Array outputs) {
            node.set("type", "library_node");
            node.set("element_id", op_id);
            node.set("implementation_type", "NONE");
            node.set("side_effect", false);
            node.set("element_type", types::primitive_type_to_string(element));
            Value flow;
            flow.set("library_node", std::move(node));
            flow.set("inputs", Value(std::move(inputs)));
            flow.set("outputs", Value(std::move(outputs)));
            Value b;
            b.set("type", "block");
            b.set("element_id", block.at("element_id").as_int());
            Value dbg = debug_info_of(*op);
            if (dbg.is_null()) dbg = debug_info_of(block);
            if (!dbg.is_null()) b.set("debug_info", std::move(dbg));
            b.set("dataflow", std::move(flow));
            children.push_back(std::move(b));
        };
        if (operands.size() == 2 && !out.scalar && out.partial()) {
            static const std::map<std::string, std::pair<std::string, int>> reductions = {
                {"ml::Add", {"ml::Sum", 0}}, {"ml::Maximum", {"ml::Max", -1}}, {"ml::Minimum", {"ml::Min", +1}}};
            auto red = reductions.find(code);
            if (red == reductions.end()) refuse(block, "a result that some loops of the nest do not index, under an operation that is not a sum, maximum or minimum");
            const std::string result = out.binding.at("data").as_string();
            int acc = -1;
            for (int k = 0; k < 2; k++) {
                const OperandWalk& w = in.at(operands[(size_t) k]);
                if (!w.scalar && w.binding.at("data").as_string() == result && w.order == out.order && w.missing == out.missing) acc = k;
            }
            if (acc < 0) refuse(block, "a result that some loops of the nest do not index and that is not accumulated onto");
            const OperandWalk& x = in.at(operands[(size_t) (1 - acc)]);
            if (x.scalar || x.partial()) refuse(block, "the operand of a reduction must be indexed by every loop of the nest");
            if (!subsequence(out.order, x.order)) refuse(block, "operand and result of the reduction walk memory differently");
            if (out.units != 0 && out.units != (int) out.missing.size()) refuse(block, "some reduced dimensions kept and others dropped");
            // the nest before this one must have set the result to the identity of the operation
            const auto identity_ok = [&](const Value& before) {
                const Value* df = before.find("dataflow");
                if (!df || !df->contains("library_node")) return false;
                const Value& n = df->at("library_node");
                if (n.at("code").as_string() != "ml::Fill") return false;
                if (df->at("outputs").as_array().at(0).at("data").as_string() != result) return false;
                const Value& x0 = df->at("inputs").as_array().at(0);
                if (!x0.contains("constant")) return false;
                std::string c = x0.at("constant").as_string();
                c.erase(std::remove_if(c.begin(), c.end(), [](char ch) { return ch == '(' || ch == ')' || ch == ' '; }), c.end());
                if (red->second.second == 0) {
                    char* end = nullptr;
                    const double v = std::strtod(c.c_str(), &end);
                    return end != c.c_str() && v == 0.0;
                }
                const bool negative = !c.empty() && c[0] == '-';
                const std::string mag = negative ? c.substr(1) : c;
                return (mag == "INFINITY" || mag == "HUGE_VAL" || mag == "HUGE_VALF") && negative == (red->second.second < 0);
            };
            if (children.empty() || !identity_ok(children.back()))
                refuse(block, "an accumulation whose result the nest before it does not set to the operation's identity");
            children.pop_back();
            Array axes;
            for (size_t d = 0; d < x.order.size(); d++)
                if (!out.uses(x.order[d])) axes.emplace_back((int64_t) d);
            Value node{Object{}};
            node.set("code", red->second.first);
            node.set("shape", Value(extents_of(x.order)));
            node.set("axes", Value(std::move(axes)));
            node.set("keepdims", out.units > 0);
            Array inputs, outputs;
            Value bx = x.binding, by = out.binding;
            bx.set("connector", "X");
            by.set("connector", "Y");
            inputs.push_back(std::move(bx));
            outputs.push_back(std::move(by));
            emit(std::move(node), std::move(inputs), std::move(outputs));
            return;
        }
        if (code == "assign" && !out.scalar && !out.partial() && !in.at(operands.at(0)).scalar && in.at(operands.at(0)).partial()) {
            const OperandWalk& x = in.at(operands[0]);
            if (!subsequence(x.order, out.order)) refuse(block, "operand and result of the repeated copy walk memory differently");
            Array in_shape;
            for (int l : out.order) in_shape.emplace_back(x.uses(l) ? loops[(size_t) l].extent : std::string("1"));
            Value node{Object{}};
            node.set("code", "ml::Broadcast");
            node.set("input_shape", Value(std::move(in_shape)));
            node.set("output_shape", Value(extents_of(out.order)));
            Array inputs, outputs;
            Value bx = x.binding, by = out.binding;
            bx.set("connector", "X");
            by.set("connector", "Y");
            inputs.push_back(std::move(bx));
            outputs.push_back(std::move(by));
            emit(std::move(node), std::move(inputs), std::move(outputs));
            return;
        }
        if (out.partial()) refuse(block, "a result that some loops of the nest do not index");
        if (operands.size() == 2 && !out.scalar) {
            // an operand of a binary operation that some loops do not move (a view with strides of 0): it is repeated into a
            // temporary of the result's shape first; the fusion pass folds that copy back into the operation's kernel
            for (auto& name : operands) {
                OperandWalk& w = in.at(name);
                if (w.scalar || !w.partial()) continue;
                if (!subsequence(w.order, out.order)) refuse(block, "a repeated operand and the result walk memory differently");
                const std::string temp = "_docc_repeat_" + std::to_string(op_id) + name;
                std::string bytes = std::to_string(types::primitive_type_size(element));
                for (int l : out.order) bytes += "*(" + loops[(size_t) l].extent + ")";
                Value c;
                c.set("type", "pointer");
                c.set("element", types::primitive_type_to_string(element));
                c.set("transient", true);
                c.set("size", bytes);
                c.set("storage", "CPU");
                containers.emplace_back(temp, std::move(c));
                Array in_shape;
                for (int l : out.order) in_shape.emplace_back(w.uses(l) ? loops[(size_t) l].extent : std::string("1"));
                Value node{Object{}};
                node.set("code", "ml::Broadcast");
                node.set("input_shape", Value(std::move(in_shape)));
                node.set("output_shape", Value(extents_of(out.order)));
                Array inputs, outputs;
                Value bx = w.binding, by{Object{}};
                bx.set("connector", "X");
                by.set("data", temp);
                by.set("connector", "Y");
                inputs.push_back(std::move(bx));
                outputs.push_back(std::move(by));
                emit(std::move(node), std::move(inputs), std::move(outputs));
                Value nb{Object{}};
                nb.set("data", temp);
                w.binding = std::move(nb);
                w.order = out.order;
                w.missing.clear();
                w.units = 0;
            }
        }
        for (auto& name : operands)
            if (in.at(name).partial()) refuse(block, "operand '" + in.at(name).binding.at("data").as_string() + "' is not indexed by every loop of the nest");

        Value node{Object{}};
        node.set("type", "library_node");
        node.set("element_id", op_id);
        node.set("implementation_type", "NONE");
        node.set("side_effect", false);
        node.set("element_type", types::primitive_type_to_string(element));
        Array inputs, outputs;
        if (code == "assign") {
            const OperandWalk& x = in.at(operands.at(0));
            if (x.scalar) {
                node.set("code", "ml::Fill");
                node.set("shape", shape_in(out.order));
                inputs.push_back(bind("X", x));
            } else {
                if (out.scalar) refuse(block, "a tensor stored to one element");
                // Y[loops in out.order] = X[loops in x.order]: output axis a is the input axis that runs over the same loop
                Array perm;
                for (int l : out.order) {
                    auto pos = std::find(x.order.begin(), x.order.end(), l);
                    perm.emplace_back((int64_t) (pos - x.order.begin()));
                }
                node.set("code", "ml::Transpose");
                node.set("shape", shape_in(x.order));
                node.set("perm", Value(std::move(perm)));
                inputs.push_back(bind("X", x));
            }
            outputs.push_back(bind("Y", out));
        } else if (operands.size() == 1) {
            const OperandWalk& x = in.at(operands[0]);
            if (x.scalar || out.scalar || x.order != out.order) refuse(block, "operand and result of the unary operation walk memory differently");
            node.set("code", code);
            node.set("shape", shape_in(out.order));
            inputs.push_back(bind("X", x));
            outputs.push_back(bind("Y", out));
        } else {
            const OperandWalk &a = in.at(operands[0]), &b = in.at(operands[1]);
            if (out.scalar || (a.scalar && b.scalar)) refuse(block, "a binary operation on scalars only");
            if ((!a.scalar && a.order != out.order) || (!b.scalar && b.order != out.order))
                refuse(block, "operands and result of the binary operation walk memory differently");
            node.set("code", code);
            node.set("shape", shape_in(out.order));
            inputs.push_back(bind("A", a));
            inputs.push_back(bind("B", b));
            outputs.push_back(bind("C", out));
        }
        Value flow;
        flow.set("library_node", std::move(node));
        flow.set("inputs", Value(std::move(inputs)));
        flow.set("outputs", Value(std::move(outputs)));
        Value b;
        b.set("type", "block");
        b.set("element_id", block.at("element_id").as_int());
        Value dbg = debug_info_of(*op);
        if (dbg.is_null()) dbg = debug_info_of(block);
        if (!dbg.is_null()) b.set("debug_info", std::move(dbg));
        b.set("dataflow", std::move(flow));
        children.push_back(std::move(b));
    }

    // Symbols a transition sets to an expression of the function's scalar arguments (the element count a mean divides
    // by, mean_node.cpp:96-107): the value is the same wherever the symbol is read, so a read of it is a read of
    // the expression. Anything else assigned between blocks has no lowering here.
    std::map<std::string, std::string> assigned;
    // does `word` occur as an identifier in any string below `v`, other than as the name an access node refers to
    // or as the left-hand side of an assignment?
    static bool word_in_expressions(const Value& v, const std::string& word) {
        if (v.is_string()) {
            const std::string& text = v.as_string();
            for (size_t at = text.find(word); at != std::string::npos; at = text.find(word, at + 1)) {
                const bool left = at == 0 || !(std::isalnum((unsigned char) text[at - 1]) || text[at - 1] == '_');
                const size_t end = at + word.size();
                const bool right = end >= text.size() || !(std::isalnum((unsigned char) text[end]) || text[end] == '_');
                if (left && right) return true;
            }
            return false;
        }
        if (v.is_array()) {
            for (auto& e : v.as_array())
                if (word_in_expressions(e, word)) return true;
            return false;
        }
        if (v.is_object()) {
            const Value* type = v.find("type");
            const bool access = type && type->is_string() && type->as_string() == "access_node";
            for (auto& kv : v.as_object()) {
                if (access && kv.first == "data") continue;
                if (kv.first == "symbol" && v.contains("expression")) continue;
                if (word_in_expressions(kv.second, word)) return true;
            }
        }
        return false;
    }
    void note_assignments(const Value& t) {
        for (auto& a : t.at("assignments").as_array()) {
            const std::string symbol = strip(a.at("symbol").as_string()), expr = strip(a.at("expression").as_expression());
            std::string word;
            auto check = [&]() {
                if (word.empty() || std::isdigit((unsigned char) word[0])) return;
                bool argument = false;
                for (auto& arg : src.at("arguments").as_array()) argument = argument || arg.as_string() == word;
                if (!argument || container(word).at("type").as_string() != "scalar")
                    throw InvalidSDFGException(describe(t) + ": symbol '" + symbol + "' is assigned '" + expr +
                                               "', which is not an expression of the function's scalar arguments");
            };
            for (char ch : expr) {
                if (std::isalnum((unsigned char) ch) || ch == '_') word += ch;
                else {
                    check();
                    word.clear();
                }
            }
            check();
            if (!src.at("containers").contains(symbol) || container(symbol).at("type").as_string() != "scalar")
                throw InvalidSDFGException(describe(t) + ": symbol assignments between blocks are not lowered by the rocm target ('" + symbol +
                                           "' is not a scalar of the function)");
            // the symbol may be read through access nodes only: inside an index, a bound or a node's attribute it would
            // have to be a variable of the generated function, which this target does not write assignments for
            if (word_in_expressions(src.at("root"), symbol))
                throw InvalidSDFGException(describe(t) + ": symbol assignments between blocks are not lowered by the rocm target ('" + symbol +
                                           "' is read inside an expression)");
            auto it = assigned.find(symbol);
            if (it != assigned.end() && it->second != expr)
                throw InvalidSDFGException(describe(t) + ": symbol '" + symbol + "' is assigned two different values");
            assigned[symbol] = expr;
        }
    }

    void import_sequence(const Value& seq, Array& children, std::string& returned) {
        if (const Value* transitions = seq.find("transitions"))
            for (auto& t : transitions->as_array()) note_assignments(t);
        for (auto& child : seq.at("children").as_array()) {
            const std::string kind = child.at("type").as_string();
            if (!returned.empty())
                throw InvalidSDFGException(describe(child) + ": code after the return");
            if (kind == "block") {
                import_block(child, children);
            } else if (kind == "sequence") {
                import_sequence(child, children, returned);
            } else if (kind == "for" || kind == "map") {
                import_loop_nest(child, children);
            } else if (kind == "return") {
                const std::string data = child.at("data").as_string();
                if (child.contains("data_type")) throw InvalidSDFGException(describe(child) + ": returning a constant");
                returned = data.empty() ? "\x01" : data;
            } else {
                throw InvalidSDFGException(describe(child) + ": control flow other than a sequence of library-node blocks and elementwise "
                                           "loop nests is not lowered by the rocm target");
            }
        }
    }

    Value run() {
        for (const char* key : {"name", "containers", "arguments", "root"})
            if (!src.contains(key)) throw InvalidSDFGException(std::string("not an SDFG: no \"") + key + "\"");
        if (const Value* t = src.find("type"))
            if (t->is_string() && t->as_string() != "CPU")
                throw InvalidSDFGException("function type " + t->as_string() + " belongs to another target");
        if (const Value* ex = src.find("externals"))
            if (!ex->as_array().empty()) throw InvalidSDFGException("externals are not supported by the rocm target");
        import_containers();
        Array children;
        std::string returned;
        import_sequence(src.at("root"), children, returned);
        out.set("type", "structured_sdfg");
        out.set("name", src.at("name").as_string());
        out.set("arguments", src.at("arguments"));
        out.set("containers", Value(std::move(containers)));
        out.set("return", returned == "\x01" ? std::string() : returned);
        Value meta{Object{}};
        if (const Value* m = src.find("metadata"))
            for (auto& kv : m->as_object()) meta.set(kv.first, kv.second);
        out.set("metadata", std::move(meta));
        Value root;
        root.set("type", "sequence");
        root.set("children", Value(std::move(children)));
        out.set("root", std::move(root));
        return out;
    }
};

// ---- export ---------------------------------------------------------------------------

Value empty_debug_info() {
    Value d;
    d.set("has", false);
    d.set("filename", "");
    d.set("function", "");
    d.set("start_line", 0);
    d.set("start_column", 0);
    d.set("end_line", 0);
    d.set("end_column", 0);
    return d;
}

Value storage_json(const Container& c) {
    Value s;
    s.set("value", c.storage == "CPU" ? (c.transient && c.is_pointer ? "CPU_Heap" : "CPU_Stack") : c.storage);
    const bool managed = c.transient && c.is_pointer && !c.size_bytes.empty();
    s.set("allocation", managed ? 1 : 0);
    s.set("deallocation", managed ? 1 : 0);
    if (managed) s.set("allocation_size", c.size_bytes);
    return s;
}

Value plain_storage() {
    Value s;
    s.set("value", "CPU_Stack");
    s.set("allocation", 0);
    s.set("deallocation", 0);
    return s;
}

Value scalar_json(types::PrimitiveType t, Value storage) {
    Value j;
    j.set("type", "scalar");
    j.set("primitive_type", reference_primitive(t));
    j.set("storage_type", std::move(storage));
    j.set("initializer", "");
    j.set("alignment", 0);
    return j;
}

Value type_json(const Container& c) {
    if (!c.is_pointer) return scalar_json(c.element, storage_json(c));
    Value j;
    j.set("type", "pointer");
    j.set("pointee_type", scalar_json(c.element, plain_storage()));
    j.set("storage_type", storage_json(c));
    j.set("initializer", "");
    j.set("alignment", 0);
    return j;
}

} // namespace

// the reference's serializer always writes "element_counter"; the block list never does
bool is_reference_format(const Value& j) { return j.is_object() && j.contains("element_counter"); }

Value import_reference_json(const Value& j) { return Import(j).run(); }

Value export_reference_json(const StructuredSDFG& sdfg) {
    size_t counter = 0;
    auto next = [&] { return (int64_t) ++counter; };
    Value j;
    j.set("name", sdfg.name());
    j.set("type", "CPU");
    Container nothing;
    nothing.element = types::PrimitiveType::Void;
    j.set("return_type", sdfg.return_container().empty() ? type_json(nothing) : type_json(sdfg.container(sdfg.return_container())));
    j.set("structures", Value(Array{}));
    Value containers{Object{}};
    for (auto& kv : sdfg.containers()) containers.set(kv.first, type_json(kv.second));
    j.set("containers", std::move(containers));
    Array args;
    for (auto& a : sdfg.arguments()) args.emplace_back(a);
    j.set("arguments", Value(std::move(args)));
    j.set("externals", Value(Array{}));
    Value meta{Object{}};
    for (auto& kv : sdfg.metadata()) meta.set(kv.first, kv.second);
    j.set("metadata", std::move(meta));

    auto debug_json = [](const structured_control_flow::DebugInfo& d) {
        if (!d.has) return empty_debug_info();
        Value v;
        v.set("has", true);
        v.set("filename", d.filename);
        v.set("function", d.function);
        v.set("start_line", (int64_t) d.start_line);
        v.set("start_column", (int64_t) d.start_column);
        v.set("end_line", (int64_t) d.end_line);
        v.set("end_column", (int64_t) d.end_column);
        return v;
    };
    auto transition = [&] {
        Value t;
        t.set("type", "transition");
        t.set("element_id", next());
        t.set("debug_info", empty_debug_info());
        t.set("assignments", Value(Array{}));
        return t;
    };

    Value root;
    root.set("type", "sequence");
    root.set("element_id", next());
    root.set("debug_info", empty_debug_info());
    Array children, transitions;
    for (auto& blk : sdfg.blocks()) {
        Value b;
        b.set("type", "block");
        b.set("element_id", next());
        b.set("debug_info", debug_json(blk.debug_info));
        Array nodes, edges;
        Value lib;
        const int64_t lib_id = next();
        lib.set("element_id", lib_id);
        lib.set("debug_info", debug_json(blk.debug_info));
        lib.set("type", "library_node");
        lib.set("implementation_type", blk.node->implementation_type());
        lib.set("code", blk.node->code());
        blk.node->to_json(lib);
        if (blk.node->code() == "ml::Cast")
            if (const Value* tt = lib.find("target_type"))
                if (tt->is_string()) lib.set("target_type", reference_primitive(types::primitive_type_from_string(tt->as_string())));
        nodes.push_back(std::move(lib));
        auto edge = [&](int64_t src, const std::string& src_conn, int64_t dst, const std::string& dst_conn, Value base_type) {
            Value e;
            e.set("element_id", next());
            e.set("debug_info", empty_debug_info());
            e.set("src", src);
            e.set("dst", dst);
            e.set("src_conn", src_conn);
            e.set("dst_conn", dst_conn);
            e.set("subset", Value(Array{}));
            e.set("base_type", std::move(base_type));
            edges.push_back(std::move(e));
        };
        for (auto& in : blk.inputs) {
            Value n;
            const int64_t id = next();
            n.set("element_id", id);
            n.set("debug_info", empty_debug_info());
            if (in.is_constant) {
                n.set("type", "constant_node");
                n.set("data", in.data);
                n.set("data_type", scalar_json(in.type, plain_storage()));
                nodes.push_back(std::move(n));
                edge(id, "void", lib_id, in.connector, scalar_json(in.type, plain_storage()));
            } else {
                n.set("type", "access_node");
                n.set("data", in.data);
                nodes.push_back(std::move(n));
                edge(id, "void", lib_id, in.connector, type_json(sdfg.container(in.data)));
            }
        }
        for (auto& out : blk.outputs) {
            Value n;
            const int64_t id = next();
            n.set("element_id", id);
            n.set("debug_info", empty_debug_info());
            n.set("type", "access_node");
            n.set("data", out.data);
            nodes.push_back(std::move(n));
            edge(lib_id, out.connector, id, "void", type_json(sdfg.container(out.data)));
        }
        Value df;
        df.set("type", "dataflow");
        df.set("nodes", Value(std::move(nodes)));
        df.set("edges", Value(std::move(edges)));
        b.set("dataflow", std::move(df));
        children.push_back(std::move(b));
        transitions.push_back(transition());
    }
    {
        // the reference's front end closes every function with a return node
        Value r;
        r.set("type", "return");
        r.set("element_id", next());
        r.set("data", sdfg.return_container());
        r.set("debug_info", empty_debug_info());
        children.push_back(std::move(r));
        transitions.push_back(transition());
    }
    root.set("children", Value(std::move(children)));
    root.set("transitions", Value(std::move(transitions)));
    j.set("root", std::move(root));
    j.set("element_counter", (int64_t) counter);
    return j;
}

} // namespace sdfg::serializer
