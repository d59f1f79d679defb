"""SDFG JSON interchange with docc's own serializer (reference sdfg/src/serializer/json_serializer.cpp:56-353).

`tests/golden/docc_tiled_matmul_sdfg.json` is a data file of the reference (examples/input/transfertuning/
matmul_sdfg.json, minified): a tiled matmul loop nest written by docc's serializer. It pins the envelope,
the type encoding (primitive type numbers, pointer -> array -> scalar) and the dataflow node / edge layout.
The library-node programs below are written by hand in the same layout, following what
PyStructuredSDFGBuilder::add_gemm builds (python/bindings/builder/py_structured_sdfg_builder.cpp:654-774: an
empty view block, one access node per edge, C bound as input and output, constants for alpha / beta) and
the node serializers (gemm_node.cpp:387-405, malloc.cpp:43-53)."""
import copy
import json
import re
from pathlib import Path

import pytest

from docc_amd.sdfg import InvalidSDFGException, Pointer, PrimitiveType, Scalar, StructuredSDFG, StructuredSDFGBuilder

GOLDEN = Path(__file__).parent / "golden" / "docc_tiled_matmul_sdfg.json"
NO_DEBUG = {"has": False, "filename": "", "function": "", "start_line": 0, "start_column": 0, "end_line": 0, "end_column": 0}
STACK = {"value": "CPU_Stack", "allocation": 0, "deallocation": 0}
FLOAT, DOUBLE, INT64 = 14, 15, 5


def scalar(prim):
    return {"type": "scalar", "primitive_type": prim, "storage_type": STACK, "initializer": "", "alignment": 0}


def pointer(prim):
    return {"type": "pointer", "pointee_type": scalar(prim), "storage_type": STACK, "initializer": "", "alignment": 0}


class Ids:
    def __init__(self):
        self.n = 0

    def __call__(self):
        self.n += 1
        return self.n


def docc_block(ids, lib, inputs, outputs, containers, debug=None):
    """One block as docc serialises it: the library node, one access / constant node per edge."""
    lib = {"element_id": ids(), "debug_info": debug or NO_DEBUG, "type": "library_node", **lib}
    nodes, edges = [lib], []
    for conn, value in inputs:
        nid = ids()
        if isinstance(value, tuple):      # (literal, primitive type): a constant node
            nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "constant_node", "data": value[0], "data_type": scalar(value[1])})
            base = scalar(value[1])
        else:
            nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "access_node", "data": value})
            base = containers[value]
        edges.append({"element_id": ids(), "debug_info": NO_DEBUG, "src": nid, "dst": lib["element_id"], "src_conn": "void",
                      "dst_conn": conn, "subset": [], "base_type": base})
    for conn, name in outputs:
        nid = ids()
        nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "access_node", "data": name})
        edges.append({"element_id": ids(), "debug_info": NO_DEBUG, "src": lib["element_id"], "dst": nid, "src_conn": conn,
                      "dst_conn": "void", "subset": [], "base_type": containers[name]})
    return {"type": "block", "element_id": ids(), "debug_info": debug or NO_DEBUG,
            "dataflow": {"type": "dataflow", "nodes": nodes, "edges": edges}}


def docc_sdfg(name, containers, arguments, children, ids):
    transitions = [{"type": "transition", "element_id": ids(), "debug_info": NO_DEBUG, "assignments": []} for _ in children]
    return {"name": name, "element_counter": ids.n + 1, "type": "CPU", "return_type": scalar(0), "structures": [],
            "containers": containers, "arguments": arguments, "externals": [], "metadata": {"sdfg_file": "/tmp/x.json"},
            "root": {"type": "sequence", "element_id": ids(), "debug_info": NO_DEBUG, "children": children, "transitions": transitions}}


def gemm_program():
    """T = A @ B (temporary from Malloc), C = 1.5 * T @ B + 0.5 * C, Free(T), return."""
    ids = Ids()
    containers = {n: pointer(DOUBLE) for n in ("A", "B", "C", "_tmp_0")}
    containers["_s0"] = scalar(INT64)
    gemm = {"implementation_type": "BLAS", "code": "GEMM", "precision": ord("d"), "layout": 101, "trans_a": 111, "trans_b": 111,
            "m": "_s0", "n": "_s0", "k": "_s0", "lda": "_s0", "ldb": "_s0", "ldc": "_s0"}
    dbg = {"has": True, "filename": "/home/u/prog.py", "function": "two_mm", "start_line": 7, "start_column": 4, "end_line": 7, "end_column": 20}
    children = [
        docc_block(ids, {"implementation_type": "NONE", "code": "Malloc", "size": "8*_s0**2"}, [], [("_ret", "_tmp_0")], containers),
        {"type": "block", "element_id": ids(), "debug_info": NO_DEBUG, "dataflow": {"type": "dataflow", "nodes": [], "edges": []}},
        docc_block(ids, gemm, [("__A", "A"), ("__B", "B"), ("__C", "_tmp_0"), ("__alpha", ("1.0", DOUBLE)), ("__beta", ("0.0", DOUBLE))],
                   [("__C", "_tmp_0")], containers, dbg),
        docc_block(ids, gemm, [("__A", "_tmp_0"), ("__B", "B"), ("__C", "C"), ("__alpha", ("1.5", DOUBLE)), ("__beta", ("0.5", DOUBLE))],
                   [("__C", "C")], containers),
        docc_block(ids, {"implementation_type": "NONE", "code": "Free"}, [("_ptr", "_tmp_0")], [("_ptr", "_tmp_0")], containers),
        {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG},
    ]
    return docc_sdfg("two_mm_sdfg", containers, ["A", "B", "C", "_s0"], children, ids)


def test_reference_data_file_pins_the_envelope_and_type_encoding():
    data = json.loads(GOLDEN.read_text())
    # a tiled loop nest (steps of 32, a reduction inside) matches no elementwise kernel: the import stops at the first map and says so
    with pytest.raises(InvalidSDFGException, match=r"map \(element \d+\): the loop's step is not 1"):
        StructuredSDFG.from_docc_json(json.dumps(data))
    # its declarations alone import: arrays behind pointers decay to their element type, type numbers as in docc's enum
    head = dict(data, root={"type": "sequence", "element_id": 1, "debug_info": NO_DEBUG, "children": [], "transitions": []})
    s = StructuredSDFG.from_docc_json(json.dumps(head))
    assert s.name == "sdfg_test" and s.arguments == ["A", "B", "C", "K", "N", "M"]
    assert s.containers["A"] == {"type": "pointer", "element": "Float", "transient": False, "storage": "CPU"}
    assert s.containers["i"]["type"] == "scalar" and s.containers["i"]["element"] == "UInt64" and s.containers["K"]["element"] == "UInt64"
    # a tasklet block on its own (an fma into C[i][j] outside its loops) is refused with its element named
    def first_block(n):
        if n.get("type") == "block":
            return n
        for c in n.get("children", []):
            r = first_block(c)
            if r:
                return r
        return first_block(n["root"]) if "root" in n and n["type"] != "sequence" else None
    blk = first_block(data["root"])
    only = dict(data, root={"type": "sequence", "element_id": 1, "debug_info": NO_DEBUG, "children": [blk],
                            "transitions": [{"type": "transition", "element_id": 2, "debug_info": NO_DEBUG, "assignments": []}]})
    with pytest.raises(InvalidSDFGException, match=r"block \(element \d+\): "):
        StructuredSDFG.from_docc_json(json.dumps(only))


def test_gemm_program_written_like_docc_imports_schedules_and_generates(tmp_path):
    text = json.dumps(gemm_program())
    s = StructuredSDFG.from_docc_json(text)
    assert s.arguments == ["A", "B", "C", "_s0"] and s.metadata("sdfg_file") == "/tmp/x.json"
    assert s.containers["_tmp_0"] == {"type": "pointer", "element": "Double", "transient": True, "storage": "CPU", "size": "8*(_s0*_s0)"}     # SymEngine's power spelled as C
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["GEMM", "GEMM"]          # Malloc / Free became the transient, the view block vanished
    assert nodes[0]["implementation_type"] == "BLAS" and nodes[0]["precision"] == ord("d") and nodes[0]["lda"] == "_s0"
    first = s._data["root"]["children"][0]
    binds = {b["connector"]: b.get("data", b.get("constant")) for b in first["dataflow"]["inputs"]}
    assert binds == {"__A": "A", "__B": "B", "__C": "_tmp_0", "__alpha": "1.0", "__beta": "0.0"}
    assert first["dataflow"]["outputs"] == [{"connector": "__C", "data": "_tmp_0"}]
    assert first["debug_info"]["function"] == "two_mm" and first["debug_info"]["start_line"] == 7
    # every entry point takes the docc format directly
    assert StructuredSDFG.parse(text).library_nodes() == nodes
    s.schedule("rocm")
    r = s.loop_report()
    assert r["H2D"] == 3 and r["D2H"] == 1            # A, B, C up (beta != 0 reads C); C down; the temporary never leaves the device
    src = Path(s.generate(str(tmp_path))["source"]).read_text()
    assert src.count("docc_rocm_dgemm(") == 2 and 'extern "C" void two_mm_sdfg(double *A, double *B, double *C, int64_t _s0)' in src


def test_import_refuses_what_it_cannot_lower():
    base = gemm_program()
    bad = copy.deepcopy(base)
    bad["root"]["children"][2]["dataflow"]["edges"][0]["subset"] = ["_s0"]
    with pytest.raises(InvalidSDFGException, match="subset on an operand of GEMM"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    bad = copy.deepcopy(base)
    bad["root"]["transitions"][0]["assignments"] = [{"symbol": "i", "expression": "0"}]
    with pytest.raises(InvalidSDFGException, match="symbol assignments"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    bad = copy.deepcopy(base)
    bad["containers"]["A"]["storage_type"] = {"value": "NV_Generic", "allocation": 0, "deallocation": 0}
    with pytest.raises(InvalidSDFGException, match="NV_Generic belongs to another target"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    bad = copy.deepcopy(base)
    bad["root"]["children"][2]["dataflow"]["nodes"][0]["code"] = "Memcpy"
    with pytest.raises(InvalidSDFGException, match="No library node serializer found for Memcpy"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    bad = copy.deepcopy(base)
    bad["root"]["children"][0]["dataflow"]["nodes"][0]["size"] = "8*_s0**_s0"
    with pytest.raises(InvalidSDFGException, match="not a small integer power"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    bad = copy.deepcopy(base)
    bad["root"]["children"][0]["dataflow"]["nodes"][0]["size"] = "8*(1 + _s0)**3"
    assert StructuredSDFG.from_docc_json(json.dumps(bad)).containers["_tmp_0"]["size"] == "8*((1 + _s0)*(1 + _s0)*(1 + _s0))"
    bad = copy.deepcopy(base)
    bad["root"]["children"].append({"type": "break", "element_id": 999, "debug_info": NO_DEBUG})
    with pytest.raises(InvalidSDFGException, match="code after the return"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    with pytest.raises(InvalidSDFGException, match="element_counter"):
        StructuredSDFG.from_docc_json(StructuredSDFGBuilder("x").move().to_json())


def test_export_writes_docc_layout_and_round_trips():
    F32 = Pointer(Scalar(PrimitiveType.Float))
    b = StructuredSDFGBuilder("dense")
    for n in ("X", "W", "bias", "Y"):
        b.add_container(n, F32, True)
    for n in ("T0", "T1", "T2"):
        b.add_container(n, F32, False, transient_bytes=32 * 16 * 4)
    b.set_debug_info("/src/m.py", "dense", 3, 5, 3, 30)
    b.add_gemm("X", "W", "T0", "1.0", "0.0", 32, 16, 8)
    b.add_broadcast("bias", "T1", [1, 16], [32, 16])
    b.add_elementwise_op("add", "T0", "T1", "T2", [32, 16])
    b.add_reduce_op("softmax", "T2", "T0", [32, 16], [-1])
    b.add_elementwise_op("mul", "T0", "0.5", "Y", [32, 16])
    s = b.move()
    d = json.loads(s.to_docc_json())
    # the keys JSONSerializer::serialize writes, in a shape its deserialize accepts
    assert set(d) == {"name", "element_counter", "type", "return_type", "structures", "containers", "arguments", "externals", "metadata", "root"}
    assert d["type"] == "CPU" and d["return_type"]["primitive_type"] == 0 and d["arguments"] == ["X", "W", "bias", "Y"]
    assert d["containers"]["X"]["pointee_type"]["primitive_type"] == FLOAT
    t0 = d["containers"]["T0"]["storage_type"]
    assert t0 == {"value": "CPU_Heap", "allocation": 1, "deallocation": 1, "allocation_size": "2048"}
    root = d["root"]
    assert root["type"] == "sequence" and len(root["children"]) == len(root["transitions"]) == 6 and root["children"][-1]["type"] == "return"
    ids = re.findall(r'"element_id": (\d+)', json.dumps(d))
    assert len(ids) == len(set(ids)) and max(map(int, ids)) == d["element_counter"]
    blk = root["children"][0]
    assert set(blk) == {"type", "element_id", "debug_info", "dataflow"} and blk["debug_info"]["start_line"] == 3
    kinds = [n["type"] for n in blk["dataflow"]["nodes"]]
    assert kinds == ["library_node", "access_node", "access_node", "access_node", "constant_node", "constant_node", "access_node"]
    lib = blk["dataflow"]["nodes"][0]
    assert lib["code"] == "GEMM" and lib["implementation_type"] == "BLAS" and lib["precision"] == ord("s") and lib["m"] == "32"
    edge = blk["dataflow"]["edges"][0]
    assert set(edge) == {"element_id", "debug_info", "src", "dst", "src_conn", "dst_conn", "subset", "base_type"}
    assert edge["dst"] == lib["element_id"] and edge["dst_conn"] == "__A" and edge["src_conn"] == "void" and edge["subset"] == []
    # and back
    again = StructuredSDFG.from_docc_json(json.dumps(d))
    strip = lambda nodes: [{k: v for k, v in n.items() if k != "element_id"} for n in nodes]
    assert strip(again.library_nodes()) == strip(s.library_nodes())
    assert again.containers == s.containers and again.arguments == s.arguments
    for a, b2 in zip(again._data["root"]["children"], s._data["root"]["children"]):
        assert a["dataflow"]["inputs"] == b2["dataflow"]["inputs"] and a["dataflow"]["outputs"] == b2["dataflow"]["outputs"]
        assert a.get("debug_info") == b2.get("debug_info")


def test_cast_and_transpose_nodes_cross_the_formats():
    """ml::Cast carries its target type as the reference's enum value there (cast_node.cpp serializer) and takes the
    input's element type from the input memlet; ml::Transpose carries shape and perm."""
    b = StructuredSDFGBuilder("ct")
    b.add_container("X", Pointer(Scalar(PrimitiveType.Float)), True)
    b.add_container("H", Pointer(Scalar(PrimitiveType.BFloat)), False, transient_bytes=6 * 4 * 2)
    b.add_container("Y", Pointer(Scalar(PrimitiveType.BFloat)), True)
    b.add_cast_op("X", "H", [6, 4])
    b.add_transpose("H", "Y", [6, 4], [1, 0])
    s = b.move()
    d = json.loads(s.to_docc_json())
    cast, tr = (c["dataflow"]["nodes"][0] for c in d["root"]["children"][:2])
    assert cast["code"] == "ml::Cast" and cast["target_type"] == 13 and cast["shape"] == ["6", "4"]      # BFloat in the reference's enum
    assert tr["code"] == "ml::Transpose" and tr["perm"] == [1, 0]
    # a dump as the reference writes it has no element_type key on the nodes
    for n in (cast, tr):
        n.pop("element_type", None)
    again = StructuredSDFG.from_docc_json(json.dumps(d))
    strip = lambda nodes: [{k: v for k, v in n.items() if k != "element_id"} for n in nodes]
    assert strip(again.library_nodes()) == strip(s.library_nodes())
    assert again.library_nodes()[0]["element_type"] == "Float" and again.library_nodes()[0]["target_type"] == "BFloat"


# ---- loop nests that are elementwise work -------------------------------------------------------------
# What the front end writes for `Y[:, :] = X` and for the copy into the return buffer (python/docc/python/
# ast_parser.py:1186-1210, :2102-2270): one For per sliced dimension (var = 0; var < extent; var = 1 + var), and in
# the innermost body a block with one assign tasklet whose memlets carry a Tensor type and one loop variable per
# dimension. The elementwise tensor nodes expand to Maps of the same shape (elementwise_node.cpp:86-240).

def tensor(prim, shape, strides=None):
    if strides is None:
        strides, acc = [], []
        for d in reversed(shape):
            strides.insert(0, "*".join(acc) if acc else "1")
            acc.insert(0, d)
    return {"type": "tensor", "element_type": scalar(prim), "shape": list(shape), "strides": list(strides), "offset": "0",
            "storage_type": STACK, "initializer": "", "alignment": 0}


def docc_nest(ids, kind, loops, op, inputs, output):
    """loops: [(variable, extent)], outermost first; inputs: [(connector, container or (literal, prim), subset, base type)];
    output: (connector, container, subset, base type); op: the tasklet or CMath node without its ids."""
    op = {"element_id": ids(), "debug_info": NO_DEBUG, **op}
    nodes, edges = [op], []
    for conn, value, subset, base in inputs:
        nid = ids()
        if isinstance(value, tuple):
            nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "constant_node", "data": value[0], "data_type": scalar(value[1])})
        else:
            nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "access_node", "data": value})
        edges.append({"element_id": ids(), "debug_info": NO_DEBUG, "src": nid, "dst": op["element_id"], "src_conn": "void", "dst_conn": conn,
                      "subset": list(subset), "base_type": base})
    conn, name, subset, base = output
    nid = ids()
    nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "access_node", "data": name})
    edges.append({"element_id": ids(), "debug_info": NO_DEBUG, "src": op["element_id"], "dst": nid, "src_conn": conn, "dst_conn": "void",
                  "subset": list(subset), "base_type": base})
    body = {"type": "block", "element_id": ids(), "debug_info": NO_DEBUG, "dataflow": {"type": "dataflow", "nodes": nodes, "edges": edges}}
    for loop in reversed(loops):
        var, extent = loop[0], loop[1]
        this_kind = loop[2] if len(loop) > 2 else kind      # a loop may name its own kind (maps around fors in a reduction)
        seq = {"type": "sequence", "element_id": ids(), "debug_info": NO_DEBUG, "children": [body],
               "transitions": [{"type": "transition", "element_id": ids(), "debug_info": NO_DEBUG, "assignments": []}]}
        body = {"type": this_kind, "element_id": ids(), "debug_info": NO_DEBUG, "indvar": var, "init": "0", "condition": f"{var} < {extent}",
                "update": f"1 + {var}", "root": seq}
        if this_kind == "map":
            body["schedule_type"] = {"value": "SEQUENTIAL", "category": 0, "properties": {}}
    return body


ASSIGN = {"type": "tasklet", "code": 0, "inputs": ["_in"], "output": "_out"}


def return_matmul_program():
    """`def f(A, B): return A @ B` as the front end leaves it: the product in a Malloc'ed temporary, a copy nest into
    the return buffer, the temporary freed, return."""
    ids = Ids()
    containers = {n: pointer(DOUBLE) for n in ("A", "B", "_docc_ret_0", "_tmp_0")}
    for n in ("_s0", "_slice_iter_0_", "_slice_iter_1_"):
        containers[n] = scalar(INT64)
    gemm = {"implementation_type": "BLAS", "code": "GEMM", "precision": ord("d"), "layout": 101, "trans_a": 111, "trans_b": 111,
            "m": "_s0", "n": "_s0", "k": "_s0", "lda": "_s0", "ldb": "_s0", "ldc": "_s0"}
    t = tensor(DOUBLE, ["_s0", "_s0"])
    idx = ["_slice_iter_0_", "_slice_iter_1_"]
    children = [
        docc_block(ids, {"implementation_type": "NONE", "code": "Malloc", "size": "8*_s0**2"}, [], [("_ret", "_tmp_0")], containers),
        docc_block(ids, gemm, [("__A", "A"), ("__B", "B"), ("__C", "_tmp_0"), ("__alpha", ("1.0", DOUBLE)), ("__beta", ("0.0", DOUBLE))],
                   [("__C", "_tmp_0")], containers),
        docc_nest(ids, "for", [("_slice_iter_0_", "_s0"), ("_slice_iter_1_", "_s0")], ASSIGN,
                  [("_in", "_tmp_0", idx, t)], ("_out", "_docc_ret_0", idx, t)),
        docc_block(ids, {"implementation_type": "NONE", "code": "Free"}, [("_ptr", "_tmp_0")], [("_ptr", "_tmp_0")], containers),
        {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG},
    ]
    return docc_sdfg("f_sdfg", containers, ["A", "B", "_s0", "_docc_ret_0"], children, ids)


def elementwise_nests_program():
    """Maps as the expanded tensor nodes leave them, over [_s0, _s1] fp32 buffers indexed by one linearised expression:
    S = X + Y; E = exp(S); T[j][i] = E[i][j] (T is [_s1, _s0]); Z = 0.5 everywhere; W = E / 3."""
    ids = Ids()
    containers = {n: pointer(FLOAT) for n in ("X", "Y", "S", "E", "T", "Z", "W")}
    for n in ("_s0", "_s1", "_i0", "_i1"):
        containers[n] = scalar(INT64)
    P = pointer(FLOAT)
    loops = [("_i0", "_s0"), ("_i1", "_s1")]
    rm, cm = ["_i1 + _i0*_s1"], ["_i0 + _i1*_s0"]
    children = [
        docc_nest(ids, "map", loops, {"type": "tasklet", "code": 2, "inputs": ["_in1", "_in2"], "output": "_out"},
                  [("_in1", "X", rm, P), ("_in2", "Y", rm, P)], ("_out", "S", rm, P)),
        docc_nest(ids, "map", loops, {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": "expf",
                                      "function_stem": "exp", "primitive_type": FLOAT},
                  [("_in1", "S", rm, P)], ("_out", "E", rm, P)),
        docc_nest(ids, "map", loops, ASSIGN, [("_in", "E", rm, P)], ("_out", "T", cm, P)),
        docc_nest(ids, "map", loops, ASSIGN, [("_in", ("0.5f", FLOAT), [], scalar(FLOAT))], ("_out", "Z", rm, P)),
        docc_nest(ids, "map", loops, {"type": "tasklet", "code": 5, "inputs": ["_in1", "_in2"], "output": "_out"},
                  [("_in1", "E", rm, P), ("_in2", ("3.0f", FLOAT), [], scalar(FLOAT))], ("_out", "W", rm, P)),
        {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG},
    ]
    return docc_sdfg("nests_sdfg", containers, ["X", "Y", "S", "E", "T", "Z", "W", "_s0", "_s1"], children, ids)


def test_return_copy_nest_imports_as_a_copy_kernel(tmp_path):
    s = StructuredSDFG.from_docc_json(json.dumps(return_matmul_program()))
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["GEMM", "ml::Transpose"]
    assert nodes[1]["shape"] == ["_s0", "_s0"] and nodes[1]["perm"] == [0, 1] and nodes[1]["element_type"] == "Double"
    copy_block = s._data["root"]["children"][1]["dataflow"]
    assert copy_block["inputs"] == [{"data": "_tmp_0", "connector": "X"}] and copy_block["outputs"] == [{"data": "_docc_ret_0", "connector": "Y"}]
    s.schedule("rocm")
    r = s.loop_report()
    assert r["H2D"] == 2 and r["D2H"] == 1            # A and B up, the return buffer down; the product never leaves the device
    src = Path(s.generate(str(tmp_path))["source"]).read_text()
    assert src.count("docc_rocm_dgemm(") == 1 and src.count("docc_rocm_transpose(") == 1
    assert 'extern "C" void f_sdfg(double *A, double *B, int64_t _s0, double *_docc_ret_0)' in src


def test_elementwise_nests_import_as_tensor_nodes():
    s = StructuredSDFG.from_docc_json(json.dumps(elementwise_nests_program()))
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["ml::Add", "ml::Exp", "ml::Transpose", "ml::Fill", "ml::Div"]
    assert all(n["shape"] == ["_s0", "_s1"] for n in nodes) and all(n["element_type"] == "Float" for n in nodes)
    assert nodes[2]["perm"] == [1, 0]
    blocks = [c["dataflow"] for c in s._data["root"]["children"][:5]]
    assert blocks[0]["inputs"] == [{"data": "X", "connector": "A"}, {"data": "Y", "connector": "B"}] and blocks[0]["outputs"] == [{"data": "S", "connector": "C"}]
    assert blocks[3]["inputs"] == [{"constant": "0.5f", "type": "Float", "connector": "X"}]
    assert blocks[4]["inputs"][1] == {"constant": "3.0f", "type": "Float", "connector": "B"}
    s.schedule("rocm")


def test_loop_nests_outside_the_elementwise_forms_are_refused():
    base = elementwise_nests_program()

    def nest(i):
        return base["root"]["children"][i]

    def inner_block(n):
        while n["type"] != "block":
            n = n["root"]["children"][0] if n["type"] in ("for", "map") else n["children"][0]
        return n

    def refused(prog, why):
        with pytest.raises(InvalidSDFGException, match=why):
            StructuredSDFG.from_docc_json(json.dumps(prog))

    bad = copy.deepcopy(base)
    bad["root"]["children"][0]["init"] = "1"
    refused(bad, r"map \(element \d+\): the loop does not start at 0")
    bad = copy.deepcopy(base)
    bad["root"]["children"][0]["condition"] = "_i0 <= _s0"
    refused(bad, "condition is not 'variable < bound'")
    bad = copy.deepcopy(base)
    inner_block(bad["root"]["children"][0])["dataflow"]["edges"][0]["subset"] = ["_i1 + _i0*_s0"]      # wrong row pitch: not the dense tensor of the nest
    refused(bad, "operand 'X' is not a dense tensor indexed by the loop variables")
    bad = copy.deepcopy(base)
    inner_block(bad["root"]["children"][0])["dataflow"]["edges"][0]["subset"] = ["1 + _i1 + _i0*_s1"]  # shifted by one element
    refused(bad, "operand 'X' is not a dense tensor")
    # several statements under a sequential loop (under maps they become a generated kernel)
    bad = copy.deepcopy(base)
    bad["root"]["children"][0]["type"] = "for"
    bad["root"]["children"][0]["root"]["children"].append(copy.deepcopy(inner_block(nest(1))))
    bad["root"]["children"][0]["root"]["transitions"].append(copy.deepcopy(bad["root"]["children"][0]["root"]["transitions"][0]))
    refused(bad, "more than one statement in a loop body")


def permuted_copy_and_scalar_program():
    """T[k][i][j] = X[i][j][k] over a [_s0, _s1, 5] array (Tensor-typed memlets, the loop order of the source), a
    difference with the scalar on the left (S = 2 - X, linearised pointers), and a scalar argument stored into the
    one-element return buffer (the scalar form of the front end's return copy, ast_parser.py:1150-1157)."""
    ids = Ids()
    containers = {n: pointer(DOUBLE) for n in ("X", "T", "S", "_docc_ret_0")}
    for n in ("_s0", "_s1", "_i0", "_i1", "_i2"):
        containers[n] = scalar(INT64)
    containers["v"] = scalar(DOUBLE)
    tx = tensor(DOUBLE, ["_s0", "_s1", "5"])
    tt = tensor(DOUBLE, ["5", "_s0", "_s1"])
    P = pointer(DOUBLE)
    loops = [("_i0", "_s0"), ("_i1", "_s1"), ("_i2", "5")]
    lin = ["_i2 + 5*_i1 + 5*_i0*_s1"]
    children = [
        docc_nest(ids, "for", loops, ASSIGN, [("_in", "X", ["_i0", "_i1", "_i2"], tx)], ("_out", "T", ["_i2", "_i0", "_i1"], tt)),
        docc_nest(ids, "map", loops, {"type": "tasklet", "code": 3, "inputs": ["_in1", "_in2"], "output": "_out"},
                  [("_in1", ("2.0", DOUBLE), [], scalar(DOUBLE)), ("_in2", "X", lin, P)], ("_out", "S", lin, P)),
        docc_nest(ids, "for", [], ASSIGN, [("_in", "v", [], scalar(DOUBLE))], ("_out", "_docc_ret_0", ["0"], P)),
        {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG},
    ]
    return docc_sdfg("perm_sdfg", containers, ["X", "T", "S", "v", "_s0", "_s1", "_docc_ret_0"], children, ids)


def test_permuted_copies_scalar_operands_and_scalar_stores_import():
    s = StructuredSDFG.from_docc_json(json.dumps(permuted_copy_and_scalar_program()))
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["ml::Transpose", "ml::Sub", "ml::Fill"]
    # output axis a of the copy is the input axis that runs over the same loop: T's axes (k, i, j) are X's axes (2, 0, 1)
    assert nodes[0]["shape"] == ["_s0", "_s1", "5"] and nodes[0]["perm"] == [2, 0, 1]
    blocks = [c["dataflow"] for c in s._data["root"]["children"][:3]]
    assert blocks[1]["inputs"] == [{"constant": "2.0", "type": "Double", "connector": "A"}, {"data": "X", "connector": "B"}]
    assert nodes[2]["shape"] == ["1"] and blocks[2]["inputs"] == [{"data": "v", "connector": "X"}]
    s.schedule("rocm")
    # a tensor type that starts past its container's first element is not matched
    bad = permuted_copy_and_scalar_program()
    blk = bad["root"]["children"][0]
    while blk["type"] != "block":
        blk = blk["root"]["children"][0]
    blk["dataflow"]["edges"][0]["base_type"]["offset"] = "3"
    with pytest.raises(InvalidSDFGException, match="operand 'X' is not a dense tensor"):
        StructuredSDFG.from_docc_json(json.dumps(bad))


def reduce_nests(ids, cmath_or_tasklet, identity, x, y, rows, cols, tx, ty):
    """Max / Sum over the last axis with keepdims as ReduceNode::expand leaves it (reduce_node.cpp:186-330): a nest of
    maps that stores the identity into every result element, then maps over the kept extent around a for over the
    reduced one, whose body combines X[i, k] with Y[i, 0] into Y[i, 0]."""
    init = docc_nest(ids, "map", [("_i_init", rows), ("_i_init_1", "1")], ASSIGN, [("_in", (identity, FLOAT), [], scalar(FLOAT))],
                     ("_out", y, ["_i_init", "_i_init_1"], ty))
    body = docc_nest(ids, "map", [("_i", rows, "map"), ("_k", cols, "for")], cmath_or_tasklet,
                     [("_in1", x, ["_i", "_k"], tx), ("_in2", y, ["_i", "0"], ty)], ("_out", y, ["_i", "0"], ty))
    return [init, body]


def expanded_softmax_program():
    """`Y = softmax(X, axis=-1)` on fp32 [_s0, _s1] after the tensor nodes were expanded: the seven steps of
    SoftmaxNode::expand (softmax_node.cpp:142-252) as the loop nests their own expansions leave (reduce_node.cpp,
    broadcast_node.cpp:110-187, the elementwise maps), over Malloc'ed temporaries."""
    ids = Ids()
    names = ("X", "Y", "_max", "_max_b", "_sub", "_exp", "_sum", "_sum_b")
    containers = {n: pointer(FLOAT) for n in names}
    for n in ("_s0", "_s1", "_i_init", "_i_init_1", "_i", "_k", "_i0", "_i1"):
        containers[n] = scalar(INT64)
    full, red = tensor(FLOAT, ["_s0", "_s1"]), tensor(FLOAT, ["_s0", "1"])
    both = [("_i0", "_s0"), ("_i1", "_s1")]
    ij = ["_i0", "_i1"]
    fmax = {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": "fmaxf", "function_stem": "fmax", "primitive_type": FLOAT}
    expf = {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": "expf", "function_stem": "exp", "primitive_type": FLOAT}
    add = {"type": "tasklet", "code": 2, "inputs": ["_in1", "_in2"], "output": "_out"}
    sub = {"type": "tasklet", "code": 3, "inputs": ["_in1", "_in2"], "output": "_out"}
    div = {"type": "tasklet", "code": 5, "inputs": ["_in1", "_in2"], "output": "_out"}
    children = []
    for name, size in (("_max", "4*_s0"), ("_max_b", "4*_s0*_s1"), ("_sub", "4*_s0*_s1"), ("_exp", "4*_s0*_s1"), ("_sum", "4*_s0"), ("_sum_b", "4*_s0*_s1")):
        children.append(docc_block(ids, {"implementation_type": "NONE", "code": "Malloc", "size": size}, [], [("_ret", name)], containers))
    children += reduce_nests(ids, fmax, "-INFINITY", "X", "_max", "_s0", "_s1", full, red)
    children.append(docc_nest(ids, "map", both, ASSIGN, [("_in", "_max", ["_i0", "0"], red)], ("_out", "_max_b", ij, full)))
    children.append(docc_nest(ids, "map", both, sub, [("_in1", "X", ij, full), ("_in2", "_max_b", ij, full)], ("_out", "_sub", ij, full)))
    children.append(docc_nest(ids, "map", both, expf, [("_in1", "_sub", ij, full)], ("_out", "_exp", ij, full)))
    children += reduce_nests(ids, add, "0.0", "_exp", "_sum", "_s0", "_s1", full, red)
    children.append(docc_nest(ids, "map", both, ASSIGN, [("_in", "_sum", ["_i0", "0"], red)], ("_out", "_sum_b", ij, full)))
    children.append(docc_nest(ids, "map", both, div, [("_in1", "_exp", ij, full), ("_in2", "_sum_b", ij, full)], ("_out", "Y", ij, full)))
    for name in ("_max", "_max_b", "_sub", "_exp", "_sum", "_sum_b"):
        children.append(docc_block(ids, {"implementation_type": "NONE", "code": "Free"}, [("_ptr", name)], [("_ptr", name)], containers))
    children.append({"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG})
    return docc_sdfg("softmax_sdfg", containers, ["X", "Y", "_s0", "_s1"], children, ids)


def test_expanded_softmax_imports_as_its_nodes_and_becomes_one_kernel(tmp_path):
    s = StructuredSDFG.from_docc_json(json.dumps(expanded_softmax_program()))
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["ml::Max", "ml::Broadcast", "ml::Sub", "ml::Exp", "ml::Sum", "ml::Broadcast", "ml::Div"]
    assert nodes[0]["shape"] == ["_s0", "_s1"] and nodes[0]["axes"] == [1] and nodes[0]["keepdims"] is True
    assert nodes[4]["axes"] == [1] and nodes[4]["keepdims"] is True
    assert nodes[1]["input_shape"] == ["_s0", "1"] and nodes[1]["output_shape"] == ["_s0", "_s1"]
    s.schedule("rocm")
    assert [n["code"] for n in s.library_nodes() if n["code"].startswith("ml::")] == ["ml::Softmax"]
    src = Path(s.generate(str(tmp_path))["source"]).read_text()
    assert "docc_rocm_softmax" in src and "docc_rocm_reduce" not in src


def test_accumulations_that_are_not_the_expansion_of_a_reduction_are_refused():
    prog = expanded_softmax_program()
    # without the nest that sets the maximum to -INFINITY the accumulation has no known starting value
    kids = prog["root"]["children"] if "root" in prog else None
    text = json.dumps(prog)
    bad = json.loads(text)
    root = bad["root"]
    maps = [i for i, c in enumerate(root["children"]) if c["type"] == "map"]
    del root["children"][maps[0]]
    del root["transitions"][maps[0]]
    with pytest.raises(Exception, match="identity"):
        StructuredSDFG.from_docc_json(json.dumps(bad))
    # a product accumulated over an axis is no node of the target
    bad = json.loads(text)
    for c in bad["root"]["children"]:
        if c["type"] == "map":
            stack = [c]
            while stack:
                e = stack.pop()
                if isinstance(e, dict):
                    if e.get("type") == "tasklet" and e.get("code") == 2:
                        e["code"] = 4
                    stack.extend(e.values())
                elif isinstance(e, list):
                    stack.extend(e)
    with pytest.raises(Exception, match="sum, maximum or minimum"):
        StructuredSDFG.from_docc_json(json.dumps(bad))


def test_reduction_nests_over_other_axes_and_index_forms():
    """The same pair of nests reducing the first axis (result without the reduced dimension), with one linearised index
    per operand, and over two separated axes of a rank-3 tensor (kept as extents of 1)."""
    add = {"type": "tasklet", "code": 2, "inputs": ["_in1", "_in2"], "output": "_out"}
    fmax = {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": "fmaxf", "function_stem": "fmax", "primitive_type": FLOAT}

    def program(symbols, nests):
        ids = Ids()
        containers = {n: pointer(FLOAT) for n in ("X", "Y")}
        for n in symbols:
            containers[n] = scalar(INT64)
        children = nests(ids) + [{"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG}]
        return docc_sdfg("r_sdfg", containers, ["X", "Y"] + [n for n in symbols if n.startswith("_s")], children, ids)

    def node(prog):
        nodes = StructuredSDFG.from_docc_json(json.dumps(prog)).library_nodes()
        assert len(nodes) == 1
        return nodes[0]

    def columns(ids):
        tx, ty = tensor(FLOAT, ["_s0", "_s1"]), tensor(FLOAT, ["_s1"])
        return [docc_nest(ids, "map", [("_ii", "_s1")], ASSIGN, [("_in", ("0.0", FLOAT), [], scalar(FLOAT))], ("_out", "Y", ["_ii"], ty)),
                docc_nest(ids, "map", [("_i", "_s1", "map"), ("_k", "_s0", "for")], add,
                          [("_in1", "X", ["_k", "_i"], tx), ("_in2", "Y", ["_i"], ty)], ("_out", "Y", ["_i"], ty))]
    n = node(program(["_s0", "_s1", "_ii", "_i", "_k"], columns))
    assert (n["code"], n["shape"], n["axes"], n["keepdims"]) == ("ml::Sum", ["_s0", "_s1"], [0], False)

    def linear(ids):
        P = pointer(FLOAT)
        return [docc_nest(ids, "map", [("_ii", "_s0")], ASSIGN, [("_in", ("-INFINITY", FLOAT), [], scalar(FLOAT))], ("_out", "Y", ["_ii"], P)),
                docc_nest(ids, "map", [("_i", "_s0", "map"), ("_k", "_s1", "for")], fmax,
                          [("_in1", "X", ["_k + _i*_s1"], P), ("_in2", "Y", ["_i"], P)], ("_out", "Y", ["_i"], P))]
    n = node(program(["_s0", "_s1", "_ii", "_i", "_k"], linear))
    assert (n["code"], n["shape"], n["axes"], n["keepdims"]) == ("ml::Max", ["_s0", "_s1"], [1], False)

    def two_axes(ids):
        tx, ty = tensor(FLOAT, ["_s0", "_s1", "_s2"]), tensor(FLOAT, ["1", "_s1", "1"])
        return [docc_nest(ids, "map", [("_a", "1"), ("_ii", "_s1"), ("_c", "1")], ASSIGN, [("_in", ("0.0", FLOAT), [], scalar(FLOAT))],
                          ("_out", "Y", ["_a", "_ii", "_c"], ty)),
                docc_nest(ids, "map", [("_i", "_s1", "map"), ("_k", "_s0", "for"), ("_k2", "_s2", "for")], add,
                          [("_in1", "X", ["_k", "_i", "_k2"], tx), ("_in2", "Y", ["0", "_i", "0"], ty)], ("_out", "Y", ["0", "_i", "0"], ty))]
    n = node(program(["_s0", "_s1", "_s2", "_ii", "_i", "_k", "_k2", "_a", "_c"], two_axes))
    assert (n["code"], n["shape"], n["axes"], n["keepdims"]) == ("ml::Sum", ["_s0", "_s1", "_s2"], [0, 2], True)

    # a maximum initialised with the identity of a sum is not the expansion of a node
    def wrong_identity(ids):
        P = pointer(FLOAT)
        return [docc_nest(ids, "map", [("_ii", "_s0")], ASSIGN, [("_in", ("0.0", FLOAT), [], scalar(FLOAT))], ("_out", "Y", ["_ii"], P)),
                docc_nest(ids, "map", [("_i", "_s0", "map"), ("_k", "_s1", "for")], fmax,
                          [("_in1", "X", ["_k + _i*_s1"], P), ("_in2", "Y", ["_i"], P)], ("_out", "Y", ["_i"], P))]
    with pytest.raises(Exception, match="identity"):
        StructuredSDFG.from_docc_json(json.dumps(program(["_s0", "_s1", "_ii", "_i", "_k"], wrong_identity)))


def expanded_mean_program():
    """`Y = mean(X, axis=1)` on fp32 [_s0, _s1] after expansion (mean_node.cpp:24-125): the two nests of the sum, an empty
    block whose transition sets `_mean_count = _s1`, and the map that divides the sums by that count."""
    ids = Ids()
    containers = {n: pointer(FLOAT) for n in ("X", "Y")}
    for n in ("_s0", "_s1", "_ii", "_i", "_k", "_j", "_mean_count"):
        containers[n] = scalar(INT64)
    tx, ty = tensor(FLOAT, ["_s0", "_s1"]), tensor(FLOAT, ["_s0"])
    add = {"type": "tasklet", "code": 2, "inputs": ["_in1", "_in2"], "output": "_out"}
    div = {"type": "tasklet", "code": 5, "inputs": ["_in1", "_in2"], "output": "_out"}
    children = [
        docc_nest(ids, "map", [("_ii", "_s0")], ASSIGN, [("_in", ("0.0", FLOAT), [], scalar(FLOAT))], ("_out", "Y", ["_ii"], ty)),
        docc_nest(ids, "map", [("_i", "_s0", "map"), ("_k", "_s1", "for")], add,
                  [("_in1", "X", ["_i", "_k"], tx), ("_in2", "Y", ["_i"], ty)], ("_out", "Y", ["_i"], ty)),
        {"type": "block", "element_id": ids(), "debug_info": NO_DEBUG, "dataflow": {"type": "dataflow", "nodes": [], "edges": []}},
        docc_nest(ids, "map", [("_j", "_s0")], div, [("_in1", "Y", ["_j"], ty), ("_in2", "_mean_count", [], tensor(FLOAT, []))],
                  ("_out", "Y", ["_j"], ty)),
        {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG},
    ]
    prog = docc_sdfg("mean_sdfg", containers, ["X", "Y", "_s0", "_s1"], children, ids)
    prog["root"]["transitions"][2]["assignments"] = [{"symbol": "_mean_count", "expression": "_s1"}]
    return prog


def test_expanded_mean_imports_with_its_count_as_an_expression(tmp_path):
    s = StructuredSDFG.from_docc_json(json.dumps(expanded_mean_program()))
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["ml::Sum", "ml::Div"]
    div = s._data["root"]["children"][1]["dataflow"]
    assert div["inputs"][1] == {"constant": "(_s1)", "type": "Float", "connector": "B"}
    s.schedule("rocm")
    src = Path(s.generate(str(tmp_path))["source"]).read_text()
    assert "docc_rocm_reduce" in src and "(_s1)" in src
    # a symbol set from something that is not an argument has no value the generated function could know
    bad = expanded_mean_program()
    bad["root"]["transitions"][2]["assignments"] = [{"symbol": "_mean_count", "expression": "_k + 1"}]
    with pytest.raises(Exception, match="scalar arguments"):
        StructuredSDFG.from_docc_json(json.dumps(bad))


def numpy_softmax_expanded_program():
    """softmax as numpy code spells it - `m = max(x, -1, keepdims)`, `e = exp(x - m)`, `e / sum(e, -1, keepdims)` - after
    expansion. The front end repeats `m` and the sum along the rows with views whose stride is 0 in the repeated
    dimension (numpy.py:1193-1232, :2679-2705), so the subtraction and the division index them with both loop variables."""
    ids = Ids()
    names = ("X", "Y", "_m", "_d", "_e", "_s")
    containers = {n: pointer(FLOAT) for n in names}
    for n in ("_s0", "_s1", "_i_init", "_i_init_1", "_i", "_k", "_i0", "_i1"):
        containers[n] = scalar(INT64)
    full, red = tensor(FLOAT, ["_s0", "_s1"]), tensor(FLOAT, ["_s0", "1"])
    view = tensor(FLOAT, ["_s0", "_s1"], ["1", "0"])          # [rows, 1] seen as [rows, cols]
    both, ij = [("_i0", "_s0"), ("_i1", "_s1")], ["_i0", "_i1"]
    fmax = {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": "fmaxf", "function_stem": "fmax", "primitive_type": FLOAT}
    expf = {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": "expf", "function_stem": "exp", "primitive_type": FLOAT}
    add = {"type": "tasklet", "code": 2, "inputs": ["_in1", "_in2"], "output": "_out"}
    sub = {"type": "tasklet", "code": 3, "inputs": ["_in1", "_in2"], "output": "_out"}
    div = {"type": "tasklet", "code": 5, "inputs": ["_in1", "_in2"], "output": "_out"}
    children = []
    for name, size in (("_m", "4*_s0"), ("_d", "4*_s0*_s1"), ("_e", "4*_s0*_s1"), ("_s", "4*_s0")):
        children.append(docc_block(ids, {"implementation_type": "NONE", "code": "Malloc", "size": size}, [], [("_ret", name)], containers))
    children += reduce_nests(ids, fmax, "-INFINITY", "X", "_m", "_s0", "_s1", full, red)
    children.append(docc_nest(ids, "map", both, sub, [("_in1", "X", ij, full), ("_in2", "_m", ij, view)], ("_out", "_d", ij, full)))
    children.append(docc_nest(ids, "map", both, expf, [("_in1", "_d", ij, full)], ("_out", "_e", ij, full)))
    children += reduce_nests(ids, add, "0.0", "_e", "_s", "_s0", "_s1", full, red)
    children.append(docc_nest(ids, "map", both, div, [("_in1", "_e", ij, full), ("_in2", "_s", ij, view)], ("_out", "Y", ij, full)))
    for name in ("_m", "_d", "_e", "_s"):
        children.append(docc_block(ids, {"implementation_type": "NONE", "code": "Free"}, [("_ptr", name)], [("_ptr", name)], containers))
    children.append({"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG})
    return docc_sdfg("np_softmax_sdfg", containers, ["X", "Y", "_s0", "_s1"], children, ids)


def test_views_with_a_stride_of_zero_import_as_repeated_operands(tmp_path):
    s = StructuredSDFG.from_docc_json(json.dumps(numpy_softmax_expanded_program()))
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["ml::Max", "ml::Broadcast", "ml::Sub", "ml::Exp", "ml::Sum", "ml::Broadcast", "ml::Div"]
    assert nodes[1]["input_shape"] == ["_s0", "1"] and nodes[1]["output_shape"] == ["_s0", "_s1"]
    s.schedule("rocm", options={"match_softmax": False})
    codes = [n["code"] for n in s.library_nodes() if n["code"].startswith("ml::")]
    assert "ml::Broadcast" not in codes                 # folded into the subtraction and the division
    s = StructuredSDFG.from_docc_json(json.dumps(numpy_softmax_expanded_program()))
    s.schedule("rocm")
    assert [n["code"] for n in s.library_nodes() if n["code"].startswith("ml::")] == ["ml::Softmax"]
    assert "docc_rocm_softmax_f32" in Path(s.generate(str(tmp_path))["source"]).read_text()


# ---- loop nests that are not one of the prebuilt kernels: the generated-kernel path (ROCMMap) -------------------

def docc_map_nest(ids, loops, blocks):
    """A nest of maps whose innermost body is a run of blocks. blocks: one list of operations per block; an operation is
    (op, inputs, outputs) with inputs [(connector, container or (literal, prim), subset, base type)] and outputs
    [(container, subset, base type)]. Within a block an access node is shared by every edge that names its container,
    so a scalar written by one operation and read by the next forms the chain tasklet -> access node -> tasklet."""
    kids = []
    for ops in blocks:
        nodes, edges, access = [], [], {}

        def access_node(name):
            if name not in access:
                access[name] = ids()
                nodes.append({"element_id": access[name], "debug_info": NO_DEBUG, "type": "access_node", "data": name})
            return access[name]

        for op, inputs, outputs in ops:
            op = {"element_id": ids(), "debug_info": NO_DEBUG, **op}
            nodes.append(op)
            for conn, value, subset, base in inputs:
                if isinstance(value, tuple):
                    nid = ids()
                    nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "constant_node", "data": value[0], "data_type": scalar(value[1])})
                else:
                    nid = access_node(value)
                edges.append({"element_id": ids(), "debug_info": NO_DEBUG, "src": nid, "dst": op["element_id"], "src_conn": "void",
                              "dst_conn": conn, "subset": list(subset), "base_type": base})
            for name, subset, base in outputs:
                # a container that is read and written in one block has two access nodes: the value before, the value after
                nid = ids()
                nodes.append({"element_id": nid, "debug_info": NO_DEBUG, "type": "access_node", "data": name})
                access[name] = nid
                edges.append({"element_id": ids(), "debug_info": NO_DEBUG, "src": op["element_id"], "dst": nid, "src_conn": "_out",
                              "dst_conn": "void", "subset": list(subset), "base_type": base})
        kids.append({"type": "block", "element_id": ids(), "debug_info": NO_DEBUG, "dataflow": {"type": "dataflow", "nodes": nodes, "edges": edges}})
    body = None
    for var, extent in reversed(loops):
        children = kids if body is None else [body]
        seq = {"type": "sequence", "element_id": ids(), "debug_info": NO_DEBUG, "children": children,
               "transitions": [{"type": "transition", "element_id": ids(), "debug_info": NO_DEBUG, "assignments": []} for _ in children]}
        body = {"type": "map", "element_id": ids(), "debug_info": NO_DEBUG, "indvar": var, "init": "0", "condition": f"{var} < {extent}",
                "update": f"1 + {var}", "root": seq, "schedule_type": {"value": "SEQUENTIAL", "category": 0, "properties": {}}}
    return body


def tasklet(code, n_inputs):
    names = ["_in"] if n_inputs == 1 and code == 0 else [f"_in{i + 1}" for i in range(n_inputs)]
    return {"type": "tasklet", "code": code, "inputs": names, "output": "_out"}


def cmath(stem, prim):
    return {"type": "library_node", "implementation_type": "NONE", "code": "CMath", "name": stem + ("f" if prim == FLOAT else ""),
            "function_stem": stem, "primitive_type": prim}


def fused_map_program(prim=FLOAT):
    """Y = relu(A * B + C) over [_s0, _s1] as MapFusion leaves three elementwise maps (map_fusion.cpp:246-330): one map
    nest whose body is three blocks, the product and the sum handed on through scalar temporaries `_fused_tmp*`, the
    last block the fmax(0, x) that ReLU expands to (relu_node.cpp:27-50). C is a row of _s1 entries repeated over the
    rows (no index in _i0). A second nest, one block holding two chained tasklets: Z = (A - Y) / 3, and W[j][i] = Z[i][j]
    stored by the same iteration."""
    ids = Ids()
    containers = {n: pointer(prim) for n in ("A", "B", "C", "Y", "Z", "W")}
    for n in ("_s0", "_s1", "_i0", "_i1"):
        containers[n] = scalar(INT64)
    for n in ("_fused_tmp", "_fused_tmp_0", "_d"):
        containers[n] = scalar(prim)
    P, S = pointer(prim), scalar(prim)
    loops = [("_i0", "_s0"), ("_i1", "_s1")]
    rm, cm, row = ["_i1 + _i0*_s1"], ["_i0 + _i1*_s0"], ["_i1"]
    lit = (lambda v: (v + "f", prim)) if prim == FLOAT else (lambda v: (v, prim))
    children = [
        docc_map_nest(ids, loops, [
            [(tasklet(4, 2), [("_in1", "A", rm, P), ("_in2", "B", rm, P)], [("_fused_tmp", [], S)])],
            [(tasklet(2, 2), [("_in1", "_fused_tmp", [], S), ("_in2", "C", row, P)], [("_fused_tmp_0", [], S)])],
            [(cmath("fmax", prim), [("_in1", lit("0.0"), [], S), ("_in2", "_fused_tmp_0", [], S)], [("Y", rm, P)])],
        ]),
        docc_map_nest(ids, loops, [
            [(tasklet(3, 2), [("_in1", "A", rm, P), ("_in2", "Y", rm, P)], [("_d", [], S)]),
             (tasklet(5, 2), [("_in1", "_d", [], S), ("_in2", lit("3.0"), [], S)], [("Z", rm, P), ("W", cm, P)])],
        ]),
        {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG},
    ]
    return docc_sdfg("fused_maps_sdfg", containers, ["A", "B", "C", "Y", "Z", "W", "_s0", "_s1"], children, ids)


def test_map_nests_with_several_operations_import_as_generated_kernels(tmp_path):
    s = StructuredSDFG.from_docc_json(json.dumps(fused_map_program()))
    first, second = s.library_nodes()
    assert first["code"] == second["code"] == "ROCMMap"
    assert first["indvars"] == ["_i0", "_i1"] and first["bounds"] == ["_s0", "_s1"] and first["symbols"] == ["_s0", "_s1"]
    assert [(r["connector"], r["strides"], r["extent"]) for r in first["reads"]] == [
        ("_in0", ["_s1", "1"], "(_s0)*_s1"), ("_in1", ["_s1", "1"], "(_s0)*_s1"), ("_in2", ["0", "1"], "_s1")]
    assert [(st["op"], st["args"]) for st in first["statements"]] == [
        ("fp_mul", ["_in0", "_in1"]), ("fp_add", ["_v0", "_in2"]), ("fmax", ["#0.0f", "_v1"])]
    assert [(w["connector"], w["strides"], w["value"]) for w in first["writes"]] == [("_out0", ["_s1", "1"], "_v2")]
    blocks = [c["dataflow"] for c in s._data["root"]["children"][:2]]
    assert blocks[0]["inputs"] == [{"data": "A", "connector": "_in0"}, {"data": "B", "connector": "_in1"}, {"data": "C", "connector": "_in2"}]
    assert blocks[0]["outputs"] == [{"data": "Y", "connector": "_out0"}]
    # two results of one statement, one of them transposed
    assert [(w["connector"], w["strides"], w["value"]) for w in second["writes"]] == [
        ("_out0", ["_s1", "1"], "_v1"), ("_out1", ["1", "_s0"], "_v1")]
    assert [(st["op"], st["args"]) for st in second["statements"]] == [("fp_sub", ["_in0", "_in1"]), ("fp_div", ["_v0", "#3.0f"])]
    # the node survives the target's own JSON
    again = StructuredSDFG.parse(s.to_json())
    assert again.library_nodes() == s.library_nodes()

    # the two nests as two kernels (the map fusion pass would make one of them: Y of the first is what the second reads)
    merged = StructuredSDFG.parse(s.to_json())
    merged.schedule("rocm")
    (one,) = [n for n in merged.library_nodes() if n["code"] == "ROCMMap"]
    assert [w["value"] for w in one["writes"]] == ["_v2", "_v4", "_v4"] and len(one["reads"]) == 3      # Y, Z, W; Y is not read back
    assert merged.loop_report()["H2D"] == 3 and merged.loop_report()["D2H"] == 3
    s.schedule("rocm", options={"fuse_maps": False})
    assert [n["implementation_type"] for n in s.library_nodes() if n["code"] == "ROCMMap"] == ["ROCMWithoutTransfers"] * 2
    r = s.loop_report()
    assert r["H2D"] == 3 and r["D2H"] == 3            # A B C up; Y Z W down; Y stays on the device between the nests
    report = s.generate(str(tmp_path))
    src = Path(report["source"]).read_text()
    kernels = sorted(p.name for p in tmp_path.glob("kernel_*.hip"))
    assert len(kernels) == 2 and all(k.startswith("kernel_fused_maps_sdfg_") for k in kernels)
    stem = kernels[0][:-4]
    assert f'"{stem}.hsaco"' in src and "docc_rocm_module_load(" in src and "docc_rocm_module_get_function(" in src
    assert src.count("docc_rocm_launch(__docc_fn, __docc_grid, __docc_block, 0, nullptr, __docc_args)") == 2
    text = (tmp_path / kernels[0]).read_text()
    assert f'extern "C" __global__ void __launch_bounds__(256) {stem}_v32(' in text and f"{stem}_s64(" in text
    assert "const float _v0 = (float) (_in0) * (float) (_in1);" in text and "fmaxf((float) (0.0f), (float) (_v1))" in text
    assert "if (gid < total) {" in text
    # the kernel text is valid gfx950 code
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    for k in kernels:
        r = subprocess.run([hipcc, "--genco", "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature",
                            "-Xclang", "-packed-fp32-ops", str(tmp_path / k), "-o", str(tmp_path / (k[:-4] + ".hsaco"))], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-3000:]


def test_what_the_prebuilt_kernels_decline_goes_to_a_generated_kernel_under_maps_only():
    base = elementwise_nests_program()

    def inner_block(n):
        while n["type"] != "block":
            n = n["root"]["children"][0] if n["type"] in ("for", "map") else n["children"][0]
        return n

    # X + Y^T: the operands walk memory in different orders
    prog = copy.deepcopy(base)
    inner_block(prog["root"]["children"][0])["dataflow"]["edges"][1]["subset"] = ["_i0 + _i1*_s0"]
    node = StructuredSDFG.from_docc_json(json.dumps(prog)).library_nodes()[0]
    assert node["code"] == "ROCMMap" and [r["strides"] for r in node["reads"]] == [["_s1", "1"], ["1", "_s0"]]
    # a remainder and a gamma function have no node of their own
    prog = copy.deepcopy(base)
    inner_block(prog["root"]["children"][0])["dataflow"]["nodes"][0]["code"] = 6
    inner_block(prog["root"]["children"][1])["dataflow"]["nodes"][0]["function_stem"] = "lgamma"
    nodes = StructuredSDFG.from_docc_json(json.dumps(prog)).library_nodes()
    assert [n["code"] for n in nodes[:2]] == ["ROCMMap", "ROCMMap"]
    assert nodes[0]["statements"][0]["op"] == "fp_rem" and nodes[1]["statements"][0]["op"] == "lgamma"
    # the same under a sequential loop: nothing says that its iterations are independent
    prog = copy.deepcopy(base)
    prog["root"]["children"][0]["type"] = "for"
    inner_block(prog["root"]["children"][0])["dataflow"]["nodes"][0]["code"] = 6
    with pytest.raises(InvalidSDFGException, match="tasklet code 6 has no kernel"):
        StructuredSDFG.from_docc_json(json.dumps(prog))
    # an element other iterations write is read: not a nest the target may run in parallel. The second nest reads Y
    # row by row and writes W column by column; reading W row by row instead meets elements of other iterations
    prog = fused_map_program()
    blk = inner_block(prog["root"]["children"][1])
    for n in blk["dataflow"]["nodes"]:
        if n["type"] == "access_node" and n["data"] == "Y":
            n["data"] = "W"
    with pytest.raises(InvalidSDFGException, match="'W' is read at other elements than the one the iteration writes"):
        StructuredSDFG.from_docc_json(json.dumps(prog))
    # a result that one loop of the nest does not index would be written by many iterations
    prog = fused_map_program()
    last = prog["root"]["children"][0]["root"]["children"][0]["root"]["children"][2]
    for e in last["dataflow"]["edges"]:
        if e["src_conn"] == "_out":
            e["subset"] = ["_i1"]
    with pytest.raises(InvalidSDFGException, match="a result that some loops of the nest do not index"):
        StructuredSDFG.from_docc_json(json.dumps(prog))
