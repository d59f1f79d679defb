"""Python face of the SDFG carrier: `StructuredSDFG`, `StructuredSDFGBuilder`
and the element types, over the C ABI of ``libdocc_rocm_target.so``
(``include/docc_rocm_target.h``).

It mirrors the part of the reference's ``docc.sdfg`` module that the hot path
uses (python/bindings/bindings.cpp:136-480): ``StructuredSDFG.{parse, validate,
expand, simplify, normalize, dump, schedule, _compile, metadata, loop_report,
arguments, name}`` and ``StructuredSDFGBuilder.{add_container, add_gemm,
add_reduce_op, add_conv, add_return}``. The SDFG itself lives as JSON text and
is handed to the native library for every step that does real work.
"""
from __future__ import annotations

import ctypes
import enum
import json
import os
from pathlib import Path
import re
from typing import Any, Dict, List, Optional, Sequence, Tuple

_LIB_DIR = Path(__file__).resolve().parent.parent / "lib"
_TARGET_LIB = _LIB_DIR / "libdocc_rocm_target.so"
_INCLUDE_DIR = Path(__file__).resolve().parent.parent.parent / "include"

_lib: Optional[ctypes.CDLL] = None

#: every symbol include/docc_rocm_target.h declares
EXPORTED_SYMBOLS = (
    "docc_rocm_target_register", "docc_rocm_target_dispatcher_keys", "docc_rocm_target_validate",
    "docc_rocm_target_schedule", "docc_rocm_target_generate", "docc_rocm_target_compile",
    "docc_rocm_target_report", "docc_rocm_target_free", "docc_rocm_target_last_error",
    "docc_rocm_target_import", "docc_rocm_target_export", "docc_rocm_target_mappers",
)


class InvalidSDFGException(RuntimeError):
    pass


def _native() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _TARGET_LIB.exists():
            raise RuntimeError(f"{_TARGET_LIB} is missing; run `python -m docc_amd.build`")
        lib = ctypes.CDLL(str(_TARGET_LIB))
        cp = ctypes.c_char_p
        lib.docc_rocm_target_register.restype = ctypes.c_int
        for name, args in (("docc_rocm_target_dispatcher_keys", []), ("docc_rocm_target_mappers", []), ("docc_rocm_target_validate", [cp]),
                           ("docc_rocm_target_schedule", [cp, cp, cp]),
                           ("docc_rocm_target_import", [cp]), ("docc_rocm_target_export", [cp]), ("docc_rocm_target_generate", [cp, cp, cp]),
                           ("docc_rocm_target_compile", [cp, cp, cp, cp, cp]), ("docc_rocm_target_report", [cp])):
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = ctypes.c_void_p  # kept as an address so that it can be freed
        lib.docc_rocm_target_free.argtypes = [ctypes.c_void_p]
        lib.docc_rocm_target_last_error.restype = cp
        lib.docc_rocm_target_register()
        _lib = lib
    return _lib


def _call(name: str, *args: Optional[str]) -> str:
    lib = _native()
    raw = getattr(lib, name)(*[a.encode() if a is not None else None for a in args])
    if not raw:
        msg = (lib.docc_rocm_target_last_error() or b"").decode()
        raise InvalidSDFGException(msg or f"{name} failed")
    try:
        return ctypes.string_at(raw).decode()
    finally:
        lib.docc_rocm_target_free(raw)


def registered_dispatchers() -> List[str]:
    """The "<code>::<implementation type>" keys the code generator can dispatch."""
    return json.loads(_call("docc_rocm_target_dispatcher_keys"))


def registered_target_mappers() -> List[Dict[str, Any]]:
    """The target mapper factories of the plugin registry, highest priority first: [{"target", "priority"}]."""
    return json.loads(_call("docc_rocm_target_mappers"))


class PrimitiveType(enum.Enum):
    Void = "Void"
    Bool = "Bool"
    Int8 = "Int8"
    Int16 = "Int16"
    Int32 = "Int32"
    Int64 = "Int64"
    UInt8 = "UInt8"
    UInt16 = "UInt16"
    UInt32 = "UInt32"
    UInt64 = "UInt64"
    Half = "Half"
    BFloat = "BFloat"
    Float = "Float"
    Double = "Double"


class Scalar:
    def __init__(self, primitive_type: PrimitiveType):
        self.primitive_type = primitive_type

    def __repr__(self):
        return f"Scalar({self.primitive_type.name})"


class Pointer:
    def __init__(self, pointee: Scalar):
        self.pointee_type = pointee

    @property
    def primitive_type(self) -> PrimitiveType:
        return self.pointee_type.primitive_type

    def __repr__(self):
        return f"Pointer({self.pointee_type!r})"


# BLAS enums as the GEMM node serialises them (reference blas_node.h:49-126)
BLAS_PRECISION = {PrimitiveType.Half: ord("h"), PrimitiveType.Float: ord("s"), PrimitiveType.Double: ord("d"),
                  PrimitiveType.BFloat: ord("b")}
ROW_MAJOR, COL_MAJOR = 101, 102
NO_TRANS, TRANS = 111, 112


def _expr(e: Any) -> str:
    return str(int(e)) if isinstance(e, (int,)) or hasattr(e, "__index__") else str(e)


class StructuredSDFG:
    """An SDFG held as JSON; every operation goes through the native target library."""

    def __init__(self, data: Dict[str, Any]):
        self._data = data

    # -- construction ---------------------------------------------------------
    @staticmethod
    def parse(text: str) -> "StructuredSDFG":
        """Parses and validates an SDFG, in this package's JSON format or in the one docc's own
        serializer writes (StructuredSDFG.dump of a docc install)."""
        return StructuredSDFG(json.loads(_call("docc_rocm_target_validate", text)))

    @staticmethod
    def from_docc_json(text: str) -> "StructuredSDFG":
        """Imports an SDFG written by docc (reference sdfg/src/serializer/json_serializer.cpp:56-353).
        Raises InvalidSDFGException naming the first element the rocm target has no lowering for."""
        return StructuredSDFG(json.loads(_call("docc_rocm_target_import", text)))

    def to_docc_json(self) -> str:
        """This SDFG in docc's JSON format."""
        return _call("docc_rocm_target_export", self.to_json())

    @staticmethod
    def from_file(path: str) -> "StructuredSDFG":
        return StructuredSDFG.parse(Path(path).read_text())

    def to_json(self) -> str:
        return json.dumps(self._data)

    # -- inspection -----------------------------------------------------------
    @property
    def name(self) -> str:
        return self._data["name"]

    @property
    def arguments(self) -> List[str]:
        return list(self._data["arguments"])

    @property
    def containers(self) -> Dict[str, Any]:
        return self._data["containers"]

    @property
    def return_container(self) -> str:
        return self._data.get("return", "") or ""

    def type(self, name: str):
        c = self._data["containers"][name]
        s = Scalar(PrimitiveType(c["element"]))
        return Pointer(s) if c["type"] == "pointer" else s

    def metadata(self, key: str) -> str:
        return self._data.get("metadata", {})[key]

    def add_metadata(self, key: str, value: str) -> None:
        self._data.setdefault("metadata", {})[key] = str(value)

    def library_nodes(self) -> List[Dict[str, Any]]:
        return [c["dataflow"]["library_node"] for c in self._data["root"]["children"]]

    def loop_report(self) -> Dict[str, int]:
        """Counts per library-node code / implementation type and transfers (there are no loops in
        these SDFGs); the analogue of the reference's loop_report (py_structured_sdfg.cpp:570-583)."""
        return json.loads(_call("docc_rocm_target_report", self.to_json()))

    # -- pipeline -------------------------------------------------------------
    def validate(self) -> None:
        self._data = json.loads(_call("docc_rocm_target_validate", self.to_json()))

    def expand(self) -> None:
        """Math library nodes are kept whole for the rocm target; nothing to expand. (The
        reference expands them into loop nests for every target except the tensor targets,
        python/docc/python/python_program.py:275-277.)"""

    def simplify(self) -> None:
        """No loop nests, so there is nothing to simplify."""

    def normalize(self) -> None:
        """No loop nests, so there is nothing to normalize."""

    def dump(self, output_folder: str, suffix: str = "") -> None:
        """Writes <name>[.<suffix>].json and records the file names in the SDFG's metadata, as the
        reference's dump does (python/bindings/py_structured_sdfg.cpp:263-292); instrumented code
        carries them into every trace event."""
        os.makedirs(output_folder, exist_ok=True)
        stem = self.name + (f".{suffix}" if suffix else "")
        meta = self._data.setdefault("metadata", {})
        meta["sdfg_file"] = str(Path(output_folder, stem + ".json"))
        meta["arg_capture_path"] = str(Path(output_folder, "arg_captures" + (f".{suffix}" if suffix else "")))
        meta["features_file"] = str(Path(output_folder, stem + ".npz"))
        meta["opt_report_file"] = str(Path(output_folder, stem + ".opt_report.json"))
        Path(output_folder, stem + ".json").write_text(json.dumps(self._data, indent=2))

    def schedule(self, target: str, category: str = "server", remote_tuning: bool = False,
                 options: Optional[Dict[str, Any]] = None) -> None:
        if target in ("none", "sequential"):
            return
        if target != "rocm":
            raise NotImplementedError(f"Target '{target}' is not supported: this package provides the 'rocm' target only")
        opts = {k: v for k, v in (options or {}).items() if k in ("offload", "require_all_mapped", "fuse", "match_softmax", "fuse_maps")}
        self._data = json.loads(_call("docc_rocm_target_schedule", self.to_json(), category, json.dumps(opts)))

    def generate(self, output_folder: str, instrumentation_mode: str = "") -> Dict[str, Any]:
        """Writes <name>.h / <name>.cpp and returns the generator's report."""
        return json.loads(_call("docc_rocm_target_generate", self.to_json(), output_folder, instrumentation_mode or ""))

    def _compile(self, output_folder: str, target: str = "rocm", instrumentation_mode: str = "",
                 capture_args: bool = False) -> str:
        """Generates, compiles and links lib<name>.so; returns its path. `instrumentation_mode`
        "" or "ols" (reference py_structured_sdfg.cpp:376-383); argument capture is not part of
        this target."""
        if capture_args:
            raise NotImplementedError("argument capture (capture_args=True) is not part of the rocm target")
        return _call("docc_rocm_target_compile", self.to_json(), output_folder, str(_INCLUDE_DIR), str(_LIB_DIR),
                     instrumentation_mode or "")


class StructuredSDFGBuilder:
    """Builds the flat block sequence. Method names and argument meaning follow the reference's
    PyStructuredSDFGBuilder (python/bindings/builder/py_structured_sdfg_builder.cpp:654-774 add_gemm,
    :960-1013 add_conv, :1041-1088 add_reduce_op)."""

    def __init__(self, name: str, return_type: Optional[Any] = None):
        self._data: Dict[str, Any] = {"type": "structured_sdfg", "name": name, "arguments": [], "containers": {},
                                      "return": "", "metadata": {}, "root": {"type": "sequence", "children": []}}
        self._ids = 0

    def exists(self, name: str) -> bool:
        return name in self._data["containers"]

    def find_new_name(self, prefix: str = "tmp_") -> str:
        i = 0
        while f"{prefix}{i}" in self._data["containers"]:
            i += 1
        return f"{prefix}{i}"

    def add_container(self, name: str, type_: Any, is_argument: bool = False, transient_bytes: Optional[Any] = None,
                      storage: str = "CPU") -> None:
        if name in self._data["containers"]:
            raise InvalidSDFGException(f"container '{name}' already exists")
        entry = {"type": "pointer" if isinstance(type_, Pointer) else "scalar", "element": type_.primitive_type.value,
                 "transient": transient_bytes is not None, "storage": storage}
        if transient_bytes is not None:
            entry["size"] = _expr(transient_bytes)
        self._data["containers"][name] = entry
        if is_argument:
            self._data["arguments"].append(name)

    def _element(self, name: str) -> PrimitiveType:
        return PrimitiveType(self._data["containers"][name]["element"])

    def set_debug_info(self, filename: str = "", function: str = "", start_line: int = 0, start_column: int = 0,
                       end_line: int = 0, end_column: int = 0) -> None:
        """Source position attached to the blocks added from now on (the reference passes a
        DebugInfo to every add_* call; its JSON keys are those of debug_info_to_json,
        sdfg/src/serializer/json_serializer.cpp). An empty filename clears it."""
        self._debug_info = None if not filename else {
            "has": True, "filename": filename, "function": function, "start_line": int(start_line),
            "start_column": int(start_column), "end_line": int(end_line), "end_column": int(end_column)}

    def _add_block(self, node: Dict[str, Any], inputs: Sequence[Dict[str, Any]], outputs: Sequence[Dict[str, Any]]) -> None:
        self._ids += 2
        node = {"type": "library_node", "element_id": self._ids, **node}
        block = {"type": "block", "element_id": self._ids - 1, "dataflow": {
            "library_node": node, "inputs": list(inputs), "outputs": list(outputs)}}
        if getattr(self, "_debug_info", None):
            block["debug_info"] = dict(self._debug_info)
        self._data["root"]["children"].append(block)

    @staticmethod
    def _operand(connector: str, value: Any, const_type: Optional[PrimitiveType] = None) -> Dict[str, Any]:
        if const_type is not None:
            return {"connector": connector, "constant": str(value), "type": const_type.value}
        return {"connector": connector, "data": value}

    def add_gemm(self, A: str, B: str, C: str, alpha: str, beta: str, m: Any, n: Any, k: Any, trans_a: bool = False,
                 trans_b: bool = False, lda: Any = None, ldb: Any = None, ldc: Any = None) -> None:
        """C = alpha * op(A) op(B) + beta * C, row-major. alpha/beta are literals ("1.0") or scalar
        container names, as in the reference. The node is created with the BLAS implementation
        type, like the reference's add_gemm; the precision follows A's element type, and bf16
        operands select the added 'b' precision (fp32 accumulate, C must be Float)."""
        elem = self._element(A)
        if self._element(B) != elem:
            raise InvalidSDFGException("GEMM: A and B must have the same element type")
        if elem not in BLAS_PRECISION:
            raise InvalidSDFGException(f"GEMM: unsupported element type {elem.name}")
        out_elem = PrimitiveType.Float if elem == PrimitiveType.BFloat else elem
        if self._element(C) != out_elem:
            raise InvalidSDFGException(f"GEMM: C must be {out_elem.name} for {elem.name} operands")
        lda = lda if lda is not None else (m if trans_a else k)
        ldb = ldb if ldb is not None else (k if trans_b else n)
        ldc = ldc if ldc is not None else n

        def scalar(connector: str, v: str) -> Dict[str, Any]:
            return self._operand(connector, v) if v in self._data["containers"] else self._operand(connector, v, out_elem)

        self._add_block(
            {"code": "GEMM", "implementation_type": "BLAS", "side_effect": False, "precision": BLAS_PRECISION[elem],
             "layout": ROW_MAJOR, "trans_a": TRANS if trans_a else NO_TRANS, "trans_b": TRANS if trans_b else NO_TRANS,
             "m": _expr(m), "n": _expr(n), "k": _expr(k), "lda": _expr(lda), "ldb": _expr(ldb), "ldc": _expr(ldc)},
            [self._operand("__A", A), self._operand("__B", B), self._operand("__C", C), scalar("__alpha", alpha), scalar("__beta", beta)],
            [self._operand("__C", C)])

    def add_matmul(self, A: str, B: str, Y: str, shape_a: Sequence[Any], shape_b: Sequence[Any]) -> None:
        """ml::MatMul, [..., M, K] @ [..., K, N] on contiguous operands."""
        self._add_block({"code": "ml::MatMul", "implementation_type": "NONE", "side_effect": False,
                         "shape_a": [_expr(s) for s in shape_a], "shape_b": [_expr(s) for s in shape_b],
                         "element_type": self._element(A).value},
                        [self._operand("A", A), self._operand("B", B)], [self._operand("Y", Y)])

    #: reduce node codes (reference .../tensor/reduce_ops/*.h); "std" is not part of the rocm target
    REDUCE_CODES = {"sum": "ml::Sum", "max": "ml::Max", "min": "ml::Min", "mean": "ml::Mean"}

    def add_reduce_op(self, op: str, X: str, Y: str, shape: Sequence[Any], axes: Sequence[int], keepdims: bool = False) -> None:
        """Reduce node "X" -> "Y" over `axes` of an input of `shape` (reference add_reduce_op,
        python/bindings/builder/py_structured_sdfg_builder.cpp:1041-1088: sum, max, min, mean, std, softmax)."""
        if op in self.REDUCE_CODES:
            self._add_block({"code": self.REDUCE_CODES[op], "implementation_type": "NONE", "side_effect": False,
                             "shape": [_expr(s) for s in shape], "axes": [int(a) for a in axes], "keepdims": bool(keepdims),
                             "element_type": self._element(X).value},
                            [self._operand("X", X)], [self._operand("Y", Y)])
            return
        if op == "std":
            self._add_std(X, Y, shape, axes, keepdims)
            return
        if op != "softmax":
            raise NotImplementedError(f"reduce op '{op}' is not part of the rocm target")
        if keepdims:
            raise InvalidSDFGException("Unsupported attribute on library node: softmax")
        self._add_block({"code": "ml::Softmax", "implementation_type": "NONE", "side_effect": False,
                         "shape": [_expr(s) for s in shape], "axes": [int(a) for a in axes], "keepdims": False,
                         "element_type": self._element(X).value},
                        [self._operand("X", X)], [self._operand("Y", Y)])

    def _add_std(self, X: str, Y: str, shape: Sequence[Any], axes: Sequence[int], keepdims: bool) -> None:
        """The node chain StdNode::expand leaves behind (reference .../reduce_ops/std_node.cpp: X*X, Mean of it,
        Mean(X), its square, their difference, Sqrt), built directly: the population standard deviation
        sqrt(mean(x^2) - mean(x)^2) with the reference's rounding at every step; temporaries are transients."""
        elem = self._element(X)
        rank = len(shape)
        norm = sorted({int(a) % rank for a in axes})
        out_shape = [("1" if d in norm else _expr(s)) for d, s in enumerate(shape) if keepdims or d not in norm] or ["1"]
        size = {PrimitiveType.Float: 4, PrimitiveType.Double: 8}.get(elem)
        if size is None:
            raise InvalidSDFGException("ml::Std: element type must be Float or Double")

        def temp(dims):
            nbytes = str(size)
            for d in dims:
                nbytes = f"({_expr(d)})*{nbytes}"
            name = self.find_new_name("_std_tmp_")
            self.add_container(name, Pointer(Scalar(elem)), False, transient_bytes=nbytes)
            return name

        x2, mean_x2, mean_x = temp(shape), temp(out_shape), temp(out_shape)
        self.add_elementwise_op("mul", X, X, x2, shape)
        self.add_reduce_op("mean", x2, mean_x2, shape, axes, keepdims)
        self.add_reduce_op("mean", X, mean_x, shape, axes, keepdims)
        self.add_elementwise_op("mul", mean_x, mean_x, mean_x, out_shape)
        self.add_elementwise_op("sub", mean_x2, mean_x, mean_x2, out_shape)
        self.add_elementwise_unary_op("sqrt", mean_x2, Y, out_shape)

    def add_conv(self, X: str, W: str, Y: str, shape: Sequence[Any], kernel_shape: Sequence[Any], strides: Sequence[Any],
                 pads: Sequence[Any], dilations: Sequence[Any], output_channels: Any, group: Any = 1, B: Optional[str] = None) -> None:
        """ml::Conv (ONNX semantics, zero padding); `pads` holds begins then ends."""
        inputs = [self._operand("X", X), self._operand("W", W)]
        if B is not None:
            inputs.append(self._operand("B", B))
        self._add_block({"code": "ml::Conv", "implementation_type": "NONE", "side_effect": False,
                         "shape": [_expr(s) for s in shape], "kernel_shape": [_expr(s) for s in kernel_shape],
                         "strides": [_expr(s) for s in strides], "pads": [_expr(s) for s in pads],
                         "dilations": [_expr(s) for s in dilations], "output_channels": _expr(output_channels),
                         "group": _expr(group), "has_bias": B is not None, "element_type": self._element(X).value},
                        inputs, [self._operand("Y", Y)])

    def add_map_nest(self, loops: Sequence[Tuple[str, Any]], reads: Sequence[Tuple[str, str, Sequence[Any]]],
                     statements: Sequence[Tuple[str, str, Sequence[Any]]], writes: Sequence[Tuple[str, Sequence[Any], str]],
                     scalars: Sequence[Tuple[str, Any]] = ()) -> None:
        """A perfect nest of maps with a body of tasklets, run as one generated kernel (node code ROCMMap). The reference's
        builder spells such a nest with begin_map / add_block / add_tasklet / add_memlet calls
        (python/bindings/builder/py_structured_sdfg_builder.cpp); the block list has no nested scopes, so the nest is
        given whole:
          loops      [(induction variable, bound)], outermost first; every loop runs from 0 in steps of 1
          reads      [(name, container, strides)]: `name` = container[sum(stride_l * variable_l)], loaded once per iteration
          scalars    [(name, scalar container or number)]
          statements [(name, operation, arguments)]: a tasklet code (assign, fp_neg, fp_add, fp_sub, fp_mul, fp_div,
                     fp_rem, fp_fma) or a libm function stem (exp, tanh, fmax, pow, ...) applied to names defined
                     before it or to numbers; every statement rounds by itself, in the element type of the first write
          writes     [(container, strides, name)]
        Iterations must be independent: no iteration may read or write an element another one writes."""
        elem = self._element(writes[0][0])
        literal = lambda v: "#" + (repr(float(v)) + ("f" if elem == PrimitiveType.Float else ""))
        names: Dict[str, str] = {}
        depth = len(loops)

        def access(connector: str, container: str, strides: Sequence[Any]) -> Dict[str, Any]:
            if len(strides) != depth:
                raise InvalidSDFGException(f"map nest: '{container}' needs one stride per loop")
            st = [_expr(x) for x in strides]
            extent = " + ".join(["1"] + [f"(({_expr(b)}) - 1)*({x})" for (_, b), x in zip(loops, st) if x != "0"])
            return {"connector": connector, "strides": st, "extent": extent, "element_type": self._element(container).value}

        node_reads, node_scalars, node_statements, node_writes, inputs, outputs = [], [], [], [], [], []
        for k, (name, container, strides) in enumerate(reads):
            names[name] = f"_in{k}"
            node_reads.append(access(names[name], container, strides))
            inputs.append(self._operand(names[name], container))
        for k, (name, value) in enumerate(scalars):
            names[name] = f"_c{k}"
            is_container = isinstance(value, str) and value in self._data["containers"]
            node_scalars.append({"connector": names[name], "element_type": (self._element(value) if is_container else elem).value})
            inputs.append(self._operand(names[name], value) if is_container else self._operand(names[name], value, elem))
        resolve = lambda a: names[a] if isinstance(a, str) and a in names else literal(a) if isinstance(a, (int, float)) else str(a)
        for k, (name, op, args) in enumerate(statements):
            node_statements.append({"out": f"_v{k}", "type": elem.value, "op": op, "args": [resolve(a) for a in args]})
            names[name] = f"_v{k}"
        for k, (container, strides, value) in enumerate(writes):
            w = access(f"_out{k}", container, strides)
            w["value"] = resolve(value)
            node_writes.append(w)
            outputs.append(self._operand(f"_out{k}", container))
        words = set()
        for text in [_expr(b) for _, b in loops] + [x for a in node_reads + node_writes for x in a["strides"]]:
            words.update(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", text))
        symbols = sorted(w for w in words if w in self._data["containers"] and self._data["containers"][w]["type"] == "scalar")
        self._add_block({"code": "ROCMMap", "implementation_type": "NONE", "side_effect": False,
                         "indvars": [v for v, _ in loops], "bounds": [_expr(b) for _, b in loops], "symbols": symbols,
                         "reads": node_reads, "writes": node_writes, "scalars": node_scalars, "statements": node_statements},
                        inputs, outputs)

    #: elementwise tensor node codes (reference .../tensor/elementwise_ops/*.h)
    UNARY_CODES = {"abs": "ml::Abs", "exp": "ml::Exp", "relu": "ml::ReLU", "sigmoid": "ml::Sigmoid", "sqrt": "ml::Sqrt",
                   "tanh": "ml::Tanh", "erf": "ml::Erf"}
    BINARY_CODES = {"add": "ml::Add", "sub": "ml::Sub", "mul": "ml::Mul", "div": "ml::Div", "max": "ml::Maximum",
                    "min": "ml::Minimum", "maximum": "ml::Maximum", "minimum": "ml::Minimum", "pow": "ml::Pow"}

    def add_elementwise_op(self, op: str, A: str, B: str, C: str, shape: Sequence[Any]) -> None:
        """Binary elementwise node "A","B" -> "C" over equally shaped operands (reference add_elementwise_op,
        python/bindings/builder/py_structured_sdfg_builder.cpp:839-908: op names add, sub, mul, div, pow, min, max).
        As there, an operand that names no container is bound as a constant of the result's element type;
        a scalar container is passed by value."""
        if op not in self.BINARY_CODES:
            raise NotImplementedError(f"elementwise op '{op}' is not part of the rocm target")
        elem = self._element(C)

        def bind(connector: str, v: Any) -> Dict[str, Any]:
            return self._operand(connector, v) if v in self._data["containers"] else self._operand(connector, v, elem)

        self._add_block({"code": self.BINARY_CODES[op], "implementation_type": "NONE", "side_effect": False,
                         "shape": [_expr(s) for s in shape], "element_type": elem.value},
                        [bind("A", A), bind("B", B)], [self._operand("C", C)])

    #: unary nodes with scalar operands on "alpha" / "beta" (reference elu_node.cpp, leaky_relu_node.cpp, hard_sigmoid_node.cpp)
    ACTIVATION_CODES = {"elu": "ml::Elu", "leaky_relu": "ml::LeakyReLU", "hard_sigmoid": "ml::HardSigmoid"}

    def add_elementwise_unary_op(self, op: str, X: str, Y: str, shape: Sequence[Any], alpha: Any = None, beta: Any = None) -> None:
        """Unary elementwise node "X" -> "Y" (reference add_elementwise_unary_op, same file :910-952). For elu,
        leaky_relu and hard_sigmoid `alpha` / `beta` (a number or the name of a scalar container) are bound to the
        connectors of those names; left out, the operator's default applies (1, 0.01, 0.2 / 0.5)."""
        if op in self.ACTIVATION_CODES:
            elem = self._element(X)
            inputs = [self._operand("X", X)]
            for connector, v in (("alpha", alpha), ("beta", beta if op == "hard_sigmoid" else None)):
                if v is not None:
                    inputs.append(self._operand(connector, v) if v in self._data["containers"] else self._operand(connector, repr(float(v)), elem))
            self._add_block({"code": self.ACTIVATION_CODES[op], "implementation_type": "NONE", "side_effect": False,
                             "shape": [_expr(s) for s in shape], "element_type": elem.value}, inputs, [self._operand("Y", Y)])
            return
        if op not in self.UNARY_CODES:
            raise NotImplementedError(f"elementwise op '{op}' is not part of the rocm target")
        self._add_block({"code": self.UNARY_CODES[op], "implementation_type": "NONE", "side_effect": False,
                         "shape": [_expr(s) for s in shape], "element_type": self._element(X).value},
                        [self._operand("X", X)], [self._operand("Y", Y)])

    def add_fill(self, value: Any, Y: str, shape: Sequence[Any]) -> None:
        """ml::Fill: every element of Y becomes `value`, a number or the name of a scalar container (reference
        fill_node.cpp:17-41; the torch path creates it for linalg.fill, LinalgToSDFGTranslator.cpp:456-500)."""
        elem = self._element(Y)
        x = self._operand("X", value) if value in self._data["containers"] else self._operand("X", repr(value), elem)
        self._add_block({"code": "ml::Fill", "implementation_type": "NONE", "side_effect": False, "shape": [_expr(s) for s in shape],
                         "element_type": elem.value}, [x], [self._operand("Y", Y)])

    def add_dot(self, X: str, Y: str, result: str, n: Any, incx: Any = 1, incy: Any = 1) -> None:
        """DOT::BLAS: result = sum_i X[i * incx] * Y[i * incy] with `result` a scalar container whose type sets the
        precision (reference add_dot, python/bindings/builder/py_structured_sdfg_builder.cpp:776-840)."""
        elem = self._element(result)
        if elem not in (PrimitiveType.Float, PrimitiveType.Double):
            raise InvalidSDFGException("DOT: the result must be a Float or Double scalar")
        self._add_block({"code": "DOT", "implementation_type": "BLAS", "side_effect": False,
                         "precision": ord("s") if elem == PrimitiveType.Float else ord("d"), "n": _expr(n), "incx": _expr(incx), "incy": _expr(incy)},
                        [self._operand("__x", X), self._operand("__y", Y)], [self._operand("__out", result)])

    def add_broadcast(self, X: str, Y: str, input_shape: Sequence[Any], output_shape: Sequence[Any]) -> None:
        """ml::Broadcast (reference .../tensor/broadcast_node.h): equal ranks, extent-1 dimensions repeat."""
        if len(input_shape) != len(output_shape):
            raise InvalidSDFGException("ml::Broadcast: input and output ranks differ")
        self._add_block({"code": "ml::Broadcast", "implementation_type": "NONE", "side_effect": False,
                         "input_shape": [_expr(s) for s in input_shape], "output_shape": [_expr(s) for s in output_shape],
                         "element_type": self._element(X).value},
                        [self._operand("X", X)], [self._operand("Y", Y)])

    def add_cast_op(self, X: str, Y: str, shape: Sequence[Any]) -> None:
        """ml::Cast "X" -> "Y": Y[i] = (type of Y) X[i] (reference add_cast_op,
        python/bindings/builder/py_structured_sdfg_builder.cpp:1015-1038; the target type is that of Y's container)."""
        self._add_block({"code": "ml::Cast", "implementation_type": "NONE", "side_effect": False, "shape": [_expr(s) for s in shape],
                         "target_type": self._element(Y).value, "element_type": self._element(X).value},
                        [self._operand("X", X)], [self._operand("Y", Y)])

    def add_transpose(self, X: str, Y: str, shape: Sequence[Any], perm: Optional[Sequence[int]] = None) -> None:
        """ml::Transpose (reference .../tensor/transpose_node.h): Y.shape[i] = shape[perm[i]]; no perm reverses the axes."""
        rank = len(shape)
        perm = [int(p) % rank if rank else int(p) for p in perm] if perm is not None else list(range(rank))[::-1]
        if sorted(perm) != list(range(rank)):
            raise InvalidSDFGException("ml::Transpose: perm is not a permutation of the axes")
        self._add_block({"code": "ml::Transpose", "implementation_type": "NONE", "side_effect": False,
                         "shape": [_expr(s) for s in shape], "perm": perm, "element_type": self._element(X).value},
                        [self._operand("X", X)], [self._operand("Y", Y)])

    def add_attention(self, Q: str, K: str, V: str, O: str, shape_q: Sequence[Any], seq_kv: Any, scale: Any, causal: bool = False) -> None:
        """ml::Attention: O = softmax(scale * Q K^T) V, Q [B,H,SQ,D], K/V [B,H,SKV,D]; `causal`: query i attends to the
        keys j <= i."""
        block = {"code": "ml::Attention", "implementation_type": "NONE", "side_effect": False,
                 "shape_q": [_expr(s) for s in shape_q], "seq_kv": _expr(seq_kv), "scale": repr(float(scale)),
                 "element_type": self._element(Q).value, "output_type": self._element(O).value}
        if causal:
            block["causal"] = True
        self._add_block(block, [self._operand("Q", Q), self._operand("K", K), self._operand("V", V)], [self._operand("O", O)])

    def add_return(self, container: str) -> None:
        self._data["return"] = container

    def add_metadata(self, key: str, value: str) -> None:
        self._data["metadata"][key] = str(value)

    def move(self) -> StructuredSDFG:
        sdfg = StructuredSDFG(self._data)
        sdfg.validate()
        return sdfg
