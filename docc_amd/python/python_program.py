"""`@native`: JIT-compiles a Python function whose body is made of the math library-node
operations (matrix products, softmax, convolution) for the `rocm` target.

Drop-in for the reference's decorator on this path (python/docc/python/python_program.py:103-339,
713-747): same decorator forms (`@native`, `@native(target=..., category=...)`), same `compile` /
`__call__` / `to_sdfg` surface, the same cache rule (one compilation per dtype and shape
*structure*: equal dimensions share a `_s<i>` symbol, :216-264), the same argument order of the
generated function (user parameters, then `_s<i>` int64 symbols, then `_docc_ret_<i>` outputs,
:594-653) and the same pipeline order validate -> expand -> simplify -> normalize -> dump ->
schedule -> compile with the target-registry hooks consulted first (:273-314).

The reference parses arbitrary numpy programs into loop nests; this front end recognises the
statements that lower to the target's library nodes and rejects everything else with
NotImplementedError (there is no CPU lowering behind it):

    A @ B, np.matmul(A, B), np.dot(A, B), A.T / np.transpose(A) as an operand, scalar * (A @ B)
    C[:] = alpha * A @ B + beta * C          (GEMM with alpha/beta, in place)
    C = A @ B, C[:] = ..., C += A @ B        (C an argument: written in place)
    scipy.special.softmax(x, axis=-1), softmax(x, axis=-1)
    the decomposed form  m = np.max(x, axis=-1, keepdims=True); e = np.exp(x - m);
                         s = np.sum(e, axis=-1, keepdims=True); e / s
    conv2d(x, w, bias, stride=, padding=, dilation=)
    x + y, x - y, x * y, x / y, x ** y, np.maximum(x, y), np.minimum(x, y) on float arrays whose shapes
        broadcast by numpy's rules (the smaller operand goes through ml::Broadcast), or on an
        array and a scalar (literal or scalar argument)
    np.abs, np.exp, np.sqrt, np.tanh, scipy.special.erf / expit, relu(x), sigmoid(x),
        np.maximum(x, 0)  (ReLU)
    np.sum / np.max / np.min / np.mean (and the array methods) over one axis or a block of
        axes, with keepdims
"""
from __future__ import annotations

import ast
import getpass
import hashlib
import inspect
import os
import shutil
import textwrap
import warnings
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np

from docc_amd.compiler import CompiledSDFG, DoccProgram
from docc_amd.python import functions as _functions
from docc_amd.python.target_registry import get_target_compile_fn, get_target_schedule_fn
from docc_amd.sdfg import Pointer, PrimitiveType, Scalar, StructuredSDFG, StructuredSDFGBuilder

_DTYPES = {np.dtype(np.float64): PrimitiveType.Double, np.dtype(np.float32): PrimitiveType.Float,
           np.dtype(np.int64): PrimitiveType.Int64, np.dtype(np.int32): PrimitiveType.Int32}
_SIZES = {PrimitiveType.Double: 8, PrimitiveType.Float: 4}


class bfloat16:
    """Names the bf16 element type in a parameter annotation: `Annotated[np.ndarray, (m, k), bfloat16]` or
    `np.ndarray[Any, np.dtype[bfloat16]]` on a parameter whose arrays arrive as `np.uint16` (the raw 16-bit words, which
    is how bf16 crosses the ctypes boundary: reference compiled_sdfg.py:28-31). The reference recognises
    `ml_dtypes.bfloat16` arrays (python_program.py:432-433); such arrays are taken here too where that package exists.
    Products of bf16 operands accumulate and return float32 (GEMM precision `b`)."""


def _is_ml_bfloat16(dtype) -> bool:
    return getattr(dtype, "name", "") == "bfloat16" and getattr(dtype, "itemsize", 0) == 2


def _map_python_type(value: Any):
    """Python/numpy value -> SDFG type (reference python_program.py:401-464)."""
    if isinstance(value, np.ndarray):
        if _is_ml_bfloat16(value.dtype):
            return Pointer(Scalar(PrimitiveType.BFloat))
        if value.dtype not in _DTYPES:
            raise TypeError(f"unsupported array dtype {value.dtype}")
        return Pointer(Scalar(_DTYPES[value.dtype]))
    if isinstance(value, (bool, np.bool_)):
        return Scalar(PrimitiveType.Bool)
    if isinstance(value, (int, np.integer)):
        return Scalar(PrimitiveType.Int64)
    if isinstance(value, (float, np.floating)):
        return Scalar(PrimitiveType.Float if isinstance(value, np.float32) else PrimitiveType.Double)
    raise TypeError(f"unsupported argument type {type(value).__name__}")


def _map_annotation(ann: Any):
    """One return annotation -> SDFG type, or None if it names nothing this front end can declare ahead of the body
    (reference python_program.py:40-100: Annotated[np.ndarray, shape, dtype], np.ndarray[shape, dtype], float, int, ...)."""
    import typing

    if typing.get_origin(ann) is typing.Annotated:
        base, *meta = typing.get_args(ann)
        if base is np.ndarray:
            elem = _map_annotation(meta[1]) if len(meta) > 1 else Scalar(PrimitiveType.Double)
            return Pointer(elem) if isinstance(elem, Scalar) else None
        return None
    if typing.get_origin(ann) is np.ndarray:
        args = typing.get_args(ann)
        if len(args) >= 2:
            dt = args[1]
            inner = typing.get_args(dt)
            elem = _map_annotation(inner[0] if typing.get_origin(dt) is np.dtype and inner else dt)
            return Pointer(elem) if isinstance(elem, Scalar) else None
        return None
    if ann is bfloat16 or _is_ml_bfloat16(ann) or getattr(ann, "__name__", "") == "bfloat16":
        return Scalar(PrimitiveType.BFloat)
    table = {float: PrimitiveType.Double, np.float64: PrimitiveType.Double, np.float32: PrimitiveType.Float, bool: PrimitiveType.Bool,
             np.bool_: PrimitiveType.Bool, int: PrimitiveType.Int64, np.int64: PrimitiveType.Int64, np.int32: PrimitiveType.Int32}
    try:
        return Scalar(table[ann]) if ann in table else None
    except TypeError:   # unhashable annotation
        return None


def _return_annotation_types(func) -> Optional[List[Any]]:
    """The types a return annotation declares (a tuple annotation: one per element), or None: no annotation, or one that
    does not map - the outputs are then inferred from the body (reference python_program.py:478-512)."""
    import typing

    ann = inspect.signature(func).return_annotation
    if ann is inspect.Signature.empty or isinstance(ann, str):
        return None
    if typing.get_origin(ann) is tuple:
        items = [a for a in typing.get_args(ann) if a is not Ellipsis]
    else:
        items = [ann]
    types = [_map_annotation(a) for a in items]
    return None if any(t is None for t in types) else types


def _mul(a: str, b: str) -> str:
    if a == "1":
        return b
    if b == "1":
        return a
    if a.isdigit() and b.isdigit():
        return str(int(a) * int(b))
    return f"{a}*{b}"


class _Array:
    """An array value during lowering: a container plus its symbolic shape."""

    def __init__(self, name: str, shape: Sequence[str], elem: PrimitiveType):
        self.name, self.shape, self.elem = name, list(shape), elem


class _Lazy:
    """A value that only exists as part of a larger pattern (scaled or transposed operands, the
    pieces of the decomposed softmax)."""

    def __init__(self, kind: str, base: Any, scalar: Any = None, src: Any = None):
        self.kind, self.base, self.scalar = kind, base, scalar
        self.src = src          # the pattern piece this one was built from
        self.array = None       # set once the value had to exist on its own


class _ScalarValue:
    def __init__(self, text: str):
        self.text = text  # literal or scalar container name


class _Lowering(ast.NodeVisitor):
    def __init__(self, func, builder: StructuredSDFGBuilder, env: Dict[str, Any], arg_names: List[str]):
        self.func = func
        self.b = builder
        self.env = env
        self.arg_names = arg_names
        self.outputs: List[str] = []
        self.output_shapes: Dict[str, List[str]] = {}
        self.globals = dict(func.__globals__)
        if func.__closure__:
            for name, cell in zip(func.__code__.co_freevars, func.__closure__):
                try:
                    self.globals[name] = cell.cell_contents
                except ValueError:
                    pass

    # ---- helpers ---------------------------------------------------------------
    def fail(self, node: ast.AST, what: str):
        raise NotImplementedError(f"{self.func.__name__}, line {getattr(node, 'lineno', '?')}: {what} "
                                  "cannot be lowered to the rocm target's library nodes")

    def resolve(self, node: ast.AST) -> Any:
        """AST of a callee -> the Python object it names, or None."""
        if isinstance(node, ast.Name):
            return self.globals.get(node.id, getattr(__import__("builtins"), node.id, None))
        if isinstance(node, ast.Attribute):
            base = self.resolve(node.value)
            return getattr(base, node.attr, None) if base is not None else None
        return None

    def new_array(self, shape: Sequence[str], elem: PrimitiveType, dest: Optional[str]) -> _Array:
        if dest is not None:
            if not self.b.exists(dest):  # a `_docc_ret_<i>` output: becomes a trailing pointer argument
                self.b.add_container(dest, Pointer(Scalar(elem)), True)
            elif self.b._data["containers"][dest]["element"] != elem.value:   # declared by the return annotation
                raise TypeError(f"{self.func.__name__}: the return annotation declares {self.b._data['containers'][dest]['element']} "
                                f"for output {dest}, the returned value is {elem.value}")
            return _Array(dest, shape, elem)
        size = str(_SIZES[elem])
        for s in shape:
            size = _mul(s, size)
        name = self.b.find_new_name("_tmp_")
        self.b.add_container(name, Pointer(Scalar(elem)), False, transient_bytes=size)
        return _Array(name, shape, elem)

    def new_output(self, shape: Sequence[str], elem: PrimitiveType) -> str:
        name = f"_docc_ret_{len(self.outputs)}"
        self.outputs.append(name)
        self.output_shapes[name] = list(shape)
        return name

    def const(self, node: ast.AST) -> Optional[float]:
        if isinstance(node, ast.Constant) and isinstance(node.value, (int, float)) and not isinstance(node.value, bool):
            return float(node.value)
        if isinstance(node, ast.UnaryOp) and isinstance(node.op, ast.USub):
            v = self.const(node.operand)
            return -v if v is not None else None
        return None

    def scalar_of(self, node: ast.AST) -> Optional[_ScalarValue]:
        c = self.const(node)
        if c is not None:
            return _ScalarValue(repr(c))
        if isinstance(node, ast.Name) and isinstance(self.env.get(node.id), _ScalarValue):
            return self.env[node.id]
        return None

    def kw(self, call: ast.Call, name: str, position: Optional[int], default: Any) -> Any:
        for k in call.keywords:
            if k.arg == name:
                return ast.literal_eval(k.value)
        if position is not None and len(call.args) > position:
            return ast.literal_eval(call.args[position])
        return default

    # ---- operations --------------------------------------------------------------
    def matmul(self, node: ast.AST, left: Any, right: Any, dest: Optional[str], alpha: str = "1.0", beta: str = "0.0") -> _Array:
        ta = tb = False
        if isinstance(left, _Lazy) and left.kind == "scaled":
            if alpha != "1.0":
                self.fail(node, "two scalar factors on one product")
            alpha, left = left.scalar.text, left.base
        if isinstance(left, _Lazy) and left.kind == "transposed":
            ta, left = True, left.base
        if isinstance(right, _Lazy) and right.kind == "transposed":
            tb, right = True, right.base
        left, right = self.array_of(node, left), self.array_of(node, right)
        if not isinstance(left, _Array) or not isinstance(right, _Array):
            self.fail(node, "a matrix product of non-array operands")
        if left.elem != right.elem:
            self.fail(node, "a matrix product of mixed element types")
        # bf16 operands: the products are accumulated and returned in float32 (GEMM precision `b`, ml::MatMul on BFloat)
        out_elem = PrimitiveType.Float if left.elem == PrimitiveType.BFloat else left.elem
        if len(left.shape) == 2 and len(right.shape) == 2:
            m, k = (left.shape[1], left.shape[0]) if ta else left.shape
            k2, n = (right.shape[1], right.shape[0]) if tb else right.shape
            if k != k2:
                raise ValueError(f"{self.func.__name__}: matmul inner dimensions differ ({k} vs {k2})")
            out = self.new_array([m, n], out_elem, dest)
            self.b.add_gemm(left.name, right.name, out.name, alpha, beta, m, n, k, ta, tb, left.shape[1], right.shape[1], n)
            return out
        # vectors, numpy's rules: matrix @ vector and vector @ matrix are GEMMs with one column / one row, the result
        # loses that axis; vector @ vector is the sum of the products
        if len(left.shape) == 2 and len(right.shape) == 1 and not tb:
            m, k = (left.shape[1], left.shape[0]) if ta else left.shape
            if k != right.shape[0]:
                raise ValueError(f"{self.func.__name__}: matmul inner dimensions differ ({k} vs {right.shape[0]})")
            out = self.new_array([m], out_elem, dest)
            self.b.add_gemm(left.name, right.name, out.name, alpha, beta, m, "1", k, ta, False, left.shape[1], "1", "1")
            return out
        if len(left.shape) == 1 and len(right.shape) == 2 and not ta:
            k2, n = (right.shape[1], right.shape[0]) if tb else right.shape
            if left.shape[0] != k2:
                raise ValueError(f"{self.func.__name__}: matmul inner dimensions differ ({left.shape[0]} vs {k2})")
            out = self.new_array([n], out_elem, dest)
            self.b.add_gemm(left.name, right.name, out.name, alpha, beta, "1", n, left.shape[0], False, tb, left.shape[0], right.shape[1], n)
            return out
        if len(left.shape) == 1 and len(right.shape) == 1 and left.elem == PrimitiveType.BFloat:
            self.fail(node, "the inner product of two bf16 vectors")
        if len(left.shape) == 1 and len(right.shape) == 1 and not (ta or tb) and alpha == "1.0" and beta == "0.0":
            if left.shape[0] != right.shape[0]:
                raise ValueError(f"{self.func.__name__}: matmul inner dimensions differ ({left.shape[0]} vs {right.shape[0]})")
            return self.reduce(node, "sum", self.elementwise(node, "mul", left, right, None), None, False, dest)
        if ta or tb or alpha != "1.0" or beta != "0.0":
            self.fail(node, "a scaled or transposed batched product")
        if len(left.shape) < 2 or len(right.shape) < 2 or (len(right.shape) > 2 and right.shape[:-2] != left.shape[:-2]):
            self.fail(node, "this broadcast in a batched product")
        if left.shape[-1] != right.shape[-2]:
            raise ValueError(f"{self.func.__name__}: matmul inner dimensions differ")
        out = self.new_array(left.shape[:-1] + [right.shape[-1]], out_elem, dest)
        self.b.add_matmul(left.name, right.name, out.name, left.shape, right.shape)
        return out

    def softmax(self, node: ast.AST, x: Any, axis: Any, dest: Optional[str]) -> _Array:
        """`axis`: an int, a tuple of ints, or None for all axes (scipy's default)."""
        if not isinstance(x, _Array):
            self.fail(node, "softmax of a non-array")
        rank = len(x.shape)
        axes = list(range(rank)) if axis is None else [axis] if isinstance(axis, int) else list(axis)
        if not axes or any(not isinstance(a, int) or a < -rank or a >= rank for a in axes):
            self.fail(node, "softmax axis out of range")
        normal = sorted({a % rank for a in axes})
        if normal[-1] - normal[0] + 1 != len(normal):
            self.fail(node, "softmax over axes that are not adjacent")
        if x.elem not in (PrimitiveType.Float, PrimitiveType.Double):
            self.fail(node, "softmax of an array that is neither float32 nor float64")
        out = self.new_array(x.shape, x.elem, dest)
        self.b.add_reduce_op("softmax", x.name, out.name, x.shape, axes)
        return out

    def conv(self, node: ast.Call, dest: Optional[str]) -> _Array:
        if len(node.args) < 2:
            self.fail(node, "conv2d without input and weight")
        x, w = self.ev(node.args[0]), self.ev(node.args[1])
        bias = None
        bias_node = node.args[2] if len(node.args) > 2 else next((k.value for k in node.keywords if k.arg == "bias"), None)
        if bias_node is not None and not (isinstance(bias_node, ast.Constant) and bias_node.value is None):
            bias = self.ev(bias_node)
        pair = lambda v: (v, v) if isinstance(v, int) else tuple(v)
        stride, pad, dil = (pair(self.kw(node, n, p, d)) for n, p, d in (("stride", 3, 1), ("padding", 4, 0), ("dilation", 5, 1)))
        if not (isinstance(x, _Array) and isinstance(w, _Array) and len(x.shape) == 4 and len(w.shape) == 4):
            self.fail(node, "conv2d on operands that are not 4-d arrays")
        dims = []
        for i in range(2):
            d, k = x.shape[2 + i], w.shape[2 + i]
            if d.isdigit() and k.isdigit():
                dims.append(str((int(d) + 2 * pad[i] - dil[i] * (int(k) - 1) - 1) // stride[i] + 1))
            else:
                dims.append(f"(({d} + {2 * pad[i]} - ({dil[i]}*({k} - 1) + 1)) // {stride[i]} + 1)")
        out_shape = [x.shape[0], w.shape[0]] + dims
        out = self.new_array(out_shape, x.elem, dest)  # `//`: these expressions are evaluated in Python only
        self.b.add_conv(x.name, w.name, out.name, x.shape, w.shape[2:], list(stride), [pad[0], pad[1], pad[0], pad[1]], list(dil),
                        w.shape[0], 1, bias.name if bias is not None else None)
        return out

    def broadcast_shape(self, node: ast.AST, a: Sequence[str], b: Sequence[str]) -> List[str]:
        rank = max(len(a), len(b))
        a, b = ["1"] * (rank - len(a)) + list(a), ["1"] * (rank - len(b)) + list(b)
        out = []
        for x, y in zip(a, b):
            if x != y and x != "1" and y != "1":
                raise ValueError(f"{self.func.__name__}: operands could not be broadcast together ({a} vs {b})")
            out.append(y if x == "1" else x)
        return out

    def expanded(self, x: _Array, shape: List[str]) -> _Array:
        """`x` repeated to `shape` through ml::Broadcast (a no-op when the shapes agree)."""
        if x.shape == shape:
            return x
        padded = ["1"] * (len(shape) - len(x.shape)) + x.shape
        if len(shape) > 6:
            raise NotImplementedError(f"{self.func.__name__}: broadcast of rank {len(shape)} (up to 6 are built)")
        out = self.new_array(shape, x.elem, None)
        self.b.add_broadcast(x.name, out.name, padded, shape)
        return out

    def array_of(self, node: ast.AST, v: Any, dest: Optional[str] = None) -> Any:
        """A pattern piece that turns out to be used on its own becomes the node(s) it stands for;
        other values pass through."""
        if not isinstance(v, _Lazy):
            return v
        if v.array is not None:
            return v.array
        if v.kind == "transposed":   # of a matrix, and not an operand of a product: the ml::Transpose node
            arr = self.transpose(node, v.base, None, dest)
        elif v.kind == "scaled":
            arr = self.elementwise(node, "mul", v.base, v.scalar, dest)
        elif v.kind == "max_keep":
            arr = self.reduce(node, "max", v.base, -1, True, dest)
        elif v.kind == "sub_max":
            arr = self.elementwise(node, "sub", v.base, self.array_of(node, v.src), dest)
        elif v.kind == "exp_sub":
            arr = self.unary(node, "exp", self.array_of(node, v.src), dest)
        elif v.kind == "sum_keep":
            arr = self.reduce(node, "sum", self.array_of(node, v.src), -1, True, dest)
        else:
            return v
        v.array = arr
        return arr

    def transpose(self, node: ast.AST, x: Any, axes: Any, dest: Optional[str]) -> _Array:
        """np.transpose(x, axes): ml::Transpose; `axes` None reverses the axes."""
        x = self.array_of(node, x)
        if not isinstance(x, _Array) or x.elem not in _SIZES:
            self.fail(node, "transposing a value that is not a float array")
        rank = len(x.shape)
        perm = list(range(rank))[::-1] if axes is None else [int(a) % rank for a in axes]
        if sorted(perm) != list(range(rank)):
            raise ValueError(f"{self.func.__name__}: axes don't match array")
        if rank > 6:
            raise NotImplementedError(f"{self.func.__name__}: transpose of rank {rank} (up to 6 are built)")
        out = self.new_array([x.shape[p] for p in perm], x.elem, dest)
        self.b.add_transpose(x.name, out.name, x.shape, perm)
        return out

    def reduce(self, node: ast.AST, op: str, x: Any, axis: Any, keepdims: bool, dest: Optional[str]) -> _Array:
        x = self.array_of(node, x)
        if not isinstance(x, _Array) or x.elem not in _SIZES:
            self.fail(node, f"'{op}' reduction of a value that is not a float array")
        rank = len(x.shape)
        axes = list(range(rank)) if axis is None else ([axis] if isinstance(axis, int) else list(axis))
        if any(not isinstance(a, int) or a < -rank or a >= rank for a in axes):
            raise ValueError(f"{self.func.__name__}: axis {axis} is out of bounds for an array of rank {rank}")
        axes = sorted({a % rank for a in axes})
        shape = [("1" if d in axes else s) for d, s in enumerate(x.shape) if keepdims or d not in axes]
        out = self.new_array(shape, x.elem, dest)
        self.b.add_reduce_op(op, x.name, out.name, x.shape, axes, keepdims)
        return out

    def elementwise(self, node: ast.AST, op: str, a: Any, b: Any, dest: Optional[str]) -> _Array:
        a, b = self.array_of(node, a), self.array_of(node, b)
        arrays = [v for v in (a, b) if isinstance(v, _Array)]
        if not arrays or not all(isinstance(v, (_Array, _ScalarValue)) for v in (a, b)):
            self.fail(node, f"elementwise '{op}' of these operands")
        elem = arrays[0].elem
        if elem not in _SIZES or any(v.elem != elem for v in arrays):
            self.fail(node, f"elementwise '{op}' of non-float or mixed element types")
        if len(arrays) == 1:
            shape = arrays[0].shape
            out = self.new_array(shape, elem, dest)
            self.b.add_elementwise_op(op, a.name if isinstance(a, _Array) else a.text, b.name if isinstance(b, _Array) else b.text,
                                      out.name, shape)
            return out
        shape = self.broadcast_shape(node, a.shape, b.shape)
        a, b = self.expanded(a, shape), self.expanded(b, shape)
        out = self.new_array(shape, elem, dest)
        self.b.add_elementwise_op(op, a.name, b.name, out.name, shape)
        return out

    def unary(self, node: ast.AST, op: str, x: Any, dest: Optional[str]) -> _Array:
        x = self.array_of(node, x)
        if not isinstance(x, _Array) or x.elem not in _SIZES:
            self.fail(node, f"'{op}' of a value that is not a float array")
        out = self.new_array(x.shape, x.elem, dest)
        self.b.add_elementwise_unary_op(op, x.name, out.name, x.shape)
        return out

    def is_product(self, n: ast.AST) -> bool:
        """`A @ B` or `scalar * (A @ B)`, syntactically."""
        if isinstance(n, ast.BinOp) and isinstance(n.op, ast.MatMult):
            return True
        if isinstance(n, ast.BinOp) and isinstance(n.op, ast.Mult):
            return any(self.scalar_of(s) is not None and isinstance(o, ast.BinOp) and isinstance(o.op, ast.MatMult)
                       for s, o in ((n.left, n.right), (n.right, n.left)))
        return False

    def gemm_accumulate(self, node: ast.BinOp, dest: Optional[str]) -> Optional[_Array]:
        """`alpha * A @ B + beta * C` written into C: one GEMM in place. Only when the statement
        names C as its destination; any other sum is an elementwise node."""
        if dest is None:
            return None
        for prod, acc in ((node.left, node.right), (node.right, node.left)):
            if not self.is_product(prod) or self.is_product(acc):
                continue
            beta, cnode = "1.0", acc
            if isinstance(acc, ast.BinOp) and isinstance(acc.op, ast.Mult):
                for sn, on in ((acc.left, acc.right), (acc.right, acc.left)):
                    s = self.scalar_of(sn)
                    if s is not None and isinstance(on, ast.Name):
                        beta, cnode = s.text, on
                        break
            if not (isinstance(cnode, ast.Name) and isinstance(self.env.get(cnode.id), _Array) and self.env[cnode.id].name == dest):
                continue
            alpha, pnode = "1.0", prod
            if isinstance(pnode.op, ast.Mult):
                for sn, on in ((pnode.left, pnode.right), (pnode.right, pnode.left)):
                    s = self.scalar_of(sn)
                    if s is not None and isinstance(on, ast.BinOp) and isinstance(on.op, ast.MatMult):
                        alpha, pnode = s.text, on
                        break
            return self.matmul(node, self.ev(pnode.left), self.ev(pnode.right), dest, alpha=alpha, beta=beta)
        return None

    # ---- expressions -------------------------------------------------------------
    def ev(self, node: ast.AST, dest: Optional[str] = None) -> Any:
        if isinstance(node, ast.Name):
            if node.id not in self.env:
                self.fail(node, f"name '{node.id}'")
            return self.env[node.id]
        s = self.scalar_of(node)
        if s is not None:
            return s
        if isinstance(node, ast.Attribute) and node.attr in ("T", "mT"):
            base = self.ev(node.value)
            if isinstance(base, _Array) and len(base.shape) == 2:
                return _Lazy("transposed", base)   # a GEMM flag when it feeds a product, else a node
            if node.attr == "mT":
                rank = len(base.shape) if isinstance(base, _Array) else 0
                return self.transpose(node, base, list(range(rank - 2)) + [rank - 1, rank - 2] if rank >= 2 else None, dest)
            return self.transpose(node, base, None, dest)
        if isinstance(node, ast.BinOp):
            return self.binop(node, dest)
        if isinstance(node, ast.UnaryOp) and isinstance(node.op, (ast.USub, ast.UAdd)):
            # -x of an array: the product with -1.0, which flips the sign of every value, zeros and NaNs included
            v = self.array_of(node, self.ev(node.operand))
            if not isinstance(v, _Array):
                self.fail(node, "a sign in front of something that is not an array or a literal")
            if isinstance(node.op, ast.UAdd):
                return v
            return self.elementwise(node, "mul", v, _ScalarValue("-1.0"), dest)
        if isinstance(node, ast.Call):
            return self.call(node, dest)
        self.fail(node, f"expression {ast.dump(node)[:60]}")

    def binop(self, node: ast.BinOp, dest: Optional[str]) -> Any:
        if isinstance(node.op, ast.MatMult):
            return self.matmul(node, self.ev(node.left), self.ev(node.right), dest)
        if isinstance(node.op, ast.Mult):
            for scalar_node, other in ((node.left, node.right), (node.right, node.left)):
                s = self.scalar_of(scalar_node)
                if s is None:
                    continue
                if isinstance(other, ast.BinOp) and isinstance(other.op, ast.MatMult):
                    return self.matmul(node, self.ev(other.left), self.ev(other.right), dest, alpha=s.text)
                v = self.ev(other)
                if isinstance(v, _Array):
                    # a factor of a product to come (alpha * A @ B parses as (alpha * A) @ B); it
                    # becomes an ml::Mul node when used as an array instead
                    return _Lazy("scaled", v, s) if dest is None else self.elementwise(node, "mul", v, s, dest)
                self.fail(node, "this multiplication")
            return self.elementwise(node, "mul", self.ev(node.left), self.ev(node.right), dest)
        if isinstance(node.op, ast.Add):
            r = self.gemm_accumulate(node, dest)
            return r if r is not None else self.elementwise(node, "add", self.ev(node.left), self.ev(node.right), dest)
        if isinstance(node.op, ast.Sub):
            x, m = self.ev(node.left), self.ev(node.right)
            if isinstance(x, _Array) and isinstance(m, _Lazy) and m.kind == "max_keep" and m.base.name == x.name:
                return _Lazy("sub_max", x, src=m)
            return self.elementwise(node, "sub", x, m, dest)
        if isinstance(node.op, ast.Div):
            e, s = self.ev(node.left), self.ev(node.right)
            if isinstance(e, _Lazy) and e.kind == "exp_sub" and isinstance(s, _Lazy) and s.kind == "sum_keep" and s.base.name == e.base.name:
                return self.softmax(node, e.base, -1, dest)
            return self.elementwise(node, "div", e, s, dest)
        if isinstance(node.op, ast.Pow):
            return self.elementwise(node, "pow", self.ev(node.left), self.ev(node.right), dest)
        self.fail(node, f"operator {type(node.op).__name__}")

    def call(self, node: ast.Call, dest: Optional[str]) -> Any:
        fn = self.resolve(node.func)
        if isinstance(node.func, ast.Attribute) and node.func.attr == "dot" and fn is None:
            return self.matmul(node, self.ev(node.func.value), self.ev(node.args[0]), dest)
        if fn in (np.matmul, np.dot):
            return self.matmul(node, self.ev(node.args[0]), self.ev(node.args[1]), dest)
        if fn is np.transpose or (fn is None and isinstance(node.func, ast.Attribute) and node.func.attr == "transpose"):
            method = fn is None
            base = self.ev(node.func.value if method else node.args[0])
            rest = node.args if method else node.args[1:]
            axes = self.kw(node, "axes", None, None)
            if rest:
                axes = [ast.literal_eval(a) for a in rest] if len(rest) > 1 else ast.literal_eval(rest[0])
                if isinstance(axes, int):
                    axes = [axes]
            if axes is None and isinstance(base, _Array) and len(base.shape) == 2:
                return _Lazy("transposed", base)
            return self.transpose(node, base, axes, dest)
        if fn is None and isinstance(node.func, ast.Attribute) and node.func.attr == "astype" and node.args:
            base = self.array_of(node, self.ev(node.func.value))
            target = {np.float32: PrimitiveType.Float, np.float64: PrimitiveType.Double}.get(self.resolve(node.args[0]))
            if target is None and isinstance(node.args[0], ast.Constant):
                target = {"float32": PrimitiveType.Float, "float64": PrimitiveType.Double}.get(node.args[0].value)
            if not isinstance(base, _Array) or target is None:
                self.fail(node, "astype to a type other than float32 / float64")
            if base.elem not in (PrimitiveType.Float, PrimitiveType.Double, PrimitiveType.Int32, PrimitiveType.Int64):
                self.fail(node, "astype of an array that is not float32, float64, int32 or int64")
            out = self.new_array(base.shape, target, dest)
            self.b.add_cast_op(base.name, out.name, base.shape)   # the same type copies
            return out
        if fn is np.swapaxes and len(node.args) == 3:
            base = self.array_of(node, self.ev(node.args[0]))
            if not isinstance(base, _Array):
                self.fail(node, "swapaxes of a value that is not an array")
            perm = list(range(len(base.shape)))
            i, j = (ast.literal_eval(a) % len(perm) for a in node.args[1:])
            perm[i], perm[j] = perm[j], perm[i]
            return self.transpose(node, base, perm, dest)
        try:
            import scipy.special as _sp
            scipy_softmax = _sp.softmax
        except Exception:  # scipy is optional
            _sp = scipy_softmax = None
        if fn is not None and fn in (scipy_softmax, _functions.softmax):
            return self.softmax(node, self.ev(node.args[0]), self.kw(node, "axis", 1, -1 if fn is _functions.softmax else None), dest)
        if fn is _functions.conv2d:
            return self.conv(node, dest)
        axis_last = lambda x: self.kw(node, "axis", 1, None) in (-1, len(x.shape) - 1) and self.kw(node, "keepdims", None, False) is True
        if fn in (np.max, np.amax):
            x = self.ev(node.args[0])
            if isinstance(x, _Array) and axis_last(x) and dest is None:
                return _Lazy("max_keep", x)
        if fn is np.exp:
            v = self.ev(node.args[0])
            if isinstance(v, _Lazy) and v.kind == "sub_max":
                return _Lazy("exp_sub", v.base, src=v)
            return self.unary(node, "exp", v, dest)
        unary_fns = {np.abs: "abs", np.absolute: "abs", np.fabs: "abs", np.sqrt: "sqrt", np.tanh: "tanh",
                     _functions.relu: "relu", _functions.sigmoid: "sigmoid", _functions.erf: "erf"}
        if _sp is not None:
            unary_fns.update({_sp.erf: "erf", _sp.expit: "sigmoid"})
        if fn is not None and len(node.args) == 1 and not node.keywords:
            for f, op in unary_fns.items():
                if fn is f:
                    return self.unary(node, op, self.ev(node.args[0]), dest)
        binary_fns = {np.maximum: "max", np.minimum: "min", np.add: "add", np.subtract: "sub", np.multiply: "mul",
                      np.divide: "div", np.true_divide: "div", np.power: "pow"}
        if fn is not None and len(node.args) == 2 and not node.keywords:
            for f, op in binary_fns.items():
                if fn is f:
                    a, b = self.ev(node.args[0]), self.ev(node.args[1])
                    if op == "max":  # np.maximum(x, 0): the ReLU node
                        for x, z in ((a, b), (b, a)):
                            if isinstance(z, _ScalarValue) and z.text in ("0.0", "-0.0") and isinstance(x, (_Array, _Lazy)):
                                return self.unary(node, "relu", x, dest)
                    return self.elementwise(node, op, a, b, dest)
        reductions = {np.sum: "sum", np.max: "max", np.amax: "max", np.min: "min", np.amin: "min", np.mean: "mean", np.std: "std"}
        if (fn is np.std or (fn is None and isinstance(node.func, ast.Attribute) and node.func.attr == "std")) and self.kw(node, "ddof", None, 0) != 0:
            self.fail(node, "a standard deviation with ddof != 0")
        if fn is np.sum:
            v = self.ev(node.args[0])
            if isinstance(v, _Lazy) and v.kind == "exp_sub" and axis_last(v.base):
                return _Lazy("sum_keep", v.base, src=v)
        for f, op in reductions.items():
            if fn is f and node.args:
                return self.reduce(node, op, self.ev(node.args[0]), self.kw(node, "axis", 1, None), bool(self.kw(node, "keepdims", None, False)), dest)
        # the same as methods of an array: x.sum(axis=..), x.max(..), x.min(..), x.mean(..)
        if fn is None and isinstance(node.func, ast.Attribute) and node.func.attr in ("sum", "max", "min", "mean", "std"):
            base = self.ev(node.func.value)
            if isinstance(base, (_Array, _Lazy)):
                return self.reduce(node, node.func.attr, base, self.kw(node, "axis", 0, None), bool(self.kw(node, "keepdims", None, False)), dest)
        self.fail(node, f"call to {ast.unparse(node.func)}")

    # ---- statements --------------------------------------------------------------
    def materialise(self, node: ast.AST, value_node: ast.AST, dest: Optional[str]) -> _Array:
        v = self.array_of(node, self.ev(value_node, dest), dest)
        if not isinstance(v, _Array):
            self.fail(node, "a statement whose value is not an array produced by a library node")
        if dest is not None and v.name != dest:
            self.fail(node, "copying one array into another")
        return v

    def visit_Assign(self, node: ast.Assign):
        if len(node.targets) != 1:
            self.fail(node, "multiple assignment targets")
        t = node.targets[0]
        if isinstance(t, ast.Subscript):
            whole = isinstance(t.slice, ast.Slice) and t.slice.lower is None and t.slice.upper is None and t.slice.step is None
            whole = whole or (isinstance(t.slice, ast.Constant) and t.slice.value is Ellipsis)
            if not (isinstance(t.value, ast.Name) and whole and isinstance(self.env.get(t.value.id), _Array)):
                self.fail(node, "a partial array assignment")
            self.materialise(node, node.value, self.env[t.value.id].name)
            return
        if not isinstance(t, ast.Name):
            self.fail(node, "this assignment target")
        if t.id in self.arg_names and isinstance(self.env.get(t.id), _Array):
            self.materialise(node, node.value, self.env[t.id].name)  # writes into the argument
            return
        self.env[t.id] = self.ev(node.value)

    def visit_AugAssign(self, node: ast.AugAssign):
        if isinstance(node.op, ast.Add) and isinstance(node.target, ast.Name) and isinstance(self.env.get(node.target.id), _Array):
            v = node.value
            if isinstance(v, ast.BinOp) and isinstance(v.op, ast.MatMult):
                self.matmul(node, self.ev(v.left), self.ev(v.right), self.env[node.target.id].name, beta="1.0")
                return
        self.fail(node, "this augmented assignment")

    def visit_Return(self, node: ast.Return):
        if node.value is None:
            return
        values = node.value.elts if isinstance(node.value, ast.Tuple) else [node.value]
        for v in values:
            # the node writes straight into a fresh output argument; its shape is known after lowering
            # into a probe, so lower once to learn the shape, into the final buffer
            name = f"_docc_ret_{len(self.outputs)}"
            before = len(self.b._data["root"]["children"])
            result = self.array_of(node, self.ev(v, name), name)
            if isinstance(result, _Array) and result.name != name and result.elem in _SIZES and 1 <= len(result.shape) <= 6:
                # a value that already has a home (a variable, an argument): the copy into the return buffer that the
                # reference's front end emits as a loop (ast_parser.py:1186-1210) is a Transpose with the identity order
                result = self.transpose(node, result, list(range(len(result.shape))), name)
            if not isinstance(result, _Array) or result.name != name or len(self.b._data["root"]["children"]) == before:
                self.fail(node, "returning a value that is not produced by a library node")
            self.outputs.append(name)
            self.output_shapes[name] = result.shape

    def visit_Expr(self, node: ast.Expr):
        if isinstance(node.value, ast.Constant):
            return  # docstring
        self.fail(node, "an expression statement")

    def visit_Pass(self, node: ast.Pass):
        return

    def generic_visit(self, node: ast.AST):
        if isinstance(node, (ast.Module, ast.FunctionDef)):
            return super().generic_visit(node)
        self.fail(node, f"statement {type(node).__name__}")

    def visit_FunctionDef(self, node: ast.FunctionDef):
        try:
            filename = inspect.getsourcefile(self.func) or ""
            first = inspect.getsourcelines(self.func)[1]
        except (OSError, TypeError):
            filename, first = "", 1
        for stmt in node.body:
            # the nodes a statement lowers to carry its source range (lines of the file, not of the snippet)
            self.b.set_debug_info(filename, self.func.__name__, first + stmt.lineno - 1, stmt.col_offset + 1,
                                  first + (stmt.end_lineno or stmt.lineno) - 1, (stmt.end_col_offset or stmt.col_offset) + 1)
            self.visit(stmt)
        self.b.set_debug_info()

    def visit_arguments(self, node):
        return


class PythonProgram(DoccProgram):
    def __init__(self, func, target: str = "none", category: str = "server", instrumentation_mode: Optional[str] = None,
                 capture_args: Optional[bool] = None, remote_tuning: bool = False, options: Optional[Dict[str, Any]] = None):
        super().__init__(name=func.__name__, target=target, category=category, instrumentation_mode=instrumentation_mode,
                         capture_args=capture_args, remote_tuning=remote_tuning)
        self.func = func
        self.options = dict(options or {})
        self.__name__ = func.__name__
        self.__doc__ = func.__doc__

    # -- DoccProgram surface -------------------------------------------------------
    def __call__(self, *args: Any) -> Any:
        compiled = self.compile(*args)
        return compiled(*self._convert_inputs(args))

    def _convert_inputs(self, args: tuple) -> tuple:
        return args

    def _convert_outputs(self, result: Any, original_args: tuple) -> Any:
        return result

    def _analyse(self, args: Sequence[Any]):
        """Shape symbols: every distinct dimension value (other than 1) gets one `_s<i>`, in order
        of first appearance; returns (types, mapping, shape_sources, signature)."""
        # a parameter annotated as bf16 takes the raw 16-bit words
        hints = self._parameter_annotations()
        arg_types = []
        for i, a in enumerate(args):
            declared = hints[i] if i < len(hints) else None
            if isinstance(a, np.ndarray) and isinstance(declared, Pointer) and declared.primitive_type == PrimitiveType.BFloat:
                if a.dtype != np.uint16 and not _is_ml_bfloat16(a.dtype):
                    raise TypeError(f"{self.name}: parameter {i} is annotated as bfloat16 and takes uint16 words, got {a.dtype}")
                arg_types.append(declared)
            else:
                arg_types.append(_map_python_type(a))
        values: List[int] = []
        sources: List[Tuple[int, int]] = []
        mapping: Dict[Tuple[int, int], int] = {}
        for i, a in enumerate(args):
            if isinstance(a, np.ndarray):
                for d, v in enumerate(a.shape):
                    if v == 1:
                        continue
                    if v not in values:
                        values.append(v)
                        sources.append((i, d))
                    mapping[(i, d)] = values.index(v)
        type_sig = ", ".join(f"{type(t).__name__}[{t.primitive_type.name}]" + (f"x{args[i].ndim}" if isinstance(args[i], np.ndarray) else "")
                             for i, t in enumerate(arg_types))
        ones = sorted((i, d) for i, a in enumerate(args) if isinstance(a, np.ndarray) for d, v in enumerate(a.shape) if v == 1)
        signature = f"{type_sig}|{sorted(mapping.items())}|{ones}"
        return arg_types, mapping, sources, signature

    def _parameter_annotations(self) -> List[Any]:
        """The SDFG type each parameter's annotation names, or None (no annotation, a string, one that does not map)."""
        if getattr(self, "_hints", None) is None:
            out = []
            for p in inspect.signature(self.func).parameters.values():
                ann = p.annotation
                out.append(None if ann is inspect.Parameter.empty or isinstance(ann, str) else _map_annotation(ann))
            self._hints = out
        return self._hints

    def _get_cache_key(self, *args: Any) -> str:
        return self._analyse(args)[3]

    def _build_sdfg(self, args: Sequence[Any], arg_types, mapping):
        params = list(inspect.signature(self.func).parameters)
        if len(params) != len(args):
            raise TypeError(f"{self.name}() takes {len(params)} positional arguments but {len(args)} were given")
        builder = StructuredSDFGBuilder(f"{self.name}_sdfg")
        env: Dict[str, Any] = {}
        # outputs a return annotation declares come first in the argument list: the reference adds them before it looks
        # at the parameters (python_program.py:515-524); a scalar is returned through a pointer
        declared = _return_annotation_types(self.func) or []
        for i, t in enumerate(declared):
            builder.add_container(f"_docc_ret_{i}", t if isinstance(t, Pointer) else Pointer(t), True)
        for i, (p, a, t) in enumerate(zip(params, args, arg_types)):
            builder.add_container(p, t, True)
            if isinstance(a, np.ndarray):
                shape = ["1" if v == 1 else f"_s{mapping[(i, d)]}" for d, v in enumerate(a.shape)]
                env[p] = _Array(p, shape, t.primitive_type)
            else:
                env[p] = _ScalarValue(p)
        nsym = (max(mapping.values()) + 1) if mapping else 0
        for s in range(nsym):
            builder.add_container(f"_s{s}", Scalar(PrimitiveType.Int64), True)
        source = textwrap.dedent(inspect.getsource(self.func))
        tree = ast.parse(source)
        fdef = next(n for n in ast.walk(tree) if isinstance(n, ast.FunctionDef) and n.name == self.func.__name__)
        lowering = _Lowering(self.func, builder, env, params)
        lowering.visit_FunctionDef(fdef)
        sdfg = builder.move()
        return sdfg, lowering.outputs, lowering.output_shapes

    def to_sdfg(self, *args: Any) -> StructuredSDFG:
        arg_types, mapping, _, _ = self._analyse(args)
        return self._build_sdfg(args, arg_types, mapping)[0]

    def compile(self, *args: Any, output_folder: Optional[str] = None, instrumentation_mode: Optional[str] = None,
                capture_args: Optional[bool] = None) -> CompiledSDFG:
        original_output_folder = output_folder
        instrumentation_mode = instrumentation_mode if instrumentation_mode is not None else (self.instrumentation_mode or "")
        capture_args = bool(capture_args if capture_args is not None else (self.capture_args or False))
        arg_types, mapping, shape_sources, signature = self._analyse(args)

        if output_folder is None:
            filename = inspect.getsourcefile(self.func)
            hash_input = f"{filename}|{self.name}|{self.target}|{self.category}|{capture_args}|{instrumentation_mode}|{self.remote_tuning}|{sorted(self.options.items())}|{signature}"
            stable_id = hashlib.sha256(hash_input.encode()).hexdigest()[:16]
            docc_tmp = os.environ.get("DOCC_TMP")
            if docc_tmp:
                output_folder = f"{docc_tmp}/{self.name}-{stable_id}"
            else:
                user = os.getenv("USER") or getpass.getuser()
                output_folder = f"/tmp/{user}/DOCC/{self.name}-{stable_id}"
        if original_output_folder is None and signature in self.cache:
            return self.cache[signature]

        if os.path.exists(output_folder):
            shutil.rmtree(output_folder)
        sdfg, out_args, out_shapes = self._build_sdfg(args, arg_types, mapping)
        sdfg.validate()
        sdfg.expand()
        sdfg.simplify()
        if self.target != "none":
            sdfg.normalize()
        sdfg.dump(output_folder)

        if self.target != "none":
            custom_schedule_fn = get_target_schedule_fn(self.target)
            if custom_schedule_fn is not None:
                custom_schedule_fn(sdfg, self.category, {"remote_tuning": self.remote_tuning, **self.options})
            else:
                print(f"Target '{self.target}' is not supported")
                sdfg.schedule(self.target, self.category, self.remote_tuning)
        self.last_sdfg = sdfg
        sdfg.dump(output_folder, "post_sched")

        custom_compile_fn = get_target_compile_fn(self.target)
        if custom_compile_fn is not None:
            lib_path = custom_compile_fn(sdfg, output_folder, instrumentation_mode, capture_args, dict(self.options))
        else:
            lib_path = sdfg._compile(output_folder=output_folder, target=self.target,
                                     instrumentation_mode=instrumentation_mode, capture_args=capture_args)
        compiled = CompiledSDFG(lib_path, sdfg, shape_sources, {}, out_args, out_shapes, {})
        if original_output_folder is None:
            self.cache[signature] = compiled
        return compiled


def native(func=None, *, target: str = "rocm", category: str = "server", instrumentation_mode: Optional[str] = None,
           capture_args: Optional[bool] = None, remote_tuning: bool = False, **options):
    """Decorator: `@native` or `@native(target="rocm", category="server")`. Extra keyword
    options (e.g. offload="node") are passed to the target's schedule hook."""
    if func is not None and callable(func):
        return PythonProgram(func, target=target, category=category, instrumentation_mode=instrumentation_mode,
                             capture_args=capture_args, remote_tuning=remote_tuning, options=options)

    def decorator(f):
        return PythonProgram(f, target=target, category=category, instrumentation_mode=instrumentation_mode,
                             capture_args=capture_args, remote_tuning=remote_tuning, options=options)

    return decorator
