"""`torch.compile(model, backend="docc")` and `compile_torch` for the `rocm` target.

Same surface as the reference's `docc.torch` (mlir/docc/torch/__init__.py:15-441): `TorchProgram`,
`compile_torch(model, example_input, target, category)`, the global `set_backend_options(target,
category)` read by the backend, a backend registered under the name "docc" that returns a tuple of
tensors to dynamo, and `metadata("return_shape")` on the SDFG.

The reference goes FX -> torch-mlir -> linalg -> SDFG and supports only 2-d matmul and
unpadded, bias-free convolution (mlir/lib/Target/SDFG/LinalgToSDFGTranslator.cpp:517-523,696-699);
this front end lowers the FX graph directly and covers what the rocm kernels implement:

    torch.matmul / @ / mm / bmm            -> GEMM (2-d, with transposed operands) or ml::MatMul (batched); bf16 operands:
                                              the bf16 GEMM with float32 accumulation - its float32 result where the model
                                              asks for it (`.float()`), else rounded once to bf16 (ml::Cast) as eager torch does
    softmax(x, dim=-1) on fp32             -> ml::Softmax
    F.conv2d / nn.Conv2d                   -> ml::Conv with padding, bias and groups
    softmax(q @ k.transpose(-2, -1) * c, dim=-1) @ v   and   F.scaled_dot_product_attention(q, k, v[, is_causal=True])
                                           -> ml::Attention (bf16; head dims 32, 64, 128 fused; causal up to 128);
                                              float32 / float64 tensors, or an additive attn_mask: ml::Transpose, ml::MatMul,
                                              ml::Softmax, ml::MatMul
    + - * / ** torch.maximum / torch.minimum on fp32/fp64 tensors (broadcasting) or a tensor and a number; on bf16
                                              tensors in float32 with one rounding to bf16, as eager torch computes them
                                              (likewise the unary operations, reductions, softmax, gelu, silu, layer_norm)
                                           -> ml::Add .. ml::Minimum, with ml::Broadcast where shapes differ
    relu, sigmoid, tanh, exp, abs, sqrt, erf (functions, methods, nn.ReLU / nn.Sigmoid / nn.Tanh),
    elu, leaky_relu, hardsigmoid (F.* and nn.ELU / nn.LeakyReLU / nn.Hardsigmoid)
                                           -> ml::ReLU .. ml::Erf
    gelu (erf and tanh forms), silu, neg, reciprocal, rsqrt, square, layer_norm (F.* / methods / nn.GELU, nn.SiLU,
    nn.LayerNorm)                          -> the chains of those nodes (and ml::Mean) that spell them; the target's map
                                              fusion makes one generated kernel of each chain
    F.linear / nn.Linear                   -> GEMM with the weight transposed, bias through Broadcast + Add
    sum / mean / amax / amin over any dims (keepdim) -> ml::Sum .. ml::Min

Tensors on a `cuda` device are passed to the generated function as device pointers (no
transfers, the kernels run on the null stream in order with torch's default stream); CPU tensors
are uploaded and downloaded by the generated code. Anything else raises NotImplementedError: this
target has no CPU lowering to fall back to.
"""
from __future__ import annotations

import ctypes
import getpass
import hashlib
import math
import operator
import os
import shutil
from typing import Any, Dict, List, Optional, Sequence, Tuple

from docc_amd import runtime
from docc_amd.compiler import CompiledSDFG, DoccProgram
from docc_amd.python.target_registry import get_target_compile_fn, get_target_schedule_fn
from docc_amd.sdfg import Pointer, PrimitiveType, Scalar, StructuredSDFG, StructuredSDFGBuilder

import docc_amd.python  # noqa: F401  (registers the rocm target hooks)


def _elem(dtype) -> PrimitiveType:
    import torch

    table = {torch.float32: PrimitiveType.Float, torch.float64: PrimitiveType.Double, torch.bfloat16: PrimitiveType.BFloat,
             torch.float16: PrimitiveType.Half, torch.int32: PrimitiveType.Int32, torch.int64: PrimitiveType.Int64}
    if dtype not in table:
        raise NotImplementedError(f"tensor dtype {dtype} is not supported by the rocm target")
    return table[dtype]


class _T:
    """A tensor held in an SDFG container."""

    def __init__(self, name: str, shape: Sequence[int], dtype):
        self.name, self.shape, self.dtype = name, [int(s) for s in shape], dtype


class _Transposed:
    def __init__(self, base: _T):
        self.base = base


class _Widened:
    """A bf16 tensor converted to float32 (`x.float()`), kept symbolic: as both operands of a product it selects the
    bf16 GEMM with float32 accumulation and result, which computes exactly that expression; anywhere else it becomes
    the ml::Cast it stands for."""

    def __init__(self, base: _T, dtype):
        self.base, self.shape, self.dtype = base, base.shape, dtype


class _Bf16Product:
    """`a @ b` of bf16 operands, kept symbolic until `.float()` / `.to(torch.float32)` asks for the float32 result:
    the GEMM then writes its float32 accumulators (without the rounding to bf16 that eager torch inserts in between)."""

    def __init__(self, a: _T, b: _T, ta: bool, tb: bool):
        self.a, self.b, self.ta, self.tb = a, b, ta, tb


class _Scores:
    """scale * q @ k^T, kept symbolic until a softmax and a product with v complete the pattern."""

    def __init__(self, q: _T, k: _T, scale: float = 1.0):
        self.q, self.k, self.scale = q, k, scale


class _Probs:
    def __init__(self, scores: _Scores):
        self.scores = scores


class _FxLowering:
    def __init__(self, gm, example_inputs: Sequence[Any], name: str):
        import torch

        self.torch = torch
        self.gm = gm
        self.builder = StructuredSDFGBuilder(name)
        self.env: Dict[Any, Any] = {}
        self.inputs: List[Tuple[str, Any]] = []      # (container, ("arg", index) | ("attr", qualified name))
        self.outputs: List[Tuple[str, List[int], Any]] = []
        self.example_inputs = list(example_inputs)
        self._propagate_shapes()

    # ---- shapes ---------------------------------------------------------------------
    def _propagate_shapes(self):
        torch = self.torch
        if all("example_value" in n.meta or "tensor_meta" in n.meta for n in self.gm.graph.nodes if n.op not in ("output",)):
            return
        if any(not isinstance(a, (torch.Tensor, int, float, bool)) for a in self.example_inputs):
            return  # symbolic inputs: dynamo has already annotated the graph
        from torch._subclasses.fake_tensor import FakeTensorMode
        from torch.fx.passes.shape_prop import ShapeProp

        mode = FakeTensorMode(allow_non_fake_inputs=True)
        fake = [mode.from_tensor(a) if isinstance(a, torch.Tensor) else a for a in self.example_inputs]
        ShapeProp(self.gm, fake_mode=mode).propagate(*fake)

    def meta(self, node):
        v = node.meta.get("example_value")
        if v is None:
            v = node.meta.get("tensor_meta")
        if v is None:
            raise NotImplementedError(f"no shape information for FX node {node.name}")
        # symbolic sizes (dynamo's automatic dynamic shapes) are specialised to their current value
        return [int(d) for d in v.shape], v.dtype

    # ---- containers ---------------------------------------------------------------------
    def add_input(self, label: str, shape, dtype, source) -> _T:
        name = self.builder.find_new_name(f"{label}_") if self.builder.exists(label) else label
        self.builder.add_container(name, Pointer(Scalar(_elem(dtype))), True)
        self.inputs.append((name, source))
        return _T(name, shape, dtype)

    def new_tensor(self, shape, dtype, dest: Optional[str]) -> _T:
        if dest is not None:
            if not self.builder.exists(dest):  # `_docc_ret_<i>`: an output pointer argument
                self.builder.add_container(dest, Pointer(Scalar(_elem(dtype))), True)
            return _T(dest, shape, dtype)
        nbytes = int(math.prod(shape)) * self.torch.empty((), dtype=dtype).element_size()
        name = self.builder.find_new_name("_tmp_")
        self.builder.add_container(name, Pointer(Scalar(_elem(dtype))), False, transient_bytes=nbytes)
        return _T(name, shape, dtype)

    def fail(self, node, what: str):
        raise NotImplementedError(f"FX node {node.name} ({node.target}): {what} is not supported by the rocm target")

    # ---- operations -----------------------------------------------------------------------
    def matmul(self, node, a, b, dest):
        torch = self.torch
        if isinstance(a, _Probs):
            return self.attention(node, a.scores.q, a.scores.k, b, a.scores.scale, dest)
        ta = tb = False
        if isinstance(a, _Transposed):
            ta, a = True, a.base
        if isinstance(b, _Transposed):
            tb, b = True, b.base
        if isinstance(a, _Widened) and isinstance(b, _Widened) and a.dtype == b.dtype == torch.float32:
            # a.float() @ b.float() of bf16 tensors: the bf16 GEMM with float32 accumulation is that product
            return self.product(node, a.base, b.base, ta, tb, torch.float32, dest)
        a, b = self.tensor(node, a), self.tensor(node, b)
        if not isinstance(a, _T) or not isinstance(b, _T):
            self.fail(node, "a product of these operands")
        if a.dtype != b.dtype:
            self.fail(node, "a product of mixed dtypes")
        if len(a.shape) > 2 and tb and not ta and a.dtype == torch.bfloat16 and len(b.shape) == len(a.shape):
            return _Scores(a, b)  # q @ k^T: waits for its softmax
        if a.dtype == torch.bfloat16:
            # bf16 operands: only the float32 result exists as a kernel; `.float()` on the product asks for it
            return _Bf16Product(a, b, ta, tb)
        return self.product(node, a, b, ta, tb, a.dtype, dest)

    def product(self, node, a: _T, b: _T, ta: bool, tb: bool, out_dtype, dest):
        """GEMM (2-d operands, transposes by flag) or ml::MatMul (batched) into a tensor of `out_dtype`: the operands'
        dtype, or float32 for bf16 operands."""
        if len(a.shape) == 2 and len(b.shape) == 2:
            m, k = (a.shape[1], a.shape[0]) if ta else a.shape
            k2, n = (b.shape[1], b.shape[0]) if tb else b.shape
            if k != k2:
                self.fail(node, f"inner dimensions {k} and {k2}")
            out = self.new_tensor([m, n], out_dtype, dest)
            one, zero = "1.0", "0.0"
            self.builder.add_gemm(a.name, b.name, out.name, one, zero, m, n, k, ta, tb, a.shape[1], b.shape[1], n)
            return out
        if ta or tb:
            self.fail(node, "a transposed operand in a batched product")
        if len(a.shape) < 2 or len(b.shape) < 2:
            self.fail(node, "a product with a vector operand")
        if len(b.shape) > 2 and b.shape[:-2] != a.shape[:-2]:
            self.fail(node, "broadcasting batch dimensions")
        if a.shape[-1] != b.shape[-2]:
            self.fail(node, f"inner dimensions {a.shape[-1]} and {b.shape[-2]}")
        out = self.new_tensor(a.shape[:-1] + [b.shape[-1]], out_dtype, dest)
        self.builder.add_matmul(a.name, b.name, out.name, a.shape, b.shape)
        return out

    def attention(self, node, q: _T, k: _T, v, scale: float, dest, causal: bool = False):
        torch = self.torch
        if not isinstance(v, _T):
            self.fail(node, "attention values of this form")
        if len(q.shape) == 3:  # [B*H, S, D] given as 3-d: treat the leading dim as batch with one head
            shape_q = [q.shape[0], 1, q.shape[1], q.shape[2]]
        elif len(q.shape) == 4:
            shape_q = list(q.shape)
        else:
            self.fail(node, "attention on tensors that are not 3-d or 4-d")
        if q.dtype != torch.bfloat16 or k.dtype != q.dtype or v.dtype != q.dtype:
            self.fail(node, "attention on tensors other than bfloat16")
        if k.shape != v.shape or k.shape[:-2] != q.shape[:-2] or k.shape[-1] != q.shape[-1]:
            self.fail(node, "attention with mismatched q/k/v shapes")
        out = self.new_tensor(q.shape, q.dtype, dest)
        if causal and q.shape[-1] > 128:
            self.fail(node, "causal attention with a head dimension above 128")
        self.builder.add_attention(q.name, k.name, v.name, out.name, shape_q, k.shape[-2], scale, causal)
        return out

    def attention_unfused(self, node, q: _T, k, v, scale: float, mask, dest):
        """softmax(scale * q k^T + mask) v as batched products around a softmax: float32 / float64 tensors, and bf16 tensors
        with an additive mask (scores, mask and softmax in float32, the probabilities rounded to bf16 for the second product,
        as eager torch's math path does)."""
        torch = self.torch
        k, v = self.tensor(node, k), self.tensor(node, v)
        if not isinstance(k, _T) or not isinstance(v, _T) or len(q.shape) < 3 or k.dtype != q.dtype or v.dtype != q.dtype:
            self.fail(node, "attention on these operands")
        if q.dtype not in (torch.float32, torch.float64, torch.bfloat16):
            self.fail(node, "attention on tensors other than float32 / float64 / bfloat16")
        bf16 = q.dtype == torch.bfloat16
        wide = torch.float32 if bf16 else q.dtype
        scores = self.product(node, q, self.tensor(node, _Transposed(k)), False, False, wide, None)
        scores = self.elementwise(node, "mul", scores, float(scale), None)
        if mask is not None:
            mask = self.widened(node, self.tensor(node, mask))
            if not isinstance(mask, _T) or mask.dtype != wide:
                self.fail(node, "a mask that is not a floating-point tensor of the scores' type (a boolean mask: add -inf where it is False)")
            scores = self.elementwise(node, "add", scores, mask, None)
        probs = self.softmax(node, scores, len(q.shape) - 1, None)
        if not bf16:
            return self.product(node, probs, v, False, False, q.dtype, dest)
        return self.narrowed(node, self.product(node, self.narrowed(node, probs, None), v, False, False, wide, None), dest)

    def softmax(self, node, x, dim, dest):
        if isinstance(x, _Scores):
            if dim not in (-1, len(x.q.shape) - 1):
                self.fail(node, "softmax of attention scores over an axis other than the last")
            return _Probs(x)
        x = self.tensor(node, x)
        if not isinstance(x, _T):
            self.fail(node, "softmax of this value")
        if not -len(x.shape) <= dim < len(x.shape):
            self.fail(node, "softmax dim out of range")
        if self.is_bf16(x):
            return self.narrowed(node, self.softmax(node, self.widened(node, x), dim, None), dest)
        if x.dtype not in (self.torch.float32, self.torch.float64):
            self.fail(node, "softmax on a dtype other than float32 / float64")
        out = self.new_tensor(x.shape, x.dtype, dest)
        self.builder.add_reduce_op("softmax", x.name, out.name, x.shape, [dim])
        return out

    def conv2d(self, node, x, w, bias, stride, padding, dilation, groups, dest):
        pair = lambda v: [int(v), int(v)] if isinstance(v, int) else [int(e) for e in v]
        if not isinstance(x, _T) or not isinstance(w, _T) or len(x.shape) != 4 or len(w.shape) != 4:
            self.fail(node, "conv2d on these operands")
        groups = int(groups)
        if groups < 1 or x.shape[1] % groups or w.shape[0] % groups or w.shape[1] * groups != x.shape[1]:
            self.fail(node, "a convolution whose groups do not divide the channels")
        if isinstance(padding, str):
            self.fail(node, "string padding modes")
        if x.dtype != self.torch.float32:
            self.fail(node, "conv2d on a dtype other than float32")
        stride, padding, dilation = pair(stride), pair(padding), pair(dilation)
        oh, ow = ((x.shape[2 + i] + 2 * padding[i] - dilation[i] * (w.shape[2 + i] - 1) - 1) // stride[i] + 1 for i in range(2))
        out = self.new_tensor([x.shape[0], w.shape[0], oh, ow], x.dtype, dest)
        self.builder.add_conv(x.name, w.name, out.name, x.shape, w.shape[2:], stride, padding + padding, dilation, w.shape[0], groups,
                              bias.name if isinstance(bias, _T) else None)
        return out

    def scale(self, node, x, factor: float, dest=None):
        if isinstance(x, _Scores):
            return _Scores(x.q, x.k, x.scale * factor)
        return self.elementwise(node, "mul", x, float(factor), dest)

    def expanded(self, node, x: _T, shape: List[int]) -> _T:
        """`x` repeated to `shape` through ml::Broadcast (a no-op when the shapes agree)."""
        if x.shape == shape:
            return x
        if len(shape) > 6:
            self.fail(node, "a broadcast of rank above 6")
        out = self.new_tensor(shape, x.dtype, None)
        self.builder.add_broadcast(x.name, out.name, [1] * (len(shape) - len(x.shape)) + x.shape, shape)
        return out

    # bf16 tensors outside products: eager torch computes elementwise operations, reductions and softmax on bf16 in float32 and
    # rounds the result once; here the operands are widened (ml::Cast), the float32 nodes do the work and one ml::Cast rounds.
    def is_bf16(self, v) -> bool:
        return isinstance(v, _T) and v.dtype == self.torch.bfloat16

    def widened(self, node, v):
        return self.tensor(node, _Widened(v, self.torch.float32)) if self.is_bf16(v) else v

    def narrowed(self, node, wide: _T, dest):
        out = self.new_tensor(wide.shape, self.torch.bfloat16, dest)
        self.builder.add_cast_op(wide.name, out.name, wide.shape)
        return out

    def elementwise(self, node, op: str, a, b, dest):
        torch = self.torch
        a, b = self.tensor(node, a), self.tensor(node, b)
        tensors = [v for v in (a, b) if isinstance(v, _T)]
        if any(self.is_bf16(v) for v in tensors) and all(v.dtype in (torch.bfloat16, torch.float32) for v in tensors):
            narrow = all(self.is_bf16(v) for v in tensors)      # bf16 with float32 promotes to float32
            wide = self.elementwise(node, op, self.widened(node, a), self.widened(node, b), None if narrow else dest)
            return self.narrowed(node, wide, dest) if narrow else wide
        if not tensors or not all(isinstance(v, (_T, int, float)) and not isinstance(v, bool) for v in (a, b)):
            self.fail(node, f"elementwise {op} of these operands")
        dtype = tensors[0].dtype
        if dtype not in (torch.float32, torch.float64) or any(v.dtype != dtype for v in tensors):
            self.fail(node, f"elementwise {op} on dtypes other than one of float32 / float64")
        if len(tensors) == 2:
            try:
                shape = list(torch.broadcast_shapes(tuple(a.shape), tuple(b.shape)))
            except RuntimeError:
                self.fail(node, f"shapes {a.shape} and {b.shape}, which do not broadcast,")
            a, b = self.expanded(node, a, shape), self.expanded(node, b, shape)
        else:
            shape = tensors[0].shape
        out = self.new_tensor(shape, dtype, dest)
        name = lambda v: v.name if isinstance(v, _T) else repr(float(v))
        self.builder.add_elementwise_op(op, name(a), name(b), out.name, shape)
        return out

    def unary(self, node, op: str, x, dest, alpha=None, beta=None):
        x = self.tensor(node, x)
        if self.is_bf16(x):
            return self.narrowed(node, self.unary(node, op, self.widened(node, x), None, alpha, beta), dest)
        if not isinstance(x, _T) or x.dtype not in (self.torch.float32, self.torch.float64):
            self.fail(node, f"{op} of a value that is not a float32 / float64 tensor")
        out = self.new_tensor(x.shape, x.dtype, dest)
        if alpha is None and beta is None:
            self.builder.add_elementwise_unary_op(op, x.name, out.name, x.shape)
        else:
            self.builder.add_elementwise_unary_op(op, x.name, out.name, x.shape, alpha=alpha, beta=beta)
        return out

    def reduce(self, node, op: str, x, dim, keepdim: bool, dest):
        x = self.tensor(node, x)
        if self.is_bf16(x):
            return self.narrowed(node, self.reduce(node, op, self.widened(node, x), dim, keepdim, None), dest)
        if not isinstance(x, _T) or x.dtype not in (self.torch.float32, self.torch.float64):
            self.fail(node, f"{op} of a value that is not a float32 / float64 tensor")
        rank = len(x.shape)
        dims = list(range(rank)) if dim is None or dim == [] or dim == () else ([dim] if isinstance(dim, int) else list(dim))
        dims = sorted({int(d) % rank for d in dims})
        shape = [(1 if d in dims else s) for d, s in enumerate(x.shape) if keepdim or d not in dims]
        out = self.new_tensor(shape, x.dtype, dest)
        self.builder.add_reduce_op(op, x.name, out.name, x.shape, dims, keepdim)
        return out

    # Operations torch has one name for and the node set spells in several: the pieces are tensor nodes, and the map
    # fusion pass of the target makes one generated kernel of each chain.
    def gelu(self, node, x, approximate: str, dest):
        """0.5 x (1 + erf(x / sqrt 2)), or with tanh(sqrt(2 / pi) (x + 0.044715 x^3)) in place of the erf."""
        x = self.tensor(node, x)
        if self.is_bf16(x):      # one rounding at the end, like eager torch's kernel
            return self.narrowed(node, self.gelu(node, self.widened(node, x), approximate, None), dest)
        if approximate == "tanh":
            cube = self.elementwise(node, "mul", self.elementwise(node, "mul", x, x, None), x, None)
            inner = self.elementwise(node, "mul", self.elementwise(node, "add", x, self.elementwise(node, "mul", cube, 0.044715, None), None),
                                     math.sqrt(2.0 / math.pi), None)
            gate = self.unary(node, "tanh", inner, None)
        elif approximate == "none":
            gate = self.unary(node, "erf", self.elementwise(node, "mul", x, 1.0 / math.sqrt(2.0), None), None)
        else:
            self.fail(node, f"gelu with approximate='{approximate}'")
        half = self.elementwise(node, "mul", x, 0.5, None)
        return self.elementwise(node, "mul", half, self.elementwise(node, "add", gate, 1.0, None), dest)

    def silu(self, node, x, dest):
        x = self.tensor(node, x)
        if self.is_bf16(x):
            return self.narrowed(node, self.silu(node, self.widened(node, x), None), dest)
        return self.elementwise(node, "mul", x, self.unary(node, "sigmoid", x, None), dest)

    def layer_norm(self, node, x, normalized_shape, weight, bias, eps: float, dest):
        """(x - mean) / sqrt(var + eps) * weight + bias over the last len(normalized_shape) axes, the variance as the
        mean of the squared differences (what torch computes)."""
        x = self.tensor(node, x)
        if not isinstance(x, _T):
            self.fail(node, "layer_norm of this value")
        if self.is_bf16(x):
            wide = self.layer_norm(node, self.widened(node, x), normalized_shape, self.widened(node, self.tensor(node, weight)),
                                   self.widened(node, self.tensor(node, bias)), eps, None)
            return self.narrowed(node, wide, dest)
        shape = [int(v) for v in ([normalized_shape] if isinstance(normalized_shape, int) else normalized_shape)]
        if not shape or x.shape[-len(shape):] != shape:
            self.fail(node, "layer_norm whose normalized_shape is not the tensor's last axes")
        dims = list(range(len(x.shape) - len(shape), len(x.shape)))
        centred = self.elementwise(node, "sub", x, self.reduce(node, "mean", x, dims, True, None), None)
        var = self.reduce(node, "mean", self.elementwise(node, "mul", centred, centred, None), dims, True, None)
        scale = self.unary(node, "sqrt", self.elementwise(node, "add", var, float(eps), None), None)
        last = weight is None and bias is None
        y = self.elementwise(node, "div", centred, scale, dest if last else None)
        if weight is not None:
            y = self.elementwise(node, "mul", y, weight, dest if bias is None else None)
        if bias is not None:
            y = self.elementwise(node, "add", y, bias, dest)
        return y

    def linear(self, node, x, w, bias, dest):
        """x [..., K] times w[N, K] transposed, plus bias [N]: one GEMM over the flattened rows."""
        out_dtype = None
        if isinstance(x, _Widened) and isinstance(w, _Widened):      # bf16 operands widened for the product: the bf16 GEMM
            x, w, out_dtype = x.base, w.base, self.torch.float32
        else:
            x, w = self.tensor(node, x), self.tensor(node, w)
        if not isinstance(x, _T) or not isinstance(w, _T) or len(w.shape) != 2 or len(x.shape) < 1 or x.shape[-1] != w.shape[1]:
            self.fail(node, "linear on these operands")
        bf16 = self.torch.bfloat16
        if x.dtype != w.dtype or (out_dtype is None and x.dtype not in (self.torch.float32, self.torch.float64, bf16)):
            self.fail(node, "linear on dtypes other than float32 / float64 / bfloat16")
        n, k = w.shape
        m = int(math.prod(x.shape[:-1]))
        shape = x.shape[:-1] + [n]
        if out_dtype is None and x.dtype == bf16:
            # bf16 throughout, as eager torch runs it: float32 accumulation, the bias added in float32, one rounding to bf16
            wide = self.new_tensor(shape, self.torch.float32, None)
            self.builder.add_gemm(x.name, w.name, wide.name, "1.0", "0.0", m, n, k, False, True, k, k, n)
            if bias is not None:
                wide = self.elementwise(node, "add", wide, self.cast(node, self.tensor(node, bias), self.torch.float32, None), None)
            out = self.new_tensor(shape, bf16, dest)
            self.builder.add_cast_op(wide.name, out.name, shape)
            return out
        out = self.new_tensor(shape, out_dtype or x.dtype, dest if bias is None else None)
        self.builder.add_gemm(x.name, w.name, out.name, "1.0", "0.0", m, n, k, False, True, k, k, n)
        if bias is None:
            return out
        return self.elementwise(node, "add", out, bias, dest)

    def transpose(self, node, x, d0: int, d1: int, dest=None):
        if isinstance(x, _Widened) and dest is None and {d0 % len(x.shape), d1 % len(x.shape)} == {len(x.shape) - 2, len(x.shape) - 1}:
            return _Transposed(x)   # still an operand of a bf16 product, or cast and transposed where it is used
        x = self.tensor(node, x)
        if not isinstance(x, _T):
            self.fail(node, "transposing this value")
        rank = len(x.shape)
        if {d0 % rank, d1 % rank} == {rank - 2, rank - 1} and dest is None:
            return _Transposed(x)   # a GEMM flag when it feeds a product; ml::Transpose when used as a tensor
        dims = list(range(rank))
        dims[d0 % rank], dims[d1 % rank] = dims[d1 % rank], dims[d0 % rank]
        return self.permute(node, x, dims, dest)

    def permute(self, node, x, dims, dest=None):
        """ml::Transpose: the result is a contiguous tensor with the permuted shape."""
        x = self.tensor(node, x)
        if not isinstance(x, _T):
            self.fail(node, "permuting this value")
        rank = len(x.shape)
        dims = [int(d) % rank for d in dims]
        if sorted(dims) != list(range(rank)):
            self.fail(node, "a permutation that does not name every dim once")
        if rank > 6:
            self.fail(node, "a permutation of rank above 6")
        out = self.new_tensor([x.shape[d] for d in dims], x.dtype, dest)
        self.builder.add_transpose(x.name, out.name, x.shape, dims)
        return out

    def cast(self, node, x, dtype, dest=None):
        """ml::Cast; the same dtype passes the tensor on."""
        torch = self.torch
        if isinstance(x, _Bf16Product) and dtype == torch.float32:
            return self.product(node, x.a, x.b, x.ta, x.tb, torch.float32, dest)   # the GEMM's own result, not rounded in between
        if dtype == torch.float32 and dest is None:
            # bf16 -> float32 that may be an operand of a product: decided where it is used
            if isinstance(x, _T) and x.dtype == torch.bfloat16:
                return _Widened(x, dtype)
            if isinstance(x, _Transposed) and isinstance(x.base, _T) and x.base.dtype == torch.bfloat16:
                return _Transposed(_Widened(x.base, dtype))
        x = self.tensor(node, x)
        if not isinstance(x, _T):
            self.fail(node, "converting this value")
        if x.dtype == dtype:
            return x
        code = {self.torch.float16: 0, self.torch.bfloat16: 1, self.torch.float32: 2, self.torch.float64: 3, self.torch.int32: 4,
                self.torch.int64: 5}
        s, d = code.get(x.dtype, -1), code.get(dtype, -1)
        f, g = s in (2, 3), d in (2, 3)
        if s < 0 or d < 0 or not ((f and g) or (s <= 1 and d == 2) or (d <= 1 and s == 2) or (s >= 4 and g) or (f and d >= 4)):
            self.fail(node, f"a conversion from {x.dtype} to {dtype} (16-bit types convert through float32, integers to and from float32 / float64)")
        out = self.new_tensor(x.shape, dtype, dest)
        self.builder.add_cast_op(x.name, out.name, x.shape)
        return out

    def tensor(self, node, v, dest=None):
        """A transposed view that is used as a tensor of its own (not as an operand of a product) is materialised."""
        if isinstance(v, _Transposed):
            rank = len(v.base.shape)
            return self.permute(node, v.base, list(range(rank - 2)) + [rank - 1, rank - 2], dest)
        if isinstance(v, _Widened):
            out = self.new_tensor(v.shape, v.dtype, dest)
            self.builder.add_cast_op(v.base.name, out.name, v.shape)
            return out
        if isinstance(v, _Bf16Product):
            # a bf16 product used as the bf16 tensor eager torch makes of it: the float32 result of the GEMM, rounded once
            wide = self.product(node, v.a, v.b, v.ta, v.tb, self.torch.float32, None)
            out = self.new_tensor(wide.shape, self.torch.bfloat16, dest)
            self.builder.add_cast_op(wide.name, out.name, wide.shape)
            return out
        return v

    # ---- graph walk -------------------------------------------------------------------------
    def arg(self, a):
        import torch.fx

        if isinstance(a, torch.fx.Node):
            return self.env[a]
        return a

    def lower(self) -> StructuredSDFG:
        import torch
        import torch.nn.functional as F

        graph = self.gm.graph
        output_node = next(n for n in graph.nodes if n.op == "output")
        out_values = output_node.args[0]
        out_list = list(out_values) if isinstance(out_values, (tuple, list)) else [out_values]
        # the node that produces output i writes straight into `_docc_ret_<i>`
        dest_of = {n: f"_docc_ret_{i}" for i, n in enumerate(out_list)}
        arg_index = 0
        for node in graph.nodes:
            dest = dest_of.get(node)
            if node.op == "placeholder":
                example = node.meta.get("example_value", self.example_inputs[arg_index] if arg_index < len(self.example_inputs) else None)
                if example is not None and not isinstance(example, torch.Tensor):
                    self.env[node] = int(example) if isinstance(example, (int, torch.SymInt)) else example  # a size passed as an input
                else:
                    shape, dtype = self.meta(node)
                    self.env[node] = self.add_input(node.name, shape, dtype, ("arg", arg_index))
                arg_index += 1
            elif node.op == "get_attr":
                t = self.gm
                for part in node.target.split("."):
                    t = getattr(t, part)
                self.env[node] = self.add_input(node.name, list(t.shape), t.dtype, ("attr", node.target))
            elif node.op == "call_module":
                mod = self.gm.get_submodule(node.target)
                activations = {torch.nn.ReLU: "relu", torch.nn.Sigmoid: "sigmoid", torch.nn.Tanh: "tanh"}
                if type(mod) in activations:
                    self.env[node] = self.unary(node, activations[type(mod)], self.arg(node.args[0]), dest)
                    continue
                # ml::Elu / ml::LeakyReLU / ml::HardSigmoid with their scalar operands (torch's hardsigmoid is relu6(x + 3) / 6)
                if type(mod) in (torch.nn.ELU, torch.nn.LeakyReLU, torch.nn.Hardsigmoid):
                    if getattr(mod, "inplace", False):
                        self.fail(node, "an in-place activation")
                    if isinstance(mod, torch.nn.ELU):
                        self.env[node] = self.unary(node, "elu", self.arg(node.args[0]), dest, alpha=float(mod.alpha))
                    elif isinstance(mod, torch.nn.LeakyReLU):
                        self.env[node] = self.unary(node, "leaky_relu", self.arg(node.args[0]), dest, alpha=float(mod.negative_slope))
                    else:
                        self.env[node] = self.unary(node, "hard_sigmoid", self.arg(node.args[0]), dest, alpha=1.0 / 6.0, beta=0.5)
                    continue
                if isinstance(mod, torch.nn.GELU):
                    self.env[node] = self.gelu(node, self.arg(node.args[0]), mod.approximate, dest)
                    continue
                if isinstance(mod, torch.nn.SiLU):
                    if mod.inplace:
                        self.fail(node, "an in-place activation")
                    self.env[node] = self.silu(node, self.arg(node.args[0]), dest)
                    continue
                if isinstance(mod, torch.nn.LayerNorm):
                    w = b = None
                    if mod.weight is not None:
                        w = self.add_input(f"{node.name}_weight", list(mod.weight.shape), mod.weight.dtype, ("attr", f"{node.target}.weight"))
                    if mod.bias is not None:
                        b = self.add_input(f"{node.name}_bias", list(mod.bias.shape), mod.bias.dtype, ("attr", f"{node.target}.bias"))
                    self.env[node] = self.layer_norm(node, self.arg(node.args[0]), list(mod.normalized_shape), w, b, mod.eps, dest)
                    continue
                if isinstance(mod, torch.nn.Linear):
                    w = self.add_input(f"{node.name}_weight", list(mod.weight.shape), mod.weight.dtype, ("attr", f"{node.target}.weight"))
                    b = None
                    if mod.bias is not None:
                        b = self.add_input(f"{node.name}_bias", list(mod.bias.shape), mod.bias.dtype, ("attr", f"{node.target}.bias"))
                    self.env[node] = self.linear(node, self.arg(node.args[0]), w, b, dest)
                    continue
                if not isinstance(mod, torch.nn.Conv2d):
                    self.fail(node, f"module {type(mod).__name__}")
                if mod.padding_mode != "zeros":
                    self.fail(node, "non-zero padding modes")
                w = self.add_input(f"{node.name}_weight", list(mod.weight.shape), mod.weight.dtype, ("attr", f"{node.target}.weight"))
                b = None
                if mod.bias is not None:
                    b = self.add_input(f"{node.name}_bias", list(mod.bias.shape), mod.bias.dtype, ("attr", f"{node.target}.bias"))
                self.env[node] = self.conv2d(node, self.arg(node.args[0]), w, b, mod.stride, mod.padding, mod.dilation, mod.groups, dest)
            elif node.op in ("call_function", "call_method"):
                self.env[node] = self.call(node, dest)
            elif node.op == "output":
                for i, n in enumerate(out_list):
                    v = self.env[n]
                    if isinstance(v, (_Transposed, _Widened, _Bf16Product)):
                        v = self.tensor(n, v, f"_docc_ret_{i}")
                    elif isinstance(v, _T) and v.name != f"_docc_ret_{i}" and 1 <= len(v.shape) <= 6:
                        # a value that lives elsewhere (an input, the operand of a view): copied into the result
                        # by a Transpose with the identity order
                        v = self.permute(n, v, list(range(len(v.shape))), f"_docc_ret_{i}")
                    if not isinstance(v, _T) or v.name != f"_docc_ret_{i}":
                        self.fail(n, "returning a value that no library node produces (inputs, views, partial patterns)")
                    self.outputs.append((v.name, v.shape, v.dtype))
        if not self.outputs:
            raise NotImplementedError("the graph has no output produced by a library node")
        self.builder.add_metadata("return_shape", "[" + ",".join(str(s) for s in self.outputs[0][1]) + "]")
        return self._finish()

    def _finish(self) -> StructuredSDFG:
        # outputs are declared after the inputs: rebuild the argument order (inputs, then _docc_ret_<i>)
        data = self.builder._data
        outs = [name for name, _, _ in self.outputs]
        data["arguments"] = [a for a in data["arguments"] if a not in outs] + outs
        return self.builder.move()

    def call(self, node, dest):
        import torch
        import torch.nn.functional as F

        t = node.target
        args = [self.arg(a) for a in node.args]
        kwargs = {k: self.arg(v) for k, v in node.kwargs.items()}
        method = t if node.op == "call_method" else None
        # shape queries and arithmetic on plain Python numbers are folded while lowering
        if t is getattr and isinstance(args[0], _T) and args[1] == "shape":
            return tuple(args[0].shape)
        if method == "size" and isinstance(args[0], _T):
            return tuple(args[0].shape) if len(args) == 1 else args[0].shape[args[1]]
        if method == "dim" and isinstance(args[0], _T):
            return len(args[0].shape)
        plain = lambda v: isinstance(v, (int, float, bool, str, type(None))) or (isinstance(v, (tuple, list)) and all(plain(e) for e in v))
        if node.op == "call_function" and all(plain(a) for a in args) and all(plain(v) for v in kwargs.values()) and \
                getattr(t, "__module__", "") in ("math", "_operator", "operator", "builtins"):
            return t(*args, **kwargs)
        if t in (torch.matmul, operator.matmul, torch.mm, torch.bmm) or method in ("matmul", "mm", "bmm"):
            return self.matmul(node, args[0], args[1], dest)
        if t is torch.transpose or method == "transpose":
            return self.transpose(node, args[0], args[1], args[2], dest)
        if method == "permute" or t is torch.permute:
            dims = list(args[1]) if isinstance(args[1], (tuple, list)) else list(args[1:])
            rank = len(dims)
            if rank >= 2 and dims[:-2] == list(range(rank - 2)) and dims[-2:] == [rank - 1, rank - 2]:
                return self.transpose(node, args[0], -2, -1, dest)
            return self.permute(node, args[0], dims, dest)
        if t is getattr and args[1] in ("mT", "T"):
            if args[1] == "T" and isinstance(args[0], _T) and len(args[0].shape) != 2:
                self.fail(node, ".T on a tensor that is not 2-d")
            return self.transpose(node, args[0], -2, -1, dest)
        if method in ("t",) or t is torch.t:
            return self.transpose(node, args[0], 0, 1, dest)
        if t in (operator.truediv, torch.div, torch.true_divide) or method in ("div", "true_divide"):
            if kwargs.get("rounding_mode") is not None:
                self.fail(node, "division with a rounding mode")
            if isinstance(args[1], (int, float)) and isinstance(args[0], _Scores):
                return self.scale(node, args[0], 1.0 / float(args[1]))
            return self.elementwise(node, "div", args[0], args[1], dest)
        if t in (operator.mul, torch.mul, torch.multiply) or method in ("mul", "multiply"):
            for x, c in ((args[0], args[1]), (args[1], args[0])):
                if isinstance(c, (int, float)) and isinstance(x, _Scores):
                    return self.scale(node, x, float(c))
            return self.elementwise(node, "mul", args[0], args[1], dest)
        if t in (operator.add, torch.add) or method == "add":
            if kwargs.get("alpha", 1) != 1:
                self.fail(node, "add with alpha")
            return self.elementwise(node, "add", args[0], args[1], dest)
        if t in (operator.sub, torch.sub, torch.subtract) or method in ("sub", "subtract"):
            if kwargs.get("alpha", 1) != 1:
                self.fail(node, "sub with alpha")
            return self.elementwise(node, "sub", args[0], args[1], dest)
        if t in (operator.pow, torch.pow) or method == "pow":
            return self.elementwise(node, "pow", args[0], args[1], dest)
        if t in (torch.maximum, torch.minimum) or method in ("maximum", "minimum"):
            return self.elementwise(node, "max" if (t is torch.maximum or method == "maximum") else "min", args[0], args[1], dest)
        unary_fns = {"relu": (torch.relu, F.relu), "sigmoid": (torch.sigmoid, F.sigmoid), "tanh": (torch.tanh, F.tanh),
                     "exp": (torch.exp,), "abs": (torch.abs, torch.absolute), "sqrt": (torch.sqrt,),
                     "erf": (torch.erf, torch.special.erf)}
        for op, fns in unary_fns.items():
            if any(t is f for f in fns) or method == op:
                if kwargs.get("inplace"):
                    self.fail(node, "an in-place activation")
                return self.unary(node, op, args[0], dest)
        if t is F.gelu:
            return self.gelu(node, args[0], kwargs.get("approximate", args[1] if len(args) > 1 else "none"), dest)
        if t is F.silu:
            if kwargs.get("inplace") or (len(args) > 1 and args[1]):
                self.fail(node, "an in-place activation")
            return self.silu(node, args[0], dest)
        if t in (torch.neg, torch.negative, operator.neg) or method in ("neg", "negative"):
            return self.elementwise(node, "mul", args[0], -1.0, dest)
        if t is torch.reciprocal or method == "reciprocal":
            return self.elementwise(node, "div", 1.0, args[0], dest)
        if t is torch.rsqrt or method == "rsqrt":
            return self.elementwise(node, "div", 1.0, self.unary(node, "sqrt", args[0], None), dest)
        if t is torch.square or method == "square":
            return self.elementwise(node, "mul", args[0], args[0], dest)
        if t is F.layer_norm:
            names = ["input", "normalized_shape", "weight", "bias", "eps"]
            bound = {"weight": None, "bias": None, "eps": 1e-5, **dict(zip(names, args)), **kwargs}
            return self.layer_norm(node, bound["input"], bound["normalized_shape"], bound["weight"], bound["bias"], bound["eps"], dest)
        if t in (F.elu, F.leaky_relu, F.hardsigmoid):
            if kwargs.get("inplace") or (len(args) > 2 and args[2]):
                self.fail(node, "an in-place activation")
            if t is F.elu:
                return self.unary(node, "elu", args[0], dest, alpha=float(kwargs.get("alpha", args[1] if len(args) > 1 else 1.0)))
            if t is F.leaky_relu:
                return self.unary(node, "leaky_relu", args[0], dest, alpha=float(kwargs.get("negative_slope", args[1] if len(args) > 1 else 0.01)))
            return self.unary(node, "hard_sigmoid", args[0], dest, alpha=1.0 / 6.0, beta=0.5)
        reductions = {"sum": (torch.sum,), "mean": (torch.mean,), "amax": (torch.amax,), "amin": (torch.amin,)}
        for name, fns in reductions.items():
            if any(t is f for f in fns) or method == name:
                if kwargs.get("dtype") is not None:
                    self.fail(node, "a reduction with a dtype conversion")
                dim = kwargs.get("dim", kwargs.get("axis", args[1] if len(args) > 1 else None))
                keepdim = bool(kwargs.get("keepdim", kwargs.get("keepdims", args[2] if len(args) > 2 else False)))
                return self.reduce(node, {"amax": "max", "amin": "min"}.get(name, name), args[0], dim, keepdim, dest)
        if t is torch.std or method == "std":
            # the node computes the population value sqrt(mean(x^2) - mean(x)^2): torch's default divides by n - 1
            correction = kwargs.get("correction", None)
            if correction is None:
                correction = 1 if kwargs.get("unbiased", True) else 0
            if correction != 0:
                self.fail(node, "a standard deviation with a correction other than 0 (pass correction=0)")
            dim = kwargs.get("dim", args[1] if len(args) > 1 else None)
            return self.reduce(node, "std", args[0], dim, bool(kwargs.get("keepdim", False)), dest)
        if t is F.linear:
            bias = args[2] if len(args) > 2 else kwargs.get("bias")
            return self.linear(node, args[0], args[1], bias, dest)
        if t in (torch.softmax, F.softmax) or method == "softmax":
            dim = kwargs.get("dim", args[1] if len(args) > 1 else None)
            if dim is None:
                self.fail(node, "softmax without an explicit dim")
            return self.softmax(node, args[0], int(dim), dest)
        if t in (F.conv2d, torch.conv2d):
            names = ["input", "weight", "bias", "stride", "padding", "dilation", "groups"]
            defaults = {"bias": None, "stride": 1, "padding": 0, "dilation": 1, "groups": 1}
            bound = {**defaults, **dict(zip(names, args)), **kwargs}
            return self.conv2d(node, bound["input"], bound["weight"], bound["bias"], bound["stride"], bound["padding"],
                               bound["dilation"], bound["groups"], dest)
        if t is F.scaled_dot_product_attention:
            names = ["query", "key", "value", "attn_mask", "dropout_p", "is_causal", "scale"]
            bound = {"attn_mask": None, "dropout_p": 0.0, "is_causal": False, "scale": None, **dict(zip(names, args)), **kwargs}
            if bound["dropout_p"] not in (0, 0.0):
                self.fail(node, "attention with dropout")
            q = bound["query"]
            if not isinstance(q, _T):
                self.fail(node, "attention on this query")
            scale = bound["scale"] if bound["scale"] is not None else 1.0 / math.sqrt(q.shape[-1])
            mask = bound["attn_mask"]
            if mask is not None or q.dtype in (torch.float32, torch.float64):
                # no fused kernel for a mask tensor or in these types: the nodes the expression is made of
                if bound["is_causal"]:
                    self.fail(node, "causal attention on float32 / float64 tensors, or together with a mask tensor,")
                return self.attention_unfused(node, q, bound["key"], bound["value"], float(scale), mask, dest)
            return self.attention(node, q, bound["key"], bound["value"], float(scale), dest, bool(bound["is_causal"]))
        casts = {"float": torch.float32, "double": torch.float64, "bfloat16": torch.bfloat16, "half": torch.float16, "int": torch.int32,
                 "long": torch.int64}
        if method in casts and len(args) == 1:
            return self.cast(node, args[0], casts[method], dest)
        if method in ("to", "type") and (len(args) > 1 or "dtype" in kwargs):
            dtype = kwargs.get("dtype", args[1] if len(args) > 1 else None)
            if isinstance(dtype, torch.dtype):
                return self.cast(node, args[0], dtype, dest)
        if method == "contiguous" or t is torch.Tensor.contiguous:
            return self.tensor(node, args[0], dest)   # a transposed view becomes the tensor it stands for
        self.fail(node, "this operation")


class _CompiledTorch:
    """Calls the generated function on torch tensors (device or host pointers)."""

    def __init__(self, lib_path: str, sdfg: StructuredSDFG, inputs, outputs, gm, on_device: bool):
        runtime.lib()
        self.lib_path, self.sdfg = lib_path, sdfg
        self.lib = ctypes.CDLL(lib_path)
        self.func = getattr(self.lib, sdfg.name)
        self.func.argtypes = [ctypes.c_void_p] * len(sdfg.arguments)
        self.func.restype = None
        self.inputs, self.outputs, self.gm, self.on_device = inputs, outputs, gm, on_device

    def _operands(self, args, device):
        """The tensors the generated function reads (kept alive by the caller) and their addresses."""
        keep, ptrs = [], []
        for name, (kind, ref) in self.inputs:
            if kind == "arg":
                t = args[ref]
            else:
                t = self.gm
                for part in ref.split("."):
                    t = getattr(t, part)
            t = t.detach()
            if t.device.type != device.type:
                raise ValueError(f"input '{name}' is on {t.device}, the program was compiled for {device.type} tensors")
            t = t.contiguous()
            keep.append(t)
            ptrs.append(t.data_ptr())
        return keep, ptrs

    def record(self, *args) -> "RecordedCall":
        """Runs the function once on a stream of its own, records a second run there as a HIP graph and returns the
        record: replay() repeats the whole function - every kernel of it - with one submission, reading the same
        input tensors (fill them in place, with copy_) and writing the same result tensors."""
        import torch

        if not self.on_device:
            raise ValueError("only a program compiled for device tensors can be recorded: its host variant waits for copies")
        device = torch.device("cuda", torch.cuda.current_device())
        keep, ptrs = self._operands(args, device)
        outs = [torch.empty(shape, dtype=dtype, device=device) for _, shape, dtype in self.outputs]
        runtime.init(device.index or 0)
        torch.cuda.synchronize()
        stream = runtime.stream_create()
        runtime.set_default_stream(stream)
        try:
            for recording in (False, True):
                if recording:
                    with runtime.Graph.capture(stream) as graph:
                        self.func(*ptrs, *[o.data_ptr() for o in outs])
                else:
                    # outside the record: kernel images load, per-stream buffers come into being
                    self.func(*ptrs, *[o.data_ptr() for o in outs])
                    code, message = runtime.take_failure()
                    if code != 0:
                        raise runtime.RocmRuntimeError(self.sdfg.name, code, message)
                    runtime.stream_sync(stream)
        except Exception:
            runtime.set_default_stream(0)
            runtime.stream_destroy(stream)
            raise
        runtime.set_default_stream(0)
        return RecordedCall(graph, stream, keep, outs)

    def __call__(self, *args):
        import torch

        device = torch.device("cuda", torch.cuda.current_device()) if self.on_device else torch.device("cpu")
        keep, ptrs = self._operands(args, device)
        # results for CPU callers of 1 MiB and more are pinned (torch caches such blocks): the device-to-host copy runs
        # at link speed instead of through the driver's staging of pageable memory
        pin = lambda shape, dtype: (not self.on_device and torch.cuda.is_available() and
                                    math.prod(shape) * torch.empty((), dtype=dtype).element_size() >= (1 << 20))
        outs = [torch.empty(shape, dtype=dtype, device=device, pin_memory=pin(shape, dtype)) for _, shape, dtype in self.outputs]
        if self.on_device:
            runtime.init(device.index or 0)
            current = torch.cuda.current_stream()
            if current != torch.cuda.default_stream():
                current.synchronize()  # the kernels run on the null stream
        self.func(*ptrs, *[o.data_ptr() for o in outs])
        code, message = runtime.take_failure()
        if code != 0:
            raise runtime.RocmRuntimeError(self.sdfg.name, code, message)
        if self.on_device and torch.cuda.current_stream() != torch.cuda.default_stream():
            torch.cuda.default_stream().synchronize()
        return outs[0] if len(outs) == 1 else tuple(outs)


class RecordedCall:
    """One call of a compiled program on device tensors, recorded as a HIP graph (see _CompiledTorch.record).

    inputs: the tensors the record reads, in the order of the function's operands; outputs: the tensors it writes.
    replay() enqueues one run on the record's own stream and, unless wait=False, waits for it; torch's streams do
    not order themselves against that stream, so synchronize torch's work on the inputs before a replay and call
    wait() before reading the outputs of a replay(wait=False)."""

    def __init__(self, graph, stream, inputs, outputs):
        self.graph, self.stream, self.inputs, self.outputs = graph, stream, inputs, outputs

    @property
    def result(self):
        return self.outputs[0] if len(self.outputs) == 1 else tuple(self.outputs)

    def replay(self, wait: bool = True):
        self.graph.launch()
        if wait:
            runtime.stream_sync(self.stream)
        return self.result

    def wait(self) -> None:
        runtime.stream_sync(self.stream)

    def close(self) -> None:
        if self.graph is not None:
            self.graph.destroy()
            runtime.stream_destroy(self.stream)
            self.graph = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class TorchProgram(DoccProgram):
    def __init__(self, model, example_input: Any = None, target: str = "none", category: str = "server",
                 remote_tuning: bool = False, instrumentation_mode: Optional[str] = None, capture_args: Optional[bool] = None,
                 name: Optional[str] = None):
        if name is None:
            name = model.__class__.__name__ if hasattr(model, "__class__") else "torch_model"
        super().__init__(name=name, target=target, category=category, remote_tuning=remote_tuning,
                         instrumentation_mode=instrumentation_mode, capture_args=capture_args)
        self.model = model
        self.example_input = example_input
        self._sdfg: Optional[StructuredSDFG] = None
        self._compiled: Optional[_CompiledTorch] = None
        self._input_info: list = []
        self._output_info: list = []
        self._gm = None

    def _examples(self, args: Sequence[Any]) -> List[Any]:
        if args:
            return list(args)
        if self.example_input is None:
            raise ValueError("TorchProgram needs an example input to compile")
        return list(self.example_input) if isinstance(self.example_input, (tuple, list)) else [self.example_input]

    def _graph_module(self):
        import torch.fx

        if self._gm is None:
            self._gm = self.model if isinstance(self.model, torch.fx.GraphModule) else torch.fx.symbolic_trace(self.model)
        return self._gm

    def _get_cache_key(self, *args: Any) -> str:
        import torch

        parts = []
        for a in self._examples(args):
            parts.append(f"{tuple(a.shape)}:{a.dtype}:{a.device.type}" if isinstance(a, torch.Tensor) else f"scalar({type(a).__name__})")
        return "|".join(parts)

    def _model_code(self) -> str:
        """Text that tells two models of the same name apart: the traced graph's code (it names every
        operation and constant argument), else the source of forward()."""
        try:
            return self._graph_module().graph.python_code("self").src
        except Exception:
            pass
        try:
            import inspect

            return inspect.getsource(type(self.model).forward)
        except Exception:
            return ""

    def _lower(self, examples):
        lowering = _FxLowering(self._graph_module(), examples, f"__docc_{self.name}")
        sdfg = lowering.lower()
        return sdfg, lowering

    def to_sdfg(self, *args: Any) -> StructuredSDFG:
        return self._lower(self._examples(args))[0]

    def compile(self, *args: Any, output_folder: Optional[str] = None) -> _CompiledTorch:
        import torch

        examples = self._examples(args)
        key = self._get_cache_key(*examples)
        if output_folder is None and key in self.cache:
            return self.cache[key]
        on_device = any(isinstance(a, torch.Tensor) and a.device.type == "cuda" for a in examples)
        sdfg, lowering = self._lower(examples)
        self._sdfg = sdfg
        folder = output_folder
        if folder is None:
            # the folder (and with it the path the library is loaded from) is specific to the graph: every
            # graph torch.compile hands over is called "GraphModule", and dlopen returns the handle it already
            # holds for a path, so two models sharing a folder would run the first one's code
            # (reference mlir/docc/torch/__init__.py:110-131 hashes the model's code for the same reason)
            stable_id = hashlib.sha256(f"{self.name}|{self.target}|{self.category}|{key}|{self._model_code()}".encode()).hexdigest()[:16]
            base = os.environ.get("DOCC_TMP") or f"/tmp/{os.getenv('USER') or getpass.getuser()}/DOCC"
            folder = f"{base}/{self.name}-{stable_id}"
        if os.path.exists(folder):
            shutil.rmtree(folder)
        sdfg.validate()
        sdfg.expand()
        sdfg.simplify()
        if self.target != "none":
            sdfg.normalize()
        sdfg.dump(folder)
        options = {"offload": "none" if on_device else "function"}
        if self.target != "none":
            schedule_fn = get_target_schedule_fn(self.target)
            if schedule_fn is not None:
                schedule_fn(sdfg, self.category, options)
            else:
                sdfg.schedule(self.target, self.category, self.remote_tuning)
        self.last_sdfg = sdfg
        sdfg.dump(folder, "post_sched")
        compile_fn = get_target_compile_fn(self.target)
        if compile_fn is not None:
            lib_path = compile_fn(sdfg, folder, self.instrumentation_mode or "", bool(self.capture_args), options)
        else:
            lib_path = sdfg._compile(output_folder=folder, target=self.target, instrumentation_mode=self.instrumentation_mode or "",
                                     capture_args=bool(self.capture_args))
        compiled = _CompiledTorch(lib_path, sdfg, lowering.inputs, lowering.outputs, self._graph_module(), on_device)
        self._output_info = [{"shape": tuple(shape)} for _, shape, _ in lowering.outputs]
        if output_folder is None:
            self.cache[key] = compiled
        self._compiled = compiled
        return compiled

    def __call__(self, *args: Any) -> Any:
        compiled = self.compile(*args)
        return self._convert_outputs(compiled(*self._convert_inputs(args)), args)

    def record(self, *args: Any) -> RecordedCall:
        """Compiles for `args` (device tensors) and records one call on them as a HIP graph."""
        return self.compile(*args).record(*args)

    def _convert_inputs(self, args: tuple) -> tuple:
        return args

    def _convert_outputs(self, result: Any, original_args: tuple) -> Any:
        return result


def compile_torch(model, example_input, target: str = "none", category: str = "server") -> TorchProgram:
    return TorchProgram(model, example_input=example_input, target=target, category=category)


_backend_options = {"target": "none", "category": "server"}


def set_backend_options(target: str = "none", category: str = "server"):
    """Global options read by the "docc" torch.compile backend; call before torch.compile."""
    _backend_options["target"] = target
    _backend_options["category"] = category


def _docc_backend(gm, example_inputs):
    """Called by torch.compile(backend="docc") with the FX graph dynamo captured."""
    example_input = example_inputs[0] if len(example_inputs) == 1 else tuple(example_inputs)
    program = TorchProgram(gm, example_input=example_input, target=_backend_options["target"],
                           category=_backend_options["category"])

    def compiled_fn(*args):
        result = program(*args)
        return result if isinstance(result, (tuple, list)) else (result,)

    return compiled_fn


def _register_backend():
    try:
        import torch._dynamo

        torch._dynamo.register_backend(name="docc")(_docc_backend)
    except ImportError:  # torch without dynamo
        pass
    except Exception:  # already registered (module imported twice)
        pass


_register_backend()
