"""Caller of a compiled SDFG: loads lib<name>.so with ctypes and marshals arguments.

Follows the reference's CompiledSDFG (python/docc/compiler/compiled_sdfg.py:34-78 load,
:309-552 call): arguments are walked in `sdfg.arguments` order by name; arrays travel as raw
element pointers, scalars by value, `_s<i>` shape symbols as int64 filled in from the argument
shapes, and `_docc_ret_<i>` outputs are buffers this class allocates and returns. bf16 and half
cross the boundary as 16-bit integers (:16-31).
"""
from __future__ import annotations

import ctypes
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np

from docc_amd import runtime
from docc_amd.sdfg import PrimitiveType, StructuredSDFG

_CTYPES = {
    PrimitiveType.Bool: ctypes.c_bool, PrimitiveType.Int8: ctypes.c_int8, PrimitiveType.Int16: ctypes.c_int16,
    PrimitiveType.Int32: ctypes.c_int32, PrimitiveType.Int64: ctypes.c_int64, PrimitiveType.UInt8: ctypes.c_uint8,
    PrimitiveType.UInt16: ctypes.c_uint16, PrimitiveType.UInt32: ctypes.c_uint32, PrimitiveType.UInt64: ctypes.c_uint64,
    PrimitiveType.Half: ctypes.c_uint16, PrimitiveType.BFloat: ctypes.c_uint16, PrimitiveType.Float: ctypes.c_float,
    PrimitiveType.Double: ctypes.c_double,
}
_NUMPY = {
    PrimitiveType.Bool: np.bool_, PrimitiveType.Int8: np.int8, PrimitiveType.Int16: np.int16, PrimitiveType.Int32: np.int32,
    PrimitiveType.Int64: np.int64, PrimitiveType.UInt8: np.uint8, PrimitiveType.UInt16: np.uint16,
    PrimitiveType.UInt32: np.uint32, PrimitiveType.UInt64: np.uint64, PrimitiveType.Half: np.float16,
    PrimitiveType.BFloat: np.uint16, PrimitiveType.Float: np.float32, PrimitiveType.Double: np.float64,
}


class CompiledSDFG:
    def __init__(self, lib_path: str, sdfg: StructuredSDFG, shape_sources: Optional[Sequence[Tuple[int, int]]] = None,
                 structure_member_info: Optional[dict] = None, output_args: Optional[Sequence[str]] = None,
                 output_shapes: Optional[Dict[str, Sequence[str]]] = None, output_strides: Optional[dict] = None):
        """shape_sources[i] = (argument index, dimension) that supplies symbol `_s<i>`;
        output_shapes[name] = list of dimension expressions over the `_s<i>`."""
        self.lib_path = lib_path
        self.sdfg = sdfg
        self.shape_sources = list(shape_sources or [])
        self.output_args = list(output_args or [])
        self.output_shapes = dict(output_shapes or {})
        runtime.lib()  # the generated library links against libdocc_rt_rocm.so: make sure it is loadable first
        self.lib = ctypes.CDLL(lib_path)
        self.func = getattr(self.lib, sdfg.name)
        self.arg_names = sdfg.arguments
        argtypes = []
        for name in self.arg_names:
            c = sdfg.containers[name]
            elem = PrimitiveType(c["element"])
            argtypes.append(ctypes.c_void_p if c["type"] == "pointer" else _CTYPES[elem])
        self.func.argtypes = argtypes
        self.func.restype = ctypes.c_void_p if sdfg.return_container else None
        self.user_args = [n for n in self.arg_names if not n.startswith("_s") and n not in self.output_args]

    def _shape_symbols(self, args: Sequence[Any]) -> Dict[str, int]:
        return {f"_s{i}": int(args[a].shape[d]) for i, (a, d) in enumerate(self.shape_sources)}

    def get_return_shape(self, *args: Any):
        if not self.output_args:
            return None
        syms = self._shape_symbols(args)
        return tuple(int(eval(e, {"__builtins__": {}}, syms)) for e in self.output_shapes[self.output_args[0]])

    def __call__(self, *args: Any):
        if len(args) != len(self.user_args):
            raise TypeError(f"{self.sdfg.name} takes {len(self.user_args)} arguments ({len(args)} given)")
        syms = self._shape_symbols(args)
        by_name: Dict[str, Any] = {}
        keep: List[np.ndarray] = []
        copies: List[Tuple[np.ndarray, np.ndarray]] = []
        for name, value in zip(self.user_args, args):
            c = self.sdfg.containers[name]
            elem = PrimitiveType(c["element"])
            if c["type"] == "pointer":
                want = _NUMPY[elem]
                arr = value if isinstance(value, np.ndarray) else np.asarray(value)
                if elem == PrimitiveType.BFloat and arr.dtype.name == "bfloat16" and arr.dtype.itemsize == 2:
                    arr = arr.view(np.uint16)      # an ml_dtypes array: the same words
                if arr.dtype != want:
                    raise TypeError(f"argument '{name}' must have dtype {np.dtype(want).name}, got {arr.dtype}")
                if not arr.flags.c_contiguous:
                    contiguous = np.ascontiguousarray(arr)
                    copies.append((arr, contiguous))
                    arr = contiguous
                keep.append(arr)
                by_name[name] = arr.ctypes.data
            else:
                by_name[name] = value
        outputs: Dict[str, np.ndarray] = {}
        for name in self.output_args:
            elem = PrimitiveType(self.sdfg.containers[name]["element"])
            shape = tuple(int(eval(e, {"__builtins__": {}}, syms)) for e in self.output_shapes[name])
            buf = runtime.result_array(shape, _NUMPY[elem])
            outputs[name] = buf
            by_name[name] = buf.ctypes.data
        call_args = [syms[n] if n in syms else by_name[n] for n in self.arg_names]
        self.func(*call_args)
        code, message = runtime.take_failure()
        if code != 0:
            raise runtime.RocmRuntimeError(self.sdfg.name, code, message)
        for original, contiguous in copies:
            if original.flags.writeable:
                np.copyto(original, contiguous)
        returned = [outputs[n] for n in self.output_args]
        if not returned:
            return None
        return returned[0] if len(returned) == 1 else tuple(returned)
