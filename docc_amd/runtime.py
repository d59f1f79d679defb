"""ctypes binding of ``libdocc_rt_rocm.so`` (``include/docc_rocm_rt.h`` and
``include/docc_rocm_ops.h``): the thin HIP runtime and the kernel launchers.

There is no fallback: when the library or a GPU is missing, calls raise.
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path
from typing import Optional

LIB_DIR = Path(__file__).resolve().parent / "lib"
LIB_PATH = LIB_DIR / "libdocc_rt_rocm.so"

NO_TRANS = 111
TRANS = 112


class RocmRuntimeError(RuntimeError):
    """A call into libdocc_rt_rocm.so returned a non-zero code."""

    def __init__(self, fn: str, code: int, message: str):
        super().__init__(f"{fn} failed with code {code}: {message}")
        self.fn = fn
        self.code = code


_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float
_f64 = ctypes.c_double

# name -> argtypes; every function returns int unless listed in _RESTYPE
_SIGNATURES = {
    "docc_rocm_init": [_int],
    "docc_rocm_device_count": [],
    "docc_rocm_device_info": [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(_int), ctypes.POINTER(_int)],
    "docc_rocm_module_load": [ctypes.c_char_p, ctypes.POINTER(_vp)],
    "docc_rocm_module_unload": [_vp],
    "docc_rocm_module_get_function": [_vp, ctypes.c_char_p, ctypes.POINTER(_vp)],
    "docc_rocm_malloc": [ctypes.POINTER(_vp), ctypes.c_size_t],
    "docc_rocm_malloc_async": [ctypes.POINTER(_vp), ctypes.c_size_t, _vp],
    "docc_rocm_free_async": [_vp, _vp],
    "docc_rocm_pool_trim": [],
    "docc_rocm_pool_stats": [ctypes.POINTER(ctypes.c_size_t)] * 3,
    "docc_rocm_pool_set_limit": [ctypes.c_size_t],
    "docc_rocm_free": [_vp],
    "docc_rocm_memset_async": [_vp, _int, ctypes.c_size_t, _vp],
    "docc_rocm_host_malloc": [ctypes.POINTER(_vp), ctypes.c_size_t],
    "docc_rocm_host_free": [_vp],
    "docc_rocm_memcpy_h2d_async": [_vp, _vp, ctypes.c_size_t, _vp],
    "docc_rocm_memcpy_d2h_async": [_vp, _vp, ctypes.c_size_t, _vp],
    "docc_rocm_memcpy_d2d_async": [_vp, _vp, ctypes.c_size_t, _vp],
    "docc_rocm_stream_create": [ctypes.POINTER(_vp)],
    "docc_rocm_stream_destroy": [_vp],
    "docc_rocm_stream_sync": [_vp],
    "docc_rocm_device_sync": [],
    "docc_rocm_launch": [_vp, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32), ctypes.c_uint32, _vp, ctypes.POINTER(_vp)],
    "docc_rocm_event_create": [ctypes.POINTER(_vp)],
    "docc_rocm_event_destroy": [_vp],
    "docc_rocm_event_record": [_vp, _vp],
    "docc_rocm_event_elapsed_ms": [_vp, _vp, ctypes.POINTER(_f32)],
    "docc_rocm_set_default_stream": [_vp],
    "docc_rocm_graph_capture_begin": [_vp],
    "docc_rocm_graph_capture_end": [ctypes.POINTER(_vp)],
    "docc_rocm_graph_launch": [_vp, _vp],
    "docc_rocm_graph_destroy": [_vp],
    "docc_rocm_report_failure": [ctypes.c_char_p, ctypes.c_char_p, _int],
    "docc_rocm_take_failure": [ctypes.c_char_p, ctypes.c_size_t],
    "docc_rocm_last_error": [],
    "docc_rocm_version": [],
    "docc_rocm_dgemm": [_vp, _int, _int, _i64, _i64, _i64, _f64, _vp, _i64, _vp, _i64, _f64, _vp, _i64],
    "docc_rocm_sgemm": [_vp, _int, _int, _i64, _i64, _i64, _f32, _vp, _i64, _vp, _i64, _f32, _vp, _i64],
    "docc_rocm_bf16gemm_f32": [_vp, _int, _int, _i64, _i64, _i64, _f32, _vp, _i64, _vp, _i64, _f32, _vp, _i64],
    "docc_rocm_dgemm_epilogue": [_vp, _int, _int, _i64, _i64, _i64, _f64, _vp, _i64, _vp, _i64, _f64, _vp, _i64, _vp, _int],
    "docc_rocm_sgemm_epilogue": [_vp, _int, _int, _i64, _i64, _i64, _f32, _vp, _i64, _vp, _i64, _f32, _vp, _i64, _vp, _int],
    "docc_rocm_bf16gemm_f32_epilogue": [_vp, _int, _int, _i64, _i64, _i64, _f32, _vp, _i64, _vp, _i64, _f32, _vp, _i64, _vp, _int],
    "docc_rocm_dgemm_batched": [_vp, _int, _int, _i64, _i64, _i64, _f64, _vp, _i64, _i64, _vp, _i64, _i64, _f64, _vp, _i64, _i64, _i64],
    "docc_rocm_sgemm_batched": [_vp, _int, _int, _i64, _i64, _i64, _f32, _vp, _i64, _i64, _vp, _i64, _i64, _f32, _vp, _i64, _i64, _i64],
    "docc_rocm_bf16gemm_f32_batched": [_vp, _int, _int, _i64, _i64, _i64, _f32, _vp, _i64, _i64, _vp, _i64, _i64, _f32, _vp, _i64, _i64, _i64],
    "docc_rocm_softmax_f32": [_vp, _i64, _i64, _vp, _vp],
    "docc_rocm_softmax": [_vp, _int, _i64, _i64, _i64, _vp, _vp],
    "docc_rocm_softmax_workspace_bytes": [_int, _i64, _i64, _i64],
    "docc_rocm_softmax_ws": [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp, _i64],
    "docc_rocm_softmax_noalloc": [_vp, _int, _i64, _i64, _i64, _vp, _vp],
    "docc_rocm_conv2d_f32": [_vp] + [_i64] * 13 + [_vp, _vp, _vp, _vp],
    "docc_rocm_conv2d_f32_pads_workspace_bytes": [_i64] * 15,
    "docc_rocm_conv2d_f32_pads": [_vp] + [_i64] * 15 + [_vp, _vp, _vp, _vp, _vp, _i64],
    "docc_rocm_conv2d_f32_grouped": [_vp] + [_i64] * 16 + [_vp, _vp, _vp, _vp, _vp, _i64],
    "docc_rocm_conv2d_f32_workspace_bytes": [_i64] * 13,
    "docc_rocm_conv2d_f32_ws": [_vp] + [_i64] * 13 + [_vp, _vp, _vp, _vp, _vp, _i64],
    "docc_rocm_attention_bf16": [_vp] + [_i64] * 5 + [_f32, _vp, _vp, _vp, _vp, _int],
    "docc_rocm_attention_bf16_workspace_bytes": [_i64] * 5 + [_int],
    "docc_rocm_attention_bf16_ws": [_vp] + [_i64] * 5 + [_f32, _vp, _vp, _vp, _vp, _int, _vp, _i64],
    "docc_rocm_attention_bf16_causal": [_vp] + [_i64] * 5 + [_f32, _vp, _vp, _vp, _vp, _int, _vp, _i64],
    "docc_rocm_convert_f32_to_bf16": [_vp, _i64, _vp, _vp],
    "docc_rocm_convert_bf16_to_f32": [_vp, _i64, _vp, _vp],
    "docc_rocm_elementwise_unary": [_vp, ctypes.c_int, ctypes.c_int, _i64, _vp, _vp],
    "docc_rocm_elementwise_binary": [_vp, ctypes.c_int, ctypes.c_int, _i64, _vp, _vp, _vp],
    "docc_rocm_elementwise_binary_scalar": [_vp, ctypes.c_int, ctypes.c_int, _i64, _vp, ctypes.c_double, ctypes.c_int, _vp],
    "docc_rocm_broadcast": [_vp, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp],
    "docc_rocm_cast": [_vp, _int, _int, _i64, _vp, _vp],
    "docc_rocm_transpose": [_vp, _int, _int, ctypes.POINTER(_i64), ctypes.POINTER(_i64), _vp, _vp],
    "docc_rocm_reduce": [_vp, ctypes.c_int, ctypes.c_int, _i64, _i64, _i64, _vp, _vp],
    "docc_rocm_elementwise_activation": [_vp, _int, _int, _i64, _vp, _vp, ctypes.c_double, ctypes.c_double],
    "docc_rocm_fill": [_vp, _int, _i64, _vp, _vp],
    "docc_rocm_dot": [_vp, _int, _i64, _vp, _i64, _vp, _i64, _vp],
    "docc_rocm_elementwise_fused": [_vp, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int, _vp, _vp, ctypes.c_double, _vp, _vp,
                                    ctypes.c_double, ctypes.c_int, _vp, _vp],
    "docc_rocm_copy_bytes": [_vp, _i64, _vp, _vp],
    "docc_rocm_mfma_probe": [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp],
    "docc_rocm_clock_probe": [_vp, ctypes.c_int, _vp],
}
_RESTYPE = {"docc_rocm_last_error": ctypes.c_char_p, "docc_rocm_version": ctypes.c_char_p,
            "docc_rocm_report_failure": None, "docc_rocm_attention_bf16_workspace_bytes": _i64, "docc_rocm_softmax_workspace_bytes": _i64,
            "docc_rocm_conv2d_f32_workspace_bytes": _i64, "docc_rocm_conv2d_f32_pads_workspace_bytes": _i64}

#: every symbol the two public headers declare
EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: ctypes.CDLL | None = None


def lib() -> ctypes.CDLL:
    """Loads ``libdocc_rt_rocm.so`` (once). Raises when it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RocmRuntimeError("load", -3, f"{LIB_PATH} is missing; run `python -m docc_amd.build`")
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPE.get(name, _int)
        _lib = handle
    return _lib


def last_error() -> str:
    return (lib().docc_rocm_last_error() or b"").decode()


def call(name: str, *args) -> None:
    """Calls an int-returning entry point and raises on a non-zero code."""
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise RocmRuntimeError(name, rc, last_error())


def take_failure() -> tuple[int, str]:
    """Collects (and clears) the failure reported by generated code, if any."""
    buf = ctypes.create_string_buffer(1024)
    code = lib().docc_rocm_take_failure(buf, 1024)
    return int(code), buf.value.decode()


def version() -> str:
    return lib().docc_rocm_version().decode()


def device_count() -> int:
    return int(lib().docc_rocm_device_count())


def init(device: int = 0) -> None:
    call("docc_rocm_init", device)


def device_info() -> dict:
    arch = ctypes.create_string_buffer(64)
    cus = _int()
    clk = _int()
    call("docc_rocm_device_info", arch, 64, ctypes.byref(cus), ctypes.byref(clk))
    return {"arch": arch.value.decode(), "compute_units": cus.value, "clock_khz": clk.value}


def malloc(nbytes: int) -> int:
    p = _vp()
    call("docc_rocm_malloc", ctypes.byref(p), nbytes)
    return p.value or 0


def free(ptr: int) -> None:
    call("docc_rocm_free", ptr)


def malloc_async(nbytes: int, stream: int = 0) -> int:
    """A block for work on `stream`: one that free_async released on that stream comes back without a wait."""
    p = _vp()
    call("docc_rocm_malloc_async", ctypes.byref(p), nbytes, stream)
    return p.value or 0


def free_async(ptr: int, stream: int = 0) -> None:
    """Returns a block whose uses were all issued on `stream`; does not wait for them."""
    call("docc_rocm_free_async", ptr, stream)


def pool_trim() -> None:
    """Returns the device blocks that free() kept to the driver."""
    call("docc_rocm_pool_trim")


def pool_stats() -> tuple[int, int, int]:
    """(cached bytes, cached blocks, limit in bytes) of the device block cache."""
    a, b, c = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    call("docc_rocm_pool_stats", ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return a.value, b.value, c.value


def pool_set_limit(nbytes: int) -> None:
    call("docc_rocm_pool_set_limit", nbytes)


def memset(ptr: int, value: int, nbytes: int, stream: int = 0) -> None:
    """Fills `nbytes` bytes of device memory with the byte `value`, in stream order."""
    call("docc_rocm_memset_async", ptr, value, nbytes, stream)


def memcpy_d2d(dst_dev: int, src_dev: int, nbytes: int, stream: int = 0) -> None:
    call("docc_rocm_memcpy_d2d_async", dst_dev, src_dev, nbytes, stream)


def memcpy_h2d(dst_dev: int, src_host: int, nbytes: int, stream: int = 0) -> None:
    call("docc_rocm_memcpy_h2d_async", dst_dev, src_host, nbytes, stream)


def memcpy_d2h(dst_host: int, src_dev: int, nbytes: int, stream: int = 0) -> None:
    call("docc_rocm_memcpy_d2h_async", dst_host, src_dev, nbytes, stream)


def stream_sync(stream: int = 0) -> None:
    call("docc_rocm_stream_sync", stream)


def device_sync() -> None:
    call("docc_rocm_device_sync")


class Event:
    """HIP event recorded on an explicit stream."""

    def __init__(self):
        p = _vp()
        call("docc_rocm_event_create", ctypes.byref(p))
        self.handle = p.value

    def record(self, stream: int = 0) -> None:
        call("docc_rocm_event_record", self.handle, stream)

    def elapsed_ms(self, stop: "Event") -> float:
        ms = _f32()
        call("docc_rocm_event_elapsed_ms", self.handle, stop.handle, ctypes.byref(ms))
        return float(ms.value)

    def __del__(self):
        try:
            if self.handle:
                lib().docc_rocm_event_destroy(self.handle)
        except Exception:
            pass


# --- kernel launchers on raw device pointers -------------------------------

def dgemm(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, trans_a=NO_TRANS, trans_b=NO_TRANS, stream=0) -> None:
    call("docc_rocm_dgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)


def sgemm(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, trans_a=NO_TRANS, trans_b=NO_TRANS, stream=0) -> None:
    call("docc_rocm_sgemm", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)


def bf16gemm_f32(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, trans_a=NO_TRANS, trans_b=NO_TRANS, stream=0) -> None:
    call("docc_rocm_bf16gemm_f32", stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)


def gemm_epilogue(kind, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias=None, activation=None, trans_a=NO_TRANS,
                  trans_b=NO_TRANS, stream=0) -> None:
    """C = act(alpha * op(A) op(B) + beta * C + bias[column]); kind "d", "s" or "b" (bf16 inputs),
    bias a device address or None, activation the name of a unary operation or None."""
    fn = {"d": "docc_rocm_dgemm_epilogue", "s": "docc_rocm_sgemm_epilogue", "b": "docc_rocm_bf16gemm_f32_epilogue"}[kind]
    act = -1 if activation is None else (UNARY_OPS[activation] if isinstance(activation, str) else activation)
    call(fn, stream, trans_a, trans_b, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias or None, act)


def gemm_batched(kind, batch, m, n, k, alpha, A, lda, stride_a, B, ldb, stride_b, beta, C, ldc, stride_c, trans_a=NO_TRANS,
                 trans_b=NO_TRANS, stream=0) -> None:
    """C[z] = alpha * op(A[z]) op(B[z]) + beta * C[z] for z < batch in one launch; strides in elements, 0 shares
    an input across the batch; kind "d", "s" or "b" (bf16 inputs)."""
    fn = {"d": "docc_rocm_dgemm_batched", "s": "docc_rocm_sgemm_batched", "b": "docc_rocm_bf16gemm_f32_batched"}[kind]
    call(fn, stream, trans_a, trans_b, m, n, k, alpha, A, lda, stride_a, B, ldb, stride_b, beta, C, ldc, stride_c, batch)


def softmax(precision, outer, reduce, inner, X, Y, stream=0) -> None:
    """Softmax over the middle extent of an [outer, reduce, inner] view; precision 32 or 64."""
    call("docc_rocm_softmax", stream, precision, outer, reduce, inner, X, Y)


def softmax_workspace_bytes(precision, outer, reduce, inner) -> int:
    return int(lib().docc_rocm_softmax_workspace_bytes(precision, outer, reduce, inner))


def softmax_ws(precision, outer, reduce, inner, X, Y, workspace, workspace_bytes, stream=0) -> None:
    """docc_rocm_softmax with the partial results of the sliced form in `workspace` (device memory of the caller)."""
    call("docc_rocm_softmax_ws", stream, precision, outer, reduce, inner, X, Y, workspace or None, workspace_bytes)


def softmax_noalloc(precision, outer, reduce, inner, X, Y, stream=0) -> None:
    """docc_rocm_softmax through the entry point that allocates nothing (fixed 1 MiB of partial results)."""
    call("docc_rocm_softmax_noalloc", stream, precision, outer, reduce, inner, X, Y)


def softmax_f32(rows, cols, X, Y, stream=0) -> None:
    call("docc_rocm_softmax_f32", stream, rows, cols, X, Y)


def conv2d_f32(N, C, H, W, OC, KH, KW, stride, pad, dilation, X, Wt, bias, Y, stream=0) -> None:
    call("docc_rocm_conv2d_f32", stream, N, C, H, W, OC, KH, KW, stride[0], stride[1], pad[0], pad[1],
         dilation[0], dilation[1], X, Wt, bias or None, Y)


def conv2d_f32_workspace_bytes(N, C, H, W, OC, KH, KW, stride, pad, dilation) -> int:
    return int(lib().docc_rocm_conv2d_f32_workspace_bytes(N, C, H, W, OC, KH, KW, stride[0], stride[1], pad[0], pad[1], dilation[0], dilation[1]))


def conv2d_f32_ws(N, C, H, W, OC, KH, KW, stride, pad, dilation, X, Wt, bias, Y, workspace, workspace_bytes, stream=0) -> None:
    """conv2d_f32 with device memory for a column matrix (conv2d_f32_workspace_bytes(...) bytes, 0 = none needed)."""
    call("docc_rocm_conv2d_f32_ws", stream, N, C, H, W, OC, KH, KW, stride[0], stride[1], pad[0], pad[1],
         dilation[0], dilation[1], X, Wt, bias or None, Y, workspace or None, workspace_bytes)


def conv2d_f32_pads_workspace_bytes(N, C, H, W, OC, KH, KW, stride, pads, dilation) -> int:
    """`pads`: (top, left, bottom, right), the node's order (begins, then ends)."""
    return int(lib().docc_rocm_conv2d_f32_pads_workspace_bytes(N, C, H, W, OC, KH, KW, stride[0], stride[1], pads[0], pads[1], pads[2], pads[3],
                                                                dilation[0], dilation[1]))


def conv2d_f32_pads(N, C, H, W, OC, KH, KW, stride, pads, dilation, X, Wt, bias, Y, workspace=0, workspace_bytes=0, stream=0) -> None:
    """The convolution with a begin and an end pad per axis: `pads` = (top, left, bottom, right)."""
    call("docc_rocm_conv2d_f32_pads", stream, N, C, H, W, OC, KH, KW, stride[0], stride[1], pads[0], pads[1], pads[2], pads[3],
         dilation[0], dilation[1], X, Wt, bias or None, Y, workspace or None, workspace_bytes)


def conv2d_f32_grouped(N, C, H, W, OC, KH, KW, stride, pads, dilation, group, X, Wt, bias, Y, workspace=0, workspace_bytes=0, stream=0) -> None:
    """The convolution with the node's `group`: weights [OC, C / group, KH, KW]; `pads` = (top, left, bottom, right)."""
    call("docc_rocm_conv2d_f32_grouped", stream, N, C, H, W, OC, KH, KW, stride[0], stride[1], pads[0], pads[1], pads[2], pads[3],
         dilation[0], dilation[1], group, X, Wt, bias or None, Y, workspace or None, workspace_bytes)


def attention_bf16(B, H, SQ, SKV, D, scale, Q, K, V, O, out_bf16=False, stream=0) -> None:
    call("docc_rocm_attention_bf16", stream, B, H, SQ, SKV, D, scale, Q, K, V, O, 1 if out_bf16 else 0)


def attention_bf16_workspace_bytes(B, H, SQ, SKV, D, out_bf16=False) -> int:
    return int(lib().docc_rocm_attention_bf16_workspace_bytes(B, H, SQ, SKV, D, 1 if out_bf16 else 0))


def attention_bf16_ws(B, H, SQ, SKV, D, scale, Q, K, V, O, workspace, workspace_bytes, out_bf16=False, stream=0) -> None:
    """Attention for any head dimension; `workspace` is device memory of attention_bf16_workspace_bytes(...) bytes."""
    call("docc_rocm_attention_bf16_ws", stream, B, H, SQ, SKV, D, scale, Q, K, V, O, 1 if out_bf16 else 0, workspace or None,
         workspace_bytes)


def attention_bf16_causal(B, H, SQ, SKV, D, scale, Q, K, V, O, workspace=0, workspace_bytes=0, out_bf16=False, stream=0) -> None:
    """Attention in which query i sees the keys j <= i; head dims up to 128 (`workspace` as for attention_bf16_ws)."""
    call("docc_rocm_attention_bf16_causal", stream, B, H, SQ, SKV, D, scale, Q, K, V, O, 1 if out_bf16 else 0, workspace or None,
         workspace_bytes)


def copy_bytes(nbytes, src, dst, stream=0) -> None:
    call("docc_rocm_copy_bytes", stream, nbytes, src, dst)


UNARY_OPS = {"abs": 0, "exp": 1, "relu": 2, "sigmoid": 3, "sqrt": 4, "tanh": 5, "erf": 6}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "maximum": 4, "minimum": 5, "pow": 6}


def elementwise_unary(op, precision, n, X, Y, stream=0) -> None:
    call("docc_rocm_elementwise_unary", stream, UNARY_OPS[op] if isinstance(op, str) else op, precision, n, X, Y)


def elementwise_binary(op, precision, n, A, B, Y, stream=0) -> None:
    call("docc_rocm_elementwise_binary", stream, BINARY_OPS[op] if isinstance(op, str) else op, precision, n, A, B, Y)


def elementwise_binary_scalar(op, precision, n, A, scalar, Y, scalar_is_lhs=False, stream=0) -> None:
    """Y = f(A, scalar), or f(scalar, A) when scalar_is_lhs."""
    call("docc_rocm_elementwise_binary_scalar", stream, BINARY_OPS[op] if isinstance(op, str) else op, precision, n, A,
         float(scalar), int(bool(scalar_is_lhs)), Y)


def broadcast(precision, in_shape, out_shape, X, Y, stream=0) -> None:
    rank = len(out_shape)
    in_shape = (1,) * (rank - len(in_shape)) + tuple(in_shape)   # numpy rule: missing leading dimensions are 1
    ins = (ctypes.c_int64 * rank)(*in_shape)
    outs = (ctypes.c_int64 * rank)(*out_shape)
    call("docc_rocm_broadcast", stream, precision, rank, ctypes.addressof(ins), ctypes.addressof(outs), X, Y)


REDUCE_OPS = {"sum": 0, "max": 1, "min": 2, "mean": 3}


ACTIVATION_OPS = {"elu": 7, "leaky_relu": 8, "hard_sigmoid": 9}


def elementwise_activation(op, precision, n, X, Y, alpha, beta=0.0, stream=0) -> None:
    """Y[i] = f(X[i]; alpha, beta) for ml::Elu / ml::LeakyReLU / ml::HardSigmoid."""
    call("docc_rocm_elementwise_activation", stream, ACTIVATION_OPS[op] if isinstance(op, str) else op, precision, n, X, Y, float(alpha), float(beta))


def fill(value, n, Y, stream=0) -> None:
    """All n elements at Y become `value`, a numpy scalar (its item size is the element size)."""
    import numpy as np

    v = np.asarray(value).reshape(1)
    call("docc_rocm_fill", stream, v.dtype.itemsize, n, v.ctypes.data, Y)


def dot(precision, n, x, incx, y, incy, stream=0):
    """sum_i x[i*incx] * y[i*incy] (device vectors), returned as a Python float once the stream has run."""
    out = (ctypes.c_double if precision == 64 else ctypes.c_float)(0)
    call("docc_rocm_dot", stream, precision, n, x, incx, y, incy, ctypes.addressof(out))
    return out.value


def reduce(op, precision, outer, extent, inner, X, Y, stream=0) -> None:
    """Y[o, i] = op over r of X[o, r, i] for X seen as [outer, extent, inner]."""
    call("docc_rocm_reduce", stream, REDUCE_OPS[op] if isinstance(op, str) else op, precision, outer, extent, inner, X, Y)


def elementwise_fused(precision, shape, binary, a, a_shape, b, b_shape, post, Y, stream=0) -> None:
    """Y = post_k(...post_1(binary(a, b))) over `shape`. `a` / `b`: a device address with its shape
    (left-padded to the output rank) or a Python number with shape None; `binary` None starts the
    chain from `a`; `post`: names of unary operations."""
    rank = len(shape)
    dims = (ctypes.c_int64 * rank)(*shape)

    def operand(value, value_shape):
        if value_shape is None:
            return None, 0, float(value)
        padded = (1,) * (rank - len(value_shape)) + tuple(value_shape)
        arr = (ctypes.c_int64 * rank)(*padded)
        return arr, value, 0.0

    a_arr, a_ptr, a_val = operand(a, a_shape)
    b_arr, b_ptr, b_val = operand(b, b_shape) if binary is not None else (None, 0, 0.0)
    ops = (ctypes.c_int * max(len(post), 1))(*[UNARY_OPS[o] if isinstance(o, str) else o for o in post])
    code = -1 if binary is None else (BINARY_OPS[binary] if isinstance(binary, str) else binary)
    call("docc_rocm_elementwise_fused", stream, precision, rank, ctypes.addressof(dims), code,
         ctypes.addressof(a_arr) if a_arr is not None else None, a_ptr, a_val,
         ctypes.addressof(b_arr) if b_arr is not None else None, b_ptr, b_val, len(post), ctypes.addressof(ops), Y)


CAST_TYPES = {"f16": 0, "bf16": 1, "f32": 2, "f64": 3, "i32": 4, "i64": 5}


def cast(src_type, dst_type, n, X, Y, stream=0) -> None:
    """Y[i] = (dst_type) X[i]; types by name (CAST_TYPES) or code."""
    code = lambda t: CAST_TYPES[t] if isinstance(t, str) else t
    call("docc_rocm_cast", stream, code(src_type), code(dst_type), n, X, Y)


def transpose(element_bytes, shape, perm, X, Y, stream=0) -> None:
    """Y = X with its axes permuted: Y.shape[i] = shape[perm[i]]."""
    rank = len(shape)
    call("docc_rocm_transpose", stream, element_bytes, rank, (_i64 * max(rank, 1))(*shape), (_i64 * max(rank, 1))(*perm), X, Y)


def mfma_probe(precision, waves_per_simd, iters, operands, sink, stream=0) -> float:
    """Launches the MFMA rate probe; returns the floating-point operations of the launch."""
    flop = ctypes.c_double(0.0)
    call("docc_rocm_mfma_probe", stream, precision, waves_per_simd, iters, operands, sink, ctypes.addressof(flop))
    return flop.value


def clock_probe(microseconds, mhz, stream=0) -> None:
    """One wave samples the shader clock for `microseconds`; mhz: device address of one float."""
    call("docc_rocm_clock_probe", stream, microseconds, mhz)


def stream_create() -> int:
    """A non-blocking stream (it does not wait for the null stream)."""
    h = _vp()
    call("docc_rocm_stream_create", ctypes.byref(h))
    return h.value


def stream_destroy(stream: int) -> None:
    call("docc_rocm_stream_destroy", stream)


def set_default_stream(stream: int = 0) -> None:
    """Names the stream that stands in for the null stream in this thread's calls of the runtime (generated code
    passes the null stream everywhere); 0 restores the null stream."""
    call("docc_rocm_set_default_stream", stream)


class Graph:
    """A recorded run of runtime calls (kernels, device copies, cached allocations) that replays with one submission.

        stream = runtime.stream_create()
        runtime.set_default_stream(stream); f(); runtime.stream_sync(stream)   # once, outside the record
        with runtime.Graph.capture(stream) as graph:
            f()                           # recorded, not run
        graph.launch(); runtime.stream_sync(stream)

    The device blocks `f` allocates while it is recorded belong to the graph until destroy(); the buffers it reads and
    writes must stay where they are. launch() without a stream replays on the stream of the capture."""

    def __init__(self, stream: int):
        self.stream = stream
        self.handle = None

    class _Capture:
        def __init__(self, graph: "Graph"):
            self.graph = graph

        def __enter__(self) -> "Graph":
            call("docc_rocm_graph_capture_begin", self.graph.stream)
            return self.graph

        def __exit__(self, kind, value, trace) -> bool:
            h = _vp()
            code = lib().docc_rocm_graph_capture_end(ctypes.byref(h))
            if kind is None:
                failed, message = take_failure()    # a failing call in generated code ends that function early
                if code != 0:
                    raise RocmRuntimeError("docc_rocm_graph_capture_end", code, last_error())
                self.graph.handle = h.value
                if failed != 0:
                    self.graph.destroy()
                    raise RocmRuntimeError("graph capture", failed, message)
            elif code == 0 and h.value:
                lib().docc_rocm_graph_destroy(h.value)
            return False

    @classmethod
    def capture(cls, stream: int) -> "Graph._Capture":
        return cls._Capture(cls(stream))

    def launch(self, stream: Optional[int] = None) -> None:
        if not self.handle:
            raise RuntimeError("the graph holds no record")
        call("docc_rocm_graph_launch", self.handle, self.stream if stream is None else stream)

    def destroy(self) -> None:
        if self.handle:
            handle, self.handle = self.handle, None
            call("docc_rocm_graph_destroy", handle)

    def __del__(self):
        try:
            if self.handle:
                lib().docc_rocm_graph_destroy(self.handle)
        except Exception:
            pass


def convert_f32_to_bf16(count, src, dst, stream=0) -> None:
    call("docc_rocm_convert_f32_to_bf16", stream, count, src, dst)


def convert_bf16_to_f32(count, src, dst, stream=0) -> None:
    call("docc_rocm_convert_bf16_to_f32", stream, count, src, dst)


# ---- result arrays in pinned host memory -------------------------------------------------------
#
# A device-to-host copy into a fresh np.empty array pays for a page fault per 4 KiB and goes through the
# driver's staging of pageable memory: 12.8 ms for 128 MiB measured on an MI355X host against 2.3 ms into
# pinned memory. Results of compiled functions are therefore allocated with hipHostMalloc; when the last
# view of such an array dies its block goes to a free list, so that a caller in a loop pins memory once.

_PINNED_MIN_BYTES = 1 << 20
_pinned_free: dict[int, list[int]] = {}
_pinned_cached = 0


def _pinned_limit() -> int:
    return int(os.environ.get("DOCC_ROCM_PINNED_RESULT_BYTES", 1 << 30))


def _pinned_release(ptr: int, nbytes: int) -> None:
    global _pinned_cached
    if _lib is None:
        return
    if _pinned_cached + nbytes <= _pinned_limit():
        _pinned_free.setdefault(nbytes, []).append(ptr)
        _pinned_cached += nbytes
    else:
        _lib.docc_rocm_host_free(ptr)


def pinned_trim() -> None:
    """Returns the cached pinned blocks to the driver."""
    global _pinned_cached
    for blocks in _pinned_free.values():
        for ptr in blocks:
            lib().docc_rocm_host_free(ptr)
    _pinned_free.clear()
    _pinned_cached = 0


def result_array(shape, dtype):
    """An uninitialised C-order ndarray for a result that the device will write: in pinned host memory when it is
    large enough to matter and a device is present (DOCC_ROCM_PINNED_RESULT_BYTES=0 switches that off), else
    np.empty. The array owns its memory through its base object, like any other ndarray."""
    import weakref

    import numpy as np

    global _pinned_cached
    dtype = np.dtype(dtype)
    nbytes = int(np.prod(shape, dtype=np.int64)) * dtype.itemsize
    if nbytes < _PINNED_MIN_BYTES or _pinned_limit() <= 0 or device_count() <= 0:
        return np.empty(shape, dtype=dtype)
    rounded = (nbytes + 4095) & ~4095
    blocks = _pinned_free.get(rounded)
    if blocks:
        ptr = blocks.pop()
        _pinned_cached -= rounded
    else:
        p = _vp()
        try:
            call("docc_rocm_host_malloc", ctypes.byref(p), rounded)
        except RocmRuntimeError:
            pinned_trim()
            return np.empty(shape, dtype=dtype)
        ptr = p.value
    owner = (ctypes.c_char * rounded).from_address(ptr)
    # not at interpreter exit: the HIP runtime may be gone by then, and the process is about to end anyway
    weakref.finalize(owner, _pinned_release, ptr, rounded).atexit = False
    return np.frombuffer(owner, dtype=dtype, count=nbytes // dtype.itemsize).reshape(shape)
