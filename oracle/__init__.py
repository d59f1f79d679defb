"""ctypes access to the CPU oracle (``oracle/docc_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU
baseline. The product (``docc_amd``) never imports this package.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "libdocc_oracle.so"

NO_TRANS = 111
TRANS = 112


def build(arch: str | None = None, out: str | None = None) -> Path:
    """Compiles the oracle (``make -C oracle``); returns the library path."""
    cmd = ["make", "-B", "-C", str(_DIR)]
    if arch:
        cmd.append(f"ARCH={arch}")
    if out:
        cmd.append(f"OUT={out}")
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + proc.stdout + proc.stderr)
    return Path(out) if out else _LIB_PATH


_i64 = ctypes.c_int64
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def _declare(lib: ctypes.CDLL) -> ctypes.CDLL:
    lib.oracle_max_threads.restype = ctypes.c_int
    lib.oracle_set_threads.argtypes = [ctypes.c_int]
    lib.oracle_f32_to_bf16_array.argtypes = [_i64, _f32p, _u16p]
    lib.oracle_bf16_to_f32_array.argtypes = [_i64, _u16p, _f32p]
    for name, ptr, sc in (("f64", _f64p, ctypes.c_double), ("f32", _f32p, ctypes.c_float)):
        getattr(lib, f"oracle_gemm_expanded_{name}").argtypes = [_i64, _i64, _i64, sc, ptr, _i64, ptr, _i64, sc, ptr, _i64]
        getattr(lib, f"oracle_gemm_blas_{name}").argtypes = [ctypes.c_int, ctypes.c_int, _i64, _i64, _i64, sc, ptr, _i64, ptr, _i64, sc, ptr, _i64]
    lib.oracle_gemm_blas_f64_ld.argtypes = lib.oracle_gemm_blas_f64.argtypes
    lib.oracle_gemm_blas_f32_acc64.argtypes = lib.oracle_gemm_blas_f32.argtypes
    lib.oracle_gemm_bf16_f32.argtypes = [ctypes.c_int, ctypes.c_int, _i64, _i64, _i64, ctypes.c_float, _u16p, _i64, _u16p, _i64, ctypes.c_float, _f32p, _i64]
    for name in ("oracle_softmax_expanded_f32", "oracle_softmax_numpy_f32"):
        getattr(lib, name).argtypes = [_i64, _i64, _f32p, _f32p]
        getattr(lib, name).restype = ctypes.c_int
    lib.oracle_softmax_expanded_f64.argtypes = [_i64, _i64, _f64p, _f64p]
    lib.oracle_softmax_expanded_f64.restype = ctypes.c_int
    lib.oracle_conv_out_dim.argtypes = [_i64] * 6
    lib.oracle_conv_out_dim.restype = _i64
    lib.oracle_conv2d_f32.argtypes = [_i64] * 13 + [_f32p, _f32p, _f32p, _f32p]
    lib.oracle_conv2d_f32_pads.argtypes = [_i64] * 15 + [_f32p, _f32p, _f32p, _f32p]
    lib.oracle_attention_bf16.argtypes = [_i64] * 5 + [ctypes.c_float, _u16p, _u16p, _u16p, _f32p]
    lib.oracle_attention_bf16.restype = ctypes.c_int
    lib.oracle_elementwise_unary_f32.argtypes = [ctypes.c_int, _i64, _f32p, _f32p]
    lib.oracle_elementwise_unary_f64.argtypes = [ctypes.c_int, _i64, _f64p, _f64p]
    lib.oracle_elementwise_activation_f32.argtypes = [ctypes.c_int, _i64, _f32p, _f32p, ctypes.c_float, ctypes.c_float]
    lib.oracle_elementwise_activation_f64.argtypes = [ctypes.c_int, _i64, _f64p, _f64p, ctypes.c_double, ctypes.c_double]
    lib.oracle_dot_f32.argtypes = [_i64, _f32p, _i64, _f32p, _i64]
    lib.oracle_dot_f32.restype = ctypes.c_float
    lib.oracle_dot_f64.argtypes = [_i64, _f64p, _i64, _f64p, _i64]
    lib.oracle_dot_f64.restype = ctypes.c_double
    lib.oracle_elementwise_binary_f32.argtypes = [ctypes.c_int, _i64, _f32p, _f32p, _f32p]
    lib.oracle_elementwise_binary_f64.argtypes = [ctypes.c_int, _i64, _f64p, _f64p, _f64p]
    lib.oracle_broadcast.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(_i64), ctypes.POINTER(_i64), ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_transpose.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(_i64), ctypes.POINTER(_i64), ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_reduce_f32.argtypes = [ctypes.c_int, _i64, _i64, _i64, _f32p, _f32p]
    lib.oracle_reduce_f64.argtypes = [ctypes.c_int, _i64, _i64, _i64, _f64p, _f64p]
    return lib


_lib: ctypes.CDLL | None = None


def load(path: str | Path | None = None) -> ctypes.CDLL:
    """Loads the oracle library, building it first when it does not exist."""
    global _lib
    if path is not None:
        return _declare(ctypes.CDLL(str(path)))
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = _declare(ctypes.CDLL(str(_LIB_PATH)))
    return _lib


def _p(a: np.ndarray, ptr):
    return a.ctypes.data_as(ptr)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def set_threads(n: int) -> None:
    load().oracle_set_threads(int(n))


def max_threads() -> int:
    return int(load().oracle_max_threads())


def f32_to_bf16(x) -> np.ndarray:
    """fp32 array -> bf16 bits (uint16), round to nearest even."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    load().oracle_f32_to_bf16_array(x.size, _p(x, _f32p), _p(out, _u16p))
    return out


def bf16_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    load().oracle_bf16_to_f32_array(h.size, _p(h, _u16p), _p(out, _f32p))
    return out


def _gemm_dims(A, B, trans_a, trans_b):
    m, k = (A.shape[1], A.shape[0]) if trans_a == TRANS else A.shape
    k2, n = (B.shape[1], B.shape[0]) if trans_b == TRANS else B.shape
    if k != k2:
        raise ValueError(f"inner dimensions differ: {k} vs {k2}")
    return m, n, k


def gemm(A, B, C=None, alpha=1.0, beta=0.0, trans_a=NO_TRANS, trans_b=NO_TRANS, variant="blas", lib=None) -> np.ndarray:
    """C = alpha*op(A)*op(B) + beta*C on fp64 or fp32 arrays.

    variant: "blas" (cblas semantics), "expanded" (the reference's loop nest,
    NN only), "ld" (fp64 data, long-double accumulate) or "acc64" (fp32 data,
    fp64 accumulate).
    """
    lib = lib or load()
    dt = np.float64 if np.asarray(A).dtype == np.float64 else np.float32
    A = _c(A, dt)
    B = _c(B, dt)
    m, n, k = _gemm_dims(A, B, trans_a, trans_b)
    out = np.zeros((m, n), dt) if C is None else np.array(C, dtype=dt, order="C", copy=True)
    ptr = _f64p if dt == np.float64 else _f32p
    sfx = "f64" if dt == np.float64 else "f32"
    lda, ldb, ldc = max(A.shape[1], 1), max(B.shape[1], 1), max(n, 1)
    if variant == "expanded":
        if trans_a != NO_TRANS or trans_b != NO_TRANS:
            raise ValueError("the reference expands NoTrans/NoTrans only")
        getattr(lib, f"oracle_gemm_expanded_{sfx}")(m, n, k, alpha, _p(A, ptr), lda, _p(B, ptr), ldb, beta, _p(out, ptr), ldc)
        return out
    name = {"blas": f"oracle_gemm_blas_{sfx}", "ld": "oracle_gemm_blas_f64_ld", "acc64": "oracle_gemm_blas_f32_acc64"}[variant]
    getattr(lib, name)(trans_a, trans_b, m, n, k, alpha, _p(A, ptr), lda, _p(B, ptr), ldb, beta, _p(out, ptr), ldc)
    return out


def gemm_bf16(A_bits, B_bits, C=None, alpha=1.0, beta=0.0, trans_a=NO_TRANS, trans_b=NO_TRANS, lib=None) -> np.ndarray:
    """bf16 bits in, fp32 accumulate and output."""
    lib = lib or load()
    A = _c(A_bits, np.uint16)
    B = _c(B_bits, np.uint16)
    m, n, k = _gemm_dims(A, B, trans_a, trans_b)
    out = np.zeros((m, n), np.float32) if C is None else np.array(C, dtype=np.float32, order="C", copy=True)
    lib.oracle_gemm_bf16_f32(trans_a, trans_b, m, n, k, alpha, _p(A, _u16p), max(A.shape[1], 1), _p(B, _u16p), max(B.shape[1], 1), beta, _p(out, _f32p), max(n, 1))
    return out


def softmax(X, variant="numpy", lib=None) -> np.ndarray:
    """Row softmax over the last axis of an fp32 array of any rank."""
    lib = lib or load()
    X = _c(X, np.float32)
    cols = X.shape[-1] if X.ndim else 1
    rows = X.size // cols if cols else 0
    out = np.empty_like(X)
    fn = lib.oracle_softmax_numpy_f32 if variant == "numpy" else lib.oracle_softmax_expanded_f32
    if fn(rows, cols, _p(X, _f32p), _p(out, _f32p)) != 0:
        raise MemoryError("oracle softmax could not allocate its temporaries")
    return out


def softmax_axes(X, axes=(-1,), lib=None) -> np.ndarray:
    """Softmax over any set of axes of an fp32 or fp64 array, the way the node's expansion computes it
    (reference softmax_node.cpp:38-265): the reduced axes are moved to the end in ascending order, which is
    the order the reduce nests visit them in, and the row form runs on that view."""
    lib = lib or load()
    X = np.asarray(X)
    dt = np.float64 if X.dtype == np.float64 else np.float32
    axes = sorted({a % X.ndim for a in axes})
    kept = [d for d in range(X.ndim) if d not in axes]
    perm = kept + axes
    Xt = _c(np.transpose(X, perm), dt)
    cols = int(np.prod([X.shape[a] for a in axes])) if axes else 1
    rows = Xt.size // cols if cols else 0
    out = np.empty_like(Xt)
    if dt == np.float64:
        rc = lib.oracle_softmax_expanded_f64(rows, cols, _p(Xt, _f64p), _p(out, _f64p))
    else:
        rc = lib.oracle_softmax_expanded_f32(rows, cols, _p(Xt, _f32p), _p(out, _f32p))
    if rc != 0:
        raise MemoryError("oracle softmax could not allocate its temporaries")
    return np.ascontiguousarray(np.transpose(out, np.argsort(perm)))


def conv_out_dim(d_in, pad, dilation, kernel, stride) -> int:
    return int(load().oracle_conv_out_dim(d_in, pad, pad, dilation, kernel, stride))


def conv2d(X, W, bias=None, stride=(1, 1), pad=(0, 0), dilation=(1, 1), lib=None, group=1) -> np.ndarray:
    """`pad`: (height, width) on both sides, or (top, left, bottom, right) as the node orders them (begins, then ends).
    `group` (reference conv_node.cpp:376-377: W [OC][C / group][KH][KW]; ONNX Conv): output channel oc belongs to group
    oc / (OC / group) and reads that group's C / group input channels - the convolution below on each group's slices."""
    lib = lib or load()
    X = _c(X, np.float32)
    W = _c(W, np.float32)
    N, C, H, Wd = X.shape
    OC, C2, KH, KW = W.shape
    if group != 1:
        if group < 1 or C % group or OC % group or C2 * group != C:
            raise ValueError("group must divide the channels, and W must hold C / group input channels")
        cg, og = C // group, OC // group
        parts = [conv2d(X[:, g * cg:(g + 1) * cg], W[g * og:(g + 1) * og], None if bias is None else np.asarray(bias)[g * og:(g + 1) * og],
                        stride, pad, dilation, lib) for g in range(group)]
        return np.concatenate(parts, axis=1)
    if C2 != C:
        raise ValueError("W holds another number of input channels than X (pass group)")
    pad = tuple(pad) if len(pad) == 4 else (pad[0], pad[1], pad[0], pad[1])
    OH = int(lib.oracle_conv_out_dim(H, pad[0], pad[2], dilation[0], KH, stride[0]))
    OW = int(lib.oracle_conv_out_dim(Wd, pad[1], pad[3], dilation[1], KW, stride[1]))
    Y = np.empty((N, OC, OH, OW), np.float32)
    b = None if bias is None else _c(bias, np.float32)
    lib.oracle_conv2d_f32_pads(N, C, H, Wd, OC, KH, KW, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3], dilation[0], dilation[1],
                               _p(X, _f32p), _p(W, _f32p), _p(b, _f32p) if b is not None else None, _p(Y, _f32p))
    return Y


def attention(Q_bits, K_bits, V_bits, scale=None, lib=None, causal=False) -> np.ndarray:
    """bf16 bits [B,H,S,D] in, fp32 [B,H,SQ,D] out. `causal`: query i attends to the keys j <= i (torch's is_causal, the
    mask aligned at the top left) - stated as what it means: row i is the attention of query i over the first i + 1 keys."""
    lib = lib or load()
    Q = _c(Q_bits, np.uint16)
    K = _c(K_bits, np.uint16)
    V = _c(V_bits, np.uint16)
    B, H, SQ, D = Q.shape
    SKV = K.shape[2]
    if scale is None:
        scale = 1.0 / float(np.sqrt(D))
    if causal:
        rows = [attention(Q[:, :, i:i + 1], K[:, :, :min(i + 1, SKV)], V[:, :, :min(i + 1, SKV)], scale, lib) for i in range(SQ)]
        return np.concatenate(rows, axis=2) if rows else np.empty((B, H, 0, D), np.float32)
    O = np.empty((B, H, SQ, D), np.float32)
    if lib.oracle_attention_bf16(B, H, SQ, SKV, D, scale, _p(Q, _u16p), _p(K, _u16p), _p(V, _u16p), _p(O, _f32p)) != 0:
        raise MemoryError("oracle attention could not allocate its scratch row")
    return O


UNARY_OPS = {"abs": 0, "exp": 1, "relu": 2, "sigmoid": 3, "sqrt": 4, "tanh": 5, "erf": 6}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "maximum": 4, "minimum": 5, "pow": 6}


def elementwise_unary(op: str, X, lib=None) -> np.ndarray:
    """Y[i] = f(X[i]) for fp32 or fp64 X of any shape."""
    lib = lib or load()
    dt = np.float64 if np.asarray(X).dtype == np.float64 else np.float32
    X = _c(X, dt)
    out = np.empty_like(X)
    ptr = _f64p if dt == np.float64 else _f32p
    fn = lib.oracle_elementwise_unary_f64 if dt == np.float64 else lib.oracle_elementwise_unary_f32
    if fn(UNARY_OPS[op], X.size, _p(X, ptr), _p(out, ptr)) != 0:
        raise ValueError(f"unknown unary operation {op}")
    return out


ACTIVATION_OPS = {"elu": 7, "leaky_relu": 8, "hard_sigmoid": 9}


def elementwise_activation(op: str, X, alpha, beta=0.0, lib=None) -> np.ndarray:
    """ml::Elu / ml::LeakyReLU / ml::HardSigmoid with their scalar operands, fp32 or fp64 X of any shape."""
    lib = lib or load()
    dt = np.float64 if np.asarray(X).dtype == np.float64 else np.float32
    X = _c(X, dt)
    out = np.empty_like(X)
    ptr = _f64p if dt == np.float64 else _f32p
    fn = lib.oracle_elementwise_activation_f64 if dt == np.float64 else lib.oracle_elementwise_activation_f32
    if fn(ACTIVATION_OPS[op], X.size, _p(X, ptr), _p(out, ptr), float(alpha), float(beta)) != 0:
        raise ValueError(f"unknown activation {op}")
    return out


def dot(x, y, incx=1, incy=1, n=None, lib=None):
    """DOT::BLAS: sum_i x[i*incx] * y[i*incy], added left to right in the element type."""
    lib = lib or load()
    dt = np.float64 if np.asarray(x).dtype == np.float64 else np.float32
    x, y = _c(x, dt).ravel(), _c(y, dt).ravel()
    if n is None:
        n = min((x.size + incx - 1) // incx if incx else x.size, (y.size + incy - 1) // incy if incy else y.size)
    ptr = _f64p if dt == np.float64 else _f32p
    fn = lib.oracle_dot_f64 if dt == np.float64 else lib.oracle_dot_f32
    return dt(fn(n, _p(x, ptr), incx, _p(y, ptr), incy))


def elementwise_binary(op: str, A, B, lib=None) -> np.ndarray:
    """Y[i] = f(A[i], B[i]) for equally shaped fp32 or fp64 operands."""
    lib = lib or load()
    dt = np.float64 if np.asarray(A).dtype == np.float64 else np.float32
    A, B = _c(A, dt), _c(B, dt)
    if A.shape != B.shape:
        raise ValueError("elementwise operands must have the same shape (broadcast first)")
    out = np.empty_like(A)
    ptr = _f64p if dt == np.float64 else _f32p
    fn = lib.oracle_elementwise_binary_f64 if dt == np.float64 else lib.oracle_elementwise_binary_f32
    if fn(BINARY_OPS[op], A.size, _p(A, ptr), _p(B, ptr), _p(out, ptr)) != 0:
        raise ValueError(f"unknown binary operation {op}")
    return out


def broadcast(X, out_shape, lib=None) -> np.ndarray:
    """ml::Broadcast: X (rank padded on the left with 1s) repeated to out_shape."""
    lib = lib or load()
    X = np.ascontiguousarray(X)
    out_shape = tuple(int(d) for d in out_shape)
    in_shape = (1,) * (len(out_shape) - X.ndim) + X.shape
    out = np.empty(out_shape, X.dtype)
    ins = (_i64 * len(out_shape))(*in_shape)
    outs = (_i64 * len(out_shape))(*out_shape)
    rc = lib.oracle_broadcast(X.dtype.itemsize, len(out_shape), ins, outs, X.ctypes.data, out.ctypes.data)
    if rc != 0:
        raise ValueError(f"cannot broadcast {X.shape} to {out_shape}")
    return out


REDUCE_OPS = {"sum": 0, "max": 1, "min": 2, "mean": 3}


def reduce(op: str, X, axes, keepdims: bool = False, lib=None) -> np.ndarray:
    """ml::Sum / ml::Max / ml::Min / ml::Mean of an fp32 or fp64 array over a block of adjacent axes,
    accumulated left to right like the reference's expansion."""
    lib = lib or load()
    dt = np.float64 if np.asarray(X).dtype == np.float64 else np.float32
    X = _c(X, dt)
    rank = X.ndim
    axes = sorted(a % rank for a in ([axes] if np.isscalar(axes) else axes))
    if axes != list(range(axes[0], axes[-1] + 1)):
        raise ValueError("the reduced axes must be adjacent")
    outer = int(np.prod(X.shape[:axes[0]], dtype=np.int64))
    extent = int(np.prod(X.shape[axes[0]:axes[-1] + 1], dtype=np.int64))
    inner = int(np.prod(X.shape[axes[-1] + 1:], dtype=np.int64))
    out = np.empty((outer, inner), dt)
    ptr = _f64p if dt == np.float64 else _f32p
    fn = lib.oracle_reduce_f64 if dt == np.float64 else lib.oracle_reduce_f32
    if fn(REDUCE_OPS[op], outer, extent, inner, _p(X, ptr), _p(out, ptr)) != 0:
        raise ValueError(f"reduce '{op}' over an extent of {extent}")
    kept = [1 if d in axes else s for d, s in enumerate(X.shape)] if keepdims else [s for d, s in enumerate(X.shape) if d not in axes]
    return out.reshape(kept)


def transpose(X, perm=None, lib=None) -> np.ndarray:
    """X with its axes permuted, out.shape[i] = X.shape[perm[i]] (reversed axes when perm is None), any dtype."""
    lib = lib or load()
    X = np.ascontiguousarray(X)
    perm = list(range(X.ndim))[::-1] if perm is None else [int(p) % X.ndim for p in perm]
    out = np.empty([X.shape[p] for p in perm], X.dtype)
    rank = X.ndim
    shape = (_i64 * max(rank, 1))(*X.shape)
    pm = (_i64 * max(rank, 1))(*perm)
    if lib.oracle_transpose(X.dtype.itemsize, rank, shape, pm, X.ctypes.data, out.ctypes.data) != 0:
        raise ValueError("invalid permutation or rank above 8")
    return out


def cast(X, dtype) -> np.ndarray:
    """ml::Cast: the conversion an assign between differently typed memlets compiles to (reference
    elementwise_ops/cast_node.cpp:39-40) - round to nearest even between floating types, truncation towards
    zero to an integer, which is what numpy's astype does for these types. `dtype` "bf16" gives the raw
    16-bit words (from fp32, through the C routine that test_oracle checks against torch); a uint16 input
    with dtype float32 is read as bf16 words."""
    X = np.ascontiguousarray(X)
    if isinstance(dtype, str) and dtype == "bf16":
        return f32_to_bf16(X.astype(np.float32, copy=False)) if X.dtype != np.uint16 else X.copy()
    dtype = np.dtype(dtype)
    if X.dtype == np.uint16:
        return bf16_to_f32(X).astype(dtype, copy=False)
    with np.errstate(all="ignore"):
        return X.astype(dtype)


def _literal(text: str) -> float:
    """A constant as generated C spells it: "0.5f", "3.0", "-INFINITY", "(2.0)"."""
    t = text.strip()
    while t.startswith("(") and t.endswith(")"):
        t = t[1:-1].strip()
    sign = 1.0
    if t.startswith("-"):
        sign, t = -1.0, t[1:].strip()
    if t in ("INFINITY", "HUGE_VAL", "HUGE_VALF"):
        return sign * float("inf")
    if t in ("NAN",):
        return float("nan")
    if t.endswith(("f", "F")) and not t.lower().startswith("0x"):
        return sign * float(np.float32(float(t[:-1])))
    return sign * float(t)


def map_nest(node: dict, operands: dict, scalars: dict | None = None, symbols: dict | None = None, lib=None) -> dict:
    """Runs a ROCMMap node's body (the payload the importer writes: indvars, bounds, reads, scalars, statements,
    writes) the way the reference's openmp target would print the nest: nested loops, one statement per tasklet.
    operands: connector -> flat numpy array (reads and writes; arrays of writes are updated in place and returned);
    scalars: connector -> value; symbols: name -> integer, for bounds and strides. Returns {write connector: array}."""
    lib = lib or load()
    lib.oracle_map_nest.restype = ctypes.c_int
    symbols = {k: int(v) for k, v in (symbols or {}).items()}
    ev = lambda e: int(eval(str(e), {"__builtins__": {}}, symbols))
    depth = len(node["indvars"])
    bounds = (ctypes.c_int64 * depth)(*[ev(b) for b in node["bounds"]])
    np_type = lambda name: np.float64 if name == "Double" else np.float32
    slots: dict = {}
    reads = node["reads"]
    keep = []
    read_ptrs = (ctypes.c_void_p * max(1, len(reads)))()
    read_strides = (ctypes.c_int64 * max(1, len(reads) * depth))()
    read_f64 = (ctypes.c_int * max(1, len(reads)))()
    for r, acc in enumerate(reads):
        a = np.ascontiguousarray(operands[acc["connector"]], dtype=np_type(acc["element_type"])).reshape(-1)
        if a.size < ev(acc["extent"]):
            raise ValueError(f"operand {acc['connector']} holds {a.size} elements, the nest walks {ev(acc['extent'])}")
        keep.append(a)
        read_ptrs[r] = a.ctypes.data
        read_f64[r] = int(acc["element_type"] == "Double")
        for l in range(depth):
            read_strides[r * depth + l] = ev(acc["strides"][l])
        slots[acc["connector"]] = r
    consts = []
    for sc in node.get("scalars", []):
        slots[sc["connector"]] = len(reads) + len(consts)
        v = (scalars or {})[sc["connector"]]
        consts.append(float(np.float32(v)) if sc["element_type"] != "Double" else float(v))
    stmts = node["statements"]
    for st in stmts:                      # literals become constants too
        for a in st["args"]:
            if a.startswith("#") and a not in slots:
                slots[a] = len(reads) + len(consts)
                consts.append(_literal(a[1:]))
    for w in node["writes"]:
        if w["value"].startswith("#") and w["value"] not in slots:
            slots[w["value"]] = len(reads) + len(consts)
            consts.append(_literal(w["value"][1:]))
    base = len(reads) + len(consts)
    ops = (ctypes.c_char_p * max(1, len(stmts)))()
    stmt_f64 = (ctypes.c_int * max(1, len(stmts)))()
    stmt_args = (ctypes.c_int * max(1, 3 * len(stmts)))(*([-1] * max(1, 3 * len(stmts))))
    for s, st in enumerate(stmts):
        ops[s] = st["op"].encode()
        stmt_f64[s] = int(st["type"] == "Double")
        for k, a in enumerate(st["args"]):
            stmt_args[3 * s + k] = slots[a]
        slots[st["out"]] = base + s
    writes = node["writes"]
    out = {}
    write_ptrs = (ctypes.c_void_p * len(writes))()
    write_strides = (ctypes.c_int64 * (len(writes) * depth))()
    write_f64 = (ctypes.c_int * len(writes))()
    write_slots = (ctypes.c_int * len(writes))()
    for w, acc in enumerate(writes):
        dt = np_type(acc["element_type"])
        given = operands.get(acc["connector"])
        a = np.zeros(ev(acc["extent"]), dt) if given is None else np.ascontiguousarray(given, dtype=dt).reshape(-1)
        out[acc["connector"]] = a
        write_ptrs[w] = a.ctypes.data
        write_f64[w] = int(acc["element_type"] == "Double")
        write_slots[w] = slots[acc["value"]]
        for l in range(depth):
            write_strides[w * depth + l] = ev(acc["strides"][l])
    cv = (ctypes.c_double * max(1, len(consts)))(*consts)
    rc = lib.oracle_map_nest(depth, bounds, len(reads), read_ptrs, read_strides, read_f64, len(consts), cv, len(stmts), ops, stmt_f64,
                             stmt_args, len(writes), write_ptrs, write_strides, write_f64, write_slots)
    if rc != 0:
        raise ValueError("oracle_map_nest: a depth outside 1..8, an unknown operation or a value used before it is computed")
    return out
