"""Elementwise tensor nodes and ml::Broadcast on the GPU against the CPU oracle, through
docc_rocm_elementwise_unary / _binary / _binary_scalar / docc_rocm_broadcast.

Bars: bit-exact for the IEEE operations and the selections (add, sub, mul, div, maximum, minimum,
abs, relu, sqrt, broadcast); exp / tanh / sigmoid / erf within 4 units in the last place of the
oracle's libm result (1e-6 relative in fp32, 1e-15 in fp64)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host

pytestmark = pytest.mark.gpu
EXACT_UNARY = ["abs", "relu", "sqrt"]
LIBM_UNARY = ["exp", "tanh", "sigmoid", "erf"]
BINARY = ["add", "sub", "mul", "div", "maximum", "minimum"]
SIZES = [0, 1, 3, 4, 255, 1000, 4099, 1 << 20]


def prec(dt):
    return 64 if dt == np.float64 else 32


def run_unary(rt, op, x, offset=0, in_place=False):
    buf = dev(np.concatenate([np.zeros(offset, x.dtype), x.ravel()]))
    out = buf if in_place else torch.full_like(buf, float("nan"))
    es = buf.element_size()
    rt.elementwise_unary(op, prec(x.dtype), x.size, buf.data_ptr() + offset * es, out.data_ptr() + offset * es)
    torch.cuda.synchronize()
    return host(out)[offset:].reshape(x.shape)


def run_binary(rt, op, a, b, offset=0):
    da = dev(np.concatenate([np.zeros(offset, a.dtype), a.ravel()]))
    db = dev(np.concatenate([np.zeros(offset, a.dtype), b.ravel()]))
    out = torch.full_like(da, float("nan"))
    es = da.element_size()
    rt.elementwise_binary(op, prec(a.dtype), a.size, da.data_ptr() + offset * es, db.data_ptr() + offset * es, out.data_ptr() + offset * es)
    torch.cuda.synchronize()
    return host(out)[offset:].reshape(a.shape)


def ulps(y, ref):
    spacing = np.spacing(np.abs(ref))
    finite = np.isfinite(ref)
    assert np.array_equal(np.isfinite(y), finite)
    return float((np.abs(y[finite].astype(np.float64) - ref[finite].astype(np.float64)) / spacing[finite]).max()) if finite.any() else 0.0


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("n", SIZES)
def test_binary_bit_exact(rt, dt, n):
    rng = np.random.default_rng(n + 1)
    a = (rng.standard_normal(n) * 10).astype(dt)
    b = (rng.standard_normal(n) * 10).astype(dt)
    if n > 100:
        b[::97] = 0.0
        a[::193] = np.nan
        a[5], b[5] = np.inf, -np.inf
    for op in BINARY:
        for offset in (0, 1):   # offset 1: operands not 16-byte aligned -> scalar path
            assert np.array_equal(run_binary(rt, op, a, b, offset), oracle.elementwise_binary(op, a, b), equal_nan=True), (op, offset)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_pow_within_libm_accuracy(rt, dt):
    """ml::Pow: the array, scalar-exponent (x ** 2, x ** 0.5) and scalar-base forms; exact on the IEEE special
    cases, within 4 ulp of the oracle's libm elsewhere."""
    rng = np.random.default_rng(12)
    a = (np.abs(rng.standard_normal(5000)) * 3 + 0.05).astype(dt)
    b = (rng.standard_normal(5000) * 3).astype(dt)
    for offset in (0, 1):
        assert ulps(run_binary(rt, "pow", a, b, offset), oracle.elementwise_binary("pow", a, b)) <= 4
    base = np.array([2, 3, 0.5, -2, -2, 0, 7, np.inf, 1, -3, 0, -0.0], dt)
    expo = np.array([10, 2, 2, 3, 0.5, 0, 0, -1, np.nan, 2, -1, -3], dt)
    with np.errstate(all="ignore"):
        assert np.array_equal(run_binary(rt, "pow", base, expo), oracle.elementwise_binary("pow", base, expo), equal_nan=True)
    for scalar, lhs in ((2.0, False), (0.5, False), (3.0, False), (-1.0, False), (2.0, True), (10.0, True)):
        x = (a if not lhs else b)
        dx = dev(x)
        out = torch.full_like(dx, float("nan"))
        rt.elementwise_binary_scalar("pow", prec(dt), x.size, dx.data_ptr(), scalar, out.data_ptr(), lhs)
        torch.cuda.synchronize()
        full = np.full(x.size, scalar, dt)
        ref = oracle.elementwise_binary("pow", full, x) if lhs else oracle.elementwise_binary("pow", x, full)
        assert ulps(host(out), ref) <= 4, (scalar, lhs)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("n", SIZES)
def test_unary(rt, dt, n):
    rng = np.random.default_rng(n + 7)
    x = (rng.standard_normal(n) * 4).astype(dt)
    if n > 100:
        x[3], x[4], x[6] = np.inf, -np.inf, np.nan
    for op in EXACT_UNARY:
        arg = np.abs(x) if op == "sqrt" else x
        for offset in (0, 1):
            assert np.array_equal(run_unary(rt, op, arg, offset), oracle.elementwise_unary(op, arg), equal_nan=True), (op, offset)
    for op in LIBM_UNARY:
        ref = oracle.elementwise_unary(op, x)
        got = run_unary(rt, op, x)
        nan = np.isnan(ref)
        assert np.array_equal(np.isnan(got), nan)
        assert ulps(got[~nan], ref[~nan]) <= 4, op
    # in place
    assert np.array_equal(run_unary(rt, "relu", x, in_place=True), oracle.elementwise_unary("relu", x), equal_nan=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 5, 1000, 4099])
def test_binary_with_a_scalar_operand_bit_exact(rt, dt, n):
    rng = np.random.default_rng(n + 3)
    a = (rng.standard_normal(n) * 10).astype(dt)
    if n > 100:
        a[7], a[8], a[9] = np.nan, np.inf, 0.0
    for scalar in (2.5, -0.1, 0.0):      # -0.1 is rounded to the element type first, as the array operand would be
        full = np.full(n, scalar, dt)
        for op in BINARY:
            for offset in (0, 1):
                for lhs in (False, True):
                    da = dev(np.concatenate([np.zeros(offset, dt), a]))
                    out = torch.full_like(da, float("nan"))
                    es = da.element_size()
                    rt.elementwise_binary_scalar(op, prec(dt), n, da.data_ptr() + offset * es, scalar, out.data_ptr() + offset * es, lhs)
                    torch.cuda.synchronize()
                    ref = oracle.elementwise_binary(op, full, a) if lhs else oracle.elementwise_binary(op, a, full)
                    assert np.array_equal(host(out)[offset:], ref, equal_nan=True), (op, scalar, offset, lhs)


def test_large_shape_and_closed_forms(rt):
    # the benchmark shape of the softmax configuration, as an elementwise problem
    rng = np.random.default_rng(0)
    a = rng.standard_normal((8192, 4096)).astype(np.float32)
    b = rng.standard_normal((8192, 4096)).astype(np.float32)
    y = run_binary(rt, "add", a, b)
    assert np.array_equal(y, a + b)
    r = run_unary(rt, "relu", a)
    assert (r >= 0).all() and np.array_equal(r, np.maximum(a, 0))
    assert np.array_equal(run_binary(rt, "sub", a, a), np.zeros_like(a))
    assert np.array_equal(run_binary(rt, "div", a, a), np.ones_like(a))
    s = run_unary(rt, "sigmoid", np.zeros(1000, np.float32))
    assert np.array_equal(s, np.full(1000, 0.5, np.float32))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("in_shape,out_shape", [((3,), (2, 3)), ((4, 1), (4, 5)), ((1, 3, 1, 2), (2, 3, 4, 2)), ((1,), (7,)),
                                                ((2, 3), (2, 3)), ((1, 64, 1, 1), (8, 64, 14, 14)), ((1, 4096), (512, 4096)),
                                                ((1, 1, 1, 1, 1, 5), (2, 3, 2, 3, 2, 5))])
def test_broadcast(rt, dt, in_shape, out_shape):
    rng = np.random.default_rng(len(out_shape))
    x = rng.standard_normal(in_shape).astype(dt)
    dx = dev(x)
    out = torch.full(out_shape, float("nan"), device="cuda", dtype=torch.float64 if dt == np.float64 else torch.float32)
    rt.broadcast(prec(dt), in_shape, out_shape, dx.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(out), oracle.broadcast(x, out_shape))
    assert np.array_equal(host(out), np.broadcast_to(x, out_shape))


def test_errors(rt):
    from docc_amd.runtime import RocmRuntimeError
    a = torch.zeros(16, device="cuda")
    with pytest.raises(RocmRuntimeError):
        rt.elementwise_unary(99, 32, 16, a.data_ptr(), a.data_ptr())
    with pytest.raises(RocmRuntimeError):
        rt.elementwise_binary("add", 16, 16, a.data_ptr(), a.data_ptr(), a.data_ptr())     # precision 16
    with pytest.raises(RocmRuntimeError):
        rt.elementwise_unary("exp", 32, 16, 0, a.data_ptr())
    with pytest.raises(RocmRuntimeError):
        rt.broadcast(32, (2, 3), (2, 4), a.data_ptr(), a.data_ptr())
    rt.elementwise_unary("exp", 32, 0, 0, 0)   # empty: no-op


FUSED_CASES = [
    # out shape, a shape (None: scalar), b shape, binary, post
    ((200, 130), (200, 130), (130,), "add", ["relu"]),                   # bias + activation after a product
    ((64, 96), (64, 1), (64, 96), "sub", ["abs", "sqrt"]),               # column operand on the left
    ((4, 8, 14, 14), (4, 8, 14, 14), (1, 8, 1, 1), "mul", []),           # NCHW channel scale
    ((37, 53), (37, 53), None, "maximum", ["relu", "abs"]),              # scalar on the right
    ((37, 53), None, (37, 53), "div", []),                               # scalar on the left
    ((1000,), (1000,), None, None, ["abs", "sqrt", "relu"]),             # unary chain only
    ((3, 5, 7), (3, 1, 7), (1, 5, 1), "minimum", ["abs"]),               # both operands repeat
    ((2, 3, 2, 3, 2, 4), (2, 3, 2, 3, 2, 4), (4,), "add", ["relu"]),     # rank 6
    ((8192, 4096), (8192, 4096), (4096,), "add", ["relu"]),              # the softmax tensor's shape
    # rows x columns of whole vectors: the kernel that walks rows (groups 2^k column vectors wide)
    ((1003, 64), (1003, 64), (64,), "add", ["relu"]),                    # narrow rows stacked in a group, a ragged last group
    ((1001, 16), (1001, 1), (1001, 16), "sub", ["abs"]),                 # column operand, four column vectors
    ((4099, 1024), (4099, 1024), (4099, 1024), "mul", ["relu"]),         # equal shapes: collapses to one run, not a multiple of 256 vectors
    ((4096, 1024), (4096, 1024), (4096, 1024), "mul", ["relu"]),         # equal shapes: one run cut into rows of 256 vectors
    ((1 << 20,), (1 << 20,), None, "maximum", ["abs", "sqrt"]),          # one run with a scalar
    ((5, 4096), (4096,), (5, 1), "add", []),                             # fewer rows than a lane takes: row and column operands
    ((7, 100), (7, 100), (100,), "minimum", ["relu"]),                   # 25 column vectors in a group of 32
    ((9, 2052), (9, 2052), (2052,), "add", ["relu"]),                    # 513 column vectors: left to the general kernel
    ((3, 70000), (3, 70000), (3, 1), "mul", []),                         # many groups along the columns
]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("case", FUSED_CASES, ids=[str(i) for i in range(len(FUSED_CASES))])
def test_fused_chain_equals_the_separate_nodes_bit_for_bit(rt, dt, case):
    """docc_rocm_elementwise_fused against the oracle's Broadcast -> binary -> unary... chain. Only
    operations whose result is exactly rounded are used here, so the bar is bit-exact."""
    shape, a_shape, b_shape, binary, post = case
    rng = np.random.default_rng(len(shape) * 7 + len(post))
    make = lambda s: (rng.standard_normal(s) * 4).astype(dt)
    a = make(a_shape) if a_shape is not None else 1.75
    b = make(b_shape) if b_shape is not None else -0.3
    if binary == "div" and b_shape is not None:
        b[b == 0] = 1
    full = lambda v, s: oracle.broadcast(v, shape) if s is not None else np.full(shape, v, dt)
    ref = full(a, a_shape)
    if binary is not None:
        ref = oracle.elementwise_binary(binary, ref, full(b, b_shape))
    for op in post:
        ref = oracle.elementwise_unary(op, ref)
    da = dev(a) if a_shape is not None else None
    db = dev(b) if (b_shape is not None and binary is not None) else None
    out = torch.full(shape, float("nan"), device="cuda", dtype=torch.float64 if dt == np.float64 else torch.float32)
    rt.elementwise_fused(prec(dt), shape, binary, da.data_ptr() if da is not None else a, a_shape,
                         db.data_ptr() if db is not None else b, b_shape if binary is not None else None, post, out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(out), ref, equal_nan=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_fused_rows_kernel_equals_the_general_kernel_and_works_in_place(rt, dt, monkeypatch):
    """The kernel for rows x columns against the general one (DOCC_ROCM_EW_FUSED_GENERAL) on the same operands,
    libm operations included (the same device functions: equal bit for bit), then with the output on the left operand."""
    rng = np.random.default_rng(31)
    tdt = torch.float64 if dt == np.float64 else torch.float32
    for shape, b_shape in [((777, 256), (256,)), ((777, 256), (777, 1)), ((777, 256), (777, 256)), ((130, 24), (24,)), ((65536,), (65536,))]:
        x, b = dev(rng.standard_normal(shape).astype(dt)), dev(rng.standard_normal(b_shape).astype(dt))
        outs = []
        for general in (False, True):
            if general:
                monkeypatch.setenv("DOCC_ROCM_EW_FUSED_GENERAL", "1")
            else:
                monkeypatch.delenv("DOCC_ROCM_EW_FUSED_GENERAL", raising=False)
            out = torch.full(shape, float("nan"), device="cuda", dtype=tdt)
            rt.elementwise_fused(prec(dt), shape, "add", x.data_ptr(), shape, b.data_ptr(), b_shape, ["tanh", "sigmoid"], out.data_ptr())
            torch.cuda.synchronize()
            outs.append(host(out))
        assert np.array_equal(outs[0], outs[1], equal_nan=True), (shape, b_shape)
        monkeypatch.delenv("DOCC_ROCM_EW_FUSED_GENERAL", raising=False)
        rt.elementwise_fused(prec(dt), shape, "add", x.data_ptr(), shape, b.data_ptr(), b_shape, ["tanh", "sigmoid"], x.data_ptr())
        torch.cuda.synchronize()
        assert np.array_equal(host(x), outs[0], equal_nan=True), (shape, b_shape)


def test_fused_chain_with_libm_operations_and_unaligned_operands(rt):
    rng = np.random.default_rng(9)
    x, bias = rng.standard_normal((65, 33)).astype(np.float32), rng.standard_normal(33).astype(np.float32)
    ref = oracle.elementwise_unary("tanh", oracle.elementwise_unary("sigmoid", oracle.elementwise_binary("add", x, oracle.broadcast(bias, x.shape))))
    dx, dbias = dev(x), dev(np.concatenate([np.zeros(1, np.float32), bias]))      # bias off a 16-byte boundary, odd inner extent
    out = torch.full(x.shape, float("nan"), device="cuda")
    rt.elementwise_fused(32, x.shape, "add", dx.data_ptr(), x.shape, dbias.data_ptr() + 4, bias.shape, ["sigmoid", "tanh"], out.data_ptr())
    torch.cuda.synchronize()
    assert ulps(host(out), ref) <= 8
    from docc_amd.runtime import RocmRuntimeError
    with pytest.raises(RocmRuntimeError):
        rt.elementwise_fused(32, (4, 4), "add", dx.data_ptr(), (4, 3), dx.data_ptr(), (4, 4), [], out.data_ptr())     # 3 cannot become 4
    with pytest.raises(RocmRuntimeError):
        rt.elementwise_fused(32, (4, 4), None, 1.0, None, 0, None, ["relu"], out.data_ptr())                           # no array operand
    with pytest.raises(RocmRuntimeError):
        rt.elementwise_fused(32, (4, 4), None, dx.data_ptr(), (4, 4), 0, None, ["relu"] * 5, out.data_ptr())           # five unary operations


CASTS = [("f32", "f64"), ("f64", "f32"), ("f32", "bf16"), ("bf16", "f32"), ("f32", "f16"), ("f16", "f32"), ("i32", "f32"), ("i32", "f64"),
         ("i64", "f32"), ("i64", "f64"), ("f32", "i32"), ("f64", "i32"), ("f32", "i64"), ("f64", "i64"), ("f32", "f32")]
NP_OF = {"f16": np.float16, "bf16": np.uint16, "f32": np.float32, "f64": np.float64, "i32": np.int32, "i64": np.int64}


@pytest.mark.parametrize("src,dst", CASTS, ids=[f"{s}_to_{d}" for s, d in CASTS])
def test_cast_bit_exact(rt, src, dst):
    """ml::Cast: round to nearest even between floating types (ties, subnormals, overflow to inf, NaN), truncation
    towards zero to integers, exact or rounded integer -> floating."""
    rng = np.random.default_rng(len(src) * 7 + len(dst))
    n = 10007
    if src.startswith("i"):
        x = rng.integers(-2 ** 30, 2 ** 30, n).astype(NP_OF[src])
        x[:6] = [0, 1, -1, 16777217, -16777219, 2 ** 30 + 1]          # 2^24 + 1: rounds in fp32
        if src == "i64":
            x[6:9] = [2 ** 53 + 1, -(2 ** 62) - 1, 2 ** 40 + 3]
    elif src == "bf16":
        x = oracle.f32_to_bf16((rng.standard_normal(n) * 100).astype(np.float32))
        x[:4] = [0x7f80, 0xff80, 0x7fc0, 0x0001]                       # inf, -inf, NaN, smallest subnormal
    else:
        x = (rng.standard_normal(n) * 1000).astype(NP_OF[src])
        with np.errstate(over="ignore"):      # 3e38 is inf in fp16
            x[:10] = [0.0, -0.0, 1.5, 2049.0, 2051.0, 1e-40, 65520.0, 3.0e38, 1.0000000596046448, -7.99]
        if dst.startswith("i"):
            x = np.clip(x, -2.0e9, 2.0e9).astype(NP_OF[src])         # out-of-range conversions are undefined in C
        else:
            x[10:13] = [np.inf, -np.inf, np.nan]
    dx = dev(x)
    out = torch.empty(n, dtype={"f16": torch.float16, "bf16": torch.int16, "f32": torch.float32, "f64": torch.float64,
                                "i32": torch.int32, "i64": torch.int64}[dst], device="cuda")
    rt.cast(src, dst, n, dx.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    got = host(out)
    want = oracle.cast(x, "bf16" if dst == "bf16" else NP_OF[dst])
    if dst == "bf16":
        got = got.view(np.uint16)
        nan = (want & 0x7fff) > 0x7f80
        assert np.array_equal(((got & 0x7fff) > 0x7f80), nan) and np.array_equal(got[~nan], want[~nan])
    else:
        assert np.array_equal(got, want, equal_nan=True)
    if (src, dst) == ("f32", "f16"):
        assert np.isinf(got[6]) and got[3] == 2048.0 and got[4] == 2052.0 and got[2] == 1.5      # 65520 overflows; ties go to even


def test_cast_rejects_what_is_not_built(rt):
    from docc_amd.runtime import RocmRuntimeError
    x = torch.zeros(64, device="cuda")
    with pytest.raises(RocmRuntimeError, match="not built"):
        rt.cast("f64", "bf16", 8, x.data_ptr(), x.data_ptr())
    with pytest.raises(RocmRuntimeError, match="unknown type"):
        rt.cast(9, 2, 8, x.data_ptr(), x.data_ptr())


def test_more_than_2_to_the_31_elements(rt):
    """The kernels switch to 64-bit indices past 2^31 elements: unary, binary with a scalar, fused chain with a
    repeated row, broadcast, transpose (rows and tiles) and cast on a tensor of 2^31 + 8192 fp32 elements (8.6 GB),
    checked on the device at the start, around the 2^31 boundary and at the end."""
    cols = 4096
    rows = (1 << 31) // cols + 2
    n = rows * cols
    assert n > (1 << 31)
    x = torch.empty(n, device="cuda")
    x.copy_(torch.arange(n, device="cuda", dtype=torch.float32) % 1021 - 510.0)      # exact small integers, both signs
    y = torch.empty(n, device="cuda")
    windows = [slice(0, 5000), slice((1 << 31) - 5000, (1 << 31) + 5000), slice(n - 5000, n)]

    def same(got, want):
        for w in windows:
            assert torch.equal(got[w], want[w])

    rt.elementwise_unary("relu", 32, n, x.data_ptr(), y.data_ptr())
    same(y, torch.relu(x))
    rt.elementwise_binary_scalar("mul", 32, n, x.data_ptr(), 2.0, y.data_ptr())
    for w in windows:
        assert torch.equal(y[w], x[w] * 2.0)
    row = torch.arange(cols, device="cuda", dtype=torch.float32)
    rt.elementwise_fused(32, (rows, cols), "add", x.data_ptr(), (rows, cols), row.data_ptr(), (cols,), ["abs"], y.data_ptr())
    for w in windows:
        idx = torch.arange(w.start, w.stop, device="cuda")
        assert torch.equal(y[w], (x[w] + row[idx % cols]).abs())
    rt.broadcast(32, (1, cols), (rows, cols), row.data_ptr(), y.data_ptr())
    for w in windows:
        idx = torch.arange(w.start, w.stop, device="cuda")
        assert torch.equal(y[w], row[idx % cols])
    # transpose [rows, cols] -> [cols, rows] (tiles), and [rows / 2, 2, cols] -> [2, rows / 2, cols] (rows kernel)
    rt.transpose(4, (rows, cols), (1, 0), x.data_ptr(), y.data_ptr())
    yt = y.view(cols, rows)
    for c, r0 in ((0, 0), (17, rows - 300), (cols - 1, rows // 2), (cols - 1, rows - 64)):
        assert torch.equal(yt[c, r0:r0 + 64], x.view(rows, cols)[r0:r0 + 64, c])
    rt.transpose(4, (rows // 2, 2, cols), (1, 0, 2), x.data_ptr(), y.data_ptr())
    y3, x3 = y.view(2, rows // 2, cols), x.view(rows // 2, 2, cols)
    for h, r in ((0, 0), (1, rows // 2 - 1), (1, 5), (0, rows // 4)):
        assert torch.equal(y3[h, r], x3[r, h])
    del y
    z = torch.empty(n, device="cuda", dtype=torch.float64)
    rt.cast("f32", "f64", n, x.data_ptr(), z.data_ptr())
    for w in windows:
        assert torch.equal(z[w], x[w].double())
