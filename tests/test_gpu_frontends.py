"""End to end on the GPU through the reference's entry points: `@native(target="rocm")` and
`torch.compile(model, backend="docc")`, compared with the CPU oracle. These tests read like the
reference's own (python/tests/python/functions/numpy/test_linalg.py:5-24,
python/benchmarks/npbench/polybench/test_gemm.py:23-89, .../deep_learning/softmax/test_softmax.py:24-84,
mlir/integration/torch/test_matmul.py, test_conv2d.py) with the target switched to rocm.

Tolerances (norm-wise relative error): fp64 1e-12, fp32 1e-5, bf16 2e-2."""
import math

import numpy as np
import pytest
import scipy.special
import torch

import docc_amd.torch as docc_torch
import oracle
from docc_amd.python import conv2d, native, relu, sigmoid
from gpu_util import rel_err_max

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def tmp_docc(tmp_path, monkeypatch):
    monkeypatch.setenv("DOCC_TMP", str(tmp_path / "docc"))
    docc_torch.set_backend_options(target="rocm", category="server")


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def test_native_matmul_config_1():
    @native(target="rocm")
    def matmul(A, B):
        return A @ B

    rng = np.random.default_rng(0)
    A, B = rng.random((1000, 1000)), rng.random((1000, 1000))
    C = matmul(A, B)
    assert C.dtype == np.float64 and C.shape == (1000, 1000) and C.flags.c_contiguous
    assert rel_err_max(C, oracle.gemm(A, B, variant="ld")) <= 1e-12
    # second call: cached program, other values and size
    A2, B2 = rng.random((37, 37)), rng.random((37, 37))
    assert rel_err_max(matmul(A2, B2), oracle.gemm(A2, B2, variant="ld")) <= 1e-12
    assert len(matmul.cache) == 1


def test_native_matmul_with_a_return_annotation():
    """The annotation moves `_docc_ret_0` to the front of the generated function's arguments
    (reference python_program.py:515-524); the caller walks the arguments by name."""
    from typing import Annotated

    @native(target="rocm")
    def annotated_mm(a, b) -> Annotated[np.ndarray, (None, None), np.float64]:
        return a @ b

    rng = np.random.default_rng(3)
    A, B = rng.random((96, 80)), rng.random((80, 72))
    C = annotated_mm(A, B)
    assert annotated_mm.last_sdfg.arguments[0] == "_docc_ret_0"
    assert C.shape == (96, 72) and rel_err_max(C, oracle.gemm(A, B, variant="ld")) <= 1e-12


@pytest.mark.parametrize("offload", ["function", "node"])
def test_native_polybench_gemm(offload):
    @native(target="rocm", offload=offload)
    def gemm(alpha, beta, C, A, B):
        C[:] = alpha * A @ B + beta * C

    rng = np.random.default_rng(42)
    NI, NJ, NK = 100, 110, 120     # non-square, like the reference benchmark's S size scaled down
    A, B, C = rng.random((NI, NK)), rng.random((NK, NJ)), rng.random((NI, NJ))
    ref = oracle.gemm(A, B, C, alpha=1.5, beta=1.2)
    gemm(1.5, 1.2, C, A, B)
    assert rel_err_max(C, ref) <= 1e-12
    report = gemm.last_sdfg.loop_report()
    assert report["GEMM"] == 1     # exactly one GEMM node, as the reference's harness expects on every target


def test_native_softmax_like_the_reference_benchmark():
    @native(target="rocm")
    def softmax(x):
        tmp_max = np.max(x, axis=-1, keepdims=True)
        tmp_out = np.exp(x - tmp_max)
        tmp_sum = np.sum(tmp_out, axis=-1, keepdims=True)
        return tmp_out / tmp_sum

    rng = np.random.default_rng(42)
    x = rng.random((16, 16, 128, 128), dtype=np.float32)      # size "S" of the reference benchmark
    y = softmax(x)
    assert y.dtype == np.float32 and y.shape == x.shape
    assert rel_err_max(y, oracle.softmax(x)) <= 1e-5
    np.testing.assert_allclose(y, scipy.special.softmax(x.astype(np.float64), axis=-1), rtol=1e-5, atol=1e-8)


def test_native_chain_keeps_the_intermediate_on_the_device():
    @native(target="rocm")
    def chain(a, b, x):
        t = a @ b
        return scipy.special.softmax(t @ x, axis=-1)

    rng = np.random.default_rng(3)
    a, b, x = (rng.standard_normal((96, 96)).astype(np.float32) * 0.2 for _ in range(3))
    y = chain(a, b, x)
    ref = oracle.softmax(oracle.gemm(oracle.gemm(a, b), x))
    assert rel_err_max(y, ref) <= 1e-4    # two chained fp32 products feed an exponential
    r = chain.last_sdfg.loop_report()
    assert r["H2D"] == 3 and r["D2H"] == 1


def test_native_intermediate_with_two_readers():
    @native(target="rocm")
    def two_readers(a, b):
        t = a @ b
        return scipy.special.softmax(t, axis=-1) @ t

    rng = np.random.default_rng(5)
    a, b = (rng.standard_normal((80, 80)).astype(np.float32) * 0.3 for _ in range(2))
    y = two_readers(a, b)
    t = oracle.gemm(a, b)
    assert rel_err_max(y, oracle.gemm(oracle.softmax(t), t)) <= 1e-5
    r = two_readers.last_sdfg.loop_report()
    assert r["H2D"] == 2 and r["D2H"] == 1          # the intermediate feeds both nodes from device memory


def test_native_conv():
    @native(target="rocm")
    def conv(x, w, b):
        return conv2d(x, w, b, stride=1, padding=1)

    g = np.load(__import__("pathlib").Path(__file__).parent / "golden" / "conv_2x3x7x7_k3_p1_bias_f32.npz")
    y = conv(g["X"], g["W"], g["b"])
    assert y.shape == (2, 4, 7, 7)
    assert rel_err_max(y, g["Y"]) <= 1e-5
    assert rel_err_max(y, oracle.conv2d(g["X"], g["W"], g["b"], pad=(1, 1))) <= 1e-5


class Attn(torch.nn.Module):
    def forward(self, q, k, v):
        s = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(q.shape[-1])
        return torch.matmul(torch.softmax(s, dim=-1), v)


def test_torch_compile_attention_config_4():
    torch.manual_seed(3)
    Q, K, V = (torch.randn(8, 16, 2048, 64).bfloat16() for _ in range(3))
    model = torch.compile(Attn(), backend="docc")
    out = model(Q.cuda(), K.cuda(), V.cuda())
    assert out.device.type == "cuda" and out.dtype == torch.bfloat16 and out.shape == (8, 16, 2048, 64)
    O = out.float().cpu().numpy()
    assert np.isfinite(O).all()
    for (b, h) in [(0, 0), (5, 9)]:
        ref = oracle.attention(bits(Q[b:b + 1, h:h + 1, 512:576]), bits(K[b:b + 1, h:h + 1]), bits(V[b:b + 1, h:h + 1]))
        assert rel_err_max(O[b, h, 512:576], ref[0, 0]) <= 2e-2


def test_torch_compile_attention_cpu_tensors_and_golden():
    g = np.load(__import__("pathlib").Path(__file__).parent / "golden" / "attn_1x2x96x64_bf16.npz")
    to_t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    model = torch.compile(Attn(), backend="docc")
    out = model(to_t(g["Q"]), to_t(g["K"]), to_t(g["V"]))      # CPU tensors: generated code does the transfers
    assert out.device.type == "cpu"
    assert rel_err_max(out.float().numpy(), g["O"]) <= 2e-2


def test_torch_compile_conv_config_5():
    torch.manual_seed(4)
    conv = torch.nn.Conv2d(64, 64, 3, stride=1, padding=1, bias=True)
    torch.nn.init.kaiming_normal_(conv.weight)
    with torch.no_grad():
        conv.bias.copy_(torch.randn(64) * 0.1)
    X = torch.randn(32, 64, 56, 56)
    program = docc_torch.compile_torch(conv.cuda(), X.cuda(), target="rocm")
    Y = program(X.cuda())
    assert Y.shape == (32, 64, 56, 56) and Y.device.type == "cuda"
    ref = oracle.conv2d(X[:2].numpy(), conv.weight.detach().cpu().numpy(), conv.bias.detach().cpu().numpy(), pad=(1, 1))
    assert rel_err_max(Y[:2].cpu().numpy(), ref) <= 1e-5


def test_torch_backend_matmul_softmax_fp32():
    class MM(torch.nn.Module):
        def forward(self, a, b):
            return torch.softmax(a @ b, dim=-1)

    torch.manual_seed(815)      # the seed of the reference's torch integration tests
    a, b = torch.randn(64, 48), torch.randn(48, 80)
    model = torch.compile(MM(), backend="docc")
    res = model(a.cuda(), b.cuda())
    assert isinstance(res, torch.Tensor)
    ref = oracle.softmax(oracle.gemm(a.numpy(), b.numpy()))
    assert rel_err_max(res.cpu().numpy(), ref) <= 1e-5

    class BMM(torch.nn.Module):
        def forward(self, a, b):
            return torch.matmul(a, b)

    a3, b3 = torch.randn(4, 20, 30, dtype=torch.float64), torch.randn(4, 30, 10, dtype=torch.float64)
    out = docc_torch.compile_torch(BMM(), (a3, b3), target="rocm")(a3, b3)   # batched: ml::MatMul
    refs = np.stack([oracle.gemm(a3[i].numpy(), b3[i].numpy(), variant="ld") for i in range(4)])
    assert rel_err_max(out.numpy(), refs) <= 1e-12


def test_native_dense_layer_stays_on_the_device():
    """relu(x @ w + b): GEMM, Broadcast, Add and ReLU nodes; only the arguments cross PCIe."""
    @native(target="rocm")
    def dense(x, w, b):
        return relu(x @ w + b)

    rng = np.random.default_rng(11)
    x, w, b = rng.standard_normal((200, 96)).astype(np.float32), rng.standard_normal((96, 130)).astype(np.float32), \
        rng.standard_normal(130).astype(np.float32)
    y = dense(x, w, b)
    t = oracle.gemm(x, w)
    ref = oracle.elementwise_unary("relu", oracle.elementwise_binary("add", t, oracle.broadcast(b, t.shape)))
    assert y.shape == (200, 130) and rel_err_max(y, ref) <= 1e-5 and (y >= 0).all()
    r = dense.last_sdfg.loop_report()
    assert r["H2D"] == 3 and r["D2H"] == 1
    assert r["GEMM"] == 1 and "ROCMFusedElementWise" not in r and "ml::Broadcast" not in r      # bias + ReLU in the store of the GEMM
    assert next(n for n in dense.last_sdfg.library_nodes() if n["code"] == "GEMM")["epilogue_activation"] == "ml::ReLU"

    # without the fusion pass: one kernel per node, the same bits
    @native(target="rocm", fuse=False)
    def dense_unfused(x, w, b):
        return relu(x @ w + b)

    y2 = dense_unfused(x, w, b)
    r = dense_unfused.last_sdfg.loop_report()
    assert [r[k] for k in ("GEMM", "ml::Broadcast", "ml::Add", "ml::ReLU")] == [1, 1, 1, 1]
    assert np.array_equal(y, y2)


def test_native_elementwise_expression_fp64():
    @native(target="rocm")
    def expr(x, y, s):
        return np.tanh(x * y - 0.5) / (s * np.abs(y) + 1.0) + np.minimum(sigmoid(x), 2.0 - np.sqrt(np.abs(y)))

    rng = np.random.default_rng(5)
    x, y = rng.standard_normal((37, 53)), rng.standard_normal((37, 53))
    got = expr(x, y, 0.75)
    ref = np.tanh(x * y - 0.5) / (0.75 * np.abs(y) + 1.0) + np.minimum(1.0 / (1.0 + np.exp(-x)), 2.0 - np.sqrt(np.abs(y)))
    assert got.dtype == np.float64 and rel_err_max(got, ref) <= 1e-12
    # in place into an argument, scalar on the left of a subtraction
    @native(target="rocm")
    def update(x, y):
        y[:] = 1.0 - np.exp(x) * y

    y2 = y.copy()
    update(x, y2)
    assert rel_err_max(y2, 1.0 - np.exp(x) * y) <= 1e-12


def test_torch_compile_mlp_fp32():
    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = torch.nn.Linear(64, 128)
            self.fc2 = torch.nn.Linear(128, 32)

        def forward(self, x):
            return torch.sigmoid(self.fc2(torch.relu(self.fc1(x)))) - 0.5

    torch.manual_seed(0)
    model = Mlp().cuda()
    x = torch.randn(16, 10, 64, device="cuda")
    program = docc_torch.compile_torch(model, x, target="rocm")
    y = program(x)
    assert y.is_cuda and y.shape == (16, 10, 32)
    with torch.no_grad():
        ref = model.double()(x.double())
    assert rel_err_max(y.cpu().numpy(), ref.cpu().numpy()) <= 1e-5
    r = program.last_sdfg.loop_report()
    assert r["GEMM"] == 2 and r["H2D"] == 0 and r["D2H"] == 0      # device tensors: no transfers at all


def test_torch_compile_activations_with_scalar_operands():
    class Acts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.elu = torch.nn.ELU(alpha=0.7)
            self.leaky = torch.nn.LeakyReLU(0.2)
            self.hs = torch.nn.Hardsigmoid()

        def forward(self, x):
            return self.hs(self.leaky(self.elu(x))) + torch.nn.functional.leaky_relu(x) + torch.nn.functional.elu(x, alpha=1.5)

    torch.manual_seed(1)
    for dtype, tol in ((torch.float32, 1e-5), (torch.float64, 1e-12)):
        x = (torch.randn(37, 129, dtype=dtype) * 3).cuda()
        program = docc_torch.compile_torch(Acts(), x, target="rocm")
        y = program(x)
        with torch.no_grad():
            ref = Acts()(x.double().cpu())
        assert y.dtype == dtype and rel_err_max(y.cpu().numpy(), ref.numpy()) <= tol
        # the same through the oracle's functions, node by node
        xh = x.cpu().numpy()
        o = oracle.elementwise_activation("hard_sigmoid", oracle.elementwise_activation("leaky_relu", oracle.elementwise_activation("elu", xh, 0.7), 0.2),
                                          1.0 / 6.0, 0.5)
        o = o + oracle.elementwise_activation("leaky_relu", xh, 0.01) + oracle.elementwise_activation("elu", xh, 1.5)
        assert rel_err_max(y.cpu().numpy(), o) <= tol


def test_builder_program_with_dot_fill_and_activations(tmp_path):
    """DOT::BLAS with a scalar result, ml::Fill from that scalar, and the activations, through the builder and
    the generated code on host arrays (function-level offloading)."""
    import ctypes

    from docc_amd.sdfg import Pointer, PrimitiveType, Scalar, StructuredSDFGBuilder

    F64p = Pointer(Scalar(PrimitiveType.Double))
    b = StructuredSDFGBuilder("dot_fill")
    for name in ("x", "y", "filled", "act"):
        b.add_container(name, F64p, True)
    b.add_container("_s0", Scalar(PrimitiveType.Int64), True)
    b.add_container("r", Scalar(PrimitiveType.Double), False)
    b.add_dot("x", "y", "r", "_s0", 1, 1)
    b.add_fill("r", "filled", ["_s0"])
    b.add_elementwise_unary_op("elu", "x", "act", ["_s0"], alpha="r")
    s = b.move()
    s.schedule("rocm")
    lib = s._compile(str(tmp_path))
    fn = getattr(ctypes.CDLL(lib), "dot_fill")
    fn.restype = None
    n = 5000
    rng = np.random.default_rng(12)
    x, y = rng.standard_normal(n) * 0.01, rng.standard_normal(n)
    filled, act = np.full(n, np.nan), np.full(n, np.nan)
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    fn(ptr(x), ptr(y), ptr(filled), ptr(act), ctypes.c_int64(n))
    from docc_amd import runtime
    assert runtime.take_failure()[0] == 0
    r = float(np.dot(x.astype(np.longdouble), y.astype(np.longdouble)))
    assert abs(filled[0] - r) <= 1e-12 * float(np.abs(x) @ np.abs(y)) and (filled == filled[0]).all()
    assert rel_err_max(act, oracle.elementwise_activation("elu", x, filled[0])) <= 1e-12


def test_torch_compile_small_batch_through_wide_layers():
    """A batch of four through 2048-wide layers: the GEMMs have few output rows and take the matrix-vector kernels
    (bias and activation as one pass over the output); same bar as any fp32 GEMM chain."""
    class Decoder(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = torch.nn.Linear(2048, 8192)
            self.down = torch.nn.Linear(8192, 2048, bias=False)

        def forward(self, x):
            return self.down(torch.relu(self.up(x)))

    torch.manual_seed(3)
    model = Decoder().cuda()
    x = torch.randn(4, 2048, device="cuda")
    program = docc_torch.compile_torch(model, x, target="rocm")
    y = program(x)
    assert y.is_cuda and y.shape == (4, 2048)
    with torch.no_grad():
        ref = model.double()(x.double())
    assert rel_err_max(y.cpu().numpy(), ref.cpu().numpy()) <= 1e-5
    assert program.last_sdfg.loop_report()["GEMM"] == 2


@pytest.mark.parametrize("mode", ["", "aggregate"])
def test_instrumented_program_writes_a_trace_with_device_times(tmp_path, mode):
    """`instrumentation_mode="ols"`: every rocm node and transfer is a region timed with HIP events;
    the trace is written when the process ends."""
    import json
    import os
    import subprocess
    import sys
    from pathlib import Path

    out = tmp_path / "trace.json"
    env = dict(os.environ, __DAISY_INSTRUMENTATION_FILE=str(out), __DAISY_INSTRUMENTATION_MODE=mode, DOCC_TMP=str(tmp_path / "docc"),
               PYTHONPATH=str(Path(__file__).resolve().parent.parent))
    r = subprocess.run([sys.executable, "-m", "docc_amd.examples.dense_instrumented"], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    events = json.loads(out.read_text())["traceEvents"]
    kinds = {}
    for e in events:
        kinds.setdefault(e["args"]["docc"]["element_type"], []).append(e)
    runs = 1 if mode == "aggregate" else 3
    assert len(kinds["math"]) == 1 * runs             # the GEMM with bias + ReLU in its store
    assert len(kinds["h2d_transfer"]) == 3 * runs and len(kinds["d2h_transfer"]) == 1 * runs
    assert all(e["args"]["target_type"] == "ROCM" and e["args"]["function"] == "dense" and e["dur"] > 0 for e in events)
    flop = [e["args"]["metrics"].get("static:::flop") for e in kinds["math"]]
    expect = 2.0 * 512 * 384 * 256 + 2.0 * 512 * 384     # multiply-adds plus the alpha/beta epilogue, as the reference counts
    assert any((f["mean"] if isinstance(f, dict) else f) == expect for f in flop if f is not None)
    pcie = sorted((e["args"]["metrics"]["static:::pcie_bytes"]["mean"] if mode == "aggregate" else e["args"]["metrics"]["static:::pcie_bytes"])
                  for e in kinds["h2d_transfer"])[-1]
    assert pcie == 512 * 256 * 4
    # even with the first launch uploading its code object a GEMM of this size stays well under 50 ms on the device;
    # a region's time is a device time, not the process's (compilation alone takes seconds)
    gemm = [e for e in kinds["math"] if e["name"].startswith("dense") and (e["args"]["metrics"].get("static:::flop") is not None)]
    assert gemm and min(e["dur"] / (3 if mode == "aggregate" else 1) for e in gemm) < 50000


def test_program_in_docc_json_format_runs(tmp_path):
    """An SDFG in the layout docc's serializer writes (two chained GEMMs with a Malloc'ed temporary) is
    imported, scheduled, compiled and run: C = 1.5 * (A @ B) @ B + 0.5 * C."""
    import ctypes
    import json

    from docc_amd import runtime
    from docc_amd.sdfg import StructuredSDFG
    from test_interchange import gemm_program

    s = StructuredSDFG.parse(json.dumps(gemm_program()))
    s.schedule("rocm")
    lib = ctypes.CDLL(s._compile(str(tmp_path)))
    fn = lib.two_mm_sdfg
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    fn.restype = None
    rng = np.random.default_rng(2)
    n = 150
    A, B, C = rng.random((n, n)), rng.random((n, n)), rng.random((n, n))
    ref = oracle.gemm(oracle.gemm(A, B), B, C, alpha=1.5, beta=0.5)
    fn(A.ctypes.data, B.ctypes.data, C.ctypes.data, n)
    assert runtime.take_failure() == (0, "")
    assert rel_err_max(C, ref) <= 1e-12


def test_docc_json_return_copy_and_elementwise_nests_run(tmp_path):
    """`return A @ B` as the front end writes it (GEMM into a temporary, a For nest copying it into `_docc_ret_0`), and
    Maps holding one tasklet or CMath call each: the nests are matched to the copy / elementwise / fill kernels."""
    import ctypes
    import json

    from docc_amd import runtime
    from docc_amd.sdfg import StructuredSDFG
    from test_interchange import elementwise_nests_program, return_matmul_program

    s = StructuredSDFG.parse(json.dumps(return_matmul_program()))
    s.schedule("rocm")
    fn = ctypes.CDLL(s._compile(str(tmp_path / "mm"))).f_sdfg
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    fn.restype = None
    rng = np.random.default_rng(5)
    n = 150
    A, B = rng.random((n, n)), rng.random((n, n))
    out = np.full((n, n), np.nan)
    fn(A.ctypes.data, B.ctypes.data, n, out.ctypes.data)
    assert runtime.take_failure() == (0, "")
    assert rel_err_max(out, oracle.gemm(A, B, variant="ld")) <= 1e-12

    s = StructuredSDFG.parse(json.dumps(elementwise_nests_program()))
    s.schedule("rocm")
    fn = ctypes.CDLL(s._compile(str(tmp_path / "ew"))).nests_sdfg
    fn.argtypes = [ctypes.c_void_p] * 7 + [ctypes.c_int64] * 2
    fn.restype = None
    r, c = 37, 129
    X, Y = (rng.standard_normal((r, c)).astype(np.float32) for _ in range(2))
    S, E, Z, W = (np.full((r, c), np.nan, np.float32) for _ in range(4))
    T = np.full((c, r), np.nan, np.float32)
    fn(*(a.ctypes.data for a in (X, Y, S, E, T, Z, W)), r, c)
    assert runtime.take_failure() == (0, "")
    assert np.array_equal(S, X + Y) and np.array_equal(Z, np.full((r, c), 0.5, np.float32))
    ref = np.exp((X + Y).astype(np.float64))
    assert rel_err_max(E, ref) <= 1e-5 and np.array_equal(T, E.T)
    assert rel_err_max(W, E.astype(np.float64) / 3.0) <= 1e-5

    # a copy that permutes the axes, a scalar on the left of a difference, a scalar stored into the return buffer
    from test_interchange import permuted_copy_and_scalar_program
    s = StructuredSDFG.parse(json.dumps(permuted_copy_and_scalar_program()))
    s.schedule("rocm")
    fn = ctypes.CDLL(s._compile(str(tmp_path / "perm"))).perm_sdfg
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_double, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]
    fn.restype = None
    Xp = rng.standard_normal((11, 7, 5))
    Tp, Sp, ret = np.full((5, 11, 7), np.nan), np.full((11, 7, 5), np.nan), np.full(1, np.nan)
    fn(Xp.ctypes.data, Tp.ctypes.data, Sp.ctypes.data, 2.75, 11, 7, ret.ctypes.data)
    assert runtime.take_failure() == (0, "")
    assert np.array_equal(Tp, Xp.transpose(2, 0, 1)) and np.array_equal(Sp, 2.0 - Xp) and ret[0] == 2.75


def test_docc_json_expanded_softmax_runs_as_the_softmax_kernel_and_as_its_pieces(tmp_path):
    """softmax after docc's tensor-node expansion - thirteen loop nests over six Malloc'ed temporaries - imports as
    Max / Broadcast / Sub / Exp / Sum / Broadcast / Div; with the pattern pass it is one softmax launch, without it the
    seven nodes run one by one (reduction nests as reduce kernels, repeated copies as broadcasts). Both against the oracle."""
    import ctypes
    import json

    from docc_amd import runtime
    from docc_amd.sdfg import StructuredSDFG
    from test_interchange import expanded_softmax_program, numpy_softmax_expanded_program

    rng = np.random.default_rng(11)
    r, c = 77, 300
    X = (rng.standard_normal((r, c)) * 8).astype(np.float32)
    ref = oracle.softmax(X)
    # the node's own expansion, and the numpy spelling with its stride-0 views of the row maximum and the row sum
    cases = [("one", expanded_softmax_program, "softmax_sdfg", {}, "docc_rocm_softmax_f32"),
             ("pieces", expanded_softmax_program, "softmax_sdfg", {"match_softmax": False}, "docc_rocm_reduce"),
             ("np_one", numpy_softmax_expanded_program, "np_softmax_sdfg", {}, "docc_rocm_softmax_f32"),
             ("np_pieces", numpy_softmax_expanded_program, "np_softmax_sdfg", {"match_softmax": False}, "docc_rocm_elementwise_fused")]
    for name, program, function, options, launcher in cases:
        s = StructuredSDFG.parse(json.dumps(program()))
        s.schedule("rocm", options=options)
        folder = tmp_path / name
        lib = s._compile(str(folder))
        assert launcher in (folder / (function + ".cpp")).read_text()
        fn = getattr(ctypes.CDLL(lib), function)
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64]
        fn.restype = None
        Y = np.full((r, c), np.nan, np.float32)
        fn(X.ctypes.data, Y.ctypes.data, r, c)
        assert runtime.take_failure() == (0, "")
        assert rel_err_max(Y, ref) <= 1e-5, name


def test_docc_json_expanded_mean_runs(tmp_path):
    """A mean after expansion: the sum's two nests, the count set on a transition, the division by it."""
    import ctypes
    import json

    from docc_amd import runtime
    from docc_amd.sdfg import StructuredSDFG
    from test_interchange import expanded_mean_program

    s = StructuredSDFG.parse(json.dumps(expanded_mean_program()))
    s.schedule("rocm")
    fn = ctypes.CDLL(s._compile(str(tmp_path / "mean"))).mean_sdfg
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64]
    fn.restype = None
    rng = np.random.default_rng(12)
    r, c = 130, 517
    X = rng.standard_normal((r, c)).astype(np.float32)
    Y = np.full(r, np.nan, np.float32)
    fn(X.ctypes.data, Y.ctypes.data, r, c)
    assert runtime.take_failure() == (0, "")
    assert rel_err_max(Y, X.astype(np.float64).mean(axis=1)) <= 1e-5


def test_reductions_over_axes_that_are_not_adjacent():
    """Axes in several blocks: the dispatcher reduces block by block through device temporaries. numpy is the pin
    (a float64 reference; sums in another order than the reference's single loop nest, inside the usual bars)."""
    @native(target="rocm")
    def scattered(x):
        return np.sum(x, axis=(0, 2)), np.max(x, axis=(0, 2, 4)), np.mean(x, axis=(1, 3), keepdims=True), np.min(x, axis=(0, 3))

    rng = np.random.default_rng(11)
    x = rng.standard_normal((6, 5, 7, 4, 9))
    s, mx, mean, mn = scattered(x)
    assert s.shape == (5, 4, 9) and mx.shape == (5, 4) and mean.shape == (6, 1, 7, 1, 9) and mn.shape == (5, 7, 9)
    assert rel_err_max(s, x.sum(axis=(0, 2))) <= 1e-12 and np.array_equal(mx, x.max(axis=(0, 2, 4)))
    assert rel_err_max(mean, x.mean(axis=(1, 3), keepdims=True)) <= 1e-12 and np.array_equal(mn, x.min(axis=(0, 3)))
    x32 = x.astype(np.float32)
    s32, _, mean32, _ = scattered(x32)
    assert rel_err_max(s32, x32.astype(np.float64).sum(axis=(0, 2))) <= 1e-5
    assert rel_err_max(mean32, x32.astype(np.float64).mean(axis=(1, 3), keepdims=True)) <= 1e-5

    class M(torch.nn.Module):
        def forward(self, t):
            return t.sum(dim=(0, 2)) + t.amax(dim=(0, 2))

    t = torch.randn(3, 8, 5, 16, device="cuda")
    y = docc_torch.compile_torch(M(), t, target="rocm")(t)
    ref = t.double().sum(dim=(0, 2)) + t.double().amax(dim=(0, 2))
    assert rel_err_max(y.cpu().numpy(), ref.cpu().numpy()) <= 1e-5


def test_arrays_named_like_the_nodes_connectors(tmp_path):
    """Containers called A, B, C, X, Y under nodes whose connectors carry the same names, every operand copied by the
    node itself (offload "node": the connectors are bound to the caller's own arrays)."""
    import ctypes

    from docc_amd import runtime
    from docc_amd.sdfg import Pointer, PrimitiveType, Scalar, StructuredSDFGBuilder

    F64p = Pointer(Scalar(PrimitiveType.Double))
    b = StructuredSDFGBuilder("clash")
    for name in ("X", "Y", "A", "B"):
        b.add_container(name, F64p, True)
    b.add_elementwise_op("add", "Y", "X", "A", [64])        # connectors A <- Y, B <- X, C -> A
    b.add_elementwise_unary_op("relu", "A", "X", [64])      # connectors X <- A, Y -> X
    b.add_elementwise_op("mul", "X", "A", "B", [64])        # connectors A <- X, B <- A, C -> B
    s = b.move()
    s.schedule("rocm", options={"offload": "node", "fuse": False})
    fn = ctypes.CDLL(s._compile(str(tmp_path))).clash
    fn.restype = None
    rng = np.random.default_rng(4)
    X, Y = rng.standard_normal(64), rng.standard_normal(64)
    x0 = X.copy()
    A, B = np.full(64, np.nan), np.full(64, np.nan)
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    fn(ptr(X), ptr(Y), ptr(A), ptr(B))
    assert runtime.take_failure()[0] == 0
    assert np.array_equal(A, Y + x0) and np.array_equal(X, np.maximum(A, 0)) and np.array_equal(B, X * A)


def test_softmax_written_in_pieces_runs_as_the_softmax_kernel(tmp_path):
    """Seven nodes (Max, Broadcast, Sub, Exp, Sum, Broadcast, Div) are matched to one ml::Softmax before the mapping."""
    import ctypes

    from docc_amd import runtime
    from test_target_codegen import softmax_in_pieces

    s = softmax_in_pieces("pieces", [8, 16, 300], [-1])
    s.schedule("rocm")
    assert s.loop_report()["ml::Softmax::ROCMWithoutTransfers"] == 1
    fn = ctypes.CDLL(s._compile(str(tmp_path))).pieces
    fn.restype = None
    rng = np.random.default_rng(8)
    X = (rng.standard_normal((8, 16, 300)) * 8).astype(np.float32)
    Y = np.full_like(X, np.nan)
    fn(X.ctypes.data_as(ctypes.c_void_p), Y.ctypes.data_as(ctypes.c_void_p))
    assert runtime.take_failure()[0] == 0
    assert rel_err_max(Y, oracle.softmax(X.reshape(-1, 300)).reshape(X.shape)) <= 1e-5


def test_native_reductions_and_layer_statistics():
    """np.sum / max / min / mean over rows, columns and blocks of axes; the softmax pieces as values of their own."""
    @native(target="rocm")
    def stats(x):
        return np.sum(x, axis=1), x.max(axis=(1, 2), keepdims=True), np.mean(x), np.min(x, axis=0)

    @native(target="rocm")
    def centred(x):
        return x - np.mean(x, axis=0, keepdims=True)

    @native(target="rocm")
    def normalise(x):
        m = np.max(x, axis=-1, keepdims=True)
        e = np.exp(x - m)
        return e / np.sum(e, axis=-1, keepdims=True), m

    rng = np.random.default_rng(21)
    x = rng.standard_normal((12, 50, 36)).astype(np.float32)
    s, mx, mean, mn = stats(x)
    assert s.shape == (12, 36) and mx.shape == (12, 1, 1) and np.shape(mean) == () and mn.shape == (50, 36)
    np.testing.assert_allclose(s, x.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-5)
    assert np.array_equal(mx, x.max(axis=(1, 2), keepdims=True)) and np.array_equal(mn, x.min(axis=0))
    np.testing.assert_allclose(mean, x.astype(np.float64).mean(), rtol=1e-5, atol=1e-6)
    assert stats.last_sdfg.loop_report()["H2D"] == 1           # x goes to the device once for the four nodes

    y = rng.standard_normal((300, 40))
    np.testing.assert_allclose(centred(y), y - y.mean(axis=0, keepdims=True), rtol=1e-12, atol=1e-12)
    p, m = normalise(x)
    assert rel_err_max(p, oracle.softmax(x)) <= 1e-5 and np.array_equal(m, x.max(axis=-1, keepdims=True))


def test_torch_reductions_fp32():
    class Pool(torch.nn.Module):
        def forward(self, x):
            return torch.mean(x, dim=(2, 3)), x.amax(dim=1, keepdim=True)

    x = torch.randn(8, 16, 14, 14, device="cuda")
    program = docc_torch.compile_torch(Pool(), x, target="rocm")
    avg, mx = program(x)
    assert avg.is_cuda and avg.shape == (8, 16) and mx.shape == (8, 1, 14, 14)
    assert torch.allclose(avg, x.double().mean(dim=(2, 3)).float(), rtol=1e-5, atol=1e-6)
    assert torch.equal(mx, x.amax(dim=1, keepdim=True))


def test_softmax_over_other_axes_and_fp64_through_both_front_ends():
    """scipy.special.softmax with an axis argument (an inner axis, a block of axes, all axes by default) on fp32
    and fp64, and torch.softmax over a leading dim."""
    @native(target="rocm")
    def over_axis_1(x):
        return scipy.special.softmax(x, axis=1)

    @native(target="rocm")
    def over_block(x):
        return scipy.special.softmax(x, axis=(0, 1))

    @native(target="rocm")
    def over_all(x):
        return scipy.special.softmax(x)

    rng = np.random.default_rng(8)
    for dt, tol in ((np.float32, 1e-5), (np.float64, 1e-12)):
        x = (rng.standard_normal((6, 40, 24)) * 4).astype(dt)
        for fn, axes in ((over_axis_1, (1,)), (over_block, (0, 1)), (over_all, (0, 1, 2))):
            y = fn(x)
            assert y.dtype == dt and y.shape == x.shape
            assert rel_err_max(y, oracle.softmax_axes(x, axes)) <= tol
            np.testing.assert_allclose(y, scipy.special.softmax(x.astype(np.float64), axis=axes), rtol=20 * tol, atol=1e-30)

    class S(torch.nn.Module):
        def forward(self, a):
            return torch.softmax(a, dim=0)

    a = torch.randn(33, 70, dtype=torch.float64)
    out = docc_torch.compile_torch(S(), (a,), target="rocm")(a)
    assert rel_err_max(out.numpy(), oracle.softmax_axes(a.numpy(), (0,))) <= 1e-12


@pytest.mark.parametrize("D", [128, 96])
def test_torch_attention_with_other_head_dimensions(D):
    """Head dimension 128 runs the fused kernel like 64; 96 is not built, and the node brings a workspace for its
    scores (GEMM, softmax, GEMM)."""
    torch.manual_seed(5)
    Q, K, V = (torch.randn(2, 3, 200, D).bfloat16() for _ in range(3))
    for dev_in in ("cuda", "cpu"):
        program = docc_torch.compile_torch(Attn(), tuple(t.to(dev_in) for t in (Q, K, V)), target="rocm")
        out = program(*(t.to(dev_in) for t in (Q, K, V)))
        assert out.device.type == dev_in and out.dtype == torch.bfloat16 and out.shape == (2, 3, 200, D)
        assert rel_err_max(out.float().cpu().numpy(), oracle.attention(bits(Q), bits(K), bits(V))) <= 2e-2


def test_torch_bf16_products_and_linear_give_bf16_like_eager():
    """A bf16 matmul and a bf16 nn.Linear return bf16 tensors as eager torch does: float32 accumulation, the bias added in
    float32, one rounding at the end. Against the float64 product of the bf16 values rounded to bf16 (eager on the GPU
    rounds the same way, so at most a last bit of bf16 differs), and against the oracle's bf16 GEMM before the rounding."""
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = torch.nn.Linear(192, 96).bfloat16()

        def forward(self, a, b):
            return torch.matmul(a, b), self.fc(a)

    torch.manual_seed(8)
    model = Net().cuda()
    a, b = torch.randn(130, 192).bfloat16().cuda(), torch.randn(192, 72).bfloat16().cuda()
    program = docc_torch.compile_torch(model, (a, b), target="rocm")
    p, l = program(a, b)
    assert p.dtype == l.dtype == torch.bfloat16 and p.shape == (130, 72) and l.shape == (130, 96)
    wide = oracle.gemm_bf16(bits(a.cpu()), bits(b.cpu()))
    assert torch.equal(p.cpu(), torch.from_numpy(wide).bfloat16())                     # the fp32 result of the bf16 GEMM, rounded to nearest even
    with torch.no_grad():
        ref = (a.double() @ model.fc.weight.double().T + model.fc.bias.double())
        eager = model.fc(a)
    assert rel_err_max(l.float().cpu().numpy(), ref.cpu().numpy()) <= 2e-2
    assert (l.float() - eager.float()).abs().max().item() <= 2.0 ** -7 * eager.float().abs().max().item()      # a last bit of bf16 at most


def test_torch_small_batch_through_wide_layers():
    """Eight rows through nn.Linear layers of 8 M weights, bf16 and fp32 (the weights stored [out, in]): the products take the
    kernels that feed the weights straight into the MFMA, the bias and the ReLU follow as a pass over the eight rows."""
    class Net(torch.nn.Module):
        def __init__(self, dtype):
            super().__init__()
            self.up = torch.nn.Linear(2048, 4096).to(dtype)
            self.down = torch.nn.Linear(4096, 2048, bias=False).to(dtype)

        def forward(self, x):
            return self.down(torch.relu(self.up(x)))

    for dtype, tol in ((torch.bfloat16, 2e-2), (torch.float32, 1e-5)):
        torch.manual_seed(12)
        model = Net(dtype).cuda()
        x = torch.randn(8, 2048).to(dtype).cuda()
        program = docc_torch.compile_torch(model, (x,), target="rocm")
        out = program(x)
        out = out[0] if isinstance(out, (tuple, list)) else out
        assert out.dtype == dtype and out.shape == (8, 2048)
        with torch.no_grad():
            h = torch.relu(x.double() @ model.up.weight.double().T + model.up.bias.double())
            if dtype == torch.bfloat16:
                h = h.bfloat16().double()          # the layer's result is rounded to bf16 before the next one reads it
            ref = h @ model.down.weight.double().T
        assert rel_err_max(out.double().cpu().numpy(), ref.cpu().numpy()) <= tol, dtype


def test_torch_bf16_elementwise_chain_like_eager():
    """bf16 tensors outside products: elementwise operations, gelu, layer_norm, softmax and a sum run in float32 and round
    once to bf16, as eager torch computes them. Against eager on the same device, a few last bits of bf16 over the chain."""
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = torch.nn.Linear(64, 128).bfloat16()
            self.ln = torch.nn.LayerNorm(128).bfloat16()

        def forward(self, x, y):
            h = torch.nn.functional.gelu(self.up(x))
            z = self.ln(h) * 0.5 + h
            return torch.softmax(z, dim=-1), (z * y).sum(dim=0), torch.relu(z) + y.float()

    torch.manual_seed(21)
    model = Net().cuda()
    x, y = torch.randn(24, 64).bfloat16().cuda(), torch.randn(24, 128).bfloat16().cuda()
    program = docc_torch.compile_torch(model, (x, y), target="rocm")
    got = program(x, y)
    with torch.no_grad():
        eager = model(x, y)
    assert [g.dtype for g in got] == [torch.bfloat16, torch.bfloat16, torch.float32]      # bf16 with float32 promotes
    for g, e in zip(got, eager):
        assert g.shape == e.shape
        scale = e.float().abs().max().item()
        assert (g.float() - e.float()).abs().max().item() <= 4 * 2.0 ** -8 * scale


def test_torch_grouped_and_depthwise_convolutions():
    """nn.Conv2d with groups: ml::Conv carries the group, the weights [out, in / groups, kh, kw] travel as they are. A grouped
    3x3 layer and a depthwise one (as in a MobileNet block) against eager torch in float64."""
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.grouped = torch.nn.Conv2d(32, 64, 3, padding=1, groups=4)
            self.depthwise = torch.nn.Conv2d(64, 64, 3, stride=2, padding=1, groups=64, bias=False)
            self.pointwise = torch.nn.Conv2d(64, 48, 1)

        def forward(self, x):
            return self.pointwise(torch.relu(self.depthwise(torch.relu(self.grouped(x)))))

    torch.manual_seed(31)
    model = Net().cuda()
    x = torch.randn(3, 32, 20, 20).cuda()
    program = docc_torch.compile_torch(model, (x,), target="rocm")
    out = program(x)
    out = out[0] if isinstance(out, (tuple, list)) else out
    convs = [n for n in program.last_sdfg.library_nodes() if n["code"] == "ml::Conv"]
    assert [n["group"] for n in convs] == ["4", "64", "1"]
    with torch.no_grad():
        ref = model.double()(x.double())
    assert out.shape == ref.shape == (3, 48, 10, 10)
    assert rel_err_max(out.cpu().numpy(), ref.cpu().numpy()) <= 1e-5


def test_torch_attention_on_float32_tensors():
    """F.scaled_dot_product_attention on float32 tensors has no fused kernel: it runs as the nodes it is made of."""
    class Net(torch.nn.Module):
        def forward(self, q, k, v):
            return torch.nn.functional.scaled_dot_product_attention(q, k, v)

    torch.manual_seed(17)
    q, k, v = torch.randn(2, 3, 70, 24).cuda(), torch.randn(2, 3, 90, 24).cuda(), torch.randn(2, 3, 90, 24).cuda()
    program = docc_torch.compile_torch(Net(), (q, k, v), target="rocm")
    out = program(q, k, v)
    out = out[0] if isinstance(out, (tuple, list)) else out
    codes = [n["code"] for n in program.last_sdfg.library_nodes()]
    assert "ml::Attention" not in codes and "ml::Softmax" in codes and codes.count("ml::MatMul") == 2
    ref = torch.nn.functional.scaled_dot_product_attention(q.double().cpu(), k.double().cpu(), v.double().cpu())
    assert out.dtype == torch.float32 and rel_err_max(out.cpu().numpy(), ref.numpy()) <= 1e-5


def test_torch_attention_with_an_additive_mask():
    """attn_mask as a float tensor: bf16 q, k, v with a [SQ, SK] mask that closes the later keys and adds a bias, and float32
    q, k, v with a mask per batch entry. No fused kernel: products around a softmax, against eager's math in float64."""
    class Net(torch.nn.Module):
        def forward(self, q, k, v, mask):
            return torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)

    torch.manual_seed(23)
    SQ, SK, D = 70, 90, 32
    for dtype, mask_shape, tol in ((torch.bfloat16, (SQ, SK), 2e-2), (torch.float32, (2, 1, SQ, SK), 1e-5)):
        q, k, v = torch.randn(2, 3, SQ, D).to(dtype).cuda(), torch.randn(2, 3, SK, D).to(dtype).cuda(), torch.randn(2, 3, SK, D).to(dtype).cuda()
        mask = torch.randn(mask_shape) * 0.5
        mask.masked_fill_(torch.arange(SK)[None, :] > torch.arange(SQ)[:, None] + 20, float("-inf"))
        mask = mask.cuda()
        program = docc_torch.compile_torch(Net(), (q, k, v, mask), target="rocm")
        out = program(q, k, v, mask)
        out = out[0] if isinstance(out, (tuple, list)) else out
        assert "ml::Attention" not in [n["code"] for n in program.last_sdfg.library_nodes()]
        ref = torch.nn.functional.scaled_dot_product_attention(q.double().cpu(), k.double().cpu(), v.double().cpu(), attn_mask=mask.double().cpu())
        assert out.dtype == dtype and rel_err_max(out.float().cpu().numpy(), ref.numpy()) <= tol, dtype


def test_torch_causal_attention():
    """F.scaled_dot_product_attention(..., is_causal=True): ml::Attention with the causal flag, on the fused kernel's causal
    form (head dim 64) and through the widened operands (head dim 80). Against eager torch's math in float64."""
    class Net(torch.nn.Module):
        def forward(self, q, k, v):
            return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)

    for D in (64, 80):
        torch.manual_seed(D)
        q, k, v = (torch.randn(2, 3, 300, D).bfloat16().cuda() for _ in range(3))
        program = docc_torch.compile_torch(Net(), (q, k, v), target="rocm")
        out = program(q, k, v)
        out = out[0] if isinstance(out, (tuple, list)) else out
        (node,) = [n for n in program.last_sdfg.library_nodes() if n["code"] == "ml::Attention"]
        assert node["causal"] is True
        ref = torch.nn.functional.scaled_dot_product_attention(q.double().cpu(), k.double().cpu(), v.double().cpu(), is_causal=True)
        assert out.dtype == torch.bfloat16 and out.shape == (2, 3, 300, D)
        assert rel_err_max(out.float().cpu().numpy(), ref.numpy()) <= 2e-2


def test_power_operator_through_both_front_ends():
    """x ** 2, x ** y and np.power lower to ml::Pow (array or scalar operand); torch.pow likewise."""
    @native(target="rocm")
    def norms(x, y):
        return np.sqrt(x ** 2 + np.power(y, 2.0)) ** (y / 4)

    rng = np.random.default_rng(21)
    x, y = rng.standard_normal((64, 50)), rng.standard_normal((64, 50))
    got = norms(x, y)
    ref = np.sqrt(x ** 2 + y ** 2) ** (y / 4)
    np.testing.assert_allclose(got, ref, rtol=1e-13)
    # the whole expression is one chain of elementwise nodes: scheduled, it is one generated kernel with the three powers
    (nest,) = [n for n in norms.last_sdfg.library_nodes() if n["code"] == "ROCMMap"]
    assert [st["op"] for st in nest["statements"]].count("pow") == 3 and len(nest["reads"]) == 2

    class P(torch.nn.Module):
        def forward(self, a, b):
            return torch.pow(a.abs(), b) + a ** 2

    a, b = torch.randn(40, 30), torch.randn(40, 30)
    out = docc_torch.compile_torch(P(), (a, b), target="rocm")(a, b)
    np.testing.assert_allclose(out.numpy(), (a.abs() ** b + a ** 2).numpy(), rtol=2e-6)


def test_transposes_through_both_front_ends():
    @native(target="rocm")
    def mix(a, b, x):
        g = a.T @ a                                  # GEMM flag
        return np.transpose(x, (2, 0, 1)) * 2.0, a.T + b, g

    rng = np.random.default_rng(31)
    a, b, x = rng.standard_normal((60, 40)), rng.standard_normal((40, 60)), rng.standard_normal((5, 6, 7))
    p, s, g = mix(a, b, x)
    assert np.array_equal(p, np.transpose(x, (2, 0, 1)) * 2.0) and np.array_equal(s, a.T + b)
    assert rel_err_max(g, oracle.gemm(np.ascontiguousarray(a.T), a, variant="ld")) <= 1e-12

    class P(torch.nn.Module):
        def forward(self, t, u):
            return (t.permute(0, 2, 1, 3) + 1.0, torch.relu(u.transpose(0, 1)), t.transpose(1, 2).contiguous())

    t, u = torch.randn(2, 3, 4, 5), torch.randn(30, 20, dtype=torch.float64)
    o1, o2, o3 = docc_torch.compile_torch(P(), (t, u), target="rocm")(t, u)
    assert torch.equal(o1, t.permute(0, 2, 1, 3) + 1.0) and torch.equal(o2, torch.relu(u.transpose(0, 1)))
    assert torch.equal(o3, t.transpose(1, 2).contiguous())


def test_standard_deviation_is_the_reference_node_chain():
    """np.std / torch.std(correction=0): Mul, Mean, Mean, Mul, Sub, Sqrt, the chain StdNode::expand builds
    (population value, sqrt(mean(x^2) - mean(x)^2))."""
    @native(target="rocm")
    def spread(x):
        return np.std(x, axis=1), x.std(axis=(0, 1), keepdims=True)

    rng = np.random.default_rng(17)
    x = rng.standard_normal((40, 300, 6)) * 3 + 1.5
    a, b = spread(x)
    codes = [n["code"] for n in spread.last_sdfg.library_nodes() if n["code"].startswith("ml::")]
    assert codes[:6] == ["ml::Mul", "ml::Mean", "ml::Mean", "ml::Mul", "ml::Sub", "ml::Sqrt"]
    np.testing.assert_allclose(a, np.std(x, axis=1), rtol=1e-10)
    np.testing.assert_allclose(b, np.std(x, axis=(0, 1), keepdims=True), rtol=1e-10)
    # the same steps on the CPU oracle, bit for bit
    m2 = oracle.reduce("mean", oracle.elementwise_binary("mul", x, x), (1,))
    m1 = oracle.reduce("mean", x, (1,))
    want = oracle.elementwise_unary("sqrt", oracle.elementwise_binary("sub", m2, oracle.elementwise_binary("mul", m1, m1)))
    np.testing.assert_allclose(a, want, rtol=1e-12)

    class S(torch.nn.Module):
        def forward(self, t):
            return torch.std(t, dim=-1, correction=0)

    t = torch.randn(64, 500)
    out = docc_torch.compile_torch(S(), (t,), target="rocm")(t)
    np.testing.assert_allclose(out.numpy(), t.std(dim=-1, correction=0).numpy(), rtol=2e-4)


def test_casts_through_both_front_ends():
    @native(target="rocm")
    def widen(x, k):
        return np.sqrt(x.astype(np.float64)) + k.astype(np.float64)

    rng = np.random.default_rng(5)
    x = np.abs(rng.standard_normal((30, 50))).astype(np.float32)
    k = rng.integers(-5, 5, (30, 50))
    got = widen(x, k)
    assert got.dtype == np.float64
    np.testing.assert_array_equal(got, np.sqrt(x.astype(np.float64)) + k.astype(np.float64))
    # the cast from integers is a prebuilt kernel; the widening of x, the square root and the addition are one generated kernel
    nodes = [n for n in widen.last_sdfg.library_nodes() if n["code"] != "ROCMOffloading"]
    assert [n["code"] for n in nodes] == ["ml::Cast", "ROCMMap"]
    assert [(st["op"], st["type"]) for st in nodes[1]["statements"]] == [("assign", "Double"), ("sqrt", "Double"), ("fp_add", "Double")]
    assert sorted(r["element_type"] for r in nodes[1]["reads"]) == ["Double", "Float"]

    class Mixed(torch.nn.Module):
        def forward(self, q, k, v):
            s = torch.matmul(q.bfloat16(), k.bfloat16().transpose(-2, -1)) / 8.0
            return torch.matmul(torch.softmax(s, dim=-1), v.bfloat16()).float()

    torch.manual_seed(9)
    q, k, v = (torch.randn(1, 2, 96, 64) for _ in range(3))
    out = docc_torch.compile_torch(Mixed(), (q, k, v), target="rocm")(q, k, v)
    assert out.dtype == torch.float32
    ref = oracle.attention(bits(q.bfloat16()), bits(k.bfloat16()), bits(v.bfloat16()))
    assert rel_err_max(out.numpy(), ref) <= 2e-2


def test_products_with_vectors_follow_numpy():
    @native(target="rocm")
    def products(a, x, y):
        return a @ x, y @ a, x @ x, a.T @ y

    rng = np.random.default_rng(2)
    a, x, y = rng.standard_normal((300, 200)), rng.standard_normal(200), rng.standard_normal(300)
    ax, ya, xx, aty = products(a, x, y)
    assert ax.shape == (300,) and ya.shape == (200,) and aty.shape == (200,) and np.ndim(xx) == 0
    assert rel_err_max(ax, a @ x) <= 1e-12 and rel_err_max(ya, y @ a) <= 1e-12 and rel_err_max(aty, a.T @ y) <= 1e-12      # the fp64 GEMM bar
    np.testing.assert_allclose(xx, x @ x, rtol=1e-13)
    codes = [n["code"] for n in products.last_sdfg.library_nodes() if not n["code"].startswith("ROCM")]
    assert codes == ["GEMM", "GEMM", "ml::Mul", "ml::Sum", "GEMM"]


@pytest.mark.parametrize("approximate", ["none", "tanh"])
def test_torch_compile_transformer_mlp_block(approximate):
    """LayerNorm -> Linear -> GELU -> Linear and the residual, on device tensors: the pieces of the norm and of the
    activation are tensor nodes that the target merges into generated kernels. Against the model in float64."""
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.LayerNorm(256)
            self.fc1 = torch.nn.Linear(256, 1024)
            self.act = torch.nn.GELU(approximate=approximate)
            self.fc2 = torch.nn.Linear(1024, 256)

        def forward(self, x):
            return x + self.fc2(self.act(self.fc1(self.norm(x))))

    torch.manual_seed(3)
    model = Block().cuda()
    with torch.no_grad():
        model.norm.weight.uniform_(0.5, 1.5)
        model.norm.bias.uniform_(-0.5, 0.5)
    x = torch.randn(8, 128, 256, device="cuda") * 2 + 0.5
    program = docc_torch.compile_torch(model, x, target="rocm")
    y = program(x)
    assert y.is_cuda and y.shape == x.shape
    with torch.no_grad():
        ref = model.double()(x.double())
    assert rel_err_max(y.cpu().numpy(), ref.cpu().numpy()) <= 1e-5
    kernels = [n["code"] for n in program.last_sdfg.library_nodes() if n["code"] != "ROCMOffloading"]
    assert kernels.count("GEMM") == 2 and kernels.count("ml::Mean") == 2 and kernels.count("ROCMMap") == 3 and len(kernels) == 8, kernels


def test_torch_compile_composite_elementwise_operations():
    class Misc(torch.nn.Module):
        def forward(self, a, b):
            F = torch.nn.functional
            return F.silu(a) * torch.rsqrt(b.square() + 1.0) - (-a).reciprocal() + F.gelu(b, approximate="tanh")

    torch.manual_seed(4)
    for dtype, tol in ((torch.float32, 1e-5), (torch.float64, 1e-12)):
        a, b = torch.randn(37, 129, dtype=dtype) + 3.0, torch.randn(37, 129, dtype=dtype)
        program = docc_torch.compile_torch(Misc(), (a, b), target="rocm")
        out = program(a, b)
        ref = Misc()(a.double(), b.double())
        assert out.dtype == dtype and rel_err_max(out.numpy(), ref.numpy()) <= tol
        assert [n["code"] for n in program.last_sdfg.library_nodes() if n["code"] != "ROCMOffloading"] == ["ROCMMap"]

    class Norm(torch.nn.Module):
        def forward(self, x, w):
            return torch.nn.functional.layer_norm(x, (6, 40), weight=w, eps=1e-3)

    x, w = torch.randn(5, 7, 6, 40), torch.rand(6, 40) + 0.5
    out = docc_torch.compile_torch(Norm(), (x, w), target="rocm")(x, w)
    assert rel_err_max(out.numpy(), Norm()(x.double(), w.double()).numpy()) <= 1e-5
