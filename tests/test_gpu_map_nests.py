"""Loop nests of maps that are not one of the prebuilt kernels, run as generated gfx950 kernels: a docc-layout program is
imported (ROCMMap nodes), scheduled, its kernels are compiled with hipcc next to the generated library, and the host
code launches them through docc_rocm_module_load / _module_get_function / _launch. Checked against the oracle's
interpreter of the same body (the loop the reference's openmp target prints) and against numpy spelled by hand.

The arithmetic tasklets are IEEE operations compiled without contraction: bit-exact. Calls into the math library
(CMath): 1e-5 (fp32) / 1e-12 (fp64) norm-wise relative error."""
import ctypes
import json

import numpy as np
import pytest

import oracle
from docc_amd import runtime
from docc_amd.sdfg import StructuredSDFG
from gpu_util import rel_err_max
from test_interchange import (DOUBLE, FLOAT, INT64, NO_DEBUG, Ids, cmath, docc_map_nest, docc_sdfg, fused_map_program, pointer,
                              scalar, tasklet)

pytestmark = pytest.mark.gpu


def compiled(program, folder, name, argtypes):
    s = StructuredSDFG.from_docc_json(json.dumps(program))
    nodes = [n for n in s.library_nodes()]
    s.schedule("rocm")
    fn = getattr(ctypes.CDLL(s._compile(str(folder))), name)
    fn.argtypes = argtypes
    fn.restype = None
    return fn, nodes


@pytest.mark.parametrize("prim,shape", [(FLOAT, (64, 256)), (FLOAT, (37, 129)), (DOUBLE, (33, 64)), (DOUBLE, (5, 7)), (FLOAT, (1, 4)),
                                        (FLOAT, (1024, 2048))])
def test_fused_maps_run_as_generated_kernels(tmp_path, prim, shape, rt):
    """Y = relu(A * B + c) as MapFusion leaves it (three blocks, scalar temporaries), then Z = (A - Y) / 3 with W = Z^T from
    one chain. Inner extents that are multiples of the vector width take the 128-bit variant, the others the scalar one."""
    dt = np.float32 if prim == FLOAT else np.float64
    fn, nodes = compiled(fused_map_program(prim), tmp_path, "fused_maps_sdfg", [ctypes.c_void_p] * 6 + [ctypes.c_int64] * 2)
    assert [n["code"] for n in nodes] == ["ROCMMap", "ROCMMap"]
    rng = np.random.default_rng(21)
    r, c = shape
    A, B = (rng.standard_normal((r, c)).astype(dt) for _ in range(2))
    C = rng.standard_normal(c).astype(dt)
    Y, Z = (np.full((r, c), np.nan, dt) for _ in range(2))
    W = np.full((c, r), np.nan, dt)
    fn(*(a.ctypes.data for a in (A, B, C, Y, Z, W)), r, c)
    assert runtime.take_failure() == (0, "")
    # numpy, spelled by hand
    y_ref = np.maximum(dt(0), A * B + C)
    z_ref = (A - y_ref) / dt(3)
    assert np.array_equal(Y, y_ref) and np.array_equal(Z, z_ref) and np.array_equal(W, z_ref.T)
    # the oracle on the imported bodies
    syms = {"_s0": r, "_s1": c}
    first = oracle.map_nest(nodes[0], {"_in0": A, "_in1": B, "_in2": C}, symbols=syms)
    assert np.array_equal(Y.reshape(-1), first["_out0"])
    second = oracle.map_nest(nodes[1], {"_in0": A, "_in1": Y}, symbols=syms)
    assert np.array_equal(Z.reshape(-1), second["_out0"]) and np.array_equal(W.reshape(-1), second["_out1"])


def math_program(prim):
    """One nest over [_s0, _s1, 6]: E = exp(X) * s + lgamma(|X| + 1) (a scalar argument, four operations in one block),
    F = fma(X, X, E) rounded once, G[k][i][j] = tanh(F[i][j][k]) stored permuted, H = fmod(X, 0.75) in place of X's copy."""
    ids = Ids()
    containers = {n: pointer(prim) for n in ("X", "E", "F", "G", "H")}
    for n in ("_s0", "_s1", "_i0", "_i1", "_i2"):
        containers[n] = scalar(INT64)
    for n in ("s", "_t0", "_t1", "_t2", "_t3", "_t4"):
        containers[n] = scalar(prim)
    P, S = pointer(prim), scalar(prim)
    loops = [("_i0", "_s0"), ("_i1", "_s1"), ("_i2", "6")]
    lin = ["_i2 + 6*_i1 + 6*_i0*_s1"]
    perm = ["_i1 + _i0*_s1 + _i2*_s0*_s1"]
    lit = (lambda v: (v + "f", prim)) if prim == FLOAT else (lambda v: (v, prim))
    body = [
        [(cmath("exp", prim), [("_in1", "X", lin, P)], [("_t0", [], S)]),
         (tasklet(4, 2), [("_in1", "_t0", [], S), ("_in2", "s", [], S)], [("_t1", [], S)]),
         (cmath("fabs", prim), [("_in1", "X", lin, P)], [("_t2", [], S)]),
         (tasklet(2, 2), [("_in1", "_t2", [], S), ("_in2", lit("1.0"), [], S)], [("_t3", [], S)]),
         (cmath("lgamma", prim), [("_in1", "_t3", [], S)], [("_t4", [], S)])],
        [(tasklet(2, 2), [("_in1", "_t1", [], S), ("_in2", "_t4", [], S)], [("E", lin, P)])],
        [(tasklet(7, 3), [("_in1", "X", lin, P), ("_in2", "X", lin, P), ("_in3", "E", lin, P)], [("F", lin, P)])],
        [(cmath("tanh", prim), [("_in1", "F", lin, P)], [("G", perm, P)])],
        [(tasklet(6, 2), [("_in1", "X", lin, P), ("_in2", lit("0.75"), [], S)], [("H", lin, P)])],
    ]
    children = [docc_map_nest(ids, loops, body), {"type": "return", "element_id": ids(), "data": "", "debug_info": NO_DEBUG}]
    return docc_sdfg("math_maps_sdfg", containers, ["X", "E", "F", "G", "H", "s", "_s0", "_s1"], children, ids)


@pytest.mark.parametrize("prim", [FLOAT, DOUBLE])
def test_math_calls_scalar_arguments_and_permuted_stores(tmp_path, prim, rt):
    dt, ct = (np.float32, ctypes.c_float) if prim == FLOAT else (np.float64, ctypes.c_double)
    tol = 1e-5 if prim == FLOAT else 1e-12
    fn, nodes = compiled(math_program(prim), tmp_path, "math_maps_sdfg", [ctypes.c_void_p] * 5 + [ct, ctypes.c_int64, ctypes.c_int64])
    (node,) = nodes
    assert node["code"] == "ROCMMap" and len(node["reads"]) == 1 and len(node["writes"]) == 4 and [s["connector"] for s in node["scalars"]] == ["_c0"]
    rng = np.random.default_rng(22)
    r, c = 19, 10
    X = (rng.standard_normal((r, c, 6)) * 1.5).astype(dt)
    E, F, H = (np.full((r, c, 6), np.nan, dt) for _ in range(3))
    G = np.full((6, r, c), np.nan, dt)
    fn(*(a.ctypes.data for a in (X, E, F, G, H)), 0.625, r, c)
    assert runtime.take_failure() == (0, "")
    ref = oracle.map_nest(node, {"_in0": X}, scalars={"_c0": 0.625}, symbols={"_s0": r, "_s1": c})
    by_container = dict(zip(("E", "F", "G", "H"), (ref[w["connector"]] for w in node["writes"])))
    assert rel_err_max(E, by_container["E"].reshape(E.shape)) <= tol
    assert rel_err_max(F, by_container["F"].reshape(F.shape)) <= tol
    assert rel_err_max(G, by_container["G"].reshape(G.shape)) <= tol
    assert np.array_equal(H, by_container["H"].reshape(H.shape))                        # fmod is exact
    # by hand, in float64
    import scipy.special as sp
    Xd = X.astype(np.float64)
    e = np.exp(Xd) * 0.625 + sp.gammaln(np.abs(Xd) + 1.0)
    assert rel_err_max(E, e) <= tol and rel_err_max(F, Xd * Xd + e) <= tol
    assert rel_err_max(G, np.tanh(Xd * Xd + e).transpose(2, 0, 1)) <= tol and np.array_equal(H, np.fmod(X, dt(0.75)))


def test_generated_kernel_at_the_size_of_the_memory_bound_configuration(tmp_path, rt):
    """[8192, 4096] fp32: the nest collapses to one loop, 32-bit indices, 128-bit accesses; checked whole against numpy."""
    fn, _ = compiled(fused_map_program(FLOAT), tmp_path, "fused_maps_sdfg", [ctypes.c_void_p] * 6 + [ctypes.c_int64] * 2)
    rng = np.random.default_rng(23)
    r, c = 8192, 4096
    A, B = (rng.standard_normal((r, c), dtype=np.float32) for _ in range(2))
    C = rng.standard_normal(c, dtype=np.float32)
    Y, Z = (np.empty((r, c), np.float32) for _ in range(2))
    W = np.empty((c, r), np.float32)
    fn(*(a.ctypes.data for a in (A, B, C, Y, Z, W)), r, c)
    assert runtime.take_failure() == (0, "")
    y_ref = np.maximum(np.float32(0), A * B + C)
    assert np.array_equal(Y, y_ref)
    z_ref = (A - y_ref) / np.float32(3)
    assert np.array_equal(Z, z_ref) and np.array_equal(W, z_ref.T)


def test_module_load_get_function_and_launch(tmp_path, rt):
    """The three runtime calls generated host code reaches its kernels through, called directly: a kernel image compiled
    from a generated snippet is loaded, its entry points are found by name, and a launch with the parameter list of
    the kernel runs it; a missing image, a missing name and an oversized block are reported as errors."""
    import torch
    s = StructuredSDFG.from_docc_json(json.dumps(fused_map_program(FLOAT)))
    s.schedule("rocm", options={"offload": "none", "fuse_maps": False})      # the two nests as they were written: two kernels
    s._compile(str(tmp_path))
    images = sorted(tmp_path.glob("kernel_*.hsaco"))
    assert len(images) == 2
    (first,) = [i for i in images if "p__in2" in i.with_suffix(".hip").read_text()]      # the nest with three operands read
    module = ctypes.c_void_p()
    rt.call("docc_rocm_module_load", str(first).encode(), ctypes.byref(module))
    fn = ctypes.c_void_p()
    rt.call("docc_rocm_module_get_function", module, (first.stem + "_v32").encode(), ctypes.byref(fn))
    assert fn.value
    with pytest.raises(rt.RocmRuntimeError, match="not found"):
        rt.call("docc_rocm_module_get_function", module, b"no_such_kernel", ctypes.byref(ctypes.c_void_p()))
    with pytest.raises(rt.RocmRuntimeError, match="cannot load"):
        rt.call("docc_rocm_module_load", str(tmp_path / "missing.hsaco").encode(), ctypes.byref(ctypes.c_void_p()))
    r, c = 48, 64
    a, b = torch.randn(r, c, device="cuda"), torch.randn(r, c, device="cuda")
    bias = torch.randn(c, device="cuda")
    y = torch.full((r, c), float("nan"), device="cuda")
    # parameters of the first nest's kernel: the four pointers, two bounds, three row strides
    values = [ctypes.c_void_p(t.data_ptr()) for t in (a, b, bias, y)] + [ctypes.c_longlong(v) for v in (r, c, c, c, c)]
    args = (ctypes.c_void_p * len(values))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in values])
    grid, block = (ctypes.c_uint32 * 3)((r * c // 4 + 255) // 256, 1, 1), (ctypes.c_uint32 * 3)(256, 1, 1)
    torch.cuda.synchronize()
    rt.call("docc_rocm_launch", fn, grid, block, 0, None, args)
    rt.device_sync()
    assert torch.equal(y, torch.relu(a * b + bias))
    # an empty grid is no launch; a block of more than 1024 threads is refused before the driver sees it
    rt.call("docc_rocm_launch", fn, (ctypes.c_uint32 * 3)(0, 1, 1), block, 0, None, args)
    with pytest.raises(rt.RocmRuntimeError, match="block of 2048 threads"):
        rt.call("docc_rocm_launch", fn, grid, (ctypes.c_uint32 * 3)(2048, 1, 1), 0, None, args)
    rt.call("docc_rocm_module_unload", module)


def test_generated_kernel_with_64_bit_indices(tmp_path, rt):
    """More than 2^31 elements per operand: the host code picks the entry points that compute indices in 64 bits (the
    vector form for the aligned extent, the element form for an extent that is no multiple of four)."""
    import torch
    from docc_amd.sdfg import Pointer, PrimitiveType, Scalar, StructuredSDFGBuilder

    b = StructuredSDFGBuilder("wide_map")
    for n in ("A", "Y"):
        b.add_container(n, Pointer(Scalar(PrimitiveType.Float)), True)
    b.add_container("_s0", Scalar(PrimitiveType.Int64), True)
    b.add_map_nest([("i", "_s0")], [("a", "A", ["1"])], [("t", "fp_mul", ["a", 2.0]), ("u", "fp_add", ["t", 1.0])], [("Y", ["1"], "u")])
    s = b.move()
    s.schedule("rocm", options={"offload": "none"})
    fn = ctypes.CDLL(s._compile(str(tmp_path))).wide_map
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    fn.restype = None
    n = (1 << 31) + 4096
    a = torch.empty(n + 3, device="cuda")
    a[: 1 << 20] = torch.arange(1 << 20, device="cuda", dtype=torch.float32)
    a[1 << 20:] = 3.0
    a[n - 5:] = torch.arange(8, device="cuda", dtype=torch.float32)        # the far end, past 2^31
    y = torch.zeros(n + 3, device="cuda")
    for count in (n, n + 3):                                                 # a multiple of four, then not
        y.zero_()
        torch.cuda.synchronize()
        fn(a.data_ptr(), y.data_ptr(), count)
        torch.cuda.synchronize()
        assert runtime.take_failure() == (0, "")
        assert torch.equal(y[: 1 << 20], a[: 1 << 20] * 2 + 1)
        assert torch.equal(y[count - 8:count], a[count - 8:count] * 2 + 1)
        assert float(y[(1 << 31) + 7]) == 7.0 and (count == n + 3 or float(y[n:].abs().max()) == 0.0)
        # a checksum over everything: 2 * sum(a) + count, in float64 by chunks
        total = sum(float(y[i:i + (1 << 28)].double().sum()) for i in range(0, count, 1 << 28))
        ref = sum(float(a[i:min(i + (1 << 28), count)].double().sum()) for i in range(0, count, 1 << 28)) * 2 + count
        assert abs(total - ref) <= 1e-9 * ref


# ---- chains of tensor nodes merged into one generated kernel (RocmMapFusionPass)

def chain_program(name, elem, shape):
    """y = sigmoid((a + b) * c - bias_row) * 0.5 + max(a, col) over `shape` = [r, c]: five two-operand operations, a
    repeated row, a repeated column and a constant, which the prebuilt fused kernel (one two-operand operation) cannot
    take in one launch."""
    from docc_amd.sdfg import Pointer, PrimitiveType, Scalar, StructuredSDFGBuilder
    T = Pointer(Scalar(PrimitiveType.Float if elem == np.float32 else PrimitiveType.Double))
    r, c = shape
    size = np.dtype(elem).itemsize
    b = StructuredSDFGBuilder(name)
    for n in ("A", "B", "C", "bias", "col", "Y"):
        b.add_container(n, T, True)
    for n in ("T0", "T1", "T2", "T3", "T4", "T5", "T6", "T7"):
        b.add_container(n, T, False, transient_bytes=r * c * size)
    b.add_elementwise_op("add", "A", "B", "T0", [r, c])
    b.add_elementwise_op("mul", "T0", "C", "T1", [r, c])
    b.add_broadcast("bias", "T2", [1, c], [r, c])
    b.add_elementwise_op("sub", "T1", "T2", "T3", [r, c])
    b.add_elementwise_unary_op("sigmoid", "T3", "T4", [r, c])
    b.add_elementwise_op("mul", "T4", "0.5", "T5", [r, c])
    b.add_broadcast("col", "T6", [r, 1], [r, c])
    b.add_elementwise_op("max", "A", "T6", "T7", [r, c])
    b.add_elementwise_op("add", "T5", "T7", "Y", [r, c])
    return b.move()


@pytest.mark.parametrize("elem,shape", [(np.float32, (64, 256)), (np.float32, (37, 129)), (np.float64, (33, 64)), (np.float32, (1, 8)),
                                        (np.float32, (2048, 1024))])
def test_chain_of_tensor_nodes_runs_as_one_generated_kernel(tmp_path, rt, elem, shape):
    r, c = shape
    rng = np.random.default_rng(31)
    A, B, C = (rng.standard_normal((r, c)).astype(elem) for _ in range(3))
    bias, col = rng.standard_normal(c).astype(elem), rng.standard_normal(r).astype(elem)
    results = {}
    for fuse_maps in (True, False):
        s = chain_program(f"chain_{int(fuse_maps)}", elem, shape)
        s.schedule("rocm", options={"fuse_maps": fuse_maps})
        kernels = [n for n in s.library_nodes() if n["code"] != "ROCMOffloading"]
        if fuse_maps:
            assert [n["code"] for n in kernels] == ["ROCMMap"] and s.loop_report()["H2D"] == 5 and s.loop_report()["D2H"] == 1
            node, fused_text = kernels[0], s.to_json()
        else:
            assert len(kernels) >= 4 and not any(n["code"] == "ROCMMap" for n in kernels)
        fn = getattr(ctypes.CDLL(s._compile(str(tmp_path / str(fuse_maps)))), f"chain_{int(fuse_maps)}")
        fn.argtypes = [ctypes.c_void_p] * 6
        fn.restype = None
        Y = np.full((r, c), np.nan, elem)
        fn(*(a.ctypes.data for a in (A, B, C, bias, col, Y)))
        assert runtime.take_failure() == (0, "")
        results[fuse_maps] = Y
    # the same operations in the same order, each rounded once: the merged kernel gives the bits of the launches it replaces
    assert np.array_equal(results[True], results[False])
    # the oracle's interpreter on the merged body, each load bound to the array its connector names
    arrays = {"A": A, "B": B, "C": C, "bias": bias, "col": col}
    operands, scalars = {}, {}
    for blk in json.loads(fused_text)["root"]["children"]:
        if blk["dataflow"]["library_node"]["code"] != "ROCMMap":
            continue
        for binding in blk["dataflow"]["inputs"]:
            if "constant" in binding:
                scalars[binding["connector"]] = float(binding["constant"])
            else:
                operands[binding["connector"]] = arrays[binding["data"].rsplit("_", 1)[1]]
    assert len(operands) == 5 and list(scalars.values()) == [0.5]           # A is loaded once for its two uses
    ref = oracle.map_nest(node, operands, scalars=scalars)
    assert rel_err_max(results[True], ref["_out0"].reshape(r, c)) <= (1e-5 if elem == np.float32 else 1e-12)
    # by hand, in float64
    d = lambda x: x.astype(np.float64)
    hand = 1.0 / (1.0 + np.exp(-((d(A) + d(B)) * d(C) - d(bias)[None, :]))) * 0.5 + np.maximum(d(A), d(col)[:, None])
    assert rel_err_max(results[True], hand) <= (2e-6 if elem == np.float32 else 1e-12)


CHAIN_SOURCES = [
    ("np.tanh(x * y + b) / (np.abs(z) + 1.5)", 1),
    ("np.maximum(x, c) - np.minimum(y, z) * np.exp(-np.abs(x))", 1),
    ("(x + b) * (y + c) + np.sqrt(np.abs(z)) * 0.25", 2),
    ("1.0 / (1.0 + np.exp(-(x * 0.5 + y * z)))", 1),
    ("np.sqrt(x * x + y * y + z * z) - b", 1),
    ("((x - y) ** 2 + c) * np.tanh(z)", 1),
]


@pytest.mark.parametrize("case", range(len(CHAIN_SOURCES)))
@pytest.mark.parametrize("dt", [np.float32, np.float64], ids=["f32", "f64"])
def test_numpy_expressions_merge_into_generated_kernels(tmp_path, case, dt):
    """numpy expressions with several two-operand operations, a bias row `b` and a column `c`, through @native: merged into
    generated kernels (at most as many as the comment says), with the bits of the unmerged program and numpy's values."""
    import importlib.util
    import sys
    from docc_amd.python import native    # noqa: F401  (the generated module imports it)
    expr, max_kernels = CHAIN_SOURCES[case]
    src = ("import numpy as np\nfrom docc_amd.python import native\n\n"
           f"@native(target='rocm')\ndef merged(x, y, z, b, c):\n    return {expr}\n\n"
           f"@native(target='rocm', fuse_maps=False)\ndef apart(x, y, z, b, c):\n    return {expr}\n")
    path = tmp_path / f"chain_case_{case}_{np.dtype(dt).name}.py"
    path.write_text(src)
    spec = importlib.util.spec_from_file_location(path.stem, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[path.stem] = mod
    spec.loader.exec_module(mod)
    rng = np.random.default_rng(40 + case)
    r, cols = 96, 200
    x, y, z = (rng.standard_normal((r, cols)).astype(dt) for _ in range(3))
    b, c = rng.standard_normal((1, cols)).astype(dt), rng.standard_normal((r, 1)).astype(dt)
    got, ref = mod.merged(x, y, z, b, c), mod.apart(x, y, z, b, c)
    assert got.dtype == dt and got.shape == (r, cols)
    assert np.array_equal(got, ref)
    want = eval(expr, {"np": np, "x": x.astype(np.float64), "y": y.astype(np.float64), "z": z.astype(np.float64),
                       "b": b.astype(np.float64), "c": c.astype(np.float64)})
    assert rel_err_max(got, want) <= (2e-5 if dt == np.float32 else 1e-12)
    kinds = [n["code"] for n in mod.merged.last_sdfg.library_nodes() if n["code"] != "ROCMOffloading"]
    assert kinds.count("ROCMMap") >= 1 and len(kinds) <= max_kernels, kinds
    assert "ROCMMap" not in [n["code"] for n in mod.apart.last_sdfg.library_nodes()]
