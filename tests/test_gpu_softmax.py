"""ml::Softmax on the GPU against the CPU oracle, through the C-ABI
(docc_rocm_softmax_f32). Tolerance: 1e-5 norm-wise relative error
(max|y - y_ref| / max|y_ref|), the fp32 bar."""
import numpy as np
import pytest
import scipy.special
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5


def run_softmax(rt, X: np.ndarray) -> np.ndarray:
    x = dev(X)
    y = torch.empty_like(x)
    cols = X.shape[-1]
    rows = X.size // cols if cols else 0
    rt.softmax_f32(rows, cols, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    return host(y)


@pytest.mark.parametrize(
    "rows,cols",
    [(1, 1), (3, 4), (8, 257), (5, 7), (64, 256), (33, 260), (17, 1024), (6, 1028), (9, 2048), (9, 2052), (11, 3000),
     (5, 4092), (16, 4096), (7, 4100), (5, 8192), (3, 16384), (2, 16388), (2, 40000), (1000, 12), (4, 3)],
)
def test_softmax_matches_oracle(rt, rows, cols):
    rng = np.random.default_rng(rows * 100003 + cols)
    X = (rng.standard_normal((rows, cols)) * 8).astype(np.float32)
    Y = run_softmax(rt, X)
    ref = oracle.softmax(X)
    assert rel_err_max(Y, ref) <= TOL_F32
    # element-wise as well: 2e-6 relative plus an absolute floor for denormal outputs
    np.testing.assert_allclose(Y, ref, rtol=2e-5, atol=1e-30)
    np.testing.assert_allclose(Y.sum(axis=-1), 1.0, rtol=0, atol=1e-5)


@pytest.mark.parametrize(
    "rows,cols",
    [(1000, 4), (999, 8), (77, 12), (513, 16), (130, 28), (4099, 32), (65, 60), (1025, 64), (300, 100), (259, 128)],
)
def test_softmax_rows_that_share_a_wavefront(rt, rows, cols):
    """Up to 128 columns several rows share a wavefront (1 to 32 lanes a row, four sets of rows per wavefront): row counts
    that end inside a set, inside a wavefront and inside a work-group, widths that fill the lanes of a row and that do not."""
    rng = np.random.default_rng(rows * 1009 + cols)
    X = (rng.standard_normal((rows, cols)) * 8).astype(np.float32)
    X[rows // 2] = -np.inf                       # max = -inf: NaN for that row only
    X[rows // 3, cols // 2] = -np.inf            # weight 0
    Y = run_softmax(rt, X)
    with np.errstate(invalid="ignore"):
        ref = oracle.softmax(X)
    assert np.isnan(Y[rows // 2]).all() and not np.isnan(np.delete(Y, rows // 2, axis=0)).any()
    ok = ~np.isnan(ref)
    assert Y[rows // 3, cols // 2] == 0.0
    np.testing.assert_allclose(Y[ok], ref[ok], rtol=2e-5, atol=1e-30)


@pytest.mark.parametrize(
    "rows,cols",
    [(130, 16388), (128, 32768), (200, 32772), (140, 65536), (129, 50000), (130, 20001), (129, 65535), (128, 32770),   # sixteen wavefronts hold a row
     (3, 16388), (2, 40000), (100, 65540), (5, 300000), (1, 1 << 22), (7, 123457), (600, 70001), (2, 4097 * 4)],  # rows cut into slices
)
def test_softmax_long_rows(rt, rows, cols):
    """Rows past 16384 columns: in the registers of sixteen wavefronts where there are rows enough for half the CUs,
    else cut into slices over two launches (any width: a row need not start on a vector boundary)."""
    rng = np.random.default_rng(rows * 7 + cols)
    X = (rng.standard_normal((rows, cols)) * 8).astype(np.float32)
    Y = run_softmax(rt, X)
    ref = scipy.special.softmax(X.astype(np.float64), axis=-1)
    assert rel_err_max(Y, ref) <= TOL_F32
    np.testing.assert_allclose(Y, ref, rtol=3e-5, atol=1e-30)
    np.testing.assert_allclose(Y.sum(axis=-1, dtype=np.float64), 1.0, rtol=0, atol=1e-5)


@pytest.mark.parametrize("cols", [257, 259, 1001, 1023, 1026, 4095, 4097, 6282, 16383])
def test_softmax_rows_that_start_off_a_vector_boundary(rt, cols):
    """A width that is not a multiple of four puts most rows off a 16-byte boundary; the work-group per row then reads
    up to three single elements, the vectors between the boundaries, and up to three single elements."""
    rng = np.random.default_rng(cols)
    X = (rng.standard_normal((13, cols)) * 8).astype(np.float32)
    X[5] = -np.inf
    X[6, cols - 1] = np.nan
    X[7, :3] = -np.inf
    Y = run_softmax(rt, X)
    with np.errstate(invalid="ignore"):
        ref = scipy.special.softmax(X.astype(np.float64), axis=-1)
    assert np.isnan(Y[5]).all() and np.isnan(Y[6]).all() and (Y[7, :3] == 0).all()
    ok = ~np.isnan(ref)
    assert not np.isnan(Y[ok]).any()
    np.testing.assert_allclose(Y[ok], ref[ok], rtol=3e-5, atol=1e-30)
    # operands placed off the boundary themselves, equally and unequally (the second goes element by element)
    for off_x, off_y in ((2, 2), (1, 3)):
        bx = torch.zeros(X.size + 8, device="cuda")
        by = torch.zeros(X.size + 8, device="cuda")
        bx[off_x:off_x + X.size] = dev(X).view(-1)
        rt.softmax_f32(13, cols, bx.data_ptr() + 4 * off_x, by.data_ptr() + 4 * off_y)
        torch.cuda.synchronize()
        got = host(by)
        np.testing.assert_allclose(got[off_y:off_y + X.size].reshape(X.shape)[ok], ref[ok], rtol=3e-5, atol=1e-30)
        assert (got[:off_y] == 0).all() and (got[off_y + X.size:] == 0).all()


F64_ROWS = [(1000, 2), (999, 4), (513, 16), (130, 28), (4099, 32), (1025, 64), (300, 100), (259, 128), (17, 512), (6, 514), (33, 1000), (9, 1024),
            (9, 2048), (11, 3000), (5, 8192), (7, 4097), (13, 1001), (140, 8194), (129, 32768), (130, 20001), (3, 16388), (2, 40001)]


@pytest.mark.parametrize("rows,cols", F64_ROWS)
def test_softmax_fp64_rows_every_form(rt, rows, cols):
    """The row kernels in fp64 (vectors of two): rows sharing a wavefront, a wavefront and a work-group per row, rows off
    a 16-byte boundary, sixteen wavefronts per row, rows cut into slices. Against scipy in float64, -inf and NaN rows included."""
    rng = np.random.default_rng(rows * 31 + cols)
    X = rng.standard_normal((rows, cols)) * 8
    X[rows // 2] = -np.inf
    X[0, cols // 2] = -np.inf                      # (every case has at least two rows)
    if rows > 4:
        X[rows - 1, cols - 1] = np.nan
    x = dev(X)
    y = torch.empty_like(x)
    rt.softmax(64, rows, cols, 1, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    Y = host(y)
    with np.errstate(invalid="ignore"):
        ref = scipy.special.softmax(X, axis=-1)
    assert np.array_equal(np.isnan(Y), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert Y[0, cols // 2] == 0.0
    np.testing.assert_allclose(Y[ok], ref[ok], rtol=1e-12, atol=1e-300)


def test_softmax_long_rows_fp64_and_misplaced_operands(rt):
    """The sliced rows in fp64 (vectors of two), and fp32 operands that are not 16-byte aligned: equally misplaced
    operands keep the vector form (head and tail by single elements), unequally placed ones go element by element."""
    rng = np.random.default_rng(12)
    X = rng.standard_normal((3, 100003)) * 9
    x = dev(X)
    y = torch.empty_like(x)
    rt.softmax(64, 3, 100003, 1, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    np.testing.assert_allclose(host(y), scipy.special.softmax(X, axis=-1), rtol=1e-12, atol=1e-300)
    Xf = (rng.standard_normal((2, 70000)) * 8).astype(np.float32)
    ref = scipy.special.softmax(Xf.astype(np.float64), axis=-1)
    for off_x, off_y in ((1, 1), (3, 3), (1, 2), (0, 3)):
        bx = torch.zeros(Xf.size + 8, device="cuda")
        by = torch.zeros(Xf.size + 8, device="cuda")
        bx[off_x:off_x + Xf.size] = dev(Xf).view(-1)
        rt.softmax_f32(2, 70000, bx.data_ptr() + 4 * off_x, by.data_ptr() + 4 * off_y)
        torch.cuda.synchronize()
        got = host(by)
        np.testing.assert_allclose(got[off_y:off_y + Xf.size].reshape(Xf.shape), ref, rtol=3e-5, atol=1e-30)
        assert (got[:off_y] == 0).all() and (got[off_y + Xf.size:] == 0).all()      # nothing written outside the rows


def test_softmax_long_rows_edge_values(rt):
    """Infinite and NaN entries in rows that are cut into slices or held by sixteen wavefronts poison their own row only."""
    for rows, cols in ((4, 200000), (140, 20000)):
        X = np.zeros((rows, cols), np.float32)
        X[0, cols - 5] = np.inf
        X[1, 70] = np.nan
        X[2, :] = -np.inf
        X[3, 9::2] = -np.inf
        Y = run_softmax(rt, X)
        assert np.isnan(Y[:3]).all()
        live = np.ones(cols, bool)
        live[9::2] = False
        assert (Y[3, ~live] == 0).all() and np.allclose(Y[3, live], 1.0 / live.sum(), rtol=1e-5)
        if rows > 4:
            assert np.allclose(Y[4:], 1.0 / cols, rtol=1e-5)
    # a slice that holds nothing but -inf next to slices with finite values, and a NaN in a slice of -inf
    X = np.full((2, 1 << 20), -np.inf, np.float32)
    X[0, 5] = 1.0
    X[0, (1 << 20) - 3] = 1.0
    X[1, 5] = 2.0
    X[1, 600000] = np.nan
    Y = run_softmax(rt, X)
    assert Y[0, 5] == 0.5 and Y[0, (1 << 20) - 3] == 0.5 and Y[0].sum() == 1.0 and np.isnan(Y[1]).all()


@pytest.mark.parametrize("force", ["wave", "block"])
@pytest.mark.parametrize("cols", [512, 1024, 2048, 3000, 4096])
def test_softmax_every_built_variant(rt, monkeypatch, force, cols):
    """The wavefront-per-row and work-group-per-row kernels are both built up to 4096 columns; the launcher
    picks by width. Forcing either must give the same result."""
    monkeypatch.setenv("DOCC_ROCM_SOFTMAX", force)
    rng = np.random.default_rng(cols)
    X = (rng.standard_normal((37, cols)) * 8).astype(np.float32)
    Y = run_softmax(rt, X)
    assert rel_err_max(Y, oracle.softmax(X)) <= TOL_F32
    np.testing.assert_allclose(Y.sum(axis=-1), 1.0, rtol=0, atol=1e-5)


def test_softmax_nd_shape_like_reference_benchmark(rt):
    # (N, H, SM, SM) with the last axis reduced, the shape of the reference's
    # softmax benchmark (python/benchmarks/npbench/deep_learning/softmax/test_softmax.py:7-28, size S)
    rng = np.random.default_rng(42)
    X = rng.random((16, 16, 128, 128), dtype=np.float32)
    Y = run_softmax(rt, X)
    assert rel_err_max(Y, oracle.softmax(X)) <= TOL_F32


def test_softmax_closed_forms(rt):
    # constant row -> 1/C exactly representable cases; shift invariance; dominant entry -> one-hot
    X = np.full((4, 1024), 3.25, np.float32)
    np.testing.assert_allclose(run_softmax(rt, X), 1.0 / 1024, rtol=1e-6)
    rng = np.random.default_rng(7)
    X = (rng.standard_normal((6, 512)) * 8).astype(np.float32)
    a = run_softmax(rt, X)
    b = run_softmax(rt, X + np.float32(64.0))  # exact shift for these magnitudes
    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-12)
    X = np.zeros((2, 300), np.float32)
    X[0, 17] = 1000.0
    X[1, 299] = 1000.0
    Y = run_softmax(rt, X)
    assert Y[0, 17] == 1.0 and Y[1, 299] == 1.0 and Y.sum() == 2.0
    # large magnitudes: max subtraction keeps everything finite
    X = (rng.standard_normal((3, 4096)) * 1e4).astype(np.float32)
    Y = run_softmax(rt, X)
    assert np.isfinite(Y).all()
    assert rel_err_max(Y, oracle.softmax(X)) <= TOL_F32


def test_softmax_in_place_and_empty(rt):
    rng = np.random.default_rng(3)
    X = (rng.standard_normal((12, 4096)) * 8).astype(np.float32)
    x = dev(X)
    rt.softmax_f32(12, 4096, x.data_ptr(), x.data_ptr())
    torch.cuda.synchronize()
    assert rel_err_max(host(x), oracle.softmax(X)) <= TOL_F32
    rt.softmax_f32(0, 4096, 0, 0)
    rt.softmax_f32(5, 0, 0, 0)


def test_softmax_full_config(rt):
    # the benchmark configuration: [8192, 4096], N(0,1)*8, seed 1
    rng = np.random.default_rng(1)
    X = (rng.standard_normal((8192, 4096)) * 8).astype(np.float32)
    Y = run_softmax(rt, X)
    # size-independent properties on the full tensor
    np.testing.assert_allclose(Y.sum(axis=-1, dtype=np.float64), 1.0, atol=2e-6)
    assert (Y >= 0).all() and np.array_equal(Y.argmax(axis=-1), X.argmax(axis=-1))
    # oracle on a slice of rows (the oracle is the slow side)
    sel = np.r_[0:64, 4000:4064, 8128:8192]
    assert rel_err_max(Y[sel], oracle.softmax(X[sel])) <= TOL_F32


# ---- the general entry point: fp64, and reductions over inner axes ------------------------------------

GENERAL = [  # shape, axes
    ((5, 7), (0,)), ((64, 300), (0,)), ((3, 1000, 8), (1,)), ((4, 257, 16), (1,)), ((2, 50, 33), (1,)), ((6, 31, 64), (1,)),
    ((2, 9, 200), (0, 1)), ((3, 4, 5, 6), (1, 2)), ((7, 129), (-1,)), ((1, 5000), (-1,)), ((4, 6, 2), (1,)), ((1, 4096, 1), (1,)),
    ((3, 3, 3), (0, 1, 2)), ((2, 2048, 4), (-2,)), ((5, 1, 70), (1,)),
    # enough (outer index, column) pairs for one launch: columns in 16-byte vectors, sixteen row groups per work-group
    ((40, 100, 68), (1,)), ((300, 7, 36), (1,)), ((9, 130, 1024), (1,)), ((64, 17, 130), (1,)), ((20, 64, 66), (1,)),
    # few columns, long extents: the rows are sliced over work-groups as well
    ((1000, 300), (0,)), ((3, 700, 130), (1,)), ((2, 4096, 65), (1,)), ((1, 257, 64), (1,)), ((5000, 40), (0,)),
    ((2, 3000, 132), (1,)), ((1, 9000, 256), (1,)), ((3, 1024, 68), (1,)),      # the same with columns in 16-byte vectors
]


@pytest.mark.parametrize("dt,tol", [(np.float32, TOL_F32), (np.float64, 1e-12)], ids=["f32", "f64"])
@pytest.mark.parametrize("shape,axes", GENERAL, ids=["x".join(map(str, s)) + "_ax" + "".join(str(a % len(s)) for a in ax) for s, ax in GENERAL])
def test_softmax_general_matches_oracle(rt, dt, tol, shape, axes):
    rng = np.random.default_rng(sum(shape) * 31 + len(axes))
    X = (rng.standard_normal(shape) * 8).astype(dt)
    norm = sorted(a % len(shape) for a in axes)
    outer = int(np.prod(shape[:norm[0]], dtype=np.int64))
    reduce_ = int(np.prod(shape[norm[0]:norm[-1] + 1], dtype=np.int64))
    inner = int(np.prod(shape[norm[-1] + 1:], dtype=np.int64))
    x = dev(X)
    y = torch.empty_like(x)
    rt.softmax(64 if dt == np.float64 else 32, outer, reduce_, inner, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    Y = host(y)
    ref = oracle.softmax_axes(X, axes)
    assert rel_err_max(Y, ref) <= tol
    np.testing.assert_allclose(Y, ref, rtol=20 * tol, atol=1e-300 if dt == np.float64 else 1e-30)
    np.testing.assert_allclose(Y.sum(axis=tuple(norm)), 1.0, rtol=0, atol=max(tol, 1e-14) * 4)


@pytest.mark.parametrize("form", ["scalar", "v16", "v4"])
@pytest.mark.parametrize("dt,tol", [(np.float32, TOL_F32), (np.float64, 1e-12)], ids=["f32", "f64"])
def test_softmax_over_inner_axes_every_kernel_form(rt, monkeypatch, form, dt, tol):
    """One column per lane, or 16-byte vectors with the extent split sixteen or four ways: every form on every shape,
    the one-launch and the sliced kernels, with a column of -inf, one with a NaN and one with +inf."""
    monkeypatch.setenv("DOCC_ROCM_SOFTMAX_TILE", form)
    rng = np.random.default_rng(8)
    for shape in ((9, 70, 260), (300, 5, 36), (2, 700, 132), (1, 2100, 64), (40, 33, 1028)):
        X = (rng.standard_normal(shape) * 6).astype(dt)
        X[0, :, 3] = -np.inf
        X[0, shape[1] // 2, 5] = np.nan
        X[0, 1, 7] = np.inf
        X[0, 2, 9] = -np.inf
        x = dev(X)
        y = torch.empty_like(x)
        rt.softmax(64 if dt == np.float64 else 32, *shape, x.data_ptr(), y.data_ptr())
        torch.cuda.synchronize()
        Y = host(y)
        with np.errstate(invalid="ignore"):
            ref = oracle.softmax_axes(X, (1,))
        assert np.array_equal(np.isnan(Y), np.isnan(ref)), shape
        assert np.isnan(Y[0, :, 3]).all() and np.isnan(Y[0, :, 5]).all() and np.isnan(Y[0, :, 7]).all() and Y[0, 2, 9] == 0
        ok = ~np.isnan(ref)
        assert rel_err_max(Y[ok], ref[ok]) <= tol, shape


def test_sliced_launch_pairs_on_two_streams_and_two_threads(rt):
    """The launchers that run as two launches with partial results in between (sliced softmax, column reduction,
    column matrix-vector product) keep those per stream: pairs issued to two streams, from two threads, many
    times over, each give what the same call gives alone."""
    import ctypes
    import threading

    streams = []
    for _ in range(2):
        h = ctypes.c_void_p()
        rt.call("docc_rocm_stream_create", ctypes.byref(h))
        streams.append(h.value)
    rng = np.random.default_rng(77)
    cases = []
    for t, (rows, cols) in enumerate([(6000, 320), (4096, 1100)]):
        X = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
        v = rng.standard_normal(rows).astype(np.float32)
        x, vd = dev(X), dev(v)
        outs = {"softmax": torch.empty_like(x), "sum": torch.empty(cols, device="cuda"), "gemv": torch.empty(cols, device="cuda")}
        cases.append((X, v, x, vd, outs, rows, cols))
    torch.cuda.synchronize()

    def issue(case, stream):
        X, v, x, vd, outs, rows, cols = case
        rt.softmax(32, 1, rows, cols, x.data_ptr(), outs["softmax"].data_ptr(), stream=stream)
        rt.reduce("sum", 32, 1, rows, cols, x.data_ptr(), outs["sum"].data_ptr(), stream=stream)
        rt.sgemm(1, cols, rows, 1.0, vd.data_ptr(), rows, x.data_ptr(), cols, 0.0, outs["gemv"].data_ptr(), cols, stream=stream)

    # what each call gives alone
    alone = []
    for case in cases:
        issue(case, 0)
        torch.cuda.synchronize()
        alone.append({k: t.clone() for k, t in case[4].items()})
        for t in case[4].values():
            t.fill_(float("nan"))
    errors = []

    def worker(i):
        try:
            for _ in range(20):
                issue(cases[i], streams[i])
        except Exception as e:      # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors
    for case, ref in zip(cases, alone):
        for k in ref:
            assert torch.equal(case[4][k], ref[k]), k
        X = case[0]
        # against the closed form in float64 (over 6000 rows the oracle's left-to-right fp32 sum is itself 1e-5 off)
        assert rel_err_max(host(case[4]["softmax"]), scipy.special.softmax(X.astype(np.float64), axis=0)) <= TOL_F32
        assert rel_err_max(host(case[4]["sum"]), X.sum(axis=0, dtype=np.float64)) <= TOL_F32
    for h in streams:
        rt.call("docc_rocm_stream_destroy", h)


def test_softmax_with_the_callers_workspace(rt):
    """docc_rocm_softmax_ws: same bits as docc_rocm_softmax, the partial results in memory of the caller."""
    rng = np.random.default_rng(5)
    for dt, precision in ((np.float32, 32), (np.float64, 64)):
        for outer, reduce_, inner in ((1, 5000, 300), (3, 700, 130), (2, 64, 40), (4, 100, 1), (2, 300, 16), (3, 90000, 1), (300, 20000, 1)):
            X = (rng.standard_normal((outer, reduce_, inner)) * 6).astype(dt)
            x = dev(X)
            y0, y1 = torch.empty_like(x), torch.full_like(x, float("nan"))
            rt.softmax(precision, outer, reduce_, inner, x.data_ptr(), y0.data_ptr())
            need = rt.softmax_workspace_bytes(precision, outer, reduce_, inner)
            assert 0 <= need <= 8 << 20
            ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
            rt.softmax_ws(precision, outer, reduce_, inner, x.data_ptr(), y1.data_ptr(), ws.data_ptr(), need)
            torch.cuda.synchronize()
            assert torch.equal(y0, y1)
            if need:
                from docc_amd.runtime import RocmRuntimeError
                with pytest.raises(RocmRuntimeError, match="workspace"):
                    rt.softmax_ws(precision, outer, reduce_, inner, x.data_ptr(), y1.data_ptr(), ws.data_ptr(), need - 1)
                with pytest.raises(RocmRuntimeError, match="workspace"):
                    rt.softmax_ws(precision, outer, reduce_, inner, x.data_ptr(), y1.data_ptr(), 0, 0)
    assert rt.softmax_workspace_bytes(32, 1, 5000, 300) > 0      # the sliced form is among the cases
    assert rt.softmax_workspace_bytes(32, 3, 90000, 1) > 0 and rt.softmax_workspace_bytes(64, 3, 90000, 1) > 0      # and rows cut into slices


def test_softmax_general_edge_values_and_empty(rt):
    """Infinite and NaN entries poison their own column only, the way the node's Sub / Exp / Sum / Div steps
    would; an empty extent launches nothing."""
    X = np.zeros((3, 6, 5), np.float64)
    X[0, 2, 1] = np.inf          # inf - inf = NaN in the Sub step: the whole column becomes NaN
    X[1, 0, 3] = np.nan
    X[2, :, 4] = -np.inf         # max = -inf: NaN as well
    X[2, 1, 0] = -np.inf         # one -inf among finite values: weight 0
    x = dev(X)
    y = torch.empty_like(x)
    rt.softmax(64, 3, 6, 5, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    Y = host(y)
    with np.errstate(invalid="ignore"):
        ref = oracle.softmax_axes(X, (1,))
    assert np.array_equal(np.isnan(Y), np.isnan(ref))
    ok = ~np.isnan(ref)
    np.testing.assert_allclose(Y[ok], ref[ok], rtol=1e-14)
    assert Y[2, 1, 0] == 0.0 and np.isnan(Y[0, :, 1]).all() and np.isnan(Y[2, :, 4]).all()
    # the same for the fp32 row kernels
    Xr = np.zeros((4, 300), np.float32)
    Xr[0, 7] = np.inf
    Xr[1, 9] = np.nan
    Xr[2, :] = -np.inf
    for cols in (300, 40004):     # block kernel, streaming kernel
        Xc = np.zeros((4, cols), np.float32)
        Xc[:, :300] = Xr
        Xc[2, :] = -np.inf
        Yr = run_softmax(rt, Xc)
        assert np.isnan(Yr[:3]).all() and np.allclose(Yr[3], 1.0 / cols)
    # sliced path: a NaN that is the only element one thread sees besides -inf, an infinite value in one slice
    for dt in (np.float32, np.float64):
        Xs = np.zeros((1, 1024, 70), dt)
        Xs[0, :, 5] = -np.inf
        Xs[0, 517, 5] = np.nan
        Xs[0, 900, 9] = np.inf
        Xs[0, 3, 11] = -np.inf
        xs = dev(Xs)
        ys = torch.empty_like(xs)
        rt.softmax(64 if dt == np.float64 else 32, 1, 1024, 70, xs.data_ptr(), ys.data_ptr())
        torch.cuda.synchronize()
        Ys = host(ys)
        with np.errstate(invalid="ignore"):
            refs = oracle.softmax_axes(Xs, (1,))
        assert np.array_equal(np.isnan(Ys), np.isnan(refs))
        assert np.isnan(Ys[0, :, 5]).all() and np.isnan(Ys[0, :, 9]).all() and Ys[0, 3, 11] == 0
        np.testing.assert_allclose(Ys[~np.isnan(refs)], refs[~np.isnan(refs)], rtol=1e-5 if dt == np.float32 else 1e-13)
    z = torch.zeros(8, device="cuda")
    rt.softmax(32, 0, 4, 2, z.data_ptr(), z.data_ptr())
    rt.softmax(64, 2, 0, 2, z.data_ptr(), z.data_ptr())
    torch.cuda.synchronize()
    assert host(z).sum() == 0
    from docc_amd.runtime import RocmRuntimeError
    with pytest.raises(RocmRuntimeError, match="precision"):
        rt.softmax(16, 1, 4, 2, z.data_ptr(), z.data_ptr())


def test_softmax_and_reductions_past_2_to_the_31_elements(rt):
    """[524290, 4096] fp32 (2^31 + 8192 elements): row offsets need 64 bits. Rows at the start, around the 2^31
    boundary and at the end against the oracle; row sums and a reduction over the rows on the device."""
    cols = 4096
    rows = (1 << 31) // cols + 2
    g = torch.Generator(device="cuda").manual_seed(6)
    x = torch.empty(rows, cols, device="cuda")
    x.normal_(0, 4, generator=g)
    y = torch.empty_like(x)
    rt.softmax_f32(rows, cols, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    for r0 in (0, rows // 2 - 2, rows - 3):
        assert rel_err_max(host(y[r0:r0 + 3]), oracle.softmax(host(x[r0:r0 + 3]))) <= TOL_F32
    sums = torch.empty(rows, device="cuda")
    rt.reduce("sum", 32, rows, cols, 1, y.data_ptr(), sums.data_ptr())
    torch.cuda.synchronize()
    assert float((sums - 1).abs().max()) <= 1e-5
    # over the rows (one result per column): the sliced column kernels walk 2^31 elements
    colmax = torch.empty(cols, device="cuda")
    rt.reduce("max", 32, 1, rows, cols, x.data_ptr(), colmax.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(colmax, x.max(dim=0).values)
    # softmax over the rows of the last 300000 x 4096 block viewed as [1, 300000, 4096] would not add coverage of
    # the index width; the general entry point is exercised past 2^31 through its row form instead
    rt.softmax(32, rows, cols, 1, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    assert rel_err_max(host(y[rows - 2:]), oracle.softmax(host(x[rows - 2:]))) <= TOL_F32
