"""ml::Softmax on the GPU against the CPU oracle, through the C-ABI
(docc_rocm_softmax_f32). Tolerance: 1e-5 norm-wise relative error
(max|y - y_ref| / max|y_ref|), the fp32 bar."""
import numpy as np
import pytest
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
