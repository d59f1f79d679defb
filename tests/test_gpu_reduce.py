"""Reduce tensor nodes (ml::Sum / ml::Max / ml::Min / ml::Mean) on the GPU against the CPU oracle, through
docc_rocm_reduce.

Bars: Max and Min bit-exact (selections); Sum and Mean bit-exact on integer-valued inputs (every partial
sum is exact, so the order of the additions does not matter) and otherwise within extent * epsilon of the
oracle relative to sum|x| (the kernel adds in a tree, the reference left to right)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

# (shape, reduced axes)
CASES = [((8192, 4096), (1,)), ((4096, 8192), (0,)), ((16, 16, 128, 128), (3,)), ((32, 64, 56, 56), (2, 3)), ((32, 64, 56, 56), (0,)),
         ((7, 33), (1,)), ((7, 33), (0,)), ((5, 1, 9), (1,)), ((3, 1000003), (1,)), ((1, 17), (0, 1)), ((2, 3, 4, 5), (1, 2)),
         ((64, 4099), (1,)), ((6, 0, 4), (1,)), ((100000, 24), (0,)), ((3, 5000, 40), (1,)),      # the last two: sliced column reductions
         ((1, 1 << 22), (1,)), ((5, 40000), (1,)), ((2, 3, 8192), (1, 2)), ((300, 9000), (1,)),    # long rows, few of them: each row in pieces
         ((1000, 4), (1,)), ((777, 8), (1,)), ((4099, 32), (1,)), ((65, 12, 5), (1, 2)), ((300, 100), (1,)), ((1025, 128), (1,))]   # short rows share a wavefront


def run(rt, op, x, axes, offset=0):
    rank = x.ndim
    axes = sorted(a % rank for a in axes)
    outer = int(np.prod(x.shape[:axes[0]], dtype=np.int64))
    extent = int(np.prod(x.shape[axes[0]:axes[-1] + 1], dtype=np.int64))
    inner = int(np.prod(x.shape[axes[-1] + 1:], dtype=np.int64))
    buf = dev(np.concatenate([np.zeros(offset, x.dtype), x.ravel()]))
    out = torch.full((max(outer * inner, 1),), float("nan"), device="cuda", dtype=buf.dtype)
    rt.reduce(op, 64 if x.dtype == np.float64 else 32, outer, extent, inner, buf.data_ptr() + offset * buf.element_size(), out.data_ptr())
    torch.cuda.synchronize()
    return host(out)[:outer * inner].reshape([s for d, s in enumerate(x.shape) if d not in axes])


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("case", CASES, ids=[f"{'x'.join(map(str, s))}_ax{'_'.join(map(str, a))}" for s, a in CASES])
def test_reduce_against_the_oracle(rt, dt, case):
    shape, axes = case
    if dt == np.float64 and np.prod(shape) > 2 ** 24:
        shape = (shape[0] // 2,) + tuple(shape[1:])
    rng = np.random.default_rng(sum(shape) + len(axes))
    x = rng.standard_normal(shape).astype(dt)
    extent = int(np.prod([shape[a] for a in axes]))
    for op in ("max", "min"):
        if extent == 0:
            continue
        assert np.array_equal(run(rt, op, x, axes), oracle.reduce(op, x, axes)), op
    ints = rng.integers(-8, 9, shape).astype(dt)
    assert np.array_equal(run(rt, "sum", ints, axes), oracle.reduce("sum", ints, axes))
    if extent:
        assert np.array_equal(run(rt, "mean", ints, axes), oracle.reduce("mean", ints, axes))      # an exact sum, divided once
    eps = np.finfo(dt).eps
    scale = np.abs(x).sum(axis=tuple(axes)) + 1e-30
    got, ref = run(rt, "sum", x, axes), oracle.reduce("sum", x, axes)
    assert (np.abs(got.astype(np.float64) - ref) <= max(extent, 1) * eps * scale).all()
    if extent:
        got, ref = run(rt, "mean", x, axes), oracle.reduce("mean", x, axes)
        assert (np.abs(got.astype(np.float64) - ref) <= eps * scale + np.abs(ref) * eps * 2).all()
        # rows that do not start on a 16-byte boundary take the scalar path
        assert np.array_equal(run(rt, "max", x, axes, offset=1), oracle.reduce("max", x, axes))


def test_reduce_special_values_and_errors(rt):
    y = np.array([[1.0, np.nan, 3.0, -2.0], [np.nan] * 4, [-np.inf, 2.0, np.inf, 0.0]], np.float32)
    assert np.array_equal(run(rt, "max", y, (1,)), oracle.reduce("max", y, (1,)))        # NaN skipped, all-NaN row -> -inf
    assert np.array_equal(run(rt, "min", y, (1,)), oracle.reduce("min", y, (1,)))
    assert np.array_equal(run(rt, "max", y, (0,)), oracle.reduce("max", y, (0,)))
    e = np.zeros((3, 0, 2), np.float64)
    assert np.array_equal(run(rt, "sum", e, (1,)), np.zeros((3, 2)))
    assert np.array_equal(run(rt, "max", e, (1,)), np.full((3, 2), -np.inf))
    from docc_amd.runtime import RocmRuntimeError
    a = torch.zeros(16, device="cuda")
    with pytest.raises(RocmRuntimeError):
        rt.reduce(9, 32, 4, 4, 1, a.data_ptr(), a.data_ptr())
    with pytest.raises(RocmRuntimeError):
        rt.reduce("mean", 32, 4, 0, 1, a.data_ptr(), a.data_ptr())
    with pytest.raises(RocmRuntimeError):
        rt.reduce("sum", 32, 4, 4, 1, 0, a.data_ptr())
    rt.reduce("sum", 32, 0, 4, 1, 0, 0)      # nothing to write
