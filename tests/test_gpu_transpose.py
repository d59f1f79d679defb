"""ml::Transpose on the GPU against the CPU oracle, through docc_rocm_transpose. The node moves bits:
bit-exact for every element size (1, 2, 4, 8 bytes), rank up to six."""
import itertools

import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

DTYPES = {1: np.uint8, 2: np.int16, 4: np.float32, 8: np.float64}


def run_transpose(rt, X, perm):
    x = dev(X)
    out_shape = [X.shape[p] for p in perm]
    y = torch.full(out_shape, 7, dtype=x.dtype, device="cuda") if X.size else torch.empty(out_shape, dtype=x.dtype, device="cuda")
    rt.transpose(X.dtype.itemsize, X.shape, perm, x.data_ptr(), y.data_ptr())
    torch.cuda.synchronize()
    return host(y)


def values(shape, dt, seed):
    rng = np.random.default_rng(seed)
    n = int(np.prod(shape, dtype=np.int64))
    if np.issubdtype(dt, np.floating):
        return rng.standard_normal(n).astype(dt).reshape(shape)
    return rng.integers(0, 200, n).astype(dt).reshape(shape)


@pytest.mark.parametrize("bytes_", [1, 2, 4, 8])
def test_every_permutation_of_small_tensors(rt, bytes_):
    dt = DTYPES[bytes_]
    for shape in ((3, 5), (4, 3, 5), (2, 3, 4, 5), (70, 3, 66)):
        X = values(shape, dt, sum(shape))
        for perm in itertools.permutations(range(len(shape))):
            got = run_transpose(rt, X, perm)
            assert np.array_equal(got, oracle.transpose(X, perm)), (shape, perm)
            assert np.array_equal(got, np.transpose(X, perm))


CASES = [  # shape, perm: tiles with ragged edges, merged axes, unit axes, rank 6, the attention and NCHW <-> NHWC forms
    ((1000, 1000), (1, 0)), ((129, 257), (1, 0)), ((64, 64), (1, 0)), ((1, 300), (1, 0)), ((300, 1), (1, 0)),
    ((8, 16, 200, 64), (0, 2, 1, 3)), ((8, 16, 200, 64), (0, 1, 3, 2)), ((32, 64, 14, 14), (0, 2, 3, 1)), ((32, 14, 14, 64), (0, 3, 1, 2)),
    ((2, 3, 4, 5, 6, 7), (5, 3, 1, 0, 2, 4)), ((2, 3, 4, 5, 6, 7), (0, 1, 2, 3, 4, 5)), ((2, 1, 3, 1, 5), (4, 3, 2, 1, 0)),
    ((5, 6, 7), (1, 0, 2)), ((0, 5), (1, 0)), ((7,), (0,)), ((3, 4, 65, 2), (2, 0, 1, 3)),
    # everything a multiple of four elements: 4-byte elements take the tile that moves 128-bit units (ragged tiles of 4, 8, 60)
    ((132, 260), (1, 0)), ((3, 68, 12, 8), (0, 3, 2, 1)), ((4, 200), (1, 0)), ((2, 124, 8, 60), (0, 3, 2, 1)),
]


@pytest.mark.parametrize("shape,perm", CASES, ids=["x".join(map(str, s)) + "_" + "".join(map(str, p)) for s, p in CASES])
def test_transpose_shapes(rt, shape, perm):
    for dt in (np.float32, np.float64, np.int16):
        X = values(shape, dt, len(shape) + sum(perm))
        assert np.array_equal(run_transpose(rt, X, perm), oracle.transpose(X, perm)), dt


def test_tile_in_128_bit_units_equals_the_one_element_tile(rt, monkeypatch):
    """4-byte elements with every extent and stride a multiple of four take another kernel: both against numpy, and a
    tensor whose address is not a multiple of 16 bytes (the one-element tile again)."""
    X = values((260, 516), np.float32, 5)
    want = np.ascontiguousarray(X.T)
    assert np.array_equal(run_transpose(rt, X, (1, 0)), want)
    monkeypatch.setenv("DOCC_ROCM_TRANSPOSE_SCALAR", "1")
    assert np.array_equal(run_transpose(rt, X, (1, 0)), want)
    monkeypatch.delenv("DOCC_ROCM_TRANSPOSE_SCALAR")
    buf = dev(np.concatenate([np.zeros(1, np.float32), X.ravel()]))
    y = torch.empty(X.size, dtype=torch.float32, device="cuda")
    rt.transpose(4, X.shape, (1, 0), buf.data_ptr() + 4, y.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(y).reshape(want.shape), want)


@pytest.mark.parametrize("wide", ["1", "0"])
def test_tiles_of_128_and_of_64_move_the_same_elements(rt, monkeypatch, wide):
    """Large tensors take tiles of 128 x 128, small ones tiles of 64 x 64: either forced, on extents that end inside a
    tile, and with batch axes in front and behind."""
    monkeypatch.setenv("DOCC_ROCM_TRANSPOSE_WIDE", wide)
    for shape, perm in (((260, 516), (1, 0)), ((3, 132, 200), (0, 2, 1)), ((128, 128), (1, 0)), ((4, 644), (1, 0)), ((2, 300, 8, 72), (0, 3, 2, 1))):
        X = values(shape, np.float32, sum(shape))
        assert np.array_equal(run_transpose(rt, X, perm), oracle.transpose(X, perm)), (shape, perm)


def test_transpose_involution_at_full_size_and_errors(rt):
    """[8192, 4096] fp32: transposing twice gives the input back; row sums become column sums."""
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn(8192, 4096, device="cuda", generator=g)
    y, z = torch.empty(4096, 8192, device="cuda"), torch.empty(8192, 4096, device="cuda")
    rt.transpose(4, (8192, 4096), (1, 0), x.data_ptr(), y.data_ptr())
    rt.transpose(4, (4096, 8192), (1, 0), y.data_ptr(), z.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(x, z) and torch.equal(y[17], x[:, 17]) and torch.equal(y[:, 8000], x[8000])
    from docc_amd.runtime import RocmRuntimeError
    p = x.data_ptr()
    with pytest.raises(RocmRuntimeError, match="permutation"):
        rt.transpose(4, (4, 4), (0, 0), p, y.data_ptr())
    with pytest.raises(RocmRuntimeError, match="in place"):
        rt.transpose(4, (4, 4), (1, 0), p, p)
    with pytest.raises(RocmRuntimeError, match="element size"):
        rt.transpose(3, (4, 4), (1, 0), p, y.data_ptr())
    with pytest.raises(RocmRuntimeError, match="rank"):
        rt.transpose(4, (2,) * 7, tuple(range(7)), p, y.data_ptr())
