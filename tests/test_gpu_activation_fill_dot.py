"""ml::Elu / ml::LeakyReLU / ml::HardSigmoid, ml::Fill and DOT::BLAS on the GPU through the C ABI
(docc_rocm_elementwise_activation, docc_rocm_fill, docc_rocm_dot) against the CPU oracle.
Tolerances: the IEEE selections and products bit for bit; exp-backed values 1e-5 (fp32) / 1e-12 (fp64)
norm-wise, as for the other libm-backed nodes; dot against the exact sum within K * u * sum|x||y|."""
import numpy as np
import pytest
import torch

import oracle
from docc_amd.runtime import RocmRuntimeError
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt,precision,tol", [(np.float32, 32, 1e-5), (np.float64, 64, 1e-12)], ids=["f32", "f64"])
@pytest.mark.parametrize("n", [1, 7, 1000, 4099, 1 << 20])
def test_activations_match_oracle(rt, dt, precision, tol, n):
    rng = np.random.default_rng(n)
    X = (rng.standard_normal(n) * 3).astype(dt)
    X[: min(n, 4)] = np.array([0.0, -0.0, 40.0, -40.0], dt)[: min(n, 4)]
    x = dev(X)
    for op, alpha, beta in (("elu", 1.0, 0.0), ("elu", 0.37, 0.0), ("leaky_relu", 0.01, 0.0), ("hard_sigmoid", 0.2, 0.5), ("hard_sigmoid", 1 / 6, 0.5)):
        y = torch.full_like(x, float("nan"))
        rt.elementwise_activation(op, precision, n, x.data_ptr(), y.data_ptr(), alpha, beta)
        torch.cuda.synchronize()
        ref = oracle.elementwise_activation(op, X, alpha, beta)
        Y = host(y)
        if op == "elu":
            assert rel_err_max(Y, ref) <= tol
            assert np.array_equal(Y[X > 0], X[X > 0])           # the positive branch passes the input through
        else:
            assert np.array_equal(Y, ref), op                    # selections, one product / one fma: exact
    # unaligned operands take the scalar path; in place is allowed
    if n > 8:
        rt.elementwise_activation("leaky_relu", precision, n - 1, x.data_ptr() + X.itemsize, x.data_ptr() + X.itemsize, 0.5)
        torch.cuda.synchronize()
        assert np.array_equal(host(x)[1:], oracle.elementwise_activation("leaky_relu", X[1:], 0.5))


def test_activation_errors(rt):
    t = torch.zeros(16, device="cuda")
    with pytest.raises(RocmRuntimeError, match="unknown operation"):
        rt.elementwise_activation(3, 32, 16, t.data_ptr(), t.data_ptr(), 1.0)
    with pytest.raises(RocmRuntimeError, match="precision"):
        rt.elementwise_activation("elu", 16, 16, t.data_ptr(), t.data_ptr(), 1.0)
    rt.elementwise_activation("elu", 32, 0, 0, 0, 1.0)


@pytest.mark.parametrize("value", [np.float32(-2.75), np.float64(1e-300), np.int64(-5), np.int32(7), np.uint16(0x3F80), np.int8(-3)],
                         ids=["f32", "f64", "i64", "i32", "u16", "i8"])
@pytest.mark.parametrize("n,offset", [(1, 0), (5, 0), (1000, 0), (4097, 1), (1 << 18, 3)])
def test_fill(rt, value, n, offset):
    size = value.dtype.itemsize
    buf = torch.full(((n + offset + 4) * size,), 0xAB, dtype=torch.uint8, device="cuda")
    rt.fill(value, n, buf.data_ptr() + offset * size)
    torch.cuda.synchronize()
    got = host(buf).view(value.dtype)
    assert np.array_equal(got[offset:offset + n], np.full(n, value))
    guard = np.frombuffer(bytes([0xAB] * size), value.dtype)[0]
    assert (got[:offset] == guard).all() and (got[offset + n:] == guard).all()      # nothing beyond the n elements


def test_fill_errors(rt):
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")
    v = np.float32(1)
    with pytest.raises(RocmRuntimeError, match="aligned"):
        rt.fill(v, 4, t.data_ptr() + 1)
    with pytest.raises(RocmRuntimeError, match="element size"):
        rt.call("docc_rocm_fill", 0, 3, 4, np.zeros(4, np.uint8).ctypes.data, t.data_ptr())
    rt.fill(v, 0, 0)


@pytest.mark.parametrize("dt,precision,u", [(np.float32, 32, 6e-8), (np.float64, 64, 1.2e-16)], ids=["f32", "f64"])
@pytest.mark.parametrize("n,incx,incy", [(1, 1, 1), (100, 1, 1), (4097, 1, 1), (1000, 3, 2), (1 << 22, 1, 1), (5000, 0, 1), (300000, 2, 5)])
def test_dot_matches_oracle(rt, dt, precision, u, n, incx, incy):
    rng = np.random.default_rng(n + incx)
    X = rng.standard_normal(max(1, (n - 1) * incx + 1)).astype(dt)
    Y = rng.standard_normal(max(1, (n - 1) * incy + 1)).astype(dt)
    x, y = dev(X), dev(Y)
    got = rt.dot(precision, n, x.data_ptr(), incx, y.data_ptr(), incy)
    xs = X[::incx][:n] if incx else np.full(n, X[0])
    ys = Y[::incy][:n] if incy else np.full(n, Y[0])
    exact = float(np.dot(xs.astype(np.longdouble), ys.astype(np.longdouble)))
    bound = float(np.dot(np.abs(xs).astype(np.longdouble), np.abs(ys).astype(np.longdouble)))
    # pairwise over work-groups: far inside the bound of the left-to-right sum the reference's loop forms
    assert abs(got - exact) <= 64 * u * bound
    assert abs(float(oracle.dot(X, Y, incx, incy, n)) - exact) <= n * u * bound + 1e-300
    assert rt.dot(precision, n, x.data_ptr(), incx, y.data_ptr(), incy) == got           # reproducible


def test_dot_exact_on_integers_and_errors(rt):
    xi, yi = np.arange(1, 3001, dtype=np.float32) % 17, np.arange(3000, 0, -1, dtype=np.float32) % 13
    x, y = dev(xi), dev(yi)
    assert rt.dot(32, 3000, x.data_ptr(), 1, y.data_ptr(), 1) == float(np.dot(xi.astype(np.float64), yi.astype(np.float64)))
    assert rt.dot(32, 0, 0, 1, 0, 1) == 0.0
    with pytest.raises(RocmRuntimeError, match="negative increments"):
        rt.dot(32, 10, x.data_ptr(), -1, y.data_ptr(), 1)
    with pytest.raises(RocmRuntimeError, match="precision"):
        rt.dot(16, 10, x.data_ptr(), 1, y.data_ptr(), 1)
