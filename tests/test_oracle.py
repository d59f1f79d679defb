"""Pins the CPU oracle (oracle/docc_oracle.c) without the reference, which holds no numeric
fixtures for these nodes: committed golden vectors (closed forms evaluated in float64 by
tests/golden/make_golden.py), library cross-checks (numpy.matmul, scipy.special.softmax, torch
conv2d / scaled_dot_product_attention in float64) and closed-form cases chosen so that a dropped
term, a wrong index or a transposed operand fails at least one of them."""
from pathlib import Path

import numpy as np
import pytest
import scipy.special
import torch

import oracle

GOLDEN = Path(__file__).resolve().parent / "golden"
N, T = oracle.NO_TRANS, oracle.TRANS


def rel(y, ref):
    return float(np.abs(np.asarray(y, np.float64) - ref).max() / np.abs(ref).max())


# ---- GEMM -----------------------------------------------------------------------------

@pytest.mark.parametrize("tag", ["f64", "f32"])
def test_gemm_golden(tag):
    g = np.load(GOLDEN / f"gemm_int_17x33x65_{tag}.npz")
    for variant in ("blas", "expanded"):
        assert np.array_equal(oracle.gemm(g["A"], g["B"], variant=variant), g["C"])
        assert np.array_equal(oracle.gemm(g["A"], g["B"], g["C0"], alpha=2.0, beta=-3.0, variant=variant), g["C_alpha2_beta_m3"])
    # transposed storage gives the same product
    assert np.array_equal(oracle.gemm(g["A"].T.copy(), g["B"], trans_a=T), g["C"])
    assert np.array_equal(oracle.gemm(g["A"], g["B"].T.copy(), trans_b=T), g["C"])
    assert np.array_equal(oracle.gemm(g["A"].T.copy(), g["B"].T.copy(), trans_a=T, trans_b=T), g["C"])


def test_gemm_bf16_golden():
    g = np.load(GOLDEN / "gemm_int_17x33x65_bf16.npz")
    assert np.array_equal(oracle.gemm_bf16(g["A"], g["B"]), g["C"])
    assert np.array_equal(oracle.gemm_bf16(g["A"].T.copy(), g["B"].T.copy(), trans_a=T, trans_b=T), g["C"])


def test_gemm_against_numpy_and_structure():
    rng = np.random.default_rng(0)
    A, B = rng.random((37, 91)), rng.random((91, 23))
    ref = A @ B
    assert rel(oracle.gemm(A, B), ref) <= 1e-14
    assert rel(oracle.gemm(A, B, variant="ld"), ref) <= 1e-14
    Af, Bf = A.astype(np.float32), B.astype(np.float32)
    assert rel(oracle.gemm(Af, Bf), Af.astype(np.float64) @ Bf.astype(np.float64)) <= 1e-5
    assert rel(oracle.gemm(Af, Bf, variant="acc64"), Af.astype(np.float64) @ Bf.astype(np.float64)) <= 1e-7
    # non-commutativity: a transposed-operand mistake cannot pass
    assert rel(oracle.gemm(A, B), (B.T @ A.T).T) <= 1e-14
    eye = np.eye(23)
    assert np.array_equal(oracle.gemm(B, eye), B)
    # rank-1 outer product and row sums
    u, v = rng.random((9, 1)), rng.random((1, 13))
    assert np.array_equal(oracle.gemm(u, v), u * v)
    assert rel(oracle.gemm(A, np.ones((91, 1))), A.sum(axis=1, keepdims=True)) <= 1e-14


def test_gemm_beta_semantics():
    rng = np.random.default_rng(1)
    A, B = rng.random((5, 6)), rng.random((6, 4))
    nan = np.full((5, 4), np.nan)
    # cblas semantics: beta == 0 does not read C; the reference's expansion multiplies it (NaN * 0 = NaN)
    assert np.isfinite(oracle.gemm(A, B, nan, beta=0.0, variant="blas")).all()
    assert np.isnan(oracle.gemm(A, B, nan, beta=0.0, variant="expanded")).all()
    # k == 0: C = beta * C
    C0 = rng.random((5, 4))
    assert np.allclose(oracle.gemm(np.zeros((5, 0)), np.zeros((0, 4)), C0, beta=2.0), 2 * C0)
    # alpha == 0: A and B are not referenced (the BLAS definition), so their NaNs stay out of C
    An = A.copy()
    An[2, 3] = np.nan
    assert np.array_equal(oracle.gemm(An, B, C0, alpha=0.0, beta=2.0, variant="blas"), 2 * C0)
    assert np.array_equal(oracle.gemm(An, B, nan, alpha=0.0, beta=0.0, variant="blas"), np.zeros((5, 4)))
    assert np.isnan(oracle.gemm(An, B, C0, alpha=1e-300, beta=2.0, variant="blas")[2]).all()


def test_bf16_conversion_matches_torch_exhaustively_on_a_sweep():
    # every bf16 value and the float32 values half-way and just around them
    hi = np.arange(0, 1 << 16, dtype=np.uint32) << 16
    for lo in (0x0000, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        bits = (hi | lo).astype(np.uint32)
        x = bits.view(np.float32)
        keep = ~np.isnan(x)
        want = torch.from_numpy(x[keep]).bfloat16().view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(oracle.f32_to_bf16(x[keep]), want)
    b = np.arange(0, 1 << 16, dtype=np.uint16)
    back = oracle.bf16_to_f32(b)
    assert np.array_equal(back.view(np.uint32), b.astype(np.uint32) << 16)


# ---- softmax --------------------------------------------------------------------------

@pytest.mark.parametrize("variant", ["numpy", "expanded"])
def test_softmax_golden_and_scipy(variant):
    g = np.load(GOLDEN / "softmax_8x257_f32.npz")
    Y = oracle.softmax(g["X"], variant=variant)
    assert rel(Y, g["Y"]) <= 1e-6
    rng = np.random.default_rng(5)
    X = (rng.standard_normal((3, 5, 64)) * 8).astype(np.float32)
    assert rel(oracle.softmax(X, variant=variant), scipy.special.softmax(X.astype(np.float64), axis=-1)) <= 1e-6


def test_softmax_closed_forms():
    X = np.full((3, 10), 2.5, np.float32)
    assert np.allclose(oracle.softmax(X), 0.1, rtol=1e-6)
    rng = np.random.default_rng(2)
    X = (rng.standard_normal((4, 33)) * 8).astype(np.float32)
    Y = oracle.softmax(X)
    assert np.allclose(Y.sum(axis=-1), 1.0, atol=1e-6)
    assert np.array_equal(Y.argmax(axis=-1), X.argmax(axis=-1))
    assert np.allclose(oracle.softmax(X + np.float32(16.0)), Y, rtol=1e-4, atol=1e-12)
    big = np.array([[1000.0, 0.0, -1000.0]], np.float32)   # max subtraction: no overflow
    assert np.array_equal(oracle.softmax(big), np.array([[1.0, 0.0, 0.0]], np.float32))
    assert oracle.softmax(np.zeros((0, 7), np.float32)).shape == (0, 7)


@pytest.mark.parametrize("dt,tol", [(np.float32, 1e-6), (np.float64, 1e-15)])
@pytest.mark.parametrize("axes", [(-1,), (0,), (1,), (1, 2), (0, 1, 2), (0, 2)])
def test_softmax_over_any_axes_against_scipy(dt, tol, axes):
    """The library cross-check (scipy in fp64), sums of one over the reduced axes, and for the last axis the
    row form itself: a transposition slip or a wrong inverse permutation fails the first two."""
    rng = np.random.default_rng(11 + len(axes))
    X = (rng.standard_normal((5, 7, 6)) * 6).astype(dt)
    Y = oracle.softmax_axes(X, axes)
    assert Y.dtype == dt and Y.shape == X.shape
    assert rel(Y, scipy.special.softmax(X.astype(np.float64), axis=axes)) <= tol
    assert np.allclose(Y.sum(axis=axes), 1.0, atol=10 * tol * X.size)
    if axes == (-1,) and dt == np.float32:
        assert np.array_equal(Y, oracle.softmax(X, variant="expanded"))


# ---- conv -----------------------------------------------------------------------------

def test_causal_attention_against_torch_and_by_hand():
    """The causal form of the oracle against torch's own (math path, float64, is_causal=True; for SQ != SKV the mask is the
    lower triangle aligned at the top left) and against a mask added by hand to the scores."""
    g = torch.Generator().manual_seed(3)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    for SQ, SKV in ((17, 17), (9, 30), (40, 12)):
        Q, K, V = (torch.randn(2, 3, s, 16, generator=g).bfloat16() for s in (SQ, SKV, SKV))
        got = oracle.attention(bits(Q), bits(K), bits(V), causal=True)
        ref = torch.nn.functional.scaled_dot_product_attention(Q.double(), K.double(), V.double(), is_causal=True).numpy()
        assert got.shape == ref.shape and rel(got, ref) <= 1e-5
        scores = Q.double() @ K.double().transpose(-2, -1) / 4.0
        scores = scores.masked_fill(torch.arange(SKV)[None, :] > torch.arange(SQ)[:, None], float("-inf"))
        assert rel(got, (torch.softmax(scores, dim=-1) @ V.double()).numpy()) <= 1e-5


def test_conv_golden():
    g = np.load(GOLDEN / "conv_2x3x7x7_k3_p1_bias_f32.npz")
    assert rel(oracle.conv2d(g["X"], g["W"], g["b"], pad=(1, 1)), g["Y"]) <= 1e-6


@pytest.mark.parametrize("stride,pad,dil", [((1, 1), (0, 0), (1, 1)), ((2, 1), (1, 2), (1, 1)), ((1, 1), (2, 2), (2, 2)), ((3, 2), (0, 1), (1, 2))])
def test_conv_against_torch(stride, pad, dil):
    g = torch.Generator().manual_seed(7)
    x, w, b = torch.randn(2, 3, 11, 9, generator=g), torch.randn(5, 3, 3, 2, generator=g), torch.randn(5, generator=g)
    ref = torch.nn.functional.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad, dilation=dil).numpy()
    Y = oracle.conv2d(x.numpy(), w.numpy(), b.numpy(), stride, pad, dil)
    assert Y.shape == ref.shape
    assert rel(Y, ref) <= 1e-6
    assert rel(oracle.conv2d(x.numpy(), w.numpy(), None, stride, pad, dil), ref - b.double().numpy()[None, :, None, None]) <= 1e-6


@pytest.mark.parametrize("group,C,OC", [(2, 6, 4), (3, 3, 6), (4, 8, 8)])
def test_conv_with_groups_two_other_statements(group, C, OC):
    """The grouped form against two statements that share none of its code: torch's conv2d with groups in float64, and the
    dense convolution with the weights laid out block-diagonally (a group's filters see zeros on the other groups' channels)."""
    g = torch.Generator().manual_seed(group)
    x, w, b = torch.randn(2, C, 9, 8, generator=g), torch.randn(OC, C // group, 3, 2, generator=g), torch.randn(OC, generator=g)
    Y = oracle.conv2d(x.numpy(), w.numpy(), b.numpy(), (2, 1), (1, 0, 0, 2), (1, 2), group=group)
    xp = torch.nn.functional.pad(x.double(), (0, 2, 1, 0))          # (left, right, top, bottom)
    ref = torch.nn.functional.conv2d(xp, w.double(), b.double(), stride=(2, 1), dilation=(1, 2), groups=group).numpy()
    assert Y.shape == ref.shape and rel(Y, ref) <= 1e-6
    dense = np.zeros((OC, C, 3, 2), np.float32)
    cg, og = C // group, OC // group
    for j in range(group):
        dense[j * og:(j + 1) * og, j * cg:(j + 1) * cg] = w.numpy()[j * og:(j + 1) * og]
    assert np.array_equal(Y, oracle.conv2d(x.numpy(), dense, b.numpy(), (2, 1), (1, 0, 0, 2), (1, 2)))
    with pytest.raises(ValueError):
        oracle.conv2d(x.numpy(), w.numpy(), None, group=group + 5)


def test_conv_closed_forms():
    # all-ones input and kernel: the output counts the taps inside the image (zero padding)
    Y = oracle.conv2d(np.ones((1, 2, 5, 5), np.float32), np.ones((1, 2, 3, 3), np.float32), pad=(1, 1))
    assert Y[0, 0, 0, 0] == 8 and Y[0, 0, 0, 2] == 12 and Y[0, 0, 2, 2] == 18
    # a delta kernel shifts the image
    X = np.arange(2 * 1 * 4 * 4, dtype=np.float32).reshape(2, 1, 4, 4)
    W = np.zeros((1, 1, 3, 3), np.float32)
    W[0, 0, 1, 1] = 1
    assert np.array_equal(oracle.conv2d(X, W, pad=(1, 1)), X)
    W[:] = 0
    W[0, 0, 2, 1] = 1   # reads X[h+1, w]
    exp = np.zeros_like(X)
    exp[:, :, :-1, :] = X[:, :, 1:, :]
    assert np.array_equal(oracle.conv2d(X, W, pad=(1, 1)), exp)
    # output extent formula of the reference (conv_node.cpp:224-233)
    assert oracle.conv_out_dim(56, 1, 1, 3, 1) == 56 and oracle.conv_out_dim(7, 0, 2, 3, 2) == 2 and oracle.conv_out_dim(2, 0, 1, 3, 1) == 0


# ---- attention ------------------------------------------------------------------------

def test_attention_golden_and_torch():
    g = np.load(GOLDEN / "attn_1x2x96x64_bf16.npz")
    assert rel(oracle.attention(g["Q"], g["K"], g["V"], 0.125), g["O"]) <= 1e-5
    gen = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(2, 2, 40, 64, generator=gen).bfloat16() for _ in range(3))
    bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double()).numpy()
    assert rel(oracle.attention(bits(q), bits(k), bits(v)), ref) <= 1e-5


def test_attention_closed_forms():
    gen = torch.Generator().manual_seed(12)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    q, v = torch.randn(1, 1, 9, 64, generator=gen).bfloat16(), torch.randn(1, 1, 20, 64, generator=gen).bfloat16()
    k = torch.randn(1, 1, 1, 64, generator=gen).bfloat16().expand(1, 1, 20, 64)
    O = oracle.attention(bits(q), bits(k), bits(v))
    assert rel(O, np.broadcast_to(v.double().mean(dim=2, keepdim=True).numpy(), O.shape)) <= 1e-5
    k = torch.randn(1, 1, 20, 64, generator=gen).bfloat16()
    perm = torch.randperm(20, generator=gen)
    a = oracle.attention(bits(q), bits(k), bits(v))
    b = oracle.attention(bits(q), bits(k[:, :, perm]), bits(v[:, :, perm]))
    assert rel(a, b.astype(np.float64)) <= 1e-5


# ---- elementwise nodes and broadcast ------------------------------------------------------

def ulp_diff(y, ref):
    """Largest distance in units in the last place of `ref`'s type."""
    ref = np.asarray(ref)
    y = np.asarray(y, ref.dtype)
    spacing = np.spacing(np.abs(ref).astype(ref.dtype))
    finite = np.isfinite(ref)
    assert np.array_equal(np.isfinite(y), finite)
    return float((np.abs(y[finite].astype(np.float64) - ref[finite].astype(np.float64)) / spacing[finite]).max()) if finite.any() else 0.0


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_elementwise_binary_matches_ieee(dt):
    rng = np.random.default_rng(3)
    a = (rng.standard_normal(1001) * 10).astype(dt)
    b = (rng.standard_normal(1001) * 10).astype(dt)
    b[::97] = 0.0                      # division by zero -> inf / nan as IEEE says
    a[::193] = np.nan                  # fmax / fmin return the other operand for one NaN
    with np.errstate(all="ignore"):
        assert np.array_equal(oracle.elementwise_binary("add", a, b), a + b, equal_nan=True)
        assert np.array_equal(oracle.elementwise_binary("sub", a, b), a - b, equal_nan=True)
        assert np.array_equal(oracle.elementwise_binary("mul", a, b), a * b, equal_nan=True)
        assert np.array_equal(oracle.elementwise_binary("div", a, b), a / b, equal_nan=True)
    assert np.array_equal(oracle.elementwise_binary("maximum", a, b), np.fmax(a, b), equal_nan=True)
    assert np.array_equal(oracle.elementwise_binary("minimum", a, b), np.fmin(a, b), equal_nan=True)
    # pow: exact cases (order of the operands, the IEEE special values), and numpy's pow within 1 ulp elsewhere
    base, expo = np.array([2, 3, 0.5, -2, -2, 0, 7, np.inf, 1], dt), np.array([10, 2, 2, 3, 0.5, 0, 0, -1, np.nan], dt)
    with np.errstate(all="ignore"):
        assert np.array_equal(oracle.elementwise_binary("pow", base, expo), np.array([1024, 9, 0.25, -8, np.nan, 1, 1, 0, 1], dt), equal_nan=True)
        p, q = np.abs(a[:500]) + dt(0.1), b[:500] / dt(4)
        assert ulp_diff(oracle.elementwise_binary("pow", p, q), np.power(p.astype(np.float64), q.astype(np.float64)).astype(dt)) <= 1
    # not commutative operations in the right order
    assert oracle.elementwise_binary("sub", np.array([5], dt), np.array([3], dt))[0] == 2
    assert oracle.elementwise_binary("div", np.array([6], dt), np.array([3], dt))[0] == 2
    with pytest.raises(ValueError):
        oracle.elementwise_binary("add", np.zeros((2, 3), dt), np.zeros((3, 2), dt))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_elementwise_unary_closed_forms_and_numpy(dt):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(2001) * 4).astype(dt)
    # exact operations
    assert np.array_equal(oracle.elementwise_unary("abs", x), np.abs(x))
    relu = oracle.elementwise_unary("relu", x)
    assert np.array_equal(relu, np.fmax(x, dt(0)))
    assert (relu >= 0).all() and np.array_equal(relu[x > 0], x[x > 0])
    assert oracle.elementwise_unary("relu", np.array([np.nan], dt))[0] == 0          # fmax(NaN, 0) = 0
    sq = oracle.elementwise_unary("sqrt", np.abs(x))
    assert np.array_equal(sq, np.sqrt(np.abs(x)))                                    # correctly rounded in both
    # transcendental ones: numpy evaluated in float64 (longdouble for fp64) and rounded is the yardstick
    wide = np.longdouble if dt == np.float64 else np.float64
    xw = x.astype(wide)
    import scipy.special as sp
    cases = {"exp": np.exp(xw), "tanh": np.tanh(xw), "sigmoid": 1 / (1 + np.exp(-xw)),
             "erf": sp.erf(x.astype(np.float64)).astype(wide)}
    for op, ref in cases.items():
        assert ulp_diff(oracle.elementwise_unary(op, x), ref.astype(dt)) <= (4 if op == "sigmoid" else 2), op
    # closed forms
    z = np.zeros(3, dt)
    assert np.array_equal(oracle.elementwise_unary("exp", z), np.ones(3, dt))
    assert np.array_equal(oracle.elementwise_unary("sigmoid", z), np.full(3, 0.5, dt))
    assert np.array_equal(oracle.elementwise_unary("tanh", -x), -oracle.elementwise_unary("tanh", x))
    assert np.array_equal(oracle.elementwise_unary("erf", -x), -oracle.elementwise_unary("erf", x))
    big = np.array([1000.0, -1000.0], dt)
    assert np.array_equal(oracle.elementwise_unary("sigmoid", big), np.array([1.0, 0.0], dt))
    assert np.array_equal(oracle.elementwise_unary("tanh", big), np.array([1.0, -1.0], dt))
    # shape is kept
    assert oracle.elementwise_unary("exp", np.zeros((2, 3, 4), dt)).shape == (2, 3, 4)


def test_broadcast_matches_numpy():
    rng = np.random.default_rng(5)
    for in_shape, out_shape in [((3,), (2, 3)), ((4, 1), (4, 5)), ((1, 3, 1, 2), (2, 3, 4, 2)), ((1,), (7,)), ((2, 3), (2, 3)),
                                ((64,), (2, 64, 1, 1))[:0] or ((1, 64, 1, 1), (2, 64, 3, 3))]:
        x = rng.standard_normal(in_shape).astype(np.float32)
        assert np.array_equal(oracle.broadcast(x, out_shape), np.broadcast_to(x, out_shape))
        xd = rng.standard_normal(in_shape)
        assert np.array_equal(oracle.broadcast(xd, out_shape), np.broadcast_to(xd, out_shape))
    with pytest.raises(ValueError):
        oracle.broadcast(np.zeros((2, 3), np.float32), (2, 4))


def test_reduce_nodes_against_numpy_and_closed_forms():
    """oracle.reduce (ml::Sum / Max / Min / Mean) pinned by numpy's reductions in float64, by integer-valued
    inputs (every partial sum exact, so the order of the additions cannot matter) and by the identities of
    an empty extent; Max / Min must be exactly numpy's reductions, and fmax / fmin where a NaN is present."""
    rng = np.random.default_rng(12)
    for dt in (np.float32, np.float64):
        x = rng.standard_normal((5, 7, 3, 4)).astype(dt)
        for axes in ((3,), (0,), (1, 2), (0, 1, 2, 3), (-1,), (2, 3)):
            for keep in (False, True):
                ax = tuple(a % 4 for a in axes)
                tol = 1e-5 if dt == np.float32 else 1e-13
                np.testing.assert_allclose(oracle.reduce("sum", x, axes, keep), x.astype(np.float64).sum(axis=ax, keepdims=keep), rtol=tol, atol=tol)
                np.testing.assert_allclose(oracle.reduce("mean", x, axes, keep), x.astype(np.float64).mean(axis=ax, keepdims=keep), rtol=tol, atol=tol)
                assert np.array_equal(oracle.reduce("max", x, axes, keep), x.max(axis=ax, keepdims=keep))
                assert np.array_equal(oracle.reduce("min", x, axes, keep), x.min(axis=ax, keepdims=keep))
                assert oracle.reduce("sum", x, axes, keep).dtype == dt
        ints = rng.integers(-8, 9, (6, 50, 3)).astype(dt)
        assert np.array_equal(oracle.reduce("sum", ints, (1,)), ints.sum(axis=1))                  # exact in any order
        assert np.array_equal(oracle.reduce("mean", np.full((4, 8), 3.0, dt), (1,)), np.full(4, 3.0, dt))
        # fmax / fmin skip a NaN; a row of nothing but NaN keeps the identity the reference starts from
        y = np.array([[1.0, np.nan, 3.0], [np.nan, np.nan, np.nan], [-np.inf, 2.0, np.inf]], dt)
        assert np.array_equal(oracle.reduce("max", y, (1,)), np.array([3.0, -np.inf, np.inf], dt))
        assert np.array_equal(oracle.reduce("min", y, (1,)), np.array([1.0, np.inf, -np.inf], dt))
        assert np.array_equal(oracle.reduce("max", y[[0, 2]], (1,)), np.fmax.reduce(y[[0, 2]], axis=1))
        # an empty extent leaves the identity
        e = np.zeros((3, 0, 2), dt)
        assert np.array_equal(oracle.reduce("sum", e, (1,)), np.zeros((3, 2), dt))
        assert np.array_equal(oracle.reduce("max", e, (1,)), np.full((3, 2), -np.inf, dt))
        assert np.array_equal(oracle.reduce("min", e, (1,)), np.full((3, 2), np.inf, dt))
    with pytest.raises(ValueError):
        oracle.reduce("sum", np.zeros((2, 3, 4)), (0, 2))        # not a block of adjacent axes
    with pytest.raises(ValueError):
        oracle.reduce("mean", np.zeros((2, 0)), (1,))


# ---- activations with scalar operands, fill, dot, transpose ------------------------------------------------

@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_activations_against_torch_and_closed_forms(dt):
    """ml::Elu / ml::LeakyReLU / ml::HardSigmoid: torch's functions of the same names (computed in float64),
    and the points where a wrong branch or a dropped operand shows: f(0), the saturation of HardSigmoid,
    the slope for negative inputs, alpha = 0."""
    rng = np.random.default_rng(8)
    x = np.concatenate([rng.standard_normal(5000) * 3, [0.0, -0.0, 1e-30, -1e-30, 50.0, -50.0, np.inf, -np.inf]]).astype(dt)
    t = torch.from_numpy(x.astype(np.float64))
    tol = 2e-7 if dt == np.float32 else 1e-15
    cases = [("elu", 1.0, 0.0, torch.nn.functional.elu(t, 1.0)), ("elu", 0.3, 0.0, torch.nn.functional.elu(t, 0.3)),
             ("leaky_relu", 0.01, 0.0, torch.nn.functional.leaky_relu(t, 0.01)), ("leaky_relu", 0.25, 0.0, torch.nn.functional.leaky_relu(t, 0.25)),
             ("hard_sigmoid", 1.0 / 6.0, 0.5, torch.nn.functional.hardsigmoid(t)), ("hard_sigmoid", 0.2, 0.5, torch.clamp(0.2 * t + 0.5, 0.0, 1.0))]
    for op, alpha, beta, ref in cases:
        y = oracle.elementwise_activation(op, x, alpha, beta)
        assert y.dtype == dt and y.shape == x.shape
        ref = ref.numpy()
        ok = np.isfinite(ref)
        assert np.array_equal(np.isnan(y), np.isnan(ref)), op
        np.testing.assert_allclose(y[ok], ref[ok], rtol=tol, atol=tol, err_msg=op)
        assert np.array_equal(y[~ok & ~np.isnan(ref)], ref[~ok & ~np.isnan(ref)].astype(dt))      # the infinities
    one = np.array([2.5, -2.5], dt)
    assert np.array_equal(oracle.elementwise_activation("elu", one, 0.0), np.array([2.5, -0.0], dt))          # alpha = 0: negatives vanish
    assert oracle.elementwise_activation("elu", one, 2.0)[1] == dt(2.0) * (np.exp(dt(-2.5)) - dt(1.0))
    assert np.array_equal(oracle.elementwise_activation("leaky_relu", one, 0.5), np.array([2.5, -1.25], dt))
    assert np.array_equal(oracle.elementwise_activation("hard_sigmoid", np.array([-10, 0, 1, 10], dt), 0.25, 0.5), np.array([0, 0.5, 0.75, 1], dt))
    with pytest.raises(KeyError):
        oracle.elementwise_activation("gelu", one, 1.0)


def test_dot_against_numpy_and_exact_cases():
    rng = np.random.default_rng(9)
    for dt, tol in ((np.float32, 1e-5), (np.float64, 1e-13)):
        x, y = rng.standard_normal(4097).astype(dt), rng.standard_normal(4097).astype(dt)
        exact = np.dot(x.astype(np.longdouble), y.astype(np.longdouble))
        scale = np.dot(np.abs(x).astype(np.longdouble), np.abs(y).astype(np.longdouble))
        assert abs(oracle.dot(x, y) - exact) <= tol * scale
        # increments: every third element of x against every second of y
        n = 1000
        assert abs(oracle.dot(x, y, 3, 2, n) - np.dot(x[:3 * n:3].astype(np.longdouble), y[:2 * n:2].astype(np.longdouble))) <= tol * scale
        # integer values are exact in any order; a swapped increment or an off-by-one in n changes them
        xi, yi = np.arange(1, 101, dtype=dt), np.arange(100, 0, -1, dtype=dt)
        assert oracle.dot(xi, yi) == dt(sum(a * b for a, b in zip(range(1, 101), range(100, 0, -1))))
        assert oracle.dot(xi, yi, 2, 1, 50) == dt(sum(a * b for a, b in zip(range(1, 101, 2), range(100, 50, -1))))
        assert oracle.dot(xi, yi, 1, 1, 0) == 0
        assert oracle.dot(xi, np.ones(1, dt), 1, 0, 100) == dt(5050)       # increment 0 repeats one element


def test_transpose_matches_numpy_for_every_permutation():
    """oracle_transpose against numpy.transpose: every permutation of rank 2-4 tensors, every element size; an
    inverted permutation or a slip in the strides fails it (the extents are pairwise different)."""
    import itertools

    rng = np.random.default_rng(10)
    for shape in ((3, 5), (2, 3, 5), (2, 3, 4, 5)):
        for dt in (np.uint8, np.int16, np.float32, np.float64):
            X = rng.integers(0, 200, size=shape).astype(dt)
            for perm in itertools.permutations(range(len(shape))):
                Y = oracle.transpose(X, perm)
                assert Y.dtype == dt and Y.flags.c_contiguous
                assert np.array_equal(Y, np.transpose(X, perm)), (shape, perm)


# ---- map nests: the interpreter of tasklet bodies -------------------------------------------------------------------

def _map_node(bounds, reads, statements, writes, scalars=()):
    """A ROCMMap payload written by hand: reads / writes are (connector, strides, extent, type[, value])."""
    acc = lambda t: {"connector": t[0], "strides": [str(x) for x in t[1]], "extent": str(t[2]), "element_type": t[3], **({"value": t[4]} if len(t) > 4 else {})}
    return {"indvars": [f"i{k}" for k in range(len(bounds))], "bounds": [str(b) for b in bounds], "symbols": [],
            "reads": [acc(r) for r in reads], "writes": [acc(w) for w in writes],
            "scalars": [{"connector": c, "element_type": t} for c, t in scalars],
            "statements": [{"out": o, "type": t, "op": op, "args": list(args)} for o, t, op, args in statements]}


def test_map_nest_follows_strides_statement_order_and_roundings():
    rng = np.random.default_rng(11)
    n, m = 7, 12
    A, B = rng.standard_normal((n, m)).astype(np.float32), rng.standard_normal((n, m)).astype(np.float32)
    c = rng.standard_normal(m).astype(np.float32)
    # relu(A * B + c), c repeated over the rows, stored row by row and transposed: pinned by numpy, whose ufuncs round
    # after every operation as separate statements do
    node = _map_node([n, m], [("a", [m, 1], n * m, "Float"), ("b", [m, 1], n * m, "Float"), ("c", [0, 1], m, "Float")],
                     [("t0", "Float", "fp_mul", ["a", "b"]), ("t1", "Float", "fp_add", ["t0", "c"]), ("t2", "Float", "fmax", ["#0.0f", "t1"])],
                     [("y", [m, 1], n * m, "Float", "t2"), ("yt", [1, n], n * m, "Float", "t2")])
    out = oracle.map_nest(node, {"a": A, "b": B, "c": c})
    ref = np.maximum(np.float32(0), A * B + c)
    assert np.array_equal(out["y"].reshape(n, m), ref) and np.array_equal(out["yt"].reshape(m, n), ref.T)
    # a transposed operand: a slip between the two stride lists fails this
    node = _map_node([n, m], [("a", [m, 1], n * m, "Float"), ("bt", [1, n], n * m, "Float")],
                     [("t0", "Float", "fp_sub", ["a", "bt"])], [("y", [m, 1], n * m, "Float", "t0")])
    Bt = rng.standard_normal((m, n)).astype(np.float32)
    assert np.array_equal(oracle.map_nest(node, {"a": A, "bt": Bt})["y"].reshape(n, m), A - Bt.T)
    # argument order of the non-commutative operations, a scalar operand, a literal, three loops
    X = rng.standard_normal((3, 4, 5))
    node = _map_node([3, 4, 5], [("x", [20, 5, 1], 60, "Double")],
                     [("t0", "Double", "fp_div", ["s", "x"]), ("t1", "Double", "fp_sub", ["t0", "#0.25"]), ("t2", "Double", "fp_neg", ["t1"]),
                      ("t3", "Double", "pow", ["t2", "#2.0"]), ("t4", "Double", "fp_rem", ["t3", "s"]), ("t5", "Double", "atan2", ["t4", "x"])],
                     [("y", [20, 5, 1], 60, "Double", "t5")], scalars=[("s", "Double")])
    ref = np.arctan2(np.fmod((-(1.5 / X - 0.25)) ** 2.0, 1.5), X)
    assert np.allclose(oracle.map_nest(node, {"x": X}, scalars={"s": 1.5})["y"].reshape(X.shape), ref, rtol=1e-15, atol=0)
    # fp_fma is one rounding: the float64 product of two float32 values is exact, so rounding a*b+c once from
    # float64 differs from the two roundings of mul-then-add on some elements and equals the fused result on all but
    # double-rounding cases (none in this sample)
    a32, b32, c32 = (rng.standard_normal(4096).astype(np.float32) for _ in range(3))
    fused = _map_node([4096], [("a", [1], 4096, "Float"), ("b", [1], 4096, "Float"), ("c", [1], 4096, "Float")],
                      [("t0", "Float", "fp_fma", ["a", "b", "c"])], [("y", [1], 4096, "Float", "t0")])
    two = _map_node([4096], [("a", [1], 4096, "Float"), ("b", [1], 4096, "Float"), ("c", [1], 4096, "Float")],
                    [("t0", "Float", "fp_mul", ["a", "b"]), ("t1", "Float", "fp_add", ["t0", "c"])], [("y", [1], 4096, "Float", "t1")])
    yf, y2 = oracle.map_nest(fused, {"a": a32, "b": b32, "c": c32})["y"], oracle.map_nest(two, {"a": a32, "b": b32, "c": c32})["y"]
    exact = a32.astype(np.float64) * b32.astype(np.float64) + c32.astype(np.float64)
    assert np.array_equal(y2, a32 * b32 + c32)
    assert (yf != y2).any() and np.abs(yf - exact).max() <= np.abs(y2 - exact).max()
    assert np.abs(yf.astype(np.float64) - exact).max() <= np.abs(exact).max() * 2.0 ** -24
    # a float32 statement on float64 operands converts first; a float64 statement on float32 operands widens
    node = _map_node([64], [("a", [1], 64, "Double")], [("t0", "Float", "fp_mul", ["a", "a"]), ("t1", "Double", "fp_add", ["t0", "a"])],
                     [("y", [1], 64, "Double", "t1")])
    a64 = rng.standard_normal(64)
    assert np.array_equal(oracle.map_nest(node, {"a": a64})["y"], (a64.astype(np.float32) * a64.astype(np.float32)).astype(np.float64) + a64)
    # errors: an unknown operation, a value used before it exists, an operand that is too small
    bad = _map_node([4], [("a", [1], 4, "Float")], [("t0", "Float", "fp_nope", ["a"])], [("y", [1], 4, "Float", "t0")])
    with pytest.raises(ValueError):
        oracle.map_nest(bad, {"a": np.zeros(4, np.float32)})
    with pytest.raises(ValueError, match="holds 3 elements"):
        oracle.map_nest(_map_node([4], [("a", [1], 4, "Float")], [("t0", "Float", "assign", ["a"])], [("y", [1], 4, "Float", "t0")]), {"a": np.zeros(3, np.float32)})


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_map_nest_cmath_calls_are_the_libm_functions(dtype):
    """Every CMath stem against numpy / scipy / math in float64 (a wrong table entry - exp for exp2, ceil for floor,
    swapped arguments - is off by far more than the tolerance)."""
    import math
    import scipy.special as sp
    rng = np.random.default_rng(12)
    n = 257
    tname = "Double" if dtype == np.float64 else "Float"
    tol = 4e-15 if dtype == np.float64 else 4e-7
    pos, unit, anyv = (rng.random(n) * 4 + 0.1).astype(dtype), (rng.random(n) * 1.8 - 0.9).astype(dtype), (rng.standard_normal(n) * 3).astype(dtype)
    other = (rng.standard_normal(n) * 2 + 0.3).astype(dtype)
    unary = {"sin": (np.sin, anyv), "cos": (np.cos, anyv), "tan": (np.tan, unit), "asin": (np.arcsin, unit), "acos": (np.arccos, unit),
             "atan": (np.arctan, anyv), "sinh": (np.sinh, anyv), "cosh": (np.cosh, anyv), "tanh": (np.tanh, anyv), "asinh": (np.arcsinh, anyv),
             "acosh": (np.arccosh, pos + 1), "atanh": (np.arctanh, unit), "exp": (np.exp, anyv), "exp2": (np.exp2, anyv),
             "exp10": (lambda x: 10.0 ** x, unit), "expm1": (np.expm1, unit), "log": (np.log, pos), "log10": (np.log10, pos),
             "log2": (np.log2, pos), "log1p": (np.log1p, pos), "sqrt": (np.sqrt, pos), "cbrt": (np.cbrt, anyv), "erf": (sp.erf, anyv),
             "erfc": (sp.erfc, unit), "tgamma": (sp.gamma, pos), "lgamma": (sp.gammaln, pos), "fabs": (np.abs, anyv), "ceil": (np.ceil, anyv),
             "floor": (np.floor, anyv), "trunc": (np.trunc, anyv), "round": (lambda x: np.sign(x) * np.floor(np.abs(x) + 0.5), anyv),
             "nearbyint": (np.rint, anyv), "rint": (np.rint, anyv)}
    for stem, (fn, x) in unary.items():
        node = _map_node([n], [("x", [1], n, tname)], [("t", tname, stem, ["x"])], [("y", [1], n, tname, "t")])
        got = oracle.map_nest(node, {"x": x})["y"].astype(np.float64)
        ref = fn(x.astype(np.float64))
        assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max()), stem
    binary = {"atan2": np.arctan2, "pow": lambda a, b: np.abs(a) ** b, "hypot": np.hypot, "fmod": np.fmod,
              "remainder": lambda a, b: np.array([math.remainder(u, v) for u, v in zip(a, b)]), "copysign": np.copysign,
              "fmax": np.fmax, "fmin": np.fmin, "fdim": lambda a, b: np.maximum(a - b, 0.0)}
    for stem, fn in binary.items():
        a = np.abs(anyv) if stem == "pow" else anyv
        node = _map_node([n], [("a", [1], n, tname), ("b", [1], n, tname)], [("t", tname, stem, ["a", "b"])], [("y", [1], n, tname, "t")])
        got = oracle.map_nest(node, {"a": a, "b": other})["y"].astype(np.float64)
        ref = fn(a.astype(np.float64), other.astype(np.float64))
        assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max()), stem


def test_conv2d_with_a_begin_and_an_end_pad_per_axis():
    """torch pads by hand (F.pad takes left, right, top, bottom) and convolves without padding, in float64: the begin pad
    moves the window, the end pad only adds output positions. Swapping begin and end, or rows and columns, fails."""
    rng = np.random.default_rng(31)
    X = rng.standard_normal((2, 3, 9, 11)).astype(np.float32)
    W = rng.standard_normal((4, 3, 3, 2)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    for pads, stride, dil in (((0, 1, 2, 0), (1, 1), (1, 1)), ((2, 0, 1, 3), (2, 1), (1, 2)), ((1, 2, 3, 4), (1, 2), (2, 1))):
        top, left, bottom, right = pads
        xp = torch.nn.functional.pad(torch.from_numpy(X).double(), (left, right, top, bottom))
        ref = torch.nn.functional.conv2d(xp, torch.from_numpy(W).double(), torch.from_numpy(b).double(), stride=stride, dilation=dil).numpy()
        got = oracle.conv2d(X, W, b, stride, pads, dil)
        assert got.shape == ref.shape and np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()
    # two-element pads mean the same on both sides
    assert np.array_equal(oracle.conv2d(X, W, b, pad=(1, 2)), oracle.conv2d(X, W, b, pad=(1, 2, 1, 2)))
