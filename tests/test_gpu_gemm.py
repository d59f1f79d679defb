"""GEMM node on the GPU against the CPU oracle, through the C-ABI
(docc_rocm_dgemm / docc_rocm_sgemm).

Tolerances (norm-wise relative error max|C - C_ref| / max|C_ref|):
fp64 1e-12, fp32 1e-5. Integer-valued inputs are compared bit-exactly: every
product and partial sum is exactly representable, so the result does not
depend on summation order.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu

TOL = {np.float64: 1e-12, np.float32: 1e-5}
N, T = oracle.NO_TRANS, oracle.TRANS


def run_gemm(rt, A, B, C=None, alpha=1.0, beta=0.0, ta=N, tb=N, lda=None, ldb=None, ldc=None, offset=0):
    """Calls the C-ABI on device copies of A, B (2-d arrays as stored) and C."""
    dt = A.dtype.type
    m, k = (A.shape[1], A.shape[0]) if ta == T else A.shape
    n = B.shape[0] if tb == T else B.shape[1]

    def padded(M, ld):
        # store M with leading dimension ld (>= cols), optionally shifted by `offset` elements
        ld = ld or max(M.shape[1], 1)
        buf = np.full(offset + max(M.shape[0], 1) * ld, np.nan, dt)
        view = buf[offset:offset + M.shape[0] * ld].reshape(M.shape[0], ld)
        view[:, :M.shape[1]] = M
        return buf, ld

    a_buf, lda = padded(A, lda)
    b_buf, ldb = padded(B, ldb)
    c_init = np.full((m, n), np.nan, dt) if C is None else C
    c_buf, ldc = padded(c_init, ldc)
    a, b, c = dev(a_buf), dev(b_buf), dev(c_buf)
    es = a.element_size()
    fn = rt.dgemm if dt == np.float64 else rt.sgemm
    fn(m, n, k, alpha, a.data_ptr() + offset * es, lda, b.data_ptr() + offset * es, ldb, beta,
       c.data_ptr() + offset * es, ldc, trans_a=ta, trans_b=tb)
    torch.cuda.synchronize()
    out = host(c)[offset:offset + m * ldc].reshape(m, ldc) if m else np.empty((0, ldc), dt)
    if ldc > n and m:
        assert np.isnan(out[:, n:]).all(), "kernel wrote into the padding of C"
    return out[:, :n].copy()


def int_matrix(rng, shape, dt, lim=8):
    return rng.integers(-lim, lim + 1, shape).astype(dt)


SHAPES = [(1, 1, 1), (17, 33, 65), (33, 17, 5), (64, 64, 64), (65, 63, 130), (128, 128, 16), (129, 257, 31),
          (257, 129, 100), (1, 300, 7), (300, 1, 7), (40, 50, 1), (200, 136, 1024)]


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_integer_exact_nn(rt, dt, m, n, k):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    A, B = int_matrix(rng, (m, k), dt), int_matrix(rng, (k, n), dt)
    C = run_gemm(rt, A, B)
    assert np.array_equal(C, oracle.gemm(A, B))
    assert np.array_equal(C, (A.astype(np.float64) @ B.astype(np.float64)).astype(dt))


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("ta,tb", [(N, T), (T, N), (T, T)])
@pytest.mark.parametrize("m,n,k", [(17, 33, 65), (130, 70, 40), (64, 128, 256), (5, 3, 2)])
def test_gemm_integer_exact_transposed(rt, dt, ta, tb, m, n, k):
    rng = np.random.default_rng(7 + m + n + k)
    A = int_matrix(rng, (k, m) if ta == T else (m, k), dt)
    B = int_matrix(rng, (n, k) if tb == T else (k, n), dt)
    C = run_gemm(rt, A, B, ta=ta, tb=tb)
    assert np.array_equal(C, oracle.gemm(A, B, trans_a=ta, trans_b=tb))


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_gemm_alpha_beta_ld_and_alignment(rt, dt):
    rng = np.random.default_rng(11)
    m, n, k = 70, 45, 33
    A, B, C0 = int_matrix(rng, (m, k), dt), int_matrix(rng, (k, n), dt), int_matrix(rng, (m, n), dt)
    ref = oracle.gemm(A, B, C0, alpha=2.0, beta=-3.0)
    # padded leading dimensions (aligned path)
    assert np.array_equal(run_gemm(rt, A, B, C0, 2.0, -3.0, lda=40, ldb=48, ldc=52), ref)
    # odd leading dimensions and a one-element pointer offset (unaligned path)
    assert np.array_equal(run_gemm(rt, A, B, C0, 2.0, -3.0, lda=35, ldb=47, ldc=49, offset=1), ref)
    # beta == 0: C is not read (it holds NaNs), as cblas specifies
    out = run_gemm(rt, A, B, None, 1.0, 0.0)
    assert np.isfinite(out).all() and np.array_equal(out, oracle.gemm(A, B))
    # k == 0: C = beta * C
    out = run_gemm(rt, np.zeros((m, 0), dt), np.zeros((0, n), dt), C0, 1.0, 2.0)
    assert np.array_equal(out, 2 * C0)
    out = run_gemm(rt, np.zeros((m, 0), dt), np.zeros((0, n), dt), None, 1.0, 0.0)
    assert np.array_equal(out, np.zeros((m, n), dt))


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_gemm_structured_cases(rt, dt):
    rng = np.random.default_rng(5)
    A = rng.standard_normal((100, 100)).astype(dt)
    eye = np.eye(100, dtype=dt)
    assert np.array_equal(run_gemm(rt, A, eye), A)
    assert np.array_equal(run_gemm(rt, eye, A), A)
    perm = eye[rng.permutation(100)]
    assert np.array_equal(run_gemm(rt, perm, A), perm @ A)
    # rank-1 outer product (m x 1 times 1 x n), the shape numpy.outer lowers to
    u, v = rng.standard_normal((37, 1)).astype(dt), rng.standard_normal((1, 91)).astype(dt)
    assert np.array_equal(run_gemm(rt, u, v), u @ v)
    # A @ ones = row sums
    ones = np.ones((100, 1), dtype=dt)
    assert rel_err_max(run_gemm(rt, A, ones), A.astype(np.float64).sum(axis=1, keepdims=True)) <= TOL[dt]


def test_gemm_errors(rt):
    from docc_amd.runtime import RocmRuntimeError
    a = torch.zeros(16, device="cuda")
    with pytest.raises(RocmRuntimeError):
        rt.sgemm(4, 4, 4, 1.0, a.data_ptr(), 2, a.data_ptr(), 4, 0.0, a.data_ptr(), 4)  # lda < k
    with pytest.raises(RocmRuntimeError):
        rt.sgemm(4, 4, 4, 1.0, a.data_ptr(), 4, a.data_ptr(), 4, 0.0, a.data_ptr(), 4, trans_a=7)
    with pytest.raises(RocmRuntimeError):
        rt.sgemm(-1, 4, 4, 1.0, a.data_ptr(), 4, a.data_ptr(), 4, 0.0, a.data_ptr(), 4)
    rt.sgemm(0, 4, 4, 1.0, 0, 4, 0, 4, 0.0, 0, 4)  # empty: no-op


def test_dgemm_config_1000(rt):
    # benchmark configuration 1: uniform[0,1) 1000x1000 fp64, seed 0, vs a long-double accumulation
    rng = np.random.default_rng(0)
    A, B = rng.random((1000, 1000)), rng.random((1000, 1000))
    C = run_gemm(rt, A, B)
    ref = oracle.gemm(A, B, variant="ld")
    assert rel_err_max(C, ref) <= 1e-12
    # and against the form the reference's openmp target computes (cblas semantics, fp64 accumulate)
    assert rel_err_max(C, oracle.gemm(A, B)) <= 1e-12


def test_sgemm_random_medium(rt):
    rng = np.random.default_rng(2)
    A = (rng.standard_normal((300, 700)) / np.sqrt(700)).astype(np.float32)
    B = (rng.standard_normal((700, 260)) / np.sqrt(700)).astype(np.float32)
    C = run_gemm(rt, A, B)
    assert rel_err_max(C, oracle.gemm(A, B, variant="acc64")) <= 1e-5
    assert rel_err_max(C, oracle.gemm(A, B)) <= 1e-5


def test_sgemm_config_4096(rt):
    # benchmark configuration 3a: N(0,1)/sqrt(K), 4096^3 fp32, seed 2
    rng = np.random.default_rng(2)
    K = 4096
    A = (rng.standard_normal((K, K)) / 64).astype(np.float32)
    B = (rng.standard_normal((K, K)) / 64).astype(np.float32)
    a, b = dev(A), dev(B)
    c = torch.full((K, K), float("nan"), device="cuda")
    rt.sgemm(K, K, K, 1.0, a.data_ptr(), K, b.data_ptr(), K, 0.0, c.data_ptr(), K)
    torch.cuda.synchronize()
    C = host(c)
    assert np.isfinite(C).all()
    # the oracle on a band of rows (the naive CPU loop nest is the slow side)
    rows = np.r_[0:24, 2040:2064, 4072:4096]
    ref = oracle.gemm(A[rows], B, variant="acc64")
    assert rel_err_max(C[rows], ref) <= 1e-5
    # size-independent property on the full result: C @ x == A @ (B @ x) for a probe vector, in fp64
    x = rng.standard_normal(K)
    lhs = C.astype(np.float64) @ x
    rhs = A.astype(np.float64) @ (B.astype(np.float64) @ x)
    assert np.abs(lhs - rhs).max() / np.abs(rhs).max() <= 1e-5


# every built tile configuration, selected through DOCC_ROCM_GEMM_CFG (BMxBNxBKxWAVES[xSTAGES[p]]; a
# trailing stage count picks the asynchronous multi-stage kernel, "p" its variant with a stage's copies
# dealt over the K-step), on shapes with ragged edges,
# a K tail and all four transpose combinations
F64_CFGS = ["64x64x16x4", "128x128x16x4", "64x64x16x4x2", "64x64x16x4x4", "64x64x16x4x6", "128x128x16x4x3",
            "64x32x16x4x4", "64x32x32x4x3", "64x64x32x4x3", "64x32x16x4x4p"]
F32_CFGS = ["64x64x16x4", "128x128x16x4", "128x128x16x4x3", "128x128x32x4x3", "128x256x16x4x3", "64x64x16x4x4", "256x256x32x4x2",
            "64x64x32x4x3", "128x256x32x4x2", "128x256x32x4x3", "128x256x16x4x4", "128x256x32x4x3p"]


@pytest.mark.parametrize("dt,cfg", [(np.float64, c) for c in F64_CFGS] + [(np.float32, c) for c in F32_CFGS])
def test_gemm_every_tile_configuration(rt, dt, cfg):
    import os
    rng = np.random.default_rng(sum(cfg.encode()))
    os.environ["DOCC_ROCM_GEMM_CFG"] = cfg
    try:
        for (m, n, k) in [(300, 260, 200), (129, 520, 72), (64, 64, 16), (4, 8, 1000)]:
            for ta in (N, T):
                for tb in (N, T):
                    A = int_matrix(rng, (k, m) if ta == T else (m, k), dt, lim=4)
                    B = int_matrix(rng, (n, k) if tb == T else (k, n), dt, lim=4)
                    C0 = int_matrix(rng, (m, n), dt, lim=4)
                    out = run_gemm(rt, A, B, C0, 2.0, -1.0, ta=ta, tb=tb)
                    assert np.array_equal(out, oracle.gemm(A, B, C0, alpha=2.0, beta=-1.0, trans_a=ta, trans_b=tb)), (cfg, m, n, k, ta, tb)
    finally:
        os.environ.pop("DOCC_ROCM_GEMM_CFG", None)


def test_gemm_with_leading_dimensions_and_batch_strides_past_32_bit_offsets(rt):
    """A with a row stride of 2^23 + 8 floats: a 128-row tile spans more than 2^32 bytes, which the asynchronous
    kernels' 32-bit tile offsets cannot address - the launcher must take the register-path kernels. And a batch
    whose stride is past 2^31 elements."""
    import torch
    m, n, k = 300, 256, 64
    lda = (1 << 23) + 8
    g = torch.Generator(device="cuda").manual_seed(12)
    a_buf = torch.zeros(m * lda, device="cuda")
    a = a_buf.view(m, lda)[:, :k]
    a.copy_(torch.randint(-4, 5, (m, k), device="cuda", generator=g).float())
    b = torch.randint(-4, 5, (k, n), device="cuda", generator=g).float()
    c = torch.full((m, n), float("nan"), device="cuda")
    rt.sgemm(m, n, k, 1.0, a_buf.data_ptr(), lda, b.data_ptr(), n, 0.0, c.data_ptr(), n)
    torch.cuda.synchronize()
    want = oracle.gemm(a.cpu().numpy(), b.cpu().numpy())
    assert np.array_equal(c.cpu().numpy(), want)            # integer-valued: exact
    # transposed: A^T stored [k, m] with the same stride
    at_buf = torch.zeros(k * lda, device="cuda")
    at = at_buf.view(k, lda)[:, :m]
    at.copy_(a.t())
    c.fill_(float("nan"))
    rt.sgemm(m, n, k, 1.0, at_buf.data_ptr(), lda, b.data_ptr(), n, 0.0, c.data_ptr(), n, trans_a=T)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), want)
    del a_buf, at_buf
    # batch of 3 with A matrices 2^31 + 64 elements apart
    stride_a = (1 << 31) + 64
    a3 = torch.zeros(2 * stride_a + m * k, device="cuda")
    mats = [torch.randint(-4, 5, (m, k), device="cuda", generator=g).float() for _ in range(3)]
    for z, mat in enumerate(mats):
        a3[z * stride_a:z * stride_a + m * k].copy_(mat.reshape(-1))
    c3 = torch.full((3, m, n), float("nan"), device="cuda")
    rt.gemm_batched("s", 3, m, n, k, 1.0, a3.data_ptr(), k, stride_a, b.data_ptr(), n, 0, 0.0, c3.data_ptr(), n, m * n)
    torch.cuda.synchronize()
    for z in range(3):
        assert np.array_equal(c3[z].cpu().numpy(), oracle.gemm(mats[z].cpu().numpy(), b.cpu().numpy())), z


@pytest.mark.parametrize("kind", ["d", "s", "b"])
def test_gemm_alpha_zero_does_not_reference_a_and_b(rt, kind):
    """The BLAS definition: with alpha == 0 the product is not formed, so NaNs in A or B stay out of C = beta * C
    (and beta == 0 stores zeros over a NaN-filled C)."""
    import torch
    m, n, k = 70, 90, 40
    dt = torch.float64 if kind == "d" else torch.float32
    a = torch.full((m, k), float("nan"), device="cuda", dtype=dt)
    b = torch.full((k, n), float("nan"), device="cuda", dtype=dt)
    if kind == "b":
        a, b = a.bfloat16(), b.bfloat16()
    c0 = torch.arange(m * n, device="cuda", dtype=dt).reshape(m, n) / 7
    fn = {"d": rt.dgemm, "s": rt.sgemm, "b": rt.bf16gemm_f32}[kind]
    c = c0.clone()
    fn(m, n, k, 0.0, a.data_ptr(), k, b.data_ptr(), n, -1.5, c.data_ptr(), n)
    torch.cuda.synchronize()
    assert torch.equal(c, c0 * -1.5)
    c = torch.full((m, n), float("nan"), device="cuda", dtype=dt)
    fn(m, n, k, 0.0, a.data_ptr(), k, b.data_ptr(), n, 0.0, c.data_ptr(), n)
    torch.cuda.synchronize()
    assert torch.equal(c, torch.zeros_like(c))
    want = oracle.gemm(np.full((m, k), np.nan, np.float64 if kind == "d" else np.float32), np.full((k, n), np.nan, np.float64 if kind == "d" else np.float32),
                       c0.cpu().numpy(), alpha=0.0, beta=-1.5)
    assert np.array_equal(want, (c0 * -1.5).cpu().numpy())


GEMV_CASES = [  # m, n, k, ta, tb: one output column or row, each operand layout; sizes that take the matrix-vector kernels
    (3000, 1, 700, N, N), (3000, 1, 701, N, T), (2048, 1, 1024, T, N), (1500, 1, 333, T, T),
    (1, 3000, 700, N, N), (1, 2048, 1024, N, T), (1, 1501, 333, T, N), (1, 4096, 96, T, T),
    (5000, 1, 8, N, N), (1, 300, 5000, N, N),
    # two to eight vectors against a matrix stored row by row along k (a small batch times W^T)
    (4, 5000, 704, N, T), (8, 4200, 333, N, T), (5000, 2, 701, N, T), (4500, 7, 96, N, T), (3, 4099, 64, N, T),
    # ... and against a matrix stored [k][n] (a small batch times W as numpy holds it), either side
    (4, 5000, 704, N, N), (8, 4200, 333, N, N), (2, 1027, 4096, N, N), (5000, 3, 701, T, N), (4100, 8, 96, T, N),
]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("case", GEMV_CASES, ids=[f"{c[0]}x{c[1]}x{c[2]}" + "nt"[c[3] == T] + "nt"[c[4] == T] for c in GEMV_CASES])
def test_gemm_with_one_column_or_one_row(rt, monkeypatch, dt, case):
    """The matrix-vector kernels behind the GEMM entry points: integer-valued operands give the oracle's integers
    (any summation order), random ones stay within the GEMM bars; the tiled kernels (DOCC_ROCM_GEMV_OFF) agree."""
    m, n, k, ta, tb = case
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    A = int_matrix(rng, (k, m) if ta == T else (m, k), dt, lim=4)
    B = int_matrix(rng, (n, k) if tb == T else (k, n), dt, lim=4)
    C0 = int_matrix(rng, (m, n), dt, lim=4)
    for alpha, beta in ((1.0, 0.0), (2.0, -1.0)):
        want = oracle.gemm(A, B, C0, alpha=alpha, beta=beta, trans_a=ta, trans_b=tb)
        assert np.array_equal(run_gemm(rt, A, B, C0, alpha, beta, ta=ta, tb=tb), want), (alpha, beta)
    # padded leading dimensions and unaligned operands take the scalar variants
    padded = run_gemm(rt, A, B, C0, 2.0, -1.0, ta=ta, tb=tb, lda=A.shape[1] + 3, ldb=B.shape[1] + 5, ldc=n + 2, offset=1)
    assert np.array_equal(padded, oracle.gemm(A, B, C0, alpha=2.0, beta=-1.0, trans_a=ta, trans_b=tb))
    Ar, Br = rng.standard_normal(A.shape).astype(dt), rng.standard_normal(B.shape).astype(dt)
    got = run_gemm(rt, Ar, Br, C0, 1.5, 0.5, ta=ta, tb=tb)
    ref = oracle.gemm(Ar, Br, C0, alpha=1.5, beta=0.5, trans_a=ta, trans_b=tb, variant="ld" if dt == np.float64 else "acc64")
    assert rel_err_max(got, ref) <= (1e-12 if dt == np.float64 else 1e-5)
    monkeypatch.setenv("DOCC_ROCM_GEMV_OFF", "1")
    tiled = run_gemm(rt, Ar, Br, C0, 1.5, 0.5, ta=ta, tb=tb)
    assert rel_err_max(tiled, ref) <= (1e-12 if dt == np.float64 else 1e-5)
