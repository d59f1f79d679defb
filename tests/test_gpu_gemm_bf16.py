"""bf16 x bf16 -> fp32 GEMM (the precision the rocm target adds to the GEMM
node) against the CPU oracle, through docc_rocm_bf16gemm_f32.

Bars: bit-exact on integer-valued inputs; 1e-5 norm-wise against the oracle's
fp32 accumulation on the same bf16 values; 2e-2 norm-wise against an fp32 GEMM
on the unrounded inputs."""
import os

import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu
N, T = oracle.NO_TRANS, oracle.TRANS


def run_bgemm(rt, A_bits, B_bits, C=None, alpha=1.0, beta=0.0, ta=N, tb=N):
    m, k = (A_bits.shape[1], A_bits.shape[0]) if ta == T else A_bits.shape
    n = B_bits.shape[0] if tb == T else B_bits.shape[1]
    a, b = dev(A_bits), dev(B_bits)
    c = dev(np.full((m, n), np.nan, np.float32) if C is None else C.astype(np.float32))
    rt.bf16gemm_f32(m, n, k, alpha, a.data_ptr(), max(A_bits.shape[1], 1), b.data_ptr(), max(B_bits.shape[1], 1),
                    beta, c.data_ptr(), max(n, 1), trans_a=ta, trans_b=tb)
    torch.cuda.synchronize()
    return host(c)


@pytest.fixture(params=["small", "big"])
def tile(request):
    os.environ["DOCC_ROCM_GEMM_TILE"] = request.param
    yield request.param
    os.environ.pop("DOCC_ROCM_GEMM_TILE", None)


@pytest.mark.parametrize("ta,tb", [(N, N), (N, T), (T, N), (T, T)])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (17, 33, 65), (128, 128, 64), (130, 70, 200), (257, 300, 72), (64, 520, 1024)])
def test_bgemm_integer_exact(rt, tile, ta, tb, m, n, k):
    rng = np.random.default_rng(m + 31 * n + 977 * k)
    A = rng.integers(-8, 9, (k, m) if ta == T else (m, k)).astype(np.float32)
    B = rng.integers(-8, 9, (n, k) if tb == T else (k, n)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    C = run_bgemm(rt, Ab, Bb, ta=ta, tb=tb)
    ref = oracle.gemm_bf16(Ab, Bb, trans_a=ta, trans_b=tb)
    assert np.array_equal(C, ref)
    opA = A.T if ta == T else A
    opB = B.T if tb == T else B
    assert np.array_equal(C, opA @ opB)


def test_bgemm_alpha_beta_and_unaligned(rt, tile):
    rng = np.random.default_rng(3)
    m, n, k = 70, 45, 33  # k and n odd: rows are not 16-byte aligned -> unaligned kernels
    A, B = rng.integers(-8, 9, (m, k)).astype(np.float32), rng.integers(-8, 9, (k, n)).astype(np.float32)
    C0 = rng.integers(-8, 9, (m, n)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    out = run_bgemm(rt, Ab, Bb, C0, alpha=2.0, beta=-3.0)
    assert np.array_equal(out, oracle.gemm_bf16(Ab, Bb, C0, alpha=2.0, beta=-3.0))
    out = run_bgemm(rt, Ab, Bb)  # beta == 0 with NaN-filled C
    assert np.isfinite(out).all()


def test_bgemm_random_vs_oracle(rt, tile):
    rng = np.random.default_rng(2)
    m, n, k = 384, 320, 1024
    A = (rng.standard_normal((m, k)) / np.sqrt(k)).astype(np.float32)
    B = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    C = run_bgemm(rt, Ab, Bb)
    assert rel_err_max(C, oracle.gemm_bf16(Ab, Bb)) <= 1e-5
    assert rel_err_max(C, oracle.gemm(A, B, variant="acc64")) <= 2e-2


def test_bgemm_config_4096(rt):
    # benchmark configuration 3b: the 3a values rounded to bf16 (RNE), fp32 accumulate/output
    rng = np.random.default_rng(2)
    K = 4096
    A = (rng.standard_normal((K, K)) / 64).astype(np.float32)
    B = (rng.standard_normal((K, K)) / 64).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    C = run_bgemm(rt, Ab, Bb)
    assert np.isfinite(C).all()
    rows = np.r_[0:16, 2040:2056, 4080:4096]
    assert rel_err_max(C[rows], oracle.gemm_bf16(Ab[rows], Bb)) <= 1e-5
    assert rel_err_max(C[rows], oracle.gemm(A[rows], B, variant="acc64")) <= 2e-2
    # full-size property: C x == A (B x) in fp64 on the bf16 values
    x = rng.standard_normal(K)
    Af, Bf = oracle.bf16_to_f32(Ab).astype(np.float64), oracle.bf16_to_f32(Bb).astype(np.float64)
    lhs, rhs = C.astype(np.float64) @ x, Af @ (Bf @ x)
    assert np.abs(lhs - rhs).max() / np.abs(rhs).max() <= 1e-5


def test_device_bf16_conversion_matches_oracle(rt):
    rng = np.random.default_rng(9)
    x = np.concatenate([rng.standard_normal(5000).astype(np.float32) * 100,
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875, 3.3895314e38], np.float32)])
    src = dev(x)
    dst = torch.empty(x.size, dtype=torch.int16, device="cuda")
    rt.convert_f32_to_bf16(x.size, src.data_ptr(), dst.data_ptr())
    back = torch.empty(x.size, dtype=torch.float32, device="cuda")
    rt.convert_bf16_to_f32(x.size, dst.data_ptr(), back.data_ptr())
    torch.cuda.synchronize()
    bits = host(dst, np.uint16)
    assert np.array_equal(bits, oracle.f32_to_bf16(x))
    assert np.array_equal(host(back), oracle.bf16_to_f32(bits))


# every built tile configuration (DOCC_ROCM_GEMM_CFG = BMxBNxBKxWAVES[xSTAGES[p|q]]; a stage count picks the
# asynchronous kernel, q the one on the 16x16x32 MFMA, which here falls back for want of a K that suits it), ragged
# edges, a K tail, all transposes
BF16_CFGS = ["128x128x64x4", "256x256x64x4", "128x128x64x4x3", "128x128x64x4x4", "128x128x32x4x4", "128x256x64x4x3",
             "256x256x64x4x2", "256x256x32x4x4", "256x256x32x4x4p", "256x256x32x4x4q"]


@pytest.mark.parametrize("cfg", BF16_CFGS)
def test_bgemm_every_tile_configuration(rt, cfg):
    rng = np.random.default_rng(sum(cfg.encode()))
    os.environ["DOCC_ROCM_GEMM_CFG"] = cfg
    try:
        for (m, n, k) in [(304, 264, 200), (136, 520, 72), (8, 16, 1000)]:
            for ta in (N, T):
                for tb in (N, T):
                    A = rng.integers(-4, 5, (k, m) if ta == T else (m, k)).astype(np.float32)
                    B = rng.integers(-4, 5, (n, k) if tb == T else (k, n)).astype(np.float32)
                    C0 = rng.integers(-4, 5, (m, n)).astype(np.float32)
                    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
                    out = run_bgemm(rt, Ab, Bb, C0, alpha=2.0, beta=-1.0, ta=ta, tb=tb)
                    ref = oracle.gemm_bf16(Ab, Bb, C0, alpha=2.0, beta=-1.0, trans_a=ta, trans_b=tb)
                    assert np.array_equal(out, ref), (cfg, m, n, k, ta, tb)
    finally:
        os.environ.pop("DOCC_ROCM_GEMM_CFG", None)


@pytest.mark.parametrize("ta,tb", [(N, N), (N, T), (T, N), (T, T)])
def test_bgemm_on_the_16x16x32_mfma(rt, ta, tb):
    """The kernel the 4096^3 configuration runs on (K a multiple of 64, four K-steps or more): exact on small integers
    for ragged m and n, the shortest K it takes, an odd number of step pairs, alpha and beta; and N(0,1) operands
    against the oracle. The same entry point on a K it does not take gives the same bits through the other kernel."""
    rng = np.random.default_rng(16 + ta + 3 * tb)
    os.environ["DOCC_ROCM_GEMM_CFG"] = "256x256x32x4x4q"
    try:
        for (m, n, k) in [(304, 264, 192), (136, 520, 128), (8, 16, 1024), (512, 256, 320), (257, 511, 448)]:
            A = rng.integers(-4, 5, (k, m) if ta == T else (m, k)).astype(np.float32)
            B = rng.integers(-4, 5, (n, k) if tb == T else (k, n)).astype(np.float32)
            C0 = rng.integers(-4, 5, (m, n)).astype(np.float32)
            Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
            out = run_bgemm(rt, Ab, Bb, C0, alpha=2.0, beta=-1.0, ta=ta, tb=tb)
            assert np.array_equal(out, oracle.gemm_bf16(Ab, Bb, C0, alpha=2.0, beta=-1.0, trans_a=ta, trans_b=tb)), (m, n, k)
            out = run_bgemm(rt, Ab, Bb, ta=ta, tb=tb)              # beta == 0 over a C full of NaN
            assert np.array_equal(out, oracle.gemm_bf16(Ab, Bb, trans_a=ta, trans_b=tb)), (m, n, k)
        m, n, k = 384, 320, 1024
        A = (rng.standard_normal((k, m) if ta == T else (m, k)) / np.sqrt(k)).astype(np.float32)
        B = (rng.standard_normal((n, k) if tb == T else (k, n)) / np.sqrt(k)).astype(np.float32)
        Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
        C = run_bgemm(rt, Ab, Bb, ta=ta, tb=tb)
        assert rel_err_max(C, oracle.gemm_bf16(Ab, Bb, trans_a=ta, trans_b=tb)) <= 1e-5
        # the two MFMA forms add the same products in the same order of k-groups: the other kernel gives the same bits
        os.environ["DOCC_ROCM_GEMM_CFG"] = "256x256x32x4x4p"
        assert np.array_equal(C, run_bgemm(rt, Ab, Bb, ta=ta, tb=tb))
    finally:
        os.environ.pop("DOCC_ROCM_GEMM_CFG", None)


BGEMV_CASES = [(3000, 1, 704, N, N), (3000, 1, 701, N, T), (2048, 1, 1024, T, N), (1504, 1, 333, T, T),
               (1, 3000, 700, N, N), (1, 2048, 1024, N, T), (1, 1501, 333, T, N), (1, 4096, 96, T, T),
               (4, 5000, 704, N, T), (3, 4200, 333, N, T), (5000, 2, 701, N, T), (4500, 4, 96, N, T),
               (8, 5000, 704, N, T), (4500, 6, 333, N, T), (4, 5000, 704, N, N), (3, 4201, 333, N, N), (5000, 2, 701, T, N), (4104, 4, 96, T, N)]


@pytest.mark.parametrize("case", BGEMV_CASES, ids=[f"{c[0]}x{c[1]}x{c[2]}" + "nt"[c[3] == T] + "nt"[c[4] == T] for c in BGEMV_CASES])
def test_bgemm_with_one_column_or_one_row(rt, monkeypatch, case):
    """bf16 products with one output column or row take the matrix-vector kernels (a decoder's x W): integer
    values give the oracle's integers, random ones stay within the bf16 bar, the tiled kernels agree."""
    m, n, k, ta, tb = case
    rng = np.random.default_rng(m + 31 * n + 977 * k)
    A = rng.integers(-8, 9, (k, m) if ta == T else (m, k)).astype(np.float32)
    B = rng.integers(-8, 9, (n, k) if tb == T else (k, n)).astype(np.float32)
    C0 = rng.integers(-8, 9, (m, n)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    for alpha, beta in ((1.0, 0.0), (2.0, -1.0)):
        got = run_bgemm(rt, Ab, Bb, C0, alpha, beta, ta=ta, tb=tb)
        assert np.array_equal(got, oracle.gemm_bf16(Ab, Bb, C0, alpha=alpha, beta=beta, trans_a=ta, trans_b=tb)), (alpha, beta)
    Ar, Br = oracle.f32_to_bf16(rng.standard_normal(A.shape).astype(np.float32)), oracle.f32_to_bf16(rng.standard_normal(B.shape).astype(np.float32))
    ref = oracle.gemm_bf16(Ar, Br, trans_a=ta, trans_b=tb)
    assert rel_err_max(run_bgemm(rt, Ar, Br, ta=ta, tb=tb), ref) <= 1e-5      # fp32 sums of exact products: far inside 2e-2
    monkeypatch.setenv("DOCC_ROCM_GEMV_OFF", "1")
    assert rel_err_max(run_bgemm(rt, Ar, Br, ta=ta, tb=tb), ref) <= 1e-5
