"""Five to 32 rows of fp32 against a wide matrix: the kernels that feed B from global memory straight into the MFMA (16 rows per
instruction up to m = 16, 32 above; B stored [k][n], and [n][k] up to 16 rows), and 3 to 32 rows of bf16 against a matrix stored
[n][k]. Through the C-ABI against the oracle, bit for bit on integer-valued operands (every product and partial sum is exact, so neither the cut of K into parts nor the order of the
wavefronts' sums changes anything), at the fp32 bar against a float64 product otherwise."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max
from test_gpu_gemm import int_matrix, run_gemm
from test_gpu_gemm_bf16 import run_bgemm

pytestmark = pytest.mark.gpu

N, T = oracle.NO_TRANS, oracle.TRANS


@pytest.fixture(autouse=True)
def skinny_for_small_matrices_too(monkeypatch):
    """By itself the launcher takes these kernels from 8 M elements of B; the tests' matrices are smaller."""
    monkeypatch.setenv("DOCC_ROCM_GEMM_SKINNY", "1")


# n off the 128 columns of a work-group, k off the chunk and off the parts, one work-group, many
SHAPES = [(16, 1024, 1024), (9, 1000, 2052), (5, 516, 512), (32, 2048, 1040), (17, 640, 4100), (12, 4096, 4096), (31, 1284, 8192)]


@pytest.mark.parametrize("tb", [N, T])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_skinny_integer_exact(rt, m, n, k, tb):
    rng = np.random.default_rng(m + 3 * n + 5 * k)
    A = int_matrix(rng, (m, k), np.float32, lim=4)
    B = int_matrix(rng, (n, k) if tb == T else (k, n), np.float32, lim=4)
    C0 = int_matrix(rng, (m, n), np.float32)
    C = run_gemm(rt, A, B, C=C0.copy(), alpha=2.0, beta=-3.0, tb=tb, ldc=n + 8)
    assert np.array_equal(C, oracle.gemm(A, B, C=C0.copy(), alpha=2.0, beta=-3.0, trans_b=tb))
    # beta == 0 must not read C (run_gemm fills it with NaN)
    assert np.array_equal(run_gemm(rt, A, B, tb=tb), oracle.gemm(A, B, trans_b=tb))


@pytest.mark.parametrize("parts", ["1", "3", "8", "64"])
@pytest.mark.parametrize("tb", [N, T])
@pytest.mark.parametrize("m", [7, 16, 29])
def test_skinny_any_number_of_parts(rt, monkeypatch, parts, tb, m):
    """One part stores alpha * sum + beta * C itself, several go through the buffer of partial products; a C whose rows are
    not 16-byte aligned takes the second way with one part too."""
    monkeypatch.setenv("DOCC_ROCM_GEMM_SPLITK", parts)
    n, k = 1152, 3072
    rng = np.random.default_rng(m + int(parts))
    A = int_matrix(rng, (m, k), np.float32, lim=4)
    B = int_matrix(rng, (n, k) if tb == T else (k, n), np.float32, lim=4)
    C0 = int_matrix(rng, (m, n), np.float32)
    expect = oracle.gemm(A, B, C=C0.copy(), alpha=-1.0, beta=2.0, trans_b=tb)
    for ldc in (n, n + 4, n + 3):
        assert np.array_equal(run_gemm(rt, A, B, C=C0.copy(), alpha=-1.0, beta=2.0, tb=tb, ldc=ldc), expect), ldc
    assert np.array_equal(run_gemm(rt, A, B, tb=tb), oracle.gemm(A, B, trans_b=tb))


@pytest.mark.parametrize("tb", [N, T])
@pytest.mark.parametrize("m,n,k", [(16, 4096, 4096), (32, 1024, 8192), (10, 11008, 2048)])
def test_skinny_random_operands(rt, monkeypatch, m, n, k, tb):
    rng = np.random.default_rng(n + k)
    A = rng.standard_normal((m, k)).astype(np.float32)
    B = rng.standard_normal((n, k) if tb == T else (k, n)).astype(np.float32)
    ref = A.astype(np.float64) @ (B.astype(np.float64).T if tb == T else B.astype(np.float64))
    got = run_gemm(rt, A, B, tb=tb)
    assert rel_err_max(got, ref) <= 1e-5
    # the kernels of the tiles give the same product to rounding
    monkeypatch.setenv("DOCC_ROCM_GEMM_SKINNY", "0")
    assert rel_err_max(run_gemm(rt, A, B, tb=tb), got.astype(np.float64)) <= 2e-5


def test_skinny_parts_larger_than_the_streams_buffer(rt, monkeypatch):
    """16 MiB of parts: a block of the device block cache for the call; the second call finds it there."""
    monkeypatch.setenv("DOCC_ROCM_GEMM_SPLITK", "8")
    m, n, k = 32, 16384, 4096
    rng = np.random.default_rng(11)
    A, B = int_matrix(rng, (m, k), np.float32, lim=3), int_matrix(rng, (k, n), np.float32, lim=3)
    expect = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    for _ in range(2):
        assert np.array_equal(run_gemm(rt, A, B), expect)


def test_skinny_is_deterministic_and_keeps_special_values(rt, monkeypatch):
    """Parts are added in order: the same bits on every call. A NaN or an infinity in B reaches exactly its column. On a matrix
    the launcher takes these kernels for by itself."""
    monkeypatch.delenv("DOCC_ROCM_GEMM_SKINNY")
    m, n, k = 16, 2048, 4096
    rng = np.random.default_rng(5)
    A = np.abs(rng.standard_normal((m, k))).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    B[100, 7] = np.nan
    B[4000, 1999] = np.inf
    first = run_gemm(rt, A, B)
    for _ in range(3):
        assert np.array_equal(run_gemm(rt, A, B), first, equal_nan=True)
    assert np.isnan(first[:, 7]).all() and np.isposinf(first[:, 1999]).all()
    rest = np.delete(first, [7, 1999], axis=1)
    assert np.isfinite(rest).all()


def test_skinny_on_two_streams(rt):
    """The parts' products live in the stream's own buffer: the same shape on two streams at once."""
    rng = np.random.default_rng(3)
    A = [int_matrix(rng, (16, 4096), np.float32) for _ in range(2)]
    B = [int_matrix(rng, (4096, 2048), np.float32) for _ in range(2)]
    a, b = [dev(x) for x in A], [dev(x) for x in B]
    c = [torch.empty(16, 2048, device="cuda") for _ in range(2)]
    streams = [rt.stream_create() for _ in range(2)]
    torch.cuda.synchronize()
    for _ in range(20):
        for i in range(2):
            rt.sgemm(16, 2048, 4096, 1.0, a[i].data_ptr(), 4096, b[i].data_ptr(), 2048, 0.0, c[i].data_ptr(), 2048, stream=streams[i])
    for st in streams:
        rt.stream_sync(st)
    for i in range(2):
        assert np.array_equal(host(c[i]), oracle.gemm(A[i], B[i]))
    for st in streams:
        rt.stream_destroy(st)


BF16_SHAPES = [(16, 1024, 1024), (9, 1000, 2056), (3, 520, 512), (32, 2048, 1032), (17, 640, 4104), (12, 4096, 4096), (31, 1288, 8192)]


@pytest.mark.parametrize("m,n,k", BF16_SHAPES)
def test_skinny_bf16_integer_exact(rt, m, n, k):
    rng = np.random.default_rng(m + 3 * n + 5 * k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (n, k)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    C0 = rng.integers(-8, 9, (m, n)).astype(np.float32)
    C = run_bgemm(rt, Ab, Bb, C=C0.copy(), alpha=0.5, beta=2.0, tb=T)
    assert np.array_equal(C, oracle.gemm_bf16(Ab, Bb, C=C0.copy(), alpha=0.5, beta=2.0, trans_b=T))
    # beta == 0 must not read C (run_bgemm fills it with NaN)
    assert np.array_equal(run_bgemm(rt, Ab, Bb, tb=T), A @ B.T)


@pytest.mark.parametrize("parts", ["1", "3", "8", "64"])
@pytest.mark.parametrize("m", [4, 16, 29])
def test_skinny_bf16_any_number_of_parts(rt, monkeypatch, parts, m):
    monkeypatch.setenv("DOCC_ROCM_GEMM_SPLITK", parts)
    n, k = 1160, 3072
    rng = np.random.default_rng(m + int(parts))
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (n, k)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    C0 = rng.integers(-8, 9, (m, n)).astype(np.float32)
    assert np.array_equal(run_bgemm(rt, Ab, Bb, C=C0.copy(), alpha=-1.0, beta=2.0, tb=T), -(A @ B.T) + 2.0 * C0)
    assert np.array_equal(run_bgemm(rt, Ab, Bb, tb=T), A @ B.T)


@pytest.mark.parametrize("m,n,k", [(16, 4096, 4096), (32, 1024, 8192), (5, 11008, 2048)])
def test_skinny_bf16_random_operands(rt, monkeypatch, m, n, k):
    """bf16 products are exact in fp32; the sums differ from the oracle's by their order only."""
    rng = np.random.default_rng(n + k)
    Ab = oracle.f32_to_bf16(rng.standard_normal((m, k)).astype(np.float32))
    Bb = oracle.f32_to_bf16(rng.standard_normal((n, k)).astype(np.float32))
    ref = oracle.bf16_to_f32(Ab).astype(np.float64) @ oracle.bf16_to_f32(Bb).astype(np.float64).T
    got = run_bgemm(rt, Ab, Bb, tb=T)
    assert rel_err_max(got, ref) <= 1e-5
    for _ in range(2):
        assert np.array_equal(run_bgemm(rt, Ab, Bb, tb=T), got)     # parts are added in order
    monkeypatch.setenv("DOCC_ROCM_GEMM_SKINNY", "0")
    assert rel_err_max(run_bgemm(rt, Ab, Bb, tb=T), got.astype(np.float64)) <= 2e-5


F64_SHAPES = [(16, 1024, 1024), (9, 1000, 2052), (5, 514, 512), (12, 4096, 4096), (13, 1286, 4098)]


@pytest.mark.parametrize("m,n,k", F64_SHAPES)
def test_skinny_f64_integer_exact(rt, m, n, k):
    """fp64, B stored [k][n], 5 to 16 rows: the same scheme on the fp64 MFMA."""
    rng = np.random.default_rng(m + 3 * n + 5 * k)
    A, B = int_matrix(rng, (m, k), np.float64, lim=4), int_matrix(rng, (k, n), np.float64, lim=4)
    C0 = int_matrix(rng, (m, n), np.float64)
    C = run_gemm(rt, A, B, C=C0.copy(), alpha=2.0, beta=-3.0, ldc=n + 6)
    assert np.array_equal(C, oracle.gemm(A, B, C=C0.copy(), alpha=2.0, beta=-3.0))
    assert np.array_equal(run_gemm(rt, A, B), oracle.gemm(A, B))      # beta == 0 must not read C


@pytest.mark.parametrize("parts", ["1", "3", "8", "64"])
@pytest.mark.parametrize("m", [7, 16])
def test_skinny_f64_any_number_of_parts_and_random_operands(rt, monkeypatch, parts, m):
    monkeypatch.setenv("DOCC_ROCM_GEMM_SPLITK", parts)
    n, k = 1154, 3072
    rng = np.random.default_rng(m + int(parts))
    A, B = int_matrix(rng, (m, k), np.float64, lim=4), int_matrix(rng, (k, n), np.float64, lim=4)
    C0 = int_matrix(rng, (m, n), np.float64)
    expect = oracle.gemm(A, B, C=C0.copy(), alpha=-1.0, beta=2.0)
    for ldc in (n, n + 2, n + 1):           # the last: rows of C off the 16-byte boundary, no direct store
        assert np.array_equal(run_gemm(rt, A, B, C=C0.copy(), alpha=-1.0, beta=2.0, ldc=ldc), expect), ldc
    A, B = rng.standard_normal((m, k)), rng.standard_normal((k, n))
    got = run_gemm(rt, A, B)
    assert rel_err_max(got, A @ B) <= 1e-12
    monkeypatch.setenv("DOCC_ROCM_GEMM_SKINNY", "0")
    assert rel_err_max(run_gemm(rt, A, B), got) <= 1e-12
