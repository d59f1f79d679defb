"""Products of a few rows (or columns) with a long K extent: K is cut into parts that run as one batched launch, and a
second launch adds the parts in order. Through the C-ABI against the oracle, bit for bit on integer-valued operands
(every product and partial sum is exact, so cutting K changes nothing), at the tolerance of the precision otherwise."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max
from test_gpu_gemm import int_matrix, run_gemm
from test_gpu_gemm_bf16 import run_bgemm

pytestmark = pytest.mark.gpu

N, T = oracle.NO_TRANS, oracle.TRANS
CASES = [(32, 512, 4096), (16, 1024, 2048), (130, 260, 8192), (64, 64, 16384), (9, 2000, 1024)]


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("ta,tb", [(N, N), (N, T), (T, N), (T, T)])
@pytest.mark.parametrize("m,n,k", CASES)
def test_gemm_with_k_in_parts_integer_exact(rt, dt, ta, tb, m, n, k):
    rng = np.random.default_rng(m + 7 * n + 13 * k)
    A = int_matrix(rng, (k, m) if ta == T else (m, k), dt, lim=4)
    B = int_matrix(rng, (n, k) if tb == T else (k, n), dt, lim=4)
    C0 = int_matrix(rng, (m, n), dt)
    C = run_gemm(rt, A, B, C=C0.copy(), alpha=2.0, beta=-3.0, ta=ta, tb=tb, ldc=n + 8)
    assert np.array_equal(C, oracle.gemm(A, B, C=C0.copy(), alpha=2.0, beta=-3.0, trans_a=ta, trans_b=tb))
    # beta == 0 must not read C
    C = run_gemm(rt, A, B, ta=ta, tb=tb)
    assert np.array_equal(C, oracle.gemm(A, B, trans_a=ta, trans_b=tb))


@pytest.mark.parametrize("splits", ["0", "2", "8", "64"])
def test_gemm_parts_forced_and_switched_off(rt, monkeypatch, splits):
    """Any number of parts gives the exact product of integer-valued operands, and random operands stay at the fp32 bar."""
    monkeypatch.setenv("DOCC_ROCM_GEMM_SPLITK", splits)
    rng = np.random.default_rng(int(splits))
    for dt, tol in ((np.float32, 1e-5), (np.float64, 1e-12)):
        A, B = int_matrix(rng, (48, 4096), dt), int_matrix(rng, (4096, 320), dt)
        assert np.array_equal(run_gemm(rt, A, B), oracle.gemm(A, B))
        A, B = rng.standard_normal((48, 4096)).astype(dt), rng.standard_normal((4096, 320)).astype(dt)
        assert rel_err_max(run_gemm(rt, A, B), A.astype(np.float64) @ B.astype(np.float64)) <= tol


@pytest.mark.parametrize("ta,tb", [(N, N), (N, T), (T, N), (T, T)])
@pytest.mark.parametrize("m,n,k", [(32, 512, 4096), (130, 260, 8192), (16, 4096, 4096)])
def test_bgemm_with_k_in_parts(rt, ta, tb, m, n, k):
    rng = np.random.default_rng(m + n + k)
    A = rng.integers(-4, 5, (k, m) if ta == T else (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (n, k) if tb == T else (k, n)).astype(np.float32)
    Ab, Bb = oracle.f32_to_bf16(A), oracle.f32_to_bf16(B)
    C0 = rng.integers(-8, 9, (m, n)).astype(np.float32)
    C = run_bgemm(rt, Ab, Bb, C=C0.copy(), alpha=0.5, beta=2.0, ta=ta, tb=tb)
    assert np.array_equal(C, oracle.gemm_bf16(Ab, Bb, C=C0.copy(), alpha=0.5, beta=2.0, trans_a=ta, trans_b=tb))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("m,n,k", [(512, 1568, 4608), (256, 4096, 4096)])
def test_gemm_parts_larger_than_the_streams_buffer(rt, dt, m, n, k):
    """More than 8 MiB of parts: they live in a block of the device block cache for the call. Integer-valued operands
    against numpy's product in float64 (exact on both sides)."""
    rng = np.random.default_rng(m + k)
    A, B = int_matrix(rng, (m, k), dt, lim=3), int_matrix(rng, (k, n), dt, lim=3)
    C0 = int_matrix(rng, (m, n), dt)
    expect = (A.astype(np.float64) @ B.astype(np.float64) - 2.0 * C0).astype(dt)
    for _ in range(2):      # the second call finds the block in the cache
        assert np.array_equal(run_gemm(rt, A, B, C=C0.copy(), alpha=1.0, beta=-2.0), expect)


def test_gemm_parts_on_two_streams_do_not_share_partial_results(rt):
    """The parts' products live in the stream's own buffer: the same shape on two streams at once."""
    rng = np.random.default_rng(3)
    A = [int_matrix(rng, (32, 4096), np.float32) for _ in range(2)]
    B = [int_matrix(rng, (4096, 1024), np.float32) for _ in range(2)]
    a, b = [dev(x) for x in A], [dev(x) for x in B]
    c = [torch.empty(32, 1024, device="cuda") for _ in range(2)]
    streams = [rt.stream_create() for _ in range(2)]
    torch.cuda.synchronize()
    for _ in range(20):
        for i in range(2):
            rt.sgemm(32, 1024, 4096, 1.0, a[i].data_ptr(), 4096, b[i].data_ptr(), 1024, 0.0, c[i].data_ptr(), 1024, stream=streams[i])
    for s in streams:
        rt.stream_sync(s)
    for i in range(2):
        assert np.array_equal(host(c[i]), oracle.gemm(A[i], B[i]))
    for s in streams:
        rt.stream_destroy(s)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("n", [2, 3, 5, 9, 17, 63])
def test_tall_matrix_times_a_few_columns_stored_by_rows(rt, dt, n):
    """A [m, k] times B [k, n] with a handful of columns: B's rows are too short for the kernels that read whole vectors,
    so B is transposed into a temporary first and the product runs against its rows. Exact on integer-valued operands,
    with alpha, beta and a padded C."""
    rng = np.random.default_rng(n)
    m, k = 1500, 512
    A, B = int_matrix(rng, (m, k), dt, lim=4), int_matrix(rng, (k, n), dt, lim=4)
    C0 = int_matrix(rng, (m, n), dt)
    C = run_gemm(rt, A, B, C=C0.copy(), alpha=-1.0, beta=2.0, ldc=n + 3)
    assert np.array_equal(C, oracle.gemm(A, B, C=C0.copy(), alpha=-1.0, beta=2.0))
    assert np.array_equal(run_gemm(rt, A, B), oracle.gemm(A, B))
