"""A batch of GEMMs in one launch (docc_rocm_{d,s}gemm_batched, docc_rocm_bf16gemm_f32_batched).

The bar is the loop it replaces: the reference expands ml::MatMul to one GEMM per batch entry
(sdfg/src/data_flow/library_nodes/math/tensor/matmul_node.cpp:366-499). Every entry is checked against
the CPU oracle at the GEMM tolerances (fp64 1e-12, fp32 1e-5, bf16 2e-2 on max|y - ref| / max|ref|),
and with the tile family pinned the batched launch must give the bits of the loop of single launches:
the batch index only moves the three base addresses."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu
N, T = oracle.NO_TRANS, oracle.TRANS
TOL = {"d": 1e-12, "s": 1e-5, "b": 2e-2}

# batch, m, n, k, ta, tb, B shared across the batch
CASES = [(1, 64, 64, 64, N, N, False), (3, 100, 130, 70, N, T, False), (5, 33, 17, 5, T, T, True), (8, 128, 256, 64, N, N, True),
         (4, 257, 129, 100, T, N, False), (16, 64, 64, 256, N, N, False), (2, 512, 512, 128, N, T, True), (7, 1, 9, 3, N, N, False),
         (3, 40, 50, 0, N, N, False), (0, 16, 16, 16, N, N, False)]


def operands(kind, batch, m, n, k, ta, tb, shared_b, seed):
    dt = np.float64 if kind == "d" else np.float32
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((max(batch, 1),) + ((k, m) if ta == T else (m, k))).astype(dt)
    B = rng.standard_normal((1 if shared_b else max(batch, 1),) + ((n, k) if tb == T else (k, n))).astype(dt)
    C0 = rng.standard_normal((max(batch, 1), m, n)).astype(dt)
    if kind == "b":
        a, b = dev(A).bfloat16().view(torch.int16), dev(B).bfloat16().view(torch.int16)
        A, B = host(a.view(torch.bfloat16).float()), host(b.view(torch.bfloat16).float())
    else:
        a, b = dev(A), dev(B)
    return dt, A, B, C0, a, b


@pytest.mark.parametrize("kind", ["d", "s", "b"])
@pytest.mark.parametrize("case", CASES, ids=[f"b{c[0]}_{c[1]}x{c[2]}x{c[3]}" + "nt"[c[4] == T] + "nt"[c[5] == T] + ("_sharedB" if c[6] else "") for c in CASES])
def test_batched_matches_oracle_and_the_loop(rt, kind, case, monkeypatch):
    batch, m, n, k, ta, tb, shared_b = case
    dt, A, B, C0, a, b = operands(kind, batch, m, n, k, ta, tb, shared_b, batch * 31 + m * 7 + n * 3 + k)
    lda, ldb = max(A.shape[2], 1), max(B.shape[2], 1)
    sa, sb, sc = A.shape[1] * A.shape[2], 0 if shared_b else B.shape[1] * B.shape[2], m * n
    esz = a.element_size()
    gemm = {"d": rt.dgemm, "s": rt.sgemm, "b": rt.bf16gemm_f32}[kind]
    for alpha, beta in ((1.0, 0.0), (1.5, -0.75)):
        for force in ("small", "big"):          # the same tile family for both forms
            monkeypatch.setenv("DOCC_ROCM_GEMM_TILE", force)
            c = dev(C0)
            rt.gemm_batched(kind, batch, m, n, k, alpha, a.data_ptr(), lda, sa, b.data_ptr(), ldb, sb, beta, c.data_ptr(), n, sc,
                            trans_a=ta, trans_b=tb)
            loop = dev(C0)
            for z in range(batch):
                gemm(m, n, k, alpha, a.data_ptr() + z * sa * esz, lda, b.data_ptr() + z * sb * esz, ldb, beta,
                     loop.data_ptr() + z * sc * loop.element_size(), n, trans_a=ta, trans_b=tb)
            torch.cuda.synchronize()
            got = host(c)
            assert np.array_equal(got, host(loop), equal_nan=True), (alpha, beta, force)
            if batch == 0:
                assert np.array_equal(got, C0)
        monkeypatch.delenv("DOCC_ROCM_GEMM_TILE")
        c = dev(C0)
        rt.gemm_batched(kind, batch, m, n, k, alpha, a.data_ptr(), lda, sa, b.data_ptr(), ldb, sb, beta, c.data_ptr(), n, sc,
                        trans_a=ta, trans_b=tb)
        torch.cuda.synchronize()
        got = host(c)
        for z in range(batch):
            Bz = B[0 if shared_b else z]
            ref = oracle.gemm(A[z], Bz, C0[z], alpha=alpha, beta=beta, trans_a=ta, trans_b=tb) if k else beta * C0[z]
            assert rel_err_max(got[z], ref) <= TOL[kind], (z, alpha, beta)


def test_batched_padded_strides_leave_the_gaps_alone(rt):
    """Leading dimensions and batch strides larger than the matrices: the padding of C keeps its values."""
    batch, m, n, k = 6, 96, 80, 48
    lda, ldb, ldc = k + 8, n + 4, n + 12
    sa, sb, sc = m * lda + 16, k * ldb + 8, m * ldc + 20
    rng = np.random.default_rng(5)
    A = rng.standard_normal(batch * sa).astype(np.float32)
    B = rng.standard_normal(batch * sb).astype(np.float32)
    C0 = rng.standard_normal(batch * sc).astype(np.float32)
    a, b, c = dev(A), dev(B), dev(C0)
    rt.gemm_batched("s", batch, m, n, k, 2.0, a.data_ptr(), lda, sa, b.data_ptr(), ldb, sb, 0.5, c.data_ptr(), ldc, sc)
    torch.cuda.synchronize()
    got = host(c)
    want = C0.copy()
    for z in range(batch):
        Az = A[z * sa:z * sa + m * lda].reshape(m, lda)[:, :k]
        Bz = B[z * sb:z * sb + k * ldb].reshape(k, ldb)[:, :n]
        Cz = C0[z * sc:z * sc + m * ldc].reshape(m, ldc)[:, :n]
        ref = oracle.gemm(np.ascontiguousarray(Az), np.ascontiguousarray(Bz), np.ascontiguousarray(Cz), alpha=2.0, beta=0.5)
        gz = got[z * sc:z * sc + m * ldc].reshape(m, ldc)
        assert rel_err_max(gz[:, :n], ref) <= 1e-5
        want[z * sc:z * sc + m * ldc].reshape(m, ldc)[:, :n] = gz[:, :n]
    assert np.array_equal(got, want)       # nothing outside the m x n windows was written


def test_batched_rejects_bad_arguments(rt):
    from docc_amd.runtime import RocmRuntimeError
    x = torch.zeros(4096, device="cuda")
    p = x.data_ptr()
    with pytest.raises(RocmRuntimeError, match="overlap"):
        rt.gemm_batched("s", 2, 16, 16, 16, 1.0, p, 16, 256, p, 16, 0, 0.0, p, 16, 100)
    with pytest.raises(RocmRuntimeError, match="negative"):
        rt.gemm_batched("s", -1, 16, 16, 16, 1.0, p, 16, 256, p, 16, 0, 0.0, p, 16, 256)
    with pytest.raises(RocmRuntimeError, match="negative batch stride"):
        rt.gemm_batched("s", 2, 16, 16, 16, 1.0, p, 16, -256, p, 16, 0, 0.0, p, 16, 256)


def test_batched_attention_scores_shape(rt):
    """[64 heads, 512, 64] x [64 heads, 64, 512]: the Q K^T of an attention layer, bf16 in, fp32 out."""
    heads, s, d = 64, 512, 64
    g = torch.Generator(device="cuda").manual_seed(11)
    q = torch.randn(heads, s, d, device="cuda", generator=g).bfloat16()
    kk = torch.randn(heads, s, d, device="cuda", generator=g).bfloat16()
    out = torch.empty(heads, s, s, device="cuda")
    rt.gemm_batched("b", heads, s, s, d, 0.125, q.data_ptr(), d, s * d, kk.data_ptr(), d, s * d, 0.0, out.data_ptr(), s, s * s,
                    trans_b=T)
    torch.cuda.synchronize()
    got = host(out)
    Q, K = host(q.float()), host(kk.float())
    for z in (0, 17, 63):
        ref = oracle.gemm(Q[z], K[z], None, alpha=0.125, beta=0.0, trans_b=T)
        assert rel_err_max(got[z], ref) <= 2e-2
