"""GEMM with bias and activation in its epilogue (docc_rocm_{d,s}gemm_epilogue, docc_rocm_bf16gemm_f32_epilogue).

The bar is the chain it replaces: the GEMM node, ml::Broadcast + ml::Add of the bias row and the unary
node, each a kernel of its own. The fused result must be the same bits (every step rounds as the
separate nodes do), and the chain itself is checked against the CPU oracle at the GEMM tolerances
(fp64 1e-12, fp32 1e-5, bf16 2e-2 on max|y - ref| / max|ref|)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu
N, T = oracle.NO_TRANS, oracle.TRANS

# m, n, k, ta, tb: aligned and ragged shapes, every tile family (small / large problems)
SHAPES = [(64, 64, 64, N, N), (100, 130, 70, N, T), (257, 129, 100, T, N), (33, 17, 5, T, T), (512, 384, 256, N, N),
          (1024, 1024, 128, N, T), (1, 300, 7, N, N), (40, 50, 0, N, N),
          # a small batch through a layer: the matrix-vector kernels, bias and activation as a pass over the few output rows
          (4, 5000, 704, N, T), (3000, 1, 700, N, N), (4, 4200, 333, N, N), (1, 4096, 512, N, T),
          # a dozen rows against a matrix of 8 M elements: the kernels that feed B straight into the MFMA, then the same pass
          (12, 4096, 2048, N, N), (12, 4096, 2048, N, T)]
ACTS = [None, "relu", "abs"]          # the activations built into the store


def chain_on_gpu(rt, kind, dt, m, n, k, alpha, a, b, beta, c0, bias, act, ta, tb, lda, ldb):
    """The unfused nodes: GEMM, then bias add and activation through the elementwise kernel."""
    c = c0.clone()
    gemm = {"d": rt.dgemm, "s": rt.sgemm, "b": rt.bf16gemm_f32}[kind]
    gemm(m, n, k, alpha, a.data_ptr(), lda, b.data_ptr(), ldb, beta, c.data_ptr(), n, trans_a=ta, trans_b=tb)
    if bias is not None or act is not None:
        rt.elementwise_fused(64 if dt == np.float64 else 32, (m, n), "add" if bias is not None else None, c.data_ptr(), (m, n),
                             bias.data_ptr() if bias is not None else 0, (n,) if bias is not None else None,
                             [act] if act else [], c.data_ptr())
    torch.cuda.synchronize()
    return host(c)


@pytest.mark.parametrize("kind", ["d", "s", "b"])
@pytest.mark.parametrize("shape", SHAPES, ids=["x".join(map(str, s[:3])) + ("t" if s[3] == T else "n") + ("t" if s[4] == T else "n") for s in SHAPES])
def test_epilogue_matches_the_separate_nodes(rt, kind, shape):
    m, n, k, ta, tb = shape
    dt = np.float64 if kind == "d" else np.float32
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    A = rng.standard_normal((k, m) if ta == T else (m, k)).astype(dt)
    B = rng.standard_normal((n, k) if tb == T else (k, n)).astype(dt)
    C0 = rng.standard_normal((m, n)).astype(dt)
    bias = rng.standard_normal(n).astype(dt)
    lda, ldb = max(A.shape[1], 1), max(B.shape[1], 1)
    if kind == "b":
        a, b = dev(A).bfloat16().view(torch.int16), dev(B).bfloat16().view(torch.int16)
        A, B = host(a.view(torch.bfloat16).float()), host(b.view(torch.bfloat16).float())
    else:
        a, b = dev(A), dev(B)
    c0, dbias = dev(C0), dev(bias)
    for alpha, beta in ((1.0, 0.0), (1.5, -0.75)):
        for act in ACTS:
            for with_bias in (True, False):
                if not with_bias and act is None:
                    continue
                c = c0.clone()
                rt.gemm_epilogue(kind, m, n, k, alpha, a.data_ptr(), lda, b.data_ptr(), ldb, beta, c.data_ptr(), n,
                                 dbias.data_ptr() if with_bias else None, act, trans_a=ta, trans_b=tb)
                torch.cuda.synchronize()
                want = chain_on_gpu(rt, kind, dt, m, n, k, alpha, a, b, beta, c0, dbias if with_bias else None, act, ta, tb, lda, ldb)
                assert np.array_equal(host(c), want, equal_nan=True), (alpha, beta, act, with_bias)
    # and the chain against the oracle, once per shape (relu, with bias, alpha/beta set)
    ref = oracle.gemm(A.astype(dt), B.astype(dt), C0, alpha=1.5, beta=-0.75, trans_a=ta, trans_b=tb) if k else -0.75 * C0
    ref = np.maximum(ref + bias[None, :], 0)
    c = c0.clone()
    rt.gemm_epilogue(kind, m, n, k, 1.5, a.data_ptr(), lda, b.data_ptr(), ldb, -0.75, c.data_ptr(), n, dbias.data_ptr(), "relu", trans_a=ta, trans_b=tb)
    torch.cuda.synchronize()
    assert rel_err_max(host(c), ref) <= {"d": 1e-12, "s": 1e-5, "b": 2e-2}[kind]


def test_epilogue_on_the_benchmark_shapes_and_padded_c(rt):
    """4096^3 fp32 (the wide asynchronous tile) and a C with a padded leading dimension."""
    n = 4096
    g = torch.Generator(device="cuda").manual_seed(3)
    a, b = torch.randn(n, n, device="cuda", generator=g) / 64, torch.randn(n, n, device="cuda", generator=g) / 64
    bias = torch.randn(n, device="cuda", generator=g)
    c = torch.empty(n, n, device="cuda")
    rt.gemm_epilogue("s", n, n, n, 1.0, a.data_ptr(), n, b.data_ptr(), n, 0.0, c.data_ptr(), n, bias.data_ptr(), "relu")
    plain = torch.empty(n, n, device="cuda")
    rt.sgemm(n, n, n, 1.0, a.data_ptr(), n, b.data_ptr(), n, 0.0, plain.data_ptr(), n)
    torch.cuda.synchronize()
    assert torch.equal(c, torch.relu(plain + bias))
    # ldc > n: only the n leading columns of each row are written
    m, k, ldc = 70, 50, 96
    a2, b2 = torch.randn(m, k, device="cuda", dtype=torch.float64), torch.randn(k, 64, device="cuda", dtype=torch.float64)
    bias2 = torch.randn(64, device="cuda", dtype=torch.float64)
    c2 = torch.full((m, ldc), float("nan"), device="cuda", dtype=torch.float64)
    rt.gemm_epilogue("d", m, 64, k, 1.0, a2.data_ptr(), k, b2.data_ptr(), 64, 0.0, c2.data_ptr(), ldc, bias2.data_ptr(), "abs")
    torch.cuda.synchronize()
    assert torch.isnan(c2[:, 64:]).all()
    ref = np.abs(oracle.gemm(host(a2), host(b2)) + host(bias2)[None, :])
    assert rel_err_max(host(c2[:, :64]), ref) <= 1e-12
    from docc_amd.runtime import RocmRuntimeError
    with pytest.raises(RocmRuntimeError):
        rt.gemm_epilogue("d", m, 64, k, 1.0, a2.data_ptr(), k, b2.data_ptr(), 64, 0.0, c2.data_ptr(), ldc, bias2.data_ptr(), 42)
    with pytest.raises(RocmRuntimeError, match="only ReLU and Abs"):       # the transcendental ones stay elementwise kernels
        rt.gemm_epilogue("d", m, 64, k, 1.0, a2.data_ptr(), k, b2.data_ptr(), 64, 0.0, c2.data_ptr(), ldc, bias2.data_ptr(), "tanh")
    with pytest.raises(RocmRuntimeError):       # an empty product with an epilogue goes through the elementwise kernel: contiguous C only
        rt.gemm_epilogue("d", m, 64, 0, 1.0, a2.data_ptr(), k, b2.data_ptr(), 64, 0.0, c2.data_ptr(), ldc, bias2.data_ptr(), "relu")


@pytest.mark.parametrize("k", [264, 320])
def test_bf16_epilogue_on_the_large_tile(rt, k):
    """A product large enough for the 256x256 tile, with a K tail (the 32x32x16 kernel that deals its copies over the
    K-step) and with K a multiple of 64 (the 16x16x32 kernel): bias and ReLU in the store give the bits of the separate nodes."""
    m, n = 4096, 3072
    g = torch.Generator(device="cuda").manual_seed(5)
    a = (torch.randn(m, k, device="cuda", generator=g) / 8).bfloat16()
    b = (torch.randn(k, n, device="cuda", generator=g) / 8).bfloat16()
    bias = torch.randn(n, device="cuda", generator=g)
    c0 = torch.randn(m, n, device="cuda", generator=g)
    fused = c0.clone()
    rt.gemm_epilogue("b", m, n, k, 1.5, a.data_ptr(), k, b.data_ptr(), n, -0.75, fused.data_ptr(), n, bias.data_ptr(), "relu")
    plain = c0.clone()
    rt.bf16gemm_f32(m, n, k, 1.5, a.data_ptr(), k, b.data_ptr(), n, -0.75, plain.data_ptr(), n)
    torch.cuda.synchronize()
    assert torch.equal(fused, torch.relu(plain + bias))
    ref = 1.5 * (a[:64].double() @ b.double()) - 0.75 * c0[:64].double()
    assert ((plain[:64].double() - ref).abs().max() / ref.abs().max()).item() <= 1e-5
