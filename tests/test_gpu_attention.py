"""ml::Attention (bf16 in, fp32 softmax/accumulate) on the GPU against the CPU
oracle, through docc_rocm_attention_bf16. Tolerance 2e-2 norm-wise against the
oracle's fp32 evaluation of softmax(scale * Q K^T) V on the same bf16 inputs
(the kernel additionally rounds the probabilities to bf16 for the second
product)."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu
TOL_BF16 = 2e-2


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def run_attention(rt, Qb, Kb, Vb, scale=None, out_bf16=False):
    B, H, SQ, D = Qb.shape
    SKV = Kb.shape[2]
    scale = scale if scale is not None else 1.0 / np.sqrt(D)
    q, k, v = dev(Qb), dev(Kb), dev(Vb)
    o = torch.full((B, H, SQ, D), float("nan"), device="cuda", dtype=torch.bfloat16 if out_bf16 else torch.float32)
    rt.attention_bf16(B, H, SQ, SKV, D, scale, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), out_bf16=out_bf16)
    torch.cuda.synchronize()
    return o.float().cpu().numpy()


@pytest.mark.parametrize("B,H,SQ,SKV", [(1, 2, 96, 96), (1, 1, 1, 1), (2, 3, 128, 64), (1, 2, 130, 200), (1, 1, 33, 65),
                                        (2, 2, 256, 512), (1, 1, 7, 1000)])
@pytest.mark.parametrize("out_bf16", [False, True])
def test_attention_matches_oracle(rt, B, H, SQ, SKV, out_bf16):
    g = torch.Generator().manual_seed(B * 7 + H * 5 + SQ * 3 + SKV)
    Q, K, V = (torch.randn(B, H, s, 64, generator=g).bfloat16() for s in (SQ, SKV, SKV))
    O = run_attention(rt, bits(Q), bits(K), bits(V), out_bf16=out_bf16)
    ref = oracle.attention(bits(Q), bits(K), bits(V))
    assert np.isfinite(O).all()
    assert rel_err_max(O, ref) <= TOL_BF16


def test_attention_closed_forms(rt):
    g = torch.Generator().manual_seed(0)
    Q = torch.randn(1, 2, 70, 64, generator=g).bfloat16()
    V = torch.randn(1, 2, 150, 64, generator=g).bfloat16()
    # all keys equal -> uniform weights -> output = mean of V over the keys
    K = torch.randn(1, 2, 1, 64, generator=g).bfloat16().expand(1, 2, 150, 64).contiguous()
    O = run_attention(rt, bits(Q), bits(K), bits(V))
    mean = V.float().mean(dim=2, keepdim=True).numpy()
    assert rel_err_max(O, np.broadcast_to(mean, O.shape)) <= TOL_BF16
    # permuting the keys (and values alike) does not change the result beyond rounding
    K = torch.randn(1, 2, 150, 64, generator=g).bfloat16()
    perm = torch.randperm(150, generator=g)
    a = run_attention(rt, bits(Q), bits(K), bits(V))
    b = run_attention(rt, bits(Q), bits(K[:, :, perm]), bits(V[:, :, perm]))
    assert rel_err_max(a, b) <= TOL_BF16
    # one dominant key -> the output is that key's value row (exactly: p = 1 and 0 elsewhere)
    Kd = torch.zeros(1, 1, 64, 64).bfloat16()
    Qd = torch.zeros(1, 1, 32, 64).bfloat16()
    Qd[..., 0] = 64.0
    Kd[0, 0, 17, 0] = 64.0   # score 4096 * 0.125 = 512 for key 17, 0 for the others
    Vd = torch.randn(1, 1, 64, 64, generator=g).bfloat16()
    O = run_attention(rt, bits(Qd), bits(Kd), bits(Vd))
    assert np.array_equal(O[0, 0], np.broadcast_to(Vd[0, 0, 17].float().numpy(), (32, 64)))


def test_attention_errors(rt):
    from docc_amd.runtime import RocmRuntimeError
    t = torch.zeros(64 * 64, dtype=torch.bfloat16, device="cuda")
    p = t.data_ptr()
    with pytest.raises(RocmRuntimeError):
        rt.attention_bf16(1, 1, 8, 8, 128, 0.1, p, p, p, p)   # head dim not built
    with pytest.raises(RocmRuntimeError):
        rt.attention_bf16(1, 1, 8, 0, 64, 0.1, p, p, p, p)    # empty key axis
    rt.attention_bf16(0, 1, 8, 8, 64, 0.1, 0, 0, 0, 0)         # empty batch: no-op


def test_attention_config_b8_h16_s2048(rt):
    # benchmark configuration 4: B=8, H=16, S=2048, D=64, seed 3, scale 1/8
    torch.manual_seed(3)
    Q, K, V = (torch.randn(8, 16, 2048, 64).bfloat16() for _ in range(3))
    O = run_attention(rt, bits(Q), bits(K), bits(V), out_bf16=True)
    assert np.isfinite(O).all()
    # oracle on three (batch, head) pairs, a band of queries each
    for (b, h) in [(0, 0), (3, 7), (7, 15)]:
        ref = oracle.attention(bits(Q[b:b + 1, h:h + 1, 1000:1128]), bits(K[b:b + 1, h:h + 1]), bits(V[b:b + 1, h:h + 1]))
        assert rel_err_max(O[b, h, 1000:1128], ref[0, 0]) <= TOL_BF16
    # full-size property: every output row is a convex combination of V rows, so it lies
    # inside the per-(b,h) min/max envelope of V (up to bf16 rounding)
    vmin = V.float().amin(dim=2, keepdim=True).numpy()
    vmax = V.float().amax(dim=2, keepdim=True).numpy()
    assert (O >= vmin - 0.02).all() and (O <= vmax + 0.02).all()


# ---- any head dimension, through docc_rocm_attention_bf16_ws ---------------------------------------

def run_attention_ws(rt, Qb, Kb, Vb, scale=None, out_bf16=False, slack=0):
    B, H, SQ, D = Qb.shape
    SKV = Kb.shape[2]
    scale = scale if scale is not None else 1.0 / np.sqrt(D)
    q, k, v = dev(Qb), dev(Kb), dev(Vb)
    o = torch.full((B, H, SQ, D), float("nan"), device="cuda", dtype=torch.bfloat16 if out_bf16 else torch.float32)
    need = rt.attention_bf16_workspace_bytes(B, H, SQ, SKV, D, out_bf16)
    ws = torch.empty(max(need + slack, 256), dtype=torch.uint8, device="cuda")
    assert ws.data_ptr() % 256 == 0
    rt.attention_bf16_ws(B, H, SQ, SKV, D, scale, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ws.data_ptr(), need,
                         out_bf16=out_bf16)
    torch.cuda.synchronize()
    return o.float().cpu().numpy(), need


@pytest.mark.parametrize("B,H,SQ,SKV,D", [(1, 2, 96, 96, 128), (2, 3, 128, 64, 32), (1, 2, 130, 200, 128), (1, 1, 33, 65, 80),
                                          (1, 1, 1, 1, 8), (2, 2, 256, 512, 128), (1, 1, 7, 1000, 16), (1, 2, 50, 70, 7),
                                          (1, 2, 96, 96, 64)])
@pytest.mark.parametrize("out_bf16", [False, True])
def test_attention_any_head_dimension_matches_oracle(rt, B, H, SQ, SKV, D, out_bf16):
    g = torch.Generator().manual_seed(B * 7 + H * 5 + SQ * 3 + SKV + D)
    Q, K, V = (torch.randn(B, H, s, D, generator=g).bfloat16() for s in (SQ, SKV, SKV))
    O, need = run_attention_ws(rt, bits(Q), bits(K), bits(V), out_bf16=out_bf16)
    assert (need == 0) == (D == 64)        # head dim 64 runs the fused kernel and needs no workspace
    ref = oracle.attention(bits(Q), bits(K), bits(V))
    assert np.isfinite(O).all()
    assert rel_err_max(O, ref) <= TOL_BF16


def test_attention_workspace_is_checked_and_chunked(rt):
    from docc_amd.runtime import RocmRuntimeError
    t = torch.zeros(1 << 16, dtype=torch.bfloat16, device="cuda")
    p = t.data_ptr()
    need = rt.attention_bf16_workspace_bytes(1, 1, 8, 8, 128)
    assert need >= 8 * 8 * 6
    with pytest.raises(RocmRuntimeError, match="workspace"):
        rt.attention_bf16_ws(1, 1, 8, 8, 128, 0.1, p, p, p, p, 0, 0)
    with pytest.raises(RocmRuntimeError, match="workspace"):
        rt.attention_bf16_ws(1, 1, 8, 8, 128, 0.1, p, p, p, p, p, need - 1)
    # more (batch, head) pairs than one 2 GiB chunk of scores holds: 40 x 4096 x 4096 x 6 B = 3.75 GiB
    B, H, S, D = 1, 40, 4096, 32
    need = rt.attention_bf16_workspace_bytes(B, H, S, S, D)
    assert need <= 2 << 30 and need < H * S * S * 6
    g = torch.Generator(device="cuda").manual_seed(9)
    Q, K, V = (torch.randn(B, H, S, D, device="cuda", generator=g).bfloat16() for _ in range(3))
    o = torch.empty(B, H, S, D, device="cuda")
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    rt.attention_bf16_ws(B, H, S, S, D, D ** -0.5, Q.data_ptr(), K.data_ptr(), V.data_ptr(), o.data_ptr(), ws.data_ptr(), need)
    torch.cuda.synchronize()
    for h in (0, 21, 39):       # heads of the first and of the second chunk
        ref = oracle.attention(bits(Q[:, h:h + 1, :256].cpu()), bits(K[:, h:h + 1].cpu()), bits(V[:, h:h + 1].cpu()))
        assert rel_err_max(o[:, h:h + 1, :256].cpu().numpy(), ref) <= TOL_BF16


def test_attention_more_pairs_than_one_grid_holds(rt):
    """70 000 (batch, head) pairs: the launcher splits them over launches of at most 65 535."""
    B, H, S = 7, 10000, 16
    g = torch.Generator(device="cuda").manual_seed(2)
    Q, K, V = (torch.randn(B, H, S, 64, device="cuda", generator=g).bfloat16() for _ in range(3))
    o = torch.full((B, H, S, 64), float("nan"), device="cuda")
    rt.attention_bf16(B, H, S, S, 64, 0.125, Q.data_ptr(), K.data_ptr(), V.data_ptr(), o.data_ptr())
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o).all())
    flat = lambda t: t.reshape(1, B * H, S, 64)
    for p in (0, 65534, 65535, 69999):
        ref = oracle.attention(bits(flat(Q)[:, p:p + 1].cpu()), bits(flat(K)[:, p:p + 1].cpu()), bits(flat(V)[:, p:p + 1].cpu()))
        assert rel_err_max(flat(o)[:, p:p + 1].cpu().numpy(), ref) <= TOL_BF16, p
