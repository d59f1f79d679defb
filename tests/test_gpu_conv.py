"""ml::Conv (2-d, NCHW, fp32) on the GPU against the CPU oracle, through
docc_rocm_conv2d_f32. Tolerance 1e-5 norm-wise (max|y - y_ref| / max|y_ref|);
integer-valued inputs are compared bit-exactly."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu


def run_conv(rt, X, W, bias=None, stride=(1, 1), pad=(0, 0), dilation=(1, 1)):
    N, C, H, Wd = X.shape
    OC, _, KH, KW = W.shape
    OH = oracle.conv_out_dim(H, pad[0], dilation[0], KH, stride[0])
    OW = oracle.conv_out_dim(Wd, pad[1], dilation[1], KW, stride[1])
    x, w = dev(X), dev(W)
    b = dev(bias) if bias is not None else None
    y = torch.full((N, OC, OH, OW), float("nan"), device="cuda")
    rt.conv2d_f32(N, C, H, Wd, OC, KH, KW, stride, pad, dilation, x.data_ptr(), w.data_ptr(),
                  b.data_ptr() if b is not None else 0, y.data_ptr())
    torch.cuda.synchronize()
    return host(y)


CASES = [
    # N, C, H, W, OC, KH, KW, stride, pad, dil, bias
    (2, 3, 7, 7, 4, 3, 3, (1, 1), (1, 1), (1, 1), True),
    (1, 2, 5, 5, 3, 3, 3, (1, 1), (0, 0), (1, 1), False),
    (2, 5, 9, 11, 70, 3, 3, (1, 1), (1, 1), (1, 1), True),     # OC > one tile of 64
    (3, 4, 12, 10, 8, 1, 1, (1, 1), (0, 0), (1, 1), True),     # 1x1
    (2, 3, 13, 9, 5, 5, 3, (2, 1), (2, 1), (1, 1), True),      # rectangular kernel, mixed stride
    (2, 3, 16, 16, 6, 3, 3, (2, 2), (1, 1), (2, 2), False),    # stride + dilation
    (1, 7, 8, 8, 9, 7, 7, (1, 1), (3, 3), (1, 1), True),       # kernel ~ image
    (4, 16, 20, 20, 32, 3, 3, (1, 1), (1, 1), (1, 1), True),
    (1, 1, 4, 4, 1, 3, 3, (1, 1), (2, 2), (1, 1), False),      # pad larger than needed
    # stride-1 3x3 / 1x1 with C % 8 == 0: the LDS-halo kernel
    (2, 8, 9, 11, 70, 3, 3, (1, 1), (1, 1), (1, 1), True),     # OC > 64 and not a multiple of 32, odd image
    (3, 16, 30, 30, 40, 3, 3, (1, 1), (0, 0), (1, 1), False),   # no padding, several strips per image (OH % TH != 0)
    (1, 24, 5, 100, 64, 3, 3, (1, 1), (2, 1), (1, 1), True),    # wide rows: 4 rows per strip, asymmetric pad sizes
    (2, 32, 12, 12, 16, 1, 1, (1, 1), (0, 0), (1, 1), True),    # 1x1
    (1, 8, 3, 448, 8, 3, 3, (1, 1), (1, 1), (1, 1), False),     # one row per strip
    (2, 32, 14, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), True),    # 7 rows of 56: 13 column tiles, the last shared by two waves
    (2, 16, 28, 28, 64, 3, 3, (1, 1), (1, 1), (1, 1), True),    # small images: strips of 8 or 4 column tiles fill the device better
    (3, 24, 14, 14, 96, 3, 3, (1, 1), (1, 1), (1, 1), False),
    (2, 32, 7, 7, 64, 3, 3, (1, 1), (1, 1), (1, 1), True),      # 49 pixels: one pixel group of the smallest strip works alone
    (2, 32, 14, 14, 70, 1, 1, (1, 1), (0, 0), (1, 1), True),
    (2, 16, 28, 28, 64, 3, 3, (2, 2), (1, 1), (1, 1), True),    # strides of 2 on the LDS-halo kernel: the patch of a strip covers the skipped pixels too
    (2, 8, 15, 21, 40, 3, 3, (2, 1), (1, 1), (1, 1), False),    # mixed strides, odd image
    (2, 32, 14, 14, 64, 1, 1, (2, 2), (0, 0), (1, 1), True),    # a 1x1 downsampling layer
    (1, 8, 9, 120, 16, 3, 3, (2, 2), (0, 0), (1, 1), True),     # wide rows: one or two output rows per strip
    (7, 16, 7, 7, 70, 3, 3, (1, 1), (1, 1), (1, 1), True),      # images of 49 pixels: several to a work-group, the last group not full
    (5, 8, 4, 6, 64, 3, 3, (1, 1), (1, 1), (1, 1), False),
    (9, 16, 9, 9, 32, 3, 3, (2, 2), (1, 1), (1, 1), True),      # 5 x 5 outputs of a strided layer
    (6, 24, 5, 5, 40, 1, 1, (1, 1), (0, 0), (1, 1), True),
]


@pytest.mark.parametrize("case", CASES)
def test_conv_integer_exact(rt, case):
    N, C, H, W, OC, KH, KW, stride, pad, dil, use_bias = case
    rng = np.random.default_rng(hash(case[:7]) & 0xffff)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, C, KH, KW)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    Y = run_conv(rt, X, Wt, b, stride, pad, dil)
    ref = oracle.conv2d(X, Wt, b, stride, pad, dil)
    assert Y.shape == ref.shape
    assert np.array_equal(Y, ref)


@pytest.mark.parametrize("case", CASES)
def test_conv_random_matches_oracle(rt, case):
    N, C, H, W, OC, KH, KW, stride, pad, dil, use_bias = case
    rng = np.random.default_rng(1 + (hash(case[:7]) & 0xffff))
    X = rng.standard_normal((N, C, H, W)).astype(np.float32)
    Wt = (rng.standard_normal((OC, C, KH, KW)) * np.sqrt(2.0 / (C * KH * KW))).astype(np.float32)
    b = (rng.standard_normal(OC) * 0.1).astype(np.float32) if use_bias else None
    Y = run_conv(rt, X, Wt, b, stride, pad, dil)
    assert rel_err_max(Y, oracle.conv2d(X, Wt, b, stride, pad, dil)) <= 1e-5


def test_conv_closed_forms(rt):
    rng = np.random.default_rng(0)
    X = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    # delta kernel per channel -> identity
    Wt = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        Wt[c, c, 1, 1] = 1.0
    assert np.array_equal(run_conv(rt, X, Wt, None, pad=(1, 1)), X)
    # shifted delta -> shift with a zero border
    Wt[:] = 0
    for c in range(3):
        Wt[c, c, 0, 2] = 1.0  # reads X[h-1, w+1]
    Y = run_conv(rt, X, Wt, None, pad=(1, 1))
    exp = np.zeros_like(X)
    exp[:, :, 1:, :-1] = X[:, :, :-1, 1:]
    assert np.array_equal(Y, exp)
    # all-ones input and weights: the output counts the taps inside the image (4 / 6 / 9 per channel)
    C = 64
    Y = run_conv(rt, np.ones((1, C, 6, 6), np.float32), np.ones((2, C, 3, 3), np.float32), None, pad=(1, 1))
    assert Y[0, 0, 0, 0] == C * 4 and Y[0, 1, 0, 3] == C * 6 and Y[0, 0, 3, 3] == C * 9 and Y[0, 1, 5, 5] == C * 4
    # zero weights: the output is the bias
    b = np.arange(5, dtype=np.float32)
    Y = run_conv(rt, X, np.zeros((5, 3, 3, 3), np.float32), b, pad=(1, 1))
    assert np.array_equal(Y, np.broadcast_to(b[None, :, None, None], Y.shape))


def test_conv_empty_and_errors(rt):
    from docc_amd.runtime import RocmRuntimeError
    rt.conv2d_f32(0, 3, 8, 8, 4, 3, 3, (1, 1), (1, 1), (1, 1), 0, 0, 0, 0)
    rt.conv2d_f32(1, 3, 2, 2, 4, 3, 3, (1, 1), (0, 0), (1, 1), 0, 0, 0, 0)  # kernel larger than image: empty output
    with pytest.raises(RocmRuntimeError):
        rt.conv2d_f32(1, 3, 8, 8, 4, 3, 3, (0, 1), (1, 1), (1, 1), 0, 0, 0, 0)


def test_conv_config_resnet_block(rt):
    # benchmark configuration 5: N=32, 64 -> 64 channels, 56x56, 3x3, stride 1, pad 1, bias
    g = torch.Generator().manual_seed(4)
    X = torch.randn(32, 64, 56, 56, generator=g).numpy()
    Wt = (torch.randn(64, 64, 3, 3, generator=g) * np.sqrt(2.0 / 576)).numpy()
    b = (torch.randn(64, generator=g) * 0.1).numpy()
    Y = run_conv(rt, X, Wt, b, pad=(1, 1))
    assert np.isfinite(Y).all()
    # oracle on two images (the first and the last)
    sel = [0, 31]
    assert rel_err_max(Y[sel], oracle.conv2d(X[sel], Wt, b, pad=(1, 1))) <= 1e-5
    # full-size property: linearity in the input, conv(X) - conv(0) summed over everything
    # equals sum_oc sum_ic sum_taps W * (sum of X over the window positions); checked through
    # the channel-summed output against a conv of the channel structure done in fp64 on the CPU
    tot = Y.astype(np.float64).sum(axis=(0, 2, 3)) - 32 * 56 * 56 * b.astype(np.float64)
    Xs = X.astype(np.float64)
    Xp = np.pad(Xs, ((0, 0), (0, 0), (1, 1), (1, 1)))
    # S[ic, kh, kw] = sum over n, oh, ow of X[n, ic, oh+kh-1, ow+kw-1]
    S = np.array([[[Xp[:, ic, kh:kh + 56, kw:kw + 56].sum() for kw in range(3)] for kh in range(3)] for ic in range(64)])
    exp = np.einsum("oikl,ikl->o", Wt.astype(np.float64), S)
    assert np.abs(tot - exp).max() / np.abs(exp).max() <= 1e-4


# ---- docc_rocm_conv2d_f32_ws: im2col + GEMM and the batched 1x1 GEMM beside the direct kernels ------------

def run_conv_ws(rt, X, W, bias=None, stride=(1, 1), pad=(0, 0), dilation=(1, 1), workspace_bytes=None):
    N, C, H, Wd = X.shape
    OC, _, KH, KW = W.shape
    OH = oracle.conv_out_dim(H, pad[0], dilation[0], KH, stride[0])
    OW = oracle.conv_out_dim(Wd, pad[1], dilation[1], KW, stride[1])
    x, w = dev(X), dev(W)
    b = dev(bias) if bias is not None else None
    y = torch.full((N, OC, OH, OW), float("nan"), device="cuda")
    need = rt.conv2d_f32_workspace_bytes(N, C, H, Wd, OC, KH, KW, stride, pad, dilation)
    size = need if workspace_bytes is None else workspace_bytes
    ws = torch.empty(max(size, 256), dtype=torch.uint8, device="cuda")
    rt.conv2d_f32_ws(N, C, H, Wd, OC, KH, KW, stride, pad, dilation, x.data_ptr(), w.data_ptr(), b.data_ptr() if b is not None else 0,
                     y.data_ptr(), ws.data_ptr() if size else 0, size)
    torch.cuda.synchronize()
    return host(y), need


@pytest.mark.parametrize("force", ["gemm", "gather", "halo", "halo-split", "halo-split-wide", "halo-whole", "halo-t4", "halo-t2", "halo-t4m", "halo-t2m", ""])
@pytest.mark.parametrize("case", CASES)
def test_conv_every_path_integer_exact(rt, monkeypatch, force, case):
    """Each way to run a layer (forced through DOCC_ROCM_CONV; a path that does not apply falls back; halo-split and
    halo-whole are the LDS-halo kernel with strips of 13 shared and 14 whole column tiles, halo-split-wide keeps the
    shared tile 32 pixels wide where the 16-pixel form would apply, halo-t4 and halo-t2 are the strips of 8 and 4 column
    tiles for small images) and the automatic choice give the oracle's integers."""
    N, C, H, W, OC, KH, KW, stride, pad, dil, use_bias = case
    if force:
        monkeypatch.setenv("DOCC_ROCM_CONV", force)
    rng = np.random.default_rng(hash(case[:7]) & 0xffff)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, C, KH, KW)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    Y, _ = run_conv_ws(rt, X, Wt, b, stride, pad, dil)
    assert np.array_equal(Y, oracle.conv2d(X, Wt, b, stride, pad, dil))


GEMM_LAYERS = [  # small images with many channels: the shapes the choice sends to im2col + GEMM, and a 1x1 layer with C >= 128
    (8, 256, 14, 14, 256, 3, 3, (1, 1), (1, 1), (1, 1), True), (8, 512, 7, 7, 512, 3, 3, (1, 1), (1, 1), (1, 1), True),
    (1, 256, 14, 14, 256, 3, 3, (1, 1), (1, 1), (1, 1), False), (4, 256, 28, 28, 64, 1, 1, (1, 1), (0, 0), (1, 1), True),
    (3, 128, 9, 9, 96, 3, 3, (2, 2), (1, 1), (1, 1), True),
]


@pytest.mark.parametrize("case", GEMM_LAYERS, ids=[f"n{c[0]}c{c[1]}_{c[2]}x{c[3]}_oc{c[4]}k{c[5]}s{c[7][0]}" for c in GEMM_LAYERS])
def test_conv_gemm_layers_match_oracle(rt, case):
    N, C, H, W, OC, KH, KW, stride, pad, dil, use_bias = case
    rng = np.random.default_rng(C + H)
    X = rng.standard_normal((N, C, H, W)).astype(np.float32)
    Wt = (rng.standard_normal((OC, C, KH, KW)) * np.sqrt(2.0 / (C * KH * KW))).astype(np.float32)
    b = (rng.standard_normal(OC) * 0.1).astype(np.float32) if use_bias else None
    Y, need = run_conv_ws(rt, X, Wt, b, stride, pad, dil)
    pointwise = KH == 1 and stride == (1, 1) and pad == (0, 0)
    assert (need == 0) == pointwise            # the 1x1 layer multiplies the tensors as they lie
    ref = oracle.conv2d(X[:2], Wt, b, stride, pad, dil)
    assert rel_err_max(Y[:2], ref) <= 1e-5
    # without the workspace the same call takes a direct kernel and agrees
    Y0, _ = run_conv_ws(rt, X, Wt, b, stride, pad, dil, workspace_bytes=0)
    assert rel_err_max(Y0, Y) <= 1e-5


def test_conv_workspace_chunks_over_images(rt, monkeypatch):
    """A workspace that holds the columns of two images at a time: the images are processed in chunks."""
    monkeypatch.setenv("DOCC_ROCM_CONV", "gemm")
    N, C, H, W, OC = 5, 16, 10, 10, 24
    rng = np.random.default_rng(77)
    X = rng.integers(-3, 4, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-3, 4, (OC, C, 3, 3)).astype(np.float32)
    b = rng.integers(-3, 4, OC).astype(np.float32)
    need = rt.conv2d_f32_workspace_bytes(N, C, H, W, OC, 3, 3, (1, 1), (1, 1), (1, 1))
    assert need > 0 and need % N == 0
    Y, _ = run_conv_ws(rt, X, Wt, b, (1, 1), (1, 1), (1, 1), workspace_bytes=need)
    assert np.array_equal(Y, oracle.conv2d(X, Wt, b, (1, 1), (1, 1), (1, 1)))


# ---- a begin and an end pad per axis (the node's `pads`: begins, then ends; conv_node.cpp:76-77, 224-233) ------------

PAD_CASES = [  # (N, C, H, W, OC, KH, KW, stride, (top, left, bottom, right), dilation, bias)
    (2, 16, 12, 20, 70, 3, 3, (1, 1), (0, 1, 2, 0), (1, 1), True),     # halo shape, nothing above, two rows below
    (1, 8, 9, 9, 64, 3, 3, (1, 1), (2, 2, 0, 1), (1, 1), False),      # halo shape, more before than after
    (3, 5, 11, 13, 17, 3, 2, (2, 1), (1, 0, 0, 3), (1, 2), True),     # strides, dilation, odd channels: the gather kernel
    (2, 24, 7, 7, 32, 1, 1, (1, 1), (0, 0, 1, 1), (1, 1), True),      # 1x1 with padding at the end only: not the pointwise GEMM
    (2, 32, 10, 10, 40, 5, 5, (1, 1), (4, 0, 0, 4), (1, 1), False),   # a large filter hanging over one corner
]


@pytest.mark.parametrize("force", ["gemm", "gather", "halo", "halo-split", ""])
@pytest.mark.parametrize("case", PAD_CASES)
def test_conv_with_different_pads_before_and_after(rt, monkeypatch, force, case):
    N, C, H, W, OC, KH, KW, stride, pads, dil, use_bias = case
    if force:
        monkeypatch.setenv("DOCC_ROCM_CONV", force)
    rng = np.random.default_rng(hash(case[:7]) & 0xffff)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, C, KH, KW)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    ref = oracle.conv2d(X, Wt, b, stride, pads, dil)
    # the extents follow begin + end; an independent statement of the same: pad the image by hand, convolve without pads
    Xp = np.pad(X, ((0, 0), (0, 0), (pads[0], pads[2]), (pads[1], pads[3])))
    assert np.array_equal(ref, oracle.conv2d(Xp, Wt, b, stride, (0, 0), dil))
    x, w = dev(X), dev(Wt)
    bd = dev(b) if b is not None else None
    y = torch.full(ref.shape, float("nan"), device="cuda")
    need = rt.conv2d_f32_pads_workspace_bytes(N, C, H, W, OC, KH, KW, stride, pads, dil)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
    rt.conv2d_f32_pads(N, C, H, W, OC, KH, KW, stride, pads, dil, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0,
                       y.data_ptr(), ws.data_ptr() if need else 0, need)
    torch.cuda.synchronize()
    assert np.array_equal(host(y), ref)
    # equal pads through the new entry point are the old entry point
    if force == "":
        sym = (pads[0], pads[1], pads[0], pads[1])
        y1 = torch.full(oracle.conv2d(X, Wt, b, stride, sym, dil).shape, float("nan"), device="cuda")
        y2 = torch.full_like(y1, float("nan"))
        rt.conv2d_f32_pads(N, C, H, W, OC, KH, KW, stride, sym, dil, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0, y1.data_ptr())
        rt.conv2d_f32(N, C, H, W, OC, KH, KW, stride, sym[:2], dil, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0, y2.data_ptr())
        torch.cuda.synchronize()
        assert torch.equal(y1, y2)
    with pytest.raises(rt.RocmRuntimeError, match="padding non-negative"):
        rt.conv2d_f32_pads(N, C, H, W, OC, KH, KW, stride, (0, 0, -1, 0), dil, x.data_ptr(), w.data_ptr(), 0, y.data_ptr())


GROUP_CASES = [
    # N, C, H, W, OC, KH, KW, stride, pads, dilation, group, bias
    (2, 32, 12, 12, 64, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 2, True),      # 16 channels a group: the LDS-halo kernel per group
    (3, 64, 9, 11, 64, 3, 3, (2, 2), (1, 0, 0, 1), (1, 1), 4, False),      # strides of 2, a begin and an end pad, four groups
    (2, 16, 10, 10, 16, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 16, True),     # depthwise: one channel a group, the gather kernel
    (1, 12, 8, 7, 30, 2, 3, (1, 2), (0, 1, 1, 0), (2, 1), 6, True),        # two channels in, five out per group, dilation
    (2, 256, 7, 7, 512, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 2, False),     # pointwise: a GEMM when whole, direct per group
    (3, 8, 13, 9, 24, 3, 3, (2, 1), (1, 1, 0, 2), (1, 1), 8, True),        # depthwise with three output channels per input channel
    (2, 24, 17, 17, 24, 5, 5, (1, 1), (2, 2, 2, 2), (1, 1), 24, False),    # depthwise 5x5
    (1, 6, 9, 20, 12, 2, 4, (1, 3), (0, 3, 1, 0), (2, 1), 6, True),        # depthwise, a 2x4 filter with dilation and a stride of 3
    (2, 40, 28, 28, 40, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 40, True),     # depthwise on planes of more than one work-group
    (3, 16, 9, 12, 32, 3, 3, (1, 1), (0, 1, 2, 1), (1, 1), 16, True),      # rows of three quads, no rows above, two below
    (2, 32, 12, 16, 32, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 8, True),      # eight groups of four channels (a ResNeXt layer in small)
    (2, 16, 9, 8, 48, 3, 3, (1, 1), (2, 1, 0, 1), (1, 1), 2, False),       # two groups of eight channels in, 24 out each
    (1, 12, 10, 12, 18, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 6, True),      # two channels in, three out per group: one output channel a lane
    (2, 10, 11, 20, 20, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 2, True),      # five channels in, ten out per group: pairs of output channels
]


# depthwise layers: four pixels of several rows a lane where rows allow, of one row (quad), one pixel, and the kernels of the other groups; those: every group in one
# launch, and a launch per group
@pytest.mark.parametrize("force", ["", "quad", "scalar", "gather", "loop"])
@pytest.mark.parametrize("case", GROUP_CASES)
def test_conv_with_groups(rt, monkeypatch, force, case):
    """The node's `group`: weights [OC, C / group, KH, KW], every group on its own channels of X and Y where they lie. Integer-
    valued operands against the oracle bit for bit; the oracle's grouped form is pinned in tests/test_oracle.py."""
    N, C, H, W, OC, KH, KW, stride, pads, dil, group, use_bias = case
    if force:
        if (group == C) == (force == "loop") or (force == "scalar" and group != C):
            pytest.skip("a form of the other kind of layer")
        monkeypatch.setenv("DOCC_ROCM_CONV", force)
    rng = np.random.default_rng(hash(case[:7]) & 0xffff)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, C // group, KH, KW)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    ref = oracle.conv2d(X, Wt, b, stride, pads, dil, group=group)
    x, w = dev(X), dev(Wt)
    bd = dev(b) if b is not None else None
    y = torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, KH, KW, stride, pads, dil, group, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0,
                          y.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(y), ref)
    # one group is the entry point without groups
    full = rng.integers(-4, 5, (OC, C, KH, KW)).astype(np.float32)
    wf = dev(full)
    y1, y2 = torch.full(ref.shape, float("nan"), device="cuda"), torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, KH, KW, stride, pads, dil, 1, x.data_ptr(), wf.data_ptr(), bd.data_ptr() if bd is not None else 0, y1.data_ptr())
    rt.conv2d_f32_pads(N, C, H, W, OC, KH, KW, stride, pads, dil, x.data_ptr(), wf.data_ptr(), bd.data_ptr() if bd is not None else 0, y2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)
    for bad in (0, -2, 5 if C % 5 else 7):
        with pytest.raises(rt.RocmRuntimeError, match="group"):
            rt.conv2d_f32_grouped(N, C, H, W, OC, KH, KW, stride, pads, dil, bad, x.data_ptr(), w.data_ptr(), 0, y.data_ptr())


@pytest.mark.parametrize("rows", ["4", "7", "8"])
@pytest.mark.parametrize("shape", [
    # N, C, H, W, channels out per channel in, pads (h, w, h end, w end), bias
    (2, 24, 19, 16, 2, (1, 1, 1, 1), True),     # 19 rows: the last block of rows is cut for every count
    (1, 8, 5, 8, 1, (2, 1, 0, 1), False),       # fewer rows than a block, two rows of padding above and none below
    (3, 5, 56, 56, 1, (1, 1, 1, 1), True),      # 15 planes of 784 quads: wavefronts run over plane borders
    (1, 3, 33, 4, 3, (0, 1, 3, 1), True),       # one quad a row
])
def test_depthwise_rows_a_lane(rt, monkeypatch, rows, shape):
    """The depthwise 3x3 kernel with 4, 7 and 8 output rows a lane (DOCC_ROCM_CONV_ROWS) against the oracle bit for bit, and equal
    to the kernel with one row a lane on random operands (same order of the sums)."""
    N, C, H, W, mult, pads, use_bias = shape
    OC = C * mult
    monkeypatch.setenv("DOCC_ROCM_CONV_ROWS", rows)
    rng = np.random.default_rng(int(rows) * 131 + H)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, 1, 3, 3)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    ref = oracle.conv2d(X, Wt, b, (1, 1), pads, (1, 1), group=C)
    x, w = dev(X), dev(Wt)
    bd = dev(b) if b is not None else None
    y = torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, 3, 3, (1, 1), pads, (1, 1), C, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0, y.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(y), ref)
    xr, wr = torch.randn(N, C, H, W, device="cuda"), torch.randn(OC, 1, 3, 3, device="cuda")
    ya, yb = torch.full(ref.shape, float("nan"), device="cuda"), torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, 3, 3, (1, 1), pads, (1, 1), C, xr.data_ptr(), wr.data_ptr(), bd.data_ptr() if bd is not None else 0, ya.data_ptr())
    monkeypatch.setenv("DOCC_ROCM_CONV", "quad")
    rt.conv2d_f32_grouped(N, C, H, W, OC, 3, 3, (1, 1), pads, (1, 1), C, xr.data_ptr(), wr.data_ptr(), bd.data_ptr() if bd is not None else 0, yb.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(ya, yb)


@pytest.mark.parametrize("rows", ["4", "7"])
@pytest.mark.parametrize("shape", [
    # N, C, H, W, channels out per channel in, stride, pads (h, w, h end, w end), bias
    (3, 20, 14, 14, 1, 1, (1, 1, 1, 1), True),     # 14 x 14 planes: rows of no whole quads
    (2, 37, 7, 7, 2, 1, (1, 1, 1, 1), False),      # 7 x 7 planes, seven lanes a plane
    (2, 6, 23, 17, 1, 2, (1, 1, 1, 1), True),      # steps of two on odd extents
    (1, 5, 30, 9, 3, 2, (0, 2, 1, 0), True),       # steps of two, pads that differ, 15 output rows
    (2, 4, 9, 13, 1, 1, (2, 0, 0, 2), False),      # no column of padding on the left, two on the right
    (2, 18, 28, 28, 1, 1, (2, 2, 2, 2), True, 5),  # 5x5 filters
    (3, 7, 17, 15, 2, 2, (2, 2, 2, 2), False, 5),  # 5x5, steps of two, odd extents
    (1, 6, 6, 9, 1, 1, (0, 1, 3, 2), True, 5),     # 5x5 on planes lower than the filter without the pads
])
def test_depthwise_column_and_rows_a_lane(rt, monkeypatch, rows, shape):
    """The depthwise 3x3 and 5x5 kernels with one output column and 4 or 7 output rows a lane (stride 1 or 2) against the oracle bit for
    bit, and equal to the kernel with a pixel a lane on random operands (same order of the sums)."""
    N, C, H, W, mult, st, pads, use_bias = shape[:8]
    K = shape[8] if len(shape) > 8 else 3
    OC = C * mult
    monkeypatch.setenv("DOCC_ROCM_CONV_ROWS", rows)
    rng = np.random.default_rng(int(rows) * 977 + H)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, 1, K, K)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    ref = oracle.conv2d(X, Wt, b, (st, st), pads, (1, 1), group=C)
    x, w = dev(X), dev(Wt)
    bd = dev(b) if b is not None else None
    y = torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, K, K, (st, st), pads, (1, 1), C, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0, y.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(y), ref)
    xr, wr = torch.randn(N, C, H, W, device="cuda"), torch.randn(OC, 1, K, K, device="cuda")
    ya, yb = torch.full(ref.shape, float("nan"), device="cuda"), torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, K, K, (st, st), pads, (1, 1), C, xr.data_ptr(), wr.data_ptr(), bd.data_ptr() if bd is not None else 0, ya.data_ptr())
    monkeypatch.setenv("DOCC_ROCM_CONV", "scalar")
    rt.conv2d_f32_grouped(N, C, H, W, OC, K, K, (st, st), pads, (1, 1), C, xr.data_ptr(), wr.data_ptr(), bd.data_ptr() if bd is not None else 0, yb.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(ya, yb)


@pytest.mark.parametrize("rows", ["8", "4"])   # set, the variable keeps small layers on this form; 4: four rows for eight channels
@pytest.mark.parametrize("shape", [
    # N, C, H, W, OC, group, pads (h, w, h end, w end), bias
    (3, 32, 19, 16, 32, 8, (1, 1, 1, 1), True),     # four in, four out per group: four rows a lane, 19 rows
    (2, 32, 13, 8, 64, 4, (1, 1, 1, 1), True),      # eight in, 16 out: two chunks of eight channels, two (or four) rows a lane
    (5, 12, 56, 56, 12, 6, (1, 1, 1, 1), False),    # two in, two out: eight rows a lane, lanes counting through the images
    (2, 9, 11, 12, 15, 3, (2, 1, 0, 1), True),      # three in, five out: one output channel and eight rows a lane, pads that differ
    (4, 512, 8, 8, 512, 32, (1, 1, 1, 1), True),    # 16 in, 16 out in 32 groups: enough work-groups for this kernel to be the choice
])
def test_small_groups_rows_a_lane(rt, monkeypatch, rows, shape):
    """Groups of a few channels with several output rows a lane against the oracle bit for bit, and equal to the kernel with one
    row a lane on random operands (same order of the sums)."""
    N, C, H, W, OC, group, pads, use_bias = shape
    monkeypatch.setenv("DOCC_ROCM_CONV_ROWS", rows)
    rng = np.random.default_rng(H * 31 + W)
    X = rng.integers(-4, 5, (N, C, H, W)).astype(np.float32)
    Wt = rng.integers(-4, 5, (OC, C // group, 3, 3)).astype(np.float32)
    b = rng.integers(-4, 5, OC).astype(np.float32) if use_bias else None
    ref = oracle.conv2d(X, Wt, b, (1, 1), pads, (1, 1), group=group)
    x, w = dev(X), dev(Wt)
    bd = dev(b) if b is not None else None
    y = torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, 3, 3, (1, 1), pads, (1, 1), group, x.data_ptr(), w.data_ptr(), bd.data_ptr() if bd is not None else 0, y.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(host(y), ref)
    xr, wr = torch.randn(N, C, H, W, device="cuda"), torch.randn(OC, C // group, 3, 3, device="cuda")
    ya, yb = torch.full(ref.shape, float("nan"), device="cuda"), torch.full(ref.shape, float("nan"), device="cuda")
    rt.conv2d_f32_grouped(N, C, H, W, OC, 3, 3, (1, 1), pads, (1, 1), group, xr.data_ptr(), wr.data_ptr(), bd.data_ptr() if bd is not None else 0, ya.data_ptr())
    monkeypatch.setenv("DOCC_ROCM_CONV", "quad")
    rt.conv2d_f32_grouped(N, C, H, W, OC, 3, 3, (1, 1), pads, (1, 1), group, xr.data_ptr(), wr.data_ptr(), bd.data_ptr() if bd is not None else 0, yb.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(ya, yb)
