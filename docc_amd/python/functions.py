"""Marker functions the `native` front end lowers to library nodes that numpy has no
spelling for. Calling them outside a `@native` function evaluates a plain numpy reference,
so the same source runs with and without the decorator."""
from __future__ import annotations

import numpy as np


def softmax(x, axis=-1):
    """Same meaning as scipy.special.softmax(x, axis=axis)."""
    m = np.max(x, axis=axis, keepdims=True)
    e = np.exp(x - m)
    return e / np.sum(e, axis=axis, keepdims=True)


def conv2d(x, w, bias=None, stride=1, padding=0, dilation=1):
    """NCHW cross-correlation with zero padding (ONNX Conv / torch.nn.functional.conv2d semantics)."""
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    ph, pw = (padding, padding) if np.isscalar(padding) else padding
    dh, dw = (dilation, dilation) if np.isscalar(dilation) else dilation
    n, c, h, wd = x.shape
    oc, _, kh, kw = w.shape
    oh = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (wd + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    xp = np.pad(x, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
    y = np.zeros((n, oc, oh, ow), dtype=x.dtype)
    for i in range(kh):
        for j in range(kw):
            patch = xp[:, :, i * dh:i * dh + sh * oh:sh, j * dw:j * dw + sw * ow:sw]
            y += np.einsum("nchw,oc->nohw", patch, w[:, :, i, j])
    if bias is not None:
        y += np.asarray(bias).reshape(1, -1, 1, 1)
    return y


def relu(x):
    """max(x, 0) elementwise (the ml::ReLU node)."""
    return np.maximum(x, 0)


def sigmoid(x):
    """1 / (1 + exp(-x)) elementwise (the ml::Sigmoid node)."""
    return 1.0 / (1.0 + np.exp(-x))


def erf(x):
    """The error function elementwise (the ml::Erf node)."""
    from scipy.special import erf as _erf
    return _erf(x)
