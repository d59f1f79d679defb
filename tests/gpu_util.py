"""Helpers shared by the GPU parity tests: torch is used only to hold device
memory; every computation goes through the C-ABI of libdocc_rt_rocm.so."""
import numpy as np
import torch


def dev(a: np.ndarray) -> torch.Tensor:
    """numpy array -> device tensor holding the same bytes (bf16 bits stay uint16)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    return torch.from_numpy(a).cuda()


def host(t: torch.Tensor, dtype=None) -> np.ndarray:
    a = t.cpu().numpy()
    if dtype is not None and a.dtype != dtype:
        a = a.view(dtype)
    return a


def rel_err_max(y: np.ndarray, ref: np.ndarray) -> float:
    """Norm-wise relative error: max|y - ref| / max|ref|."""
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    denom = np.abs(ref).max() if ref.size else 1.0
    return float(np.abs(y - ref).max() / (denom if denom > 0 else 1.0)) if ref.size else 0.0


def rel_err_fro(y: np.ndarray, ref: np.ndarray) -> float:
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    denom = np.linalg.norm(ref.ravel())
    return float(np.linalg.norm((y - ref).ravel()) / (denom if denom > 0 else 1.0))
