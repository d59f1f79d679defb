"""docc_rocm_softmax_noalloc, the entry point for callers that cannot allocate: through the C ABI, against
docc_rocm_softmax (same kernels and launch geometry, so the same bits), on calls in a row that share the fixed
array of partial results, the later ones smaller than the first."""
import numpy as np
import pytest
import scipy.special
import torch

from docc_amd.runtime import RocmRuntimeError
from gpu_util import dev, host, rel_err_max

pytestmark = pytest.mark.gpu


def both(rt, X, precision):
    outer, reduce_, inner = X.shape
    x = dev(X)
    ref, out = torch.empty_like(x), torch.full_like(x, float("nan"))
    rt.softmax(precision, outer, reduce_, inner, x.data_ptr(), ref.data_ptr())
    rt.softmax_noalloc(precision, outer, reduce_, inner, x.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    return host(ref), host(out)


@pytest.mark.parametrize("dt,precision,tol", [(np.float32, 32, 1e-5), (np.float64, 64, 1e-12)], ids=["f32", "f64"])
def test_no_alloc_softmax_matches_the_allocating_entry_point(rt, dt, precision, tol):
    rng = np.random.default_rng(precision)
    # sliced form (partial results in the fixed array), large then small, then shapes of the one-launch forms
    shapes = [(1, 6000, 320), (1, 900, 130), (2, 512, 70), (3, 700, 130), (1, 257, 64), (4, 100, 1), (2, 300, 16), (5, 40, 33),
              (2, 150000, 1), (3, 20000, 1)]      # rows cut into slices: their pairs go through the fixed array as well
    assert rt.softmax_workspace_bytes(precision, *shapes[0]) > rt.softmax_workspace_bytes(precision, *shapes[1]) > 0
    for shape in shapes:
        X = (rng.standard_normal(shape) * 6).astype(dt)
        ref, out = both(rt, X, precision)
        assert np.array_equal(ref, out), shape
        assert rel_err_max(out, scipy.special.softmax(X.astype(np.float64), axis=1)) <= tol, shape


def test_no_alloc_softmax_refuses_what_does_not_fit(rt):
    # fp64, 19200 columns in 300 tiles: four slices of (maximum, sum) pairs are 1.2 MiB
    outer, reduce_, inner = 1, 4096, 19200
    need = rt.softmax_workspace_bytes(64, outer, reduce_, inner)
    assert need > 1 << 20
    x = torch.zeros(outer * reduce_ * inner, dtype=torch.float64, device="cuda")
    y = torch.empty_like(x)
    with pytest.raises(RocmRuntimeError, match=f"needs {need} bytes of partial results, the entry point holds {1 << 20}"):
        rt.softmax_noalloc(64, outer, reduce_, inner, x.data_ptr(), y.data_ptr())
    rt.softmax(64, outer, reduce_, inner, x.data_ptr(), y.data_ptr())      # the allocating entry point takes it
    torch.cuda.synchronize()
    assert bool((y == 1.0 / reduce_).all())
    with pytest.raises(RocmRuntimeError, match="precision"):
        rt.softmax_noalloc(16, 1, 8, 8, x.data_ptr(), y.data_ptr())
    rt.softmax_noalloc(32, 0, 8, 8, 0, 0)                                    # empty: nothing to do


def test_no_alloc_softmax_takes_no_device_memory_on_a_new_stream(rt):
    """What the entry point is for: a sliced shape on a stream that has never been used allocates nothing (the
    allocating entry point would create its 8 MiB of partial results for that stream here)."""
    outer, reduce_, inner = 1, 6000, 320
    assert rt.softmax_workspace_bytes(32, outer, reduce_, inner) > 0            # the sliced form
    rng = np.random.default_rng(9)
    X = (rng.standard_normal((outer, reduce_, inner)) * 6).astype(np.float32)
    x = dev(X)
    y = torch.full_like(x, float("nan"))
    s = rt.stream_create()
    try:
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        rt.softmax_noalloc(32, outer, reduce_, inner, x.data_ptr(), y.data_ptr(), stream=s)
        rt.stream_sync(s)
        assert torch.cuda.mem_get_info()[0] >= free_before - (1 << 20)
        assert rel_err_max(host(y), scipy.special.softmax(X.astype(np.float64), axis=1)) <= 1e-5
        # the allocating entry point on the same new stream does take its buffer, and gives it back with the stream
        rt.softmax(32, outer, reduce_, inner, x.data_ptr(), y.data_ptr(), stream=s)
        rt.stream_sync(s)
        assert free_before - torch.cuda.mem_get_info()[0] >= 8 << 20
    finally:
        rt.stream_destroy(s)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before - (1 << 20)


def test_no_alloc_softmax_wants_the_device_set_up_first():
    """In a process that has not called docc_rocm_init the entry point loads nothing by itself: it says what is missing."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    code = (
        "import ctypes, sys\n"
        f"lib = ctypes.CDLL(r'{root / 'docc_amd' / 'lib' / 'libdocc_rt_rocm.so'}')\n"
        "lib.docc_rocm_last_error.restype = ctypes.c_char_p\n"
        "f = lib.docc_rocm_softmax_noalloc\n"
        "f.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]\n"
        "rc = f(None, 32, 2, 300, 16, 4096, 8192)\n"
        "print(rc, lib.docc_rocm_last_error().decode())\n"
    )
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.startswith("-1 ") and "has not been set up; call docc_rocm_init(0) first" in r.stdout, r.stdout
