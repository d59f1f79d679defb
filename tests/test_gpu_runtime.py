"""The thin HIP runtime on a device: memory, copies and the device block cache behind
docc_rocm_malloc / docc_rocm_free (include/docc_rocm_rt.h)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_copies_round_trip(rt):
    x = np.arange(100000, dtype=np.float64)
    y = np.zeros_like(x)
    p = rt.malloc(x.nbytes)
    rt.memcpy_h2d(p, x.ctypes.data, x.nbytes)
    rt.memcpy_d2h(y.ctypes.data, p, x.nbytes)
    rt.stream_sync()
    rt.free(p)
    assert np.array_equal(x, y)


def test_free_keeps_blocks_for_the_next_malloc_of_that_size(rt):
    rt.pool_trim()
    _, _, limit = rt.pool_stats()
    try:
        rt.pool_set_limit(1 << 30)
        a = rt.malloc(1000)               # rounded up to 1024
        b = rt.malloc(5 << 20)
        rt.free(a)
        rt.free(b)
        assert rt.pool_stats()[:2] == (1024 + (5 << 20), 2)
        assert rt.malloc(1024) == a       # same rounded size: the cached block
        assert rt.malloc(5 << 20) == b
        c = rt.malloc(5 << 20)            # the cache is empty for this size: a new block
        assert c not in (a, b) and rt.pool_stats()[:2] == (0, 0)
        for p in (a, b, c):
            rt.free(p)
        assert rt.pool_stats()[1] == 3
        # a block larger than what the cache may still hold goes back to the driver
        rt.pool_set_limit(8 << 20)        # shrinking trims
        assert rt.pool_stats()[:2] == (0, 0)
        big = rt.malloc(16 << 20)
        rt.free(big)
        assert rt.pool_stats()[:2] == (0, 0)
        # limit 0: no caching at all
        rt.pool_set_limit(0)
        p = rt.malloc(4096)
        rt.free(p)
        assert rt.pool_stats()[:2] == (0, 0)
    finally:
        rt.pool_set_limit(limit)


def test_cached_blocks_hold_no_stale_work(rt):
    """free() waits for the device before it keeps a block, so the next owner cannot race with a kernel of the last."""
    import torch
    n = 1 << 22
    src = torch.arange(n, dtype=torch.float32, device="cuda")
    p = rt.malloc(n * 4)
    rt.elementwise_unary("abs", 32, n, src.data_ptr(), p)     # enqueued, not awaited
    rt.free(p)
    q = rt.malloc(n * 4)
    assert q == p
    out = np.empty(n, np.float32)
    rt.memcpy_d2h(out.ctypes.data, q, n * 4)
    rt.stream_sync()
    rt.free(q)
    assert np.array_equal(out, np.arange(n, dtype=np.float32))


def test_blocks_freed_on_a_stream_come_back_in_stream_order(rt):
    """free_async records the release on the stream and does not wait; the next owner sees the block only behind that
    release: on the same stream by stream order, on another stream through an event wait, on the host after a wait."""
    import torch
    n = 1 << 24
    src = torch.arange(n, dtype=torch.float32, device="cuda")
    neg, neg2 = -src, -2 * src
    expected = np.arange(n, dtype=np.float32)
    a, b = rt.stream_create(), rt.stream_create()
    try:
        torch.cuda.synchronize()
        rt.pool_trim()
        # same stream: a chain of kernels into p, release, the block again, its contents are the chain's result
        p = rt.malloc_async(n * 4, a)
        for _ in range(8):
            rt.elementwise_unary("abs", 32, n, neg.data_ptr(), p, stream=a)
        rt.free_async(p, a)
        assert rt.pool_stats()[1] == 1                     # kept at once, nothing was waited for
        q = rt.malloc_async(n * 4, a)
        assert q == p
        out = np.empty(n, np.float32)
        rt.memcpy_d2h(out.ctypes.data, q, n * 4, a)
        rt.stream_sync(a)
        assert np.array_equal(out, expected)
        # another stream: its work on the block starts behind the first stream's
        for _ in range(8):
            rt.elementwise_unary("abs", 32, n, neg.data_ptr(), q, stream=a)
        rt.free_async(q, a)
        r = rt.malloc_async(n * 4, b)
        assert r == p
        rt.elementwise_unary("abs", 32, n, neg2.data_ptr(), r, stream=b)     # must land after the eight launches on a
        rt.memcpy_d2h(out.ctypes.data, r, n * 4, b)
        rt.stream_sync(b)
        rt.stream_sync(a)
        assert np.array_equal(out, expected * 2)
        # the host-ordered malloc waits for a release that is still pending
        for _ in range(8):
            rt.elementwise_unary("abs", 32, n, neg.data_ptr(), r, stream=b)
        rt.free_async(r, b)
        t = rt.malloc(n * 4)
        assert t == p
        rt.memcpy_d2h(out.ctypes.data, t, n * 4)           # the null stream does not wait for b by itself
        rt.stream_sync()
        assert np.array_equal(out, expected)
        rt.free(t)
        # a block freed the plain way is not pending: any stream takes it without an event
        assert rt.malloc_async(n * 4, b) == p
        rt.free_async(p, b)
    finally:
        rt.stream_sync(a)
        rt.stream_sync(b)
        rt.stream_destroy(a)
        rt.stream_destroy(b)
        rt.pool_trim()


def test_a_destroyed_stream_gives_its_partial_results_back(rt):
    """The two-launch kernels keep 8 MiB per stream they ran on; destroying the stream releases it."""
    import torch
    x = torch.randn(8192, 256, device="cuda")
    y = torch.empty(256, device="cuda")
    ref = x.double().sum(0)

    def once():
        s = rt.stream_create()
        rt.reduce("sum", 32, 1, 8192, 256, x.data_ptr(), y.data_ptr(), stream=s)      # few columns, long extent: sliced
        rt.stream_sync(s)
        rt.stream_destroy(s)

    once()
    torch.cuda.synchronize()
    assert float((y.double() - ref).abs().max() / ref.abs().max()) < 1e-5
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(12):
        once()
    torch.cuda.synchronize()
    assert free_before - torch.cuda.mem_get_info()[0] < (16 << 20), "partial-result buffers of destroyed streams were kept"


def test_uploads_from_memory_the_caller_pinned_go_straight_to_the_driver(rt):
    """Memory pinned by someone else (torch's pin_memory) is recognised: the upload is one asynchronous copy, and
    arrives intact."""
    import torch
    n = (24 << 20) + 3
    host = torch.randint(0, 255, (n,), dtype=torch.uint8).pin_memory()
    p = rt.malloc(n)
    rt.memcpy_h2d(p, host.data_ptr(), n)
    back = torch.empty(n, dtype=torch.uint8)
    rt.memcpy_d2h(back.data_ptr(), p, n)
    rt.stream_sync()
    rt.free(p)
    assert torch.equal(host, back)


def test_result_arrays_are_pinned_and_reused(rt):
    import gc
    rt.pinned_trim()
    small = rt.result_array((10, 10), np.float32)
    assert small.base is None                                    # below 1 MiB: ordinary memory
    a = rt.result_array((512, 1024), np.float64)                 # 4 MiB
    assert a.shape == (512, 1024) and a.dtype == np.float64 and a.flags.c_contiguous and a.flags.writeable
    a[:] = 3.0
    addr = a.ctypes.data
    # a device copy lands in it
    p = rt.malloc(a.nbytes)
    src = np.arange(a.size, dtype=np.float64).reshape(a.shape)
    rt.memcpy_h2d(p, src.ctypes.data, a.nbytes)
    rt.memcpy_d2h(a.ctypes.data, p, a.nbytes)
    rt.stream_sync()
    rt.free(p)
    assert np.array_equal(a, src)
    view = a[5:7]
    del a
    gc.collect()
    b = rt.result_array((512, 1024), np.float64)
    assert b.ctypes.data != addr                                  # a view still holds the first block
    del view
    gc.collect()
    c = rt.result_array((1024, 512), np.float64)
    assert c.ctypes.data == addr                                  # released with its last view, reused for the same size
    del b, c
    gc.collect()
    rt.pinned_trim()


def test_large_uploads_from_pageable_memory_are_staged_through_pinned_chunks(rt):
    """Uploads of 16 MiB and more from memory the runtime did not pin go through its ring of pinned 8 MiB chunks (helper
    threads fill them while earlier chunks travel); sizes that are no multiple of the chunk, sources the call may not
    keep, two uploads in a row, another stream, and pinned sources (straight to the driver) all arrive intact."""
    import ctypes
    rng = np.random.default_rng(5)
    for nbytes in (4 << 20, (33 << 20) + 13, (16 << 20) - 1, (16 << 20), (24 << 20) + 1):
        x = rng.integers(0, 256, nbytes, dtype=np.uint8)
        expected = x.copy()
        p = rt.malloc(nbytes)
        rt.memcpy_h2d(p, x.ctypes.data, nbytes)
        x[:] = 0                        # the source has been read when the call returns
        y = np.empty(nbytes, np.uint8)
        rt.memcpy_d2h(y.ctypes.data, p, nbytes)
        rt.stream_sync()
        assert np.array_equal(y, expected)
        rt.free(p)
    # a stream of its own, and a pinned source
    s = ctypes.c_void_p()
    rt.call("docc_rocm_stream_create", ctypes.byref(s))
    n = (20 << 20) + 5
    x = rng.integers(0, 256, n, dtype=np.uint8)
    hp = ctypes.c_void_p()
    rt.call("docc_rocm_host_malloc", ctypes.byref(hp), n)
    pinned = np.frombuffer((ctypes.c_uint8 * n).from_address(hp.value), dtype=np.uint8)
    pinned[:] = x[::-1]
    p, q = rt.malloc(n), rt.malloc(n)
    rt.memcpy_h2d(p, x.ctypes.data, n, s.value)
    rt.memcpy_h2d(q, hp.value, n, s.value)
    y, z = np.empty(n, np.uint8), np.empty(n, np.uint8)
    rt.memcpy_d2h(y.ctypes.data, p, n, s.value)
    rt.memcpy_d2h(z.ctypes.data, q, n, s.value)
    rt.stream_sync(s.value)
    assert np.array_equal(y, x) and np.array_equal(z, x[::-1])
    rt.free(p); rt.free(q)
    rt.call("docc_rocm_host_free", hp)
    rt.call("docc_rocm_stream_destroy", s)


@pytest.mark.parametrize("precision", [64, 32, 16, 116])
def test_mfma_probe_times_its_loop_and_nothing_else(rt, precision):
    """The ceiling probe's launch time must be its MFMA loop: twice the rounds take twice as long (operand
    set-up that costs as much as thousands of rounds once passed for matrix time), and the flop count it
    reports is 32 MFMAs per round and wave."""
    import statistics
    import torch
    ops = torch.randn(4096, device="cuda")
    sink = torch.empty(2 * 256 * 512, device="cuda")

    def timed(iters):
        flop = rt.mfma_probe(precision, 1, iters, ops.data_ptr(), sink.data_ptr())
        for _ in range(3):
            rt.mfma_probe(precision, 1, iters, ops.data_ptr(), sink.data_ptr())
        rt.device_sync()
        ts = []
        for _ in range(5):
            e0, e1 = rt.Event(), rt.Event()
            e0.record()
            rt.mfma_probe(precision, 1, iters, ops.data_ptr(), sink.data_ptr())
            e1.record()
            ts.append(e0.elapsed_ms(e1))
        return statistics.median(ts), flop

    for _ in range(20):   # clocks up
        rt.mfma_probe(precision, 1, 2000, ops.data_ptr(), sink.data_ptr())
    t1, f1 = timed(2000)
    t2, f2 = timed(4000)
    per_mfma = {64: 2048, 32: 4096, 16: 32768, 116: 16384}[precision]
    groups = f1 / (per_mfma * 32.0 * 2000 * 4)
    assert groups == int(groups) and groups >= 1 and f2 == 2 * f1
    assert 1.75 < t2 / t1 < 2.25, (t1, t2)
    assert torch.isfinite(sink[: int(groups) * 256]).all()
    with pytest.raises(rt.RocmRuntimeError):
        rt.mfma_probe(8, 1, 10, ops.data_ptr(), sink.data_ptr())
    with pytest.raises(rt.RocmRuntimeError):
        rt.mfma_probe(precision, 3, 10, ops.data_ptr(), sink.data_ptr())


def test_clock_probe_reports_a_plausible_shader_clock(rt):
    import torch
    out = torch.zeros(1, device="cuda")
    rt.clock_probe(200, out.data_ptr())
    rt.device_sync()
    assert 100.0 < float(out.item()) < 3000.0
    with pytest.raises(rt.RocmRuntimeError):
        rt.clock_probe(0, out.data_ptr())


@pytest.mark.parametrize("nbytes", [16, 16 * 1023, 16 * 1024, 16 * 1025, 16 * 777777])
def test_copy_bytes_moves_exactly_the_bytes_asked_for(rt, nbytes):
    import torch
    x = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda")
    y = torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")
    rt.copy_bytes(nbytes, x.data_ptr(), y.data_ptr())
    rt.device_sync()
    assert torch.equal(x, y[:nbytes]) and int(y[nbytes:].sum().item()) == 0
    with pytest.raises(rt.RocmRuntimeError):
        rt.copy_bytes(24, x.data_ptr(), y.data_ptr())
