"""Runs of runtime calls recorded as HIP graphs (include/docc_rocm_rt.h, docc_rocm_graph_*): a replay gives the bits
of the same calls made one by one, every time, with other work on the device between the replays; the device blocks a
record allocates stay with it; calls that cannot be recorded say so."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import docc_amd.torch as docc_torch
from docc_amd.runtime import RocmRuntimeError

pytestmark = pytest.mark.gpu


def chain(rt, m, n, k, a, b, bias, out, stream=0):
    """softmax(relu(a @ b + bias row)) with a temporary from the block cache, then a byte fill of the temporary's
    first row: GEMM, a fused elementwise kernel, the softmax and a fill, around a cached allocation."""
    tmp = rt.malloc_async(m * n * 4, stream)
    rt.sgemm(m, n, k, 1.0, a, k, b, n, 0.0, tmp, n, stream=stream)
    rt.elementwise_fused(32, (m, n), "add", tmp, (m, n), bias, (n,), ["relu"], tmp, stream=stream)
    rt.softmax(32, m, n, 1, tmp, out, stream=stream)
    rt.free_async(tmp, stream)
    return tmp


# the tiles; sixteen rows against a wide matrix (B straight into the MFMA, the parts' products in the stream's buffer); the same
# kernels with 16 MiB of parts, which take a block of the block cache inside the record
@pytest.mark.parametrize("m,n,k,parts,blocks", [(384, 512, 256, None, 1), (16, 4096, 2048, None, 1), (32, 8192, 4096, "16", 2)])
def test_replays_give_the_bits_of_the_eager_calls(rt, monkeypatch, m, n, k, parts, blocks):
    if parts:
        monkeypatch.setenv("DOCC_ROCM_GEMM_SPLITK", parts)
    g = torch.Generator(device="cpu").manual_seed(11)
    a = torch.randn(m, k, generator=g).cuda()
    b = torch.randn(k, n, generator=g).cuda()
    bias = torch.randn(n, generator=g).cuda()
    out = torch.empty(m, n, device="cuda")
    eager = torch.empty(m, n, device="cuda")
    other_in = torch.randn(1024, 1024, generator=g).cuda()
    other_out = torch.empty_like(other_in)
    torch.cuda.synchronize()

    stream = rt.stream_create()
    rt.set_default_stream(stream)
    try:
        chain(rt, m, n, k, a.data_ptr(), b.data_ptr(), bias.data_ptr(), out.data_ptr())   # null stream -> `stream`
        rt.stream_sync()
        first = out.clone()
        with rt.Graph.capture(stream) as graph:
            held = chain(rt, m, n, k, a.data_ptr(), b.data_ptr(), bias.data_ptr(), out.data_ptr())
            rt.memset(out.data_ptr(), 0, n * 4 + 3)          # a fill inside the record: row 0 and three bytes more
    finally:
        rt.set_default_stream(0)
    assert graph.handle
    # recorded, not run: `out` still holds the run before the record
    torch.cuda.synchronize()
    assert torch.equal(out, first)
    # the temporary belongs to the graph: the cache hands the next caller another block
    p = rt.malloc(m * n * 4)
    assert p != held
    rt.free(p)

    for replay in range(4):
        a.copy_(torch.randn(m, k, generator=g))
        bias.copy_(torch.randn(n, generator=g))
        torch.cuda.synchronize()
        chain(rt, m, n, k, a.data_ptr(), b.data_ptr(), bias.data_ptr(), eager.data_ptr())
        rt.stream_sync()
        expect = eager.clone()
        expect.view(-1).view(torch.uint8)[: n * 4 + 3] = 0
        out.fill_(-1.0)
        # other work of the program between the replays, on the null stream, and a synchronization
        rt.softmax(32, 1024, 1024, 1, other_in.data_ptr(), other_out.data_ptr())
        rt.device_sync()
        graph.launch()
        rt.stream_sync(stream)
        assert torch.equal(out, expect), f"replay {replay}"
    rows = torch.softmax(other_in.double(), dim=1)
    assert (other_out.double() - rows).abs().max().item() < 1e-6

    cached_before = rt.pool_stats()[1]
    graph.destroy()
    assert rt.pool_stats()[1] == cached_before + blocks     # the temporary (and the block of parts) are back in the cache
    rt.stream_destroy(stream)


def test_blocks_freed_inside_a_record_serve_its_later_allocations(rt):
    n = 1 << 16
    x = torch.arange(n, dtype=torch.float32, device="cuda") - n / 2
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    stream = rt.stream_create()
    with rt.Graph.capture(stream) as graph:
        t1 = rt.malloc_async(n * 4)
        rt.elementwise_unary("abs", 32, n, x.data_ptr(), t1)
        rt.free_async(t1)
        t2 = rt.malloc(n * 4)                                  # the plain pair as well: nothing waits inside a record
        rt.elementwise_unary("sqrt", 32, n, t2, y.data_ptr())
        rt.free(t2)
    assert t1 == t2
    for _ in range(2):
        y.zero_()
        torch.cuda.synchronize()
        graph.launch()
        rt.stream_sync(stream)
        assert torch.equal(y, torch.sqrt(torch.abs(x)))
    graph.destroy()
    rt.stream_destroy(stream)


def test_calls_that_cannot_be_recorded_refuse(rt):
    with pytest.raises(RocmRuntimeError, match="null stream"):
        rt.call("docc_rocm_graph_capture_begin", 0)
    with pytest.raises(RocmRuntimeError, match="no capture"):
        import ctypes
        h = ctypes.c_void_p()
        rt.call("docc_rocm_graph_capture_end", ctypes.byref(h))
    x = torch.ones(1000, dtype=torch.float64, device="cuda")
    torch.cuda.synchronize()
    stream = rt.stream_create()
    with rt.Graph.capture(stream) as graph:
        with pytest.raises(RocmRuntimeError, match="cannot be captured"):
            rt.dot(64, 1000, x.data_ptr(), 1, x.data_ptr(), 1)
        with pytest.raises(RocmRuntimeError, match="already open"):
            rt.call("docc_rocm_graph_capture_begin", stream)
        with pytest.raises(RocmRuntimeError, match="capture is open"):
            rt.set_default_stream(0)
    graph.launch()                                             # an empty record replays as nothing
    rt.stream_sync(stream)
    graph.destroy()
    rt.stream_destroy(stream)
    assert rt.dot(64, 1000, x.data_ptr(), 1, x.data_ptr(), 1) == 1000.0


def test_a_compiled_torch_program_replays_as_one_submission():
    """LayerNorm -> Linear -> GELU -> Linear + residual: eight kernels per call, one graph launch per replay."""
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.LayerNorm(256)
            self.fc1 = torch.nn.Linear(256, 1024)
            self.act = torch.nn.GELU()
            self.fc2 = torch.nn.Linear(1024, 256)

        def forward(self, x):
            return x + self.fc2(self.act(self.fc1(self.norm(x))))

    torch.manual_seed(5)
    model = Block().cuda()
    x = torch.randn(8, 128, 256, device="cuda")
    program = docc_torch.compile_torch(model, x, target="rocm")
    recorded = program.record(x)
    assert recorded.inputs[0].data_ptr() == x.data_ptr()
    for replay in range(3):
        x.copy_(torch.randn(8, 128, 256) * (replay + 1))
        torch.cuda.synchronize()
        expect = program(x).clone()                           # the same kernels, launched one by one on the null stream
        torch.cuda.synchronize()
        recorded.result.fill_(float("nan"))
        torch.cuda.synchronize()
        got = recorded.replay()
        assert torch.equal(got, expect), f"replay {replay}"
    with torch.no_grad():
        ref = model.double()(x.double())
    assert ((recorded.result.double() - ref).abs().max() / ref.abs().max()).item() <= 1e-5
    recorded.close()
    # a program compiled for host arrays waits for its copies and cannot be recorded
    host = docc_torch.compile_torch(Block(), x.cpu(), target="rocm")
    with pytest.raises(ValueError, match="device tensors"):
        host.record(x.cpu())
