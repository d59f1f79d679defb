"""`@native` and the torch front end up to (not including) execution: lowering to library nodes,
argument order of the generated function, the compile cache rule, target-registry hooks. Modelled
on the reference's python/tests/python/program/test_caching.py:6-57 and
python/tests/python/targets/test_overrides.py:9-72."""
import math

import numpy as np
import pytest
import scipy.special
import torch
from pathlib import Path

import docc_amd.torch as docc_torch
from docc_amd.python import (conv2d, erf, native, register_target, register_target_overrides, relu, sigmoid, softmax,
                             unregister_target)


@pytest.fixture(autouse=True)
def tmp_docc(tmp_path, monkeypatch):
    monkeypatch.setenv("DOCC_TMP", str(tmp_path / "docc"))


def test_matmul_lowers_to_one_gemm_with_reference_argument_order():
    @native(target="rocm")
    def matmul_op(a, b):
        return a @ b

    a = np.random.rand(10, 10)
    sdfg = matmul_op.to_sdfg(a, a)
    # user parameters, then one shape symbol (all dims equal), then the output pointer
    assert sdfg.arguments == ["a", "b", "_s0", "_docc_ret_0"]
    assert sdfg.name == "matmul_op_sdfg"
    (node,) = sdfg.library_nodes()
    assert node["code"] == "GEMM" and node["precision"] == ord("d") and node["m"] == node["n"] == node["k"] == "_s0"
    sdfg = matmul_op.to_sdfg(np.zeros((5, 7), np.float32), np.zeros((7, 3), np.float32))
    assert sdfg.arguments == ["a", "b", "_s0", "_s1", "_s2", "_docc_ret_0"]
    node = sdfg.library_nodes()[0]
    assert (node["precision"], node["m"], node["n"], node["k"], node["lda"], node["ldb"], node["ldc"]) == (ord("s"), "_s0", "_s2", "_s1", "_s1", "_s2", "_s2")


def test_other_matmul_spellings_and_polybench_gemm():
    @native
    def np_matmul(a, b):
        return np.matmul(a, b)

    @native
    def dot_t(a, b):
        return np.dot(a, b.T)

    @native
    def gemm(alpha, beta, C, A, B):
        C[:] = alpha * A @ B + beta * C

    @native
    def into_arg(A, B, C):
        C = A @ B

    a = np.zeros((6, 6))
    assert np_matmul.to_sdfg(a, a).library_nodes()[0]["code"] == "GEMM"
    batched = np_matmul.to_sdfg(np.zeros((4, 5, 6), np.float32), np.zeros((4, 6, 3), np.float32))
    (node,) = batched.library_nodes()
    assert node["code"] == "ml::MatMul" and node["shape_a"] == ["_s0", "_s1", "_s2"] and node["shape_b"] == ["_s0", "_s2", "_s3"]
    assert batched._data["root"]["children"][0]["dataflow"]["outputs"] == [{"connector": "Y", "data": "_docc_ret_0"}]
    assert dot_t.to_sdfg(a, a).library_nodes()[0]["trans_b"] == 112
    sdfg = gemm.to_sdfg(1.5, 1.2, a, a, a)
    assert sdfg.arguments == ["alpha", "beta", "C", "A", "B", "_s0"]     # in place: no return buffer
    df = sdfg._data["root"]["children"][0]["dataflow"]
    binds = {b["connector"]: b.get("data") for b in df["inputs"]}
    assert binds == {"__A": "A", "__B": "B", "__C": "C", "__alpha": "alpha", "__beta": "beta"}
    assert len(sdfg.library_nodes()) == 1                                  # exactly one GEMM node, no loops
    assert into_arg.to_sdfg(a, a, a).arguments == ["A", "B", "C", "_s0"]


def test_softmax_forms_and_conv():
    @native
    def sp(x):
        return scipy.special.softmax(x, axis=-1)

    @native
    def decomposed(x):
        tmp_max = np.max(x, axis=-1, keepdims=True)
        tmp_out = np.exp(x - tmp_max)
        tmp_sum = np.sum(tmp_out, axis=-1, keepdims=True)
        return tmp_out / tmp_sum

    @native
    def conv(x, w, b):
        return conv2d(x, w, b, stride=1, padding=1)

    x = np.zeros((4, 3, 8, 8), np.float32)
    for prog in (sp, decomposed):
        (node,) = prog.to_sdfg(x).library_nodes()
        assert node["code"] == "ml::Softmax" and node["axes"] == [-1] and node["shape"] == ["_s0", "_s1", "_s2", "_s2"]
    (node,) = conv.to_sdfg(x, np.zeros((5, 3, 3, 3), np.float32), np.zeros(5, np.float32)).library_nodes()
    assert node["code"] == "ml::Conv" and node["pads"] == ["1", "1", "1", "1"] and node["has_bias"] is True
    # the marker functions compute the same thing in plain numpy
    y = np.random.rand(3, 7).astype(np.float32)
    assert np.allclose(softmax(y), scipy.special.softmax(y, axis=-1))
    xs, ws = np.random.rand(1, 2, 5, 5), np.random.rand(3, 2, 3, 3)
    ref = torch.nn.functional.conv2d(torch.from_numpy(xs), torch.from_numpy(ws), padding=1).numpy()
    assert np.allclose(conv2d(xs, ws, padding=1), ref)


def test_unsupported_code_is_rejected_not_run_on_the_cpu():
    @native
    def loop(a, b):
        for i in range(a.shape[0]):
            b[i] = a[i]

    @native
    def power(a, b):
        return a ** b

    @native
    def modulo(a, b):
        return a % b

    @native
    def add(a, b):
        return a + b

    a = np.zeros(4)
    with pytest.raises(NotImplementedError, match="rocm target"):
        loop.to_sdfg(a, a)
    with pytest.raises(NotImplementedError):
        modulo.to_sdfg(a, a)
    assert [n["code"] for n in power.to_sdfg(a, a).library_nodes()] == ["ml::Pow"]
    with pytest.raises(NotImplementedError):          # integer arrays have no elementwise kernels
        add.to_sdfg(np.zeros(4, np.int64), np.zeros(4, np.int64))
    with pytest.raises(ValueError, match="broadcast"):
        add.to_sdfg(np.zeros((4, 3)), np.zeros((4, 2)))


def test_elementwise_expressions_lower_to_tensor_nodes():
    @native
    def dense(x, w, b):
        return relu(x @ w + b)

    @native
    def mixed(x, y, s):
        return np.tanh(x * y - 0.5) / (s * y)

    @native
    def clip(x, y):
        return np.minimum(np.maximum(x, 0), np.abs(y))

    @native
    def in_place(x, y):
        y[:] = np.exp(x) + y

    @native
    def negated(x, y):
        return np.exp(-np.abs(x)) + -2.5

    x, w, b = np.zeros((8, 5), np.float32), np.zeros((5, 3), np.float32), np.zeros(3, np.float32)
    sdfg = dense.to_sdfg(x, w, b)
    codes = [n["code"] for n in sdfg.library_nodes()]
    assert codes == ["GEMM", "ml::Broadcast", "ml::Add", "ml::ReLU"]
    bc = sdfg.library_nodes()[1]
    assert bc["input_shape"] == ["1", "_s2"] and bc["output_shape"] == ["_s0", "_s2"]
    blocks = [c["dataflow"] for c in sdfg._data["root"]["children"]]
    assert {i["connector"] for i in blocks[2]["inputs"]} == {"A", "B"} and blocks[2]["outputs"][0]["connector"] == "C"
    assert blocks[3]["inputs"][0]["connector"] == "X" and blocks[3]["outputs"][0] == {"connector": "Y", "data": "_docc_ret_0"}
    # intermediates are transients of the generated function, only the result is an argument
    assert sdfg.arguments == ["x", "w", "b", "_s0", "_s1", "_s2", "_docc_ret_0"]

    z = np.zeros((4, 6))
    sdfg = mixed.to_sdfg(z, z, 2.0)
    assert [n["code"] for n in sdfg.library_nodes()] == ["ml::Mul", "ml::Sub", "ml::Tanh", "ml::Mul", "ml::Div"]
    blocks = [c["dataflow"] for c in sdfg._data["root"]["children"]]
    sub_b = next(i for i in blocks[1]["inputs"] if i["connector"] == "B")
    assert sub_b == {"connector": "B", "constant": "0.5", "type": "Double"}
    mul_s = {i["connector"]: i for i in blocks[3]["inputs"]}
    assert mul_s["B"] == {"connector": "B", "data": "s"} and mul_s["A"]["data"] == "y"   # scalar argument by value
    assert all(n["element_type"] == "Double" for n in sdfg.library_nodes())

    assert [n["code"] for n in clip.to_sdfg(z, z).library_nodes()] == ["ml::ReLU", "ml::Abs", "ml::Minimum"]
    # a sign in front of an array is the product with -1.0; in front of a literal it is the literal's
    sdfg = negated.to_sdfg(z, z)
    assert [n["code"] for n in sdfg.library_nodes()] == ["ml::Abs", "ml::Mul", "ml::Exp", "ml::Add"]
    blocks = [c["dataflow"] for c in sdfg._data["root"]["children"]]
    assert {i["connector"]: i.get("constant") for i in blocks[1]["inputs"]}["B"] == "-1.0"
    assert {i["connector"]: i.get("constant") for i in blocks[3]["inputs"]}["B"] == "-2.5"
    sdfg = in_place.to_sdfg(z, z)
    assert sdfg.arguments == ["x", "y", "_s0", "_s1"]
    assert sdfg._data["root"]["children"][1]["dataflow"]["outputs"][0]["data"] == "y"
    # the marker functions are plain numpy outside @native
    v = np.linspace(-3, 3, 7)
    assert np.allclose(relu(v), np.maximum(v, 0)) and np.allclose(sigmoid(v), scipy.special.expit(v))
    assert np.allclose(erf(v), scipy.special.erf(v))


def test_compile_cache_follows_shape_structure():
    @native
    def mm(a, b):
        return a @ b

    c1 = mm.compile(np.random.rand(16, 16), np.random.rand(16, 16))
    c2 = mm.compile(np.random.rand(32, 32), np.random.rand(32, 32))   # same structure, other values
    assert c1 is c2
    c3 = mm.compile(np.random.rand(16, 8), np.random.rand(8, 16))     # different structure
    assert c3 is not c1 and c3.sdfg.arguments == ["a", "b", "_s0", "_s1", "_docc_ret_0"]
    c4 = mm.compile(np.zeros((16, 16), np.float32), np.zeros((16, 16), np.float32))   # different dtype
    assert c4 is not c1
    assert c1.get_return_shape(np.zeros((5, 5)), np.zeros((5, 5))) == (5, 5)


def test_target_overrides_are_consulted(capsys):
    calls = []

    def schedule(sdfg, category, options):
        calls.append(("schedule", category, sorted(options)))
        sdfg.schedule("rocm", category, False, {"offload": "node"})

    def schedule_legacy(sdfg, category):
        calls.append(("legacy", category))
        sdfg.schedule("rocm", category, False)

    def compile_(sdfg, out_dir, inst_mode, capture, options):
        calls.append(("compile", inst_mode, capture))
        return sdfg._compile(out_dir, "rocm", inst_mode, capture)

    register_target_overrides("special", schedule, compile_)
    register_target("special_legacy", schedule_legacy)
    try:
        @native(target="special", category="desktop")
        def f(a, b):
            return a @ b

        @native(target="special_legacy")
        def g(a, b):
            return a @ b

        a = np.zeros((4, 4), np.float32)
        f.compile(a, a)
        g.compile(a, a)
        out = capsys.readouterr().out
        assert "is not supported" not in out
        assert calls == [("schedule", "desktop", ["remote_tuning"]), ("compile", "", False), ("legacy", "server")]
        assert f.last_sdfg.library_nodes()[0]["implementation_type"] == "ROCMWithTransfers"
    finally:
        unregister_target("special")
        unregister_target("special_legacy")

    @native(target="openmp")
    def h(a, b):
        return a @ b

    with pytest.raises(NotImplementedError):
        h.compile(np.zeros((4, 4)), np.zeros((4, 4)))
    assert "Target 'openmp' is not supported" in capsys.readouterr().out


class Attn(torch.nn.Module):
    def forward(self, q, k, v):
        s = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(q.shape[-1])
        return torch.matmul(torch.softmax(s, dim=-1), v)


def test_torch_lowering_recognises_attention_conv_and_matmul():
    q = torch.randn(2, 4, 128, 64).bfloat16()
    sdfg = docc_torch.TorchProgram(Attn(), (q, q, q), target="rocm").to_sdfg()
    assert sdfg.name == "__docc_Attn" and sdfg.arguments == ["q", "k", "v", "_docc_ret_0"]
    (node,) = sdfg.library_nodes()
    assert node["code"] == "ml::Attention" and float(node["scale"]) == 0.125 and node["shape_q"] == ["2", "4", "128", "64"]
    assert sdfg.metadata("return_shape") == "[2,4,128,64]"

    class Sdpa(torch.nn.Module):
        def forward(self, q, k, v):
            return torch.nn.functional.scaled_dot_product_attention(q, k, v)

    assert docc_torch.TorchProgram(Sdpa(), (q, q, q), target="rocm").to_sdfg().library_nodes()[0]["code"] == "ml::Attention"

    class Conv(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = torch.nn.Conv2d(8, 16, 3, padding=1)

        def forward(self, x):
            return self.conv(x)

    sdfg = docc_torch.compile_torch(Conv(), torch.randn(2, 8, 14, 14), target="rocm").to_sdfg()
    assert sdfg.arguments == ["x", "conv_weight", "conv_bias", "_docc_ret_0"]
    assert sdfg.library_nodes()[0]["pads"] == ["1", "1", "1", "1"]

    class MM(torch.nn.Module):
        def forward(self, a, b):
            return torch.softmax(a @ b.t(), dim=-1)

    sdfg = docc_torch.TorchProgram(MM(), (torch.randn(8, 6), torch.randn(5, 6)), target="rocm").to_sdfg()
    assert [n["code"] for n in sdfg.library_nodes()] == ["GEMM", "ml::Softmax"] and sdfg.library_nodes()[0]["trans_b"] == 112

    class Unsupported(torch.nn.Module):
        def forward(self, a):
            return torch.cumsum(a, 0)

    with pytest.raises(NotImplementedError):
        docc_torch.TorchProgram(Unsupported(), torch.randn(4), target="rocm").to_sdfg()


def test_torch_lowering_of_elementwise_operations_and_linear():
    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = torch.nn.Linear(12, 20)
            self.act = torch.nn.ReLU()
            self.fc2 = torch.nn.Linear(20, 6, bias=False)

        def forward(self, x):
            return torch.tanh(self.fc2(self.act(self.fc1(x)))) * 0.5

    x = torch.randn(4, 7, 12)
    sdfg = docc_torch.TorchProgram(Mlp(), (x,), target="rocm").to_sdfg()
    codes = [n["code"] for n in sdfg.library_nodes()]
    assert codes == ["GEMM", "ml::Broadcast", "ml::Add", "ml::ReLU", "GEMM", "ml::Tanh", "ml::Mul"]
    g = sdfg.library_nodes()[0]
    assert (g["m"], g["n"], g["k"], g["trans_b"], g["ldb"]) == ("28", "20", "12", 112, "12")    # rows flattened, weight [N, K] transposed
    assert sdfg.library_nodes()[1]["input_shape"] == ["1", "1", "20"] and sdfg.metadata("return_shape") == "[4,7,6]"
    last = sdfg._data["root"]["children"][-1]["dataflow"]
    assert {"connector": "B", "constant": "0.5", "type": "Float"} in last["inputs"] and last["outputs"][0]["data"] == "_docc_ret_0"

    class Arith(torch.nn.Module):
        def forward(self, a, b):
            return torch.maximum(a - b, b / 3) + torch.sigmoid(a).exp() * torch.sqrt(b.abs())

    sdfg = docc_torch.TorchProgram(Arith(), (torch.randn(5, 3, dtype=torch.float64), torch.randn(3, dtype=torch.float64)),
                                   target="rocm").to_sdfg()
    codes = [n["code"] for n in sdfg.library_nodes()]
    assert codes == ["ml::Broadcast", "ml::Sub", "ml::Div", "ml::Broadcast", "ml::Maximum", "ml::Sigmoid", "ml::Exp", "ml::Abs",
                     "ml::Sqrt", "ml::Broadcast", "ml::Mul", "ml::Add"]
    assert all(n["element_type"] == "Double" for n in sdfg.library_nodes())

    class Norm(torch.nn.Module):
        def forward(self, x):
            return x - x.mean(dim=-1, keepdim=True)

    sdfg = docc_torch.TorchProgram(Norm(), (torch.randn(4, 5, 6),), target="rocm").to_sdfg()
    assert [n["code"] for n in sdfg.library_nodes()] == ["ml::Mean", "ml::Broadcast", "ml::Sub"]
    assert sdfg.library_nodes()[0]["axes"] == [2] and sdfg.library_nodes()[0]["keepdims"] is True

    class Pool(torch.nn.Module):
        def forward(self, x):
            return torch.sum(x, (2, 3)), x.amax(dim=1)

    sdfg = docc_torch.TorchProgram(Pool(), (torch.randn(2, 3, 4, 5),), target="rocm").to_sdfg()
    assert [(n["code"], n["axes"]) for n in sdfg.library_nodes()] == [("ml::Sum", [2, 3]), ("ml::Max", [1])]

    class Ints(torch.nn.Module):
        def forward(self, a):
            return a + a

    with pytest.raises(NotImplementedError):
        docc_torch.TorchProgram(Ints(), torch.ones(4, dtype=torch.int32), target="rocm").to_sdfg()


def test_torch_lowering_of_activations_with_scalar_operands():
    class Acts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.elu = torch.nn.ELU(alpha=0.7)
            self.leaky = torch.nn.LeakyReLU(0.2)
            self.hs = torch.nn.Hardsigmoid()

        def forward(self, x):
            return self.hs(self.leaky(self.elu(x))) + torch.nn.functional.leaky_relu(x) + torch.nn.functional.elu(x, alpha=1.5)

    sdfg = docc_torch.TorchProgram(Acts(), (torch.randn(4, 6),), target="rocm").to_sdfg()
    codes = [n["code"] for n in sdfg.library_nodes()]
    assert codes == ["ml::Elu", "ml::LeakyReLU", "ml::HardSigmoid", "ml::LeakyReLU", "ml::Add", "ml::Elu", "ml::Add"]
    flows = [c["dataflow"] for c in sdfg._data["root"]["children"]]
    operands = lambda f: {b["connector"]: b.get("constant") for b in f["inputs"] if "constant" in b}
    assert operands(flows[0]) == {"alpha": "0.7"} and operands(flows[1]) == {"alpha": "0.2"}
    assert operands(flows[2]) == {"alpha": repr(1.0 / 6.0), "beta": "0.5"}
    assert operands(flows[3]) == {"alpha": "0.01"} and operands(flows[5]) == {"alpha": "1.5"}
    sdfg.schedule("rocm")          # the mapper takes all of them
    assert sdfg.loop_report()["ml::Elu::ROCMWithoutTransfers"] == 2


def test_torch_backend_is_registered_and_reads_global_options():
    import torch._dynamo

    assert "docc" in torch._dynamo.list_backends(None)
    docc_torch.set_backend_options(target="rocm", category="server")
    assert docc_torch._backend_options == {"target": "rocm", "category": "server"}
    captured = {}

    def schedule(sdfg, category, options):
        captured["options"] = options
        sdfg.schedule("rocm", category, False, options)

    register_target_overrides("probe", schedule, None)
    try:
        docc_torch.set_backend_options(target="probe")
        program = docc_torch.TorchProgram(Attn(), None, target="probe")
        q = torch.randn(1, 1, 64, 64).bfloat16()
        compiled = program.compile(q, q, q)
        assert captured["options"] == {"offload": "function"}      # CPU tensors: the generated code moves the data
        assert program.last_sdfg.loop_report()["H2D"] == 3 and program.last_sdfg.loop_report()["D2H"] == 1
        assert program.compile(q, q, q) is compiled                 # cached per shapes/dtypes/device
    finally:
        unregister_target("probe")
        docc_torch.set_backend_options(target="rocm")


def test_torch_models_of_one_name_and_shape_get_libraries_of_their_own(tmp_path, monkeypatch):
    """Two different models with the same class name and input shapes (under torch.compile every graph is a
    "GraphModule"): folder and library path differ, so loading the second cannot return the first's handle
    (reference mlir/docc/torch/__init__.py:110-131)."""
    monkeypatch.setenv("DOCC_TMP", str(tmp_path))

    def make(fn):
        return type("Net", (torch.nn.Module,), {"forward": lambda self, x: fn(x)})()

    x = torch.randn(4, 8)
    first = docc_torch.TorchProgram(make(torch.tanh), None, target="rocm").compile(x)
    second = docc_torch.TorchProgram(make(torch.relu), None, target="rocm").compile(x)
    assert first.sdfg.name == second.sdfg.name
    assert first.lib_path != second.lib_path and Path(first.lib_path).parent != Path(second.lib_path).parent
    assert first.lib._handle != second.lib._handle
    codes = [c.sdfg.library_nodes() for c in (first, second)]
    assert any(n["code"] == "ml::Tanh" for n in codes[0]) and any(n["code"] == "ml::ReLU" for n in codes[1])
    # the same model again maps to the same place
    again = docc_torch.TorchProgram(make(torch.tanh), None, target="rocm").compile(x)
    assert again.lib_path == first.lib_path


def test_reductions_and_softmax_pieces_used_on_their_own():
    @native
    def stats(x):
        return np.sum(x, axis=1), x.max(axis=(1, 2), keepdims=True), np.mean(x), np.min(x, axis=0)

    @native
    def normalise(x):
        m = np.max(x, axis=-1, keepdims=True)
        e = np.exp(x - m)
        return e / np.sum(e, axis=-1, keepdims=True), m          # the softmax node, and the maximum as a value of its own

    @native
    def centred(x):
        return x - np.mean(x, axis=0, keepdims=True)

    x = np.zeros((4, 5, 6), np.float32)
    sdfg = stats.to_sdfg(x)
    nodes = sdfg.library_nodes()
    assert [(n["code"], n["axes"], n["keepdims"]) for n in nodes] == [("ml::Sum", [1], False), ("ml::Max", [1, 2], True),
                                                                      ("ml::Mean", [0, 1, 2], False), ("ml::Min", [0], False)]
    assert all(n["shape"] == ["_s0", "_s1", "_s2"] and n["element_type"] == "Float" for n in nodes)
    assert sdfg.arguments == ["x", "_s0", "_s1", "_s2", "_docc_ret_0", "_docc_ret_1", "_docc_ret_2", "_docc_ret_3"]
    assert [n["code"] for n in normalise.to_sdfg(x).library_nodes()] == ["ml::Softmax", "ml::Max"]
    sdfg = centred.to_sdfg(np.zeros((7, 3)))
    assert [n["code"] for n in sdfg.library_nodes()] == ["ml::Mean", "ml::Broadcast", "ml::Sub"]
    assert sdfg.library_nodes()[1]["input_shape"] == ["1", "_s1"]

    @native
    def scattered(x):
        return np.sum(x, axis=(0, 2))

    (node,) = scattered.to_sdfg(x).library_nodes()       # axes in two blocks: one node, the dispatcher chains the blocks
    assert node["code"] == "ml::Sum" and node["axes"] == [0, 2]
    with pytest.raises(ValueError, match="out of bounds"):
        native(_bad_axis).to_sdfg(x)


def _bad_axis(x):
    return np.sum(x, axis=5)


def test_transposes_lower_to_a_gemm_flag_or_a_transpose_node():
    @native
    def gram(a):
        return a.T @ a                        # operand of a product: the flag of the GEMM, no node

    @native
    def flipped(a, b):
        return a.T + b                        # used as an array: ml::Transpose

    @native
    def permuted(x):
        return np.transpose(x, (2, 0, 1)) * 2.0

    @native
    def reversed_axes(x):
        return np.exp(x.T)                    # rank 3: axes reversed

    @native
    def swapped(x):
        return np.swapaxes(x, 0, 1)

    a = np.zeros((6, 4))
    g = gram.to_sdfg(a).library_nodes()
    assert [n["code"] for n in g] == ["GEMM"] and g[0]["trans_a"] == 112 and g[0]["trans_b"] == 111
    f = flipped.to_sdfg(a, np.zeros((4, 6))).library_nodes()
    assert [n["code"] for n in f] == ["ml::Transpose", "ml::Add"] and f[0]["perm"] == [1, 0]
    x = np.zeros((3, 4, 5), np.float32)
    p = permuted.to_sdfg(x).library_nodes()
    assert [n["code"] for n in p] == ["ml::Transpose", "ml::Mul"] and p[0]["perm"] == [2, 0, 1]
    assert reversed_axes.to_sdfg(x).library_nodes()[0]["perm"] == [2, 1, 0]
    s = swapped.to_sdfg(x)
    assert s.library_nodes()[0]["perm"] == [1, 0, 2]
    @native
    def repeated_axis(x):
        return np.transpose(x, (0, 0, 1))

    with pytest.raises(ValueError, match="axes"):
        repeated_axis.to_sdfg(x)


def test_return_annotation_puts_the_outputs_first():
    """With a return annotation the reference declares `_docc_ret_<i>` before it looks at the parameters
    (python/docc/python/python_program.py:515-524): the outputs lead the argument list of the generated function."""
    from typing import Annotated, Tuple

    @native(target="rocm")
    def annotated(a, b) -> Annotated[np.ndarray, (None, None), np.float64]:
        return a @ b

    a = np.random.rand(6, 6)
    sdfg = annotated.to_sdfg(a, a)
    assert sdfg.arguments == ["_docc_ret_0", "a", "b", "_s0"]
    sdfg.schedule("rocm")
    src = Path(sdfg.generate(str(Path(__import__("os").environ["DOCC_TMP"]) / "annotated"))["source"]).read_text()
    assert 'extern "C" void annotated_sdfg(double *_docc_ret_0, double *a, double *b, int64_t _s0)' in src

    @native(target="rocm")
    def two(a, b) -> Tuple[Annotated[np.ndarray, (None, None), np.float32], Annotated[np.ndarray, (None, None), np.float32]]:
        return a @ b, relu(a)

    f = np.zeros((4, 4), np.float32)
    assert two.to_sdfg(f, f).arguments == ["_docc_ret_0", "_docc_ret_1", "a", "b", "_s0"]

    # an element type other than the declared one is an error, not a silent reinterpretation
    with pytest.raises(TypeError, match="declares Double for output _docc_ret_0, the returned value is Float"):
        annotated.to_sdfg(f, f)

    # an annotation that maps to nothing leaves the outputs to the body, as without one
    @native(target="rocm")
    def loose(a, b) -> "whatever":
        return a @ b

    assert loose.to_sdfg(a, a).arguments == ["a", "b", "_s0", "_docc_ret_0"]


def test_bf16_products_lower_to_the_gemm_with_float32_accumulation():
    """bf16 operands reach GEMM precision `b` (float32 accumulate and result) from both front ends: `@native` through a
    parameter annotation on arrays of the 16-bit words (the reference carries bf16 across ctypes as c_uint16,
    compiled_sdfg.py:28-31), torch through `(a @ b).float()` or `a.float() @ b.float()`."""
    from typing import Annotated, Any

    from docc_amd.python import bfloat16

    @native(target="rocm")
    def mm(a: Annotated[np.ndarray, ("M", "K"), bfloat16], b: np.ndarray[Any, np.dtype[bfloat16]]):
        return a @ b

    a, b = np.zeros((64, 32), np.uint16), np.zeros((32, 48), np.uint16)
    sdfg = mm.to_sdfg(a, b)
    (node,) = sdfg.library_nodes()
    assert node["code"] == "GEMM" and node["precision"] == ord("b")
    elements = {k: v["element"] for k, v in sdfg.containers.items()}
    assert elements["a"] == elements["b"] == "BFloat" and elements["_docc_ret_0"] == "Float"
    assert "BFloat" in mm._get_cache_key(a, b)
    with pytest.raises(TypeError, match="bfloat16"):
        mm.to_sdfg(np.zeros((64, 32), np.float32), b)

    @native(target="rocm")
    def batched(a: Annotated[np.ndarray, (), bfloat16], b: Annotated[np.ndarray, (), bfloat16]):
        return a @ b

    sdfg = batched.to_sdfg(np.zeros((4, 64, 32), np.uint16), np.zeros((4, 32, 48), np.uint16))
    (node,) = sdfg.library_nodes()
    assert node["code"] == "ml::MatMul" and sdfg.containers["_docc_ret_0"]["element"] == "Float"

    @native(target="rocm")
    def plain_words(a, b):          # no annotation: uint16 is not an element type of the math nodes
        return a @ b

    with pytest.raises(TypeError, match="uint16"):
        plain_words.to_sdfg(a, b)

    class ProductThenFloat(torch.nn.Module):
        def forward(self, a, b):
            return torch.matmul(a, b).float()

    class Widened(torch.nn.Module):
        def forward(self, a, b):
            return a.float() @ b.float().T

    class WidenedLinear(torch.nn.Module):
        def forward(self, x, w):
            return torch.nn.functional.linear(x.float(), w.float())

    class OneWidened(torch.nn.Module):
        def forward(self, a, b):
            return torch.relu(a.float()) @ b.float()

    class Rounded(torch.nn.Module):
        def forward(self, a, b):
            return torch.matmul(a, b)

    ta, tb, tbt = (torch.zeros(s, dtype=torch.bfloat16) for s in ((64, 32), (32, 48), (48, 32)))
    for model, args, trans_b in ((ProductThenFloat(), (ta, tb), 111), (Widened(), (ta, tbt), 112), (WidenedLinear(), (ta, tbt), 112)):
        sdfg = docc_torch.TorchProgram(model, target="rocm").to_sdfg(*args)
        (node,) = sdfg.library_nodes()
        assert (node["code"], node["precision"], node["trans_b"]) == ("GEMM", ord("b"), trans_b), type(model).__name__
        assert sdfg.containers["_docc_ret_0"]["element"] == "Float"
    sdfg = docc_torch.TorchProgram(ProductThenFloat(), target="rocm").to_sdfg(torch.zeros(4, 64, 32, dtype=torch.bfloat16), torch.zeros(4, 32, 48, dtype=torch.bfloat16))
    assert [n["code"] for n in sdfg.library_nodes()] == ["ml::MatMul"] and sdfg.containers["_docc_ret_0"]["element"] == "Float"
    # one operand that is more than a widened bf16 tensor: the casts are real, the product is a float32 GEMM
    sdfg = docc_torch.TorchProgram(OneWidened(), target="rocm").to_sdfg(ta, tb)
    assert [n["code"] for n in sdfg.library_nodes()] == ["ml::Cast", "ml::ReLU", "ml::Cast", "GEMM"]
    assert sdfg.library_nodes()[-1]["precision"] == ord("s")
    # the product as the bf16 tensor eager torch makes of it: the float32 result of the bf16 GEMM, rounded once
    sdfg = docc_torch.TorchProgram(Rounded(), target="rocm").to_sdfg(ta, tb)
    assert [n["code"] for n in sdfg.library_nodes()] == ["GEMM", "ml::Cast"] and sdfg.library_nodes()[0]["precision"] == ord("b")
    assert sdfg.containers["_docc_ret_0"]["element"] == "BFloat"

    class Bf16Linear(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = torch.nn.Linear(32, 48).bfloat16()

        def forward(self, x):
            return self.fc(x)

    sdfg = docc_torch.TorchProgram(Bf16Linear(), target="rocm").to_sdfg(ta)
    codes = [n["code"] for n in sdfg.library_nodes()]
    assert codes[0] == "GEMM" and codes[-1] == "ml::Cast" and "ml::Add" in codes and sdfg.containers["_docc_ret_0"]["element"] == "BFloat"


def test_torch_lowering_of_composite_activations_and_layer_norm():
    """gelu, silu, neg, reciprocal, rsqrt, square and layer_norm are spelled with the tensor nodes there are; scheduled, the
    chains between the reductions and products are single generated kernels."""
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.LayerNorm(16)
            self.fc1 = torch.nn.Linear(16, 32)
            self.act = torch.nn.GELU()
            self.fc2 = torch.nn.Linear(32, 16)

        def forward(self, x):
            return x + self.fc2(self.act(self.fc1(self.norm(x))))

    x = torch.randn(2, 5, 16)
    sdfg = docc_torch.TorchProgram(Block(), (x,), target="rocm").to_sdfg()
    codes = [n["code"] for n in sdfg.library_nodes()]
    # layer norm: mean, centre, mean of squares, + eps, sqrt, divide, weight, bias
    assert codes[:13] == ["ml::Mean", "ml::Broadcast", "ml::Sub", "ml::Mul", "ml::Mean", "ml::Add", "ml::Sqrt", "ml::Broadcast", "ml::Div",
                          "ml::Broadcast", "ml::Mul", "ml::Broadcast", "ml::Add"]
    assert codes[13:] == ["GEMM", "ml::Broadcast", "ml::Add", "ml::Mul", "ml::Erf", "ml::Mul", "ml::Add", "ml::Mul",
                          "GEMM", "ml::Broadcast", "ml::Add", "ml::Add"]
    sdfg.schedule("rocm")
    kernels = [n["code"] for n in sdfg.library_nodes() if n["code"] != "ROCMOffloading"]
    # mean | centre and square in one kernel each (the centred value has two readers) | mean | the rest of the norm |
    # GEMM with its bias | gelu | GEMM with its bias | the residual
    assert kernels.count("GEMM") == 2 and kernels.count("ml::Mean") == 2 and kernels.count("ROCMMap") >= 2
    assert len(kernels) <= 9, kernels

    class Misc(torch.nn.Module):
        def forward(self, a, b):
            return F.silu(a) * torch.rsqrt(b.square() + 1.0) - (-a).reciprocal() + F.gelu(b, approximate="tanh")

    F = torch.nn.functional
    sdfg = docc_torch.TorchProgram(Misc(), (torch.randn(6, 7), torch.randn(6, 7)), target="rocm").to_sdfg()
    codes = [n["code"] for n in sdfg.library_nodes()]
    assert codes.count("ml::Sigmoid") == 1 and codes.count("ml::Sqrt") == 1 and codes.count("ml::Tanh") == 1 and codes.count("ml::Div") == 2
    sdfg.schedule("rocm")
    assert [n["code"] for n in sdfg.library_nodes() if n["code"] != "ROCMOffloading"] == ["ROCMMap"]      # one kernel for all of it

    class Bad(torch.nn.Module):
        def forward(self, a):
            return F.gelu(a, approximate="sigmoid")

    with pytest.raises((NotImplementedError, RuntimeError)):      # torch itself refuses the word while it traces
        docc_torch.TorchProgram(Bad(), (torch.randn(4),), target="rocm").to_sdfg()
