"""The rocm target's C++ side, driven through its C ABI: SDFG (de)serialisation with the
reference's node payload keys, the "<code>::<implementation type>" dispatcher registry, the node
mapper, the offloading transform with transfer minimisation, and the emitted host C++ (checked
as text, the way the reference tests its dispatchers: opt/tests/cuda/cuda_library_nodes_test.cpp:513-651)."""
import ctypes
import json
import re
from pathlib import Path

import numpy as np
import pytest

from docc_amd import runtime
from docc_amd.sdfg import (InvalidSDFGException, Pointer, PrimitiveType, Scalar, StructuredSDFG, StructuredSDFGBuilder,
                           registered_dispatchers)

F64, F32, BF16, I64 = (Pointer(Scalar(PrimitiveType.Double)), Pointer(Scalar(PrimitiveType.Float)),
                       Pointer(Scalar(PrimitiveType.BFloat)), Scalar(PrimitiveType.Int64))


def gemm_sdfg(ptr=F64, name="matmul_sdfg"):
    b = StructuredSDFGBuilder(name)
    b.add_container("A", ptr, True)
    b.add_container("B", ptr, True)
    b.add_container("_s0", I64, True)
    b.add_container("_docc_ret_0", F32 if ptr is BF16 else ptr, True)
    b.add_gemm("A", "B", "_docc_ret_0", "1.0", "0.0", "_s0", "_s0", "_s0")
    return b.move()


def source_of(sdfg, tmp_path):
    report = sdfg.generate(str(tmp_path))
    return Path(report["source"]).read_text(), report


def test_registry_holds_every_rocm_key():
    keys = registered_dispatchers()
    for code in ("GEMM", "ml::MatMul", "ml::Softmax", "ml::Conv", "ml::Attention", "ml::Broadcast", "ml::Abs", "ml::Exp",
                 "ml::ReLU", "ml::Sigmoid", "ml::Sqrt", "ml::Tanh", "ml::Erf", "ml::Add", "ml::Sub", "ml::Mul", "ml::Div",
                 "ml::Maximum", "ml::Minimum", "ml::Sum", "ml::Max", "ml::Min", "ml::Mean", "ROCMFusedElementWise", "ml::Elu",
                 "ml::LeakyReLU", "ml::HardSigmoid", "ml::Fill", "DOT"):
        assert f"{code}::ROCMWithTransfers" in keys and f"{code}::ROCMWithoutTransfers" in keys
    assert "ROCMOffloading::NONE" in keys


def test_gemm_node_json_uses_the_reference_keys():
    node = gemm_sdfg().library_nodes()[0]
    # keys of GEMMNodeSerializer (reference gemm_node.cpp:387-405) inside the library_node envelope
    for key in ("type", "element_id", "code", "implementation_type", "precision", "layout", "trans_a", "trans_b",
                "m", "n", "k", "lda", "ldb", "ldc"):
        assert key in node
    assert node["code"] == "GEMM" and node["implementation_type"] == "BLAS"
    assert node["precision"] == ord("d") and node["layout"] == 101 and node["trans_a"] == 111 and node["trans_b"] == 111
    # a round trip through the native parser keeps everything
    again = StructuredSDFG.parse(gemm_sdfg().to_json())
    assert again.library_nodes()[0] == node and again.arguments == ["A", "B", "_s0", "_docc_ret_0"]


def test_dot_and_activation_nodes_use_the_reference_keys(tmp_path):
    b = StructuredSDFGBuilder("dots")
    b.add_container("x", F32, True)
    b.add_container("y", F32, True)
    b.add_container("_s0", I64, True)
    b.add_container("r", Scalar(PrimitiveType.Float), False)
    b.add_container("out", F32, True)
    b.add_dot("x", "y", "r", "_s0", 1, 2)
    b.add_fill("r", "out", [1])
    b.add_elementwise_unary_op("leaky_relu", "x", "y", ["_s0"], alpha="r")
    s = b.move()
    dot, fill, leaky = s.library_nodes()
    # DotNodeSerializer (reference dot_node.cpp:189-202) and ElementWiseUnaryNodeSerializer keys
    assert dot["code"] == "DOT" and dot["precision"] == ord("s") and (dot["n"], dot["incx"], dot["incy"]) == ("_s0", "1", "2")
    assert dot["implementation_type"] == "BLAS"
    assert fill["code"] == "ml::Fill" and fill["shape"] == ["1"]
    assert leaky["code"] == "ml::LeakyReLU" and leaky["shape"] == ["_s0"]
    again = StructuredSDFG.parse(s.to_json())
    assert [n["code"] for n in again.library_nodes()] == ["DOT", "ml::Fill", "ml::LeakyReLU"]
    s.schedule("rocm", options={"offload": "none"})
    src, _ = source_of(s, tmp_path)
    assert "docc_rocm_dot(nullptr, 32, _s0, __x, 1, __y, 2, &__out)" in src and "r = __out;" in src
    assert "docc_rocm_fill(nullptr, (int) sizeof(__docc_value), 1, &__docc_value, Y)" in src
    assert "docc_rocm_elementwise_activation(nullptr, 8 /* ml::LeakyReLU */, 32, _s0, X, Y, (double) alpha, 0.0)" in src
    # a pointer where a scalar belongs is refused when the code is generated
    b = StructuredSDFGBuilder("bad_dot")
    for n in ("x", "y", "r"):
        b.add_container(n, F64, True)
    b._add_block({"code": "DOT", "implementation_type": "BLAS", "side_effect": False, "precision": ord("d"), "n": "4", "incx": "1", "incy": "1"},
                 [b._operand("__x", "x"), b._operand("__y", "y")], [b._operand("__out", "r")])
    bad = b.move()
    bad.schedule("rocm", options={"offload": "none"})
    with pytest.raises(InvalidSDFGException, match="scalar"):
        bad.generate(str(tmp_path / "bad"))


def test_validation_errors():
    b = StructuredSDFGBuilder("bad")
    b.add_container("A", F64, True)
    with pytest.raises(InvalidSDFGException):
        b.add_container("A", F64, True)
    data = json.loads(gemm_sdfg().to_json())
    data["root"]["children"][0]["dataflow"]["inputs"][0]["data"] = "nope"
    with pytest.raises(InvalidSDFGException, match="unknown container"):
        StructuredSDFG.parse(json.dumps(data))
    data = json.loads(gemm_sdfg().to_json())
    data["root"]["children"][0]["dataflow"]["library_node"]["code"] = "Mystery"
    with pytest.raises(InvalidSDFGException, match="No library node serializer"):
        StructuredSDFG.parse(json.dumps(data))
    data = json.loads(gemm_sdfg().to_json())
    del data["root"]["children"][0]["dataflow"]["inputs"][4]
    with pytest.raises(InvalidSDFGException, match="__beta"):
        StructuredSDFG.parse(json.dumps(data))


def test_unscheduled_node_has_no_dispatcher(tmp_path):
    # the BLAS implementation type belongs to the reference's CPU path, which this target does not carry
    with pytest.raises(InvalidSDFGException, match="No library node dispatcher found for library node code: GEMM::BLAS"):
        gemm_sdfg().generate(str(tmp_path))


def test_mapper_sets_implementation_types_and_declines_what_the_kernels_lack():
    s = gemm_sdfg()
    s.schedule("rocm", options={"offload": "node"})
    assert s.library_nodes()[0]["implementation_type"] == "ROCMWithTransfers"
    s = gemm_sdfg()
    s.schedule("rocm", options={"offload": "none"})
    assert s.library_nodes()[0]["implementation_type"] == "ROCMWithoutTransfers"
    assert s.loop_report()["H2D"] == 0
    # column-major GEMM is declined; with no CPU lowering that is an error, not a silent fallback
    data = json.loads(gemm_sdfg().to_json())
    data["root"]["children"][0]["dataflow"]["library_node"]["layout"] = 102
    with pytest.raises(InvalidSDFGException, match="row-major"):
        StructuredSDFG.parse(json.dumps(data)).schedule("rocm")
    s = StructuredSDFG.parse(json.dumps(data))
    s.schedule("rocm", options={"require_all_mapped": False})
    assert s.library_nodes()[0]["implementation_type"] == "BLAS"
    # softmax over scattered axes, grouped conv, head dim != 64
    b = StructuredSDFGBuilder("s")
    b.add_container("X", F32, True)
    b.add_container("Y", F32, True)
    b.add_reduce_op("softmax", "X", "Y", [4, 8, 3], [0, 2])
    with pytest.raises(InvalidSDFGException, match="adjacent"):
        b.move().schedule("rocm")
    b = StructuredSDFGBuilder("c")
    for n in ("X", "W", "Y"):
        b.add_container(n, F32, True)
    b.add_conv("X", "W", "Y", [1, 4, 8, 8], [3, 3], [1, 1], [1, 1, 1, 1], [1, 1], 4, group=0)
    with pytest.raises(InvalidSDFGException, match="group"):
        b.move().schedule("rocm")
    # the node's group is taken: the launcher for grouped convolutions, the weights [C_out, C_in / group, kh, kw] on the device
    b = StructuredSDFGBuilder("cg")
    for n in ("X", "W", "Y"):
        b.add_container(n, F32, True)
    b.add_conv("X", "W", "Y", [1, 4, 8, 8], [3, 3], [1, 1], [1, 1, 1, 1], [1, 1], 6, group=2)
    s = b.move()
    s.schedule("rocm")
    import tempfile
    with tempfile.TemporaryDirectory() as folder:
        text = re.sub(r"\s+", " ", Path(s.generate(folder)["source"]).read_text())
    assert "docc_rocm_conv2d_f32_grouped(nullptr, 1, 4, 8, 8, 6, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, (int64_t) (2), (const float *)" in text
    assert "nullptr, 0));" in text and "docc_rocm_conv2d_f32_pads(" not in text
    assert "docc_rocm_memcpy_h2d_async(_dst, _src, (size_t) (((216) / 2)*4), nullptr)" in text       # W: 6 x 4 / 2 x 3 x 3 floats
    # a convolution whose pads differ between begin and end is taken: the launcher gets all four (begins, then ends)
    b = StructuredSDFGBuilder("cp")
    for n in ("X", "W", "Y"):
        b.add_container(n, F32, True)
    b.add_conv("X", "W", "Y", [1, 4, 8, 8], [3, 3], [1, 1], [0, 1, 2, 0], [1, 1], 4)
    s = b.move()
    s.schedule("rocm", options={"offload": "none"})
    assert s.library_nodes()[0]["implementation_type"] == "ROCMWithoutTransfers"
    import tempfile
    with tempfile.TemporaryDirectory() as folder:
        text = re.sub(r"\s+", " ", Path(s.generate(folder)["source"]).read_text())
    assert "docc_rocm_conv2d_f32_pads(nullptr, 1, 4, 8, 8, 4, 3, 3, 1, 1, 0, 1, 2, 0, 1, 1, (const float *) X" in text
    assert "docc_rocm_conv2d_f32_pads_workspace_bytes(1, 4, 8, 8, 4, 3, 3, 1, 1, 0, 1, 2, 0, 1, 1)" in text
    b = StructuredSDFGBuilder("a")
    for n in ("Q", "K", "V"):
        b.add_container(n, F32, True)
    b.add_container("O", F32, True)
    b.add_attention("Q", "K", "V", "O", [1, 2, 16, 64], 16, 0.1)
    with pytest.raises(InvalidSDFGException, match="BFloat"):
        b.move().schedule("rocm")
    with pytest.raises(NotImplementedError):
        gemm_sdfg().schedule("openmp")


def test_with_transfers_dispatcher_text(tmp_path):
    s = gemm_sdfg()
    s.schedule("rocm", options={"offload": "node"})
    src, report = source_of(s, tmp_path)
    assert report["function"] == 'extern "C" void matmul_sdfg(double *A, double *B, int64_t _s0, double *_docc_ret_0)'
    flat = re.sub(r"\s+", " ", src)
    # connector locals, constants printed verbatim, write-back (reference block_dispatcher.cpp:333-438)
    for piece in ("double *__A = A;", "double *__B = B;", "double *__C = _docc_ret_0;", "double __alpha = 1.0;",
                  "double __beta = 0.0;", "_docc_ret_0 = __C;"):
        assert piece in flat
    # alloc x3, upload of A and B only (beta == 0: C is not read), launch, download, sync, free x3
    assert flat.count("docc_rocm_malloc_async(") == 3 and flat.count("docc_rocm_free_async(") == 3
    assert flat.count("docc_rocm_memcpy_h2d_async(") == 2 and flat.count("docc_rocm_memcpy_d2h_async(") == 1
    assert "docc_rocm_dgemm(nullptr, 111, 111, _s0, _s0, _s0, __alpha, (const double *) d___A, _s0, (const double *) d___B, _s0, __beta, (double *) d___C, _s0)" in flat
    assert flat.index("docc_rocm_memcpy_h2d_async") < flat.index("docc_rocm_dgemm") < flat.index("docc_rocm_memcpy_d2h_async") < flat.index("docc_rocm_stream_sync")
    assert "if ((_s0) != 0 && (_s0) != 0)" in flat            # zero-size guard, as the cuBLAS dispatcher has
    assert '#include "docc_rocm_rt.h"' in src and src.count("#define DOCC_ROCM_CHECK") == 1
    metrics = report["instrumentation"][0]
    assert metrics["target_type"] == "ROCM" and "flop" in metrics["metrics"] and "pcie_bytes" in metrics["metrics"]


def test_beta_nonzero_uploads_c(tmp_path):
    b = StructuredSDFGBuilder("gemm_acc")
    for n in ("A", "B", "C"):
        b.add_container(n, F32, True)
    b.add_gemm("A", "B", "C", "1.5", "1.2", 8, 8, 8)
    s = b.move()
    s.schedule("rocm", options={"offload": "node"})
    src, _ = source_of(s, tmp_path)
    assert src.count("docc_rocm_memcpy_h2d_async(") == 3 and "docc_rocm_sgemm(" in src and "float __alpha = 1.5;" in src


def test_bf16_gemm_text(tmp_path):
    s = gemm_sdfg(BF16, "bf")
    s.schedule("rocm", options={"offload": "none"})
    src, report = source_of(s, tmp_path)
    assert report["function"] == 'extern "C" void bf(__bf16 *A, __bf16 *B, int64_t _s0, float *_docc_ret_0)'
    assert "docc_rocm_bf16gemm_f32(nullptr, 111, 111, _s0, _s0, _s0, __alpha, (const uint16_t *) __A" in src
    assert "float __alpha = 1.0;" in src and "docc_rocm_malloc" not in src


def test_softmax_over_inner_axes_and_fp64(tmp_path):
    """A block of adjacent axes is the middle extent of an [outer, extent, inner] view; the last axis of an
    fp32 tensor keeps its own entry point."""
    cases = [(F32, [4, 8, 6], [1], "docc_rocm_softmax(nullptr, 32, 4, 8, 6, (const void *) X, (void *) Y)"),
             (F32, [4, 8, 6], [0, 1], "docc_rocm_softmax(nullptr, 32, 1, 32, 6, (const void *) X, (void *) Y)"),
             (F64, [4, 8, 6], [-1], "docc_rocm_softmax(nullptr, 64, 32, 6, 1, (const void *) X, (void *) Y)"),
             (F64, [4, 8, 6], [-2, 2], "docc_rocm_softmax(nullptr, 64, 4, 48, 1, (const void *) X, (void *) Y)"),
             (F32, [4, 8, 6], [2], "docc_rocm_softmax_f32(nullptr, 32, 6, (const float *) X, (float *) Y)")]
    for ptr, shape, axes, text in cases:
        b = StructuredSDFGBuilder("sm")
        b.add_container("X", ptr, True)
        b.add_container("Y", ptr, True)
        b.add_reduce_op("softmax", "X", "Y", shape, axes)
        s = b.move()
        s.schedule("rocm", options={"offload": "none"})
        src, _ = source_of(s, tmp_path)
        assert text in src, (axes, src)


def test_attention_with_another_head_dimension_brings_its_workspace(tmp_path):
    for d, fused in ((64, True), (128, True), (32, True), (96, False)):
        b = StructuredSDFGBuilder("att")
        for n in ("Q", "K", "V", "O"):
            b.add_container(n, BF16, True)
        b.add_attention("Q", "K", "V", "O", [2, 4, 256, d], 192, 0.125)
        s = b.move()
        s.schedule("rocm", options={"offload": "none"})
        src, _ = source_of(s, tmp_path)
        if fused:
            assert f"docc_rocm_attention_bf16(nullptr, 2, 4, 256, 192, {d}, (float) (0.125)," in src and "_ws" not in src
        else:
            assert "docc_rocm_attention_bf16_workspace_bytes(2, 4, 256, 192, 96, 1);" in src
            assert "docc_rocm_attention_bf16_ws(nullptr, 2, 4, 256, 192, 96, (float) (0.125), (const uint16_t *) Q" in src
            assert src.index("docc_rocm_malloc_async(&__ws") < src.index("docc_rocm_attention_bf16_ws(") < src.index("docc_rocm_free_async(__ws, nullptr)")


def test_transpose_node_round_trips_and_dispatches(tmp_path):
    b = StructuredSDFGBuilder("tr")
    b.add_container("X", F32, True)
    b.add_container("Y", F32, True)
    b.add_container("_s0", I64, True)
    b.add_transpose("X", "Y", ["_s0", 3, 5], [2, 0, 1])
    s = b.move()
    node = s.library_nodes()[0]
    assert node["code"] == "ml::Transpose" and node["perm"] == [2, 0, 1] and node["shape"] == ["_s0", "3", "5"]
    again = StructuredSDFG.parse(s.to_json()).library_nodes()[0]
    assert {k: v for k, v in again.items() if k != "element_id"} == {k: v for k, v in node.items() if k != "element_id"}
    s.schedule("rocm", options={"offload": "node"})
    src, _ = source_of(s, tmp_path)
    assert "const int64_t __docc_shape[] = {(int64_t) (_s0), (int64_t) (3), (int64_t) (5)};" in src
    assert "const int64_t __docc_perm[] = {2, 0, 1};" in src
    assert "docc_rocm_transpose(nullptr, 4, 3, __docc_shape, __docc_perm, d_X, d_Y)" in src
    # no permutation: the axes are reversed, as in the reference's constructor
    b = StructuredSDFGBuilder("tr2")
    b.add_container("X", F64, True)
    b.add_container("Y", F64, True)
    b.add_transpose("X", "Y", [2, 3, 4])
    assert b.move().library_nodes()[0]["perm"] == [2, 1, 0]
    with pytest.raises(InvalidSDFGException, match="permutation"):
        b = StructuredSDFGBuilder("bad")
        b.add_container("X", F32, True)
        b.add_container("Y", F32, True)
        b.add_transpose("X", "Y", [2, 3], [0, 0])


def test_cast_node_dispatches_and_declines(tmp_path):
    b = StructuredSDFGBuilder("cast")
    b.add_container("X", F32, True)
    b.add_container("Y", BF16, True)
    b.add_container("_s0", I64, True)
    b.add_cast_op("X", "Y", ["_s0", 8])
    s = b.move()
    node = s.library_nodes()[0]
    assert node["code"] == "ml::Cast" and node["target_type"] == "BFloat" and node["element_type"] == "Float"
    s.schedule("rocm", options={"offload": "none"})
    src, _ = source_of(s, tmp_path)
    assert "docc_rocm_cast(nullptr, 2 /* Float */, 1 /* BFloat */, _s0*8, X, Y)" in src
    b = StructuredSDFGBuilder("cast2")
    b.add_container("X", F64, True)
    b.add_container("Y", BF16, True)
    b.add_cast_op("X", "Y", [4])
    with pytest.raises(InvalidSDFGException, match="Double -> BFloat is not built"):
        b.move().schedule("rocm")


def test_matmul_node_is_one_batched_launch(tmp_path):
    """[6, 32, 16] @ [16, 24]: B is shared (stride 0); with a batched B its stride is k*n."""
    for shape_b, stride_b in (([16, 24], "0"), ([6, 16, 24], "384")):
        b = StructuredSDFGBuilder("bmm")
        for n in ("A", "B", "Y"):
            b.add_container(n, F32, True)
        b.add_matmul("A", "B", "Y", [6, 32, 16], shape_b)
        s = b.move()
        s.schedule("rocm", options={"offload": "none"})
        src, _ = source_of(s, tmp_path)
        assert ("docc_rocm_sgemm_batched(nullptr, 111, 111, 32, 24, 16, 1.0f, (const float *) A, 16, (int64_t) (512), "
                f"(const float *) B, 24, (int64_t) ({stride_b}), 0.0f, (float *) Y, 24, (int64_t) (768), (int64_t) (6)));") in src
        assert "for (int64_t __b" not in src


def chain_sdfg():
    """T = A @ B; Y = softmax(T): the intermediate T is a transient."""
    b = StructuredSDFGBuilder("chain")
    b.add_container("A", F32, True)
    b.add_container("B", F32, True)
    b.add_container("Y", F32, True)
    b.add_container("T", F32, False, transient_bytes=64 * 64 * 4)
    b.add_gemm("A", "B", "T", "1.0", "0.0", 64, 64, 64)
    b.add_reduce_op("softmax", "T", "Y", [64, 64], [-1])
    return b.move()


def test_offloading_keeps_intermediates_on_the_device(tmp_path):
    s = chain_sdfg()
    s.schedule("rocm")                     # default: function-level offloading
    report = s.loop_report()
    assert report["GEMM::ROCMWithoutTransfers"] == 1 and report["ml::Softmax::ROCMWithoutTransfers"] == 1
    assert report["H2D"] == 2 and report["D2H"] == 1          # A, B up; Y down; T never crosses PCIe
    assert "size" not in s.containers["T"]                     # and needs no host memory any more
    codes = [(n["code"], n.get("transfer_direction"), n.get("buffer_lifecycle")) for n in s.library_nodes()]
    assert codes.index(("GEMM", None, None)) < codes.index(("ml::Softmax", None, None))
    src, _ = source_of(s, tmp_path)
    assert "malloc(" not in src.replace("docc_rocm_malloc_async(", "")  # no host allocation left
    assert src.count("docc_rocm_malloc_async(") == src.count("docc_rocm_free_async(") == 4
    # without minimisation (per-node transfers) T would cross twice
    s2 = chain_sdfg()
    s2.schedule("rocm", options={"offload": "node"})
    assert s2.loop_report()["H2D"] == 0 and "ROCMOffloading" not in s2.loop_report()
    src2, _ = source_of(s2, tmp_path / "node")
    assert src2.count("docc_rocm_memcpy_h2d_async(") == 3 and src2.count("docc_rocm_memcpy_d2h_async(") == 2


def test_offloading_reuses_a_read_only_operand(tmp_path):
    b = StructuredSDFGBuilder("reuse")
    for n in ("A", "B", "C", "D"):
        b.add_container(n, F64, True)
    b.add_gemm("A", "B", "C", "1.0", "0.0", 16, 16, 16)
    b.add_gemm("C", "B", "D", "1.0", "0.0", 16, 16, 16)
    s = b.move()
    s.schedule("rocm")
    r = s.loop_report()
    assert r["H2D"] == 2          # A and B once each; C stays on the device
    assert r["D2H"] == 2          # C and D are arguments: both come back
    offload = [n for n in s.library_nodes() if n["code"] == "ROCMOffloading"]
    # payload keys of the reference's offloading node (cuda_data_offloading_node.cpp:198-256)
    assert all({"size", "device_id", "transfer_direction", "buffer_lifecycle"} <= set(n) for n in offload)
    d2h_only = [n for n in offload if n["transfer_direction"] == -1 and n["buffer_lifecycle"] == 0]
    assert len(d2h_only) == 1     # C's download no longer frees: the second GEMM still reads the device copy


def every_node_type():
    """One single-node program per node type the target lowers; arguments p0..p3 (names no connector has)."""
    def build(name, fill, ptrs):
        b = StructuredSDFGBuilder(name)
        for n, t in ptrs.items():
            b.add_container(n, t, True)
        fill(b)
        return b.move()

    f3 = {"p0": F32, "p1": F32, "p3": F32}
    yield build("n_gemm", lambda b: b.add_gemm("p0", "p1", "p3", "1.0", "0.5", 8, 8, 8), f3)
    yield build("n_gemm_bf16", lambda b: b.add_gemm("p0", "p1", "p3", "1.0", "0.0", 8, 8, 8), {"p0": BF16, "p1": BF16, "p3": F32})
    yield build("n_matmul", lambda b: b.add_matmul("p0", "p1", "p3", [6, 32, 16], [6, 16, 24]), f3)
    yield build("n_softmax", lambda b: b.add_reduce_op("softmax", "p0", "p3", [4, 8], [-1]), {"p0": F32, "p3": F32})
    yield build("n_softmax_inner", lambda b: b.add_reduce_op("softmax", "p0", "p3", [4, 8, 6], [1]), {"p0": F64, "p3": F64})
    for op in ("sum", "max", "min", "mean"):
        yield build("n_" + op, lambda b, op=op: b.add_reduce_op(op, "p0", "p3", [4, 8, 6], [1]), {"p0": F32, "p3": F32})
    yield build("n_conv", lambda b: b.add_conv("p0", "p1", "p3", [2, 8, 9, 9], [3, 3], [1, 1], [1, 1, 1, 1], [1, 1], 16, B="p2"),
                {"p0": F32, "p1": F32, "p2": F32, "p3": F32})
    yield build("n_conv_gemm", lambda b: b.add_conv("p0", "p1", "p3", [2, 7, 9, 9], [3, 3], [2, 2], [0, 0, 0, 0], [1, 1], 16),
                {"p0": F32, "p1": F32, "p3": F32})
    for d in (64, 128):
        yield build(f"n_attention{d}", lambda b, d=d: b.add_attention("p0", "p1", "p2", "p3", [2, 4, 96, d], 80, 0.125),
                    {"p0": BF16, "p1": BF16, "p2": BF16, "p3": F32})
    for op in StructuredSDFGBuilder.UNARY_CODES:
        yield build("n_" + op, lambda b, op=op: b.add_elementwise_unary_op(op, "p0", "p3", [4, 8]), {"p0": F32, "p3": F32})
    for op in sorted(set(StructuredSDFGBuilder.BINARY_CODES) - {"max", "min"}):
        yield build("n_" + op, lambda b, op=op: b.add_elementwise_op(op, "p0", "p1", "p3", [4, 8]), f3)
    yield build("n_scalar", lambda b: b.add_elementwise_op("mul", "p0", 2.5, "p3", [4, 8]), {"p0": F64, "p3": F64})
    yield build("n_elu", lambda b: b.add_elementwise_unary_op("elu", "p0", "p3", [4, 8], alpha=0.5), {"p0": F32, "p3": F32})
    yield build("n_leaky", lambda b: b.add_elementwise_unary_op("leaky_relu", "p0", "p3", [4, 8]), {"p0": F64, "p3": F64})
    yield build("n_hardsig", lambda b: b.add_elementwise_unary_op("hard_sigmoid", "p0", "p3", [4, 8], alpha=0.25, beta=0.5), {"p0": F32, "p3": F32})
    yield build("n_fill", lambda b: b.add_fill(1.5, "p3", [4, 8]), {"p3": F32})

    def dot(b):
        b.add_container("res", Scalar(PrimitiveType.Double), False)
        b.add_dot("p0", "p1", "res", 32, 1, 2)
        b.add_fill("res", "p3", [1])          # the scalar result reaches an argument through a fill of one element
    yield build("n_dot", dot, {"p0": F64, "p1": F64, "p3": F64})
    yield build("n_broadcast", lambda b: b.add_broadcast("p0", "p3", [1, 8], [4, 8]), {"p0": F32, "p3": F32})
    yield build("n_transpose", lambda b: b.add_transpose("p0", "p3", [4, 8, 3], [2, 0, 1]), {"p0": F32, "p3": F32})
    yield build("n_cast", lambda b: b.add_cast_op("p0", "p3", [4, 8]), {"p0": F32, "p3": BF16})


LAUNCHER_CALL = re.compile(r"DOCC_ROCM_CHECK\((docc_rocm_\w+)\((.*)\)\);")
NOT_A_KERNEL = {"docc_rocm_malloc_async", "docc_rocm_free_async", "docc_rocm_memcpy_h2d_async", "docc_rocm_memcpy_d2h_async",
                "docc_rocm_stream_sync"}


@pytest.mark.parametrize("offload", ["node", "function", "none"])
def test_every_node_type_generates_valid_code_on_device_pointers(tmp_path, offload):
    """Each node type, alone, under each offloading mode: the emitted C++ passes the compiler's syntax and
    type checks against the runtime headers, and where the function receives host pointers no launcher is
    handed one of them (a host address in a kernel is a memory fault on the device)."""
    include = Path(runtime.__file__).resolve().parent.parent / "include"
    for s in every_node_type():
        pointers = {n for n in s.arguments if s.containers[n].get("pointer", True)}
        s.schedule("rocm", options={"offload": offload})
        folder = tmp_path / s.name
        src, report = source_of(s, folder)
        cxx = __import__("os").environ.get("DOCC_CXX", "/opt/rocm/lib/llvm/bin/clang++")     # the compiler the target's JIT step runs
        proc = __import__("subprocess").run([cxx, "-std=c++17", "-fsyntax-only", "-Wall",
                                             "-I", str(include), "-I", str(folder), report["source"]], capture_output=True, text=True)
        assert proc.returncode == 0, f"{s.name} under offload={offload}:\n{proc.stderr}\n{src}"
        calls = [m for m in LAUNCHER_CALL.finditer(src) if m.group(1) not in NOT_A_KERNEL and not m.group(1).endswith("_workspace_bytes")]
        assert calls, s.name
        if offload == "none":
            continue
        connectors = set()
        for node in s.library_nodes():
            if node["code"] != "ROCMOffloading":
                connectors |= {c for c in node.get("inputs", []) + node.get("outputs", [])}
        for m in calls:
            tokens = set(re.findall(r"[A-Za-z_]\w*", m.group(2)))
            if offload == "node":
                # the node's connector locals are host pointers here; only their device copies d_<connector> may be passed
                bare = {t for t in tokens if t in connectors and not t.startswith("__alpha") and not t.startswith("__beta")}
                assert not (bare & {"A", "B", "C", "X", "Y", "W", "Q", "K", "V", "O", "__A", "__B", "__C", "__bias"}), (s.name, m.group(0))
            assert not (tokens & pointers), (s.name, m.group(0))


def check_transfers(s):
    """Walks the scheduled block list the way the generated code runs and fails on: an upload from host
    memory that holds no value (a transient nothing has written or downloaded into), a node or download
    that uses a device buffer before it is allocated or after it is freed, a buffer freed twice or never."""
    live, host_valid = set(), set(s.arguments)
    for child in s._data["root"]["children"]:
        flow, node = child["dataflow"], child["dataflow"]["library_node"]
        ins = [b["data"] for b in flow["inputs"] if "data" in b]
        outs = [b["data"] for b in flow["outputs"]]
        if node["code"] == "ROCMOffloading":
            direction, life = node["transfer_direction"], node["buffer_lifecycle"]
            if life == 1:
                assert outs[0] not in live, f"{outs[0]} allocated twice"
                live.add(outs[0])
            if direction == 1:
                assert ins[0] in host_valid, f"upload from {ins[0]}, which holds no value"
                assert outs[0] in live
            if direction == -1:
                assert ins[0] in live
                host_valid.add(outs[0])
            if life == -1:
                assert ins[0] in live, f"{ins[0]} freed while not allocated"
                live.discard(ins[0])
        else:
            for name in ins + outs:
                if s.containers[name].get("storage") == "ROCM_Generic":
                    assert name in live, f"{node['code']} uses {name} outside its lifetime"
    assert not live, f"never freed: {sorted(live)}"
    return host_valid


def test_offloading_a_transient_with_two_readers(tmp_path):
    """T = A @ B; Y = softmax(T); Z = T @ B: both readers of T, and both readers of B, use the buffers
    the first node filled; nothing is uploaded from T's (never written) host memory."""
    b = StructuredSDFGBuilder("two_readers")
    for n in ("A", "B", "Y", "Z"):
        b.add_container(n, F32, True)
    b.add_container("T", F32, False, transient_bytes=64 * 64 * 4)
    b.add_gemm("A", "B", "T", "1.0", "0.0", 64, 64, 64)
    b.add_reduce_op("softmax", "T", "Y", [64, 64], [-1])
    b.add_gemm("T", "B", "Z", "1.0", "0.0", 64, 64, 64)
    s = b.move()
    s.schedule("rocm")
    r = s.loop_report()
    assert r["H2D"] == 2 and r["D2H"] == 2                     # A, B up; Y, Z down
    valid = check_transfers(s)
    assert "T" not in valid and "size" not in s.containers["T"]
    src, _ = source_of(s, tmp_path)
    assert "malloc(" not in src.replace("docc_rocm_malloc_async(", "")
    assert src.count("docc_rocm_malloc_async(") == src.count("docc_rocm_free_async(") == 5   # A B T Y Z


def test_offloading_longer_chains_keep_every_lifetime_whole(tmp_path):
    """Reuse patterns the pairwise view of transfers gets wrong: three readers with other nodes in between,
    a container rewritten between its readers, an argument written twice."""
    b = StructuredSDFGBuilder("lifetimes")
    for n in ("A", "B", "C", "Y"):
        b.add_container(n, F32, True)
    for n in ("T", "U", "V"):
        b.add_container(n, F32, False, transient_bytes=32 * 32 * 4)
    b.add_gemm("A", "B", "T", "1.0", "0.0", 32, 32, 32)         # T = A B
    b.add_gemm("T", "B", "U", "1.0", "0.0", 32, 32, 32)         # U = T B
    b.add_reduce_op("softmax", "T", "V", [32, 32], [-1])        # V = softmax(T)
    b.add_gemm("T", "U", "C", "1.0", "0.0", 32, 32, 32)         # C = T U      (third reader of T)
    b.add_gemm("V", "C", "T", "1.0", "0.0", 32, 32, 32)         # T = V C      (T rewritten)
    b.add_gemm("T", "A", "C", "1.0", "0.0", 32, 32, 32)         # C = T A      (C written a second time)
    b.add_reduce_op("softmax", "C", "Y", [32, 32], [-1])
    s = b.move()
    s.schedule("rocm")
    r = s.loop_report()
    assert r["H2D"] == 2                                        # A and B, once each
    assert r["D2H"] == 2                                        # C once (its first value is never seen by the host) and Y
    valid = check_transfers(s)
    assert not ({"T", "U", "V"} & valid)
    src, _ = source_of(s, tmp_path)
    assert src.count("docc_rocm_malloc_async(") == src.count("docc_rocm_free_async(")


def test_generated_function_honours_the_calling_convention(tmp_path):
    """Compiles an emitted function and calls it through ctypes the way CompiledSDFG does. Without a
    GPU the first runtime call fails; the function must return early and report through the failure
    channel instead of touching its arguments or aborting."""
    import torch

    s = gemm_sdfg()
    s.schedule("rocm", options={"offload": "node"})
    lib_path = s._compile(str(tmp_path))
    assert Path(lib_path).name == "libmatmul_sdfg.so"
    runtime.lib()
    lib = ctypes.CDLL(lib_path)
    fn = lib.matmul_sdfg
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    fn.restype = None
    A, B = np.ones((4, 4)), np.ones((4, 4))
    out = np.full((4, 4), -1.0)
    # zero-sized problem: the guard skips every device call, on any machine
    fn(A.ctypes.data, B.ctypes.data, 0, out.ctypes.data)
    assert runtime.take_failure() == (0, "") and (out == -1.0).all()
    if not torch.cuda.is_available():
        fn(A.ctypes.data, B.ctypes.data, 4, out.ctypes.data)
        code, message = runtime.take_failure()
        assert code != 0 and "matmul_sdfg" in message and "docc_rocm_malloc" in message
        assert (out == -1.0).all()


def test_device_pointer_mode_allocates_transients_on_the_device(tmp_path):
    """offload == "none": the caller passes device pointers, so an intermediate must be a device
    allocation too - a host malloc'ed buffer handed to a kernel faults the GPU."""
    s = chain_sdfg()
    s.schedule("rocm", options={"offload": "none"})
    r = s.loop_report()
    assert r["H2D"] == 0 and r["D2H"] == 0 and r["ROCMOffloading"] == 2       # ALLOC and FREE of T
    assert s.containers["T"]["storage"] == "ROCM_Generic" and "size" not in s.containers["T"]
    src, _ = source_of(s, tmp_path)
    assert "malloc(" not in src.replace("docc_rocm_malloc_async(", "")
    flat = re.sub(r"\s+", " ", src)
    assert flat.index("docc_rocm_malloc_async(") < flat.index("docc_rocm_sgemm(") < flat.index("docc_rocm_softmax_f32(") < flat.index("docc_rocm_free_async(")
    assert src.count("docc_rocm_malloc_async(") == 1 and src.count("docc_rocm_free_async(") == 1


def dense_sdfg():
    """Y = relu(X @ W + bias) * 0.5: GEMM, Broadcast of the bias row, Add, ReLU, Mul by a constant."""
    b = StructuredSDFGBuilder("dense")
    for n in ("X", "W", "bias", "Y"):
        b.add_container(n, F32, True)
    for n in ("T0", "T1", "T2", "T3"):
        b.add_container(n, F32, False, transient_bytes=32 * 16 * 4)
    b.add_gemm("X", "W", "T0", "1.0", "0.0", 32, 16, 8)
    b.add_broadcast("bias", "T1", [1, 16], [32, 16])
    b.add_elementwise_op("add", "T0", "T1", "T2", [32, 16])
    b.add_elementwise_unary_op("relu", "T2", "T3", [32, 16])
    b.add_elementwise_op("mul", "T3", "0.5", "Y", [32, 16])
    return b.move()


def test_elementwise_nodes_round_trip_and_dispatch(tmp_path):
    s = dense_sdfg()
    nodes = s.library_nodes()
    assert [n["code"] for n in nodes] == ["GEMM", "ml::Broadcast", "ml::Add", "ml::ReLU", "ml::Mul"]
    # payload keys of the reference's serializers: shape (elementwise_node.cpp), input_shape / output_shape (broadcast_node.cpp)
    assert nodes[2]["shape"] == ["32", "16"] and nodes[1]["input_shape"] == ["1", "16"] and nodes[1]["output_shape"] == ["32", "16"]
    assert StructuredSDFG.parse(s.to_json()).library_nodes() == nodes
    s.schedule("rocm", options={"fuse": False})      # one launcher call per node
    r = s.loop_report()
    assert r["H2D"] == 3 and r["D2H"] == 1          # X, W, bias up; Y down; T0..T3 stay in device memory
    for t in ("T0", "T1", "T2", "T3"):
        assert "size" not in s.containers[t]
    src, _ = source_of(s, tmp_path)
    flat = re.sub(r"\s+", " ", src)
    assert "docc_rocm_broadcast(nullptr, 32, 2, __docc_in_shape, __docc_out_shape, X, Y)" in flat
    assert "const int64_t __docc_in_shape[] = {(int64_t) (1), (int64_t) (16)};" in flat
    assert "docc_rocm_elementwise_binary(nullptr, 0 /* ml::Add */, 32, 512, A, B, C)" in flat
    assert "docc_rocm_elementwise_unary(nullptr, 2 /* ml::ReLU */, 32, 512, X, Y)" in flat
    # the constant operand is passed by value, the array one as the only pointer
    assert "float B = 0.5;" in flat
    assert "docc_rocm_elementwise_binary_scalar(nullptr, 2 /* ml::Mul */, 32, 512, A, (double) B, 0, C)" in flat
    order = [flat.index(k) for k in ("docc_rocm_sgemm(", "docc_rocm_broadcast(", "docc_rocm_elementwise_binary(",
                                     "docc_rocm_elementwise_unary(", "docc_rocm_elementwise_binary_scalar(")]
    assert order == sorted(order)


def test_elementwise_with_transfers_and_scalar_on_the_left(tmp_path):
    b = StructuredSDFGBuilder("rsub")
    b.add_container("x", F64, True)
    b.add_container("s", Scalar(PrimitiveType.Double), True)
    b.add_container("y", F64, True)
    b.add_elementwise_op("sub", "s", "x", "y", ["_n"])
    b.add_container("_n", I64, True)
    s = b.move()
    s.schedule("rocm", options={"offload": "node"})
    src, report = source_of(s, tmp_path)
    flat = re.sub(r"\s+", " ", src)
    assert "docc_rocm_elementwise_binary_scalar(nullptr, 1 /* ml::Sub */, 64, _n, d_B, (double) A, 1, d_C)" in flat
    assert flat.count("docc_rocm_malloc_async(") == 2 and flat.count("docc_rocm_memcpy_h2d_async(") == 1   # the scalar is not an operand buffer
    assert flat.count("docc_rocm_memcpy_d2h_async(") == 1
    # what the kernels lack is declined, not run elsewhere
    b = StructuredSDFGBuilder("ints")
    for n in ("a", "c"):
        b.add_container(n, Pointer(Scalar(PrimitiveType.Int32)), True)
    b.add_elementwise_unary_op("abs", "a", "c", [8])
    with pytest.raises(InvalidSDFGException, match="Float or Double"):
        b.move().schedule("rocm")
    b = StructuredSDFGBuilder("bc")
    for n in ("a", "c"):
        b.add_container(n, F32, True)
    with pytest.raises(InvalidSDFGException, match="cannot be broadcast"):
        b.add_broadcast("a", "c", [3, 4], [5, 4])
        b.move().validate()


def test_fusion_folds_the_chain_into_one_kernel(tmp_path):
    """relu(X @ W + bias) * 0.5: the Broadcast moves into the Add, the ReLU into the Add, and the whole chain into
    the store of the GEMM; the multiplication by a constant is a binary node of its own and stays. Two
    launches instead of five, the intermediates gone."""
    s = dense_sdfg()
    s.schedule("rocm")
    r = s.loop_report()
    assert r["GEMM"] == 1 and r["ml::Mul"] == 1
    for gone in ("ml::Broadcast", "ml::Add", "ml::ReLU", "ROCMFusedElementWise"):
        assert gone not in r
    assert r["H2D"] == 3 and r["D2H"] == 1
    assert "T3" in s.containers and not {"T0", "T1", "T2"} & set(s.containers)
    gemm = next(n for n in s.library_nodes() if n["code"] == "GEMM")
    assert gemm["epilogue_bias"] is True and gemm["epilogue_activation"] == "ml::ReLU" and gemm["implementation_type"] == "ROCMWithoutTransfers"
    strip = lambda nodes: [{k: v for k, v in n.items() if k != "element_id"} for n in nodes]       # ids are renumbered by a parse
    assert strip(StructuredSDFG.parse(s.to_json()).library_nodes()) == strip(s.library_nodes())    # the epilogue fields serialise
    flat = re.sub(r"\s+", " ", source_of(s, tmp_path)[0])
    assert ("docc_rocm_sgemm_epilogue(nullptr, 111, 111, 32, 16, 8, __alpha, (const float *) __A, 8, (const float *) __B, 16, __beta, "
            "(float *) __C, 16, (const float *) __bias, 2 /* ml::ReLU */)") in flat
    assert "float *__bias = __daisy_rocm_" in flat
    assert flat.count("docc_rocm_malloc_async(") == 5      # X W bias on the device, T3, Y

    # without the GEMM in front the chain is one elementwise launch
    b = StructuredSDFGBuilder("ew")
    for n in ("A", "bias", "Y"):
        b.add_container(n, F32, True)
    for n in ("T1", "T2"):
        b.add_container(n, F32, False, transient_bytes=32 * 16 * 4)
    b.add_broadcast("bias", "T1", [1, 16], [32, 16])
    b.add_elementwise_op("add", "A", "T1", "T2", [32, 16])
    b.add_elementwise_unary_op("relu", "T2", "Y", [32, 16])
    s = b.move()
    s.schedule("rocm")
    fused = next(n for n in s.library_nodes() if n["code"] == "ROCMFusedElementWise")
    assert fused["binary"] == "ml::Add" and fused["a_shape"] == ["32", "16"] and fused["b_shape"] == ["1", "16"]
    assert fused["post"] == ["ml::ReLU"] and fused["implementation_type"] == "ROCMWithoutTransfers"
    assert strip(StructuredSDFG.parse(s.to_json()).library_nodes()) == strip(s.library_nodes())
    flat = re.sub(r"\s+", " ", source_of(s, tmp_path / "ew")[0])
    assert "const int64_t __docc_b_shape[] = {(int64_t) (1), (int64_t) (16)};" in flat
    assert "const int __docc_post[] = {2 /* ml::ReLU */};" in flat
    assert ("docc_rocm_elementwise_fused(nullptr, 32, 2, __docc_shape, 0 /* ml::Add */, __docc_a_shape, A, 0.0, __docc_b_shape, B, 0.0, "
            "1, __docc_post, Y)") in flat

    # an activation that is not one instruction stays behind the GEMM; the bias still moves into the store
    b = StructuredSDFGBuilder("tanh_layer")
    for n in ("X", "W", "bias", "Y"):
        b.add_container(n, F64, True)
    for n in ("T0", "T1", "T2"):
        b.add_container(n, F64, False, transient_bytes=32 * 16 * 8)
    b.add_gemm("X", "W", "T0", "1.0", "0.0", 32, 16, 8)
    b.add_broadcast("bias", "T1", [1, 16], [32, 16])
    b.add_elementwise_op("add", "T1", "T0", "T2", [32, 16])      # bias on the left
    b.add_elementwise_unary_op("tanh", "T2", "Y", [32, 16])
    s = b.move()
    s.schedule("rocm")
    nodes = [n for n in s.library_nodes() if n["code"] != "ROCMOffloading"]
    assert [n["code"] for n in nodes] == ["GEMM", "ROCMFusedElementWise"]
    assert nodes[0]["epilogue_bias"] is True and nodes[0]["epilogue_activation"] == ""
    assert nodes[1]["binary"] == "" and nodes[1]["post"] == ["ml::Tanh"]
    flat = re.sub(r"\s+", " ", source_of(s, tmp_path / "tanh")[0])
    assert "(const double *) __bias, -1)" in flat and "docc_rocm_dgemm_epilogue(" in flat

    # beta != 0 makes the GEMM a reader of its own output: the chain is left alone; so is a C with a padded leading dimension
    b = StructuredSDFGBuilder("acc")
    for n in ("X", "W", "T0", "Y"):
        b.add_container(n, F32, True)
    b.add_gemm("X", "W", "T0", "1.0", "1.0", 32, 16, 8)
    b.add_elementwise_unary_op("relu", "T0", "Y", [32, 16])
    s = b.move()
    s.schedule("rocm")
    assert "epilogue_activation" not in next(n for n in s.library_nodes() if n["code"] == "GEMM")

    # unary chains fold too, up to four operations; a value that something else reads is not folded away
    b = StructuredSDFGBuilder("chain")
    for n in ("X", "Y", "Z"):
        b.add_container(n, F64, True)
    for n in ("T0", "T1", "T2"):
        b.add_container(n, F64, False, transient_bytes=800)
    b.add_elementwise_unary_op("abs", "X", "T0", [100])
    b.add_elementwise_unary_op("sqrt", "T0", "T1", [100])
    b.add_elementwise_unary_op("tanh", "T1", "T2", [100])
    b.add_elementwise_op("sub", "T2", "T1", "Y", [100])        # T1 has a second reader
    b.add_elementwise_unary_op("exp", "Y", "Z", [100])         # Y is an argument: stays
    s = b.move()
    text = s.to_json()
    s.schedule("rocm", options={"fuse_maps": False})
    nodes = [(n["code"], n.get("post"), n.get("binary")) for n in s.library_nodes() if not n["code"].startswith("ROCMOff")]
    assert nodes == [("ROCMFusedElementWise", ["ml::Abs", "ml::Sqrt"], ""), ("ml::Tanh", None, None), ("ml::Sub", None, None),
                     ("ml::Exp", None, None)]
    # what the prebuilt kernels leave as separate launches becomes one generated kernel: tanh and the subtraction are
    # one nest, which is then the only reader of T1, so the chain in front joins it; Y, an argument, is still written,
    # and the exponential of it is a second result of the same nest
    s = StructuredSDFG.parse(text)
    s.schedule("rocm")
    nodes = [n for n in s.library_nodes() if not n["code"].startswith("ROCMOff")]
    assert [n["code"] for n in nodes] == ["ROCMMap"]
    assert [(st["op"], st["args"]) for st in nodes[0]["statements"]] == [
        ("fabs", ["_in0"]), ("sqrt", ["_v0"]), ("tanh", ["_v1"]), ("fp_sub", ["_v2", "_v1"]), ("exp", ["_v3"])]
    assert nodes[0]["bounds"] == ["100"] and len(nodes[0]["reads"]) == 1 and [w["value"] for w in nodes[0]["writes"]] == ["_v3", "_v4"]
    assert not {"T0", "T1", "T2"} & set(s.containers)
    assert s.loop_report()["H2D"] == 1 and s.loop_report()["D2H"] == 2

    # without a device compiler on the machine the chain keeps its prebuilt kernels
    import os
    s = StructuredSDFG.parse(text)
    saved = os.environ.get("DOCC_HIPCC")
    os.environ["DOCC_HIPCC"] = "/nonexistent/bin/hipcc"
    try:
        s.schedule("rocm")
    finally:
        if saved is None:
            del os.environ["DOCC_HIPCC"]
        else:
            os.environ["DOCC_HIPCC"] = saved
    assert "ROCMMap" not in [n["code"] for n in s.library_nodes()]

    # a GEMM in front of a merged chain: its result stays on the device although the two nodes spell its size differently
    b = StructuredSDFGBuilder("gemm_chain")
    for n in ("X", "W", "C", "D", "Y"):
        b.add_container(n, F32, True)
    for n in ("T0", "T1", "T2"):
        b.add_container(n, F32, False, transient_bytes=32 * 16 * 4)
    b.add_gemm("X", "W", "T0", "1.0", "0.0", 32, 16, 8)
    b.add_elementwise_op("mul", "T0", "C", "T1", [32, 16])
    b.add_elementwise_op("sub", "T1", "D", "T2", [32, 16])
    b.add_elementwise_op("mul", "T2", "0.5", "Y", [32, 16])
    s = b.move()
    s.schedule("rocm")
    r = s.loop_report()
    assert r["GEMM"] == 1 and r["ROCMMap"] == 1 and r["H2D"] == 4 and r["D2H"] == 1

    # per-node transfers keep working on the fused node, scalars are passed by value
    b = StructuredSDFGBuilder("scalar")
    b.add_container("x", F32, True)
    b.add_container("y", F32, True)
    b.add_container("t", F32, False, transient_bytes=40)
    b.add_elementwise_op("max", "x", "0.25", "t", [10])
    b.add_elementwise_unary_op("sigmoid", "t", "y", [10])
    s = b.move()
    s.schedule("rocm", options={"offload": "node"})
    flat = re.sub(r"\s+", " ", source_of(s, tmp_path / "scalar")[0])
    assert "docc_rocm_elementwise_fused(nullptr, 32, 1, __docc_shape, 4 /* ml::Maximum */, __docc_a_shape, d_A, 0.0, nullptr, nullptr, (double) B, 1, __docc_post, d_Y)" in flat
    assert flat.count("docc_rocm_memcpy_h2d_async(") == 1 and flat.count("docc_rocm_memcpy_d2h_async(") == 1


def test_reduce_nodes_dispatch_and_decline(tmp_path):
    b = StructuredSDFGBuilder("red")
    for n in ("X", "S", "M"):
        b.add_container(n, F32, True)
    b.add_container("_n", I64, True)
    b.add_reduce_op("sum", "X", "S", ["_n", 64, 56, 56], [2, 3])            # [_n, 64, 56*56] -> [_n, 64]
    b.add_reduce_op("max", "X", "M", ["_n", 64, 56, 56], [-3], keepdims=True)   # over the channels: inner extent 56*56
    s = b.move()
    nodes = s.library_nodes()
    # payload keys of the reference's reduce serializer (reduce_node.h:194-245)
    assert nodes[0]["code"] == "ml::Sum" and nodes[0]["axes"] == [2, 3] and nodes[0]["keepdims"] is False
    assert nodes[1]["code"] == "ml::Max" and nodes[1]["axes"] == [-3] and nodes[1]["keepdims"] is True
    s.schedule("rocm")
    r = s.loop_report()
    assert r["ml::Sum::ROCMWithoutTransfers"] == 1 and r["H2D"] == 1 and r["D2H"] == 2     # X goes up once for both nodes
    flat = re.sub(r"\s+", " ", source_of(s, tmp_path)[0])
    assert "docc_rocm_reduce(nullptr, 0 /* ml::Sum */, 32, _n*64, 3136, 1, X, Y)" in flat
    assert "docc_rocm_reduce(nullptr, 1 /* ml::Max */, 32, _n, 64, 3136, X, Y)" in flat
    assert "(size_t) (_n*64*4)" in flat.replace("(_n*64)*4", "_n*64*4")                      # Y of the sum: the kept extents
    # axes in several blocks are reduced block by block
    b = StructuredSDFGBuilder("scattered")
    for n in ("X", "Y"):
        b.add_container(n, F64, True)
    b.add_container("_n", I64, True)
    b.add_reduce_op("mean", "X", "Y", [4, 5, "_n", 6, 7], [0, 2, 3])
    s = b.move()
    s.schedule("rocm", options={"offload": "none"})
    flat = re.sub(r"\s+", " ", source_of(s, tmp_path / "scattered")[0])
    # axes in two blocks: the inner block (axes 2, 3) first into a device temporary, then axis 0 of what is left
    assert "docc_rocm_malloc_async(&__docc_part[0], (size_t) (1120), nullptr)" in flat                      # [4, 5, 7] doubles
    assert "docc_rocm_reduce(nullptr, 3 /* ml::Mean */, 64, 20, _n*6, 7, X, __docc_part[0])" in flat
    assert "docc_rocm_reduce(nullptr, 3 /* ml::Mean */, 64, 1, 4, 35, __docc_part[0], Y)" in flat
    assert "docc_rocm_free_async(__docc_part[0], nullptr)" in flat
    # std is the chain of nodes the reference's StdNode expands to
    b = StructuredSDFGBuilder("s")
    for n in ("X", "Y"):
        b.add_container(n, F32, True)
    b.add_reduce_op("std", "X", "Y", [4, 9], [1])
    s = b.move()
    assert [n["code"] for n in s.library_nodes()] == ["ml::Mul", "ml::Mean", "ml::Mean", "ml::Mul", "ml::Sub", "ml::Sqrt"]
    assert sorted(k for k, c in s.containers.items() if c["transient"]) == ["_std_tmp_0", "_std_tmp_1", "_std_tmp_2"]
    with pytest.raises(NotImplementedError, match="var"):
        StructuredSDFGBuilder("s").add_reduce_op("var", "X", "Y", [4], [0])
    b = StructuredSDFGBuilder("axis")
    for n in ("X", "Y"):
        b.add_container(n, F64, True)
    b.add_reduce_op("sum", "X", "Y", [4, 5], [2])
    with pytest.raises(InvalidSDFGException, match="Axis value out of bounds"):
        b.move().validate()


def test_cpp_plugin_door_has_the_reference_signatures(tmp_path):
    """A plugin source written against the reference's interfaces compiles against this target's headers and runs:
    the dispatcher factory takes (LanguageExtension&, const Function&, const data_flow::DataFlowGraph&, const
    data_flow::LibraryNode&) (sdfg/include/sdfg/codegen/dispatchers/node_dispatcher_registry.h:140-141), a dispatcher
    overrides dispatch_code(PrettyPrinter&, PrettyPrinter&, CodeSnippetFactory&), target mappers arrive through
    TargetMapperFactory / TargetMapperRegistry (sdfg/include/sdfg/plugins/target_mapping.h:24-37) and a plugin registers
    through plugins::Context (targets/et/src/et/target.cpp:21-36)."""
    import subprocess
    from docc_amd.sdfg import registered_target_mappers

    assert {"target": "rocm", "priority": 100} in registered_target_mappers()
    root = Path(__file__).resolve().parent.parent
    src = tmp_path / "plugin.cpp"
    src.write_text(r'''
#include <cstdio>
#include <functional>
#include <memory>
#include <type_traits>
#include "rocm_target.h"
using namespace sdfg;

// the reference's factory type, spelled out
using RefFn = std::function<std::unique_ptr<codegen::LibraryNodeDispatcher>(codegen::LanguageExtension&, const Function&,
                                                                             const data_flow::DataFlowGraph&, const data_flow::LibraryNode&)>;
static_assert(std::is_same<codegen::LibraryNodeDispatcherFn, RefFn>::value, "dispatcher factory signature");
static_assert(std::is_abstract<plugins::TargetMapperFactory>::value && std::is_abstract<plugins::TargetMapper>::value, "mapper interfaces");

class MyDispatcher : public codegen::LibraryNodeDispatcher {
public:
    MyDispatcher(codegen::LanguageExtension& le, const Function& f, const data_flow::DataFlowGraph& g, const data_flow::LibraryNode& n)
        : codegen::LibraryNodeDispatcher(le, f, g, n) {}
    void dispatch_code(codegen::PrettyPrinter& stream, codegen::PrettyPrinter&, codegen::CodeSnippetFactory&) override {
        stream << "/* " << node_.code() << " with " << data_flow_graph_.inputs.size() << " inputs */" << std::endl;
    }
};

class MyMapper : public plugins::TargetMapper {
public:
    bool try_map(builder::StructuredSDFGBuilder&, analysis::AnalysisManager&, data_flow::LibraryNode&) const override { return false; }
};
class MyFactory : public plugins::TargetMapperFactory {
public:
    std::unique_ptr<plugins::TargetMapper> create() const override { return std::make_unique<MyMapper>(); }
    int priority() override { return 500; }
    const std::string& for_target() const override { static const std::string t = "mine"; return t; }
};

static void register_mine(plugins::Context& context) {
    context.library_node_dispatcher_registry.register_library_node_dispatcher(
        "GEMM::MINE", [](codegen::LanguageExtension& le, const Function& f, const data_flow::DataFlowGraph& g, const data_flow::LibraryNode& n) {
            return std::make_unique<MyDispatcher>(le, f, g, n);
        });
}

int main() {
    auto context = plugins::Context::global_context();
    rocm::register_plugin(context);     // the rocm plugin's own entry, as docc would call it
    register_mine(context);
    auto& reg = codegen::LibraryNodeDispatcherRegistry::instance();
    if (!reg.get_library_node_dispatcher("GEMM::MINE") || !reg.get_library_node_dispatcher("GEMM::ROCMWithoutTransfers")) return 1;
    rocm::register_rocm_plugin();
    auto& mappers = plugins::TargetMapperRegistry::instance();
    mappers.register_target_mapper(std::make_shared<MyFactory>());
    auto all = mappers.get_all_mappers();
    if (all.size() != 2 || all[0]->for_target() != "mine" || all[1]->for_target() != "rocm") return 2;     // by priority
    auto rocm_mappers = mappers.create_for_target("rocm");
    if (rocm_mappers.size() != 1 || dynamic_cast<rocm::RocmLibNodeMapper*>(rocm_mappers[0].get()) == nullptr) return 3;
    std::puts("ok");
    return 0;
}
''')
    exe = tmp_path / "plugin"
    lib_dir = root / "docc_amd" / "lib"
    r = subprocess.run(["g++", "-std=c++17", "-I", str(root / "docc_amd" / "csrc" / "target"), str(src), "-o", str(exe),
                        "-L", str(lib_dir), "-ldocc_rocm_target", f"-Wl,-rpath,{lib_dir}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip() == "ok", (r.returncode, r.stdout, r.stderr)


def test_containers_named_like_connectors_do_not_shadow_each_other(tmp_path):
    """The tensor nodes' connectors are X, Y, A, B, C - names a user's arrays may carry too. A connector's local would
    hide such a container (`double *X = X;` reads the local itself), so the containers are captured under other names
    first and written back outside the connectors' scope."""
    import subprocess

    b = StructuredSDFGBuilder("clash")
    for n in ("X", "Y", "A"):
        b.add_container(n, F64, True)
    b.add_elementwise_op("add", "Y", "X", "A", [8])       # connector A <- Y, B <- X, C -> A
    b.add_elementwise_unary_op("relu", "A", "X", [8])     # connector X <- A, Y -> X
    s = b.move()
    s.schedule("rocm", options={"offload": "none", "fuse": False})
    src_path = s.generate(str(tmp_path))["source"]
    flat = re.sub(r"\s+", " ", Path(src_path).read_text())
    assert "double *__docc_bound_0 = Y; double *__docc_bound_1 = X; double *__docc_bound_2 = A; { double *A = __docc_bound_0; double *B = __docc_bound_1; double *C = __docc_bound_2;" in flat
    assert "__docc_bound_2 = C; } A = __docc_bound_2;" in flat
    assert "double *X = X;" not in flat and "double *A = A;" not in flat
    # nodes whose connectors meet no container keep the reference's plain text
    b = StructuredSDFGBuilder("plain")
    for n in ("P", "Q"):
        b.add_container(n, F64, True)
    b.add_elementwise_unary_op("relu", "P", "Q", [8])
    s2 = b.move()
    s2.schedule("rocm", options={"offload": "none"})
    flat2 = re.sub(r"\s+", " ", Path(s2.generate(str(tmp_path / "plain"))["source"]).read_text())
    assert "{ double *X = P; double *Y = Q;" in flat2 and "__docc_bound" not in flat2
    root = Path(__file__).resolve().parent.parent
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror=uninitialized", "-I", str(root / "include"), "-I", str(tmp_path), src_path],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]


def softmax_in_pieces(name, shape, axes, extra_reader=False):
    """m = Max(X); e = Exp(X - broadcast(m)); Y = e / broadcast(Sum(e)) as seven nodes, the way a builder client or an
    imported program spells softmax (the nodes the reference's SoftmaxNode::expand chains, softmax_node.cpp:142-252)."""
    b = StructuredSDFGBuilder(name)
    for n in ("X", "Y") + (("Z",) if extra_reader else ()):
        b.add_container(n, F32, True)
    kept = [1 if d in [a % len(shape) for a in axes] else s for d, s in enumerate(shape)]
    count = 1
    for s_ in shape:
        count *= s_
    for n in ("m", "mb", "d", "e", "s", "sb"):
        b.add_container(n, F32, False, transient_bytes=4 * count)
    b.add_reduce_op("max", "X", "m", shape, axes, True)
    b.add_broadcast("m", "mb", kept, shape)
    b.add_elementwise_op("sub", "X", "mb", "d", shape)
    b.add_elementwise_unary_op("exp", "d", "e", shape)
    b.add_reduce_op("sum", "e", "s", shape, axes, True)
    b.add_broadcast("s", "sb", kept, shape)
    b.add_elementwise_op("div", "e", "sb", "Y", shape)
    if extra_reader:
        b.add_elementwise_unary_op("relu", "e", "Z", shape)       # the exponentials are looked at from outside
    return b.move()


def test_softmax_written_in_pieces_becomes_one_node(tmp_path):
    s = softmax_in_pieces("pieces", [8, 16, 32], [-1])
    assert [n["code"] for n in s.library_nodes()] == ["ml::Max", "ml::Broadcast", "ml::Sub", "ml::Exp", "ml::Sum", "ml::Broadcast", "ml::Div"]
    s.schedule("rocm")
    nodes = [n for n in s.library_nodes() if n["code"] != "ROCMOffloading"]
    assert [n["code"] for n in nodes] == ["ml::Softmax"] and nodes[0]["axes"] == [2] and nodes[0]["shape"] == ["8", "16", "32"]
    assert set(s.containers) >= {"X", "Y"} and not {"m", "mb", "d", "e", "s", "sb"} & set(s.containers)
    r = s.loop_report()
    assert r["H2D"] == 1 and r["D2H"] == 1
    assert "docc_rocm_softmax_f32(nullptr, " in source_of(s, tmp_path)[0]
    # a block of axes in the middle
    s = softmax_in_pieces("middle", [4, 5, 6, 7], [1, 2])
    s.schedule("rocm")
    (node,) = [n for n in s.library_nodes() if n["code"] != "ROCMOffloading"]
    assert node["code"] == "ml::Softmax" and node["axes"] == [1, 2]
    # not when a value in between is used elsewhere, and not when switched off
    s = softmax_in_pieces("shared", [8, 32], [1], extra_reader=True)
    s.schedule("rocm")
    assert "ml::Softmax" not in [n["code"] for n in s.library_nodes()]
    s = softmax_in_pieces("off", [8, 32], [1])
    s.schedule("rocm", options={"match_softmax": False})
    assert "ml::Softmax" not in [n["code"] for n in s.library_nodes()]
    # reduced axes that are not one block: no softmax kernel takes them, so the seven nodes stay (the mapper takes
    # each of them: reductions over several blocks run block by block) and the schedule does not fail
    s = softmax_in_pieces("apart", [4, 5, 6], [0, 2])
    s.schedule("rocm", options={"require_all_mapped": True})
    codes = [n["code"] for n in s.library_nodes() if n["code"] != "ROCMOffloading"]
    assert "ml::Softmax" not in codes and "ml::Max" in codes and "ml::Sum" in codes
    assert all(n["implementation_type"].startswith("ROCM") for n in s.library_nodes() if n["code"] != "ROCMOffloading")


def test_builder_map_nest_generates_a_kernel_and_its_launch(tmp_path):
    """add_map_nest: relu(a * b + bias row) over [_s0, _s1] spelled as three statements. The two loops are one walk
    for a, b and y but not for the bias, so the kernel keeps both; with equally shaped operands only, the nest
    collapses to a single loop and the kernel takes no strides."""
    b = StructuredSDFGBuilder("mapped")
    for n in ("A", "B", "Y"):
        b.add_container(n, F32, True)
    b.add_container("bias", F32, True)
    b.add_container("alpha", Scalar(PrimitiveType.Float), True)
    for n in ("_s0", "_s1"):
        b.add_container(n, Scalar(PrimitiveType.Int64), True)
    row = ["_s1", "1"]
    b.add_map_nest([("i", "_s0"), ("j", "_s1")], [("a", "A", row), ("b", "B", row), ("c", "bias", ["0", "1"])],
                   [("p", "fp_mul", ["a", "b"]), ("q", "fp_fma", ["p", "s", "c"]), ("r", "fmax", [0.0, "q"])], [("Y", row, "r")],
                   scalars=[("s", "alpha")])
    b.add_map_nest([("i", "_s0"), ("j", "_s1")], [("a", "A", row)], [("t", "tanh", ["a"]), ("u", "fp_sub", ["t", 0.5])], [("B", row, "u")])
    s = b.move()
    s.validate()
    first, second = s.library_nodes()
    assert first["symbols"] == ["_s0", "_s1"] and first["reads"][2]["extent"] == "1 + ((_s1) - 1)*(1)"
    assert first["statements"][2] == {"out": "_v2", "type": "Float", "op": "fmax", "args": ["#0.0f", "_v1"]}
    s.schedule("rocm", options={"offload": "none"})
    report = s.generate(str(tmp_path))
    src = Path(report["source"]).read_text()
    texts = {p.name: p.read_text() for p in sorted(tmp_path.glob("kernel_mapped_*.hip"))}
    assert len(texts) == 2
    one, two = texts.values()
    assert "float _c0, long long b0, long long b1, long long st__in0_0" in one and "__builtin_fmaf((float) (_v0), (float) (_c0), (float) (_in2))" in one
    assert "long long b0)" in two and "b1" not in two and "st_" not in two          # one merged loop, no strides
    assert "const I i0 = gid * V;" in two and "tanhf(" in two
    assert '(void *) &_c0' in src and "(long long) ((_s0)*(_s1))" in src
    # statements may only use what is defined before them; operations must be known
    bad = StructuredSDFGBuilder("bad")
    bad.add_container("A", F32, True)
    bad.add_map_nest([("i", 8)], [("a", "A", ["1"])], [("p", "fp_add", ["a", "later"]), ("later", "assign", ["a"])], [("A", ["1"], "p")])
    with pytest.raises(InvalidSDFGException, match="before it is defined"):
        bad.move().validate()
    bad = StructuredSDFGBuilder("bad2")
    bad.add_container("A", F32, True)
    bad.add_map_nest([("i", 8)], [("a", "A", ["1"])], [("p", "fp_sqrt", ["a"])], [("A", ["1"], "p")])
    with pytest.raises(InvalidSDFGException, match="unknown operation 'fp_sqrt'"):
        bad.move().validate()


def test_bf16_tensors_between_float32_nodes_join_the_generated_kernel(tmp_path):
    """A bf16 tensor widened to float32, two float32 nodes and the rounding back to bf16 - what the torch front end makes of an
    elementwise chain on bf16 tensors - become one generated kernel that loads and stores bf16: the conversions are the
    assignments of the nest, the arithmetic stays in float32. A nest may not compute in bf16."""
    b = StructuredSDFGBuilder("bf16_chain")
    b.add_container("x", BF16, True)
    b.add_container("y", BF16, True)
    b.add_container("out", BF16, True)
    for n in ("xw", "yw", "t0", "t1"):
        b.add_container(n, F32, False, transient_bytes=64 * 48 * 4)
    b.add_cast_op("x", "xw", [64, 48])
    b.add_cast_op("y", "yw", [64, 48])
    b.add_elementwise_op("mul", "xw", "yw", "t0", [64, 48])
    b.add_elementwise_unary_op("tanh", "t0", "t1", [64, 48])
    b.add_cast_op("t1", "out", [64, 48])
    s = b.move()
    s.schedule("rocm")
    nodes = [n for n in s.library_nodes() if not n["code"].startswith("ROCMOff")]
    assert [n["code"] for n in nodes] == ["ROCMMap"]
    (nest,) = nodes
    assert [r["element_type"] for r in nest["reads"]] == ["BFloat", "BFloat"] and [w["element_type"] for w in nest["writes"]] == ["BFloat"]
    assert [(st["op"], st["type"]) for st in nest["statements"]] == [("assign", "Float"), ("assign", "Float"), ("fp_mul", "Float"),
                                                                     ("tanh", "Float"), ("assign", "BFloat")]
    assert not {"xw", "yw", "t0", "t1"} & set(s.containers)
    s.generate(str(tmp_path))
    (text,) = [p.read_text() for p in sorted(tmp_path.glob("kernel_*.hip"))]
    assert "const __bf16* p__in0, const __bf16* p__in1, __bf16* p__out0" in text
    assert "docc_load<__bf16, V, true>" in text and "docc_store<__bf16, V>" in text
    assert "const float _v0 = (float) (_in0);" in text and "const __bf16 _v4 = (__bf16) (_v3);" in text
    # arithmetic on bf16 values is not a nest
    bad = StructuredSDFGBuilder("bad_bf16")
    bad.add_container("A", BF16, True)
    bad.add_map_nest([("i", 8)], [("a", "A", ["1"])], [("p", "fp_add", ["a", "a"])], [("A", ["1"], "p")])
    with pytest.raises(InvalidSDFGException, match="must be Float or Double"):
        bad.move().validate()


def test_causal_attention_binds_its_entry_point(tmp_path):
    """The Attention node's causal flag serialises and selects docc_rocm_attention_bf16_causal with the workspace the widened
    head dimensions need; a head dimension above 128 is declined."""
    b = StructuredSDFGBuilder("ca")
    for n in ("Q", "K", "V", "O"):
        b.add_container(n, BF16, True)
    b.add_attention("Q", "K", "V", "O", [2, 4, 128, 80], 128, 0.1, causal=True)
    s = b.move()
    assert StructuredSDFG.parse(s.to_json()).library_nodes()[0]["causal"] is True
    s.schedule("rocm", options={"offload": "none"})
    text = re.sub(r"\s+", " ", source_of(s, tmp_path)[0])
    assert "docc_rocm_attention_bf16_workspace_bytes(2, 4, 128, 128, 80, 1)" in text
    assert "docc_rocm_attention_bf16_causal(nullptr, 2, 4, 128, 128, 80, (float) (0.1), (const uint16_t *) Q" in text and "__ws, __ws_bytes));" in text
    b = StructuredSDFGBuilder("cb")
    for n in ("Q", "K", "V", "O"):
        b.add_container(n, BF16, True)
    b.add_attention("Q", "K", "V", "O", [1, 1, 64, 256], 64, 0.1, causal=True)
    with pytest.raises(InvalidSDFGException, match="causal"):
        b.move().schedule("rocm")
    # without the flag nothing changes
    b = StructuredSDFGBuilder("cc")
    for n in ("Q", "K", "V", "O"):
        b.add_container(n, BF16, True)
    b.add_attention("Q", "K", "V", "O", [1, 1, 64, 64], 64, 0.1)
    s = b.move()
    assert "causal" not in s.library_nodes()[0]
