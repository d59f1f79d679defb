"""Instrumentation of generated code: the text of the `__daisy_instrumentation_*` brackets (as
the reference prints them, sdfg/src/codegen/instrumentation/instrumentation_plan.cpp:22-141), the
"ols" / "" / unknown modes (python/bindings/py_structured_sdfg.cpp:376-383), and the runtime behind
the calls: regions, aggregation, and the Chrome trace layout of the reference's
rtl/src/instrumentation.cpp:173-456. Runs without a GPU (the ROCm event set then measures wall-clock time)."""
import ctypes
import json
import re
import subprocess
import sys
import textwrap
from pathlib import Path

import numpy as np
import pytest

from docc_amd import runtime
from docc_amd.python import native, relu
from docc_amd.sdfg import InvalidSDFGException, Pointer, PrimitiveType, Scalar, StructuredSDFGBuilder

ROOT = Path(__file__).resolve().parent.parent
RTL = runtime.LIB_DIR / "libdocc_rtl_rocm.so"
F32 = Pointer(Scalar(PrimitiveType.Float))


def small_sdfg():
    b = StructuredSDFGBuilder("inst")
    for n in ("A", "B", "C"):
        b.add_container(n, F32, True)
    b.add_container("T", F32, False, transient_bytes=16 * 16 * 4)
    b.set_debug_info("/src/model.py", "forward", 10, 5, 11, 30)
    b.add_gemm("A", "B", "T", "1.0", "0.0", 16, 16, 16)
    b.set_debug_info("/src/model.py", "forward", 12, 5, 12, 22)
    b.add_elementwise_unary_op("relu", "T", "C", [16, 16])
    return b.move()


def test_rtl_header_and_library_agree():
    text = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / "docc_rocm_rtl.h").read_text(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(__daisy_instrumentation_\w+|docc_rocm_rtl_\w+)\s*\(", text)))
    assert declared == ["__daisy_instrumentation_enter", "__daisy_instrumentation_exit", "__daisy_instrumentation_finalize",
                        "__daisy_instrumentation_increment", "__daisy_instrumentation_init", "__daisy_instrumentation_metric",
                        "docc_rocm_rtl_flush"]
    lib = ctypes.CDLL(str(RTL))
    for name in declared:
        assert hasattr(lib, name), name
    # the event sets of the reference's header keep their values; ROCM is the added one
    assert re.findall(r"__DAISY_EVENT_SET_(\w+) = (\d)", text) == [("CPU", "0"), ("CUDA", "1"), ("NONE", "2"), ("ROCM", "3")]


def test_brackets_in_the_generated_code(tmp_path):
    s = small_sdfg()
    assert s._data["root"]["children"][0]["debug_info"]["start_line"] == 10
    s.dump(str(tmp_path))                       # records sdfg_file etc. in the metadata
    s.schedule("rocm")
    plain = Path(s.generate(str(tmp_path / "plain"))["source"]).read_text()
    assert "__daisy_instrumentation" not in plain and "docc_rocm_rtl.h" not in (tmp_path / "plain" / "inst.h").read_text()
    report = s.generate(str(tmp_path / "ols"), "ols")
    src = Path(report["source"]).read_text()
    assert '#include "docc_rocm_rtl.h"' in Path(report["header"]).read_text()
    regions = {r["element_type"]: r for r in report["instrumentation"]}
    assert regions["math"]["target_type"] == "ROCM" and regions["h2d_transfer"]["metrics"]["pcie_bytes"] == "1024"
    gemm_id = next(r["element_id"] for r in report["instrumentation"] if r["region"] == "GEMM")
    stem = f"inst_{gemm_id}"
    flat = re.sub(r"\s+", " ", src)
    for piece in (f"__daisy_metadata_t {stem}_md;", f'{stem}_md.file_name = "/src/model.py";', f'{stem}_md.function_name = "forward";',
                  f"{stem}_md.line_begin = 10;", f"{stem}_md.line_end = 11;", f"{stem}_md.column_begin = 5;",
                  f'{stem}_md.sdfg_name = "inst";', f'{stem}_md.sdfg_file = "{tmp_path}/inst.json";',
                  f"{stem}_md.element_id = {gemm_id};", f'{stem}_md.element_type = "math";', f'{stem}_md.target_type = "ROCM";',
                  f"{stem}_md.loopnest_index = -1;", f"{stem}_md.num_loops = 0;", f"{stem}_md.is_perfectly_nested = 0;",
                  f'{stem}_md.region_uuid = "{stem}";',
                  f"long long {stem}_id = __daisy_instrumentation_init(&{stem}_md, __DAISY_EVENT_SET_ROCM);",
                  f"__daisy_instrumentation_enter({stem}_id);", f"__daisy_instrumentation_exit({stem}_id);",
                  f'__daisy_instrumentation_metric({stem}_id, "flop", ', f"__daisy_instrumentation_finalize({stem}_id);"):
        assert piece in flat, piece
    # init < enter < launch < exit < metric < finalize
    order = [flat.index(k) for k in (f"__daisy_instrumentation_init(&{stem}_md", f"__daisy_instrumentation_enter({stem}_id)",
                                     "docc_rocm_sgemm_epilogue(", f"__daisy_instrumentation_exit({stem}_id)",
                                     f"__daisy_instrumentation_metric({stem}_id", f"__daisy_instrumentation_finalize({stem}_id)")]
    assert order == sorted(order)
    # math nodes and transfers are regions; allocations and frees are not
    assert flat.count("__daisy_instrumentation_enter(") == 1 + 2 + 1      # the GEMM with the ReLU in its store; A, B up; C down
    with pytest.raises(InvalidSDFGException, match="Unsupported instrumentation plan: loops"):
        s.generate(str(tmp_path / "bad"), "loops")
    with pytest.raises(NotImplementedError, match="capture"):
        s._compile(str(tmp_path / "cap"), capture_args=True)


def test_native_passes_source_positions_and_mode(tmp_path, monkeypatch):
    monkeypatch.setenv("DOCC_TMP", str(tmp_path / "docc"))

    @native(target="rocm", instrumentation_mode="ols")
    def dense(x, w):
        t = x @ w
        return relu(t)

    x = np.zeros((8, 8), np.float32)
    sdfg = dense.to_sdfg(x, x)
    infos = [c["debug_info"] for c in sdfg._data["root"]["children"]]
    assert all(i["filename"] == __file__ and i["function"] == "dense" for i in infos)
    assert infos[1]["start_line"] == infos[0]["start_line"] + 1
    src_line = Path(__file__).read_text().splitlines()[infos[0]["start_line"] - 1]
    assert src_line.strip() == "t = x @ w"
    compiled = dense.compile(x, x, output_folder=str(tmp_path / "out"))
    text = (tmp_path / "out" / "dense_sdfg.cpp").read_text()
    assert "__daisy_instrumentation_enter" in text and f'.file_name = "{__file__}"' in text
    needed = subprocess.run(["readelf", "-d", str(tmp_path / "out" / "libdense_sdfg.so")], capture_output=True, text=True).stdout
    assert "libdocc_rtl_rocm.so" in needed and "libdocc_rt_rocm.so" in needed
    assert compiled is not None


DRIVER = """
import ctypes, sys
lib = ctypes.CDLL(sys.argv[1])

class MD(ctypes.Structure):
    _fields_ = [("file_name", ctypes.c_char_p), ("function_name", ctypes.c_char_p), ("line_begin", ctypes.c_long),
                ("line_end", ctypes.c_long), ("column_begin", ctypes.c_long), ("column_end", ctypes.c_long),
                ("sdfg_name", ctypes.c_char_p), ("sdfg_file", ctypes.c_char_p), ("arg_capture_path", ctypes.c_char_p),
                ("features_file", ctypes.c_char_p), ("opt_report_file", ctypes.c_char_p), ("element_id", ctypes.c_size_t),
                ("element_type", ctypes.c_char_p), ("target_type", ctypes.c_char_p), ("loopnest_index", ctypes.c_int),
                ("num_loops", ctypes.c_size_t), ("num_maps", ctypes.c_size_t), ("num_fors", ctypes.c_size_t),
                ("num_whiles", ctypes.c_size_t), ("max_depth", ctypes.c_size_t), ("is_perfectly_nested", ctypes.c_bool),
                ("is_perfectly_parallel", ctypes.c_bool), ("is_elementwise", ctypes.c_bool), ("has_side_effects", ctypes.c_bool),
                ("region_uuid", ctypes.c_char_p)]

lib.__daisy_instrumentation_init.restype = ctypes.c_size_t
lib.__daisy_instrumentation_init.argtypes = [ctypes.POINTER(MD), ctypes.c_int]
for f in ("enter", "exit", "finalize"):
    getattr(lib, "__daisy_instrumentation_" + f).argtypes = [ctypes.c_size_t]
lib.__daisy_instrumentation_metric.argtypes = [ctypes.c_size_t, ctypes.c_char_p, ctypes.c_double]
lib.__daisy_instrumentation_increment.argtypes = [ctypes.c_size_t, ctypes.c_char_p, ctypes.c_longlong]

def region(uuid, event_set, element_id, line):
    md = MD(b'/src/"quoted".py', b"forward", line, line + 1, 3, 9, b"net", b"/tmp/net.json", b"", b"", b"", element_id, b"math",
            b"ROCM", -1, 0, 0, 0, 0, 0, False, False, False, False, uuid)
    return lib.__daisy_instrumentation_init(ctypes.byref(md), event_set)

import time
for call in range(3):                 # the generated function runs three times
    a = region(b"net_4", 3, 4, 10)    # ROCM event set (wall clock without a GPU)
    lib.__daisy_instrumentation_enter(a); time.sleep(0.002); lib.__daisy_instrumentation_exit(a)
    lib.__daisy_instrumentation_metric(a, b"flop", 1000.0 * (call + 1))
    lib.__daisy_instrumentation_finalize(a)
    b = region(b"net_6", 0, 6, 20)    # CPU event set
    lib.__daisy_instrumentation_enter(b); lib.__daisy_instrumentation_exit(b)
    lib.__daisy_instrumentation_increment(b, b"calls", 1)
    lib.__daisy_instrumentation_finalize(b)
    assert a != b and region(b"net_4", 3, 4, 10) == a
n = region(b"net_8", 2, 8, 30)        # NONE: metrics only, never timed
lib.__daisy_instrumentation_enter(n); lib.__daisy_instrumentation_exit(n)
lib.__daisy_instrumentation_metric(n, b"bytes", 64.0)
"""


@pytest.mark.parametrize("mode", ["", "aggregate"])
def test_runtime_writes_the_chrome_trace(tmp_path, mode):
    out = tmp_path / "trace.json"
    env = {"PATH": "/usr/bin:/bin", "__DAISY_INSTRUMENTATION_FILE": str(out), "__DAISY_INSTRUMENTATION_MODE": mode}
    r = subprocess.run([sys.executable, "-c", textwrap.dedent(DRIVER), str(RTL)], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    trace = json.loads(out.read_text())            # written at process exit, valid JSON (the quote in the file name is escaped)
    events = trace["traceEvents"]
    by_id = {}
    for e in events:
        by_id.setdefault(e["args"]["docc"]["element_id"], []).append(e)
    first = by_id[4][0]
    # the reference's event layout
    assert first["ph"] == "X" and first["name"] == "forward [L10-11]" and first["pid"] > 0 and first["tid"] > 0
    assert first["args"]["function"] == "forward" and first["args"]["module"] == '"quoted".py'
    assert first["args"]["source_ranges"] == [{"file": '/src/"quoted".py', "from": {"line": 10, "col": 3}, "to": {"line": 11, "col": 9}}]
    docc = first["args"]["docc"]
    assert docc["sdfg_name"] == "net" and docc["sdfg_file"] == "/tmp/net.json" and docc["element_type"] == "math"
    assert docc["loop_info"] == {"loopnest_index": -1, "num_loops": 0, "num_maps": 0, "num_fors": 0, "num_whiles": 0, "max_depth": 0,
                                 "is_perfectly_nested": False, "is_perfectly_parallel": False, "is_elementwise": False,
                                 "has_side_effects": False}
    assert first["args"]["target_type"] == "ROCM"
    if mode == "aggregate":
        assert first["cat"] == "aggregated_region,daisy" and len(by_id[4]) == 1 and len(by_id[6]) == 1
        m = first["args"]["metrics"]
        assert m["static:::flop"] == {"mean": 2000.0, "variance": pytest.approx(2e6 / 3), "count": 3, "min": 1000.0, "max": 3000.0}
        assert m["runtime"]["count"] == 3 and m["runtime"]["min"] >= 2000 and first["dur"] >= 6000      # microseconds
        assert by_id[6][0]["args"]["metrics"]["static:::calls"]["count"] == 3
        assert by_id[8][0]["args"]["metrics"]["static:::bytes"]["mean"] == 64.0 and by_id[8][0]["args"]["metrics"]["runtime"]["count"] == 0
    else:
        assert first["cat"] == "region,daisy" and len(by_id[4]) == 3 and len(by_id[6]) == 3 and 8 not in by_id
        assert all(e["dur"] >= 2000 for e in by_id[4]) and by_id[4][0]["ts"] <= by_id[4][1]["ts"] <= by_id[4][2]["ts"]
        assert first["args"]["metrics"]["static:::flop"] == 2000.0
