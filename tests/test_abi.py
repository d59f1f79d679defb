"""The C-ABI libraries load on a machine without a GPU and export every symbol the public
headers declare; no compute entry point is called here."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
INCLUDE = ROOT / "include"


def declared_functions(header: Path):
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(docc_rocm_\w+)\s*\(", text)))


def test_runtime_library_exports_every_declared_symbol():
    from docc_amd import runtime

    lib = ctypes.CDLL(str(runtime.LIB_PATH))
    declared = declared_functions(INCLUDE / "docc_rocm_rt.h") + declared_functions(INCLUDE / "docc_rocm_ops.h")
    assert len(declared) >= 35
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported"
    # and the Python binding covers exactly the declared set
    assert sorted(runtime.EXPORTED_SYMBOLS) == sorted(declared)


def test_target_library_exports_every_declared_symbol():
    import docc_amd.sdfg as sdfg

    lib = ctypes.CDLL(str(sdfg._TARGET_LIB))
    declared = declared_functions(INCLUDE / "docc_rocm_target.h")
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported"
    assert sorted(sdfg.EXPORTED_SYMBOLS) == sorted(declared)


def test_kernel_images_are_built():
    from docc_amd import build, runtime

    for family in build.KERNEL_FAMILIES:
        assert (runtime.LIB_DIR / f"docc_rocm_{family}.hsaco").exists(), family
    # the runtime's image list and the build's family list name the same files
    src = (ROOT / "docc_amd" / "csrc" / "rt" / "runtime.cpp").read_text()
    listed = set(re.findall(r'"docc_rocm_(\w+)\.hsaco"', src))
    assert listed == set(build.KERNEL_FAMILIES)


def test_kernels_the_launchers_name_are_in_the_images():
    """Every kernel a launcher names outright (a string literal, not a pattern filled in at run time) is a symbol
    of one of the built images."""
    from docc_amd import runtime

    # the images are offload bundles around an ELF object: a kernel's name stands in its string table, NUL-terminated
    images = b"\0".join(image.read_bytes() for image in sorted(runtime.LIB_DIR.glob("docc_rocm_*.hsaco")))
    named = set()
    for src in (ROOT / "docc_amd" / "csrc" / "rt").glob("*.cpp"):
        named.update(re.findall(r'"(docc_[a-z0-9_]+)"', src.read_text()))
    named = {n for n in named if not n.startswith("docc_rocm_")}      # entry points of the library itself, not kernels
    assert {"docc_transpose_tile4_b32", "docc_copy_b128", "docc_splitk_combine_f32", "docc_pad_rows_b16"} <= named
    # names the launchers put together at run time: the forms of the row softmax in both precisions (ops_softmax.cpp,
    # noalloc.hip), the LDS-halo convolution (ops_conv.cpp) and the attention kernels (ops_attention.cpp)
    forms = ["stream", "slab", "tile", "tilev16", "tilev4", "sliced_partial", "sliced_finish", "slicedv_partial", "slicedv_finish", "rowslice_partial", "rowslice_finish", "block8_v2", "block16_v8",
             "block16_v16", "any4_v1", "any4_v4", "any4_v16", "any16_v8", "any16_v16"]
    forms += [f"wave_v{v}" for v in (1, 2, 4, 8, 16)] + [f"block_v{v}" for v in (1, 2, 4, 8, 16)] + [f"sub{v}" for v in (1, 2, 4, 8, 16, 32)]
    named |= {f"docc_softmax_{t}_{form}" for t in ("f32", "f64") for form in forms}
    named |= {f"docc_conv2d_f32_halo_{k}{form}" for k, fs in (("3x3", ("", "_split", "_split16", "_t4", "_t2", "_t4m", "_t2m")), ("1x1", ("", "_t4", "_t2", "_t4m", "_t2m"))) for form in fs}
    named |= {f"docc_attention_bf16_d{d}_q{q}_{o}" for d in (32, 64, 128) for q in (128, 256) for o in ("f32out", "bf16out")}
    # the entry point that may look nothing up at a call resolves every one of these forms at set-up
    listed = re.search(r"forms\[\] = \{(.*?)\};", (ROOT / "docc_amd" / "csrc" / "rt" / "noalloc.hip").read_text(), re.S).group(1)
    assert set(re.findall(r'"([a-z0-9_]+)"', listed)) == set(forms)
    missing = sorted(n for n in named if b"\0" + n.encode() + b"\0" not in images)
    assert not missing, missing
    assert b"\0docc_conv2d_f32_halo_3x3_split17\0" not in images      # the check can fail


def test_runtime_reports_errors_without_a_gpu_or_with_bad_arguments():
    import torch

    from docc_amd import runtime

    assert runtime.version().startswith("docc-rocm")
    assert runtime.take_failure() == (0, "")
    if torch.cuda.is_available():
        pytest.skip("error paths below are for a machine without a GPU")
    assert runtime.device_count() == 0
    with pytest.raises(runtime.RocmRuntimeError) as e:
        runtime.init(0)
    assert e.value.code == -4 and "no HIP device" in str(e.value)
    # argument validation comes before any device work
    with pytest.raises(runtime.RocmRuntimeError) as e:
        runtime.sgemm(4, 4, 4, 1.0, 1, 2, 1, 4, 0.0, 1, 4)
    assert e.value.code == -1
    with pytest.raises(runtime.RocmRuntimeError):
        runtime.attention_bf16(1, 1, 8, 8, 128, 0.1, 16, 16, 16, 16)
    # there is no CPU fallback: a well-formed call fails loudly when no device is present
    with pytest.raises(runtime.RocmRuntimeError):
        runtime.softmax_f32(4, 4, 16, 16)
    # the failure channel of generated code keeps the first report
    runtime.lib().docc_rocm_report_failure(b"f", b"docc_rocm_malloc_async(...)", 2)
    runtime.lib().docc_rocm_report_failure(b"g", b"later", 3)
    code, message = runtime.take_failure()
    assert code == 2 and "docc_rocm_malloc" in message
    assert runtime.take_failure() == (0, "")
