"""Builds the native parts of the docc `rocm` target, in-tree.

Products (all under ``docc_amd/lib/``):

* ``docc_rocm_<family>.hsaco``  gfx950 code objects, one per kernel family
  (``hipcc --genco --offload-arch=gfx950``);
* ``libdocc_rt_rocm.so``       the thin C-ABI runtime and the op launchers
  (``include/docc_rocm_rt.h``, ``include/docc_rocm_ops.h``);
* ``libdocc_rocm_target.so``   the library-node descriptors, dispatcher
  registry, rocm plugin and host-code generator (``include/docc_rocm_target.h``).

The reference drives its own compile steps with ``std::system`` from
``python/bindings/py_structured_sdfg.cpp:355-560``; this module is the
counterpart for the pre-built pieces and is what ``__graft_entry__.build()``
calls.  Run ``python -m docc_amd.build`` to (re)build everything.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
PKG = ROOT / "docc_amd"
CSRC = PKG / "csrc"
LIB = PKG / "lib"
INCLUDE = ROOT / "include"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

# kernel family -> source file; keep in step with kKernelImages in csrc/rt/runtime.cpp
KERNEL_FAMILIES = {
    "util": "util.hip",
    "softmax": "softmax.hip",
    "gemm_f32": "gemm_f32.hip",
    "gemm_f64": "gemm_f64.hip",
    "gemm_bf16": "gemm_bf16.hip",
    "gemm_bf16_async": "gemm_bf16_async.hip",
    "gemm_bf16_async_big": "gemm_bf16_async_big.hip",
    "gemm_f32_epilogue": "gemm_f32_epilogue.hip",
    "gemm_f64_epilogue": "gemm_f64_epilogue.hip",
    "gemm_bf16_epilogue": "gemm_bf16_epilogue.hip",
    "gemm_bf16_async_epilogue": "gemm_bf16_async_epilogue.hip",
    "gemm_bf16_async_big_epilogue": "gemm_bf16_async_big_epilogue.hip",
    "gemm_f32_big": "gemm_f32_big.hip",
    "gemm_f32_big_epilogue": "gemm_f32_big_epilogue.hip",
    "conv2d": "conv2d.hip",
    "attention": "attention.hip",
    "elementwise": "elementwise.hip",
    "reduce": "reduce.hip",
    "transpose": "transpose.hip",
    "gemv": "gemv.hip",
    "gemm_skinny": "gemm_skinny.hip",
}

# Per-family extra device flags. "-amdgpu-mfma-vgpr-form" keeps MFMA accumulators in ordinary
# VGPRs: without it the compiler parks loop-carried accumulators in VGPRs and copies them to and
# from AGPRs around the MFMAs of every K-step (64 extra VALU instructions per step for a
# 32-register accumulator). Families whose accumulators alone need more than 256 registers
# (the 256x256 bf16 tile) cannot use it.
FAMILY_FLAGS = {
    "gemm_f64": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_f32": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_bf16_async": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_f64_epilogue": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_f32_epilogue": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_bf16_async_epilogue": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "conv2d": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "attention": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_skinny": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}

# packed fp32 VALU ops are switched off for every device compile
DEVICE_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or str(ROCM / "bin" / "hipcc")
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; the rocm target needs the ROCm toolchain to build")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed:\n  " + " ".join(cmd) + "\n" + proc.stdout + proc.stderr)


def _newer(target: Path, sources: list[Path]) -> bool:
    if not target.exists():
        return False
    t = target.stat().st_mtime
    return all(s.stat().st_mtime <= t for s in sources)


def build_kernel_family(family: str, force: bool = True) -> Path:
    src = CSRC / "kernels" / KERNEL_FAMILIES[family]
    out = LIB / f"docc_rocm_{family}.hsaco"
    deps = [src] + sorted((CSRC / "kernels").glob("*.h")) + sorted((CSRC / "kernels").glob("gemm*.hip"))
    if not force and _newer(out, deps):
        return out
    LIB.mkdir(parents=True, exist_ok=True)
    _run([hipcc(), "--genco", *DEVICE_FLAGS, *FAMILY_FLAGS.get(family, []), "-I", str(CSRC / "kernels"), str(src), "-o", str(out)])
    return out


def build_kernels(force: bool = True, jobs: int = 8) -> list[Path]:
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        return list(pool.map(lambda f: build_kernel_family(f, force), KERNEL_FAMILIES))


def build_runtime(force: bool = True) -> Path:
    srcs = sorted((CSRC / "rt").glob("*.cpp"))
    hip_srcs = sorted((CSRC / "rt").glob("*.hip"))
    deps = srcs + hip_srcs + sorted((CSRC / "rt").glob("*.h")) + sorted(INCLUDE.glob("*.h"))
    out = LIB / "libdocc_rt_rocm.so"
    if not force and _newer(out, deps):
        return out
    LIB.mkdir(parents=True, exist_ok=True)
    # the one HIP source of the runtime (a device array whose address host code asks for) goes through hipcc;
    # its object carries the device image and registers it when the library is loaded
    objs = []
    for src in hip_srcs:
        obj = LIB / (src.stem + ".o")
        _run([hipcc(), "-c", "-fPIC", *DEVICE_FLAGS, "-I", str(INCLUDE), "-I", str(CSRC / "rt"), str(src), "-o", str(obj)])
        objs.append(obj)
    _run([
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-D__HIP_PLATFORM_AMD__",
        "-I", str(INCLUDE), "-I", str(CSRC / "rt"), "-I", str(ROCM / "include"),
        *map(str, srcs), *map(str, objs), "-o", str(out),
        "-L", str(ROCM / "lib"), "-lamdhip64", "-ldl", f"-Wl,-rpath,{ROCM / 'lib'}",
    ])
    return out


def build_rtl(force: bool = True) -> Path:
    """libdocc_rtl_rocm.so: the `__daisy_instrumentation_*` runtime with the ROCm event set
    (needs libdocc_rt_rocm.so, built first)."""
    srcs = sorted((CSRC / "rtl").glob("*.cpp"))
    deps = srcs + sorted(INCLUDE.glob("*.h"))
    out = LIB / "libdocc_rtl_rocm.so"
    if not force and _newer(out, deps):
        return out
    LIB.mkdir(parents=True, exist_ok=True)
    _run([
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", str(INCLUDE), *map(str, srcs), "-o", str(out),
        "-L", str(LIB), "-ldocc_rt_rocm", "-ldl", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{ROCM / 'lib'}",
    ])
    return out


def build_target(force: bool = True) -> Path | None:
    srcs = sorted((CSRC / "target").glob("*.cpp"))
    if not srcs:
        return None
    deps = srcs + sorted((CSRC / "target").glob("*.h")) + sorted(INCLUDE.glob("*.h"))
    out = LIB / "libdocc_rocm_target.so"
    if not force and _newer(out, deps):
        return out
    LIB.mkdir(parents=True, exist_ok=True)
    _run([
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
        "-I", str(INCLUDE), "-I", str(CSRC / "target"), *map(str, srcs), "-o", str(out),
    ])
    return out


def build_all(force: bool = True) -> dict[str, list[str]]:
    built = {"kernels": [str(p) for p in build_kernels(force)], "runtime": [str(build_runtime(force))]}
    built["rtl"] = [str(build_rtl(force))]
    target = build_target(force)
    if target:
        built["target"] = [str(target)]
    return built


if __name__ == "__main__":
    force = "--if-stale" not in sys.argv
    for kind, paths in build_all(force).items():
        for p in paths:
            print(f"{kind}: {p}")
