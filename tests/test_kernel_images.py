"""Checks on the built kernel images that no run on a GPU makes visible.

The bf16 GEMM on the 16x16x32 MFMA (csrc/kernels/gemm_async16.h) writes its MFMAs as asm statements with the
accumulator tied to its registers. The compiler therefore does not know their latency: an accumulator register read by
another instruction right behind the MFMA that writes it would see the old value now and then. The kernel is written
so that the compiler has no reason to touch accumulators between the first and the last MFMA (one loop of identical
straight code) and puts no-ops before the epilogue; this test holds the compiled code to that."""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
LLVM = Path("/opt/rocm/lib/llvm/bin")


def disassembly(image: Path, tmp_path: Path) -> str:
    bundler, objdump = LLVM / "clang-offload-bundler", LLVM / "llvm-objdump"
    if not bundler.exists() or not objdump.exists():
        pytest.skip("no clang-offload-bundler / llvm-objdump in this ROCm installation")
    obj = tmp_path / (image.stem + ".co")
    subprocess.run([str(bundler), "--unbundle", "--type=o", f"--input={image}", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950",
                    f"--output={obj}"], check=True, capture_output=True)
    return subprocess.run([str(objdump), "-d", str(obj)], check=True, capture_output=True, text=True).stdout


@pytest.mark.parametrize("image", ["docc_rocm_gemm_bf16_async_big.hsaco", "docc_rocm_gemm_bf16_async_big_epilogue.hsaco"])
def test_no_accumulator_is_touched_between_the_mfmas_of_the_16x16x32_gemm(tmp_path, image):
    path = ROOT / "docc_amd" / "lib" / image
    if not path.exists():
        pytest.skip("kernel images are not built")
    text = disassembly(path, tmp_path)
    functions = re.split(r"\n(?=[0-9a-f]{16} <)", text)
    seen = 0
    for body in functions:
        m = re.match(r"[0-9a-f]{16} <(docc_bgemma_256x256x32q4_\w+)>:", body)
        if not m:
            continue
        seen += 1
        lines = [ln.split("//")[0].strip() for ln in body.splitlines()[1:]]
        lines = [ln for ln in lines if ln]
        mfma = [i for i, ln in enumerate(lines) if ln.startswith("v_mfma_f32_16x16x32_bf16")]
        assert len(mfma) == 128, (m.group(1), len(mfma))                      # two K-steps of 64, nothing peeled
        inside = lines[mfma[0]:mfma[-1] + 1]
        touched = [ln for ln in inside if ln.startswith("v_accvgpr") or re.match(r"v_\w+ .*\ba\[?\d", ln) and not ln.startswith("v_mfma")]
        assert not touched, (m.group(1), touched[:5])
        # every MFMA accumulates in place
        for i in mfma:
            ops = [o.strip() for o in lines[i].split(None, 1)[1].split(",")]
            assert ops[0] == ops[3] and ops[0].startswith("a["), (m.group(1), lines[i])
        # behind the last MFMA: the no-ops, before anything reads an accumulator
        after = lines[mfma[-1] + 1:]
        first_read = next(i for i, ln in enumerate(after) if ln.startswith("v_accvgpr"))
        assert sum(1 for ln in after[:first_read] if ln == "s_nop 15") >= 2, (m.group(1), after[:first_read][-6:])
    assert seen == 4, seen
