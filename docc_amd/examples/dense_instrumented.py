"""relu(x @ w + b) through `@native(target="rocm", instrumentation_mode="ols")`.

Every rocm node and transfer of the generated function is a region of the instrumentation
runtime: run it with __DAISY_INSTRUMENTATION_FILE=trace.json (and optionally
__DAISY_INSTRUMENTATION_MODE=aggregate) to get a Chrome trace with device times, `flop` and
`pcie_bytes` per region, or under `rocprofv3 --marker-trace` to see the same regions as roctx
ranges.

    python -m docc_amd.examples.dense_instrumented [rows] [repeats]
"""
import sys

import numpy as np

from docc_amd.python import native, relu


@native(target="rocm", instrumentation_mode="ols")
def dense(x, w, b):
    t = x @ w + b
    return relu(t)


def main(rows: int = 512, repeats: int = 3) -> None:
    rng = np.random.default_rng(0)
    x = rng.standard_normal((rows, 256)).astype(np.float32)
    w = rng.standard_normal((256, 384)).astype(np.float32)
    b = rng.standard_normal(384).astype(np.float32)
    for _ in range(repeats):
        y = dense(x, w, b)
    if not np.allclose(y, np.maximum(x @ w + b, 0), rtol=1e-4, atol=1e-4):
        raise SystemExit("dense_instrumented: result differs from numpy")
    print(f"dense_instrumented: {repeats} x relu([{rows},256] @ [256,384] + b) ok")


if __name__ == "__main__":
    main(*(int(a) for a in sys.argv[1:3]))
