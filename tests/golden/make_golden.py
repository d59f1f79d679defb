"""Writes the golden vectors under tests/golden/ (run once; the .npz files are committed).

The reference holds no numeric fixtures for GEMM, softmax, conv or attention (its tests
recompute expectations with numpy/torch on unseeded inputs), so these vectors come from the
closed forms, evaluated here in float64 with numpy only - independently of the oracle and of the
GPU kernels, both of which are tested against them. Nothing from the reference is imported.

    python tests/golden/make_golden.py
"""
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bits (uint16), round to nearest even."""
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_to_f64(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def main():
    rng = np.random.default_rng(20240)
    # GEMM 17x33x65, integer-valued: exact in every dtype and summation order
    A = rng.integers(-8, 9, (17, 65))
    B = rng.integers(-8, 9, (65, 33))
    C0 = rng.integers(-8, 9, (17, 33))
    C = A @ B
    for tag, dt in (("f64", np.float64), ("f32", np.float32)):
        np.savez(HERE / f"gemm_int_17x33x65_{tag}.npz", A=A.astype(dt), B=B.astype(dt), C0=C0.astype(dt), C=C.astype(dt),
                 C_alpha2_beta_m3=(2 * C - 3 * C0).astype(dt))
    np.savez(HERE / "gemm_int_17x33x65_bf16.npz", A=bf16_round(A.astype(np.float32)), B=bf16_round(B.astype(np.float32)),
             C=C.astype(np.float32))

    # softmax 8x257 fp32 (odd width: exercises the unaligned path), N(0,1)*8
    X = (rng.standard_normal((8, 257)) * 8).astype(np.float32)
    x64 = X.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=-1, keepdims=True))
    np.savez(HERE / "softmax_8x257_f32.npz", X=X, Y=(e / e.sum(axis=-1, keepdims=True)))

    # conv 2x3x7x7, 4 output channels, 3x3, pad 1, bias: seven nested loops in float64
    Xc = rng.standard_normal((2, 3, 7, 7)).astype(np.float32)
    Wc = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    bc = rng.standard_normal(4).astype(np.float32)
    Y = np.zeros((2, 4, 7, 7))
    for n in range(2):
        for oc in range(4):
            for oh in range(7):
                for ow in range(7):
                    acc = float(bc[oc])
                    for ic in range(3):
                        for kh in range(3):
                            for kw in range(3):
                                ih, iw = oh - 1 + kh, ow - 1 + kw
                                if 0 <= ih < 7 and 0 <= iw < 7:
                                    acc += float(Xc[n, ic, ih, iw]) * float(Wc[oc, ic, kh, kw])
                    Y[n, oc, oh, ow] = acc
    np.savez(HERE / "conv_2x3x7x7_k3_p1_bias_f32.npz", X=Xc, W=Wc, b=bc, Y=Y)

    # attention 1x2x96x64 bf16, scale 1/8: softmax(Q K^T / 8) V in float64 on the bf16 values
    Q, K, V = (bf16_round(rng.standard_normal((1, 2, 96, 64)).astype(np.float32)) for _ in range(3))
    q, k, v = bf16_to_f64(Q), bf16_to_f64(K), bf16_to_f64(V)
    s = np.einsum("bhid,bhjd->bhij", q, k) * 0.125
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    np.savez(HERE / "attn_1x2x96x64_bf16.npz", Q=Q, K=K, V=V, O=np.einsum("bhij,bhjd->bhid", p, v).astype(np.float32))
    for f in sorted(HERE.glob("*.npz")):
        print(f.name, f.stat().st_size)


if __name__ == "__main__":
    main()
