"""Writes tests/golden/q8_0_quantizer_vectors.npz.

An INDEPENDENT restatement, in numpy float32 arithmetic, of the reference's Q8_0
activation quantizer (wick/src/backend/simd.rs:255-323).  The reference holds no
test vector for the exact bits of that function and cannot be built here (Rust,
aarch64-only), but every step is a single correctly rounded IEEE-754 binary32
operation (divide, divide, multiply, round-to-nearest-even, f32->f16 RNE), so any
two faithful implementations agree bit for bit.  The C oracle and the HIP kernel
are both checked against this file.

Run from the repository root:  python tests/golden/make_q8_0_quantizer_vectors.py
"""
import os

import numpy as np

F = np.float32


def quantize_q8_0_numpy(x: np.ndarray):
    x = np.asarray(x, F).reshape(-1, 32)
    amax = np.abs(x).max(axis=1).astype(F)
    d = (amax / F(127.0)).astype(F)
    with np.errstate(divide="ignore"):
        inv = (F(1.0) / d).astype(F)
    idv = np.where(d != 0, inv, F(0.0)).astype(F)
    scaled = (x * idv[:, None]).astype(F)
    q = np.rint(scaled).astype(np.int32).astype(np.int8)  # rint = ties-to-even; i32 -> i8 truncates
    with np.errstate(over="ignore"):
        scales = d.astype(np.float16).astype(F)  # stored scale = f32(f16(d)), may be inf or 0
    return scales, q.reshape(-1)


def edge_blocks() -> np.ndarray:
    rng = np.random.default_rng(20260101)
    blocks = []
    blocks.append(np.zeros(32, F))  # all zero: d = 0, id = 0
    b = np.zeros(32, F); b[5] = 3.25; blocks.append(b)  # single +max
    b = np.zeros(32, F); b[31] = -7.5; blocks.append(b)  # single -max
    # amax = 127 -> d = id = 1: exact ties at .5 go to even
    b = np.array([127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 126.5, -126.5, 125.5, 0.49999997, 0.50000006] + [0.0] * 19, F)
    blocks.append(b)
    # amax = 127 * 2^n exact
    for e in (-20, -3, 4, 17):
        b = rng.integers(-127, 128, 32).astype(F) * F(2.0**e); b[0] = F(127.0 * 2.0**e); blocks.append(b)
    # stored f16 scale is subnormal (d < 2^-14) / rounds to zero (d < 2^-25) / overflows to inf (d >= 65520)
    for amax in (1e-3, 5e-4, 1e-6, 3e-7, 8.4e6, 1e9):
        b = (rng.standard_normal(32) * 0.3).astype(F); b = b / np.abs(b).max() * F(amax); blocks.append(b.astype(F))
    # very small / very large but normal f32 all the way through
    for amax in (1e-30, 1e30):
        b = rng.uniform(-1, 1, 32).astype(F) * F(amax); blocks.append(b)
    # values whose product with id lands just beside .5
    for amax in (1.0, 3.0, 10.0, 0.1, 77.7):
        d = F(amax) / F(127.0)
        ks = rng.integers(-126, 126, 32).astype(F) + F(0.5)
        b = (ks * d).astype(F); b[0] = F(amax); blocks.append(b)
    # negative zero, mixed signs
    b = np.full(32, -0.0, F); b[3] = 1.0; b[4] = -1.0; blocks.append(b)
    return np.concatenate(blocks).astype(F)


def main():
    rng = np.random.default_rng(7)
    x_normal = rng.standard_normal(64 * 32).astype(F)
    x_wide = (rng.standard_normal(64 * 32) * np.exp(rng.uniform(-8, 8, 64 * 32))).astype(F)
    x_edge = edge_blocks()
    out = {}
    for name, x in (("normal", x_normal), ("wide", x_wide), ("edge", x_edge)):
        s, q = quantize_q8_0_numpy(x)
        out[f"{name}_x"] = x
        out[f"{name}_scales"] = s
        out[f"{name}_quants"] = q
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "q8_0_quantizer_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
