"""Pins the oracle's f16 conversions, block decoding and integer block dots.

Sources of truth: numpy float16 (IEEE binary16, RNE), the closed-form blocks of the
reference's own unit tests (wick/src/quant.rs:501-741), python integers."""
import numpy as np
import pytest

from conftest import GOLDEN  # noqa: F401


def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_bits_to_f32(int(b)) for b in bits], np.float32)
    same = (ref.view(np.uint32) == got.view(np.uint32)) | (np.isnan(ref) & np.isnan(got))
    assert same.all()


def test_f32_to_f16_rne(oracle):
    rng = np.random.default_rng(3)
    xs = [rng.standard_normal(4000).astype(np.float32) * np.float32(s) for s in (1e-9, 3e-8, 1e-6, 6e-5, 1e-3, 1, 300, 6.5e4)]
    # exact ties between neighbouring halfs, smallest subnormal boundaries, overflow boundary
    h = np.arange(0, 0x7BFF, 7, dtype=np.uint16).view(np.float16).astype(np.float64)
    hn = np.arange(1, 0x7C00, 7, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((h + hn) / 2).astype(np.float32)
    edge = np.array([0.0, -0.0, 2.0**-25, np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-24, 1.5 * 2.0**-24,
                     2.0**-14, np.nextafter(np.float32(2.0**-14), np.float32(0)), 65504.0, 65519.99, 65520.0, 1e9, np.inf, -np.inf],
                    np.float32)
    allx = np.concatenate(xs + [ties, -ties, edge])
    with np.errstate(over="ignore"):
        ref = allx.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16_bits(float(v)) for v in allx], np.uint16)
    assert np.array_equal(got, ref)


def _q4_block(d_bits, qs):
    return np.concatenate([np.array([d_bits & 0xFF, d_bits >> 8], np.uint8), np.asarray(qs, np.uint8)])


def _q8_block(d_bits, quants):
    return np.concatenate([np.array([d_bits & 0xFF, d_bits >> 8], np.uint8), np.asarray(quants, np.int8).view(np.uint8)])


def _h(f):
    return int(np.float16(f).view(np.uint16))


def test_dequant_q4_0_closed_forms(oracle):
    # wick/src/quant.rs:502-514: all nibbles 8 -> zero
    out = oracle.dequant_row(oracle.Q4_0, _q4_block(_h(1.0), [0x88] * 16))
    assert np.array_equal(out, np.zeros(32, np.float32))
    # wick/src/quant.rs:516-544: lo nibble i, hi nibble 15, d = 0.5
    out = oracle.dequant_row(oracle.Q4_0, _q4_block(_h(0.5), [i | (15 << 4) for i in range(16)]))
    assert np.array_equal(out[:16], (np.arange(16) - 8) * 0.5)
    assert np.array_equal(out[16:], np.full(16, 3.5))


def test_dequant_q8_0_closed_forms(oracle):
    # wick/src/quant.rs:569-586
    out = oracle.dequant_row(oracle.Q8_0, _q8_block(_h(0.5), np.arange(32)))
    assert np.array_equal(out, np.arange(32) * 0.5)
    # wick/src/quant.rs:589-631: two blocks in one row
    row = np.concatenate([_q8_block(_h(1.0), np.arange(32) - 16), _q8_block(_h(0.25), [1] * 32)])
    out = oracle.dequant_row(oracle.Q8_0, row)
    assert np.array_equal(out[:32], np.arange(32) - 16.0)
    assert np.array_equal(out[32:], np.full(32, 0.25))


def _py_block_dot(dtype, blk, xq):
    if dtype == 2:
        qs = blk[2:18]
        return sum((int(qs[i] & 0xF) - 8) * int(xq[i]) + (int(qs[i] >> 4) - 8) * int(xq[16 + i]) for i in range(16))
    w = blk[2:34].view(np.int8)
    return sum(int(w[i]) * int(xq[i]) for i in range(32))


@pytest.mark.parametrize("dtype", [2, 8])
def test_block_dots_extremes_and_random(oracle, dtype):
    rng = np.random.default_rng(dtype)
    bb = 18 if dtype == 2 else 34
    blocks, xs = [], []
    # every combination of the integer extremes on both sides
    w_ext = ([0x00, 0xFF, 0x0F, 0xF0, 0x88] if dtype == 2 else [-128, 127, -1, 0, 1])
    x_ext = [-128, -127, 127, 0, 1]
    for wv in w_ext:
        for xv in x_ext:
            if dtype == 2:
                blocks.append(_q4_block(0x3C00, [wv] * 16))
            else:
                blocks.append(_q8_block(0x3C00, [wv] * 32))
            xs.append(np.full(32, xv, np.int8))
    for _ in range(200):
        blocks.append(rng.integers(0, 256, bb).astype(np.uint8))
        xs.append(rng.integers(-128, 128, 32).astype(np.int8))
    # each (block, x) pair as its own m=1, n=1, k=32 problem
    for blk, xq in zip(blocks, xs):
        got = oracle.block_dots_i32(dtype, blk, xq, 1, 1, 32)[0, 0, 0]
        assert got == _py_block_dot(dtype, blk, xq)
    # bounds stated for the contract: |isum| <= 32*8*128 (Q4_0), 32*128*128 (Q8_0)
    lim = 32 * 8 * 128 if dtype == 2 else 32 * 128 * 128
    big = max(abs(_py_block_dot(dtype, b, x)) for b, x in zip(blocks, xs))
    assert big <= lim


@pytest.mark.parametrize("dtype", [2, 8])
def test_block_dots_layout(oracle, dtype):
    """out[(j*m + i)*nb + b] indexing against a direct python loop."""
    rng = np.random.default_rng(10 + dtype)
    m, n, k = 3, 2, 96
    bb = 18 if dtype == 2 else 34
    a = rng.integers(0, 256, m * (k // 32) * bb).astype(np.uint8)
    xq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    got = oracle.block_dots_i32(dtype, a, xq, m, n, k)
    for j in range(n):
        for i in range(m):
            for b in range(k // 32):
                blk = a[(i * (k // 32) + b) * bb:(i * (k // 32) + b + 1) * bb]
                assert got[j, i, b] == _py_block_dot(dtype, blk, xq[j, b * 32:(b + 1) * 32])
