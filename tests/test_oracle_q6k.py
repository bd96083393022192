"""Pins the oracle's Q6_K functions without the reference at hand: the reference's own
closed-form blocks (wick/src/quant.rs:819-880), an independent numpy restatement of the
bit layout (written from dequantize_q6_k_block's index arithmetic, quant.rs:380-412, with
array slicing instead of the oracle's per-element formula), python-integer brute force for
the group dots and an f64 dequantize-then-dot for the GEMV."""
import numpy as np
import pytest

from oracle import oracle as O


def numpy_dequant_q6_k(blocks: np.ndarray) -> np.ndarray:
    """blocks: uint8 [nblocks, 210] -> f32 [nblocks, 256], slice by slice like the reference's loop."""
    nbk = blocks.shape[0]
    ql, qh = blocks[:, :128].astype(np.int32), blocks[:, 128:192].astype(np.int32)
    sc = blocks[:, 192:208].view(np.int8).astype(np.float32)
    d = blocks[:, 208:210].copy().view(np.float16).astype(np.float32)  # [nbk, 1]
    out = np.zeros((nbk, 256), np.float32)
    for n in range(2):
        lo, hi, h = ql[:, 64 * n:64 * n + 32], ql[:, 64 * n + 32:64 * n + 64], qh[:, 32 * n:32 * n + 32]
        q1 = ((lo & 15) | ((h & 3) << 4)) - 32
        q2 = ((hi & 15) | (((h >> 2) & 3) << 4)) - 32
        q3 = ((lo >> 4) | (((h >> 4) & 3) << 4)) - 32
        q4 = ((hi >> 4) | (((h >> 6) & 3) << 4)) - 32
        isx = np.arange(32) // 16
        for j, q in enumerate((q1, q2, q3, q4)):
            s = sc[:, 8 * n + isx + 2 * j]
            out[:, 128 * n + 32 * j:128 * n + 32 * j + 32] = (d * s).astype(np.float32) * q.astype(np.float32)
    return out


def random_q6k(rng, m, k):
    nbk = m * (k // 256)
    b = rng.integers(0, 256, (nbk, 210)).astype(np.uint8)
    b[:, 208:210] = np.array([0.01], np.float16).view(np.uint8)  # a sane super-block scale
    return b.reshape(-1)


def test_reference_block_all_quants_32_is_zero():
    """test_dequantize_q6_k_basic (quant.rs:819-846): ql = 0, qh = 0xAA, scales = 1, d = 1 -> all zeros."""
    blk = np.zeros(210, np.uint8)
    blk[128:192] = 0xAA
    blk[192:208] = 1
    blk[208:210] = np.array([1.0], np.float16).view(np.uint8)
    assert np.all(O.dequant_q6_k(blk, 1, 256) == 0.0)


def test_reference_varied_block_both_ways():
    """test_vec_dot_q6_k_matches_dequantize (quant.rs:849-880): the varied block, dequantized by the
    oracle and by the numpy restatement, and its dot with y = (i - 128) * 0.01."""
    blk = np.zeros(210, np.uint8)
    i = np.arange(128)
    blk[:128] = (i % 13) | ((i % 9) << 4)
    blk[128:192] = np.arange(64) % 256
    blk[192:208] = (np.arange(16) % 5 + 1).astype(np.int8).view(np.uint8)
    blk[208:210] = np.array([0.5], np.float16).view(np.uint8)
    a = O.dequant_q6_k(blk, 1, 256)[0]
    b = numpy_dequant_q6_k(blk.reshape(1, 210))[0]
    assert np.array_equal(a, b)
    # spot values by hand: element 0: ql[0] = 0 -> low nibble 0, qh[0] = 0 -> q = -32, scale 1, d 0.5
    assert a[0] == 0.5 * 1 * -32
    # element 255 = n 1, j 3, l 31: ql[64+32+31] = 127 % 13 | (127 % 9) << 4 = 10 | 1 << 4 -> high nibble 1;
    # qh[32+31] = 63 -> bits 6-7 = 0 -> q = 1 - 32; scale index 15 -> 15 % 5 + 1 = 1
    assert a[255] == 0.5 * 1 * (1 - 32)
    y = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    assert abs(float(np.dot(a.astype(np.float64), y)) - float(np.dot(b.astype(np.float64), y))) == 0.0


@pytest.mark.parametrize("m,k", [(3, 256), (5, 1024), (2, 1536)])
def test_dequant_matches_numpy_restatement(m, k):
    rng = np.random.default_rng(m * 1000 + k)
    a = random_q6k(rng, m, k)
    ref = numpy_dequant_q6_k(a.reshape(-1, 210)).reshape(m, k)
    assert np.array_equal(O.dequant_q6_k(a, m, k), ref)


def test_group_dots_brute_force_with_python_ints():
    rng = np.random.default_rng(7)
    m, k = 2, 512
    a = random_q6k(rng, m, k)
    q = rng.integers(-128, 128, k).astype(np.int8)
    q[:32] = 127
    q[32:64] = -128
    got = O.q6k_group_dots_i32(a, q, m, k)
    # integer weights = dequant with d = 1 and scales = 1
    ints = a.reshape(-1, 210).copy()
    ints[:, 192:208] = 1
    ints[:, 208:210] = np.array([1.0], np.float16).view(np.uint8)
    w = numpy_dequant_q6_k(ints).reshape(m, k)
    for i in range(m):
        for g in range(k // 16):
            ref = sum(int(w[i, 16 * g + t]) * int(q[16 * g + t]) for t in range(16))
            assert got[i, g] == ref
    assert got.min() >= -32 * 128 * 16 and got.max() <= 32 * 128 * 16


@pytest.mark.parametrize("m,k", [(4, 256), (7, 1024), (3, 2048)])
def test_gemv_matches_f64_dequantize_then_dot(m, k):
    rng = np.random.default_rng(k + m)
    a = O.synth_weight(O.Q6_K, m, k, seed=5 + m)
    x = O.fill_normal(99, 1.0, k)
    s, q = O.quantize_q8_0(x)
    y = O.gemv_q6k_q8(a, s, q, m, k)
    y64 = O.gemv_q6k_q8(a, s, q, m, k, f64=True)
    w = O.dequant_q6_k(a, m, k).astype(np.float64)
    xd = (q.astype(np.float64).reshape(-1, 32) * s.astype(np.float64)[:, None]).reshape(-1)
    ref = w @ xd
    assert np.allclose(y64, ref, rtol=1e-12, atol=1e-12)
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-6


def test_generator_round_trip_error():
    """The synthetic Q6_K encoder is only an input generator; still, dequantizing what it wrote must
    land within half a quantization step (+ the rounding of the int8 group scale) of the input."""
    m, k = 4, 1024
    v = O.fill_normal(3, 0.02, m * k)
    a = O.build_q6_k(v, m, k)
    w = O.dequant_q6_k(a, m, k).reshape(-1)
    amax = np.abs(v.reshape(-1, 16)).max(axis=1)
    err = np.abs(w - v).reshape(-1, 16).max(axis=1)
    assert np.all(err <= amax / 31.0 * 1.1 + 1e-7)
