"""Pins the oracle's GEMV / GEMM and the input generators.

* against a float64 dequantize-then-dot (textbook GEMM): catches a dropped term,
  wrong nibble order, transposed operand, wrong scale index;
* GEMM == per-column GEMV on the reference's own shapes and inputs
  (wick/src/backend/simd.rs:1440-1623);
* the Q8_0 closed form y = -16/(row+1) of test_q8_0_gemm_standalone
  (wick/tests/bench_perf.rs:852-971);
* the dequantize-and-multiply references of the reference's GPU tests
  (wick/tests/gemv_q4_0_bench.rs:38-56, wick/src/backend/wgpu.rs:747-769) at their
  tolerance max_abs < 1e-2 or max_rel < 1e-3."""
import numpy as np
import pytest

from conftest import rel_l2


def ref_weights(m, k):  # simd.rs:1448-1450
    i = np.arange(m * k)
    return (((i * 17 + 3) % 29).astype(np.float32) * np.float32(0.1) - np.float32(1.4)).astype(np.float32)


def ref_inputs(n, k):  # simd.rs:1454-1460
    i = np.arange(k)
    return np.stack([(((i * 13 + j * 7 + 5) % 23).astype(np.float32) * np.float32(0.2) - np.float32(2.3)) for j in range(n)]).astype(np.float32)


def dequant_f64(oracle, dtype, a, s, q, m, k):
    W = oracle.dequant_matrix(dtype, a, m, k).astype(np.float64)
    X = q.reshape(-1, k // 32, 32).astype(np.float64) * s.reshape(-1, k // 32, 1).astype(np.float64)
    return W @ X.reshape(-1, k).T  # [m, n]


@pytest.mark.parametrize("dtype", [2, 8])
@pytest.mark.parametrize("m,k", [(4, 32), (8, 64), (5, 96), (64, 256), (33, 2048)])
def test_gemv_vs_f64_dequant(oracle, dtype, m, k):
    a = oracle.synth_weight(dtype, m, k, seed=m * 1000 + k, sigma=0.02)
    s, q = oracle.quantize_q8_0(oracle.fill_normal(k, 1.0, k))
    y = oracle.gemv_q8(dtype, a, s, q, m, k)
    y64 = oracle.gemv_q8(dtype, a, s, q, m, k, f64=True)
    ref = dequant_f64(oracle, dtype, a, s, q, m, k)[:, 0]
    assert rel_l2(y64, ref) < 1e-12  # exact integer dots x exact scales
    assert rel_l2(y, ref) < 1e-6  # f32 accumulation in the reference's order


@pytest.mark.parametrize("dtype,n", [(2, 7), (8, 5), (2, 8), (2, 11), (2, 16)])
def test_gemm_equals_sequential_gemv_reference_shapes(oracle, dtype, n):
    m, k = 8, 64
    a = oracle.build_matrix(dtype, ref_weights(m, k), m, k)
    s, q = oracle.quantize_q8_0_batch(ref_inputs(n, k), n, k)
    c = oracle.gemm_q8(dtype, a, s, q, m, n, k)
    for j in range(n):
        y = oracle.gemv_q8(dtype, a, s[j], q[j], m, k)
        assert np.abs(c[:, j] - y).max() < 1e-4  # the reference's bound; ours is bit-equal
        assert np.array_equal(c[:, j], y)
    assert rel_l2(c, dequant_f64(oracle, dtype, a, s, q, m, k)) < 1e-6


def test_gemm_single_column_reference_shape(oracle):  # simd.rs:1596-1623
    m, k = 4, 32
    w = ((np.arange(m * k) % 11).astype(np.float32) * np.float32(0.3) - np.float32(1.5)).astype(np.float32)
    x = ((np.arange(k) % 7).astype(np.float32) * np.float32(0.5) - np.float32(1.75)).astype(np.float32)
    a = oracle.build_matrix(2, w, m, k)
    s, q = oracle.quantize_q8_0_batch(x, 1, k)
    c = oracle.gemm_q8(2, a, s, q, m, 1, k)
    assert np.array_equal(c[:, 0], oracle.gemv_q8(2, a, s[0], q[0], m, k))


def test_q8_0_gemm_closed_form(oracle):
    """m=64, k=32, n=4, scale 1/(row+1), quants -16..15, x == 1 -> -16/(row+1)."""
    m, k, n = 64, 32, 4
    rows = []
    for r in range(m):
        h = int(np.float16(1.0 / (r + 1.0)).view(np.uint16))
        rows.append(np.concatenate([np.array([h & 0xFF, h >> 8], np.uint8), (np.arange(32) - 16).astype(np.int8).view(np.uint8)]))
    a = np.concatenate(rows)
    s, q = oracle.quantize_q8_0_batch(np.ones(n * k, np.float32), n, k)
    c = oracle.gemm_q8(8, a, s, q, m, n, k)
    # x == 1 quantizes to q = 127, scale = f16(1/127): the activation is reproduced to f16 precision
    expect = np.array([-16.0 * float(np.float16(1.0 / (r + 1.0))) for r in range(m)])
    for j in range(n):
        assert np.abs(c[:, j] - expect).max() < 1.0  # the reference's own (loose) bound
        assert np.allclose(c[:, j], expect * 127.0 * float(np.float16(1.0 / 127.0)), rtol=1e-6)


def test_against_gpu_test_references(oracle):
    """x = sin(0.013 i), weights from the multiplicative hash of the reference's GPU
    parity tests, compared with their dequantize-and-multiply CPU reference."""
    m, k = 64, 256
    i = np.arange(m * k, dtype=np.uint64)
    w = ((((i * np.uint64(2654435761)) & np.uint64(0xFFFFFFFF)) >> np.uint64(16)).astype(np.float32) / np.float32(32768.0) - np.float32(1.0)) * np.float32(0.5)
    x = np.sin(0.013 * np.arange(k)).astype(np.float32)
    a = oracle.build_matrix(2, w, m, k)
    W = oracle.dequant_matrix(2, a, m, k)
    expect = np.zeros(m, np.float32)
    for b in range(k // 32):  # f32 accumulation like q4_0_gemv_cpu
        expect += (W[:, b * 32:(b + 1) * 32] * x[b * 32:(b + 1) * 32]).sum(axis=1, dtype=np.float32)
    s, q = oracle.quantize_q8_0(x)
    y = oracle.gemv_q8(2, a, s, q, m, k)
    # (1) the same dequantize-and-multiply reference fed the DEQUANTIZED activations
    #     must agree at the GPU tests' tolerance (the integer path is that product, regrouped)
    xhat = (q.reshape(-1, 32).astype(np.float32) * s[:, None]).reshape(-1)
    expect_hat = np.zeros(m, np.float32)
    for b in range(k // 32):
        expect_hat += (W[:, b * 32:(b + 1) * 32] * xhat[b * 32:(b + 1) * 32]).sum(axis=1, dtype=np.float32)
    max_abs = np.abs(y - expect_hat).max()
    max_rel = (np.abs(y - expect_hat) / np.maximum(np.abs(expect_hat), 1e-6)).max()
    assert max_abs < 1e-2 or max_rel < 1e-3
    assert max_abs < 1e-4
    # (2) against the f32-activation reference the only extra term is the Q8_0 rounding of x,
    #     bounded per row by sum_b (sum_i |w_i|) * d_b / 2 (+ the f16 rounding of d_b)
    d = np.abs(x.reshape(-1, 32)).max(axis=1) / 127.0
    bound = (np.abs(W).reshape(m, -1, 32).sum(axis=2) * (d * (0.5 + 127 * 2.0**-11))[None, :]).sum(axis=1)
    assert np.all(np.abs(y - expect) <= bound + 1e-5)


def test_weight_quantizers_vs_numpy(oracle):
    """Input generators: Q4_0 d = amax/7, q = min(15, trunc(x*id + 8.5)); Q8_0
    d = amax/127, q = round-half-away (simd.rs:1371-1419)."""
    rng = np.random.default_rng(2)
    m, k = 16, 128
    v = (rng.standard_normal(m * k) * 0.02).astype(np.float32)
    vb = v.reshape(-1, 32)
    amax = np.abs(vb).max(axis=1)
    # Q4_0
    d = (amax / np.float32(7)).astype(np.float32)
    idv = (np.float32(1) / d).astype(np.float32)
    t = ((vb * idv[:, None]).astype(np.float32) + np.float32(8.5)).astype(np.float32)
    qn = np.minimum(np.clip(np.trunc(t), 0, 255), 15).astype(np.uint8)
    a = oracle.build_matrix(2, v, m, k).reshape(-1, 18)
    assert np.array_equal(a[:, :2].copy().view(np.uint16)[:, 0], d.astype(np.float16).view(np.uint16))
    assert np.array_equal(a[:, 2:] & 0xF, qn[:, :16]) and np.array_equal(a[:, 2:] >> 4, qn[:, 16:])
    # Q8_0
    d = (amax / np.float32(127)).astype(np.float32)
    idv = (np.float32(1) / d).astype(np.float32)
    t = (vb * idv[:, None]).astype(np.float32)
    qn = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -128, 127).astype(np.int8)
    a = oracle.build_matrix(8, v, m, k).reshape(-1, 34)
    assert np.array_equal(a[:, :2].copy().view(np.uint16)[:, 0], d.astype(np.float16).view(np.uint16))
    assert np.array_equal(a[:, 2:].view(np.int8), qn)


def test_x86_baseline_matches_f64(oracle):
    """The timing baseline (f32 path, no activation quantization) is a different
    function from the oracle; it only has to be a correct dequantize-and-dot."""
    for dtype in (2, 8):
        m, k = 700, 512
        a = oracle.synth_weight(dtype, m, k, seed=4)
        x = oracle.fill_normal(8, 1.0, k)
        y, used = oracle.x86_gemv_f32(dtype, a, x, m, k, threads=4)
        ref = oracle.dequant_matrix(dtype, a, m, k).astype(np.float64) @ x.astype(np.float64)
        assert rel_l2(y, ref) < 1e-5
        assert used == (1 if dtype == 2 else 2)  # Q4_0 serial; Q8_0 chunk = max(700/4, 512) -> 2 chunks
