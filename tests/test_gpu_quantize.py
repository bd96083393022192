"""Q8_0 activation quantizer on the GPU: BIT-EXACT against the oracle and the
golden fixture (int8 quants and the f32 bits of the f16-rounded scales)."""
import os

import numpy as np
import pytest

from conftest import GOLDEN

pytestmark = pytest.mark.gpu


def run_quantizer(ctx, x, n, k, stride):
    d_x = ctx.to_device(x)
    d_q = ctx.alloc(max(n * k, 4))
    d_s = ctx.alloc(max(n * (k // 32) * 4, 4))
    ctx.quantize_q8_0(d_x, n, k, stride, d_q, d_s)
    q = d_q.download(np.int8, n * k).reshape(n, k)
    s = d_s.download(np.float32, n * (k // 32)).reshape(n, k // 32)
    for b in (d_x, d_q, d_s):
        b.free()
    return s, q


@pytest.mark.parametrize("name", ["normal", "wide", "edge"])
def test_golden_fixture(ctx, name):
    v = np.load(os.path.join(GOLDEN, "q8_0_quantizer_vectors.npz"))
    x = v[f"{name}_x"]
    s, q = run_quantizer(ctx, x, 1, x.size, x.size)
    assert np.array_equal(q[0], v[f"{name}_quants"])
    assert np.array_equal(s[0].view(np.uint32), v[f"{name}_scales"].view(np.uint32))


@pytest.mark.parametrize("n,k,stride", [(1, 32, 32), (1, 2048, 2048), (3, 64, 64), (7, 1024, 1024), (5, 96, 100), (4, 4608, 4609),
                                        (33, 6912, 6912), (2002, 2048, 2048)])
def test_matches_oracle(ctx, oracle, n, k, stride):
    x = oracle.fill_normal(n * 31 + k, 1.0, (n - 1) * stride + k)
    s, q = run_quantizer(ctx, x, n, k, stride)
    s_ref, q_ref = oracle.quantize_q8_0_batch(x, n, k, stride)
    assert np.array_equal(q, q_ref)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))


def test_wide_dynamic_range(ctx, oracle):
    rng = np.random.default_rng(17)
    n, k = 64, 512
    x = (rng.standard_normal(n * k) * np.exp(rng.uniform(-20, 20, n * k))).astype(np.float32)
    s, q = run_quantizer(ctx, x, n, k, k)
    s_ref, q_ref = oracle.quantize_q8_0_batch(x, n, k)
    assert np.array_equal(q, q_ref)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))


def test_unaligned_source_offset(ctx, oracle):
    """A source that is only 4-byte aligned takes the scalar-load variant."""
    n, k = 3, 256
    x = oracle.fill_normal(5, 1.0, n * k + 1)
    d_x = ctx.to_device(x)
    d_q, d_s = ctx.alloc(n * k), ctx.alloc(n * (k // 32) * 4)
    ctx.quantize_q8_0(d_x.ptr + 4, n, k, k, d_q, d_s)
    q = d_q.download(np.int8, n * k).reshape(n, k)
    s = d_s.download(np.float32, n * (k // 32)).reshape(n, -1)
    s_ref, q_ref = oracle.quantize_q8_0_batch(x[1:], n, k)
    assert np.array_equal(q, q_ref) and np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))


def test_empty_and_bad_arguments(ctx):
    import wick_amd as W

    d = ctx.alloc(1024)
    ctx.quantize_q8_0(d, 0, 64, 64, d, d)  # n = 0 is a no-op
    with pytest.raises(W.RocmError) as e:
        ctx.quantize_q8_0(d, 1, 48, 48, d, d)  # k % 32 != 0
    assert e.value.status == -3
    with pytest.raises(W.RocmError) as e:
        ctx.quantize_q8_0(d, 2, 64, 32, d, d)  # stride < k
    assert e.value.status == -1
    with pytest.raises(W.RocmError) as e:
        ctx.quantize_q8_0(None, 1, 64, 64, d, d)
    assert e.value.status == -1
    d.free()
