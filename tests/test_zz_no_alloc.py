"""The entry point that allocates nothing (wick_rocm_matmul_f32_noalloc) against the entry point it is a variant of
(wick_rocm_matmul_f32): same kernels, so the same bits, on two calls in a row through the C ABI, the second one smaller
than the first (the static scratch then still holds the tail of the first call's activations)."""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity

pytestmark = pytest.mark.gpu


def _both(ctx, oracle, dtype, m, k, n, x_stride, y_stride, seed, accumulate=False):
    wb = oracle.synth_weight(dtype, m, k, seed=seed)
    w = ctx.upload_weight(wb, dtype, m, k)
    x = oracle.fill_normal(seed + 1, 1.0, n * x_stride)
    y0 = oracle.fill_normal(seed + 2, 1.0, n * y_stride)
    d_x = ctx.to_device(x)
    d_a, d_b = ctx.to_device(y0), ctx.to_device(y0)
    # the K split of launches with few tiles keeps its partial sums in context scratch, so the no-alloc entry point never takes
    # it: same kernels = same bits with the split switched off, the f32 bar (checked below) with it on
    ctx.set_gemm_max_k_splits(1)
    ctx.encode_gemm(w, d_x, 0, d_a, 0, n, x_stride, y_stride, accumulate=accumulate)
    ctx.set_gemm_max_k_splits(0)
    ctx.encode_gemm_noalloc(w, d_x, 0, d_b, 0, n, x_stride, y_stride, accumulate=accumulate)
    a, b = d_a.download(np.float32, y0.size), d_b.download(np.float32, y0.size)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"no-alloc result differs ({dtype}, {m}x{n}x{k})"
    assert not np.array_equal(a, y0)
    # and both are the oracle's result
    s, q = oracle.quantize_q8_0_batch(x, n, k, x_stride)
    if dtype == W.Q6_K:  # no batched Q6_K kernel in the reference either: one GEMV per token
        ref = np.stack([oracle.gemv_q6k_q8(wb, s[j], q[j], m, k) for j in range(n)], axis=1).astype(np.float64)
    else:
        ref = oracle.gemm_q8(dtype, wb, s, q, m, n, k, f64=True)
    ref = ref + (y0.reshape(n, y_stride)[:, :m].T if accumulate else 0.0)
    assert_f32_parity(b.reshape(n, y_stride)[:, :m].T, ref, "no-alloc matmul")
    w.free()
    for buf in (d_x, d_a, d_b):
        buf.free()


def test_no_alloc_matches_matmul_f32_twice_in_a_row(ctx, oracle):
    # first call: 600 tokens x 2048 on the int8-MFMA kernel; second call: smaller (40 x 1024), then single tokens
    _both(ctx, oracle, W.Q4_0, 768, 2048, 600, 2048 + 64, 768 + 8, seed=1)
    _both(ctx, oracle, W.Q4_0, 300, 1024, 40, 1024, 300, seed=2)
    _both(ctx, oracle, W.Q8_0, 512, 1024, 3, 1024 + 32, 512, seed=3, accumulate=True)  # multi-token GEMV
    _both(ctx, oracle, W.Q8_0, 512, 2048, 1, 2048, 512, seed=4)                        # decode GEMV
    _both(ctx, oracle, W.Q6_K, 96, 512, 2, 512, 96, seed=5)                            # Q6_K: one GEMV per token


def test_no_alloc_against_a_split_launch_at_default_settings(ctx, oracle):
    """With the library's default K split the two entry points take different launches on a shape that splits (few tokens over a
    long K): not the same low-order bits, both inside the f32 bar against the oracle and against each other."""
    m, k, n = 2048, 6912, 20
    wb = oracle.synth_weight(W.Q8_0, m, k, seed=31)
    w = ctx.upload_weight(wb, W.Q8_0, m, k)
    x = oracle.fill_normal(32, 1.0, n * k)
    d_x, d_a, d_b = ctx.to_device(x), ctx.alloc(n * m * 4), ctx.alloc(n * m * 4)
    ctx.set_gemm_max_k_splits(0)  # the default
    ctx.encode_gemm(w, d_x, 0, d_a, 0, n, k, m)
    ctx.encode_gemm_noalloc(w, d_x, 0, d_b, 0, n, k, m)
    a, b = d_a.download(np.float32, n * m).reshape(n, m).T, d_b.download(np.float32, n * m).reshape(n, m).T
    s, q = oracle.quantize_q8_0_batch(x, n, k)
    ref = oracle.gemm_q8(W.Q8_0, wb, s, q, m, n, k, f64=True)
    assert_f32_parity(a, ref, "matmul_f32 (split launch)")
    assert_f32_parity(b, ref, "no-alloc matmul (unsplit launch)")
    assert_f32_parity(b, a, "no-alloc vs split")
    w.free(), d_x.free(), d_a.free(), d_b.free()


def test_no_alloc_refuses_a_second_context_until_the_first_has_synchronised(ctx, oracle):
    """One static array per GPU, shared by every context: the overlap the host can see is refused instead of raced."""
    m, k, n = 64, 256, 4
    wb = oracle.synth_weight(W.Q4_0, m, k, seed=41)
    x = oracle.fill_normal(42, 1.0, n * k)
    s, q = oracle.quantize_q8_0_batch(x, n, k)
    ref = oracle.gemm_q8(W.Q4_0, wb, s, q, m, n, k)
    other = W.RocmContext(0)
    try:
        wa, wo = ctx.upload_weight(wb, W.Q4_0, m, k), other.upload_weight(wb, W.Q4_0, m, k)
        xa, ya, xo, yo = ctx.to_device(x), ctx.alloc(n * m * 4), other.to_device(x), other.alloc(n * m * 4)
        ctx.sync()
        ctx.encode_gemm_noalloc(wa, xa, 0, ya, 0, n, k, m)  # enqueued, not synchronised: the array is ctx's
        with pytest.raises(W.RocmError, match="another context") as e:
            other.encode_gemm_noalloc(wo, xo, 0, yo, 0, n, k, m)
        assert e.value.status == -6
        ctx.sync()
        other.encode_gemm_noalloc(wo, xo, 0, yo, 0, n, k, m)  # free again
        with pytest.raises(W.RocmError, match="another context"):
            ctx.encode_gemm_noalloc(wa, xa, 0, ya, 0, n, k, m)
        assert_f32_parity(yo.download(np.float32, n * m).reshape(n, m).T, ref, "second context")  # the download synchronises
        ctx.encode_gemm_noalloc(wa, xa, 0, ya, 0, n, k, m)
        assert_f32_parity(ya.download(np.float32, n * m).reshape(n, m).T, ref, "first context again")
        wa.free(), xa.free(), ya.free(), wo.free(), xo.free(), yo.free()
    finally:
        other.close()


def test_no_alloc_inside_a_graph_capture(ctx, oracle):
    """What it is for: a capture in which nothing may allocate.  No wick_rocm_reserve_scratch beforehand."""
    m, k, n = 256, 2080, 20  # 2080: a shape wick_rocm_matmul_f32 would need context scratch for
    wb = oracle.synth_weight(W.Q4_0, m, k, seed=11)
    w = ctx.upload_weight(wb, W.Q4_0, m, k)
    x = oracle.fill_normal(12, 1.0, n * k)
    d_x, d_y = ctx.to_device(x), ctx.alloc(n * m * 4)
    ctx.graph_begin()
    ctx.encode_gemm_noalloc(w, d_x, 0, d_y, 0, n, k, m)
    g = ctx.graph_end()
    s, q = oracle.quantize_q8_0_batch(x, n, k)
    ref = oracle.gemm_q8(W.Q4_0, wb, s, q, m, n, k)
    for rep in range(3):
        d_y.upload(np.zeros(n * m, np.float32))
        ctx.graph_launch(g)
        assert_f32_parity(d_y.download(np.float32, n * m).reshape(n, m).T, ref, f"replay {rep}")
        ctx.encode_gemm_noalloc(w, d_x, 0, d_y, 0, 5, k, m)  # eager work on the same scratch between replays
        ctx.sync()
    ctx.graph_destroy(g)
    w.free(), d_x.free(), d_y.free()


def test_no_alloc_rejects_what_does_not_fit(ctx, oracle):
    m, k = 32, 8192
    w = ctx.upload_weight(oracle.synth_weight(W.Q8_0, m, k, seed=21), W.Q8_0, m, k)
    n = 513  # 513 * 8192 > 4194304
    d_x, d_y = ctx.alloc(n * k * 4), ctx.alloc(n * m * 4)
    with pytest.raises(W.RocmError, match="exceeds the static scratch") as e:
        ctx.encode_gemm_noalloc(w, d_x, 0, d_y, 0, n, k, m)
    assert e.value.status == -3
    ctx.encode_gemm_noalloc(w, d_x, 0, d_y, 0, 512, k, m)  # exactly at the limit
    ctx.sync()
    ctx.kernel_timing_begin()
    try:
        with pytest.raises(W.RocmError, match="kernel timing") as e:
            ctx.encode_gemm_noalloc(w, d_x, 0, d_y, 0, 4, k, m)
        assert e.value.status == -6
    finally:
        ctx.kernel_timing_end()
    w.free(), d_x.free(), d_y.free()
