"""The reference's GPU call-site shape (f32 in, f32 out, byte offsets, strides):
encode_gemv_impl / encode_gemm of wick/src/model/metal_lfm2.rs:881-992, 1231-1335,
checked end to end (device quantizer + GEMV/GEMM) against the oracle; plus one
submission per token through graph capture."""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_encode_gemv_with_offsets(ctx, oracle, dtype):
    m, k = 1024, 2048
    wb = oracle.synth_weight(dtype, m, k, seed=31)
    w = ctx.upload_weight(wb, dtype, m, k)
    x = oracle.fill_normal(6, 1.0, k + 16)
    d_x = ctx.to_device(x)
    d_y = ctx.to_device(np.zeros(m + 8, np.float32))
    ctx.encode_gemv(w, d_x, 16 * 4, d_y, 8 * 4)
    s, q = oracle.quantize_q8_0(x[16:])
    got = d_y.download(np.float32, m + 8)
    assert np.all(got[:8] == 0)
    assert_f32_parity(got[8:], oracle.gemv_q8(dtype, wb, s, q, m, k), "encode_gemv")
    ctx.encode_gemv(w, d_x, 16 * 4, d_y, 8 * 4, accumulate=True)
    assert_f32_parity(d_y.download(np.float32, m + 8)[8:], 2.0 * oracle.gemv_q8(dtype, wb, s, q, m, k, f64=True), "encode_gemv accumulate")
    w.free(), d_x.free(), d_y.free()


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("n", [1, 3, 15, 16, 100])
def test_encode_gemm_strided(ctx, oracle, dtype, n):
    """X[col*x_stride + i], Y[col*y_stride + row] with strides larger than k and m,
    like the prefill buffers (x_stride = hs | is, y_stride = 3hs | hs | kv_dim | is)."""
    m, k, xs, ys = 512, 1024, 1024 + 32, 3 * 512
    wb = oracle.synth_weight(dtype, m, k, seed=41)
    w = ctx.upload_weight(wb, dtype, m, k)
    x = oracle.fill_normal(n, 1.0, n * xs)
    d_x = ctx.to_device(x)
    d_y = ctx.to_device(np.full(n * ys, 3.0, np.float32))
    ctx.encode_gemm(w, d_x, 0, d_y, 0, n, xs, ys)
    s, q = oracle.quantize_q8_0_batch(x, n, k, xs)
    got = d_y.download(np.float32, n * ys).reshape(n, ys)
    assert np.all(got[:, m:] == 3.0)
    assert_f32_parity(got[:, :m].T, oracle.gemm_q8(dtype, wb, s, q, m, n, k), f"encode_gemm n={n}")
    w.free(), d_x.free(), d_y.free()


def test_graph_replay_matches_eager(ctx, oracle):
    """One submission per token: capture quantize + {gate, up} + down, replay it
    several times with eager work and synchronisation in between, and check every
    replay against the eager result (inputs change between replays)."""
    hs, is_ = 1024, 4608
    wg = oracle.synth_weight(W.Q4_0, is_, hs, 1)
    wu = oracle.synth_weight(W.Q4_0, is_, hs, 2)
    wd = oracle.synth_weight(W.Q4_0, hs, is_, 3)
    g, u, d = (ctx.upload_weight(b, W.Q4_0, m, k) for b, m, k in ((wg, is_, hs), (wu, is_, hs), (wd, hs, is_)))
    d_x = ctx.alloc(hs * 4)
    d_q, d_s = ctx.alloc(is_), ctx.alloc(is_ // 32 * 4)
    d_g, d_u, d_o = ctx.alloc(is_ * 4), ctx.alloc(is_ * 4), ctx.alloc(hs * 4)

    def step():
        ctx.quantize_q8_0(d_x, 1, hs, hs, d_q, d_s)
        ctx.gemv_with_preq_multi([g, u], d_s, d_q, [d_g, d_u])
        ctx.quantize_q8_0(d_g, 1, is_, is_, d_q, d_s)
        ctx.gemv_with_preq(d, d_s, d_q, d_o)

    ctx.graph_begin()
    step()
    graph = ctx.graph_end()
    for it in range(4):
        x = oracle.fill_normal(50 + it, 1.0, hs)
        d_x.upload(x)
        step()
        eager = d_o.download(np.float32, hs)
        d_o.upload(np.zeros(hs, np.float32))
        ctx.graph_launch(graph)
        replay = d_o.download(np.float32, hs)
        assert np.array_equal(eager, replay), f"replay {it} differs from eager"
        s0, q0 = oracle.quantize_q8_0(x)
        gate = oracle.gemv_q8(W.Q4_0, wg, s0, q0, is_, hs)
        s1, q1 = oracle.quantize_q8_0(d_g.download(np.float32, is_))
        assert_f32_parity(d_g.download(np.float32, is_), gate, "gate")
        assert_f32_parity(replay, oracle.gemv_q8(W.Q4_0, wd, s1, q1, hs, is_), "down")
    ctx.graph_destroy(graph)
    with pytest.raises(W.RocmError) as e:
        ctx.graph_end()
    assert e.value.status == -6
    for w in (g, u, d):
        w.free()
    for b in (d_x, d_q, d_s, d_g, d_u, d_o):
        b.free()
