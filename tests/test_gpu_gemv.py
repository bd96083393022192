"""Decode GEMV on the GPU against the oracle: per-block i32 dots BIT-EXACT, f32
outputs within rel-L2 1e-5 / max-abs 1e-4 x RMS."""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity
from gpu_util import Problem

pytestmark = pytest.mark.gpu

# (m, k): every lanes-per-row tier of the pair kernel, two-chunk rows (k=4608, 6912), odd block
# counts and k > 8192 (generic kernel), m below / above one wave pass, the LFM2 shapes.
SHAPES = [(1, 32), (5, 32), (7, 96), (8, 64), (3, 128), (64, 256), (100, 512), (300, 1024), (513, 2048), (6912, 2048),
          (64, 4096), (1024, 4608), (2048, 6912), (40, 8192), (16, 16384), (33, 2080), (1024, 1024), (3072, 1024),
          (512, 1024), (4608, 1024)]


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("m,k", SHAPES)
def test_gemv_parity(ctx, oracle, dtype, m, k):
    with Problem(ctx, oracle, dtype, m, k, seed=m + 3 * k + dtype) as p:
        d_y = p.alloc(m * 4)
        ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_y)
        y = d_y.download(np.float32, m)
        assert_f32_parity(y, oracle.gemv_q8(dtype, p.wb, p.s[0], p.q[0], m, k), f"gemv {dtype} {m}x{k}")
        d_d = p.alloc(m * (k // 32) * 4)
        ctx.block_dots_i32(p.w, p.d_q, 1, d_d)
        dots = d_d.download(np.int32, m * (k // 32)).reshape(1, m, k // 32)
        assert np.array_equal(dots, oracle.block_dots_i32(dtype, p.wb, p.q, m, 1, k))


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_extreme_blocks(ctx, oracle, dtype):
    """Random BYTES as weights (every nibble / int8 value, arbitrary f16 scales made
    finite) and saturated activations: the integer path must stay exact."""
    rng = np.random.default_rng(99 + dtype)
    m, k = 96, 512
    bb = 18 if dtype == W.Q4_0 else 34
    wb = rng.integers(0, 256, m * (k // 32) * bb).astype(np.uint8).reshape(-1, bb)
    wb[:, 1] &= 0x3B  # clear the top exponent bits: scales finite and modest
    wb = wb.reshape(-1)
    with Problem(ctx, oracle, dtype, m, k, seed=3, weight_bytes=wb) as p:
        q = rng.choice(np.array([-127, 127, -1, 0, 1, 126], np.int8), size=k).astype(np.int8)
        d_q = p.to_device(q)
        d_y, d_d = p.alloc(m * 4), p.alloc(m * (k // 32) * 4)
        ctx.gemv_with_preq(p.w, p.d_s, d_q, d_y)
        ctx.block_dots_i32(p.w, d_q, 1, d_d)
        assert np.array_equal(d_d.download(np.int32, m * (k // 32)).reshape(1, m, -1), oracle.block_dots_i32(dtype, wb, q, m, 1, k))
        assert_f32_parity(d_y.download(np.float32, m), oracle.gemv_q8(dtype, wb, p.s[0], q, m, k), "extreme blocks")


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_accumulate(ctx, oracle, dtype):
    """y += W x, the residual form of encode_gemv_weight_accumulate."""
    m, k = 1024, 2048
    with Problem(ctx, oracle, dtype, m, k, seed=21) as p:
        y0 = oracle.fill_normal(77, 1.0, m)
        d_y = p.to_device(y0)
        ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_y, accumulate=True)
        ref = y0.astype(np.float64) + oracle.gemv_q8(dtype, p.wb, p.s[0], p.q[0], m, k, f64=True)
        assert_f32_parity(d_y.download(np.float32, m), ref, "accumulate")


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("ms,k", [((1024, 512, 512), 1024), ((4608, 4608), 1024), ((2048, 512, 512, 7), 2048), ((5, 3), 96)])
def test_multi_weight_one_activation(ctx, oracle, dtype, ms, k):
    """{Q,K,V} / {gate,up}: several weights against one quantized activation in one launch."""
    s, q = oracle.quantize_q8_0(oracle.fill_normal(5, 1.0, k))
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    wbs = [oracle.synth_weight(dtype, m, k, seed=100 + i) for i, m in enumerate(ms)]
    ws = [ctx.upload_weight(wb, dtype, m, k) for wb, m in zip(wbs, ms)]
    ys = [ctx.alloc(m * 4) for m in ms]
    ctx.gemv_with_preq_multi(ws, d_s, d_q, ys)
    for wb, m, y in zip(wbs, ms, ys):
        assert_f32_parity(y.download(np.float32, m), oracle.gemv_q8(dtype, wb, s, q, m, k), f"multi m={m}")
    for b in [d_q, d_s] + ys:
        b.free()
    for w in ws:
        w.free()


def test_argument_errors(ctx, oracle):
    with Problem(ctx, oracle, W.Q4_0, 8, 64) as p:
        d_y = p.alloc(32)
        with pytest.raises(W.RocmError) as e:
            ctx.gemv_with_preq(p.w, p.d_s, p.d_q, None)
        assert e.value.status == -1
        w2 = ctx.upload_weight(oracle.synth_weight(W.Q4_0, 8, 128, 1), W.Q4_0, 8, 128)
        with pytest.raises(W.RocmError) as e:  # weights of one batch must share k
            ctx.gemv_with_preq_multi([p.w, w2], p.d_s, p.d_q, [d_y, d_y])
        assert e.value.status == -3
        w2.free()
    blocks = np.zeros(18 * 2, np.uint8)
    with pytest.raises(W.RocmError) as e:
        ctx.upload_weight(blocks, 12, 1, 64)  # Q4_K: not on this path
    assert e.value.status == -2
    with pytest.raises(W.RocmError) as e:
        ctx.upload_weight(blocks, W.Q4_0, 1, 48)  # k % 32 != 0
    assert e.value.status == -3
    with pytest.raises(W.RocmError) as e:
        ctx.upload_weight(blocks, W.Q4_0, 3, 64)  # byte count mismatch
    assert e.value.status == -3


# Both ways of fetching the weights on: every lanes-per-row tier, k/64 not a power of two
# (spans shorter than 64 pairs), two-chunk rows, m below one pass and not a multiple of the
# rows per pass (the last span hangs over the matrix end), many passes per wave.
STREAM_SHAPES = [(1, 64), (9, 128), (33, 192), (100, 256), (1, 512), (3, 512), (1000, 512), (2, 1024), (4, 1024), (37, 1024),
                 (4099, 1024), (77, 1536), (1, 2048), (2, 2048), (515, 2048), (9001, 2048), (1, 4096), (7, 4096), (3001, 4096),
                 (130, 4608), (1025, 4608), (65, 6912), (19, 8192), (70001, 1024)]


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("m,k", STREAM_SHAPES)
def test_gemv_streaming_variant(ctx, oracle, dtype, m, k):
    """Both ways of fetching the weights (per-lane loads, whole-line span loads through LDS)
    give the reference's result, pre-quantized and fused-quantizer entry points alike; the
    fused and the pre-quantized launch of one policy agree bit for bit, and the parity hook of each
    (the same kernel with the scaling replaced by a store) writes the oracle's i32 block dots."""
    with Problem(ctx, oracle, dtype, m, k, seed=5 * m + k + dtype) as p:
        ref = oracle.gemv_q8(dtype, p.wb, p.s[0], p.q[0], m, k)
        d_x = p.to_device(p.x)
        d_y, d_yf, d_d = p.alloc(m * 4), p.alloc(m * 4), p.alloc(m * (k // 32) * 4)
        want_dots = oracle.block_dots_i32(dtype, p.wb, p.q, m, 1, k)
        try:
            for direct_max in (1 << 62, 0):
                ctx.set_gemv_policy(direct_max)
                d_y.upload(np.full(m, np.nan, np.float32))
                d_yf.upload(np.full(m, np.nan, np.float32))
                ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_y)
                ctx.encode_gemv_fused([p.w], d_x, 0, [d_yf])
                y, yf = d_y.download(np.float32, m), d_yf.download(np.float32, m)
                assert_f32_parity(y, ref, f"gemv direct_max={direct_max} {dtype} {m}x{k}")
                assert np.array_equal(y, yf), "fused quantizer differs from pre-quantized launch"
                # the raw i32 block dots of THESE kernels (same fetch mode, pre-quantized and fused quantizer), bit for bit
                for fused in (False, True):
                    if fused and (k // 32) % 2:
                        continue  # odd block counts never take the fused kernel
                    d_d.upload(np.full(m * (k // 32), -1, np.int32))
                    if fused:
                        ctx.block_dots_f32_i32(p.w, d_x, d_d)
                    else:
                        ctx.block_dots_i32(p.w, p.d_q, 1, d_d)
                    assert np.array_equal(d_d.download(np.int32, m * (k // 32)).reshape(1, m, -1), want_dots), f"block dots, fused={fused}, direct_max={direct_max}"
        finally:
            ctx.set_gemv_policy(-1)


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_gemv_streaming_accumulate(ctx, oracle, dtype):
    m, k = 2051, 1024
    with Problem(ctx, oracle, dtype, m, k, seed=31) as p:
        y0 = oracle.fill_normal(78, 1.0, m)
        d_y = p.to_device(y0)
        try:
            ctx.set_gemv_policy(0)
            ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_y, accumulate=True)
        finally:
            ctx.set_gemv_policy(-1)
        ref = y0 + oracle.gemv_q8(dtype, p.wb, p.s[0], p.q[0], m, k)
        assert_f32_parity(d_y.download(np.float32, m), ref, "streaming gemv accumulate")


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_block_dots_through_the_product_kernel_at_full_size(ctx, oracle, dtype):
    """6912 x 2048 (the LFM2-1.2B ffn_up decode shape): the i32 block dots written by the GEMV kernel itself, in the
    fetch mode the library picks for this size and in the other one, pre-quantized and with the in-kernel quantizer."""
    m, k = 6912, 2048
    with Problem(ctx, oracle, dtype, m, k, seed=1234) as p:
        want = oracle.block_dots_i32(dtype, p.wb, p.q, m, 1, k)
        d_x, d_d = p.to_device(p.x), p.alloc(m * (k // 32) * 4)
        try:
            for policy in (-1, 1 << 62, 0):
                ctx.set_gemv_policy(policy)
                for fused in (False, True):
                    d_d.upload(np.full(m * (k // 32), -1, np.int32))
                    ctx.block_dots_f32_i32(p.w, d_x, d_d) if fused else ctx.block_dots_i32(p.w, p.d_q, 1, d_d)
                    assert np.array_equal(d_d.download(np.int32, m * (k // 32)).reshape(1, m, -1), want), (policy, fused)
        finally:
            ctx.set_gemv_policy(-1)
    with Problem(ctx, oracle, W.Q6_K, 8, 256) as p6:
        with pytest.raises(W.RocmError) as e:
            ctx.block_dots_f32_i32(p6.w, p6.d_q, p6.d_q)
        assert e.value.status == -2
