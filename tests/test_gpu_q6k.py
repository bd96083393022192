"""Q6_K decode GEMV on the GPU against the oracle (wick/src/backend/simd.rs:547-640):
the i32 dot of every 16-weight group BIT-EXACT, f32 outputs within rel-L2 1e-5 /
max-abs 1e-4 x RMS."""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity
from gpu_util import Problem, fetch_gemm
from oracle import lfm2_oracle as L
from wick_amd.lfm2 import Lfm2Ops

pytestmark = pytest.mark.gpu

# (m, k): every lanes-per-row tier (k/128 half blocks per row, padded to a power of two),
# m below / above one wave pass and ragged against rows-per-wave, the LFM2 LM head width.
SHAPES = [(1, 256), (3, 256), (33, 256), (7, 512), (130, 512), (65, 768), (257, 1024), (4099, 1024), (19, 1536), (300, 2048),
          (1025, 2048), (31, 2560), (64, 4096), (9, 6144), (17, 8192), (65536, 1024)]


@pytest.mark.parametrize("m,k", SHAPES)
def test_q6k_gemv_parity(ctx, oracle, m, k):
    with Problem(ctx, oracle, W.Q6_K, m, k, seed=m + 3 * k) as p:
        d_y = p.alloc(m * 4)
        ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_y)
        assert_f32_parity(d_y.download(np.float32, m), oracle.gemv_q6k_q8(p.wb, p.s[0], p.q[0], m, k), f"q6k gemv {m}x{k}")
        d_d = p.alloc(m * (k // 16) * 4)
        ctx.block_dots_i32(p.w, p.d_q, 1, d_d)
        dots = d_d.download(np.int32, m * (k // 16)).reshape(m, k // 16)
        assert np.array_equal(dots, oracle.q6k_group_dots_i32(p.wb, p.q[0], m, k))


def test_q6k_extreme_blocks(ctx, oracle):
    """Random BYTES as blocks (every 6-bit value, every int8 group scale, arbitrary finite
    f16 super-scales) against saturated activations: the integer path must stay exact."""
    rng = np.random.default_rng(1406)
    m, k = 96, 1024
    wb = rng.integers(0, 256, m * (k // 256) * 210).astype(np.uint8).reshape(-1, 210)
    wb[:, 209] &= 0x3B  # clear the top exponent bits of d: finite and modest
    wb = wb.reshape(-1)
    with Problem(ctx, oracle, W.Q6_K, m, k, seed=3, weight_bytes=wb) as p:
        q = rng.choice(np.array([-127, 127, -1, 0, 1, 126], np.int8), size=k).astype(np.int8)
        d_q = p.to_device(q)
        d_y, d_d = p.alloc(m * 4), p.alloc(m * (k // 16) * 4)
        ctx.gemv_with_preq(p.w, p.d_s, d_q, d_y)
        ctx.block_dots_i32(p.w, d_q, 1, d_d)
        assert np.array_equal(d_d.download(np.int32, m * (k // 16)).reshape(m, -1), oracle.q6k_group_dots_i32(wb, q, m, k))
        assert_f32_parity(d_y.download(np.float32, m), oracle.gemv_q6k_q8(wb, p.s[0], q, m, k), "q6k extreme blocks")


def test_q6k_accumulate_and_multi(ctx, oracle):
    """y += W x, and two weights behind one call."""
    m, k = 777, 1024
    with Problem(ctx, oracle, W.Q6_K, m, k, seed=21) as p:
        y0 = oracle.fill_normal(77, 1.0, m)
        d_y = p.to_device(y0)
        ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_y, accumulate=True)
        ref = oracle.gemv_q6k_q8(p.wb, p.s[0], p.q[0], m, k)
        assert_f32_parity(d_y.download(np.float32, m), y0 + ref, "q6k accumulate")
        wb2 = oracle.synth_weight(W.Q6_K, 50, k, 5)
        w2 = ctx.upload_weight(wb2, W.Q6_K, 50, k)
        d_a, d_b = p.alloc(m * 4), p.alloc(50 * 4)
        ctx.gemv_with_preq_multi([p.w, w2], p.d_s, p.d_q, [d_a, d_b])
        assert_f32_parity(d_a.download(np.float32, m), ref, "q6k multi[0]")
        assert_f32_parity(d_b.download(np.float32, 50), oracle.gemv_q6k_q8(wb2, p.s[0], p.q[0], 50, k), "q6k multi[1]")
        w2.free()


def test_q6k_f32_call_site(ctx, oracle):
    """The reference's call-site form (f32 in, f32 out; wick/src/backend/cpu.rs:423-470 quantizes x
    to Q8_0 first) equals quantize + pre-quantized GEMV bit for bit."""
    m, k = 1030, 2048
    with Problem(ctx, oracle, W.Q6_K, m, k, seed=8) as p:
        d_x = p.to_device(p.x)
        d_y, d_z = p.alloc(m * 4), p.alloc(m * 4)
        ctx.encode_gemv(p.w, d_x, 0, d_y, 0)
        ctx.gemv_with_preq(p.w, p.d_s, p.d_q, d_z)
        y, z = d_y.download(np.float32, m), d_z.download(np.float32, m)
        assert np.array_equal(y.view(np.uint32), z.view(np.uint32))
        ctx.encode_gemv_fused([p.w], d_x, 0, [d_y])
        assert np.array_equal(d_y.download(np.float32, m).view(np.uint32), z.view(np.uint32))


@pytest.mark.parametrize("layout", [W.LAYOUT_ROW_MAJOR, W.LAYOUT_TOKEN_MAJOR])
def test_q6k_batched(ctx, oracle, layout):
    """Batched calls on a Q6_K weight run the GEMV per token: every column equals the oracle's GEMV."""
    m, k, n = 203, 512, 5
    with Problem(ctx, oracle, W.Q6_K, m, k, n=n, seed=4) as p:
        stride = (n + 3) if layout == W.LAYOUT_ROW_MAJOR else (m + 5)
        d_y = p.alloc(max(m, n) * stride * 4)
        ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, stride, layout)
        y = fetch_gemm(d_y, m, n, stride, layout)
        for j in range(n):
            assert_f32_parity(y[:, j], oracle.gemv_q6k_q8(p.wb, p.s[j], p.q[j], m, k), f"q6k batched col {j}")


@pytest.mark.parametrize("m,k", [(1, 256), (130, 512), (65, 768), (4099, 1024), (300, 2048), (31, 2560), (17, 8192), (65536, 1024)])
def test_q6k_norm_and_quantizer_inside_the_gemv_launch(ctx, oracle, m, k):
    """y = W rmsnorm(x), the LM head's form: every wave of the Q6_K GEMV norms and quantizes x itself.  Bit-identical to the norm +
    quantizer launch followed by the pre-quantized GEMV (also with accumulate), and within the f32 bar of the oracle's GEMV on the
    same quants."""
    ops, eps = Lfm2Ops(ctx), 1e-5
    with Problem(ctx, oracle, W.Q6_K, m, k, seed=2 * m + k) as p:
        x = oracle.fill_normal(m + k, 1.7, k)
        nw = (1 + 0.3 * oracle.fill_normal(k, 1.0, k)).astype(np.float32)
        d_x, d_nw = p.to_device(x), p.to_device(nw)
        d_q, d_s = p.alloc(k), p.alloc(k // 32 * 4)
        ops.rmsnorm_quantize(d_x, d_nw, 1, k, eps, d_q, d_s)
        y0 = oracle.fill_normal(5, 1.0, m)
        d_y, d_z, d_ya, d_za = p.alloc(m * 4), p.alloc(m * 4), p.to_device(y0), p.to_device(y0)
        ctx.gemv_with_preq(p.w, d_s, d_q, d_z)
        ctx.encode_gemv_rmsnorm_fused([p.w], d_x, d_nw, eps, [d_y])
        y, z = d_y.download(np.float32, m), d_z.download(np.float32, m)
        assert np.array_equal(y.view(np.uint32), z.view(np.uint32))
        ctx.gemv_with_preq(p.w, d_s, d_q, d_za, accumulate=True)
        ctx.encode_gemv_rmsnorm_fused([p.w], d_x, d_nw, eps, [d_ya], accumulate=True)
        assert np.array_equal(d_ya.download(np.float32, m).view(np.uint32), d_za.download(np.float32, m).view(np.uint32))
        q, sc = d_q.download(np.int8, k), d_s.download(np.float32, k // 32)
        assert_f32_parity(y, oracle.gemv_q6k_q8(p.wb, sc, q, m, k), f"q6k norm-fused gemv {m}x{k}")
        # the quants themselves: the oracle's norm then quantizer (inv_rms may differ in its last bit: at most a quant step)
        sr, qr = oracle.quantize_q8_0(L.rmsnorm(x, nw, eps))
        assert np.abs(q.astype(np.int32) - qr.astype(np.int32)).max() <= 1 and np.allclose(sc, sr, rtol=1e-3, atol=0)  # scales: f16 values, at most one step apart


@pytest.mark.parametrize("dtype,m,k", [(W.Q6_K, 5000, 1024), (W.Q6_K, 65536, 1024), (W.Q6_K, 300, 512), (W.Q6_K, 3, 256), (W.Q4_0, 5000, 1024), (W.Q8_0, 777, 256)])
def test_lm_head_and_greedy_pick_in_two_launches(ctx, oracle, dtype, m, k):
    """Output norm + LM head + greedy pick as one call: logits bit-identical to the norm-fused GEMV, the pick is cpu_argmax of them
    (wick/src/sampler.rs:7-19) -- for a Q6_K head taken from the keys its waves leave behind."""
    ops, eps = Lfm2Ops(ctx), 1e-5
    with Problem(ctx, oracle, dtype, m, k, seed=m + k) as p:
        x = oracle.fill_normal(3 * m + k, 1.3, k)
        nw = (1 + 0.3 * oracle.fill_normal(k + 1, 1.0, k)).astype(np.float32)
        d_x, d_nw = p.to_device(x), p.to_device(nw)
        d_y, d_z, d_out = p.alloc(m * 4), p.alloc(m * 4), p.alloc(4)
        d_tok, d_pos = p.to_device(np.array([0], np.uint32)), p.to_device(np.array([9], np.uint32))
        ctx.encode_gemv_rmsnorm_fused([p.w], d_x, d_nw, eps, [d_z])
        ops.lm_head_greedy(p.w, d_x, d_nw, eps, d_y, d_out, d_token=d_tok, d_pos=d_pos)
        y, z = d_y.download(np.float32, m), d_z.download(np.float32, m)
        assert np.array_equal(y.view(np.uint32), z.view(np.uint32))
        pick = int(d_out.download(np.uint32, 1)[0])
        assert pick == L.argmax(y) and int(d_tok.download(np.uint32, 1)[0]) == pick and int(d_pos.download(np.uint32, 1)[0]) == 10


def test_lm_head_greedy_pick_takes_the_last_of_equal_logits(ctx, oracle):
    """Every row of the head is the same row: all logits are equal and the pick is the last index, whichever wave holds it."""
    ops, m, k = Lfm2Ops(ctx), 3001, 1024
    row = oracle.synth_weight(W.Q6_K, 1, k, 12)
    wb = np.tile(row, m)
    with Problem(ctx, oracle, W.Q6_K, m, k, seed=1, weight_bytes=wb) as p:
        d_x, d_nw = p.to_device(oracle.fill_normal(4, 1.0, k)), p.to_device(np.ones(k, np.float32))
        d_y, d_out = p.alloc(m * 4), p.alloc(4)
        ops.lm_head_greedy(p.w, d_x, d_nw, 1e-5, d_y, d_out)
        y = d_y.download(np.float32, m)
        assert (y == y[0]).all() and int(d_out.download(np.uint32, 1)[0]) == m - 1


def test_q6k_rejects(ctx, oracle):
    wb = oracle.synth_weight(W.Q6_K, 4, 256, 1)
    with pytest.raises(W.RocmError):
        ctx.upload_weight(wb[:-1], W.Q6_K, 4, 256)
    with pytest.raises(W.RocmError):
        ctx.upload_weight(np.zeros(4 * 210 // 2, np.uint8), W.Q6_K, 4, 128)
