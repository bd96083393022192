"""The decode step's non-matmul operations on the GPU against the oracle (wick/src/backend/cpu.rs:577-731,
1320-1401, 2113-2161; wick/src/model/lfm2.rs:621-726).  Bit-exact where the kernel keeps the reference's
operation order (embedding rows, SiLU gate, short conv, attention scores, argmax); within a stated
tolerance where a sum is taken in another order or sin/cos come from the device library."""
import numpy as np
import pytest

import wick_amd as W
from oracle import lfm2_oracle as L
from wick_amd.lfm2 import Lfm2Ops, attention_block_scratch_bytes, attention_scratch_floats, rope_theta_scale

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ops(ctx):
    return Lfm2Ops(ctx)


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def max_ulp(a, b):
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    return int(np.abs(a - b).max())


@pytest.mark.parametrize("dtype,k", [(W.Q4_0, 256), (W.Q8_0, 1024), (W.Q6_K, 512), (W.Q6_K, 1024)])
def test_embed_row(ctx, ops, oracle, dtype, k):
    m = 77
    wb = oracle.synth_weight(dtype, m, k, seed=k + dtype)
    w = ctx.upload_weight(wb, dtype, m, k)
    d_out, d_tok = ctx.alloc(k * 4), ctx.to_device(np.array([m - 1], np.uint32))
    for token in (0, 13, m - 1):
        ops.embed_row(w, d_out, token)
        assert np.array_equal(bits(d_out.download(np.float32, k)), bits(L.embed_row(dtype, wb, token, k)))
    ops.embed_row(w, d_out, 0, d_token=d_tok)  # device-side token wins over the by-value one
    assert np.array_equal(bits(d_out.download(np.float32, k)), bits(L.embed_row(dtype, wb, m - 1, k)))
    with pytest.raises(W.RocmError):
        ops.embed_row(w, d_out, m)
    w.free(), d_out.free(), d_tok.free()


@pytest.mark.parametrize("rows,dim", [(1, 4), (1, 1024), (1, 2048), (16, 64), (3, 100), (1, 5000)])
def test_rmsnorm(ctx, ops, oracle, rows, dim):
    x = oracle.fill_normal(rows * dim, 1.5, rows * dim)
    w = 1.0 + 0.3 * oracle.fill_normal(dim, 1.0, dim)
    d_x, d_w, d_y = ctx.to_device(x), ctx.to_device(w), ctx.alloc(rows * dim * 4)
    ops.encode_rmsnorm(d_x, d_w, d_y, dim, 1e-5, rows=rows)
    y = d_y.download(np.float32, rows * dim).reshape(rows, dim)
    ref = np.stack([L.rmsnorm(x[r * dim:(r + 1) * dim], w, 1e-5) for r in range(rows)])
    # the f64 sum of squares is taken in another order: inv_rms may differ in its last bit
    assert max_ulp(y, ref) <= 2
    ops.encode_rmsnorm(d_x, d_w, d_x, dim, 1e-5, rows=rows)  # in place
    assert np.array_equal(d_x.download(np.float32, rows * dim).reshape(rows, dim), y)
    for b in (d_x, d_w, d_y):
        b.free()


def test_rmsnorm_reference_closed_forms(ctx, ops):
    d_x, d_w, d_y = ctx.to_device(np.array([1, 2, 3, 4], np.float32)), ctx.to_device(np.ones(4, np.float32)), ctx.alloc(16)
    ops.encode_rmsnorm(d_x, d_w, d_y, 4, 1e-5)  # wick/src/backend/cpu.rs:2278-2295
    assert np.allclose(d_y.download(np.float32, 4), np.array([1, 2, 3, 4]) / np.sqrt(7.5 + 1e-5), atol=1e-6)
    for b in (d_x, d_w, d_y):
        b.free()


@pytest.mark.parametrize("n", [1, 255, 4608, 10000])
def test_silu_mul_bit_exact(ctx, ops, oracle, n):
    g = oracle.fill_normal(n + 1, 4.0, n)
    g[: min(n, 8)] = np.array([0.0, -0.0, 90.0, -90.0, 104.0, -104.0, 1e-30, -200.0], np.float32)[: min(n, 8)]  # every range branch of expf
    u = oracle.fill_normal(n + 2, 1.0, n)
    d_g, d_u = ctx.to_device(g), ctx.to_device(u)
    ops.silu_mul_inplace(d_g, d_u, n)
    assert np.array_equal(bits(d_g.download(np.float32, n)), bits(L.silu_mul(g, u)))
    d_g.free(), d_u.free()


@pytest.mark.parametrize("hidden,kernel", [(96, 3), (1024, 3), (300, 4), (64, 2), (128, 1)])
def test_shortconv_steps_bit_exact(ctx, ops, oracle, hidden, kernel):
    w = oracle.fill_normal(kernel, 0.5, hidden * kernel)
    buf = np.zeros(max(kernel - 1, 1) * hidden, np.float32)
    d_w, d_buf, d_out = ctx.to_device(w), ctx.to_device(buf), ctx.alloc(hidden * 4)
    ref_buf = np.zeros((kernel - 1) * hidden, np.float32)
    for step in range(5):
        proj = oracle.fill_normal(100 + step, 1.0, 3 * hidden)
        d_proj = ctx.to_device(proj)
        ops.encode_conv1d_fused(d_proj, d_buf, d_w, d_out, hidden, kernel)
        ref = L.shortconv_step(proj, ref_buf, w, hidden, kernel)
        assert np.array_equal(bits(d_out.download(np.float32, hidden)), bits(ref))
        if kernel > 1:
            assert np.array_equal(bits(d_buf.download(np.float32, (kernel - 1) * hidden)), bits(ref_buf))
        d_proj.free()
    for b in (d_w, d_buf, d_out):
        b.free()


@pytest.mark.parametrize("hidden,kernel,n,start", [(1024, 3, 70, 0), (96, 3, 5, 2), (320, 4, 9, 1), (64, 2, 3, 0), (128, 1, 4, 0), (1024, 3, 1, 3),
                                                   (300, 3, 6, 0)])
def test_shortconv_of_a_prompt(ctx, ops, oracle, hidden, kernel, n, start):
    """The convolution of n prompt tokens at once (wick/src/model/lfm2.rs:1306-1350) == n single steps, bit for bit, state included
    (`start` single steps first, so the rolling state is not all zero); its quantizing form == the float form + the Q8_0 quantizer."""
    w = oracle.fill_normal(kernel, 0.5, hidden * kernel)
    d_w = ctx.to_device(w)
    ref_buf = np.zeros((kernel - 1) * hidden, np.float32)
    d_buf = ctx.to_device(np.zeros(max(kernel - 1, 1) * hidden, np.float32))
    d_out1 = ctx.alloc(hidden * 4)
    for step in range(start):
        proj = oracle.fill_normal(50 + step, 1.0, 3 * hidden)
        d_p = ctx.to_device(proj)
        ops.encode_conv1d_fused(d_p, d_buf, d_w, d_out1, hidden, kernel)
        L.shortconv_step(proj, ref_buf, w, hidden, kernel)
        d_p.free()
    state0 = d_buf.download(np.float32, max(kernel - 1, 1) * hidden)
    projs = oracle.fill_normal(200 + n, 1.0, n * 3 * hidden)
    want = np.stack([L.shortconv_step(projs[j * 3 * hidden:(j + 1) * 3 * hidden], ref_buf, w, hidden, kernel) for j in range(n)])
    d_projs, d_out = ctx.to_device(projs), ctx.alloc(n * hidden * 4)
    ops.encode_conv1d_seq(d_projs, d_buf, d_w, d_out, hidden, kernel, n)
    got = d_out.download(np.float32, n * hidden).reshape(n, hidden)
    assert np.array_equal(bits(got), bits(want))
    if kernel > 1:
        assert np.array_equal(bits(d_buf.download(np.float32, (kernel - 1) * hidden)), bits(ref_buf))
    d_q, d_s = ctx.alloc(n * hidden), ctx.alloc(n * (hidden // 32 + 1) * 4)
    if hidden % 32 == 0:
        d_buf2 = ctx.to_device(state0)
        ops.encode_conv1d_seq_quantize(d_projs, d_buf2, d_w, d_q, d_s, hidden, kernel, n)
        fq, fs = d_q.download(np.int8, n * hidden), d_s.download(np.float32, n * (hidden // 32))
        ctx.quantize_q8_0(d_out, n, hidden, hidden, d_q, d_s)
        assert np.array_equal(fq, d_q.download(np.int8, n * hidden)) and np.array_equal(bits(fs), bits(d_s.download(np.float32, n * (hidden // 32))))
        rs, rq = oracle.quantize_q8_0_batch(want.reshape(-1), n, hidden)
        assert np.array_equal(fq, rq.reshape(-1)) and np.array_equal(bits(fs), bits(rs.reshape(-1)))
        if kernel > 1:
            assert np.array_equal(bits(d_buf2.download(np.float32, (kernel - 1) * hidden)), bits(ref_buf))
        d_buf2.free()
    else:
        with pytest.raises(W.RocmError, match="hidden % 32"):
            ops.encode_conv1d_seq_quantize(d_projs, d_buf, d_w, d_q, d_s, hidden, kernel, n)
    for b in (d_w, d_buf, d_out1, d_projs, d_out, d_q, d_s):
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,hd,pos", [(4, 2, 64, 0), (16, 8, 64, 5), (8, 8, 32, 300), (4, 1, 128, 4095), (2, 2, 256, 17)])
def test_qk_norm_rope_and_append(ctx, ops, oracle, n_heads, n_kv, hd, pos):
    max_seq, eps, base = 4096, 1e-5, 1_000_000.0
    kv_dim = n_kv * hd
    q, k, v = oracle.fill_normal(1, 1.0, n_heads * hd), oracle.fill_normal(2, 1.0, kv_dim), oracle.fill_normal(3, 1.0, kv_dim)
    qn, kn = 1 + 0.2 * oracle.fill_normal(4, 1.0, hd), 1 + 0.2 * oracle.fill_normal(5, 1.0, hd)
    d = {n: ctx.to_device(a) for n, a in dict(q=q, k=k, v=v, qn=qn, kn=kn).items()}
    d_kc, d_vc = ctx.to_device(np.full(max_seq * kv_dim, 7.0, np.float32)), ctx.to_device(np.full(max_seq * kv_dim, 7.0, np.float32))
    ts = rope_theta_scale(hd, base)
    assert ts == L.rope_theta_scale(hd, base)
    ops.encode_qk_norm_rope(d["q"], d["k"], d["v"], d["qn"], d["kn"], d_kc, d_vc, pos, max_seq, hd, n_heads, n_kv, eps, ts)
    qr = np.concatenate([L.rmsnorm(q[h * hd:(h + 1) * hd], qn, eps) for h in range(n_heads)])
    kr = np.concatenate([L.rmsnorm(k[h * hd:(h + 1) * hd], kn, eps) for h in range(n_kv)])
    qr, kr = L.rope(qr, kr, pos, n_heads, n_kv, hd, base)
    got_q, got_k = d["q"].download(np.float32, n_heads * hd), d["k"].download(np.float32, kv_dim)
    # sin/cos of the device library vs libm (an ulp or two of a value <= 1) on top of the norm's last-bit freedom
    assert np.allclose(got_q, qr, rtol=0, atol=2e-6 * np.abs(qr).max()) and np.allclose(got_k, kr, rtol=0, atol=2e-6 * np.abs(kr).max())
    kc = d_kc.download(np.float32, max_seq * kv_dim).reshape(max_seq, kv_dim)
    vc = d_vc.download(np.float32, max_seq * kv_dim).reshape(max_seq, kv_dim)
    assert np.array_equal(bits(kc[pos]), bits(got_k)) and np.array_equal(bits(vc[pos]), bits(v))
    untouched = np.ones(max_seq, bool)
    untouched[pos] = False
    assert (kc[untouched] == 7.0).all() and (vc[untouched] == 7.0).all()
    with pytest.raises(W.RocmError):
        ops.encode_qk_norm_rope(d["q"], d["k"], d["v"], d["qn"], d["kn"], d_kc, d_vc, max_seq, max_seq, hd, n_heads, n_kv, eps, ts)
    for b in list(d.values()) + [d_kc, d_vc]:
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,hd,max_seq", [(16, 8, 64, 4096), (4, 2, 64, 100), (8, 2, 128, 512), (3, 1, 96, 70)])
def test_attention_over_one_position_returns_the_value_row(ctx, ops, oracle, n_heads, n_kv, hd, max_seq):
    """The closed form the reference's own test leans on (wick/tests/single_token_attn.rs:33-43): with one cached position
    softmax([score]) = [1] for every head, so the attention's output is the value row, repeated for the query heads of a
    group -- bit for bit here, since ggml_expf(0) = 1 and v * 1 / 1 = v.  Through both decode paths (plain attention over a
    cache that holds the row, and the block that appends the row itself) and the prompt kernel with one token."""
    kv_dim = n_kv * hd
    q, v = oracle.fill_normal(1, 3.0, n_heads * hd), oracle.fill_normal(2, 1.0, kv_dim)
    kc = oracle.fill_normal(3, 1.0, max_seq * kv_dim)
    vc = np.full(max_seq * kv_dim, np.nan, np.float32)  # nothing past the first row may be looked at
    vc[:kv_dim] = v
    want = np.concatenate([v[(h // (n_heads // n_kv)) * hd:(h // (n_heads // n_kv) + 1) * hd] for h in range(n_heads)])
    d_q, d_kc, d_vc = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc)
    d_out, d_sc = ctx.alloc(n_heads * hd * 4), ctx.alloc(attention_block_scratch_bytes(max_seq, n_heads, hd))
    ops.encode_attention(d_q, d_kc, d_vc, d_out, d_sc, 1, max_seq, n_heads, n_kv, hd)
    assert np.array_equal(bits(d_out.download(np.float32, n_heads * hd)), bits(want))
    if hd != 96:  # the prompt kernels take head dims 32 / 64 / 128 / 256 (a model with another one attends token by token)
        ops.encode_attention_prefill(d_q, n_heads * hd, d_kc, d_vc, d_out, n_heads * hd, 0, 1, max_seq, n_heads, n_kv, hd)
        assert np.array_equal(bits(d_out.download(np.float32, n_heads * hd)), bits(want))
    # the block: norms and rotates q and k, appends k and v at position 0, attends over that one row
    d_k, d_v = ctx.to_device(oracle.fill_normal(4, 1.0, kv_dim)), ctx.to_device(v)
    d_qn, d_kn = ctx.to_device(1 + 0.2 * oracle.fill_normal(5, 1.0, hd)), ctx.to_device(1 + 0.2 * oracle.fill_normal(6, 1.0, hd))
    d_vc2 = ctx.to_device(np.full(max_seq * kv_dim, np.nan, np.float32))
    ops.encode_attention_block(d_q, d_k, d_v, d_qn, d_kn, d_kc, d_vc2, d_out, d_sc, 0, max_seq, hd, n_heads, n_kv, 1e-5, rope_theta_scale(hd, 1_000_000.0))
    assert np.array_equal(bits(d_out.download(np.float32, n_heads * hd)), bits(want))
    for b in (d_q, d_kc, d_vc, d_out, d_sc, d_k, d_v, d_qn, d_kn, d_vc2):
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,hd,pos0,n,pad", [(16, 8, 64, 0, 40, 0), (4, 2, 64, 4000, 96, 8), (3, 1, 128, 7, 5, 0), (2, 2, 256, 100, 3, 4),
                                                        (5, 5, 32, 0, 1, 0)])
def test_qk_norm_rope_of_a_prompt(ctx, ops, oracle, n_heads, n_kv, hd, pos0, n, pad):
    """Pass A of the batched prefill (wick/src/model/lfm2.rs:1557-1620): one launch for the n tokens == n single-token launches, bit for bit
    (the prompt kernel shares a position's sin / cos between the heads; same operations per element)."""
    max_seq, eps, base = 4096, 1e-5, 1_000_000.0
    kv_dim = n_kv * hd
    q_stride, kv_stride = n_heads * hd + 2 * kv_dim + pad, n_heads * hd + 2 * kv_dim + pad  # one [q | k | v] row per token, like the prompt pass
    rows = oracle.fill_normal(11 + n, 1.0, n * q_stride)
    qn, kn = 1 + 0.2 * oracle.fill_normal(4, 1.0, hd), 1 + 0.2 * oracle.fill_normal(5, 1.0, hd)
    d_qn, d_kn = ctx.to_device(qn), ctx.to_device(kn)
    ts = rope_theta_scale(hd, base)
    out = []
    for batched in (True, False):
        d_rows = ctx.to_device(rows)
        d_kc, d_vc = ctx.to_device(np.full(max_seq * kv_dim, 7.0, np.float32)), ctx.to_device(np.full(max_seq * kv_dim, 7.0, np.float32))
        q_ptr, k_ptr, v_ptr = d_rows.ptr, d_rows.ptr + 4 * n_heads * hd, d_rows.ptr + 4 * (n_heads * hd + kv_dim)
        if batched:
            ops.encode_qk_norm_rope_tokens(q_ptr, q_stride, k_ptr, v_ptr, kv_stride, d_qn, d_kn, d_kc, d_vc, pos0, n, max_seq, hd, n_heads, n_kv, eps, ts)
        else:
            for j in range(n):
                o = 4 * j * q_stride
                ops.encode_qk_norm_rope(q_ptr + o, k_ptr + o, v_ptr + o, d_qn, d_kn, d_kc, d_vc, pos0 + j, max_seq, hd, n_heads, n_kv, eps, ts)
        out.append((d_rows.download(np.float32, n * q_stride), d_kc.download(np.float32, max_seq * kv_dim), d_vc.download(np.float32, max_seq * kv_dim)))
        for b in (d_rows, d_kc, d_vc):
            b.free()
    for a, b in zip(*out):
        assert np.array_equal(bits(a), bits(b))
    got = out[0][0].reshape(n, q_stride)
    assert np.array_equal(bits(got[:, n_heads * hd + kv_dim:]), bits(rows.reshape(n, q_stride)[:, n_heads * hd + kv_dim:]))  # v and the padding untouched
    kc = out[0][1].reshape(max_seq, kv_dim)
    assert np.array_equal(bits(kc[pos0:pos0 + n]), bits(got[:, n_heads * hd: n_heads * hd + kv_dim])) and (kc[:pos0] == 7.0).all() and (kc[pos0 + n:] == 7.0).all()
    with pytest.raises(W.RocmError, match="beyond the cache"):
        ops.encode_qk_norm_rope_tokens(d_qn, q_stride, d_qn, d_qn, kv_stride, d_qn, d_kn, d_qn, d_qn, max_seq - n + 1, n, max_seq, hd, n_heads, n_kv, eps, ts)
    d_qn.free(), d_kn.free()


# contexts of <= 256 positions (and head_dim 96) run the one-workgroup kernel, longer ones the sequence-split kernel;
# 20000 positions make every workgroup walk several chunks
@pytest.mark.parametrize("n_heads,n_kv,hd,seq", [(4, 2, 64, 1), (16, 8, 64, 10), (16, 8, 64, 253), (16, 8, 64, 257), (8, 2, 64, 1500), (4, 4, 32, 33),
                                                 (3, 1, 96, 70), (3, 1, 96, 600), (2, 1, 256, 19), (4, 4, 32, 700), (4, 1, 128, 600),
                                                 (2, 1, 256, 300), (16, 8, 64, 4096), (2, 1, 64, 20000)])
def test_attention_decode(ctx, ops, oracle, n_heads, n_kv, hd, seq):
    max_seq, kv_dim = seq + 3, n_kv * hd
    single = max_seq <= 256 or hd == 96
    q = oracle.fill_normal(seq, 1.0, n_heads * hd)
    kc, vc = oracle.fill_normal(seq + 1, 1.0, max_seq * kv_dim), oracle.fill_normal(seq + 2, 1.0, max_seq * kv_dim)
    d_q, d_kc, d_vc = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc)
    d_out, d_sc = ctx.alloc(n_heads * hd * 4), ctx.alloc(attention_scratch_floats(max_seq, n_heads, hd) * 4)
    ops.encode_attention(d_q, d_kc, d_vc, d_out, d_sc, seq, max_seq, n_heads, n_kv, hd)
    got = d_out.download(np.float32, n_heads * hd)
    ref = L.attention(q, kc[: seq * kv_dim], vc[: seq * kv_dim], n_heads, n_kv, hd, seq)
    # probabilities: exp bit-exact, their f64 sum in another order; values summed in four interleaved parts
    assert np.allclose(got, ref, rtol=0, atol=4e-6 * max(np.abs(ref).max(), 1e-3))
    if single:  # this kernel's scratch holds the unnormalised exp(score - max): bit-exact against the oracle's scores
        sc = d_sc.download(np.float32, n_heads * max_seq).reshape(n_heads, max_seq)[:, :seq]
        scale = np.float32(1.0) / np.sqrt(np.float32(hd))
        for h in (0, n_heads - 1):
            s = L.attn_scores(q[h * hd:(h + 1) * hd], kc, kv_dim, (h // (n_heads // n_kv)) * hd, hd, scale, seq)
            e = np.array([L.ggml_expf(float(np.float32(x) - s.max())) for x in s], np.float32)
            assert np.array_equal(bits(sc[h]), bits(e))
    # device-side position: seq_len = *d_pos + 1
    d_pos = ctx.to_device(np.array([seq - 1], np.uint32))
    ops.encode_attention(d_q, d_kc, d_vc, d_out, d_sc, 0, max_seq, n_heads, n_kv, hd, d_pos=d_pos)
    assert np.array_equal(bits(d_out.download(np.float32, n_heads * hd)), bits(got))
    if seq > 300:  # a shorter prefix of the same cache: workgroups past the end stay out, partials of an earlier call are not picked up
        ops.encode_attention(d_q, d_kc, d_vc, d_out, d_sc, 290, max_seq, n_heads, n_kv, hd)
        ref = L.attention(q, kc[: 290 * kv_dim], vc[: 290 * kv_dim], n_heads, n_kv, hd, 290)
        assert np.allclose(d_out.download(np.float32, n_heads * hd), ref, rtol=0, atol=4e-6 * np.abs(ref).max())
    for b in (d_q, d_kc, d_vc, d_out, d_sc, d_pos):
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,hd,pos0,n,pad", [
    (4, 2, 64, 0, 16, 0), (4, 4, 64, 0, 63, 4), (8, 2, 64, 5, 130, 0), (4, 1, 64, 100, 64, 8), (2, 2, 64, 0, 200, 0), (16, 8, 64, 61, 67, 0),
    (4, 2, 64, 37, 450, 0), (2, 1, 64, 0, 1000, 0),  # 8 and 16 blocks of 64 queries, taken in (long, short) pairs
    (4, 2, 64, 0, 9, 0),     # fewer than 16 tokens: the scalar kernel
    (4, 2, 32, 3, 40, 0), (2, 1, 128, 0, 70, 4),  # head dims without a matrix-core kernel
])
def test_attention_prefill(ctx, ops, oracle, n_heads, n_kv, hd, pos0, n, pad):
    """Causal attention over a prompt (wick/src/model/lfm2.rs:1640-1700): token j == the decode attention with seq_len = pos0 + j + 1.
    head_dim 64 runs on the matrix cores (f32 operands as f16 hi + lo, three exact-product MFMAs per product), sums in tiles of 64
    positions."""
    kv_dim, seq_total = n_kv * hd, pos0 + n
    max_seq = seq_total + 2
    q_stride, out_stride = n_heads * hd + 2 * kv_dim + pad, n_heads * hd + pad
    q = oracle.fill_normal(7 * n + pos0, 1.0, n * q_stride)
    kc, vc = oracle.fill_normal(n + 1, 1.0, max_seq * kv_dim), oracle.fill_normal(n + 2, 1.0, max_seq * kv_dim)
    d_q, d_kc, d_vc = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc)
    d_out = ctx.to_device(np.full(n * out_stride, 7.5, np.float32))
    ops.encode_attention_prefill(d_q, q_stride, d_kc, d_vc, d_out, out_stride, pos0, n, max_seq, n_heads, n_kv, hd)
    got = d_out.download(np.float32, n * out_stride).reshape(n, out_stride)
    assert np.all(got[:, n_heads * hd:] == 7.5)  # padding between rows is left alone
    for j in sorted({0, 1, 15, 16, 17, 63, 64, 65, 127, 128, n // 2, n - 65, n - 64, n - 2, n - 1} & set(range(n))) if n > 80 else range(n):
        seq = pos0 + j + 1
        ref = L.attention(q[j * q_stride: j * q_stride + n_heads * hd], kc[: seq * kv_dim], vc[: seq * kv_dim], n_heads, n_kv, hd, seq)
        assert np.allclose(got[j, : n_heads * hd], ref, rtol=0, atol=4e-6 * max(np.abs(ref).max(), 1e-3)), f"token {j}"
    with pytest.raises(W.RocmError, match="beyond the cache"):
        ops.encode_attention_prefill(d_q, q_stride, d_kc, d_vc, d_out, out_stride, 3, n, n + 2, n_heads, n_kv, hd)
    for b in (d_q, d_kc, d_vc, d_out):
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,pos0,n,qscale", [(4, 2, 0, 300, 1.0), (4, 2, 50, 300, 3.0), (16, 8, 0, 2002, 1.0), (4, 2, 0, 200, 6.0)])
def test_attention_prefill_accuracy_against_f64(ctx, ops, n_heads, n_kv, pos0, n, qscale):
    """The matrix-core prompt attention takes its two products from f16 hi + lo halves of the f32 operands (three exact-product
    MFMAs per product).  Held against an f64 evaluation of the same attention (textbook softmax(QK^T / sqrt(d)) V, causal): rel-L2
    <= 1e-6 and max error <= 2e-6 of the largest output, also with logits of a few tens (qscale) -- the f32 bar of this path
    (north star: rel-L2 1e-5) with an order of magnitude to spare.  Measured: 2e-7 .. 4e-7 / 1.4e-7 .. 8e-7."""
    hd = 64
    rng = np.random.default_rng(n + pos0)
    kv_dim, max_seq, qs = n_kv * hd, pos0 + n + 4, n_heads * hd + 2 * n_kv * hd
    q = (rng.standard_normal(n * qs) * qscale).astype(np.float32)
    kc, vc = rng.standard_normal(max_seq * kv_dim).astype(np.float32), rng.standard_normal(max_seq * kv_dim).astype(np.float32)
    d_q, d_k, d_v, d_o = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc), ctx.alloc(n * n_heads * hd * 4)
    ops.encode_attention_prefill(d_q, qs, d_k, d_v, d_o, n_heads * hd, pos0, n, max_seq, n_heads, n_kv, hd)
    got = d_o.download(np.float32, n * n_heads * hd).reshape(n, n_heads * hd).astype(np.float64)
    rows = np.arange(n) if n <= 400 else np.unique(np.concatenate([np.arange(0, n, 37), np.arange(n - 70, n), np.arange(0, 130)]))
    want = np.zeros((len(rows), n_heads * hd))
    for h in range(n_heads):
        kvh = h // (n_heads // n_kv)
        K = kc.reshape(-1, kv_dim)[:, kvh * hd:(kvh + 1) * hd].astype(np.float64)
        V = vc.reshape(-1, kv_dim)[:, kvh * hd:(kvh + 1) * hd].astype(np.float64)
        Q = q.reshape(n, qs)[rows, h * hd:(h + 1) * hd].astype(np.float64) / np.sqrt(hd)
        S = Q @ K[:pos0 + n].T
        for i, j in enumerate(rows):
            sj = S[i, :pos0 + j + 1]
            p = np.exp(sj - sj.max())
            want[i, h * hd:(h + 1) * hd] = (p @ V[:pos0 + j + 1]) / p.sum()
    err = np.abs(got[rows] - want)
    assert np.linalg.norm(got[rows] - want) / np.linalg.norm(want) <= 1e-6
    assert err.max() <= 2e-6 * np.abs(want).max()
    for b in (d_q, d_k, d_v, d_o):
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,pos0,n", [(4, 2, 0, 16), (16, 8, 61, 67), (2, 1, 0, 200), (4, 4, 37, 450)])
def test_attention_prefill_quantizing_epilogue(ctx, ops, oracle, n_heads, n_kv, pos0, n):
    """The prompt attention writing Q8_0 blocks (the out projection's input) == the float result + the quantizer, bit for bit."""
    hd = 64
    kv_dim, max_seq = n_kv * hd, pos0 + n + 2
    q_stride, hs = n_heads * hd + 2 * kv_dim, n_heads * hd
    q = oracle.fill_normal(7 * n + pos0, 1.0, n * q_stride)
    kc, vc = oracle.fill_normal(n + 1, 1.0, max_seq * kv_dim), oracle.fill_normal(n + 2, 1.0, max_seq * kv_dim)
    d_q, d_kc, d_vc = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc)
    d_out, d_oq, d_os = ctx.alloc(n * hs * 4), ctx.to_device(np.full(n * hs, 99, np.int8)), ctx.alloc(n * (hs // 32) * 4)
    ops.encode_attention_prefill_quantize(d_q, q_stride, d_kc, d_vc, d_oq, d_os, pos0, n, max_seq, n_heads, n_kv, hd)
    fq, fs = d_oq.download(np.int8, n * hs), d_os.download(np.float32, n * (hs // 32))
    ops.encode_attention_prefill(d_q, q_stride, d_kc, d_vc, d_out, hs, pos0, n, max_seq, n_heads, n_kv, hd)
    ctx.quantize_q8_0(d_out, n, hs, hs, d_oq, d_os)
    assert np.array_equal(fq, d_oq.download(np.int8, n * hs)) and np.array_equal(bits(fs), bits(d_os.download(np.float32, n * (hs // 32))))
    with pytest.raises(W.RocmError, match="head_dim 64"):
        ops.encode_attention_prefill_quantize(d_q, q_stride, d_kc, d_vc, d_oq, d_os, pos0, 8, max_seq, n_heads, n_kv, hd)
    with pytest.raises(W.RocmError, match="beyond the cache"):
        ops.encode_attention_prefill_quantize(d_q, q_stride, d_kc, d_vc, d_oq, d_os, 3, n, n + 2, n_heads, n_kv, hd)
    for b in (d_q, d_kc, d_vc, d_out, d_oq, d_os):
        b.free()


@pytest.mark.parametrize("n_heads,n_kv,hd,max_seq,steps", [(4, 2, 64, 300, [0, 1, 2, 63, 64, 65, 130, 299]), (16, 8, 64, 4096, [0, 700, 4095]),
                                                           (4, 4, 32, 64, [0, 5, 63]), (2, 1, 128, 5000, [4100, 4999]), (2, 1, 256, 100, [99]),
                                                           (3, 1, 96, 80, [0, 7, 79])])
def test_attention_block_equals_the_separate_launches(ctx, ops, oracle, n_heads, n_kv, hd, max_seq, steps):
    """The block (norm + RoPE + append folded into the attention kernel) against qk_norm_rope followed by attention,
    bit for bit, over several positions of one cache; head_dim 96 takes the block's unfused path."""
    kv_dim, eps, ts = n_kv * hd, 1e-5, rope_theta_scale(hd, 1_000_000.0)
    cache = oracle.fill_normal(max_seq, 1.0, 2 * max_seq * kv_dim)
    kc_a, vc_a = ctx.to_device(cache[: max_seq * kv_dim]), ctx.to_device(cache[max_seq * kv_dim:])
    kc_b, vc_b = ctx.to_device(cache[: max_seq * kv_dim]), ctx.to_device(cache[max_seq * kv_dim:])
    d_qn, d_kn = ctx.to_device(1 + 0.2 * oracle.fill_normal(4, 1.0, hd)), ctx.to_device(1 + 0.2 * oracle.fill_normal(5, 1.0, hd))
    nbytes = attention_block_scratch_bytes(max_seq, n_heads, hd)
    d_scr = ctx.alloc(nbytes)
    d_sc2 = ctx.alloc(attention_scratch_floats(max_seq, n_heads, hd) * 4)
    d_oa, d_ob = ctx.alloc(n_heads * hd * 4), ctx.alloc(n_heads * hd * 4)
    for pos in steps:
        q, k, v = (oracle.fill_normal(10 * pos + i, 1.0, n) for i, n in enumerate((n_heads * hd, kv_dim, kv_dim)))
        qa, ka, va = ctx.to_device(q), ctx.to_device(k), ctx.to_device(v)
        qb, kb = ctx.to_device(q), ctx.to_device(k)
        ops.encode_attention_block(qa, ka, va, d_qn, d_kn, kc_a, vc_a, d_oa, d_scr, pos, max_seq, hd, n_heads, n_kv, eps, ts)
        ops.encode_qk_norm_rope(qb, kb, va, d_qn, d_kn, kc_b, vc_b, pos, max_seq, hd, n_heads, n_kv, eps, ts)
        ops.encode_attention(qb, kc_b, vc_b, d_ob, d_sc2, pos + 1, max_seq, n_heads, n_kv, hd)
        got, sep = d_oa.download(np.float32, n_heads * hd), d_ob.download(np.float32, n_heads * hd)
        if max_seq > 256 or hd == 96:  # the separate launches take the same sequence-split arithmetic (or the block its unfused path)
            assert np.array_equal(bits(got), bits(sep)), f"pos {pos}"
        else:  # short contexts: the separate attention call is the one-workgroup kernel, which sums in another order
            assert np.allclose(got, sep, rtol=0, atol=4e-6 * np.abs(sep).max()), f"pos {pos}"
        for b in (qa, ka, va, qb, kb):
            b.free()
    assert np.array_equal(bits(kc_a.download(np.float32, max_seq * kv_dim)), bits(kc_b.download(np.float32, max_seq * kv_dim)))
    assert np.array_equal(bits(vc_a.download(np.float32, max_seq * kv_dim)), bits(vc_b.download(np.float32, max_seq * kv_dim)))
    for b in (kc_a, vc_a, kc_b, vc_b, d_qn, d_kn, d_scr, d_sc2, d_oa, d_ob):
        b.free()


def test_argmax_rules(ctx, ops):
    """cpu_argmax (wick/src/sampler.rs:7-19): last of equal maxima, NaN = -inf, -0.0 < +0.0."""
    cases = [[1.0, 3.0, 2.0], [3.0, 1.0, 3.0, 2.0], [np.nan, 1.0, np.nan], [np.nan, np.nan], [np.nan, -np.inf], [0.0, -0.0], [-0.0, 0.0, -0.0],
             [-5.0], [-np.inf, -np.inf, -np.inf]]
    rng = np.random.default_rng(6)
    cases += [rng.integers(-3, 4, n).astype(np.float32) for n in (1000, 1024, 1025, 65536)]
    cases += [rng.standard_normal(65536).astype(np.float32)]
    d_out = ctx.alloc(4)
    for c in cases:
        x = np.asarray(c, np.float32)
        d_x = ctx.to_device(x)
        ops.argmax(d_x, x.size, d_out)
        assert int(d_out.download(np.uint32, 1)[0]) == L.argmax(x), c if x.size < 10 else x.size
        d_x.free()
    d_tok, d_pos = ctx.to_device(np.array([0], np.uint32)), ctx.to_device(np.array([41], np.uint32))
    d_x = ctx.to_device(np.array([0.5, 9.0, 1.0], np.float32))
    ops.argmax(d_x, 3, d_out, d_token=d_tok, d_pos=d_pos)
    assert d_tok.download(np.uint32, 1)[0] == 1 and d_pos.download(np.uint32, 1)[0] == 42
    for b in (d_out, d_tok, d_pos, d_x):
        b.free()


@pytest.mark.parametrize("rows,dim,pad", [(1, 32, 0), (3, 256, 0), (17, 1024, 8), (5, 4608, 0), (2, 2080, 4)])
def test_rmsnorm_quantize_equals_the_two_launches(ctx, ops, oracle, rows, dim, pad):
    """Norm and Q8_0 quantizer in one pass: quants and scale bits of rmsnorm followed by quantize_q8_0, and of the oracle."""
    stride, eps = dim + pad, 1e-5
    x = oracle.fill_normal(rows * 3 + dim, 1.5, rows * stride)
    wt = (1 + 0.3 * oracle.fill_normal(dim, 1.0, dim)).astype(np.float32)
    d_x, d_w = ctx.to_device(x), ctx.to_device(wt)
    d_n, d_q1, d_s1 = ctx.alloc(rows * dim * 4), ctx.alloc(rows * dim), ctx.alloc(rows * dim // 32 * 4)
    d_q2, d_s2 = ctx.alloc(rows * dim), ctx.alloc(rows * dim // 32 * 4)
    ops.encode_rmsnorm(d_x, d_w, d_n, dim, eps, rows=rows, x_stride=stride, y_stride=dim)
    ctx.quantize_q8_0(d_n, rows, dim, dim, d_q1, d_s1)
    ops.rmsnorm_quantize(d_x, d_w, rows, dim, eps, d_q2, d_s2, x_stride=stride)
    assert np.array_equal(d_q1.download(np.int8, rows * dim), d_q2.download(np.int8, rows * dim))
    assert np.array_equal(bits(d_s1.download(np.float32, rows * dim // 32)), bits(d_s2.download(np.float32, rows * dim // 32)))
    normed = np.concatenate([L.rmsnorm(x[r * stride: r * stride + dim], wt, eps) for r in range(rows)])
    if np.array_equal(bits(normed), bits(d_n.download(np.float32, rows * dim))):  # the f64 sum of squares is taken in another order than the oracle's loop
        s, q = oracle.quantize_q8_0_batch(normed, rows, dim)
        assert np.array_equal(q.ravel(), d_q2.download(np.int8, rows * dim))
    with pytest.raises(W.RocmError):
        ops.rmsnorm_quantize(d_x, d_w, rows, dim + 8, eps, d_q2, d_s2, x_stride=stride + 8)
    for b in (d_x, d_w, d_n, d_q1, d_s1, d_q2, d_s2):
        b.free()


@pytest.mark.parametrize("rows,dim", [(1, 32), (4, 256), (9, 4608), (33, 1024)])
def test_silu_mul_quantize_equals_the_two_launches(ctx, ops, oracle, rows, dim):
    g, u = oracle.fill_normal(rows + dim, 2.0, rows * dim), oracle.fill_normal(rows + dim + 1, 1.0, rows * dim)
    d_g, d_u = ctx.to_device(g), ctx.to_device(u)
    d_q1, d_s1, d_q2, d_s2 = ctx.alloc(rows * dim), ctx.alloc(rows * dim // 32 * 4), ctx.alloc(rows * dim), ctx.alloc(rows * dim // 32 * 4)
    ops.silu_mul_quantize(d_g, d_u, rows, dim, d_q2, d_s2)
    ops.silu_mul_inplace(d_g, d_u, rows * dim)
    ctx.quantize_q8_0(d_g, rows, dim, dim, d_q1, d_s1)
    assert np.array_equal(d_q1.download(np.int8, rows * dim), d_q2.download(np.int8, rows * dim))
    assert np.array_equal(bits(d_s1.download(np.float32, rows * dim // 32)), bits(d_s2.download(np.float32, rows * dim // 32)))
    s, q = oracle.quantize_q8_0_batch(L.silu_mul(g, u), rows, dim)  # silu_mul is bit-exact, so the oracle's quantizer must agree too
    assert np.array_equal(q.ravel(), d_q2.download(np.int8, rows * dim))
    for b in (d_g, d_u, d_q1, d_s1, d_q2, d_s2):
        b.free()


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("hidden,inter", [(256, 512), (1024, 4608), (2048, 1024), (192, 320)])
def test_shortconv_folded_into_its_neighbours(ctx, ops, oracle, dtype, hidden, inter):
    """Two launches instead of three per gated-conv layer: the convolution in the out projection's prologue (state read only),
    the state advance in the gate / up launch.  Hidden state, gate output and conv state after three tokens are bit-identical
    to shortconv_step + out projection (accumulate) + gate / up, and the conv output is the oracle's."""
    K, eps = 3, float(np.float32(1e-5))
    w_out = ctx.upload_weight(oracle.synth_weight(dtype, hidden, hidden, 61), dtype, hidden, hidden)
    w_gate = ctx.upload_weight(oracle.synth_weight(dtype, inter, hidden, 62), dtype, inter, hidden)
    w_up = ctx.upload_weight(oracle.synth_weight(dtype, inter, hidden, 63), dtype, inter, hidden)
    assert ops.shortconv_fusable(w_out, w_gate, w_up, K)
    assert not ops.shortconv_fusable(w_out, w_gate, w_up, 4)
    rng = np.random.default_rng(hidden + inter)
    conv_w = rng.standard_normal(hidden * K).astype(np.float32)
    norm_w = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    d_cw, d_nw = ctx.to_device(conv_w), ctx.to_device(norm_w)
    state0 = rng.standard_normal((K - 1) * hidden).astype(np.float32)
    h0 = rng.standard_normal(hidden).astype(np.float32)
    bufs = {name: (ctx.to_device(state0), ctx.to_device(h0), ctx.alloc(inter * 4)) for name in ("fused", "plain")}
    d_proj, d_gated = ctx.alloc(3 * hidden * 4), ctx.alloc(hidden * 4)
    ref_buf = state0.copy()
    for step in range(3):
        proj = rng.standard_normal(3 * hidden).astype(np.float32)
        d_proj.upload(proj)
        st, hid, act = bufs["fused"]
        ops.encode_shortconv_out_proj(w_out, d_proj, st, d_cw, K, hid, accumulate=True)
        ops.encode_ffn_gate_up_conv_advance(w_gate, w_up, hid, d_nw, eps, act, d_proj, st, hidden, K)
        st, hid, act = bufs["plain"]
        ops.encode_conv1d_fused(d_proj, st, d_cw, d_gated, hidden, K)
        ctx.encode_gemv(w_out, d_gated, 0, hid, 0, accumulate=True)
        ctx.encode_ffn_gate_up(w_gate, w_up, hid, d_nw, eps, act)
        want_gated = L.shortconv_step(proj, ref_buf, conv_w, hidden, K)
        assert np.array_equal(d_gated.download(np.float32, hidden).view(np.uint32), want_gated.view(np.uint32))
        for i, n in enumerate(((K - 1) * hidden, hidden, inter)):
            a, b = bufs["fused"][i].download(np.uint32, n), bufs["plain"][i].download(np.uint32, n)
            assert np.array_equal(a, b), f"step {step}: {('conv state', 'hidden', 'gate output')[i]} differs"
        assert np.array_equal(bufs["fused"][0].download(np.float32, (K - 1) * hidden).view(np.uint32), ref_buf.view(np.uint32))
    with pytest.raises(W.RocmError, match="kernel size 3") as e:
        ops.encode_shortconv_out_proj(w_out, d_proj, bufs["fused"][0], d_cw, 4, bufs["fused"][1])
    assert e.value.status == -3
    for w in (w_out, w_gate, w_up):
        w.free()
    for b in (d_cw, d_nw, d_proj, d_gated) + bufs["fused"] + bufs["plain"]:
        b.free()


@pytest.mark.parametrize("dtype,m,k,n", [(W.Q4_0, 4608, 1024, 2002), (W.Q8_0, 2080, 256, 1100), (W.Q4_0, 2048, 128, 1153)])
def test_gate_up_gemm_with_gate_and_quantizer_in_its_epilogue(ctx, ops, oracle, dtype, m, k, n):
    """gemm_preq(ffn_gate), gemm_preq(ffn_up), silu_mul_inplace and quantize_columns of the batched prefill
    (wick/src/model/lfm2.rs:2025-2090) as one launch: quants and scales bit-identical to the three-launch sequence, which the
    other tests hold against the oracle; a sampled band is checked against the oracle directly as well."""
    wg, wu = oracle.synth_weight(dtype, m, k, seed=31), oracle.synth_weight(dtype, m, k, seed=32)
    d_wg, d_wu = ctx.upload_weight(wg, dtype, m, k), ctx.upload_weight(wu, dtype, m, k)
    xs, xq = oracle.quantize_q8_0_batch(oracle.fill_normal(5, 1.0, n * k), n, k)
    d_xq, d_xs = ctx.to_device(xq), ctx.to_device(xs)
    assert ops.ffn_gate_up_silu_quantize_applies(d_wg, d_wu, n)
    d_oq, d_os = ctx.to_device(np.full(n * m, 99, np.int8)), ctx.alloc(n * (m // 32) * 4)
    ops.encode_ffn_gate_up_silu_quantize(d_wg, d_wu, d_xs, d_xq, n, d_oq, d_os)
    fq, fs = d_oq.download(np.int8, n * m), d_os.download(np.float32, n * (m // 32))
    d_g, d_u = ctx.alloc(n * m * 4), ctx.alloc(n * m * 4)
    ctx.gemm_preq_multi([d_wg, d_wu], d_xs, d_xq, n, [d_g, d_u], m)
    ops.silu_mul_quantize(d_g, d_u, n, m, d_oq, d_os)
    assert np.array_equal(fq, d_oq.download(np.int8, n * m)) and np.array_equal(bits(fs), bits(d_os.download(np.float32, n * (m // 32))))
    # the oracle on a few tokens: its own GEMV route, gate and quantizer (f32 sums in another order: a quant may differ by one
    # where a value sits on a rounding tie, never more)
    for j in (0, n // 2, n - 1):
        g = oracle.gemv_q8(dtype, wg, xs[j], xq[j], m, k)
        u = oracle.gemv_q8(dtype, wu, xs[j], xq[j], m, k)
        rs, rq = oracle.quantize_q8_0_batch(L.silu_mul(g, u), 1, m)
        got = fq.reshape(n, m)[j].astype(np.int32)
        assert np.abs(got - rq.reshape(-1).astype(np.int32)).max() <= 1 and np.allclose(fs.reshape(n, m // 32)[j], rs.reshape(-1), rtol=2e-3)
    assert not ops.ffn_gate_up_silu_quantize_applies(d_wg, d_wu, 64)
    with pytest.raises(W.RocmError, match="ffn_gate_up_silu_quantize"):
        ops.encode_ffn_gate_up_silu_quantize(d_wg, d_wu, d_xs, d_xq, 64, d_oq, d_os)
    for b in (d_xq, d_xs, d_oq, d_os, d_g, d_u):
        b.free()
    d_wg.free(), d_wu.free()
