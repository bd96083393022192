"""The benchmark's large configurations under the same parity bar as the small shapes:

* the nine per-layer prefill call sites of an LFM2-1.2B-shaped layer at n = 4096 tokens, Q8_0 weights
  (wick/src/model/lfm2.rs:1262-1937: conv in/out proj, attention Q / K / V / O, FFN gate / up / down), through the
  f32 call-site entry point with the prompt pass's strides;
* the tied LM head, Q8_0 65536 x 2048, at n = 1, 4, 16, 64 tokens through BOTH kernels (multi-token GEMV and int8
  MFMA), i.e. on either side of the hand-off (wick/src/backend/cpu.rs:3146-3248 times this shape).

Outputs of these sizes are checked the way the full-size ffn_up shape is: an oracle row band over ALL tokens plus
scattered rows, GEMM column j == GEMV of column j, both output layouts bit-equal, and the raw i32 block dots of a
band bit-exact.
"""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity, rel_l2
from gpu_util import fetch_gemm

pytestmark = pytest.mark.gpu

HS, IS, KV = 2048, 6912, 512
N_TOKENS = 4096
# (site, m, k, y_stride of the prompt pass's token-major buffer the site writes into)
SITES = [
    ("conv_in_proj", 3 * HS, HS, 3 * HS),
    ("conv_out_proj", HS, HS, HS),
    ("attn_q", HS, HS, HS + 2 * KV),   # Q | K | V share one [n][q|k|v] row
    ("attn_k", KV, HS, HS + 2 * KV),
    ("attn_v", KV, HS, HS + 2 * KV),
    ("attn_o", HS, HS, HS),
    ("ffn_gate", IS, HS, IS),
    ("ffn_up", IS, HS, IS),
    ("ffn_down", HS, IS, HS),
]
_BB = {W.Q4_0: 18, W.Q8_0: 34}


def _band(m):
    """Rows the oracle checks: both ends (ragged last tile included) and a stride through the middle."""
    rows = np.concatenate([np.arange(0, min(24, m)), np.arange(max(m - 24, 0), m), np.arange(37, m, max(m // 16, 1))])
    return np.unique(rows)


def _sub_weight(wb, dtype, m, k, rows):
    per_row = (k // 32) * _BB[dtype]
    return np.ascontiguousarray(wb.reshape(m, per_row)[rows]).ravel()


class _Activations:
    """4096 x k f32 activations, quantized once by the device quantizer and checked bit for bit against the oracle."""

    cache = {}

    @classmethod
    def get(cls, ctx, oracle, k):
        if k not in cls.cache:
            n = N_TOKENS
            x = oracle.fill_normal(4000 + k, 1.0, n * k)
            s, q = oracle.quantize_q8_0_batch(x, n, k)
            d_x, d_q, d_s = ctx.to_device(x), ctx.alloc(n * k), ctx.alloc(n * (k // 32) * 4)
            ctx.quantize_q8_0(d_x, n, k, k, d_q, d_s)
            assert np.array_equal(d_q.download(np.int8, n * k).reshape(n, k), q), "device quants differ from the oracle"
            assert np.array_equal(d_s.download(np.float32, s.size).view(np.uint32), s.ravel().view(np.uint32)), "device scales differ"
            cls.cache[k] = (x, s, q, d_x, d_q, d_s)
        return cls.cache[k]


@pytest.mark.parametrize("site,m,k,y_stride", SITES, ids=[s[0] for s in SITES])
def test_prefill_sites_c4(ctx, oracle, site, m, k, y_stride):
    n, dtype = N_TOKENS, W.Q8_0
    x, s, q, d_x, d_q, d_s = _Activations.get(ctx, oracle, k)
    wb = oracle.synth_weight(dtype, m, k, seed=300 + len(site) + m)
    w = ctx.upload_weight(wb, dtype, m, k)
    col0 = {"attn_k": HS, "attn_v": HS + KV}.get(site, 0)  # K and V land behind Q in the shared row
    d_y = ctx.to_device(np.full(n * y_stride, -3.0, np.float32))
    # the literal call-site shape: f32 in (x_stride = k), f32 out at a byte offset, quantizer inside
    ctx.encode_gemm(w, d_x, 0, d_y, col0 * 4, n, k, y_stride)
    full = d_y.download(np.float32, n * y_stride).reshape(n, y_stride)
    y = full[:, col0:col0 + m].T
    assert np.isfinite(y).all()
    untouched = np.ones(y_stride, bool)
    untouched[col0:col0 + m] = False
    assert np.all(full[:, untouched] == -3.0), "columns outside the site's slice were written"
    rows = _band(m)
    assert_f32_parity(y[rows], oracle.gemm_q8(dtype, _sub_weight(wb, dtype, m, k, rows), s, q, len(rows), n, k), f"C4 {site} row band")
    # column j of the GEMM == the GEMV of column j (same kernel family the decode step uses)
    d_v = ctx.alloc(m * 4)
    for j in (0, 127, 128, 2047, 2048, 4095):
        ctx.gemv_with_preq(w, d_s.ptr + j * (k // 32) * 4, d_q.ptr + j * k, d_v)
        assert rel_l2(y[:, j], d_v.download(np.float32, m)) < 1e-6
    # both output layouts of the pre-quantized entry point agree bit for bit with the call-site result
    d_a = ctx.alloc(m * n * 4)
    ctx.gemm_preq(w, d_s, d_q, n, d_a, layout=W.LAYOUT_TOKEN_MAJOR)
    a = fetch_gemm(d_a, m, n, m, W.LAYOUT_TOKEN_MAJOR)
    assert np.array_equal(a.view(np.uint32), np.ascontiguousarray(y).view(np.uint32))
    ctx.gemm_preq(w, d_s, d_q, n, d_a, layout=W.LAYOUT_ROW_MAJOR)
    assert np.array_equal(fetch_gemm(d_a, m, n, n, W.LAYOUT_ROW_MAJOR).view(np.uint32), np.ascontiguousarray(a).view(np.uint32))
    # raw i32 block dots of a band (last 128-row tile x the last 160 tokens: ragged in neither, but past tile 31 of the token axis)
    br = np.arange(max(m - 128, 0), m)
    bt0, bn = n - 160, 160
    wband = ctx.upload_weight(_sub_weight(wb, dtype, m, k, br), dtype, len(br), k)
    d_d = ctx.alloc(bn * len(br) * (k // 32) * 4)
    ctx.block_dots_i32(wband, d_q.ptr + bt0 * k, bn, d_d)
    dots = d_d.download(np.int32, bn * len(br) * (k // 32)).reshape(bn, len(br), k // 32)
    assert np.array_equal(dots, oracle.block_dots_i32(dtype, _sub_weight(wb, dtype, m, k, br), q[bt0:], len(br), bn, k))
    for b in (d_y, d_v, d_a, d_d):
        b.free()
    w.free(), wband.free()


def test_prefill_qkv_in_one_launch_c4(ctx, oracle):
    """Q, K and V of the 1.2B-shaped layer at n = 4096 the way the prompt pass issues them: one launch over three
    weights into one [n][q|k|v] row, bit-identical to one launch per weight."""
    n, k, dtype = N_TOKENS, HS, W.Q8_0
    _, s, q, _, d_q, d_s = _Activations.get(ctx, oracle, k)
    ms = (HS, KV, KV)
    ws = [ctx.upload_weight(oracle.synth_weight(dtype, m, k, seed=700 + i), dtype, m, k) for i, m in enumerate(ms)]
    stride = sum(ms)
    d_a, d_b = ctx.alloc(n * stride * 4), ctx.alloc(n * stride * 4)
    offs = (0, HS, HS + KV)
    ctx.gemm_preq_multi(ws, d_s, d_q, n, [d_a.ptr + 4 * o for o in offs], stride, layout=W.LAYOUT_TOKEN_MAJOR)
    for w, o in zip(ws, offs):
        ctx.gemm_preq(w, d_s, d_q, n, d_b.ptr + 4 * o, y_stride=stride, layout=W.LAYOUT_TOKEN_MAJOR)
    a, b = d_a.download(np.uint32, n * stride), d_b.download(np.uint32, n * stride)
    assert np.array_equal(a, b)
    for w in ws:
        w.free()
    d_a.free(), d_b.free()


class _LmHead:
    cache = None

    @classmethod
    def get(cls, ctx, oracle):
        if cls.cache is None:
            m, k, dtype = 65536, 2048, W.Q8_0
            wb = oracle.synth_weight(dtype, m, k, seed=999)
            cls.cache = (wb, ctx.upload_weight(wb, dtype, m, k))
        return cls.cache


@pytest.mark.parametrize("route", ["gemv", "mfma"])
@pytest.mark.parametrize("n", [1, 4, 16, 64])
def test_lm_head_c5(ctx, oracle, n, route):
    """Q8_0 65536 x 2048 at n tokens through the multi-token GEMV (hand-off forced up) and through the int8-MFMA
    kernel (hand-off forced down to 1; n = 1 then runs the narrow MFMA tile on a single token column)."""
    m, k, dtype = 65536, 2048, W.Q8_0
    wb, w = _LmHead.get(ctx, oracle)
    x = oracle.fill_normal(50 + n, 1.0, n * k)
    s, q = oracle.quantize_q8_0_batch(x, n, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    d_y = ctx.to_device(np.full(n * m, -5.0, np.float32))
    ctx.set_gemm_min_n(1 << 30 if route == "gemv" else 1)
    try:
        ctx.gemm_preq(w, d_s, d_q, n, d_y, y_stride=m, layout=W.LAYOUT_TOKEN_MAJOR)
        y = fetch_gemm(d_y, m, n, m, W.LAYOUT_TOKEN_MAJOR)
        assert np.isfinite(y).all() and not np.any(y == -5.0)
        rows = _band(m)
        sub = _sub_weight(wb, dtype, m, k, rows)
        assert_f32_parity(y[rows], oracle.gemm_q8(dtype, sub, s, q, len(rows), n, k), f"C5 n={n} {route} row band")
        # every row against the f64 dequantize-and-dot of the oracle for the first and the last token
        for j in {0, n - 1}:
            ref = oracle.gemv_q8(dtype, wb, s[j], q[j], m, k)
            assert_f32_parity(y[:, j], ref, f"C5 n={n} {route} token {j}, all 65536 rows")
        # raw i32 block dots through the same route, on the last 256 rows (the ragged end of the row axis does not exist
        # here: 65536 = 512 tiles; the band covers the last two)
        br = np.arange(m - 256, m)
        wband = ctx.upload_weight(_sub_weight(wb, dtype, m, k, br), dtype, len(br), k)
        d_d = ctx.alloc(n * len(br) * (k // 32) * 4)
        ctx.block_dots_i32(wband, d_q, n, d_d)
        dots = d_d.download(np.int32, n * len(br) * (k // 32)).reshape(n, len(br), k // 32)
        assert np.array_equal(dots, oracle.block_dots_i32(dtype, _sub_weight(wb, dtype, m, k, br), q, len(br), n, k))
        wband.free(), d_d.free()
    finally:
        ctx.set_gemm_min_n(0)
    for b in (d_q, d_s, d_y):
        b.free()


def test_lm_head_routes_agree_c5(ctx, oracle):
    """Either side of the hand-off computes the same block dots and the same scaling; only the f32 summation order
    differs (lane tree vs per-block accumulation): n = 16 through both kernels within 1e-6."""
    m, k, n, dtype = 65536, 2048, 16, W.Q8_0
    wb, w = _LmHead.get(ctx, oracle)
    s, q = oracle.quantize_q8_0_batch(oracle.fill_normal(77, 1.0, n * k), n, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    d_a, d_b = ctx.alloc(n * m * 4), ctx.alloc(n * m * 4)
    try:
        ctx.set_gemm_min_n(1 << 30)
        ctx.gemm_preq(w, d_s, d_q, n, d_a, y_stride=m, layout=W.LAYOUT_TOKEN_MAJOR)
        ctx.set_gemm_min_n(1)
        ctx.gemm_preq(w, d_s, d_q, n, d_b, y_stride=m, layout=W.LAYOUT_TOKEN_MAJOR)
    finally:
        ctx.set_gemm_min_n(0)
    assert rel_l2(d_a.download(np.float32, n * m), d_b.download(np.float32, n * m)) < 1e-6
    for b in (d_q, d_s, d_a, d_b):
        b.free()


def test_free_cached_inputs(ctx):
    """Releases the device copies the tests above share (runs last in this file)."""
    for _, _, _, d_x, d_q, d_s in _Activations.cache.values():
        d_x.free(), d_q.free(), d_s.free()
    _Activations.cache.clear()
    if _LmHead.cache is not None:
        _LmHead.cache[1].free()
        _LmHead.cache = None
