"""Pins oracle/wick_oracle_ops.c: the reference's own known-answer tests for these operations
(wick/src/backend/cpu.rs:2278-2391, 2751-2810, 2905-3010) plus what the mathematics fixes
(float64 restatements, closed forms, invariants).  Runs without a GPU."""
import numpy as np
import pytest

from oracle import lfm2_oracle as L


def ulp_diff(a, b):
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    return np.abs(a - b)


def test_ggml_expf_reference_values_and_sweep():
    for x in [0.0, 1.0, -1.0, 2.0, -5.0, -10.0, -50.0, 80.0]:  # cpu.rs:2751-2766
        got, exp = L.ggml_expf(x), float(np.exp(np.float64(x)))
        assert abs(got - exp) / exp < 1e-5
    assert L.ggml_expf(0.0) == 1.0
    assert np.isinf(L.ggml_expf(100.0)) and L.ggml_expf(-200.0) == 0.0  # cpu.rs:2768-2769
    xs = np.linspace(-87.0, 88.0, 20001, dtype=np.float32)
    got = np.array([L.ggml_expf(float(x)) for x in xs], np.float32)
    ref = np.exp(xs.astype(np.float64)).astype(np.float32)
    assert ulp_diff(got, ref).max() <= 2  # "1.45358 + 0.5 ULPs", cpu.rs:599
    # the two range branches (|n| in (126, 192] and beyond)
    for x in [-90.0, -100.0, -103.0, 88.5]:
        got, exp = L.ggml_expf(x), float(np.exp(np.float64(x)))
        assert abs(got - exp) <= 1e-5 * exp + 1e-45
    assert L.ggml_expf(-140.0) == 0.0 and np.isinf(L.ggml_expf(140.0))


def test_rmsnorm_closed_forms():
    eps = 1e-5
    got = L.rmsnorm([1.0, 2.0, 3.0, 4.0], [1.0] * 4, eps)  # cpu.rs:2278-2295
    assert np.allclose(got, np.array([1, 2, 3, 4]) / np.sqrt(7.5 + eps), atol=1e-6)
    got = L.rmsnorm([2.0, 2.0], [3.0, 0.5], eps)  # cpu.rs:2298-2315
    assert np.allclose(got, [2 * 3 / np.sqrt(4 + eps), 2 * 0.5 / np.sqrt(4 + eps)], atol=1e-6)
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal(1024).astype(np.float32), rng.standard_normal(1024).astype(np.float32)
    inv = np.float32(1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2) + np.float64(np.float32(eps))))
    assert np.array_equal(L.rmsnorm(x, w, eps), x * inv * w)  # same f64 sum order, same f32 products


def test_silu_mul_known_values():
    got = L.silu_mul([0.0, 1.0, -1.0, 5.0], [1.0, 1.0, 1.0, 1.0])  # cpu.rs:2318-2327
    assert abs(got[0]) < 1e-6 and abs(got[1] - 0.7311) < 1e-3 and abs(got[2] + 0.2689) < 1e-3 and abs(got[3] - 4.9665) < 1e-3
    rng = np.random.default_rng(1)
    g, u = (rng.standard_normal(4096) * 4).astype(np.float32), rng.standard_normal(4096).astype(np.float32)
    ref = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(L.silu_mul(g, u), ref, rtol=2e-6, atol=1e-7)


def test_softmax_known_values_and_stability():
    got = L.softmax([1.0, 2.0, 3.0])  # cpu.rs:2374-2391
    assert np.allclose(got, [0.0900, 0.2447, 0.6652], atol=1e-3) and abs(got.sum() - 1) < 1e-6
    got = L.softmax([1000.0, 1001.0, 1002.0])  # cpu.rs:2773-2780
    assert np.isfinite(got).all() and abs(got.sum() - 1) < 1e-6
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(777) * 3).astype(np.float32)
    e = np.exp(x.astype(np.float64) - x.max())
    assert np.allclose(L.softmax(x), e / e.sum(), rtol=3e-6, atol=1e-9)
    assert np.array_equal(L.softmax([5.0]), [1.0])


def test_rope_identity_closed_form_and_composition():
    q, k = np.array([1, 2, 3, 4], np.float32), np.array([5, 6, 7, 8], np.float32)
    q2, k2 = L.rope(q, k, 0, 1, 1, 4, 10000.0)  # cpu.rs:2783-2797
    assert np.array_equal(q2, q) and np.array_equal(k2, k)
    rng = np.random.default_rng(3)
    hd, nh, nkv, base = 64, 4, 2, 1_000_000.0
    q, k = rng.standard_normal(nh * hd).astype(np.float32), rng.standard_normal(nkv * hd).astype(np.float32)
    for pos in (1, 7, 100, 4000):
        q2, k2 = L.rope(q, k, pos, nh, nkv, hd, base)
        theta = pos * np.float64(base) ** (-2.0 * np.arange(hd // 2) / hd)
        for src, dst, n in ((q, q2, nh), (k, k2, nkv)):
            s = src.reshape(n, 2, hd // 2).astype(np.float64)
            ref = np.stack([s[:, 0] * np.cos(theta) - s[:, 1] * np.sin(theta), s[:, 0] * np.sin(theta) + s[:, 1] * np.cos(theta)], 1)
            # theta is multiplied up in f32 (cpu.rs:2150-2160): the angle error grows with pos
            assert np.allclose(dst.reshape(n, 2, hd // 2), ref, atol=2e-6 * max(pos, 8))
            pair_norm = lambda a: np.hypot(a.reshape(n, 2, hd // 2)[:, 0], a.reshape(n, 2, hd // 2)[:, 1])
            assert np.allclose(pair_norm(dst), pair_norm(src), rtol=1e-6)
    a, _ = L.rope(*L.rope(q, k, 5, nh, nkv, hd, base), 9, nh, nkv, hd, base)
    b, _ = L.rope(q, k, 14, nh, nkv, hd, base)
    assert np.allclose(a, b, atol=1e-5)
    assert L.rope_theta_scale(64, 1_000_000.0) == np.float32(np.float32(1_000_000.0) ** np.float32(-2.0 / 64))


def _rope_head(head, pos, hd, base):
    return L.rope(head, np.zeros(hd, np.float32), pos, 1, 1, hd, base)[0]


def test_rope_delta_on_the_reference_cases():
    hd, base = 64, 10_000.0  # wick/tests/n_keep_shift.rs:47-78: the same position pairs and head values
    raw = (np.arange(hd) * 0.01).astype(np.float32)
    for p_old in (0, 1, 7, 64, 2048):
        for p_new in (0, 1, 5, 63, 2000):
            via = L.rope_delta(_rope_head(raw, p_old, hd, base), p_new - p_old, hd, base)
            assert np.abs(via - _rope_head(raw, p_new, hd, base)).max() < 1e-3, (p_old, p_new)
    orig = (np.arange(32) * 0.1 + 1.0).astype(np.float32)  # wick/tests/n_keep_shift.rs:80-91
    assert np.abs(L.rope_delta(orig, 0, 32, base) - orig).max() < 1e-5
    assert np.array_equal(L.rope_delta(orig, 0, 32, base), orig)  # cos 0 = 1, sin 0 = 0 exactly
    # a non-negative delta walks the very same angles as a rotation for that position
    rng = np.random.default_rng(11)
    h = rng.standard_normal(hd).astype(np.float32)
    for d in (1, 5, 777):
        assert np.array_equal(L.rope_delta(h, d, hd, 1_000_000.0), _rope_head(h, d, hd, 1_000_000.0))
    # a negative delta is the inverse rotation: closed form in float64, and there-and-back returns the head
    for d in (-1, -7, -300):
        theta = d * np.float64(1_000_000.0) ** (-2.0 * np.arange(hd // 2) / hd)
        x = h.reshape(2, hd // 2).astype(np.float64)
        ref = np.concatenate([x[0] * np.cos(theta) - x[1] * np.sin(theta), x[0] * np.sin(theta) + x[1] * np.cos(theta)])
        assert np.allclose(L.rope_delta(h, d, hd, 1_000_000.0), ref, atol=2e-6 * max(-d, 8))
        assert np.allclose(L.rope_delta(L.rope_delta(h, d, hd, 1_000_000.0), -d, hd, 1_000_000.0), h, atol=1e-5)


def test_shift_kv_on_the_reference_case():
    hd, base, seq, n_keep, shift = 16, 10_000.0, 24, 5, 7  # wick/tests/n_keep_shift.rs:138-236
    for layer, n_kv in enumerate((4, 2)):
        kvd = n_kv * hd
        raw = np.array([[layer + 0.1 * h + 0.01 * d for d in range(hd)] for h in range(n_kv)], np.float32)
        k = np.stack([np.concatenate([_rope_head(raw[h], t, hd, base) for h in range(n_kv)]) for t in range(seq)])
        v = np.stack([(raw + np.float32(0.001) * np.float32(t)).astype(np.float32).ravel() for t in range(seq)])
        k2, v2 = L.shift_kv(k.ravel(), v.ravel(), seq, n_keep, shift, n_kv, hd, base)
        k2, v2 = k2.reshape(seq, kvd), v2.reshape(seq, kvd)
        assert np.array_equal(k2[:n_keep], k[:n_keep]) and np.array_equal(v2[:n_keep], v[:n_keep])  # kept rows untouched
        for t_new in range(n_keep, seq - shift):
            fresh = np.concatenate([_rope_head(raw[h], t_new, hd, base) for h in range(n_kv)])
            assert np.abs(k2[t_new] - fresh).max() < 1e-3
            assert np.array_equal(v2[t_new], v[t_new + shift])  # the row kept its identity
        # the row move itself, restated: keys are the old rows rotated back by `shift`
        for t_new in (n_keep, seq - shift - 1):
            for h in range(n_kv):
                assert np.array_equal(k2[t_new, h * hd:(h + 1) * hd], L.rope_delta(k[t_new + shift, h * hd:(h + 1) * hd], -shift, hd, base))
    # dropping everything behind n_keep leaves the kept rows and nothing to rotate
    k = np.arange(6 * 8, dtype=np.float32)
    k2, v2 = L.shift_kv(k, k + 1, 6, 2, 4, 1, 8, base)
    assert np.array_equal(k2[:16], k[:16]) and np.array_equal(v2[:16], k[:16] + 1)


def test_attention_helpers_on_the_reference_inputs():
    hd, kv_dim, seq = 64, 128, 10  # cpu.rs:2910-2925
    q = ((np.arange(hd) - 32.0) * 0.05).astype(np.float32)
    kc = (((np.arange(seq * kv_dim) * 7 + 3) % 31) * 0.04 - 0.6).astype(np.float32)
    got = L.attn_scores(q, kc, kv_dim, 64, hd, 1 / 8.0, seq)
    ref = kc.reshape(seq, kv_dim)[:, 64:128].astype(np.float64) @ q.astype(np.float64) / 8.0
    assert np.allclose(got, ref, atol=1e-5)
    sc = ((np.arange(seq) + 1.0) / seq).astype(np.float32)  # cpu.rs:2958-2970
    vc = (((np.arange(seq * kv_dim) * 11 + 5) % 29) * 0.03 - 0.4).astype(np.float32)
    got = L.attn_values(sc, vc, kv_dim, 0, hd, seq)
    assert np.allclose(got, sc.astype(np.float64) @ vc.reshape(seq, kv_dim)[:, :64].astype(np.float64), atol=1e-5)
    assert L.attn_scores(q, np.zeros(0, np.float32), 64, 0, 64, 0.125, 0).size == 0  # cpu.rs:3005-3010
    assert np.array_equal(L.attn_values(np.zeros(0, np.float32), np.zeros(0, np.float32), 64, 0, 64, 0), np.zeros(64, np.float32))
    # whole decode attention (GQA) against float64 softmax(QK^T)V
    rng = np.random.default_rng(4)
    nh, nkv, seq = 8, 2, 37
    qq = rng.standard_normal(nh * hd).astype(np.float32)
    kk, vv = rng.standard_normal((seq, nkv * hd)).astype(np.float32), rng.standard_normal((seq, nkv * hd)).astype(np.float32)
    got = L.attention(qq, kk, vv, nh, nkv, hd, seq).reshape(nh, hd)
    for h in range(nh):
        g = h // (nh // nkv)
        s = kk[:, g * hd:(g + 1) * hd].astype(np.float64) @ qq[h * hd:(h + 1) * hd].astype(np.float64) / 8.0
        p = np.exp(s - s.max())
        assert np.allclose(got[h], (p / p.sum()) @ vv[:, g * hd:(g + 1) * hd].astype(np.float64), atol=2e-6)


@pytest.mark.parametrize("kernel", [1, 2, 3, 4])
def test_shortconv_step_against_numpy(kernel):
    rng = np.random.default_rng(5 + kernel)
    hs, steps = 96, 6
    w = rng.standard_normal((hs, kernel)).astype(np.float32)
    buf = np.zeros((kernel - 1) * hs, np.float32)
    hist = [np.zeros(hs, np.float32)] * (kernel - 1)  # bx of the previous steps, oldest first
    for _ in range(steps):
        proj = rng.standard_normal(3 * hs).astype(np.float32)
        b, c, x = proj[:hs], proj[hs:2 * hs], proj[2 * hs:]
        bx = b * x
        taps = hist + [bx]
        s = np.zeros(hs, np.float32)
        for kk in range(kernel):
            s = s + taps[kk] * w[:, kk]
        out = L.shortconv_step(proj, buf, w.ravel(), hs, kernel)
        assert np.array_equal(out, c * s)
        hist = (hist + [bx])[1:] if kernel > 1 else []
        if kernel > 1:
            assert np.array_equal(buf.reshape(kernel - 1, hs), np.stack(hist))
    # identity kernel (only the newest tap): out = c * b * x
    proj = rng.standard_normal(3 * hs).astype(np.float32)
    ident = np.zeros((hs, kernel), np.float32)
    ident[:, kernel - 1] = 1
    out = L.shortconv_step(proj, np.ones((kernel - 1) * hs, np.float32), ident.ravel(), hs, kernel)
    assert np.array_equal(out, proj[hs:2 * hs] * (proj[:hs] * proj[2 * hs:]))


def test_argmax_keeps_the_last_maximum():
    """cpu_argmax (wick/src/sampler.rs:7-19): Iterator::max_by returns the last of equal maxima,
    NaN counts as -inf, total_cmp orders -0.0 below +0.0."""
    assert L.argmax([1.0, 3.0, 2.0]) == 1
    assert L.argmax([3.0, 1.0, 3.0, 2.0]) == 2
    assert L.argmax([np.nan, 1.0, np.nan]) == 1
    assert L.argmax([np.nan, np.nan]) == 1 and L.argmax([np.nan, -np.inf]) == 1
    assert L.argmax([0.0, -0.0]) == 0 and L.argmax([-0.0, 0.0, -0.0]) == 1
    assert L.argmax([]) == 0
    rng = np.random.default_rng(6)
    for _ in range(50):
        x = rng.integers(-3, 4, 200).astype(np.float32)
        assert L.argmax(x) == 199 - int(np.argmax(x[::-1]))
