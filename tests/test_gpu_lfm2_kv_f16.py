"""The model handle with KV caches of f16 rows (wick_rocm_lfm2_load_kv, WICK_ROCM_KV_F16: the caches of the reference's GPU
models, wick/src/model/metal_lfm2.rs:4117-4247, 2906-3364) against the oracle running the same steps with every cached value
rounded to f16 when it is appended or shifted.

Rounding to f16 is one more discontinuity on top of the Q8_0 quantizer's: a key or value that the GPU computes one f32 ulp
away from the oracle's can land on the other side of an f16 rounding boundary and then differs by a whole f16 step (2^-11 of
the value).  The tests therefore read the GPU's caches back (snapshot_state) and compare them with the oracle's as f16 bit
patterns: while they are identical (and no activation came near a Q8_0 tie) the logits are held to the f32 bar, 1e-5 rel-L2;
a handful of one-step differences in the caches loosens the bar to what those can do."""
import numpy as np
import pytest

import lfm2_synth
import wick_amd as W
from conftest import rel_l2
from oracle import lfm2_oracle as L
from wick_amd import gguf as G
from wick_amd.lfm2 import RocmLfm2Model

pytestmark = pytest.mark.gpu

NEAR_TIE = 3e-5
STRICT, LOOSE = 1e-5, 5e-3


def load(ctx, oracle, tmp_path, context=64, kv_f16=True, **kw):
    img, cfg, tensors = lfm2_synth.build(oracle, **kw)
    path = tmp_path / "lfm2_synth.gguf"
    path.write_bytes(img)
    with G.GgufFile.open(str(path)) as g:
        model = RocmLfm2Model(ctx, g, context, kv_f16=kv_f16)
    return model, L.Lfm2Oracle(cfg, tensors, kv_f16=kv_f16), cfg


def cache_differences(model, ref_state, cfg, seq_len, conv_bar=1e-5, only_first_attention_layer=False):
    """(elements that differ, elements that differ by more than one f16 step, elements) between the GPU's f16 caches and the
    oracle's; conv buffers must agree to `conv_bar` (f32 rounding while nothing upstream has flipped).
    only_first_attention_layer: the one layer whose keys and values no earlier cache rounding has touched."""
    first = min(i for i, n in enumerate(cfg["kv_heads_per_layer"]) if n)
    snap = model.snapshot_state(seq_len)
    hd, off, differ, far, total = cfg["hidden_size"] // cfg["n_heads"], 0, 0, 0, 0
    for i, n_kv in enumerate(cfg["kv_heads_per_layer"]):
        nbytes = model.layer_state_bytes(i, seq_len)
        piece = snap[off:off + nbytes]
        off += nbytes
        if n_kv == 0:
            got = piece.view(np.float32)
            assert rel_l2(got, ref_state["layers"][i]["buf"]) <= conv_bar, f"conv buffer of layer {i}"
            continue
        if only_first_attention_layer and i != first:
            continue
        assert nbytes == 2 * seq_len * n_kv * hd * 2  # keys then values, two bytes per element
        got = piece.view(np.float16).reshape(2, seq_len * n_kv * hd)
        for j, key in enumerate(("k", "v")):
            want = np.concatenate(ref_state["layers"][i][key]).astype(np.float16)
            g, w = got[j].view(np.int16).astype(np.int32), want.view(np.int16).astype(np.int32)
            d = np.abs(g - w)
            differ, far, total = differ + int((d != 0).sum()), far + int((d > 1).sum()), total + d.size
    assert off == snap.size
    return differ, far, total


def clean_rows_of_first_attention_layer(model, ref_state, cfg, seq_len):
    """(token rows of the first attention layer whose keys and values equal the oracle's f16 values up to a few single-step
    differences, rows).  A row is off as a whole when a Q8_0 quant flipped upstream of it (the gated convolution in front mixes
    three tokens, so one flip can take three rows along): a few such rows are arithmetic, most rows off is a bug."""
    snap = model.snapshot_state(seq_len)
    hd, off = cfg["hidden_size"] // cfg["n_heads"], 0
    for i, n_kv in enumerate(cfg["kv_heads_per_layer"]):
        nbytes = model.layer_state_bytes(i, seq_len)
        if n_kv:
            got = snap[off:off + nbytes].view(np.float16).reshape(2, seq_len, n_kv * hd).view(np.int16).astype(np.int32)
            clean = np.ones(seq_len, bool)
            for j, key in enumerate(("k", "v")):
                want = np.stack(ref_state["layers"][i][key][:seq_len]).astype(np.float16).view(np.int16).astype(np.int32)
                d = np.abs(got[j] - want)
                clean &= ((d > 1).sum(axis=1) == 0) & ((d == 1).sum(axis=1) <= max(2, d.shape[1] // 50))
            return int(clean.sum()), seq_len
        off += nbytes
    raise AssertionError("no attention layer")


def cosine(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))


def check(logits, want, caches_equal, margin, what):
    assert np.isfinite(logits).all(), what
    err = rel_l2(logits, want)
    if caches_equal and margin >= NEAR_TIE:
        assert err <= STRICT, f"{what}: rel-L2 {err:.2e} with identical f16 caches"
        return True
    assert err <= LOOSE, f"{what}: rel-L2 {err:.2e}"
    return False


def test_f16_caches_halve_the_state_and_steps_match_the_oracle(ctx, oracle, tmp_path):
    kw = dict(hidden=256, inter=256, vocab=256, seed=16)
    model, ref, cfg = load(ctx, oracle, tmp_path, **kw)
    m32, _, _ = load(ctx, oracle, tmp_path, kv_f16=False, **kw)
    assert model.kv_f16 and not m32.kv_f16
    attn_layers = [i for i, n in enumerate(cfg["kv_heads_per_layer"]) if n]
    for i in attn_layers:
        assert model.layer_state_bytes(i, 7) * 2 == m32.layer_state_bytes(i, 7)
    state = ref.new_state()
    # token seed 256: the first six steps of this model stay clear of Q8_0 ties with f16 caches (searched on the oracle alone;
    # the margin is re-checked below), the last four are whatever they are
    tokens = np.random.default_rng(256).integers(0, cfg["vocab_size"], 10)
    strict = 0
    for pos, tok in enumerate(tokens):
        logits, l32 = model.forward(int(tok), pos), m32.forward(int(tok), pos)
        want = ref.forward(int(tok), pos, state)
        differ, far, total = cache_differences(model, state, cfg, pos + 1, 1e-5 if ref.min_margin >= NEAR_TIE else 5e-2)
        assert far == 0 and differ <= max(2, total // 500), f"pos {pos}: {differ} of {total} cache elements differ ({far} by more than a step)"
        strict += check(logits, want, differ == 0, ref.min_margin, f"pos {pos}")
        if pos:  # the two cache types are different models from the second position on, and close ones
            assert not np.array_equal(logits, l32) and rel_l2(logits, l32) <= 0.1  # (a random model amplifies a flipped quant)
        if pos < 6:
            assert ref.min_margin >= NEAR_TIE, "this token seed no longer stays clear of quantizer ties: search another"
    assert strict >= 1  # (every later step is strict too until the first cache element lands on the other side of an f16 boundary)
    model.free(), m32.free()


@pytest.mark.parametrize("n_prompt", [5, 40, 300])
def test_f16_caches_prompt_then_steps(ctx, oracle, tmp_path, n_prompt):
    """Prompts through both batched attention kernels (the scalar one below 16 tokens, the matrix-core one without low halves
    from there on) against the oracle's token-by-token steps and against the model's own single steps.  Over a whole prompt
    some cached value always lands on the other side of an f16 boundary (and everything downstream of it then differs by more
    than a step), so the caches are compared where no earlier rounding has been: the first attention layer."""
    context = 64 if n_prompt < 60 else 512
    model, ref, cfg = load(ctx, oracle, tmp_path, context=context, hidden=256, inter=256, vocab=256, seed=16)
    state = ref.new_state()
    tokens = np.random.default_rng(n_prompt).integers(0, cfg["vocab_size"], n_prompt + 3)
    want = None
    for pos in range(n_prompt):
        want = ref.forward(int(tokens[pos]), pos, state)
    logits = model.forward_prefill(tokens[:n_prompt], 0)
    # a prompt pass sums its projections in the GEMM's order, a step in the GEMV's: an f32 ulp apart in front of the cache rounding;
    # a Q8_0 quant that flips in the first layer moves that token's keys by a few f16 steps
    clean, rows = clean_rows_of_first_attention_layer(model, state, cfg, n_prompt)
    assert clean >= rows - max(3, rows // 10), f"only {clean} of {rows} cache rows match the oracle's f16 values"
    assert np.isfinite(logits).all() and rel_l2(logits, want) <= 5e-2 and cosine(logits, want) >= 0.999, f"prompt logits rel-L2 {rel_l2(logits, want):.2e}"
    for pos in range(n_prompt, n_prompt + 3):
        got, want = model.forward(int(tokens[pos]), pos), ref.forward(int(tokens[pos]), pos, state)
        assert np.isfinite(got).all() and rel_l2(got, want) <= 5e-2 and cosine(got, want) >= 0.999, f"step {pos}: rel-L2 {rel_l2(got, want):.2e}"
    # the prompt pass against the same model's single steps
    model.reset()
    single = None
    for pos in range(n_prompt):
        single = model.forward(int(tokens[pos]), pos)
    assert cosine(logits, single) >= 0.999 and rel_l2(logits, single) <= 5e-2
    model.free()


def test_f16_caches_context_shift_and_restore(ctx, oracle, tmp_path):
    model, ref, cfg = load(ctx, oracle, tmp_path, hidden=256, inter=256, vocab=256, seed=16)
    state = ref.new_state()
    tokens = np.random.default_rng(9).integers(0, cfg["vocab_size"], 20)
    for pos in range(12):
        model.forward(int(tokens[pos]), pos), ref.forward(int(tokens[pos]), pos, state)
    snap = model.snapshot_state(12)
    new_len = model.shift_kv(12, 2, 5)
    ref.shift_kv(state, 2, 5)
    assert new_len == 7 == state["seq_len"]
    differ, far, total = cache_differences(model, state, cfg, 7, 0.1, only_first_attention_layer=True)
    assert differ <= total // 4 and far <= total // 10  # rotated keys: device sin / cos, then the f16 rounding
    got, want = model.forward(int(tokens[12]), 7), ref.forward(int(tokens[12]), 7, state)
    assert rel_l2(got, want) <= 5e-2 and cosine(got, want) >= 0.999
    # back to the snapshot: the same step as before the shift, bit for bit
    model.restore_state(snap, 12)
    a = model.forward(int(tokens[12]), 12)
    model.restore_state(snap, 12)
    b = model.forward(int(tokens[12]), 12)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    model.free()


def test_f16_caches_with_a_head_dim_without_fused_kernels(ctx, oracle, tmp_path):
    """head_dim 48: QK-norm + RoPE + append, the one-workgroup decode attention and (for prompts) the same kernel token by token,
    all over f16 rows."""
    kw = dict(hidden=384, inter=256, n_heads=8, kv_heads=(0, 4, 0, 8), vocab=256, embd_type=W.Q4_0, seed=4)
    model, ref, cfg = load(ctx, oracle, tmp_path, **kw)
    state = ref.new_state()
    tokens = np.random.default_rng(3).integers(0, cfg["vocab_size"], 8)
    for pos, tok in enumerate(tokens[:5]):
        got, want = model.forward(int(tok), pos), ref.forward(int(tok), pos, state)
        clean, rows = clean_rows_of_first_attention_layer(model, state, cfg, pos + 1)
        assert clean >= rows - 2
        check(got, want, False, ref.min_margin, f"head_dim 48, pos {pos}")
    model.reset()
    state = ref.new_state()
    want = None
    for pos, tok in enumerate(tokens):
        want = ref.forward(int(tok), pos, state)
    got = model.forward_prefill(tokens, 0)
    assert np.isfinite(got).all() and rel_l2(got, want) <= 5e-2 and cosine(got, want) >= 0.999
    model.free()


def test_bad_kv_dtype_is_refused(ctx, oracle, tmp_path):
    import ctypes as C

    from wick_amd import lfm2 as M

    img, _, _ = lfm2_synth.build(oracle, hidden=256, inter=256, vocab=256, seed=16)
    path = tmp_path / "m.gguf"
    path.write_bytes(img)
    with G.GgufFile.open(str(path)) as g:
        h = C.c_void_p()
        assert M._lib().wick_rocm_lfm2_load_kv(ctx._h, g.handle, 64, 7, C.byref(h)) == -1 and not h.value
