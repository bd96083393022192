"""One LFM2 decode step on the GPU (GGUF file -> model handle -> forward) against the oracle's restatement
of the reference's aarch64 CPU model (wick/src/model/lfm2.rs:1020-1124, 2258-2289) on seeded random models."""
import numpy as np
import pytest

import lfm2_synth
import wick_amd as W
from conftest import rel_l2
from oracle import lfm2_oracle as L
from wick_amd import gguf as G
from wick_amd.lfm2 import RocmLfm2Model

pytestmark = pytest.mark.gpu

# f32 tolerance of a whole step: every operation is within a few ulp of the oracle's, a 4..6-layer
# residual stream amplifies that to ~1e-6; 1e-5 rel-L2 is the bar of the matmul path itself.
LOGITS_REL_L2 = 1e-5


def load(ctx, oracle, tmp_path, context=64, **kw):
    img, cfg, tensors = lfm2_synth.build(oracle, **kw)
    path = tmp_path / "lfm2_synth.gguf"
    path.write_bytes(img)
    with G.GgufFile.open(str(path)) as g:
        model = RocmLfm2Model(ctx, g, context)
    return model, L.Lfm2Oracle(cfg, tensors), cfg


@pytest.mark.parametrize("kw", [
    dict(),                                                                              # Q4_0 body, Q6_K embedding (a shipped Q4_0 file)
    dict(wtype=W.Q8_0, embd_type=W.Q8_0, seed=2),
    dict(n_layers=6, hidden=512, inter=1024, n_heads=8, kv_heads=(0, 0, 4, 0, 8, 2), vocab=1000, embd_type=W.Q4_0, seed=3),
    dict(kernel=4, kv_heads=(2, 0, 0, 4), seed=4, rope_theta=10000.0, eps=1e-6),
    dict(mixed_qkv=True, seed=5),                                                        # Q/K Q4_0, V Q8_0: separate launches
], ids=["q4_0+q6k", "q8_0", "6-layer", "kernel4", "mixed-qkv"])
def test_forward_matches_the_oracle_step_by_step(ctx, oracle, tmp_path, kw):
    model, ref, cfg = load(ctx, oracle, tmp_path, **kw)
    assert model.kv_heads_per_layer == cfg["kv_heads_per_layer"]
    assert model.config["max_seq_len"] == 64 and model.config["n_kv_heads"] == max(cfg["kv_heads_per_layer"])
    state = ref.new_state()
    rng = np.random.default_rng(11)
    tokens = rng.integers(0, cfg["vocab_size"], 9)
    for pos, tok in enumerate(tokens):
        logits = model.forward(int(tok), pos)
        want = ref.forward(int(tok), pos, state)
        assert np.isfinite(logits).all()
        assert rel_l2(logits, want) <= LOGITS_REL_L2, f"pos {pos}: rel-L2 {rel_l2(logits, want):.2e}"
        assert int(np.argmax(logits)) == int(np.argmax(want))
    model.free()


def test_reset_starts_a_fresh_state(ctx, oracle, tmp_path):
    model, ref, cfg = load(ctx, oracle, tmp_path)
    first = [model.forward(t, p) for p, t in enumerate([5, 9, 200])]
    model.reset()
    again = [model.forward(t, p) for p, t in enumerate([5, 9, 200])]
    for a, b in zip(first, again):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    model.free()


def test_greedy_generation_stays_on_the_device(ctx, oracle, tmp_path):
    """forward_greedy == argmax(forward) with the reference's tie rule; n steps without a host round trip
    give the same tokens as n single steps."""
    model, ref, cfg = load(ctx, oracle, tmp_path, seed=7)
    state, tok, want = ref.new_state(), 17, []
    for pos in range(12):
        tok = L.argmax(ref.forward(tok, pos, state))
        want.append(tok)
    got = model.generate_greedy(17, 0, 12)
    assert got.tolist() == want
    model.reset()
    tok, single = 17, []
    for pos in range(12):
        tok = model.forward_greedy(tok, pos)
        single.append(tok)
    assert single == want
    # the two kinds of step interleave on one state: logits of the next position follow the greedy prefix
    logits = model.forward(want[-1], 12)
    assert rel_l2(logits, ref.forward(want[-1], 12, state)) <= LOGITS_REL_L2
    model.free()


def test_load_and_step_errors(ctx, oracle, tmp_path):
    model, ref, cfg = load(ctx, oracle, tmp_path, context=8, context_length=6)
    assert model.config["max_seq_len"] == 6  # min(context_size, lfm2.context_length), wick/src/model/lfm2.rs:121-125
    assert model.gpu_memory_bytes() > 0
    with pytest.raises(W.RocmError, match="token_id out of range"):
        model.forward(cfg["vocab_size"], 0)
    with pytest.raises(W.RocmError, match="beyond the context"):
        model.forward(1, 6)
    with pytest.raises(W.RocmError, match="beyond the context"):
        model.generate_greedy(1, 4, 3)
    model.free()
    img, _, _ = lfm2_synth.build(oracle)
    with G.GgufFile.from_bytes(img) as g:
        with pytest.raises(W.RocmError, match="context_size"):
            RocmLfm2Model(ctx, g, 0)
    # a file without the LFM2 metadata / tensors is refused with the missing name
    import gguf_writer as GW
    with G.GgufFile.from_bytes(GW.build([("general.architecture", GW.T_STRING, "llama")])[0]) as g:
        with pytest.raises(W.RocmError, match="missing lfm2.block_count"):
            RocmLfm2Model(ctx, g, 16)
