"""The Model-trait methods around the decode / prompt step on the GPU: the n_keep context shift (wick/src/kv_cache.rs:601-700,
wick/src/model/lfm2.rs:2507-2516), state snapshots (wick/src/model/metal_lfm2.rs:2535-2634) and the embedding-input steps
(wick/src/model/lfm2.rs:2295-2349, 2452-2487), each against the oracle's restatement of the reference's CPU model."""
import numpy as np
import pytest

import wick_amd as W
from conftest import rel_l2
from oracle import lfm2_oracle as L
from test_gpu_lfm2_model import CLEAR, check_step, load
from wick_amd.lfm2 import Lfm2Ops, rope_theta_scale

pytestmark = pytest.mark.gpu


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def _rope_head(head, pos, hd, base):
    return L.rope(head, np.zeros(hd, np.float32), pos, 1, 1, hd, base)[0]


# ---- the shift of one layer's caches -------------------------------------------------------------

@pytest.mark.parametrize("seq,n_keep,shift,n_kv,hd,base", [
    (24, 5, 7, 4, 16, 10_000.0), (24, 5, 7, 2, 16, 10_000.0),  # the reference's own case (wick/tests/n_keep_shift.rs:138-146)
    (300, 32, 100, 8, 64, 1_000_000.0), (300, 0, 1, 8, 64, 1_000_000.0), (4096, 32, 2032, 8, 64, 1_000_000.0),
    (50, 3, 40, 1, 256, 10_000.0), (9, 0, 8, 3, 2, 10_000.0), (77, 70, 3, 2, 96, 500_000.0), (20, 4, 16, 2, 32, 10_000.0)])
def test_kv_shift_of_one_layer(ctx, oracle, seq, n_keep, shift, n_kv, hd, base):
    ops = Lfm2Ops(ctx)
    kvd, rows = n_kv * hd, seq + 3  # three rows past seq_len: must stay as they are
    k = oracle.fill_normal(seq + shift, 1.0, rows * kvd)
    v = oracle.fill_normal(seq + 2 * shift, 1.0, rows * kvd)
    d_k, d_v = ctx.to_device(k), ctx.to_device(v)
    n_scratch = ops.kv_shift_scratch_floats(seq, n_keep, shift, n_kv, hd)
    assert n_scratch == 2 * (seq - n_keep - shift) * kvd
    d_s = ctx.alloc(max(n_scratch, 1) * 4)
    ops.encode_kv_shift(d_k, d_v, d_s if n_scratch else None, seq, n_keep, shift, n_kv, hd, rope_theta_scale(hd, base))
    got_k, got_v = d_k.download(np.float32, rows * kvd), d_v.download(np.float32, rows * kvd)
    want_k, want_v = L.shift_kv(k, v, seq, n_keep, shift, n_kv, hd, base)
    assert np.array_equal(bits(got_v), bits(want_v))  # values only move
    new_len = seq - shift
    keep = np.r_[0:n_keep * kvd, new_len * kvd:rows * kvd]  # rows in front of the drop and everything from the new length on
    assert np.array_equal(bits(got_k[keep]), bits(want_k[keep])) and np.array_equal(bits(got_k[:n_keep * kvd]), bits(k[:n_keep * kvd]))
    moved = slice(n_keep * kvd, new_len * kvd)
    # same f32 angles and the same four roundings per pair; sin / cos come from the device library (an ulp or two from libm's)
    if new_len > n_keep:
        assert np.abs(got_k[moved] - want_k[moved]).max() <= 1e-6 * float(np.abs(k).max())
        assert rel_l2(got_k[moved], want_k[moved]) <= 1e-6
    for b in (d_k, d_v, d_s):
        b.free()


def test_kv_shift_reference_closed_form_and_errors(ctx, oracle):
    """Caches filled with raw heads rotated for their row: after the shift every moved key equals a fresh rotation for its new row
    (wick/tests/n_keep_shift.rs:138-236, bound 1e-3 there), kept rows byte-identical, value rows keep their identity."""
    ops = Lfm2Ops(ctx)
    hd, base, seq, n_keep, shift = 16, 10_000.0, 24, 5, 7
    for layer, n_kv in enumerate((4, 2)):
        kvd = n_kv * hd
        raw = np.array([[layer + 0.1 * h + 0.01 * d for d in range(hd)] for h in range(n_kv)], np.float32)
        k = np.stack([np.concatenate([_rope_head(raw[h], t, hd, base) for h in range(n_kv)]) for t in range(seq)])
        v = np.stack([(raw + np.float32(0.001) * np.float32(t)).astype(np.float32).ravel() for t in range(seq)])
        d_k, d_v, d_s = ctx.to_device(k.ravel()), ctx.to_device(v.ravel()), ctx.alloc(2 * seq * kvd * 4)
        ops.encode_kv_shift(d_k, d_v, d_s, seq, n_keep, shift, n_kv, hd, rope_theta_scale(hd, base))
        k2, v2 = d_k.download(np.float32, seq * kvd).reshape(seq, kvd), d_v.download(np.float32, seq * kvd).reshape(seq, kvd)
        assert np.array_equal(bits(k2[:n_keep]), bits(k[:n_keep]))
        for t_new in range(n_keep, seq - shift):
            fresh = np.concatenate([_rope_head(raw[h], t_new, hd, base) for h in range(n_kv)])
            assert np.abs(k2[t_new] - fresh).max() < 1e-3
            assert np.array_equal(bits(v2[t_new]), bits(v[t_new + shift]))
        with pytest.raises(W.RocmError, match="shift must be > 0"):
            ops.encode_kv_shift(d_k, d_v, d_s, seq, n_keep, 0, n_kv, hd, 0.5)
        with pytest.raises(W.RocmError, match="out of bounds"):
            ops.encode_kv_shift(d_k, d_v, d_s, seq, 20, 5, n_kv, hd, 0.5)
        with pytest.raises(W.RocmError, match="head_dim"):
            ops.encode_kv_shift(d_k, d_v, d_s, seq, n_keep, shift, n_kv, 15, 0.5)
        with pytest.raises(W.RocmError, match="scratch"):
            ops.encode_kv_shift(d_k, d_v, None, seq, n_keep, shift, n_kv, hd, 0.5)
        for b in (d_k, d_v, d_s):
            b.free()


# ---- the model ------------------------------------------------------------------------------------

@pytest.mark.parametrize("name,n,n_keep,shift", [("q4_0+q6k", 20, 4, 6), ("kernel4", 30, 0, 11), ("3-layer-q4embd", 25, 8, 17), ("q8_0", 12, 2, 1)])
def test_shift_kv_then_decode(ctx, oracle, tmp_path, name, n, n_keep, shift):
    """Prompt, shift, then single steps at the shifted positions: the GPU state follows the oracle's through the shift
    (Session::append_tokens' overflow sequence, wick/tests/n_keep_shift.rs:238-330)."""
    model, ref, cfg = load(ctx, oracle, tmp_path, **CLEAR[name])
    tokens = np.random.default_rng(n + shift).integers(0, cfg["vocab_size"], n + 4)
    state = ref.new_state()
    for pos in range(n):
        want = ref.forward(int(tokens[pos]), pos, state)
    got = model.forward_prefill(tokens[:n], 0)
    check_step(got, want, ref.min_margin, f"{name}: prompt")
    ref.shift_kv(state, n_keep, shift)
    assert model.shift_kv(n, n_keep, shift) == n - shift == state["seq_len"]
    for j in range(4):
        pos = n - shift + j
        check_step(model.forward(int(tokens[n + j]), pos), ref.forward(int(tokens[n + j]), pos, state), ref.min_margin, f"{name}: step {j} after the shift")
    with pytest.raises(W.RocmError, match="shift must be > 0"):
        model.shift_kv(10, 2, 0)
    with pytest.raises(W.RocmError, match="out of bounds"):
        model.shift_kv(10, 6, 5)
    with pytest.raises(W.RocmError, match="out of bounds"):
        model.shift_kv(65, 1, 1)  # beyond the context of 64
    model.free()


def test_shift_that_drops_everything_behind_n_keep(ctx, oracle, tmp_path):
    """cur_len == n_keep + shift: nothing to move (the boundary case of wick/src/model/metal_lfm2.rs:2499-2508)."""
    model, ref, cfg = load(ctx, oracle, tmp_path, **CLEAR["q4_0+q6k"])
    state = ref.new_state()
    tokens = [7, 19, 3, 200, 41, 5]
    for pos, t in enumerate(tokens):
        want = ref.forward(t, pos, state)
        got = model.forward(t, pos)
    check_step(got, want, ref.min_margin, "before the shift")
    ref.shift_kv(state, 2, 4)
    assert model.shift_kv(6, 2, 4) == 2
    check_step(model.forward(9, 2), ref.forward(9, 2, state), ref.min_margin, "after dropping the tail")
    model.free()


def test_snapshot_and_restore(ctx, oracle, tmp_path):
    """snapshot_state / restore_state: the steps after a restore repeat the steps after the snapshot bit for bit, in the same
    model and in a second one loaded from the same file; the bytes are the K / V rows and conv buffers in model order."""
    model, ref, cfg = load(ctx, oracle, tmp_path, **CLEAR["kernel4"])
    other, _, _ = load(ctx, oracle, tmp_path, **CLEAR["kernel4"])
    rng = np.random.default_rng(4)
    tokens = rng.integers(0, cfg["vocab_size"], 14)
    state = ref.new_state()
    model.forward_prefill(tokens[:10], 0)
    for pos in range(10):
        ref.forward(int(tokens[pos]), pos, state)
    snap = model.snapshot_state(10)
    hs, hd, kernel = cfg["hidden_size"], cfg["hidden_size"] // cfg["n_heads"], cfg["conv_kernel_size"]
    sizes = [model.layer_state_bytes(i, 10) for i in range(cfg["n_layers"])]
    assert sizes == [2 * 10 * n_kv * hd * 4 if n_kv else (kernel - 1) * hs * 4 for n_kv in cfg["kv_heads_per_layer"]]
    assert snap.size == sum(sizes)
    at = 0
    for i, n_kv in enumerate(cfg["kv_heads_per_layer"]):  # the pieces are what the oracle's state holds
        piece = snap[at:at + sizes[i]].view(np.float32)
        at += sizes[i]
        if n_kv:
            k, v = piece[:piece.size // 2], piece[piece.size // 2:]
            assert rel_l2(k, np.concatenate(state["layers"][i]["k"])) <= 1e-5 and rel_l2(v, np.concatenate(state["layers"][i]["v"])) <= 1e-5
        else:
            assert rel_l2(piece, state["layers"][i]["buf"]) <= 1e-5
    first = [model.forward(int(t), 10 + j) for j, t in enumerate(tokens[10:])]
    model.restore_state(snap, 10)
    again = [model.forward(int(t), 10 + j) for j, t in enumerate(tokens[10:])]
    other.forward_prefill(rng.integers(0, cfg["vocab_size"], 20), 0)  # some other history, overwritten by the restore
    other.restore_state(snap, 10)
    third = [other.forward(int(t), 10 + j) for j, t in enumerate(tokens[10:])]
    for a, b, c in zip(first, again, third):
        assert np.array_equal(bits(a), bits(b)) and np.array_equal(bits(a), bits(c))
    assert model.snapshot_state(0).size == sum(model.layer_state_bytes(i, 0) for i in range(cfg["n_layers"]))  # conv buffers only
    with pytest.raises(W.RocmError, match="exactly"):
        model.restore_state(snap[:-4], 10)
    with pytest.raises(W.RocmError, match="exactly"):
        model.restore_state(snap, 11)
    with pytest.raises(W.RocmError, match="beyond the context"):
        model.snapshot_state(65)
    model.free(), other.free()


@pytest.mark.parametrize("name", ["q4_0+q6k", "q8_0"])
def test_embedding_input_steps(ctx, oracle, tmp_path, name):
    """forward_from_embedding / forward_embedding / forward_hidden_from_embedding interleaved with token steps, each against the
    oracle running the same sequence (wick/src/model/lfm2.rs:2295-2349)."""
    model, ref, cfg = load(ctx, oracle, tmp_path, **CLEAR[name])
    hs = cfg["hidden_size"]
    gt, dims, data = ref.t["token_embd.weight"]
    # a token's own embedding row as the input vector is the token step itself
    row = L.embed_row(gt, data, 5, dims[0])
    a = model.forward(5, 0)
    model.reset()
    b = model.forward_from_embedding(row, 0)
    assert np.array_equal(bits(a), bits(b))
    model.reset()
    state = ref.new_state()
    rng = np.random.default_rng(8)
    emb = [(0.05 * rng.standard_normal(hs)).astype(np.float32) for _ in range(3)]
    check_step(model.forward(17, 0), ref.forward(17, 0, state), ref.min_margin, "token step")
    got, want = model.forward_embedding(23, 1), ref.hidden_after_layers(23, 1, state)
    assert rel_l2(got, want) <= (1e-5 if ref.min_margin >= 3e-5 else 5e-2), "forward_embedding"
    check_step(model.forward_from_embedding(emb[0], 2), ref.forward_from_embedding(emb[0], 2, state), ref.min_margin, "forward_from_embedding")
    got, want = model.forward_hidden_from_embedding(emb[1], 3), ref.hidden_after_layers(None, 3, state, emb[1])
    assert rel_l2(got, want) <= (1e-5 if ref.min_margin >= 3e-5 else 5e-2), "forward_hidden_from_embedding"
    check_step(model.forward(99, 4), ref.forward(99, 4, state), ref.min_margin, "token step after the embedding steps")
    # replayed graphs and plain launches agree for the hidden-state step as well
    model.reset()
    h1 = [model.forward_embedding(t, p) for p, t in enumerate([4, 8])]
    model.reset()
    model.set_graph_replay(False)
    h2 = [model.forward_embedding(t, p) for p, t in enumerate([4, 8])]
    for x, y in zip(h1, h2):
        assert np.array_equal(bits(x), bits(y))
    with pytest.raises(ValueError):
        model.forward_from_embedding(np.zeros(hs - 1, np.float32), 0)
    with pytest.raises(W.RocmError, match="beyond the context"):
        model.forward_from_embedding(emb[2], 64)
    model.free()


@pytest.mark.parametrize("name,n", [("q4_0+q6k", 24), ("q8_0", 5), ("q4_0+q6k", 2), ("q8_0", 1)])
def test_prefill_from_embeddings(ctx, oracle, tmp_path, name, n):
    """forward_prefill_from_embeddings (wick/src/model/lfm2.rs:2452-2487): the tokens' own rows give the token prompt bit for bit;
    arbitrary frames follow the oracle's frame-by-frame forward_from_embedding (the trait's default, wick/src/model/mod.rs:241-268)."""
    model, ref, cfg = load(ctx, oracle, tmp_path, **CLEAR[name])
    hs = cfg["hidden_size"]
    gt, dims, data = ref.t["token_embd.weight"]
    tokens = np.random.default_rng(n).integers(0, cfg["vocab_size"], n)
    rows = np.stack([L.embed_row(gt, data, int(t), dims[0]) for t in tokens])
    a = model.forward_prefill(tokens, 0)
    model.reset()
    b = model.forward_prefill_from_embeddings(rows, 0)
    assert np.array_equal(bits(a), bits(b))
    model.reset()
    frames = (0.05 * np.random.default_rng(n + 1).standard_normal((n, hs))).astype(np.float32)
    state = ref.new_state()
    for j in range(n):
        want = ref.forward_from_embedding(frames[j], j, state)
    check_step(model.forward_prefill_from_embeddings(frames, 0), want, ref.min_margin, f"{name}: {n} frames")
    check_step(model.forward(3, n), ref.forward(3, n, state), ref.min_margin, f"{name}: step after the frames")
    with pytest.raises(W.RocmError, match="at least one frame"):
        model.forward_prefill_from_embeddings(np.zeros((0, hs), np.float32), 0)
    with pytest.raises(W.RocmError, match="beyond the context"):
        model.forward_prefill_from_embeddings(frames, 64 - n + 1)
    model.free()


def test_two_threads_share_one_context(ctx, oracle, tmp_path):
    """The context serialises its callers (the reference's infer_lock, wick/src/model/metal_lfm2.rs:254-267): a model stepping in one
    thread and another thread issuing matmuls and a second model's steps on the same context leave every result as it is when each runs
    alone -- nothing of one caller ends up in the other's captured step or scratch."""
    import threading
    model, ref, cfg = load(ctx, oracle, tmp_path, **CLEAR["q4_0+q6k"])
    other, _, _ = load(ctx, oracle, tmp_path, **CLEAR["q8_0"])
    tokens = np.random.default_rng(2).integers(0, cfg["vocab_size"], 24)
    m, k, n = 300, 1024, 40
    wb = oracle.synth_weight(W.Q4_0, m, k, seed=9)
    w = ctx.upload_weight(wb, W.Q4_0, m, k)
    x = oracle.fill_normal(3, 1.0, n * k)
    d_x, d_y = ctx.to_device(x), ctx.alloc(n * m * 4)

    def steps(mod):
        mod.reset()
        return [mod.forward(int(t), p) for p, t in enumerate(tokens)]

    def matmuls(reps):
        out = []
        for _ in range(reps):
            ctx.encode_gemm(w, d_x, 0, d_y, 0, n, k, m)
            out.append(d_y.download(np.float32, n * m))
        return out

    alone_a, alone_b, alone_mm = steps(model), steps(other), matmuls(1)[0]
    got, errors = {}, []

    def run(name, fn, *args):
        try:
            got[name] = fn(*args)
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((name, e))

    threads = [threading.Thread(target=run, args=("a", steps, model)), threading.Thread(target=run, args=("b", steps, other)),
               threading.Thread(target=run, args=("mm", matmuls, 30))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for name, alone in (("a", alone_a), ("b", alone_b)):
        for x1, x2 in zip(alone, got[name]):
            assert np.array_equal(bits(x1), bits(x2)), name
    for y in got["mm"]:
        assert np.array_equal(bits(y), bits(alone_mm))
    model.free(), other.free(), w.free(), d_x.free(), d_y.free()
