"""A seeded, randomly initialised LFM2-shaped model as a GGUF image plus the same tensors for the
oracle (not collected by pytest).  Tensor names, metadata keys and shapes are the ones
Lfm2Model::from_gguf_with_id reads (wick/src/model/lfm2.rs:97-300)."""
import numpy as np

import gguf_writer as GW

F32, Q4_0, Q8_0, Q6_K = 0, 2, 8, 14


def build(oracle, n_layers=4, hidden=256, inter=512, n_heads=4, kv_heads=(0, 2, 0, 4), vocab=320, kernel=3, rope_theta=1_000_000.0,
          eps=1e-5, wtype=Q4_0, embd_type=Q6_K, seed=1, context_length=None, sigma=0.08, mixed_qkv=False):
    """Returns (gguf image bytes, cfg dict for the oracle, {name: (ggml_type, dims, array)})."""
    assert len(kv_heads) == n_layers
    rng = np.random.default_rng(seed)
    hd = hidden // n_heads
    tensors = {}
    counter = [seed * 1000]

    def quant(name, m, k, t):
        counter[0] += 1
        tensors[name] = (t, [k, m], oracle.synth_weight(t, m, k, counter[0], sigma))

    def f32(name, dims, center=1.0, spread=0.2):
        n = int(np.prod(dims))
        tensors[name] = (F32, list(dims), (center + spread * rng.standard_normal(n)).astype(np.float32))

    quant("token_embd.weight", vocab, hidden, embd_type)
    f32("token_embd_norm.weight", [hidden])
    for i, n_kv in enumerate(kv_heads):
        p = f"blk.{i}."
        f32(p + "attn_norm.weight", [hidden])
        f32(p + "ffn_norm.weight", [hidden])
        if n_kv:
            quant(p + "attn_q.weight", hidden, hidden, wtype)
            quant(p + "attn_k.weight", n_kv * hd, hidden, wtype)
            quant(p + "attn_v.weight", n_kv * hd, hidden, Q8_0 if mixed_qkv else wtype)
            quant(p + "attn_output.weight", hidden, hidden, wtype)
            f32(p + "attn_q_norm.weight", [hd])
            f32(p + "attn_k_norm.weight", [hd])
        else:
            quant(p + "shortconv.in_proj.weight", 3 * hidden, hidden, wtype)
            quant(p + "shortconv.out_proj.weight", hidden, hidden, wtype)
            f32(p + "shortconv.conv.weight", [kernel, hidden], center=0.0, spread=0.5)
        quant(p + "ffn_gate.weight", inter, hidden, wtype)
        quant(p + "ffn_up.weight", inter, hidden, wtype)
        quant(p + "ffn_down.weight", hidden, inter, wtype)
    meta = [
        ("general.architecture", GW.T_STRING, "lfm2"),
        ("lfm2.block_count", GW.T_U32, n_layers),
        ("lfm2.embedding_length", GW.T_U32, hidden),
        ("lfm2.feed_forward_length", GW.T_U32, inter),
        ("lfm2.attention.head_count", GW.T_U32, n_heads),
        ("lfm2.vocab_size", GW.T_U32, vocab),
        ("lfm2.rope.freq_base", GW.T_F32, rope_theta),
        ("lfm2.attention.layer_norm_rms_epsilon", GW.T_F32, eps),
        ("lfm2.shortconv.l_cache", GW.T_U32, kernel),
        ("lfm2.attention.head_count_kv", GW.T_ARRAY, (GW.T_I32, list(kv_heads))),
    ]
    if context_length is not None:
        meta.append(("lfm2.context_length", GW.T_U32, context_length))
    img, _ = GW.build(meta, [(n, d, t, a) for n, (t, d, a) in tensors.items()])
    cfg = {"n_layers": n_layers, "hidden_size": hidden, "intermediate_size": inter, "n_heads": n_heads, "vocab_size": vocab,
           "rope_theta": float(np.float32(rope_theta)), "rms_norm_eps": float(np.float32(eps)), "conv_kernel_size": kernel,
           "kv_heads_per_layer": list(kv_heads)}
    return img, cfg, tensors
