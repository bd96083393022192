"""GGUF file -> device weight -> GEMV: the loader hands the kernels the same bytes, m and k
an explicit upload would (resolve_weight, wick/src/model/lfm2.rs:310-338)."""
import numpy as np
import pytest

import gguf_writer as GW
import wick_amd as W
from conftest import assert_f32_parity
from wick_amd import gguf as G

pytestmark = pytest.mark.gpu


def test_weights_from_a_gguf_file(ctx, oracle, tmp_path):
    k = 1024
    shapes = {"blk.0.attn_q.weight": (W.Q4_0, 300), "blk.0.ffn_down.weight": (W.Q8_0, 130), "token_embd.weight": (W.Q6_K, 515)}
    blobs = {name: oracle.synth_weight(t, m, k, seed=m) for name, (t, m) in shapes.items()}
    tensors = [(name, [k, m], t, blobs[name]) for name, (t, m) in shapes.items()]
    tensors.append(("blk.0.attn_norm.weight", [k], 0, np.ones(k, np.float32)))
    img, _ = GW.build([("general.architecture", GW.T_STRING, "lfm2")], tensors)
    path = tmp_path / "synthetic.gguf"
    path.write_bytes(img)

    x = oracle.fill_normal(11, 1.0, k)
    s, q = oracle.quantize_q8_0_batch(x, 1, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    with G.GgufFile.open(str(path)) as g:
        for name, (t, m) in shapes.items():
            w = ctx.weight_from_gguf(g, name)
            assert (w.dtype, w.m, w.k, w.nbytes) == (t, m, k, blobs[name].nbytes)
            d_y = ctx.alloc(m * 4)
            ctx.gemv_with_preq(w, d_s, d_q, d_y)
            ref = oracle.gemv_q6k_q8(blobs[name], s[0], q[0], m, k) if t == W.Q6_K else oracle.gemv_q8(t, blobs[name], s[0], q[0], m, k)
            assert_f32_parity(d_y.download(np.float32, m), ref, name)
            d_y.free(), w.free()
        # an f32 norm vector is a valid tensor but not a matmul weight; a missing name is an error too
        with pytest.raises(W.RocmError, match="Q4_0"):
            ctx.weight_from_gguf(g, "blk.0.attn_norm.weight")
        with pytest.raises(W.RocmError, match="tensor not found"):
            ctx.weight_from_gguf(g, "blk.9.attn_q.weight")
    d_q.free(), d_s.free()
