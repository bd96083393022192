"""Host mirror of ``include/wick_rocm_lfm2.h``: the decode step's non-matmul operations under the
names of the reference's encoder call sites (wick/src/model/metal_lfm2.rs:1380-1990), and the LFM2
model handle with ``forward`` / ``forward_greedy`` of ``trait Model`` (wick/src/model/mod.rs:72-323).
Test / bench plumbing over ctypes, like ``wick_amd.rocm``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import numpy as np

from . import rocm
from .rocm import RocmContext, RocmWeight, _ptr

_P = C.c_void_p
_U32, _F = C.c_uint32, C.c_float


class Lfm2Config(C.Structure):
    """wick_rocm_lfm2_config (ModelConfig, wick/src/model/mod.rs:27-46)."""
    _fields_ = [(n, _U32) for n in ("n_layers", "hidden_size", "intermediate_size", "n_heads", "n_kv_heads", "vocab_size", "max_seq_len",
                                    "conv_kernel_size")] + [("rope_theta", _F), ("rms_norm_eps", _F)]


_SIGNATURES = {
    "wick_rocm_embed_row": (C.c_int, [_P, _P, _U32, _P, _P]),
    "wick_rocm_rmsnorm": (C.c_int, [_P, _P, _P, _P, _U32, _U32, _U32, _U32, _F]),
    "wick_rocm_qk_norm_rope": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _U32, _P, _U32, _U32, _U32, _U32, _F, _F]),
    "wick_rocm_attention_prefill_quantize_q8_0": (C.c_int, [_P, _P, _U32, _P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _U32]),
    "wick_rocm_shortconv_seq": (C.c_int, [_P, _P, _P, _P, _P, _U32, _U32, _U32]),
    "wick_rocm_shortconv_seq_quantize_q8_0": (C.c_int, [_P, _P, _P, _P, _P, _P, _U32, _U32, _U32]),
    "wick_rocm_ffn_gate_up_silu_quantize_applies": (C.c_int, [_P, _P, _U32]),
    "wick_rocm_ffn_gate_up_silu_quantize_q8": (C.c_int, [_P, _P, _P, _P, _P, _U32, _P, _P]),
    "wick_rocm_qk_norm_rope_tokens": (C.c_int, [_P, _P, _U32, _P, _P, _U32, _P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _U32, _F, _F]),
    "wick_rocm_rope_theta_scale": (_F, [_U32, _F]),
    "wick_rocm_attention_decode": (C.c_int, [_P, _P, _P, _P, _P, _P, _U32, _P, _U32, _U32, _U32, _U32]),
    "wick_rocm_attention_scratch_floats": (C.c_size_t, [_U32, _U32, _U32]),
    "wick_rocm_attention_prefill": (C.c_int, [_P, _P, _U32, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _U32, _U32]),
    "wick_rocm_attention_block_scratch_bytes": (C.c_size_t, [_U32, _U32, _U32]),
    "wick_rocm_attention_block": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _U32, _P, _U32, _U32, _U32, _U32, _F, _F]),
    "wick_rocm_shortconv_step": (C.c_int, [_P, _P, _P, _P, _P, _U32, _U32]),
    "wick_rocm_silu_mul": (C.c_int, [_P, _P, _P, _U32]),
    "wick_rocm_argmax": (C.c_int, [_P, _P, _U32, _P, _P, _P]),
    "wick_rocm_lm_head_greedy_f32": (C.c_int, [_P, _P, _P, _P, _F, _P, _P, _P, _P]),
    "wick_rocm_rmsnorm_quantize_q8_0": (C.c_int, [_P, _P, _P, _U32, _U32, _U32, _F, _P, _P]),
    "wick_rocm_silu_mul_quantize_q8_0": (C.c_int, [_P, _P, _P, _U32, _U32, _P, _P]),
    "wick_rocm_lfm2_load": (C.c_int, [_P, _P, _U32, C.POINTER(_P)]),
    "wick_rocm_lfm2_load_kv": (C.c_int, [_P, _P, _U32, C.c_int, C.POINTER(_P)]),
    "wick_rocm_lfm2_kv_dtype": (C.c_int, [_P]),
    "wick_rocm_lfm2_free": (C.c_int, [_P, _P]),
    "wick_rocm_lfm2_get_config": (C.c_int, [_P, C.POINTER(Lfm2Config)]),
    "wick_rocm_lfm2_layer_kv_heads": (C.c_int, [_P, _U32, C.POINTER(_U32)]),
    "wick_rocm_lfm2_gpu_memory_bytes": (C.c_size_t, [_P]),
    "wick_rocm_lfm2_reset": (C.c_int, [_P, _P]),
    "wick_rocm_shortconv_fusable": (C.c_int, [_P, _P, _P, _U32]),
    "wick_rocm_shortconv_out_proj_f32": (C.c_int, [_P, _P, _P, _P, _P, _U32, _P, C.c_int]),
    "wick_rocm_ffn_gate_up_conv_advance_f32": (C.c_int, [_P, _P, _P, _P, _P, C.c_float, _P, _P, _P, _U32, _U32]),
    "wick_rocm_lfm2_set_graph_replay": (C.c_int, [_P, C.c_int]),
    "wick_rocm_lfm2_forward": (C.c_int, [_P, _P, _U32, _U32, _P]),
    "wick_rocm_lfm2_forward_prefill": (C.c_int, [_P, _P, _P, _U32, _U32, _P]),
    "wick_rocm_lfm2_forward_prefill_chunked": (C.c_int, [_P, _P, _P, _U32, _U32, _U32, _P, C.POINTER(_U32), _P]),
    "wick_rocm_lfm2_forward_greedy": (C.c_int, [_P, _P, _U32, _U32, C.POINTER(_U32)]),
    "wick_rocm_lfm2_generate_greedy": (C.c_int, [_P, _P, _U32, _U32, _U32, _P]),
    "wick_rocm_lfm2_logits_device": (_P, [_P]),
    "wick_rocm_kv_shift_scratch_floats": (C.c_size_t, [_U32, _U32, _U32, _U32, _U32]),
    "wick_rocm_kv_shift": (C.c_int, [_P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _F]),
    "wick_rocm_lfm2_forward_prefill_from_embeddings": (C.c_int, [_P, _P, _P, _U32, _U32, _P]),
    "wick_rocm_lfm2_forward_from_embedding": (C.c_int, [_P, _P, _P, _U32, _P]),
    "wick_rocm_lfm2_forward_embedding": (C.c_int, [_P, _P, _U32, _U32, _P]),
    "wick_rocm_lfm2_forward_hidden_from_embedding": (C.c_int, [_P, _P, _P, _U32, _P]),
    "wick_rocm_lfm2_layer_state_bytes": (C.c_size_t, [_P, _U32, _U32]),
    "wick_rocm_lfm2_state_bytes": (C.c_size_t, [_P, _U32]),
    "wick_rocm_lfm2_snapshot_state": (C.c_int, [_P, _P, _U32, _P, C.c_size_t]),
    "wick_rocm_lfm2_restore_state": (C.c_int, [_P, _P, _U32, _P, C.c_size_t]),
    "wick_rocm_lfm2_shift_kv": (C.c_int, [_P, _P, _U32, _U32, _U32]),
}

_bound = False


def _lib() -> C.CDLL:
    global _bound
    lib = rocm.load_library()
    if not _bound:
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _bound = True
    return lib


def attention_scratch_floats(max_seq: int, n_heads: int, head_dim: int) -> int:
    return int(_lib().wick_rocm_attention_scratch_floats(max_seq, n_heads, head_dim))


def attention_block_scratch_bytes(max_seq: int, n_heads: int, head_dim: int) -> int:
    return int(_lib().wick_rocm_attention_block_scratch_bytes(max_seq, n_heads, head_dim))


def rope_theta_scale(head_dim: int, freq_base: float) -> float:
    return float(_lib().wick_rocm_rope_theta_scale(head_dim, freq_base))


class Lfm2Ops:
    """The operations as calls on a context (device buffers in, device buffers out)."""

    def __init__(self, ctx: RocmContext):
        self.ctx, self._l = ctx, _lib()

    def embed_row(self, w: RocmWeight, out, token: int = 0, d_token=None) -> None:
        self.ctx._check(self._l.wick_rocm_embed_row(self.ctx._h, w.handle, token, _ptr(d_token), _ptr(out)))

    def encode_rmsnorm(self, x, weight, y, dim: int, eps: float, rows: int = 1, x_stride: Optional[int] = None,
                       y_stride: Optional[int] = None) -> None:
        self.ctx._check(self._l.wick_rocm_rmsnorm(self.ctx._h, _ptr(x), _ptr(weight), _ptr(y), rows, dim, x_stride or dim, y_stride or dim, eps))

    def encode_qk_norm_rope(self, q, k, v, q_norm, k_norm, k_cache, v_cache, pos: int, max_seq: int, head_dim: int, n_heads: int,
                            n_kv_heads: int, eps: float, theta_scale: float, d_pos=None) -> None:
        self.ctx._check(self._l.wick_rocm_qk_norm_rope(self.ctx._h, _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(k_cache),
                                                       _ptr(v_cache), pos, _ptr(d_pos), max_seq, head_dim, n_heads, n_kv_heads, eps, theta_scale))

    def encode_qk_norm_rope_tokens(self, q, q_stride: int, k, v, kv_stride: int, q_norm, k_norm, k_cache, v_cache, pos0: int, n: int, max_seq: int,
                                   head_dim: int, n_heads: int, n_kv_heads: int, eps: float, theta_scale: float) -> None:
        """encode_qk_norm_rope for the n tokens of a prompt at positions pos0.. (token j's heads at j * stride floats)."""
        self.ctx._check(self._l.wick_rocm_qk_norm_rope_tokens(self.ctx._h, _ptr(q), q_stride, _ptr(k), _ptr(v), kv_stride, _ptr(q_norm), _ptr(k_norm),
                                                              _ptr(k_cache), _ptr(v_cache), pos0, n, max_seq, head_dim, n_heads, n_kv_heads, eps,
                                                              theta_scale))

    def kv_shift_scratch_floats(self, seq_len: int, n_keep: int, shift: int, n_kv_heads: int, head_dim: int) -> int:
        return int(self._l.wick_rocm_kv_shift_scratch_floats(seq_len, n_keep, shift, n_kv_heads, head_dim))

    def encode_kv_shift(self, k_cache, v_cache, scratch, seq_len: int, n_keep: int, shift: int, n_kv_heads: int, head_dim: int,
                        theta_scale: float) -> None:
        """One layer's n_keep context shift: cache rows [n_keep, n_keep + shift) dropped, the keys behind them re-rotated."""
        self.ctx._check(self._l.wick_rocm_kv_shift(self.ctx._h, _ptr(k_cache), _ptr(v_cache), _ptr(scratch), seq_len, n_keep, shift, n_kv_heads,
                                                   head_dim, theta_scale))

    def encode_attention(self, q, k_cache, v_cache, out, scores, seq_len: int, max_seq: int, n_heads: int, n_kv_heads: int, head_dim: int,
                         d_pos=None) -> None:
        self.ctx._check(self._l.wick_rocm_attention_decode(self.ctx._h, _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(scores), seq_len,
                                                           _ptr(d_pos), max_seq, n_heads, n_kv_heads, head_dim))

    def encode_attention_prefill(self, q, q_stride: int, k_cache, v_cache, out, out_stride: int, pos0: int, n: int, max_seq: int, n_heads: int,
                                 n_kv_heads: int, head_dim: int) -> None:
        """Causal attention of n prompt tokens at positions pos0.. over caches that already hold their K / V rows."""
        self.ctx._check(self._l.wick_rocm_attention_prefill(self.ctx._h, _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(out), out_stride,
                                                            pos0, n, max_seq, n_heads, n_kv_heads, head_dim))

    def encode_attention_prefill_quantize(self, q, q_stride: int, k_cache, v_cache, out_q, out_scales, pos0: int, n: int, max_seq: int, n_heads: int,
                                          n_kv_heads: int, head_dim: int) -> None:
        """encode_attention_prefill with the result written as Q8_0 blocks (the out projection's input)."""
        self.ctx._check(self._l.wick_rocm_attention_prefill_quantize_q8_0(self.ctx._h, _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(out_q),
                                                                          _ptr(out_scales), pos0, n, max_seq, n_heads, n_kv_heads, head_dim))

    def encode_conv1d_seq(self, proj, buffer, conv_weight, out, hidden: int, kernel_size: int, n: int) -> None:
        """The gated short convolution of n prompt tokens (proj [n][3*hidden] -> out [n][hidden]), then the rolling state."""
        self.ctx._check(self._l.wick_rocm_shortconv_seq(self.ctx._h, _ptr(proj), _ptr(buffer), _ptr(conv_weight), _ptr(out), hidden, kernel_size, n))

    def encode_conv1d_seq_quantize(self, proj, buffer, conv_weight, out_q, out_scales, hidden: int, kernel_size: int, n: int) -> None:
        """encode_conv1d_seq with the result written as Q8_0 blocks."""
        self.ctx._check(self._l.wick_rocm_shortconv_seq_quantize_q8_0(self.ctx._h, _ptr(proj), _ptr(buffer), _ptr(conv_weight), _ptr(out_q),
                                                                      _ptr(out_scales), hidden, kernel_size, n))

    def ffn_gate_up_silu_quantize_applies(self, w_gate: RocmWeight, w_up: RocmWeight, n: int) -> bool:
        return bool(self._l.wick_rocm_ffn_gate_up_silu_quantize_applies(w_gate.handle, w_up.handle, n))

    def encode_ffn_gate_up_silu_quantize(self, w_gate: RocmWeight, w_up: RocmWeight, scales, quants, n: int, out_q, out_scales) -> None:
        """Q8_0(silu(W_gate x) * (W_up x)) for n quantized activation rows: gate / up GEMM with the gate and the quantizer in its epilogue."""
        self.ctx._check(self._l.wick_rocm_ffn_gate_up_silu_quantize_q8(self.ctx._h, w_gate.handle, w_up.handle, _ptr(quants), _ptr(scales), n,
                                                                       _ptr(out_q), _ptr(out_scales)))

    def shortconv_fusable(self, w_out: RocmWeight, w_gate: RocmWeight, w_up: RocmWeight, kernel_size: int) -> bool:
        return bool(self._l.wick_rocm_shortconv_fusable(w_out.handle, w_gate.handle, w_up.handle, kernel_size))

    def encode_shortconv_out_proj(self, w_out: RocmWeight, proj, buffer, conv_weight, kernel_size: int, y, accumulate: bool = False) -> None:
        """y (+)= W_out quantize(c * conv(b * x)): the gated short convolution in the out projection's prologue (state read only)."""
        self.ctx._check(self._l.wick_rocm_shortconv_out_proj_f32(self.ctx._h, w_out.handle, _ptr(proj), _ptr(buffer), _ptr(conv_weight), kernel_size,
                                                                 _ptr(y), int(accumulate)))

    def encode_ffn_gate_up_conv_advance(self, w_gate: RocmWeight, w_up: RocmWeight, x, norm_weight, eps: float, act, proj, buffer, hidden: int,
                                        kernel_size: int) -> None:
        """encode_ffn_gate_up + the conv state of the same layer advanced by this token, in one launch."""
        self.ctx._check(self._l.wick_rocm_ffn_gate_up_conv_advance_f32(self.ctx._h, w_gate.handle, w_up.handle, _ptr(x), _ptr(norm_weight), eps, _ptr(act),
                                                                       _ptr(proj), _ptr(buffer), hidden, kernel_size))

    def encode_attention_block(self, q, k, v, q_norm, k_norm, k_cache, v_cache, out, scratch, pos: int, max_seq: int, head_dim: int,
                               n_heads: int, n_kv_heads: int, eps: float, theta_scale: float, d_pos=None) -> None:
        """QK-norm + RoPE + KV append folded into the attention kernel (then the merge)."""
        self.ctx._check(self._l.wick_rocm_attention_block(self.ctx._h, _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(k_cache),
                                                          _ptr(v_cache), _ptr(out), _ptr(scratch), pos, _ptr(d_pos), max_seq, head_dim, n_heads,
                                                          n_kv_heads, eps, theta_scale))

    def encode_conv1d_fused(self, proj, buffer, conv_weight, out, hidden: int, kernel_size: int) -> None:
        self.ctx._check(self._l.wick_rocm_shortconv_step(self.ctx._h, _ptr(proj), _ptr(buffer), _ptr(conv_weight), _ptr(out), hidden, kernel_size))

    def silu_mul_inplace(self, gate, up, n: int) -> None:
        self.ctx._check(self._l.wick_rocm_silu_mul(self.ctx._h, _ptr(gate), _ptr(up), n))

    def rmsnorm_quantize(self, x, weight, rows: int, dim: int, eps: float, quants, scales, x_stride: Optional[int] = None) -> None:
        """encode_rmsnorm + quantize_q8_0 of `rows` vectors without the f32 round trip."""
        self.ctx._check(self._l.wick_rocm_rmsnorm_quantize_q8_0(self.ctx._h, _ptr(x), _ptr(weight), rows, dim, x_stride or dim, eps, _ptr(quants),
                                                                _ptr(scales)))

    def silu_mul_quantize(self, gate, up, rows: int, dim: int, quants, scales) -> None:
        """silu_mul_inplace + quantize_q8_0 of [rows][dim] gate / up values, the gated f32 values never written."""
        self.ctx._check(self._l.wick_rocm_silu_mul_quantize_q8_0(self.ctx._h, _ptr(gate), _ptr(up), rows, dim, _ptr(quants), _ptr(scales)))

    def argmax(self, logits, n: int, out, d_token=None, d_pos=None) -> None:
        self.ctx._check(self._l.wick_rocm_argmax(self.ctx._h, _ptr(logits), n, _ptr(out), _ptr(d_token), _ptr(d_pos)))

    def lm_head_greedy(self, w, x, norm_weight, eps: float, logits, out, d_token=None, d_pos=None) -> None:
        """Output norm + LM head + greedy pick: logits = W rmsnorm(x), out[0] = argmax (and the device-side token / position)."""
        self.ctx._check(self._l.wick_rocm_lm_head_greedy_f32(self.ctx._h, w.handle, _ptr(x), _ptr(norm_weight), eps, _ptr(logits), _ptr(out),
                                                             _ptr(d_token), _ptr(d_pos)))


KV_F32, KV_F16 = 0, 1  # wick_rocm_lfm2_load_kv's kv_dtype


class RocmLfm2Model:
    """load_model_* counterpart (wick/src/model/mod.rs:385-403): owns weights, KV caches, conv state and scratch on the GPU."""

    def __init__(self, ctx: RocmContext, gguf, context_size: int, kv_f16: bool = False):
        """kv_f16: KV caches of f16 rows like the reference's GPU models (default: f32 rows like its CPU model)."""
        self.ctx, self._l = ctx, _lib()
        h = _P()
        if kv_f16:
            ctx._check(self._l.wick_rocm_lfm2_load_kv(ctx._h, gguf.handle, context_size, KV_F16, C.byref(h)))
        else:
            ctx._check(self._l.wick_rocm_lfm2_load(ctx._h, gguf.handle, context_size, C.byref(h)))
        self._h = h.value
        self.kv_f16 = self._l.wick_rocm_lfm2_kv_dtype(self._h) == KV_F16
        cfg = Lfm2Config()
        ctx._check(self._l.wick_rocm_lfm2_get_config(self._h, C.byref(cfg)))
        self.config = {n: getattr(cfg, n) for n, _ in Lfm2Config._fields_}
        kv = _U32()
        self.kv_heads_per_layer = []
        for i in range(cfg.n_layers):
            ctx._check(self._l.wick_rocm_lfm2_layer_kv_heads(self._h, i, C.byref(kv)))
            self.kv_heads_per_layer.append(kv.value)

    def free(self) -> None:
        if self._h:
            self.ctx._check(self._l.wick_rocm_lfm2_free(self.ctx._h, self._h))
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()

    def gpu_memory_bytes(self) -> int:
        return self._l.wick_rocm_lfm2_gpu_memory_bytes(self._h)

    def reset(self) -> None:
        self.ctx._check(self._l.wick_rocm_lfm2_reset(self.ctx._h, self._h))

    def set_graph_replay(self, enabled: bool) -> None:
        self.ctx._check(self._l.wick_rocm_lfm2_set_graph_replay(self._h, int(enabled)))

    def forward(self, token: int, pos: int) -> np.ndarray:
        logits = np.empty(self.config["vocab_size"], np.float32)
        self.ctx._check(self._l.wick_rocm_lfm2_forward(self.ctx._h, self._h, token, pos, logits.ctypes.data))
        return logits

    def forward_prefill(self, tokens, start_pos: int) -> np.ndarray:
        """Model::forward_prefill: the logits of the last prompt token."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.config["vocab_size"], np.float32)
        self.ctx._check(self._l.wick_rocm_lfm2_forward_prefill(self.ctx._h, self._h, t.ctypes.data, t.size, start_pos, logits.ctypes.data))
        return logits

    def forward_prefill_chunked(self, tokens, start_pos: int, ubatch: int, cancel=None):
        """Model::forward_prefill_chunked: (tokens consumed, logits of the last processed chunk or None).  `cancel` is a
        ctypes.c_int32 another thread may set; it is looked at after every chunk."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.config["vocab_size"], np.float32)
        consumed = _U32()
        self.ctx._check(self._l.wick_rocm_lfm2_forward_prefill_chunked(self.ctx._h, self._h, t.ctypes.data, t.size, start_pos, ubatch,
                                                                       C.addressof(cancel) if cancel is not None else None, C.byref(consumed),
                                                                       logits.ctypes.data))
        return consumed.value, (logits if consumed.value else None)

    def forward_prefill_from_embeddings(self, embeddings, start_pos: int) -> np.ndarray:
        """Model::forward_prefill_from_embeddings: `embeddings` is [n][hidden_size]; logits of the last frame."""
        e = np.ascontiguousarray(embeddings, dtype=np.float32).reshape(-1, self.config["hidden_size"])
        logits = np.empty(self.config["vocab_size"], np.float32)
        self.ctx._check(self._l.wick_rocm_lfm2_forward_prefill_from_embeddings(self.ctx._h, self._h, e.ctypes.data, e.shape[0], start_pos,
                                                                               logits.ctypes.data))
        return logits

    def _embedding(self, embedding) -> np.ndarray:
        e = np.ascontiguousarray(embedding, dtype=np.float32).ravel()
        if e.size != self.config["hidden_size"]:
            raise ValueError(f"embedding has {e.size} elements, hidden_size is {self.config['hidden_size']}")
        return e

    def forward_from_embedding(self, embedding, pos: int) -> np.ndarray:
        """Model::forward_from_embedding: a step fed with a hidden-size vector instead of a token -> logits."""
        e, logits = self._embedding(embedding), np.empty(self.config["vocab_size"], np.float32)
        self.ctx._check(self._l.wick_rocm_lfm2_forward_from_embedding(self.ctx._h, self._h, e.ctypes.data, pos, logits.ctypes.data))
        return logits

    def forward_embedding(self, token: int, pos: int) -> np.ndarray:
        """Model::forward_embedding: a token step that returns the hidden state after the output norm (no LM head)."""
        hidden = np.empty(self.config["hidden_size"], np.float32)
        self.ctx._check(self._l.wick_rocm_lfm2_forward_embedding(self.ctx._h, self._h, token, pos, hidden.ctypes.data))
        return hidden

    def forward_hidden_from_embedding(self, embedding, pos: int) -> np.ndarray:
        e, hidden = self._embedding(embedding), np.empty(self.config["hidden_size"], np.float32)
        self.ctx._check(self._l.wick_rocm_lfm2_forward_hidden_from_embedding(self.ctx._h, self._h, e.ctypes.data, pos, hidden.ctypes.data))
        return hidden

    def layer_state_bytes(self, layer: int, seq_len: int) -> int:
        return int(self._l.wick_rocm_lfm2_layer_state_bytes(self._h, layer, seq_len))

    def snapshot_state(self, seq_len: int) -> np.ndarray:
        """Model::snapshot_state: the state after seq_len positions as bytes (layer by layer: keys then values, or the conv buffer)."""
        out = np.empty(int(self._l.wick_rocm_lfm2_state_bytes(self._h, seq_len)), np.uint8)
        self.ctx._check(self._l.wick_rocm_lfm2_snapshot_state(self.ctx._h, self._h, seq_len, out.ctypes.data, out.size))
        return out

    def restore_state(self, snapshot, seq_len: int) -> None:
        """Model::restore_state: the inverse of snapshot_state(seq_len)."""
        b = np.ascontiguousarray(snapshot, dtype=np.uint8)
        self.ctx._check(self._l.wick_rocm_lfm2_restore_state(self.ctx._h, self._h, seq_len, b.ctypes.data, b.size))

    def shift_kv(self, seq_len: int, n_keep: int, shift: int) -> int:
        """Model::shift_kv on a state of seq_len positions; returns the new position count."""
        self.ctx._check(self._l.wick_rocm_lfm2_shift_kv(self.ctx._h, self._h, seq_len, n_keep, shift))
        return seq_len - shift

    def forward_greedy(self, token: int, pos: int) -> int:
        nxt = _U32()
        self.ctx._check(self._l.wick_rocm_lfm2_forward_greedy(self.ctx._h, self._h, token, pos, C.byref(nxt)))
        return nxt.value

    def generate_greedy(self, token: int, pos: int, n: int) -> np.ndarray:
        out = np.empty(n, np.uint32)
        self.ctx._check(self._l.wick_rocm_lfm2_generate_greedy(self.ctx._h, self._h, token, pos, n, out.ctypes.data))
        return out
