"""CPU oracle of wick's LFM2 decode step (TEST INFRASTRUCTURE, not product code).

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu-baseline leg may import this
module.  The per-operation functions wrap ``oracle/wick_oracle_ops.c`` one to one; the
step itself (``Lfm2Oracle.forward``) is the aarch64 branch of the reference's CPU model:
every GEMV runs on Q8_0-quantized activations (wick/src/model/lfm2.rs:1020-1124 run_layers,
:646-730 conv block, :733-1017 attention block, :2258-2289 forward).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import oracle as O

F32 = 0  # ggml type id

_ops = None


def ops() -> C.CDLL:
    global _ops
    if _ops is None:
        L = O._load("libwick_oracle_ops.so")
        L.orc_ggml_expf.restype = C.c_float
        L.orc_ggml_expf.argtypes = [C.c_float]
        L.orc_rope_theta_scale.restype = C.c_float
        L.orc_rope_theta_scale.argtypes = [C.c_int64, C.c_float]
        L.orc_argmax.restype = C.c_int64
        _ops = L
    return _ops


_p, _c = O._p, O._c


def ggml_expf(x: float) -> float:
    return float(ops().orc_ggml_expf(C.c_float(float(x))))


def rmsnorm(x, weight, eps: float) -> np.ndarray:
    y = _c(x, np.float32).copy()
    ops().orc_rmsnorm(_p(y), _p(_c(weight, np.float32)), C.c_int64(y.size), C.c_float(eps))
    return y


def silu_mul(gate, up) -> np.ndarray:
    g = _c(gate, np.float32).copy()
    ops().orc_silu_mul(_p(g), _p(_c(up, np.float32)), C.c_int64(g.size))
    return g


def softmax(x) -> np.ndarray:
    y = _c(x, np.float32).copy()
    ops().orc_softmax(_p(y), C.c_int64(y.size))
    return y


def rope(q, k, pos: int, n_heads: int, n_kv_heads: int, head_dim: int, freq_base: float):
    q2, k2 = _c(q, np.float32).copy(), _c(k, np.float32).copy()
    ops().orc_rope(_p(q2), _p(k2), C.c_int64(pos), C.c_int64(n_heads), C.c_int64(n_kv_heads), C.c_int64(head_dim), C.c_float(freq_base))
    return q2, k2


def rope_delta(head, delta_pos: int, head_dim: int, freq_base: float) -> np.ndarray:
    h = _c(head, np.float32).copy()
    ops().orc_rope_delta(_p(h), C.c_int32(delta_pos), C.c_int64(head_dim), C.c_float(freq_base))
    return h


def shift_kv(k_cache, v_cache, seq_len: int, n_keep: int, shift: int, n_kv_heads: int, head_dim: int, freq_base: float):
    """The caches of one attention layer ([>= seq_len][n_kv_heads * head_dim]) after dropping rows [n_keep, n_keep + shift)."""
    assert shift > 0 and n_keep + shift <= seq_len
    k2, v2 = _c(k_cache, np.float32).copy(), _c(v_cache, np.float32).copy()
    ops().orc_shift_kv(_p(k2), _p(v2), C.c_int64(seq_len), C.c_int64(n_keep), C.c_int64(shift), C.c_int64(n_kv_heads), C.c_int64(head_dim),
                       C.c_float(freq_base))
    return k2, v2


def rope_theta_scale(head_dim: int, freq_base: float) -> float:
    return float(ops().orc_rope_theta_scale(head_dim, C.c_float(freq_base)))


def attn_scores(q_head, k_cache, kv_dim: int, kv_h_offset: int, head_dim: int, scale: float, seq_len: int) -> np.ndarray:
    out = np.zeros(seq_len, np.float32)
    ops().orc_attn_scores(_p(_c(q_head, np.float32)), _p(_c(k_cache, np.float32)), _p(out), C.c_int64(kv_dim), C.c_int64(kv_h_offset),
                          C.c_int64(head_dim), C.c_float(scale), C.c_int64(seq_len))
    return out


def attn_values(scores, v_cache, kv_dim: int, kv_h_offset: int, head_dim: int, seq_len: int) -> np.ndarray:
    out = np.zeros(head_dim, np.float32)
    ops().orc_attn_values(_p(_c(scores, np.float32)), _p(_c(v_cache, np.float32)), _p(out), C.c_int64(kv_dim), C.c_int64(kv_h_offset),
                          C.c_int64(head_dim), C.c_int64(seq_len))
    return out


def attention(q, k_cache, v_cache, n_heads: int, n_kv_heads: int, head_dim: int, seq_len: int) -> np.ndarray:
    """All heads of one decode position (wick/src/model/lfm2.rs:984-1006): [n_heads * head_dim]."""
    q = _c(q, np.float32)
    kc, vc = _c(k_cache, np.float32), _c(v_cache, np.float32)
    kv_dim, group = n_kv_heads * head_dim, n_heads // n_kv_heads
    scale = np.float32(1.0) / np.sqrt(np.float32(head_dim))
    out = np.zeros(n_heads * head_dim, np.float32)
    scratch = np.zeros(max(seq_len, 1), np.float32)
    for h in range(n_heads):
        ops().orc_attention_head(_p(q[h * head_dim:]), _p(kc), _p(vc), _p(scratch), _p(out[h * head_dim:]), C.c_int64(kv_dim),
                                 C.c_int64((h // group) * head_dim), C.c_int64(head_dim), C.c_float(scale), C.c_int64(seq_len))
    return out


def shortconv_step(proj, buffer, conv_weight, hidden: int, kernel_size: int) -> np.ndarray:
    """One decode step of the gated short convolution; `buffer` ([(kernel-1) * hidden] f32) is updated in place."""
    assert buffer.dtype == np.float32 and buffer.flags.c_contiguous and buffer.size == (kernel_size - 1) * hidden
    out = np.empty(hidden, np.float32)
    ops().orc_shortconv_step(_p(_c(proj, np.float32)), _p(buffer), _p(_c(conv_weight, np.float32)), _p(out), C.c_int64(hidden),
                             C.c_int64(kernel_size))
    return out


def argmax(x) -> int:
    x = _c(x, np.float32)
    return int(ops().orc_argmax(_p(x), C.c_int64(x.size))) if x.size else 0


def embed_row(ggml_type: int, data: np.ndarray, row: int, k: int) -> np.ndarray:
    """dequantize_row_into, wick/src/model/lfm2.rs:621-643."""
    if ggml_type == F32:
        return data.view(np.float32)[row * k:(row + 1) * k].copy()
    if ggml_type == O.Q6_K:
        rb = k // 256 * 210
        return O.dequant_q6_k(data[row * rb:(row + 1) * rb], 1, k)[0]
    rb = k // 32 * O.BLOCK_BYTES[ggml_type]
    return O.dequant_row(ggml_type, data[row * rb:(row + 1) * rb])


def gemv(ggml_type: int, data: np.ndarray, x: np.ndarray, m: int, k: int) -> np.ndarray:
    """The aarch64 GEMV dispatch: quantize x to Q8_0, integer dots (wick/src/backend/cpu.rs:334-354, 423-470)."""
    s, q = O.quantize_q8_0(x)
    if ggml_type == O.Q6_K:
        return O.gemv_q6k_q8(data, s, q, m, k)
    return O.gemv_q8(ggml_type, data, s, q, m, k)


def quantizer_margin(x) -> float:
    """How far the Q8_0 quantization of `x` (wick/src/backend/simd.rs:255-323) is from changing under a
    last-bit perturbation of x, as the smaller of
      - the distance of any x*id from a rounding tie (in units of one quant step), and
      - 1e3 x the relative distance of any block's amax/127 from an f16 rounding boundary of its scale.
    The quantizer is discontinuous there: two correct f32 pipelines that differ in the last bit of one
    activation can then legitimately differ by a whole quant step (or a whole f16 scale step) downstream."""
    x = np.asarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(x).max(1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    r = (x * idv[:, None]).astype(np.float32)
    tie = float(np.abs(r - np.floor(r) - np.float32(0.5)).min())
    nz = d[d != 0].astype(np.float64)
    if nz.size == 0:
        return tie
    h = nz.astype(np.float16).astype(np.float64)
    up, dn = np.nextafter(h.astype(np.float16), np.float16(np.inf)).astype(np.float64), np.nextafter(h.astype(np.float16), np.float16(-np.inf)).astype(np.float64)
    edge = np.minimum(np.abs(nz - (h + up) / 2), np.abs(nz - (h + dn) / 2)) / nz
    return min(tie, float(edge.min()) * 1e3)


def _f16_round(x) -> np.ndarray:
    """f32 -> nearest-even f16 -> f32 (what a cache of f16 rows keeps of a value)."""
    with np.errstate(over="ignore"):
        return np.asarray(x, np.float32).astype(np.float16).astype(np.float32)


class Lfm2Oracle:
    """`cfg`: n_layers, hidden_size, intermediate_size, n_heads, vocab_size, rope_theta, rms_norm_eps,
    conv_kernel_size, kv_heads_per_layer (0 = gated-conv layer).  `tensors`: GGUF name -> (ggml_type, dims, array),
    quantized weights as raw block bytes (dims [k, m]), norms / conv kernels as float32."""

    def __init__(self, cfg: dict, tensors: dict, jitter_seed=None, kv_f16=False):
        self.cfg, self.t = cfg, tensors
        # KV caches of f16 rows, the reference's GPU models' caches (wick/src/model/metal_lfm2.rs:4117-4247: K after QK-norm and
        # RoPE and V are cast to half on their way in, the attention reads half): every cached value is rounded to nearest even
        # f16 when it is appended or moved by a context shift; the arithmetic on the widened values is the f32 one below.
        self.kv_f16 = kv_f16
        self.min_margin = float("inf")  # smallest quantizer_margin over every GEMV input so far
        # Sensitivity probe: with a seed, every GEMV output is moved by up to 2^-22 of its value (about two ulp), which is
        # what another order of the f32 block sums does to it -- the order is not part of the contract (rel-L2 1e-5 is).
        # How far the logits of a jittered run move is how far a correct implementation may sit from this oracle once
        # activations come near quantizer ties.
        self.jitter = np.random.default_rng(jitter_seed) if jitter_seed is not None else None

    def new_state(self) -> dict:
        c = self.cfg
        hs, dconv = c["hidden_size"], c["conv_kernel_size"] - 1
        st = {"seq_len": 0, "layers": []}
        for n_kv in c["kv_heads_per_layer"]:
            st["layers"].append({"k": [], "v": []} if n_kv else {"buf": np.zeros(dconv * hs, np.float32)})
        return st

    def _f32(self, name):
        return self.t[name][2].view(np.float32).ravel()

    def _gemv(self, name, x):
        gt, dims, data = self.t[name]
        self.min_margin = min(self.min_margin, quantizer_margin(x))
        y = gemv(gt, data, x, dims[1], dims[0])
        if self.jitter is not None:
            y = (y * (np.float32(1.0) + self.jitter.uniform(-1.0, 1.0, y.size).astype(np.float32) * np.float32(2.0 ** -22))).astype(np.float32)
        return y

    def hidden_after_layers(self, token, pos: int, state: dict, embedding=None) -> np.ndarray:
        """run_layers (wick/src/model/lfm2.rs:1020-1124) on the token's embedding row, or on `embedding` when given
        (forward_embedding / forward_hidden_from_embedding, :2325-2349): the hidden state after the output norm."""
        c = self.cfg
        hs, eps = c["hidden_size"], c["rms_norm_eps"]
        if embedding is None:
            gt, dims, data = self.t["token_embd.weight"]
            hidden = embed_row(gt, data, token, dims[0])
        else:
            hidden = _c(embedding, np.float32).copy()
            assert hidden.size == hs
        for i, n_kv in enumerate(c["kv_heads_per_layer"]):
            normed = rmsnorm(hidden, self._f32(f"blk.{i}.attn_norm.weight"), eps)
            if n_kv == 0:
                proj = self._gemv(f"blk.{i}.shortconv.in_proj.weight", normed)
                gated = shortconv_step(proj, state["layers"][i]["buf"], self._f32(f"blk.{i}.shortconv.conv.weight"), hs, c["conv_kernel_size"])
                out = self._gemv(f"blk.{i}.shortconv.out_proj.weight", gated)
            else:
                hd = hs // c["n_heads"]
                q = self._gemv(f"blk.{i}.attn_q.weight", normed)
                k = self._gemv(f"blk.{i}.attn_k.weight", normed)
                v = self._gemv(f"blk.{i}.attn_v.weight", normed)
                qn, kn = self._f32(f"blk.{i}.attn_q_norm.weight"), self._f32(f"blk.{i}.attn_k_norm.weight")
                for h in range(c["n_heads"]):
                    q[h * hd:(h + 1) * hd] = rmsnorm(q[h * hd:(h + 1) * hd], qn, eps)
                for h in range(n_kv):
                    k[h * hd:(h + 1) * hd] = rmsnorm(k[h * hd:(h + 1) * hd], kn, eps)
                q, k = rope(q, k, pos, c["n_heads"], n_kv, hd, c["rope_theta"])
                ls = state["layers"][i]
                if self.kv_f16:
                    k, v = _f16_round(k), _f16_round(v)
                ls["k"].append(k), ls["v"].append(v)
                attn = attention(q, np.concatenate(ls["k"]), np.concatenate(ls["v"]), c["n_heads"], n_kv, hd, len(ls["k"]))
                out = self._gemv(f"blk.{i}.attn_output.weight", attn)
            hidden = hidden + out
            ffn_in = rmsnorm(hidden, self._f32(f"blk.{i}.ffn_norm.weight"), eps)
            gate = self._gemv(f"blk.{i}.ffn_gate.weight", ffn_in)
            up = self._gemv(f"blk.{i}.ffn_up.weight", ffn_in)
            hidden = hidden + self._gemv(f"blk.{i}.ffn_down.weight", silu_mul(gate, up))
        state["seq_len"] += 1
        return rmsnorm(hidden, self._f32("token_embd_norm.weight"), eps)

    def forward(self, token: int, pos: int, state: dict) -> np.ndarray:
        """Logits of one decode step (tied embedding as LM head, wick/src/model/lfm2.rs:2258-2289)."""
        hidden = self.hidden_after_layers(token, pos, state)
        return self._gemv("token_embd.weight", hidden)

    def forward_from_embedding(self, embedding, pos: int, state: dict) -> np.ndarray:
        """Logits of one step whose input is a hidden-size vector instead of a token (wick/src/model/lfm2.rs:2295-2323)."""
        return self._gemv("token_embd.weight", self.hidden_after_layers(None, pos, state, embedding))

    def shift_kv(self, state: dict, n_keep: int, shift: int) -> None:
        """Lfm2Model::shift_kv (wick/src/model/lfm2.rs:2507-2516): every attention layer drops cache rows [n_keep, n_keep + shift)
        and re-rotates the keys behind them; conv layers are left alone; seq_len shrinks by `shift`."""
        c = self.cfg
        hd, seq = c["hidden_size"] // c["n_heads"], state["seq_len"]
        assert shift > 0 and n_keep + shift <= seq
        for n_kv, ls in zip(c["kv_heads_per_layer"], state["layers"]):
            if n_kv == 0 or not ls["k"]:
                continue
            assert len(ls["k"]) == seq
            k, v = shift_kv(np.concatenate(ls["k"]), np.concatenate(ls["v"]), seq, n_keep, shift, n_kv, hd, c["rope_theta"])
            if self.kv_f16:  # the re-rotated keys go back into f16 rows (kept rows and values are f16 values already)
                k = _f16_round(k)
            kvd = n_kv * hd
            ls["k"] = [k[t * kvd:(t + 1) * kvd].copy() for t in range(seq - shift)]
            ls["v"] = [v[t * kvd:(t + 1) * kvd].copy() for t in range(seq - shift)]
        state["seq_len"] = seq - shift
