/* wick_rocm_lfm2.h -- the LFM2 decode step around the matmul path, on one gfx950 GPU.
 *
 * Two layers, both on top of include/wick_rocm.h (same context, same status codes, same
 * enqueue-only semantics, device pointers named d_*):
 *
 *  1. The non-matmul operations of a decode step as single calls, shaped like the reference's
 *     GPU encoder call sites (wick/src/model/metal_lfm2.rs:1380-1990) and computing what its CPU
 *     operations compute (wick/src/backend/cpu.rs:577-731, 1320-1401, 2113-2161).
 *  2. A model handle that owns weights, KV caches, conv state and scratch, like the reference's
 *     GPU models (wick/src/model/metal_lfm2.rs:254-267), with forward / forward_greedy of
 *     `trait Model` (wick/src/model/mod.rs:72-323).  The step follows the aarch64 CPU model:
 *     every GEMV runs on Q8_0-quantized activations, the KV cache holds f32
 *     (wick/src/model/lfm2.rs:646-1124, 2258-2289).
 *
 * "pos" / "token" arguments come in pairs: a by-value number and a device pointer.  When the
 * pointer is non-null the kernel reads it instead, so a captured graph of the step can be
 * replayed for every token.
 */
#ifndef WICK_ROCM_LFM2_H
#define WICK_ROCM_LFM2_H

#include "wick_rocm.h"

#ifdef __cplusplus
extern "C" {
#endif

struct wick_gguf;

/* ---- operations ---------------------------------------------------------------------- */

/* Embedding lookup = dequantize_row_into (wick/src/model/lfm2.rs:621-643): row `token` (or *d_token) of a
 * Q4_0 / Q8_0 / Q6_K weight as k floats.  A by-value token >= m is an error; a device-side one leaves d_out untouched. */
int wick_rocm_embed_row(wick_rocm_ctx *ctx, const wick_rocm_weight *w, uint32_t token, const uint32_t *d_token, float *d_out);

/* encode_rmsnorm / encode_per_head_rmsnorm (wick/src/model/metal_lfm2.rs:1380-1398, 1480-1496) = cpu::rmsnorm
 * (wick/src/backend/cpu.rs:577-594) on `rows` vectors of `dim` floats that share one weight vector:
 * y[r*y_stride + i] = x[r*x_stride + i] * inv_rms_r * weight[i].  d_y may equal d_x. */
int wick_rocm_rmsnorm(wick_rocm_ctx *ctx, const float *d_x, const float *d_weight, float *d_y, uint32_t rows, uint32_t dim,
                      uint32_t x_stride, uint32_t y_stride, float eps);

/* encode_qk_norm_rope + the KV append (wick/src/model/metal_lfm2.rs:1542-1580, 4178-4193; CPU:
 * wick/src/model/lfm2.rs:783-857, cpu::rope wick/src/backend/cpu.rs:2113-2161): per-head RMSNorm of Q and K
 * with the layer's q_norm / k_norm weights, RoPE at `pos`, both in place; then K and V of this position are
 * stored at row `pos` of the caches ([max_seq][n_kv_heads*head_dim] floats).  theta_scale = freq_base^(-2/head_dim)
 * as an f32 (wick_rocm_rope_theta_scale).  head_dim even, <= 256. */
int wick_rocm_qk_norm_rope(wick_rocm_ctx *ctx, float *d_q, float *d_k, const float *d_v, const float *d_q_norm, const float *d_k_norm,
                           float *d_k_cache, float *d_v_cache, uint32_t pos, const uint32_t *d_pos, uint32_t max_seq, uint32_t head_dim,
                           uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale);
float wick_rocm_rope_theta_scale(uint32_t head_dim, float freq_base);

/* The same for the n tokens of a prompt at positions pos0 .. pos0 + n - 1: pass A of the reference's batched prefill
 * (QK norm, RoPE and the cache append per token, wick/src/model/lfm2.rs:1557-1620).  Token j's query heads start at
 * d_q + j * q_stride, its key and value heads at d_k / d_v + j * kv_stride (floats).  Bit-identical to n calls of
 * wick_rocm_qk_norm_rope. */
int wick_rocm_qk_norm_rope_tokens(wick_rocm_ctx *ctx, float *d_q, uint32_t q_stride, float *d_k, const float *d_v, uint32_t kv_stride,
                                  const float *d_q_norm, const float *d_k_norm, float *d_k_cache, float *d_v_cache, uint32_t pos0, uint32_t n,
                                  uint32_t max_seq, uint32_t head_dim, uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale);

/* One attention layer's part of the n_keep context shift (InferenceState::shift_kv_with_rope, wick/src/kv_cache.rs:601-700;
 * Metal: encode_kv_shift_layers, wick/src/model/metal_lfm2.rs:2657-2761): rows [n_keep, n_keep + shift) of both caches
 * ([>= seq_len][n_kv_heads*head_dim] floats) are dropped, the rows behind them move down by `shift`, and every key head that
 * moved is rotated by -shift positions (apply_rope_delta_to_head, wick/src/backend/cpu.rs:2174-2187), so that it reads as if it
 * had been rotated for its new row.  Values move unchanged.  Rows from seq_len - shift on are left as they were; the caller's
 * seq_len becomes seq_len - shift.  d_scratch holds wick_rocm_kv_shift_scratch_floats(...) floats (may be null when
 * n_keep + shift == seq_len: nothing moves).  shift > 0, n_keep + shift <= seq_len.  Not available inside a graph capture. */
size_t wick_rocm_kv_shift_scratch_floats(uint32_t seq_len, uint32_t n_keep, uint32_t shift, uint32_t n_kv_heads, uint32_t head_dim);
int wick_rocm_kv_shift(wick_rocm_ctx *ctx, float *d_k_cache, float *d_v_cache, float *d_scratch, uint32_t seq_len, uint32_t n_keep,
                       uint32_t shift, uint32_t n_kv_heads, uint32_t head_dim, float theta_scale);

/* encode_attention (wick/src/model/metal_lfm2.rs:1736-1867) = attn_scores + softmax_inplace + attn_values per
 * query head (wick/src/model/lfm2.rs:984-1006) over cache rows [0, seq_len) (seq_len = *d_pos + 1 when d_pos is
 * given), grouped-query: head h reads KV head h / (n_heads / n_kv_heads).  d_scratch holds
 * wick_rocm_attention_scratch_floats(max_seq, n_heads, head_dim) floats (contents need not be kept between calls).
 * head_dim % 4 == 0, <= 256.  Contexts longer than 256 positions with head_dim 32 / 64 / 128 / 256 are split over the
 * sequence (many workgroups per head, streaming softmax, a second small launch merges the partials). */
size_t wick_rocm_attention_scratch_floats(uint32_t max_seq, uint32_t n_heads, uint32_t head_dim);
int wick_rocm_attention_decode(wick_rocm_ctx *ctx, const float *d_q, const float *d_k_cache, const float *d_v_cache, float *d_out,
                               float *d_scratch, uint32_t seq_len, const uint32_t *d_pos, uint32_t max_seq, uint32_t n_heads,
                               uint32_t n_kv_heads, uint32_t head_dim);

/* Causal attention for the n tokens of a prompt whose K / V rows are already in the caches: pass B of the reference's
 * batched prefill (wick/src/model/lfm2.rs:1640-1700), i.e. for token j the decode attention above with
 * seq_len = pos0 + j + 1.  d_q: [n][q_stride] floats (a token's n_heads * head_dim query values first), d_out:
 * [n][out_stride].  head_dim 32 / 64 / 128 / 256; head_dim 64 with 16-byte aligned rows and n >= 16 runs on the matrix
 * cores with every f32 operand split into two f16 halves and three exact-product MFMAs per product (f32 accuracy: measured
 * rel-L2 2e-7 against an f64 evaluation; sums in another order than the reference's loops, softmax weights from the hardware's exp2
 * instead of ggml_expf: an ulp or two apart).  That path needs |q| / sqrt(head_dim),
 * |k| and |v| below the f16 range (65504) -- the range the reference's own GPU path assumes when it keeps its KV caches in f16
 * (encode_cast_f32_to_f16, wick/src/model/metal_lfm2.rs:4178-4193). */
int wick_rocm_attention_prefill(wick_rocm_ctx *ctx, const float *d_q, uint32_t q_stride, const float *d_k_cache, const float *d_v_cache,
                                float *d_out, uint32_t out_stride, uint32_t pos0, uint32_t n, uint32_t max_seq, uint32_t n_heads,
                                uint32_t n_kv_heads, uint32_t head_dim);

/* The same with the result written as Q8_0 blocks ([n][n_heads * head_dim] quants, [n][n_heads * head_dim / 32] scales), which is
 * what the output projection reads (the reference quantizes that input inside its GEMM call, wick/src/model/lfm2.rs:571-592):
 * bit-identical to wick_rocm_attention_prefill + wick_rocm_quantize_q8_0, one launch and one float round trip less.  Only where
 * the matrix-core kernel runs (head_dim 64, n >= 16, 16-byte aligned q and caches, q_stride % 4 == 0): WICK_ROCM_ERR_BAD_SHAPE
 * otherwise. */
int wick_rocm_attention_prefill_quantize_q8_0(wick_rocm_ctx *ctx, const float *d_q, uint32_t q_stride, const float *d_k_cache,
                                              const float *d_v_cache, int8_t *d_out_q, float *d_out_scales, uint32_t pos0, uint32_t n,
                                              uint32_t max_seq, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim);

/* The attention block between the Q/K/V projections and the output projection: what wick_rocm_qk_norm_rope followed
 * by wick_rocm_attention_decode compute (wick/src/model/lfm2.rs:783-1006), bit for bit, with the norm, the rotation and
 * the KV append folded into the attention kernel (workgroups norm and rotate their own query head; those that own the
 * new position norm, rotate and append K and V themselves), one launch less.  d_scratch:
 * wick_rocm_attention_block_scratch_bytes(...) bytes, contents need not be kept.  d_q / d_k may be overwritten (head
 * dims without a fused kernel run the separate launches, which work in place). */
size_t wick_rocm_attention_block_scratch_bytes(uint32_t max_seq, uint32_t n_heads, uint32_t head_dim);
int wick_rocm_attention_block(wick_rocm_ctx *ctx, float *d_q, float *d_k, const float *d_v, const float *d_q_norm, const float *d_k_norm,
                              float *d_k_cache, float *d_v_cache, float *d_out, void *d_scratch, uint32_t pos, const uint32_t *d_pos,
                              uint32_t max_seq, uint32_t head_dim, uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale);

/* encode_conv1d_fused (wick/src/model/metal_lfm2.rs:1959-1991) = the middle of forward_conv_block
 * (wick/src/model/lfm2.rs:694-726): d_proj = [b | c | x] (hidden floats each), d_buffer the rolling state
 * ((kernel_size-1) * hidden floats, updated in place), d_conv_weight [hidden][kernel_size]; d_out = c * conv(b*x). */
int wick_rocm_shortconv_step(wick_rocm_ctx *ctx, const float *d_proj, float *d_buffer, const float *d_conv_weight, float *d_out,
                             uint32_t hidden, uint32_t kernel_size);
/* The gated short convolution for the n tokens of a prompt (the sequential core of the reference's batched prefill,
 * wick/src/model/lfm2.rs:1306-1350): d_proj [n][3 * hidden] = a token's [b | c | x], d_out [n][hidden]; token j sees the gated
 * inputs b*x of tokens j-(K-1) .. j, those before the prompt from the rolling state, which is brought up to date afterwards.
 * Bit-identical to n calls of wick_rocm_shortconv_step.  The _quantize_q8_0 form writes the result as Q8_0 blocks for the out
 * projection instead ([n][hidden] quants, [n][hidden / 32] scales; bit-identical to the float form + wick_rocm_quantize_q8_0;
 * hidden % 32 == 0 and 16-byte aligned buffers, WICK_ROCM_ERR_BAD_SHAPE otherwise). */
int wick_rocm_shortconv_seq(wick_rocm_ctx *ctx, const float *d_proj, float *d_buffer, const float *d_conv_weight, float *d_out,
                            uint32_t hidden, uint32_t kernel_size, uint32_t n);
int wick_rocm_shortconv_seq_quantize_q8_0(wick_rocm_ctx *ctx, const float *d_proj, float *d_buffer, const float *d_conv_weight,
                                          int8_t *d_out_q, float *d_out_scales, uint32_t hidden, uint32_t kernel_size, uint32_t n);
/* The same convolution folded into the launches on either side of it, two launches instead of three per gated-conv layer
 * (the Metal path fuses its dispatches the same way, e.g. encode_gemv_rmsnorm_gate_up, wick/src/model/metal_lfm2.rs:1157-1186):
 *   wick_rocm_shortconv_out_proj_f32        y (+)= W_out * quantize(c * conv(b * x)): the out projection computes the gated
 *                                           convolution in its prologue from d_proj, the conv weight and the rolling state,
 *                                           which it only READS (every workgroup needs the old state);
 *   wick_rocm_ffn_gate_up_conv_advance_f32  wick_rocm_ffn_gate_up_f32 of the same layer, whose first workgroups also advance
 *                                           the rolling state by this token (slot s <- slot s + 1, last slot <- b * x).
 * Called in this order, y, d_act and the state are bit-identical to wick_rocm_shortconv_step + wick_rocm_matmul_f32(accumulate)
 * + wick_rocm_ffn_gate_up_f32.  Shapes: kernel size 3, hidden <= 2048 (even block count), Q4_0 / Q8_0 weights the one-launch
 * kernels take, 16-byte aligned buffers; wick_rocm_shortconv_fusable says so beforehand (1 / 0), the calls themselves return
 * WICK_ROCM_ERR_BAD_SHAPE otherwise (no silent fallback: the two halves only make sense together). */
int wick_rocm_shortconv_fusable(const wick_rocm_weight *w_out, const wick_rocm_weight *w_gate, const wick_rocm_weight *w_up, uint32_t kernel_size);
int wick_rocm_shortconv_out_proj_f32(wick_rocm_ctx *ctx, const wick_rocm_weight *w_out, const float *d_proj, const float *d_buffer,
                                     const float *d_conv_weight, uint32_t kernel_size, float *d_y, int accumulate);
int wick_rocm_ffn_gate_up_conv_advance_f32(wick_rocm_ctx *ctx, const wick_rocm_weight *w_gate, const wick_rocm_weight *w_up, const float *d_x,
                                           const float *d_norm_weight, float eps, float *d_act, const float *d_proj, float *d_buffer,
                                           uint32_t hidden, uint32_t kernel_size);

/* encode_elementwise(silu_mul_inplace) (wick/src/model/metal_lfm2.rs:1701-1715) = cpu::silu_mul_inplace
 * (wick/src/backend/cpu.rs:668-673): gate = silu(gate) * up. */
int wick_rocm_silu_mul(wick_rocm_ctx *ctx, float *d_gate, const float *d_up, uint32_t n);

/* Prompt-pass forms of the two steps in front of a batched projection, without the f32 round trip through memory:
 * wick_rocm_rmsnorm followed by wick_rocm_quantize_q8_0, and wick_rocm_silu_mul followed by wick_rocm_quantize_q8_0
 * (quantize_columns after the norm / the gate, wick/src/model/lfm2.rs:1163-1200, 1990-2050), bit for bit.  Outputs in the
 * split Q8_0 layout of wick_rocm_quantize_q8_0: d_quants [rows][dim] int8, d_scales [rows][dim / 32] f32.  dim % 32 == 0;
 * rows of d_x (x_stride floats apart, x_stride % 4 == 0), d_weight, d_gate and d_up 16-byte aligned; gate / up contiguous. */
int wick_rocm_rmsnorm_quantize_q8_0(wick_rocm_ctx *ctx, const float *d_x, const float *d_weight, uint32_t rows, uint32_t dim, uint32_t x_stride,
                                    float eps, int8_t *d_quants, float *d_scales);
int wick_rocm_silu_mul_quantize_q8_0(wick_rocm_ctx *ctx, const float *d_gate, const float *d_up, uint32_t rows, uint32_t dim, int8_t *d_quants,
                                     float *d_scales);

/* The feed-forward block's gate and up projections over n prompt tokens with the SiLU gate and the Q8_0 quantizer of the
 * down projection's input in the GEMM's epilogue (wick/src/model/lfm2.rs:2025-2090: gemm_preq(ffn_gate), gemm_preq(ffn_up),
 * silu_mul_inplace, quantize_columns): d_out_quants [n][m] int8, d_out_scales [n][m / 32] f32, bit-identical to
 * wick_rocm_gemm_q8_multi + wick_rocm_silu_mul_quantize_q8_0; the two float projections (2 * n * m * 4 bytes) are never written.
 * d_quants / d_scales: the n quantized activation rows (wick_rocm_quantize_q8_0 layout).  Only where the wide matrix-core tile
 * runs: both weights Q4_0 or both Q8_0 with the same m and k, m % 32 == 0, k % 128 == 0, n > 64 and more than 256 tiles of
 * 64 rows x 128 tokens; wick_rocm_ffn_gate_up_silu_quantize_applies says so beforehand (1 / 0), the call returns
 * WICK_ROCM_ERR_BAD_SHAPE otherwise. */
int wick_rocm_ffn_gate_up_silu_quantize_applies(const wick_rocm_weight *w_gate, const wick_rocm_weight *w_up, uint32_t n);
int wick_rocm_ffn_gate_up_silu_quantize_q8(wick_rocm_ctx *ctx, const wick_rocm_weight *w_gate, const wick_rocm_weight *w_up,
                                           const int8_t *d_quants, const float *d_scales, uint32_t n, int8_t *d_out_quants,
                                           float *d_out_scales);

/* argmax_f32 dispatch of forward_greedy (wick/src/model/metal_lfm2.rs:2187-2195) with the tie / NaN rules of
 * cpu_argmax (wick/src/sampler.rs:7-19).  d_out[0] = pick; when given, *d_token = pick and *d_pos += 1. */
int wick_rocm_argmax(wick_rocm_ctx *ctx, const float *d_logits, uint32_t n, uint32_t *d_out, uint32_t *d_token, uint32_t *d_pos);

/* The tail of forward_greedy as one call (encode_rmsnorm + encode_gemv_output + argmax_f32, wick/src/model/metal_lfm2.rs:2180-2195):
 * d_logits[w->m] = W rmsnorm(d_x) with the output norm's weights, then wick_rocm_argmax over them.  A Q6_K head (the tied
 * embedding of shipped Q4_0 files) norms and quantizes its input inside the GEMV's launch and leaves the pick's first stage
 * behind as one key per wave: two launches, where wick_rocm_gemv_rmsnorm_f32_multi + wick_rocm_argmax take three; logits and
 * pick are bit-identical to that sequence.  d_x, d_norm_weight, d_logits 16-byte aligned. */
int wick_rocm_lm_head_greedy_f32(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const float *d_x, const float *d_norm_weight, float eps,
                                 float *d_logits, uint32_t *d_out, uint32_t *d_token, uint32_t *d_pos);

/* ---- the model --------------------------------------------------------------------------- */

typedef struct wick_rocm_lfm2 wick_rocm_lfm2;

/* ModelConfig (wick/src/model/mod.rs:23-70) as far as the step needs it. */
typedef struct wick_rocm_lfm2_config {
    uint32_t n_layers, hidden_size, intermediate_size, n_heads, n_kv_heads /* max over layers */, vocab_size, max_seq_len,
        conv_kernel_size;
    float rope_theta, rms_norm_eps;
} wick_rocm_lfm2_config;

/* load_model_metal's counterpart (wick/src/model/mod.rs:385-403; metadata keys, tensor names and checks of
 * Lfm2Model::from_gguf_with_id, wick/src/model/lfm2.rs:97-300): reads the config, uploads every weight, allocates
 * KV caches for min(context_size, lfm2.context_length) positions, conv state and scratch.  The GGUF handle is not
 * referenced after the call returns. */
int wick_rocm_lfm2_load(wick_rocm_ctx *ctx, const struct wick_gguf *gguf, uint32_t context_size, wick_rocm_lfm2 **out);
/* The same with the element type of the KV caches chosen by the caller.  WICK_ROCM_KV_F32 (what wick_rocm_lfm2_load takes):
 * f32 rows, the CPU model's caches (wick/src/kv_cache.rs) -- what the oracle of this backend computes on.  WICK_ROCM_KV_F16:
 * f16 rows, the reference's GPU models' caches (K after QK-norm and RoPE and V are cast to half on their way in and the
 * attention kernels read half, wick/src/model/metal_lfm2.rs:4117-4247, 2906-3364): half the cache memory and half the
 * attention's cache traffic; every cached value is rounded once, to nearest even, when it is appended (or moved by
 * wick_rocm_lfm2_shift_kv), all arithmetic stays f32.  Snapshots then hold f16 rows (wick_rocm_lfm2_layer_state_bytes says
 * how many bytes). */
enum { WICK_ROCM_KV_F32 = 0, WICK_ROCM_KV_F16 = 1 };
int wick_rocm_lfm2_load_kv(wick_rocm_ctx *ctx, const struct wick_gguf *gguf, uint32_t context_size, int kv_dtype, wick_rocm_lfm2 **out);
int wick_rocm_lfm2_kv_dtype(const wick_rocm_lfm2 *model);
int wick_rocm_lfm2_free(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model);
int wick_rocm_lfm2_get_config(const wick_rocm_lfm2 *model, wick_rocm_lfm2_config *out);
/* kv_heads_per_layer (0 = gated-conv layer). */
int wick_rocm_lfm2_layer_kv_heads(const wick_rocm_lfm2 *model, uint32_t layer, uint32_t *n_kv_heads);
/* Model::gpu_memory_bytes. */
size_t wick_rocm_lfm2_gpu_memory_bytes(const wick_rocm_lfm2 *model);
/* A fresh InferenceState: conv state zeroed, caches logically empty. */
int wick_rocm_lfm2_reset(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model);

/* Steps replay a captured graph (the counterpart of one command buffer per token, wick/src/model/metal_lfm2.rs:1-4).
 * With enabled = 0 the same launches are enqueued one by one instead, which per-dispatch timing
 * (wick_rocm_kernel_timing_begin) and kernel tracers need; results are identical.  While per-dispatch timing is on,
 * steps are enqueued one by one whatever this switch says.  The counterpart of the
 * reference's profiled encode path (encode_layers_profiled, wick/src/model/metal_lfm2.rs:4559-4712). */
int wick_rocm_lfm2_set_graph_replay(wick_rocm_lfm2 *model, int enabled);

/* Model::forward (wick/src/model/lfm2.rs:2258-2289): one token at position `pos` (= tokens seen so far) ->
 * vocab_size logits copied to `logits` (host memory; may be null to leave them on the device).  Waits for the step. */
int wick_rocm_lfm2_forward(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t token, uint32_t pos, float *logits);
/* Model::forward_prefill (wick/src/model/lfm2.rs:2351-2443, prefill_layers_and_logits :1139-2109): n prompt tokens at
 * positions start_pos .. start_pos + n - 1 in passes of up to 2048; projections run as GEMMs over the tokens, the conv
 * state and the KV append are walked in token order, attention is causal per (head, token).  Leaves the state as n
 * single steps would (up to the rounding of GEMM against GEMV sums) and returns the logits of the LAST token. */
int wick_rocm_lfm2_forward_prefill(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, const uint32_t *tokens, uint32_t n, uint32_t start_pos,
                                   float *logits);
/* Model::forward_prefill_from_embeddings (wick/src/model/lfm2.rs:2452-2487, wick/src/model/metal_lfm2.rs:2426-2464): the same
 * passes over n frames given as hidden-size vectors (frame j at embeddings[j * hidden_size], host memory) instead of token ids;
 * logits of the LAST frame. */
int wick_rocm_lfm2_forward_prefill_from_embeddings(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, const float *embeddings, uint32_t n,
                                                   uint32_t start_pos, float *logits);
/* Model::forward_prefill_chunked (wick/src/model/mod.rs:111-140): the prompt in chunks of `ubatch` tokens (0 = one chunk),
 * each a wick_rocm_lfm2_forward_prefill of its own; `cancel` (may be null) is read after every chunk and a non-zero value
 * stops the call there.  *consumed = tokens that made it into the state (0 < consumed <= n for n > 0; 0 and no logits for an
 * empty prompt); `logits` (may be null) are those of the last processed chunk. */
int wick_rocm_lfm2_forward_prefill_chunked(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, const uint32_t *tokens, uint32_t n, uint32_t start_pos,
                                           uint32_t ubatch, const volatile int32_t *cancel, uint32_t *consumed, float *logits);
/* Model::forward_greedy (wick/src/model/metal_lfm2.rs:2151-2200): same step, the pick is made on the device. */
int wick_rocm_lfm2_forward_greedy(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t token, uint32_t pos, uint32_t *next_token);
/* n greedy steps starting with `token` at `pos`, without a host round trip between steps: out_tokens[i] is the
 * pick after step i (which is also step i+1's input). */
int wick_rocm_lfm2_generate_greedy(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t token, uint32_t pos, uint32_t n,
                                   uint32_t *out_tokens);
/* The embedding-input steps of the audio / soft-token paths (Model::supports_embedding_input is true for this backend).
 * forward_from_embedding (wick/src/model/lfm2.rs:2295-2323): a step whose input is `embedding` ([hidden_size] floats, host
 * memory) instead of a token's embedding row -> logits.
 * forward_embedding (:2325-2337, wick/src/model/metal_lfm2.rs:2204-2250): a token step that stops after the output norm ->
 * `hidden` ([hidden_size] floats, host memory; may be null), no LM head.
 * forward_hidden_from_embedding (:2339-2349): both at once. */
int wick_rocm_lfm2_forward_from_embedding(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, const float *embedding, uint32_t pos, float *logits);
int wick_rocm_lfm2_forward_embedding(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t token, uint32_t pos, float *hidden);
int wick_rocm_lfm2_forward_hidden_from_embedding(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, const float *embedding, uint32_t pos,
                                                 float *hidden);

/* Model::snapshot_state / restore_state (wick/src/model/mod.rs:301-315; snapshot_state_locked / restore_state_locked,
 * wick/src/model/metal_lfm2.rs:2535-2634): the model's state after seq_len positions as host bytes, layer by layer in model
 * order -- an attention layer contributes its key rows [0, seq_len) then its value rows [0, seq_len) (f32, or f16 for a model
 * loaded with WICK_ROCM_KV_F16, [seq_len][kv_dim];
 * LayerSnapshot::Attention's k_data, v_data), a gated-conv layer its rolling buffer ((conv_kernel_size - 1) * hidden_size f32;
 * LayerSnapshot::Conv's buffer).  wick_rocm_lfm2_layer_state_bytes gives one layer's share (an attention layer's is split
 * evenly between keys and values), wick_rocm_lfm2_state_bytes the total; `nbytes` must equal it.  The position count itself
 * stays with the caller (StateSnapshot::seq_len), as `pos` does in the step calls. */
size_t wick_rocm_lfm2_layer_state_bytes(const wick_rocm_lfm2 *model, uint32_t layer, uint32_t seq_len);
size_t wick_rocm_lfm2_state_bytes(const wick_rocm_lfm2 *model, uint32_t seq_len);
int wick_rocm_lfm2_snapshot_state(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t seq_len, void *out, size_t nbytes);
int wick_rocm_lfm2_restore_state(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t seq_len, const void *in, size_t nbytes);

/* Model::shift_kv (wick/src/model/lfm2.rs:2507-2516, wick/src/model/metal_lfm2.rs:2473-2531; supports_kv_shift is true for
 * this backend): wick_rocm_kv_shift on every attention layer of a state of seq_len positions; gated-conv layers keep their
 * rolling buffer.  The next step's position is seq_len - shift.  Waits for the shift. */
int wick_rocm_lfm2_shift_kv(wick_rocm_ctx *ctx, wick_rocm_lfm2 *model, uint32_t seq_len, uint32_t n_keep, uint32_t shift);

/* The logits of the last step on the device ([vocab_size] floats). */
const float *wick_rocm_lfm2_logits_device(const wick_rocm_lfm2 *model);

#ifdef __cplusplus
}
#endif
#endif /* WICK_ROCM_LFM2_H */
