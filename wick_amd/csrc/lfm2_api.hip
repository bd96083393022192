// C ABI of include/wick_rocm_lfm2.h: the decode step's non-matmul operations as entry points, and the
// LFM2 model handle (weights, KV caches, conv state, scratch, one captured graph per kind of step).
// Host code only.  The model is a composition of public entry points; a step, a prompt pass or a capture holds the
// model's own lock (the reference's infer_lock) and the context's (recursive) lock from start to end.
#include "../../include/wick_rocm_lfm2.h"

#include <cmath>
#include <cstring>
#include <memory>
#include <vector>

#include "../../include/wick_gguf.h"
#include "wick_rocm_ctx.h"

namespace {

bool misaligned(const void* p, size_t a) { return reinterpret_cast<uintptr_t>(p) % a != 0; }

}  // namespace

extern "C" {

int wick_rocm_embed_row(wick_rocm_ctx* ctx, const wick_rocm_weight* w, uint32_t token, const uint32_t* d_token, float* d_out) {
    WR_ENTER(ctx);
    if (!w || !w->d || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "embed_row: null argument");
    if (!d_token && token >= w->m) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "embed_row: token out of range");
    hipError_t e = launch_embed_row(static_cast<const uint8_t*>(w->d), w->type, w->m, w->k, token, d_token, d_out, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "embed_row launch");
}

int wick_rocm_rmsnorm(wick_rocm_ctx* ctx, const float* d_x, const float* d_weight, float* d_y, uint32_t rows, uint32_t dim, uint32_t x_stride,
                      uint32_t y_stride, float eps) {
    WR_ENTER(ctx);
    if (!d_x || !d_weight || !d_y) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "rmsnorm: null device pointer");
    if (dim == 0 || (rows > 1 && (x_stride < dim || y_stride < dim))) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "rmsnorm: dim 0 or stride < dim");
    hipError_t e = launch_rmsnorm(d_x, d_weight, d_y, rows, dim, x_stride, y_stride, eps, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "rmsnorm launch");
}

size_t wick_rocm_attention_scratch_floats(uint32_t max_seq, uint32_t n_heads, uint32_t head_dim) {
    return attention_scratch_floats(max_seq, n_heads, head_dim);
}

float wick_rocm_rope_theta_scale(uint32_t head_dim, float freq_base) { return powf(freq_base, -2.0f / (float)head_dim); }

int wick_rocm_qk_norm_rope(wick_rocm_ctx* ctx, float* d_q, float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm,
                           float* d_k_cache, float* d_v_cache, uint32_t pos, const uint32_t* d_pos, uint32_t max_seq, uint32_t head_dim,
                           uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale) {
    WR_ENTER(ctx);
    if (!d_q || !d_k || !d_v || !d_q_norm || !d_k_norm || !d_k_cache || !d_v_cache)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "qk_norm_rope: null device pointer");
    if (head_dim == 0 || head_dim % 2u != 0 || head_dim > 256u || n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "qk_norm_rope: head_dim must be even and <= 256, n_kv_heads must divide n_heads");
    if (!d_pos && pos >= max_seq) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "qk_norm_rope: pos beyond the cache");
    hipError_t e = launch_qk_norm_rope(d_q, d_k, d_v, d_q_norm, d_k_norm, d_k_cache, d_v_cache, pos, d_pos, max_seq, head_dim, n_heads, n_kv_heads,
                                       eps, theta_scale, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "qk_norm_rope launch");
}

int wick_rocm_qk_norm_rope_tokens(wick_rocm_ctx* ctx, float* d_q, uint32_t q_stride, float* d_k, const float* d_v, uint32_t kv_stride,
                                  const float* d_q_norm, const float* d_k_norm, float* d_k_cache, float* d_v_cache, uint32_t pos0, uint32_t n,
                                  uint32_t max_seq, uint32_t head_dim, uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale) {
    WR_ENTER(ctx);
    if (!d_q || !d_k || !d_v || !d_q_norm || !d_k_norm || !d_k_cache || !d_v_cache)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "qk_norm_rope_tokens: null device pointer");
    if (head_dim == 0 || head_dim % 2u != 0 || head_dim > 256u || n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "qk_norm_rope_tokens: head_dim must be even and <= 256, n_kv_heads must divide n_heads");
    if (q_stride < n_heads * head_dim || kv_stride < n_kv_heads * head_dim)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "qk_norm_rope_tokens: strides must cover a token's heads");
    if ((uint64_t)pos0 + n > max_seq) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "qk_norm_rope_tokens: positions beyond the cache");
    hipError_t e = launch_qk_norm_rope(d_q, d_k, d_v, d_q_norm, d_k_norm, d_k_cache, d_v_cache, pos0, nullptr, max_seq, head_dim, n_heads, n_kv_heads,
                                       eps, theta_scale, ctx->launch(), n, q_stride, kv_stride);
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "qk_norm_rope_tokens launch");
}

size_t wick_rocm_kv_shift_scratch_floats(uint32_t seq_len, uint32_t n_keep, uint32_t shift, uint32_t n_kv_heads, uint32_t head_dim) {
    if ((uint64_t)n_keep + shift > seq_len) return 0;
    return 2 * (size_t)(seq_len - n_keep - shift) * n_kv_heads * head_dim;
}

int wick_rocm_kv_shift(wick_rocm_ctx* ctx, float* d_k_cache, float* d_v_cache, float* d_scratch, uint32_t seq_len, uint32_t n_keep, uint32_t shift,
                       uint32_t n_kv_heads, uint32_t head_dim, float theta_scale) {
    WR_ENTER(ctx);
    if (!d_k_cache || !d_v_cache) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "kv_shift: null device pointer");
    if (shift == 0) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "kv_shift: shift must be > 0");
    if ((uint64_t)n_keep + shift > seq_len) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "kv_shift: shift range out of bounds (n_keep + shift > seq_len)");
    if (head_dim == 0 || head_dim % 2u != 0 || head_dim > 256u || n_kv_heads == 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "kv_shift: head_dim must be even and <= 256, n_kv_heads > 0");
    if (seq_len - n_keep - shift != 0 && !d_scratch) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "kv_shift: null scratch pointer");
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "kv_shift: not available inside a graph capture");
    hipError_t e = launch_kv_shift(d_k_cache, d_v_cache, d_scratch, seq_len, n_keep, shift, n_kv_heads, head_dim, theta_scale, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "kv_shift launch");
}

int wick_rocm_attention_decode(wick_rocm_ctx* ctx, const float* d_q, const float* d_k_cache, const float* d_v_cache, float* d_out,
                               float* d_scores, uint32_t seq_len, const uint32_t* d_pos, uint32_t max_seq, uint32_t n_heads, uint32_t n_kv_heads,
                               uint32_t head_dim) {
    WR_ENTER(ctx);
    if (!d_q || !d_k_cache || !d_v_cache || !d_out || !d_scores) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention: null device pointer");
    if (head_dim == 0 || head_dim % 4u != 0 || head_dim > 256u || n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "attention: head_dim must be a multiple of 4 and <= 256, n_kv_heads must divide n_heads");
    if (misaligned(d_k_cache, 16) || misaligned(d_q, 16)) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention: q and the key cache must be 16-byte aligned");
    if (!d_pos && seq_len > max_seq) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention: seq_len beyond the cache");
    const float scale = 1.0f / sqrtf((float)head_dim);  // wick/src/model/lfm2.rs:862
    hipError_t e = launch_attention_decode(d_q, d_k_cache, d_v_cache, d_out, d_scores, seq_len, d_pos, max_seq, n_heads, n_kv_heads, head_dim, scale,
                                           ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "attention launch");
}

int wick_rocm_attention_prefill(wick_rocm_ctx* ctx, const float* d_q, uint32_t q_stride, const float* d_k_cache, const float* d_v_cache,
                                float* d_out, uint32_t out_stride, uint32_t pos0, uint32_t n, uint32_t max_seq, uint32_t n_heads,
                                uint32_t n_kv_heads, uint32_t head_dim) {
    WR_ENTER(ctx);
    if (!d_q || !d_k_cache || !d_v_cache || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_prefill: null device pointer");
    if ((head_dim != 32u && head_dim != 64u && head_dim != 128u && head_dim != 256u) || n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "attention_prefill: head_dim must be 32, 64, 128 or 256, n_kv_heads must divide n_heads");
    if (q_stride < n_heads * head_dim || out_stride < n_heads * head_dim || q_stride % 4u != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "attention_prefill: strides must cover n_heads * head_dim (q_stride a multiple of 4)");
    if (misaligned(d_q, 16) || misaligned(d_k_cache, 16) || misaligned(d_v_cache, 16))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_prefill: q and the caches must be 16-byte aligned");
    if ((uint64_t)pos0 + n > max_seq) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_prefill: positions beyond the cache");
    const float scale = 1.0f / sqrtf((float)head_dim);  // wick/src/model/lfm2.rs:862
    hipError_t e = launch_attention_prefill(d_q, d_k_cache, d_v_cache, d_out, nullptr, pos0, nullptr, n, q_stride, out_stride, max_seq, n_heads,
                                            n_kv_heads, head_dim, scale, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "attention_prefill launch");
}

int wick_rocm_attention_prefill_quantize_q8_0(wick_rocm_ctx* ctx, const float* d_q, uint32_t q_stride, const float* d_k_cache, const float* d_v_cache,
                                              int8_t* d_out_q, float* d_out_scales, uint32_t pos0, uint32_t n, uint32_t max_seq, uint32_t n_heads,
                                              uint32_t n_kv_heads, uint32_t head_dim) {
    WR_ENTER(ctx);
    if (!d_q || !d_k_cache || !d_v_cache || !d_out_q || !d_out_scales)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_prefill_quantize: null device pointer");
    if (n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0 || q_stride < n_heads * head_dim)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "attention_prefill_quantize: n_kv_heads must divide n_heads, q_stride must cover n_heads * head_dim");
    if (!attention_prefill_quantize_applies(d_q, d_k_cache, d_v_cache, n, q_stride, head_dim) || misaligned(d_out_q, 4))
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE,
                    "attention_prefill_quantize: needs head_dim 64, n >= 16, q_stride % 4 == 0 and 16-byte aligned q and caches (use attention_prefill + quantize_q8_0)");
    if ((uint64_t)pos0 + n > max_seq) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_prefill_quantize: positions beyond the cache");
    const float scale = 1.0f / sqrtf((float)head_dim);  // wick/src/model/lfm2.rs:862
    hipError_t e = launch_attention_prefill(d_q, d_k_cache, d_v_cache, nullptr, nullptr, pos0, nullptr, n, q_stride, 0, max_seq, n_heads, n_kv_heads,
                                            head_dim, scale, ctx->launch(), d_out_q, d_out_scales);
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "attention_prefill_quantize launch");
}

int wick_rocm_ffn_gate_up_silu_quantize_applies(const wick_rocm_weight* w_gate, const wick_rocm_weight* w_up, uint32_t n) {
    if (!w_gate || !w_up || !w_gate->d_gemm || !w_up->d_gemm) return 0;
    if (w_gate->type != w_up->type || (w_gate->type != kTypeQ4_0 && w_gate->type != kTypeQ8_0)) return 0;
    if (w_gate->m != w_up->m || w_gate->k != w_up->k) return 0;
    return gemm_gated_applies(w_gate->m, n, w_gate->k) ? 1 : 0;
}

int wick_rocm_ffn_gate_up_silu_quantize_q8(wick_rocm_ctx* ctx, const wick_rocm_weight* w_gate, const wick_rocm_weight* w_up, const int8_t* d_quants,
                                           const float* d_scales, uint32_t n, int8_t* d_out_quants, float* d_out_scales) {
    WR_ENTER(ctx);
    if (!w_gate || !w_up || !d_quants || !d_scales || !d_out_quants || !d_out_scales)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "ffn_gate_up_silu_quantize: null argument");
    if (!wick_rocm_ffn_gate_up_silu_quantize_applies(w_gate, w_up, n) || misaligned(d_quants, 16) || misaligned(d_scales, 16))
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE,
                    "ffn_gate_up_silu_quantize: needs two Q4_0 or two Q8_0 weights of one shape, m % 32 == 0, k % 128 == 0, n > 64, more than 256 "
                    "tiles and 16-byte aligned activations (use gemm_q8_multi + silu_mul_quantize_q8_0)");
    hipError_t e = launch_gemm_mfma_gated(w_gate->type, static_cast<const uint8_t*>(w_gate->d_gemm), static_cast<const uint8_t*>(w_up->d_gemm), w_gate->m, w_gate->k,
                                          d_quants, d_scales, n, d_out_quants, d_out_scales, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "ffn_gate_up_silu_quantize launch");
}

int wick_rocm_shortconv_seq(wick_rocm_ctx* ctx, const float* d_proj, float* d_buffer, const float* d_conv_weight, float* d_out, uint32_t hidden,
                            uint32_t kernel_size, uint32_t n) {
    WR_ENTER(ctx);
    if (!d_proj || !d_buffer || !d_conv_weight || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "shortconv_seq: null device pointer");
    if (hidden == 0 || kernel_size == 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "shortconv_seq: hidden and kernel_size must be > 0");
    hipError_t e = launch_shortconv_seq(d_proj, d_buffer, d_conv_weight, d_out, hidden, kernel_size, n, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "shortconv_seq launch");
}

int wick_rocm_shortconv_seq_quantize_q8_0(wick_rocm_ctx* ctx, const float* d_proj, float* d_buffer, const float* d_conv_weight, int8_t* d_out_q,
                                          float* d_out_scales, uint32_t hidden, uint32_t kernel_size, uint32_t n) {
    WR_ENTER(ctx);
    if (!d_proj || !d_buffer || !d_conv_weight || !d_out_q || !d_out_scales)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "shortconv_seq_quantize: null device pointer");
    if (hidden == 0 || kernel_size == 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "shortconv_seq_quantize: hidden and kernel_size must be > 0");
    if (!shortconv_seq_quantize_applies(d_proj, d_buffer, hidden) || misaligned(d_out_q, 4))
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "shortconv_seq_quantize: needs hidden % 32 == 0 and 16-byte aligned buffers (use shortconv_seq + quantize_q8_0)");
    hipError_t e = launch_shortconv_seq_quantize(d_proj, d_buffer, d_conv_weight, d_out_q, d_out_scales, hidden, kernel_size, n, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "shortconv_seq_quantize launch");
}

size_t wick_rocm_attention_block_scratch_bytes(uint32_t max_seq, uint32_t n_heads, uint32_t head_dim) {
    return attention_scratch_floats(max_seq, n_heads, head_dim) * sizeof(float);
}

}  // extern "C"

// The attention block over caches of either element type (the model handle's route; the public entry point below is the
// f32-cache form).
static int attention_block_kv(wick_rocm_ctx* ctx, float* d_q, float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm,
                              void* d_k_cache, void* d_v_cache, float* d_out, void* d_scratch, uint32_t pos, const uint32_t* d_pos,
                              uint32_t max_seq, uint32_t head_dim, uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale, bool kv_f16) {
    WR_ENTER(ctx);
    if (!d_q || !d_k || !d_v || !d_q_norm || !d_k_norm || !d_k_cache || !d_v_cache || !d_out || !d_scratch)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_block: null device pointer");
    if (head_dim == 0 || head_dim % 4u != 0 || head_dim > 256u || n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "attention_block: head_dim must be a multiple of 4 and <= 256, n_kv_heads must divide n_heads");
    if (misaligned(d_k_cache, 16) || misaligned(d_q, 16) || misaligned(d_scratch, 16))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_block: q, the key cache and the scratch must be 16-byte aligned");
    if (!d_pos && pos >= max_seq) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "attention_block: pos beyond the cache");
    const float scale = 1.0f / sqrtf((float)head_dim);  // wick/src/model/lfm2.rs:862
    float* partials = static_cast<float*>(d_scratch);
    hipError_t e;
    if (attention_layer_applies(head_dim)) {
        e = launch_attention_layer(d_q, d_k, d_v, d_q_norm, d_k_norm, d_k_cache, d_v_cache, d_out, partials, pos, d_pos, max_seq, n_heads,
                                   n_kv_heads, head_dim, eps, theta_scale, scale, ctx->launch(), kv_f16);
    } else {
        e = launch_qk_norm_rope(d_q, d_k, d_v, d_q_norm, d_k_norm, d_k_cache, d_v_cache, pos, d_pos, max_seq, head_dim, n_heads, n_kv_heads, eps,
                                theta_scale, ctx->launch(), 1, 0, 0, kv_f16);
        if (e == hipSuccess)
            e = launch_attention_decode(d_q, d_k_cache, d_v_cache, d_out, partials, pos + 1u, d_pos, max_seq, n_heads, n_kv_heads, head_dim, scale,
                                        ctx->launch(), kv_f16);
    }
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "attention_block launch");
}

extern "C" {

int wick_rocm_attention_block(wick_rocm_ctx* ctx, float* d_q, float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm,
                              float* d_k_cache, float* d_v_cache, float* d_out, void* d_scratch, uint32_t pos, const uint32_t* d_pos,
                              uint32_t max_seq, uint32_t head_dim, uint32_t n_heads, uint32_t n_kv_heads, float eps, float theta_scale) {
    return attention_block_kv(ctx, d_q, d_k, d_v, d_q_norm, d_k_norm, d_k_cache, d_v_cache, d_out, d_scratch, pos, d_pos, max_seq, head_dim, n_heads,
                              n_kv_heads, eps, theta_scale, false);
}

int wick_rocm_shortconv_step(wick_rocm_ctx* ctx, const float* d_proj, float* d_buffer, const float* d_conv_weight, float* d_out, uint32_t hidden,
                             uint32_t kernel_size) {
    WR_ENTER(ctx);
    if (!d_proj || !d_conv_weight || !d_out || (!d_buffer && kernel_size > 1)) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "shortconv: null device pointer");
    if (hidden == 0 || kernel_size == 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "shortconv: hidden and kernel_size must be > 0");
    hipError_t e = launch_shortconv_step(d_proj, d_buffer, d_conv_weight, d_out, hidden, kernel_size, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "shortconv launch");
}

int wick_rocm_silu_mul(wick_rocm_ctx* ctx, float* d_gate, const float* d_up, uint32_t n) {
    WR_ENTER(ctx);
    if (!d_gate || !d_up) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "silu_mul: null device pointer");
    hipError_t e = launch_silu_mul(d_gate, d_up, n, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "silu_mul launch");
}

int wick_rocm_rmsnorm_quantize_q8_0(wick_rocm_ctx* ctx, const float* d_x, const float* d_weight, uint32_t rows, uint32_t dim, uint32_t x_stride,
                                    float eps, int8_t* d_quants, float* d_scales) {
    WR_ENTER(ctx);
    if (!d_x || !d_weight || !d_quants || !d_scales) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "rmsnorm_quantize: null device pointer");
    if (dim == 0 || dim % 32u != 0 || x_stride < dim || x_stride % 4u != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "rmsnorm_quantize: dim % 32 != 0 or stride < dim or stride % 4 != 0");
    if (misaligned(d_x, 16) || misaligned(d_weight, 16) || misaligned(d_quants, 4))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "rmsnorm_quantize: x and weight must be 16-byte aligned");
    hipError_t e = launch_rmsnorm_quantize(d_x, d_weight, rows, dim, x_stride, eps, d_quants, d_scales, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "rmsnorm_quantize launch");
}

int wick_rocm_silu_mul_quantize_q8_0(wick_rocm_ctx* ctx, const float* d_gate, const float* d_up, uint32_t rows, uint32_t dim, int8_t* d_quants,
                                     float* d_scales) {
    WR_ENTER(ctx);
    if (!d_gate || !d_up || !d_quants || !d_scales) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "silu_mul_quantize: null device pointer");
    if (dim % 32u != 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "silu_mul_quantize: dim % 32 != 0");
    if (misaligned(d_gate, 16) || misaligned(d_up, 16) || misaligned(d_quants, 4))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "silu_mul_quantize: gate and up must be 16-byte aligned");
    hipError_t e = launch_silu_mul_quantize(d_gate, d_up, rows, dim, d_quants, d_scales, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "silu_mul_quantize launch");
}

int wick_rocm_argmax(wick_rocm_ctx* ctx, const float* d_logits, uint32_t n, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos) {
    WR_ENTER(ctx);
    if (!d_logits || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "argmax: null device pointer");
    if (misaligned(d_logits, 16)) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "argmax: logits must be 16-byte aligned");
    if (!ctx->argmax_partial) {
        if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "argmax: first use inside a graph capture (call it once before capturing)");
        WR_HIP(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->argmax_partial), kArgmaxPartials * sizeof(unsigned long long)));
    }
    hipError_t e = launch_argmax(d_logits, n, ctx->argmax_partial, d_out, d_token, d_pos, nullptr, 0, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "argmax launch");
}

}  // extern "C"

namespace {

// Output norm + LM head + greedy pick (lock held).  A Q6_K head norms and quantizes its input itself and leaves one pick key
// per wave, so the pick's first stage is not launched: two launches instead of four.  `history` / `emb_out`: the model's
// extras of launch_argmax (may be null).
int lm_head_greedy_locked(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const float* d_x, const float* d_norm_weight, float eps, float* d_logits,
                          unsigned long long* d_partial, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos, uint32_t* d_history,
                          uint32_t history_len, float* d_emb_out) {
    const uint8_t* wd = static_cast<const uint8_t*>(w->d);
    const uint32_t waves = w->type == kTypeQ6_K ? gemv_q6k_waves(w->m, w->k, ctx->num_cus) : 0u;
    if (waves != 0 && waves <= kArgmaxPartials && !misaligned(d_x, 16) && !misaligned(d_norm_weight, 16)) {
        hipError_t e = launch_gemv_q6k_rmsnorm(wd, w->m, w->k, d_x, d_norm_weight, eps, d_logits, 0, ctx->num_cus, ctx->launch(), d_partial);
        if (e != hipSuccess) return fail_hip(ctx, e, "Q6_K gemv launch");
        e = launch_argmax_final(d_partial, waves, w->m, d_out, d_token, d_pos, d_history, history_len, ctx->launch(), wd, w->type, w->m, w->k, d_emb_out);
        return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "argmax launch");
    }
    if (int rc = wick_rocm_gemv_rmsnorm_f32_multi(ctx, &w, &d_logits, 1, d_x, d_norm_weight, eps, 0)) return rc;
    hipError_t e = launch_argmax(d_logits, w->m, d_partial, d_out, d_token, d_pos, d_history, history_len, ctx->launch(), wd, w->type, w->m, w->k, d_emb_out);
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "argmax launch");
}

}  // namespace

extern "C" int wick_rocm_lm_head_greedy_f32(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const float* d_x, const float* d_norm_weight, float eps,
                                            float* d_logits, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos) {
    WR_ENTER(ctx);
    if (!w || !w->d) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "null weight handle");
    if (!d_x || !d_norm_weight || !d_logits || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lm_head_greedy: null device pointer");
    if (misaligned(d_logits, 16)) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lm_head_greedy: logits must be 16-byte aligned");
    if (!ctx->argmax_partial) {
        if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "lm_head_greedy: first use inside a graph capture (call it once before capturing)");
        WR_HIP(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->argmax_partial), kArgmaxPartials * sizeof(unsigned long long)));
    }
    return lm_head_greedy_locked(ctx, w, d_x, d_norm_weight, eps, d_logits, ctx->argmax_partial, d_out, d_token, d_pos, nullptr, 0, nullptr);
}

// ---------------------------------------------------------------------------------------------
// The model.

namespace {

struct LayerWeights {
    uint32_t n_kv = 0;  // 0: gated-conv layer
    wick_rocm_weight *in_proj = nullptr, *out_proj = nullptr;               // conv
    wick_rocm_weight *q = nullptr, *k = nullptr, *v = nullptr, *o = nullptr;  // attention
    wick_rocm_weight *gate = nullptr, *up = nullptr, *down = nullptr;
    float *attn_norm = nullptr, *ffn_norm = nullptr, *q_norm = nullptr, *k_norm = nullptr, *conv_w = nullptr;
    void *k_cache = nullptr, *v_cache = nullptr;  // [max_seq][kv_dim] of the model's cache element type
    float* conv_state = nullptr;
    bool conv_fused = false;  // gated-conv layer whose convolution rides in its out projection and gate / up launches
};

}  // namespace

struct wick_rocm_lfm2 {
    wick_rocm_lfm2_config cfg{};
    std::vector<LayerWeights> layers;
    wick_rocm_weight* embd = nullptr;
    float* out_norm = nullptr;
    std::vector<wick_rocm_weight*> weights;  // everything uploaded, for release
    std::vector<void*> buffers;              // every device buffer, for release
    size_t bytes = 0;
    float theta_scale = 0.0f;
    // step scratch (device)
    float *hidden = nullptr, *proj = nullptr, *gated = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr,
          *gate = nullptr, *scores = nullptr, *logits = nullptr;
    uint32_t *d_token = nullptr, *d_pos = nullptr, *d_pick = nullptr, *d_history = nullptr;
    unsigned long long* d_argmax_partial = nullptr;
    // prompt (prefill) buffers for up to `prefill_cap` tokens, allocated by the first prefill
    uint32_t prefill_cap = 0;
    float *pX = nullptr, *pA = nullptr, *pG = nullptr, *pGate = nullptr, *pUp = nullptr, *pS = nullptr, *pS2 = nullptr, *pAttn = nullptr;
    int8_t *pQ = nullptr, *pQ2 = nullptr;
    uint32_t* pTokens = nullptr;
    void* shift_stage = nullptr;   // staging rows of a context shift, allocated by the first one
    bool kv_f16 = false;           // the KV caches hold f16 rows (wick_rocm_lfm2_load_kv); f32 otherwise
    size_t kv_elem() const { return kv_f16 ? 2 : 4; }
    wick_rocm_graph* g_step[3] = {nullptr, nullptr, nullptr};  // one captured step per StepMode
    bool use_graph = true;
    std::mutex mu;
};

namespace {

// What a step ends with: the tied LM head's logits, the greedy pick on top of them, or only the hidden state after the
// output norm (forward_embedding / forward_hidden_from_embedding, wick/src/model/lfm2.rs:2325-2349).
enum StepMode { kStepLogits = 0, kStepGreedy = 1, kStepHidden = 2 };

int ctx_fail(wick_rocm_ctx* ctx, int code, const std::string& what) {
    std::lock_guard<std::recursive_mutex> lk(ctx->mu);
    return fail(ctx, code, what.c_str());
}

int alloc(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, size_t nbytes, void** out) {
    if (int rc = wick_rocm_buffer_alloc(ctx, nbytes, out)) return rc;
    m->buffers.push_back(*out);
    m->bytes += nbytes;
    return WICK_ROCM_OK;
}

template <typename T>
int alloc_t(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, size_t count, T** out) {
    return alloc(ctx, m, count * sizeof(T), reinterpret_cast<void**>(out));
}

// An f32 tensor of exactly `count` elements -> device buffer (the reference's get_tensor(..).to_f32_vec()).
int upload_f32(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, const wick_gguf* g, const std::string& name, uint64_t count, float** out) {
    int type = 0;
    uint32_t nd = 0;
    uint64_t dims[8], off = 0, size = 0;
    if (wick_gguf_tensor_info(g, name.c_str(), &type, &nd, dims, &off, &size) != 0)
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, std::string("lfm2_load: ") + wick_gguf_last_error());
    if (type != 0) return ctx_fail(ctx, WICK_ROCM_ERR_UNSUPPORTED_DTYPE, "lfm2_load: " + name + " must be F32");
    if (size != count * 4) return ctx_fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "lfm2_load: " + name + " has an unexpected element count");
    const void* data = nullptr;
    size_t nbytes = 0;
    if (wick_gguf_tensor_data(g, name.c_str(), &data, &nbytes) != 0)
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, std::string("lfm2_load: ") + wick_gguf_last_error());
    if (int rc = alloc_t(ctx, m, count, out)) return rc;
    return wick_rocm_upload(ctx, *out, data, nbytes);
}

int upload_weight(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, const wick_gguf* g, const std::string& name, uint32_t rows, uint32_t cols,
                  wick_rocm_weight** out) {
    if (int rc = wick_rocm_weight_from_gguf(ctx, g, name.c_str(), out)) return rc;
    m->weights.push_back(*out);
    m->bytes += (*out)->nbytes + (*out)->gemm_bytes;
    if ((*out)->m != rows || (*out)->k != cols)
        return ctx_fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "lfm2_load: " + name + " has an unexpected shape");
    return WICK_ROCM_OK;
}

void release(wick_rocm_ctx* ctx, wick_rocm_lfm2* m) {
    wick_rocm_sync(ctx);
    for (wick_rocm_graph* g : m->g_step)
        if (g) wick_rocm_graph_destroy(ctx, g);
    for (wick_rocm_weight* w : m->weights) wick_rocm_weight_free(ctx, w);
    for (void* b : m->buffers) wick_rocm_buffer_free(ctx, b);
    delete m;
}

// y_i = W_i rmsnorm(x) for 1..3 weights that share x, the norm folded into the projection's launch; one launch when
// the weights' types agree.
int gemv_normed(wick_rocm_ctx* ctx, std::initializer_list<const wick_rocm_weight*> ws, std::initializer_list<float*> ys, const float* x,
                const float* norm_weight, float eps) {
    bool same = true;
    for (const wick_rocm_weight* w : ws) same = same && w->type == (*ws.begin())->type;
    if (same) return wick_rocm_gemv_rmsnorm_f32_multi(ctx, ws.begin(), ys.begin(), (uint32_t)ws.size(), x, norm_weight, eps, 0);
    auto y = ys.begin();
    for (const wick_rocm_weight* const& w : ws) {
        float* const out = *y++;
        if (int rc = wick_rocm_gemv_rmsnorm_f32_multi(ctx, &w, &out, 1, x, norm_weight, eps, 0)) return rc;
    }
    return WICK_ROCM_OK;
}

// y += W x (the residual form of the out / output projections).
int gemv_residual(wick_rocm_ctx* ctx, const wick_rocm_weight* w, float* y, const float* x) {
    return wick_rocm_matmul_f32(ctx, w, x, 0, 1, w->k, y, 0, w->m, 1);
}

// Enqueues one decode step that reads token / pos from the device: run_layers + the tied LM head
// (wick/src/model/lfm2.rs:1020-1124, 2258-2289), optionally the greedy pick.
int enqueue_step(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, StepMode mode) {
    const wick_rocm_lfm2_config& c = m->cfg;
    const uint32_t hs = c.hidden_size, hd = hs / c.n_heads;
    // m->hidden already holds the token's embedding row: set_step (or the previous step's greedy pick) looked it up
    int rc = 0;
    for (uint32_t i = 0; rc == 0 && i < c.n_layers; i++) {
        const LayerWeights& L = m->layers[i];
        if (L.n_kv == 0) {
            if ((rc = gemv_normed(ctx, {L.in_proj}, {m->proj}, m->hidden, L.attn_norm, c.rms_norm_eps))) break;
            if (L.conv_fused) {  // the convolution in the out projection's prologue, its state advance in the gate / up launch below
                if ((rc = wick_rocm_shortconv_out_proj_f32(ctx, L.out_proj, m->proj, L.conv_state, L.conv_w, c.conv_kernel_size, m->hidden, 1))) break;
            } else {
                if ((rc = wick_rocm_shortconv_step(ctx, m->proj, L.conv_state, L.conv_w, m->gated, hs, c.conv_kernel_size))) break;
                if ((rc = gemv_residual(ctx, L.out_proj, m->hidden, m->gated))) break;
            }
        } else {
            if ((rc = gemv_normed(ctx, {L.q, L.k, L.v}, {m->q, m->k, m->v}, m->hidden, L.attn_norm, c.rms_norm_eps))) break;
            if ((rc = attention_block_kv(ctx, m->q, m->k, m->v, L.q_norm, L.k_norm, L.k_cache, L.v_cache, m->attn, m->scores, 0, m->d_pos,
                                         c.max_seq_len, hd, c.n_heads, L.n_kv, c.rms_norm_eps, m->theta_scale, m->kv_f16)))
                break;
            if ((rc = gemv_residual(ctx, L.o, m->hidden, m->attn))) break;
        }
        // gate = silu(W_gate n(hidden)) * (W_up n(hidden)); hidden += W_down gate
        if (L.conv_fused)
            rc = wick_rocm_ffn_gate_up_conv_advance_f32(ctx, L.gate, L.up, m->hidden, L.ffn_norm, c.rms_norm_eps, m->gate, m->proj, L.conv_state, hs,
                                                        c.conv_kernel_size);
        else
            rc = wick_rocm_ffn_gate_up_f32(ctx, L.gate, L.up, m->hidden, L.ffn_norm, c.rms_norm_eps, m->gate);
        if (rc) break;
        rc = gemv_residual(ctx, L.down, m->hidden, m->gate);
    }
    if (rc) return rc;
    if (mode == kStepHidden) return wick_rocm_rmsnorm(ctx, m->hidden, m->out_norm, m->gated, 1, hs, hs, hs, c.rms_norm_eps);  // m->gated is free here
    if (mode != kStepGreedy) return gemv_normed(ctx, {m->embd}, {m->logits}, m->hidden, m->out_norm, c.rms_norm_eps);
    std::lock_guard<std::recursive_mutex> lk(ctx->mu);
    return lm_head_greedy_locked(ctx, m->embd, m->hidden, m->out_norm, c.rms_norm_eps, m->logits, m->d_argmax_partial, m->d_pick, m->d_token, m->d_pos,
                                 m->d_history, c.max_seq_len, m->hidden);
}

int step_graph(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, StepMode mode, wick_rocm_graph** out) {
    wick_rocm_graph*& g = m->g_step[mode];
    if (g && graph_is_stale(ctx, g)) {  // the context's scratch moved since the capture (another model, a wider matmul): capture again
        wick_rocm_graph_destroy(ctx, g);
        g = nullptr;
    }
    if (!g) {
        if (int rc = wick_rocm_graph_begin(ctx)) return rc;
        const int rc = enqueue_step(ctx, m, mode);
        wick_rocm_graph* captured = nullptr;
        const int rc_end = wick_rocm_graph_end(ctx, &captured);  // always end the capture
        if (rc) {
            if (captured) wick_rocm_graph_destroy(ctx, captured);
            return rc;
        }
        if (rc_end) return rc_end;
        g = captured;
    }
    *out = g;
    return WICK_ROCM_OK;
}

// One step on the context's stream: a replay of the captured graph, or the same launches enqueued one by one.
int run_step(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, StepMode mode) {
    // per-dispatch timing cannot see inside a graph: while it is on, steps are enqueued launch by launch
    bool timing;
    {
        std::lock_guard<std::recursive_mutex> lk(ctx->mu);
        timing = ctx->timer.enabled;
    }
    if (!m->use_graph || timing) return enqueue_step(ctx, m, mode);
    wick_rocm_graph* g = nullptr;
    if (int rc = step_graph(ctx, m, mode, &g)) return rc;
    return wick_rocm_graph_launch(ctx, g);
}

constexpr uint32_t kPromptAsStepsMax = 2;  // prompts this short run as single steps (prefill_locked)
constexpr uint32_t kPrefillChunk = 2048;  // tokens per pass of a prompt (the reference's Metal path uses 512, MAX_PREFILL_TOKENS, wick/src/model/metal_lfm2.rs:25;
                                          // 288 GB of HBM afford four times that, and the GEMMs run better the wider they are)

int ensure_prefill_buffers(wick_rocm_ctx* ctx, wick_rocm_lfm2* m) {
    if (m->prefill_cap) return WICK_ROCM_OK;
    const wick_rocm_lfm2_config& c = m->cfg;
    const size_t P = c.max_seq_len < kPrefillChunk ? c.max_seq_len : kPrefillChunk;
    const size_t hs = c.hidden_size, inter = c.intermediate_size, hd = hs / c.n_heads, wide = hs > inter ? hs : inter;
    int rc;
    if ((rc = alloc_t(ctx, m, P * hs, &m->pX)) || (rc = alloc_t(ctx, m, P * 3 * hs, &m->pA)) ||
        (rc = alloc_t(ctx, m, P * hs, &m->pG)) || (rc = alloc_t(ctx, m, P * inter, &m->pGate)) || (rc = alloc_t(ctx, m, P * inter, &m->pUp)) ||
        (rc = alloc_t(ctx, m, P * wide, &m->pQ)) || (rc = alloc_t(ctx, m, P * (wide / 32), &m->pS)) ||
        (rc = alloc_t(ctx, m, P * inter, &m->pQ2)) || (rc = alloc_t(ctx, m, P * (inter / 32), &m->pS2)) ||
        (rc = alloc_t(ctx, m, attention_prefill_scratch_floats((uint32_t)P, c.n_heads, (uint32_t)hd), &m->pAttn)) ||
        (rc = alloc_t(ctx, m, P, &m->pTokens)))
        return rc;
    // room for the K shares of a split projection, once: no prompt then regrows the context's scratch (a regrow waits for the
    // stream and makes every captured step graph stale)
    if ((rc = wick_rocm_reserve_scratch(ctx, (uint32_t)P, 0))) return rc;
    m->prefill_cap = (uint32_t)P;
    return WICK_ROCM_OK;
}

// y[n][y_stride] (+)= W x for n tokens: quantized activations (q, s) against one weight, token-major output.
int gemm(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const wick_rocm_lfm2* m, uint32_t n, float* y, uint32_t y_stride, int accumulate) {
    return wick_rocm_gemm_q8(ctx, w, m->pQ, m->pS, n, y, y_stride, WICK_ROCM_LAYOUT_TOKEN_MAJOR, accumulate);
}

// The same for projections that share their input (Q / K / V, gate / up): one launch when dtype and k agree.
int gemm_group(wick_rocm_ctx* ctx, std::initializer_list<const wick_rocm_weight*> ws, std::initializer_list<float*> ys, const wick_rocm_lfm2* m,
               uint32_t n, uint32_t y_stride) {
    bool same = true;
    for (const wick_rocm_weight* w : ws) same = same && w->type == (*ws.begin())->type && w->k == (*ws.begin())->k;
    if (same) return wick_rocm_gemm_q8_multi(ctx, ws.begin(), ys.begin(), (uint32_t)ws.size(), m->pQ, m->pS, n, y_stride, WICK_ROCM_LAYOUT_TOKEN_MAJOR, 0);
    auto y = ys.begin();
    for (const wick_rocm_weight* w : ws)
        if (int rc = gemm(ctx, w, m, n, *y++, y_stride, 0)) return rc;
    return WICK_ROCM_OK;
}

// One pass of a prompt: n <= prefill_cap tokens (already in pTokens) at positions pos0 .. pos0 + n - 1.  The batched form
// of enqueue_step (prefill_layers_and_logits, wick/src/model/lfm2.rs:1139-2109): projections as GEMMs over the tokens,
// the short conv per (token, channel) with the rolling state behind it, the KV append per token, causal attention per
// (head, token).
int enqueue_prompt_pass(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, uint32_t n, uint32_t pos0, bool lookup = true) {
    const wick_rocm_lfm2_config& c = m->cfg;
    const uint32_t hs = c.hidden_size, hd = hs / c.n_heads, inter = c.intermediate_size;
    const float scale = 1.0f / sqrtf((float)hd);
    auto locked = [&](auto&& launch, const char* what) {
        std::lock_guard<std::recursive_mutex> lk(ctx->mu);
        const hipError_t e = launch();
        return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, what);
    };
    // the pass's input rows: the tokens' embedding rows, or what the caller put into pX (a prompt given as embeddings)
    int rc = !lookup ? WICK_ROCM_OK
                     : locked([&] { return launch_embed_rows(static_cast<const uint8_t*>(m->embd->d), m->embd->type, m->embd->m, hs, m->pTokens, n, m->pX, ctx->launch()); },
                              "embed_rows launch");
    // A residual projection and the norm + quantizer behind it go out as one call (a split projection's shares are then added
    // up by the norm's kernel): the out projection with the FFN norm, the down projection with the NEXT layer's first norm.
    auto project_and_norm = [&](const wick_rocm_weight* w, const int8_t* q, const float* s, const float* norm_weight) {
        return wick_rocm_gemm_q8_residual_rmsnorm_quantize(ctx, w, q, s, n, m->pX, hs, norm_weight, c.rms_norm_eps, m->pQ, m->pS);
    };
    for (uint32_t i = 0; rc == 0 && i < c.n_layers; i++) {
        const LayerWeights& L = m->layers[i];
        const float* next_norm = i + 1 < c.n_layers ? m->layers[i + 1].attn_norm : nullptr;
        // layer 0 norms its own input; every later layer's came with the previous layer's down projection
        if (i == 0 && (rc = wick_rocm_rmsnorm_quantize_q8_0(ctx, m->pX, L.attn_norm, n, hs, hs, c.rms_norm_eps, m->pQ, m->pS))) break;
        bool quantized = false;
        if (L.n_kv == 0) {
            if ((rc = gemm(ctx, L.in_proj, m, n, m->pA, 3 * hs, 0))) break;
            quantized = shortconv_seq_quantize_applies(m->pA, L.conv_state, hs);
            if ((rc = locked([&] {
                     return quantized ? launch_shortconv_seq_quantize(m->pA, L.conv_state, L.conv_w, m->pQ, m->pS, hs, c.conv_kernel_size, n, ctx->launch())
                                      : launch_shortconv_seq(m->pA, L.conv_state, L.conv_w, m->pG, hs, c.conv_kernel_size, n, ctx->launch());
                 }, "shortconv_seq launch")))
                break;
        } else {
            const uint32_t kvd = L.n_kv * hd, S = hs + 2 * kvd;  // a token's [q | k | v]
            float *q = m->pA, *k = m->pA + hs, *v = m->pA + hs + kvd;
            if ((rc = gemm_group(ctx, {L.q, L.k, L.v}, {q, k, v}, m, n, S))) break;
            if ((rc = locked([&] {
                     return launch_qk_norm_rope(q, k, v, L.q_norm, L.k_norm, L.k_cache, L.v_cache, pos0, nullptr, c.max_seq_len, hd, c.n_heads, L.n_kv,
                                                c.rms_norm_eps, m->theta_scale, ctx->launch(), n, S, S, m->kv_f16);
                 }, "qk_norm_rope launch")))
                break;
            if (attention_layer_applies(hd)) {
                quantized = attention_prefill_quantize_applies(q, L.k_cache, L.v_cache, n, S, hd);
                rc = locked([&] {
                    return launch_attention_prefill(q, L.k_cache, L.v_cache, m->pG, m->pAttn, pos0, nullptr, n, S, hs, c.max_seq_len, c.n_heads, L.n_kv, hd,
                                                    scale, ctx->launch(), quantized ? m->pQ : nullptr, quantized ? m->pS : nullptr, m->kv_f16);
                }, "attention_prefill launch");
            } else {  // head dims without a batched kernel: the decode kernel, token by token
                for (uint32_t j = 0; rc == 0 && j < n; j++)
                    rc = locked([&] {
                        return launch_attention_decode(q + (size_t)j * S, L.k_cache, L.v_cache, m->pG + (size_t)j * hs, m->scores, pos0 + j + 1, nullptr,
                                                       c.max_seq_len, c.n_heads, L.n_kv, hd, scale, ctx->launch(), m->kv_f16);
                    }, "attention_decode launch");
            }
            if (rc) break;
        }
        // the out projection's input: already Q8_0 blocks when its producer wrote them itself
        if (!quantized && (rc = wick_rocm_quantize_q8_0(ctx, m->pG, n, hs, hs, m->pQ, m->pS))) break;
        if ((rc = project_and_norm(L.n_kv == 0 ? L.out_proj : L.o, m->pQ, m->pS, L.ffn_norm))) break;  // hidden += out projection; FFN norm
        if (L.gate->type == kTypeQ4_0 && L.gate->k <= 1024 && wick_rocm_ffn_gate_up_silu_quantize_applies(L.gate, L.up, n)) {
            // gate, up, SiLU gate and the down projection's quantizer in one launch; its output cannot overwrite its own input.
            // (Where it pays, measured on one GPU against GEMM + gate kernel: Q4_0 with k = 1024 6-7 % faster; k = 2048 2-8 %
            // slower -- the epilogue's exp / divide work sits on the vector ALU that bounds the GEMM; Q8_0, whose kernel is
            // two registers over its budget, 11 % slower.)
            if ((rc = wick_rocm_ffn_gate_up_silu_quantize_q8(ctx, L.gate, L.up, m->pQ, m->pS, n, m->pQ2, m->pS2))) break;
            rc = next_norm ? project_and_norm(L.down, m->pQ2, m->pS2, next_norm)
                           : wick_rocm_gemm_q8(ctx, L.down, m->pQ2, m->pS2, n, m->pX, hs, WICK_ROCM_LAYOUT_TOKEN_MAJOR, 1);
            continue;
        }
        if ((rc = gemm_group(ctx, {L.gate, L.up}, {m->pGate, m->pUp}, m, n, inter))) break;
        if ((rc = wick_rocm_silu_mul_quantize_q8_0(ctx, m->pGate, m->pUp, n, inter, m->pQ, m->pS))) break;
        rc = next_norm ? project_and_norm(L.down, m->pQ, m->pS, next_norm) : gemm(ctx, L.down, m, n, m->pX, hs, 1);
    }
    return rc;
}

int set_step(wick_rocm_ctx* ctx, wick_rocm_lfm2* m, uint32_t token, uint32_t pos) {
    std::lock_guard<std::recursive_mutex> lk(ctx->mu);
    hipError_t e = launch_set_step(m->d_token, token, m->d_pos, pos, ctx->launch(), static_cast<const uint8_t*>(m->embd->d), m->embd->type, m->embd->m,
                                   m->cfg.hidden_size, m->hidden);
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "set_step launch");
}

int check_step(wick_rocm_ctx* ctx, const wick_rocm_lfm2* m, uint32_t token, uint32_t pos, uint32_t n) {
    if (token >= m->cfg.vocab_size) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: token_id out of range");
    if ((uint64_t)pos + n > m->cfg.max_seq_len) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: position beyond the context size");
    return WICK_ROCM_OK;
}

// Walks the layers' state in snapshot order and hands every piece (device pointer, bytes) to `piece`.
template <typename F>
int for_each_state_piece(const wick_rocm_lfm2* model, uint32_t seq_len, F&& piece) {
    const wick_rocm_lfm2_config& c = model->cfg;
    for (const LayerWeights& L : model->layers) {
        if (L.n_kv) {
            const size_t half = (size_t)seq_len * L.n_kv * (c.hidden_size / c.n_heads) * model->kv_elem();
            if (half == 0) continue;
            if (int rc = piece(L.k_cache, half)) return rc;
            if (int rc = piece(L.v_cache, half)) return rc;
        } else if (L.conv_state) {
            if (int rc = piece(L.conv_state, (size_t)(c.conv_kernel_size - 1) * c.hidden_size * sizeof(float))) return rc;
        }
    }
    return WICK_ROCM_OK;
}

}  // namespace

extern "C" {

int wick_rocm_lfm2_load(wick_rocm_ctx* ctx, const wick_gguf* g, uint32_t context_size, wick_rocm_lfm2** out) {
    return wick_rocm_lfm2_load_kv(ctx, g, context_size, WICK_ROCM_KV_F32, out);
}

int wick_rocm_lfm2_kv_dtype(const wick_rocm_lfm2* model) { return model && model->kv_f16 ? WICK_ROCM_KV_F16 : WICK_ROCM_KV_F32; }

int wick_rocm_lfm2_load_kv(wick_rocm_ctx* ctx, const wick_gguf* g, uint32_t context_size, int kv_dtype, wick_rocm_lfm2** out) {
    if (!ctx) return WICK_ROCM_ERR_INVALID_ARG;
    if (!g || !out) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2_load: null argument");
    *out = nullptr;
    if (kv_dtype != WICK_ROCM_KV_F32 && kv_dtype != WICK_ROCM_KV_F16)
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2_load: kv_dtype must be WICK_ROCM_KV_F32 or WICK_ROCM_KV_F16");
    if (context_size == 0) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2_load: context_size must be > 0");

    // metadata, wick/src/model/lfm2.rs:104-136
    wick_rocm_lfm2_config c{};
    struct Key {
        const char* name;
        uint32_t* dst;
    } required[] = {{"lfm2.block_count", &c.n_layers},
                    {"lfm2.embedding_length", &c.hidden_size},
                    {"lfm2.feed_forward_length", &c.intermediate_size},
                    {"lfm2.attention.head_count", &c.n_heads},
                    {"lfm2.vocab_size", &c.vocab_size}};
    for (const Key& k : required)
        if (wick_gguf_get_u32(g, k.name, k.dst) != 0) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, std::string("lfm2_load: missing ") + k.name);
    uint32_t ctx_len = 128000, l_cache = 3;
    wick_gguf_get_u32(g, "lfm2.context_length", &ctx_len);
    c.max_seq_len = context_size < ctx_len ? context_size : ctx_len;
    c.rope_theta = 1000000.0f, c.rms_norm_eps = 1e-5f;
    wick_gguf_get_f32(g, "lfm2.rope.freq_base", &c.rope_theta);
    wick_gguf_get_f32(g, "lfm2.attention.layer_norm_rms_epsilon", &c.rms_norm_eps);
    wick_gguf_get_u32(g, "lfm2.shortconv.l_cache", &l_cache);  // kernel size, default 3 (wick/src/model/lfm2.rs:650)
    c.conv_kernel_size = l_cache;
    const void* kv_data = nullptr;
    uint64_t kv_count = 0;
    if (wick_gguf_get_array(g, "lfm2.attention.head_count_kv", WICK_GGUF_T_I32, &kv_data, &kv_count) != 0)
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2_load: missing lfm2.attention.head_count_kv");
    if (kv_count < c.n_layers) return ctx_fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "lfm2_load: head_count_kv array shorter than block_count");
    if (c.n_layers == 0 || c.hidden_size == 0 || c.n_heads == 0 || c.hidden_size % c.n_heads != 0 || c.vocab_size == 0 || c.conv_kernel_size == 0 ||
        c.intermediate_size == 0)
        return ctx_fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "lfm2_load: degenerate model dimensions");
    const uint32_t hs = c.hidden_size, hd = hs / c.n_heads, inter = c.intermediate_size;
    if (hd % 4u != 0 || hd > 256u) return ctx_fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "lfm2_load: head_dim must be a multiple of 4 and <= 256");

    std::unique_ptr<wick_rocm_lfm2> holder(new wick_rocm_lfm2);
    wick_rocm_lfm2* m = holder.get();
    m->kv_f16 = kv_dtype == WICK_ROCM_KV_F16;
    auto bail = [&](int rc) {
        release(ctx, holder.release());
        return rc;
    };
    m->layers.resize(c.n_layers);
    int rc = 0;
    // block types from tensor presence, wick/src/model/lfm2.rs:151-170
    for (uint32_t i = 0; i < c.n_layers; i++) {
        const std::string p = "blk." + std::to_string(i) + ".";
        LayerWeights& L = m->layers[i];
        const bool is_attn = wick_gguf_tensor_info(g, (p + "attn_q.weight").c_str(), nullptr, nullptr, nullptr, nullptr, nullptr) == 0;
        if (is_attn) {
            int32_t n_kv;
            memcpy(&n_kv, static_cast<const uint8_t*>(kv_data) + 4 * i, 4);
            if (n_kv <= 0 || c.n_heads % (uint32_t)n_kv != 0)
                return bail(ctx_fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "lfm2_load: layer " + std::to_string(i) + ": n_kv_heads must be > 0 and divide n_heads"));
            L.n_kv = (uint32_t)n_kv;
            c.n_kv_heads = L.n_kv > c.n_kv_heads ? L.n_kv : c.n_kv_heads;
        }
        if ((rc = upload_f32(ctx, m, g, p + "attn_norm.weight", hs, &L.attn_norm))) return bail(rc);
        if ((rc = upload_f32(ctx, m, g, p + "ffn_norm.weight", hs, &L.ffn_norm))) return bail(rc);
        if (is_attn) {
            const uint32_t kv_dim = L.n_kv * hd;
            if ((rc = upload_f32(ctx, m, g, p + "attn_q_norm.weight", hd, &L.q_norm))) return bail(rc);
            if ((rc = upload_f32(ctx, m, g, p + "attn_k_norm.weight", hd, &L.k_norm))) return bail(rc);
            if ((rc = upload_weight(ctx, m, g, p + "attn_q.weight", hs, hs, &L.q))) return bail(rc);
            if ((rc = upload_weight(ctx, m, g, p + "attn_k.weight", kv_dim, hs, &L.k))) return bail(rc);
            if ((rc = upload_weight(ctx, m, g, p + "attn_v.weight", kv_dim, hs, &L.v))) return bail(rc);
            if ((rc = upload_weight(ctx, m, g, p + "attn_output.weight", hs, hs, &L.o))) return bail(rc);
            if ((rc = alloc(ctx, m, (size_t)c.max_seq_len * kv_dim * m->kv_elem(), &L.k_cache))) return bail(rc);
            if ((rc = alloc(ctx, m, (size_t)c.max_seq_len * kv_dim * m->kv_elem(), &L.v_cache))) return bail(rc);
        } else {
            if ((rc = upload_f32(ctx, m, g, p + "shortconv.conv.weight", (uint64_t)hs * c.conv_kernel_size, &L.conv_w))) return bail(rc);
            if ((rc = upload_weight(ctx, m, g, p + "shortconv.in_proj.weight", 3 * hs, hs, &L.in_proj))) return bail(rc);
            if ((rc = upload_weight(ctx, m, g, p + "shortconv.out_proj.weight", hs, hs, &L.out_proj))) return bail(rc);
            if (c.conv_kernel_size > 1 && (rc = alloc_t(ctx, m, (size_t)(c.conv_kernel_size - 1) * hs, &L.conv_state))) return bail(rc);
        }
        if ((rc = upload_weight(ctx, m, g, p + "ffn_gate.weight", inter, hs, &L.gate))) return bail(rc);
        if ((rc = upload_weight(ctx, m, g, p + "ffn_up.weight", inter, hs, &L.up))) return bail(rc);
        if ((rc = upload_weight(ctx, m, g, p + "ffn_down.weight", hs, inter, &L.down))) return bail(rc);
        L.conv_fused = L.n_kv == 0 && L.conv_state && reinterpret_cast<uintptr_t>(L.conv_state) % 16u == 0 && reinterpret_cast<uintptr_t>(L.conv_w) % 16u == 0 &&
                       wick_rocm_shortconv_fusable(L.out_proj, L.gate, L.up, c.conv_kernel_size) != 0;
    }
    if ((rc = upload_f32(ctx, m, g, "token_embd_norm.weight", hs, &m->out_norm))) return bail(rc);
    {
        // The tied embedding serves row lookups and the LM head over ONE token (a prompt pass takes the last token's logits only,
        // wick/src/model/lfm2.rs:2190-2212): it never runs as a batched GEMM, so it keeps its raw blocks only.
        std::lock_guard<std::recursive_mutex> lk(ctx->mu);
        const bool packing = ctx->gemm_packing;
        ctx->gemm_packing = false;
        rc = upload_weight(ctx, m, g, "token_embd.weight", c.vocab_size, hs, &m->embd);
        ctx->gemm_packing = packing;
        if (rc) return bail(rc);
    }

    const uint32_t kv_max = (c.n_kv_heads ? c.n_kv_heads : 1) * hd;
    if ((rc = alloc_t(ctx, m, hs, &m->hidden)) || (rc = alloc_t(ctx, m, 3 * (size_t)hs, &m->proj)) ||
        (rc = alloc_t(ctx, m, hs, &m->gated)) || (rc = alloc_t(ctx, m, hs, &m->q)) || (rc = alloc_t(ctx, m, kv_max, &m->k)) ||
        (rc = alloc_t(ctx, m, kv_max, &m->v)) || (rc = alloc_t(ctx, m, hs, &m->attn)) || (rc = alloc_t(ctx, m, inter, &m->gate)) ||
        (rc = alloc_t(ctx, m, attention_scratch_floats(c.max_seq_len, c.n_heads, hd), &m->scores)) ||
        (rc = alloc_t(ctx, m, c.vocab_size, &m->logits)) || (rc = alloc_t(ctx, m, 1, &m->d_token)) ||
        (rc = alloc_t(ctx, m, 1, &m->d_pos)) || (rc = alloc_t(ctx, m, 1, &m->d_pick)) || (rc = alloc_t(ctx, m, kArgmaxPartials, &m->d_argmax_partial)) || (rc = alloc_t(ctx, m, c.max_seq_len, &m->d_history)))
        return bail(rc);
    // GEMVs that cannot take the fused-quantizer kernel quantize into the context's scratch: size it before any capture
    if ((rc = wick_rocm_reserve_scratch(ctx, 1, hs > inter ? hs : inter))) return bail(rc);
    m->cfg = c;
    m->theta_scale = wick_rocm_rope_theta_scale(hd, c.rope_theta);
    if ((rc = wick_rocm_lfm2_reset(ctx, m))) return bail(rc);
    if ((rc = wick_rocm_sync(ctx))) return bail(rc);  // uploads read the GGUF image: done before the caller may close it
    *out = holder.release();
    return WICK_ROCM_OK;
}

int wick_rocm_lfm2_free(wick_rocm_ctx* ctx, wick_rocm_lfm2* model) {
    if (!ctx) return WICK_ROCM_ERR_INVALID_ARG;
    if (model) release(ctx, model);
    return WICK_ROCM_OK;
}

int wick_rocm_lfm2_get_config(const wick_rocm_lfm2* model, wick_rocm_lfm2_config* out) {
    if (!model || !out) return WICK_ROCM_ERR_INVALID_ARG;
    *out = model->cfg;
    return WICK_ROCM_OK;
}

int wick_rocm_lfm2_layer_kv_heads(const wick_rocm_lfm2* model, uint32_t layer, uint32_t* n_kv_heads) {
    if (!model || !n_kv_heads || layer >= model->cfg.n_layers) return WICK_ROCM_ERR_INVALID_ARG;
    *n_kv_heads = model->layers[layer].n_kv;
    return WICK_ROCM_OK;
}

size_t wick_rocm_lfm2_gpu_memory_bytes(const wick_rocm_lfm2* model) { return model ? model->bytes : 0; }

int wick_rocm_lfm2_reset(wick_rocm_ctx* ctx, wick_rocm_lfm2* model) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);  // nothing else gets onto the context's stream (or into a capture) in between
    const size_t state_floats = (size_t)(model->cfg.conv_kernel_size - 1) * model->cfg.hidden_size;
    if (state_floats) {
        const std::vector<float> zeros(state_floats, 0.0f);
        for (const LayerWeights& L : model->layers)
            if (L.conv_state)
                if (int rc = wick_rocm_upload(ctx, L.conv_state, zeros.data(), state_floats * sizeof(float))) return rc;
    }
    return WICK_ROCM_OK;
}

int wick_rocm_lfm2_set_graph_replay(wick_rocm_lfm2* model, int enabled) {
    if (!model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    model->use_graph = enabled != 0;
    return WICK_ROCM_OK;
}

int wick_rocm_lfm2_forward(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t token, uint32_t pos, float* logits) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);  // nothing else gets onto the context's stream (or into a capture) in between
    if (int rc = check_step(ctx, model, token, pos, 1)) return rc;
    if (int rc = set_step(ctx, model, token, pos)) return rc;
    if (int rc = run_step(ctx, model, kStepLogits)) return rc;
    if (logits) return wick_rocm_download(ctx, logits, model->logits, (size_t)model->cfg.vocab_size * sizeof(float));
    return wick_rocm_sync(ctx);
}

// Shared body of the two prompt entry points: exactly one of tokens / embeddings is given.
static int prefill_locked(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, const uint32_t* tokens, const float* embeddings, uint32_t n, uint32_t start_pos,
                          float* logits) {
    const wick_rocm_lfm2_config& c = model->cfg;
    if ((uint64_t)start_pos + n > c.max_seq_len) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: position beyond the context size");
    if (n <= kPromptAsStepsMax) {
        // One or two tokens (the tail of a chunked prompt, a short turn): single steps, whose graph replays in 0.3 ms each, beat a
        // pass of ~130 launches (0.7 ms whatever its length).  Same arithmetic per token; the LM head runs for the last one only.
        for (uint32_t j = 0; j < n; j++) {
            const StepMode mode = j + 1 == n ? kStepLogits : kStepHidden;
            if (tokens) {
                if (int rc = set_step(ctx, model, tokens[j], start_pos + j)) return rc;
            } else {
                const hipError_t e = launch_set_step(nullptr, 0, model->d_pos, start_pos + j, ctx->launch());
                if (e != hipSuccess) return fail_hip(ctx, e, "set_step launch");
                if (int rc = wick_rocm_upload(ctx, model->hidden, embeddings + (size_t)j * c.hidden_size, (size_t)c.hidden_size * sizeof(float))) return rc;
            }
            if (int rc = run_step(ctx, model, mode)) return rc;
        }
        if (logits) return wick_rocm_download(ctx, logits, model->logits, (size_t)c.vocab_size * sizeof(float));
        return wick_rocm_sync(ctx);
    }
    if (int rc = ensure_prefill_buffers(ctx, model)) return rc;
    uint32_t last = 0;
    for (uint32_t done = 0; done < n; done += model->prefill_cap) {
        last = n - done < model->prefill_cap ? n - done : model->prefill_cap;
        if (tokens) {
            if (int rc = wick_rocm_upload(ctx, model->pTokens, tokens + done, (size_t)last * sizeof(uint32_t))) return rc;
        } else {  // frame j of the prompt is row j of the pass's input (wick/src/model/lfm2.rs:2452-2487)
            if (int rc = wick_rocm_upload(ctx, model->pX, embeddings + (size_t)done * c.hidden_size, (size_t)last * c.hidden_size * sizeof(float))) return rc;
        }
        if (int rc = enqueue_prompt_pass(ctx, model, last, start_pos + done, tokens != nullptr)) return rc;
    }
    // output norm + tied LM head on the last token only (wick/src/model/lfm2.rs:2080-2109)
    const float* h_last = model->pX + (size_t)(last - 1) * c.hidden_size;
    if (int rc = gemv_normed(ctx, {model->embd}, {model->logits}, h_last, model->out_norm, c.rms_norm_eps)) return rc;
    if (logits) return wick_rocm_download(ctx, logits, model->logits, (size_t)c.vocab_size * sizeof(float));
    return wick_rocm_sync(ctx);
}

int wick_rocm_lfm2_forward_prefill(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, const uint32_t* tokens, uint32_t n, uint32_t start_pos, float* logits) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    if (!tokens || n == 0) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 prefill: empty prompt");
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);  // nothing else gets onto the context's stream (or into a capture) in between
    for (uint32_t j = 0; j < n; j++)
        if (tokens[j] >= model->cfg.vocab_size) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: token_id out of range");
    return prefill_locked(ctx, model, tokens, nullptr, n, start_pos, logits);
}

int wick_rocm_lfm2_forward_prefill_from_embeddings(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, const float* embeddings, uint32_t n, uint32_t start_pos,
                                                   float* logits) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    if (!embeddings || n == 0) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 prefill: at least one frame is required");
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);
    return prefill_locked(ctx, model, nullptr, embeddings, n, start_pos, logits);
}

int wick_rocm_lfm2_forward_prefill_chunked(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                           uint32_t ubatch, const volatile int32_t* cancel, uint32_t* consumed, float* logits) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    if (!consumed) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 prefill: null consumed pointer");
    *consumed = 0;
    if (n == 0) return WICK_ROCM_OK;  // the reference's (0, None)
    if (!tokens) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 prefill: null token pointer");
    const uint32_t step = ubatch == 0 ? n : ubatch;  // 0 = one chunk covering everything
    while (*consumed < n) {
        const uint32_t len = n - *consumed < step ? n - *consumed : step;
        if (int rc = wick_rocm_lfm2_forward_prefill(ctx, model, tokens + *consumed, len, start_pos + *consumed, logits)) return rc;
        *consumed += len;
        // looked at AFTER each chunk, so a call always makes progress by at least one chunk
        if (cancel && __atomic_load_n(cancel, __ATOMIC_RELAXED) != 0) break;
    }
    return WICK_ROCM_OK;
}

int wick_rocm_lfm2_forward_greedy(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t token, uint32_t pos, uint32_t* next_token) {
    return wick_rocm_lfm2_generate_greedy(ctx, model, token, pos, 1, next_token);
}

int wick_rocm_lfm2_generate_greedy(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t token, uint32_t pos, uint32_t n, uint32_t* out_tokens) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    if (!out_tokens) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: null output pointer");
    if (n == 0) return WICK_ROCM_OK;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);  // nothing else gets onto the context's stream (or into a capture) in between
    if (int rc = check_step(ctx, model, token, pos, n)) return rc;
    if (int rc = set_step(ctx, model, token, pos)) return rc;
    for (uint32_t i = 0; i < n; i++)  // the pick of step i is written to the device-side token and position pos + i of the history
        if (int rc = run_step(ctx, model, kStepGreedy)) return rc;
    return wick_rocm_download(ctx, out_tokens, model->d_history + pos, (size_t)n * sizeof(uint32_t));
}

// One step whose input is the token's embedding row (embedding == null) or the caller's hidden-size vector; ends per `mode`.
static int step_locked(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t token, const float* embedding, uint32_t pos, StepMode mode, float* out) {
    const wick_rocm_lfm2_config& c = model->cfg;
    if (int rc = check_step(ctx, model, embedding ? 0u : token, pos, 1)) return rc;
    if (embedding) {  // position only; the input vector goes where the lookup would have put the row
        {
            std::lock_guard<std::recursive_mutex> lk(ctx->mu);
            const hipError_t e = launch_set_step(nullptr, 0, model->d_pos, pos, ctx->launch());
            if (e != hipSuccess) return fail_hip(ctx, e, "set_step launch");
        }
        if (int rc = wick_rocm_upload(ctx, model->hidden, embedding, (size_t)c.hidden_size * sizeof(float))) return rc;
    } else if (int rc = set_step(ctx, model, token, pos)) {
        return rc;
    }
    if (int rc = run_step(ctx, model, mode)) return rc;
    if (!out) return wick_rocm_sync(ctx);
    return mode == kStepHidden ? wick_rocm_download(ctx, out, model->gated, (size_t)c.hidden_size * sizeof(float))
                               : wick_rocm_download(ctx, out, model->logits, (size_t)c.vocab_size * sizeof(float));
}

int wick_rocm_lfm2_forward_from_embedding(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, const float* embedding, uint32_t pos, float* logits) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    if (!embedding) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: null embedding pointer");
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);
    return step_locked(ctx, model, 0, embedding, pos, kStepLogits, logits);
}

int wick_rocm_lfm2_forward_embedding(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t token, uint32_t pos, float* hidden) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);
    return step_locked(ctx, model, token, nullptr, pos, kStepHidden, hidden);
}

int wick_rocm_lfm2_forward_hidden_from_embedding(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, const float* embedding, uint32_t pos, float* hidden) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    if (!embedding) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2: null embedding pointer");
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole_step(ctx->mu);
    return step_locked(ctx, model, 0, embedding, pos, kStepHidden, hidden);
}

// ---- state snapshots and the context shift -------------------------------------------------

size_t wick_rocm_lfm2_layer_state_bytes(const wick_rocm_lfm2* model, uint32_t layer, uint32_t seq_len) {
    if (!model || layer >= model->cfg.n_layers || seq_len > model->cfg.max_seq_len) return 0;
    const wick_rocm_lfm2_config& c = model->cfg;
    const LayerWeights& L = model->layers[layer];
    if (L.n_kv) return 2 * (size_t)seq_len * L.n_kv * (c.hidden_size / c.n_heads) * model->kv_elem();
    return (size_t)(c.conv_kernel_size - 1) * c.hidden_size * sizeof(float);
}

size_t wick_rocm_lfm2_state_bytes(const wick_rocm_lfm2* model, uint32_t seq_len) {
    if (!model) return 0;
    size_t total = 0;
    for (uint32_t i = 0; i < model->cfg.n_layers; i++) total += wick_rocm_lfm2_layer_state_bytes(model, i, seq_len);
    return total;
}

int wick_rocm_lfm2_snapshot_state(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t seq_len, void* out, size_t nbytes) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole(ctx->mu);
    if (seq_len > model->cfg.max_seq_len) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 snapshot: seq_len beyond the context size");
    if (nbytes != wick_rocm_lfm2_state_bytes(model, seq_len) || (!out && nbytes))
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 snapshot: the buffer must hold exactly wick_rocm_lfm2_state_bytes(model, seq_len) bytes");
    uint8_t* at = static_cast<uint8_t*>(out);
    return for_each_state_piece(model, seq_len, [&](const void* d, size_t n) {
        const int rc = wick_rocm_download(ctx, at, d, n);
        at += n;
        return rc;
    });
}

int wick_rocm_lfm2_restore_state(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t seq_len, const void* in, size_t nbytes) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole(ctx->mu);
    if (seq_len > model->cfg.max_seq_len) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 restore: seq_len beyond the context size");
    if (nbytes != wick_rocm_lfm2_state_bytes(model, seq_len) || (!in && nbytes))
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 restore: the snapshot must hold exactly wick_rocm_lfm2_state_bytes(model, seq_len) bytes");
    const uint8_t* at = static_cast<const uint8_t*>(in);
    return for_each_state_piece(model, seq_len, [&](void* d, size_t n) {
        const int rc = wick_rocm_upload(ctx, d, at, n);
        at += n;
        return rc;
    });
}

int wick_rocm_lfm2_shift_kv(wick_rocm_ctx* ctx, wick_rocm_lfm2* model, uint32_t seq_len, uint32_t n_keep, uint32_t shift) {
    if (!ctx || !model) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(model->mu);
    std::lock_guard<std::recursive_mutex> whole(ctx->mu);
    const wick_rocm_lfm2_config& c = model->cfg;
    if (shift == 0) return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 shift_kv: shift must be > 0");
    if (seq_len > c.max_seq_len || (uint64_t)n_keep + shift > seq_len)
        return ctx_fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "lfm2 shift_kv: shift range out of bounds (n_keep + shift > seq_len)");
    if (seq_len - n_keep - shift == 0) return WICK_ROCM_OK;  // nothing behind the dropped rows: only the caller's seq_len changes
    const uint32_t hd = c.hidden_size / c.n_heads;
    if (!model->shift_stage && c.n_kv_heads)
        if (int rc = alloc(ctx, model, 2 * (size_t)c.max_seq_len * c.n_kv_heads * hd * model->kv_elem(), &model->shift_stage)) return rc;
    for (const LayerWeights& L : model->layers)  // conv layers keep their rolling buffer (wick/src/kv_cache.rs:584-590)
        if (L.n_kv) {
            const hipError_t e = launch_kv_shift(L.k_cache, L.v_cache, model->shift_stage, seq_len, n_keep, shift, L.n_kv, hd, model->theta_scale,
                                                 ctx->launch(), model->kv_f16);
            if (e != hipSuccess) return fail_hip(ctx, e, "kv_shift launch");
        }
    return wick_rocm_sync(ctx);
}

const float* wick_rocm_lfm2_logits_device(const wick_rocm_lfm2* model) { return model ? model->logits : nullptr; }

}  // extern "C"
