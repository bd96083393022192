/*
 * wick_oracle_ops.c -- CPU restatement of the non-matmul operations of wick's LFM2 decode
 * step (the operations either side of the block-quantized GEMVs).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE: only tests, the smoke check and the
 * benchmark's cpu-baseline leg may link or load it; the shipped library never does.
 *
 * Every function cites the reference lines it follows (paths relative to the reference
 * checkout).  binary32 arithmetic with separate multiply and add (-ffp-contract=off),
 * double only where the reference uses f64.  Loops run in the reference's order.
 *
 * How each function is pinned (tests/test_oracle_ops.py):
 *   orc_ggml_expf      the reference's own check (cpu.rs:2751-2770: within 1e-5 of exp on eight
 *                      values, overflow / underflow edges) extended to a dense sweep against
 *                      numpy's exp (<= 2 ulp on [-87, 88]); exp(0) == 1 exactly
 *   orc_rmsnorm        closed forms of cpu.rs:2278-2316; numpy float64 restatement
 *   orc_silu_mul       known values of cpu.rs:2318-2348; x / (1 + exp(-x)) * u in float64
 *   orc_softmax        known values / stability cases of cpu.rs:2374-2391, 2773-2780; sums to 1
 *   orc_rope           pos = 0 is the identity (cpu.rs:2783-2797); closed form
 *                      theta_i = pos * base^(-2 i / d) in float64; norm of every pair preserved;
 *                      R(p + q) = R(q) R(p)
 *   orc_rope_delta     the reference's own checks (wick/tests/n_keep_shift.rs:47-91): a head rotated for
 *                      p_old and then by p_new - p_old equals the head rotated for p_new within 1e-3
 *                      on the same 25 position pairs and inputs, delta 0 is the identity; for
 *                      delta >= 0 bit-equal to orc_rope at pos = delta
 *   orc_shift_kv       the reference's closed-form case (wick/tests/n_keep_shift.rs:138-236: caches filled
 *                      with raw heads rotated for their row, 24 rows, n_keep 5, shift 7): kept rows
 *                      byte-identical, moved keys within 1e-3 of a fresh rotation for the new row, moved
 *                      value rows bit-equal to their old rows; numpy restatement of the row move
 *   orc_attn_scores /  the reference's own inputs (cpu.rs:2910-3003) against numpy matmul;
 *   orc_attn_values    seq_len = 0 leaves the output untouched / zero (cpu.rs:3005-3010)
 *   orc_shortconv_step identity kernel reproduces b*x*c; numpy restatement over several steps
 *                      of the rolling buffer (lfm2.rs:694-726)
 *   orc_argmax         numpy restatement incl. ties (the last maximum wins), NaN and signed zeros
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

static float from_bits(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint32_t to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* ggml_expf, wick/src/backend/cpu.rs:604-652 (ggml's ggml_v_expf polynomial). */
ORC_API float orc_ggml_expf(float x) {
    const float R = from_bits(0x4B400000u), LOG2E = from_bits(0x3FB8AA3Bu);
    const float LN2_HI = from_bits(0x3F317200u), LN2_LO = from_bits(0x35BFBE8Eu);
    const float C1 = from_bits(0x3F7FFFF6u), C2 = from_bits(0x3EFFFEDBu), C3 = from_bits(0x3E2AAF33u);
    const float C4 = from_bits(0x3D2B9F17u), C5 = from_bits(0x3C072010u);
    const float z = R + x * LOG2E;
    const float n = z - R;
    const float b = x - n * LN2_HI - n * LN2_LO;
    const uint32_t e = to_bits(z) << 23;
    const float k = from_bits(e + to_bits(1.0f));
    const float u = b * b;
    const float j = C1 * b + (C2 + C3 * b + (C4 + C5 * b) * u) * u;
    const float abs_n = from_bits(to_bits(n) & 0x7FFFFFFFu);
    if (abs_n <= 126.0f) return k + j * k;
    if (abs_n > 192.0f) return n > 0.0f ? INFINITY : 0.0f;
    const uint32_t d = n <= 0.0f ? 0x82000000u : 0u;
    const float s1 = from_bits(d + 0x7f000000u);
    const float s2 = from_bits(e - d);
    return (s2 + s2 * j) * s1;
}

/* rmsnorm, wick/src/backend/cpu.rs:577-594: f64 sum of squares, x * inv_rms * weight. */
ORC_API void orc_rmsnorm(float* x, const float* weight, int64_t n, float eps) {
    double sum_sq = 0.0;
    for (int64_t i = 0; i < n; i++) sum_sq += (double)x[i] * (double)x[i];
    const double mean = sum_sq / (double)n;
    const double rms = sqrt(mean + (double)eps);
    const float inv_rms = (float)(1.0 / rms);
    for (int64_t i = 0; i < n; i++) x[i] = x[i] * inv_rms * weight[i];
}

/* silu_mul_inplace, wick/src/backend/cpu.rs:668-673: g / (1 + expf(-g)) * u. */
ORC_API void orc_silu_mul(float* gate, const float* up, int64_t n) {
    for (int64_t i = 0; i < n; i++) gate[i] = gate[i] / (1.0f + orc_ggml_expf(-gate[i])) * up[i];
}

/* softmax_inplace, wick/src/backend/cpu.rs:715-731: max, ggml_expf, f64 sum, one f32 reciprocal. */
ORC_API void orc_softmax(float* x, int64_t n) {
    float mx = -INFINITY;
    for (int64_t i = 0; i < n; i++) mx = x[i] > mx ? x[i] : mx; /* f32::max: NaN-free inputs */
    double sum = 0.0;
    for (int64_t i = 0; i < n; i++) {
        x[i] = orc_ggml_expf(x[i] - mx);
        sum += (double)x[i];
    }
    const float inv = (float)(1.0 / sum);
    for (int64_t i = 0; i < n; i++) x[i] *= inv;
}

/* apply_rope_to_head, wick/src/backend/cpu.rs:2148-2161: split-halves pairs, theta multiplied up in f32. */
static void rope_head(float* head, int64_t pos, int64_t head_dim, float freq_base) {
    const int64_t half = head_dim / 2;
    const float theta_scale = powf(freq_base, -2.0f / (float)head_dim);
    float theta = (float)pos;
    for (int64_t i = 0; i < half; i++) {
        const float s = sinf(theta), c = cosf(theta);
        const float x0 = head[i], x1 = head[i + half];
        head[i] = x0 * c - x1 * s;
        head[i + half] = x0 * s + x1 * c;
        theta *= theta_scale;
    }
}

/* rope, wick/src/backend/cpu.rs:2113-2137. */
ORC_API void orc_rope(float* q, float* k, int64_t pos, int64_t n_heads, int64_t n_kv_heads, int64_t head_dim, float freq_base) {
    for (int64_t h = 0; h < n_heads; h++) rope_head(q + h * head_dim, pos, head_dim, freq_base);
    for (int64_t h = 0; h < n_kv_heads; h++) rope_head(k + h * head_dim, pos, head_dim, freq_base);
}

/* apply_rope_delta_to_head, wick/src/backend/cpu.rs:2174-2187: the same pairs and theta schedule from a signed start angle. */
ORC_API void orc_rope_delta(float* head, int32_t delta_pos, int64_t head_dim, float freq_base) {
    const int64_t half = head_dim / 2;
    const float theta_scale = powf(freq_base, -2.0f / (float)head_dim);
    float theta = (float)delta_pos;
    for (int64_t i = 0; i < half; i++) {
        const float s = sinf(theta), c = cosf(theta);
        const float x0 = head[i], x1 = head[i + half];
        head[i] = x0 * c - x1 * s;
        head[i + half] = x0 * s + x1 * c;
        theta *= theta_scale;
    }
}

/* InferenceState::shift_kv_with_rope for one attention layer, wick/src/kv_cache.rs:601-700: rows [n_keep, n_keep + shift) of
 * both caches ([seq_len][n_kv_heads * head_dim]) are dropped, the rows behind them move down by `shift`, and every key head
 * that moved is rotated by -shift positions.  The caller's seq_len becomes seq_len - shift; rows past it are left as they are. */
ORC_API void orc_shift_kv(float* k_cache, float* v_cache, int64_t seq_len, int64_t n_keep, int64_t shift, int64_t n_kv_heads, int64_t head_dim,
                          float freq_base) {
    const int64_t kv_dim = n_kv_heads * head_dim, new_len = seq_len - shift;
    memmove(k_cache + n_keep * kv_dim, k_cache + (n_keep + shift) * kv_dim, (size_t)((new_len - n_keep) * kv_dim) * sizeof(float));
    memmove(v_cache + n_keep * kv_dim, v_cache + (n_keep + shift) * kv_dim, (size_t)((new_len - n_keep) * kv_dim) * sizeof(float));
    for (int64_t t = n_keep; t < new_len; t++)
        for (int64_t h = 0; h < n_kv_heads; h++) orc_rope_delta(k_cache + t * kv_dim + h * head_dim, -(int32_t)shift, head_dim, freq_base);
}

/* The f32 theta_scale the reference derives from freq_base (cpu.rs:2150), for callers that hand it to the device. */
ORC_API float orc_rope_theta_scale(int64_t head_dim, float freq_base) { return powf(freq_base, -2.0f / (float)head_dim); }

/* attn_scores, scalar branch, wick/src/backend/cpu.rs:1346-1355. */
ORC_API void orc_attn_scores(const float* q_head, const float* k_cache, float* scores, int64_t kv_dim, int64_t kv_h_offset,
                             int64_t head_dim, float scale, int64_t seq_len) {
    for (int64_t t = 0; t < seq_len; t++) {
        float dot = 0.0f;
        const float* kr = k_cache + t * kv_dim + kv_h_offset;
        for (int64_t d = 0; d < head_dim; d++) dot += q_head[d] * kr[d];
        scores[t] = dot * scale;
    }
}

/* attn_values, scalar branch, wick/src/backend/cpu.rs:1391-1401. */
ORC_API void orc_attn_values(const float* scores, const float* v_cache, float* attn_out, int64_t kv_dim, int64_t kv_h_offset,
                             int64_t head_dim, int64_t seq_len) {
    for (int64_t d = 0; d < head_dim; d++) attn_out[d] = 0.0f;
    for (int64_t t = 0; t < seq_len; t++) {
        const float s = scores[t];
        const float* vr = v_cache + t * kv_dim + kv_h_offset;
        for (int64_t d = 0; d < head_dim; d++) attn_out[d] += s * vr[d];
    }
}

/* One head of decode attention as forward_attn_block runs it (wick/src/model/lfm2.rs:984-1006):
 * scores -> softmax -> weighted values.  `scores` is scratch of seq_len floats. */
ORC_API void orc_attention_head(const float* q_head, const float* k_cache, const float* v_cache, float* scores, float* out,
                                int64_t kv_dim, int64_t kv_h_offset, int64_t head_dim, float scale, int64_t seq_len) {
    orc_attn_scores(q_head, k_cache, scores, kv_dim, kv_h_offset, head_dim, scale, seq_len);
    orc_softmax(scores, seq_len);
    orc_attn_values(scores, v_cache, out, kv_dim, kv_h_offset, head_dim, seq_len);
}

/* The gated short convolution of one decode step, wick/src/model/lfm2.rs:694-726:
 * proj = [b | c | x] (hidden floats each); bx = b*x; out = c * (sum_k buffer[k]*w[ch][k] + bx*w[ch][d_conv]);
 * the rolling buffer ((kernel-1) slots of hidden floats) shifts left by one slot and takes bx. */
ORC_API void orc_shortconv_step(const float* proj, float* buffer, const float* conv_weight, float* out, int64_t hidden,
                                int64_t kernel_size) {
    const int64_t d_conv = kernel_size - 1;
    const float *b = proj, *c = proj + hidden, *x = proj + 2 * hidden;
    for (int64_t ch = 0; ch < hidden; ch++) {
        const float bx = b[ch] * x[ch];
        float sum = 0.0f;
        for (int64_t k = 0; k < d_conv; k++) sum += buffer[k * hidden + ch] * conv_weight[ch * kernel_size + k];
        sum += bx * conv_weight[ch * kernel_size + d_conv];
        for (int64_t k = 0; k + 1 < d_conv; k++) buffer[k * hidden + ch] = buffer[(k + 1) * hidden + ch];
        if (d_conv > 0) buffer[(d_conv - 1) * hidden + ch] = bx;
        out[ch] = c[ch] * sum;
    }
}

/* cpu_argmax, wick/src/sampler.rs:7-19: NaN counts as -inf, values compare by f32::total_cmp
 * (-0.0 below +0.0), and Iterator::max_by keeps the LAST of several equal maxima; 0 for an empty slice. */
static int32_t total_order_key(float f) {
    if (f != f) f = -INFINITY;
    int32_t b = (int32_t)to_bits(f);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1); /* f32::total_cmp's transform */
}
ORC_API int64_t orc_argmax(const float* x, int64_t n) {
    int64_t best = 0;
    for (int64_t i = 1; i < n; i++)
        if (total_order_key(x[i]) >= total_order_key(x[best])) best = i;
    return best;
}
