// Internal declarations shared by the kernel translation units and the C ABI
// layer.  Not installed; the public surface is include/wick_rocm.h.
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

namespace wick_rocm {

constexpr int kTypeQ4_0 = 2;  // ggml ids, wick/src/gguf.rs:36-51
constexpr int kTypeQ8_0 = 8;
constexpr int kQ4BlockBytes = 18;  // wick/src/quant.rs:13-20
constexpr int kQ8BlockBytes = 34;  // wick/src/quant.rs:27-34
constexpr int kMaxGemvBatch = 4;

inline int block_bytes(int type) { return type == kTypeQ4_0 ? kQ4BlockBytes : (type == kTypeQ8_0 ? kQ8BlockBytes : 0); }

// Up to kMaxGemvBatch weights that share one quantized activation.  row_end is the
// running total of rows (row_end[i] - row_end[i-1] = rows of weight i).
struct GemvBatch {
    const uint8_t* w[kMaxGemvBatch];
    float* y[kMaxGemvBatch];
    uint32_t row_end[kMaxGemvBatch];
    uint32_t count;
};

// Per-dispatch GPU timestamps (the counterpart of the reference's GpuTimer,
// wick/src/model/metal_lfm2.rs:3367-4116).  While enabled, every kernel is
// launched with a start/stop event pair bound to its own dispatch packet
// (hipExtLaunchKernelGGL), so the elapsed time is the kernel's execution time
// alone, the same quantity a kernel trace reports.
enum KernelFamily { kFamQuantize = 0, kFamGemv = 1, kFamGemm = 2, kFamOther = 3, kNumFamilies = 4 };

struct KernelTimer {
    struct Rec {
        hipEvent_t start, stop;
        int family;
    };
    bool enabled = false;
    std::vector<Rec> recs;    // launches since timing began
    std::vector<Rec> spares;  // event pairs kept for reuse
};

struct Launch {
    hipStream_t stream;
    KernelTimer* timer;  // may be null
    int64_t gemv_direct_max_bytes = -1;  // single-token GEMV: per-lane loads below, span loads from here on; < 0 = per-dtype default
    bool gemm_mfma16 = false;            // plain wide GEMM launches: the 16x16x32 block loop instead of the 32x32x32 one
};

template <typename... KArgs, typename... Args>
inline hipError_t launch_kernel(const Launch& L, int family, void (*kernel)(KArgs...), dim3 grid, dim3 block,
                                Args... args) {
    if (L.timer && L.timer->enabled) {
        KernelTimer::Rec r{};
        if (!L.timer->spares.empty()) {
            r = L.timer->spares.back();
            L.timer->spares.pop_back();
        } else {
            hipError_t e = hipEventCreate(&r.start);
            if (e != hipSuccess) return e;
            e = hipEventCreate(&r.stop);
            if (e != hipSuccess) return e;
        }
        r.family = family;
        hipExtLaunchKernelGGL(kernel, grid, block, 0, L.stream, r.start, r.stop, 0, args...);
        L.timer->recs.push_back(r);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, 0, L.stream, args...);
    }
    return hipGetLastError();
}

// Launchers.  All only enqueue on L.stream; callers have validated shapes.
// They return hipGetLastError() after the launch.

hipError_t launch_quantize_q8_0(const float* d_x, uint32_t n, uint32_t k, uint32_t x_stride, int8_t* d_q,
                                float* d_scales, const Launch& L);

// Decode GEMV, one token.  k % 32 == 0.
hipError_t launch_gemv(int type, const GemvBatch& batch, uint32_t k, const int8_t* d_q, const float* d_scales,
                       int accumulate, int num_cus, const Launch& L);

// Decode GEMV straight from f32 activations (Q8_0 quantization fused into the
// kernel).  Only when pairs_kernel_applies() and d_x is 16-byte aligned.
bool pairs_kernel_applies(const GemvBatch& batch, uint32_t k);
// xform: what is done to x before it is quantized (d_aux: the RMSNorm weights / the "up" vector, k floats, 16-byte aligned).
enum { kXformNone = 0, kXformRmsNorm = 1, kXformSiluMul = 2, kXformShortConv = 3 };
hipError_t launch_gemv_f32(int type, const GemvBatch& batch, uint32_t k, const float* d_x, int accumulate, int num_cus,
                           const Launch& L, int xform = kXformNone, const float* d_aux = nullptr, float eps = 0.0f);

// The FFN's gate and up projections with the gate applied to the row sums: out[r] = silu(W_gate[r] . x') * (W_up[r] . x'),
// x' = xform(x) quantized to Q8_0 (xform: none or RMSNorm).  Only when gated_kernel_applies() (even block count,
// k <= 4096, 4-byte aligned weights) and d_x / d_aux are 16-byte aligned.
bool gated_kernel_applies(const uint8_t* d_w_gate, const uint8_t* d_w_up, uint32_t k);
// conv_state non-null: the first workgroups also advance that rolling short-conv state by one token (slot s <- slot s + 1, last
// slot <- b * x of conv_proj = [b | c | x], conv_hidden floats each, conv_hidden % 4 == 0, 16-byte aligned): what
// launch_shortconv_step does to the state, for a layer whose conv output went through launch_gemv_shortconv_f32.
hipError_t launch_gemv_gated_f32(int type, const uint8_t* d_w_gate, const uint8_t* d_w_up, uint32_t m, uint32_t k, const float* d_x,
                                 float* d_out, int num_cus, const Launch& L, int xform = kXformNone, const float* d_aux = nullptr,
                                 float eps = 0.0f, float* conv_state = nullptr, const float* conv_proj = nullptr, uint32_t conv_hidden = 0,
                                 uint32_t conv_kernel = 0);
// y (+)= W * quantize(c * conv(b * x)) for d_proj = [b | c | x] (k floats each), the rolling state d_state ([2][k], read only) and
// the conv kernel d_conv_w ([k][3]): the gated short convolution folded into its out projection.  Only when
// shortconv_kernel_applies() (kernel size 3, k <= 2048, even block count) and all pointers are 16-byte aligned.
bool shortconv_kernel_applies(const uint8_t* d_w, uint32_t k, uint32_t kernel_size);
hipError_t launch_gemv_shortconv_f32(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const float* d_proj, const float* d_state,
                                     const float* d_conv_w, float* d_y, int accumulate, int num_cus, const Launch& L);

// Q6_K decode GEMV, one token (gemv_q6k.hip).  k % 256 == 0, k <= 8192; the weight allocation is padded by
// 16 bytes; y[row * y_row_stride].  launch_group_dots_q6k is its parity hook: out[i * (k/16) + g] = exact i32 dot of 16-weight group g.
constexpr int kTypeQ6_K = 14;  // ggml id, wick/src/gguf.rs:36-51
constexpr int kQ6KBlockBytes = 210;
// y = W rmsnorm(x) with the norm and the Q8_0 quantizer inside the GEMV's launch (bit-identical to launch_rmsnorm_quantize +
// launch_gemv_q6k); d_x / d_norm_weight 16-byte aligned.  d_partial non-null: gemv_q6k_waves(m, k, num_cus) greedy-pick keys, one
// per wave, for launch_argmax_final.
uint32_t gemv_q6k_waves(uint32_t m, uint32_t k, int num_cus);
hipError_t launch_gemv_q6k_rmsnorm(const uint8_t* d_w, uint32_t m, uint32_t k, const float* d_x, const float* d_norm_weight, float eps, float* d_y,
                                   int accumulate, int num_cus, const Launch& L, unsigned long long* d_partial = nullptr);
hipError_t launch_gemv_q6k(const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, const float* d_scales, float* d_y,
                           uint32_t y_row_stride, int accumulate, int num_cus, const Launch& L);
hipError_t launch_group_dots_q6k(const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, int32_t* d_out, int num_cus,
                                 const Launch& L);

// Small-n GEMM done as a multi-token GEMV (weights streamed once per 1..kGemvTokens tokens).
hipError_t launch_gemv_tokens(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                              const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                              int accumulate, int num_cus, const Launch& L);

// int8-MFMA GEMM.  Requires k % 128 == 0.  d_w / d_w_gate / d_w_up of the GEMM launchers are the weights' PACKED copies
// (gemm_packed_bytes bytes, made by launch_gemm_pack from the raw blocks when the weight is uploaded), not the raw blocks.
size_t gemm_packed_bytes(uint32_t m, uint32_t k);
hipError_t launch_gemm_pack(int type, const uint8_t* d_raw, uint32_t m, uint32_t k, uint8_t* d_packed, const Launch& L);
hipError_t launch_gemm_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                            const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                            int accumulate, const Launch& L, uint32_t splits = 1, float* d_partial = nullptr, bool defer_reduce = false);
// defer_reduce (splits > 1 only): the shares stay in d_partial ([splits][n][m], token-major) and the caller's next kernel adds them
// up in ascending order onto y itself (launch_residual_rmsnorm_quantize).
// Ways (1, 2, 4 or 8, at most max_splits) the launch above may be split over K: > 1 only for launches of few tiles and long K.
uint32_t gemm_split_k(uint32_t m, uint32_t n, uint32_t k, uint32_t max_splits);
hipError_t launch_gemm_mfma_multi(int type, const uint8_t* const* d_w, const uint32_t* m, uint32_t count, uint32_t k, const int8_t* d_q,
                                  const float* d_scales, uint32_t n, float* const* d_y, uint32_t y_stride, int y_layout, int accumulate,
                                  const Launch& L);
// out = Q8_0(silu(W_gate x) * (W_up x)) over n tokens in one launch (wide tiles only: gemm_gated_applies).
bool gemm_gated_applies(uint32_t m, uint32_t n, uint32_t k);
hipError_t launch_gemm_mfma_gated(int type, const uint8_t* d_w_gate, const uint8_t* d_w_up, uint32_t m, uint32_t k, const int8_t* d_q,
                                  const float* d_scales, uint32_t n, int8_t* d_out_q, float* d_out_scales, const Launch& L);

// Per-block i32 dots, out[(j*m + i)*nb + b], through the GEMM's loads / LDS layout / MFMA (k % 128 == 0): launch_block_dots_mfma
// below.  The same through the decode GEMV's own kernels (gemv_dump.hip): every fetch mode, token count and the fused
// in-kernel quantizer, exactly as a product launch of that shape would run them.
hipError_t launch_block_dots_gemv(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n, int32_t* d_out,
                                  int num_cus, const Launch& L);
hipError_t launch_block_dots_gemv_f32(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const float* d_x, int32_t* d_out, int num_cus,
                                      const Launch& L);
hipError_t launch_block_dots_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n,
                                  int32_t* d_out, const Launch& L);

// The non-matmul operations of an LFM2 decode step (lfm2_ops.hip).  d_pos / d_token, when non-null, are read on the
// device in place of the by-value pos / token.
hipError_t launch_embed_row(const uint8_t* d_w, int type, uint32_t m, uint32_t k, uint32_t token, const uint32_t* d_token, float* d_out,
                            const Launch& L);
hipError_t launch_rmsnorm(const float* d_x, const float* d_weight, float* d_y, uint32_t rows, uint32_t dim, uint32_t x_stride,
                          uint32_t y_stride, float eps, const Launch& L);
// The KV caches of the launchers below hold f32 rows, or f16 rows with kv_f16 (values rounded once when they are appended or
// moved, widened exactly when they are read; all arithmetic f32).
hipError_t launch_qk_norm_rope(float* d_q, float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm, void* d_k_cache,
                               void* d_v_cache, uint32_t pos, const uint32_t* d_pos, uint32_t max_seq, uint32_t head_dim, uint32_t n_heads,
                               uint32_t n_kv_heads, float eps, float theta_scale, const Launch& L, uint32_t n_tokens = 1, uint32_t q_stride = 0,
                               uint32_t kv_stride = 0, bool kv_f16 = false);
// Drops cache rows [n_keep, n_keep + shift) of one attention layer and re-rotates the keys that move; d_stage holds
// 2 * (seq_len - n_keep - shift) * n_kv_heads * head_dim cache elements.
hipError_t launch_kv_shift(void* d_k_cache, void* d_v_cache, void* d_stage, uint32_t seq_len, uint32_t n_keep, uint32_t shift,
                           uint32_t n_kv_heads, uint32_t head_dim, float theta_scale, const Launch& L, bool kv_f16 = false);
// A prompt of n tokens at once (token j at position pos + j): embedding rows [n][k], the short conv of every (token, channel), causal attention over caches that already hold the prompt's K / V rows (head_dim 32 / 64 / 128 / 256;
// scratch: attention_prefill_scratch_floats).
hipError_t launch_embed_rows(const uint8_t* d_w, int type, uint32_t m, uint32_t k, const uint32_t* d_tokens, uint32_t n, float* d_out,
                             const Launch& L);
hipError_t launch_shortconv_seq(const float* d_proj, float* d_buffer, const float* d_conv_w, float* d_out, uint32_t hidden,
                                uint32_t kernel_size, uint32_t n, const Launch& L);
size_t attention_prefill_scratch_floats(uint32_t n, uint32_t n_heads, uint32_t head_dim);
hipError_t launch_attention_prefill(const float* d_q, const void* d_k_cache, const void* d_v_cache, float* d_out, float* d_scratch,
                                    uint32_t pos0, const uint32_t* d_pos, uint32_t n, uint32_t q_stride, uint32_t out_stride, uint32_t max_seq,
                                    uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, float scale, const Launch& L, int8_t* d_q8 = nullptr,
                                    float* d_q8_scales = nullptr, bool kv_f16 = false);
// The two producers of an out projection's input written directly as Q8_0 blocks (no float result in memory).
bool attention_prefill_quantize_applies(const float* d_q, const void* d_k_cache, const void* d_v_cache, uint32_t n, uint32_t q_stride,
                                        uint32_t head_dim);
bool shortconv_seq_quantize_applies(const float* d_proj, const float* d_buffer, uint32_t hidden);
hipError_t launch_shortconv_seq_quantize(const float* d_proj, float* d_buffer, const float* d_conv_w, int8_t* d_q, float* d_scales, uint32_t hidden,
                                         uint32_t kernel_size, uint32_t n, const Launch& L);
// d_scores is scratch of attention_scratch_floats(max_seq, n_heads, head_dim) floats.
uint32_t attention_splits(uint32_t max_seq);
size_t attention_scratch_floats(uint32_t max_seq, uint32_t n_heads, uint32_t head_dim);
hipError_t launch_attention_decode(const float* d_q, const void* d_k_cache, const void* d_v_cache, float* d_out, float* d_scores,
                                   uint32_t seq_len, const uint32_t* d_pos, uint32_t max_seq, uint32_t n_heads, uint32_t n_kv_heads,
                                   uint32_t head_dim, float scale, const Launch& L, bool kv_f16 = false);
// QK-norm + RoPE + KV append folded into the sequence-split attention kernel, then the merge (head_dim 32 / 64 / 128 / 256).
// d_scratch as for launch_attention_decode.
bool attention_layer_applies(uint32_t head_dim);
hipError_t launch_attention_layer(const float* d_q, const float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm,
                                  void* d_k_cache, void* d_v_cache, float* d_out, float* d_scratch, uint32_t pos,
                                  const uint32_t* d_pos, uint32_t max_seq, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, float eps,
                                  float theta_scale, float scale, const Launch& L, bool kv_f16 = false);
hipError_t launch_shortconv_step(const float* d_proj, float* d_buffer, const float* d_conv_w, float* d_out, uint32_t hidden,
                                 uint32_t kernel_size, const Launch& L);
hipError_t launch_rmsnorm_quantize(const float* d_x, const float* d_weight, uint32_t rows, uint32_t dim, uint32_t x_stride, float eps, int8_t* d_q,
                                   float* d_scales, const Launch& L);
// The same with a residual update in front: x[r][i] += partial[0][r][i] + partial[1][r][i] + .. (the K shares of a split projection,
// added in that order; the sum first, then onto x -- what the split's own reduce launch computes), then norm and quantizer
// of the updated rows.  dim <= kResidualNormMaxDim.
constexpr uint32_t kResidualNormMaxDim = 8192;
hipError_t launch_residual_rmsnorm_quantize(float* d_x, const float* d_partial, uint32_t splits, const float* d_weight, uint32_t rows, uint32_t dim,
                                            uint32_t x_stride, float eps, int8_t* d_q, float* d_scales, const Launch& L);
hipError_t launch_silu_mul_quantize(const float* d_gate, const float* d_up, uint32_t n, uint32_t dim, int8_t* d_q, float* d_scales, const Launch& L);
hipError_t launch_silu_mul(float* d_gate, const float* d_up, uint32_t n, const Launch& L);
// d_history[pos] = pick (pos = *d_pos before it is advanced), when given.  d_partial: scratch of kArgmaxPartials keys, 8-byte aligned;
// d_x 16-byte aligned.
constexpr uint32_t kArgmaxPartials = 4096;  // 64 for the two-stage pick; up to one key per wave of a Q6_K LM head that leaves its own
// d_embd_out non-null: the pick's row of the embedding (d_embd, type, m x k) is written there as the next step's input.
hipError_t launch_argmax(const float* d_x, uint32_t n, unsigned long long* d_partial, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos,
                         uint32_t* d_history, uint32_t history_len, const Launch& L, const uint8_t* d_embd = nullptr, int embd_type = 0,
                         uint32_t embd_m = 0, uint32_t embd_k = 0, float* d_embd_out = nullptr);
// The second stage on its own, over n_partials keys that a producer has left in d_partial (n = the number of candidates; 0: pick 0).
hipError_t launch_argmax_final(const unsigned long long* d_partial, uint32_t n_partials, uint32_t n, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos,
                               uint32_t* d_history, uint32_t history_len, const Launch& L, const uint8_t* d_embd = nullptr, int embd_type = 0,
                               uint32_t embd_m = 0, uint32_t embd_k = 0, float* d_embd_out = nullptr);
hipError_t launch_set_step(uint32_t* d_token, uint32_t token, uint32_t* d_pos, uint32_t pos, const Launch& L, const uint8_t* d_embd = nullptr,
                           int embd_type = 0, uint32_t embd_m = 0, uint32_t embd_k = 0, float* d_embd_out = nullptr);
hipError_t launch_advance_pos(uint32_t* d_pos, const Launch& L);

// n at and above which gemm_q8 uses the MFMA kernel (when k % 128 == 0): the counterpart of GEMM_MIN_N = 16
// (wick/src/model/metal_lfm2.rs:18-21), set where the two routes cross on this GPU.  The multi-token GEMV streams the weight
// once per group of four tokens; the narrow MFMA kernel streams it once and computes 16 token columns at a time.  A 1024 x 1024
// projection inside a prompt pass: up to two groups (n <= 8) the GEMV wins, from n = 9 the MFMA kernel (passes of 12 / 15 tokens
// 0.98 / 1.07 -> 0.89 ms).  A weight whose stream is what a launch costs (16 MB and more: an LM head): one group 29 us, two 58 us,
// the MFMA kernel 34 us for any n <= 16, so it takes over from n = 5.
constexpr uint32_t kGemmMinN = 9;
constexpr uint32_t kGemmMinNLarge = 5;
constexpr size_t kGemmLargeWeightBytes = 16u << 20;
constexpr uint32_t kGemmMaxSplits = 8;  // most K shares of a GEMM launch with few tiles
// Most floats the shares of a split launch can take: (tile, share) pairs fill at most the chip's 512 workgroup slots, a tile is
// at most 128 x 128 sums, and shares x n x m <= pairs x tile.
constexpr size_t kGemmSplitScratchFloats = 512u * 128u * 128u;

}  // namespace wick_rocm
