/*
 * wick_rocm.h -- C ABI of the MI355X (gfx950) backend for wick's block-quantized
 * matmul path: Q8_0 activation quantization, decode GEMV, batched prefill GEMM
 * over GGUF Q4_0 / Q8_0 weight blocks.
 *
 * The reference has no C ABI for this path; its boundary is Rust-internal.  Each
 * entry point below names the reference interface it stands in for (paths are
 * relative to the reference checkout).  A Rust host (`backend/rocm.rs`) binds
 * these with a plain `extern "C"` block and links `libwick_rocm.a`.
 *
 * Conventions
 *   - Every function returns a wick_rocm_status (0 = ok, negative = error) and
 *     never throws or aborts across the boundary.  `wick_rocm_last_error` gives
 *     the message of the last failure on that context (thread-safe copy-out).
 *   - Pointers named d_* are device pointers (HBM); all others are host pointers.
 *   - The caller owns activation / output buffers; the library owns the context,
 *     its stream and uploaded weights.
 *   - All hot-path calls only ENQUEUE work on the context's stream (like encoding
 *     into a Metal command encoder, wick/src/model/metal_lfm2.rs:1-4); nothing
 *     synchronises except wick_rocm_sync / wick_rocm_download / event queries.
 *   - Calls on one context serialise on an internal mutex, the counterpart of the
 *     GPU models' `infer_lock` (wick/src/model/metal_lfm2.rs:254-267).
 *   - Weight bytes keep the GGUF block layout verbatim (wick/src/quant.rs:13-34):
 *     row-major, m rows of k/32 blocks; Q4_0 block = {f16 d; u8 qs[16]} (18 B),
 *     Q8_0 block = {f16 d; i8 qs[32]} (34 B).  That is what is uploaded and what the decode
 *     GEMVs read; the prefill GEMM reads a second layout of the same values that the library
 *     derives on the device at upload (wick_rocm_set_gemm_packing).
 *   - Q6_K weights (wick/src/quant.rs:54-70: {u8 ql[128]; u8 qh[64]; i8 scales[16];
 *     f16 d}, 210 B per 256 weights, k % 256 == 0, k <= 8192) take the decode path
 *     only: the integer Q6_K x Q8_0 GEMV of wick/src/backend/simd.rs:547-640
 *     (one f32 scale product per 16-weight group).  Batched calls run that GEMV once
 *     per token; their quants must be 16-byte aligned.
 *   - Quantized activations use the reference's split layout
 *     (wick/src/kv_cache.rs:103-106, wick/src/backend/simd.rs:683-685):
 *     scales f32 [n][k/32] (values are f16-representable), quants i8 [n][k].
 */
#ifndef WICK_ROCM_H
#define WICK_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum wick_rocm_status {
    WICK_ROCM_OK = 0,
    WICK_ROCM_ERR_INVALID_ARG = -1, /* null pointer, zero size, bad stride or alignment */
    WICK_ROCM_ERR_UNSUPPORTED_DTYPE = -2, /* ggml type other than Q4_0 (2) / Q8_0 (8) / Q6_K (14) */
    WICK_ROCM_ERR_BAD_SHAPE = -3,   /* k % 32 != 0 (Q6_K: k % 256, k > 8192), byte count != rows * row bytes */
    WICK_ROCM_ERR_HIP = -4,         /* a HIP runtime call failed (message has the HIP error) */
    WICK_ROCM_ERR_NO_DEVICE = -5,   /* no gfx950 device with that index */
    WICK_ROCM_ERR_STATE = -6        /* capture begun twice, graph launched while capturing, ... */
} wick_rocm_status;

/* ggml tensor type ids, wick/src/gguf.rs:36-51 */
enum { WICK_ROCM_TYPE_Q4_0 = 2, WICK_ROCM_TYPE_Q8_0 = 8, WICK_ROCM_TYPE_Q6_K = 14 };

/* Output layouts of the batched GEMM. */
enum {
    /* Y[col * y_stride + row]: the GPU call-site convention of encode_gemm,
     * wick/src/model/metal_lfm2.rs:770-776, 881-992. */
    WICK_ROCM_LAYOUT_TOKEN_MAJOR = 0,
    /* out[row * y_stride + col] (y_stride >= n): the CPU kernels' convention,
     * wick/src/backend/simd.rs:685, 696-704. */
    WICK_ROCM_LAYOUT_ROW_MAJOR = 1
};

typedef struct wick_rocm_ctx wick_rocm_ctx;
typedef struct wick_rocm_weight wick_rocm_weight;
typedef struct wick_rocm_graph wick_rocm_graph;
typedef struct wick_rocm_event wick_rocm_event;

/* ---- context ------------------------------------------------------------
 * Stands in for MetalContext::new / GpuContext::new
 * (wick/src/backend/metal.rs:21-191, wick/src/backend/wgpu.rs:15-580): one
 * device, one in-order queue (HIP stream at default priority). */
int wick_rocm_device_count(int *count);
int wick_rocm_ctx_create(int device_id, wick_rocm_ctx **out);
void wick_rocm_ctx_destroy(wick_rocm_ctx *ctx);
/* Copies the last error message of this context into buf (NUL-terminated). */
int wick_rocm_last_error(wick_rocm_ctx *ctx, char *buf, size_t buf_len);
/* "gfx950 ..." device name and CU count, for logs (wick-cli prints the backend label,
 * wick-cli/src/main.rs:869-878). */
int wick_rocm_device_info(wick_rocm_ctx *ctx, char *name_buf, size_t name_len, int *compute_units,
                          size_t *hbm_bytes);
/* The context's hipStream_t, as an opaque pointer, for interop with other HIP code. */
void *wick_rocm_ctx_stream(wick_rocm_ctx *ctx);

/* ---- device buffers (activation / output storage the caller owns) ---------
 * Counterpart of MetalContext::create_buffer / read_f32 (wick/src/backend/metal.rs). */
int wick_rocm_buffer_alloc(wick_rocm_ctx *ctx, size_t nbytes, void **d_ptr);
int wick_rocm_buffer_free(wick_rocm_ctx *ctx, void *d_ptr);
int wick_rocm_upload(wick_rocm_ctx *ctx, void *d_dst, const void *src, size_t nbytes);   /* H2D, ordered on the stream */
int wick_rocm_download(wick_rocm_ctx *ctx, void *dst, const void *d_src, size_t nbytes); /* D2H, waits for the stream */
int wick_rocm_sync(wick_rocm_ctx *ctx);
/* ---- weights ----------------------------------------------------------------
 * Stands in for MetalWeight {mmap_offset, dtype, m, k} (wick/src/model/metal_lfm2.rs:28-36,
 * 409-421).  A discrete GPU cannot wrap the GGUF mmap in place, so the block
 * bytes are copied once, verbatim, into HBM.  `nbytes` must equal
 * m * (k/32) * block_bytes(ggml_type), for Q6_K m * (k/256) * 210.  Q4_0 / Q8_0 weights with k % 128 == 0 also get
 * the prefill GEMM's own layout of the same values (see wick_rocm_set_gemm_packing).  The handle stays valid until
 * wick_rocm_weight_free or context destruction. */
int wick_rocm_weight_upload(wick_rocm_ctx *ctx, const void *host_blocks, size_t nbytes, int ggml_type,
                            uint32_t m, uint32_t k, wick_rocm_weight **out);
/* resolve_weight + upload (wick/src/model/lfm2.rs:310-338, wick/src/model/metal_lfm2.rs:409-421): looks the
 * tensor up in an open GGUF file (include/wick_gguf.h), takes k = ne0 and m = ne1 (m = 1 for rank 1)
 * and uploads its bytes.  Fails like wick_rocm_weight_upload for types / shapes the kernels do not take. */
struct wick_gguf;
int wick_rocm_weight_from_gguf(wick_rocm_ctx *ctx, const struct wick_gguf *gguf, const char *tensor_name, wick_rocm_weight **out);
int wick_rocm_weight_free(wick_rocm_ctx *ctx, wick_rocm_weight *w);
int wick_rocm_weight_info(const wick_rocm_weight *w, int *ggml_type, uint32_t *m, uint32_t *k, size_t *nbytes);
const void *wick_rocm_weight_device_ptr(const wick_rocm_weight *w);

/* ---- Q8_0 activation quantizer ------------------------------------------
 * quantize_f32_to_q8_0_neon (wick/src/backend/simd.rs:255-323; wrapper
 * wick/src/backend/cpu.rs:315-328) applied to n columns, as quantize_to_scratch /
 * quantize_columns do (wick/src/model/lfm2.rs:571-612).  Column j is read from
 * d_x[j * x_stride + 0..k) (token-major f32, x_stride >= k).  Writes
 * d_scales[j * (k/32) + b] and d_quants[j * k + i].  Bit-exact with the
 * reference: d = amax/127, id = 1/d from the unrounded d, stored scale =
 * f32(f16(d)), q = (i8) round-ties-even(x * id). */
int wick_rocm_quantize_q8_0(wick_rocm_ctx *ctx, const float *d_x, uint32_t n, uint32_t k, uint32_t x_stride,
                            int8_t *d_quants, float *d_scales);

/* ---- decode GEMV (n = 1) ----------------------------------------------------
 * gemv_with_preq (wick/src/backend/cpu.rs:334-354) -> gemv_q4_0_q8_0_neon /
 * gemv_q8_0_q8_0_neon (wick/src/backend/simd.rs:328-415, 440-524):
 *   y[i] (+)= sum_b f32(isum_{i,b}) * (f32(d_w[i,b]) * x_scales[b]).
 * `accumulate` != 0 gives y += W x, the residual form of
 * encode_gemv_weight_accumulate (wick/src/model/metal_lfm2.rs:702-710). */
int wick_rocm_gemv_q8(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const int8_t *d_quants, const float *d_scales,
                      float *d_y, int accumulate);

/* Several weights against ONE quantized activation in a single launch: the
 * shared-quantization groups of the decode step ({Q,K,V}, {gate,up};
 * wick/src/model/lfm2.rs:752-775, 1053-1067; fused Metal forms
 * wick/src/model/metal_lfm2.rs:1043-1119).  All weights must share k and dtype. */
int wick_rocm_gemv_q8_multi(wick_rocm_ctx *ctx, const wick_rocm_weight *const *ws, float *const *d_ys, uint32_t count,
                            const int8_t *d_quants, const float *d_scales, int accumulate);

/* ---- batched prefill GEMM -----------------------------------------------
 * gemm_q4_0_q8_0_neon / gemm_q8_0_q8_0_neon (wick/src/backend/simd.rs:696-925,
 * 937-1019; caller gemm_preq, wick/src/model/lfm2.rs:539-565):
 *   C[i,j] (+)= sum_b f32(isum_{i,j,b}) * (f32(d_w[i,b]) * scales[j*nb + b]).
 * Written as Y[j * y_stride + i] (TOKEN_MAJOR, y_stride >= m) or
 * out[i * y_stride + j] (ROW_MAJOR, y_stride >= n).  Any n >= 1; small n takes the
 * bandwidth-bound multi-token GEMV, larger n the int8-MFMA kernel (the hand-off
 * mirrors GEMM_MIN_N, wick/src/model/metal_lfm2.rs:18-21, 899-927). */
int wick_rocm_gemm_q8(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const int8_t *d_quants, const float *d_scales,
                      uint32_t n, float *d_y, uint32_t y_stride, int y_layout, int accumulate);

/* The same for 1..3 weights of one dtype and k over the same quantized activations (Q / K / V, gate / up of a prompt
 * pass: the batched counterpart of encode_gemv_qkv / encode_gemv_gate_up, wick/src/model/metal_lfm2.rs:1043-1119) in
 * one launch, y_i written like wick_rocm_gemm_q8 writes it (shared stride, layout, accumulate flag); results are those
 * of one wick_rocm_gemm_q8 call per weight taken without the K split (wick_rocm_set_gemm_max_k_splits), bit for bit. */
int wick_rocm_gemm_q8_multi(wick_rocm_ctx *ctx, const wick_rocm_weight *const *ws, float *const *d_ys, uint32_t count,
                            const int8_t *d_quants, const float *d_scales, uint32_t n, uint32_t y_stride, int y_layout, int accumulate);

/* A residual projection of a prompt pass together with the norm and quantizer behind it (encode_gemm_add + encode_rmsnorm_batch /
 * encode_add_rmsnorm_batch + quantize_columns, wick/src/model/metal_lfm2.rs:998-1041, 1400-1460; CPU: wick/src/model/lfm2.rs:1380-1420):
 * x[j][.] += W * (activation j) for n token rows x[j * x_stride ..] (w->m floats each), then d_out_quants / d_out_scales =
 * Q8_0(rmsnorm(x[j]) * norm_weight) ([n][m] quants, [n][m / 32] scales).  The same bits as wick_rocm_gemm_q8 (token-major,
 * accumulate) followed by wick_rocm_rmsnorm_quantize_q8_0; when the projection is split over K, the norm's kernel adds the shares
 * up and the split's own reduce launch is not made.  The output may be the projection's own input buffers.  m % 32 == 0. */
int wick_rocm_gemm_q8_residual_rmsnorm_quantize(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const int8_t *d_quants, const float *d_scales,
                                                uint32_t n, float *d_x, uint32_t x_stride, const float *d_norm_weight, float eps,
                                                int8_t *d_out_quants, float *d_out_scales);

/* wick_rocm_weight_upload keeps the raw blocks (what the decode GEMVs stream, as the reference's MetalWeight does,
 * wick/src/model/metal_lfm2.rs:28-36) and, for Q4_0 / Q8_0 weights with k % 128 == 0, also makes the prefill GEMM's own copy on
 * the device: the same int8 values and scales laid out in the order the GEMM's workgroups read them (32-row granules, one
 * contiguous 5 KB slab per granule and 128 K-elements; 1.25 bytes per weight), so that a stage of weights reaches the matrix
 * cores' operand buffer with plain coalesced copies and no unpacking in the main loop.  Results do not depend on it (same
 * integers, same scales).  enabled = 0 switches the copy off for weights uploaded from then on: they take the multi-token GEMV
 * route for any n (slower prompts, 1.25 bytes per weight less memory); so does a weight for whose copy the device had no memory
 * left at upload.  wick_rocm_weight_device_bytes: what a weight holds on
 * the device, both copies.  No counterpart in the reference (its GPU GEMM reads the raw blocks). */
int wick_rocm_set_gemm_packing(wick_rocm_ctx *ctx, int enabled);
size_t wick_rocm_weight_device_bytes(const wick_rocm_weight *w);

/* The n at and above which wick_rocm_gemm_q8 / wick_rocm_matmul_f32 hand off from the
 * multi-token GEMV to the MFMA GEMM: the counterpart of the reference's GEMM_MIN_N = 16
 * (wick/src/model/metal_lfm2.rs:18-21).  Default (min_n = 0): where the two routes cross on
 * this GPU, per weight -- 9, and 5 for weights of 16 MB and more (an LM head).  Results agree
 * to the f32 bar on either side.  A tuning knob, like the reference's WICK_Q4_FAST /
 * WICK_SPLITS switches (wick/src/backend/cpu.rs:23-27). */
int wick_rocm_set_gemm_min_n(wick_rocm_ctx *ctx, uint32_t min_n);

/* A GEMM launch that would leave at least half of the CUs without a tile while walking a long K (few tokens x few rows x
 * k >= 2048: the down projection of a short prompt) is split over K in up to max_splits shares (1, 2, 4, 8): the shares' sums go
 * to context scratch and a second small launch adds them up in a fixed order -- deterministic, but not the same low-order bits
 * as the unsplit sum (both inside the f32 bar).  max_splits = 1 switches it off, 0 restores the default (8).  A tuning knob like
 * the one above; wick_rocm_matmul_f32_noalloc never splits. */
int wick_rocm_set_gemm_max_k_splits(wick_rocm_ctx *ctx, uint32_t max_splits);

/* Which matrix-core instruction the GEMM's block loops are built on: 32 (the default, also 0) = v_mfma_i32_32x32x32_i8
 * (two per block and wave on the wide tile, one on the narrow tile when the launch has more than 48 tokens), 16 = eight / four
 * v_mfma_i32_16x16x32_i8 (what the gated feed-forward launch and narrow launches of up to 48 tokens always use).  Block dots are bit-identical either way, f32 sums agree to the last bit or two (the order in
 * which a row's blocks are added is the same, the lanes that hold them differ).  A tuning knob like the ones above. */
int wick_rocm_set_gemm_mfma_shape(wick_rocm_ctx *ctx, int shape);

/* How the single-token GEMV fetches its weights, by bytes of weights in one launch: below
 * direct_max_bytes every lane loads its own block pair; from there on a wave loads whole
 * cache lines and redistributes them through LDS.  Negative = the built-in default (3 MiB
 * for Q4_0, 512 KiB for Q8_0).  Results do not depend on it.  A tuning knob, like the
 * reference's WICK_Q4_FAST / WICK_SPLITS switches (wick/src/backend/cpu.rs:23-27). */
int wick_rocm_set_gemv_policy(wick_rocm_ctx *ctx, int64_t direct_max_bytes);

/* ---- the literal call-site shape ---------------------------------------
 * encode_gemm(w, x, x_off_bytes, y, y_off_bytes, n, x_stride, y_stride, accumulate)
 * and, with n = 1, encode_gemv_impl(w, input, input_off, output, output_off, accumulate)
 * (wick/src/model/metal_lfm2.rs:881-992, 1231-1335): X[col*x_stride + i] f32 in,
 * Y[col*y_stride + row] f32 out.  Quantizes the n columns into context-owned
 * scratch (grown on demand, never inside a graph capture) and runs GEMV or GEMM.
 * Offsets are in bytes like the reference's. */
int wick_rocm_matmul_f32(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const float *d_x, size_t x_off_bytes, uint32_t n,
                         uint32_t x_stride, float *d_y, size_t y_off_bytes, uint32_t y_stride, int accumulate);
/* wick_rocm_matmul_f32 for callers that cannot allocate.  It has no counterpart in the reference; it exists for callers
 * that must not reach hipMalloc / hipFree: code running under HIP graph capture, tight serving loops, harnesses that
 * forbid allocation.  Same arguments and same kernels, but the Q8_0-quantized activations go into a fixed array in device
 * memory that is part of the library's image (4.5 MiB per GPU, held until the process ends) instead of context scratch that
 * grows on demand.  Results are bit-identical to wick_rocm_matmul_f32 wherever that call does not split its launch over K
 * (wick_rocm_set_gemm_max_k_splits: always with max_splits = 1; with the default only prompts of few tokens over a long K
 * split) and within the f32 bar of it otherwise: this entry point never splits, the shares would need scratch of their own.
 * Limits and rules:
 *   - n * k <= 4194304 elements (e.g. 2048 tokens x 2048, 512 x 8192); larger calls return WICK_ROCM_ERR_BAD_SHAPE;
 *   - no hipMalloc, hipFree or other allocating call is made, on any path; with per-dispatch kernel timing on
 *     (which creates events) the call returns WICK_ROCM_ERR_STATE instead;
 *   - every call on one GPU uses that GPU's one array, from any context: calls that overlap in time on one GPU race
 *     (calls on one context's stream are ordered and safe).  The library refuses the overlap it can see: while one context's
 *     calls (or replays of graphs that captured them) may still be running, a call from ANOTHER context of the same GPU
 *     returns WICK_ROCM_ERR_STATE until the first context has synchronised (wick_rocm_sync, wick_rocm_download);
 *   - the array keeps the last call's contents, and nothing in it needs clearing, because the quantizer rewrites every
 *     byte the matmul reads. */
int wick_rocm_matmul_f32_noalloc(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const float *d_x, size_t x_off_bytes, uint32_t n,
                                 uint32_t x_stride, float *d_y, size_t y_off_bytes, uint32_t y_stride, int accumulate);
/* encode_gemv_qkv / encode_gemv_gate_up (wick/src/model/metal_lfm2.rs:1043-1119):
 * up to four weights sharing k and dtype against ONE f32 activation vector read at
 * d_x + x_off_bytes, y_i (+)= W_i x, in a single launch.  The Q8_0 quantization of x
 * happens inside the GEMV kernel (bit-identical to wick_rocm_quantize_q8_0); shapes
 * the fused kernel does not take (odd block count per row, k > 8192, x not 16-byte
 * aligned) quantize into context scratch first.  wick_rocm_matmul_f32 with n = 1
 * takes the same route. */
int wick_rocm_gemv_f32_multi(wick_rocm_ctx *ctx, const wick_rocm_weight *const *ws, float *const *d_ys, uint32_t count,
                             const float *d_x, size_t x_off_bytes, int accumulate);

/* encode_gemv_rmsnorm_gate_up (wick/src/model/metal_lfm2.rs:1157-1186), for any group of 1..4 weights that share
 * the activation: y_i (+)= W_i * quantize(rmsnorm(x, norm_weight, eps)) in one launch.  cpu::rmsnorm
 * (wick/src/backend/cpu.rs:577-594) is applied to the f32 vector inside the GEMV kernel, in front of its Q8_0
 * quantization; results equal wick_rocm_rmsnorm followed by wick_rocm_gemv_f32_multi up to the last bit of the f64
 * sum of squares.  Weights that cannot take the fused kernel (Q6_K, odd block counts, k > 8192) run the norm as
 * a launch of its own into context scratch (wick_rocm_reserve_scratch before a capture). */
int wick_rocm_gemv_rmsnorm_f32_multi(wick_rocm_ctx *ctx, const wick_rocm_weight *const *ws, float *const *d_ys, uint32_t count,
                                     const float *d_x, const float *d_norm_weight, float eps, int accumulate);
/* The FFN's down projection with its gate folded in: y (+)= W * quantize(silu(gate) * up), cpu::silu_mul_inplace
 * (wick/src/backend/cpu.rs:668-673) applied inside the GEMV kernel (bit-identical to the two separate launches).
 * d_gate is left unchanged. */
int wick_rocm_gemv_silu_mul_f32(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const float *d_gate, const float *d_up, float *d_y,
                                int accumulate);

/* The FFN's gate and up projections with the gate applied in the same launch:
 *   d_act[r] = silu(W_gate[r] . x') * (W_up[r] . x'),  x' = rmsnorm(x, norm_weight, eps) (or x when d_norm_weight is
 * null), quantized to Q8_0 inside the kernel.  One lane ends up with both row sums and applies cpu::silu_mul_inplace
 * (wick/src/backend/cpu.rs:668-673) to them: bit-identical to encode_gemv_rmsnorm_gate_up followed by the silu_mul
 * dispatch (wick/src/model/metal_lfm2.rs:1157-1186, 4225-4238), one launch and one round trip through memory less.
 * Both weights m x k of one type; shapes the kernel does not take (k > 4096, odd block counts, Q6_K) run the three
 * steps separately through context scratch. */
int wick_rocm_ffn_gate_up_f32(wick_rocm_ctx *ctx, const wick_rocm_weight *w_gate, const wick_rocm_weight *w_up, const float *d_x,
                              const float *d_norm_weight, float eps, float *d_act);

/* Pre-sizes the context's scratch for up to max_n columns of up to max_k elements (max_k: the largest row length
 * or row count of any weight used; call before capturing a graph).  Used by wick_rocm_matmul_f32 (n > 1 or a shape
 * the fused kernels do not take) and by the unfused fallbacks of the calls above.  With max_n >= 5 it also holds the room
 * the K shares of a split GEMM launch can take (32 MiB), so that no later batched call regrows the scratch. */
int wick_rocm_reserve_scratch(wick_rocm_ctx *ctx, uint32_t max_n, uint32_t max_k);

/* ---- parity hook ----------------------------------------------------------
 * The exact per-block i32 dots the kernels scale and accumulate
 * (wick/src/backend/simd.rs:369-383, 478-492): d_out[(j*m + i)*(k/32) + b], written by the product kernel
 * that a wick_rocm_gemm_q8 call of the same weight, n and tuning knobs would run (decode GEMV, multi-token GEMV
 * or int8-MFMA GEMM) with the scaling replaced by a store.
 * For Q6_K weights: the i32 dot of every 16-weight group (wick/src/backend/simd.rs:583-630),
 * d_out[(j*m + i)*(k/16) + g]. */
int wick_rocm_block_dots_i32(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const int8_t *d_quants, uint32_t n,
                             int32_t *d_out);
/* The same dots as the fused decode GEMV sees them: one f32 activation vector (16-byte aligned) quantized to Q8_0
 * INSIDE the GEMV kernel (quantize_f32_to_q8_0_neon, wick/src/backend/simd.rs:255-323, then the block dots above),
 * d_out[i*(k/32) + b].  Only shapes the fused kernel takes (even block count per row, k <= 8192); Q4_0 / Q8_0. */
int wick_rocm_block_dots_f32_i32(wick_rocm_ctx *ctx, const wick_rocm_weight *w, const float *d_x, int32_t *d_out);

/* ---- one submission per token -------------------------------------------
 * The reference's GPU backends encode a whole token into one command buffer and
 * commit once (wick/src/model/metal_lfm2.rs:1-4).  The HIP counterpart is stream
 * capture into a graph: begin, enqueue any hot-path calls, end, then launch the
 * graph as often as needed. */
int wick_rocm_graph_begin(wick_rocm_ctx *ctx);
int wick_rocm_graph_end(wick_rocm_ctx *ctx, wick_rocm_graph **out);
int wick_rocm_graph_launch(wick_rocm_ctx *ctx, wick_rocm_graph *g);
int wick_rocm_graph_destroy(wick_rocm_ctx *ctx, wick_rocm_graph *g);

/* ---- GPU timestamps -----------------------------------------------------
 * Counterpart of the reference's GpuTimer (MTLCounterSampleBuffer timestamps,
 * wick/src/model/metal_lfm2.rs:3367-4116): events recorded on the context's stream. */
int wick_rocm_event_create(wick_rocm_ctx *ctx, wick_rocm_event **out);
int wick_rocm_event_record(wick_rocm_ctx *ctx, wick_rocm_event *e);
int wick_rocm_event_elapsed_ms(wick_rocm_ctx *ctx, wick_rocm_event *start, wick_rocm_event *stop, float *ms); /* waits for stop */
int wick_rocm_event_destroy(wick_rocm_ctx *ctx, wick_rocm_event *e);

/* Per-dispatch kernel timestamps, the counterpart of WICK_PROFILE=gpu
 * (per-dispatch counter samples, wick/src/model/metal_lfm2.rs:3367-4116).  Between
 * begin and end every kernel the hot-path calls launch carries its own start/stop
 * timestamps; end waits for the stream and returns, per kernel family
 * (0 = quantizer, 1 = GEMV, 2 = GEMM, 3 = other), the summed execution time in ms
 * and the number of launches.  Arrays hold n_families (<= 4) entries.  Not usable
 * during graph capture. */
int wick_rocm_kernel_timing_begin(wick_rocm_ctx *ctx);
int wick_rocm_kernel_timing_end(wick_rocm_ctx *ctx, double *total_ms, uint64_t *launches, int n_families);

/* Library version string, e.g. "wick-rocm 0.1 (gfx950)". */
const char *wick_rocm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* WICK_ROCM_H */
