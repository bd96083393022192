/*
 * wick_oracle.c -- CPU restatement of wick's block-quantized matmul arithmetic.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists so that the HIP
 * kernels can be checked against the arithmetic of the reference's CPU integer
 * kernels (which are aarch64-NEON-only and therefore cannot run on an x86 host).
 * Only tests, the smoke check and the benchmark's cpu-baseline leg may link or
 * load it; the shipped library never does.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference checkout).  All arithmetic is IEEE-754 binary32 with separate
 * multiply and add (compile with -ffp-contract=off), unless a function name
 * ends in _f64.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_f16_bits_to_f32 / orc_f32_to_f16_bits   numpy float16, exhaustively / on edge values
 *   orc_dequant_q4_0_row / orc_dequant_q8_0_row closed-form blocks of wick/src/quant.rs:502-631
 *   orc_quantize_q8_0                           independent numpy-float32 restatement (golden
 *                                               fixture) + invariants; the reference holds no
 *                                               vector for its exact bits
 *   orc_block_dots_*                            brute force over integer extremes; python ints
 *   orc_gemv_* / orc_gemm_*                     f64 dequantize-then-dot, GEMM == per-column GEMV on
 *                                               the reference's own shapes (simd.rs:1440-1623),
 *                                               Q8_0 closed form -16/(row+1) (bench_perf.rs:852-971)
 *   orc_build_q4_0_matrix / orc_build_q8_0_matrix   input generators only; numpy restatement
 *   orc_dequant_q6_k_row                        the reference's closed-form block (all quants 32 -> 0,
 *                                               quant.rs:819-846) + an independent numpy bit-twiddling
 *                                               restatement of quant.rs:380-412 on random bytes
 *   orc_q6k_group_dots_i32, orc_gemv_q6k_q8     python-integer brute force; f64 dequantize-then-dot;
 *                                               the reference's varied block (quant.rs:849-880) dotted
 *                                               both ways
 *   orc_build_q6_k_matrix                       input generator only (round trip error bound)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))
/* Rows are independent (the reference itself hands row chunks to a thread pool, par_rows,
 * wick/src/backend/cpu.rs:222-234), so the row loops may run on several threads without
 * changing any result. */
#define ORC_PAR_ROWS _Pragma("omp parallel for schedule(static)")

enum { Q4_0_BLOCK_BYTES = 18, Q8_0_BLOCK_BYTES = 34, QK = 32 };
enum { ORC_Q4_0 = 2, ORC_Q8_0 = 8 }; /* ggml type ids, wick/src/gguf.rs:36-51 */

/* ---------------------------------------------------------------- f16 <-> f32
 * `half::f16::{from_f32,to_f32}` as used at wick/src/backend/simd.rs:295,385 and
 * wick/src/quant.rs:79,155: IEEE binary16, round-to-nearest-even, subnormals kept. */
ORC_API float orc_f16_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

ORC_API uint16_t orc_f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t a = x & 0x7fffffffu;
    if (a >= 0x7f800000u) { /* inf / nan */
        uint16_t m = (a > 0x7f800000u) ? (uint16_t)(0x200u | ((a >> 13) & 0x3ffu)) : 0;
        return (uint16_t)(sign | 0x7c00u | m);
    }
    if (a < 0x38800000u) { /* |f| < 2^-14: subnormal half or zero */
        uint32_t e = a >> 23;
        if (e < 102) return sign; /* |f| < 2^-25 rounds to zero */
        uint32_t m = (a & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126 - e; /* 14..24 */
        uint32_t r = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return (uint16_t)(sign | r);
    }
    uint32_t e = (a >> 23) - 112u;
    uint32_t m = a & 0x7fffffu;
    uint32_t r = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++; /* carry may roll into inf */
    if (r >= 0x7c00u) r = 0x7c00u;
    return (uint16_t)(sign | r);
}

/* ------------------------------------------------------------ block decoding
 * wick/src/quant.rs:78-90 (Q4_0: element i<16 = low nibble of qs[i], element
 * i+16 = high nibble, value = (nibble-8)*d) and :154-161 (Q8_0). */
ORC_API void orc_dequant_q4_0_row(const uint8_t *src, int64_t n_blocks, float *dst) {
    for (int64_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = src + b * Q4_0_BLOCK_BYTES;
        float d = orc_f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 16; i++) {
            int lo = (blk[2 + i] & 0xF) - 8;
            int hi = (blk[2 + i] >> 4) - 8;
            dst[b * 32 + i] = (float)lo * d;
            dst[b * 32 + i + 16] = (float)hi * d;
        }
    }
}

ORC_API void orc_dequant_q8_0_row(const uint8_t *src, int64_t n_blocks, float *dst) {
    for (int64_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = src + b * Q8_0_BLOCK_BYTES;
        float d = orc_f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 32; i++) dst[b * 32 + i] = (float)(int8_t)blk[2 + i] * d;
    }
}

/* ------------------------------------------------- Q8_0 activation quantizer
 * wick/src/backend/simd.rs:255-323 (quantize_f32_to_q8_0_neon):
 *   amax = max|x|; d = amax/127; id = d != 0 ? 1/d : 0;
 *   scales[b] = f32(f16(d));  q = (i8)(i32) round_ties_even(x * id)   (FCVTNS)
 * `id` comes from the UNROUNDED d.  Returns the number of blocks written. */
ORC_API int64_t orc_quantize_q8_0(const float *x, int64_t k, float *scales, int8_t *quants) {
    int64_t nb = k / QK;
    for (int64_t b = 0; b < nb; b++) {
        const float *xb = x + b * QK;
        float amax = 0.0f;
        for (int i = 0; i < QK; i++) {
            float a = fabsf(xb[i]);
            if (a > amax) amax = a;
        }
        volatile float d = amax / 127.0f;
        volatile float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        scales[b] = orc_f16_bits_to_f32(orc_f32_to_f16_bits(d));
        for (int i = 0; i < QK; i++) {
            volatile float v = xb[i] * id;
            quants[b * QK + i] = (int8_t)(int32_t)nearbyintf(v); /* default mode = ties-to-even */
        }
    }
    return nb;
}

/* n columns, column j starts at x + j*x_stride (token-major source).  Output is
 * the batched layout of wick/src/backend/simd.rs:683-685: scales[j*nb + b],
 * quants[j*k + ...].  (The reference's quantize_columns, wick/src/model/lfm2.rs:571-592,
 * gathers stride-n columns into a contiguous temporary first and then calls the
 * same quantizer per column; the arithmetic per column is identical.) */
ORC_API void orc_quantize_q8_0_batch(const float *x, int64_t n, int64_t k, int64_t x_stride,
                                     float *scales, int8_t *quants) {
    int64_t nb = k / QK;
    for (int64_t j = 0; j < n; j++)
        orc_quantize_q8_0(x + j * x_stride, k, scales + j * nb, quants + j * k);
}

/* ------------------------------------------------------ integer block dots
 * NEON keeps each block dot as four i32 lane partials p[0..3]
 * (vdotq_s32(vdotq_s32(0, w_lo, y_lo), w_hi, y_hi), simd.rs:382, :491): lane l
 * sums elements 4l..4l+3 of the low half and of the high half. */
static inline void q4_0_lane_partials(const uint8_t *blk, const int8_t *xq, int32_t p[4]) {
    for (int l = 0; l < 4; l++) {
        int32_t s = 0;
        for (int i = 4 * l; i < 4 * l + 4; i++) {
            s += ((int)(blk[2 + i] & 0xF) - 8) * (int)xq[i];
            s += ((int)(blk[2 + i] >> 4) - 8) * (int)xq[16 + i];
        }
        p[l] = s;
    }
}

static inline void q8_0_lane_partials(const uint8_t *blk, const int8_t *xq, int32_t p[4]) {
    const int8_t *w = (const int8_t *)(blk + 2);
    for (int l = 0; l < 4; l++) {
        int32_t s = 0;
        for (int i = 4 * l; i < 4 * l + 4; i++) {
            s += (int)w[i] * (int)xq[i];
            s += (int)w[16 + i] * (int)xq[16 + i];
        }
        p[l] = s;
    }
}

static inline int block_bytes_of(int ggml_type) {
    return ggml_type == ORC_Q4_0 ? Q4_0_BLOCK_BYTES : (ggml_type == ORC_Q8_0 ? Q8_0_BLOCK_BYTES : 0);
}

/* out[(j*m + i)*nb + b] = sum of the four lane partials = the exact i32 block dot
 * the parity contract names (simd.rs:369-383 for Q4_0, :478-492 for Q8_0). */
ORC_API int orc_block_dots_i32(int ggml_type, const uint8_t *a, const int8_t *xq, int64_t m,
                               int64_t n, int64_t k, int32_t *out) {
    int bb = block_bytes_of(ggml_type);
    if (!bb || k % QK) return -1;
    int64_t nb = k / QK;
    for (int64_t j = 0; j < n; j++)
        for (int64_t i = 0; i < m; i++)
            for (int64_t b = 0; b < nb; b++) {
                int32_t p[4];
                const uint8_t *blk = a + (i * nb + b) * bb;
                if (ggml_type == ORC_Q4_0)
                    q4_0_lane_partials(blk, xq + j * k + b * QK, p);
                else
                    q8_0_lane_partials(blk, xq + j * k + b * QK, p);
                out[(j * m + i) * nb + b] = p[0] + p[1] + p[2] + p[3];
            }
    return 0;
}

/* ------------------------------------------------------------- GEMV / GEMM
 * One output element in the reference's f32 order (simd.rs:346-407 for Q4_0,
 * :458-516 for Q8_0; the GEMM macros simd.rs:59-86 accumulate the same way):
 *   s = f32(d_w) * xs[b]                             (one rounding)
 *   acc[b&1][l] = acc[b&1][l] + f32(p[l]) * s        (vmlaq_n_f32: mul, then add)
 *   y = vaddvq(acc0) + vaddvq(acc1),  vaddvq = (a0+a1)+(a2+a3)
 * A trailing odd block goes to acc0 (simd.rs:392-404). */
static float row_dot_neon_order(int ggml_type, const uint8_t *row, const float *xs,
                                const int8_t *xq, int64_t nb) {
    int bb = block_bytes_of(ggml_type);
    float acc[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * bb;
        int32_t p[4];
        if (ggml_type == ORC_Q4_0)
            q4_0_lane_partials(blk, xq + b * QK, p);
        else
            q8_0_lane_partials(blk, xq + b * QK, p);
        float dw = orc_f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        volatile float s = dw * xs[b];
        int which = (b + 1 == nb && (nb & 1)) ? 0 : (int)(b & 1);
        for (int l = 0; l < 4; l++) {
            volatile float prod = (float)p[l] * s;
            acc[which][l] = acc[which][l] + prod;
        }
    }
    volatile float h0a = acc[0][0] + acc[0][1], h0b = acc[0][2] + acc[0][3];
    volatile float h1a = acc[1][0] + acc[1][1], h1b = acc[1][2] + acc[1][3];
    volatile float h0 = h0a + h0b, h1 = h1a + h1b;
    return h0 + h1;
}

static double row_dot_f64(int ggml_type, const uint8_t *row, const float *xs, const int8_t *xq,
                          int64_t nb) {
    int bb = block_bytes_of(ggml_type);
    double acc = 0.0;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * bb;
        int32_t p[4];
        if (ggml_type == ORC_Q4_0)
            q4_0_lane_partials(blk, xq + b * QK, p);
        else
            q8_0_lane_partials(blk, xq + b * QK, p);
        double dw = (double)orc_f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        acc += (double)(p[0] + p[1] + p[2] + p[3]) * (dw * (double)xs[b]);
    }
    return acc;
}

/* gemv_q4_0_q8_0_neon / gemv_q8_0_q8_0_neon (simd.rs:328-415, :440-524), reached
 * through gemv_with_preq (wick/src/backend/cpu.rs:334-354). */
ORC_API int orc_gemv_q8(int ggml_type, const uint8_t *a, const float *x_scales,
                        const int8_t *x_quants, float *y, int64_t m, int64_t k) {
    int bb = block_bytes_of(ggml_type);
    if (!bb || k % QK) return -1;
    int64_t nb = k / QK;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++)
        y[i] = row_dot_neon_order(ggml_type, a + i * nb * bb, x_scales, x_quants, nb);
    return 0;
}

ORC_API int orc_gemv_q8_f64(int ggml_type, const uint8_t *a, const float *x_scales,
                            const int8_t *x_quants, double *y, int64_t m, int64_t k) {
    int bb = block_bytes_of(ggml_type);
    if (!bb || k % QK) return -1;
    int64_t nb = k / QK;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++)
        y[i] = row_dot_f64(ggml_type, a + i * nb * bb, x_scales, x_quants, nb);
    return 0;
}

/* gemm_q4_0_q8_0_neon / gemm_q8_0_q8_0_neon (simd.rs:696-925, :937-1019):
 * b_scales[j*nb + b], b_quants[j*k + ...], out[i*n + j] row-major m x n.  Every
 * column tier (8 / 4 / 1 columns) accumulates one (i,j) exactly like the GEMV. */
ORC_API int orc_gemm_q8(int ggml_type, const uint8_t *a, const float *b_scales,
                        const int8_t *b_quants, float *out, int64_t m, int64_t n, int64_t k) {
    int bb = block_bytes_of(ggml_type);
    if (!bb || k % QK) return -1;
    int64_t nb = k / QK;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++)
            out[i * n + j] =
                row_dot_neon_order(ggml_type, a + i * nb * bb, b_scales + j * nb, b_quants + j * k, nb);
    return 0;
}

ORC_API int orc_gemm_q8_f64(int ggml_type, const uint8_t *a, const float *b_scales,
                            const int8_t *b_quants, double *out, int64_t m, int64_t n, int64_t k) {
    int bb = block_bytes_of(ggml_type);
    if (!bb || k % QK) return -1;
    int64_t nb = k / QK;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++)
            out[i * n + j] = row_dot_f64(ggml_type, a + i * nb * bb, b_scales + j * nb, b_quants + j * k, nb);
    return 0;
}

/* ------------------------------------------------------- input generators
 * Weight quantizers the reference's own tests use to make inputs
 * (simd.rs:1371-1394 = tests/gemv_q4_0_bench.rs:14-35 for Q4_0: d = amax/7,
 * q = min(15, (u8)(x*id + 8.5)) with Rust's saturating float->u8 cast;
 * simd.rs:1398-1419 for Q8_0: d = amax/127, q = round-half-away(x*id) clamped). */
static inline uint8_t rust_f32_as_u8(float v) {
    if (!(v > 0.0f)) return 0; /* NaN and negatives saturate to 0 */
    if (v >= 255.0f) return 255;
    return (uint8_t)v;
}

ORC_API void orc_build_q4_0_matrix(const float *values, int64_t m, int64_t k, uint8_t *bytes) {
    int64_t nb = k / QK;
    for (int64_t r = 0; r < m; r++)
        for (int64_t b = 0; b < nb; b++) {
            const float *blk = values + r * k + b * QK;
            uint8_t *o = bytes + (r * nb + b) * Q4_0_BLOCK_BYTES;
            float amax = 0.0f;
            for (int i = 0; i < QK; i++) amax = fmaxf(amax, fabsf(blk[i]));
            volatile float d = amax / 7.0f;
            volatile float id = (d != 0.0f) ? 1.0f / d : 0.0f;
            uint16_t h = orc_f32_to_f16_bits(d);
            o[0] = (uint8_t)(h & 0xff);
            o[1] = (uint8_t)(h >> 8);
            for (int i = 0; i < 16; i++) {
                volatile float t0 = blk[i] * id, t1 = blk[16 + i] * id;
                volatile float u0 = t0 + 8.5f, u1 = t1 + 8.5f;
                uint8_t lo = rust_f32_as_u8(u0), hi = rust_f32_as_u8(u1);
                if (lo > 15) lo = 15;
                if (hi > 15) hi = 15;
                o[2 + i] = (uint8_t)(lo | (hi << 4));
            }
        }
}

ORC_API void orc_build_q8_0_matrix(const float *values, int64_t m, int64_t k, uint8_t *bytes) {
    int64_t nb = k / QK;
    for (int64_t r = 0; r < m; r++)
        for (int64_t b = 0; b < nb; b++) {
            const float *blk = values + r * k + b * QK;
            uint8_t *o = bytes + (r * nb + b) * Q8_0_BLOCK_BYTES;
            float amax = 0.0f;
            for (int i = 0; i < QK; i++) amax = fmaxf(amax, fabsf(blk[i]));
            volatile float d = amax / 127.0f;
            volatile float id = (d != 0.0f) ? 1.0f / d : 0.0f;
            uint16_t h = orc_f32_to_f16_bits(d);
            o[0] = (uint8_t)(h & 0xff);
            o[1] = (uint8_t)(h >> 8);
            for (int i = 0; i < QK; i++) {
                volatile float t = blk[i] * id;
                float q = roundf(t); /* f32::round: half away from zero */
                if (q < -128.0f) q = -128.0f;
                if (q > 127.0f) q = 127.0f;
                o[2 + i] = (uint8_t)(int8_t)q;
            }
        }
}

/* ------------------------------------------------------------------ Q6_K
 * BlockQ6K (wick/src/quant.rs:60-70): 256 weights in 210 bytes
 *   ql[128]  low 4 bits, qh[64]  high 2 bits, scales[16] int8 (one per 16 weights), d f16.
 * Element e = 128 n + 32 j + l  (n < 2, j < 4, l < 32), from dequantize_q6_k_block
 * (quant.rs:380-412):
 *   q = ((ql[64 n + 32 (j & 1) + l] >> 4 (j >> 1)) & 15) | (((qh[32 n + l] >> 2 j) & 3) << 4)
 *   w = f32(d) * scales[e / 16] * (q - 32)
 * (the reference indexes scales as 8 n + l / 16 + 2 j, which is e / 16). */
#define Q6K_BLOCK_BYTES 210
#define Q6K_SUPER 256

static inline int q6k_quant(const uint8_t *blk, int e) {
    int n = e >> 7, j = (e >> 5) & 3, l = e & 31;
    int lo = (blk[64 * n + 32 * (j & 1) + l] >> (4 * (j >> 1))) & 15;
    int hi = (blk[128 + 32 * n + l] >> (2 * j)) & 3;
    return (lo | (hi << 4)) - 32;
}

ORC_API void orc_dequant_q6_k_row(const uint8_t *src, int64_t n_blocks, float *dst) {
    for (int64_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = src + b * Q6K_BLOCK_BYTES;
        const int8_t *sc = (const int8_t *)(blk + 192);
        float d = orc_f16_bits_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
        for (int e = 0; e < Q6K_SUPER; e++) {
            /* d * sc * q, left to right, like quant.rs:400-403 */
            volatile float ds = d * (float)sc[e >> 4];
            dst[b * Q6K_SUPER + e] = ds * (float)q6k_quant(blk, e);
        }
    }
}

/* Exact i32 dot of every 16-weight group with its 16 activation quants:
 * out[(i * (k/16)) + g]  (one token; what gemv_q6k_q8_0_neon feeds to vaddvq_s32). */
ORC_API int orc_q6k_group_dots_i32(const uint8_t *a, const int8_t *xq, int64_t m, int64_t k, int32_t *out) {
    if (k % Q6K_SUPER) return -1;
    int64_t nbk = k / Q6K_SUPER;
    for (int64_t i = 0; i < m; i++)
        for (int64_t b = 0; b < nbk; b++) {
            const uint8_t *blk = a + (i * nbk + b) * Q6K_BLOCK_BYTES;
            for (int g = 0; g < 16; g++) {
                int32_t s = 0;
                for (int t = 0; t < 16; t++) s += q6k_quant(blk, 16 * g + t) * (int32_t)xq[b * Q6K_SUPER + 16 * g + t];
                out[(i * nbk + b) * 16 + g] = s;
            }
        }
    return 0;
}

/* gemv_q6k_q8_0_neon (wick/src/backend/simd.rs:552-679): per row one f32 accumulator;
 * per block, passes n = 0, 1; halves h = 0, 1; then the four groups j = 0..3 of
 * elements 128 n + 32 j + 16 h .. + 15:
 *   dj   = (d * f32(scales[8 n + h + 2 j])) * xs[(256 b + 128 n + 32 j + 16 h) / 32]
 *   sumf = sumf + dj * f32(idot)            (separate multiply and add) */
ORC_API int orc_gemv_q6k_q8(const uint8_t *a, const float *x_scales, const int8_t *x_quants, float *y,
                            int64_t m, int64_t k) {
    if (k % Q6K_SUPER) return -1;
    int64_t nbk = k / Q6K_SUPER;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++) {
        volatile float sumf = 0.0f;
        for (int64_t b = 0; b < nbk; b++) {
            const uint8_t *blk = a + (i * nbk + b) * Q6K_BLOCK_BYTES;
            const int8_t *sc = (const int8_t *)(blk + 192);
            float d = orc_f16_bits_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
            for (int n = 0; n < 2; n++)
                for (int h = 0; h < 2; h++)
                    for (int j = 0; j < 4; j++) {
                        int e0 = 128 * n + 32 * j + 16 * h;
                        int32_t idot = 0;
                        for (int t = 0; t < 16; t++) idot += q6k_quant(blk, e0 + t) * (int32_t)x_quants[b * Q6K_SUPER + e0 + t];
                        volatile float ds = d * (float)sc[8 * n + h + 2 * j];
                        volatile float dj = ds * x_scales[(b * Q6K_SUPER + e0) / 32];
                        volatile float prod = dj * (float)idot;
                        sumf = sumf + prod;
                    }
        }
        y[i] = sumf;
    }
    return 0;
}

ORC_API int orc_gemv_q6k_q8_f64(const uint8_t *a, const float *x_scales, const int8_t *x_quants, double *y,
                                int64_t m, int64_t k) {
    if (k % Q6K_SUPER) return -1;
    int64_t nbk = k / Q6K_SUPER;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++) {
        double acc = 0.0;
        for (int64_t b = 0; b < nbk; b++) {
            const uint8_t *blk = a + (i * nbk + b) * Q6K_BLOCK_BYTES;
            const int8_t *sc = (const int8_t *)(blk + 192);
            double d = (double)orc_f16_bits_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
            for (int e = 0; e < Q6K_SUPER; e++)
                acc += d * (double)sc[e >> 4] * (double)q6k_quant(blk, e) * (double)x_scales[(b * Q6K_SUPER + e) / 32] *
                       (double)x_quants[b * Q6K_SUPER + e];
        }
        y[i] = acc;
    }
    return 0;
}

/* Input generator only (the reference has no Q6_K quantizer; real files come from
 * llama.cpp): a plain round-to-nearest Q6_K encoder.  Per 16 weights s = amax / 31; the
 * super-block scale d = max(s) / 127 (stored as f16); scales[g] = round(s_g / d);
 * q = clamp(round(w / (d * scales[g])), -32, 31) + 32. */
ORC_API void orc_build_q6_k_matrix(const float *values, int64_t m, int64_t k, uint8_t *bytes) {
    int64_t nbk = k / Q6K_SUPER;
    ORC_PAR_ROWS
    for (int64_t i = 0; i < m; i++)
        for (int64_t b = 0; b < nbk; b++) {
            const float *w = values + i * k + b * Q6K_SUPER;
            uint8_t *blk = bytes + (i * nbk + b) * Q6K_BLOCK_BYTES;
            memset(blk, 0, Q6K_BLOCK_BYTES);
            float smax = 0.0f, s[16];
            for (int g = 0; g < 16; g++) {
                float amax = 0.0f;
                for (int t = 0; t < 16; t++) amax = fmaxf(amax, fabsf(w[16 * g + t]));
                s[g] = amax / 31.0f;
                smax = fmaxf(smax, s[g]);
            }
            uint16_t dh = orc_f32_to_f16_bits(smax / 127.0f);
            float d = orc_f16_bits_to_f32(dh);
            blk[208] = (uint8_t)(dh & 0xff);
            blk[209] = (uint8_t)(dh >> 8);
            for (int g = 0; g < 16; g++) {
                int sc = d > 0.0f ? (int)lrintf(s[g] / d) : 0;
                if (sc > 127) sc = 127;
                ((int8_t *)(blk + 192))[g] = (int8_t)sc;
                float step = d * (float)sc;
                for (int t = 0; t < 16; t++) {
                    int e = 16 * g + t;
                    int q = step > 0.0f ? (int)lrintf(w[e] / step) : 0;
                    if (q < -32) q = -32;
                    if (q > 31) q = 31;
                    q += 32;
                    int n = e >> 7, j = (e >> 5) & 3, l = e & 31;
                    blk[64 * n + 32 * (j & 1) + l] |= (uint8_t)((q & 15) << (4 * (j >> 1)));
                    blk[128 + 32 * n + l] |= (uint8_t)((q >> 4) << (2 * j));
                }
            }
        }
}

/* Seeded synthetic data: splitmix64 -> Box-Muller normal deviates, N(0, sigma^2).
 * The reference has no normal generator on this path; this one is this
 * repository's own and only fixes the value distribution of test/bench inputs. */
static inline uint64_t splitmix64(uint64_t *s) {
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

ORC_API void orc_fill_normal(uint64_t seed, float sigma, int64_t n, float *out) {
    uint64_t s = seed;
    for (int64_t i = 0; i < n; i += 2) {
        double u1 = ((double)(splitmix64(&s) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        double u2 = (double)(splitmix64(&s) >> 11) * (1.0 / 9007199254740992.0);
        double r = sqrt(-2.0 * log(u1));
        double a = 6.283185307179586476925286766559 * u2;
        out[i] = (float)(r * cos(a) * (double)sigma);
        if (i + 1 < n) out[i + 1] = (float)(r * sin(a) * (double)sigma);
    }
}
