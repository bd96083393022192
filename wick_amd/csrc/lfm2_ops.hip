// The non-matmul operations of one LFM2 decode step for gfx950: embedding-row dequantization,
// RMSNorm, per-head QK-norm + RoPE + KV append, decode attention, the gated short convolution,
// SiLU-gate and the greedy pick.  Arithmetic follows the reference's CPU operations
// (wick/src/backend/cpu.rs:577-731, 1320-1401, 2113-2161; wick/src/model/lfm2.rs:621-726);
// each kernel says which steps reproduce them bit for bit and which only to rounding.
//
// Every product / sum that the reference computes as separate f32 operations uses
// __fmul_rn / __fadd_rn / __fsub_rn / __fdiv_rn here: the translation unit is compiled with
// contraction on, and a fused multiply-add would round differently.
//
// "pos" and "token" may live in device memory (d_pos / d_token non-null): a captured graph of
// the step can then be replayed for every token without new kernel arguments.
#include <type_traits>

#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

// The KV caches hold f32 rows, like the reference's CPU model (wick/src/kv_cache.rs), or f16 rows, like its GPU models
// (wick/src/model/metal_lfm2.rs:4117-4247: K after QK-norm and RoPE and V are cast to half on their way into the caches and
// the attention kernels read half).  Every kernel that touches a cache is a template over the element type KV: a value is
// rounded once, to nearest even, when it is appended (or moved by a context shift) and widened exactly when it is read; all
// arithmetic stays f32.
typedef _Float16 kv_h4 __attribute__((ext_vector_type(4)));
template <typename KV>
__device__ __forceinline__ float4 kv_load4(const KV* p) {
    if constexpr (std::is_same<KV, float>::value) {
        return *reinterpret_cast<const float4*>(p);
    } else {
        const kv_h4 v = *reinterpret_cast<const kv_h4*>(p);
        return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
    }
}
template <typename KV>
__device__ __forceinline__ float kv_load(const KV* p) { return (float)*p; }
template <typename KV>
__device__ __forceinline__ void kv_store(KV* p, float v) { *p = (KV)v; }
// launch_kernel over the cache element type: F(float{}) or F(_Float16{}).
template <typename F>
inline hipError_t with_kv_type(bool kv_f16, F&& f) { return kv_f16 ? f(_Float16{}) : f(float{}); }

// Sum over a block of up to 16 waves; every thread gets the total.  `slots` holds 16 doubles.
__device__ __forceinline__ double block_sum_f64(double v, double* slots) {
    v = wave_sum_f64(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();  // slots may still be read from an earlier call
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < nw; i++) t += slots[i];
    return t;
}

// ---- embedding row -------------------------------------------------------------------
// dequantize_row_into (wick/src/model/lfm2.rs:621-643) for Q4_0 / Q8_0 (quant.rs:78-90, 154-161) and
// Q6_K (quant.rs:380-412: d * sc * q left to right): bit-exact.
__device__ __forceinline__ float dequant_element(const uint8_t* __restrict__ w, int type, uint32_t row, uint32_t k, uint32_t e) {
    if (type == kTypeQ6_K) {
        const uint8_t* blk = w + ((size_t)row * (k >> 8) + (e >> 8)) * kQ6KBlockBytes;
        const uint32_t i = e & 255u, n = i >> 7, j = (i >> 5) & 3u, l = i & 31u;
        const uint32_t lo = (blk[64 * n + 32 * (j & 1u) + l] >> (4 * (j >> 1))) & 15u;
        const uint32_t hi = (blk[128 + 32 * n + l] >> (2 * j)) & 3u;
        const int q = (int)(lo | (hi << 4)) - 32;
        const float d = f16_bits_to_f32((uint32_t)blk[208] | ((uint32_t)blk[209] << 8));
        const float sc = (float)(int)(int8_t)blk[192 + (i >> 4)];
        return __fmul_rn(__fmul_rn(d, sc), (float)q);
    }
    if (type == kTypeQ4_0) {
        const uint8_t* blk = w + ((size_t)row * (k >> 5) + (e >> 5)) * kQ4BlockBytes;
        const uint32_t i = e & 31u;
        const uint32_t byte = blk[2 + (i & 15u)];
        const int q = (int)((i < 16u) ? (byte & 15u) : (byte >> 4)) - 8;
        return __fmul_rn((float)q, f16_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8)));
    }
    const uint8_t* blk = w + ((size_t)row * (k >> 5) + (e >> 5)) * kQ8BlockBytes;
    return __fmul_rn((float)(int)(int8_t)blk[2 + (e & 31u)], f16_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8)));
}

__global__ __launch_bounds__(256) void embed_row_kernel(const uint8_t* __restrict__ w, int type, uint32_t m, uint32_t k, uint32_t token,
                                                        const uint32_t* __restrict__ d_token, float* __restrict__ out) {
    const uint32_t row = d_token ? *d_token : token;
    if (row >= m) return;  // the host checks a by-value token; a device-side token out of range leaves `out` untouched
    for (uint32_t e = blockIdx.x * blockDim.x + threadIdx.x; e < k; e += gridDim.x * blockDim.x) out[e] = dequant_element(w, type, row, k, e);
}

// The rows of a whole prompt: out[j][k] = row d_tokens[j] (blockIdx.y = j).
__global__ __launch_bounds__(256) void embed_rows_kernel(const uint8_t* __restrict__ w, int type, uint32_t m, uint32_t k,
                                                         const uint32_t* __restrict__ d_tokens, float* __restrict__ out) {
    const uint32_t row = d_tokens[blockIdx.y];
    if (row >= m) return;
    float* o = out + (size_t)blockIdx.y * k;
    for (uint32_t e = blockIdx.x * blockDim.x + threadIdx.x; e < k; e += gridDim.x * blockDim.x) o[e] = dequant_element(w, type, row, k, e);
}

// ---- RMSNorm ---------------------------------------------------------------------------
// rmsnorm (wick/src/backend/cpu.rs:577-594): f64 sum of squares (summed in another order than the
// reference's loop: the f64 total can differ in its last bits, inv_rms as f32 almost never), then the
// reference's two f32 products.  One block per row; `weight` is shared by all rows.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ weight, float* __restrict__ y,
                                                      uint32_t dim, uint32_t x_stride, uint32_t y_stride, float eps) {
    __shared__ double slots[16];
    const float* xr = x + (size_t)blockIdx.x * x_stride;
    float* yr = y + (size_t)blockIdx.x * y_stride;
    double s = 0.0;
    for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) {
        const double v = (double)xr[i];
        s += v * v;
    }
    const double total = block_sum_f64(s, slots);
    const float inv_rms = (float)(1.0 / sqrt(total / (double)dim + (double)eps));
    for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) yr[i] = __fmul_rn(__fmul_rn(xr[i], inv_rms), weight[i]);
}

// ---- per-head QK-norm + RoPE + KV append ----------------------------------------------------
// forward_attn_block's middle (wick/src/model/lfm2.rs:783-857): every Q and K head is RMS-normalised with
// the shared per-layer weights, rotated (apply_rope_to_head, cpu.rs:2148-2161: split halves, theta
// multiplied up in f32 -- reproduced exactly -- sin/cos from the device library, within an ulp or two
// of libm's), and K / V of this position are appended to the caches [t][kv_dim].
// One 64-thread block per head: blocks [0, n_heads) are Q heads, the rest K heads (which also copy V).
struct QkNormRopeArgs {
    float* q;               // [n_heads * head_dim], in place
    float* k;               // [n_kv_heads * head_dim], in place
    const float* v;         // [n_kv_heads * head_dim]
    const float* q_norm;    // [head_dim]
    const float* k_norm;    // [head_dim]
    void* k_cache;          // [max_seq][kv_dim] of the cache's element type
    void* v_cache;
    const uint32_t* d_pos;  // may be null
    uint32_t pos, max_seq, head_dim, n_heads, n_kv_heads;
    float eps, theta_scale;
    uint32_t q_stride, kv_stride;  // floats between consecutive tokens of q / of k and v (a prompt: blockIdx.y = token, position pos + token)
};

// The rotation of pair i at position pos: angle = pos * theta_scale^i, the power by repeated multiplication as in the
// reference.
__device__ __forceinline__ void rope_sincos(uint32_t pos, uint32_t i, float theta_scale, float& sn, float& cs) {
    float theta = (float)pos;
    for (uint32_t j = 0; j < i; j++) theta = __fmul_rn(theta, theta_scale);
    sincosf(theta, &sn, &cs);
}

// RMSNorm + RoPE of one head by the calling wave: dst[] (and dst2[], when given) receive the result; src may equal dst.
// sn_tab / cs_tab: the position's sines and cosines per pair when the caller has them already (else computed here).
template <typename D1, typename D2>
__device__ __forceinline__ void norm_rope_head(const float* src, const float* w, uint32_t hd, uint32_t pos, float eps, float theta_scale,
                                               D1* dst, D2* dst2, const float* sn_tab = nullptr, const float* cs_tab = nullptr) {
    const uint32_t lane = threadIdx.x & 63u, half = hd >> 1;
    double s = 0.0;
    for (uint32_t i = lane; i < hd; i += 64) {
        const double v = (double)src[i];
        s += v * v;
    }
    const float inv_rms = (float)(1.0 / sqrt(wave_sum_f64(s) / (double)hd + (double)eps));
    for (uint32_t i = lane; i < half; i += 64) {
        float sn, cs;
        if (sn_tab) sn = sn_tab[i], cs = cs_tab[i];
        else rope_sincos(pos, i, theta_scale, sn, cs);
        const float x0 = __fmul_rn(__fmul_rn(src[i], inv_rms), w[i]);
        const float x1 = __fmul_rn(__fmul_rn(src[i + half], inv_rms), w[i + half]);
        const float r0 = __fsub_rn(__fmul_rn(x0, cs), __fmul_rn(x1, sn));
        const float r1 = __fadd_rn(__fmul_rn(x0, sn), __fmul_rn(x1, cs));
        kv_store(dst + i, r0), kv_store(dst + i + half, r1);
        if (dst2) kv_store(dst2 + i, r0), kv_store(dst2 + i + half, r1);
    }
}

template <typename KV>
__device__ __forceinline__ void qk_norm_rope_one_head(const QkNormRopeArgs& a, uint32_t tok, uint32_t pos, uint32_t hh, const float* sn_tab,
                                                      const float* cs_tab) {
    const bool is_q = hh < a.n_heads;
    const uint32_t h = is_q ? hh : hh - a.n_heads;
    const uint32_t hd = a.head_dim, kv_dim = a.n_kv_heads * hd;
    float* head = (is_q ? a.q + (size_t)tok * a.q_stride : a.k + (size_t)tok * a.kv_stride) + (size_t)h * hd;
    const bool store = !is_q && pos < a.max_seq;  // the host checks a by-value pos; a device-side pos past the cache is dropped
    norm_rope_head(head, is_q ? a.q_norm : a.k_norm, hd, pos, a.eps, a.theta_scale, head,
                   store ? static_cast<KV*>(a.k_cache) + (size_t)pos * kv_dim + (size_t)h * hd : static_cast<KV*>(nullptr), sn_tab, cs_tab);
    if (store) {
        const float* vh = a.v + (size_t)tok * a.kv_stride + (size_t)h * hd;
        KV* vc = static_cast<KV*>(a.v_cache) + (size_t)pos * kv_dim + (size_t)h * hd;
        for (uint32_t i = threadIdx.x & 63u; i < hd; i += 64) kv_store(vc + i, vh[i]);
    }
}

template <typename KV>
__global__ __launch_bounds__(64) void qk_norm_rope_kernel(QkNormRopeArgs a) {
    const uint32_t tok = blockIdx.y;
    const uint32_t pos = (a.d_pos ? *a.d_pos : a.pos) + tok;
    qk_norm_rope_one_head<KV>(a, tok, pos, blockIdx.x, nullptr, nullptr);
}

// The same for the tokens of a prompt: one workgroup per token works out the position's sines and cosines once (every
// head of the token uses the same ones) and its four waves share the heads.  Same operations per element: bit-identical.
constexpr uint32_t kRopeTableMax = 128;  // pairs = head_dim / 2
template <typename KV>
__global__ __launch_bounds__(256) void qk_norm_rope_tokens_kernel(QkNormRopeArgs a) {
    __shared__ float sn_tab[kRopeTableMax], cs_tab[kRopeTableMax];
    const uint32_t tok = blockIdx.x;
    const uint32_t pos = (a.d_pos ? *a.d_pos : a.pos) + tok;
    for (uint32_t i = threadIdx.x; i < (a.head_dim >> 1); i += 256) rope_sincos(pos, i, a.theta_scale, sn_tab[i], cs_tab[i]);
    __syncthreads();
    for (uint32_t hh = threadIdx.x >> 6; hh < a.n_heads + a.n_kv_heads; hh += 4) qk_norm_rope_one_head<KV>(a, tok, pos, hh, sn_tab, cs_tab);
}

// head_dim 64: a lane owns one element of a head, so a wave keeps up to six heads in flight -- all their loads first,
// then the arithmetic, then the stores: one memory round trip per wave instead of one per head.  The rotation partner
// (element i +- 32) comes through a lane exchange of the normalised value.  Same operations per element: bit-identical.
template <typename KV>
__global__ __launch_bounds__(256) void qk_norm_rope_tokens64_kernel(QkNormRopeArgs a) {
    constexpr uint32_t HD = 64, HB = 6;
    __shared__ float sn_tab[HD / 2], cs_tab[HD / 2];
    const uint32_t tok = blockIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t pos = (a.d_pos ? *a.d_pos : a.pos) + tok;
    if (threadIdx.x < HD / 2) rope_sincos(pos, threadIdx.x, a.theta_scale, sn_tab[threadIdx.x], cs_tab[threadIdx.x]);
    const uint32_t heads = a.n_heads + a.n_kv_heads, kv_dim = a.n_kv_heads * HD;
    const bool store = pos < a.max_seq;  // the host checks a by-value pos; a device-side pos past the cache is dropped
    const float wq = a.q_norm[lane], wk = a.k_norm[lane];
    for (uint32_t first = 0; first < heads; first += 4u * HB) {  // the same number of trips for every wave: there is a barrier inside
        const uint32_t hh0 = first + wave;
        float v[HB], vv[HB];
        float* head[HB];
#pragma unroll
        for (uint32_t t = 0; t < HB; t++) {
            const uint32_t hh = hh0 + 4u * t;
            const bool is_q = hh < a.n_heads;
            const uint32_t h = is_q ? hh : hh - a.n_heads;
            head[t] = hh < heads ? (is_q ? a.q + (size_t)tok * a.q_stride : a.k + (size_t)tok * a.kv_stride) + (size_t)h * HD : nullptr;
            v[t] = head[t] ? head[t][lane] : 0.0f;
            vv[t] = head[t] && !is_q ? a.v[(size_t)tok * a.kv_stride + (size_t)h * HD + lane] : 0.0f;
        }
        __syncthreads();  // the table (first trip; later trips find it published already)
        const float sn = sn_tab[lane & 31u], cs = cs_tab[lane & 31u];
#pragma unroll
        for (uint32_t t = 0; t < HB; t++) {
            const uint32_t hh = hh0 + 4u * t;  // wave-uniform
            if (hh >= heads) break;
            const bool is_q = hh < a.n_heads;
            const double sq = (double)v[t] * (double)v[t];
            const float inv_rms = (float)(1.0 / sqrt(wave_sum_f64(sq) / (double)HD + (double)a.eps));
            const float xn = __fmul_rn(__fmul_rn(v[t], inv_rms), is_q ? wq : wk);
            const float other = __shfl_xor(xn, 32);
            // lanes 0-31 hold x0 and write r0 = x0 cs - x1 sn; lanes 32-63 hold x1 and write r1 = x0 sn + x1 cs
            const float r = lane < 32u ? __fsub_rn(__fmul_rn(xn, cs), __fmul_rn(other, sn)) : __fadd_rn(__fmul_rn(other, sn), __fmul_rn(xn, cs));
            head[t][lane] = r;
            if (!is_q && store) {
                const size_t at = (size_t)pos * kv_dim + (size_t)(hh - a.n_heads) * HD + lane;
                kv_store(static_cast<KV*>(a.k_cache) + at, r);
                kv_store(static_cast<KV*>(a.v_cache) + at, vv[t]);
            }
        }
    }
}

// ---- n_keep context shift -----------------------------------------------------------------
// InferenceState::shift_kv_with_rope for one attention layer (wick/src/kv_cache.rs:601-700): cache rows
// [n_keep, n_keep + shift) are dropped, the `retained` rows behind them move down by `shift`, and every key head that
// moves is rotated by -shift positions (apply_rope_delta_to_head, wick/src/backend/cpu.rs:2174-2187: the pairs and the
// f32 theta schedule of the forward rotation, started from the angle (float)(-shift); separate multiplies and adds).
// Source and destination rows overlap, so this kernel writes the moved rows -- keys rotated, values as they are -- to
// staging buffers ([retained][kv_dim] each) and plain device copies put them in place afterwards.  A workgroup takes
// kShiftRows rows and computes the sines and cosines once for all of them.
struct KvShiftArgs {
    const void* k_cache;  // caches and staging buffers of the cache's element type
    const void* v_cache;
    void* k_stage;
    void* v_stage;
    uint32_t n_keep, shift, retained, n_kv_heads, head_dim;
    float theta_scale;
};
constexpr uint32_t kShiftRows = 8;

template <typename KV>
__global__ __launch_bounds__(256) void kv_shift_stage_kernel(KvShiftArgs a) {
    __shared__ float sn_tab[kRopeTableMax], cs_tab[kRopeTableMax];
    const uint32_t hd = a.head_dim, half = hd >> 1, kv_dim = a.n_kv_heads * hd;
    for (uint32_t i = threadIdx.x; i < half; i += 256) {
        float theta = -(float)a.shift;
        for (uint32_t j = 0; j < i; j++) theta = __fmul_rn(theta, a.theta_scale);
        sincosf(theta, &sn_tab[i], &cs_tab[i]);
    }
    __syncthreads();
    const uint32_t r0 = blockIdx.x * kShiftRows, r1 = r0 + kShiftRows < a.retained ? r0 + kShiftRows : a.retained;
    for (uint32_t r = r0; r < r1; r++) {
        const KV* ks = static_cast<const KV*>(a.k_cache) + (size_t)(a.n_keep + a.shift + r) * kv_dim;
        const KV* vs = static_cast<const KV*>(a.v_cache) + (size_t)(a.n_keep + a.shift + r) * kv_dim;
        KV* kd = static_cast<KV*>(a.k_stage) + (size_t)r * kv_dim;
        KV* vd = static_cast<KV*>(a.v_stage) + (size_t)r * kv_dim;
        for (uint32_t e = threadIdx.x; e < a.n_kv_heads * half; e += 256) {
            const uint32_t at = (e / half) * hd + e % half;
            const float sn = sn_tab[e % half], cs = cs_tab[e % half];
            const float x0 = kv_load(ks + at), x1 = kv_load(ks + at + half);
            kv_store(kd + at, __fsub_rn(__fmul_rn(x0, cs), __fmul_rn(x1, sn)));
            kv_store(kd + at + half, __fadd_rn(__fmul_rn(x0, sn), __fmul_rn(x1, cs)));
        }
        for (uint32_t e = threadIdx.x; e < kv_dim; e += 256) vd[e] = vs[e];
    }
}

// ---- decode attention -----------------------------------------------------------------
// forward_attn_block's tail (wick/src/model/lfm2.rs:984-1006) = attn_scores -> softmax_inplace -> attn_values
// (cpu.rs:1346-1355, 715-731, 1391-1401), one 256-thread block per query head over positions [0, seq_len).
//   scores: one thread per position, the dot summed in the reference's order: bit-exact;
//   softmax: ggml_expf bit-exact, f64 sum in another order (inverse may differ in the last f32 bit);
//   values: four waves take positions t = wave (mod 4), one lane per dimension, partial sums added at
//           the end: rounding differs from the sequential loop at the 1e-7 level.
// `scores` is scratch [n_heads][max_seq].
struct AttentionArgs {
    const float* q;
    const void* k_cache;  // of the cache's element type
    const void* v_cache;
    float* out;     // [n_heads * head_dim]
    float* scores;  // [n_heads][max_seq]
    const uint32_t* d_pos;  // seq_len = *d_pos + 1 when non-null
    uint32_t seq_len, max_seq, n_heads, n_kv_heads, head_dim;
    float scale;
};

template <typename KV>
__global__ __launch_bounds__(256) void attention_decode_kernel(AttentionArgs a) {
    __shared__ double slots[16];
    __shared__ float red[256];
    __shared__ float qs[256];
    const uint32_t h = blockIdx.x, hd = a.head_dim, kv_dim = a.n_kv_heads * hd;
    uint32_t seq = a.d_pos ? *a.d_pos + 1u : a.seq_len;
    if (seq > a.max_seq) seq = a.max_seq;
    const uint32_t kvh = h / (a.n_heads / a.n_kv_heads);
    const KV* kbase = static_cast<const KV*>(a.k_cache) + (size_t)kvh * hd;
    const KV* vbase = static_cast<const KV*>(a.v_cache) + (size_t)kvh * hd;
    float* sc = a.scores + (size_t)h * a.max_seq;
    const uint32_t tid = threadIdx.x;

    for (uint32_t i = tid; i < hd; i += 256) qs[i] = a.q[(size_t)h * hd + i];
    __syncthreads();

    float mx = -__builtin_inff();
    for (uint32_t t = tid; t < seq; t += 256) {
        const KV* kr = kbase + (size_t)t * kv_dim;
        float dot = 0.0f;
        for (uint32_t d = 0; d < hd; d += 4) {
            const float4 kv = kv_load4(kr + d);
            dot = __fadd_rn(dot, __fmul_rn(qs[d], kv.x));
            dot = __fadd_rn(dot, __fmul_rn(qs[d + 1], kv.y));
            dot = __fadd_rn(dot, __fmul_rn(qs[d + 2], kv.z));
            dot = __fadd_rn(dot, __fmul_rn(qs[d + 3], kv.w));
        }
        const float s = __fmul_rn(dot, a.scale);
        sc[t] = s;
        mx = fmaxf(mx, s);
    }
    red[tid] = mx;
    __syncthreads();
    for (uint32_t off = 128; off > 0; off >>= 1) {
        if (tid < off) red[tid] = fmaxf(red[tid], red[tid + off]);
        __syncthreads();
    }
    mx = red[0];

    double sum = 0.0;
    for (uint32_t t = tid; t < seq; t += 256) {  // each thread revisits the positions it wrote
        const float e = ggml_expf(__fsub_rn(sc[t], mx));
        sc[t] = e;
        sum += (double)e;
    }
    const double total = block_sum_f64(sum, slots);  // its barriers also publish sc[] to the block
    const float inv = (float)(1.0 / total);

    // values: thread = (part, dim); parts take interleaved positions
    const uint32_t lanes = hd < 256u ? hd : 256u;     // hd <= 256 (checked by the host)
    const uint32_t parts = 256u / lanes;               // 4 for head_dim 64
    const uint32_t d = tid % lanes, part = tid / lanes;
    float acc = 0.0f;
    if (part < parts) {
        for (uint32_t t = part; t < seq; t += parts) acc = __fadd_rn(acc, __fmul_rn(__fmul_rn(sc[t], inv), kv_load(vbase + (size_t)t * kv_dim + d)));
    }
    __syncthreads();
    red[tid] = acc;
    __syncthreads();
    if (tid < lanes) {
        float r = red[tid];
        for (uint32_t p = 1; p < parts; p++) r = __fadd_rn(r, red[p * lanes + tid]);
        a.out[(size_t)h * hd + tid] = r;
    }
}

// Long sequences: the same attention split over the sequence.  Workgroup (head, split) walks chunks
// split, split + splits, ... of kAttnChunk positions with a running maximum and rescaled sums (the usual
// streaming softmax), reading whole cache rows with consecutive lanes (a float4 per lane), and leaves
// {max, sum, acc[head_dim]} in scratch; attention_combine_kernel merges the partials of a head.
// Against the single-workgroup kernel above only the summation order and the point where exp() is taken
// change: results agree to a few 1e-7.  head_dim in {32, 64, 128, 256}.
constexpr uint32_t kAttnChunk = 64;       // positions a workgroup handles per pass
constexpr uint32_t kAttnMaxSplits = 64;   // workgroups per head; contexts beyond 64 * 64 positions make them loop

// The chunks of workgroup (h, split): scores against q (HD floats, 16-byte aligned, global or LDS), streaming softmax,
// weighted values; leaves {max, sum, acc[HD]} in the partial record of (h, split).  All 256 threads call it.
template <int HD, typename KV>
__device__ __forceinline__ void attention_chunks(const AttentionArgs& a, uint32_t splits, uint32_t h, uint32_t split, uint32_t seq, const float* q) {
    constexpr uint32_t LR = HD / 4;                  // lanes per cache row
    constexpr uint32_t RPP = 256 / LR;               // rows per pass of the block
    constexpr uint32_t KROWS = kAttnChunk / RPP;     // key rows per thread and chunk
    constexpr uint32_t KB = KROWS < 8 ? KROWS : 8;   // ... loaded in batches of
    constexpr uint32_t VG = 256 / HD;                // position groups of the value sum
    constexpr uint32_t VROWS = kAttnChunk / VG;
    constexpr uint32_t VB = VROWS < 16 ? VROWS : 16;
    static_assert(KROWS >= 1 && KROWS % KB == 0 && VROWS % VB == 0, "chunk does not tile");
    __shared__ float sc[kAttnChunk];
    __shared__ float red[256];
    const uint32_t kv_dim = a.n_kv_heads * HD;
    const uint32_t kvh = h / (a.n_heads / a.n_kv_heads);
    const KV* kbase = static_cast<const KV*>(a.k_cache) + (size_t)kvh * HD;
    const KV* vbase = static_cast<const KV*>(a.v_cache) + (size_t)kvh * HD;
    const uint32_t tid = threadIdx.x, quad = tid % LR, prow = tid / LR, d = tid % HD, g = tid / HD;
    const float4 q4 = reinterpret_cast<const float4*>(q)[quad];
    const uint32_t last = seq - 1u;

    float m_run = -__builtin_inff(), l_run = 0.0f, acc = 0.0f;
    for (uint32_t c = split; c * kAttnChunk < seq; c += splits) {
        const uint32_t t0 = c * kAttnChunk;
        const uint32_t nt = seq - t0 < kAttnChunk ? seq - t0 : kAttnChunk;
        // Loads are unconditional (rows past the end are clamped to the last one and masked afterwards), so the
        // compiler can put a whole batch of them in flight instead of one round trip per row.
#pragma unroll
        for (uint32_t i = 0; i < KROWS; i += KB) {
            float4 kv[KB];
#pragma unroll
            for (uint32_t j = 0; j < KB; j++) {
                const uint32_t row = t0 + prow + (i + j) * RPP;
                kv[j] = kv_load4(kbase + (size_t)(row < last ? row : last) * kv_dim + 4u * quad);
            }
#pragma unroll
            for (uint32_t j = 0; j < KB; j++) {
                const uint32_t r = prow + (i + j) * RPP;
                float p = q4.x * kv[j].x + q4.y * kv[j].y + q4.z * kv[j].z + q4.w * kv[j].w;
                p = group_sum<LR>(p);  // DPP adds inside 16 lanes: no trip through the LDS crossbar
                if (quad == 0) sc[r] = r < nt ? p * a.scale : -__builtin_inff();
            }
        }
        __syncthreads();
        // Every wave takes the chunk's 64 scores (one per lane) and reduces them on its own: no cross-wave exchange,
        // the exponentials are computed four times over instead.
        const uint32_t lane = tid & 63u;
        const float s = sc[lane];
        const float m_new = fmaxf(m_run, wave_max_f32(s));
        const float e = lane < nt ? ggml_expf(s - m_new) : 0.0f;  // positions past the end weigh 0
        const float l_chunk = wave_sum_f32(e);
        __syncthreads();  // every wave has read the scores
        if (tid < kAttnChunk) sc[tid] = e;
        __syncthreads();
        const float corr = ggml_expf(m_run - m_new);    // 0 on the first chunk (m_run = -inf)
        l_run = l_run * corr + l_chunk;
        acc *= corr;
#pragma unroll
        for (uint32_t i = 0; i < VROWS; i += VB) {
            float vv[VB];
#pragma unroll
            for (uint32_t j = 0; j < VB; j++) {
                const uint32_t row = t0 + g + (i + j) * VG;
                vv[j] = kv_load(vbase + (size_t)(row < last ? row : last) * kv_dim + d);
            }
#pragma unroll
            for (uint32_t j = 0; j < VB; j++) acc += sc[g + (i + j) * VG] * vv[j];
        }
        m_run = m_new;
        __syncthreads();  // sc[] is rewritten by the next chunk
    }
    red[tid] = acc;
    __syncthreads();
    float* part = a.scores + ((size_t)h * splits + split) * (HD + 2);
    if (tid < HD) {
        float r = red[tid];
#pragma unroll
        for (uint32_t p = 1; p < VG; p++) r += red[p * HD + tid];
        part[2 + tid] = r;
    }
    if (tid == 0) part[0] = m_run, part[1] = l_run;
}

// Merges the partials of head h: the first wave turns the (max, sum) pairs into weights, then every thread sums its
// share of the weighted accumulators (again with its loads batched).  All 256 threads call it.
template <int HD>
__device__ __forceinline__ void attention_merge(const AttentionArgs& a, uint32_t splits, uint32_t h, uint32_t seq) {
    constexpr uint32_t G = 256 / HD;  // partial groups
    __shared__ float wts[kAttnMaxSplits];
    __shared__ float mred[256];
    __shared__ float total;
    const uint32_t tid = threadIdx.x, d = tid % HD, grp = tid / HD;
    uint32_t active = (seq + kAttnChunk - 1) / kAttnChunk;
    active = active < splits ? active : splits;
    const float* parts = a.scores + (size_t)h * splits * (HD + 2);
    if (tid < 64) {  // splits <= 64: one lane per partial
        const bool on = tid < active;
        const float m_i = on ? parts[(size_t)tid * (HD + 2)] : -__builtin_inff();
        const float l_i = on ? parts[(size_t)tid * (HD + 2) + 1] : 0.0f;
        const float m = wave_max_f32(m_i);
        const float w = on ? ggml_expf(m_i - m) : 0.0f;
        const float l = wave_sum_f32(l_i * w);
        wts[tid] = w;
        if (tid == 0) total = l;
    }
    __syncthreads();
    float o = 0.0f;
    for (uint32_t i0 = grp; i0 < active; i0 += 4 * G) {
        float v[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
            const uint32_t i = i0 + j * G;
            v[j] = parts[(size_t)(i < active ? i : i0) * (HD + 2) + 2 + d];
        }
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
            const uint32_t i = i0 + j * G;
            o += i < active ? v[j] * wts[i] : 0.0f;
        }
    }
    mred[tid] = o;
    __syncthreads();
    if (tid < HD) {
        float r = mred[tid];
#pragma unroll
        for (uint32_t p = 1; p < G; p++) r += mred[p * HD + tid];
        a.out[(size_t)h * HD + tid] = active ? __fdiv_rn(r, total) : 0.0f;
    }
}

__device__ __forceinline__ uint32_t attention_seq(const AttentionArgs& a) {
    const uint32_t seq = a.d_pos ? *a.d_pos + 1u : a.seq_len;
    return seq > a.max_seq ? a.max_seq : seq;
}

template <int HD, typename KV>
__global__ __launch_bounds__(256) void attention_split_kernel(AttentionArgs a, uint32_t splits) {
    const uint32_t h = blockIdx.x / splits, split = blockIdx.x % splits;
    const uint32_t seq = attention_seq(a);
    if (split * kAttnChunk >= seq) return;  // the combine step derives the number of partials from seq as well
    attention_chunks<HD, KV>(a, splits, h, split, seq, a.q + (size_t)h * HD);
}

template <int HD>
__global__ __launch_bounds__(256) void attention_combine_kernel(AttentionArgs a, uint32_t splits) {
    attention_merge<HD>(a, splits, blockIdx.x, attention_seq(a));
}

// The attention block between the Q/K/V projections and the output projection with QK-norm, RoPE and the KV append
// folded into the sequence-split kernel (wick/src/model/lfm2.rs:783-1006): every workgroup (head, split) norms and
// rotates its own query head into LDS (same arithmetic as qk_norm_rope_kernel); the workgroups whose chunk holds the
// new position norm and rotate the key head, append it and the value row to the caches (query heads that share a KV
// head write identical bytes) and read them back after a barrier.  No workgroup depends on another; the partials are
// merged by attention_combine_kernel as before.  Results are bit-identical to qk_norm_rope + attention_split +
// attention_combine, one launch less.  (Merging in the last workgroup to finish, behind a ticket counter, was built
// and measured: the device-scope fences it needs write back and invalidate the L2 per workgroup and cost far more
// than the launch they save.)
struct AttentionLayerArgs {
    AttentionArgs at;     // q unused; caches as read
    const float* q_raw;   // [n_heads * HD] projection output, left unchanged
    const float* k_raw;   // [n_kv_heads * HD]
    const float* v;       // [n_kv_heads * HD]
    const float* q_norm;
    const float* k_norm;
    void* k_cache;        // the same caches, writable
    void* v_cache;
    float eps, theta_scale;
};

template <int HD, typename KV>
__global__ __launch_bounds__(256) void attention_layer_kernel(AttentionLayerArgs f, uint32_t splits) {
    __shared__ __align__(16) float qh[HD];
    const AttentionArgs& a = f.at;
    const uint32_t h = blockIdx.x / splits, split = blockIdx.x % splits, tid = threadIdx.x;
    const uint32_t seq = attention_seq(a);
    if (seq == 0 || split * kAttnChunk >= seq) return;
    const uint32_t pos = seq - 1u, kv_dim = a.n_kv_heads * HD, kvh = h / (a.n_heads / a.n_kv_heads);
    if (tid < 64) norm_rope_head(f.q_raw + (size_t)h * HD, f.q_norm, HD, pos, f.eps, f.theta_scale, qh, static_cast<float*>(nullptr));
    if ((pos / kAttnChunk) % splits == split) {  // this workgroup's chunks include the new position
        if (tid >= 64 && tid < 128)
            norm_rope_head(f.k_raw + (size_t)kvh * HD, f.k_norm, HD, pos, f.eps, f.theta_scale,
                           static_cast<KV*>(f.k_cache) + (size_t)pos * kv_dim + (size_t)kvh * HD, static_cast<float*>(nullptr));
        if (tid >= 128) {
            const float* vh = f.v + (size_t)kvh * HD;
            KV* vc = static_cast<KV*>(f.v_cache) + (size_t)pos * kv_dim + (size_t)kvh * HD;
            for (uint32_t i = tid - 128; i < HD; i += 128) kv_store(vc + i, vh[i]);
        }
    }
    __syncthreads();  // qh[] and this workgroup's cache rows are complete
    attention_chunks<HD, KV>(a, splits, h, split, seq, qh);
}

// Causal attention for the n tokens of a prompt whose K / V rows are already in the caches (pass B of the reference's
// batched prefill, wick/src/model/lfm2.rs:1640-1700).  A workgroup takes QB = 8 consecutive query tokens of one head and
// walks the 64-position chunks of the cache once for all of them: every key / value row it loads serves eight queries
// (one workgroup per query re-read the caches 2002 times for a 2002-token prompt and was L2-bound at 1 ms per layer).
// Per chunk: scores of the 8 queries (rows past a query's own position masked), streaming softmax with each wave
// owning two queries (64 positions = one wave: shuffles only), then the weighted value sums for all eight from one set
// of value loads.  q: [n][q_stride] floats, out: [n][out_stride].
template <int HD, typename KV>
__global__ __launch_bounds__(256) void attention_prefill_kernel(AttentionArgs a, uint32_t pos0, uint32_t n, uint32_t q_stride, uint32_t out_stride) {
    constexpr uint32_t QB = 8;
    constexpr uint32_t LR = HD / 4, RPP = 256 / LR, KROWS = kAttnChunk / RPP, KB = KROWS < 4 ? KROWS : 4;
    constexpr uint32_t VG = 256 / HD, VROWS = kAttnChunk / VG, VB = VROWS < 8 ? VROWS : 8;
    static_assert(VB % 4 == 0, "weights are read four at a time");
    static_assert(kAttnChunk == 64 && KROWS % KB == 0 && VROWS % VB == 0, "one wave per query's softmax needs 64-position chunks");
    __shared__ __align__(16) float sc[QB][kAttnChunk];
    __shared__ float corr[QB], lsum[QB];
    __shared__ float red[256];
    const uint32_t h = blockIdx.x, j0 = blockIdx.y * QB;
    const uint32_t nq = n - j0 < QB ? n - j0 : QB;  // queries of this workgroup
    const uint32_t base = a.d_pos ? *a.d_pos : pos0;
    const uint32_t kv_dim = a.n_kv_heads * HD, kvh = h / (a.n_heads / a.n_kv_heads);
    const KV* kbase = static_cast<const KV*>(a.k_cache) + (size_t)kvh * HD;
    const KV* vbase = static_cast<const KV*>(a.v_cache) + (size_t)kvh * HD;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, quad = tid % LR, prow = tid / LR, d = tid % HD, g = tid / HD;
    uint32_t seq_max = base + j0 + nq;  // positions the last query sees
    if (seq_max > a.max_seq) seq_max = a.max_seq;
    const uint32_t last = seq_max - 1u;

    float4 q4[QB];
#pragma unroll
    for (uint32_t q = 0; q < QB; q++)
        q4[q] = reinterpret_cast<const float4*>(a.q + (size_t)(j0 + (q < nq ? q : 0u)) * q_stride + (size_t)h * HD)[quad];
    float acc[QB];
#pragma unroll
    for (uint32_t q = 0; q < QB; q++) acc[q] = 0.0f;
    float m_run[2] = {-__builtin_inff(), -__builtin_inff()}, l_run[2] = {0.0f, 0.0f};  // of queries 2 * wave, 2 * wave + 1

    for (uint32_t t0 = 0; t0 < seq_max; t0 += kAttnChunk) {
#pragma unroll
        for (uint32_t i = 0; i < KROWS; i += KB) {
            float4 kv[KB];
#pragma unroll
            for (uint32_t jj = 0; jj < KB; jj++) {
                const uint32_t row = t0 + prow + (i + jj) * RPP;
                kv[jj] = kv_load4(kbase + (size_t)(row < last ? row : last) * kv_dim + 4u * quad);
            }
#pragma unroll
            for (uint32_t jj = 0; jj < KB; jj++) {
                const uint32_t r = prow + (i + jj) * RPP;
#pragma unroll
                for (uint32_t q = 0; q < QB; q++) {
                    float p = q4[q].x * kv[jj].x + q4[q].y * kv[jj].y + q4[q].z * kv[jj].z + q4[q].w * kv[jj].w;
                    p = group_sum<LR>(p);  // DPP adds inside 16 lanes: no trip through the LDS crossbar
                    // causal: query q (token j0 + q) sees positions <= base + j0 + q
                    if (quad == 0) sc[q][r] = (q < nq && t0 + r <= base + j0 + q && t0 + r < a.max_seq) ? p * a.scale : -__builtin_inff();
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t w2 = 0; w2 < 2; w2++) {  // this wave's two queries: one lane per position of the chunk
            const uint32_t q = 2 * wave + w2;
            const float s = sc[q][lane];
            const float m_new = fmaxf(m_run[w2], wave_max_f32(s));
            // a chunk (or a query slot) with nothing to see keeps -inf: weights 0, nothing rescaled
            const float e = m_new == -__builtin_inff() ? 0.0f : ggml_expf(s - m_new);
            const float l = wave_sum_f32(e);
            const float c = m_new == -__builtin_inff() ? 1.0f : ggml_expf(m_run[w2] - m_new);
            sc[q][lane] = e;
            l_run[w2] = l_run[w2] * c + l;
            m_run[w2] = m_new;
            if (lane == 0) corr[q] = c;
        }
        __syncthreads();
#pragma unroll
        for (uint32_t q = 0; q < QB; q++) acc[q] *= corr[q];
        // group g takes the contiguous positions g * VROWS .. of the chunk: its weights come as 16-byte LDS reads
#pragma unroll
        for (uint32_t i = 0; i < VROWS; i += VB) {
            float vv[VB];
#pragma unroll
            for (uint32_t jj = 0; jj < VB; jj++) {
                const uint32_t row = t0 + g * VROWS + i + jj;
                vv[jj] = kv_load(vbase + (size_t)(row < last ? row : last) * kv_dim + d);
            }
#pragma unroll
            for (uint32_t q = 0; q < QB; q++) {
#pragma unroll
                for (uint32_t jj = 0; jj < VB; jj += 4) {
                    const float4 w4 = *reinterpret_cast<const float4*>(&sc[q][g * VROWS + i + jj]);
                    acc[q] += w4.x * vv[jj] + w4.y * vv[jj + 1] + w4.z * vv[jj + 2] + w4.w * vv[jj + 3];
                }
            }
        }
        __syncthreads();  // sc[] and corr[] are rewritten by the next chunk
    }
    if (lane == 0) lsum[2 * wave] = l_run[0], lsum[2 * wave + 1] = l_run[1];
#pragma unroll
    for (uint32_t q = 0; q < QB; q++) {
        __syncthreads();  // red[] of the previous query has been read; lsum[] is published before the first read
        red[tid] = acc[q];
        __syncthreads();
        if (tid < HD && q < nq) {
            float r = red[tid];
#pragma unroll
            for (uint32_t p = 1; p < VG; p++) r += red[p * HD + tid];
            a.out[(size_t)(j0 + q) * out_stride + (size_t)h * HD + tid] = __fdiv_rn(r, lsum[q]);
        }
    }
}

// The same causal attention on the matrix cores, head_dim 64.  Sixteen queries of one head per wave; the cache is walked in
// tiles of 64 positions that a workgroup's waves share through LDS.
//   scores, transposed:  S^T[key][q] = sum_d K[key][d] Q[q][d]   A = K (keys are the M rows), B = Q^T;
//     in the 16 x 16 result lane l holds keys 4 * (l / 16) + r of query l % 16.
//   weighted values, transposed:  O^T[d][q] = sum_key V[key][d] P[key][q]   A = V^T, B = P: the B operand wants, per lane,
//     consecutive K-steps (= keys) of one query -- exactly what the score MFMA left in the lane's registers, so the softmax
//     weights go from one product into the next without leaving their registers (the order of an MFMA's K steps is free as
//     long as both operands agree on it).
// Streaming softmax per query across the tiles (running maximum shared by the four lane groups of a query, partial sums of
// the weights kept per lane and added up at the end).
// Causal work grows with the query's position, so with HALVES == 2 a workgroup takes two blocks of 64 queries, block
// (last - y) and block y: every workgroup then covers the same number of (wave, tile) steps and the two blocks share
// one copy of each K/V tile; the short block's waves drop out of the arithmetic (not the barriers) once their
// queries are past.  Each block of 64 queries is served by 8 waves: a second wave per 16 queries takes the upper 32
// keys of every tile with a softmax state of its own, and the two states are merged at the end through LDS -- four
// waves per SIMD while both blocks run and two when only the long one is left, so that one wave's exp / rescale work
// overlaps another's MFMAs.  Two tiles sit in LDS: tile t+1 is written (and tile t+2 requested) after the arithmetic
// of tile t, into the buffer that tile t-1 left -- one barrier per tile, and no wave waits for global memory before it
// multiplies.
typedef float v4f __attribute__((ext_vector_type(4)));

// Both products run on the f16 matrix cores at f32 accuracy: every f32 operand x is
// split into hi = f16(x) and lo = f16(x - hi) (22-23 significant bits together) and a product a * b is taken as
// a_hi b_hi + a_hi b_lo + a_lo b_hi, each an exact f16 x f16 product accumulated in f32 by v_mfma_f32_16x16x32_f16 (the
// dropped a_lo b_lo term is below 2^-22 of the product).  Three MFMAs of K = 32 in 16 cycles each replace eight f32 MFMAs
// of K = 4 in 32 cycles each: the matrix time drops by a factor of five and the kernel becomes bound by the softmax's
// vector work.  K tiles sit in LDS as f16 hi / lo rows, V tiles transposed ([dim][key]) so that the second product's A
// operand (V^T: 8 keys of one dim per lane) is two 8-byte reads; the softmax weights are scaled by 2^12 before the
// split (exact, undone at the end) so that small weights keep their bits in f16.  Slot j of lane group g stands for
// key 4 g + j of the wave's first 16-key sub-tile (j < 4) or of its second (j >= 4) in both operands of the second
// product, which is again exactly how the first product leaves the weights in the registers.
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void split_f16(float x, _Float16& hi, _Float16& lo) {
    hi = (_Float16)x;
    lo = (_Float16)(x - (float)hi);
}

// Reductions over the four lane groups of a query (lanes l, l ^ 16, l ^ 32, l ^ 48) with gfx950's row / half swaps: swapping a
// register with a copy of itself leaves the two partners' values in the pair, so their maximum (or sum) needs no select
// and no trip through the LDS crossbar.  Every lane ends with the result.
__device__ __forceinline__ float groups_max(float v) {
    const uint32_t b = __float_as_uint(v);
    auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    const uint32_t c = __float_as_uint(v);
    auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
    return fmaxf(__uint_as_float(q[0]), __uint_as_float(q[1]));
}
__device__ __forceinline__ float groups_sum(float v) {
    const uint32_t b = __float_as_uint(v);
    auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    const uint32_t c = __float_as_uint(v);
    auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

// exp(x) for x <= 0 (-inf included) on the hardware's exp2 (v_exp_f32, about one ulp): two instructions where the polynomial of
// ggml_expf takes about thirty, and the softmax of a tile is nine of them per lane.  The weights differ from ggml_expf's in the
// last bit or two; the streaming softmax of this kernel differs from the reference's two-pass one at that level anyway.
__device__ __forceinline__ float exp_nonpos_hw(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// KV = _Float16 (f16 caches): K and V are their own high halves and have no low halves, so the K_lo Q_hi and V_lo P_hi
// products, their operand reads and the low planes' LDS writes drop out (8 of the 12 MFMAs per wave and tile remain).
template <int HALVES, typename KV>
__global__ __launch_bounds__(512 * HALVES) void attention_prefill_f16x3_kernel(AttentionArgs a, uint32_t pos0, uint32_t n, uint32_t q_stride, uint32_t out_stride,
                                                                                int8_t* q_out, float* s_out) {
    constexpr bool LO = std::is_same<KV, float>::value;  // the caches' values have low halves
    constexpr int HD = 64, KT = 64, NT = 512 * HALVES;
    constexpr int LDH = 72;  // f16 per K row: 64 + 8 (144 bytes: 16-byte aligned rows, conflict-free 16-byte operand reads)
    constexpr int LDV = 68;  // f16 per V^T row: 64 + 4 (136 bytes: 8-byte aligned rows; 64 rows' 8-byte writes cover all banks twice)
    constexpr float kPScale = 4096.0f;
    __shared__ __align__(16) _Float16 kbuf[2][2][KT][LDH];  // [buffer][hi | lo][key][dim]
    __shared__ __align__(16) _Float16 vbuf[2][2][HD][LDV];  // [buffer][hi | lo][dim][key]
    const uint32_t h = blockIdx.x;
    const uint32_t qblocks = (n + 63u) / 64u;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
    const uint32_t wave_id = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t wave = wave_id & 3u, ksp = (wave_id >> 2) & 1u, half = wave_id >> 3;
    const uint32_t qb_long = qblocks - 1u - blockIdx.y;
    const uint32_t qb = half == 0 ? qb_long : blockIdx.y;
    const bool active = half == 0 || qb != qb_long;
    const uint32_t j0 = qb * 64u;
    const uint32_t base = a.d_pos ? *a.d_pos : pos0;
    const uint32_t kv_dim = a.n_kv_heads * HD, kvh = h / (a.n_heads / a.n_kv_heads);
    const KV* kbase = static_cast<const KV*>(a.k_cache) + (size_t)kvh * HD;
    const KV* vbase = static_cast<const KV*>(a.v_cache) + (size_t)kvh * HD;
    const uint32_t jq = j0 + 16u * wave + l16;
    const uint32_t jl = jq < n ? jq : n - 1u;
    const uint32_t pq = base + jl;
    uint32_t wg_last = base + (qb_long * 64u + 63u < n ? qb_long * 64u + 63u : n - 1u);
    if (wg_last >= a.max_seq) wg_last = a.max_seq - 1u;
    const uint32_t wave_last = min(base + min(j0 + 16u * wave + 15u, n - 1u), wg_last);

    // this lane's query, dims 32 s + 8 g .. + 7 of slab s, scaled and split
    h8 qh[2], ql[2];
    {
        const float* qp = a.q + (size_t)jl * q_stride + (size_t)h * HD + 8u * g;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const float4 v0 = *reinterpret_cast<const float4*>(qp + 32 * s), v1 = *reinterpret_cast<const float4*>(qp + 32 * s + 4);
            const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                _Float16 hi, lo;
                split_f16(f[i] * a.scale, hi, lo);
                qh[s][i] = hi, ql[s][i] = lo;
            }
        }
    }
    v4f o[4];
#pragma unroll
    for (int c = 0; c < 4; c++) o[c] = v4f{0.f, 0.f, 0.f, 0.f};
    float m_run = -__builtin_inff(), l_run = 0.0f;

    constexpr int C4 = HD / 4, RPP = NT / C4, NR = KT / RPP;
    const uint32_t c4 = tid % C4, r0 = tid / C4;
    float4 kk[NR], vv[NR];
    auto fetch_tile = [&](uint32_t t0) {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const uint32_t key = min(t0 + r0 + i * RPP, wg_last);
            kk[i] = kv_load4(kbase + (size_t)key * kv_dim + 4u * c4);
            vv[i] = kv_load4(vbase + (size_t)key * kv_dim + 4u * c4);
        }
    };
    // A thread holds one key x four dims of K and of V.  K rows go to LDS as they are; V is transposed on the way: the four
    // lane groups of a wave hold four consecutive keys of the same dims, so a 4 x 4 transpose across them (two rounds of
    // row / half swaps on {hi, lo} pairs packed into one register) leaves every lane with four keys of one dim = one
    // 8-byte write per half, instead of eight conflicting 2-byte writes.
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const uint32_t key = r0 + i * RPP;
            const float kf[4] = {kk[i].x, kk[i].y, kk[i].z, kk[i].w}, vf[4] = {vv[i].x, vv[i].y, vv[i].z, vv[i].w};
            h4 khi, klo;
            uint32_t vp[4];  // V of this key: dim j as {hi, lo}
#pragma unroll
            for (int j = 0; j < 4; j++) {
                _Float16 hi, lo;
                split_f16(kf[j], hi, lo);
                khi[j] = hi, klo[j] = lo;
                split_f16(vf[j], hi, lo);
                vp[j] = (uint32_t)__builtin_bit_cast(uint16_t, hi) | ((uint32_t)__builtin_bit_cast(uint16_t, lo) << 16);
            }
            *reinterpret_cast<h4*>(&kbuf[buf][0][key][4 * c4]) = khi;
            if constexpr (LO) *reinterpret_cast<h4*>(&kbuf[buf][1][key][4 * c4]) = klo;
            // transpose M[g][j] (g = lane group = key, j = register = dim) in 2 x 2 blocks, then the blocks themselves
            auto s01 = __builtin_amdgcn_permlane16_swap(vp[0], vp[1], false, false);
            auto s23 = __builtin_amdgcn_permlane16_swap(vp[2], vp[3], false, false);
            auto t02 = __builtin_amdgcn_permlane32_swap(s01[0], s23[0], false, false);
            auto t13 = __builtin_amdgcn_permlane32_swap(s01[1], s23[1], false, false);
            const uint32_t w[4] = {t02[0], t13[0], t02[1], t13[1]};  // this lane's dim 4 c4 + g, keys (key & ~3) + 0 .. 3
            uint2 vhi, vlo;
            vhi.x = __builtin_amdgcn_perm(w[1], w[0], 0x05040100u), vhi.y = __builtin_amdgcn_perm(w[3], w[2], 0x05040100u);
            vlo.x = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u), vlo.y = __builtin_amdgcn_perm(w[3], w[2], 0x07060302u);
            const uint32_t key4 = key & ~3u;
            *reinterpret_cast<uint2*>(&vbuf[buf][0][4 * c4 + g][key4]) = vhi;
            if constexpr (LO) *reinterpret_cast<uint2*>(&vbuf[buf][1][4 * c4 + g][key4]) = vlo;
        }
    };
    fetch_tile(0);
    store_tile(0);
    if (KT <= wg_last) fetch_tile(KT);
    __syncthreads();
    int cur = 0;
    for (uint32_t t0 = 0; t0 <= wg_last; t0 += KT, cur ^= 1) {
        const uint32_t key0 = t0 + 32u * ksp;  // this wave's 32 keys of the tile
        if (active && key0 <= wave_last) {
            // scores: 2 sub-tiles of 16 keys x 2 slabs of 32 dims x 3 products
            v4f sc[2] = {v4f{0.f, 0.f, 0.f, 0.f}, v4f{0.f, 0.f, 0.f, 0.f}};
            h8 kh[2][2], kl[2][2];  // [slab][sub-tile]
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    kh[s][u] = *reinterpret_cast<const h8*>(&kbuf[cur][0][32u * ksp + 16 * u + l16][32 * s + 8 * g]);
                    if constexpr (LO) kl[s][u] = *reinterpret_cast<const h8*>(&kbuf[cur][1][32u * ksp + 16 * u + l16][32 * s + 8 * g]);
                }
#pragma unroll
            for (int s = 0; s < 2; s++) {
                if constexpr (LO) {
#pragma unroll
                    for (int u = 0; u < 2; u++) sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kl[s][u], qh[s], sc[u], 0, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < 2; u++) sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh[s][u], ql[s], sc[u], 0, 0, 0);
#pragma unroll
                for (int u = 0; u < 2; u++) sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh[s][u], qh[s], sc[u], 0, 0, 0);
            }
            // the V operands of the second product are on their way while the softmax runs
            h8 vh[4], vl[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const h4 a0 = *reinterpret_cast<const h4*>(&vbuf[cur][0][16 * c + l16][32u * ksp + 4 * g]);
                const h4 a1 = *reinterpret_cast<const h4*>(&vbuf[cur][0][16 * c + l16][32u * ksp + 16 + 4 * g]);
                vh[c] = h8{a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                if constexpr (LO) {
                    const h4 b0 = *reinterpret_cast<const h4*>(&vbuf[cur][1][16 * c + l16][32u * ksp + 4 * g]);
                    const h4 b1 = *reinterpret_cast<const h4*>(&vbuf[cur][1][16 * c + l16][32u * ksp + 16 + 4 * g]);
                    vl[c] = h8{b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
                }
            }
            float tmax = -__builtin_inff();
            const bool masked_tile = key0 + 31u > base + min(j0 + 16u * wave, n - 1u);
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (masked_tile && key0 + 16u * u + 4u * g + r > pq) sc[u][r] = -__builtin_inff();
                    tmax = fmaxf(tmax, sc[u][r]);
                }
            tmax = groups_max(tmax);
            const float m_new = fmaxf(m_run, tmax);
            const float m_sub = m_new == -__builtin_inff() ? 0.0f : m_new;
            const float alpha = exp_nonpos_hw(m_run - m_sub);
            m_run = m_new;
            float psum = 0.0f;
            h8 ph, pl;
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float pw = exp_nonpos_hw(sc[u][r] - m_sub);
                    psum += pw;
                    _Float16 hi, lo;
                    split_f16(pw * kPScale, hi, lo);
                    ph[4 * u + r] = hi, pl[4 * u + r] = lo;
                }
            l_run = l_run * alpha + psum;
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] *= alpha;
            if constexpr (LO) {
#pragma unroll
                for (int c = 0; c < 4; c++) o[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vl[c], ph, o[c], 0, 0, 0);
            }
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vh[c], pl, o[c], 0, 0, 0);
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vh[c], ph, o[c], 0, 0, 0);
        }
        if (t0 + KT <= wg_last) {
            store_tile(cur ^ 1);
            if (t0 + 2 * KT <= wg_last) fetch_tile(t0 + 2 * KT);
        }
        __syncthreads();
    }
    l_run = groups_sum(l_run);
    {
        // the upper-key waves hand (maximum, weight sum, weighted values) to their partners through the K buffers
        constexpr int NS = 18;
        static_assert(sizeof(kbuf) >= sizeof(float) * NS * 64 * 4 * HALVES, "K buffers hold the partner states");
        float* xch = reinterpret_cast<float*>(&kbuf[0][0][0][0]) + (size_t)(half * 4u + wave) * NS * 64u + lane;
        if (ksp == 1) {
            xch[0] = m_run, xch[64] = l_run;
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int r = 0; r < 4; r++) xch[(2 + 4 * c + r) * 64] = o[c][r];
        }
        __syncthreads();
        if (ksp == 1) return;
        const float m_b = xch[0], l_b = xch[64];
        const float m_all = fmaxf(m_run, m_b);
        const float fa = exp_nonpos_hw(m_run - m_all), fb = exp_nonpos_hw(m_b - m_all);
        l_run = l_run * fa + l_b * fb;
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int r = 0; r < 4; r++) o[c][r] = (o[c][r] * fa + xch[(2 + 4 * c + r) * 64] * fb) * (1.0f / kPScale);
    }
    // register r of tile c holds dim 16 c + 4 g + r of query l16
    if (q_out) {
        float v[4][4];
        float amax[2] = {0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                v[c][r] = __fdiv_rn(o[c][r], l_run);
                amax[c >> 1] = fmaxf(amax[c >> 1], fabsf(v[c][r]));
            }
#pragma unroll
        for (int b = 0; b < 2; b++) {
            amax[b] = groups_max(amax[b]);
        }
        if (active && jq < n) {
            const size_t row = (size_t)jq * a.n_heads * HD + (size_t)h * HD;
#pragma unroll
            for (int b = 0; b < 2; b++) {
                float id;
                const float scale = q8_scale_and_inverse(amax[b], id);
#pragma unroll
                for (int cc = 0; cc < 2; cc++) {
                    const int c = 2 * b + cc;
                    *reinterpret_cast<uint32_t*>(q_out + row + 16 * c + 4 * g) = q8_pack4(v[c][0], v[c][1], v[c][2], v[c][3], id);
                }
                if (g == 0) s_out[(row >> 5) + b] = scale;
            }
        }
        return;
    }
    if (active && jq < n) {
        float* dst = a.out + (size_t)jq * out_stride + (size_t)h * HD;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float4 v;
            v.x = __fdiv_rn(o[c][0], l_run), v.y = __fdiv_rn(o[c][1], l_run), v.z = __fdiv_rn(o[c][2], l_run), v.w = __fdiv_rn(o[c][3], l_run);
            *reinterpret_cast<float4*>(dst + 16 * c + 4 * g) = v;
        }
    }
}

// ---- gated short convolution, one step ---------------------------------------------------
// forward_conv_block's middle (wick/src/model/lfm2.rs:694-726): proj = [b | c | x]; bx = b*x;
// out = c * (sum_k buffer[k][ch]*w[ch][k] + bx*w[ch][K-1]); the rolling buffer shifts by one slot and takes bx.
// One thread per channel, the reference's operation order: bit-exact.
__global__ __launch_bounds__(256) void shortconv_step_kernel(const float* __restrict__ proj, float* __restrict__ buffer,
                                                             const float* __restrict__ conv_w, float* __restrict__ out, uint32_t hidden,
                                                             uint32_t kernel_size) {
    const uint32_t ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= hidden) return;
    const uint32_t d_conv = kernel_size - 1;
    const float bx = __fmul_rn(proj[ch], proj[2 * hidden + ch]);
    const float* w = conv_w + (size_t)ch * kernel_size;
    float sum = 0.0f;
    for (uint32_t k = 0; k < d_conv; k++) {
        const float tap = buffer[(size_t)k * hidden + ch];
        sum = __fadd_rn(sum, __fmul_rn(tap, w[k]));
        if (k > 0) buffer[(size_t)(k - 1) * hidden + ch] = tap;
    }
    sum = __fadd_rn(sum, __fmul_rn(bx, w[d_conv]));
    if (d_conv > 0) buffer[(size_t)(d_conv - 1) * hidden + ch] = bx;
    out[ch] = __fmul_rn(proj[hidden + ch], sum);
}

// The same step for the n tokens of a prompt (the sequential core of the reference's batched prefill,
// wick/src/model/lfm2.rs:1306-1350).  The convolution has no recurrence -- token j sees the gated inputs b*x of
// tokens j - (K-1) .. j, the ones before the prompt coming from the rolling state -- so every (token, channel) is
// computed on its own, taps summed oldest first exactly like shortconv_step_kernel: bit-exact.  The state is brought
// up to date by a second small kernel once every token has read the old one.
// proj [n][3 * hidden], out [n][hidden]; blockIdx.y = token.
__global__ __launch_bounds__(256) void shortconv_seq_kernel(const float* __restrict__ proj, const float* __restrict__ buffer,
                                                            const float* __restrict__ conv_w, float* __restrict__ out, uint32_t hidden,
                                                            uint32_t kernel_size) {
    const uint32_t ch = blockIdx.x * blockDim.x + threadIdx.x, j = blockIdx.y;
    if (ch >= hidden) return;
    const uint32_t d_conv = kernel_size - 1;
    const float* w = conv_w + (size_t)ch * kernel_size;
    float sum = 0.0f;
    for (uint32_t k = 0; k < d_conv; k++) {
        const int t = (int)j - (int)d_conv + (int)k;  // token of this tap, < 0: before the prompt
        float tap;
        if (t < 0) {
            tap = buffer[(size_t)(t + (int)d_conv) * hidden + ch];
        } else {
            const float* p = proj + (size_t)t * 3 * hidden;
            tap = __fmul_rn(p[ch], p[2 * hidden + ch]);
        }
        sum = __fadd_rn(sum, __fmul_rn(tap, w[k]));
    }
    const float* p = proj + (size_t)j * 3 * hidden;
    sum = __fadd_rn(sum, __fmul_rn(__fmul_rn(p[ch], p[2 * hidden + ch]), w[d_conv]));
    out[(size_t)j * hidden + ch] = __fmul_rn(p[hidden + ch], sum);
}

// shortconv_seq_kernel followed by the Q8_0 quantizer, bit for bit: a thread takes four consecutive channels of one
// token (16-byte loads), eight threads one 32-channel block, and the gated convolution goes straight into Q8_0 blocks
// for the out projection -- the f32 result never touches memory.  hidden % 32 == 0, 16-byte aligned buffers.
// KS: the kernel size when known at compile time (3, the reference's default: the taps unroll and all of a thread's loads are
// issued together), 0: read from kernel_size.
template <int KS>
__global__ __launch_bounds__(256) void shortconv_seq_quantize_kernel(const float* __restrict__ proj, const float* __restrict__ buffer,
                                                                     const float* __restrict__ conv_w, int8_t* __restrict__ q,
                                                                     float* __restrict__ scales, uint32_t hidden, uint32_t kernel_size_arg,
                                                                     uint64_t total_quads) {
    const uint32_t kernel_size = KS ? (uint32_t)KS : kernel_size_arg;
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = t < total_quads;
    const uint64_t tt = live ? t : 0;
    const uint32_t qpr = hidden >> 2;
    const uint32_t j = (uint32_t)(tt / qpr), c0 = 4u * (uint32_t)(tt % qpr);
    const uint32_t d_conv = kernel_size - 1;
    const float* w = conv_w + (size_t)c0 * kernel_size;
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t k = 0; k < d_conv; k++) {
        const int src = (int)j - (int)d_conv + (int)k;  // token of this tap, < 0: before the prompt
        // Both candidates are loaded (clamped addresses) and one is selected: no branch between the loads, so the taps' loads
        // and the token's own go out together.
        const float4 s4 = *reinterpret_cast<const float4*>(buffer + (size_t)(src < 0 ? src + (int)d_conv : 0) * hidden + c0);
        const float* p = proj + (size_t)(src < 0 ? 0 : src) * 3 * hidden;
        const float4 b = *reinterpret_cast<const float4*>(p + c0), x = *reinterpret_cast<const float4*>(p + 2 * hidden + c0);
        float tap[4] = {__fmul_rn(b.x, x.x), __fmul_rn(b.y, x.y), __fmul_rn(b.z, x.z), __fmul_rn(b.w, x.w)};
        if (src < 0) tap[0] = s4.x, tap[1] = s4.y, tap[2] = s4.z, tap[3] = s4.w;
#pragma unroll
        for (int i = 0; i < 4; i++) sum[i] = __fadd_rn(sum[i], __fmul_rn(tap[i], w[(size_t)i * kernel_size + k]));
    }
    const float* p = proj + (size_t)j * 3 * hidden;
    const float4 b = *reinterpret_cast<const float4*>(p + c0), c = *reinterpret_cast<const float4*>(p + hidden + c0),
                 x = *reinterpret_cast<const float4*>(p + 2 * hidden + c0);
    const float bx[4] = {__fmul_rn(b.x, x.x), __fmul_rn(b.y, x.y), __fmul_rn(b.z, x.z), __fmul_rn(b.w, x.w)};
    const float cc[4] = {c.x, c.y, c.z, c.w};
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = __fmul_rn(cc[i], __fadd_rn(sum[i], __fmul_rn(bx[i], w[(size_t)i * kernel_size + d_conv])));
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = group_max8(amax);
    float id;
    const float scale = q8_scale_and_inverse(amax, id);
    const uint32_t packed = q8_pack4(v[0], v[1], v[2], v[3], id);
    if (live) {
        reinterpret_cast<uint32_t*>(q)[tt] = packed;
        if ((tt & 7u) == 0) scales[tt >> 3] = scale;
    }
}

// New rolling state after n prompt tokens: slot s holds b*x of token n - (K-1) + s (an old slot when that is negative).
__global__ __launch_bounds__(256) void shortconv_state_kernel(const float* __restrict__ proj, float* __restrict__ buffer, uint32_t hidden,
                                                              uint32_t kernel_size, uint32_t n) {
    const uint32_t ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= hidden) return;
    const int d_conv = (int)kernel_size - 1;
    for (int s = 0; s < d_conv; s++) {  // ascending: slot s only ever takes a value from a slot above it
        const int t = (int)n - d_conv + s;
        float v;
        if (t < 0) {
            v = buffer[(size_t)(t + d_conv) * hidden + ch];
        } else {
            const float* p = proj + (size_t)t * 3 * hidden;
            v = __fmul_rn(p[ch], p[2 * hidden + ch]);
        }
        buffer[(size_t)s * hidden + ch] = v;
    }
}

// ---- SiLU gate ------------------------------------------------------------------------
// silu_mul_inplace (wick/src/backend/cpu.rs:668-673): g / (1 + expf(-g)) * u, bit-exact.
__global__ __launch_bounds__(256) void silu_mul_kernel(float* __restrict__ gate, const float* __restrict__ up, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i];
    gate[i] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, ggml_expf(-g))), up[i]);
}

// ---- normalise / gate and quantize in one pass (prompt passes) -----------------------------------
// What rmsnorm_kernel followed by the Q8_0 quantizer compute (wick/src/backend/cpu.rs:577-594, wick/src/backend/simd.rs:255-323),
// bit for bit, without the f32 round trip through memory: the sum of squares is taken over the same elements per thread
// and in the same order as rmsnorm_kernel does, the normalised values are formed by the same two products, and eight
// lanes own one 32-element block exactly as in the quantizer.  One block per row; dim % 32 == 0, rows 16-byte aligned.
__global__ __launch_bounds__(256) void rmsnorm_quantize_kernel(const float* __restrict__ x, const float* __restrict__ weight, int8_t* __restrict__ q,
                                                               float* __restrict__ scales, uint32_t dim, uint32_t x_stride, float eps) {
    __shared__ double slots[16];
    const float* xr = x + (size_t)blockIdx.x * x_stride;
    double s = 0.0;
    for (uint32_t i0 = threadIdx.x; i0 < dim; i0 += 4u * 256u) {  // four loads in flight; elements t, t + 256, .. in order, as rmsnorm_kernel sums them
        float xv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) xv[j] = xr[i0 + 256u * j < dim ? i0 + 256u * j : i0];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (i0 + 256u * j < dim) {
                const double v = (double)xv[j];
                s += v * v;
            }
        }
    }
    const double total = block_sum_f64(s, slots);
    const float inv_rms = (float)(1.0 / sqrt(total / (double)dim + (double)eps));
    const uint32_t quads = dim >> 2;
    for (uint32_t quad0 = 0; quad0 < quads; quad0 += blockDim.x) {  // groups of 8 lanes stay together: quads % 8 == 0
        const uint32_t quad = quad0 + threadIdx.x;
        const bool live = quad < quads;
        const uint32_t qd = live ? quad : 0;
        const float4 v = reinterpret_cast<const float4*>(xr)[qd];
        const float4 w = reinterpret_cast<const float4*>(weight)[qd];
        const float v0 = __fmul_rn(__fmul_rn(v.x, inv_rms), w.x), v1 = __fmul_rn(__fmul_rn(v.y, inv_rms), w.y);
        const float v2 = __fmul_rn(__fmul_rn(v.z, inv_rms), w.z), v3 = __fmul_rn(__fmul_rn(v.w, inv_rms), w.w);
        float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
        amax = group_max8(amax);
        float id;
        const float scale = q8_scale_and_inverse(amax, id);
        const uint32_t packed = q8_pack4(v0, v1, v2, v3, id);
        if (live) {
            *reinterpret_cast<uint32_t*>(q + (size_t)blockIdx.x * dim + 4u * quad) = packed;
            if ((quad & 7u) == 0) scales[(size_t)blockIdx.x * (dim >> 5) + (quad >> 3)] = scale;
        }
    }
}

// The K shares of a split projection added onto the residual rows, then rmsnorm_quantize_kernel of the updated rows, bit for bit
// what gemm_splitk_reduce_kernel (accumulating) followed by rmsnorm_quantize_kernel leave: the shares are summed in ascending
// order and then added to x; thread t covers the same elements t, t + 256, .. in the same order for the f64 sum of squares.  The
// updated row is written back and kept in LDS for the quantizer's pass.  partial: [splits][rows][dim].
template <int S>
__global__ __launch_bounds__(256) void residual_rmsnorm_quantize_kernel(float* __restrict__ x, const float* __restrict__ partial, size_t share_stride,
                                                                        const float* __restrict__ weight, int8_t* __restrict__ q,
                                                                        float* __restrict__ scales, uint32_t dim, uint32_t x_stride, float eps) {
    __shared__ double slots[16];
    __shared__ __align__(16) float row[kResidualNormMaxDim];
    float* xr = x + (size_t)blockIdx.x * x_stride;
    const float* pr = partial + (size_t)blockIdx.x * dim;
    double s = 0.0;
    for (uint32_t i0 = threadIdx.x; i0 < dim; i0 += 4u * 256u) {  // four elements' loads (S + 1 each) in flight together
        float xv[4], pv[4][S];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t i = i0 + 256u * j < dim ? i0 + 256u * j : i0;
            xv[j] = xr[i];
#pragma unroll
            for (int p = 0; p < S; p++) pv[j][p] = pr[(size_t)p * share_stride + i];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t i = i0 + 256u * j;
            if (i < dim) {
                float sum = pv[j][0];
#pragma unroll
                for (int p = 1; p < S; p++) sum += pv[j][p];
                const float h = xv[j] + sum;
                xr[i] = h, row[i] = h;
                const double v = (double)h;
                s += v * v;
            }
        }
    }
    const double total = block_sum_f64(s, slots);  // its barriers also publish row[]
    const float inv_rms = (float)(1.0 / sqrt(total / (double)dim + (double)eps));
    const uint32_t quads = dim >> 2;
    for (uint32_t quad0 = 0; quad0 < quads; quad0 += blockDim.x) {
        const uint32_t quad = quad0 + threadIdx.x;
        const bool live = quad < quads;
        const uint32_t qd = live ? quad : 0;
        const float4 v = reinterpret_cast<const float4*>(row)[qd];
        const float4 w = reinterpret_cast<const float4*>(weight)[qd];
        const float v0 = __fmul_rn(__fmul_rn(v.x, inv_rms), w.x), v1 = __fmul_rn(__fmul_rn(v.y, inv_rms), w.y);
        const float v2 = __fmul_rn(__fmul_rn(v.z, inv_rms), w.z), v3 = __fmul_rn(__fmul_rn(v.w, inv_rms), w.w);
        float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
        amax = group_max8(amax);
        float id;
        const float scale = q8_scale_and_inverse(amax, id);
        const uint32_t packed = q8_pack4(v0, v1, v2, v3, id);
        if (live) {
            *reinterpret_cast<uint32_t*>(q + (size_t)blockIdx.x * dim + 4u * quad) = packed;
            if ((quad & 7u) == 0) scales[(size_t)blockIdx.x * (dim >> 5) + (quad >> 3)] = scale;
        }
    }
}

// silu_mul_kernel followed by the quantizer, bit for bit: the gated values go straight into Q8_0 blocks.
// gate / up: [n][dim] floats, contiguous, 16-byte aligned.
__global__ __launch_bounds__(256) void silu_mul_quantize_kernel(const float* __restrict__ gate, const float* __restrict__ up, int8_t* __restrict__ q,
                                                                float* __restrict__ scales, uint64_t total_quads) {
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = t < total_quads;
    const uint64_t tt = live ? t : 0;
    const float4 g = reinterpret_cast<const float4*>(gate)[tt];
    const float4 u = reinterpret_cast<const float4*>(up)[tt];
    const float v0 = silu_mul(g.x, u.x), v1 = silu_mul(g.y, u.y), v2 = silu_mul(g.z, u.z), v3 = silu_mul(g.w, u.w);
    float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
    amax = group_max8(amax);
    float id;
    const float scale = q8_scale_and_inverse(amax, id);
    const uint32_t packed = q8_pack4(v0, v1, v2, v3, id);
    if (live) {
        reinterpret_cast<uint32_t*>(q)[tt] = packed;
        if ((tt & 7u) == 0) scales[tt >> 3] = scale;
    }
}

// ---- greedy pick ----------------------------------------------------------------------
// cpu_argmax (wick/src/sampler.rs:7-19): NaN counts as -inf, values order by f32::total_cmp, the LAST of
// equal maxima wins; bit-exact.  Two small launches (64 blocks, then one wave over their partial keys): a single
// block would spend 20 us walking a 65536-entry vocabulary.  Optionally publishes the pick as the next step's
// token and advances the device-side position.

constexpr uint32_t kArgmaxBlocks = 64;

// Stage 1: every block leaves the best key of its slice (float4 loads, all of a thread's loads in flight at once).
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ x, uint32_t n, unsigned long long* __restrict__ partial) {
    __shared__ unsigned long long red[4];
    unsigned long long best = 0ull;  // below every real key
    const uint32_t quads = n >> 2, stride = gridDim.x * 256u;
    for (uint32_t q0 = blockIdx.x * 256u + threadIdx.x; q0 < quads; q0 += 4u * stride) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t q = q0 + j * stride;
            v[j] = reinterpret_cast<const float4*>(x)[q < quads ? q : q0];  // clamped: a repeated quad cannot change the maximum
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t q = q0 + j * stride;
            const uint32_t i = 4u * (q < quads ? q : q0);
            const unsigned long long k0 = argmax_key(v[j].x, i), k1 = argmax_key(v[j].y, i + 1), k2 = argmax_key(v[j].z, i + 2),
                                     k3 = argmax_key(v[j].w, i + 3);
            const unsigned long long a = k0 > k1 ? k0 : k1, b = k2 > k3 ? k2 : k3, c = a > b ? a : b;
            best = c > best ? c : best;
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {  // the last n % 4 elements
        const uint32_t i = (n & ~3u) + threadIdx.x;
        const unsigned long long k = argmax_key(x[i], i);
        best = k > best ? k : best;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(best, off, 64);
        best = o > best ? o : best;
    }
    if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned long long a = red[0] > red[1] ? red[0] : red[1], b = red[2] > red[3] ? red[2] : red[3];
        partial[blockIdx.x] = a > b ? a : b;
    }
}

// Stage 2: one workgroup (one wave when there are at most 64 keys and nothing to look up) merges the partial keys and
// publishes the pick.
// An embedding to look the next step's input up in (w null: none): row `token` of w as k floats into `out`.
struct EmbedArgs {
    const uint8_t* w;
    float* out;
    int type;
    uint32_t m, k;
};

// Row `row` of the embedding into emb.out by the calling workgroup, four elements per thread at a time: their loads are all issued
// before the first store (the stores could alias the loads as far as the compiler knows, which would chain the round trips).
__device__ __forceinline__ void embed_row_batched(const EmbedArgs& emb, uint32_t row) {
    for (uint32_t e0 = threadIdx.x; e0 < emb.k; e0 += 4u * blockDim.x) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t e = e0 + j * blockDim.x;
            v[j] = dequant_element(emb.w, emb.type, row, emb.k, e < emb.k ? e : e0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t e = e0 + j * blockDim.x;
            if (e < emb.k) emb.out[e] = v[j];
        }
    }
}

__global__ __launch_bounds__(256) void argmax_final_kernel(const unsigned long long* __restrict__ partial, uint32_t blocks, uint32_t n,
                                                           uint32_t* __restrict__ out, uint32_t* __restrict__ d_token, uint32_t* __restrict__ d_pos,
                                                           uint32_t* __restrict__ d_history, uint32_t history_len, EmbedArgs emb) {
    __shared__ uint32_t picked;
    __shared__ unsigned long long red[4];
    const uint32_t waves = blockDim.x >> 6;  // 1 (at most 64 partial keys) or 4
    unsigned long long best = 0ull;
    for (uint32_t i0 = threadIdx.x; i0 < blocks; i0 += 8u * blockDim.x) {  // eight keys per thread in flight (one round trip for <= 2048 keys)
        unsigned long long k[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t i = i0 + j * blockDim.x;
            k[j] = partial[i < blocks ? i : i0];  // clamped: a repeated key cannot change the maximum
        }
#pragma unroll
        for (int j = 0; j < 8; j++) best = k[j] > best ? k[j] : best;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(best, off, 64);
        best = o > best ? o : best;
    }
    if (waves > 1) {
        if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = best;
        __syncthreads();
        if (threadIdx.x == 0) {
            const unsigned long long a = red[0] > red[1] ? red[0] : red[1], b = red[2] > red[3] ? red[2] : red[3];
            best = a > b ? a : b;
        }
    }
    if (threadIdx.x == 0) {
        const uint32_t pick = n ? (uint32_t)(best & 0xffffffffull) : 0u;
        picked = pick;
        out[0] = pick;
        if (d_token) *d_token = pick;
        if (d_pos) {
            const uint32_t pos = *d_pos;
            if (d_history && pos < history_len) d_history[pos] = pick;  // the pick made after the token at `pos`
            *d_pos = pos + 1u;
        }
    }
    if (!emb.w) return;
    __syncthreads();
    const uint32_t pick = picked;  // the pick is the next step's token: its embedding row is that step's input
    if (pick < emb.m) embed_row_batched(emb, pick);
}

// Sets the device-side token / position of the next step (either may be null) and, when an embedding is given, looks
// the token's row up as that step's input.
__global__ __launch_bounds__(256) void set_step_kernel(uint32_t* d_token, uint32_t token, uint32_t* d_pos, uint32_t pos, EmbedArgs emb) {
    if (threadIdx.x == 0) {
        if (d_token) *d_token = token;
        if (d_pos) *d_pos = pos;
    }
    if (emb.w && token < emb.m) embed_row_batched(emb, token);
}

__global__ void advance_pos_kernel(uint32_t* d_pos) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *d_pos = *d_pos + 1u;
}

}  // namespace

hipError_t launch_embed_row(const uint8_t* d_w, int type, uint32_t m, uint32_t k, uint32_t token, const uint32_t* d_token, float* d_out,
                            const Launch& L) {
    const uint32_t blocks = (k + 255u) / 256u;
    return launch_kernel(L, kFamOther, embed_row_kernel, dim3(blocks < 64u ? blocks : 64u), dim3(256), d_w, type, m, k, token, d_token, d_out);
}

hipError_t launch_rmsnorm(const float* d_x, const float* d_weight, float* d_y, uint32_t rows, uint32_t dim, uint32_t x_stride,
                          uint32_t y_stride, float eps, const Launch& L) {
    if (rows == 0) return hipSuccess;
    return launch_kernel(L, kFamOther, rmsnorm_kernel, dim3(rows), dim3(256), d_x, d_weight, d_y, dim, x_stride, y_stride, eps);
}

hipError_t launch_qk_norm_rope(float* d_q, float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm, void* d_k_cache,
                               void* d_v_cache, uint32_t pos, const uint32_t* d_pos, uint32_t max_seq, uint32_t head_dim, uint32_t n_heads,
                               uint32_t n_kv_heads, float eps, float theta_scale, const Launch& L, uint32_t n_tokens, uint32_t q_stride,
                               uint32_t kv_stride, bool kv_f16) {
    if (n_tokens == 0) return hipSuccess;
    QkNormRopeArgs a{d_q, d_k, d_v, d_q_norm, d_k_norm, d_k_cache, d_v_cache, d_pos, pos, max_seq, head_dim, n_heads, n_kv_heads, eps, theta_scale,
                     q_stride, kv_stride};
    return with_kv_type(kv_f16, [&](auto kv) {
        using KV = decltype(kv);
        if (n_tokens > 1 && head_dim == 64) return launch_kernel(L, kFamOther, qk_norm_rope_tokens64_kernel<KV>, dim3(n_tokens), dim3(256), a);
        if (n_tokens > 1 && head_dim / 2 <= kRopeTableMax) return launch_kernel(L, kFamOther, qk_norm_rope_tokens_kernel<KV>, dim3(n_tokens), dim3(256), a);
        return launch_kernel(L, kFamOther, qk_norm_rope_kernel<KV>, dim3(n_heads + n_kv_heads, n_tokens), dim3(64), a);
    });
}

hipError_t launch_kv_shift(void* d_k_cache, void* d_v_cache, void* d_stage, uint32_t seq_len, uint32_t n_keep, uint32_t shift,
                           uint32_t n_kv_heads, uint32_t head_dim, float theta_scale, const Launch& L, bool kv_f16) {
    const uint32_t retained = seq_len - n_keep - shift;
    if (retained == 0) return hipSuccess;  // everything behind n_keep is dropped: nothing moves
    const size_t kv_dim = (size_t)n_kv_heads * head_dim, elems = (size_t)retained * kv_dim, esize = kv_f16 ? 2 : 4;
    uint8_t* const stage = static_cast<uint8_t*>(d_stage);
    KvShiftArgs a{d_k_cache, d_v_cache, stage, stage + elems * esize, n_keep, shift, retained, n_kv_heads, head_dim, theta_scale};
    hipError_t e = with_kv_type(kv_f16, [&](auto kv) {
        return launch_kernel(L, kFamOther, kv_shift_stage_kernel<decltype(kv)>, dim3((retained + kShiftRows - 1) / kShiftRows), dim3(256), a);
    });
    if (e != hipSuccess) return e;
    e = hipMemcpyAsync(static_cast<uint8_t*>(d_k_cache) + (size_t)n_keep * kv_dim * esize, a.k_stage, elems * esize, hipMemcpyDeviceToDevice, L.stream);
    if (e != hipSuccess) return e;
    return hipMemcpyAsync(static_cast<uint8_t*>(d_v_cache) + (size_t)n_keep * kv_dim * esize, a.v_stage, elems * esize, hipMemcpyDeviceToDevice, L.stream);
}

hipError_t launch_attention_decode(const float* d_q, const void* d_k_cache, const void* d_v_cache, float* d_out, float* d_scores,
                                   uint32_t seq_len, const uint32_t* d_pos, uint32_t max_seq, uint32_t n_heads, uint32_t n_kv_heads,
                                   uint32_t head_dim, float scale, const Launch& L, bool kv_f16) {
    AttentionArgs a{d_q, d_k_cache, d_v_cache, d_out, d_scores, d_pos, seq_len, max_seq, n_heads, n_kv_heads, head_dim, scale};
    const uint32_t splits = attention_splits(max_seq);
    auto split_path = [&](auto hd) -> hipError_t {
        constexpr int HD = decltype(hd)::value;
        hipError_t e = with_kv_type(kv_f16, [&](auto kv) {
            return launch_kernel(L, kFamOther, attention_split_kernel<HD, decltype(kv)>, dim3(n_heads * splits), dim3(256), a, splits);
        });
        if (e != hipSuccess) return e;
        return launch_kernel(L, kFamOther, attention_combine_kernel<HD>, dim3(n_heads), dim3(256), a, splits);
    };
    // a short context gains nothing from the second launch
    if (max_seq > 256u) {
        switch (head_dim) {
            case 32: return split_path(std::integral_constant<int, 32>{});
            case 64: return split_path(std::integral_constant<int, 64>{});
            case 128: return split_path(std::integral_constant<int, 128>{});
            case 256: return split_path(std::integral_constant<int, 256>{});
            default: break;
        }
    }
    return with_kv_type(kv_f16, [&](auto kv) { return launch_kernel(L, kFamOther, attention_decode_kernel<decltype(kv)>, dim3(n_heads), dim3(256), a); });
}

// The fused attention block; false when head_dim has no fused variant (the caller then runs the three launches).
bool attention_layer_applies(uint32_t head_dim) { return head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256; }

hipError_t launch_attention_layer(const float* d_q, const float* d_k, const float* d_v, const float* d_q_norm, const float* d_k_norm,
                                  void* d_k_cache, void* d_v_cache, float* d_out, float* d_scratch, uint32_t pos,
                                  const uint32_t* d_pos, uint32_t max_seq, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, float eps,
                                  float theta_scale, float scale, const Launch& L, bool kv_f16) {
    AttentionLayerArgs f{};
    f.at = AttentionArgs{nullptr, d_k_cache, d_v_cache, d_out, d_scratch, d_pos, pos + 1u, max_seq, n_heads, n_kv_heads, head_dim, scale};
    f.q_raw = d_q, f.k_raw = d_k, f.v = d_v, f.q_norm = d_q_norm, f.k_norm = d_k_norm;
    f.k_cache = d_k_cache, f.v_cache = d_v_cache, f.eps = eps, f.theta_scale = theta_scale;
    const uint32_t splits = attention_splits(max_seq);
    const dim3 grid(n_heads * splits), block(256);
    auto run = [&](auto hd) -> hipError_t {
        constexpr int HD = decltype(hd)::value;
        hipError_t e = with_kv_type(kv_f16, [&](auto kv) { return launch_kernel(L, kFamOther, attention_layer_kernel<HD, decltype(kv)>, grid, block, f, splits); });
        if (e != hipSuccess) return e;
        return launch_kernel(L, kFamOther, attention_combine_kernel<HD>, dim3(n_heads), block, f.at, splits);
    };
    switch (head_dim) {
        case 32: return run(std::integral_constant<int, 32>{});
        case 64: return run(std::integral_constant<int, 64>{});
        case 128: return run(std::integral_constant<int, 128>{});
        case 256: return run(std::integral_constant<int, 256>{});
        default: return hipErrorInvalidValue;
    }
}

uint32_t attention_splits(uint32_t max_seq) {
    const uint32_t chunks = (max_seq + kAttnChunk - 1) / kAttnChunk;
    return chunks < 1u ? 1u : (chunks < kAttnMaxSplits ? chunks : kAttnMaxSplits);
}

size_t attention_scratch_floats(uint32_t max_seq, uint32_t n_heads, uint32_t head_dim) {
    const size_t single = (size_t)n_heads * max_seq;                                        // scores of the one-workgroup kernel
    const size_t split = (size_t)n_heads * attention_splits(max_seq) * (head_dim + 2);      // {max, sum, acc[head_dim]} per partial
    return single > split ? single : split;
}

hipError_t launch_shortconv_step(const float* d_proj, float* d_buffer, const float* d_conv_w, float* d_out, uint32_t hidden,
                                 uint32_t kernel_size, const Launch& L) {
    return launch_kernel(L, kFamOther, shortconv_step_kernel, dim3((hidden + 255u) / 256u), dim3(256), d_proj, d_buffer, d_conv_w, d_out, hidden,
                         kernel_size);
}

hipError_t launch_embed_rows(const uint8_t* d_w, int type, uint32_t m, uint32_t k, const uint32_t* d_tokens, uint32_t n, float* d_out,
                             const Launch& L) {
    if (n == 0) return hipSuccess;
    const uint32_t blocks = (k + 255u) / 256u;
    return launch_kernel(L, kFamOther, embed_rows_kernel, dim3(blocks < 16u ? blocks : 16u, n), dim3(256), d_w, type, m, k, d_tokens, d_out);
}

hipError_t launch_shortconv_seq(const float* d_proj, float* d_buffer, const float* d_conv_w, float* d_out, uint32_t hidden,
                                uint32_t kernel_size, uint32_t n, const Launch& L) {
    if (n == 0) return hipSuccess;
    const uint32_t blocks = (hidden + 255u) / 256u;
    hipError_t e = launch_kernel(L, kFamOther, shortconv_seq_kernel, dim3(blocks, n), dim3(256), d_proj, static_cast<const float*>(d_buffer), d_conv_w,
                                 d_out, hidden, kernel_size);
    if (e != hipSuccess || kernel_size < 2) return e;
    return launch_kernel(L, kFamOther, shortconv_state_kernel, dim3(blocks), dim3(256), d_proj, d_buffer, hidden, kernel_size, n);
}

bool shortconv_seq_quantize_applies(const float* d_proj, const float* d_buffer, uint32_t hidden) {
    return hidden % 32u == 0 && ((uintptr_t)d_proj | (uintptr_t)d_buffer) % 16u == 0;
}

// The convolution of n tokens written as Q8_0 blocks ([n][hidden] quants, [n][hidden / 32] scales), then the state.
hipError_t launch_shortconv_seq_quantize(const float* d_proj, float* d_buffer, const float* d_conv_w, int8_t* d_q, float* d_scales, uint32_t hidden,
                                         uint32_t kernel_size, uint32_t n, const Launch& L) {
    if (n == 0) return hipSuccess;
    if (!shortconv_seq_quantize_applies(d_proj, d_buffer, hidden)) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)n * (hidden >> 2);
    const auto go = [&](auto kernel) {
        return launch_kernel(L, kFamQuantize, kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), d_proj, static_cast<const float*>(d_buffer),
                             d_conv_w, d_q, d_scales, hidden, kernel_size, total);
    };
    hipError_t e = kernel_size == 3 ? go(shortconv_seq_quantize_kernel<3>) : go(shortconv_seq_quantize_kernel<0>);
    if (e != hipSuccess || kernel_size < 2) return e;
    return launch_kernel(L, kFamOther, shortconv_state_kernel, dim3((hidden + 255u) / 256u), dim3(256), d_proj, d_buffer, hidden, kernel_size, n);
}

size_t attention_prefill_scratch_floats(uint32_t, uint32_t, uint32_t) { return 4; }  // the kernel keeps everything on chip

bool attention_prefill_quantize_applies(const float* d_q, const void* d_k_cache, const void* d_v_cache, uint32_t n, uint32_t q_stride,
                                        uint32_t head_dim) {
    return head_dim == 64 && n >= 16 && q_stride % 4u == 0 && ((uintptr_t)d_q | (uintptr_t)d_k_cache | (uintptr_t)d_v_cache) % 16u == 0;
}

// d_q8 / d_q8_scales given (attention_prefill_quantize_applies): the result is written as Q8_0 blocks, rows of
// n_heads * head_dim quants, bit-identical to quantizing the float result; d_out is not written then.
hipError_t launch_attention_prefill(const float* d_q, const void* d_k_cache, const void* d_v_cache, float* d_out, float* d_scratch,
                                    uint32_t pos0, const uint32_t* d_pos, uint32_t n, uint32_t q_stride, uint32_t out_stride, uint32_t max_seq,
                                    uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, float scale, const Launch& L, int8_t* d_q8,
                                    float* d_q8_scales, bool kv_f16) {
    if (n == 0) return hipSuccess;
    AttentionArgs a{d_q, d_k_cache, d_v_cache, d_out, d_scratch, d_pos, 0u, max_seq, n_heads, n_kv_heads, head_dim, scale};
    // the matrix-core kernel needs 16-byte aligned rows (q, caches, out) and whole tiles of head dims
    const bool aligned = q_stride % 4u == 0 && ((uintptr_t)d_q | (uintptr_t)d_k_cache | (uintptr_t)d_v_cache) % 16u == 0 &&
                         (d_q8 || (out_stride % 4u == 0 && (uintptr_t)d_out % 16u == 0));
    if (d_q8 && !(aligned && attention_prefill_quantize_applies(d_q, d_k_cache, d_v_cache, n, q_stride, head_dim))) return hipErrorInvalidValue;
    if (head_dim == 64 && aligned && n >= 16) {
        const uint32_t qblocks = (n + 63u) / 64u;
        // (long, short) pairs balance the causal work once there are more query blocks than CUs; below that one block per
        // workgroup (longest first) spreads wider: 17.7 -> 14.9, 25.8 -> 23.5, 43.5 -> 41.7 us at 256 / 512 / 1024 tokens of 16
        // heads, but 82 -> 94 us at 2002.  The same arithmetic per query either way.
        return with_kv_type(kv_f16, [&](auto kv) {
            using KV = decltype(kv);
            if (n_heads * qblocks <= 256u)
                return launch_kernel(L, kFamOther, attention_prefill_f16x3_kernel<1, KV>, dim3(n_heads, qblocks), dim3(512), a, pos0, n, q_stride, out_stride,
                                     d_q8, d_q8_scales);
            return launch_kernel(L, kFamOther, attention_prefill_f16x3_kernel<2, KV>, dim3(n_heads, (qblocks + 1u) / 2u), dim3(1024), a, pos0, n, q_stride,
                                 out_stride, d_q8, d_q8_scales);
        });
    }
    const dim3 grid(n_heads, (n + 7u) / 8u), block(256);
    return with_kv_type(kv_f16, [&](auto kv) {
        using KV = decltype(kv);
        switch (head_dim) {
            case 32: return launch_kernel(L, kFamOther, attention_prefill_kernel<32, KV>, grid, block, a, pos0, n, q_stride, out_stride);
            case 64: return launch_kernel(L, kFamOther, attention_prefill_kernel<64, KV>, grid, block, a, pos0, n, q_stride, out_stride);
            case 128: return launch_kernel(L, kFamOther, attention_prefill_kernel<128, KV>, grid, block, a, pos0, n, q_stride, out_stride);
            case 256: return launch_kernel(L, kFamOther, attention_prefill_kernel<256, KV>, grid, block, a, pos0, n, q_stride, out_stride);
            default: return hipErrorInvalidValue;
        }
    });
}

hipError_t launch_rmsnorm_quantize(const float* d_x, const float* d_weight, uint32_t rows, uint32_t dim, uint32_t x_stride, float eps, int8_t* d_q,
                                   float* d_scales, const Launch& L) {
    if (rows == 0) return hipSuccess;
    return launch_kernel(L, kFamQuantize, rmsnorm_quantize_kernel, dim3(rows), dim3(256), d_x, d_weight, d_q, d_scales, dim, x_stride, eps);
}

hipError_t launch_residual_rmsnorm_quantize(float* d_x, const float* d_partial, uint32_t splits, const float* d_weight, uint32_t rows, uint32_t dim,
                                            uint32_t x_stride, float eps, int8_t* d_q, float* d_scales, const Launch& L) {
    if (rows == 0) return hipSuccess;
    if (dim > kResidualNormMaxDim) return hipErrorInvalidValue;
    const auto go = [&](auto kernel) {
        return launch_kernel(L, kFamQuantize, kernel, dim3(rows), dim3(256), d_x, d_partial, (size_t)rows * dim, d_weight, d_q, d_scales, dim, x_stride, eps);
    };
    if (splits == 2) return go(residual_rmsnorm_quantize_kernel<2>);
    if (splits == 4) return go(residual_rmsnorm_quantize_kernel<4>);
    if (splits == 8) return go(residual_rmsnorm_quantize_kernel<8>);
    return hipErrorInvalidValue;  // the K split makes 2, 4 or 8 shares
}

hipError_t launch_silu_mul_quantize(const float* d_gate, const float* d_up, uint32_t n, uint32_t dim, int8_t* d_q, float* d_scales, const Launch& L) {
    const uint64_t total = (uint64_t)n * (dim >> 2);
    if (total == 0) return hipSuccess;
    return launch_kernel(L, kFamQuantize, silu_mul_quantize_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), d_gate, d_up, d_q, d_scales, total);
}

hipError_t launch_silu_mul(float* d_gate, const float* d_up, uint32_t n, const Launch& L) {
    if (n == 0) return hipSuccess;
    return launch_kernel(L, kFamOther, silu_mul_kernel, dim3((n + 255u) / 256u), dim3(256), d_gate, d_up, n);
}

hipError_t launch_argmax(const float* d_x, uint32_t n, unsigned long long* d_partial, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos,
                         uint32_t* d_history, uint32_t history_len, const Launch& L, const uint8_t* d_embd, int embd_type, uint32_t embd_m,
                         uint32_t embd_k, float* d_embd_out) {
    const uint32_t blocks = n >= 4096u ? kArgmaxBlocks : 1u;
    hipError_t e = launch_kernel(L, kFamOther, argmax_partial_kernel, dim3(blocks), dim3(256), d_x, n, d_partial);
    if (e != hipSuccess) return e;
    return launch_argmax_final(d_partial, blocks, n, d_out, d_token, d_pos, d_history, history_len, L, d_embd, embd_type, embd_m, embd_k, d_embd_out);
}

hipError_t launch_argmax_final(const unsigned long long* d_partial, uint32_t n_partials, uint32_t n, uint32_t* d_out, uint32_t* d_token, uint32_t* d_pos,
                               uint32_t* d_history, uint32_t history_len, const Launch& L, const uint8_t* d_embd, int embd_type, uint32_t embd_m,
                               uint32_t embd_k, float* d_embd_out) {
    const EmbedArgs emb{d_embd_out ? d_embd : nullptr, d_embd_out, embd_type, embd_m, embd_k};
    return launch_kernel(L, kFamOther, argmax_final_kernel, dim3(1), dim3(emb.w || n_partials > 64u ? 256 : 64), d_partial, n_partials, n, d_out, d_token,
                         d_pos, d_history, history_len, emb);
}

hipError_t launch_set_step(uint32_t* d_token, uint32_t token, uint32_t* d_pos, uint32_t pos, const Launch& L, const uint8_t* d_embd, int embd_type,
                           uint32_t embd_m, uint32_t embd_k, float* d_embd_out) {
    const EmbedArgs emb{d_embd_out ? d_embd : nullptr, d_embd_out, embd_type, embd_m, embd_k};
    return launch_kernel(L, kFamOther, set_step_kernel, dim3(1), dim3(256), d_token, token, d_pos, pos, emb);
}

hipError_t launch_advance_pos(uint32_t* d_pos, const Launch& L) {
    return launch_kernel(L, kFamOther, advance_pos_kernel, dim3(1), dim3(64), d_pos);
}

}  // namespace wick_rocm
