// Decode GEMV over raw GGUF Q6_K blocks against Q8_0-quantized activations, for gfx950.
// Shipped LFM2 Q4_0 files keep the tied embedding / LM head -- the largest GEMV of a decode
// step -- in Q6_K (wick/src/model/metal_lfm2.rs:175-180, 1345-1355).
//
// Arithmetic: gemv_q6k_q8_0_neon (wick/src/backend/simd.rs:552-679):
//   y[i] = sum over 16-weight groups g:  ((f32(f16 d) * f32(scales[g])) * xs[q8 block of g]) * f32(idot_g)
//   idot_g = sum_16 (q - 32) * xq, q the 6-bit quant, exact i32.
// The f32 summation order differs from NEON's (per-lane partial sums, then a tree over the
// lanes of a row); the contract is rel-L2 <= 1e-5, not bit equality.
//
// Block layout (wick/src/quant.rs:60-70): ql[128] low nibbles, qh[64] high 2-bit pairs,
// scales[16] int8, d f16 = 210 bytes for 256 weights; element e = 128 n + 32 j + l
// (n < 2, j < 4, l < 32): low nibble = ql[64 n + 32 (j & 1) + l] >> 4 (j >> 1),
// high bits = qh[32 n + l] >> 2 j, scale = scales[e / 16].
//
// Shape of the kernel (HBM-bound): a lane owns one HALF block (n fixed: 128 weights =
// 64 bytes of ql, 32 of qh, 8 scales) of every row it visits, so its 128 activation quants,
// their four scales and the eight 16-element sums live in registers.  A row is 2 k/256
// consecutive lanes (padded to a power of two), 64 lanes cover consecutive rows, and the
// rows of one pass are one contiguous span of the matrix: the wave fetches it as whole
// consecutive 16-byte pieces (nontemporal, every cache line exactly once), parks it in a
// wave-private LDS slot and each lane reads its runs back.  Blocks are only 2-byte aligned,
// so runs are read as aligned dwords and funnel-shifted by 0 or 2 bytes.
#include <type_traits>

#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

constexpr int kQ6kBlockBytes = 210;
constexpr int kHalfBytes = kQ6kBlockBytes / 2;  // a row is a whole number of half blocks (105 bytes each)
constexpr int kSlotBytes = 64 * kHalfBytes + 32;  // + up to 15 lead bytes, + the overhang of the last runs

struct Q6kArgs {
    const uint8_t* w;
    const int8_t* xq;   // [k]
    const float* xs;    // [k / 32]
    float* y;
    int32_t* dots;      // parity hook: [m][k / 16] group dots instead of y
    uint32_t m, k;
    uint32_t rows_per_wave;
    uint32_t y_row_stride;  // y[row * y_row_stride]
    int accumulate;
    // FUSED variant: the f32 activations and the RMSNorm weights in front of them (xq / xs unused)
    const float* xf;        // [k]
    const float* norm_w;    // [k]
    float eps;
    // when given, every wave also leaves the greedy-pick key of its best row here (partial[blockIdx.x])
    unsigned long long* partial;
};

// NDW dwords starting at byte `off` (even) of the LDS slot.
template <int NDW>
__device__ __forceinline__ void read_run(const uint8_t* slot, uint32_t off, uint32_t (&out)[NDW]) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(slot + (off & ~3u));
    const uint32_t sh = off & 3u;
    uint32_t t[NDW + 1];
#pragma unroll
    for (int i = 0; i <= NDW; i++) t[i] = p[i];
#pragma unroll
    for (int i = 0; i < NDW; i++) out[i] = __builtin_amdgcn_alignbyte(t[i + 1], t[i], sh);
}

// FUSED: the wave norms and quantizes the f32 activation vector itself (rmsnorm_quantize_kernel's arithmetic, bit for bit:
// its 256 threads are played by the wave's lanes four at a time, so that every f64 partial sum is taken over the same
// elements in the same order; eight lanes per 32-element block in the quantizer) into LDS, under the latency of its first
// weight span, and reads its half block's quants and scales back from there.  One launch less in front of the LM head;
// every wave redoes the vector (k floats from the L2), which costs less than that launch.
template <int LPR, bool DUMP, bool FUSED = false>
__global__ __launch_bounds__(64) void gemv_q6k_kernel(Q6kArgs a) {
    static_assert(!(DUMP && FUSED), "the parity hook runs on pre-quantized activations");
    constexpr int RPW = 64 / LPR;  // rows per pass
    constexpr int PIECES = (15 + RPW * LPR * kHalfBytes + 15) / 16;  // upper bound of 16-byte pieces per span
    constexpr int PPL = (PIECES + 63) / 64;                      // pieces per lane
    const uint32_t lane = threadIdx.x;
    const uint32_t sub = lane % LPR, rsel = lane / LPR;
    const uint32_t halves = a.k >> 7;  // half blocks per row (<= LPR)
    const uint32_t row_bytes = halves * kHalfBytes;
    const bool hvalid = sub < halves;
    const uint32_t hb = hvalid ? sub : 0;
    const uint32_t blk = hb >> 1, n = hb & 1u;

    __shared__ __align__(16) uint8_t slot[kSlotBytes];

    const uint32_t wave_row0 = blockIdx.x * a.rows_per_wave;
    const uint32_t wave_row1 = min(wave_row0 + a.rows_per_wave, a.m);

    // The span of one pass as 16-byte pieces from the 16-byte boundary at or below its first
    // byte (rows are only 2-byte aligned; the matrix base is 256-byte aligned); pieces past the
    // span read offset 0 instead (the allocation is padded, so the last piece of the last row
    // may hang over by < 16 bytes).  lead(row0) = bytes of the first piece before the span.
    uint4 piece[PPL];
    auto lead_of = [&](uint32_t row0) { return (uint32_t)(((size_t)row0 * row_bytes) & 15u); };
    auto issue = [&](uint32_t row0) {
        const uint32_t nrows = row0 < a.m ? min((uint32_t)RPW, a.m - row0) : 0u;
        const size_t first = (size_t)row0 * row_bytes;
        const uint32_t span = (uint32_t)(first & 15u) + nrows * row_bytes;
        const uint8_t* sp = a.w + (first & ~(size_t)15);
#pragma unroll
        for (int j = 0; j < PPL; j++) {
            const uint32_t o = 16u * (64u * j + lane);
            const bool ok = o < span;
            const u32x4_native_a4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_native_a4*>(ok ? sp + o : a.w));
            piece[j] = make_uint4(t.x, t.y, t.z, t.w);
        }
    };

    // FUSED: the activations and norm weights are requested before the weight span (they come from the L2 and the load
    // counter retires in order), so that the norm and the quantizer run while the span is still on its way from HBM.
    constexpr int XE = FUSED ? 2 * LPR : 1;        // k / 64 elements per lane in the order of the f64 sums
    constexpr int XQ = FUSED ? (LPR + 1) / 2 : 1;  // k / 256 quads per lane for the quantizer
    float xe[XE];
    float4 xv4[XQ], wv4[XQ];
    if constexpr (FUSED) {
        const uint32_t quads = a.k >> 2;  // a multiple of 64
#pragma unroll
        for (int j = 0; j < XE; j++) {
            const uint32_t e = 64u * j + lane;
            xe[j] = a.xf[e < a.k ? e : lane];
        }
#pragma unroll
        for (int j = 0; j < XQ; j++) {
            const uint32_t quad = lane + 64u * j;
            xv4[j] = reinterpret_cast<const float4*>(a.xf)[quad < quads ? quad : lane];
            wv4[j] = reinterpret_cast<const float4*>(a.norm_w)[quad < quads ? quad : lane];
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }

    issue(wave_row0);

    __shared__ __align__(16) uint32_t fq[FUSED ? LPR * 32 : 4];  // k <= 128 LPR quants
    __shared__ float fs[FUSED ? LPR * 4 : 1];
    if constexpr (FUSED) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        double part[4] = {0.0, 0.0, 0.0, 0.0};  // of the four threads (lane, lane + 64, ..) this lane stands for
#pragma unroll
        for (int b = 0; b < XE / 4; b++) {
            if (256u * b < a.k) {  // uniform; k % 256 == 0
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const double x = (double)xe[4 * b + v];
                    part[v] += x * x;
                }
            }
        }
        double total = 0.0;
#pragma unroll
        for (int v = 0; v < 4; v++) total += wave_sum_f64(part[v]);
        const float inv_rms = (float)(1.0 / sqrt(total / (double)a.k + (double)a.eps));
        const uint32_t quads = a.k >> 2;
#pragma unroll
        for (int j = 0; j < XQ; j++) {
            const uint32_t quad = lane + 64u * j;
            if (64u * j < quads) {  // uniform: whole rounds
                const float4 v = xv4[j], w = wv4[j];
                const float v0 = __fmul_rn(__fmul_rn(v.x, inv_rms), w.x), v1 = __fmul_rn(__fmul_rn(v.y, inv_rms), w.y);
                const float v2 = __fmul_rn(__fmul_rn(v.z, inv_rms), w.z), v3 = __fmul_rn(__fmul_rn(v.w, inv_rms), w.w);
                float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
                amax = group_max8(amax);
                float id;
                const float scale = q8_scale_and_inverse(amax, id);
                fq[quad] = q8_pack4(v0, v1, v2, v3, id);
                if ((quad & 7u) == 0) fs[quad >> 3] = scale;
            }
        }
        // the same wave reads the vector back below; LDS operations of a wave execute in order
    }

    // This lane's 128 activation quants (4 Q8_0 blocks), their scales and the eight 16-element sums.
    uint32_t xq[32];
    float xsc[4];
    int xsum[8];
    {
        const uint4* src = FUSED ? reinterpret_cast<const uint4*>(fq + blk * 64 + 32 * n)
                                 : reinterpret_cast<const uint4*>(a.xq + (size_t)blk * 256 + 128 * n);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint4 v = src[i];
            xq[4 * i + 0] = hvalid ? v.x : 0, xq[4 * i + 1] = hvalid ? v.y : 0, xq[4 * i + 2] = hvalid ? v.z : 0, xq[4 * i + 3] = hvalid ? v.w : 0;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if constexpr (DUMP) xsc[i] = 0.0f;  // no scales behind the parity hook
            else if constexpr (FUSED) xsc[i] = hvalid ? fs[blk * 8 + 4 * n + i] : 0.0f;
            else xsc[i] = hvalid ? a.xs[blk * 8 + 4 * n + i] : 0.0f;
        }
#pragma unroll
        for (int g = 0; g < 8; g++) {
            int s = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) s = __builtin_amdgcn_sdot4(0x01010101, (int)xq[4 * g + i], s, false);
            xsum[g] = s;
        }
    }

    unsigned long long best = 0ull;  // below every real key
    for (uint32_t row0 = wave_row0; row0 < wave_row1; row0 += RPW) {
        // span -> LDS (same wave writes and reads; LDS operations of a wave execute in order)
#pragma unroll
        for (int j = 0; j < PPL; j++) {
            const uint32_t o = 16u * (64u * j + lane);
            if (o + 16u <= (uint32_t)kSlotBytes) *reinterpret_cast<uint4*>(slot + o) = piece[j];
        }
        const uint32_t base = lead_of(row0) + rsel * row_bytes + blk * kQ6kBlockBytes;
        uint32_t ql[16], qh[8], scw[2], dwd[1];
        read_run<16>(slot, base + 64 * n, ql);
        read_run<8>(slot, base + 128 + 32 * n, qh);
        read_run<2>(slot, base + 192 + 8 * n, scw);
        read_run<1>(slot, base + 208, dwd);
        if (row0 + RPW < wave_row1) issue(row0 + RPW);  // next pass, under this pass's arithmetic

        const float d = f16_bits_to_f32(dwd[0] & 0xffffu);
        float acc = 0.0f;
        const uint32_t row = row0 + rsel;
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int g = 2 * j + h;  // 16-element group within the half block
                int dot = 0;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t lo = (ql[8 * (j & 1) + 4 * h + i] >> (4 * (j >> 1))) & 0x0f0f0f0fu;
                    const uint32_t hi = ((qh[4 * h + i] >> (2 * j)) & 0x03030303u) << 4;
                    dot = __builtin_amdgcn_sdot4((int)(lo | hi), (int)xq[8 * j + 4 * h + i], dot, false);
                }
                dot -= 32 * xsum[g];
                if constexpr (DUMP) {
                    if (hvalid && row < a.m) a.dots[(size_t)row * (a.k >> 4) + 16 * blk + 8 * n + g] = dot;
                } else {
                    const int sc = (int)(int8_t)((scw[g >> 2] >> (8 * (g & 3))) & 0xffu);
                    const float f = (d * (float)sc) * xsc[g >> 1];
                    acc += f * (float)dot;
                }
            }
        }
        if constexpr (!DUMP) {
            const float tot = group_sum<LPR>(hvalid ? acc : 0.0f);
            if (sub == 0 && row < wave_row1) {
                float* dst = a.y + (size_t)row * a.y_row_stride;
                const float out = a.accumulate ? *dst + tot : tot;
                *dst = out;
                if (a.partial) {
                    const unsigned long long key = argmax_key(out, row);
                    best = key > best ? key : best;
                }
            }
        }
    }
    if constexpr (!DUMP) {
        if (a.partial) {  // uniform
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const unsigned long long o = __shfl_xor(best, off, 64);
                best = o > best ? o : best;
            }
            if (lane == 0) a.partial[blockIdx.x] = best;
        }
    }
}

// The norm-fused variant runs fewer, longer waves: each redoes the norm once (4, 6, 8, 12, 16 per CU measured inside a decode
// step: 8 best by 0.1 - 0.8 %).
constexpr uint32_t kFusedWavesPerCu = 8;

// Rows per wave and waves of a launch over m rows with LPR lanes per row.
template <int LPR>
uint32_t plan_lpr(uint32_t m, int num_cus, uint32_t& rows_per_wave, uint32_t waves_per_cu = 12u) {
    constexpr uint32_t RPW = 64 / LPR;
    const uint32_t passes = (m + RPW - 1) / RPW;
    const uint32_t max_waves = (uint32_t)num_cus * waves_per_cu;  // 12: measured best on the 65536 x 1024 LM head (8..16 within 7 %)
    uint32_t ppw = (passes + max_waves - 1) / max_waves;
    if (ppw == 0) ppw = 1;
    rows_per_wave = ppw * RPW;
    return (m + rows_per_wave - 1) / rows_per_wave;
}

template <int LPR, bool DUMP, bool FUSED>
hipError_t launch_lpr(Q6kArgs& a, int num_cus, const Launch& L) {
    const uint32_t waves = plan_lpr<LPR>(a.m, num_cus, a.rows_per_wave, FUSED ? kFusedWavesPerCu : 12u);
    return launch_kernel(L, kFamGemv, gemv_q6k_kernel<LPR, DUMP, FUSED>, dim3(waves), dim3(64), a);
}

template <typename F>
auto with_lpr(uint32_t k, F&& f) {
    const uint32_t halves = k >> 7;
    if (halves <= 2) return f(std::integral_constant<int, 2>{});
    if (halves <= 4) return f(std::integral_constant<int, 4>{});
    if (halves <= 8) return f(std::integral_constant<int, 8>{});
    if (halves <= 16) return f(std::integral_constant<int, 16>{});
    if (halves <= 32) return f(std::integral_constant<int, 32>{});
    return f(std::integral_constant<int, 64>{});
}

template <bool DUMP, bool FUSED = false>
hipError_t dispatch(Q6kArgs& a, int num_cus, const Launch& L) {
    if (a.m == 0) return hipSuccess;
    if ((a.k >> 7) > 64) return hipErrorInvalidValue;  // k > 8192: callers reject it
    return with_lpr(a.k, [&](auto lpr) { return launch_lpr<decltype(lpr)::value, DUMP, FUSED>(a, num_cus, L); });
}

}  // namespace

hipError_t launch_gemv_q6k(const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, const float* d_scales, float* d_y,
                           uint32_t y_row_stride, int accumulate, int num_cus, const Launch& L) {
    Q6kArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = d_scales, a.y = d_y, a.dots = nullptr;
    a.m = m, a.k = k, a.y_row_stride = y_row_stride, a.accumulate = accumulate;
    return dispatch<false>(a, num_cus, L);
}

uint32_t gemv_q6k_waves(uint32_t m, uint32_t k, int num_cus) {
    if (m == 0 || (k >> 7) > 64) return 0;
    uint32_t rpw = 0;
    return with_lpr(k, [&](auto lpr) { return plan_lpr<decltype(lpr)::value>(m, num_cus, rpw, kFusedWavesPerCu); });
}

hipError_t launch_gemv_q6k_rmsnorm(const uint8_t* d_w, uint32_t m, uint32_t k, const float* d_x, const float* d_norm_weight, float eps, float* d_y,
                                   int accumulate, int num_cus, const Launch& L, unsigned long long* d_partial) {
    Q6kArgs a{};
    a.w = d_w, a.y = d_y, a.xf = d_x, a.norm_w = d_norm_weight, a.eps = eps, a.partial = d_partial;
    a.m = m, a.k = k, a.y_row_stride = 1, a.accumulate = accumulate;
    return dispatch<false, true>(a, num_cus, L);
}

hipError_t launch_group_dots_q6k(const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, int32_t* d_out, int num_cus,
                                 const Launch& L) {
    Q6kArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = nullptr, a.y = nullptr, a.dots = d_out;
    a.m = m, a.k = k;
    return dispatch<true>(a, num_cus, L);
}

}  // namespace wick_rocm
