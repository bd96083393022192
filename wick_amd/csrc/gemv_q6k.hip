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

template <int LPR, bool DUMP>
__global__ __launch_bounds__(64) void gemv_q6k_kernel(Q6kArgs a) {
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

    issue(wave_row0);

    // This lane's 128 activation quants (4 Q8_0 blocks), their scales and the eight 16-element sums.
    uint32_t xq[32];
    float xsc[4];
    int xsum[8];
    {
        const uint4* src = reinterpret_cast<const uint4*>(a.xq + (size_t)blk * 256 + 128 * n);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint4 v = src[i];
            xq[4 * i + 0] = hvalid ? v.x : 0, xq[4 * i + 1] = hvalid ? v.y : 0, xq[4 * i + 2] = hvalid ? v.z : 0, xq[4 * i + 3] = hvalid ? v.w : 0;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if constexpr (DUMP) xsc[i] = 0.0f;  // no scales behind the parity hook
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
                *dst = a.accumulate ? *dst + tot : tot;
            }
        }
    }
}

template <int LPR, bool DUMP>
hipError_t launch_lpr(Q6kArgs& a, int num_cus, const Launch& L) {
    constexpr uint32_t RPW = 64 / LPR;
    const uint32_t passes = (a.m + RPW - 1) / RPW;
    const uint32_t max_waves = (uint32_t)num_cus * 12u;  // measured best on the 65536 x 1024 LM head (8..16 within 7 %)
    uint32_t ppw = (passes + max_waves - 1) / max_waves;
    if (ppw == 0) ppw = 1;
    a.rows_per_wave = ppw * RPW;
    const uint32_t waves = (a.m + a.rows_per_wave - 1) / a.rows_per_wave;
    return launch_kernel(L, kFamGemv, gemv_q6k_kernel<LPR, DUMP>, dim3(waves), dim3(64), a);
}

template <bool DUMP>
hipError_t dispatch(Q6kArgs& a, int num_cus, const Launch& L) {
    if (a.m == 0) return hipSuccess;
    const uint32_t halves = a.k >> 7;
    if (halves <= 2) return launch_lpr<2, DUMP>(a, num_cus, L);
    if (halves <= 4) return launch_lpr<4, DUMP>(a, num_cus, L);
    if (halves <= 8) return launch_lpr<8, DUMP>(a, num_cus, L);
    if (halves <= 16) return launch_lpr<16, DUMP>(a, num_cus, L);
    if (halves <= 32) return launch_lpr<32, DUMP>(a, num_cus, L);
    if (halves <= 64) return launch_lpr<64, DUMP>(a, num_cus, L);
    return hipErrorInvalidValue;  // k > 8192: callers reject it
}

}  // namespace

hipError_t launch_gemv_q6k(const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, const float* d_scales, float* d_y,
                           uint32_t y_row_stride, int accumulate, int num_cus, const Launch& L) {
    Q6kArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = d_scales, a.y = d_y, a.dots = nullptr;
    a.m = m, a.k = k, a.y_row_stride = y_row_stride, a.accumulate = accumulate;
    return dispatch<false>(a, num_cus, L);
}

hipError_t launch_group_dots_q6k(const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, int32_t* d_out, int num_cus,
                                 const Launch& L) {
    Q6kArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = nullptr, a.y = nullptr, a.dots = d_out;
    a.m = m, a.k = k;
    return dispatch<true>(a, num_cus, L);
}

}  // namespace wick_rocm
