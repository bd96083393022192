// Decode GEMV (and small-n multi-token GEMV) over raw GGUF Q4_0 / Q8_0 blocks
// against Q8_0-quantized activations, for gfx950.
//
// Arithmetic: gemv_q4_0_q8_0_neon / gemv_q8_0_q8_0_neon
// (wick/src/backend/simd.rs:328-415, 440-524):
//   y[i] = sum_b f32(isum_{i,b}) * (f32(f16 d_w[i,b]) * xs[b]),  isum exact i32.
// The f32 summation order differs from NEON's (tree over lanes instead of
// even/odd block accumulators); the contract is rel-L2 <= 1e-5, not bit equality.
//
// Shape of the kernel (HBM-bandwidth-bound, no matrix cores):
//   * The weight matrix is a flat stream of 36-byte (Q4_0) / 68-byte (Q8_0)
//     block PAIRS; a row of k elements is k/64 consecutive pairs and rows follow
//     each other without padding, so 64 consecutive lanes read 64 consecutive
//     pairs = one contiguous 2304 / 4352 byte span with dword-aligned wide loads.
//   * A row is owned by LPR lanes (power of two, <= 64); a lane always meets the
//     same pair index of every row it visits, so its slice of the activation
//     vector (64 int8 + 2 scales per pair) lives in REGISTERS for the whole
//     kernel.  Nothing is staged through LDS.
//   * Nibbles are unpacked with and/shift and dotted with v_dot4_i32_i8; the
//     "-8" of Q4_0 is folded into one subtraction of 8*sum(x) per block.
//   * U rows are in flight per lane before any is consumed, and every wave is
//     its own workgroup so small matrices still spread over all 256 CUs.
//   * Rows are reduced across their LPR lanes with lane swaps.
#pragma once
#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

#include <cstdlib>
#include <type_traits>

namespace wick_rocm {

namespace {

struct GemvArgs {
    GemvBatch batch;
    const int8_t* xq;   // [n][k]      (pre-quantized activations)
    const float* xs;    // [n][k/32]
    const float* xf;    // [n][x_stride] f32 activations, quantized in-kernel (FUSEQ variants)
    const float* xaux;  // FUSEQ with a transform: RMSNorm weights [k] / the "up" vector [k] / the conv kernel [k][3]
    const float* xaux2; // kXformShortConv: the rolling conv state [2][k] (read only)
    // GATED with a side job: the rolling state of the layer's short convolution is advanced by the first workgroups
    // (conv_state[s] <- conv_state[s + 1], last slot <- b * x of conv_proj = [b | c | x]); null: no side job
    float* conv_state;
    const float* conv_proj;
    uint32_t conv_hidden, conv_kernel;
    float eps;          // RMSNorm epsilon
    int32_t* dots;      // parity hook (DUMP variants): raw i32 block dots, [token][row][block], instead of y
    int xform;          // kXformNone / kXformRmsNorm / kXformSiluMul (host-side selector of the kernel variant)
    int gated;          // host-side selector of the GATED variant: batch.w[0] = gate, batch.w[1] = up, y[0][r] = silu(gate_r) * up_r
    uint32_t x_stride;
    uint32_t k;
    uint32_t n;         // tokens (1 for decode)
    uint32_t y_stride;  // token-major: >= rows of that weight; row-major: >= n
    uint32_t rows_per_wave;
    uint32_t total_waves;
    int y_row_major;
    int accumulate;
    uint32_t wave_end[kMaxGemvBatch];  // running total of waves per weight (a wave never straddles weights); UINT32_MAX past the batch
};

template <int TYPE, int NT>
struct ActRegs {
    uint32_t q[NT][2][8];  // two blocks of 32 int8
    float s[NT][2];
    int sum[NT][2];  // sum of the block's quants (used by Q4_0 only)
};

// FUSEQ workgroups have four waves that quantize the activation vector together.
constexpr int kFusedWaves = 4;
constexpr int kFusedMaxK = 8192;
constexpr int kConvMaxK = 2048;  // kXformShortConv: eight operands per quad instead of two

// How a lane gets its pair (MODE):
//   kDirect    each lane loads its own 36 / 68 bytes (two / four 16-byte loads + one dword);
//   kDirectNT  the same, loads marked nontemporal;
//   kSpan      the wave loads the contiguous span that holds its 64 pairs as whole consecutive
//              16-byte pieces (lane l takes bytes 16 l .. 16 l + 15 of every KB: each load
//              instruction covers whole cache lines once, nontemporal), parks the span in a
//              wave-private LDS slot and every lane reads its pair back from there (lane
//              stride 9 / 17 dwords: odd, conflict-free).  The same wave writes and reads the
//              slot and LDS operations of a wave execute in order, so no barrier is involved.
enum { kDirect = 0, kDirectNT = 1, kSpan = 2 };

// What the fused variant does to the f32 activations before quantizing them (XF):
//   kXformRmsNorm  x * inv_rms * weight (cpu::rmsnorm, wick/src/backend/cpu.rs:577-594): the norm in front of
//                  every projection of a decode step, folded into the projection's launch like the reference's
//                  encode_gemv_rmsnorm_gate_up (wick/src/model/metal_lfm2.rs:1157-1186);
//   kXformSiluMul  silu(x) * up (cpu::silu_mul_inplace, wick/src/backend/cpu.rs:668-673) in front of the FFN's
//                  down projection.
//   kXformShortConv  the gated short convolution of a decode step (forward_conv_block's middle, wick/src/model/lfm2.rs:694-726)
//                  in front of its out projection: x = [b | c | x'] (3k floats), out = c * (s0 w0 + s1 w1 + (b x') w2)
//                  with the rolling state s0, s1 READ ONLY -- many workgroups read it, so it is advanced by a later
//                  launch (the side job of the gate / up kernel).  Kernel size 3, k <= 2048.
// Every workgroup redoes the transform on the whole vector (k <= 8192 floats, a few per thread): cheaper than a
// launch of its own.

// The leading scalar parameters repeat fields of `a` (x = a.xf for the fused variant, a.xq
// otherwise; w0 / y0 / rows0 = weight 0 of the batch).  Passed on their own, at the front,
// they are the kernel arguments the hardware preloads into SGPRs at wave launch (the build
// asks for that, -amdgpu-kernarg-preload-count): everything needed to issue the activation
// and weight loads of a single-weight launch is there at the first instruction, instead of
// after one or two scalar-load round trips (~0.15 us each, on the critical path of a
// 2-3 us launch).  The rest of `a` is still fetched the ordinary way, under those loads.
// GATED: the FFN's gate and up projections in one pass with the gate applied to the results.  Lane slots u = 0, 2, ..
// hold rows of weight 0 (gate), u = 1, 3, .. the same rows of weight 1 (up); the lane that ends up with both row sums
// stores silu(gate) * up (cpu::silu_mul_inplace, wick/src/backend/cpu.rs:668-673): the same f32 values the two plain
// projections would have written, so the result is bit-identical to projection + projection + silu_mul, without the
// launch and the round trip through memory in between.
// DUMP: the parity hook.  The same loads, LDS hand-over, unpack and v_dot4 as the product kernel; the exact i32 dot of
// every (token, row, block) is written out where the product kernel would scale and sum it.
// SPAN: the timing hook.  The product instruction stream plus two reads of the 100 MHz wall clock per wave: the wave's first
// instruction and, after its last store has been acknowledged, its last.  Both go to a.dots (as [wave][2] 64-bit words); the
// host takes first start -> last end as the launch's execution span (the counterpart of the reference's per-dispatch GPU
// timestamps, wick/src/model/metal_lfm2.rs:3367-4116, for launches inside a graph replay, which carry no events).
template <int TYPE, int LPR, int NCHUNK, int U, int NT, bool FUSEQ, bool MULTI, int MODE, int XF = kXformNone, bool GATED = false, bool DUMP = false,
          bool SPAN = false>
__global__ __launch_bounds__(FUSEQ ? 64 * kFusedWaves : 64) void gemv_pairs_kernel(const void* p_x, const uint8_t* p_w0, float* p_y0,
                                                                                  uint32_t p_k, uint32_t p_rows0,
                                                                                  uint32_t p_rows_per_wave, uint32_t p_total_waves,
                                                                                  int p_accumulate, GemvArgs a) {
    static_assert(XF == kXformNone || FUSEQ, "activation transforms belong to the fused-quantizer variant");
    static_assert(!GATED || (FUSEQ && !MULTI && NT == 1 && U % 2 == 0), "the gated variant pairs lane slots");
    static_assert(!DUMP || (!MULTI && !GATED && XF == kXformNone), "the parity hook runs the plain single-weight variants");
    static_assert(!SPAN || (!DUMP && !FUSEQ && !MULTI && NT == 1), "the timing hook runs the plain single-token variants");
    unsigned long long span_t0 = 0;
    if constexpr (SPAN) span_t0 = __builtin_amdgcn_s_memrealtime();
    constexpr int UR = GATED ? U / 2 : U;  // distinct rows per lane and pass
    using PT = PairTraits<TYPE>;
    constexpr int RPW = 64 / LPR;  // rows per wave pass
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t sub = lane % LPR;
    const uint32_t rsel = lane / LPR;
    const uint32_t ppr = p_k >> 6;  // pairs per row
    const uint32_t nb = p_k >> 5;
    const uint32_t tok0 = blockIdx.y * NT;

    const uint32_t gwave =
        FUSEQ ? blockIdx.x * kFusedWaves + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) : blockIdx.x;
    // The f32 activations are requested first of all (fused variant): they need only two
    // scalars of the argument block, and everything below overlaps with their latency.
    constexpr int kQuadRounds = XF == kXformShortConv ? kConvMaxK / 4 / (64 * kFusedWaves)  // 2: eight operands per quad
                                                      : kFusedMaxK / 4 / (64 * kFusedWaves);  // 8
    float4 xv[FUSEQ ? kQuadRounds : 1];
    float4 av[XF != kXformNone && XF != kXformShortConv ? kQuadRounds : 1];  // the transform's second operand, same quads
    float4 cv[XF == kXformShortConv ? kQuadRounds : 1][7];  // conv operands: c, x', state 0, state 1, three quads of the kernel (xv holds b)
    if constexpr (FUSEQ) {
        const uint32_t quads = p_k >> 2;
#pragma unroll
        for (int i = 0; i < kQuadRounds; i++) {
            const uint32_t quad = threadIdx.x + i * 64 * kFusedWaves;
            // whole rounds past the end of the vector are skipped (uniform, one taken branch);
            // within a round: clamped
            if (i > 0 && i * 64 * kFusedWaves >= quads) break;
            xv[i] = reinterpret_cast<const float4*>(p_x)[min(quad, quads - 1)];
        }
        if constexpr (XF == kXformShortConv) {
            const float4 *px = reinterpret_cast<const float4*>(p_x), *st = reinterpret_cast<const float4*>(a.xaux2),
                         *cw = reinterpret_cast<const float4*>(a.xaux);
#pragma unroll
            for (int i = 0; i < kQuadRounds; i++) {
                if (i > 0 && i * 64 * kFusedWaves >= quads) break;
                const uint32_t quad = min(threadIdx.x + i * 64 * kFusedWaves, quads - 1);
                cv[i][0] = px[quads + quad], cv[i][1] = px[2 * quads + quad];
                cv[i][2] = st[quad], cv[i][3] = st[quads + quad];
                cv[i][4] = cw[3 * quad], cv[i][5] = cw[3 * quad + 1], cv[i][6] = cw[3 * quad + 2];  // [channel][tap] of four channels
            }
        } else if constexpr (XF != kXformNone) {
            const float4* aux = reinterpret_cast<const float4*>(a.xaux);
#pragma unroll
            for (int i = 0; i < kQuadRounds; i++) {
                const uint32_t quad = threadIdx.x + i * 64 * kFusedWaves;
                if (i > 0 && i * 64 * kFusedWaves >= quads) break;
                av[i] = aux[min(quad, quads - 1)];
            }
        }
        // keep the compiler from moving the weight loads in front of these
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }

    if constexpr (GATED) {
        // Side job of the FFN's gate / up launch in a gated-conv layer: advance the layer's rolling conv state.  The out
        // projection before this launch has read the old state; nothing reads it again before the next token.  One thread
        // per four channels, slots ascending, exactly what shortconv_step_kernel does to the state.
        if (a.conv_state != nullptr && blockIdx.x * (64u * kFusedWaves) < (a.conv_hidden >> 2)) {
            const uint32_t cq = a.conv_hidden >> 2, d_conv = a.conv_kernel - 1;
            const float4* pj = reinterpret_cast<const float4*>(a.conv_proj);
            float4* st = reinterpret_cast<float4*>(a.conv_state);
            for (uint32_t q = blockIdx.x * (64u * kFusedWaves) + threadIdx.x; q < cq; q += gridDim.x * (64u * kFusedWaves)) {  // any grid covers every channel
                const float4 b = pj[q], x = pj[2 * cq + q];
                for (uint32_t s_ = 1; s_ < d_conv; s_++) st[(size_t)(s_ - 1) * cq + q] = st[(size_t)s_ * cq + q];
                st[(size_t)(d_conv - 1) * cq + q] = make_float4(__fmul_rn(b.x, x.x), __fmul_rn(b.y, x.y), __fmul_rn(b.z, x.z), __fmul_rn(b.w, x.w));
            }
        }
    }

    // Which weight of the batch this wave works on.  Every per-weight field is copied out of
    // the argument block first (one scalar-load round trip for all of them; the empty asm
    // keeps the compiler from sinking the loads into the selection below, which would make
    // them a second, dependent round trip) and then picked with scalar selects.
    // wave_end[] entries past the batch are UINT32_MAX (set_wave_ends).
    uint32_t widx = 0;
    const uint8_t* wbase = p_w0;
    float* ybase = p_y0;
    uint32_t row_hi = p_rows0, row_lo = 0, wave_lo = 0;
    if constexpr (MULTI) {
        uint64_t w0 = (uint64_t)a.batch.w[0], w1 = (uint64_t)a.batch.w[1], w2 = (uint64_t)a.batch.w[2], w3 = (uint64_t)a.batch.w[3];
        uint64_t y0 = (uint64_t)a.batch.y[0], y1 = (uint64_t)a.batch.y[1], y2 = (uint64_t)a.batch.y[2], y3 = (uint64_t)a.batch.y[3];
        uint32_t r0 = a.batch.row_end[0], r1 = a.batch.row_end[1], r2 = a.batch.row_end[2], r3 = a.batch.row_end[3];
        uint32_t e0 = a.wave_end[0], e1 = a.wave_end[1], e2 = a.wave_end[2], cnt = a.batch.count;
        // (the inputs only pull the remaining fields into the same round trip)
        asm(""
            : "+s"(w0), "+s"(w1), "+s"(w2), "+s"(w3), "+s"(y0), "+s"(y1), "+s"(y2), "+s"(y3), "+s"(r0), "+s"(r1), "+s"(r2),
              "+s"(r3), "+s"(e0), "+s"(e1), "+s"(e2), "+s"(cnt)
            : "s"(a.xs));
        widx = min((uint32_t)(gwave >= e0) + (uint32_t)(gwave >= e1) + (uint32_t)(gwave >= e2), cnt - 1u);
        // Masks instead of ?: -- the compiler turns a chain of scalar selects into a chain of
        // branches, and a taken scalar branch costs more than all of this arithmetic.
        const uint64_t m0 = 0ull - (uint64_t)(widx == 0), m1 = 0ull - (uint64_t)(widx == 1), m2 = 0ull - (uint64_t)(widx == 2),
                       m3 = 0ull - (uint64_t)(widx == 3);
        auto pick = [&](uint64_t v0, uint64_t v1, uint64_t v2, uint64_t v3) { return (v0 & m0) | (v1 & m1) | (v2 & m2) | (v3 & m3); };
        // (the integers came out of an asm: say again that these are global addresses)
        wbase = (const uint8_t*)(const uint8_t __attribute__((address_space(1)))*)pick(w0, w1, w2, w3);
        ybase = (float*)(float __attribute__((address_space(1)))*)pick(y0, y1, y2, y3);
        row_hi = (uint32_t)pick(r0, r1, r2, r3);
        row_lo = (uint32_t)pick(0u, r0, r1, r2);
        wave_lo = (uint32_t)pick(0u, e0, e1, e2);
    }
    const uint32_t rows = row_hi - row_lo;
    const uint32_t wave = gwave - wave_lo;
    // Waves past the end of the batch (last workgroup of a fused launch) get an empty row
    // range but still take part in the cooperative quantization and its barrier.
    const bool live_wave = gwave < p_total_waves;
    const uint32_t wave_row0 = live_wave ? wave * p_rows_per_wave : 0;
    const uint32_t wave_row1 = live_wave ? min(wave_row0 + p_rows_per_wave, rows) : 0;

    bool pvalid[NCHUNK];
#pragma unroll
    for (int c = 0; c < NCHUNK; c++) pvalid[c] = c * LPR + sub < ppr;

    // Weight registers of one pass (U rows per lane) and where each row's result goes.
    constexpr int WREGS = PT::DWORDS;
    constexpr int WIDE = PT::BYTES / 16;  // 16-byte pieces per lane and span (kSpan)
    uint32_t w[U][NCHUNK][WREGS];
    uint32_t span_tail[U][NCHUNK];  // kSpan: where the dword remainder of the span starts
    bool rvalid[U];
    uint32_t lrow[U];
    __shared__ __align__(16) uint8_t span_lds[MODE == kSpan ? (FUSEQ ? kFusedWaves : 1) * 64 * PT::BYTES : 16];
    // Loads are unconditional (row and pair indices clamped into range) so that the number
    // of outstanding loads is known at every wait; a clamped load's data is neutralised by
    // zero activation scales (pair out of range) or simply not stored (row out of range).
    const uint8_t* const wbase_of_wave = wbase;
    const uint8_t* wbase1 = GATED ? a.batch.w[1] : wbase;
    auto issue_pass = [&](uint32_t base) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int ur = GATED ? u >> 1 : u;
            const uint8_t* wbase = (GATED && (u & 1)) ? wbase1 : wbase_of_wave;
            lrow[u] = base + ur * RPW + rsel;
            rvalid[u] = lrow[u] < wave_row1;
            if constexpr (MODE == kSpan) {
                // First row of this pass (wave-uniform) and the rows of it that exist.
                const uint32_t row0 = base + ur * RPW;
                const uint32_t nrows = row0 < rows ? min((uint32_t)RPW, rows - row0) : 0u;
#pragma unroll
                for (int c = 0; c < NCHUNK; c++) {
                    const uint32_t pairs = NCHUNK == 1 ? nrows * ppr : (nrows && ppr > 64u * c ? min(64u, ppr - 64u * c) : 0u);
                    const uint32_t span = pairs * PT::BYTES;
                    const uint8_t* sp = wbase + (span ? ((size_t)row0 * ppr + 64u * c) * PT::BYTES : 0);
#pragma unroll
                    for (int j = 0; j < WIDE; j++) {
                        const uint32_t o = 1024u * j + 16u * lane;
                        const u32x4_native_a4 t =
                            __builtin_nontemporal_load(reinterpret_cast<const u32x4_native_a4*>(sp + (o + 16u <= span ? o : 0u)));
                        w[u][c][4 * j + 0] = t.x, w[u][c][4 * j + 1] = t.y, w[u][c][4 * j + 2] = t.z, w[u][c][4 * j + 3] = t.w;
                    }
                    // What the 16-byte pieces leave over (256 bytes of a full span, the last
                    // 4-12 bytes of a short one) goes as single dwords.
                    const uint32_t o = (min(span, 1024u * WIDE) & ~15u) + 4u * lane;
                    w[u][c][WREGS - 1] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(sp + (o + 4u <= span ? o : 0u)));
                    span_tail[u][c] = min(span, 1024u * WIDE) & ~15u;
                }
            } else {
                const uint8_t* rowp = wbase + (size_t)min(lrow[u], rows - 1) * ppr * PT::BYTES;
#pragma unroll
                for (int c = 0; c < NCHUNK; c++) {
                    const uint32_t p = pvalid[c] ? c * LPR + sub : 0;
                    load_pair<PT::DWORDS, MODE == kDirectNT>(rowp + (size_t)p * PT::BYTES, w[u][c]);
                }
            }
        }
    };
    // kSpan: the span pieces in w[u][c] go through this wave's LDS slot and come back as
    // this lane's own pair (position rsel * ppr + sub of the span, or sub for a row chunk).
    auto own_pair = [&](uint32_t (&piece)[WREGS], uint32_t tail) {
        if constexpr (MODE == kSpan) {
            uint8_t* slot = span_lds + (FUSEQ ? (threadIdx.x >> 6) * 64 * PT::BYTES : 0);
#pragma unroll
            for (int j = 0; j < WIDE; j++)
                *reinterpret_cast<uint4*>(slot + 1024 * j + 16 * lane) =
                    make_uint4(piece[4 * j], piece[4 * j + 1], piece[4 * j + 2], piece[4 * j + 3]);
            // after the pieces: a piece that straddles the span's end holds filler
            *reinterpret_cast<uint32_t*>(slot + tail + 4 * lane) = piece[WREGS - 1];
            const uint32_t pos = NCHUNK == 1 ? rsel * ppr + sub : sub;
            const uint32_t* mine = reinterpret_cast<const uint32_t*>(slot + (size_t)min(pos, 63u) * PT::BYTES);
#pragma unroll
            for (int i = 0; i < WREGS; i++) piece[i] = mine[i];
        }
    };

    // Order of the memory operations matters because the load counter retires in order:
    //   1. (fused) this thread's share of the f32 activation vector,
    //   2. the weight loads of the first pass (the long pole, HBM),
    //   3. wait for (1) only, quantize into LDS, barrier -- all under the latency of (2).
    __shared__ __align__(16) uint32_t fq[FUSEQ ? kFusedMaxK / 4 : 4];
    __shared__ float fs[FUSEQ ? kFusedMaxK / 32 : 1];
    issue_pass(wave_row0);
    if constexpr (FUSEQ) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }

    // Fused variant: the workgroup quantizes the f32 activation vector ONCE, together,
    // into LDS (eight lanes per 32-element block, exactly like the stand-alone quantizer
    // kernel), instead of every wave redoing it.  Only n = 1 uses this variant.
    if constexpr (FUSEQ) {
        const uint32_t quads = p_k >> 2;
        if constexpr (XF == kXformSiluMul) {
#pragma unroll
            for (int i = 0; i < kQuadRounds; i++) {
                if (i * 64 * kFusedWaves < quads) {
                    xv[i].x = silu_mul(xv[i].x, av[i].x), xv[i].y = silu_mul(xv[i].y, av[i].y);
                    xv[i].z = silu_mul(xv[i].z, av[i].z), xv[i].w = silu_mul(xv[i].w, av[i].w);
                }
            }
        }
        if constexpr (XF == kXformShortConv) {
            // per channel, the operations and their order are shortconv_step_kernel's: bit-identical
#pragma unroll
            for (int i = 0; i < kQuadRounds; i++) {
                if (i * 64 * kFusedWaves < quads) {
                    const float w[12] = {cv[i][4].x, cv[i][4].y, cv[i][4].z, cv[i][4].w, cv[i][5].x, cv[i][5].y,
                                         cv[i][5].z, cv[i][5].w, cv[i][6].x, cv[i][6].y, cv[i][6].z, cv[i][6].w};
                    const float b[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w}, c[4] = {cv[i][0].x, cv[i][0].y, cv[i][0].z, cv[i][0].w};
                    const float xx[4] = {cv[i][1].x, cv[i][1].y, cv[i][1].z, cv[i][1].w};
                    const float s0[4] = {cv[i][2].x, cv[i][2].y, cv[i][2].z, cv[i][2].w}, s1[4] = {cv[i][3].x, cv[i][3].y, cv[i][3].z, cv[i][3].w};
                    float o[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float sum = __fadd_rn(0.0f, __fmul_rn(s0[j], w[3 * j]));
                        sum = __fadd_rn(sum, __fmul_rn(s1[j], w[3 * j + 1]));
                        sum = __fadd_rn(sum, __fmul_rn(__fmul_rn(b[j], xx[j]), w[3 * j + 2]));
                        o[j] = __fmul_rn(c[j], sum);
                    }
                    xv[i] = make_float4(o[0], o[1], o[2], o[3]);
                }
            }
        }
        if constexpr (XF == kXformRmsNorm) {
            // f64 sum of squares over the whole vector (clamped duplicates of the last quad left out), one barrier
            __shared__ double sq[kFusedWaves];
            double part = 0.0;
#pragma unroll
            for (int i = 0; i < kQuadRounds; i++) {
                const uint32_t quad = threadIdx.x + i * 64 * kFusedWaves;
                if (i * 64 * kFusedWaves < quads && quad < quads) {
                    const double x0 = xv[i].x, x1 = xv[i].y, x2 = xv[i].z, x3 = xv[i].w;
                    part += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
                }
            }
            part = wave_sum_f64(part);
            if (lane == 0) sq[threadIdx.x >> 6] = part;
            __syncthreads();
            const double total = (sq[0] + sq[1]) + (sq[2] + sq[3]);
            const float inv_rms = (float)(1.0 / sqrt(total / (double)p_k + (double)a.eps));
#pragma unroll
            for (int i = 0; i < kQuadRounds; i++) {
                if (i * 64 * kFusedWaves < quads) {
                    xv[i].x = __fmul_rn(__fmul_rn(xv[i].x, inv_rms), av[i].x), xv[i].y = __fmul_rn(__fmul_rn(xv[i].y, inv_rms), av[i].y);
                    xv[i].z = __fmul_rn(__fmul_rn(xv[i].z, inv_rms), av[i].z), xv[i].w = __fmul_rn(__fmul_rn(xv[i].w, inv_rms), av[i].w);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kQuadRounds; i++) {
            const uint32_t quad = threadIdx.x + i * 64 * kFusedWaves;
            if (i * 64 * kFusedWaves < quads) {  // uniform: whole rounds only differ in their tail
                const float4 v = xv[i];
                float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
                amax = group_max8(amax);
                float id;
                const float scale = q8_scale_and_inverse(amax, id);
                if (quad < quads) {
                    fq[quad] = q8_pack4(v.x, v.y, v.z, v.w, id);
                    if ((quad & 7u) == 0) fs[quad >> 3] = scale;
                }
            }
        }
        __syncthreads();
    }

    // This lane's slice of the activations, kept in registers.
    ActRegs<TYPE, NT> act[NCHUNK];
#pragma unroll
    for (int c = 0; c < NCHUNK; c++) {
        const uint32_t p = c * LPR + sub;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const bool ok = pvalid[c] && (tok0 + t < a.n);
            const uint32_t tok = ok ? tok0 + t : 0;
            const uint32_t pp = ok ? p : 0;
            if constexpr (FUSEQ) {
                // This lane's two blocks, from the copy the workgroup quantized into LDS.
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const uint4 lo = *reinterpret_cast<const uint4*>(&fq[pp * 16 + h * 8]);
                    const uint4 hi = *reinterpret_cast<const uint4*>(&fq[pp * 16 + h * 8 + 4]);
                    act[c].q[t][h][0] = ok ? lo.x : 0, act[c].q[t][h][1] = ok ? lo.y : 0;
                    act[c].q[t][h][2] = ok ? lo.z : 0, act[c].q[t][h][3] = ok ? lo.w : 0;
                    act[c].q[t][h][4] = ok ? hi.x : 0, act[c].q[t][h][5] = ok ? hi.y : 0;
                    act[c].q[t][h][6] = ok ? hi.z : 0, act[c].q[t][h][7] = ok ? hi.w : 0;
                    act[c].sum[t][h] = (TYPE == 2) ? block_xsum(act[c].q[t][h]) : 0;
                    act[c].s[t][h] = ok ? fs[2 * pp + h] : 0.0f;
                }
            } else {
                const uint4* src = reinterpret_cast<const uint4*>(static_cast<const int8_t*>(p_x) + (size_t)tok * p_k + (size_t)pp * 64);
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    uint4 lo = src[2 * h], hi = src[2 * h + 1];
                    if (!ok) lo = hi = make_uint4(0, 0, 0, 0);
                    act[c].q[t][h][0] = lo.x, act[c].q[t][h][1] = lo.y, act[c].q[t][h][2] = lo.z, act[c].q[t][h][3] = lo.w;
                    act[c].q[t][h][4] = hi.x, act[c].q[t][h][5] = hi.y, act[c].q[t][h][6] = hi.z, act[c].q[t][h][7] = hi.w;
                    act[c].sum[t][h] = (TYPE == 2) ? block_xsum(act[c].q[t][h]) : 0;
                    const float sc = a.xs[(size_t)tok * nb + 2 * pp + h];
                    act[c].s[t][h] = ok ? sc : 0.0f;
                }
            }
        }
    }

    for (uint32_t base = wave_row0; base < wave_row1; base += RPW * UR) {
        if (base != wave_row0) issue_pass(base);
        // Consume.
        float gate_sum = 0.0f;  // GATED: the row sum of the even slot, waiting for its odd partner
#pragma unroll
        for (int u = 0; u < U; u++) {
            float acc[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) acc[t] = 0.0f;
#pragma unroll
            for (int c = 0; c < NCHUNK; c++) {
                uint32_t d0, d1, q0[PT::NQ], q1[PT::NQ];
                own_pair(w[u][c], span_tail[u][c]);
                split_pair<TYPE>(w[u][c], d0, d1, q0, q1);
                const float dw0 = pvalid[c] ? f16_bits_to_f32(d0) : 0.0f, dw1 = pvalid[c] ? f16_bits_to_f32(d1) : 0.0f;
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int i0 = block_dot<TYPE>(q0, act[c].q[t][0], act[c].sum[t][0]);
                    const int i1 = block_dot<TYPE>(q1, act[c].q[t][1], act[c].sum[t][1]);
                    if constexpr (DUMP) {
                        if (rvalid[u] && pvalid[c] && tok0 + t < a.n) {
                            int32_t* o = a.dots + ((size_t)(tok0 + t) * p_rows0 + lrow[u]) * nb + 2u * (c * LPR + sub);
                            o[0] = i0, o[1] = i1;
                        }
                    }
                    acc[t] += (float)i0 * (dw0 * act[c].s[t][0]);
                    acc[t] += (float)i1 * (dw1 * act[c].s[t][1]);
                }
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const float tot = group_sum<LPR>(acc[t]);
                if constexpr (DUMP) {
                    (void)tot;
                } else if constexpr (GATED) {
                    if ((u & 1) == 0) gate_sum = tot;
                    else if (sub == 0 && rvalid[u]) ybase[lrow[u]] = silu_mul(gate_sum, tot);
                } else if (sub == 0 && rvalid[u] && tok0 + t < a.n) {
                    float* dst = a.y_row_major ? ybase + (size_t)lrow[u] * a.y_stride + (tok0 + t)
                                               : ybase + (size_t)(tok0 + t) * a.y_stride + lrow[u];
                    *dst = p_accumulate ? *dst + tot : tot;
                }
            }
        }
    }
    if constexpr (SPAN) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the wave's stores have been acknowledged
        const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
        if (lane == 0) {
            unsigned long long* o = reinterpret_cast<unsigned long long*>(a.dots) + 2 * (size_t)gwave;
            o[0] = span_t0, o[1] = t1;
        }
    }
}

// Any k % 32 == 0, any byte alignment: one wave per row, lanes stride over single
// blocks, two-byte loads.  Correctness path for shapes the pair kernel does not
// take (odd block count per row, k > 8192); not tuned.
template <int TYPE, int NT, bool DUMP = false>
__global__ __launch_bounds__(64) void gemv_generic_kernel(GemvArgs a) {
    constexpr int BB = (TYPE == 2) ? kQ4BlockBytes : kQ8BlockBytes;
    constexpr int NQ = PairTraits<TYPE>::NQ;
    const uint32_t lane = threadIdx.x;
    const uint32_t nb = a.k >> 5;
    const uint32_t tok0 = blockIdx.y * NT;
    const uint8_t* wp = a.batch.w[0];
    float* yp = a.batch.y[0];
    uint32_t rows = a.batch.row_end[0];
    uint32_t wave = blockIdx.x;
    for (uint32_t i = 1; i < a.batch.count; i++) {
        if (blockIdx.x >= a.wave_end[i - 1]) {
            wp = a.batch.w[i];
            yp = a.batch.y[i];
            rows = a.batch.row_end[i] - a.batch.row_end[i - 1];
            wave = blockIdx.x - a.wave_end[i - 1];
        }
    }
    const uint32_t row0 = wave * a.rows_per_wave;
    const uint32_t row1 = min(row0 + a.rows_per_wave, rows);
    for (uint32_t lrow = row0; lrow < row1; lrow++) {
        const uint8_t* rowp = wp + (size_t)lrow * nb * BB;
        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) acc[t] = 0.0f;
        for (uint32_t b = lane; b < nb; b += 64) {
            const uint16_t* hp = reinterpret_cast<const uint16_t*>(rowp + (size_t)b * BB);
            const float dw = f16_bits_to_f32(hp[0]);
            uint32_t q[NQ];
#pragma unroll
            for (int j = 0; j < NQ; j++) q[j] = (uint32_t)hp[1 + 2 * j] | ((uint32_t)hp[2 + 2 * j] << 16);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if (tok0 + t < a.n) {
                    const uint32_t* xp = reinterpret_cast<const uint32_t*>(a.xq + (size_t)(tok0 + t) * a.k + (size_t)b * 32);
                    uint32_t x[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) x[j] = xp[j];
                    const int isum = block_dot<TYPE>(q, x, (TYPE == 2) ? block_xsum(x) : 0);
                    if constexpr (DUMP) a.dots[((size_t)(tok0 + t) * rows + lrow) * nb + b] = isum;
                    else acc[t] += (float)isum * (dw * a.xs[(size_t)(tok0 + t) * nb + b]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const float tot = group_sum<64>(acc[t]);
            if (!DUMP && lane == 0 && tok0 + t < a.n) {
                float* dst = a.y_row_major ? yp + (size_t)lrow * a.y_stride + (tok0 + t)
                                           : yp + (size_t)(tok0 + t) * a.y_stride + lrow;
                *dst = a.accumulate ? *dst + tot : tot;
            }
        }
    }
}

// Every weight of the batch gets its own whole number of waves.
inline uint32_t set_wave_ends(GemvArgs& a) {
    uint32_t waves = 0, prev = 0;
    for (uint32_t i = 0; i < a.batch.count; i++) {
        const uint32_t rows = a.batch.row_end[i] - prev;
        prev = a.batch.row_end[i];
        waves += (rows + a.rows_per_wave - 1) / a.rows_per_wave;
        a.wave_end[i] = waves;
    }
    for (uint32_t i = a.batch.count; i < kMaxGemvBatch; i++) a.wave_end[i] = UINT32_MAX;
    a.total_waves = waves;
    return waves;
}

// How the weights of a single-token launch are fetched, by bytes of weights in the launch
// (measured on MI355X, HBM-cold, inside a graph):
//   * small launches are latency-bound and per-lane loads save the LDS round trip.  For
//     Q4_0 nontemporal per-lane loads are 0.3-0.4 us faster than ordinary ones; for Q8_0
//     they are slower (a lane's 68 bytes take five load instructions that share cache
//     lines, and without L1 retention every one of them goes to L2 again), so Q8_0 keeps
//     ordinary loads and switches to span loads much earlier;
//   * from the threshold on, whole-line span loads (kSpan): 10-25 % faster on 5-150 MB
//     matrices, 6.4 TB/s kernel-time on a 142 MB Q8_0 matrix.
constexpr uint64_t kDirectMaxBytesQ4 = 3ull << 20;
constexpr uint64_t kDirectMaxBytesQ8 = 512ull << 10;
template <int TYPE, int LPR, int NCHUNK, int NT, bool FUSEQ, int U, bool DUMP, bool SPAN = false>
hipError_t launch_pairs_u(GemvArgs& a, uint32_t total_rows, int num_cus, const Launch& L) {
    const uint32_t pass_rows = (64 / LPR) * (a.gated ? U / 2 : U);
    // Enough waves to give every CU ~16, and every wave at least one full pass.
    const uint32_t max_waves = (uint32_t)num_cus * 16u;
    uint32_t passes = (total_rows + pass_rows - 1) / pass_rows;
    uint32_t passes_per_wave = (passes + max_waves - 1) / max_waves;
    if (passes_per_wave == 0) passes_per_wave = 1;
    a.rows_per_wave = passes_per_wave * pass_rows;
    const uint32_t waves = set_wave_ends(a);
    const dim3 grid = FUSEQ ? dim3((waves + kFusedWaves - 1) / kFusedWaves, 1) : dim3(waves, (a.n + NT - 1) / NT);
    const dim3 block(FUSEQ ? 64 * kFusedWaves : 64);
    const uint64_t bytes = (uint64_t)total_rows * (a.k >> 5) * (TYPE == 2 ? 18u : 34u) * (a.gated ? 2u : 1u);
    constexpr int kSmall = TYPE == 2 ? kDirectNT : kDirect;
    const uint64_t direct_max = L.gemv_direct_max_bytes >= 0 ? (uint64_t)L.gemv_direct_max_bytes : (TYPE == 2 ? kDirectMaxBytesQ4 : kDirectMaxBytesQ8);
    const bool multi = a.batch.count > 1;
    // Several token groups re-read the weights (they should stay cached): only launches of ONE group -- a single token, or up
    // to NT tokens of one Q8_0 weight -- stream them with whole-line nontemporal span loads (Q8_0 65536 x 2048 over four tokens:
    // 34.7 -> 29.5 us; a Q4_0 lane's 36 bytes are three loads either way and the span form is 3 % slower there).
    const bool one_group = NT == 1 || (TYPE == 8 && a.n <= (uint32_t)NT && !multi);
    const int mode = !one_group ? kDirect : (bytes < direct_max ? (NT > 1 ? kDirect : kSmall) : kSpan);
    // hot scalars first (preloaded into SGPRs), then the whole argument block
    auto go = [&](auto kernel) {
        return launch_kernel(L, kFamGemv, kernel, grid, block, FUSEQ ? static_cast<const void*>(a.xf) : static_cast<const void*>(a.xq),
                             a.batch.w[0], a.batch.y[0], a.k, a.batch.row_end[0], a.rows_per_wave, a.total_waves, a.accumulate, a);
    };
    if constexpr (DUMP) {  // the parity hook: plain single-weight variants, same fetch mode as the product launch of this size
        if constexpr (NT == 1) {
            if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, kXformNone, false, true>);
            return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall, kXformNone, false, true>);
        } else {
            if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, kXformNone, false, true>);
            return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kDirect, kXformNone, false, true>);
        }
    } else if constexpr (NT == 1 && FUSEQ) {
        // the activation transforms exist for the fused single-token variant only
        if (a.gated) {  // gate | up pairs: two lane slots per row, no transform other than the norm
            if constexpr (U == 2 && NCHUNK == 1) {
                if (a.xform == kXformRmsNorm) {
                    if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, kXformRmsNorm, true>);
                    return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall, kXformRmsNorm, true>);
                }
                if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, kXformNone, true>);
                return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall, kXformNone, true>);
            } else {
                return hipErrorInvalidValue;  // launch_pairs picks U = 2 for gated launches; gated_kernel_applies() keeps NCHUNK at 1
            }
        }
        auto with_xform = [&](auto xf) {
            constexpr int XF = decltype(xf)::value;
            if (mode == kSpan && multi) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, true, kSpan, XF>);
            if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, XF>);
            if (multi) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, true, kSmall, XF>);
            return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall, XF>);
        };
        if (a.xform == kXformShortConv) {  // k <= 2048: rows of at most 32 pairs; one weight
            if constexpr (LPR <= 32 && NCHUNK == 1) {
                if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, kXformShortConv>);
                return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall, kXformShortConv>);
            } else {
                return hipErrorInvalidValue;  // shortconv_kernel_applies() keeps such shapes away
            }
        }
        if (a.xform == kXformRmsNorm) return with_xform(std::integral_constant<int, kXformRmsNorm>{});
        if (a.xform == kXformSiluMul) return with_xform(std::integral_constant<int, kXformSiluMul>{});
        return with_xform(std::integral_constant<int, kXformNone>{});
    } else if constexpr (SPAN) {  // the timing hook: single weight, the fetch mode of the product launch
        if (multi) return hipErrorInvalidValue;
        if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan, kXformNone, false, false, true>);
        return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall, kXformNone, false, false, true>);
    } else if constexpr (NT == 1) {
        if (mode == kSpan && multi) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, true, kSpan>);
        if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan>);
        if (multi) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, true, kSmall>);
        return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSmall>);
    } else {
        if (multi) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, true, kDirect>);
        if (mode == kSpan) return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kSpan>);
        return go(gemv_pairs_kernel<TYPE, LPR, NCHUNK, U, NT, FUSEQ, false, kDirect>);
    }
}

// Rows in flight per lane (U).  Small matrices are latency-bound: the finer the waves,
// the sooner every byte is requested and the shorter each wave's unpack/dot tail, so U
// drops until there are enough waves to cover the chip; big matrices stream with U = 4
// (Q4_0) / 2 (Q8_0, whose pairs are 17 dwords).  WICK_ROCM_GEMV_U overrides (tuning knob,
// like the reference's WICK_Q4_FAST / WICK_SPLITS environment switches).
inline int gemv_u_override() {
    static const int v = [] {
        const char* e = getenv("WICK_ROCM_GEMV_U");
        return e ? atoi(e) : 0;
    }();
    return v;
}

template <int TYPE, int LPR, int NCHUNK, int NT, bool FUSEQ, bool DUMP, bool SPAN = false>
hipError_t launch_pairs(GemvArgs& a, uint32_t total_rows, int num_cus, const Launch& L) {
    constexpr int UMAX = (NT > 1 || NCHUNK > 1) ? (TYPE == 2 && NT == 1 ? 2 : 1) : (TYPE == 2 ? 4 : 2);
    if (a.gated) {  // one gate row and one up row per lane and pass
        if constexpr (FUSEQ && NT == 1 && NCHUNK == 1) return launch_pairs_u<TYPE, LPR, NCHUNK, NT, FUSEQ, 2, DUMP, SPAN>(a, total_rows, num_cus, L);
        else return hipErrorInvalidValue;
    }
    int u = UMAX;
    const uint32_t want_waves = (uint32_t)num_cus * 8u;
    while (u > 1 && total_rows / ((64 / LPR) * u) < want_waves) u >>= 1;
    if (gemv_u_override() > 0) u = gemv_u_override() < UMAX ? gemv_u_override() : UMAX;
    if constexpr (UMAX >= 4)
        if (u >= 4) return launch_pairs_u<TYPE, LPR, NCHUNK, NT, FUSEQ, 4, DUMP, SPAN>(a, total_rows, num_cus, L);
    if constexpr (UMAX >= 2)
        if (u >= 2) return launch_pairs_u<TYPE, LPR, NCHUNK, NT, FUSEQ, 2, DUMP, SPAN>(a, total_rows, num_cus, L);
    return launch_pairs_u<TYPE, LPR, NCHUNK, NT, FUSEQ, 1, DUMP, SPAN>(a, total_rows, num_cus, L);
}

// FUSEQ callers have checked that the pair kernel applies (pairs_kernel_applies).
template <int TYPE, int NT, bool FUSEQ = false, bool DUMP = false, bool SPAN = false>
hipError_t dispatch(GemvArgs& a, int num_cus, const Launch& L) {
    const uint32_t total_rows = a.batch.row_end[a.batch.count - 1];
    if (total_rows == 0 || a.n == 0) return hipSuccess;
    const uint32_t nb = a.k >> 5;
    const uint32_t ppr = nb >> 1;
    bool aligned = (nb % 2u) == 0 && (FUSEQ || (reinterpret_cast<uintptr_t>(a.xq) % 16u) == 0);
    for (uint32_t i = 0; i < a.batch.count; i++) aligned = aligned && (reinterpret_cast<uintptr_t>(a.batch.w[i]) % 4u) == 0;
    if (aligned && ppr <= 128) {
        if (ppr <= 4) return launch_pairs<TYPE, 4, 1, NT, FUSEQ, DUMP, SPAN>(a, total_rows, num_cus, L);
        if (ppr <= 8) return launch_pairs<TYPE, 8, 1, NT, FUSEQ, DUMP, SPAN>(a, total_rows, num_cus, L);
        if (ppr <= 16) return launch_pairs<TYPE, 16, 1, NT, FUSEQ, DUMP, SPAN>(a, total_rows, num_cus, L);
        if (ppr <= 32) return launch_pairs<TYPE, 32, 1, NT, FUSEQ, DUMP, SPAN>(a, total_rows, num_cus, L);
        if (ppr <= 64) return launch_pairs<TYPE, 64, 1, NT, FUSEQ, DUMP, SPAN>(a, total_rows, num_cus, L);
        return launch_pairs<TYPE, 64, 2, NT, FUSEQ, DUMP, SPAN>(a, total_rows, num_cus, L);
    }
    if (FUSEQ || SPAN) return hipErrorInvalidValue;  // FUSEQ: unreachable, see pairs_kernel_applies; the timing hook: pair kernel only
    a.rows_per_wave = 1;
    dim3 grid(set_wave_ends(a), (a.n + NT - 1) / NT);
    return launch_kernel(L, kFamGemv, gemv_generic_kernel<TYPE, NT, DUMP>, dim3(grid), dim3(64), a);
}

}  // namespace

}  // namespace wick_rocm
