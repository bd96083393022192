// Batched prefill GEMM: raw GGUF Q4_0 / Q8_0 weight blocks x Q8_0-quantized
// activations -> f32, on the gfx950 int8 matrix cores.
//
// Arithmetic: gemm_q4_0_q8_0_neon / gemm_q8_0_q8_0_neon
// (wick/src/backend/simd.rs:696-925, 937-1019):
//   C[i,j] = sum_b f32(isum_{i,j,b}) * (f32(f16 d_w[i,b]) * xs[j,b]),  isum exact i32
// with one scale pair per 32-element block, so i32 accumulation cannot run across
// blocks: every v_mfma_i32_32x32x32_i8 covers exactly one block (K = 32) and its
// 32x32 i32 result is scaled into f32 accumulators on the vector ALU.
//
// Workgroup = 256 threads = 4 waves, tile = 128 weight rows x 128 tokens, each
// wave owns 64 x 64 (2 x 2 MFMA tiles).  One stage = 4 blocks (128 elements of K):
//   * weights: each thread reads one 36/68-byte block pair with dword-aligned wide
//     loads, unpacks nibbles to int8 and writes 16-byte operand rows to LDS;
//   * activations: copied global -> LDS directly (global_load_lds_dwordx4, asynchronous,
//     no registers); token scales through registers (f32 -> f16, lane order).
// LDS holds two stages.  The global loads of stage s+1 are issued before stage s is
// computed and written to the other LDS buffer after it, so there is one barrier
// per stage and the load latency hides behind the stage's ALU work.
//
// LDS operand layout: [block][khalf][row][16 bytes].  An MFMA lane supplies 16
// consecutive K-bytes of one operand row, lanes 0-31 the first half of the block
// and lanes 32-63 the second, so 32 consecutive lanes read 512 consecutive bytes:
// conflict-free.  For Q4_0 the low nibbles of a block ARE its first 16 elements and
// the high nibbles its last 16 (wick/src/quant.rs:82-88), so the two halves fall
// out of one and / shift each.  (The K order inside an MFMA is irrelevant as long
// as both operands use the same one.)
//
// Roles: tokens are the MFMA "A" (M) operand, weight rows the "B" (N) operand, so
// in the 32x32 result a lane holds ONE weight row (n = lane % 32) and 16 tokens
// (m = 8*(r/4) + 4*(lane/32) + r%4).  Its weight scale is one register per block;
// the 16 token scales are kept as f16 in LDS, stored in the order a lane consumes
// them (32 contiguous bytes per lane half, tile and block) and fed to the FMA as
// f16 operands (v_fma_mix_f32), which is exact because they ARE f16 values.
//
// Scaling is what bounds this kernel (vector ALU, not the matrix core), so it is
// cut to two FMAs per result:
//   * Q4_0 nibbles are stored as 16*(nibble-8) (the nibble moved to the top of the
//     byte, sign bit flipped: two ALU ops per four weights, no per-byte subtract);
//     the 1/16 is folded into the weight scale.
//   * The MFMA accumulates onto C = 0x4B400000 in every lane, i.e. the bit pattern
//     of 12582912.0f = 1.5 * 2^23.  Integer-adding v (|v| < 2^22) to that pattern
//     gives exactly the f32 12582912 + v, so the i32 -> f32 conversion is free.
//   * t = fma(D_as_f32, dw, -12582912*dw) = round(v * dw) exactly (single rounding;
//     12582912*dw is exact because dw has an 11-bit significand);
//     acc = fma(t, dx, acc).
#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

constexpr int BM = 128;       // weight rows per workgroup
constexpr int BN = 128;       // tokens per workgroup
constexpr int KB = 4;         // blocks per stage
constexpr int THREADS = 256;  // 4 waves: 2 (rows) x 2 (tokens)
constexpr uint32_t kBiasBits = 0x4B400000u;  // 12582912.0f
constexpr float kBias = 12582912.0f;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct GemmArgs {
    const uint8_t* w;
    const int8_t* xq;
    const float* xs;
    float* y;
    int32_t* dots;  // parity hook output (DUMP only)
    uint32_t m, n, k;
    uint32_t y_stride;
    uint32_t row_tiles, tok_tiles;
    int y_row_major;
    int accumulate;
};

// One stage of operands.  Row counts are padded (one 16-byte operand row per
// plane, two float2 per scale row) so that the stage WRITES, where neighbouring
// lanes hit different planes of the same row, spread over the LDS banks; reads
// walk consecutive rows of one plane.
struct Stage {
    uint4 wt[2][KB][BM + 2];    // [khalf][block][row]  int8 weights (Q4_0: x16)
    uint4 xt[KB][2][BN + 1];    // [block][khalf][token] int8 activations
    float2 dws[KB][BM + 2];     // {dw, -12582912*dw} per block and row (dw x 1/16 for Q4_0)
    float4 dxf[KB][BN / 32][2][4];  // [block][token tile][lane half][16 floats]: token scales in the order a lane consumes them
};

struct Smem {
    Stage st[2];
};

// 16*(nibble-8) for the four low / four high nibbles of each byte of q.
__device__ __forceinline__ uint32_t q4_lo_x16(uint32_t q) { return ((q << 4) & 0xf0f0f0f0u) ^ 0x80808080u; }
__device__ __forceinline__ uint32_t q4_hi_x16(uint32_t q) { return (q & 0xf0f0f0f0u) ^ 0x80808080u; }

template <int TYPE>
struct StageRegs {
    uint32_t w[PairTraits<TYPE>::DWORDS];
    float4 dx;
};

// Activation tiles go global -> LDS directly (global_load_lds_dwordx4): no staging
// registers, no unpack, no ds_write, and the copy runs asynchronously under the stage's
// ALU work.  One wave instruction fills 64 consecutive tokens of one [block][khalf]
// plane (lane l -> token l, 16 bytes each, contiguous 1 KB in LDS); a stage has
// 8 planes x 2 token halves = 16 such instructions, four per wave.
__device__ __forceinline__ void dma_activations(const GemmArgs& a, Stage& s, uint32_t tok0, uint32_t kb0) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // = block of the stage
#pragma unroll
    for (int half = 0; half < 2; half++) {
        const uint32_t tok = min(tok0 + 64u * half + lane, a.n - 1);
        const int8_t* src = a.xq + (size_t)tok * a.k + (size_t)(kb0 + wave) * 32;
#pragma unroll
        for (int kh = 0; kh < 2; kh++) {
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(src + 16 * kh),
                                             (void __attribute__((address_space(3)))*)&s.xt[wave][kh][64 * half], 16, 0, 0);
        }
    }
}

// Thread -> work of one stage:
//   weights      256 pairs   = 128 rows x 2 pairs             : row = t >> 1, pair = t & 1
//   activations  direct-to-LDS, see dma_activations
//   token scales 128 tokens x 4 blocks (one float4)           : threads 0..127, token = t
template <int TYPE>
__device__ __forceinline__ void load_stage(const GemmArgs& a, uint32_t row0, uint32_t tok0, uint32_t kb0,
                                           StageRegs<TYPE>& r) {
    using PT = PairTraits<TYPE>;
    const uint32_t t = threadIdx.x;
    const uint32_t nb = a.k >> 5;
    {
        const uint32_t row = min(row0 + (t >> 1), a.m - 1);
        const uint8_t* p = a.w + ((size_t)row * nb + kb0 + 2 * (t & 1u)) * (PT::BYTES / 2);
        load_pair<PT::DWORDS>(p, r.w);
    }
    if (t < BN && a.xs) {  // xs is null only for the parity hook, which never scales
        const uint32_t tok = min(tok0 + t, a.n - 1);
        r.dx = *reinterpret_cast<const float4*>(a.xs + (size_t)tok * nb + kb0);
    } else {
        r.dx = make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

template <int TYPE>
__device__ __forceinline__ void store_stage(Stage& s, const StageRegs<TYPE>& r) {
    using PT = PairTraits<TYPE>;
    const uint32_t t = threadIdx.x;
    {
        const uint32_t row = t >> 1;
        const uint32_t b0 = 2 * (t & 1u);
        uint32_t d0, d1, q0[PT::NQ], q1[PT::NQ];
        split_pair<TYPE>(r.w, d0, d1, q0, q1);
        const float scale = (TYPE == 2) ? 0.0625f : 1.0f;
        const float dw0 = f16_bits_to_f32(d0) * scale, dw1 = f16_bits_to_f32(d1) * scale;
        s.dws[b0][row] = make_float2(dw0, -kBias * dw0);
        s.dws[b0 + 1][row] = make_float2(dw1, -kBias * dw1);
        if constexpr (TYPE == 2) {
            s.wt[0][b0][row] = make_uint4(q4_lo_x16(q0[0]), q4_lo_x16(q0[1]), q4_lo_x16(q0[2]), q4_lo_x16(q0[3]));
            s.wt[1][b0][row] = make_uint4(q4_hi_x16(q0[0]), q4_hi_x16(q0[1]), q4_hi_x16(q0[2]), q4_hi_x16(q0[3]));
            s.wt[0][b0 + 1][row] = make_uint4(q4_lo_x16(q1[0]), q4_lo_x16(q1[1]), q4_lo_x16(q1[2]), q4_lo_x16(q1[3]));
            s.wt[1][b0 + 1][row] = make_uint4(q4_hi_x16(q1[0]), q4_hi_x16(q1[1]), q4_hi_x16(q1[2]), q4_hi_x16(q1[3]));
        } else {
            s.wt[0][b0][row] = make_uint4(q0[0], q0[1], q0[2], q0[3]);
            s.wt[1][b0][row] = make_uint4(q0[4], q0[5], q0[6], q0[7]);
            s.wt[0][b0 + 1][row] = make_uint4(q1[0], q1[1], q1[2], q1[3]);
            s.wt[1][b0 + 1][row] = make_uint4(q1[4], q1[5], q1[6], q1[7]);
        }
    }
    if (t < BN) {
        // token t of the tile sits at MFMA row t % 32 = 8*gq + 4*g + e -> lane half g, slot 4*gq + e
        const uint32_t tile = t >> 5, g = (t >> 2) & 1u, slot = ((t >> 3) & 3u) * 4 + (t & 3u);
        float* base = reinterpret_cast<float*>(&s.dxf[0][tile][g][0]) + slot;
        constexpr int kBlockStride = sizeof(s.dxf[0]) / sizeof(float);
        base[0 * kBlockStride] = r.dx.x;
        base[1 * kBlockStride] = r.dx.y;
        base[2 * kBlockStride] = r.dx.z;
        base[3 * kBlockStride] = r.dx.w;
    }
}

// Per-block operands of a wave's 2 x 2 MFMA tiles.
struct Mats {
    v4i av[2], bv[2];  // [token tile], [row tile]: 16 K-bytes of this lane's operand row
};
struct RowScales {
    float2 dw[2];  // {dw, -12582912*dw} of this lane's weight row, per row tile
};
struct TokScales {
    v4f dx[4];  // the 16 token scales of one token tile, in result-register order
};

// All LDS reads of the main loop are inline assembly on purpose.  While direct-to-LDS
// copies (of the NEXT stage, into the other buffer) are in flight, the compiler makes
// every LDS read it can see wait for all of them, which would put the whole global-memory
// latency at the start of each stage.  These reads touch only the current buffer; the
// copies are waited for explicitly before the barrier that ends the stage.  Data arrives
// in issue order; the *_ready functions are the matching waits (at most N later LDS reads
// still outstanding) and tie the registers, so nothing can use them earlier.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const void __attribute__((address_space(3)))*)p;
}
// A lane's four LDS read addresses (its rows of xt / wt / dws / dxf for the block being
// fetched).  Token tile, row tile and the pieces of a scale row are immediate offsets, so
// moving to the next block costs four additions instead of one per read.
struct LaneAddr {
    uint32_t xt, wt, dws, dxf;
};
constexpr int kOffXt = sizeof(uint4) * 2 * (BN + 1);         // one block of xt
constexpr int kOffWt = sizeof(uint4) * (BM + 2);             // one block of wt (within a khalf plane)
constexpr int kOffDws = sizeof(float2) * (BM + 2);           // one block of dws
constexpr int kOffDxf = sizeof(float4) * (BN / 32) * 2 * 4;  // one block of dxf
__device__ __forceinline__ void next_block(LaneAddr& la, bool advance) {
    la.xt += advance ? kOffXt : 0;
    la.wt += advance ? kOffWt : 0;
    la.dws += advance ? kOffDws : 0;
    la.dxf += advance ? kOffDxf : 0;
}
template <int OFF>
__device__ __forceinline__ void lds_read16(uint32_t addr, v4i& dst) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read16(uint32_t addr, v4f& dst) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read8(uint32_t addr, float2& dst) {
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ void load_mats(const LaneAddr& la, Mats& m) {
    lds_read16<0>(la.xt, m.av[0]);
    lds_read16<32 * 16>(la.xt, m.av[1]);
    lds_read16<0>(la.wt, m.bv[0]);
    lds_read16<32 * 16>(la.wt, m.bv[1]);
}
__device__ __forceinline__ void load_row_scales(const LaneAddr& la, RowScales& r) {
    lds_read8<0>(la.dws, r.dw[0]);
    lds_read8<32 * 8>(la.dws, r.dw[1]);
}
template <int TT>
__device__ __forceinline__ void load_tok_scales(const LaneAddr& la, TokScales& t) {
    lds_read16<TT * 128 + 0>(la.dxf, t.dx[0]);
    lds_read16<TT * 128 + 16>(la.dxf, t.dx[1]);
    lds_read16<TT * 128 + 32>(la.dxf, t.dx[2]);
    lds_read16<TT * 128 + 48>(la.dxf, t.dx[3]);
}
template <int N>
__device__ __forceinline__ void mats_ready(Mats& m, RowScales& r) {
    asm volatile("s_waitcnt lgkmcnt(%6)"
                 : "+v"(m.av[0]), "+v"(m.av[1]), "+v"(m.bv[0]), "+v"(m.bv[1]), "+v"(r.dw[0]), "+v"(r.dw[1])
                 : "n"(N)
                 : "memory");
}
template <int N>
__device__ __forceinline__ void tok_scales_ready(TokScales& t) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(t.dx[0]), "+v"(t.dx[1]), "+v"(t.dx[2]), "+v"(t.dx[3]) : "n"(N) : "memory");
}

// Scales one 32 x 32 MFMA result into the f32 accumulators: two full-rate v_fma_f32 per
// value (a v_fma_mix_f32 with an f16 scale operand would save registers but issues at half
// the rate, and this kernel is bound by exactly these instructions).
__device__ __forceinline__ void scale_tile(const v16i& d, const float2 dw, const TokScales& t, float (&acc)[16]) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const float v = __builtin_fmaf(__int_as_float(d[r]), dw.x, dw.y);
        acc[r] = __builtin_fmaf(v, t.dx[r >> 2][r & 3], acc[r]);
    }
}

// Parity hook: the raw i32 block dots of one MFMA result.
template <int TYPE>
__device__ __forceinline__ void dump_tile(const GemmArgs& a, const v16i& d, uint32_t row, uint32_t tok_base, uint32_t g, uint32_t nb,
                                          uint32_t block) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const uint32_t tok = tok_base + 8 * (r >> 2) + 4 * g + (r & 3);
        if (row < a.m && tok < a.n) {
            int v = d[r] - (int)kBiasBits;
            if (TYPE == 2) v >>= 4;  // weights were stored x16; exact
            a.dots[((size_t)tok * a.m + row) * nb + block] = v;
        }
    }
}

// Workgroup -> tile, XCD- and L2-aware.  Hardware hands consecutive workgroup ids to
// the 8 XCDs round-robin, so ids with equal (id % 8) share an L2 (4 MB).  Each XCD
// takes a contiguous run of a tile list that walks the output in 8 x 8 "supertiles"
// (8 row tiles x 8 token tiles, row-major inside): the ~64 workgroups resident on an
// XCD at one time then touch 8 weight panels + 8 activation panels (~3.3 MB at
// k = 2048), which fit its L2, instead of a 4 x 16 strip whose activation panels
// alone overflow it.
__device__ __forceinline__ void tile_of_block(uint32_t bid, uint32_t row_tiles, uint32_t tok_tiles, uint32_t& row_tile,
                                              uint32_t& tok_tile, bool& valid) {
    constexpr uint32_t S = 8;
    const uint32_t tiles = row_tiles * tok_tiles;
    const uint32_t per_xcd = (tiles + 7u) / 8u;
    const uint32_t t = (bid & 7u) * per_xcd + (bid >> 3);
    valid = (bid >> 3) < per_xcd && t < tiles;
    const uint32_t tt = valid ? t : 0;
    const uint32_t sr_count = (row_tiles + S - 1) / S, sc_count = (tok_tiles + S - 1) / S;
    const uint32_t sr = min(tt / (S * tok_tiles), sr_count - 1);  // supertile row (all but the last hold S*tok_tiles tiles)
    const uint32_t t1 = tt - sr * S * tok_tiles;
    const uint32_t h = min(S, row_tiles - sr * S);
    const uint32_t sc = min(t1 / (h * S), sc_count - 1);
    const uint32_t t2 = t1 - sc * h * S;
    const uint32_t w = min(S, tok_tiles - sc * S);
    row_tile = sr * S + t2 / w;
    tok_tile = sc * S + t2 % w;
}

template <int TYPE, bool DUMP>
__global__ __launch_bounds__(THREADS, 2) void gemm_mfma_kernel(GemmArgs a) {
    __shared__ Smem sm;
    uint32_t row_tile, tok_tile;
    bool valid_tile;
    tile_of_block(blockIdx.x, a.row_tiles, a.tok_tiles, row_tile, tok_tile, valid_tile);
    if (!valid_tile) return;  // whole workgroup leaves together
    const uint32_t row0 = row_tile * BM;
    const uint32_t tok0 = tok_tile * BN;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t l32 = lane & 31u;
    const uint32_t g = lane >> 5;             // which 16-byte half of the block this lane feeds
    const uint32_t wrow0 = (wave >> 1) * 64;  // wave's rows within the tile
    const uint32_t wtok0 = (wave & 1u) * 64;
    const uint32_t nb = a.k >> 5;
    const uint32_t stages = nb / KB;

    float acc[2][2][16];
#pragma unroll
    for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[tt][rt][r] = 0.0f;

    v16i cbias;
#pragma unroll
    for (int r = 0; r < 16; r++) cbias[r] = (int)kBiasBits;
    asm volatile("" : "+v"(cbias));  // keep it in registers: left alone, the compiler rebuilds all 16 before every MFMA group

    StageRegs<TYPE> regs;
    dma_activations(a, sm.st[0], tok0, 0);
    load_stage<TYPE>(a, row0, tok0, 0, regs);
    store_stage<TYPE>(sm.st[0], regs);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's direct-to-LDS copies have landed
    __syncthreads();

    for (uint32_t st = 0; st < stages; st++) {
        const Stage& s = sm.st[st & 1u];
        if (st + 1 < stages) {
            // the other LDS stage was last read in stage st-1 and every wave has passed the
            // barrier that ended it, so it can be refilled from here on
            dma_activations(a, sm.st[(st + 1) & 1u], tok0, (st + 1) * KB);
            load_stage<TYPE>(a, row0, tok0, (st + 1) * KB, regs);
        }

        // 16 MFMA tiles per stage, software-pipelined at MFMA granularity: the matrix core
        // works on tile i+1 while the vector ALU scales tile i (two result buffers), and the
        // operands of block b+1 are fetched from LDS into registers as soon as block b has
        // released them, so neither LDS nor MFMA latency sits in the wave's dependency chain.
        // The scheduling barriers pin that order; the block loop stays rolled (unrolled, the
        // compiler issues all 16 MFMAs of the stage up front and spills their results).
        // Tile order within a block: (token tile, row tile) = (0,0) (0,1) (1,0) (1,1).
        Mats mt;
        RowScales rs, rs_next;
        TokScales ts0, ts1;
        LaneAddr la;  // block 0 of this stage's buffer
        la.xt = lds_addr(&s.xt[0][g][wtok0 + l32]);
        la.wt = lds_addr(&s.wt[g][0][wrow0 + l32]);
        la.dws = lds_addr(&s.dws[0][wrow0 + l32]);
        la.dxf = lds_addr(&s.dxf[0][wtok0 >> 5][g][0]);
        load_mats(la, mt);
        load_row_scales(la, rs);
        load_tok_scales<0>(la, ts0);
        load_tok_scales<1>(la, ts1);
        mats_ready<8>(mt, rs);
        v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.av[0], mt.bv[0], cbias, 0, 0, 0), d1;
        tok_scales_ready<4>(ts0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
        for (int b = 0; b < KB; b++) {
            next_block(la, b + 1 < KB);  // last iteration: harmless re-read of its own block
            const uint32_t row = row0 + wrow0 + l32, tokb = tok0 + wtok0, blk = st * KB + b;
            d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.av[0], mt.bv[1], cbias, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (DUMP) dump_tile<TYPE>(a, d0, row, tokb, g, nb, blk); else scale_tile(d0, rs.dw[0], ts0, acc[0][0]);
            __builtin_amdgcn_sched_barrier(0);
            d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.av[1], mt.bv[0], cbias, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (DUMP) dump_tile<TYPE>(a, d1, row + 32, tokb, g, nb, blk); else scale_tile(d1, rs.dw[1], ts0, acc[0][1]);
            __builtin_amdgcn_sched_barrier(0);
            d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.av[1], mt.bv[1], cbias, 0, 0, 0);
            // block b needs its matrices and the scales of token tile 0 no longer: fetch block b+1's
            load_tok_scales<0>(la, ts0);    // 4 reads (ts1 of this block arrived long ago)
            load_mats(la, mt);              // 4 reads
            load_row_scales(la, rs_next);   // 2 reads
            tok_scales_ready<10>(ts1);  // issued at the end of the previous iteration, before the ten reads above
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (DUMP) dump_tile<TYPE>(a, d0, row, tokb + 32, g, nb, blk); else scale_tile(d0, rs.dw[0], ts1, acc[1][0]);
            __builtin_amdgcn_sched_barrier(0);
            mats_ready<0>(mt, rs_next);
            tok_scales_ready<0>(ts0);
            d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.av[0], mt.bv[0], cbias, 0, 0, 0);  // first tile of block b+1
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (DUMP) dump_tile<TYPE>(a, d1, row + 32, tokb + 32, g, nb, blk); else scale_tile(d1, rs.dw[1], ts1, acc[1][1]);
            __builtin_amdgcn_sched_barrier(0);
            load_tok_scales<1>(la, ts1);    // waited for by the next iteration's lgkmcnt(0)
            rs = rs_next;
        }
        tok_scales_ready<0>(ts1);  // nothing of this stage's buffer is read past this point

        // The other buffer was last read in stage st-1; every wave has passed the barrier
        // that ended that stage, so it is free to be refilled now.
        if (st + 1 < stages) store_stage<TYPE>(sm.st[(st + 1) & 1u], regs);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS copies of the next stage have landed
        __syncthreads();
    }

    if constexpr (!DUMP) {
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const uint32_t row = row0 + wrow0 + rt * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const uint32_t tok = tok0 + wtok0 + tt * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                    if (row < a.m && tok < a.n) {
                        float* dst = a.y_row_major ? a.y + (size_t)row * a.y_stride + tok : a.y + (size_t)tok * a.y_stride + row;
                        *dst = a.accumulate ? *dst + acc[tt][rt][r] : acc[tt][rt][r];
                    }
                }
            }
    }
}

template <bool DUMP>
hipError_t launch(int type, GemmArgs& a, const Launch& L) {
    if (a.m == 0 || a.n == 0) return hipSuccess;
    a.row_tiles = (a.m + BM - 1) / BM;
    a.tok_tiles = (a.n + BN - 1) / BN;
    const uint32_t tiles = a.row_tiles * a.tok_tiles;
    const uint32_t blocks = ((tiles + 7u) / 8u) * 8u;  // every XCD gets the same number of slots
    if (type == kTypeQ4_0)
        return launch_kernel(L, kFamGemm, gemm_mfma_kernel<2, DUMP>, dim3(blocks), dim3(THREADS), a);
    return launch_kernel(L, kFamGemm, gemm_mfma_kernel<8, DUMP>, dim3(blocks), dim3(THREADS), a);
}

}  // namespace

hipError_t launch_gemm_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                            const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                            int accumulate, const Launch& L) {
    GemmArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = d_scales, a.y = d_y, a.dots = nullptr;
    a.m = m, a.n = n, a.k = k, a.y_stride = y_stride;
    a.y_row_major = (y_layout == 1);
    a.accumulate = accumulate;
    return launch<false>(type, a, L);
}

// Parity hook through the matrix-core path: the same loads, unpack, LDS layout and
// MFMA as the GEMM, writing the raw i32 block dots instead of scaling them.
hipError_t launch_block_dots_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n,
                                  int32_t* d_out, const Launch& L) {
    GemmArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = nullptr, a.y = nullptr, a.dots = d_out;
    a.m = m, a.n = n, a.k = k, a.y_stride = 0;
    return launch<true>(type, a, L);
}

}  // namespace wick_rocm
