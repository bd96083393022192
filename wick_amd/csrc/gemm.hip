// Batched prefill GEMM: Q4_0 / Q8_0 weights x Q8_0-quantized activations -> f32, on the gfx950 int8 matrix cores.
//
// Arithmetic: gemm_q4_0_q8_0_neon / gemm_q8_0_q8_0_neon
// (wick/src/backend/simd.rs:696-925, 937-1019):
//   C[i,j] = sum_b f32(isum_{i,j,b}) * (f32(f16 d_w[i,b]) * xs[j,b]),  isum exact i32
// with one scale pair per 32-element block, so i32 accumulation cannot run across
// blocks: every MFMA covers exactly one block (K = 32) and its i32 result is scaled
// into f32 accumulators on the vector ALU.
//
// Workgroup = 512 threads = 8 waves, tile = 128 weight rows x 128 tokens, each wave
// owns 64 rows x 32 tokens.  Two block loops exist for that wave tile:
//   * gemm_mfma32_kernel (plain projections, the default): 2 x v_mfma_i32_32x32x32_i8 per block, one 16-register
//     result buffer, 16-register bias tuple, 16 token scales and 2 row-scale pairs per block -- 125 VGPRs
//     (gemm_narrow32_kernel is the same loop with one MFMA per block on the 128 x 64 tile);
//   * gemm_mfma_kernel (the gated feed-forward launch, and plain projections on request): 4 x 2 tiles of
//     v_mfma_i32_16x16x32_i8, four 4-register result buffers, 4-register bias -- 109 VGPRs.
// Both stay under 128 VGPRs so that FOUR waves share a SIMD, which matters more than anything else here: a wave can
// issue a vector-ALU instruction only every ~4.7 cycles while a SIMD retires one every ~2.2, and the kernel is bound by
// the two scaling FMAs per result plus the matrix instructions, which a SIMD does not overlap with them.  The small
// shape runs the matrix unit at a third of the large one's rate (1.7 vs 4.9 POP/s measured), which is what the
// 32x32x32 loop recovers part of (3 - 8 % of a launch).
// One stage = 4 blocks (128 elements of K).  Both operands are copied global -> LDS directly
// (global_load_lds_dwordx4: asynchronous, no registers, 1 KB per wave instruction):
//   * weights from the GEMM's own copy of the matrix, made from the raw GGUF blocks when the
//     weight is uploaded (gemm_pack_kernel, layout at StageT): int8 operand rows and
//     {scale, -bias * scale} pairs already in the order a stage of LDS holds them, so the main
//     loop neither unpacks nibbles nor converts scales nor stores to LDS;
//   * activations from the token-major Q8_0 quants; token scales through registers (they are
//     stored block-major).
// LDS holds two stages (76 KB, two workgroups per CU).  The copies of stage s+1 are issued
// before stage s is computed, so there is one barrier per stage and the load latency hides
// behind the stage's ALU work.
//
// LDS operand layout: weights [granule of 32 rows][khalf][block][row][16 bytes], activations
// [token][8 x 16 bytes, swizzled].  An MFMA lane supplies 8 consecutive K-bytes of operand row
// lane % 16, K-quarter lane / 16, so 32 consecutive lanes read 256 consecutive bytes (the two
// 8-byte halves of 16 rows): conflict-free.  For Q4_0 the low nibbles of a block ARE its first
// 16 elements and the high nibbles its last 16 (wick/src/quant.rs:82-88): the two khalf planes.
// (The K order inside an MFMA is irrelevant as long as both operands use the same one.)
//
// Roles: tokens are the MFMA "A" (M) operand, weight rows the "B" (N) operand, so in the
// 16x16 result a lane holds ONE weight row (n = lane % 16) and 4 consecutive tokens
// (m = 4*(lane/16) + r).  Its weight scale is one register pair per block and row tile;
// the token scales sit in LDS as f32, token-major, and a lane reads its four with one
// 16-byte read (a broadcast within each group of 16 lanes).
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
//     acc = fma(t, dx, acc), both plain v_fma_f32 (v_fma_mix_f32 with an f16 scale
//     operand would save registers but issues at half the rate).
#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

constexpr int BM = 128;       // weight rows per workgroup
constexpr int BN = 128;       // tokens per workgroup
constexpr int BN_NARROW = 64;  // ... of the narrow kernel (n <= 64)
constexpr int KB = 4;         // blocks per stage
constexpr int THREADS = 512;  // 8 waves: 2 (rows) x 4 (tokens)
constexpr int TT = 2;          // 16-token MFMA tiles per wave
constexpr int RT = 4;          // 16-row MFMA tiles per wave
constexpr uint32_t kBiasBits = 0x4B400000u;  // 12582912.0f
constexpr float kBias = 12582912.0f;

typedef int v4i __attribute__((ext_vector_type(4)));
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
    // Up to two more weights that share the activations (Q / K / V, gate / up): their row tiles follow the first
    // weight's in the launch's tile list.  tile_start[i]: first row tile of weight i + 1 (UINT32_MAX: absent).
    const uint8_t* w_more[2];
    float* y_more[2];
    uint32_t m_more[2];
    uint32_t tile_start[2];
    // Gated feed-forward launch (GATED kernels only): w = gate, w_up = up, the output is the Q8_0-quantized silu(gate) * up.
    const uint8_t* w_up;
    int8_t* q_out;   // [n][m]
    float* s_out;    // [n][m / 32]
    // K split of a narrow launch with few tiles: workgroup (tile, split) walks its share of the stages and leaves its sums
    // in partial[split][n][m]; gemm_splitk_reduce_kernel adds the shares up in a fixed order.  ksplit <= 1: off.
    uint32_t ksplit;
    float* partial;
};

// Makes `a` describe the weight that owns row tile `row_tile` and rebases the tile index to that weight.
__device__ __forceinline__ void select_weight(GemmArgs& a, uint32_t& row_tile) {
    const bool second = row_tile >= a.tile_start[0], third = row_tile >= a.tile_start[1];
    if (second) {
        a.w = third ? a.w_more[1] : a.w_more[0];
        a.y = third ? a.y_more[1] : a.y_more[0];
        a.m = third ? a.m_more[1] : a.m_more[0];
        row_tile -= third ? a.tile_start[1] : a.tile_start[0];
    }
}

// The weights a GEMM launch reads are not the raw GGUF blocks but a copy laid out for this kernel, made once when the
// weight is uploaded (gemm_pack_kernel): rows in granules of 32, and per (granule, stage of 4 blocks) one 5120-byte slab
//   [khalf 2][block 4][row 32][16 bytes]   int8 operand rows (Q4_0: 16 * (nibble - 8)), 4096 bytes
//   [block 4][row 32] {dw, -12582912 * dw}  scale pairs (dw x 1/16 for Q4_0), 1024 bytes
// laid out [pair of granules][stage][granule of the pair]: the 64 rows x 128 K-elements a wave works on are 10 KB in one piece.  A slab is exactly what a stage of LDS holds for those 32 rows, so the weights go
// global -> LDS directly like the activations: five 1 KB copies per granule, no staging registers, no unpack and no LDS
// stores in the main loop, fully coalesced.  A tile is four granules (a gated tile: two of the gate weight and the same
// two of the up weight).  1.25 bytes per weight instead of 0.5625 (Q4_0) / 1.0625 (Q8_0).
constexpr int GR = 32;                              // rows per granule
constexpr int kSlabWt = 2 * KB * GR * 16;           // 4096
constexpr int kSlabDws = KB * GR * 8;               // 1024
constexpr int kSlab = kSlabWt + kSlabDws;           // 5120
constexpr int kSlabChunks = kSlab / 1024;           // 5 direct-to-LDS copies of 1 KB

// One stage of operands.
template <int NTOK>  // tokens per workgroup tile: BN, or BN_NARROW for the narrow kernel
struct StageT {
    uint4 wt[BM / GR][2][KB][GR];  // [granule][khalf][block][row]  int8 weights: the slabs' first 4 KB
    uint4 xt[NTOK][2 * KB];        // [token][16-byte K-chunk, swizzled] int8 activations, see dma_activations
    float2 dws[BM / GR][KB][GR];   // {dw, -12582912*dw} per granule, block and row: the slabs' last 1 KB
    float dxf[KB][NTOK];           // token scales
};
using Stage = StageT<BN>;

template <int NTOK>
struct SmemT {
    StageT<NTOK> st[2];
};
using Smem = SmemT<BN>;

// 16*(nibble-8) for the four low / four high nibbles of each byte of q.
__device__ __forceinline__ uint32_t q4_lo_x16(uint32_t q) { return ((q << 4) & 0xf0f0f0f0u) ^ 0x80808080u; }
__device__ __forceinline__ uint32_t q4_hi_x16(uint32_t q) { return (q & 0xf0f0f0f0u) ^ 0x80808080u; }

struct StageRegs {
    float4 dx;
};

// Raw blocks -> slabs.  One workgroup per (granule, stage): thread (row = t % 32, block = t / 32).  Rows past the end of
// the matrix become zero rows with zero scales.  For Q4_0 the low nibbles of a block ARE its first 16 elements and the high
// nibbles its last 16 (wick/src/quant.rs:82-88): the two khalf planes.
template <int TYPE>
__global__ __launch_bounds__(GR * KB) void gemm_pack_kernel(const uint8_t* __restrict__ raw, uint32_t m, uint32_t nb, uint8_t* __restrict__ packed) {
    constexpr int BB = TYPE == 2 ? 18 : 34;
    const uint32_t stages = nb / KB, granule = blockIdx.x / stages, stage = blockIdx.x % stages;
    const uint32_t within = threadIdx.x % GR, b = threadIdx.x / GR, row = granule * GR + within;
    uint32_t lo[4] = {0, 0, 0, 0}, hi[4] = {0, 0, 0, 0};
    float dw = 0.0f;
    if (row < m) {
        const uint16_t* blk = reinterpret_cast<const uint16_t*>(raw + ((size_t)row * nb + stage * KB + b) * BB);  // blocks are 2-byte aligned
        dw = f16_bits_to_f32(blk[0]) * (TYPE == 2 ? 0.0625f : 1.0f);
        uint32_t q[8];
#pragma unroll
        for (int i = 0; i < (BB - 2) / 4; i++) q[i] = (uint32_t)blk[1 + 2 * i] | ((uint32_t)blk[2 + 2 * i] << 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = TYPE == 2 ? q4_lo_x16(q[i]) : q[i];
            hi[i] = TYPE == 2 ? q4_hi_x16(q[i]) : q[4 + i];
        }
    }
    uint8_t* slab = packed + (((size_t)(granule >> 1) * stages + stage) * 2 + (granule & 1u)) * kSlab;
    reinterpret_cast<uint4*>(slab)[(0 * KB + b) * GR + within] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    reinterpret_cast<uint4*>(slab)[(1 * KB + b) * GR + within] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    reinterpret_cast<float2*>(slab + kSlabWt)[b * GR + within] = make_float2(dw, -kBias * dw);
}

// Activation tiles go global -> LDS directly (global_load_lds_dwordx4): no staging
// registers, no unpack, no ds_write, and the copy runs asynchronously under the stage's
// ALU work.  A token's 128 K-bytes of the stage are exactly one cache line, so one wave
// instruction fetches 8 tokens x 8 16-byte chunks = 8 whole lines (lane l -> token l / 8,
// position l % 8; the address unit works per line touched, and a chunk-major split would
// touch 64 lines per instruction).  Direct-to-LDS data lands lane-contiguous, i.e. as
// [token][8 positions] rows of 128 bytes, which an MFMA operand read (16 tokens, same
// chunk) would hit with an 8-way bank conflict.  So position p of token t holds K-chunk
// p ^ ((t >> 1) & 7): the lane picks its GLOBAL chunk accordingly, and 16 consecutive
// tokens reading one chunk then spread over all banks.  16 instructions per stage, four
// per loader wave (dma_stage).
__device__ __forceinline__ uint32_t xt_swizzle(uint32_t token_in_tile) { return (token_in_tile >> 1) & 7u; }
// A thread's global read positions of the stage to fetch next.  Set up once per tile; every fetch moves them one stage
// (128 K-elements) on, one 64-bit add each, instead of rebuilding row / token / block addresses per stage.
// Only the first kLoaderWaves waves of a workgroup issue the stage's global -> LDS copies (and fetch the token scales): the
// address unit takes a copy instruction every 16 cycles, so 36 of them per stage and workgroup queue up, and a wave waiting in
// that queue issues nothing else.  The later waves of a workgroup are the ones that lag in the block loop (the SIMD favours the
// older wave), so they get no copies to issue at all and the earlier ones, which would otherwise idle at the stage barrier, all.
constexpr int kLoaderWaves = 4;
template <int NTOK>
struct StagePtrs {
    const int8_t* x[NTOK / 8 / kLoaderWaves];  // this lane's 16-byte activation chunks (direct-to-LDS copies)
    const uint8_t* wc;                          // this lane's 16 bytes of the first kilobyte of granule `wave`'s slab
    const uint8_t* dx;                          // threads 0 .. NTOK - 1: a token's four scales
};
// Where chunk c (0 .. 19) of a tile's stage lands: granule c / 5, its weights' kilobyte c % 5 or (the fifth) its scale pairs.
template <int NTOK>
__device__ __forceinline__ void* chunk_dst(StageT<NTOK>& s, uint32_t c) {
    const uint32_t g = c / kSlabChunks, part = c % kSlabChunks;
    return part < 4 ? static_cast<void*>(reinterpret_cast<uint8_t*>(&s.wt[g][0][0][0]) + 1024u * part) : static_cast<void*>(&s.dws[g][0][0]);
}
template <int NTOK>
__device__ __forceinline__ void dma_stage(StagePtrs<NTOK>& p, StageT<NTOK>& s) {
    constexpr int PER_WAVE = NTOK / 8 / kLoaderWaves;  // activation instructions per loader wave and stage
    static_assert(BM / GR == kLoaderWaves, "one granule's slab per loader wave");
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (wave >= (uint32_t)kLoaderWaves) return;  // uniform per wave
#pragma unroll
    for (int j = 0; j < PER_WAVE; j++) {
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)p.x[j],
                                         (void __attribute__((address_space(3)))*)&s.xt[8u * (PER_WAVE * wave + j)][0], 16, 0, 0);
        p.x[j] += KB * 32;
    }
#pragma unroll
    for (int part = 0; part < kSlabChunks; part++)
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(p.wc + 1024 * part),
                                         (void __attribute__((address_space(3)))*)chunk_dst(s, kSlabChunks * wave + part), 16, 0, 0);
    p.wc += 2 * kSlab;
}

template <int NTOK, bool GATED = false>
__device__ __forceinline__ void init_stage_ptrs(const GemmArgs& a, uint32_t row_tile, uint32_t tok0, uint32_t kb0, StagePtrs<NTOK>& p) {
    constexpr int PER_WAVE = NTOK / 8 / kLoaderWaves;
    const uint32_t t = threadIdx.x, lane = t & 63u;
    const uint32_t wave = min((uint32_t)__builtin_amdgcn_readfirstlane((int)(t >> 6)), (uint32_t)kLoaderWaves - 1u);  // (later waves: unused values)
    const uint32_t nb = a.k >> 5, stages = nb / KB;
#pragma unroll
    for (int j = 0; j < PER_WAVE; j++) {
        const uint32_t tt = 8u * (PER_WAVE * wave + j) + (lane >> 3);  // token within the tile
        const uint32_t chunk = (lane & 7u) ^ xt_swizzle(tt);
        const uint32_t tok = min(tok0 + tt, a.n - 1);
        p.x[j] = a.xq + (size_t)tok * a.k + (size_t)kb0 * 32 + 16u * chunk;
    }
    const uint32_t granules = (a.m + GR - 1) / GR;
    {
        const uint32_t g = wave;
        // the tile's granule g: rows 32 g .. of a plain tile; of a gated tile (64 output rows) gate, up, gate, up of its two
        uint32_t granule = GATED ? 2u * row_tile + (g >> 1) : (BM / GR) * row_tile + g;
        const uint8_t* w = GATED && (g & 1u) ? a.w_up : a.w;
        granule = min(granule, granules - 1u);  // past the end of the matrix: any rows, their results are not stored
        p.wc = w + (((size_t)(granule >> 1) * stages + kb0 / KB) * 2 + (granule & 1u)) * kSlab + 16u * lane;
    }
    p.dx = nullptr;
    if (t < NTOK && a.xs) {  // xs is null only for the parity hook, which never scales
        const uint32_t tok = min(tok0 + t, a.n - 1);
        p.dx = reinterpret_cast<const uint8_t*>(a.xs + (size_t)tok * nb + kb0);
    }
}

// Thread -> rest of a stage: one float4 (4 blocks) of token scales per token, threads 0 .. NTOK - 1 (loader waves), through registers
// (they are stored block-major).
template <int NTOK>
__device__ __forceinline__ void load_stage(StagePtrs<NTOK>& p, StageRegs& r) {
    if (p.dx) {
        r.dx = *reinterpret_cast<const float4*>(p.dx);
        p.dx += KB * sizeof(float);
    } else {
        r.dx = make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

template <int NTOK>
__device__ __forceinline__ void store_stage(StageT<NTOK>& s, const StageRegs& r) {
    const uint32_t t = threadIdx.x;
    if (t < NTOK) {
        const uint32_t u = t;
        s.dxf[0][u] = r.dx.x;
        s.dxf[1][u] = r.dx.y;
        s.dxf[2][u] = r.dx.z;
        s.dxf[3][u] = r.dx.w;
    }
}

// Per-block operands of a wave's TT x RT MFMA tiles: 8 K-bytes of this lane's operand row.
struct Mats {
    long av[TT], bv[RT];
};
struct Scales {
    float2 dw[RT];  // {dw, -12582912*dw} of this lane's weight row, per row tile
    v4f dx[TT];     // scales of this lane's four tokens, per token tile
};

// All LDS reads of the main loop are inline assembly on purpose.  While direct-to-LDS
// copies (of the NEXT stage, into the other buffer) are in flight, the compiler makes
// every LDS read it can see wait for all of them, which would put the whole global-memory
// latency at the start of each stage.  These reads touch only the current buffer; the
// copies are waited for explicitly before the barrier that ends the stage.  Data arrives
// in issue order; lds_wait<N> is the matching wait (at most N later LDS reads still
// outstanding) and ties the registers, so nothing can use them earlier.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const void __attribute__((address_space(3)))*)p;
}
// A lane's four LDS read addresses (its rows of xt / wt / dws and its tokens of dxf for the
// block being fetched).  Tile indices are immediate offsets; moving to the next block costs
// three additions and, for the swizzled activation tile, one xor + shift-add:
// xt = xbase + ((block ^ xsh) << 5).
struct LaneAddr {
    uint32_t xt, wt, dws, dxf;
    uint32_t xbase, xsh;
};
constexpr int kOffWt = sizeof(uint4) * GR;            // one block of wt (within a granule's khalf plane)
constexpr int kOffDws = sizeof(float2) * GR;          // one block of dws (within a granule)
constexpr int kOffDxf = sizeof(float) * BN;           // one block of dxf
__device__ __forceinline__ void next_block(LaneAddr& la, uint32_t block, bool advance) {
    la.xt = la.xbase + (((advance ? block + 1 : block) ^ la.xsh) << 5);
    la.wt += advance ? kOffWt : 0;
    la.dws += advance ? kOffDws : 0;
    la.dxf += advance ? kOffDxf : 0;
}
template <int OFF>
__device__ __forceinline__ void lds_read16(uint32_t addr, v4f& dst) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read8(uint32_t addr, long& dst) {
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read8(uint32_t addr, float2& dst) {
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ void load_mats(const LaneAddr& la, Mats& m) {  // TT + RT = 6 reads
    lds_read8<0 * 16 * 128>(la.xt, m.av[0]);  // 16 tokens further: same swizzle
    lds_read8<1 * 16 * 128>(la.xt, m.av[1]);
    lds_read8<0>(la.wt, m.bv[0]);  // row tiles 0, 1: the two halves of the wave's first granule; 2, 3: of its second
    lds_read8<256>(la.wt, m.bv[1]);
    lds_read8<kSlabWt>(la.wt, m.bv[2]);
    lds_read8<kSlabWt + 256>(la.wt, m.bv[3]);
}
__device__ __forceinline__ void load_row_scales(const LaneAddr& la, Scales& s) {  // RT = 4 reads
    lds_read8<0>(la.dws, s.dw[0]);
    lds_read8<128>(la.dws, s.dw[1]);
    lds_read8<kSlabDws>(la.dws, s.dw[2]);
    lds_read8<kSlabDws + 128>(la.dws, s.dw[3]);
}
template <int T>
__device__ __forceinline__ void load_tok_scales(const LaneAddr& la, Scales& s) {  // 1 read
    lds_read16<T * 64>(la.dxf, s.dx[T]);
}
template <int N>
__device__ __forceinline__ void lds_wait(Mats& m) {
    asm volatile("s_waitcnt lgkmcnt(%6)"
                 : "+v"(m.av[0]), "+v"(m.av[1]), "+v"(m.bv[0]), "+v"(m.bv[1]), "+v"(m.bv[2]), "+v"(m.bv[3])
                 : "n"(N)
                 : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait(Scales& s) {
    asm volatile("s_waitcnt lgkmcnt(%6)"
                 : "+v"(s.dw[0]), "+v"(s.dw[1]), "+v"(s.dw[2]), "+v"(s.dw[3]), "+v"(s.dx[0]), "+v"(s.dx[1])
                 : "n"(N)
                 : "memory");
}

// Scales one 16 x 16 MFMA result (4 values per lane) into the f32 accumulators: two
// full-rate v_fma_f32 per value.
__device__ __forceinline__ void scale_tile(const v4i& d, const float2 dw, const v4f& dx, float (&acc)[4]) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const float v = __builtin_fmaf(__int_as_float(d[r]), dw.x, dw.y);
        acc[r] = __builtin_fmaf(v, dx[r], acc[r]);
    }
}

// Parity hook: the raw i32 block dots of one MFMA result.  row = this lane's weight row,
// tok = the first of its four tokens.
template <int TYPE>
__device__ __forceinline__ void dump_tile(const GemmArgs& a, const v4i& d, uint32_t row, uint32_t tok, uint32_t nb, uint32_t block) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (row < a.m && tok + r < a.n) {
            int v = d[r] - (int)kBiasBits;
            if (TYPE == 2) v >>= 4;  // weights were stored x16; exact
            a.dots[((size_t)(tok + r) * a.m + row) * nb + block] = v;
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

// Results of a wave's MFMA tiles into the output (or into a K share's partial sums): element (tt, rt, r) of the wave tile is
// (row + RSTEP rt, tok + TSTEP tt + r), `row` / `tok` being this lane's first row and token (16 / 16 for the 16x16 MFMA
// layout: a lane holds 4 consecutive tokens of one row per tile; 8 / 32 for the 32x32 layout: 4 groups of 4 tokens, 8 apart).  One instantiation per output layout
// so that the inner index is an immediate offset of the store; CHECK = false for wave tiles that lie inside the matrix (no
// predicates at all), ACC adds onto what is there.  The mode is uniform per launch, the bounds are uniform per wave: the
// callers branch once, not per element.
template <int NTT, int NRT, int TSTEP, int RSTEP, bool ROW_MAJOR, bool CHECK, bool ACC, typename F>
__device__ __forceinline__ void store_results(float* __restrict__ base, size_t stride, uint32_t row, uint32_t tok, uint32_t m, uint32_t n,
                                              F&& value) {
    if constexpr (ROW_MAJOR) {
#pragma unroll
        for (int rt = 0; rt < NRT; rt++) {
            float* q = base + (size_t)(row + RSTEP * rt) * stride + tok;
#pragma unroll
            for (int tt = 0; tt < NTT; tt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (CHECK && !(row + RSTEP * rt < m && tok + TSTEP * tt + r < n)) continue;
                    const float v = value(tt, rt, r);
                    q[TSTEP * tt + r] = ACC ? q[TSTEP * tt + r] + v : v;
                }
        }
    } else {
#pragma unroll
        for (int tt = 0; tt < NTT; tt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float* q = base + (size_t)(tok + TSTEP * tt + r) * stride + row;
#pragma unroll
                for (int rt = 0; rt < NRT; rt++) {
                    if (CHECK && !(row + RSTEP * rt < m && tok + TSTEP * tt + r < n)) continue;
                    const float v = value(tt, rt, r);
                    q[RSTEP * rt] = ACC ? q[RSTEP * rt] + v : v;
                }
            }
    }
}
// The launch's output mode picked once per wave: a K share's partial sums [share][n][m], or y in either layout, plain or accumulating.
template <int NTT, int NRT, int TSTEP = 16, int RSTEP = 16, typename F>
__device__ __forceinline__ void store_wave_tile(const GemmArgs& a, uint32_t ksplit, uint32_t split, uint32_t row, uint32_t tok, F&& value) {
    // the wave tile's corner is the same for every lane: keep the test (and the branches on it) scalar
    const uint32_t row_end = (uint32_t)__builtin_amdgcn_readfirstlane((int)(row - (row & (uint32_t)(RSTEP - 1)))) + (uint32_t)(RSTEP * NRT);
    const uint32_t tok_end = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tok - (tok & (uint32_t)(TSTEP - 1)))) + (uint32_t)(TSTEP * NTT);
    const bool inside = row_end <= a.m && tok_end <= a.n;
    if (ksplit > 1) {  // this share's sums; the reduce launch (or the caller's next kernel) adds the shares up
        float* base = a.partial + (size_t)split * a.n * a.m;
        if (inside) store_results<NTT, NRT, TSTEP, RSTEP, false, false, false>(base, a.m, row, tok, a.m, a.n, value);
        else store_results<NTT, NRT, TSTEP, RSTEP, false, true, false>(base, a.m, row, tok, a.m, a.n, value);
    } else if (a.y_row_major) {
        if (a.accumulate) store_results<NTT, NRT, TSTEP, RSTEP, true, true, true>(a.y, a.y_stride, row, tok, a.m, a.n, value);
        else if (inside) store_results<NTT, NRT, TSTEP, RSTEP, true, false, false>(a.y, a.y_stride, row, tok, a.m, a.n, value);
        else store_results<NTT, NRT, TSTEP, RSTEP, true, true, false>(a.y, a.y_stride, row, tok, a.m, a.n, value);
    } else {
        if (a.accumulate) store_results<NTT, NRT, TSTEP, RSTEP, false, true, true>(a.y, a.y_stride, row, tok, a.m, a.n, value);
        else if (inside) store_results<NTT, NRT, TSTEP, RSTEP, false, false, false>(a.y, a.y_stride, row, tok, a.m, a.n, value);
        else store_results<NTT, NRT, TSTEP, RSTEP, false, true, false>(a.y, a.y_stride, row, tok, a.m, a.n, value);
    }
}

// Maximum over the 16 lanes of a DPP row (lanes that share lane / 16); every lane of the row ends with it.
__device__ __forceinline__ float row_max16(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false)));   // quad_perm [1,0,3,2]
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false)));   // quad_perm [2,3,0,1]
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false)));  // row_half_mirror
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false)));  // row_mirror
    return v;
}

template <int TYPE, bool DUMP, bool GATED = false>
__global__ __launch_bounds__(THREADS, 4) void gemm_mfma_kernel(GemmArgs a) {
    static_assert(!(DUMP && GATED), "the parity hook dumps plain projections");
    __shared__ Smem sm;
    uint32_t row_tile, tok_tile;
    bool valid_tile;
    // K split (plain single-weight launches only): workgroup (tile, share) walks the stages [first, first + stages) of its tile
    const uint32_t ksplit = DUMP || GATED || a.ksplit < 2 ? 1u : a.ksplit;
    const uint32_t split = ksplit > 1 ? blockIdx.x % ksplit : 0u;
    tile_of_block(ksplit > 1 ? blockIdx.x / ksplit : blockIdx.x, a.row_tiles, a.tok_tiles, row_tile, tok_tile, valid_tile);
    if (!valid_tile) return;  // whole workgroup leaves together
    if constexpr (!GATED) select_weight(a, row_tile);
    const uint32_t row0 = row_tile * (GATED ? BM / 2 : BM);  // GATED: 64 output rows per tile, see load_stage
    const uint32_t tok0 = tok_tile * BN;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t l16 = lane & 15u;
    const uint32_t kq = lane >> 4;            // which 8-byte quarter of the block this lane feeds
    const uint32_t wrow0 = (wave >> 2) * 64;  // wave's rows within the tile
    const uint32_t wtok0 = (wave & 3u) * 32;  // wave's tokens within the tile
    const uint32_t nb = a.k >> 5;
    const uint32_t all_stages = nb / KB;
    const uint32_t first = split * all_stages / ksplit;  // shares differ by at most one stage, none is empty
    const uint32_t stages = (split + 1u) * all_stages / ksplit - first;

    float acc[TT][RT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[tt][rt][r] = 0.0f;

    v4i cbias = {(int)kBiasBits, (int)kBiasBits, (int)kBiasBits, (int)kBiasBits};
    asm volatile("" : "+v"(cbias));  // keep it in registers (left alone, the compiler rebuilds it before every MFMA)

    StageRegs regs;
    StagePtrs<BN> ptrs;
    init_stage_ptrs<BN, GATED>(a, row_tile, tok0, first * KB, ptrs);
    dma_stage(ptrs, sm.st[0]);
    load_stage(ptrs, regs);
    store_stage(sm.st[0], regs);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's direct-to-LDS copies have landed
    __syncthreads();

    // This lane's LDS read addresses: block 0 of buffer 0 here, moved from block to block by next_block and from one buffer to
    // the other at the end of every stage (four additions instead of rebuilding them).
    LaneAddr la;
    {
        const Stage& s = sm.st[0];
        // this lane's token row; K-chunk 2*block + (kq >> 1) sits at position chunk ^ swizzle
        la.xsh = xt_swizzle(wtok0 + l16) >> 1;
        la.xbase = lds_addr(&s.xt[wtok0 + l16][0]) + ((((kq >> 1) ^ xt_swizzle(wtok0 + l16)) & 1u) << 4) + 8 * (kq & 1u);
        la.xt = la.xbase + (la.xsh << 5);
        la.wt = lds_addr(&s.wt[wrow0 / GR][kq >> 1][0][l16]) + 8 * (kq & 1u);  // the wave's 64 rows are two granules
        la.dws = lds_addr(&s.dws[wrow0 / GR][0][l16]);
        la.dxf = lds_addr(&s.dxf[0][wtok0 + 4 * kq]);
    }

    for (uint32_t st = 0; st < stages; st++) {
        if (st + 1 < stages) {
            // the other LDS stage was last read in stage st-1 and every wave has passed the
            // barrier that ended it, so it can be refilled from here on
            dma_stage(ptrs, sm.st[(st + 1) & 1u]);
            load_stage(ptrs, regs);
        }

        // 8 MFMA tiles per block, software-pipelined by hand: four result buffers, the matrix
        // core runs up to four tiles ahead of the vector ALU, and every operand register is
        // refilled from LDS (for block b+1) as soon as its last use in block b has been
        // issued, so LDS latency stays out of the wave's dependency chain.  The scheduling
        // barriers pin that order; the block loop stays rolled.
        // Tile order: t = 4 * token tile + row tile.
        Mats mt;
        Scales sc;
        load_mats(la, mt);              // 6 reads
        load_tok_scales<0>(la, sc);     // 1
        load_tok_scales<1>(la, sc);     // 1
        load_row_scales(la, sc);        // 4
#pragma unroll 1
        for (int b = 0; b < KB; b++) {
            next_block(la, (uint32_t)b, b + 1 < KB);  // last iteration: harmless re-read of its own block
            const uint32_t row = row0 + wrow0 + l16, tok = tok0 + wtok0 + 4 * kq, blk = (first + st) * KB + b;
            v4i d[4];
            lds_wait<6>(mt);  // the six reads issued after the matrices may still be in flight
#pragma unroll
            for (int t = 0; t < 4; t++) d[t] = __builtin_amdgcn_mfma_i32_16x16x32_i8(mt.av[0], mt.bv[t], cbias, 0, 0, 0);
            lds_wait<0>(sc);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const int tt = t >> 2, rt = t & 3;
                if constexpr (DUMP) dump_tile<TYPE>(a, d[t & 3], row + 16 * rt, tok + 16 * tt, nb, blk);
                else scale_tile(d[t & 3], sc.dw[rt], sc.dx[tt], acc[tt][rt]);
                __builtin_amdgcn_sched_barrier(0);
                if (t < 4) {
                    d[t & 3] = __builtin_amdgcn_mfma_i32_16x16x32_i8(mt.av[1], mt.bv[t], cbias, 0, 0, 0);
                    if (t == 3) {
                        load_mats(la, mt);           // all eight MFMAs of this block have been issued
                        load_tok_scales<0>(la, sc);  // token tile 0 is done
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            load_tok_scales<1>(la, sc);
            load_row_scales(la, sc);
        }
        lds_wait<0>(sc);  // nothing of this stage's buffer is read past this point
        {   // block 0 of the other buffer (the block loop left wt / dws / dxf at block KB - 1)
            const uint32_t other = (st & 1u) ? 0u - (uint32_t)sizeof(Stage) : (uint32_t)sizeof(Stage);
            la.xbase += other;
            la.xt = la.xbase + (la.xsh << 5);
            la.wt += other - (KB - 1) * kOffWt;
            la.dws += other - (KB - 1) * kOffDws;
            la.dxf += other - (KB - 1) * kOffDxf;
        }

        // The other buffer was last read in stage st-1; every wave has passed the barrier
        // that ended that stage, so it is free to be refilled now.
        if (st + 1 < stages) store_stage(sm.st[(st + 1) & 1u], regs);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS copies of the next stage have landed
        __syncthreads();
    }

    if constexpr (GATED) {
        // silu(gate) * up and the Q8_0 quantizer on the wave's registers, element for element what silu_mul_quantize_kernel
        // computes from the two float results: row tiles 0 / 1 are gate rows A / B, 2 / 3 the same rows of up; the 16 lanes
        // of a DPP row hold the 16 rows of a tile for the same four tokens, so one row reduction gives a block's maximum.
        static_assert(RT == 4, "two gate and two up row tiles per wave");
        const uint32_t rbase = row0 + (wrow0 >> 1);  // first of this wave's 32 output rows = one Q8_0 block
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t tok = tok0 + wtok0 + 16 * tt + 4 * kq + r;
                const float ha = silu_mul(acc[tt][0][r], acc[tt][2][r]), hb = silu_mul(acc[tt][1][r], acc[tt][3][r]);
                const float amax = row_max16(fmaxf(fabsf(ha), fabsf(hb)));
                float id;
                const float scale = q8_scale_and_inverse(amax, id);
                const int qa = (int)__builtin_rintf(__fmul_rn(ha, id)), qb = (int)__builtin_rintf(__fmul_rn(hb, id));
                if (tok < a.n && rbase < a.m) {  // m % 32 == 0: a block is inside the matrix or not at all
                    int8_t* dst = a.q_out + (size_t)tok * a.m + rbase;
                    dst[l16] = (int8_t)qa;
                    dst[16 + l16] = (int8_t)qb;
                    if (l16 == 0) a.s_out[(size_t)tok * (a.m >> 5) + (rbase >> 5)] = scale;
                }
            }
    } else if constexpr (!DUMP) {
        store_wave_tile<TT, RT>(a, ksplit, split, row0 + wrow0 + l16, tok0 + wtok0 + 4 * kq,
                                [&](int tt, int rt, int r) { return acc[tt][rt][r]; });
    }
}

// ---------------------------------------------------------------------------------------
// The wide tile on the large MFMA shape: same workgroup tile (128 rows x 128 tokens), same stages, copies and LDS layouts
// as gemm_mfma_kernel, but a wave's 64 rows x 32 tokens are TWO v_mfma_i32_32x32x32_i8 per block (rows 0..31 and 32..63 of
// the wave against its 32 tokens) instead of eight 16x16x32: the small shape runs the matrix unit at a third of its rate and
// its time adds to the scaling FMAs' (a SIMD does not overlap the two), so a block's matrix work drops from ~160 to ~57 cycles.
// Layout of the 32x32 result: lane l holds weight row n = l % 32 (of its row half) and the 16 tokens
// m = 8 g + 4 (l / 32) + r, g = 0..3, r = 0..3 -- one row-scale pair per MFMA and 16 token scales per block (four 16-byte LDS
// reads, shared by both MFMAs).  ONE result buffer: MFMA -> its 32 FMAs -> MFMA -> its 32 FMAs; the other waves of the SIMD
// cover the MFMA's latency (measured: faster than two buffers, and 16 registers cheaper, which is what lets the 16-register
// bias tuple, 16 token scales and 32 accumulators fit four waves per SIMD).  Operands of block b+1 are requested as soon as
// the second MFMA of block b has been issued, token scales group by group behind their last use.
// Plain projections only (the gated launch keeps the 16x16 kernel, whose epilogue is written for that result layout).
typedef int v16i __attribute__((ext_vector_type(16)));
struct Mats32 {
    v4i a, b0, b1;  // 16 K-bytes of this lane's token / of its row in the wave's first and second 32 rows
};
struct Scales32 {
    float2 dw0, dw1;  // {dw, -12582912*dw} of this lane's two rows
    v4f dx[4];        // token scales of its four token groups
};
template <int OFF>
__device__ __forceinline__ void lds_read16(uint32_t addr, v4i& dst) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ void load_mats(const LaneAddr& la, Mats32& m) {  // 3 reads
    lds_read16<0>(la.xt, m.a);
    lds_read16<0>(la.wt, m.b0);
    lds_read16<kSlabWt>(la.wt, m.b1);  // the wave's second granule
}
template <int G>
__device__ __forceinline__ void load_tok_scales32(const LaneAddr& la, Scales32& s) {  // 1 read
    lds_read16<32 * G>(la.dxf, s.dx[G]);
}
// (the waits tie the registers that become valid, so nothing that uses them can be scheduled above)
template <int N>
__device__ __forceinline__ void lds_wait_a_b0(Mats32& m) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(m.a), "+v"(m.b0) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait_phase_a(Mats32& m, Scales32& s) {
    asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(m.b1), "+v"(s.dw0), "+v"(s.dx[0]), "+v"(s.dx[1]), "+v"(s.dx[2]), "+v"(s.dx[3]) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait_dw1(Scales32& s) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(s.dw1) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait_all(Mats32& m, Scales32& s) {
    asm volatile("s_waitcnt lgkmcnt(%9)"
                 : "+v"(m.a), "+v"(m.b0), "+v"(m.b1), "+v"(s.dw0), "+v"(s.dw1), "+v"(s.dx[0]), "+v"(s.dx[1]), "+v"(s.dx[2]), "+v"(s.dx[3])
                 : "n"(N)
                 : "memory");
}

template <int TYPE, bool DUMP>
__global__ __launch_bounds__(THREADS, 4) void gemm_mfma32_kernel(GemmArgs a) {
    __shared__ Smem sm;
    uint32_t row_tile, tok_tile;
    bool valid_tile;
    const uint32_t ksplit = DUMP || a.ksplit < 2 ? 1u : a.ksplit;
    const uint32_t split = ksplit > 1 ? blockIdx.x % ksplit : 0u;
    tile_of_block(ksplit > 1 ? blockIdx.x / ksplit : blockIdx.x, a.row_tiles, a.tok_tiles, row_tile, tok_tile, valid_tile);
    if (!valid_tile) return;  // whole workgroup leaves together
    select_weight(a, row_tile);
    const uint32_t row0 = row_tile * BM;
    const uint32_t tok0 = tok_tile * BN;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t l32 = lane & 31u;
    const uint32_t kh = lane >> 5;            // which 16-byte half of the block this lane feeds
    const uint32_t wrow0 = (wave >> 2) * 64;  // wave's rows within the tile
    const uint32_t wtok0 = (wave & 3u) * 32;  // wave's tokens within the tile
    const uint32_t nb = a.k >> 5;
    const uint32_t all_stages = nb / KB;
    const uint32_t first = split * all_stages / ksplit;  // shares differ by at most one stage, none is empty
    const uint32_t stages = (split + 1u) * all_stages / ksplit - first;

    float acc[2][16];  // [row half][4 g + r]
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[j][i] = 0.0f;

    v16i cbias;
#pragma unroll
    for (int i = 0; i < 16; i++) cbias[i] = (int)kBiasBits;
    asm volatile("" : "+v"(cbias));  // keep it in registers (left alone, the compiler rebuilds it before every MFMA)

    StageRegs regs;
    StagePtrs<BN> ptrs;
    init_stage_ptrs<BN, false>(a, row_tile, tok0, first * KB, ptrs);
    dma_stage(ptrs, sm.st[0]);
    load_stage(ptrs, regs);
    store_stage(sm.st[0], regs);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's direct-to-LDS copies have landed
    __syncthreads();

    LaneAddr la;
    {
        const Stage& s = sm.st[0];
        // this lane's token row; K-chunk 2*block + kh sits at position chunk ^ swizzle
        const uint32_t sw = xt_swizzle(wtok0 + l32);
        la.xsh = sw >> 1;
        la.xbase = lds_addr(&s.xt[wtok0 + l32][0]) + (((kh ^ sw) & 1u) << 4);
        la.xt = la.xbase + (la.xsh << 5);
        la.wt = lds_addr(&s.wt[wrow0 / GR][kh][0][l32]);  // the wave's 64 rows are two granules
        la.dws = lds_addr(&s.dws[wrow0 / GR][0][l32]);
        la.dxf = lds_addr(&s.dxf[0][wtok0 + 4 * kh]);
    }

    for (uint32_t st = 0; st < stages; st++) {
        if (st + 1 < stages) {
            dma_stage(ptrs, sm.st[(st + 1) & 1u]);
            load_stage(ptrs, regs);
        }

        // Reads of a block, in issue order (LDS data returns in that order): a, b0, b1, dw0, dx0..dx3, dw1.
        Mats32 mt;
        Scales32 sc;
        load_mats(la, mt);                  // 3
        lds_read8<0>(la.dws, sc.dw0);       // 1
        load_tok_scales32<0>(la, sc);       // 4
        load_tok_scales32<1>(la, sc);
        load_tok_scales32<2>(la, sc);
        load_tok_scales32<3>(la, sc);
        lds_read8<kSlabDws>(la.dws, sc.dw1);  // 1
#pragma unroll 1
        for (int b = 0; b < KB; b++) {
            next_block(la, (uint32_t)b, b + 1 < KB);  // last iteration: harmless re-read of its own block
            const uint32_t row = row0 + wrow0 + l32, tok = tok0 + wtok0 + 4 * kh, blk = (first + st) * KB + b;
            auto consume = [&](const v16i& d, int j, const float2 dw) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    if constexpr (DUMP) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            if (row + 32 * j < a.m && tok + 8 * g + r < a.n) {
                                int v = d[4 * g + r] - (int)kBiasBits;
                                if (TYPE == 2) v >>= 4;  // weights were stored x16; exact
                                a.dots[((size_t)(tok + 8 * g + r) * a.m + row + 32 * j) * nb + blk] = v;
                            }
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const float v = __builtin_fmaf(__int_as_float(d[4 * g + r]), dw.x, dw.y);
                            acc[j][4 * g + r] = __builtin_fmaf(v, sc.dx[g][r], acc[j][4 * g + r]);
                        }
                    }
                    if (j == 1) {  // this group's token scales are done with: request the next block's
                        if (g == 0) load_tok_scales32<0>(la, sc);
                        if (g == 1) load_tok_scales32<1>(la, sc);
                        if (g == 2) load_tok_scales32<2>(la, sc);
                        if (g == 3) load_tok_scales32<3>(la, sc);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            lds_wait_a_b0<7>(mt);  // the seven reads issued after a and b0 may still be in flight
            v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.a, mt.b0, cbias, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);  // (the MFMA goes out before the wait for what only the FMAs need)
            lds_wait_phase_a<1>(mt, sc);  // everything but dw1
            __builtin_amdgcn_sched_barrier(0);
            consume(d, 0, sc.dw0);
            d = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.a, mt.b1, cbias, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            load_mats(la, mt);             // both MFMAs of this block have been issued
            lds_read8<0>(la.dws, sc.dw0);  // the first row half is done
            lds_wait_dw1<4>(sc);           // (the four reads just issued stay in flight)
            __builtin_amdgcn_sched_barrier(0);
            consume(d, 1, sc.dw1);
            lds_read8<kSlabDws>(la.dws, sc.dw1);
        }
        lds_wait_all<0>(mt, sc);  // nothing of this stage's buffer is read past this point
        {   // block 0 of the other buffer (the block loop left wt / dws / dxf at block KB - 1)
            const uint32_t other = (st & 1u) ? 0u - (uint32_t)sizeof(Stage) : (uint32_t)sizeof(Stage);
            la.xbase += other;
            la.xt = la.xbase + (la.xsh << 5);
            la.wt += other - (KB - 1) * kOffWt;
            la.dws += other - (KB - 1) * kOffDws;
            la.dxf += other - (KB - 1) * kOffDxf;
        }
        if (st + 1 < stages) store_stage(sm.st[(st + 1) & 1u], regs);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS copies of the next stage have landed
        __syncthreads();
    }

    if constexpr (!DUMP) {
        store_wave_tile<4, 2, 8, 32>(a, ksplit, split, row0 + wrow0 + l32, tok0 + wtok0 + 4 * kh,
                                     [&](int g, int j, int r) { return acc[j][4 * g + r]; });
    }
}

// ---------------------------------------------------------------------------------------
// Narrow variant for 16 <= n <= 64 (an LM head or a projection over a short prompt): tile =
// 128 weight rows x 64 tokens, every one of the 8 waves owns 16 rows x all 64 tokens (one
// row tile x four token tiles), so no matrix or scaling work is spent on token columns that
// do not exist beyond the 64, and the weights -- the only large operand -- are streamed
// exactly once.  Same staging, LDS layouts and arithmetic as the wide kernel; 60 KB of LDS,
// two workgroups per CU.  TTN (1 .. 4): how many of the four token tiles the launch has tokens
// for -- a launch of n <= 16 / 32 / 48 tokens reads and multiplies only those (these launches
// are bound by their block loop, so the unused tiles were a third to three quarters of their time).
struct NarrowMats {
    long av[4], bv;
};
struct NarrowScales {
    float2 dw;
    v4f dx[4];
};
constexpr int kOffDxfNarrow = sizeof(float) * BN_NARROW;
// TTN: the token tiles (of 16) the launch has tokens for; the others are neither read nor multiplied.
template <int TTN>
__device__ __forceinline__ void load_mats(const LaneAddr& la, NarrowMats& m) {  // TTN + 1 reads
    lds_read8<0 * 16 * 128>(la.xt, m.av[0]);
    if constexpr (TTN > 1) lds_read8<1 * 16 * 128>(la.xt, m.av[1]);
    if constexpr (TTN > 2) lds_read8<2 * 16 * 128>(la.xt, m.av[2]);
    if constexpr (TTN > 3) lds_read8<3 * 16 * 128>(la.xt, m.av[3]);
    lds_read8<0>(la.wt, m.bv);
}
template <int TTN>
__device__ __forceinline__ void load_scales(const LaneAddr& la, NarrowScales& s) {  // TTN + 1 reads
    lds_read8<0>(la.dws, s.dw);
    lds_read16<0 * 64>(la.dxf, s.dx[0]);
    if constexpr (TTN > 1) lds_read16<1 * 64>(la.dxf, s.dx[1]);
    if constexpr (TTN > 2) lds_read16<2 * 64>(la.dxf, s.dx[2]);
    if constexpr (TTN > 3) lds_read16<3 * 64>(la.dxf, s.dx[3]);
}
template <int N>
__device__ __forceinline__ void lds_wait(NarrowMats& m) {
    asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(m.av[0]), "+v"(m.av[1]), "+v"(m.av[2]), "+v"(m.av[3]), "+v"(m.bv) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait(NarrowScales& s) {
    asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(s.dw), "+v"(s.dx[0]), "+v"(s.dx[1]), "+v"(s.dx[2]), "+v"(s.dx[3]) : "n"(N) : "memory");
}

template <int TYPE, bool DUMP, int TTN = 4>
__global__ __launch_bounds__(THREADS, 4) void gemm_narrow_kernel(GemmArgs a) {
    __shared__ SmemT<BN_NARROW> sm;
    uint32_t row_tile, tok_tile;
    bool valid_tile;
    const uint32_t ksplit = DUMP || a.ksplit < 2 ? 1u : a.ksplit;
    const uint32_t split = ksplit > 1 ? blockIdx.x % ksplit : 0u;  // the splits of a tile are neighbours: different XCDs, same time
    tile_of_block(ksplit > 1 ? blockIdx.x / ksplit : blockIdx.x, a.row_tiles, a.tok_tiles, row_tile, tok_tile, valid_tile);
    if (!valid_tile) return;  // whole workgroup leaves together
    select_weight(a, row_tile);
    const uint32_t row0 = row_tile * BM;
    const uint32_t tok0 = tok_tile * BN_NARROW;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t l16 = lane & 15u;
    const uint32_t kq = lane >> 4;      // which 8-byte quarter of the block this lane feeds
    const uint32_t wrow0 = wave * 16;   // wave's rows within the tile
    const uint32_t nb = a.k >> 5;
    // this workgroup's stages: [first, first + stages)
    const uint32_t all_stages = nb / KB;
    // shares differ by at most one stage and none is empty (the host splits only where all_stages >= 2 * ksplit)
    const uint32_t first = split * all_stages / ksplit;
    const uint32_t stages = (split + 1u) * all_stages / ksplit - first;

    float acc[4][4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[tt][r] = 0.0f;

    v4i cbias = {(int)kBiasBits, (int)kBiasBits, (int)kBiasBits, (int)kBiasBits};
    asm volatile("" : "+v"(cbias));

    StageRegs regs;
    StagePtrs<BN_NARROW> ptrs;
    init_stage_ptrs<BN_NARROW>(a, row_tile, tok0, first * KB, ptrs);
    dma_stage(ptrs, sm.st[0]);
    load_stage(ptrs, regs);
    store_stage(sm.st[0], regs);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's direct-to-LDS copies have landed
    __syncthreads();

    LaneAddr la;  // block 0 of buffer 0; moved on as in the wide kernel
    {
        const StageT<BN_NARROW>& s = sm.st[0];
        la.xsh = xt_swizzle(l16) >> 1;
        la.xbase = lds_addr(&s.xt[l16][0]) + ((((kq >> 1) ^ xt_swizzle(l16)) & 1u) << 4) + 8 * (kq & 1u);
        la.xt = la.xbase + (la.xsh << 5);
        la.wt = lds_addr(&s.wt[wrow0 / GR][kq >> 1][0][(wrow0 % GR) + l16]) + 8 * (kq & 1u);  // the wave's 16 rows: half a granule
        la.dws = lds_addr(&s.dws[wrow0 / GR][0][(wrow0 % GR) + l16]);
        la.dxf = lds_addr(&s.dxf[0][4 * kq]);
    }

    for (uint32_t st = 0; st < stages; st++) {
        if (st + 1 < stages) {
            dma_stage(ptrs, sm.st[(st + 1) & 1u]);
            load_stage(ptrs, regs);
        }

        NarrowMats mt{};
        NarrowScales sc{};
        load_mats<TTN>(la, mt);    // TTN + 1 reads
        load_scales<TTN>(la, sc);  // TTN + 1 reads
#pragma unroll 1
        for (int b = 0; b < KB; b++) {
            // addresses of block b+1 (last iteration: harmless re-read of its own block)
            const bool adv = b + 1 < KB;
            la.xt = la.xbase + ((((uint32_t)(adv ? b + 1 : b)) ^ la.xsh) << 5);
            la.wt += adv ? kOffWt : 0;
            la.dws += adv ? kOffDws : 0;
            la.dxf += adv ? kOffDxfNarrow : 0;
            const uint32_t row = row0 + wrow0 + l16, tok = tok0 + 4 * kq, blk = (first + st) * KB + b;
            v4i d[TTN];
            lds_wait<TTN + 1>(mt);  // the scale reads issued after the matrices may still be in flight
#pragma unroll
            for (int tt = 0; tt < TTN; tt++) d[tt] = __builtin_amdgcn_mfma_i32_16x16x32_i8(mt.av[tt], mt.bv, cbias, 0, 0, 0);
            load_mats<TTN>(la, mt);  // in place: the MFMAs that read block b's operands have been issued
            lds_wait<TTN + 1>(sc);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tt = 0; tt < TTN; tt++) {
                if constexpr (DUMP) dump_tile<TYPE>(a, d[tt], row, tok + 16 * tt, nb, blk);
                else scale_tile(d[tt], sc.dw, sc.dx[tt], acc[tt]);
            }
            __builtin_amdgcn_sched_barrier(0);
            load_scales<TTN>(la, sc);
        }
        lds_wait<0>(sc);  // nothing of this stage's buffer is read past this point
        {
            const uint32_t other = (st & 1u) ? 0u - (uint32_t)sizeof(StageT<BN_NARROW>) : (uint32_t)sizeof(StageT<BN_NARROW>);
            la.xbase += other;
            la.xt = la.xbase + (la.xsh << 5);
            la.wt += other - (KB - 1) * kOffWt;
            la.dws += other - (KB - 1) * kOffDws;
            la.dxf += other - (KB - 1) * kOffDxfNarrow;
        }

        if (st + 1 < stages) store_stage(sm.st[(st + 1) & 1u], regs);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS copies of the next stage have landed
        __syncthreads();
    }

    if constexpr (!DUMP) {
        store_wave_tile<TTN, 1>(a, ksplit, split, row0 + wrow0 + l16, tok0 + 4 * kq, [&](int tt, int, int r) { return acc[tt][r]; });
    }
}

// The narrow tile (128 rows x 64 tokens) on the large MFMA shape, for launches that have tokens for the whole tile
// (n > 48; the shorter ones keep gemm_narrow_kernel's 16-token tiles): wave w owns rows 32 (w / 2) .. of the tile (one
// granule) against tokens 32 (w % 2) .., ONE v_mfma_i32_32x32x32_i8 per block instead of four 16x16x32, the result layout,
// scale reads and single result buffer of gemm_mfma32_kernel.  Same stages, copies and LDS layouts as gemm_narrow_kernel.
struct NarrowMats32 {
    v4i a, b;
};
struct NarrowScales32 {
    float2 dw;
    v4f dx[4];
};
template <int N>
__device__ __forceinline__ void lds_wait(NarrowMats32& m) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(m.a), "+v"(m.b) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait(NarrowScales32& s) {
    asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(s.dw), "+v"(s.dx[0]), "+v"(s.dx[1]), "+v"(s.dx[2]), "+v"(s.dx[3]) : "n"(N) : "memory");
}

template <int TYPE, bool DUMP>
__global__ __launch_bounds__(THREADS, 4) void gemm_narrow32_kernel(GemmArgs a) {
    __shared__ SmemT<BN_NARROW> sm;
    uint32_t row_tile, tok_tile;
    bool valid_tile;
    const uint32_t ksplit = DUMP || a.ksplit < 2 ? 1u : a.ksplit;
    const uint32_t split = ksplit > 1 ? blockIdx.x % ksplit : 0u;
    tile_of_block(ksplit > 1 ? blockIdx.x / ksplit : blockIdx.x, a.row_tiles, a.tok_tiles, row_tile, tok_tile, valid_tile);
    if (!valid_tile) return;  // whole workgroup leaves together
    select_weight(a, row_tile);
    const uint32_t row0 = row_tile * BM;
    const uint32_t tok0 = tok_tile * BN_NARROW;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t l32 = lane & 31u;
    const uint32_t kh = lane >> 5;             // which 16-byte half of the block this lane feeds
    const uint32_t wrow0 = (wave >> 1) * 32;   // wave's rows within the tile: one granule
    const uint32_t wtok0 = (wave & 1u) * 32;   // wave's tokens within the tile
    const uint32_t nb = a.k >> 5;
    const uint32_t all_stages = nb / KB;
    const uint32_t first = split * all_stages / ksplit;
    const uint32_t stages = (split + 1u) * all_stages / ksplit - first;

    float acc[16];  // [4 g + r]
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.0f;
    v16i cbias;
#pragma unroll
    for (int i = 0; i < 16; i++) cbias[i] = (int)kBiasBits;
    asm volatile("" : "+v"(cbias));

    StageRegs regs;
    StagePtrs<BN_NARROW> ptrs;
    init_stage_ptrs<BN_NARROW>(a, row_tile, tok0, first * KB, ptrs);
    dma_stage(ptrs, sm.st[0]);
    load_stage(ptrs, regs);
    store_stage(sm.st[0], regs);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's direct-to-LDS copies have landed
    __syncthreads();

    LaneAddr la;  // block 0 of buffer 0; moved on as in the wide kernel
    {
        const StageT<BN_NARROW>& s = sm.st[0];
        const uint32_t sw = xt_swizzle(wtok0 + l32);
        la.xsh = sw >> 1;
        la.xbase = lds_addr(&s.xt[wtok0 + l32][0]) + (((kh ^ sw) & 1u) << 4);
        la.xt = la.xbase + (la.xsh << 5);
        la.wt = lds_addr(&s.wt[wrow0 / GR][kh][0][l32]);
        la.dws = lds_addr(&s.dws[wrow0 / GR][0][l32]);
        la.dxf = lds_addr(&s.dxf[0][wtok0 + 4 * kh]);
    }

    for (uint32_t st = 0; st < stages; st++) {
        if (st + 1 < stages) {
            dma_stage(ptrs, sm.st[(st + 1) & 1u]);
            load_stage(ptrs, regs);
        }

        // Reads of a block, in issue order: a, b, dx0..dx3, dw.
        NarrowMats32 mt;
        NarrowScales32 sc;
        lds_read16<0>(la.xt, mt.a);
        lds_read16<0>(la.wt, mt.b);
        lds_read16<0>(la.dxf, sc.dx[0]);
        lds_read16<32>(la.dxf, sc.dx[1]);
        lds_read16<64>(la.dxf, sc.dx[2]);
        lds_read16<96>(la.dxf, sc.dx[3]);
        lds_read8<0>(la.dws, sc.dw);
#pragma unroll 1
        for (int b = 0; b < KB; b++) {
            const bool adv = b + 1 < KB;  // last iteration: harmless re-read of its own block
            la.xt = la.xbase + ((((uint32_t)(adv ? b + 1 : b)) ^ la.xsh) << 5);
            la.wt += adv ? kOffWt : 0;
            la.dws += adv ? kOffDws : 0;
            la.dxf += adv ? kOffDxfNarrow : 0;
            const uint32_t row = row0 + wrow0 + l32, tok = tok0 + wtok0 + 4 * kh, blk = (first + st) * KB + b;
            lds_wait<5>(mt);  // the five scale reads issued after a and b may still be in flight
            const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(mt.a, mt.b, cbias, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            lds_read16<0>(la.xt, mt.a);  // the MFMA that reads block b's operands has been issued
            lds_read16<0>(la.wt, mt.b);
            lds_wait<2>(sc);  // (the two reads just issued stay in flight)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if constexpr (DUMP) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        if (row < a.m && tok + 8 * g + r < a.n) {
                            int v = d[4 * g + r] - (int)kBiasBits;
                            if (TYPE == 2) v >>= 4;  // weights were stored x16; exact
                            a.dots[((size_t)(tok + 8 * g + r) * a.m + row) * nb + blk] = v;
                        }
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float v = __builtin_fmaf(__int_as_float(d[4 * g + r]), sc.dw.x, sc.dw.y);
                        acc[4 * g + r] = __builtin_fmaf(v, sc.dx[g][r], acc[4 * g + r]);
                    }
                }
                // this group's token scales are done with: request the next block's
                if (g == 0) lds_read16<0>(la.dxf, sc.dx[0]);
                if (g == 1) lds_read16<32>(la.dxf, sc.dx[1]);
                if (g == 2) lds_read16<64>(la.dxf, sc.dx[2]);
                if (g == 3) lds_read16<96>(la.dxf, sc.dx[3]);
                __builtin_amdgcn_sched_barrier(0);
            }
            lds_read8<0>(la.dws, sc.dw);
        }
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(mt.a), "+v"(mt.b), "+v"(sc.dw), "+v"(sc.dx[0]), "+v"(sc.dx[1]), "+v"(sc.dx[2]), "+v"(sc.dx[3])
                     :
                     : "memory");  // nothing of this stage's buffer is read past this point
        {
            const uint32_t other = (st & 1u) ? 0u - (uint32_t)sizeof(StageT<BN_NARROW>) : (uint32_t)sizeof(StageT<BN_NARROW>);
            la.xbase += other;
            la.xt = la.xbase + (la.xsh << 5);
            la.wt += other - (KB - 1) * kOffWt;
            la.dws += other - (KB - 1) * kOffDws;
            la.dxf += other - (KB - 1) * kOffDxfNarrow;
        }
        if (st + 1 < stages) store_stage(sm.st[(st + 1) & 1u], regs);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS copies of the next stage have landed
        __syncthreads();
    }

    if constexpr (!DUMP) {
        store_wave_tile<4, 1, 8, 32>(a, ksplit, split, row0 + wrow0 + l32, tok0 + wtok0 + 4 * kh, [&](int g, int, int r) { return acc[4 * g + r]; });
    }
}

// y (+)= partial[0] + partial[1] + ... in that order, element by element (token-major partials [split][n][m]).
// (S a template parameter: all of an element's loads are in flight together instead of one round trip per share.)
template <int S>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ partial, uint32_t n, uint32_t m,
                                                                 float* __restrict__ y, uint32_t y_stride, int y_row_major, int accumulate) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, total = (size_t)n * m;
    if (i >= total) return;
    const uint32_t tok = (uint32_t)(i / m), row = (uint32_t)(i % m);
    float* dst = y_row_major ? y + (size_t)row * y_stride + tok : y + (size_t)tok * y_stride + row;
    float p[S];
#pragma unroll
    for (int s_ = 0; s_ < S; s_++) p[s_] = partial[(size_t)s_ * total + i];
    const float old = accumulate ? *dst : 0.0f;
    float sum = p[0];
#pragma unroll
    for (int s_ = 1; s_ < S; s_++) sum += p[s_];
    *dst = accumulate ? old + sum : sum;
}

// How many ways a single-weight launch is split over K: only narrow launches that leave at least half of the CUs without
// a tile, with K long enough (>= 8 stages) that the shorter walk pays for the second launch, every share >= 2 stages (a stage
// of a launch with few tiles costs a whole memory round trip, 1.2 - 1.4 us: nothing else is there to hide it).
// The same on the wide tile: a long-K launch of 64 .. 256 wide tiles (the down projection of a long prompt: 1024 x 2002 x 4608 is
// 128 of them) fills the chip's 512 workgroup slots with (tile, share) pairs of the wide kernel, whose block loop is the faster one,
// instead of one narrow tile per CU.  Shares of >= 8 stages.
uint32_t wide_split_factor(uint32_t m, uint32_t n, uint32_t k, uint32_t max_splits) {
    const uint32_t tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN), stages = (k >> 5) / KB;
    if (n <= BN_NARROW || tiles < 64 || tiles > 256 || stages < 32) return 1;
    uint32_t s_ = 1;
    while (2 * s_ <= max_splits && tiles * 2 * s_ <= 512 && stages / (2 * s_) >= 8) s_ *= 2;
    return s_;
}

uint32_t split_k_factor(uint32_t m, uint32_t n, uint32_t k, uint32_t max_splits) {
    const uint32_t ws = wide_split_factor(m, n, k, max_splits);
    if (ws > 1) return ws;
    const uint32_t row_tiles = (m + BM - 1) / BM;
    const bool narrow = n <= BN_NARROW || row_tiles * ((n + BN - 1) / BN) <= 256;
    if (!narrow) return 1;
    const uint32_t tiles = row_tiles * ((n + BN_NARROW - 1) / BN_NARROW), stages = (k >> 5) / KB;
    if (stages < 8) return 1;
    uint32_t s_ = 1;
    while (2 * s_ <= max_splits && tiles * 2 * s_ <= 256 && stages / (2 * s_) >= 2) s_ *= 2;
    return s_;
}

// The second launch of a split GEMM: y (+)= the shares in ascending order.
hipError_t launch_reduce(const GemmArgs& a, const Launch& L) {
    const size_t total = (size_t)a.n * a.m;
    const auto reduce = [&](auto kernel) {
        return launch_kernel(L, kFamGemm, kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), static_cast<const float*>(a.partial), a.n, a.m, a.y,
                             a.y_stride, a.y_row_major, a.accumulate);
    };
    if (a.ksplit == 2) return reduce(gemm_splitk_reduce_kernel<2>);
    if (a.ksplit == 4) return reduce(gemm_splitk_reduce_kernel<4>);
    if (a.ksplit == 8) return reduce(gemm_splitk_reduce_kernel<8>);
    return hipErrorInvalidValue;  // split_k_factor makes 2, 4 or 8 shares
}

template <bool DUMP>
hipError_t launch(int type, GemmArgs& a, const Launch& L, uint32_t more = 0, bool defer_reduce = false) {
    if (a.m == 0 || a.n == 0) return hipSuccess;
    a.row_tiles = (a.m + BM - 1) / BM;
    a.tile_start[0] = a.tile_start[1] = UINT32_MAX;
    for (uint32_t i = 0; i < more; i++) {
        a.tile_start[i] = a.row_tiles;
        a.row_tiles += (a.m_more[i] + BM - 1) / BM;
    }
    // The narrow tile also serves small problems that would leave more than half of the
    // 512 resident workgroup slots (2 per CU) empty with the wide tile: twice the tiles.
    const bool wide_split = !DUMP && more == 0 && a.ksplit > 1 && wide_split_factor(a.m, a.n, a.k, a.ksplit) == a.ksplit;
    const bool narrow = !wide_split && (a.n <= BN_NARROW || a.row_tiles * ((a.n + BN - 1) / BN) <= 256);
    a.tok_tiles = narrow ? (a.n + BN_NARROW - 1) / BN_NARROW : (a.n + BN - 1) / BN;
    if ((uint64_t)a.row_tiles * a.tok_tiles > 0x7fffff00ull) return hipErrorInvalidValue;  // beyond a launch's grid
    const uint32_t tiles = a.row_tiles * a.tok_tiles;
    const uint32_t blocks = ((tiles + 7u) / 8u) * 8u;  // every XCD gets the same number of slots
    if (narrow) {
        // a launch of at most 16 / 32 / 48 tokens computes one / two / three of the tile's four 16-token MFMA tiles (the parity
        // hook: all four).  These launches are bound by their block loop, not by memory: 65536 x 16 x 2048 40 -> 34 us.
        const auto narrow_launch = [&](uint32_t grid) {
            if constexpr (!DUMP) {
                if (a.n <= 16) return launch_kernel(L, kFamGemm, gemm_narrow_kernel<2, false, 1>, dim3(grid), dim3(THREADS), a);
                if (a.n <= 32) return launch_kernel(L, kFamGemm, gemm_narrow_kernel<2, false, 2>, dim3(grid), dim3(THREADS), a);
                if (a.n <= 48) return launch_kernel(L, kFamGemm, gemm_narrow_kernel<2, false, 3>, dim3(grid), dim3(THREADS), a);
            }
            // (the product kernels do not depend on the weight type any more: the copy they read is the same for both)
            if (!L.gemm_mfma16 && a.n > 48)
                return type == kTypeQ4_0 ? launch_kernel(L, kFamGemm, gemm_narrow32_kernel<2, DUMP>, dim3(grid), dim3(THREADS), a)
                                         : launch_kernel(L, kFamGemm, gemm_narrow32_kernel<8, DUMP>, dim3(grid), dim3(THREADS), a);
            return type == kTypeQ4_0 ? launch_kernel(L, kFamGemm, gemm_narrow_kernel<2, DUMP>, dim3(grid), dim3(THREADS), a)
                                     : launch_kernel(L, kFamGemm, gemm_narrow_kernel<8, DUMP>, dim3(grid), dim3(THREADS), a);
        };
        if (!DUMP && a.ksplit > 1) {
            // tile id = blockIdx.x / ksplit must run over all `blocks` slots of the tile map
            hipError_t e = narrow_launch(blocks * a.ksplit);
            if (e != hipSuccess || defer_reduce) return e;  // deferred: the caller's next kernel adds the shares up itself
            return launch_reduce(a, L);
        }
        return narrow_launch(blocks);
    }
    if (wide_split) {
        hipError_t e = !L.gemm_mfma16
                           ? (type == kTypeQ4_0 ? launch_kernel(L, kFamGemm, gemm_mfma32_kernel<2, DUMP>, dim3(blocks * a.ksplit), dim3(THREADS), a)
                                                : launch_kernel(L, kFamGemm, gemm_mfma32_kernel<8, DUMP>, dim3(blocks * a.ksplit), dim3(THREADS), a))
                           : (type == kTypeQ4_0 ? launch_kernel(L, kFamGemm, gemm_mfma_kernel<2, DUMP>, dim3(blocks * a.ksplit), dim3(THREADS), a)
                                                : launch_kernel(L, kFamGemm, gemm_mfma_kernel<8, DUMP>, dim3(blocks * a.ksplit), dim3(THREADS), a));
        if (e != hipSuccess || defer_reduce) return e;
        return launch_reduce(a, L);
    }
    a.ksplit = 1;  // an unsplit launch of the wide kernel
    if (!L.gemm_mfma16) {
        if (type == kTypeQ4_0) return launch_kernel(L, kFamGemm, gemm_mfma32_kernel<2, DUMP>, dim3(blocks), dim3(THREADS), a);
        return launch_kernel(L, kFamGemm, gemm_mfma32_kernel<8, DUMP>, dim3(blocks), dim3(THREADS), a);
    }
    if (type == kTypeQ4_0)
        return launch_kernel(L, kFamGemm, gemm_mfma_kernel<2, DUMP>, dim3(blocks), dim3(THREADS), a);
    return launch_kernel(L, kFamGemm, gemm_mfma_kernel<8, DUMP>, dim3(blocks), dim3(THREADS), a);
}

}  // namespace

uint32_t gemm_split_k(uint32_t m, uint32_t n, uint32_t k, uint32_t max_splits) { return split_k_factor(m, n, k, max_splits); }

// The GEMM's own copy of a weight (slabs, see StageT): its size, and the kernel that makes it from the raw blocks.
size_t gemm_packed_bytes(uint32_t m, uint32_t k) { return (size_t)((m + 2 * GR - 1) / (2 * GR)) * 2 * ((k >> 5) / KB) * kSlab; }

hipError_t launch_gemm_pack(int type, const uint8_t* d_raw, uint32_t m, uint32_t k, uint8_t* d_packed, const Launch& L) {
    const uint32_t nb = k >> 5;
    if (m == 0 || nb == 0 || nb % KB != 0) return hipErrorInvalidValue;
    const uint64_t blocks = (uint64_t)((m + 2 * GR - 1) / (2 * GR)) * 2 * (nb / KB);  // whole pairs: a last odd granule gets a zero partner
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    if (type == kTypeQ4_0) return launch_kernel(L, kFamOther, gemm_pack_kernel<2>, dim3((uint32_t)blocks), dim3(GR * KB), d_raw, m, nb, d_packed);
    if (type == kTypeQ8_0) return launch_kernel(L, kFamOther, gemm_pack_kernel<8>, dim3((uint32_t)blocks), dim3(GR * KB), d_raw, m, nb, d_packed);
    return hipErrorInvalidValue;
}

// splits > 1 (= gemm_split_k(m, n, k, ...)) with d_partial holding splits * n * m floats: the K-split launch pair.
hipError_t launch_gemm_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                            const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                            int accumulate, const Launch& L, uint32_t splits, float* d_partial, bool defer_reduce) {
    GemmArgs a{};
    a.w = d_w, a.xq = d_q, a.xs = d_scales, a.y = d_y, a.dots = nullptr;
    a.m = m, a.n = n, a.k = k, a.y_stride = y_stride;
    a.y_row_major = (y_layout == 1);
    a.accumulate = accumulate;
    if (splits > 1 && d_partial) {
        if (splits != split_k_factor(m, n, k, splits)) return hipErrorInvalidValue;  // the shape does not carry that split
        a.ksplit = splits, a.partial = d_partial;
    } else if (defer_reduce) {
        return hipErrorInvalidValue;  // nothing to defer on an unsplit launch
    }
    return launch<false>(type, a, L, 0, defer_reduce);
}

// The same launch over up to three weights of one type and k that share the activations: outputs y[i] (same stride,
// layout and accumulate flag), tiles of all weights in one tile list.
hipError_t launch_gemm_mfma_multi(int type, const uint8_t* const* d_w, const uint32_t* m, uint32_t count, uint32_t k, const int8_t* d_q,
                                  const float* d_scales, uint32_t n, float* const* d_y, uint32_t y_stride, int y_layout, int accumulate,
                                  const Launch& L) {
    if (count == 0 || count > 3) return hipErrorInvalidValue;
    GemmArgs a{};
    a.w = d_w[0], a.xq = d_q, a.xs = d_scales, a.y = d_y[0], a.dots = nullptr;
    a.m = m[0], a.n = n, a.k = k, a.y_stride = y_stride;
    a.y_row_major = (y_layout == 1);
    a.accumulate = accumulate;
    for (uint32_t i = 1; i < count; i++) a.w_more[i - 1] = d_w[i], a.y_more[i - 1] = d_y[i], a.m_more[i - 1] = m[i];
    return launch<false>(type, a, L, count - 1);
}

// Gate and up projection of a feed-forward block over n tokens in one launch whose epilogue applies the SiLU gate and
// quantizes: out = Q8_0(silu(W_gate x) * (W_up x)), [n][m] quants + [n][m / 32] scales, bit-identical to the two
// projections + silu_mul_quantize_kernel.  The float projections (2 * n * m * 4 bytes) are never written.
bool gemm_gated_applies(uint32_t m, uint32_t n, uint32_t k) {
    // wide tiles only (the narrow kernel's waves own 16 rows: no block in one wave), and enough of them to fill the chip
    return m % 32u == 0 && k % 128u == 0 && n > BN_NARROW && (uint64_t)((m + 63u) / 64u) * ((n + BN - 1) / BN) > 256u;
}

hipError_t launch_gemm_mfma_gated(int type, const uint8_t* d_w_gate, const uint8_t* d_w_up, uint32_t m, uint32_t k, const int8_t* d_q,
                                  const float* d_scales, uint32_t n, int8_t* d_out_q, float* d_out_scales, const Launch& L) {
    if (m == 0 || n == 0) return hipSuccess;
    if (!gemm_gated_applies(m, n, k)) return hipErrorInvalidValue;
    GemmArgs a{};
    a.w = d_w_gate, a.w_up = d_w_up, a.xq = d_q, a.xs = d_scales, a.q_out = d_out_q, a.s_out = d_out_scales;
    a.m = m, a.n = n, a.k = k;
    a.row_tiles = (m + 63u) / 64u;
    a.tok_tiles = (n + BN - 1) / BN;
    a.tile_start[0] = a.tile_start[1] = UINT32_MAX;
    if ((uint64_t)a.row_tiles * a.tok_tiles > 0x7fffff00ull) return hipErrorInvalidValue;
    const uint32_t blocks = ((a.row_tiles * a.tok_tiles + 7u) / 8u) * 8u;
    if (type == kTypeQ4_0) return launch_kernel(L, kFamGemm, gemm_mfma_kernel<2, false, true>, dim3(blocks), dim3(THREADS), a);
    return launch_kernel(L, kFamGemm, gemm_mfma_kernel<8, false, true>, dim3(blocks), dim3(THREADS), a);
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
