// Device-side helpers shared by the GEMV, GEMM and parity-hook kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wick_rocm {

// f16 bit pattern -> f32 (v_cvt_f32_f16; exact, subnormals kept).
__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
    uint16_t b = (uint16_t)bits;
    _Float16 h;
    __builtin_memcpy(&h, &b, 2);
    return (float)h;
}

// 4- and 16-byte vectors that only promise 4-byte alignment, so the compiler may
// still issue one wide global load for them.
struct __attribute__((packed, aligned(4))) u32x4_a4 {
    uint32_t v[4];
};
struct __attribute__((packed, aligned(4))) u32x2_a4 {
    uint32_t v[2];
};

// A "pair" is two consecutive weight blocks of one row: 36 B (Q4_0) or 68 B
// (Q8_0).  Rows hold an even number of blocks on the fast paths, so every pair
// starts 4-byte aligned and is read as whole dwords:
//   dword 0            = [ d0 (f16) | first two quant bytes of block 0 ]
//   dwords 1 .. NQ-1   = block 0 quants, shifted by two bytes
//   dword NQ           = [ last two quant bytes of block 0 | d1 (f16) ]
//   dwords NQ+1 .. 2NQ = block 1 quants, dword aligned
// NQ = quant dwords per block: 4 (Q4_0: 16 nibble bytes) or 8 (Q8_0: 32 int8).
template <int TYPE>
struct PairTraits;
template <>
struct PairTraits<2> {
    static constexpr int NQ = 4;
    static constexpr int DWORDS = 9;
    static constexpr int BYTES = 36;
};
template <>
struct PairTraits<8> {
    static constexpr int NQ = 8;
    static constexpr int DWORDS = 17;
    static constexpr int BYTES = 68;
};

// Native vectors with only 4-byte alignment promised, for the streaming builtin.
typedef uint32_t u32x4_native_a4 __attribute__((ext_vector_type(4), aligned(4)));

// STREAM = true marks the loads nontemporal: a GEMV reads every weight byte exactly
// once, and on MI355X streaming reads that do not allocate in the caches sustain
// about 10 % more HBM bandwidth than ordinary ones.  Tiles that are re-read by
// other workgroups (the GEMM) keep the default policy.
template <int DWORDS, bool STREAM = false>
__device__ __forceinline__ void load_pair(const uint8_t* __restrict__ p, uint32_t (&w)[DWORDS]) {
    static_assert(DWORDS % 4 == 1, "pair = 4*j + 1 dwords");
#pragma unroll
    for (int i = 0; i < DWORDS / 4; i++) {
        if constexpr (STREAM) {
            const u32x4_native_a4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_native_a4*>(p + 16 * i));
            w[4 * i + 0] = t.x;
            w[4 * i + 1] = t.y;
            w[4 * i + 2] = t.z;
            w[4 * i + 3] = t.w;
        } else {
            u32x4_a4 t = *reinterpret_cast<const u32x4_a4*>(p + 16 * i);
            w[4 * i + 0] = t.v[0];
            w[4 * i + 1] = t.v[1];
            w[4 * i + 2] = t.v[2];
            w[4 * i + 3] = t.v[3];
        }
    }
    if constexpr (STREAM) {
        w[DWORDS - 1] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p + 4 * (DWORDS - 1)));
    } else {
        w[DWORDS - 1] = *reinterpret_cast<const uint32_t*>(p + 4 * (DWORDS - 1));
    }
}

// Splits a pair into the two f16 scale bit patterns and the two blocks' quant
// dwords (block 0 needs a two-byte funnel shift, v_alignbyte_b32).
template <int TYPE>
__device__ __forceinline__ void split_pair(const uint32_t (&w)[PairTraits<TYPE>::DWORDS], uint32_t& d0, uint32_t& d1,
                                           uint32_t (&q0)[PairTraits<TYPE>::NQ], uint32_t (&q1)[PairTraits<TYPE>::NQ]) {
    constexpr int NQ = PairTraits<TYPE>::NQ;
    d0 = w[0] & 0xffffu;
    d1 = w[NQ] >> 16;
#pragma unroll
    for (int j = 0; j < NQ; j++) {
        q0[j] = __builtin_amdgcn_alignbyte(w[j + 1], w[j], 2);
        q1[j] = w[NQ + 1 + j];
    }
}

// Exact i32 dot of one weight block with one Q8_0 activation block (8 dwords of
// int8: x[0..3] = elements 0..15, x[4..7] = elements 16..31).
//
// Q4_0 (wick/src/quant.rs:82-88): byte i of qs holds element i in its low nibble
// and element i+16 in its high nibble, value = nibble - 8.  The unsigned nibbles
// are dotted as they are and 8 * sum(x) is subtracted once; `xsum` is that
// block's sum of activation quants.
__device__ __forceinline__ int block_dot_q4_0(const uint32_t (&q)[4], const uint32_t (&x)[8], int xsum) {
    int s = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t lo = q[j] & 0x0f0f0f0fu;
        uint32_t hi = (q[j] >> 4) & 0x0f0f0f0fu;
        s = __builtin_amdgcn_sdot4((int)lo, (int)x[j], s, false);
        s = __builtin_amdgcn_sdot4((int)hi, (int)x[4 + j], s, false);
    }
    return s - 8 * xsum;
}

__device__ __forceinline__ int block_dot_q8_0(const uint32_t (&q)[8], const uint32_t (&x)[8]) {
    int s = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) s = __builtin_amdgcn_sdot4((int)q[j], (int)x[j], s, false);
    return s;
}

__device__ __forceinline__ int block_xsum(const uint32_t (&x)[8]) {
    int s = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) s = __builtin_amdgcn_sdot4(0x01010101, (int)x[j], s, false);
    return s;
}

template <int TYPE>
__device__ __forceinline__ int block_dot(const uint32_t (&q)[PairTraits<TYPE>::NQ], const uint32_t (&x)[8], int xsum) {
    if constexpr (TYPE == 2) {
        return block_dot_q4_0(q, x, xsum);
    } else {
        (void)xsum;
        return block_dot_q8_0(q, x);
    }
}

// Q8_0 activation quantization arithmetic shared by the stand-alone quantizer and the
// fused GEMV (quantize_f32_to_q8_0_neon, wick/src/backend/simd.rs:255-323): d = amax/127,
// id = 1/d from the unrounded d, stored scale = f32(f16(d)),
// q = (i8)(i32) round-ties-even(x * id).  Every step is one correctly rounded
// binary32 operation.
__device__ __forceinline__ float q8_scale_and_inverse(float amax, float& id) {
    const float d = __fdiv_rn(amax, 127.0f);
    id = (d != 0.0f) ? __fdiv_rn(1.0f, d) : 0.0f;
    return (float)(_Float16)d;
}

__device__ __forceinline__ uint32_t q8_pack4(float v0, float v1, float v2, float v3, float id) {
    const int q0 = (int)__builtin_rintf(__fmul_rn(v0, id));
    const int q1 = (int)__builtin_rintf(__fmul_rn(v1, id));
    const int q2 = (int)__builtin_rintf(__fmul_rn(v2, id));
    const int q3 = (int)__builtin_rintf(__fmul_rn(v3, id));
    return (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) | ((uint32_t)(q3 & 0xff) << 24);
}

// Sum over groups of WIDTH consecutive lanes (WIDTH a power of two <= 64); every
// lane of a group ends with the group's total.  Within a row of 16 lanes the four
// butterfly steps are DPP operand modifiers on the add itself (no LDS crossbar, no
// wait): xor 1 and xor 2 as quad permutes, then the two mirror patterns, which
// complete the 8- and 16-lane sums because the smaller groups are already uniform.
// Only the 32- and 64-lane steps go through ds_bpermute.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
    return v + __builtin_bit_cast(float, moved);
}

// Maximum over groups of 8 consecutive lanes (the eight lanes that share one 32-element
// activation block in the quantizers), same three DPP steps, no LDS crossbar.
__device__ __forceinline__ float group_max8(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false)));
    return v;
}

template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (WIDTH >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    if constexpr (WIDTH >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if constexpr (WIDTH >= 8) v = dpp_add<0x141>(v);  // row_half_mirror
    if constexpr (WIDTH >= 16) v = dpp_add<0x140>(v); // row_mirror
    if constexpr (WIDTH >= 32) v += __shfl_xor(v, 16, 64);
    if constexpr (WIDTH >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// The same for a double over the whole wave, every lane gets the total: four DPP steps inside the rows of 16 lanes
// (each moves the two halves of the double), then the four row totals through scalar registers.  A butterfly of
// 64-bit shuffles costs twelve trips through the LDS crossbar, which is most of an RMSNorm prologue.
template <int CTRL>
__device__ __forceinline__ double dpp_add_f64(double v) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, 0xf, 0xf, false);
    return v + __hiloint2double(hi, lo);
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    v = dpp_add_f64<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add_f64<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add_f64<0x141>(v);  // row_half_mirror
    v = dpp_add_f64<0x140>(v);  // row_mirror: every lane of a row holds the row's sum
    const int lo = __double2loint(v), hi = __double2hiint(v);
    const double r0 = __hiloint2double(__builtin_amdgcn_readlane(hi, 0), __builtin_amdgcn_readlane(lo, 0));
    const double r1 = __hiloint2double(__builtin_amdgcn_readlane(hi, 16), __builtin_amdgcn_readlane(lo, 16));
    const double r2 = __hiloint2double(__builtin_amdgcn_readlane(hi, 32), __builtin_amdgcn_readlane(lo, 32));
    const double r3 = __hiloint2double(__builtin_amdgcn_readlane(hi, 48), __builtin_amdgcn_readlane(lo, 48));
    return (r0 + r1) + (r2 + r3);
}

// f32 sum / maximum over the whole wave, every lane gets the result: DPP inside the rows, row results through scalar
// registers.
__device__ __forceinline__ float wave_sum_f32(float v) {
    v = group_sum<16>(v);
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    return fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false)));
}
__device__ __forceinline__ float wave_max_f32(float v) {
    v = dpp_max<0xB1>(v), v = dpp_max<0x4E>(v), v = dpp_max<0x141>(v), v = dpp_max<0x140>(v);
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// The greedy pick's ordering (cpu_argmax, wick/src/sampler.rs:7-19) as one unsigned key: NaN counts as -inf, values order
// by f32::total_cmp, and of equal values the larger index wins; 0 is below every real key.
__device__ __forceinline__ unsigned long long argmax_key(float f, uint32_t index) {
    if (f != f) f = -__builtin_inff();
    int32_t b = (int32_t)__float_as_uint(f);
    b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);                 // total_cmp's transform: signed order
    const uint32_t ordered = (uint32_t)b ^ 0x80000000u;          // ... as unsigned order
    return ((unsigned long long)ordered << 32) | index;          // equal values: the larger index wins
}

__device__ __forceinline__ float bits_f(uint32_t u) { return __uint_as_float(u); }

// ggml_expf (wick/src/backend/cpu.rs:604-652), operation for operation: bit-exact.
__device__ __forceinline__ float ggml_expf(float x) {
    const float R = bits_f(0x4B400000u), LOG2E = bits_f(0x3FB8AA3Bu);
    const float LN2_HI = bits_f(0x3F317200u), LN2_LO = bits_f(0x35BFBE8Eu);
    const float C1 = bits_f(0x3F7FFFF6u), C2 = bits_f(0x3EFFFEDBu), C3 = bits_f(0x3E2AAF33u);
    const float C4 = bits_f(0x3D2B9F17u), C5 = bits_f(0x3C072010u);
    const float z = __fadd_rn(R, __fmul_rn(x, LOG2E));
    const float n = __fsub_rn(z, R);
    const float b = __fsub_rn(__fsub_rn(x, __fmul_rn(n, LN2_HI)), __fmul_rn(n, LN2_LO));
    const uint32_t e = __float_as_uint(z) << 23;
    const float k = bits_f(e + 0x3F800000u);
    const float u = __fmul_rn(b, b);
    const float inner = __fadd_rn(__fadd_rn(C2, __fmul_rn(C3, b)), __fmul_rn(__fadd_rn(C4, __fmul_rn(C5, b)), u));
    const float j = __fadd_rn(__fmul_rn(C1, b), __fmul_rn(inner, u));
    const float abs_n = fabsf(n);
    if (abs_n <= 126.0f) return __fadd_rn(k, __fmul_rn(j, k));
    if (abs_n > 192.0f) return n > 0.0f ? __builtin_inff() : 0.0f;
    const uint32_t d = n <= 0.0f ? 0x82000000u : 0u;
    const float s1 = bits_f(d + 0x7f000000u);
    const float s2 = bits_f(e - d);
    return __fmul_rn(__fadd_rn(s2, __fmul_rn(s2, j)), s1);
}

// silu_mul_inplace's element (wick/src/backend/cpu.rs:668-673): g / (1 + expf(-g)) * u, bit-exact.
__device__ __forceinline__ float silu_mul(float g, float u) { return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, ggml_expf(-g))), u); }

}  // namespace wick_rocm
