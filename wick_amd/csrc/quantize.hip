// Q8_0 activation quantizer for gfx950.
//
// Arithmetic of quantize_f32_to_q8_0_neon (wick/src/backend/simd.rs:255-323),
// applied per column as quantize_to_scratch / quantize_columns do
// (wick/src/model/lfm2.rs:571-612).  Bit-exact by construction: every step is one
// correctly rounded IEEE binary32 operation (divide, divide, multiply,
// round-to-nearest-even, f32->f16 RNE), so the order in which amax is reduced is
// the only freedom, and max is associative.
//
// HBM-bound: reads 4*n*k bytes, writes n*k + 4*n*k/32.  Eight lanes own one
// 32-element block (one float4 each); amax is reduced with three lane swaps.
#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

template <bool VEC4>
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float* __restrict__ x, uint32_t n, uint32_t k,
                                                            uint32_t x_stride, int8_t* __restrict__ q,
                                                            float* __restrict__ scales) {
    const uint32_t quads_per_col = k >> 2;  // k % 32 == 0, so groups of 8 lanes never straddle a column
    const uint64_t total = (uint64_t)n * quads_per_col;
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = t < total;
    const uint64_t tt = live ? t : 0;
    const uint32_t col = (uint32_t)(tt / quads_per_col);
    const uint32_t quad = (uint32_t)(tt % quads_per_col);
    const float* src = x + (size_t)col * x_stride + 4u * quad;

    float v0, v1, v2, v3;
    if constexpr (VEC4) {
        float4 v = *reinterpret_cast<const float4*>(src);
        v0 = v.x, v1 = v.y, v2 = v.z, v3 = v.w;
    } else {
        v0 = src[0], v1 = src[1], v2 = src[2], v3 = src[3];
    }

    float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
    amax = group_max8(amax);

    float id;
    const float scale = q8_scale_and_inverse(amax, id);
    const uint32_t packed = q8_pack4(v0, v1, v2, v3, id);
    if (live) {
        *reinterpret_cast<uint32_t*>(q + (size_t)col * k + 4u * quad) = packed;
        if ((quad & 7u) == 0) scales[(size_t)col * (k >> 5) + (quad >> 3)] = scale;
    }
}

}  // namespace

hipError_t launch_quantize_q8_0(const float* d_x, uint32_t n, uint32_t k, uint32_t x_stride, int8_t* d_q,
                                float* d_scales, const Launch& L) {
    const uint64_t total = (uint64_t)n * (k >> 2);
    if (total == 0) return hipSuccess;
    const uint32_t blocks = (uint32_t)((total + 255) / 256);
    const bool vec4 = ((reinterpret_cast<uintptr_t>(d_x) & 15u) == 0) && (x_stride % 4u == 0);
    if (vec4)
        return launch_kernel(L, kFamQuantize, quantize_q8_0_kernel<true>, dim3(blocks), dim3(256), d_x, n, k, x_stride, d_q, d_scales);
    else
        return launch_kernel(L, kFamQuantize, quantize_q8_0_kernel<false>, dim3(blocks), dim3(256), d_x, n, k, x_stride, d_q, d_scales);
    return hipGetLastError();
}

}  // namespace wick_rocm
