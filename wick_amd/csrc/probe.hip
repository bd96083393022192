// Register-only probes that measure this GPU's own ceilings for the two instructions the
// prefill GEMM is priced against (no memory traffic: operands never leave registers).
// They exist so that "fraction of peak" can be stated against a measured denominator as
// well as the datasheet one; nothing on the matmul path calls them.
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kProbeThreads = 256;
constexpr int kProbeChains = 4;  // independent accumulators per wave, enough to cover the MFMA latency

// SHAPE 0: v_mfma_i32_32x32x32_i8 (65536 ops), 1: v_mfma_i32_16x16x32_i8 (16384 ops),
// 2: v_fma_f32 on 16 independent registers (64 lanes x 2 flops each).
template <int SHAPE>
__global__ __launch_bounds__(kProbeThreads) void probe_kernel(int* sink, uint32_t iters) {
    v4i a4 = {(int)threadIdx.x, 2, 3, 4}, b4 = {5, 6, (int)threadIdx.x, 8};
    long a8 = (long)threadIdx.x * 0x0101010101010101L, b8 = 0x0203040506070809L + (long)threadIdx.x;
    v16i c[kProbeChains];
    v4i d[kProbeChains];
    float f[16];
#pragma unroll
    for (int i = 0; i < kProbeChains; i++) {
        d[i] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int r = 0; r < 16; r++) c[i][r] = 0;
    }
#pragma unroll
    for (int r = 0; r < 16; r++) f[r] = (float)(threadIdx.x + r);
    const float m = 1.0f + 1e-7f * (float)threadIdx.x, ad = 1e-3f;
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < kProbeChains; i++) {
            if constexpr (SHAPE == 0) c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, b4, c[i], 0, 0, 0);
            if constexpr (SHAPE == 1) d[i] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a8, b8, d[i], 0, 0, 0);
            if constexpr (SHAPE == 2) {
#pragma unroll
                for (int r = 0; r < 4; r++) f[4 * i + r] = __builtin_fmaf(f[4 * i + r], m, ad);
            }
        }
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < kProbeChains; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s += c[i][r];
#pragma unroll
        for (int r = 0; r < 4; r++) s += d[i][r];
    }
#pragma unroll
    for (int r = 0; r < 16; r++) s += (int)f[r];
    if (s == 0x7fffffff) sink[0] = s;  // keeps the loop alive, practically never stores
}

}  // namespace

// Enqueues one probe launch that fills the chip (8 workgroups of 4 waves per CU) and returns
// the number of operations it performs (int8 ops for the MFMA shapes, flops for the FMA one).
hipError_t launch_probe(int shape, uint32_t iters, int num_cus, int* d_sink, double* ops, const Launch& L) {
    const dim3 grid((uint32_t)num_cus * 8u), block(kProbeThreads);
    const double waves = (double)grid.x * (kProbeThreads / 64);
    const double per_iter = kProbeChains * (shape == 0 ? 65536.0 : shape == 1 ? 16384.0 : 4 * 64 * 2.0);
    *ops = waves * per_iter * iters;
    if (shape == 0) return launch_kernel(L, kFamOther, probe_kernel<0>, grid, block, d_sink, iters);
    if (shape == 1) return launch_kernel(L, kFamOther, probe_kernel<1>, grid, block, d_sink, iters);
    return launch_kernel(L, kFamOther, probe_kernel<2>, grid, block, d_sink, iters);
}

}  // namespace wick_rocm
