// Measurement aids of the benchmark, built into a library of their own (libwick_rocm_bench.so): nothing here is part of
// the backend's C ABI and libwick_rocm.{so,a} does not contain it.
//   * Register-only probes that measure this GPU's own ceilings for the two instructions the prefill GEMM is priced
//     against (no memory traffic: operands never leave registers), so that "fraction of peak" can be stated against a
//     measured denominator as well as the datasheet one.
//   * A device-to-device copy of known size (calibration of the memory-traffic counters).
//   * The decode GEMV with the timing hook (gemv_impl.h, SPAN): the product kernel plus two wall-clock reads per wave, for
//     the execution span of launches inside a graph replay.
// Every entry point takes the hipStream_t to enqueue on (wick_rocm_ctx_stream of the backend's context).
#include "gemv_impl.h"
#include "wick_rocm_bench.h"

namespace wick_rocm {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kProbeThreads = 256;
constexpr int kProbeChains = 4;  // independent accumulators per wave, enough to cover the MFMA latency

// SHAPE 0: v_mfma_i32_32x32x32_i8 (65536 ops), 1: v_mfma_i32_16x16x32_i8 (16384 ops),
// 2: v_fma_f32 on 16 independent registers (64 lanes x 2 flops each); 3, 4: probe_mix_kernel below.
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

// The GEMM's block loop without its memory side: per iteration one 32-element block of a wave's 64 x 32 tile, i.e.
// 8 v_mfma_i32_16x16x32_i8 (SHAPE 3) or 2 v_mfma_i32_32x32x32_i8 (SHAPE 4) onto the float-bias constant, and the two
// scaling FMAs of each of the 32 results per lane (per-lane scale registers, the second FMA four instructions behind
// the first).  512-thread workgroups, two per CU: four waves per SIMD, the GEMM's occupancy.
constexpr int kMixThreads = 512;
template <int SHAPE>
__global__ __launch_bounds__(kMixThreads) void probe_mix_kernel(int* sink, uint32_t iters) {
    float acc[32];
#pragma unroll
    for (int i = 0; i < 32; i++) acc[i] = (float)(threadIdx.x + i);
    const float dw = 1e-3f + 1e-9f * (float)threadIdx.x, nb = -12582912.0f * dw, dx = 2e-3f + 1e-9f * (float)threadIdx.x;
    long a8 = (long)threadIdx.x * 0x0101010101010101L;
    const long b8 = 0x0203040506070809L + (long)threadIdx.x;
    v4i c4 = {0x4B400000, 0x4B400000, 0x4B400000, 0x4B400000};
    v16i c16;
#pragma unroll
    for (int r = 0; r < 16; r++) c16[r] = 0x4B400000;
    asm volatile("" : "+v"(c4), "+v"(c16));
    for (uint32_t it = 0; it < iters; it++) {
        int d[32];
        if constexpr (SHAPE == 3) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const v4i r4 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a8 + j, b8, c4, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; r++) d[4 * j + r] = r4[r];
            }
        } else {
            const v4i a4 = {(int)a8, (int)(a8 >> 32), 3, 4}, b4 = {(int)b8, 6, 7, 8};
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const v16i r16 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, b4 + j, c16, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) d[16 * j + r] = r16[r];
            }
        }
#pragma unroll
        for (int g = 0; g < 8; g++) {
            float t[4];
#pragma unroll
            for (int r = 0; r < 4; r++) t[r] = __builtin_fmaf(__int_as_float(d[4 * g + r]), dw, nb);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[4 * g + r] = __builtin_fmaf(t[r], dx, acc[4 * g + r]);
            __builtin_amdgcn_sched_barrier(0);
        }
        a8 += 0x0101;
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) s += acc[i];
    if (s == 123.456f) sink[0] = 1;  // keeps the loop alive, practically never stores
}

static __device__ int probe_sink[16];  // the probes may (practically never do) store here

// One probe launch that fills the chip (8 workgroups of 4 waves per CU); *ops = the operations it performs (int8 ops for the
// MFMA shapes, flops for the FMA one).
hipError_t launch_probe(int shape, uint32_t iters, int num_cus, double* ops, const Launch& L) {
    int* d_sink = nullptr;
    hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&d_sink), HIP_SYMBOL(probe_sink));
    if (e != hipSuccess) return e;
    if (shape >= 3) {  // the block loop: 2 * 64 * 32 * 32 int8 ops per wave and iteration
        const dim3 grid((uint32_t)num_cus * 2u), block(kMixThreads);
        *ops = (double)grid.x * (kMixThreads / 64) * 131072.0 * iters;
        if (shape == 3) return launch_kernel(L, kFamOther, probe_mix_kernel<3>, grid, block, d_sink, iters);
        return launch_kernel(L, kFamOther, probe_mix_kernel<4>, grid, block, d_sink, iters);
    }
    const dim3 grid((uint32_t)num_cus * 8u), block(kProbeThreads);
    const double waves = (double)grid.x * (kProbeThreads / 64);
    const double per_iter = kProbeChains * (shape == 0 ? 65536.0 : shape == 1 ? 16384.0 : 4 * 64 * 2.0);
    *ops = waves * per_iter * iters;
    if (shape == 0) return launch_kernel(L, kFamOther, probe_kernel<0>, grid, block, d_sink, iters);
    if (shape == 1) return launch_kernel(L, kFamOther, probe_kernel<1>, grid, block, d_sink, iters);
    return launch_kernel(L, kFamOther, probe_kernel<2>, grid, block, d_sink, iters);
}

}  // namespace

}  // namespace wick_rocm

using namespace wick_rocm;

extern "C" {

int wick_bench_probe_rate(void* stream, int shape, uint32_t iters, int num_cus, double* ops) {
    if (!ops || shape < 0 || shape > 4 || iters == 0 || num_cus <= 0) return -1;
    return launch_probe(shape, iters, num_cus, ops, Launch{static_cast<hipStream_t>(stream), nullptr}) == hipSuccess ? 0 : -4;
}

int wick_bench_copy(void* stream, void* d_dst, const void* d_src, size_t nbytes) {
    if (!d_dst || !d_src) return -1;
    return hipMemcpyAsync(d_dst, d_src, nbytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)) == hipSuccess ? 0 : -4;
}

int wick_bench_gemv_q8_span(void* stream, int ggml_type, const void* d_w, uint32_t m, uint32_t k, const int8_t* d_quants, const float* d_scales,
                            float* d_y, int num_cus, unsigned long long* d_span, uint32_t span_capacity_waves, uint32_t* waves) {
    if (!d_w || !d_quants || !d_scales || !d_y || !d_span || !waves || m == 0 || k == 0 || k % 64u != 0 || num_cus <= 0) return -1;
    if (ggml_type != kTypeQ4_0 && ggml_type != kTypeQ8_0) return -2;
    // the launch writes one record per wave: refuse a buffer that cannot hold the most waves any split of the rows makes
    if (span_capacity_waves < m) return -1;
    GemvArgs a{};
    a.batch.w[0] = static_cast<const uint8_t*>(d_w), a.batch.y[0] = d_y, a.batch.row_end[0] = m, a.batch.count = 1;
    a.xq = d_quants, a.xs = d_scales;
    a.k = k, a.n = 1;
    a.dots = reinterpret_cast<int32_t*>(d_span);
    const Launch L{static_cast<hipStream_t>(stream), nullptr};
    const hipError_t e = ggml_type == kTypeQ4_0 ? dispatch<2, 1, false, false, true>(a, num_cus, L) : dispatch<8, 1, false, false, true>(a, num_cus, L);
    *waves = a.total_waves;
    return e == hipSuccess ? 0 : -4;
}

}  // extern "C"
