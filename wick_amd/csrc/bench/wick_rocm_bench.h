// Entry points of libwick_rocm_bench.so (bench_kernels.hip): measurement aids of bench.py, not part of the backend's C ABI
// (include/wick_rocm.h) and not linked into libwick_rocm.{so,a}.  Return 0 on success, -1 bad argument, -2 bad type,
// -4 HIP error.  `stream`: the hipStream_t to enqueue on (wick_rocm_ctx_stream).
#pragma once
#include <stddef.h>
#include <stdint.h>

extern "C" {
// A register-only kernel that issues one instruction (shape 0 = v_mfma_i32_32x32x32_i8, 1 = v_mfma_i32_16x16x32_i8,
// 2 = v_fma_f32) `iters` x 4 times per wave on every SIMD; shapes 3 / 4: the prefill GEMM's whole block loop from registers
// (one 32-element block of a 64 x 32 tile per wave and iteration = 8 v_mfma_i32_16x16x32_i8 / 2 v_mfma_i32_32x32x32_i8 plus
// the two scaling FMAs of each of the 32 results per lane, at the GEMM's occupancy).  *ops: operations performed.
int wick_bench_probe_rate(void* stream, int shape, uint32_t iters, int num_cus, double* ops);
// Device-to-device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters.
int wick_bench_copy(void* stream, void* d_dst, const void* d_src, size_t nbytes);
// y = W x through the decode GEMV's product kernel with the timing hook: d_span[2 w], d_span[2 w + 1] = 100 MHz wall-clock
// reading at wave w's first instruction / after its last store was acknowledged; *waves = records written.
// d_w: the raw blocks (wick_rocm_weight_device_ptr), k % 64 == 0; span_capacity_waves >= m.
int wick_bench_gemv_q8_span(void* stream, int ggml_type, const void* d_w, uint32_t m, uint32_t k, const int8_t* d_quants, const float* d_scales,
                            float* d_y, int num_cus, unsigned long long* d_span, uint32_t span_capacity_waves, uint32_t* waves);
}
