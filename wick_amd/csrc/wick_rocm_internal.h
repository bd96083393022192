// Internal declarations shared by the kernel translation units and the C ABI
// layer.  Not installed; the public surface is include/wick_rocm.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wick_rocm {

constexpr int kTypeQ4_0 = 2;  // ggml ids, wick/src/gguf.rs:36-51
constexpr int kTypeQ8_0 = 8;
constexpr int kQ4BlockBytes = 18;  // wick/src/quant.rs:13-20
constexpr int kQ8BlockBytes = 34;  // wick/src/quant.rs:27-34
constexpr int kMaxGemvBatch = 4;

inline int block_bytes(int type) { return type == kTypeQ4_0 ? kQ4BlockBytes : (type == kTypeQ8_0 ? kQ8BlockBytes : 0); }

// Up to kMaxGemvBatch weights that share one quantized activation.  Rows of all
// weights form one concatenated row space [0, row_end[count-1]).
struct GemvBatch {
    const uint8_t* w[kMaxGemvBatch];
    float* y[kMaxGemvBatch];
    uint32_t row_end[kMaxGemvBatch];
    uint32_t count;
};

// Launchers.  All only enqueue on `stream`; callers have validated shapes.
// They return hipGetLastError() after the launch.

hipError_t launch_quantize_q8_0(const float* d_x, uint32_t n, uint32_t k, uint32_t x_stride, int8_t* d_q,
                                float* d_scales, hipStream_t stream);

// Decode GEMV, one token.  k % 32 == 0.
hipError_t launch_gemv(int type, const GemvBatch& batch, uint32_t k, const int8_t* d_q, const float* d_scales,
                       int accumulate, int num_cus, hipStream_t stream);

// Small-n GEMM done as a multi-token GEMV (weights streamed once per 1..kGemvTokens tokens).
hipError_t launch_gemv_tokens(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                              const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                              int accumulate, int num_cus, hipStream_t stream);

// int8-MFMA GEMM.  Requires k % 256 == 0.
hipError_t launch_gemm_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                            const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                            int accumulate, hipStream_t stream);

// Per-block i32 dots, out[(j*m + i)*nb + b], through the same unpack + v_dot4 code
// as the GEMV, or through the GEMM's loads / LDS layout / MFMA (k % 256 == 0).
hipError_t launch_block_dots_dot4(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n,
                                  int32_t* d_out, hipStream_t stream);
hipError_t launch_block_dots_mfma(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n,
                                  int32_t* d_out, hipStream_t stream);

// n at and above which gemm_q8 uses the MFMA kernel (when k % 256 == 0).
constexpr uint32_t kGemmMinN = 16;  // cf. GEMM_MIN_N, wick/src/model/metal_lfm2.rs:18-21

}  // namespace wick_rocm
