// Public launchers of the decode GEMV (kernel and dispatch: gemv_impl.h).
#include "gemv_impl.h"

namespace wick_rocm {

bool pairs_kernel_applies(const GemvBatch& batch, uint32_t k) {
    const uint32_t nb = k >> 5;
    if (nb % 2u != 0 || (nb >> 1) > 128) return false;
    for (uint32_t i = 0; i < batch.count; i++)
        if (reinterpret_cast<uintptr_t>(batch.w[i]) % 4u != 0) return false;
    return true;
}

// f32 activations in, quantized inside the GEMV kernel: one launch instead of two.
hipError_t launch_gemv_f32(int type, const GemvBatch& batch, uint32_t k, const float* d_x, int accumulate, int num_cus,
                           const Launch& L, int xform, const float* d_aux, float eps) {
    GemvArgs a{};
    a.batch = batch;
    a.xf = d_x;
    a.xform = xform, a.xaux = d_aux, a.eps = eps;
    a.x_stride = k;
    a.k = k;
    a.n = 1;
    a.accumulate = accumulate;
    return type == kTypeQ4_0 ? dispatch<2, 1, true>(a, num_cus, L) : dispatch<8, 1, true>(a, num_cus, L);
}

bool gated_kernel_applies(const uint8_t* d_w_gate, const uint8_t* d_w_up, uint32_t k) {
    const uint32_t nb = k >> 5;
    return nb % 2u == 0 && (nb >> 1) <= 64 && reinterpret_cast<uintptr_t>(d_w_gate) % 4u == 0 && reinterpret_cast<uintptr_t>(d_w_up) % 4u == 0;
}

// out[r] = silu(W_gate[r] . x') * (W_up[r] . x'), x' = xform(x) quantized to Q8_0, in one launch.
bool shortconv_kernel_applies(const uint8_t* d_w, uint32_t k, uint32_t kernel_size) {
    const uint32_t nb = k >> 5;
    return kernel_size == 3 && k <= (uint32_t)kConvMaxK && nb % 2u == 0 && reinterpret_cast<uintptr_t>(d_w) % 4u == 0;
}

hipError_t launch_gemv_shortconv_f32(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const float* d_proj, const float* d_state,
                                     const float* d_conv_w, float* d_y, int accumulate, int num_cus, const Launch& L) {
    GemvArgs a{};
    a.batch.w[0] = d_w, a.batch.y[0] = d_y, a.batch.row_end[0] = m, a.batch.count = 1;
    a.xf = d_proj;
    a.xform = kXformShortConv, a.xaux = d_conv_w, a.xaux2 = d_state;
    a.x_stride = k;
    a.k = k;
    a.n = 1;
    a.accumulate = accumulate;
    return type == kTypeQ4_0 ? dispatch<2, 1, true>(a, num_cus, L) : dispatch<8, 1, true>(a, num_cus, L);
}

hipError_t launch_gemv_gated_f32(int type, const uint8_t* d_w_gate, const uint8_t* d_w_up, uint32_t m, uint32_t k, const float* d_x,
                                 float* d_out, int num_cus, const Launch& L, int xform, const float* d_aux, float eps, float* conv_state,
                                 const float* conv_proj, uint32_t conv_hidden, uint32_t conv_kernel) {
    GemvArgs a{};
    a.batch.w[0] = d_w_gate, a.batch.w[1] = d_w_up;
    a.batch.y[0] = d_out;
    a.batch.row_end[0] = m;
    a.batch.count = 1;  // the waves are laid out over the rows of one weight; each handles both
    a.xf = d_x;
    a.xform = xform, a.xaux = d_aux, a.eps = eps, a.gated = 1;
    a.conv_state = conv_state, a.conv_proj = conv_proj, a.conv_hidden = conv_hidden, a.conv_kernel = conv_kernel;
    a.x_stride = k;
    a.k = k;
    a.n = 1;
    return type == kTypeQ4_0 ? dispatch<2, 1, true>(a, num_cus, L) : dispatch<8, 1, true>(a, num_cus, L);
}

hipError_t launch_gemv(int type, const GemvBatch& batch, uint32_t k, const int8_t* d_q, const float* d_scales,
                       int accumulate, int num_cus, const Launch& L) {
    GemvArgs a{};
    a.batch = batch;
    a.xq = d_q;
    a.xs = d_scales;
    a.k = k;
    a.n = 1;
    a.y_stride = 0;
    a.y_row_major = 0;
    a.accumulate = accumulate;
    return type == kTypeQ4_0 ? dispatch<2, 1>(a, num_cus, L) : dispatch<8, 1>(a, num_cus, L);
}

hipError_t launch_gemv_tokens(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q,
                              const float* d_scales, uint32_t n, float* d_y, uint32_t y_stride, int y_layout,
                              int accumulate, int num_cus, const Launch& L) {
    GemvArgs a{};
    a.batch.w[0] = d_w;
    a.batch.y[0] = d_y;
    a.batch.row_end[0] = m;
    a.batch.count = 1;
    a.xq = d_q;
    a.xs = d_scales;
    a.k = k;
    a.n = n;
    a.y_stride = y_stride;
    a.y_row_major = (y_layout == 1);
    a.accumulate = accumulate;
    if (n == 1) return type == kTypeQ4_0 ? dispatch<2, 1>(a, num_cus, L) : dispatch<8, 1>(a, num_cus, L);
    return type == kTypeQ4_0 ? dispatch<2, 4>(a, num_cus, L) : dispatch<8, 4>(a, num_cus, L);
}

}  // namespace wick_rocm
