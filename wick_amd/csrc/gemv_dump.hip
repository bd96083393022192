// Parity hook of the decode GEMV: the DUMP instantiations of the product kernels (gemv_impl.h), kept in a translation
// unit of their own so that they compile next to the product variants instead of after them.
#include "gemv_impl.h"

namespace wick_rocm {

// out[(j*m + i)*nb + b]: the exact i32 dot of block b of row i against token j's quants, through the GEMV kernel that a
// product launch of this shape, token count and fetch policy runs.
hipError_t launch_block_dots_gemv(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n, int32_t* d_out,
                                  int num_cus, const Launch& L) {
    GemvArgs a{};
    a.batch.w[0] = d_w;
    a.batch.row_end[0] = m;
    a.batch.count = 1;
    a.xq = d_q;
    a.k = k;
    a.n = n;
    a.dots = d_out;
    if (n == 1) return type == kTypeQ4_0 ? dispatch<2, 1, false, true>(a, num_cus, L) : dispatch<8, 1, false, true>(a, num_cus, L);
    return type == kTypeQ4_0 ? dispatch<2, 4, false, true>(a, num_cus, L) : dispatch<8, 4, false, true>(a, num_cus, L);
}

// The same for the fused variant: one f32 activation vector, quantized to Q8_0 inside the kernel.  Callers have checked
// pairs_kernel_applies() and the 16-byte alignment of d_x.
hipError_t launch_block_dots_gemv_f32(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const float* d_x, int32_t* d_out, int num_cus,
                                      const Launch& L) {
    GemvArgs a{};
    a.batch.w[0] = d_w;
    a.batch.row_end[0] = m;
    a.batch.count = 1;
    a.xf = d_x;
    a.x_stride = k;
    a.k = k;
    a.n = 1;
    a.dots = d_out;
    return type == kTypeQ4_0 ? dispatch<2, 1, true, true>(a, num_cus, L) : dispatch<8, 1, true, true>(a, num_cus, L);
}

}  // namespace wick_rocm
