// Parity hook: the exact per-block i32 dots (wick/src/backend/simd.rs:369-383,
// 478-492) computed with the SAME device functions the GEMV uses (pair load,
// funnel shift, nibble unpack, v_dot4_i32_i8, 8*sum(x) correction) and written
// out unscaled: out[(j*m + i)*nb + b].
#include "wick_rocm_device.h"
#include "wick_rocm_internal.h"

namespace wick_rocm {

namespace {

template <int TYPE>
__global__ __launch_bounds__(256) void block_dots_pairs_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ xq,
                                                               uint32_t m, uint32_t n, uint32_t k, int32_t* __restrict__ out) {
    using PT = PairTraits<TYPE>;
    const uint32_t ppr = k >> 6, nb = k >> 5;
    const uint64_t total = (uint64_t)n * m * ppr;
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    const uint32_t p = (uint32_t)(t % ppr);
    const uint32_t i = (uint32_t)((t / ppr) % m);
    const uint32_t j = (uint32_t)(t / ((uint64_t)ppr * m));
    uint32_t wr[PT::DWORDS];
    load_pair<PT::DWORDS>(w + ((size_t)i * ppr + p) * PT::BYTES, wr);
    uint32_t d0, d1, q0[PT::NQ], q1[PT::NQ];
    split_pair<TYPE>(wr, d0, d1, q0, q1);
    const uint32_t* xp = reinterpret_cast<const uint32_t*>(xq + (size_t)j * k + (size_t)p * 64);
    uint32_t x0[8], x1[8];
#pragma unroll
    for (int c = 0; c < 8; c++) x0[c] = xp[c], x1[c] = xp[8 + c];
    int32_t* o = out + ((size_t)j * m + i) * nb + 2 * p;
    o[0] = block_dot<TYPE>(q0, x0, block_xsum(x0));
    o[1] = block_dot<TYPE>(q1, x1, block_xsum(x1));
}

// Odd block counts / unaligned bases: one block per thread, two-byte loads.
template <int TYPE>
__global__ __launch_bounds__(256) void block_dots_generic_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ xq,
                                                                 uint32_t m, uint32_t n, uint32_t k, int32_t* __restrict__ out) {
    constexpr int BB = (TYPE == 2) ? kQ4BlockBytes : kQ8BlockBytes;
    constexpr int NQ = PairTraits<TYPE>::NQ;
    const uint32_t nb = k >> 5;
    const uint64_t total = (uint64_t)n * m * nb;
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    const uint32_t b = (uint32_t)(t % nb);
    const uint32_t i = (uint32_t)((t / nb) % m);
    const uint32_t j = (uint32_t)(t / ((uint64_t)nb * m));
    const uint16_t* hp = reinterpret_cast<const uint16_t*>(w + ((size_t)i * nb + b) * BB);
    uint32_t q[NQ];
#pragma unroll
    for (int c = 0; c < NQ; c++) q[c] = (uint32_t)hp[1 + 2 * c] | ((uint32_t)hp[2 + 2 * c] << 16);
    const uint32_t* xp = reinterpret_cast<const uint32_t*>(xq + (size_t)j * k + (size_t)b * 32);
    uint32_t x[8];
#pragma unroll
    for (int c = 0; c < 8; c++) x[c] = xp[c];
    out[((size_t)j * m + i) * nb + b] = block_dot<TYPE>(q, x, block_xsum(x));
}

}  // namespace

hipError_t launch_block_dots_dot4(int type, const uint8_t* d_w, uint32_t m, uint32_t k, const int8_t* d_q, uint32_t n,
                                  int32_t* d_out, const Launch& L) {
    const uint32_t nb = k >> 5;
    if ((uint64_t)m * n * nb == 0) return hipSuccess;
    const bool pairs = (nb % 2u == 0) && (reinterpret_cast<uintptr_t>(d_w) % 4u == 0);
    const uint64_t total = pairs ? (uint64_t)n * m * (nb / 2) : (uint64_t)n * m * nb;
    const uint32_t blocks = (uint32_t)((total + 255) / 256);
    if (pairs) {
        if (type == kTypeQ4_0)
            return launch_kernel(L, kFamOther, block_dots_pairs_kernel<2>, dim3(blocks), dim3(256), d_w, d_q, m, n, k, d_out);
        else
            return launch_kernel(L, kFamOther, block_dots_pairs_kernel<8>, dim3(blocks), dim3(256), d_w, d_q, m, n, k, d_out);
    } else {
        if (type == kTypeQ4_0)
            return launch_kernel(L, kFamOther, block_dots_generic_kernel<2>, dim3(blocks), dim3(256), d_w, d_q, m, n, k, d_out);
        else
            return launch_kernel(L, kFamOther, block_dots_generic_kernel<8>, dim3(blocks), dim3(256), d_w, d_q, m, n, k, d_out);
    }
    return hipGetLastError();
}

}  // namespace wick_rocm
