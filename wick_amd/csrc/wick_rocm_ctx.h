// Context, handle structs and the entry-point prologue shared by the translation units that
// implement the C ABI (api.hip, lfm2_api.hip).  Not installed.
#pragma once

#include <mutex>
#include <string>

#include "../../include/wick_rocm.h"
#include "wick_rocm_internal.h"

using namespace wick_rocm;

struct wick_rocm_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    // Serialises calls on this context, like the reference's infer_lock.  Recursive: the model handle holds it for a whole
    // step or capture while it composes public entry points, which take it again.
    std::recursive_mutex mu;
    std::string err;
    std::string name;
    int num_cus = 0;
    size_t hbm_bytes = 0;
    bool capturing = false;
    // scratch for wick_rocm_matmul_f32 (quantized activations)
    int8_t* scratch_q = nullptr;
    float* scratch_s = nullptr;
    size_t scratch_q_cap = 0;  // bytes
    size_t scratch_s_cap = 0;  // floats
    float* scratch_f = nullptr;  // one transformed f32 activation vector (norm / gate folded into a GEMV that cannot take the fused kernel)
    size_t scratch_f_cap = 0;  // floats
    // A captured graph has the scratch addresses baked in.  Every regrow bumps the generation; a graph that used the
    // scratch remembers the generation it was captured under and refuses to launch under another one.
    // One generation per scratch buffer (quants, scales, K-split partial sums): a graph that only quantizes is not made stale
    // by a larger partial-sum buffer.
    uint64_t scratch_gen[3] = {0, 0, 0};
    unsigned capture_used_scratch = 0;  // bit i: the capture in progress holds the address of scratch buffer i
    bool capture_used_noalloc = false;  // the capture in progress holds a wick_rocm_matmul_f32_noalloc call
    unsigned char* noalloc_scratch = nullptr;  // this device's address of the static scratch array of wick_rocm_matmul_f32_noalloc
    uint32_t gemm_min_n = 0;  // hand-off from the multi-token GEMV to the MFMA GEMM; 0: the per-weight default (min_n_for)
    uint32_t min_n_for(size_t weight_bytes) const {
        return gemm_min_n ? gemm_min_n : (weight_bytes >= kGemmLargeWeightBytes ? kGemmMinNLarge : kGemmMinN);
    }
    bool gemm_packing = true;         // weight_upload also makes the GEMM's own copy of a Q4_0 / Q8_0 weight
    uint32_t gemm_max_splits = kGemmMaxSplits;  // K split of GEMM launches with few tiles (1: off)
    KernelTimer timer;
    int64_t gemv_direct_max_bytes = -1;
    bool gemm_mfma16 = false;  // wick_rocm_set_gemm_mfma_shape(ctx, 16)
    unsigned long long* argmax_partial = nullptr;  // kArgmaxPartials keys for wick_rocm_argmax
    Launch launch() { return Launch{stream, &timer, gemv_direct_max_bytes, gemm_mfma16}; }
};

struct wick_rocm_weight {
    void* d = nullptr;       // the raw blocks, as uploaded: what the decode GEMVs stream
    size_t nbytes = 0;
    void* d_gemm = nullptr;  // the prefill GEMM's own copy (gemm_packed_bytes, see gemm.hip); null: the weight takes the GEMV route for any n
    size_t gemm_bytes = 0;
    int type = 0;
    uint32_t m = 0, k = 0;
};

struct wick_rocm_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    unsigned uses_scratch = 0;             // bit i: some captured launch reads or writes scratch buffer i of the context
    uint64_t scratch_gen[3] = {0, 0, 0};   // ... as they were laid out then
    bool uses_noalloc = false;  // some captured launch uses the GPU's static scratch array (wick_rocm_matmul_f32_noalloc)
};

// True when the graph refers to scratch memory that has been freed and reallocated since its capture.
inline bool graph_is_stale(const wick_rocm_ctx* ctx, const wick_rocm_graph* g) {
    for (int i = 0; i < 3; i++)
        if ((g->uses_scratch >> i & 1u) && g->scratch_gen[i] != ctx->scratch_gen[i]) return true;
    return false;
}

struct wick_rocm_event {
    hipEvent_t ev = nullptr;
};


inline int fail(wick_rocm_ctx* ctx, int code, const char* what) {
    if (ctx) ctx->err = what;
    return code;
}

inline int fail_hip(wick_rocm_ctx* ctx, hipError_t e, const char* where) {
    if (ctx) {
        ctx->err = std::string(where) + ": " + hipGetErrorString(e);
    }
    return WICK_ROCM_ERR_HIP;
}

#define WR_HIP(ctx, call)                                      \
    do {                                                       \
        hipError_t e_ = (call);                                \
        if (e_ != hipSuccess) return fail_hip(ctx, e_, #call); \
    } while (0)

// Takes the context lock and makes its device current for the calling thread.
struct Guard {
    std::unique_lock<std::recursive_mutex> lk;
    hipError_t status;
    explicit Guard(wick_rocm_ctx* ctx) : lk(ctx->mu), status(hipSetDevice(ctx->device)) {}
};

#define WR_ENTER(ctx)                                                   \
    if (!(ctx)) return WICK_ROCM_ERR_INVALID_ARG;                       \
    Guard guard_(ctx);                                                  \
    if (guard_.status != hipSuccess) return fail_hip(ctx, guard_.status, "hipSetDevice")
