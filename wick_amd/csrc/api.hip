// C ABI of the gfx950 backend (see include/wick_rocm.h for the contract and the
// reference interfaces each entry point stands in for).  Host code only: argument
// validation, ownership, stream / graph / event plumbing, kernel routing.
#include "../../include/wick_rocm.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>

#include "wick_rocm_ctx.h"
#include "../../include/wick_gguf.h"

// Scratch of wick_rocm_matmul_f32_noalloc: the Q8_0-quantized activations (quants, then scales) of one call, in
// device memory that exists from load time on, one copy per GPU.  `scratch` is a host-side stand-in for the symbol, not a
// device address: host code only ever uses the address hipGetSymbolAddress returns for the current device
// (wick_rocm_ctx::noalloc_scratch, looked up in wick_rocm_ctx_create).
constexpr size_t kNoallocMaxElems = 4u << 20;  // n * k of one call: 4 Mi quants (4 MiB) + 128 Ki scales (512 KiB)
constexpr size_t kNoallocScratchBytes = kNoallocMaxElems + kNoallocMaxElems / 32 * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kNoallocScratchBytes];

namespace {

// Every context on a GPU shares that GPU's one array, and nothing orders the streams of two contexts.  The host therefore
// keeps, per device, the context whose calls (or graph replays of them) may still be using the array: a call from another
// context is refused until the owner has synchronised (wick_rocm_sync, a download, destruction), which is when its work on
// the array is known to have finished.
constexpr int kNoallocMaxDevices = 64;
std::mutex g_noalloc_mu;
wick_rocm_ctx* g_noalloc_owner[kNoallocMaxDevices] = {};

int noalloc_claim(wick_rocm_ctx* ctx) {
    if (ctx->device < 0 || ctx->device >= kNoallocMaxDevices) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32_noalloc: device index out of range");
    std::lock_guard<std::mutex> lk(g_noalloc_mu);
    wick_rocm_ctx*& owner = g_noalloc_owner[ctx->device];
    if (owner && owner != ctx)
        return fail(ctx, WICK_ROCM_ERR_STATE, "matmul_f32_noalloc: another context's work on this GPU's static scratch may still be in flight; "
                                              "wick_rocm_sync that context first");
    owner = ctx;
    return WICK_ROCM_OK;
}

// The context's stream has drained (or the context goes away): whatever it enqueued on the array has finished.
void noalloc_release(wick_rocm_ctx* ctx) {
    if (ctx->device < 0 || ctx->device >= kNoallocMaxDevices) return;
    std::lock_guard<std::mutex> lk(g_noalloc_mu);
    if (g_noalloc_owner[ctx->device] == ctx) g_noalloc_owner[ctx->device] = nullptr;
}

int check_weight(wick_rocm_ctx* ctx, const wick_rocm_weight* w) {
    if (!w || !w->d) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "null weight handle");
    return WICK_ROCM_OK;
}

int ensure_scratch(wick_rocm_ctx* ctx, size_t q_bytes, size_t s_floats, size_t f_floats = 0) {
    // the graph being captured will hold the addresses of the buffers this call asks for
    if (ctx->capturing) ctx->capture_used_scratch |= (q_bytes ? 1u : 0u) | (s_floats ? 2u : 0u) | (f_floats ? 4u : 0u);
    if (q_bytes <= ctx->scratch_q_cap && s_floats <= ctx->scratch_s_cap && f_floats <= ctx->scratch_f_cap) return WICK_ROCM_OK;
    if (ctx->capturing)
        return fail(ctx, WICK_ROCM_ERR_STATE, "activation scratch too small during graph capture; call wick_rocm_reserve_scratch first");
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));  // earlier launches may still read the old scratch
    // graphs captured against a buffer that moves are stale from here on (wick_rocm_graph_launch refuses them)
    if (q_bytes > ctx->scratch_q_cap) ctx->scratch_gen[0]++;
    if (s_floats > ctx->scratch_s_cap) ctx->scratch_gen[1]++;
    if (f_floats > ctx->scratch_f_cap) ctx->scratch_gen[2]++;
    if (q_bytes > ctx->scratch_q_cap) {
        if (ctx->scratch_q) WR_HIP(ctx, hipFree(ctx->scratch_q));
        ctx->scratch_q = nullptr, ctx->scratch_q_cap = 0;
        WR_HIP(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->scratch_q), q_bytes));
        ctx->scratch_q_cap = q_bytes;
    }
    if (s_floats > ctx->scratch_s_cap) {
        if (ctx->scratch_s) WR_HIP(ctx, hipFree(ctx->scratch_s));
        ctx->scratch_s = nullptr, ctx->scratch_s_cap = 0;
        WR_HIP(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->scratch_s), s_floats * sizeof(float)));
        ctx->scratch_s_cap = s_floats;
    }
    if (f_floats > ctx->scratch_f_cap) {
        if (ctx->scratch_f) WR_HIP(ctx, hipFree(ctx->scratch_f));
        ctx->scratch_f = nullptr, ctx->scratch_f_cap = 0;
        WR_HIP(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->scratch_f), f_floats * sizeof(float)));
        ctx->scratch_f_cap = f_floats;
    }
    return WICK_ROCM_OK;
}

// Routing shared by wick_rocm_gemm_q8 and wick_rocm_matmul_f32 (lock already held).
// may_split: the call may take the K-split launch pair, whose partial sums live in context scratch (never the entry point
// that must not allocate, never during a capture that has not reserved the room).
// deferred (may be null): when given and the launch is split, the shares are left in ctx->scratch_f for the caller's next
// kernel to add up (*deferred = their number); otherwise *deferred = 0 and y is complete.
int gemm_locked(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const int8_t* d_q, const float* d_s, uint32_t n,
                float* d_y, uint32_t y_stride, int y_layout, int accumulate, bool may_split = true, uint32_t* deferred = nullptr) {
    if (deferred) *deferred = 0;
    if (!d_q || !d_s || !d_y) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "null device pointer");
    if (n == 0) return WICK_ROCM_OK;
    if (y_layout != WICK_ROCM_LAYOUT_TOKEN_MAJOR && y_layout != WICK_ROCM_LAYOUT_ROW_MAJOR)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "unknown output layout");
    if (y_layout == WICK_ROCM_LAYOUT_TOKEN_MAJOR ? (y_stride < w->m && n > 1) : (y_stride < n))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "y_stride smaller than the output extent");
    if (w->type == kTypeQ6_K) {  // no batched kernel for Q6_K: one GEMV per token (the LM head sees one or a few)
        if (reinterpret_cast<uintptr_t>(d_q) % 16u != 0) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "Q6_K gemm: quants must be 16-byte aligned");
        const bool tm = y_layout == WICK_ROCM_LAYOUT_TOKEN_MAJOR;
        for (uint32_t j = 0; j < n; j++) {
            hipError_t e = launch_gemv_q6k(static_cast<const uint8_t*>(w->d), w->m, w->k, d_q + (size_t)j * w->k, d_s + (size_t)j * (w->k / 32u),
                                           tm ? d_y + (size_t)j * y_stride : d_y + j, tm ? 1u : y_stride, accumulate, ctx->num_cus, ctx->launch());
            if (e != hipSuccess) return fail_hip(ctx, e, "Q6_K gemv launch");
        }
        return WICK_ROCM_OK;
    }
    const bool mfma_ok = w->d_gemm && (w->k % 128u == 0) && (reinterpret_cast<uintptr_t>(d_q) % 16u == 0) &&
                         (reinterpret_cast<uintptr_t>(d_s) % 16u == 0);
    hipError_t e;
    if (n >= ctx->min_n_for(w->nbytes) && mfma_ok) {
        uint32_t splits = may_split && ctx->gemm_max_splits > 1 ? gemm_split_k(w->m, n, w->k, ctx->gemm_max_splits) : 1u;
        if (splits > 1) {
            const size_t floats = (size_t)splits * n * w->m;
            if (ctx->capturing && floats > ctx->scratch_f_cap) splits = 1;  // no room reserved: the unsplit launch, same result to the f32 bar
            else if (int rc = ensure_scratch(ctx, 0, 0, floats)) return rc;
        }
        const bool defer = deferred && splits > 1;
        e = launch_gemm_mfma(w->type, static_cast<const uint8_t*>(w->d_gemm), w->m, w->k, d_q, d_s, n, d_y, y_stride,
                             y_layout, accumulate, ctx->launch(), splits, splits > 1 ? ctx->scratch_f : nullptr, defer);
        if (defer && e == hipSuccess) *deferred = splits;
    } else
        e = launch_gemv_tokens(w->type, static_cast<const uint8_t*>(w->d), w->m, w->k, d_q, d_s, n, d_y, y_stride,
                               y_layout, accumulate, ctx->num_cus, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "gemm launch");
    return WICK_ROCM_OK;
}

}  // namespace

extern "C" {

const char* wick_rocm_version(void) { return "wick-rocm 0.1 (gfx950)"; }

int wick_rocm_device_count(int* count) {
    if (!count) return WICK_ROCM_ERR_INVALID_ARG;
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess) {
        *count = 0;
        return e == hipErrorNoDevice ? WICK_ROCM_OK : WICK_ROCM_ERR_HIP;
    }
    *count = c;
    return WICK_ROCM_OK;
}

int wick_rocm_ctx_create(int device_id, wick_rocm_ctx** out) {
    if (!out) return WICK_ROCM_ERR_INVALID_ARG;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device_id < 0 || device_id >= count) return WICK_ROCM_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_id) != hipSuccess) return WICK_ROCM_ERR_HIP;
    // The kernels are built for gfx950 only; refuse anything else up front instead
    // of failing at the first launch.
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) return WICK_ROCM_ERR_NO_DEVICE;
    wick_rocm_ctx* ctx = new (std::nothrow) wick_rocm_ctx();
    if (!ctx) return WICK_ROCM_ERR_HIP;
    ctx->device = device_id;
    ctx->name = std::string(prop.gcnArchName) + " " + prop.name;
    ctx->num_cus = prop.multiProcessorCount;
    ctx->hbm_bytes = prop.totalGlobalMem;
    if (hipSetDevice(device_id) != hipSuccess || hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
        delete ctx;
        return WICK_ROCM_ERR_HIP;
    }
    // This device's copy of the static scratch array (every GPU has its own, at its own address); the device is current.
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) {
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return WICK_ROCM_ERR_HIP;
    }
    ctx->noalloc_scratch = static_cast<unsigned char*>(sym);
    *out = ctx;
    return WICK_ROCM_OK;
}

void wick_rocm_ctx_destroy(wick_rocm_ctx* ctx) {
    if (!ctx) return;
    {
        Guard g(ctx);
        if (ctx->stream) {
            (void)hipStreamSynchronize(ctx->stream);
            (void)hipStreamDestroy(ctx->stream);
        }
        noalloc_release(ctx);
        if (ctx->scratch_q) (void)hipFree(ctx->scratch_q);
        if (ctx->scratch_s) (void)hipFree(ctx->scratch_s);
        if (ctx->scratch_f) (void)hipFree(ctx->scratch_f);
        if (ctx->argmax_partial) (void)hipFree(ctx->argmax_partial);
        for (auto* v : {&ctx->timer.recs, &ctx->timer.spares})
            for (KernelTimer::Rec& r : *v) {
                (void)hipEventDestroy(r.start);
                (void)hipEventDestroy(r.stop);
            }
    }
    delete ctx;
}

int wick_rocm_last_error(wick_rocm_ctx* ctx, char* buf, size_t buf_len) {
    if (!ctx || !buf || buf_len == 0) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::recursive_mutex> lk(ctx->mu);
    std::snprintf(buf, buf_len, "%s", ctx->err.c_str());
    return WICK_ROCM_OK;
}

int wick_rocm_device_info(wick_rocm_ctx* ctx, char* name_buf, size_t name_len, int* compute_units, size_t* hbm_bytes) {
    if (!ctx) return WICK_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::recursive_mutex> lk(ctx->mu);
    if (name_buf && name_len) std::snprintf(name_buf, name_len, "%s", ctx->name.c_str());
    if (compute_units) *compute_units = ctx->num_cus;
    if (hbm_bytes) *hbm_bytes = ctx->hbm_bytes;
    return WICK_ROCM_OK;
}

void* wick_rocm_ctx_stream(wick_rocm_ctx* ctx) { return ctx ? static_cast<void*>(ctx->stream) : nullptr; }

int wick_rocm_buffer_alloc(wick_rocm_ctx* ctx, size_t nbytes, void** d_ptr) {
    WR_ENTER(ctx);
    if (!d_ptr || nbytes == 0) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "buffer_alloc: null out pointer or zero size");
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "buffer_alloc during graph capture");
    *d_ptr = nullptr;
    WR_HIP(ctx, hipMalloc(d_ptr, nbytes));
    return WICK_ROCM_OK;
}

int wick_rocm_buffer_free(wick_rocm_ctx* ctx, void* d_ptr) {
    WR_ENTER(ctx);
    if (!d_ptr) return WICK_ROCM_OK;
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "buffer_free during graph capture");
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    WR_HIP(ctx, hipFree(d_ptr));
    return WICK_ROCM_OK;
}

int wick_rocm_upload(wick_rocm_ctx* ctx, void* d_dst, const void* src, size_t nbytes) {
    WR_ENTER(ctx);
    if (nbytes == 0) return WICK_ROCM_OK;
    if (!d_dst || !src) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "upload: null pointer");
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "upload during graph capture");
    WR_HIP(ctx, hipMemcpyAsync(d_dst, src, nbytes, hipMemcpyHostToDevice, ctx->stream));
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));  // the host buffer may be reused on return
    return WICK_ROCM_OK;
}

int wick_rocm_download(wick_rocm_ctx* ctx, void* dst, const void* d_src, size_t nbytes) {
    WR_ENTER(ctx);
    if (nbytes == 0) return WICK_ROCM_OK;
    if (!dst || !d_src) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "download: null pointer");
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "download during graph capture");
    WR_HIP(ctx, hipMemcpyAsync(dst, d_src, nbytes, hipMemcpyDeviceToHost, ctx->stream));
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    noalloc_release(ctx);
    return WICK_ROCM_OK;
}

int wick_rocm_set_gemv_policy(wick_rocm_ctx* ctx, int64_t direct_max_bytes) {
    WR_ENTER(ctx);
    ctx->gemv_direct_max_bytes = direct_max_bytes < 0 ? -1 : direct_max_bytes;
    return WICK_ROCM_OK;
}

int wick_rocm_set_gemm_max_k_splits(wick_rocm_ctx* ctx, uint32_t max_splits) {
    WR_ENTER(ctx);
    ctx->gemm_max_splits = max_splits == 0 ? kGemmMaxSplits : (max_splits > 8 ? 8u : max_splits);
    return WICK_ROCM_OK;
}

int wick_rocm_set_gemm_packing(wick_rocm_ctx* ctx, int enabled) {
    WR_ENTER(ctx);
    ctx->gemm_packing = enabled != 0;
    return WICK_ROCM_OK;
}

size_t wick_rocm_weight_device_bytes(const wick_rocm_weight* w) { return w ? w->nbytes + w->gemm_bytes : 0; }

int wick_rocm_set_gemm_mfma_shape(wick_rocm_ctx* ctx, int shape) {
    WR_ENTER(ctx);
    if (shape != 0 && shape != 16 && shape != 32) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "set_gemm_mfma_shape: 0 (default), 16 or 32");
    ctx->gemm_mfma16 = shape == 16;
    return WICK_ROCM_OK;
}

int wick_rocm_set_gemm_min_n(wick_rocm_ctx* ctx, uint32_t min_n) {
    WR_ENTER(ctx);
    ctx->gemm_min_n = min_n;  // 0: back to the per-weight default
    return WICK_ROCM_OK;
}

int wick_rocm_sync(wick_rocm_ctx* ctx) {
    WR_ENTER(ctx);
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "sync during graph capture");
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    noalloc_release(ctx);
    return WICK_ROCM_OK;
}

int wick_rocm_weight_upload(wick_rocm_ctx* ctx, const void* host_blocks, size_t nbytes, int ggml_type, uint32_t m,
                            uint32_t k, wick_rocm_weight** out) {
    WR_ENTER(ctx);
    if (!out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "weight_upload: null out pointer");
    *out = nullptr;
    if (!host_blocks) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "weight_upload: null host pointer");
    if (ggml_type == kTypeQ6_K) {
        if (m == 0 || k == 0 || k % 256u != 0 || k > 8192u)
            return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "weight_upload: Q6_K needs m > 0 and k a multiple of 256, at most 8192");
        if (nbytes != (size_t)m * (k / 256u) * (size_t)kQ6KBlockBytes)
            return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "weight_upload: nbytes != m * (k/256) * 210");
    } else {
        const int bb = block_bytes(ggml_type);
        if (bb == 0)
            return fail(ctx, WICK_ROCM_ERR_UNSUPPORTED_DTYPE, "weight_upload: only Q4_0 (2), Q8_0 (8) and Q6_K (14) are supported");
        if (m == 0 || k == 0 || k % 32u != 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "weight_upload: m, k must be > 0 and k % 32 == 0");
        if (nbytes != (size_t)m * (k / 32u) * (size_t)bb)
            return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "weight_upload: nbytes != m * (k/32) * block_bytes");
    }
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "weight_upload during graph capture");
    wick_rocm_weight* w = new (std::nothrow) wick_rocm_weight();
    if (!w) return fail(ctx, WICK_ROCM_ERR_HIP, "out of host memory");
    // (+64: the Q6_K kernel reads its last 16-byte piece whole)
    hipError_t e = hipMalloc(&w->d, nbytes + 64);
    if (e == hipSuccess) e = hipMemcpyAsync(w->d, host_blocks, nbytes, hipMemcpyHostToDevice, ctx->stream);
    // The prefill GEMM reads its own layout of the weight (see gemm.hip): made here, once, on the device.  Weights the GEMM does
    // not take (Q6_K, k % 128 != 0) or uploaded with packing switched off keep the raw blocks only and run as GEMVs for any n.
    if (e == hipSuccess && ctx->gemm_packing && ggml_type != kTypeQ6_K && k % 128u == 0) {
        w->gemm_bytes = gemm_packed_bytes(m, k);
        e = hipMalloc(&w->d_gemm, w->gemm_bytes);
        if (e == hipErrorOutOfMemory) {  // no room for the second layout: the weight works without it (GEMV route for any n)
            (void)hipGetLastError();
            w->d_gemm = nullptr, w->gemm_bytes = 0;
            e = hipSuccess;
        } else if (e == hipSuccess) {
            e = launch_gemm_pack(ggml_type, static_cast<const uint8_t*>(w->d), m, k, static_cast<uint8_t*>(w->d_gemm), ctx->launch());
        }
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        if (w->d) (void)hipFree(w->d);
        if (w->d_gemm) (void)hipFree(w->d_gemm);
        delete w;
        return fail_hip(ctx, e, "weight_upload");
    }
    w->nbytes = nbytes, w->type = ggml_type, w->m = m, w->k = k;
    *out = w;
    return WICK_ROCM_OK;
}

int wick_rocm_weight_from_gguf(wick_rocm_ctx* ctx, const wick_gguf* gguf, const char* tensor_name, wick_rocm_weight** out) {
    WR_ENTER(ctx);
    if (!gguf || !tensor_name || !out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "weight_from_gguf: null argument");
    uint64_t offset = 0, rows = 0, cols = 0;
    int type = 0;
    const void* bytes = nullptr;
    size_t nbytes = 0;
    if (wick_gguf_tensor_meta(gguf, tensor_name, &offset, &rows, &cols, &type) != 0 ||
        wick_gguf_tensor_data(gguf, tensor_name, &bytes, &nbytes) != 0)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, (std::string("weight_from_gguf: ") + wick_gguf_last_error()).c_str());
    if (rows > UINT32_MAX || cols > UINT32_MAX) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "weight_from_gguf: dimension exceeds 32 bits");
    return wick_rocm_weight_upload(ctx, bytes, nbytes, type, (uint32_t)rows, (uint32_t)cols, out);
}

int wick_rocm_weight_free(wick_rocm_ctx* ctx, wick_rocm_weight* w) {
    WR_ENTER(ctx);
    if (!w) return WICK_ROCM_OK;
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "weight_free during graph capture");
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (w->d) WR_HIP(ctx, hipFree(w->d));
    if (w->d_gemm) WR_HIP(ctx, hipFree(w->d_gemm));
    delete w;
    return WICK_ROCM_OK;
}

int wick_rocm_weight_info(const wick_rocm_weight* w, int* ggml_type, uint32_t* m, uint32_t* k, size_t* nbytes) {
    if (!w) return WICK_ROCM_ERR_INVALID_ARG;
    if (ggml_type) *ggml_type = w->type;
    if (m) *m = w->m;
    if (k) *k = w->k;
    if (nbytes) *nbytes = w->nbytes;
    return WICK_ROCM_OK;
}

const void* wick_rocm_weight_device_ptr(const wick_rocm_weight* w) { return w ? w->d : nullptr; }

int wick_rocm_quantize_q8_0(wick_rocm_ctx* ctx, const float* d_x, uint32_t n, uint32_t k, uint32_t x_stride,
                            int8_t* d_quants, float* d_scales) {
    WR_ENTER(ctx);
    if (n == 0) return WICK_ROCM_OK;
    if (!d_x || !d_quants || !d_scales) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "quantize_q8_0: null device pointer");
    if (k == 0 || k % 32u != 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "quantize_q8_0: k % 32 != 0");
    if (x_stride < k && n > 1) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "quantize_q8_0: x_stride < k");
    if (reinterpret_cast<uintptr_t>(d_x) % 4u || reinterpret_cast<uintptr_t>(d_quants) % 4u ||
        reinterpret_cast<uintptr_t>(d_scales) % 4u)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "quantize_q8_0: pointers must be 4-byte aligned");
    hipError_t e = launch_quantize_q8_0(d_x, n, k, x_stride, d_quants, d_scales, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "quantize_q8_0 launch");
    return WICK_ROCM_OK;
}

namespace {

// Validates a group of weights sharing one activation and fills the launch batch.
int make_batch(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count, GemvBatch& b) {
    if (!ws || !d_ys) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv: null pointer");
    if (count == 0 || count > (uint32_t)kMaxGemvBatch) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv multi: count must be 1..4");
    uint32_t rows = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (int rc = check_weight(ctx, ws[i])) return rc;
        if (!d_ys[i]) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv: null output pointer");
        if (ws[i]->k != ws[0]->k || ws[i]->type != ws[0]->type)
            return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "gemv multi: weights must share k and dtype");
        if ((uint64_t)rows + ws[i]->m > 0xffffffffull) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "gemv multi: too many rows");
        rows += ws[i]->m;
        b.w[i] = static_cast<const uint8_t*>(ws[i]->d);
        b.y[i] = d_ys[i];
        b.row_end[i] = rows;
    }
    b.count = count;
    return WICK_ROCM_OK;
}

// Q6_K weights (the LM head of shipped LFM2 Q4_0 files): one GEMV launch per weight.
int q6k_gemv_locked(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count,
                    const int8_t* d_q, const float* d_s, int accumulate) {
    if (reinterpret_cast<uintptr_t>(d_q) % 16u != 0) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "Q6_K gemv: quants must be 16-byte aligned");
    for (uint32_t i = 0; i < count; i++) {
        hipError_t e = launch_gemv_q6k(static_cast<const uint8_t*>(ws[i]->d), ws[i]->m, ws[i]->k, d_q, d_s, d_ys[i], 1, accumulate,
                                       ctx->num_cus, ctx->launch());
        if (e != hipSuccess) return fail_hip(ctx, e, "Q6_K gemv launch");
    }
    return WICK_ROCM_OK;
}

// f32 activations -> y for a group of weights (lock held): fused quantize+GEMV when
// the pair kernel takes the shape, otherwise quantize into scratch, then GEMV.
int gemv_f32_locked(wick_rocm_ctx* ctx, const GemvBatch& b, int type, uint32_t k, const float* x, int accumulate) {
    if (pairs_kernel_applies(b, k) && reinterpret_cast<uintptr_t>(x) % 16u == 0) {
        hipError_t e = launch_gemv_f32(type, b, k, x, accumulate, ctx->num_cus, ctx->launch());
        if (e != hipSuccess) return fail_hip(ctx, e, "fused gemv launch");
        return WICK_ROCM_OK;
    }
    if (int rc = ensure_scratch(ctx, k, k / 32u)) return rc;
    hipError_t e = launch_quantize_q8_0(x, 1, k, k, ctx->scratch_q, ctx->scratch_s, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "quantize_q8_0 launch");
    e = launch_gemv(type, b, k, ctx->scratch_q, ctx->scratch_s, accumulate, ctx->num_cus, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "gemv launch");
    return WICK_ROCM_OK;
}

}  // namespace

int wick_rocm_gemv_q8_multi(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count,
                            const int8_t* d_quants, const float* d_scales, int accumulate) {
    WR_ENTER(ctx);
    if (!d_quants || !d_scales) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv: null pointer");
    GemvBatch b{};
    if (int rc = make_batch(ctx, ws, d_ys, count, b)) return rc;
    if (ws[0]->type == kTypeQ6_K) return q6k_gemv_locked(ctx, ws, d_ys, count, d_quants, d_scales, accumulate);
    hipError_t e = launch_gemv(ws[0]->type, b, ws[0]->k, d_quants, d_scales, accumulate, ctx->num_cus, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "gemv launch");
    return WICK_ROCM_OK;
}

namespace {

// y_i (+)= W_i x for weights that share the f32 activation x (lock held).
int gemv_plain_locked(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count, const float* x, int accumulate) {
    GemvBatch b{};
    if (int rc = make_batch(ctx, ws, d_ys, count, b)) return rc;
    if (ws[0]->type == kTypeQ6_K) {  // quantize into scratch, then one launch per weight
        const uint32_t k = ws[0]->k;
        if (int rc = ensure_scratch(ctx, k, k / 32u)) return rc;
        hipError_t e = launch_quantize_q8_0(x, 1, k, k, ctx->scratch_q, ctx->scratch_s, ctx->launch());
        if (e != hipSuccess) return fail_hip(ctx, e, "quantize_q8_0 launch");
        return q6k_gemv_locked(ctx, ws, d_ys, count, ctx->scratch_q, ctx->scratch_s, accumulate);
    }
    return gemv_f32_locked(ctx, b, ws[0]->type, ws[0]->k, x, accumulate);
}

// y_i (+)= W_i xform(x) for weights that share x (lock held).  The fused kernel applies the transform in its
// prologue; shapes / types it does not take run the transform as a launch of its own into scratch first.
int gemv_xform_locked(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count, const float* x, int xform,
                      const float* d_aux, float eps, int accumulate) {
    if (!x || !d_aux) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv: null activation pointer");
    GemvBatch b{};
    if (int rc = make_batch(ctx, ws, d_ys, count, b)) return rc;
    const uint32_t k = ws[0]->k;
    const auto aligned16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16u == 0; };
    if (ws[0]->type != kTypeQ6_K && pairs_kernel_applies(b, k) && aligned16(x) && aligned16(d_aux)) {
        hipError_t e = launch_gemv_f32(ws[0]->type, b, k, x, accumulate, ctx->num_cus, ctx->launch(), xform, d_aux, eps);
        return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "fused gemv launch");
    }
    hipError_t e;
    if (xform == kXformRmsNorm && ws[0]->type == kTypeQ6_K && aligned16(x) && aligned16(d_aux)) {  // norm and quantizer inside the GEMV's launch
        for (uint32_t i = 0; i < count; i++) {
            e = launch_gemv_q6k_rmsnorm(static_cast<const uint8_t*>(ws[i]->d), ws[i]->m, k, x, d_aux, eps, d_ys[i], accumulate, ctx->num_cus, ctx->launch());
            if (e != hipSuccess) return fail_hip(ctx, e, "Q6_K gemv launch");
        }
        return WICK_ROCM_OK;
    }
    if (int rc = ensure_scratch(ctx, k, k / 32u, k)) return rc;
    if (xform == kXformRmsNorm) {
        e = launch_rmsnorm(x, d_aux, ctx->scratch_f, 1, k, k, k, eps, ctx->launch());
    } else {
        e = hipMemcpyAsync(ctx->scratch_f, x, (size_t)k * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream);
        if (e == hipSuccess) e = launch_silu_mul(ctx->scratch_f, d_aux, k, ctx->launch());
    }
    if (e != hipSuccess) return fail_hip(ctx, e, "activation transform launch");
    if (ws[0]->type == kTypeQ6_K) {
        e = launch_quantize_q8_0(ctx->scratch_f, 1, k, k, ctx->scratch_q, ctx->scratch_s, ctx->launch());
        if (e != hipSuccess) return fail_hip(ctx, e, "quantize_q8_0 launch");
        return q6k_gemv_locked(ctx, ws, d_ys, count, ctx->scratch_q, ctx->scratch_s, accumulate);
    }
    return gemv_f32_locked(ctx, b, ws[0]->type, k, ctx->scratch_f, accumulate);
}

}  // namespace

int wick_rocm_gemv_rmsnorm_f32_multi(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count,
                                     const float* d_x, const float* d_norm_weight, float eps, int accumulate) {
    WR_ENTER(ctx);
    return gemv_xform_locked(ctx, ws, d_ys, count, d_x, kXformRmsNorm, d_norm_weight, eps, accumulate);
}

int wick_rocm_gemv_silu_mul_f32(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const float* d_gate, const float* d_up, float* d_y,
                                int accumulate) {
    WR_ENTER(ctx);
    const wick_rocm_weight* ws[1] = {w};
    float* ys[1] = {d_y};
    return gemv_xform_locked(ctx, ws, ys, 1, d_gate, kXformSiluMul, d_up, 0.0f, accumulate);
}

namespace {

const auto aligned16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16u == 0; };

// Whether the one-launch gate / up kernel takes these weights (lock held or not: reads handles only).
bool gate_up_fused(const wick_rocm_weight* w_gate, const wick_rocm_weight* w_up) {
    return w_gate->type == w_up->type && w_gate->type != kTypeQ6_K && w_gate->m == w_up->m && w_gate->k == w_up->k &&
           gated_kernel_applies(static_cast<const uint8_t*>(w_gate->d), static_cast<const uint8_t*>(w_up->d), w_gate->k);
}

}  // namespace

int wick_rocm_ffn_gate_up_f32(wick_rocm_ctx* ctx, const wick_rocm_weight* w_gate, const wick_rocm_weight* w_up, const float* d_x,
                              const float* d_norm_weight, float eps, float* d_act) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w_gate)) return rc;
    if (int rc = check_weight(ctx, w_up)) return rc;
    if (!d_x || !d_act) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "ffn_gate_up: null device pointer");
    if (w_gate->m != w_up->m || w_gate->k != w_up->k) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "ffn_gate_up: gate and up must have one shape");
    const uint32_t m = w_gate->m, k = w_gate->k;
    const auto *g = static_cast<const uint8_t*>(w_gate->d), *u = static_cast<const uint8_t*>(w_up->d);
    if (gate_up_fused(w_gate, w_up) && aligned16(d_x) && (!d_norm_weight || aligned16(d_norm_weight))) {
        hipError_t e = launch_gemv_gated_f32(w_gate->type, g, u, m, k, d_x, d_act, ctx->num_cus, ctx->launch(),
                                             d_norm_weight ? kXformRmsNorm : kXformNone, d_norm_weight, eps);
        return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "gated gemv launch");
    }
    // Shapes / types the gated kernel does not take: gate into d_act, up into scratch (after the quantization /
    // transform scratch of k floats), then the gate as a launch of its own.
    if (int rc = ensure_scratch(ctx, k, k / 32u, (size_t)k + m)) return rc;
    float* up_out = ctx->scratch_f + k;
    const wick_rocm_weight* ws[2] = {w_gate, w_up};
    float* ys[2] = {d_act, up_out};
    for (int i = 0; i < 2; i++) {
        const int rc = d_norm_weight ? gemv_xform_locked(ctx, ws + i, ys + i, 1, d_x, kXformRmsNorm, d_norm_weight, eps, 0)
                                     : gemv_plain_locked(ctx, ws + i, ys + i, 1, d_x, 0);
        if (rc) return rc;
    }
    hipError_t e = launch_silu_mul(d_act, up_out, m, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "silu_mul launch");
}

int wick_rocm_shortconv_fusable(const wick_rocm_weight* w_out, const wick_rocm_weight* w_gate, const wick_rocm_weight* w_up, uint32_t kernel_size) {
    if (!w_out || !w_gate || !w_up || !w_out->d || !w_gate->d || !w_up->d) return 0;
    return w_out->type != kTypeQ6_K && w_out->k % 4u == 0 &&
           shortconv_kernel_applies(static_cast<const uint8_t*>(w_out->d), w_out->k, kernel_size) && gate_up_fused(w_gate, w_up);
}

int wick_rocm_shortconv_out_proj_f32(wick_rocm_ctx* ctx, const wick_rocm_weight* w_out, const float* d_proj, const float* d_buffer,
                                     const float* d_conv_weight, uint32_t kernel_size, float* d_y, int accumulate) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w_out)) return rc;
    if (!d_proj || !d_buffer || !d_conv_weight || !d_y) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "shortconv_out_proj: null device pointer");
    if (w_out->type == kTypeQ6_K || !shortconv_kernel_applies(static_cast<const uint8_t*>(w_out->d), w_out->k, kernel_size))
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "shortconv_out_proj: needs kernel size 3, hidden <= 2048 with an even block count and a Q4_0 / Q8_0 weight; "
                                                  "use wick_rocm_shortconv_step + wick_rocm_matmul_f32");
    if (!aligned16(d_proj) || !aligned16(d_buffer) || !aligned16(d_conv_weight))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "shortconv_out_proj: proj, buffer and conv weight must be 16-byte aligned");
    hipError_t e = launch_gemv_shortconv_f32(w_out->type, static_cast<const uint8_t*>(w_out->d), w_out->m, w_out->k, d_proj, d_buffer, d_conv_weight,
                                             d_y, accumulate, ctx->num_cus, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "shortconv gemv launch");
}

int wick_rocm_ffn_gate_up_conv_advance_f32(wick_rocm_ctx* ctx, const wick_rocm_weight* w_gate, const wick_rocm_weight* w_up, const float* d_x,
                                           const float* d_norm_weight, float eps, float* d_act, const float* d_proj, float* d_buffer,
                                           uint32_t hidden, uint32_t kernel_size) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w_gate)) return rc;
    if (int rc = check_weight(ctx, w_up)) return rc;
    if (!d_x || !d_act || !d_proj || !d_buffer) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "ffn_gate_up_conv_advance: null device pointer");
    if (!gate_up_fused(w_gate, w_up) || hidden == 0 || hidden % 4u != 0 || kernel_size < 2)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "ffn_gate_up_conv_advance: shapes the one-launch gate / up kernel does not take (or hidden % 4 != 0, kernel size < 2); "
                                                  "use wick_rocm_shortconv_step and wick_rocm_ffn_gate_up_f32");
    if (!aligned16(d_x) || (d_norm_weight && !aligned16(d_norm_weight)) || !aligned16(d_proj) || !aligned16(d_buffer))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "ffn_gate_up_conv_advance: x, norm weight, proj and buffer must be 16-byte aligned");
    hipError_t e = launch_gemv_gated_f32(w_gate->type, static_cast<const uint8_t*>(w_gate->d), static_cast<const uint8_t*>(w_up->d), w_gate->m, w_gate->k, d_x,
                                         d_act, ctx->num_cus, ctx->launch(), d_norm_weight ? kXformRmsNorm : kXformNone, d_norm_weight, eps, d_buffer, d_proj,
                                         hidden, kernel_size);
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "gated gemv launch");
}

int wick_rocm_gemv_f32_multi(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count,
                             const float* d_x, size_t x_off_bytes, int accumulate) {
    WR_ENTER(ctx);
    if (!d_x) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv_f32_multi: null activation pointer");
    if (x_off_bytes % 4u) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemv_f32_multi: offset must be a multiple of 4");
    return gemv_plain_locked(ctx, ws, d_ys, count, reinterpret_cast<const float*>(reinterpret_cast<const char*>(d_x) + x_off_bytes), accumulate);
}

int wick_rocm_gemv_q8(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const int8_t* d_quants, const float* d_scales,
                      float* d_y, int accumulate) {
    const wick_rocm_weight* ws[1] = {w};
    float* ys[1] = {d_y};
    return wick_rocm_gemv_q8_multi(ctx, ws, ys, 1, d_quants, d_scales, accumulate);
}

int wick_rocm_gemm_q8(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const int8_t* d_quants, const float* d_scales,
                      uint32_t n, float* d_y, uint32_t y_stride, int y_layout, int accumulate) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w)) return rc;
    return gemm_locked(ctx, w, d_quants, d_scales, n, d_y, y_stride, y_layout, accumulate);
}

int wick_rocm_gemm_q8_residual_rmsnorm_quantize(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const int8_t* d_quants, const float* d_scales,
                                                uint32_t n, float* d_x, uint32_t x_stride, const float* d_norm_weight, float eps,
                                                int8_t* d_out_quants, float* d_out_scales) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w)) return rc;
    if (!d_x || !d_norm_weight || !d_out_quants || !d_out_scales) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemm + norm: null device pointer");
    if (w->m % 32u != 0 || x_stride < w->m || x_stride % 4u != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "gemm + norm: rows must be a multiple of 32, x_stride >= rows and a multiple of 4");
    if (reinterpret_cast<uintptr_t>(d_x) % 16u != 0 || reinterpret_cast<uintptr_t>(d_norm_weight) % 16u != 0 ||
        reinterpret_cast<uintptr_t>(d_out_quants) % 4u != 0)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemm + norm: x and the norm weights must be 16-byte aligned");
    if (n == 0) return WICK_ROCM_OK;
    uint32_t shares = 0;
    if (int rc = gemm_locked(ctx, w, d_quants, d_scales, n, d_x, x_stride, WICK_ROCM_LAYOUT_TOKEN_MAJOR, 1, true,
                             w->m <= kResidualNormMaxDim ? &shares : nullptr))
        return rc;
    // a split projection's shares are added up by the norm's kernel instead of a launch of their own
    const hipError_t e = shares > 1 ? launch_residual_rmsnorm_quantize(d_x, ctx->scratch_f, shares, d_norm_weight, n, w->m, x_stride, eps, d_out_quants,
                                                                       d_out_scales, ctx->launch())
                                    : launch_rmsnorm_quantize(d_x, d_norm_weight, n, w->m, x_stride, eps, d_out_quants, d_out_scales, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "rmsnorm_quantize launch");
}

int wick_rocm_gemm_q8_multi(wick_rocm_ctx* ctx, const wick_rocm_weight* const* ws, float* const* d_ys, uint32_t count, const int8_t* d_quants,
                            const float* d_scales, uint32_t n, uint32_t y_stride, int y_layout, int accumulate) {
    WR_ENTER(ctx);
    if (!ws || !d_ys || count == 0 || count > 3) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "gemm_q8_multi: 1..3 weights");
    for (uint32_t i = 0; i < count; i++) {
        if (int rc = check_weight(ctx, ws[i])) return rc;
        if (ws[i]->type != ws[0]->type || ws[i]->k != ws[0]->k) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "gemm_q8_multi: weights must share k and dtype");
    }
    const wick_rocm_weight* w0 = ws[0];
    bool packed = true;
    for (uint32_t i = 0; i < count; i++) packed = packed && ws[i]->d_gemm != nullptr;
    size_t bytes = 0;  // the launch streams all of them
    for (uint32_t i = 0; i < count; i++) bytes += ws[i]->nbytes;
    const bool one_launch = count > 1 && packed && w0->type != kTypeQ6_K && n >= ctx->min_n_for(bytes) && w0->k % 128u == 0 && d_quants && d_scales &&
                            reinterpret_cast<uintptr_t>(d_quants) % 16u == 0 && reinterpret_cast<uintptr_t>(d_scales) % 16u == 0;
    if (!one_launch) {  // shapes without a batched launch: one call per weight, same results
        for (uint32_t i = 0; i < count; i++)
            if (int rc = gemm_locked(ctx, ws[i], d_quants, d_scales, n, d_ys[i], y_stride, y_layout, accumulate)) return rc;
        return WICK_ROCM_OK;
    }
    if (y_layout != WICK_ROCM_LAYOUT_TOKEN_MAJOR && y_layout != WICK_ROCM_LAYOUT_ROW_MAJOR)
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "unknown output layout");
    const uint8_t* wp[3];
    uint32_t ms[3];
    for (uint32_t i = 0; i < count; i++) {
        if (!d_ys[i]) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "null device pointer");
        if (y_layout == WICK_ROCM_LAYOUT_TOKEN_MAJOR ? y_stride < ws[i]->m : y_stride < n)
            return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "y_stride smaller than the output extent");
        wp[i] = static_cast<const uint8_t*>(ws[i]->d_gemm), ms[i] = ws[i]->m;
    }
    hipError_t e = launch_gemm_mfma_multi(w0->type, wp, ms, count, w0->k, d_quants, d_scales, n, d_ys, y_stride, y_layout, accumulate, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "gemm launch");
}

int wick_rocm_reserve_scratch(wick_rocm_ctx* ctx, uint32_t max_n, uint32_t max_k) {
    WR_ENTER(ctx);
    if (max_k % 32u != 0) return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "reserve_scratch: max_k % 32 != 0");
    // f32 scratch: one transformed activation vector + one projection output of the unfused fallbacks and, for batched calls
    // that may take the MFMA GEMM, the K shares of a split launch ([shares][n][m] <= 512 tiles of 128 x 128 sums, whatever the shape)
    const size_t split_floats = max_n >= kGemmMinNLarge && ctx->gemm_max_splits > 1 ? kGemmSplitScratchFloats : 0;
    const size_t f_floats = 2 * (size_t)max_k > split_floats ? 2 * (size_t)max_k : split_floats;
    return ensure_scratch(ctx, (size_t)max_n * max_k, (size_t)max_n * (max_k / 32u), f_floats);
}

int wick_rocm_matmul_f32(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const float* d_x, size_t x_off_bytes, uint32_t n,
                         uint32_t x_stride, float* d_y, size_t y_off_bytes, uint32_t y_stride, int accumulate) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w)) return rc;
    if (!d_x || !d_y) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32: null device pointer");
    if (n == 0) return WICK_ROCM_OK;
    if (x_off_bytes % 4u || y_off_bytes % 4u) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32: offsets must be multiples of 4");
    if (n > 1 && (x_stride < w->k || y_stride < w->m))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32: stride smaller than the vector length");
    const float* x = reinterpret_cast<const float*>(reinterpret_cast<const char*>(d_x) + x_off_bytes);
    float* y = reinterpret_cast<float*>(reinterpret_cast<char*>(d_y) + y_off_bytes);
    if (n == 1 && w->type != kTypeQ6_K) {
        GemvBatch b{};
        b.w[0] = static_cast<const uint8_t*>(w->d), b.y[0] = y, b.row_end[0] = w->m, b.count = 1;
        return gemv_f32_locked(ctx, b, w->type, w->k, x, accumulate);
    }
    if (int rc = ensure_scratch(ctx, (size_t)n * w->k, (size_t)n * (w->k / 32u))) return rc;
    hipError_t e = launch_quantize_q8_0(x, n, w->k, x_stride, ctx->scratch_q, ctx->scratch_s, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "quantize_q8_0 launch");
    return gemm_locked(ctx, w, ctx->scratch_q, ctx->scratch_s, n, y, n == 1 ? w->m : y_stride,
                       WICK_ROCM_LAYOUT_TOKEN_MAJOR, accumulate);
}

int wick_rocm_matmul_f32_noalloc(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const float* d_x, size_t x_off_bytes, uint32_t n,
                                 uint32_t x_stride, float* d_y, size_t y_off_bytes, uint32_t y_stride, int accumulate) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w)) return rc;
    if (!d_x || !d_y) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32_noalloc: null device pointer");
    if (n == 0) return WICK_ROCM_OK;
    if (x_off_bytes % 4u || y_off_bytes % 4u) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32_noalloc: offsets must be multiples of 4");
    if (n > 1 && (x_stride < w->k || y_stride < w->m))
        return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "matmul_f32_noalloc: stride smaller than the vector length");
    if ((uint64_t)n * w->k > kNoallocMaxElems)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "matmul_f32_noalloc: n * k exceeds the static scratch (4194304 elements); use wick_rocm_matmul_f32");
    if (ctx->timer.enabled) return fail(ctx, WICK_ROCM_ERR_STATE, "matmul_f32_noalloc: per-dispatch kernel timing creates events; switch it off");
    if (int rc = noalloc_claim(ctx)) return rc;
    if (ctx->capturing) ctx->capture_used_noalloc = true;  // every replay of the graph will use the array again
    const float* x = reinterpret_cast<const float*>(reinterpret_cast<const char*>(d_x) + x_off_bytes);
    float* y = reinterpret_cast<float*>(reinterpret_cast<char*>(d_y) + y_off_bytes);
    // this device's copy of the static array, never the array's name: quants first, scales behind them
    int8_t* q = reinterpret_cast<int8_t*>(ctx->noalloc_scratch);
    float* s = reinterpret_cast<float*>(ctx->noalloc_scratch + kNoallocMaxElems);
    // Nothing in the scratch has to start at zero: the quantizer writes every byte the matmul reads.
    hipError_t e = launch_quantize_q8_0(x, n, w->k, n == 1 ? w->k : x_stride, q, s, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "quantize_q8_0 launch");
    return gemm_locked(ctx, w, q, s, n, y, n == 1 ? w->m : y_stride, WICK_ROCM_LAYOUT_TOKEN_MAJOR, accumulate, /*may_split=*/false);
}

int wick_rocm_block_dots_i32(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const int8_t* d_quants, uint32_t n,
                             int32_t* d_out) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w)) return rc;
    if (!d_quants || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "block_dots: null device pointer");
    if (n == 0) return WICK_ROCM_OK;
    if (w->type == kTypeQ6_K) {  // 16-weight groups: out[(j*m + i) * (k/16) + g]
        if (reinterpret_cast<uintptr_t>(d_quants) % 16u != 0) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "block_dots: quants must be 16-byte aligned");
        for (uint32_t j = 0; j < n; j++) {
            hipError_t e = launch_group_dots_q6k(static_cast<const uint8_t*>(w->d), w->m, w->k, d_quants + (size_t)j * w->k,
                                                 d_out + (size_t)j * w->m * (w->k / 16u), ctx->num_cus, ctx->launch());
            if (e != hipSuccess) return fail_hip(ctx, e, "block_dots launch");
        }
        return WICK_ROCM_OK;
    }
    const bool mfma = w->d_gemm && n >= ctx->min_n_for(w->nbytes) && (w->k % 128u == 0) && (reinterpret_cast<uintptr_t>(d_quants) % 16u == 0);
    hipError_t e = mfma ? launch_block_dots_mfma(w->type, static_cast<const uint8_t*>(w->d_gemm), w->m, w->k, d_quants, n, d_out, ctx->launch())
                        : launch_block_dots_gemv(w->type, static_cast<const uint8_t*>(w->d), w->m, w->k, d_quants, n, d_out, ctx->num_cus, ctx->launch());
    if (e != hipSuccess) return fail_hip(ctx, e, "block_dots launch");
    return WICK_ROCM_OK;
}

int wick_rocm_block_dots_f32_i32(wick_rocm_ctx* ctx, const wick_rocm_weight* w, const float* d_x, int32_t* d_out) {
    WR_ENTER(ctx);
    if (int rc = check_weight(ctx, w)) return rc;
    if (!d_x || !d_out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "block_dots_f32: null device pointer");
    if (w->type == kTypeQ6_K) return fail(ctx, WICK_ROCM_ERR_UNSUPPORTED_DTYPE, "block_dots_f32: Q6_K has no fused-quantizer kernel");
    GemvBatch b{};
    b.w[0] = static_cast<const uint8_t*>(w->d), b.row_end[0] = w->m, b.count = 1;
    if (!pairs_kernel_applies(b, w->k) || reinterpret_cast<uintptr_t>(d_x) % 16u != 0)
        return fail(ctx, WICK_ROCM_ERR_BAD_SHAPE, "block_dots_f32: shape not taken by the fused kernel (odd block count, k > 8192 or x not 16-byte aligned)");
    hipError_t e = launch_block_dots_gemv_f32(w->type, b.w[0], w->m, w->k, d_x, d_out, ctx->num_cus, ctx->launch());
    return e == hipSuccess ? WICK_ROCM_OK : fail_hip(ctx, e, "block_dots_f32 launch");
}

int wick_rocm_graph_begin(wick_rocm_ctx* ctx) {
    WR_ENTER(ctx);
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "graph_begin: capture already in progress");
    if (ctx->timer.enabled) return fail(ctx, WICK_ROCM_ERR_STATE, "graph_begin: kernel timing is on");
    WR_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    ctx->capture_used_scratch = 0;
    ctx->capture_used_noalloc = false;
    return WICK_ROCM_OK;
}

int wick_rocm_graph_end(wick_rocm_ctx* ctx, wick_rocm_graph** out) {
    WR_ENTER(ctx);
    if (!out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "graph_end: null out pointer");
    *out = nullptr;
    if (!ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "graph_end: no capture in progress");
    // the capture ends whatever happens next, so that no failure leaves the stream capturing
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    wick_rocm_graph* g = e == hipSuccess ? new (std::nothrow) wick_rocm_graph() : nullptr;
    if (e == hipSuccess && !g) {
        (void)hipGraphDestroy(graph);
        return fail(ctx, WICK_ROCM_ERR_HIP, "out of host memory");
    }
    if (e == hipSuccess) {
        g->graph = graph;
        e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    }
    if (e != hipSuccess) {
        if (graph) (void)hipGraphDestroy(graph);
        delete g;
        return fail_hip(ctx, e, "graph_end");
    }
    g->uses_scratch = ctx->capture_used_scratch;
    for (int i = 0; i < 3; i++) g->scratch_gen[i] = ctx->scratch_gen[i];
    g->uses_noalloc = ctx->capture_used_noalloc;
    *out = g;
    return WICK_ROCM_OK;
}

int wick_rocm_graph_launch(wick_rocm_ctx* ctx, wick_rocm_graph* g) {
    WR_ENTER(ctx);
    if (!g || !g->exec) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "graph_launch: null graph");
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "graph_launch during capture");
    if (graph_is_stale(ctx, g))
        return fail(ctx, WICK_ROCM_ERR_STATE, "graph_launch: the context's scratch was regrown after this graph was captured (it holds freed addresses); "
                                              "capture it again, and size the scratch with wick_rocm_reserve_scratch before capturing");
    if (g->uses_noalloc)
        if (int rc = noalloc_claim(ctx)) return rc;
    WR_HIP(ctx, hipGraphLaunch(g->exec, ctx->stream));
    return WICK_ROCM_OK;
}

int wick_rocm_graph_destroy(wick_rocm_ctx* ctx, wick_rocm_graph* g) {
    WR_ENTER(ctx);
    if (!g) return WICK_ROCM_OK;
    WR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return WICK_ROCM_OK;
}

int wick_rocm_event_create(wick_rocm_ctx* ctx, wick_rocm_event** out) {
    WR_ENTER(ctx);
    if (!out) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "event_create: null out pointer");
    wick_rocm_event* e = new (std::nothrow) wick_rocm_event();
    if (!e) return fail(ctx, WICK_ROCM_ERR_HIP, "out of host memory");
    hipError_t he = hipEventCreate(&e->ev);
    if (he != hipSuccess) {
        delete e;
        return fail_hip(ctx, he, "hipEventCreate");
    }
    *out = e;
    return WICK_ROCM_OK;
}

int wick_rocm_event_record(wick_rocm_ctx* ctx, wick_rocm_event* e) {
    WR_ENTER(ctx);
    if (!e) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "event_record: null event");
    WR_HIP(ctx, hipEventRecord(e->ev, ctx->stream));
    return WICK_ROCM_OK;
}

int wick_rocm_event_elapsed_ms(wick_rocm_ctx* ctx, wick_rocm_event* start, wick_rocm_event* stop, float* ms) {
    WR_ENTER(ctx);
    if (!start || !stop || !ms) return fail(ctx, WICK_ROCM_ERR_INVALID_ARG, "event_elapsed_ms: null argument");
    WR_HIP(ctx, hipEventSynchronize(stop->ev));
    WR_HIP(ctx, hipEventElapsedTime(ms, start->ev, stop->ev));
    return WICK_ROCM_OK;
}

int wick_rocm_kernel_timing_begin(wick_rocm_ctx* ctx) {
    WR_ENTER(ctx);
    if (ctx->capturing) return fail(ctx, WICK_ROCM_ERR_STATE, "kernel_timing_begin during graph capture");
    if (ctx->timer.enabled) return fail(ctx, WICK_ROCM_ERR_STATE, "kernel timing already on");
    ctx->timer.enabled = true;
    return WICK_ROCM_OK;
}

int wick_rocm_kernel_timing_end(wick_rocm_ctx* ctx, double* total_ms, uint64_t* launches, int n_families) {
    WR_ENTER(ctx);
    if (!ctx->timer.enabled) return fail(ctx, WICK_ROCM_ERR_STATE, "kernel timing is not on");
    ctx->timer.enabled = false;
    for (int f = 0; f < n_families; f++) {
        if (total_ms) total_ms[f] = 0.0;
        if (launches) launches[f] = 0;
    }
    hipError_t first = hipStreamSynchronize(ctx->stream);
    for (KernelTimer::Rec& r : ctx->timer.recs) {
        float ms = 0.f;
        hipError_t e = hipEventElapsedTime(&ms, r.start, r.stop);
        if (e != hipSuccess && first == hipSuccess) first = e;
        if (e == hipSuccess && r.family < n_families) {
            if (total_ms) total_ms[r.family] += (double)ms;
            if (launches) launches[r.family] += 1;
        }
        ctx->timer.spares.push_back(r);
    }
    ctx->timer.recs.clear();
    if (first != hipSuccess) return fail_hip(ctx, first, "kernel_timing_end");
    return WICK_ROCM_OK;
}

int wick_rocm_event_destroy(wick_rocm_ctx* ctx, wick_rocm_event* e) {
    WR_ENTER(ctx);
    if (!e) return WICK_ROCM_OK;
    (void)hipEventDestroy(e->ev);
    delete e;
    return WICK_ROCM_OK;
}

}  // extern "C"
