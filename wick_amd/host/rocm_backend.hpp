// Host-side C++ mirror of wick's GPU-backend matmul call sites over the C ABI in
// include/wick_rocm.h.  This is the role `backend/rocm.rs` + `model/rocm_lfm2.rs`
// play in the Rust tree (which cannot be compiled in this environment): same
// method names, argument order and error behaviour as the reference's
//   MetalWeight                       wick/src/model/metal_lfm2.rs:28-36
//   encode_gemv_impl                  wick/src/model/metal_lfm2.rs:1231-1335
//   encode_gemm                       wick/src/model/metal_lfm2.rs:881-992
//   encode_gemv_qkv / _gate_up        wick/src/model/metal_lfm2.rs:1043-1119
//   quantize_to_scratch / _columns    wick/src/model/lfm2.rs:571-612
//   gemv_with_preq                    wick/src/backend/cpu.rs:334-354
//   gemm_preq                         wick/src/model/lfm2.rs:539-565
//   trait Model (forward / forward_prefill / forward_greedy)   wick/src/model/mod.rs:72-323
//   load_model_metal                  wick/src/model/mod.rs:385-403
// Errors become exceptions here (anyhow::Result on the Rust side); contract
// violations the reference asserts on (null buffers, bad strides) are reported the
// same way instead of aborting.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/wick_gguf.h"
#include "../../include/wick_rocm.h"
#include "../../include/wick_rocm_lfm2.h"

namespace wick {

enum class DType : int { Q4_0 = WICK_ROCM_TYPE_Q4_0, Q8_0 = WICK_ROCM_TYPE_Q8_0, Q6_K = WICK_ROCM_TYPE_Q6_K };

struct BackendError : std::runtime_error {
    int status;
    BackendError(int s, const std::string& m) : std::runtime_error("rocm backend: " + m + " (status " + std::to_string(s) + ")"), status(s) {}
};

class RocmContext;

// An open GGUF file (GgufFile::open, wick/src/gguf.rs:331-341).
class GgufFile {
public:
    explicit GgufFile(const std::string& path) {
        const int rc = wick_gguf_open(path.c_str(), &g_);
        if (rc != 0) throw BackendError(rc, wick_gguf_last_error());
    }
    ~GgufFile() { wick_gguf_close(g_); }
    GgufFile(const GgufFile&) = delete;
    GgufFile& operator=(const GgufFile&) = delete;
    const wick_gguf* raw() const { return g_; }

private:
    wick_gguf* g_ = nullptr;
};

// Device-resident weight: GGUF block bytes verbatim.
struct RocmWeight {
    wick_rocm_weight* handle = nullptr;
    DType dtype = DType::Q4_0;
    uint32_t m = 0, k = 0;
};

// A caller-owned device buffer (a Metal `Buffer` in the reference).
struct Buffer {
    void* ptr = nullptr;
    size_t nbytes = 0;
};

class RocmContext {
public:
    explicit RocmContext(int device = 0) {
        int rc = wick_rocm_ctx_create(device, &ctx_);
        if (rc != 0) throw BackendError(rc, rc == WICK_ROCM_ERR_NO_DEVICE ? "no gfx950 device" : "context creation failed");
    }
    ~RocmContext() { wick_rocm_ctx_destroy(ctx_); }
    RocmContext(const RocmContext&) = delete;
    RocmContext& operator=(const RocmContext&) = delete;

    Buffer create_buffer(size_t nbytes) {
        Buffer b;
        b.nbytes = nbytes;
        check(wick_rocm_buffer_alloc(ctx_, nbytes, &b.ptr));
        return b;
    }
    void free_buffer(Buffer& b) {
        check(wick_rocm_buffer_free(ctx_, b.ptr));
        b.ptr = nullptr;
    }
    void write(const Buffer& b, const void* src, size_t nbytes, size_t off = 0) {
        check(wick_rocm_upload(ctx_, static_cast<char*>(b.ptr) + off, src, nbytes));
    }
    void read(const Buffer& b, void* dst, size_t nbytes, size_t off = 0) {
        check(wick_rocm_download(ctx_, dst, static_cast<const char*>(b.ptr) + off, nbytes));
    }
    std::vector<float> read_f32(const Buffer& b, size_t count, size_t off = 0) {
        std::vector<float> v(count);
        read(b, v.data(), count * sizeof(float), off);
        return v;
    }
    void sync() { check(wick_rocm_sync(ctx_)); }
    // whether upload_weight / weight_from_gguf also make the prefill GEMM's own layout of a Q4_0 / Q8_0 weight (default: yes)
    void set_gemm_packing(bool enabled) { check(wick_rocm_set_gemm_packing(ctx_, enabled ? 1 : 0)); }

    RocmWeight upload_weight(const void* blocks, size_t nbytes, DType dtype, uint32_t m, uint32_t k) {
        RocmWeight w;
        w.dtype = dtype, w.m = m, w.k = k;
        check(wick_rocm_weight_upload(ctx_, blocks, nbytes, static_cast<int>(dtype), m, k, &w.handle));
        return w;
    }
    // resolve_weight (wick/src/model/lfm2.rs:310-338) + upload: k = ne0, m = ne1.
    RocmWeight weight_from_gguf(const GgufFile& gguf, const std::string& tensor_name) {
        RocmWeight w;
        check(wick_rocm_weight_from_gguf(ctx_, gguf.raw(), tensor_name.c_str(), &w.handle));
        int type = 0;
        size_t nbytes = 0;
        check(wick_rocm_weight_info(w.handle, &type, &w.m, &w.k, &nbytes));
        w.dtype = static_cast<DType>(type);
        return w;
    }
    void free_weight(RocmWeight& w) {
        check(wick_rocm_weight_free(ctx_, w.handle));
        w.handle = nullptr;
    }

    // ---- GPU call sites: f32 activations in, f32 out, byte offsets ------------------
    void encode_gemv(const RocmWeight& w, const Buffer& input, uint64_t input_off_bytes, const Buffer& output,
                     uint64_t output_off_bytes, bool accumulate = false) {
        check(wick_rocm_matmul_f32(ctx_, w.handle, static_cast<const float*>(input.ptr), input_off_bytes, 1, w.k,
                                   static_cast<float*>(output.ptr), output_off_bytes, w.m, accumulate));
    }
    void encode_gemm(const RocmWeight& w, const Buffer& x, uint64_t x_off_bytes, const Buffer& y, uint64_t y_off_bytes,
                     uint32_t n, uint32_t x_stride, uint32_t y_stride, bool accumulate = false) {
        check(wick_rocm_matmul_f32(ctx_, w.handle, static_cast<const float*>(x.ptr), x_off_bytes, n, x_stride,
                                   static_cast<float*>(y.ptr), y_off_bytes, y_stride, accumulate));
    }
    // {Q,K,V} or {gate,up}: one activation, several weights, one launch.
    void encode_gemv_fused(const std::vector<const RocmWeight*>& ws, const Buffer& x, uint64_t x_off_bytes,
                           const std::vector<Buffer>& ys, bool accumulate = false) {
        std::vector<const wick_rocm_weight*> hs;
        std::vector<float*> ps;
        for (auto* w : ws) hs.push_back(w->handle);
        for (auto& y : ys) ps.push_back(static_cast<float*>(y.ptr));
        check(wick_rocm_gemv_f32_multi(ctx_, hs.data(), ps.data(), static_cast<uint32_t>(hs.size()),
                                       static_cast<const float*>(x.ptr), x_off_bytes, accumulate));
    }

    // ---- CPU call sites on pre-quantized activations ---------------------------------
    void quantize_columns(const Buffer& x, uint32_t n, uint32_t k, uint32_t x_stride, const Buffer& quants, const Buffer& scales) {
        check(wick_rocm_quantize_q8_0(ctx_, static_cast<const float*>(x.ptr), n, k, x_stride, static_cast<int8_t*>(quants.ptr),
                                      static_cast<float*>(scales.ptr)));
    }
    void gemv_with_preq(const RocmWeight& w, const Buffer& scales, const Buffer& quants, const Buffer& y, bool accumulate = false) {
        check(wick_rocm_gemv_q8(ctx_, w.handle, static_cast<const int8_t*>(quants.ptr), static_cast<const float*>(scales.ptr),
                                static_cast<float*>(y.ptr), accumulate));
    }
    // out[i*n + j], like gemm_*_q8_0_neon
    void gemm_preq(const RocmWeight& w, const Buffer& scales, const Buffer& quants, uint32_t n, const Buffer& out) {
        check(wick_rocm_gemm_q8(ctx_, w.handle, static_cast<const int8_t*>(quants.ptr), static_cast<const float*>(scales.ptr), n,
                                static_cast<float*>(out.ptr), n, WICK_ROCM_LAYOUT_ROW_MAJOR, 0));
    }

    wick_rocm_ctx* raw() { return ctx_; }

    void check(int rc) {
        if (rc == 0) return;
        char buf[512] = {0};
        wick_rocm_last_error(ctx_, buf, sizeof buf);
        throw BackendError(rc, buf);
    }

private:
    wick_rocm_ctx* ctx_ = nullptr;
};

// An LFM2 model on the GPU with the `Model` trait's methods (wick/src/model/mod.rs:72-323); what
// load_model_metal returns for the Metal backend (wick/src/model/mod.rs:385-403).  Owns weights, KV caches,
// conv state and scratch; the GGUF file may be closed once the constructor has returned.
class RocmLfm2Model {
public:
    // kv_f16: K / V rows kept in half like the reference's GPU model (wick/src/model/metal_lfm2.rs:4117-4247) instead of
    // the CPU model's f32 rows.
    RocmLfm2Model(RocmContext& ctx, const GgufFile& gguf, uint32_t context_size, bool kv_f16 = false) : ctx_(ctx) {
        ctx_.check(wick_rocm_lfm2_load_kv(ctx_.raw(), gguf.raw(), context_size, kv_f16 ? WICK_ROCM_KV_F16 : WICK_ROCM_KV_F32, &m_));
        ctx_.check(wick_rocm_lfm2_get_config(m_, &cfg_));
    }
    bool kv_f16() const { return wick_rocm_lfm2_kv_dtype(m_) == WICK_ROCM_KV_F16; }
    ~RocmLfm2Model() { wick_rocm_lfm2_free(ctx_.raw(), m_); }
    RocmLfm2Model(const RocmLfm2Model&) = delete;
    RocmLfm2Model& operator=(const RocmLfm2Model&) = delete;

    const wick_rocm_lfm2_config& config() const { return cfg_; }
    size_t gpu_memory_bytes() const { return wick_rocm_lfm2_gpu_memory_bytes(m_); }
    // A fresh InferenceState.
    void reset() { ctx_.check(wick_rocm_lfm2_reset(ctx_.raw(), m_)); }

    // forward(tokens = [token], pos) -> logits [vocab_size]
    std::vector<float> forward(uint32_t token, uint32_t pos) {
        std::vector<float> logits(cfg_.vocab_size);
        ctx_.check(wick_rocm_lfm2_forward(ctx_.raw(), m_, token, pos, logits.data()));
        return logits;
    }
    // forward_prefill(tokens, start_pos) -> logits of the last token
    std::vector<float> forward_prefill(const std::vector<uint32_t>& tokens, uint32_t start_pos) {
        std::vector<float> logits(cfg_.vocab_size);
        ctx_.check(wick_rocm_lfm2_forward_prefill(ctx_.raw(), m_, tokens.data(), static_cast<uint32_t>(tokens.size()), start_pos, logits.data()));
        return logits;
    }
    // forward_greedy(tokens = [token], pos) -> next token id, picked on the device
    uint32_t forward_greedy(uint32_t token, uint32_t pos) {
        uint32_t next = 0;
        ctx_.check(wick_rocm_lfm2_forward_greedy(ctx_.raw(), m_, token, pos, &next));
        return next;
    }
    // n greedy steps without a host round trip between them
    std::vector<uint32_t> generate_greedy(uint32_t token, uint32_t pos, uint32_t n) {
        std::vector<uint32_t> out(n);
        ctx_.check(wick_rocm_lfm2_generate_greedy(ctx_.raw(), m_, token, pos, n, out.data()));
        return out;
    }

    // supports_embedding_input() == true: steps and prompts fed with hidden-size vectors, and steps that stop after the output norm
    std::vector<float> forward_from_embedding(const std::vector<float>& embedding, uint32_t pos) {
        check_embedding(embedding.size(), 1);
        std::vector<float> logits(cfg_.vocab_size);
        ctx_.check(wick_rocm_lfm2_forward_from_embedding(ctx_.raw(), m_, embedding.data(), pos, logits.data()));
        return logits;
    }
    std::vector<float> forward_embedding(uint32_t token, uint32_t pos) {
        std::vector<float> hidden(cfg_.hidden_size);
        ctx_.check(wick_rocm_lfm2_forward_embedding(ctx_.raw(), m_, token, pos, hidden.data()));
        return hidden;
    }
    std::vector<float> forward_hidden_from_embedding(const std::vector<float>& embedding, uint32_t pos) {
        check_embedding(embedding.size(), 1);
        std::vector<float> hidden(cfg_.hidden_size);
        ctx_.check(wick_rocm_lfm2_forward_hidden_from_embedding(ctx_.raw(), m_, embedding.data(), pos, hidden.data()));
        return hidden;
    }
    std::vector<float> forward_prefill_from_embeddings(const std::vector<float>& embeddings, uint32_t n_tokens, uint32_t start_pos) {
        check_embedding(embeddings.size(), n_tokens);
        std::vector<float> logits(cfg_.vocab_size);
        ctx_.check(wick_rocm_lfm2_forward_prefill_from_embeddings(ctx_.raw(), m_, embeddings.data(), n_tokens, start_pos, logits.data()));
        return logits;
    }

    // snapshot_state / restore_state: the state after seq_len positions as bytes (per layer: keys then values, or the conv buffer)
    std::vector<uint8_t> snapshot_state(uint32_t seq_len) {
        std::vector<uint8_t> out(wick_rocm_lfm2_state_bytes(m_, seq_len));
        ctx_.check(wick_rocm_lfm2_snapshot_state(ctx_.raw(), m_, seq_len, out.data(), out.size()));
        return out;
    }
    void restore_state(const std::vector<uint8_t>& snapshot, uint32_t seq_len) {
        ctx_.check(wick_rocm_lfm2_restore_state(ctx_.raw(), m_, seq_len, snapshot.data(), snapshot.size()));
    }
    // supports_kv_shift() == true: shift_kv on a state of seq_len positions; returns the new position count
    uint32_t shift_kv(uint32_t seq_len, uint32_t n_keep, uint32_t shift) {
        ctx_.check(wick_rocm_lfm2_shift_kv(ctx_.raw(), m_, seq_len, n_keep, shift));
        return seq_len - shift;
    }

private:
    void check_embedding(size_t len, size_t frames) const {
        if (frames == 0 || len != frames * cfg_.hidden_size) throw std::invalid_argument("embedding length != frames * hidden_size");
    }
    RocmContext& ctx_;
    wick_rocm_lfm2* m_ = nullptr;
    wick_rocm_lfm2_config cfg_{};
};

}  // namespace wick
