// Self-test of the C++ host mirror, linked STATICALLY against libwick_rocm.a the way a
// Rust build.rs would link it.  Self-contained checks (closed forms and invariants):
//   * the Q8_0 closed form of the reference's test_q8_0_gemm_standalone
//     (wick/tests/bench_perf.rs:852-971): m=64, k=32, n=4, scale 1/(row+1),
//     quants -16..15, x == 1  ->  y[col*m + row] ~= -16/(row+1);
//   * GEMM column j == GEMV of column j (the reference's invariant, simd.rs:1440-1623);
//   * encode_gemv (fused quantize) == quantize_columns + gemv_with_preq, bit for bit;
//   * error statuses instead of aborts.
// Prints "selftest OK" and exits 0 on success.
// With a GGUF file as argument it instead loads that LFM2 model through the mirror's RocmLfm2Model and prints
//   tokens: <ten greedy picks from token 17 at position 0>
//   prefill: <argmax of forward_prefill over those picks> <argmax of the same tokens fed one by one>
// for the caller to compare with another binding of the same library.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "rocm_backend.hpp"

// f32 -> f16 bits, round-to-nearest-even, for normal-range positive values (the scales used here).
static uint16_t f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t e = ((x >> 23) & 0xff) - 112u, m = x & 0x7fffffu;
    uint32_t r = (e << 10) | (m >> 13), rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
    return (uint16_t)r;
}

static size_t argmax(const std::vector<float>& v) {
    size_t best = 0;
    for (size_t i = 1; i < v.size(); i++)
        if (v[i] >= v[best]) best = i;  // the last of equal maxima, as the reference's cpu_argmax picks
    return best;
}

static int model_check(const char* path) {
    wick::RocmContext ctx(0);
    std::vector<uint32_t> picks;
    {
        wick::GgufFile gguf(path);
        wick::RocmLfm2Model model(ctx, gguf, 64);
        if (model.config().vocab_size == 0 || model.gpu_memory_bytes() == 0) return 1;
        picks = model.generate_greedy(17, 0, 10);
        std::printf("tokens:");
        for (uint32_t t : picks) std::printf(" %u", t);
        std::printf("\n");
        model.reset();
        uint32_t tok = 17;
        for (uint32_t pos = 0; pos < 10; pos++) {
            tok = model.forward_greedy(tok, pos);
            if (tok != picks[pos]) { std::printf("forward_greedy differs from generate_greedy at %u\n", pos); return 1; }
        }
        model.reset();
        const size_t a = argmax(model.forward_prefill(picks, 0));
        model.reset();
        std::vector<float> logits;
        for (uint32_t pos = 0; pos < picks.size(); pos++) logits = model.forward(picks[pos], pos);
        std::printf("prefill: %zu %zu\n", a, argmax(logits));
        // state snapshot: the step after a restore repeats the step after the snapshot
        const std::vector<uint8_t> snap = model.snapshot_state(10);
        const std::vector<float> first = model.forward(picks[0], 10);
        model.restore_state(snap, 10);
        if (model.forward(picks[0], 10) != first) { std::printf("restore_state does not bring the snapshot back\n"); return 1; }
        // a token's hidden state fed back as an embedding-input step, a context shift, then a step at the shifted position
        const std::vector<float> hidden = model.forward_embedding(picks[1], 11);
        const std::vector<float> after = model.forward_from_embedding(hidden, 12);
        if (hidden.size() != model.config().hidden_size || after.size() != model.config().vocab_size || !std::isfinite(after[0])) return 1;
        if (model.shift_kv(13, 2, 5) != 8 || !std::isfinite(model.forward(picks[2], 8)[0])) { std::printf("shift_kv failed\n"); return 1; }
        bool bad_len = false;
        try { model.forward_prefill_from_embeddings(hidden, 2, 0); } catch (const std::invalid_argument&) { bad_len = true; }
        if (!bad_len) { std::printf("embedding length not checked\n"); return 1; }
        bool threw = false;
        try { model.forward(model.config().vocab_size, 0); } catch (const wick::BackendError& e) { threw = e.status == WICK_ROCM_ERR_INVALID_ARG; }
        if (!threw) { std::printf("token out of range not reported\n"); return 1; }
    }
    std::printf("selftest OK\n");
    return 0;
}

int main(int argc, char** argv) {
    try {
        if (argc > 1) return model_check(argv[1]);
        wick::RocmContext ctx(0);
        // --- closed form ---------------------------------------------------------
        const uint32_t m = 64, k = 32, n = 4;
        std::vector<uint8_t> wbytes;
        for (uint32_t r = 0; r < m; r++) {
            uint16_t h = f32_to_f16(1.0f / (float)(r + 1));
            wbytes.push_back(h & 0xff), wbytes.push_back(h >> 8);
            for (int j = 0; j < 32; j++) wbytes.push_back((uint8_t)(int8_t)(j - 16));
        }
        auto w = ctx.upload_weight(wbytes.data(), wbytes.size(), wick::DType::Q8_0, m, k);
        std::vector<float> x(n * k, 1.0f);
        auto bx = ctx.create_buffer(x.size() * 4), by = ctx.create_buffer(m * n * 4);
        ctx.write(bx, x.data(), x.size() * 4);
        ctx.encode_gemm(w, bx, 0, by, 0, n, k, m);
        auto y = ctx.read_f32(by, m * n);
        for (uint32_t c = 0; c < n; c++)
            for (uint32_t r = 0; r < m; r++) {
                float expect = -16.0f / (float)(r + 1);
                if (!(std::fabs(y[c * m + r] - expect) < 1e-2f * std::fabs(expect) + 1e-6f)) {
                    std::printf("closed form mismatch at col %u row %u: %g vs %g\n", c, r, y[c * m + r], expect);
                    return 1;
                }
            }
        // --- GEMM column == GEMV, fused == two-step ---------------------------------
        const uint32_t M = 300, K = 512, N = 40;
        std::vector<uint8_t> wb((size_t)M * (K / 32) * 18);
        uint64_t s = 88172645463325252ull;
        for (size_t i = 0; i < wb.size(); i++) { s ^= s << 13; s ^= s >> 7; s ^= s << 17; wb[i] = (uint8_t)(s >> 24); }
        for (size_t b = 0; b < wb.size(); b += 18) wb[b + 1] = (wb[b + 1] & 0x3b);  // finite, modest f16 scales
        auto W = ctx.upload_weight(wb.data(), wb.size(), wick::DType::Q4_0, M, K);
        std::vector<float> X((size_t)N * K);
        for (auto& v : X) { s ^= s << 13; s ^= s >> 7; s ^= s << 17; v = (float)((int64_t)(s >> 40) - (1 << 23)) / (float)(1 << 22); }
        auto bX = ctx.create_buffer(X.size() * 4), bQ = ctx.create_buffer((size_t)N * K), bS = ctx.create_buffer((size_t)N * (K / 32) * 4);
        auto bC = ctx.create_buffer((size_t)M * N * 4), bV = ctx.create_buffer(M * 4), bV2 = ctx.create_buffer(M * 4);
        ctx.write(bX, X.data(), X.size() * 4);
        ctx.quantize_columns(bX, N, K, K, bQ, bS);
        ctx.gemm_preq(W, bS, bQ, N, bC);
        auto C = ctx.read_f32(bC, (size_t)M * N);
        for (uint32_t j : {0u, 7u, 39u}) {
            wick::Buffer q{static_cast<char*>(bQ.ptr) + (size_t)j * K, K}, sc{static_cast<char*>(bS.ptr) + (size_t)j * (K / 32) * 4, K / 32 * 4};
            ctx.gemv_with_preq(W, sc, q, bV);
            ctx.encode_gemv(W, bX, (uint64_t)j * K * 4, bV2, 0);
            auto v = ctx.read_f32(bV, M), v2 = ctx.read_f32(bV2, M);
            double num = 0, den = 0;
            for (uint32_t i = 0; i < M; i++) {
                if (std::memcmp(&v[i], &v2[i], 4) != 0) { std::printf("fused != two-step at row %u col %u\n", i, j); return 1; }
                double d = (double)C[(size_t)i * N + j] - (double)v[i];
                num += d * d, den += (double)v[i] * v[i];
            }
            if (!(std::sqrt(num / den) < 1e-5)) { std::printf("gemm column %u differs from gemv: rel %g\n", j, std::sqrt(num / den)); return 1; }
        }
        // --- errors are statuses, not aborts -------------------------------------------
        bool threw = false;
        try { ctx.upload_weight(wb.data(), 18, static_cast<wick::DType>(12), 1, 32); } catch (const wick::BackendError& e) { threw = e.status == WICK_ROCM_ERR_UNSUPPORTED_DTYPE; }
        if (!threw) { std::printf("unsupported dtype not reported\n"); return 1; }
        threw = false;
        try { ctx.upload_weight(wb.data(), 18, wick::DType::Q4_0, 1, 48); } catch (const wick::BackendError& e) { threw = e.status == WICK_ROCM_ERR_BAD_SHAPE; }
        if (!threw) { std::printf("k %% 32 != 0 not reported\n"); return 1; }
        ctx.free_weight(w), ctx.free_weight(W);
        std::printf("selftest OK\n");
        return 0;
    } catch (const std::exception& e) {
        std::printf("selftest FAILED: %s\n", e.what());
        return 1;
    }
}
