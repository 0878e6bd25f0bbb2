// C++ tests of include/agpu_nn.hpp, written like the reference's own unit tests: closed-form
// deterministic inputs, an inline CPU loop as the expected value, an absolute tolerance.
// Sources of the cases: nn/ops/quantize.rs:198-267, nn/layers/int4_linear.rs:71-147,
// tests_transformer.rs:12-206,739-833,1963-2120, nn/models/gpt2.rs:1601-1843 (int4 model: finite, >= 1 token),
// tests_inference.rs:6114-6171 (cached == uncached).  Needs a GPU; run by tests/test_gpu_cpp.py.
#include <cmath>
#include <cstdio>
#include <functional>
#include <string>
#include <vector>

#include "../../include/agpu_nn.hpp"

using namespace agpu::nn;

static int g_failed = 0;
#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("  CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++g_failed;                                                    \
        }                                                                  \
    } while (0)

static void run(const char *name, const std::function<void()> &fn) {
    const int before = g_failed;
    try {
        fn();
    } catch (const std::exception &e) {
        std::printf("  unexpected exception: %s\n", e.what());
        ++g_failed;
    }
    std::printf("%s %s\n", g_failed == before ? "ok  " : "FAIL", name);
    std::fflush(stdout);
}

template <class F>
static bool throws_kind(NnError::Kind k, F &&f) {
    try {
        f();
    } catch (const NnError &e) {
        return e.kind == k;
    }
    return false;
}

static float max_abs_diff(const std::vector<float> &a, const std::vector<double> &b) {
    float m = 0;
    for (size_t i = 0; i < a.size(); ++i) m = std::fmax(m, std::fabs(a[i] - (float)b[i]));
    return m;
}

// deterministic pseudo-random floats in [-1, 1)
static float lcg(uint32_t &s) {
    s = s * 1664525u + 1013904223u;
    return (float)((s >> 8) & 0xFFFF) / 32768.0f - 1.0f;
}

int main() {
    Registry reg = KernelRegistry::init_default(0);

    run("registry.get", [&] {
        CHECK(reg->get("int4_gemm_w4a16") == "agpu_int4_linear");
        CHECK(reg->get("flash_attention_kv") == "agpu_attention");
        CHECK(throws_kind(NnError::Kind::KernelNotFound, [&] { reg->get("winograd_f23"); }));
    });

    run("gpu_tensor", [&] {
        std::vector<float> h(24);
        for (size_t i = 0; i < h.size(); ++i) h[i] = (float)i * 0.5f;
        GpuTensor t = GpuTensor::from_host(h, {2, 3, 4}, reg);
        CHECK(t.ndim() == 3 && t.numel() == 24 && t.dim(2) == 4);
        CHECK(t.to_host() == h);
        GpuTensor r = t.reshape({6, 4});
        CHECK(r.data() == t.data());  // shares memory (tensor.rs:201-222)
        GpuTensor c = t.clone_tensor();
        CHECK(c.data() != t.data() && c.to_host() == h);
        CHECK(GpuTensor::zeros({5}, reg).to_host() == std::vector<float>(5, 0.0f));
        CHECK(throws_kind(NnError::Kind::ShapeMismatch, [&] { t.reshape({5, 5}); }));
        CHECK(throws_kind(NnError::Kind::ShapeMismatch, [&] { GpuTensor::from_host(h, {5, 5}, reg); }));
        CHECK(throws_kind(NnError::Kind::DimOutOfRange, [&] { t.dim(3); }));
    });

    run("gpu_array_residency", [&] {  // gpu_array.rs:516-640: upload on demand, kernel output synced back on read
        for (size_t n : {size_t(100), size_t(16384 + 77)}) {  // pinned mapped backend, then device memory
            std::vector<float> h(n);
            for (size_t i = 0; i < n; ++i) h[i] = ((float)(i % 41) - 20.0f) * 0.125f;
            auto in = GpuArray<float>::from_vec(h);
            auto out = GpuArray<float>::zeroed(n);
            CHECK(in.residency() == Residency::HostOnly);
            const float *din = in.device_ptr(reg);
            float *dout = out.device_ptr(reg);
            CHECK(in.residency() == Residency::Synced && out.residency() == Residency::Synced);
            CHECK(in.is_mapped() == (n * 4 < kGpuArrayMappedThresholdBytes));
            CHECK(in.device_ptr(reg) == din);  // Synced: no new storage, no copy
            // y = x + x through the device copies; the kernel's output is marked, the next read syncs it back
            reg->check(agpu_memcpy_d2d(reg->device(), dout, din, n * sizeof(float)));
            reg->check(agpu_add_inplace(reg->device(), dout, din, n));
            out.mark_device_dirty();
            CHECK(out.residency() == Residency::DeviceOnly);
            bool ok = true;
            for (size_t i = 0; i < n; ++i) ok = ok && out[i] == 2.0f * h[i];
            CHECK(ok);
            CHECK(out.residency() == Residency::Synced);
            // a host write makes the device copy stale; the next ensure_device uploads into the same storage
            in.write()[3] = 1000.0f;
            CHECK(in.residency() == Residency::HostDirty);
            CHECK(in.device_ptr(reg) == din && in.residency() == Residency::Synced);
            reg->check(agpu_memcpy_d2d(reg->device(), dout, din, n * sizeof(float)));
            out.mark_device_dirty();
            CHECK(out[3] == 1000.0f && out[4] == h[4]);
            // a write while the device copy is the newer one syncs back first, so the kernel's results are kept
            reg->check(agpu_add_inplace(reg->device(), dout, din, n));
            out.mark_device_dirty();
            out.write()[0] = -1.0f;
            CHECK(out.residency() == Residency::HostDirty && out[3] == 2000.0f && out[0] == -1.0f);
        }
        auto empty = GpuArray<float>::from_vec({});
        CHECK(empty.ensure_device(reg) == 0 && empty.residency() == Residency::Synced);  // gpu_array.rs:262-266
    });

    run("quantize_weight_int4_roundtrip", [&] {  // quantize.rs:217-267
        const size_t k = 8, n = 4;
        std::vector<float> w(k * n);
        for (size_t i = 0; i < w.size(); ++i) w[i] = ((float)i - 16.0f) * 0.1f;
        auto [packed, scales] = ops::quantize::quantize_weight_int4(w, k, n, 128);
        CHECK(packed.size() == 4 && scales.size() == 4);
        for (size_t col = 0; col < n; ++col)
            for (size_t bit = 0; bit < 8; ++bit) {
                const float rec = (float)ops::quantize::unpack_int4(packed[col], bit) * scales[col];
                CHECK(std::fabs(rec - w[bit * n + col]) < scales[col] + 1e-6f);
            }
        uint32_t word = 0;
        for (int i = 0; i < 8; ++i) word |= ((uint32_t)(i - 4 + 8) & 0xF) << (i * 4);
        for (int i = 0; i < 8; ++i) CHECK(ops::quantize::unpack_int4(word, i) == i - 4);
        CHECK(throws_kind(NnError::Kind::ShapeMismatch, [&] { ops::quantize::quantize_weight_int4(std::vector<float>(24), 12, 2, 4); }));
    });

    run("int4_linear_forward", [&] {  // int4_linear.rs:71-147 against an f64 loop over the dequantised weights
        const size_t K = 768, N = 200, g = 32;
        uint32_t s = 7;
        std::vector<float> w(K * N), bias(N), x(3 * K);
        for (auto &v : w) v = lcg(s) * 0.05f;
        for (auto &v : bias) v = lcg(s) * 0.1f;
        for (auto &v : x) v = lcg(s);
        auto [packed, scales] = ops::quantize::quantize_weight_int4(w, K, N, g);
        Int4Linear lin(packed, scales, bias, K, N, g, reg);
        CHECK(lin.memory_bytes() == K / 8 * N * 4 + K / g * N * 4 + N * 4);
        std::vector<double> ref(3 * N);
        for (size_t m = 0; m < 3; ++m)
            for (size_t n = 0; n < N; ++n) {
                double acc = 0;
                for (size_t k = 0; k < K; ++k) {
                    const float wq = (float)ops::quantize::unpack_int4(packed[(k / 8) * N + n], k % 8) * scales[(k / g) * N + n];
                    acc += (double)x[m * K + k] * (double)wq;
                }
                ref[m * N + n] = acc + bias[n];
            }
        GpuTensor y = lin.forward(GpuTensor::from_host(x, {3, K}, reg));
        CHECK(y.shape() == (std::vector<size_t>{3, N}));
        CHECK(max_abs_diff(y.to_host(), ref) <= 1e-4f);
        GpuTensor y3 = lin.forward(GpuTensor::from_host(x, {1, 3, K}, reg));  // leading dims kept for rank > 2
        CHECK(y3.shape() == (std::vector<size_t>{1, 3, N}));
        GpuTensor y1 = lin.forward(GpuTensor::from_host(std::vector<float>(x.begin(), x.begin() + K), {K}, reg));
        CHECK(y1.shape() == (std::vector<size_t>{1, N}));  // rank 1 -> [1, N]
        CHECK(throws_kind(NnError::Kind::ShapeMismatch, [&] { lin.forward(GpuTensor::zeros({2, 100}, reg)); }));
        // ops::int4_matmul quantizes B itself (group 128): close to the f32 product within the quantisation error
        GpuTensor b = GpuTensor::from_host(w, {K, N}, reg);
        GpuTensor c = ops::int4_matmul(GpuTensor::from_host(x, {3, K}, reg), b, reg);
        GpuTensor cf = ops::matmul(GpuTensor::from_host(x, {3, K}, reg), b, reg);
        float worst = 0;
        auto hc = c.to_host(), hf = cf.to_host();
        for (size_t i = 0; i < hc.size(); ++i) worst = std::fmax(worst, std::fabs(hc[i] - hf[i]));
        CHECK(worst < 0.2f && worst > 0.0f);
    });

    run("layer_norm_4x768", [&] {  // tests_transformer.rs:12-125
        const size_t rows = 4, d = 768;
        std::vector<float> x(rows * d), gamma(d), beta(d);
        for (size_t i = 0; i < rows; ++i)
            for (size_t j = 0; j < d; ++j) x[i * d + j] = ((float)((i * 7 + j * 3) % 11) - 5.0f) * 0.1f;
        for (size_t j = 0; j < d; ++j) {
            gamma[j] = 1.0f + (float)j * 0.001f;
            beta[j] = (float)j * 0.0001f;
        }
        LayerNorm ln(gamma, beta, 1e-5f, reg);
        std::vector<double> ref(rows * d);
        for (size_t i = 0; i < rows; ++i) {
            double mean = 0, var = 0;
            for (size_t j = 0; j < d; ++j) mean += x[i * d + j];
            mean /= d;
            for (size_t j = 0; j < d; ++j) var += (x[i * d + j] - mean) * (x[i * d + j] - mean);
            var /= d;
            for (size_t j = 0; j < d; ++j) ref[i * d + j] = gamma[j] * (x[i * d + j] - mean) / std::sqrt(var + 1e-5) + beta[j];
        }
        CHECK(max_abs_diff(ln.forward(GpuTensor::from_host(x, {rows, d}, reg)).to_host(), ref) <= 1e-5f);
    });

    run("gelu_grid", [&] {  // tests_transformer.rs:128-206, tolerance 1e-4 there
        const size_t n = 1024;
        std::vector<float> x(n);
        std::vector<double> ref(n);
        for (size_t i = 0; i < n; ++i) {
            x[i] = -5.0f + 10.0f * (float)i / (float)(n - 1);
            const double v = x[i];
            ref[i] = v * 0.5 * (1.0 + std::tanh(0.7978845608028654 * (v + 0.044715 * v * v * v)));
        }
        CHECK(max_abs_diff(Gelu(reg).forward(GpuTensor::from_host(x, {n}, reg)).to_host(), ref) <= 1e-6f);
    });

    run("embedding_exact", [&] {  // tests_transformer.rs:739-833
        const size_t V = 50257, P = 16, d = 8;
        std::vector<float> wte(V * d), wpe(P * d);
        for (size_t i = 0; i < wte.size(); ++i) wte[i] = (float)(i % 977) * 0.001f;
        for (size_t i = 0; i < wpe.size(); ++i) wpe[i] = (float)(i % 13) * 0.01f;
        Embedding emb(wte, wpe, V, P, d, reg);
        std::vector<uint32_t> ids = {0, 50256, 17, 50256};
        GpuBufferU32 dev_ids(ids, reg);
        auto out = emb.forward_tokens_with_offset(dev_ids, ids.size(), 5).to_host();
        for (size_t p = 0; p < ids.size(); ++p)
            for (size_t j = 0; j < d; ++j) CHECK(out[p * d + j] == wte[ids[p] * d + j] + wpe[(p + 5) * d + j]);
        CHECK(throws_kind(NnError::Kind::DimOutOfRange, [&] { emb.forward_tokens_with_offset(dev_ids, ids.size(), 14); }));
    });

    run("attention_kv_equals_last_row", [&] {  // tests_transformer.rs:1963-2120
        const size_t seq = 32, dh = 64;
        std::vector<float> q(seq * dh), k(seq * dh), v(seq * dh);
        for (size_t i = 0; i < seq * dh; ++i) {
            q[i] = (float)((i * 7 + 3) % 100) * 0.01f - 0.5f;
            k[i] = (float)((i * 13 + 5) % 100) * 0.01f - 0.5f;
            v[i] = (float)((i * 17 + 9) % 100) * 0.01f - 0.5f;
        }
        GpuTensor dq = GpuTensor::from_host(q, {seq, dh}, reg), dk = GpuTensor::from_host(k, {seq, dh}, reg),
                  dv = GpuTensor::from_host(v, {seq, dh}, reg);
        auto full = ops::multi_head_flash_attention(dq, dk, dv, seq, 1, dh, true, reg).to_host();
        GpuTensor q_last = GpuTensor::from_host(std::vector<float>(q.end() - dh, q.end()), {1, dh}, reg);
        auto one = ops::scaled_dot_product_attention_kv(q_last, dk, dv, 1, seq, seq - 1, seq, dh, reg).to_host();
        float worst = 0;
        for (size_t e = 0; e < dh; ++e) worst = std::fmax(worst, std::fabs(one[e] - full[(seq - 1) * dh + e]));
        CHECK(worst <= 1e-4f);
        for (size_t e = 0; e < dh; ++e) CHECK(std::fabs(full[e] - v[e]) <= 1e-6f);  // row 0 sees only key 0
        CHECK(throws_kind(NnError::Kind::ShapeMismatch,
                          [&] { ops::multi_head_flash_attention(dq, dk, dv, seq, 2, 32, true, reg); }));  // d_head must be 64
    });

    run("int4_gpt2_model", [&] {  // gpt2.rs:1601-1843 (finite logits, >= 1 token), tests_inference.rs:6114-6171
        Gpt2Config cfg{2, 128, 2, 503, 64, 1e-5f};
        Gpt2Weights w;
        uint32_t s = 99;
        auto fill = [&](std::vector<float> &v, size_t n, float scale) {
            v.resize(n);
            for (auto &e : v) e = lcg(s) * scale;
        };
        const size_t d = cfg.n_embd, ff = cfg.ffn_dim();
        fill(w.wte, cfg.vocab_size * d, 0.1f);
        fill(w.wpe, cfg.n_positions * d, 0.1f);
        w.ln_f_weight.assign(d, 1.0f);
        w.ln_f_bias.assign(d, 0.0f);
        w.layers.resize(cfg.n_layer);
        for (auto &L : w.layers) {
            L.ln_1_weight.assign(d, 1.0f); L.ln_1_bias.assign(d, 0.0f);
            L.ln_2_weight.assign(d, 1.0f); L.ln_2_bias.assign(d, 0.0f);
            fill(L.c_attn_weight, d * 3 * d, 0.1f); fill(L.c_attn_bias, 3 * d, 0.02f);
            fill(L.c_proj_weight, d * d, 0.1f); fill(L.c_proj_bias, d, 0.02f);
            fill(L.mlp_fc_weight, d * ff, 0.1f); fill(L.mlp_fc_bias, ff, 0.02f);
            fill(L.mlp_proj_weight, ff * d, 0.1f); fill(L.mlp_proj_bias, d, 0.02f);
        }
        for (int head : {AGPU_LM_HEAD_F32, AGPU_LM_HEAD_INT4}) {
            Int4Gpt2Model model = Int4Gpt2Model::from_weights(w, cfg, 32, reg, head);
            size_t per = 0;
            for (auto kn : {std::pair<size_t, size_t>{d, 3 * d}, {d, d}, {d, ff}, {ff, d}})
                per += kn.first / 8 * kn.second * 4 + kn.first / 32 * kn.second * 4 + kn.second * 4;
            CHECK(model.quantized_memory_bytes() == cfg.n_layer * per);
            std::vector<uint32_t> prompt = {5, 77, 300, 12, 499};
            GpuBufferU32 ids(prompt, reg);
            auto logits = model.forward(ids, prompt.size());
            CHECK(logits.shape() == (std::vector<size_t>{prompt.size(), cfg.vocab_size}));
            bool finite = true;
            for (float v : logits.to_host()) finite = finite && std::isfinite(v);
            CHECK(finite);
            auto unc = model.generate(prompt, 10, -1);
            auto cac = model.generate_cached(prompt, 10, -1);
            CHECK(unc.size() == prompt.size() + 10 && unc == cac);
            CHECK(model.cache_len() == prompt.size() + 9);
            CHECK(throws_kind(NnError::Kind::DimOutOfRange, [&] { model.generate_cached(prompt, 61, -1); }));
            // sampling: same seed, same continuation; k = 1 is the greedy one; the generator is xorshift64
            SimpleRng r1(7), r2(7), r3(9);
            auto s1 = model.generate_cached_sampling(prompt, 12, 8, 0.9f, r1, -1);
            auto s2 = model.generate_cached_sampling(prompt, 12, 8, 0.9f, r2, -1);
            CHECK(s1.size() == prompt.size() + 12 && s1 == s2);
            auto g1 = model.generate_cached_sampling(prompt, 10, 1, 1.0f, r3, -1);
            CHECK(g1 == cac);
            SimpleRng r4(1);
            CHECK(r4.next_f32() == 0.0f && *r4.state() == 0x40822041ull);  // one xorshift64 step from 1 (13, 7, 17)
            CHECK(r4.next_f32() == (float)(1048641ull) / 16777216.0f);
            // early exit: an unreachable threshold is greedy decoding, threshold 0 leaves after the first block
            auto ee = model.generate_cached_early_exit(prompt, 10, 2.0f, -1);
            CHECK(ee.first == cac && ee.second == std::vector<size_t>(10, model.config().n_layer));
            auto e0 = model.generate_cached_early_exit(prompt, 10, 0.0f, -1);
            CHECK(e0.first.size() == prompt.size() + 10 && e0.second.size() == 10 && e0.second[0] == model.config().n_layer);
            for (size_t i = 1; i < e0.second.size(); ++i) CHECK(e0.second[i] == 1);
            auto fe = model.forward_early_exit(prompt, 2.0f);
            CHECK(fe.second == model.config().n_layer && fe.first.shape() == std::vector<size_t>({prompt.size(), model.config().vocab_size}));
            CHECK(model.forward_early_exit(prompt, 0.0f).second == 1);
            CHECK(model.generate_cached(prompt, 10, -1) == cac);
        }
    });

    std::printf("%s: %d failed check(s)\n", g_failed ? "FAILED" : "PASSED", g_failed);
    return g_failed ? 1 : 0;
}
