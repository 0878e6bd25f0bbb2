// The GPT-2 example of the reference (examples/std/gpt2-inference/src/main.rs:22-135) in C++ over include/agpu_nn.hpp,
// step by step as there: initialise the device and the kernel registry, load a safetensors file of fp32 GPT-2 weights
// (model.rs:308-378: Conv1D [in, out] matrices, names with or without the "transformer." prefix), build the int4 model
// (every dense layer quantized at load, gpt2.rs:1362-1433), encode three prompts, one diagnostic forward, then for
// every prompt a greedy generation without and with the KV cache, their timings, and the check that both give the
// same tokens.
//
//   gpt2_inference MODEL.safetensors VOCAB.tiktoken [--max-new-tokens 50] [--group-size 32] [--int4-head] [--dry-run]
//                  [--print-tokens] [--prompt TEXT]...
//
// --prompt (repeatable) replaces the three prompts of the reference's program.
// --print-tokens adds a line with the token ids of every cached generation.  --dry-run stops before the device is
// touched: it reads both files and prints the model's geometry and the token ids of the three prompts (a check of the
// two readers on a machine without a GPU).
//
// VOCAB is the tokenizer's table in tiktoken's one-file format (base64 token, rank per line: r50k_base.tiktoken for
// GPT-2).  The tokenizer here is the published byte-pair scheme, lowest rank first, behind GPT-2's split pattern with
// ASCII letter and digit classes (bytes of multi-byte UTF-8 characters count as letters): enough for the prompts of
// this program; async-gpu_amd/tokenizer.py has the pattern with the Unicode classes.
#include <chrono>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "agpu_nn.hpp"

namespace {

using agpu::nn::Gpt2Config;
using agpu::nn::Gpt2LayerWeights;
using agpu::nn::Gpt2Weights;

// ---- safetensors: 8 bytes of header length, a JSON header {name: {dtype, shape, data_offsets}}, then the data ----
struct TensorInfo {
    std::string dtype;
    std::vector<size_t> shape;
    size_t begin = 0, end = 0;
};

class SafeTensors {
public:
    explicit SafeTensors(const std::string &path) {
        std::ifstream f(path, std::ios::binary);
        if (!f) throw std::runtime_error("Model file not found: " + path);
        unsigned char len8[8];
        f.read(reinterpret_cast<char *>(len8), 8);
        if (!f) throw std::runtime_error("safetensors: file too short");
        size_t n = 0;
        for (int i = 7; i >= 0; --i) n = (n << 8) | len8[i];
        std::string header(n, '\0');
        f.read(&header[0], (std::streamsize)n);
        if (!f) throw std::runtime_error("safetensors: header cut short");
        data_.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
        parse(header);
    }
    bool has(const std::string &name) const { return t_.count(name) != 0; }
    const TensorInfo &info(const std::string &name) const {
        auto it = t_.find(name);
        if (it == t_.end()) throw std::runtime_error("tensor '" + name + "' not found");
        return it->second;
    }
    // fp32 tensor `name` of exactly `numel` elements
    std::vector<float> f32(const std::string &name, size_t numel) const {
        const TensorInfo &ti = info(name);
        if (ti.dtype != "F32") throw std::runtime_error("tensor '" + name + "': expected F32, got " + ti.dtype);
        size_t n = 1;
        for (size_t s : ti.shape) n *= s;
        if (n != numel || ti.end - ti.begin != 4 * n || ti.end > data_.size())
            throw std::runtime_error("tensor '" + name + "': expected " + std::to_string(numel) + " elements, got " + std::to_string(n));
        std::vector<float> v(n);
        std::memcpy(v.data(), data_.data() + ti.begin, 4 * n);
        return v;
    }
    size_t total_params() const {
        size_t n = 0;
        for (const auto &kv : t_) {
            size_t e = 1;
            for (size_t s : kv.second.shape) e *= s;
            n += e;
        }
        return n;
    }
    size_t data_bytes() const { return data_.size(); }
    const std::map<std::string, TensorInfo> &tensors() const { return t_; }

private:
    // a JSON reader for this header: objects, arrays, strings, numbers
    const char *p_ = nullptr, *e_ = nullptr;
    void ws() {
        while (p_ < e_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
    }
    void expect(char c) {
        ws();
        if (p_ >= e_ || *p_ != c) throw std::runtime_error(std::string("safetensors header: expected '") + c + "'");
        ++p_;
    }
    std::string str() {
        expect('"');
        std::string s;
        while (p_ < e_ && *p_ != '"') {
            if (*p_ == '\\' && p_ + 1 < e_) {
                ++p_;
                switch (*p_) {
                    case 'n': s += '\n'; break;
                    case 't': s += '\t'; break;
                    case 'u': s += '?'; p_ += 4; break;  // names and dtypes are ASCII
                    default: s += *p_;
                }
                ++p_;
            } else {
                s += *p_++;
            }
        }
        expect('"');
        return s;
    }
    size_t number() {
        ws();
        size_t v = 0;
        if (p_ >= e_ || *p_ < '0' || *p_ > '9') throw std::runtime_error("safetensors header: expected a number");
        while (p_ < e_ && *p_ >= '0' && *p_ <= '9') v = v * 10 + (size_t)(*p_++ - '0');
        return v;
    }
    void skip_value() {  // the values of __metadata__
        ws();
        if (p_ >= e_) return;
        if (*p_ == '"') {
            (void)str();
        } else if (*p_ == '{' || *p_ == '[') {
            const char open = *p_, close = open == '{' ? '}' : ']';
            ++p_;
            ws();
            while (p_ < e_ && *p_ != close) {
                if (open == '{') {
                    (void)str();
                    expect(':');
                }
                skip_value();
                ws();
                if (p_ < e_ && *p_ == ',') ++p_;
                ws();
            }
            expect(close);
        } else {
            while (p_ < e_ && *p_ != ',' && *p_ != '}' && *p_ != ']') ++p_;
        }
    }
    void parse(const std::string &h) {
        p_ = h.data();
        e_ = p_ + h.size();
        expect('{');
        ws();
        while (p_ < e_ && *p_ != '}') {
            const std::string name = str();
            expect(':');
            if (name == "__metadata__") {
                skip_value();
            } else {
                TensorInfo ti;
                expect('{');
                ws();
                while (p_ < e_ && *p_ != '}') {
                    const std::string key = str();
                    expect(':');
                    if (key == "dtype") {
                        ti.dtype = str();
                    } else if (key == "shape" || key == "data_offsets") {
                        std::vector<size_t> v;
                        expect('[');
                        ws();
                        while (p_ < e_ && *p_ != ']') {
                            v.push_back(number());
                            ws();
                            if (p_ < e_ && *p_ == ',') ++p_;
                            ws();
                        }
                        expect(']');
                        if (key == "shape") {
                            ti.shape = v;
                        } else {
                            if (v.size() != 2) throw std::runtime_error("safetensors header: data_offsets of '" + name + "'");
                            ti.begin = v[0];
                            ti.end = v[1];
                        }
                    } else {
                        skip_value();
                    }
                    ws();
                    if (p_ < e_ && *p_ == ',') ++p_;
                    ws();
                }
                expect('}');
                t_[name] = ti;
            }
            ws();
            if (p_ < e_ && *p_ == ',') ++p_;
            ws();
        }
    }
    std::map<std::string, TensorInfo> t_;
    std::vector<char> data_;
};

// load_gpt2_weights (model.rs:308-378): the geometry from the shapes, every tensor checked against it
Gpt2Weights load_gpt2_weights(const SafeTensors &st, Gpt2Config &cfg) {
    const std::string pre = st.has("wte.weight") ? "" : "transformer.";
    const TensorInfo &wte = st.info(pre + "wte.weight"), &wpe = st.info(pre + "wpe.weight");
    if (wte.shape.size() != 2 || wpe.shape.size() != 2 || wpe.shape[1] != wte.shape[1]) throw std::runtime_error("wte / wpe: unexpected shapes");
    size_t n_layer = 0;
    while (st.has(pre + "h." + std::to_string(n_layer) + ".ln_1.weight")) ++n_layer;
    if (n_layer == 0) throw std::runtime_error("tensor '" + pre + "h.0.ln_1.weight' not found");
    cfg = Gpt2Config{n_layer, wte.shape[1], wte.shape[1] / 64, wte.shape[0], wpe.shape[0]};
    const size_t d = cfg.n_embd, ff = cfg.ffn_dim();
    Gpt2Weights w;
    w.wte = st.f32(pre + "wte.weight", cfg.vocab_size * d);
    w.wpe = st.f32(pre + "wpe.weight", cfg.n_positions * d);
    w.ln_f_weight = st.f32(pre + "ln_f.weight", d);
    w.ln_f_bias = st.f32(pre + "ln_f.bias", d);
    for (size_t l = 0; l < n_layer; ++l) {
        const std::string h = pre + "h." + std::to_string(l) + ".";
        Gpt2LayerWeights L;
        L.ln_1_weight = st.f32(h + "ln_1.weight", d);
        L.ln_1_bias = st.f32(h + "ln_1.bias", d);
        L.c_attn_weight = st.f32(h + "attn.c_attn.weight", d * 3 * d);
        L.c_attn_bias = st.f32(h + "attn.c_attn.bias", 3 * d);
        L.c_proj_weight = st.f32(h + "attn.c_proj.weight", d * d);
        L.c_proj_bias = st.f32(h + "attn.c_proj.bias", d);
        L.ln_2_weight = st.f32(h + "ln_2.weight", d);
        L.ln_2_bias = st.f32(h + "ln_2.bias", d);
        L.mlp_fc_weight = st.f32(h + "mlp.c_fc.weight", d * ff);
        L.mlp_fc_bias = st.f32(h + "mlp.c_fc.bias", ff);
        L.mlp_proj_weight = st.f32(h + "mlp.c_proj.weight", ff * d);
        L.mlp_proj_bias = st.f32(h + "mlp.c_proj.bias", d);
        w.layers.push_back(std::move(L));
    }
    return w;
}

// ---- tokenizer (tokenizer.rs:1-62: tiktoken's r50k_base behind encode / decode) ----
class Tokenizer {
public:
    explicit Tokenizer(const std::string &path) {
        std::ifstream f(path);
        if (!f) throw std::runtime_error("Vocabulary file not found: " + path);
        std::string line;
        while (std::getline(f, line)) {
            const size_t sp = line.find(' ');
            if (sp == std::string::npos) continue;
            const std::string tok = base64(line.substr(0, sp));
            const uint32_t rank = (uint32_t)std::stoul(line.substr(sp + 1));
            ranks_[tok] = rank;
            if (by_rank_.size() <= rank) by_rank_.resize(rank + 1);
            by_rank_[rank] = tok;
        }
        if (ranks_.empty()) throw std::runtime_error("Vocabulary file holds no tokens: " + path);
    }
    std::vector<uint32_t> encode(const std::string &text) const {
        std::vector<uint32_t> out;
        size_t i = 0;
        while (i < text.size()) {
            const size_t n = piece_len(text, i);
            merge(text.substr(i, n), out);
            i += n;
        }
        return out;
    }
    // the text of `ids`; "[decode error]" (main.rs:90-92) for an unknown id or bytes that are not UTF-8
    std::string decode(const std::vector<uint32_t> &ids) const {
        std::string s;
        for (uint32_t id : ids) {
            if (id >= by_rank_.size()) return "[decode error]";
            s += by_rank_[id];
        }
        for (size_t i = 0; i < s.size();) {
            const unsigned char c = (unsigned char)s[i];
            const size_t n = c < 0x80 ? 1 : (c >> 5) == 6 ? 2 : (c >> 4) == 14 ? 3 : (c >> 3) == 30 ? 4 : 0;
            if (n == 0 || i + n > s.size()) return "[decode error]";
            for (size_t k = 1; k < n; ++k)
                if (((unsigned char)s[i + k] >> 6) != 2) return "[decode error]";
            i += n;
        }
        return s;
    }

private:
    static bool is_space(unsigned char c) { return c == ' ' || (c >= 9 && c <= 13); }
    static bool is_letter(unsigned char c) { return (c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || c >= 0x80; }
    static bool is_digit(unsigned char c) { return c >= '0' && c <= '9'; }
    static bool is_other(unsigned char c) { return !is_space(c) && !is_letter(c) && !is_digit(c); }
    // 's|'t|'re|'ve|'m|'ll|'d| ?L+| ?N+| ?[^\s L N]+|\s+(?!\S)|\s+ : length of the piece that starts at i
    static size_t piece_len(const std::string &t, size_t i) {
        const size_t n = t.size();
        auto at = [&](size_t k) { return k < n ? (unsigned char)t[k] : (unsigned char)0; };
        if (t[i] == '\'') {
            for (const char *c : {"'s", "'t", "'re", "'ve", "'m", "'ll", "'d"})
                if (t.compare(i, std::strlen(c), c) == 0) return std::strlen(c);
        }
        const size_t j = (t[i] == ' ' && i + 1 < n && !is_space(at(i + 1))) ? i + 1 : i;
        if (j < n && !is_space(at(j))) {
            bool (*cls)(unsigned char) = is_letter(at(j)) ? is_letter : (is_digit(at(j)) ? is_digit : is_other);
            size_t k = j;
            while (k < n && cls(at(k))) ++k;
            return k - i;
        }
        size_t k = i;
        while (k < n && is_space(at(k))) ++k;
        if (k < n && k - i > 1) --k;  // whitespace before a word leaves its last character to that word
        return k - i;
    }
    void merge(const std::string &piece, std::vector<uint32_t> &out) const {
        std::vector<std::string> parts;
        for (char c : piece) parts.emplace_back(1, c);
        for (;;) {
            size_t best = parts.size();
            uint32_t best_rank = 0xffffffffu;
            for (size_t k = 0; k + 1 < parts.size(); ++k) {
                auto it = ranks_.find(parts[k] + parts[k + 1]);
                if (it != ranks_.end() && it->second < best_rank) {
                    best_rank = it->second;
                    best = k;
                }
            }
            if (best == parts.size()) break;
            parts[best] += parts[best + 1];
            parts.erase(parts.begin() + (long)best + 1);
        }
        for (const std::string &p : parts) {
            auto it = ranks_.find(p);
            if (it == ranks_.end()) throw std::runtime_error("tokenizer: a byte of the text is not in the vocabulary");
            out.push_back(it->second);
        }
    }
    static std::string base64(const std::string &s) {
        std::string out;
        unsigned acc = 0;
        int bits = 0;
        for (char c : s) {
            int v;
            if (c >= 'A' && c <= 'Z') v = c - 'A';
            else if (c >= 'a' && c <= 'z') v = c - 'a' + 26;
            else if (c >= '0' && c <= '9') v = c - '0' + 52;
            else if (c == '+') v = 62;
            else if (c == '/') v = 63;
            else continue;  // padding
            acc = (acc << 6) | (unsigned)v;
            bits += 6;
            if (bits >= 8) {
                bits -= 8;
                out += (char)((acc >> bits) & 0xffu);
            }
        }
        return out;
    }
    std::map<std::string, uint32_t> ranks_;
    std::vector<std::string> by_rank_;
};

double ms_since(const std::chrono::steady_clock::time_point &t0) {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

using Prompts = std::vector<std::string>;
const Prompts kPrompts = {"The capital of France is", "In a world where AI", "Once upon a time"};

int dry_run(const std::string &model_path, const std::string &vocab_path, const Prompts &prompts) {
    const SafeTensors st(model_path);
    Gpt2Config config{};
    const Gpt2Weights weights = load_gpt2_weights(st, config);
    std::printf("Loaded %.1fM params (%.1f MB)\n", st.total_params() / 1e6, st.data_bytes() / 1e6);
    std::printf("Config: n_layer=%zu n_embd=%zu n_head=%zu vocab_size=%zu n_positions=%zu\n", config.n_layer, config.n_embd, config.n_head,
                config.vocab_size, config.n_positions);
    double sum = 0.0;
    for (float v : weights.layers.back().mlp_proj_weight) sum += v;
    std::printf("Checksum of the last mlp.c_proj.weight: %.9g\n", sum);
    const Tokenizer tokenizer(vocab_path);
    for (const std::string &prompt : prompts) {
        const std::vector<uint32_t> tokens = tokenizer.encode(prompt);
        std::printf("Tokens:");
        for (uint32_t t : tokens) std::printf(" %u", t);
        std::printf("\nDecoded: %s\n", tokenizer.decode(tokens).c_str());
    }
    return 0;
}

int run(const std::string &model_path, const std::string &vocab_path, size_t max_new_tokens, size_t group_size, bool int4_head,
        bool print_tokens, const Prompts &prompts) {
    // 1. Initialize the device and the kernels
    auto registry = agpu::nn::KernelRegistry::init_default(0);
    std::printf("HIP device initialized\n");
    // the reference's kernel names on this path (nn/registry.rs:45-112): the registry answers get(name) for each
    const char *kernels[] = {"int4_gemm_w4a16", "layer_norm_v3",      "gelu_forward_v2",  "elementwise_add_v3", "bias_add",         "split_qkv",
                             "concat_heads",    "flash_attention_v2", "flash_attention_kv", "kv_cache_append",  "embedding_lookup", "gemm_f32"};
    int served = 0;
    for (const char *k : kernels) {
        try {
            (void)registry->get(k);
            ++served;
        } catch (const std::exception &) {
        }
    }
    std::printf("Kernel registry loaded (%d ML kernels)\n", served);

    // 3. Load model weights from safetensors
    auto t0 = std::chrono::steady_clock::now();
    const SafeTensors st(model_path);
    Gpt2Config config{};
    const Gpt2Weights weights = load_gpt2_weights(st, config);
    std::printf("Loaded %.1fM params (%.1f MB) in %.1fms\n", st.total_params() / 1e6, st.data_bytes() / 1e6, ms_since(t0));

    // 4. Build model from weights
    auto t1 = std::chrono::steady_clock::now();
    const agpu::nn::Int4Gpt2Model model = agpu::nn::Int4Gpt2Model::from_weights(weights, config, group_size, registry,
                                                                                 int4_head ? AGPU_LM_HEAD_INT4 : AGPU_LM_HEAD_F32);
    std::printf("Model built on GPU in %.1fms\n", ms_since(t1));

    // 5. Tokenize prompts
    const Tokenizer tokenizer(vocab_path);

    // 6. Diagnostic: single forward pass on first prompt
    {
        const std::vector<uint32_t> tokens = tokenizer.encode(prompts[0]);
        std::fprintf(stderr, "\n[diag] Running diagnostic forward on '%s' (%zu tokens)\n", prompts[0].c_str(), tokens.size());
        const agpu::nn::GpuBufferU32 ids(tokens, registry);
        (void)model.forward_diagnostic(ids, tokens.size());
    }

    // 7. Generate text for each prompt
    bool all_match = true;
    for (const std::string &prompt : prompts) {
        const std::vector<uint32_t> tokens = tokenizer.encode(prompt);
        std::printf("\n--- Prompt: \"%s\" (%zu tokens) ---\n", prompt.c_str(), tokens.size());

        // Greedy generation (no KV cache)
        auto t2 = std::chrono::steady_clock::now();
        const std::vector<uint32_t> output_tokens = model.generate(tokens, max_new_tokens);
        const double gen_ms = ms_since(t2);
        const size_t new_tokens = output_tokens.size() - tokens.size();
        std::printf("Output: %s\n", tokenizer.decode(output_tokens).c_str());
        std::printf("Generated %zu tokens in %.1fms (%.1fms/token)\n", new_tokens, gen_ms, new_tokens ? gen_ms / (double)new_tokens : 0.0);

        // KV-cached generation for comparison
        auto t3 = std::chrono::steady_clock::now();
        const std::vector<uint32_t> cached_tokens = model.generate_cached(tokens, max_new_tokens);
        const double cached_ms = ms_since(t3);
        const size_t cached_new = cached_tokens.size() - tokens.size();
        std::printf("Cached: %s\n", tokenizer.decode(cached_tokens).c_str());
        std::printf("Cached: %zu tokens in %.1fms (%.1fms/token)\n", cached_new, cached_ms, cached_new ? cached_ms / (double)cached_new : 0.0);

        // Verify outputs match
        if (output_tokens == cached_tokens) {
            std::printf("MATCH: cached and non-cached outputs agree\n");
        } else {
            all_match = false;
            std::printf("MISMATCH: cached=%zu tokens, non-cached=%zu tokens\n", cached_tokens.size(), output_tokens.size());
        }
        if (print_tokens) {
            std::printf("Tokens:");
            for (uint32_t t : cached_tokens) std::printf(" %u", t);
            std::printf("\n");
        }
    }
    std::printf("\nDone.\n");
    return all_match ? 0 : 2;
}

}  // namespace

int main(int argc, char **argv) {
    std::string model, vocab;
    size_t max_new_tokens = 50, group_size = 32;
    bool int4_head = false, dry = false, print_tokens = false;
    Prompts prompts;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        if (a == "--max-new-tokens" && i + 1 < argc) max_new_tokens = (size_t)std::stoul(argv[++i]);
        else if (a == "--group-size" && i + 1 < argc) group_size = (size_t)std::stoul(argv[++i]);
        else if (a == "--int4-head") int4_head = true;
        else if (a == "--dry-run") dry = true;
        else if (a == "--prompt" && i + 1 < argc) prompts.push_back(argv[++i]);
        else if (a == "--print-tokens") print_tokens = true;
        else if (model.empty()) model = a;
        else if (vocab.empty()) vocab = a;
    }
    if (model.empty() || vocab.empty()) {
        std::fprintf(stderr, "usage: gpt2_inference MODEL.safetensors VOCAB.tiktoken [--max-new-tokens N] [--group-size G] [--int4-head] [--print-tokens] [--dry-run] [--prompt TEXT]...\n");
        return 1;
    }
    try {
        if (prompts.empty()) prompts = kPrompts;
        return dry ? dry_run(model, vocab, prompts) : run(model, vocab, max_new_tokens, group_size, int4_head, print_tokens, prompts);
    } catch (const std::exception &e) {  // the reference prints the error and exits with status 1
        std::fprintf(stderr, "Error: %s\n", e.what());
        return 1;
    }
}
