// Driver configuration: the per-launch TOML the Pie server writes for a driver
// (`[model] [batching] [runtime]`, driver/portable/src/config.hpp:52-116,
// server/src/embedded_driver.rs:319-358), parsed by a small TOML subset reader
// (sections, `key = value` with string / integer / float / boolean values, comments).
// Unknown `[batching]` keys are rejected like the reference does.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <fstream>
#include <map>
#include <sstream>
#include <stdexcept>
#include <cctype>
#include <string>

namespace pie_hip_driver {

struct ModelConfig {
    // architecture: "llama3" (dense, adjacent-pair RoPE) | "qwen3" (dense, qk-norm, half-split
    // RoPE) | "qwen3_moe"
    std::string arch = "llama3";
    int hidden = 0, layers = 0, q_heads = 0, kv_heads = 0, head_dim = 0, intermediate = 0;
    int vocab = 0;
    float rope_theta = 500000.f, rms_eps = 1e-5f;
    // llama3 wavelength-band RoPE scaling; factor <= 0 disables it
    float rope_factor = 0.f, rope_low_freq_factor = 1.f, rope_high_freq_factor = 4.f;
    int rope_original_max_pos = 8192;
    // rope_scaling = "llama3" (wavelength bands, the default when rope_factor > 0) or "yarn"
    // (ramp over the rotation dims between beta_fast and beta_slow, cos / sin times the
    // attention factor; 0 = 0.1 ln(factor) + 1)
    std::string rope_scaling;
    float rope_beta_fast = 32.f, rope_beta_slow = 1.f, rope_attention_factor = 0.f;
    int rope_interleaved = -1;  // -1: half split, the pairing of Llama / Mistral / Qwen checkpoints
    bool tie_embeddings = false;
    // storage format of the decoder linears: "int4b8" | "int8" | "fp8" | "bf16"
    std::string quant = "int4b8";
    int group_size = 128;
    std::string scale_dtype = "bf16";  // row scales of int8/fp8: "bf16" | "f32"
    // MoE (qwen3_moe)
    int num_experts = 0, top_k = 0, expert_intermediate = 0;
    bool norm_topk = true;
    int sliding_window = 0;   // > 0: a query at position p sees keys p - W + 1 .. p only
    // synthetic random-init weights: N(0, init_std) in bf16, then quantised
    std::uint64_t seed = 0x9E3779B97F4A7C15ull;
    float init_std = 0.02f;
    float router_std = 0.f;  // MoE router rows; 0 = init_std
    float embed_std = 0.f;   // embedding rows; 0 = init_std (a large value lets a token's own embedding
                             // dominate the residual stream, so distinct tokens take distinct MoE routes)
    // `[model] hf_path` (portable driver's key) or `snapshot_dir` (CUDA driver's key): a Hugging
    // Face snapshot directory; its config.json then fixes the shape fields above and the weights
    // come from its safetensors files instead of the synthetic initialiser
    std::string checkpoint_dir;
};

struct BatchingConfig {
    int kv_page_size = 32;       // driver/portable/src/config.hpp:30
    int total_pages = 1024;      // server/src/config.rs:727-743
    int max_forward_tokens = 10240;
    int max_forward_requests = 512;
    int cpu_pages = 0;
    // KV-cache storage (driver/cuda/src/config.hpp:66, kv_cache_format.cpp:46-110): auto | bf16 |
    // bfloat16 | fp8_e4m3 | int8_per_token_head | fp8_per_token_head
    std::string kv_cache_dtype = "auto";
};

struct RuntimeConfig {
    bool verbose = false;
    bool use_graphs = true;
    // a second copy of every decoder linear in the skinny GEMM's tile-major layout (doubles the
    // weight memory, ~25 % off the 5-32-row and MoE grouped GEMMs)
    bool tiled_weights = true;
    // one synthetic full-size prefill chunk and a decode step at start-up, so that the first
    // request does not pay one-time costs (measured: 58 ms cold against 47 ms for a 2048-token
    // prefill of an 8B model); writes only KV pages nobody owns yet
    bool warmup = true;
    // time the candidate kernels of every decoder linear at start-up (2-4 and 17-128 rows, a few
    // tens of milliseconds) and dispatch on the measurements instead of the fitted cost model
    bool tune_linears = true;
    // one or two decode rows: the attention output projection merges the attention's splits in
    // its prologue where that is measured to pay (no separate merge launch; the attention output
    // rows are then never stored)
    bool attn_merge_proj = true;
    std::string snapshot_dir;
};

struct DriverConfig {
    ModelConfig model;
    BatchingConfig batching;
    RuntimeConfig runtime;
};

namespace detail {
inline std::string trim(const std::string& s) {
    const auto b = s.find_first_not_of(" \t\r\n");
    if (b == std::string::npos) return "";
    const auto e = s.find_last_not_of(" \t\r\n");
    return s.substr(b, e - b + 1);
}
inline std::string unquote(const std::string& v) {
    if (v.size() >= 2 && (v.front() == '"' || v.front() == '\'') && v.back() == v.front())
        return v.substr(1, v.size() - 2);
    return v;
}
inline bool to_bool(const std::string& v, const std::string& key) {
    if (v == "true") return true;
    if (v == "false") return false;
    throw std::runtime_error("config: " + key + " must be true or false");
}
inline long long to_int(const std::string& v, const std::string& key) {
    std::string t;
    for (char c : v)
        if (c != '_') t.push_back(c);
    char* end = nullptr;
    const long long r = std::strtoll(t.c_str(), &end, 0);
    if (end == t.c_str() || *end != '\0') throw std::runtime_error("config: " + key + " must be an integer");
    return r;
}
inline double to_float(const std::string& v, const std::string& key) {
    char* end = nullptr;
    const double r = std::strtod(v.c_str(), &end);
    if (end == v.c_str() || *end != '\0') throw std::runtime_error("config: " + key + " must be a number");
    return r;
}
}  // namespace detail

// Parses TOML text into section -> key -> raw value.
inline std::map<std::string, std::map<std::string, std::string>> parse_toml_lite(
    const std::string& text) {
    std::map<std::string, std::map<std::string, std::string>> out;
    std::istringstream in(text);
    std::string line, section;
    int lineno = 0;
    while (std::getline(in, line)) {
        ++lineno;
        // strip comments outside quotes
        bool inq = false;
        char qc = 0;
        for (size_t i = 0; i < line.size(); ++i) {
            const char c = line[i];
            if (inq) {
                if (c == qc) inq = false;
            } else if (c == '"' || c == '\'') {
                inq = true;
                qc = c;
            } else if (c == '#') {
                line.erase(i);
                break;
            }
        }
        line = detail::trim(line);
        if (line.empty()) continue;
        if (line.front() == '[') {
            if (line.back() != ']') throw std::runtime_error("config: bad section at line " + std::to_string(lineno));
            section = detail::trim(line.substr(1, line.size() - 2));
            out[section];
            continue;
        }
        const auto eq = line.find('=');
        if (eq == std::string::npos) throw std::runtime_error("config: expected key = value at line " + std::to_string(lineno));
        out[section][detail::trim(line.substr(0, eq))] = detail::trim(line.substr(eq + 1));
    }
    return out;
}

// The kernel library's PIE_HIP_KV_* code of a kv_cache_dtype value; the reference's other values
// (fp8_e5m2, fp4_e2m1, nvfp4) are recognised and refused, anything else is invalid
// (driver/cuda/src/kv_cache_format.cpp:105-108).
inline int kv_format_code(const std::string& value) {
    std::string v;
    for (char ch : value) v.push_back(static_cast<char>(std::tolower(static_cast<unsigned char>(ch))));
    if (v.empty() || v == "auto" || v == "bf16" || v == "bfloat16") return 0;
    if (v == "fp8_e4m3") return 1;
    if (v == "int8_per_token_head") return 2;
    if (v == "fp8_per_token_head") return 3;
    if (v == "fp8_e5m2") return 4;
    if (v == "fp4_e2m1" || v == "nvfp4") return 5;   // one scheme under two names (kv_cache_format.cpp:99-107)
    throw std::runtime_error("invalid kv_cache_dtype '" + value +
                             "'; expected one of: auto, bf16, bfloat16, fp8_e4m3, fp8_e5m2, "
                             "int8_per_token_head, fp8_per_token_head, fp4_e2m1, nvfp4");
}

// Shape and range checks, defaults that depend on other fields.
inline void finalize_config(DriverConfig& c) {
    auto& m = c.model;
    if (m.hidden <= 0 || m.layers <= 0 || m.q_heads <= 0 || m.kv_heads <= 0 || m.vocab <= 0)
        throw std::runtime_error("config: [model] needs hidden, layers, q_heads, kv_heads, vocab");
    if (m.head_dim <= 0) m.head_dim = m.hidden / m.q_heads;
    if (m.q_heads % m.kv_heads != 0) throw std::runtime_error("config: q_heads must be a multiple of kv_heads");
    const bool moe = m.arch == "qwen3_moe";
    if (m.arch != "llama3" && m.arch != "qwen3" && !moe)
        throw std::runtime_error("config: unsupported arch '" + m.arch + "'");
    if (moe) {
        if (m.num_experts <= 0 || m.top_k <= 0 || m.expert_intermediate <= 0 || m.top_k > m.num_experts)
            throw std::runtime_error("config: qwen3_moe needs num_experts, top_k, expert_intermediate");
    } else if (m.intermediate <= 0) {
        throw std::runtime_error("config: [model] needs intermediate");
    }
    if (m.quant != "int4b8" && m.quant != "int8" && m.quant != "fp8" && m.quant != "bf16")
        throw std::runtime_error("config: unsupported quant '" + m.quant + "'");
    if (m.scale_dtype != "bf16" && m.scale_dtype != "f32")
        throw std::runtime_error("config: scale_dtype must be bf16 or f32");
    // (i, i + d/2) pairs for every architecture here, as the reference rotates them
    // (driver/cuda/src/kernels/rope.cu:10-21 keeps adjacent pairs for GLM only)
    if (m.rope_interleaved < 0) m.rope_interleaved = 0;
    if (m.rope_scaling.empty()) m.rope_scaling = "llama3";
    if (m.rope_scaling != "llama3" && m.rope_scaling != "yarn")
        throw std::runtime_error("config: rope_scaling must be llama3 or yarn");
    const auto& b = c.batching;
    if (b.kv_page_size <= 0 || b.kv_page_size % 16 != 0)
        throw std::runtime_error("config: kv_page_size must be a positive multiple of 16");
    if (b.total_pages <= 0 || b.max_forward_tokens <= 0 || b.max_forward_requests <= 0)
        throw std::runtime_error("config: [batching] sizes must be positive");
    (void)kv_format_code(b.kv_cache_dtype);
}

inline DriverConfig parse_config_text(const std::string& text) {
    using namespace detail;
    DriverConfig c;
    const auto t = parse_toml_lite(text);
    for (const auto& [sec, kv] : t) {
        for (const auto& [k, raw] : kv) {
            const std::string v = unquote(raw);
            const std::string key = sec + "." + k;
            if (sec == "model") {
                auto& m = c.model;
                if (k == "arch") m.arch = v;
                else if (k == "hidden" || k == "hidden_size") m.hidden = (int)to_int(v, key);
                else if (k == "layers" || k == "num_hidden_layers") m.layers = (int)to_int(v, key);
                else if (k == "q_heads" || k == "num_attention_heads") m.q_heads = (int)to_int(v, key);
                else if (k == "kv_heads" || k == "num_key_value_heads") m.kv_heads = (int)to_int(v, key);
                else if (k == "head_dim") m.head_dim = (int)to_int(v, key);
                else if (k == "intermediate" || k == "intermediate_size") m.intermediate = (int)to_int(v, key);
                else if (k == "vocab" || k == "vocab_size") m.vocab = (int)to_int(v, key);
                else if (k == "rope_theta") m.rope_theta = (float)to_float(v, key);
                else if (k == "rms_eps" || k == "rms_norm_eps") m.rms_eps = (float)to_float(v, key);
                else if (k == "rope_factor") m.rope_factor = (float)to_float(v, key);
                else if (k == "rope_low_freq_factor") m.rope_low_freq_factor = (float)to_float(v, key);
                else if (k == "rope_high_freq_factor") m.rope_high_freq_factor = (float)to_float(v, key);
                else if (k == "rope_original_max_pos") m.rope_original_max_pos = (int)to_int(v, key);
                else if (k == "rope_scaling") m.rope_scaling = v;
                else if (k == "rope_beta_fast") m.rope_beta_fast = (float)to_float(v, key);
                else if (k == "rope_beta_slow") m.rope_beta_slow = (float)to_float(v, key);
                else if (k == "rope_attention_factor") m.rope_attention_factor = (float)to_float(v, key);
                else if (k == "rope_interleaved") m.rope_interleaved = to_bool(v, key) ? 1 : 0;
                else if (k == "tie_embeddings") m.tie_embeddings = to_bool(v, key);
                else if (k == "quant") m.quant = v;
                else if (k == "group_size") m.group_size = (int)to_int(v, key);
                else if (k == "scale_dtype") m.scale_dtype = v;
                else if (k == "num_experts") m.num_experts = (int)to_int(v, key);
                else if (k == "top_k") m.top_k = (int)to_int(v, key);
                else if (k == "expert_intermediate") m.expert_intermediate = (int)to_int(v, key);
                else if (k == "norm_topk") m.norm_topk = to_bool(v, key);
                else if (k == "sliding_window") m.sliding_window = (int)to_int(v, key);
                else if (k == "seed") m.seed = (std::uint64_t)to_int(v, key);
                else if (k == "init_std") m.init_std = (float)to_float(v, key);
                else if (k == "router_std") m.router_std = (float)to_float(v, key);
                else if (k == "embed_std") m.embed_std = (float)to_float(v, key);
                else if (k == "hf_path" || k == "snapshot_dir") m.checkpoint_dir = v;
                // other [model] keys (paths, dtype hints) belong to loaders this driver lacks
            } else if (sec == "batching") {
                auto& b = c.batching;
                if (k == "kv_page_size") b.kv_page_size = (int)to_int(v, key);
                else if (k == "total_pages") b.total_pages = (int)to_int(v, key);
                else if (k == "max_forward_tokens") b.max_forward_tokens = (int)to_int(v, key);
                else if (k == "max_forward_requests") b.max_forward_requests = (int)to_int(v, key);
                else if (k == "cpu_pages") b.cpu_pages = (int)to_int(v, key);
                else if (k == "kv_cache_dtype") b.kv_cache_dtype = v;
                else throw std::runtime_error("config: unknown [batching] key '" + k + "'");
            } else if (sec == "runtime") {
                auto& r = c.runtime;
                if (k == "verbose") r.verbose = to_bool(v, key);
                else if (k == "use_graphs") r.use_graphs = to_bool(v, key);
                else if (k == "tiled_weights") r.tiled_weights = to_bool(v, key);
                else if (k == "warmup") r.warmup = to_bool(v, key);
                else if (k == "tune_linears") r.tune_linears = to_bool(v, key);
                else if (k == "attn_merge_proj") r.attn_merge_proj = to_bool(v, key);
                else if (k == "snapshot_dir") r.snapshot_dir = v;
            }
        }
    }
    if (c.model.checkpoint_dir.empty()) finalize_config(c);   // else after config.json is applied
    return c;
}

// `src` is a file path, or inline TOML when it contains a newline.
inline DriverConfig load_config(const std::string& src) {
    if (src.find('\n') != std::string::npos) return parse_config_text(src);
    std::ifstream f(src);
    if (!f) throw std::runtime_error("config: cannot open '" + src + "'");
    std::stringstream ss;
    ss << f.rdbuf();
    return parse_config_text(ss.str());
}

}  // namespace pie_hip_driver
