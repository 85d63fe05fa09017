// Hugging Face snapshot reader: `config.json` -> ModelConfig, `*.safetensors` -> named tensors
// (memory-mapped, zero copies on the host).  Pure host C++.
//
// Takes the place of the reference's loaders for this path: the portable driver's safetensors
// archive + HF config reader (driver/portable/src/safetensors.cpp, driver/portable/src/
// hf_config.cpp; tensor names bound in driver/portable/src/model.cpp:1476-1479 via
// build_dense_) and the storage-program loader of the CUDA driver (driver/weight_loader).
// File format: 8-byte little-endian header length, a JSON header
// {name: {dtype, shape, data_offsets: [begin, end]}, "__metadata__": {...}}, then the data.
#pragma once

#include <dirent.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "config.hpp"

namespace pie_hip_driver {

// ---- a small JSON reader (objects, arrays, strings, numbers, true / false / null) ------------
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool b = false;
    double num = 0.0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;

    const Json* get(const std::string& key) const {
        if (kind != Object) return nullptr;
        for (const auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    double number_or(const std::string& key, double dflt) const {
        const Json* j = get(key);
        return j && j->kind == Number ? j->num : dflt;
    }
    std::string string_or(const std::string& key, const std::string& dflt) const {
        const Json* j = get(key);
        return j && j->kind == String ? j->str : dflt;
    }
    bool bool_or(const std::string& key, bool dflt) const {
        const Json* j = get(key);
        return j && j->kind == Bool ? j->b : dflt;
    }
};

class JsonParser {
  public:
    JsonParser(const char* p, size_t n) : p_(p), end_(p + n) {}
    Json parse() {
        Json v = value();
        ws();
        if (p_ != end_) fail("trailing characters");
        return v;
    }

  private:
    [[noreturn]] void fail(const char* what) const { throw std::runtime_error(std::string("json: ") + what); }
    void ws() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
    }
    bool eat(char c) {
        ws();
        if (p_ < end_ && *p_ == c) {
            ++p_;
            return true;
        }
        return false;
    }
    Json value() {
        ws();
        if (p_ >= end_) fail("unexpected end");
        Json v;
        const char c = *p_;
        if (c == '{') {
            ++p_;
            v.kind = Json::Object;
            if (eat('}')) return v;
            do {
                ws();
                std::string key = string();
                if (!eat(':')) fail("expected ':'");
                v.obj.emplace_back(std::move(key), value());
            } while (eat(','));
            if (!eat('}')) fail("expected '}'");
        } else if (c == '[') {
            ++p_;
            v.kind = Json::Array;
            if (eat(']')) return v;
            do v.arr.push_back(value());
            while (eat(','));
            if (!eat(']')) fail("expected ']'");
        } else if (c == '"') {
            v.kind = Json::String;
            v.str = string();
        } else if (literal("true")) {
            v.kind = Json::Bool;
            v.b = true;
        } else if (literal("false")) {
            v.kind = Json::Bool;
        } else if (literal("null")) {
        } else {
            char* e = nullptr;
            const std::string tmp(p_, std::min<size_t>(end_ - p_, 64));
            v.num = std::strtod(tmp.c_str(), &e);
            if (e == tmp.c_str()) fail("bad value");
            p_ += e - tmp.c_str();
            v.kind = Json::Number;
        }
        return v;
    }
    bool literal(const char* s) {
        const size_t n = std::strlen(s);
        if (static_cast<size_t>(end_ - p_) >= n && std::memcmp(p_, s, n) == 0) {
            p_ += n;
            return true;
        }
        return false;
    }
    std::string string() {
        if (p_ >= end_ || *p_ != '"') fail("expected string");
        ++p_;
        std::string out;
        while (p_ < end_ && *p_ != '"') {
            if (*p_ == '\\') {
                if (++p_ >= end_) fail("bad escape");
                switch (*p_) {
                    case 'n': out.push_back('\n'); break;
                    case 't': out.push_back('\t'); break;
                    case 'r': out.push_back('\r'); break;
                    case 'b': out.push_back('\b'); break;
                    case 'f': out.push_back('\f'); break;
                    case 'u':   // names here are ASCII; keep the low byte of the code unit
                        if (end_ - p_ < 5) fail("bad \\u escape");
                        out.push_back(static_cast<char>(std::strtol(std::string(p_ + 1, 4).c_str(), nullptr, 16)));
                        p_ += 4;
                        break;
                    default: out.push_back(*p_); break;
                }
                ++p_;
            } else {
                out.push_back(*p_++);
            }
        }
        if (p_ >= end_) fail("unterminated string");
        ++p_;
        return out;
    }
    const char* p_;
    const char* end_;
};

inline Json parse_json_file(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("snapshot: cannot open '" + path + "'");
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string text = ss.str();
    return JsonParser(text.data(), text.size()).parse();
}

// ---- safetensors --------------------------------------------------------------------------
// Bytes per element of a safetensors dtype name (0: not a dtype of that format).
inline size_t st_dtype_size(const std::string& dt) {
    if (dt == "F64" || dt == "I64" || dt == "U64") return 8;
    if (dt == "F32" || dt == "I32" || dt == "U32") return 4;
    if (dt == "BF16" || dt == "F16" || dt == "I16" || dt == "U16") return 2;
    if (dt == "I8" || dt == "U8" || dt == "BOOL" || dt == "F8_E4M3" || dt == "F8_E5M2") return 1;
    return 0;
}

struct StTensor {
    std::string dtype;            // "BF16", "F16", "F32", "I32", "U8", "I8", "F8_E4M3", ...
    std::vector<int64_t> shape;
    const uint8_t* data = nullptr;
    size_t bytes = 0;
    int64_t elems() const {
        int64_t n = 1;
        for (int64_t s : shape) n *= s;
        return n;
    }
};

class Snapshot {
  public:
    explicit Snapshot(const std::string& dir) : dir_(dir) {
        std::vector<std::string> files;
        if (DIR* d = opendir(dir.c_str())) {
            while (const dirent* e = readdir(d)) {
                const std::string n = e->d_name;
                if (n.size() > 12 && n.compare(n.size() - 12, 12, ".safetensors") == 0) files.push_back(n);
            }
            closedir(d);
        } else {
            throw std::runtime_error("snapshot: cannot list '" + dir + "'");
        }
        std::sort(files.begin(), files.end());
        if (files.empty()) throw std::runtime_error("snapshot: no .safetensors file in '" + dir + "'");
        for (const std::string& f : files) map_file(dir + "/" + f);
    }
    ~Snapshot() {
        for (const auto& m : maps_) munmap(m.first, m.second);
    }
    Snapshot(const Snapshot&) = delete;
    Snapshot& operator=(const Snapshot&) = delete;

    const StTensor* find(const std::string& name) const {
        const auto it = tensors_.find(name);
        return it == tensors_.end() ? nullptr : &it->second;
    }
    const StTensor& at(const std::string& name) const {
        const StTensor* t = find(name);
        if (!t) throw std::runtime_error("snapshot: tensor '" + name + "' not found in " + dir_);
        return *t;
    }
    const std::map<std::string, StTensor>& tensors() const { return tensors_; }

  private:
    void map_file(const std::string& path) {
        const int fd = open(path.c_str(), O_RDONLY);
        if (fd < 0) throw std::runtime_error("snapshot: cannot open '" + path + "'");
        struct stat st {};
        if (fstat(fd, &st) != 0 || st.st_size < 8) {
            close(fd);
            throw std::runtime_error("snapshot: '" + path + "' is too short");
        }
        void* base = mmap(nullptr, static_cast<size_t>(st.st_size), PROT_READ, MAP_PRIVATE, fd, 0);
        close(fd);
        if (base == MAP_FAILED) throw std::runtime_error("snapshot: mmap failed for '" + path + "'");
        maps_.emplace_back(base, static_cast<size_t>(st.st_size));
        const auto* bytes = static_cast<const uint8_t*>(base);
        uint64_t hlen = 0;
        std::memcpy(&hlen, bytes, 8);
        if (hlen > static_cast<uint64_t>(st.st_size) - 8 || hlen > (128ull << 20))
            throw std::runtime_error("snapshot: bad header length in '" + path + "'");
        const Json header = JsonParser(reinterpret_cast<const char*>(bytes + 8), hlen).parse();
        if (header.kind != Json::Object) throw std::runtime_error("snapshot: header of '" + path + "' is not an object");
        const uint8_t* data0 = bytes + 8 + hlen;
        const uint64_t data_bytes = static_cast<uint64_t>(st.st_size) - 8 - hlen;
        for (const auto& kv : header.obj) {
            if (kv.first == "__metadata__") continue;
            const Json* dt = kv.second.get("dtype");
            const Json* sh = kv.second.get("shape");
            const Json* off = kv.second.get("data_offsets");
            if (!dt || !sh || !off || off->arr.size() != 2)
                throw std::runtime_error("snapshot: malformed entry '" + kv.first + "'");
            // Nothing in the header is trusted: kinds, dtype names, dimensions (whole, >= 0, no
            // overflow of the element count), offsets inside the file, and a byte count that is
            // exactly elements * element size — later copies size themselves from these.
            if (dt->kind != Json::String || sh->kind != Json::Array || off->kind != Json::Array ||
                off->arr[0].kind != Json::Number || off->arr[1].kind != Json::Number)
                throw std::runtime_error("snapshot: malformed entry '" + kv.first + "'");
            StTensor t;
            t.dtype = dt->str;
            const size_t esize = st_dtype_size(t.dtype);
            if (esize == 0) throw std::runtime_error("snapshot: unknown dtype '" + t.dtype + "' in '" + kv.first + "'");
            uint64_t elems = 1;
            for (const Json& s : sh->arr) {
                if (s.kind != Json::Number || !(s.num >= 0.0) || s.num > 9.0e15 ||
                    s.num != static_cast<double>(static_cast<int64_t>(s.num)))
                    throw std::runtime_error("snapshot: bad dimension in '" + kv.first + "'");
                const uint64_t dim = static_cast<uint64_t>(s.num);
                if (dim != 0 && elems > (uint64_t(1) << 62) / dim)
                    throw std::runtime_error("snapshot: element count of '" + kv.first + "' overflows");
                elems *= dim;
                t.shape.push_back(static_cast<int64_t>(dim));
            }
            auto whole = [](double v) { return v >= 0.0 && v <= 9.0e15 && v == static_cast<double>(static_cast<uint64_t>(v)); };
            if (!whole(off->arr[0].num) || !whole(off->arr[1].num))
                throw std::runtime_error("snapshot: offsets of '" + kv.first + "' out of range");
            const uint64_t b = static_cast<uint64_t>(off->arr[0].num), e = static_cast<uint64_t>(off->arr[1].num);
            if (b > e || e > data_bytes) throw std::runtime_error("snapshot: offsets of '" + kv.first + "' out of range");
            if (e - b != elems * esize)
                throw std::runtime_error("snapshot: '" + kv.first + "' holds " + std::to_string(e - b) +
                                         " bytes, its shape and dtype need " + std::to_string(elems * esize));
            t.data = data0 + b;
            t.bytes = e - b;
            tensors_[kv.first] = std::move(t);
        }
    }
    std::string dir_;
    std::vector<std::pair<void*, size_t>> maps_;
    std::map<std::string, StTensor> tensors_;
};

// ---- config.json -> ModelConfig ----------------------------------------------------------------
// Field names as transformers writes them (llama / qwen3 / qwen3_moe); the reference reads the
// same keys in driver/portable/src/hf_config.cpp.  Checkpoints use the half-split RoPE pairing
// (the CUDA driver's default, driver/cuda/src/kernels/rope.cu:10-21) unless the TOML says otherwise.
inline void apply_hf_config(ModelConfig& m, const std::string& dir) {
    const Json c = parse_json_file(dir + "/config.json");
    const std::string type = c.string_or("model_type", "");
    if (type == "llama" || type == "mistral") m.arch = "llama3";
    else if (type == "qwen3") m.arch = "qwen3";
    else if (type == "qwen3_moe") m.arch = "qwen3_moe";
    else throw std::runtime_error("snapshot: unsupported model_type '" + type + "'");
    m.hidden = static_cast<int>(c.number_or("hidden_size", 0));
    // (Mistral-type checkpoints: "sliding_window": N or null; Qwen3 writes one next to
    // "use_sliding_window": false, which switches it off)
    if (m.sliding_window <= 0 && c.bool_or("use_sliding_window", true))
        m.sliding_window = static_cast<int>(c.number_or("sliding_window", 0));
    m.layers = static_cast<int>(c.number_or("num_hidden_layers", 0));
    m.q_heads = static_cast<int>(c.number_or("num_attention_heads", 0));
    m.kv_heads = static_cast<int>(c.number_or("num_key_value_heads", m.q_heads));
    m.head_dim = static_cast<int>(c.number_or("head_dim", m.q_heads ? m.hidden / m.q_heads : 0));
    m.intermediate = static_cast<int>(c.number_or("intermediate_size", 0));
    m.vocab = static_cast<int>(c.number_or("vocab_size", 0));
    m.rms_eps = static_cast<float>(c.number_or("rms_norm_eps", 1e-5));
    m.rope_theta = static_cast<float>(c.number_or("rope_theta", 10000.0));
    m.tie_embeddings = c.bool_or("tie_word_embeddings", false);
    m.rope_factor = 0.f;
    if (const Json* rs = c.get("rope_scaling"); rs && rs->kind == Json::Object) {
        const std::string rt = rs->string_or("rope_type", rs->string_or("type", ""));
        if (rt == "llama3") {
            m.rope_factor = static_cast<float>(rs->number_or("factor", 8.0));
            m.rope_low_freq_factor = static_cast<float>(rs->number_or("low_freq_factor", 1.0));
            m.rope_high_freq_factor = static_cast<float>(rs->number_or("high_freq_factor", 4.0));
            m.rope_original_max_pos = static_cast<int>(rs->number_or("original_max_position_embeddings", 8192));
        } else if (rt == "yarn") {
            m.rope_scaling = "yarn";
            m.rope_factor = static_cast<float>(rs->number_or("factor", 1.0));
            m.rope_beta_fast = static_cast<float>(rs->number_or("beta_fast", 32.0));
            m.rope_beta_slow = static_cast<float>(rs->number_or("beta_slow", 1.0));
            m.rope_attention_factor = static_cast<float>(rs->number_or("attention_factor", 0.0));
            m.rope_original_max_pos = static_cast<int>(rs->number_or(
                "original_max_position_embeddings", c.number_or("max_position_embeddings", 8192)));
        } else if (!rt.empty() && rt != "default") {
            throw std::runtime_error("snapshot: unsupported rope_scaling type '" + rt + "'");
        }
    }
    if (m.arch == "qwen3_moe") {
        m.num_experts = static_cast<int>(c.number_or("num_experts", 0));
        m.top_k = static_cast<int>(c.number_or("num_experts_per_tok", 0));
        m.expert_intermediate = static_cast<int>(c.number_or("moe_intermediate_size", 0));
        m.norm_topk = c.bool_or("norm_topk_prob", true);
    }
    if (m.rope_interleaved < 0) m.rope_interleaved = 0;
}

}  // namespace pie_hip_driver
