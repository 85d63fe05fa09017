#include "model.hpp"

#include <cmath>
#include <stdexcept>

#include "pie_hip_kernels.h"
#include "snapshot.hpp"

namespace pie_hip_driver {

#define PIE_HIP_CHECK(expr)                                                              \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess)                                                            \
            throw std::runtime_error(std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

namespace {

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// out[i] = bf16(mean + std * z_i): z_i is the centred sum of four 16-bit uniforms drawn from
// a counter hash of (seed, i) — integer arithmetic plus one exact int->float conversion and
// two IEEE operations, so the stream is a pure function of (seed, i).
__global__ void fill_normal_bf16_kernel(uint16_t* __restrict__ out, size_t n, uint64_t seed,
                                        float mean, float std) {
    const size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (i >= n) return;
    const uint64_t h = splitmix64(seed ^ (i * 0xD1342543DE82EF95ull));
    const int sum = static_cast<int>(h & 0xFFFF) + static_cast<int>((h >> 16) & 0xFFFF) +
                    static_cast<int>((h >> 32) & 0xFFFF) + static_cast<int>(h >> 48);
    const float z = static_cast<float>(sum - 131070) * (1.0f / 37837.227f);
    const float v = mean + std * z;
    const __bf16 b = static_cast<__bf16>(v);
    out[i] = __builtin_bit_cast(uint16_t, b);
}

void fill_normal(uint16_t* dst, size_t n, uint64_t seed, float mean, float std,
                 hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(fill_normal_bf16_kernel, dim3(static_cast<unsigned>((n + 255) / 256)),
                       dim3(256), 0, stream, dst, n, seed, mean, std);
    PIE_HIP_CHECK(hipGetLastError());
}

// Inside every block of 2*half rows: dst row 2i = src row i (gate_i), dst row 2i+1 = src row
// half + i (up_i); rows of row_bytes bytes (always even), moved two bytes at a time — a
// load-time kernel.  One block for a dense FFN, one block per expert for stacked MoE experts.
__global__ void interleave_rows_kernel(const unsigned char* __restrict__ src,
                                       unsigned char* __restrict__ dst, size_t half,
                                       size_t row_bytes, size_t rows_total) {
    const size_t total = rows_total * row_bytes;
    for (size_t b = (blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x) * 2; b < total;
         b += static_cast<size_t>(gridDim.x) * blockDim.x * 2) {
        const size_t grow = b / row_bytes, off = b - grow * row_bytes;
        const size_t blk = grow / (2 * half), drow = grow - blk * 2 * half;
        const size_t srow = blk * 2 * half + ((drow & 1) ? half + (drow >> 1) : (drow >> 1));
        *reinterpret_cast<uint16_t*>(dst + b) =
            *reinterpret_cast<const uint16_t*>(src + srow * row_bytes + off);
    }
}

Quant parse_quant(const std::string& q) {
    if (q == "int4b8") return Quant::Int4b8;
    if (q == "int8") return Quant::Int8;
    if (q == "fp8") return Quant::Fp8;
    return Quant::Bf16;
}

__global__ void f32_to_bf16_kernel(const float* __restrict__ in, uint16_t* __restrict__ out,
                                   int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const __bf16 b = static_cast<__bf16>(in[i]);
    out[i] = __builtin_bit_cast(uint16_t, b);
}

}  // namespace

std::vector<float> rope_inv_freq(const ModelConfig& cfg) {
    const int d = cfg.head_dim, half = d / 2;
    std::vector<float> out(half);
    const double pi = 3.14159265358979323846;
    for (int i = 0; i < half; ++i) {
        const double base = std::pow(static_cast<double>(cfg.rope_theta), -2.0 * i / d);
        double f = base;
        if (cfg.rope_factor > 0.f && cfg.rope_original_max_pos > 0 && cfg.rope_scaling == "yarn") {
            // YaRN: full rotations below low_dim, frequencies divided by the factor above
            // high_dim, a linear ramp between (launch_rope_yarn_original_bf16,
            // driver/cuda/src/kernels/rope.cu:495-507,552-589)
            const double ln_theta = std::log(static_cast<double>(cfg.rope_theta));
            auto corr = [&](double rot) {
                return d * std::log(cfg.rope_original_max_pos / (rot * 2.0 * pi)) / (2.0 * ln_theta);
            };
            double lo = std::floor(corr(cfg.rope_beta_fast)), hi = std::ceil(corr(cfg.rope_beta_slow));
            lo = std::max(lo, 0.0);
            hi = std::min(hi, static_cast<double>(half) - 1.0);
            hi = std::max(hi, lo);
            const double denom = hi == lo ? hi + 1e-3 - lo : hi - lo;
            const double ramp = std::min(1.0, std::max(0.0, (i - lo) / denom));
            f = base * ((1.0 - ramp) + ramp / cfg.rope_factor);
        } else if (cfg.rope_factor > 0.f && cfg.rope_original_max_pos > 0) {
            const double low_wl = cfg.rope_original_max_pos / static_cast<double>(cfg.rope_low_freq_factor);
            const double high_wl = cfg.rope_original_max_pos / static_cast<double>(cfg.rope_high_freq_factor);
            const double wl = 2.0 * pi / base;
            if (wl < high_wl) {
                f = base;
            } else if (wl > low_wl) {
                f = base / cfg.rope_factor;
            } else {
                const double smooth = (cfg.rope_original_max_pos / wl - cfg.rope_low_freq_factor) /
                                      (cfg.rope_high_freq_factor - cfg.rope_low_freq_factor);
                f = (1.0 - smooth) * base / cfg.rope_factor + smooth * base;
            }
        }
        out[i] = static_cast<float>(f);
    }
    return out;
}

float rope_mscale(const ModelConfig& cfg) {
    if (cfg.rope_scaling != "yarn" || !(cfg.rope_factor > 0.f)) return 1.f;
    if (cfg.rope_attention_factor > 0.f) return cfg.rope_attention_factor;
    return cfg.rope_factor <= 1.f ? 1.f : 0.1f * std::log(cfg.rope_factor) + 1.f;
}

Model::~Model() {
    for (void* p : allocs_) (void)hipFree(p);
}

void Model::build_tiled_copies(hipStream_t stream) {
    for (LayerWeights& l : layers)
        for (Linear* w : {&l.wqkv, &l.wo, &l.wgu, &l.wdown}) {
            if (!w->data || w->data_tiled || w->N <= 0 || w->N % 16 != 0) continue;
            const size_t row_bytes = w->data_bytes() / static_cast<size_t>(w->N);
            if (row_bytes % 64 != 0) continue;
            w->data_tiled = alloc(w->data_bytes(), "");
            const int st = w->kind == Quant::Int4b8
                               ? pie_hip_repack_mfma_tiles_int4(w->data, w->data_tiled, w->N, row_bytes, stream)
                               : pie_hip_repack_mfma_tiles(w->data, w->data_tiled, w->N, row_bytes, stream);
            if (st != PIE_HIP_OK)
                throw std::runtime_error("model: weight repack failed");
            if (w->kind == Quant::Int4b8) {
                w->scale_tiled = alloc(w->scale_bytes(), "");
                if (pie_hip_repack_scale_tiles(static_cast<const uint16_t*>(w->scale),
                                               static_cast<uint16_t*>(w->scale_tiled), w->N, w->K / w->group,
                                               stream) != PIE_HIP_OK)
                    throw std::runtime_error("model: scale repack failed");
            }
        }
    PIE_HIP_CHECK(hipStreamSynchronize(stream));
}

void* Model::alloc(size_t bytes, const std::string& name) {
    void* p = nullptr;
    PIE_HIP_CHECK(hipMalloc(&p, bytes ? bytes : 16));
    allocs_.push_back(p);
    if (!name.empty()) names_[name] = TensorRef{p, bytes};
    return p;
}

void Model::prepare_linear(Linear& lin, int N, int K, const std::string& name) {
    lin.kind = quant_;
    lin.N = N;
    lin.K = K;
    lin.group = cfg_.group_size;
    lin.scale_bf16 = cfg_.scale_dtype == "bf16";
    if (quant_ == Quant::Int4b8 && (K % lin.group != 0 || lin.group % 32 != 0))
        throw std::runtime_error("model: int4b8 needs K % group == 0 and group % 32 == 0 (" + name + ")");
    lin.data = alloc(lin.data_bytes(), name + ".data");
    if (lin.scale_bytes()) lin.scale = alloc(lin.scale_bytes(), name + ".scale");
    decode_bytes_ += lin.data_bytes() + lin.scale_bytes();
    if (quant_ != Quant::Bf16 && static_cast<size_t>(N) * K > tmp_elems_)
        throw std::runtime_error("model: scratch too small for " + name);
}

// [N, K] bf16 in the scratch buffer -> the linear's storage format.
void Model::quantise_scratch(Linear& lin, const std::string& name, hipStream_t stream) {
    const int N = lin.N, K = lin.K;
    int st = 0;
    if (quant_ == Quant::Bf16) {
        PIE_HIP_CHECK(hipMemcpyAsync(lin.data, tmp_bf16_, lin.data_bytes(), hipMemcpyDeviceToDevice, stream));
        return;
    }
    if (quant_ == Quant::Int4b8) {
        st = pie_hip_quant_int4b8_group(tmp_bf16_, static_cast<uint32_t*>(lin.data),
                                        static_cast<uint16_t*>(lin.scale), N, K, lin.group, stream);
    } else {
        // row-scale formats quantise into an f32 scale first; bf16 scales are its rounding
        float* s32 = lin.scale_bf16 ? static_cast<float*>(alloc(static_cast<size_t>(N) * 4, ""))
                                    : static_cast<float*>(lin.scale);
        if (quant_ == Quant::Int8)
            st = pie_hip_quant_int8_per_channel(tmp_bf16_, static_cast<int8_t*>(lin.data), s32, N, K, stream);
        else
            st = pie_hip_quant_fp8_per_channel(tmp_bf16_, static_cast<uint8_t*>(lin.data), s32, N, K, stream);
        if (st == 0 && lin.scale_bf16) {
            hipLaunchKernelGGL(f32_to_bf16_kernel, dim3((N + 255) / 256), dim3(256), 0, stream, s32,
                               static_cast<uint16_t*>(lin.scale), N);
            PIE_HIP_CHECK(hipGetLastError());
        }
    }
    if (st != 0) throw std::runtime_error("model: quantiser failed for " + name);
}

void Model::make_linear(Linear& lin, int N, int K, const std::string& name, std::uint64_t seed,
                        hipStream_t stream) {
    prepare_linear(lin, N, K, name);
    const size_t nk = static_cast<size_t>(N) * K;
    if (quant_ == Quant::Bf16) {
        fill_normal(static_cast<uint16_t*>(lin.data), nk, seed, 0.f, cfg_.init_std, stream);
        return;
    }
    fill_normal(tmp_bf16_, nk, seed, 0.f, cfg_.init_std, stream);
    quantise_scratch(lin, name, stream);
}

// Re-orders the rows of a fused gate/up projection from (all gate rows, all up rows) to
// (gate_0, up_0, gate_1, up_1, ...), the row order the SwiGLU epilogue of the fused projection
// kernel pairs up.  A pure row permutation of the canonical [N, K] layout: data and scales move
// together, no value changes.
void Model::interleave_gate_up(Linear& lin, int blocks, hipStream_t stream) {
    interleave_row_blocks(lin, static_cast<size_t>(lin.N) / blocks / 2, static_cast<size_t>(lin.N), stream);
}

// Inside every block of 2*half rows among the first `rows` rows: row 2i <- row i, row 2i+1 <-
// row half + i; data and scales together, later rows untouched.
void Model::interleave_row_blocks(Linear& lin, size_t half, size_t rows, hipStream_t stream) {
    auto permute = [&](void* buf, size_t bytes) {
        if (!buf || bytes == 0 || rows == 0) return;
        const size_t row_bytes = bytes / lin.N;
        const size_t part = rows * row_bytes;
        void* tmp = nullptr;
        PIE_HIP_CHECK(hipMalloc(&tmp, part));
        hipLaunchKernelGGL(interleave_rows_kernel, dim3(2048), dim3(256), 0, stream,
                           static_cast<const unsigned char*>(buf), static_cast<unsigned char*>(tmp),
                           half, row_bytes, rows);
        PIE_HIP_CHECK(hipGetLastError());
        PIE_HIP_CHECK(hipMemcpyAsync(buf, tmp, part, hipMemcpyDeviceToDevice, stream));
        PIE_HIP_CHECK(hipStreamSynchronize(stream));
        (void)hipFree(tmp);
    };
    permute(lin.data, lin.data_bytes());
    permute(lin.scale, lin.scale_bytes());
}

// Half-split RoPE (pairs (i, i + d/2), driver/cuda/src/kernels/rope.cu:10-21) without a per-head
// q/k norm: the q and k rows of the fused projection are re-ordered so that a pair's two outputs
// are neighbours, which lets the projection kernels rotate them in their epilogue; the stores
// put them back at i and i + d/2, so q and the KV pool hold what the original row order gives.
void Model::pair_qk_rows(hipStream_t stream) {
    const int d = cfg_.head_dim;
    if (cfg_.rope_interleaved || has_qk_norm() || d < 2 || (d & (d - 1)) != 0) return;
    const size_t rows = static_cast<size_t>(cfg_.q_heads + cfg_.kv_heads) * d;
    for (LayerWeights& l : layers) interleave_row_blocks(l.wqkv, static_cast<size_t>(d) / 2, rows, stream);
    qk_rows_paired_ = true;
}

void Model::init_synthetic(const ModelConfig& cfg, hipStream_t stream) {
    cfg_ = cfg;
    quant_ = parse_quant(cfg.quant);
    const int H = cfg.hidden, d = cfg.head_dim, hq = cfg.q_heads, hk = cfg.kv_heads;
    const int V = cfg.vocab, L = cfg.layers;
    const bool moe = is_moe();
    const int I = moe ? cfg.expert_intermediate : cfg.intermediate;
    if (H % 32 != 0 || d % 8 != 0 || I % 32 != 0 || V % 8 != 0)
        throw std::runtime_error("model: hidden/intermediate must be multiples of 32, head_dim and vocab of 8");

    size_t biggest = static_cast<size_t>((hq + 2 * hk) * d) * H;
    biggest = std::max(biggest, static_cast<size_t>(2 * I) * H * (moe ? cfg.num_experts : 1));
    biggest = std::max(biggest, static_cast<size_t>(H) * hq * d);
    tmp_elems_ = biggest;
    PIE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&tmp_bf16_), biggest * 2));

    std::uint64_t seed = cfg.seed;
    auto next_seed = [&]() { return seed += 0xA0761D6478BD642Full; };

    embed = static_cast<uint16_t*>(alloc(static_cast<size_t>(V) * H * 2, "embed"));
    fill_normal(embed, static_cast<size_t>(V) * H, next_seed(), 0.f, cfg.embed_std > 0.f ? cfg.embed_std : cfg.init_std, stream);
    if (cfg.tie_embeddings) {
        lm_head = embed;
        names_["lm_head"] = names_["embed"];
    } else {
        lm_head = static_cast<uint16_t*>(alloc(static_cast<size_t>(V) * H * 2, "lm_head"));
        fill_normal(lm_head, static_cast<size_t>(V) * H, next_seed(), 0.f, cfg.init_std, stream);
    }
    decode_bytes_ += static_cast<size_t>(V) * H * 2;
    final_norm = static_cast<uint16_t*>(alloc(static_cast<size_t>(H) * 2, "final_norm"));
    fill_normal(final_norm, H, next_seed(), 1.f, 0.1f, stream);

    const std::vector<float> f = rope_inv_freq(cfg);
    inv_freq = static_cast<float*>(alloc(f.size() * 4, "inv_freq"));
    PIE_HIP_CHECK(hipMemcpyAsync(inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice, stream));
    PIE_HIP_CHECK(hipStreamSynchronize(stream));

    layers.resize(L);
    for (int l = 0; l < L; ++l) {
        LayerWeights& w = layers[l];
        const std::string p = "layers." + std::to_string(l) + ".";
        w.attn_norm = static_cast<uint16_t*>(alloc(static_cast<size_t>(H) * 2, p + "attn_norm"));
        fill_normal(w.attn_norm, H, next_seed(), 1.f, 0.1f, stream);
        w.ffn_norm = static_cast<uint16_t*>(alloc(static_cast<size_t>(H) * 2, p + "ffn_norm"));
        fill_normal(w.ffn_norm, H, next_seed(), 1.f, 0.1f, stream);
        if (has_qk_norm()) {
            w.q_norm = static_cast<uint16_t*>(alloc(static_cast<size_t>(d) * 2, p + "q_norm"));
            fill_normal(w.q_norm, d, next_seed(), 1.f, 0.1f, stream);
            w.k_norm = static_cast<uint16_t*>(alloc(static_cast<size_t>(d) * 2, p + "k_norm"));
            fill_normal(w.k_norm, d, next_seed(), 1.f, 0.1f, stream);
        }
        make_linear(w.wqkv, (hq + 2 * hk) * d, H, p + "wqkv", next_seed(), stream);
        make_linear(w.wo, H, hq * d, p + "wo", next_seed(), stream);
        if (!moe) {
            make_linear(w.wgu, 2 * I, H, p + "wgu", next_seed(), stream);
            interleave_gate_up(w.wgu, 1, stream);
            make_linear(w.wdown, H, I, p + "wdown", next_seed(), stream);
        } else {
            // experts stacked along the rows: wgu [E * 2I, H] (gate/up interleaved inside each
            // expert), wdown [E * H, I]; row / group scales make the stacking exact
            const int E = cfg.num_experts;
            w.router.kind = Quant::Bf16;
            w.router.N = E;
            w.router.K = H;
            w.router.data = alloc(static_cast<size_t>(E) * H * 2, p + "router");
            fill_normal(static_cast<uint16_t*>(w.router.data), static_cast<size_t>(E) * H, next_seed(), 0.f,
                        cfg.router_std > 0.f ? cfg.router_std : cfg.init_std, stream);
            const size_t before = decode_bytes_;
            make_linear(w.wgu, E * 2 * I, H, p + "wgu", next_seed(), stream);
            interleave_gate_up(w.wgu, E, stream);
            make_linear(w.wdown, E * H, I, p + "wdown", next_seed(), stream);
            // a batch-1 decode step touches top_k of the E experts
            const size_t all = decode_bytes_ - before;
            decode_bytes_ = before + all / E * cfg.top_k + static_cast<size_t>(E) * H * 2;
        }
    }
    PIE_HIP_CHECK(hipStreamSynchronize(stream));
    (void)hipFree(tmp_bf16_);
    tmp_bf16_ = nullptr;
    pair_qk_rows(stream);
}

namespace {

// Widens / narrows a checkpoint tensor to bf16 bits on the host when it is not bf16 already.
const uint16_t* as_bf16(const StTensor& t, std::vector<uint16_t>& staging) {
    const size_t n = static_cast<size_t>(t.elems());
    if (t.dtype == "BF16") {
        if (t.bytes != n * 2) throw std::runtime_error("snapshot: BF16 tensor with a wrong byte count");
        return reinterpret_cast<const uint16_t*>(t.data);
    }
    staging.resize(n);
    auto rne = [](float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
        return static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    };
    if (t.dtype == "F32") {
        if (t.bytes != n * 4) throw std::runtime_error("snapshot: F32 tensor with a wrong byte count");
        for (size_t i = 0; i < n; ++i) {
            float f;
            std::memcpy(&f, t.data + 4 * i, 4);
            staging[i] = rne(f);
        }
    } else if (t.dtype == "F16") {
        if (t.bytes != n * 2) throw std::runtime_error("snapshot: F16 tensor with a wrong byte count");
        for (size_t i = 0; i < n; ++i) {
            uint16_t h;
            std::memcpy(&h, t.data + 2 * i, 2);
            const uint32_t sign = (h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
            uint32_t u;
            if (exp == 0) {
                if (man == 0) u = sign;
                else {   // subnormal half: normalise
                    int e = -1;
                    uint32_t m2 = man;
                    do { ++e; m2 <<= 1; } while (!(m2 & 0x400u));
                    u = sign | ((127 - 15 - e) << 23) | ((m2 & 0x3FFu) << 13);
                }
            } else if (exp == 31) u = sign | 0x7F800000u | (man << 13);
            else u = sign | ((exp + 112) << 23) | (man << 13);
            float f;
            std::memcpy(&f, &u, 4);
            staging[i] = rne(f);
        }
    } else {
        throw std::runtime_error("snapshot: dtype " + t.dtype + " is not a floating weight");
    }
    return staging.data();
}

void expect_shape(const StTensor& t, const std::string& name, int64_t rows, int64_t cols) {
    const bool ok = cols < 0 ? (t.shape.size() == 1 && t.shape[0] == rows)
                             : (t.shape.size() == 2 && t.shape[0] == rows && t.shape[1] == cols);
    if (!ok) throw std::runtime_error("snapshot: tensor '" + name + "' has an unexpected shape");
}

}  // namespace

void Model::load_snapshot(const ModelConfig& cfg, hipStream_t stream) {
    cfg_ = cfg;
    quant_ = parse_quant(cfg.quant);
    const Snapshot snap(cfg.checkpoint_dir);
    const int H = cfg.hidden, d = cfg.head_dim, hq = cfg.q_heads, hk = cfg.kv_heads;
    const int V = cfg.vocab, L = cfg.layers;
    const bool moe = is_moe();
    const int I = moe ? cfg.expert_intermediate : cfg.intermediate;
    const int E = moe ? cfg.num_experts : 1;
    if (H % 32 != 0 || d % 8 != 0 || I % 32 != 0 || V % 8 != 0)
        throw std::runtime_error("model: hidden/intermediate must be multiples of 32, head_dim and vocab of 8");

    size_t biggest = static_cast<size_t>((hq + 2 * hk) * d) * H;
    biggest = std::max(biggest, static_cast<size_t>(2 * I) * H * E);
    biggest = std::max(biggest, static_cast<size_t>(H) * hq * d);
    tmp_elems_ = biggest;
    PIE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&tmp_bf16_), biggest * 2));
    std::vector<uint16_t> staging;

    // rows of a checkpoint tensor -> device bf16 at `dst` (+ row offset)
    auto upload = [&](const std::string& name, uint16_t* dst, int64_t rows, int64_t cols) {
        const StTensor& t = snap.at(name);
        expect_shape(t, name, rows, cols);
        const uint16_t* src = as_bf16(t, staging);
        PIE_HIP_CHECK(hipMemcpyAsync(dst, src, static_cast<size_t>(t.elems()) * 2, hipMemcpyHostToDevice, stream));
        PIE_HIP_CHECK(hipStreamSynchronize(stream));   // `staging` is reused by the next tensor
    };
    auto vector_param = [&](const std::string& src, const std::string& name, int n) {
        auto* p = static_cast<uint16_t*>(alloc(static_cast<size_t>(n) * 2, name));
        upload(src, p, n, -1);
        return p;
    };

    embed = static_cast<uint16_t*>(alloc(static_cast<size_t>(V) * H * 2, "embed"));
    upload("model.embed_tokens.weight", embed, V, H);
    if (cfg.tie_embeddings || !snap.find("lm_head.weight")) {
        lm_head = embed;
        names_["lm_head"] = names_["embed"];
    } else {
        lm_head = static_cast<uint16_t*>(alloc(static_cast<size_t>(V) * H * 2, "lm_head"));
        upload("lm_head.weight", lm_head, V, H);
    }
    decode_bytes_ += static_cast<size_t>(V) * H * 2;
    final_norm = vector_param("model.norm.weight", "final_norm", H);
    const std::vector<float> f = rope_inv_freq(cfg);
    inv_freq = static_cast<float*>(alloc(f.size() * 4, "inv_freq"));
    PIE_HIP_CHECK(hipMemcpyAsync(inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice, stream));
    PIE_HIP_CHECK(hipStreamSynchronize(stream));

    // One fused linear from several checkpoint projections, rows concatenated in order.
    struct Part {
        std::string prefix;   // e.g. "model.layers.0.self_attn.q_proj"
        int rows;
    };
    auto fused = [&](Linear& lin, const std::vector<Part>& parts, int K, const std::string& name) {
        int N = 0;
        for (const Part& p : parts) N += p.rows;
        prepare_linear(lin, N, K, name);
        const bool packed = snap.find(parts[0].prefix + ".weight_packed") != nullptr;
        if (packed) {
            // compressed-tensors pack-quantized int4: nibble j of word w = element 8w + j,
            // stored value + 8 (the layout of driver/cuda/src/kernels/dequant_wna16.cu:31-36)
            if (quant_ != Quant::Int4b8)
                throw std::runtime_error("snapshot: '" + name + "' is packed int4; set quant = \"int4b8\"");
            size_t row = 0;
            for (const Part& p : parts) {
                const StTensor& w = snap.at(p.prefix + ".weight_packed");
                const StTensor& sc = snap.at(p.prefix + ".weight_scale");
                if (w.dtype != "I32" && w.dtype != "U32") throw std::runtime_error("snapshot: weight_packed must be I32");
                expect_shape(w, p.prefix + ".weight_packed", p.rows, K / 8);
                expect_shape(sc, p.prefix + ".weight_scale", p.rows, K / lin.group);
                if (w.bytes != static_cast<size_t>(p.rows) * (K / 2) ||
                    (row + p.rows) * (static_cast<size_t>(K) / 2) > lin.data_bytes())
                    throw std::runtime_error("snapshot: '" + p.prefix + ".weight_packed' does not fit its rows");
                PIE_HIP_CHECK(hipMemcpyAsync(static_cast<uint8_t*>(lin.data) + row * (K / 2), w.data, w.bytes,
                                             hipMemcpyHostToDevice, stream));
                const uint16_t* sb = as_bf16(sc, staging);
                PIE_HIP_CHECK(hipMemcpyAsync(static_cast<uint16_t*>(lin.scale) + row * (K / lin.group), sb,
                                             static_cast<size_t>(sc.elems()) * 2, hipMemcpyHostToDevice, stream));
                PIE_HIP_CHECK(hipStreamSynchronize(stream));
                row += p.rows;
            }
            return;
        }
        uint16_t* dst = quant_ == Quant::Bf16 ? static_cast<uint16_t*>(lin.data) : tmp_bf16_;
        size_t row = 0;
        for (const Part& p : parts) {
            upload(p.prefix + ".weight", dst + row * K, p.rows, K);
            row += p.rows;
        }
        if (quant_ != Quant::Bf16) quantise_scratch(lin, name, stream);
    };

    layers.resize(L);
    for (int l = 0; l < L; ++l) {
        LayerWeights& w = layers[l];
        const std::string p = "layers." + std::to_string(l) + ".";
        const std::string hf = "model.layers." + std::to_string(l) + ".";
        w.attn_norm = vector_param(hf + "input_layernorm.weight", p + "attn_norm", H);
        w.ffn_norm = vector_param(hf + "post_attention_layernorm.weight", p + "ffn_norm", H);
        if (has_qk_norm()) {
            w.q_norm = vector_param(hf + "self_attn.q_norm.weight", p + "q_norm", d);
            w.k_norm = vector_param(hf + "self_attn.k_norm.weight", p + "k_norm", d);
        }
        fused(w.wqkv, {{hf + "self_attn.q_proj", hq * d}, {hf + "self_attn.k_proj", hk * d},
                       {hf + "self_attn.v_proj", hk * d}}, H, p + "wqkv");
        fused(w.wo, {{hf + "self_attn.o_proj", H}}, hq * d, p + "wo");
        if (!moe) {
            fused(w.wgu, {{hf + "mlp.gate_proj", I}, {hf + "mlp.up_proj", I}}, H, p + "wgu");
            interleave_gate_up(w.wgu, 1, stream);
            fused(w.wdown, {{hf + "mlp.down_proj", H}}, I, p + "wdown");
        } else {
            w.router.kind = Quant::Bf16;
            w.router.N = E;
            w.router.K = H;
            w.router.data = alloc(static_cast<size_t>(E) * H * 2, p + "router");
            upload(hf + "mlp.gate.weight", static_cast<uint16_t*>(w.router.data), E, H);
            std::vector<Part> gu, down;
            for (int e = 0; e < E; ++e) {
                const std::string ex = hf + "mlp.experts." + std::to_string(e) + ".";
                gu.push_back({ex + "gate_proj", I});
                gu.push_back({ex + "up_proj", I});
                down.push_back({ex + "down_proj", H});
            }
            const size_t before = decode_bytes_;
            fused(w.wgu, gu, H, p + "wgu");
            interleave_gate_up(w.wgu, E, stream);
            fused(w.wdown, down, I, p + "wdown");
            const size_t all = decode_bytes_ - before;
            decode_bytes_ = before + all / E * cfg.top_k + static_cast<size_t>(E) * H * 2;
        }
    }
    PIE_HIP_CHECK(hipStreamSynchronize(stream));
    (void)hipFree(tmp_bf16_);
    tmp_bf16_ = nullptr;
    pair_qk_rows(stream);
}

}  // namespace pie_hip_driver
