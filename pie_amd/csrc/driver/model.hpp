// Model weights resident in HBM, in the storage formats the kernels stream.
//
// Layout per decoder layer (llama-like; op sequence of
// driver/portable/src/graph_qwen3.cpp:225-829 and driver/cuda/src/model/llama_like.cpp:364-762):
//   attn_norm [H] bf16, wqkv [(hq+2hk)d, H] (q rows, then k rows, then v rows — per-row /
//   per-group scales make the fusion exact), optional q_norm/k_norm [d], wo [H, hq*d],
//   ffn_norm [H], then either wgu [2I, H] (rows interleaved gate_0, up_0, gate_1, ... for the
//   fused SwiGLU epilogue) + wdown [H, I], or the
//   MoE block: router [E, H] bf16, experts stacked along the rows — wgu [E * 2Ie, H] (gate/up
//   interleaved inside each expert) and wdown [E * H, Ie].
// embed [V, H] bf16, final_norm [H], lm_head [V, H] bf16 (aliases embed when tied); those
// three stay unquantised like the reference (driver/cuda/src/config.hpp:20-30).
#pragma once

#include <array>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "config.hpp"

namespace pie_hip_driver {

enum class Quant { Int4b8, Int8, Fp8, Bf16 };

struct Linear {
    Quant kind = Quant::Bf16;
    void* data = nullptr;   // packed weights, [N, K] in the format's element size
    void* scale = nullptr;  // int4: bf16 [N, K/G]; int8/fp8: f32 or bf16 [N]; bf16: null
    bool scale_bf16 = true;
    int N = 0, K = 0, group = 0;
    // optional copies in the skinny GEMM's tile-major layout (pie_hip_repack_mfma_tiles)
    void* data_tiled = nullptr;
    void* scale_tiled = nullptr;   // int4 group scales; other formats keep `scale`
    // kernel that measured fastest for M activation rows at start-up (index M, 0..128):
    // 0 GEMV, 1 skinny GEMM, 2 tiled GEMM, 3 tiled GEMM in K shares; -1: not measured, the cost
    // model decides
    std::array<int8_t, 129> tuned = [] { std::array<int8_t, 129> t{}; t.fill(-1); return t; }();
    size_t data_bytes() const {
        const size_t nk = static_cast<size_t>(N) * K;
        switch (kind) {
            case Quant::Int4b8: return nk / 2;
            case Quant::Bf16: return nk * 2;
            default: return nk;
        }
    }
    size_t scale_bytes() const {
        switch (kind) {
            case Quant::Int4b8: return static_cast<size_t>(N) * (K / group) * 2;
            case Quant::Bf16: return 0;
            default: return static_cast<size_t>(N) * (scale_bf16 ? 2 : 4);
        }
    }
};

struct LayerWeights {
    uint16_t* attn_norm = nullptr;
    uint16_t* ffn_norm = nullptr;
    uint16_t* q_norm = nullptr;
    uint16_t* k_norm = nullptr;
    Linear wqkv, wo, wgu, wdown;  // MoE: wgu / wdown hold the experts stacked along the rows
    Linear router;                // MoE: [E, H] bf16
};

struct TensorRef {
    void* ptr;
    size_t bytes;
};

class Model {
  public:
    Model() = default;
    ~Model();
    Model(const Model&) = delete;
    Model& operator=(const Model&) = delete;

    // Allocates every tensor and fills it with seeded synthetic weights on the device:
    // N(0, init_std) rounded to bf16, then quantised by the library's quantiser kernels.
    void init_synthetic(const ModelConfig& cfg, hipStream_t stream);

    // The same layout filled from a Hugging Face snapshot (cfg.checkpoint_dir): bf16 / f16 / f32
    // `*.weight` tensors are fused (q|k|v rows, gate/up interleaved, experts stacked) and
    // quantised on the device to cfg.quant; compressed-tensors int4 checkpoints
    // (`weight_packed` int32 [N, K/8] + `weight_scale` [N, K/group]) are taken as stored.
    void load_snapshot(const ModelConfig& cfg, hipStream_t stream);

    // Builds the tile-major copies of every decoder linear whose shape the skinny GEMM takes.
    void build_tiled_copies(hipStream_t stream);

    const ModelConfig& cfg() const { return cfg_; }
    bool is_moe() const { return cfg_.arch == "qwen3_moe"; }
    bool has_qk_norm() const { return cfg_.arch != "llama3"; }
    // True when the q and k rows of every layer's wqkv were re-ordered at load so that rows
    // (2i, 2i+1) of a head hold the half-split RoPE pair (i, i + d/2): the fused projection
    // epilogues then rotate neighbouring outputs and store them at i and i + d/2.
    bool qk_rows_paired() const { return qk_rows_paired_; }
    Quant quant() const { return quant_; }

    uint16_t* embed = nullptr;
    uint16_t* lm_head = nullptr;
    uint16_t* final_norm = nullptr;
    float* inv_freq = nullptr;  // [d/2] device
    std::vector<LayerWeights> layers;

    // bytes streamed from HBM by one decode step at batch 1 (every weight once)
    size_t decode_weight_bytes() const { return decode_bytes_; }
    const std::map<std::string, TensorRef>& tensors() const { return names_; }

  private:
    void* alloc(size_t bytes, const std::string& name);
    void make_linear(Linear& lin, int N, int K, const std::string& name, std::uint64_t seed,
                     hipStream_t stream);
    void prepare_linear(Linear& lin, int N, int K, const std::string& name);
    void quantise_scratch(Linear& lin, const std::string& name, hipStream_t stream);
    void interleave_gate_up(Linear& lin, int blocks, hipStream_t stream);
    void interleave_row_blocks(Linear& lin, size_t half, size_t rows, hipStream_t stream);
    void pair_qk_rows(hipStream_t stream);
    bool qk_rows_paired_ = false;
    ModelConfig cfg_;
    Quant quant_ = Quant::Bf16;
    std::vector<void*> allocs_;
    std::map<std::string, TensorRef> names_;
    uint16_t* tmp_bf16_ = nullptr;  // scratch for the largest bf16 tensor being quantised
    size_t tmp_elems_ = 0;
    size_t decode_bytes_ = 0;
};

// Host-side inv_freq table (theta^(-2i/d) with optional llama3 band scaling,
// driver/portable/src/model.cpp:1414-1448: the stored factor divides the base frequency).
std::vector<float> rope_inv_freq(const ModelConfig& cfg);
// What cos and sin are multiplied by: YaRN's attention factor (0.1 ln(factor) + 1 unless the
// config states one), 1 for every other scheme.
float rope_mscale(const ModelConfig& cfg);

}  // namespace pie_hip_driver
