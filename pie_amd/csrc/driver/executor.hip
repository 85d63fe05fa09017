#include "executor.hpp"

#include <algorithm>
#include <chrono>
#include <cstring>
#include <stdexcept>
#include <string>

#include "pie_hip_kernels.h"

namespace pie_hip_driver {

#define PIE_HIP_CHECK(expr)                                                              \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess)                                                            \
            throw std::runtime_error(std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

#define PIE_KERNEL(expr)                                                                     \
    do {                                                                                     \
        const int st_ = (expr);                                                              \
        if (st_ != PIE_HIP_OK)                                                               \
            throw std::runtime_error(std::string(#expr) + " failed with status " +          \
                                     std::to_string(st_));                                   \
    } while (0)

namespace {

using clk = std::chrono::steady_clock;
uint32_t us_since(clk::time_point t0) {
    return static_cast<uint32_t>(
        std::chrono::duration_cast<std::chrono::microseconds>(clk::now() - t0).count());
}

template <typename T>
T* dmalloc(size_t elems) {
    void* p = nullptr;
    PIE_HIP_CHECK(hipMalloc(&p, std::max<size_t>(elems, 1) * sizeof(T)));
    return static_cast<T*>(p);
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int fmt_code(Quant q) {
    switch (q) {
        case Quant::Int4b8: return PIE_HIP_FMT_INT4B8;
        case Quant::Int8: return PIE_HIP_FMT_INT8;
        case Quant::Fp8: return PIE_HIP_FMT_FP8;
        default: return PIE_HIP_FMT_BF16;
    }
}

// Measured cost models (MI355X, microseconds, int4 8B-class shapes at 16-128 rows).  Skinny GEMM:
// ~5 us + the weights at ~2.8 TB/s for the first 16-row pass, each further (side-by-side) pass
// adding 85 % of that stream; from the tile-major copy (wave-private form) ~3.8 TB/s and 52 % per
// further pass, the pass count rounded up to a power of two.  Tiled GEMM (eight-wave blocks): K in
// 64-wide steps of ~0.60 us with 64-row block tiles (M <= 64), ~0.68 us with 128-row tiles, while
// the tiles fit the machine (512 resident blocks).  Split-K tiled GEMM: the steps of one share
// (+3 of prologue) at 1.06 / 1.36 us with two blocks per CU, per round of 512 blocks, plus ~15 us
// for the second kernel and the partials.
enum class GemmPath { Skinny, Tiled, TiledSplitK };
GemmPath pick_gemm(const Linear& w, int M, size_t ws_bytes) {
    if (w.K % 64 != 0 || M < 17) return GemmPath::Skinny;
    const int passes = (M + 15) / 16;
    // the wave-private form runs its passes side by side: cost steps at powers of two; above 32
    // rows a pass covers 32 rows and costs 1.38 of a 16-row one
    const int wpasses = M > 32 ? (M + 31) / 32 : passes;
    int p2 = 1;
    while (p2 < wpasses) p2 <<= 1;
    // (past eight passes the machine is full: the cost grows in proportion)
    const double wave_form = (M > 32 ? 1.38 : 1.0) *
                             (p2 <= 8 ? 1.0 + 0.52 * (p2 - 1) : (1.0 + 0.52 * 7) * wpasses / 8.0);
    const double skinny = w.data_tiled
                              ? 5.0 + static_cast<double>(w.data_bytes()) / 3.8e6 * wave_form
                              : 5.0 + static_cast<double>(w.data_bytes()) / 2.8e6 * (1.0 + 0.85 * (passes - 1));
    const int steps = w.K / 64;
    const double tiles = static_cast<double>((w.N + 127) / 128) * (M <= 64 ? 1 : (M + 127) / 128);
    const double tiled = 2.0 + steps * (M <= 64 ? 0.60 : 0.68) * std::max(1.0, tiles / 512.0);
    double split = 1e30;
    const size_t need = M <= 128 ? pie_hip_gemm_mfma_workspace_bytes(M, w.N, w.K) : 0;
    if (need && need <= ws_bytes) {
        const int shares = static_cast<int>(need / (static_cast<size_t>(M) * w.N * sizeof(float)));
        const int per = (steps + shares - 1) / shares;
        split = 15.0 + (per + 3) * (M <= 64 ? 1.06 : 1.36) * std::ceil(tiles * shares / 512.0);
    }
    if (split < skinny && split < tiled) return GemmPath::TiledSplitK;
    return tiled < skinny ? GemmPath::Tiled : GemmPath::Skinny;
}

// The fitted cost model's kernel for M rows of `w`: 0 GEMV, 1 skinny GEMM, 2 tiled GEMM, 3 tiled GEMM
// in K shares.  Two to four rows: the GEMV pays its dot products once per row, the skinny GEMM over
// the tile-major copy does not but needs the norm as its own launch (~4.8 us).  Costs fitted to
// the 8B shapes decide (decode steps of 2 / 3 / 4 rows over 512-token contexts: 1.91 / 2.46 /
// 2.79 ms with the GEMV everywhere, 2.01 / 2.08 / 2.14 ms with the skinny GEMM everywhere);
// without a tile-major copy the GEMV keeps all four.
int model_route(const Linear& w, int M, bool has_norm, size_t ws_bytes) {
    if (M <= 4) {
        if (M < 2 || !w.data_tiled) return 0;
        const double bytes = static_cast<double>(w.data_bytes());
        const double t_gemv = 3.4 + bytes / 5.5e6 * (M == 2 ? 1.35 : 1.0 + 0.5 * (M - 1));   // (a second row costs the GEMV less than the third and fourth)
        const double t_skinny = 4.4 + bytes / 4.2e6 + (has_norm ? 4.8 : 0.0);
        if (t_gemv <= t_skinny) return 0;
    }
    const GemmPath p = pick_gemm(w, M, ws_bytes);
    return p == GemmPath::Skinny ? 1 : p == GemmPath::Tiled ? 2 : 3;
}

// (PIE_GEMV_MAX_ROWS = n: rows up to n take the GEMV, more the skinny GEMM, whatever the costs say)
int forced_gemv_rows() {
    static const int forced_rows = [] { const char* e = getenv("PIE_GEMV_MAX_ROWS"); return e ? atoi(e) : -1; }();
    return forced_rows;
}

// Whether linear_fused sends M rows of this linear to the GEMV (its first choice, before any
// refusal by the kernel).
bool routes_to_gemv(const Linear& w, int M, bool has_norm, size_t ws_bytes) {
    const int tuned = M <= 128 ? w.tuned[M] : -1;
    if (tuned >= 0) return tuned == 0 && M <= 4;
    if (forced_gemv_rows() >= 0) return M <= std::min(forced_gemv_rows(), 4);
    return model_route(w, M, has_norm, ws_bytes) == 0;
}

// y = epilogue(rmsnorm?(act) · W^T) by the weight's storage format — the dispatcher role of
// gemm_act_x_w (driver/cuda/src/ops/gemm.cpp:1414-1583).  Up to four rows: the weight-streaming
// GEMV with the norm riding in its activation staging and SwiGLU in its epilogue.  More rows
// (norm as its own kernel into `norm_tmp`): the matrix-core skinny GEMM, which streams the
// weights once per 16 rows, or the tiled matrix-core GEMM where its cost model wins; shapes those do
// not take fall back to the GEMV path.
// `force`: -1 = pick (the start-up measurement when there is one, else the cost model); 0..3 = that
// kernel whatever the costs (the tuner's own launches).  Returns false when a forced kernel does
// not take the shape.
bool linear_fused(const Linear& w, const uint16_t* act, const uint16_t* norm_w, float eps,
                  uint16_t* y, int M, int beta, int swiglu, uint16_t* norm_tmp, void* gemm_ws,
                  size_t gemm_ws_bytes, hipStream_t s, int force = -1) {
    const int fmt = fmt_code(w.kind);
    const int sbf = w.scale_bf16 ? 1 : 0;
    const int forced_rows = forced_gemv_rows();
    int tuned = force >= 0 ? force : (M <= 128 ? w.tuned[M] : -1);
    bool gemv;
    if (tuned >= 0) {
        gemv = tuned == 0 && M <= 4;
    } else if (forced_rows >= 0) {
        gemv = M <= std::min(forced_rows, 4);
    } else {
        tuned = model_route(w, M, norm_w != nullptr, gemm_ws_bytes);
        gemv = tuned == 0;
    }
    if (gemv) {
        const int st = pie_hip_linear_fused(fmt, act, norm_w, eps, w.data, w.scale, sbf, w.group, y, M, w.N, w.K,
                                            beta, swiglu, s);
        if (st == PIE_HIP_OK) return true;
        if (st != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(st);
        if (force >= 0) return false;
        // (a row too long for the GEMV's staged activations: the matrix-core kernels take any K)
    }
    {
        const uint16_t* a = act;
        if (norm_w) {
            PIE_KERNEL(pie_hip_rmsnorm(act, norm_w, norm_tmp, M, w.K, eps, s));
            a = norm_tmp;
        }
        const GemmPath path = tuned == 1   ? GemmPath::Skinny
                              : tuned == 2 ? GemmPath::Tiled
                              : tuned == 3 ? GemmPath::TiledSplitK
                                           : pick_gemm(w, M, gemm_ws_bytes);   // (forced row limit, GEMV refusal)
        if (path != GemmPath::Skinny) {
            // the tiled GEMM (weights dequantised to bf16 while staged), in K shares for a
            // decode batch whose output has few tiles
            const int sg = path == GemmPath::TiledSplitK
                               ? pie_hip_gemm_mfma_splitk(fmt, a, w.data, w.scale, sbf, w.group, y, M, w.N,
                                                          w.K, beta, swiglu, gemm_ws, gemm_ws_bytes, s)
                               : pie_hip_gemm_mfma(fmt, a, w.data, w.scale, sbf, w.group, y, M, w.N, w.K,
                                                   beta, swiglu, s);
            if (sg == PIE_HIP_OK) return true;
            if (sg != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(sg);
            if (force >= 0) return false;
        }
        const int st = w.data_tiled
                           ? pie_hip_gemm_skinny_tiled(fmt, a, w.data_tiled, w.scale_tiled ? w.scale_tiled : w.scale,
                                                       sbf, w.group, y, M, w.N, w.K, beta, swiglu, s)
                           : pie_hip_gemm_skinny(fmt, a, w.data, w.scale, sbf, w.group, y, M, w.N, w.K, beta,
                                                 swiglu, s);
        if (st == PIE_HIP_OK) return true;
        if (st != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(st);
        if (force >= 0) return false;
        PIE_KERNEL(pie_hip_linear_fused(fmt, a, nullptr, eps, w.data, w.scale, sbf, w.group, y, M,
                                        w.N, w.K, beta, swiglu, s));
    }
    return true;
}

}  // namespace

// Staged inputs are packed back to back in an order that makes every offset a function of
// (rows, sampled rows) only — the page list goes last — so one contiguous host-to-device copy
// feeds a forward and a captured graph's pointers stay valid for its (rows, sampled rows) key.
Executor::Inputs Executor::input_layout(int N, int S) {
    Inputs in{};
    size_t off = 0;
    in.off_tokens = off;       off = align_up(off + static_cast<size_t>(N) * 4, 256);
    in.off_positions = off;    off = align_up(off + static_cast<size_t>(N) * 4, 256);
    in.off_slots = off;        off = align_up(off + static_cast<size_t>(N) * 8, 256);
    in.off_row_begin = off;    off = align_up(off + static_cast<size_t>(N) * 4, 256);
    in.off_row_len = off;      off = align_up(off + static_cast<size_t>(N) * 4, 256);
    in.off_sample_rows = off;  off = align_up(off + static_cast<size_t>(S) * 4, 256);
    in.off_pages = off;
    in.total = off;
    return in;
}

Executor::Executor(const DriverConfig& cfg, Model& model) : cfg_(cfg), model_(model) {
    PIE_HIP_CHECK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    page_size_ = cfg.batching.kv_page_size;
    total_pages_ = cfg.batching.total_pages;
    max_tokens_ = cfg.batching.max_forward_tokens;
    max_page_refs_ = 4 * total_pages_ + max_tokens_;
    kv_format_ = kv_format_code(cfg.batching.kv_cache_dtype);
    alloc_kv();
    cpu_pages_ = std::max(0, cfg.batching.cpu_pages);
    if (cpu_pages_ > 0) {
        const size_t bytes = static_cast<size_t>(model.cfg().layers) * 2 * cpu_pages_ *
                             (page_bytes() + scale_page_bytes());
        PIE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&swap_pool_), bytes, hipHostMallocDefault));
        std::memset(swap_pool_, 0, bytes);
    }

    const ModelConfig& m = model.cfg();
    const size_t T = static_cast<size_t>(max_tokens_);
    const int H = m.hidden, d = m.head_dim, hq = m.q_heads, hk = m.kv_heads;
    const int I = model.is_moe() ? m.expert_intermediate : m.intermediate;
    x_ = dmalloc<uint16_t>(T * H);
    xn_ = dmalloc<uint16_t>(T * H);
    qkv_ = dmalloc<uint16_t>(T * (hq + 2 * hk) * d);
    q_ = dmalloc<uint16_t>(T * hq * d);
    attn_ = dmalloc<uint16_t>(T * hq * d);
    gu_ = dmalloc<uint16_t>(T * 2 * I);
    if (model.is_moe()) {
        // one row per route (token, k): expert activations and per-route outputs, the router
        // logits, and the grouped layout the routing kernel builds
        const size_t R = T * m.top_k;
        act_ = dmalloc<uint16_t>(R * I);
        moe_y_ = dmalloc<uint16_t>(R * H);
        moe_logits_ = dmalloc<uint16_t>(T * m.num_experts);
        moe_idx_ = dmalloc<int32_t>(R);
        moe_w_ = dmalloc<float>(R);
        moe_offsets_ = dmalloc<int32_t>(m.num_experts + 1);
        moe_route_token_ = dmalloc<int32_t>(R);
        moe_route_pos_ = dmalloc<int32_t>(R);
    } else {
        act_ = dmalloc<uint16_t>(T * I);
    }
    rope_tab_ = dmalloc<float>(T * d);
    const size_t srows = std::min<size_t>(T, 2 * static_cast<size_t>(cfg.batching.max_forward_requests));
    xs_ = dmalloc<uint16_t>(srows * H);
    logits_ = dmalloc<uint16_t>(srows * m.vocab);
    out_tokens_ = dmalloc<uint32_t>(T);
    out_cap_ = T;
    amax_ws_bytes_ = pie_hip_lm_head_argmax_workspace_bytes(4, m.vocab);
    if (amax_ws_bytes_) PIE_HIP_CHECK(hipMalloc(&amax_ws_, amax_ws_bytes_));
    // Bound of the split-K partial buffers over every (rows, context) the planner can pick:
    // rows * splits <= 3072/hk + rows.
    attn_ws_bytes_ = (3072 / static_cast<size_t>(hk) + 1 + T) * hq * (d + 2) * sizeof(float);
    PIE_HIP_CHECK(hipMalloc(&attn_ws_, attn_ws_bytes_));
    if (kv_format_ != PIE_HIP_KV_BF16) {
        k_rows_ = dmalloc<uint16_t>(T * hk * d);
        v_rows_ = dmalloc<uint16_t>(T * hk * d);
        iota_slots_ = dmalloc<int64_t>(T);
        std::vector<int64_t> iota(T);
        for (size_t i = 0; i < T; ++i) iota[i] = static_cast<int64_t>(i);
        PIE_HIP_CHECK(hipMemcpy(iota_slots_, iota.data(), T * sizeof(int64_t), hipMemcpyHostToDevice));
    }
    // fp32 partials of the split-K GEMM for decode batches of up to 128 rows (dense layers)
    if (!model.layers.empty()) {
        const LayerWeights& l0 = model.layers[0];
        for (const Linear* w : {&l0.wqkv, &l0.wo, &l0.wgu, &l0.wdown})
            for (int rows : {64, 128})
                if (w->data && w->K % 64 == 0)
                    gemm_ws_bytes_ = std::max(gemm_ws_bytes_, pie_hip_gemm_mfma_workspace_bytes(rows, w->N, w->K));
        gemm_ws_bytes_ = std::min<size_t>(gemm_ws_bytes_, size_t(64) << 20);
        if (gemm_ws_bytes_) PIE_HIP_CHECK(hipMalloc(&gemm_ws_, gemm_ws_bytes_));
    }

    in_ = input_layout(max_tokens_, max_tokens_);
    in_.total = align_up(in_.off_pages + static_cast<size_t>(max_page_refs_) * 4, 256);
    PIE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&in_host_), in_.total, hipHostMallocDefault));
    PIE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&in_dev_), in_.total));
    PIE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&out_host_), T * 4, hipHostMallocDefault));
    tune_linears();
}

Executor::~Executor() {
    if (stream_) (void)hipStreamSynchronize(stream_);
    for (auto& kv : graphs_) (void)hipGraphExecDestroy(kv.second);
    for (auto* p : k_pool_) (void)hipFree(p);
    for (auto* p : v_pool_) (void)hipFree(p);
    for (void* p : {static_cast<void*>(x_), static_cast<void*>(xn_), static_cast<void*>(qkv_),
                    static_cast<void*>(q_), static_cast<void*>(attn_), static_cast<void*>(gu_),
                    static_cast<void*>(act_), static_cast<void*>(xs_), static_cast<void*>(logits_),
                    static_cast<void*>(rope_tab_), static_cast<void*>(out_tokens_), attn_ws_, gemm_ws_, amax_ws_,
                    static_cast<void*>(in_dev_), static_cast<void*>(copy_ids_),
                    static_cast<void*>(moe_y_), static_cast<void*>(moe_logits_),
                    static_cast<void*>(moe_idx_), static_cast<void*>(moe_w_),
                    static_cast<void*>(moe_offsets_), static_cast<void*>(moe_route_token_),
                    static_cast<void*>(moe_route_pos_), static_cast<void*>(k_rows_),
                    static_cast<void*>(v_rows_), static_cast<void*>(iota_slots_)})
        if (p) (void)hipFree(p);
    for (auto* p : k_scale_pool_) (void)hipFree(p);
    for (auto* p : v_scale_pool_) (void)hipFree(p);
    if (kv_shadow_k_) (void)hipFree(kv_shadow_k_);
    if (kv_shadow_v_) (void)hipFree(kv_shadow_v_);
    for (Growable* g : {&mask_in_host_, &mask_in_dev_, &mask_bitmap_, &tile_in_host_, &tile_in_dev_}) g->release();
    for (Growable* g : {&samp_f32_, &samp_ws_, &samp_in_dev_, &samp_in_host_, &samp_out_dev_, &samp_out_host_})
        g->release();
    if (swap_pool_) (void)hipHostFree(swap_pool_);
    if (in_host_) (void)hipHostFree(in_host_);
    if (out_host_) (void)hipHostFree(out_host_);
    if (stream_) (void)hipStreamDestroy(stream_);
}

// Page sizes of the storage formats: kv_bytes_per_page / scale_bytes_per_page,
// driver/cuda/src/kv_cache_format.cpp:27-49.
size_t Executor::page_bytes() const {
    const ModelConfig& m = model_.cfg();
    const size_t elems = static_cast<size_t>(page_size_) * m.kv_heads * m.head_dim;
    if (kv_format_ == PIE_HIP_KV_FP4_BLOCK) return elems / 2;   // two codes per byte
    return elems * (kv_format_ == PIE_HIP_KV_BF16 ? 2 : 1);
}
size_t Executor::scale_page_bytes() const {
    const ModelConfig& m = model_.cfg();
    if (kv_format_ == PIE_HIP_KV_FP4_BLOCK)   // one scale per block of 16 elements
        return static_cast<size_t>(page_size_) * m.kv_heads * ((m.head_dim + 15) / 16) * sizeof(float);
    const bool scaled = kv_format_ == PIE_HIP_KV_INT8_PER_TOKEN_HEAD || kv_format_ == PIE_HIP_KV_FP8_PER_TOKEN_HEAD;
    return scaled ? static_cast<size_t>(page_size_) * m.kv_heads * sizeof(float) : 0;
}

// Start-up measurement of the decoder linears' candidate kernels.  For every role (q|k|v, wo,
// gate|up, down) and a ladder of row counts the GEMV (2-4 rows), the skinny GEMM and the tiled GEMM
// (17-128 rows; in K shares where the workspace allows) run over the weights of successive layers
// (so that they come from HBM, as in a forward pass) on zeroed activations; the fastest goes into
// every layer's table for the row counts up to the next rung.
void Executor::tune_linears() {
    const ModelConfig& m = model_.cfg();
    if (model_.layers.empty() || !cfg_.runtime.tune_linears || getenv("PIE_NO_TUNE")) return;
    hipStream_t s = stream_;
    const size_t T = static_cast<size_t>(max_tokens_);
    const int H = m.hidden, d = m.head_dim, hq = m.q_heads, hk = m.kv_heads;
    const int I = model_.is_moe() ? m.expert_intermediate : m.intermediate;
    PIE_HIP_CHECK(hipMemsetAsync(x_, 0, T * H * 2, s));
    PIE_HIP_CHECK(hipMemsetAsync(attn_, 0, T * hq * d * 2, s));
    if (!model_.is_moe()) PIE_HIP_CHECK(hipMemsetAsync(act_, 0, T * I * 2, s));
    struct Role {
        Linear LayerWeights::*lin;
        uint16_t* LayerWeights::*norm;
        const uint16_t* act;
        uint16_t* y;
        int beta, swiglu;
        double tiled_handicap_us;   // what the tiled route costs beyond the GEMM (a separate RoPE launch)
    };
    std::vector<Role> roles = {
        {&LayerWeights::wqkv, &LayerWeights::attn_norm, x_, qkv_, 0, 0, 4.0},
        {&LayerWeights::wo, nullptr, attn_, x_, 1, 0, 0.0},
    };
    if (!model_.is_moe()) {
        roles.push_back({&LayerWeights::wgu, &LayerWeights::ffn_norm, x_, act_, 0, 1, 0.0});
        roles.push_back({&LayerWeights::wdown, nullptr, act_, x_, 1, 0, 0.0});
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    PIE_HIP_CHECK(hipEventCreate(&e0));
    PIE_HIP_CHECK(hipEventCreate(&e1));
    const int L = static_cast<int>(model_.layers.size());
    int rot = 0;
    // (the smaller of two timed rounds: a round disturbed by something else on the machine would
    // otherwise decide the dispatch for the life of the process)
    auto time_us = [&](const Role& r, int M, int force) -> double {
        constexpr int kWarm = 1, kReps = 4, kRounds = 2;
        double best = 1e30;
        for (int round = 0; round < kRounds; ++round) {
            for (int i = 0; i < kWarm + kReps; ++i) {
                if (i == kWarm) PIE_HIP_CHECK(hipEventRecord(e0, s));
                LayerWeights& lw = model_.layers[static_cast<size_t>(rot++ % L)];
                const uint16_t* nw = r.norm ? lw.*(r.norm) : nullptr;
                if (!linear_fused(lw.*(r.lin), r.act, nw, m.rms_eps, r.y, M, r.beta, r.swiglu, xn_, gemm_ws_,
                                  gemm_ws_bytes_, s, force))
                    return 1e30;
            }
            PIE_HIP_CHECK(hipEventRecord(e1, s));
            PIE_HIP_CHECK(hipEventSynchronize(e1));
            float ms = 0.f;
            PIE_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
            best = std::min(best, static_cast<double>(ms) * 1e3 / kReps);
        }
        return best;
    };
    const int ladder[] = {2, 3, 4, 17, 24, 32, 33, 40, 48, 56, 64, 65, 72, 80, 88, 96, 97, 104, 112, 120, 128};
    for (const Role& r : roles) {
        const Linear& l0 = model_.layers[0].*(r.lin);
        if (!l0.data || !l0.data_tiled) continue;   // (without the tile-major copy the cost model's defaults stand)
        int prev = 1;
        // llama-type layers send two to four decode rows of q|k|v to the GEMV with the RoPE
        // epilogue whatever a measurement says (Executor::body): those rungs would decide nothing
        const bool qkv_fused_rows = r.lin == &LayerWeights::wqkv && !model_.layers[0].q_norm &&
                                    (m.rope_interleaved || model_.qk_rows_paired()) && (d & (d - 1)) == 0 &&
                                    kv_format_ == PIE_HIP_KV_BF16;
        for (int M : ladder) {
            if (M > max_tokens_) break;
            if (M <= 4 && qkv_fused_rows) {
                prev = M;
                continue;
            }
            int best = -1;
            double best_t = 1e30, model_t = 1e30;
            const int by_model = model_route(l0, M, r.norm != nullptr, gemm_ws_bytes_);
            for (int cand = M <= 4 ? 0 : 1; cand <= (M <= 4 ? 1 : 3); ++cand) {
                if (cand == 3 && (M > 128 || pie_hip_gemm_mfma_workspace_bytes(M, l0.N, l0.K) == 0 ||
                                  pie_hip_gemm_mfma_workspace_bytes(M, l0.N, l0.K) > gemm_ws_bytes_))
                    continue;
                if (cand >= 2 && l0.K % 64 != 0) continue;
                double t = time_us(r, M, cand);
                if (cand >= 2) t += r.tiled_handicap_us;
                if (cand == by_model) model_t = t;
                if (t < best_t) {
                    best_t = t;
                    best = cand;
                }
            }
            // A measurement overrides the cost model only where it is clearly faster (a tenth and
            // half a microsecond): candidates that tie keep the model's kernel, so that timing noise
            // does not change which kernel — and with it which rounding — a restart gets.
            if (model_t < 1e29 && !(best_t < 0.9 * model_t && best_t + 0.5 < model_t)) best = by_model;
            // rows 5..16 stay with the skinny GEMM; a rung decides for the row counts above the
            // previous rung up to itself
            const int lo = M <= 4 ? M : std::max(prev + 1, 17);
            if (best >= 0)
                for (auto& lw : model_.layers)
                    for (int mm = lo; mm <= M; ++mm) (lw.*(r.lin)).tuned[static_cast<size_t>(mm)] = static_cast<int8_t>(best);
            prev = M;
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    PIE_HIP_CHECK(hipStreamSynchronize(s));
}

// Allocate the pool; on out-of-memory halve the page count down to 64 pages
// (driver/portable/src/entry.cpp:327-348).
void Executor::alloc_kv() {
    const int L = model_.cfg().layers;
    for (;;) {
        const size_t bytes = page_bytes() * static_cast<size_t>(total_pages_);
        const size_t sbytes = scale_page_bytes() * static_cast<size_t>(total_pages_);
        bool ok = true;
        for (int l = 0; l < L && ok; ++l) {
            void *k = nullptr, *v = nullptr;
            if (hipMalloc(&k, bytes) != hipSuccess) { ok = false; break; }
            k_pool_.push_back(static_cast<uint16_t*>(k));
            if (hipMalloc(&v, bytes) != hipSuccess) { ok = false; break; }
            v_pool_.push_back(static_cast<uint16_t*>(v));
            if (sbytes) {
                if (hipMalloc(&k, sbytes) != hipSuccess) { ok = false; break; }
                k_scale_pool_.push_back(static_cast<float*>(k));
                if (hipMalloc(&v, sbytes) != hipSuccess) { ok = false; break; }
                v_scale_pool_.push_back(static_cast<float*>(v));
            }
        }
        if (ok && kv_format_ == PIE_HIP_KV_FP4_BLOCK) {
            // the bf16 pages the attention kernels read (k_bf16_pages / v_bf16_pages of the
            // reference's layer view, driver/cuda/src/kernels/kv_paged.cu:698-770)
            const ModelConfig& m = model_.cfg();
            const size_t shadow = static_cast<size_t>(total_pages_) * page_size_ * m.kv_heads * m.head_dim * 2;
            void *k = nullptr, *v = nullptr;
            if (hipMalloc(&k, shadow) != hipSuccess || hipMalloc(&v, shadow) != hipSuccess) {
                if (k) (void)hipFree(k);
                ok = false;
            } else {
                kv_shadow_k_ = static_cast<uint16_t*>(k);
                kv_shadow_v_ = static_cast<uint16_t*>(v);
                PIE_HIP_CHECK(hipMemsetAsync(kv_shadow_k_, 0, shadow, stream_));
                PIE_HIP_CHECK(hipMemsetAsync(kv_shadow_v_, 0, shadow, stream_));
            }
        }
        if (ok) {
            // Pages start zeroed so slots no request has written hold finite values.
            for (int l = 0; l < L; ++l) {
                PIE_HIP_CHECK(hipMemsetAsync(k_pool_[l], 0, bytes, stream_));
                PIE_HIP_CHECK(hipMemsetAsync(v_pool_[l], 0, bytes, stream_));
                if (sbytes) {
                    PIE_HIP_CHECK(hipMemsetAsync(k_scale_pool_[l], 0, sbytes, stream_));
                    PIE_HIP_CHECK(hipMemsetAsync(v_scale_pool_[l], 0, sbytes, stream_));
                }
            }
            PIE_HIP_CHECK(hipStreamSynchronize(stream_));
            return;
        }
        (void)hipGetLastError();
        for (auto* p : k_pool_) (void)hipFree(p);
        for (auto* p : v_pool_) (void)hipFree(p);
        for (auto* p : k_scale_pool_) (void)hipFree(p);
        for (auto* p : v_scale_pool_) (void)hipFree(p);
        k_pool_.clear();
        v_pool_.clear();
        k_scale_pool_.clear();
        v_scale_pool_.clear();
        if (total_pages_ <= 64) throw std::runtime_error("executor: cannot allocate the KV pool");
        total_pages_ = std::max(64, total_pages_ / 2);
    }
}

// x += sum_k w_k * down_e(swiglu(gate_up_e(norm(x)))) over each token's top-k experts
// (driver/portable/src/graph_common.cpp:237-345; kernel-by-kernel form
// driver/cuda/src/model/kimi_forward.cpp:662-714): norm, router GEMM, one routing kernel, two
// grouped expert GEMMs that read every touched expert once, one combine onto the residual.
void Executor::moe_block(const LayerWeights& w, int N, const uint16_t* next_norm, hipStream_t s) {
    const ModelConfig& m = model_.cfg();
    const int H = m.hidden, E = m.num_experts, K = m.top_k, Ie = m.expert_intermediate;
    const int fmt = fmt_code(w.wgu.kind);
    const int sbf = w.wgu.scale_bf16 ? 1 : 0;
    // a decode batch: norm, router logits and top-k per token in one launch (every token's block
    // reads the router matrix through the L2, which stops paying at a few hundred rows)
    // (PIE_MOE_FUSED=0: the separate launches, for measurement)
    static const bool fused_on = [] { const char* e = getenv("PIE_MOE_FUSED"); return !e || atoi(e) != 0; }();
    if (!fused_on) next_norm = nullptr;
    int routed = PIE_HIP_ERR_UNSUPPORTED;
    if (fused_on && N <= kFusedRouteRows && w.router.kind == Quant::Bf16)
        routed = pie_hip_moe_norm_route(x_, w.ffn_norm, m.rms_eps, static_cast<const uint16_t*>(w.router.data), xn_,
                                        moe_logits_, moe_idx_, moe_w_, moe_offsets_, moe_route_token_,
                                        moe_route_pos_, N, H, E, K, m.norm_topk ? 1 : 0, s);
    if (routed == PIE_HIP_ERR_UNSUPPORTED) {
    PIE_KERNEL(pie_hip_rmsnorm(x_, w.ffn_norm, xn_, N, H, m.rms_eps, s));
    linear_fused(w.router, xn_, nullptr, m.rms_eps, moe_logits_, N, 0, 0, nullptr, gemm_ws_, gemm_ws_bytes_, s);
    PIE_KERNEL(pie_hip_moe_route_opt(moe_logits_, moe_idx_, moe_w_, moe_offsets_, moe_route_token_,
                                     moe_route_pos_, N, E, K, m.norm_topk ? 1 : 0, s));
    } else {
        PIE_KERNEL(routed);
    }
    const int hint = std::max(1, std::min(N, 2 * ((N * K + E - 1) / E)));
    // experts stacked along the rows: the tile-major copy of the stack keeps expert e at the same
    // byte stride (every expert has a multiple of 16 rows)
    const bool tiled = w.wgu.data_tiled && w.wdown.data_tiled && (2 * Ie) % 16 == 0 && H % 16 == 0;
    auto grouped = tiled ? pie_hip_moe_grouped_gemm_tiled : pie_hip_moe_grouped_gemm;
    auto wptr = [&](const Linear& l) { return tiled ? l.data_tiled : l.data; };
    auto sptr = [&](const Linear& l) { return tiled && l.scale_tiled ? l.scale_tiled : l.scale; };
    PIE_KERNEL(grouped(fmt, xn_, moe_route_token_, moe_offsets_, E, hint, wptr(w.wgu),
                       w.wgu.data_bytes() / E, sptr(w.wgu), w.wgu.scale_bytes() / E, sbf, w.wgu.group,
                       act_, 2 * Ie, H, 1, s));
    PIE_KERNEL(grouped(fmt, act_, nullptr, moe_offsets_, E, hint, wptr(w.wdown), w.wdown.data_bytes() / E,
                       sptr(w.wdown), w.wdown.scale_bytes() / E, sbf, w.wdown.group, moe_y_, H, Ie, 0, s));
    // with the next layer's attention norm riding along when that layer takes its rows normalised
    int combined = PIE_HIP_ERR_UNSUPPORTED;
    if (next_norm)
        combined = pie_hip_moe_combine_norm(moe_y_, moe_route_pos_, moe_w_, x_, next_norm, m.rms_eps, xn_, N, K, H, s);
    if (combined == PIE_HIP_ERR_UNSUPPORTED) {
        PIE_KERNEL(pie_hip_moe_combine(moe_y_, moe_route_pos_, moe_w_, x_, N, K, H, 1, s));
        xn_holds_next_norm_ = false;
    } else {
        PIE_KERNEL(combined);
        xn_holds_next_norm_ = true;
    }
}

void Executor::body(int N, int S, int max_kv_len) {
    xn_holds_next_norm_ = false;
    const Inputs in_ = input_layout(N, S);
    const ModelConfig& m = model_.cfg();
    const int H = m.hidden, d = m.head_dim, hq = m.q_heads, hk = m.kv_heads;
    hipStream_t s = stream_;
    const auto* tokens = reinterpret_cast<const uint32_t*>(in_dev_ + in_.off_tokens);
    const auto* positions = reinterpret_cast<const int32_t*>(in_dev_ + in_.off_positions);
    const auto* slots = reinterpret_cast<const int64_t*>(in_dev_ + in_.off_slots);
    const auto* row_begin = reinterpret_cast<const uint32_t*>(in_dev_ + in_.off_row_begin);
    const auto* row_len = reinterpret_cast<const int32_t*>(in_dev_ + in_.off_row_len);
    const auto* sample_rows = reinterpret_cast<const uint32_t*>(in_dev_ + in_.off_sample_rows);
    const auto* pages = reinterpret_cast<const uint32_t*>(in_dev_ + in_.off_pages);

    PIE_KERNEL(pie_hip_embed(tokens, model_.embed, x_, N, H, m.vocab, s));
    PIE_KERNEL(pie_hip_rope_table_scaled(positions, model_.inv_freq, rope_tab_, N, d, rope_mscale(m), s));
    // RoPE pairing as the rotation kernels take it: adjacent pairs, half-split pairs, or
    // half-split pairs over projection rows re-ordered at load (then the fused epilogues apply)
    const int pairing = m.rope_interleaved ? PIE_HIP_ROPE_ADJACENT
                        : model_.qk_rows_paired() ? PIE_HIP_ROPE_HALF_PAIRED_ROWS : PIE_HIP_ROPE_HALF;
    const bool fused_rope = pairing != PIE_HIP_ROPE_HALF && (d & (d - 1)) == 0;
    for (int l = 0; l < m.layers; ++l) {
        const LayerWeights& w = model_.layers[l];
        const bool kvq = kv_format_ != PIE_HIP_KV_BF16;
        float* ksc = kvq && !k_scale_pool_.empty() ? k_scale_pool_[l] : nullptr;
        float* vsc = kvq && !v_scale_pool_.empty() ? v_scale_pool_[l] : nullptr;
        // (the previous layer's MoE combine may have left this layer's normalised rows in xn_)
        const bool prenormed = xn_holds_next_norm_;
        xn_holds_next_norm_ = false;
        if (kvq) {
            // one-byte pools: the rotated K / V rows of this step are staged as bf16 rows (row t
            // in "slot" t) and quantised into the tokens' real slots
            linear_fused(w.wqkv, prenormed ? xn_ : x_, prenormed ? nullptr : w.attn_norm, m.rms_eps, qkv_, N, 0, 0, xn_,
                         gemm_ws_, gemm_ws_bytes_, s);
            // rotation and quantising write in one launch; head dims past 256 take the two kernels
            const int st = pie_hip_qkv_rope_kvwrite_quant(kv_format_, qkv_, q_, k_pool_[l], v_pool_[l], ksc, vsc,
                                                          w.q_norm, w.k_norm, rope_tab_, slots, N, hq, hk, d,
                                                          page_size_, pairing, m.rms_eps, s);
            if (st == PIE_HIP_ERR_UNSUPPORTED) {
                PIE_KERNEL(pie_hip_qkv_rope_kvwrite(qkv_, q_, k_rows_, v_rows_, w.q_norm, w.k_norm, rope_tab_,
                                                    iota_slots_, N, hq, hk, d, pairing, m.rms_eps, s));
                PIE_KERNEL(pie_hip_kv_write_quant(kv_format_, k_rows_, v_rows_, slots, k_pool_[l], v_pool_[l],
                                                  ksc, vsc, N, hk, d, page_size_, s));
            } else {
                PIE_KERNEL(st);
            }
        } else {
            // decode rows of llama-type layers: rotation and KV write ride in the projection
            // (a hidden size past the GEMV's staged-activation limit takes the general route)
            int fused_st = PIE_HIP_ERR_UNSUPPORTED;
            if (N <= 4 && fused_rope && !w.q_norm) {
                fused_st = pie_hip_qkv_rope_fused(fmt_code(w.wqkv.kind), x_, w.attn_norm, m.rms_eps, w.wqkv.data,
                                                  w.wqkv.scale, w.wqkv.scale_bf16 ? 1 : 0, w.wqkv.group, N, H,
                                                  rope_tab_, slots, q_, k_pool_[l], v_pool_[l], hq, hk, d,
                                                  pairing, s);
                if (fused_st != PIE_HIP_OK && fused_st != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(fused_st);
            }
            if (fused_st != PIE_HIP_OK) {
            // a decode batch of llama-type layers on the skinny GEMM: rotation and KV write ride
            // in its epilogue too (one launch less per layer)
            bool done = false;
            const int tuned_qkv = N <= 128 ? w.wqkv.tuned[N] : -1;
            if (fused_rope && !w.q_norm && w.wqkv.data_tiled &&
                (tuned_qkv >= 0 ? tuned_qkv <= 1 : pick_gemm(w.wqkv, N, gemm_ws_bytes_) == GemmPath::Skinny)) {
                PIE_KERNEL(pie_hip_rmsnorm(x_, w.attn_norm, xn_, N, H, m.rms_eps, s));
                const int st = pie_hip_qkv_rope_skinny_tiled(
                    fmt_code(w.wqkv.kind), xn_, w.wqkv.data_tiled,
                    w.wqkv.scale_tiled ? w.wqkv.scale_tiled : w.wqkv.scale, w.wqkv.scale_bf16 ? 1 : 0,
                    w.wqkv.group, N, H, rope_tab_, slots, q_, k_pool_[l], v_pool_[l], hq, hk, d, pairing, s);
                if (st == PIE_HIP_OK) done = true;
                else if (st != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(st);
            }
            if (!done) {
                linear_fused(w.wqkv, prenormed ? xn_ : x_, prenormed ? nullptr : w.attn_norm, m.rms_eps, qkv_, N, 0, 0,
                             xn_, gemm_ws_, gemm_ws_bytes_, s);
                PIE_KERNEL(pie_hip_qkv_rope_kvwrite(qkv_, q_, k_pool_[l], v_pool_[l], w.q_norm, w.k_norm,
                                                    rope_tab_, slots, N, hq, hk, d, pairing, m.rms_eps, s));
            }
            }
        }
        // 4-bit blocks: the pages this batch reads become bf16 in the shared pool pair, which the
        // bf16 attention kernels then read under the same page ids
        const bool fp4 = kv_format_ == PIE_HIP_KV_FP4_BLOCK;
        if (fp4)
            PIE_KERNEL(pie_hip_kv_dequant_pages(kv_format_, k_pool_[l], v_pool_[l], ksc, vsc, kv_shadow_k_,
                                                kv_shadow_v_, pages, n_page_refs_, hk, d, page_size_, s));
        const uint16_t* kat = fp4 ? kv_shadow_k_ : k_pool_[l];
        const uint16_t* vat = fp4 ? kv_shadow_v_ : v_pool_[l];
        const bool kvq_attn = kvq && !fp4;
        // One or two decode rows whose output projection runs the GEMV: the attention stops at its
        // splits' partial results and the projection merges them while its first weights travel —
        // one launch less per layer, but EVERY block of the projection reads all the partial results,
        // so only where those are few: measured on the 1B shape (32 heads of 64, four splits, 32 KB)
        // 0.578 -> 0.560 ms per step and on the 8B shape with four splits (64 KB, contexts below 512)
        // 1.589 -> 1.553; with eight splits (128 KB) the projection grows from 4.7 to 8.8 us, more than
        // the merge launch it saves (1.580 -> 1.601).  ([runtime] attn_merge_proj = false
        // or PIE_ATTN_MERGE_PROJ=0 keeps the separate merge.)
        bool merged_into_wo = false;
        if (N <= 2 && n_tiles_ == 0 && !masked_ && cfg_.runtime.attn_merge_proj) {
            static const bool merge_on = [] { const char* e = getenv("PIE_ATTN_MERGE_PROJ"); return !e || atoi(e) != 0; }();
            int ups = 0, ns = 1;
            if (merge_on && routes_to_gemv(w.wo, N, false, gemm_ws_bytes_) &&
                pie_hip_attn_decode_plan(N, hk, max_kv_len, &ups, &ns) == PIE_HIP_OK && ns >= 2 &&
                static_cast<size_t>(N) * hq * ns * d * sizeof(float) <= kMergeProjMaxBytes &&
                pie_hip_linear_attn_merge_supported(fmt_code(w.wo.kind), N, ns, hq, d, w.wo.group)) {
                PIE_KERNEL(pie_hip_attn_rows_paged_partials(kvq_attn ? kv_format_ : PIE_HIP_KV_BF16, q_,
                                                            kvq_attn ? static_cast<const void*>(k_pool_[l]) : kat,
                                                            kvq_attn ? static_cast<const void*>(v_pool_[l]) : vat,
                                                            kvq_attn ? ksc : nullptr, kvq_attn ? vsc : nullptr, pages,
                                                            row_begin, row_len, N, hq, hk, d, page_size_, -1.f,
                                                            max_kv_len, attn_ws_, attn_ws_bytes_, s));
                PIE_KERNEL(pie_hip_linear_attn_merge(fmt_code(w.wo.kind), attn_ws_, ns, ups, row_len, hq, d, w.wo.data,
                                                     w.wo.scale, w.wo.scale_bf16 ? 1 : 0, w.wo.group, x_, N, w.wo.N, 1,
                                                     s));
                merged_into_wo = true;
            }
        }
        if (merged_into_wo) {
        } else if (kvq_attn && n_tiles_ > 0 && !masked_) {
            const auto* td = static_cast<const int32_t*>(tile_in_dev_.ptr);
            PIE_KERNEL(pie_hip_attn_prefill_tiles_kvq(kv_format_, q_, k_pool_[l], v_pool_[l], ksc, vsc, attn_,
                                                      pages, row_begin, row_len, td, td + n_tiles_, n_tiles_,
                                                      tile_rows_, hq, hk, d, page_size_, -1.f, s));
        } else if (kvq_attn && masked_) {
            PIE_KERNEL(pie_hip_attn_rows_paged_kvq_masked(
                kv_format_, q_, k_pool_[l], v_pool_[l], ksc, vsc, attn_, nullptr, pages, row_begin, row_len,
                static_cast<const uint16_t*>(mask_bitmap_.ptr), mask_stride_, N, hq, hk, d, page_size_, -1.f,
                max_kv_len, attn_ws_, attn_ws_bytes_, s));
        } else if (kvq_attn) {
            PIE_KERNEL((uniform_rows_ ? pie_hip_attn_rows_paged_kvq_uniform : pie_hip_attn_rows_paged_kvq)(
                kv_format_, q_, k_pool_[l], v_pool_[l], ksc, vsc, attn_, nullptr, pages, row_begin, row_len, N, hq,
                hk, d, page_size_, -1.f, max_kv_len, attn_ws_, attn_ws_bytes_, s));
        } else if (n_tiles_ > 0) {
            const auto* td = static_cast<const int32_t*>(tile_in_dev_.ptr);
            PIE_KERNEL(pie_hip_attn_prefill_tiles(q_, kat, vat, attn_, pages, row_begin,
                                                  row_len, td, td + n_tiles_, n_tiles_, tile_rows_, hq,
                                                  hk, d, page_size_, -1.f, s));
        } else if (masked_) {
            PIE_KERNEL(pie_hip_attn_rows_paged_masked(
                q_, kat, vat, attn_, nullptr, pages, row_begin, row_len,
                static_cast<const uint16_t*>(mask_bitmap_.ptr), mask_stride_, N, hq, hk, d, page_size_,
                -1.f, max_kv_len, attn_ws_, attn_ws_bytes_, s));
        } else if (uniform_rows_) {
            PIE_KERNEL(pie_hip_attn_rows_paged_kvq_uniform(PIE_HIP_KV_BF16, q_, kat, vat, nullptr, nullptr, attn_,
                                                           nullptr, pages, row_begin, row_len, N, hq, hk, d,
                                                           page_size_, -1.f, max_kv_len, attn_ws_, attn_ws_bytes_, s));
        } else {
            PIE_KERNEL(pie_hip_attn_rows_paged(q_, kat, vat, attn_, nullptr, pages,
                                               row_begin, row_len, N, hq, hk, d, page_size_, -1.f,
                                               max_kv_len, attn_ws_, attn_ws_bytes_, s));
        }
        if (!merged_into_wo)
        linear_fused(w.wo, attn_, nullptr, m.rms_eps, x_, N, 1, 0, xn_, gemm_ws_, gemm_ws_bytes_, s);
        if (model_.is_moe()) {
            // the next layer's rows come normalised when that layer runs the plain projection
            // (q/k norm: no fused RoPE epilogue) on more than the GEMV's four rows
            const bool next_plain = l + 1 < m.layers && N > 4 && model_.layers[l + 1].q_norm != nullptr;
            moe_block(w, N, next_plain ? model_.layers[l + 1].attn_norm : nullptr, s);
            continue;
        }
        linear_fused(w.wgu, x_, w.ffn_norm, m.rms_eps, act_, N, 0, 1, xn_, gemm_ws_, gemm_ws_bytes_, s);
        linear_fused(w.wdown, act_, nullptr, m.rms_eps, x_, N, 1, 0, xn_, gemm_ws_, gemm_ws_bytes_, s);
    }
    // lm_head only on the sampled rows (driver/portable/src/graph_qwen3.cpp:867-896)
    const int cap = static_cast<int>(std::min<size_t>(max_tokens_, 2 * static_cast<size_t>(cfg_.batching.max_forward_requests)));
    for (int s0 = 0; s0 < S; s0 += cap) {
        const int n = std::min(cap, S - s0);
        PIE_KERNEL(pie_hip_embed(sample_rows + s0, x_, xs_, n, H, N, s));  // row gather
        Linear head;
        head.kind = Quant::Bf16;
        head.data = model_.lm_head;
        head.N = m.vocab;
        head.K = H;
        // up to four rows: the GEMV keeps (largest value, row) pairs while it stores the logits
        const int fused = n <= 4 ? pie_hip_lm_head_argmax(xs_, model_.final_norm, m.rms_eps, model_.lm_head, logits_,
                                                          out_tokens_ + s0, n, m.vocab, H, amax_ws_, amax_ws_bytes_, s)
                                 : PIE_HIP_ERR_UNSUPPORTED;
        if (fused == PIE_HIP_ERR_UNSUPPORTED) {
            linear_fused(head, xs_, model_.final_norm, m.rms_eps, logits_, n, 0, 0, xn_, gemm_ws_, gemm_ws_bytes_, s);
            PIE_KERNEL(pie_hip_argmax(logits_, out_tokens_ + s0, n, m.vocab, s));
        } else {
            PIE_KERNEL(fused);
        }
        if (samp_gather_in_body_) {   // more sampled rows than one chunk: keep each chunk's f32 rows
            const auto* in = static_cast<const unsigned char*>(samp_in_dev_.ptr);
            PIE_KERNEL(pie_hip_sample_gather_logits(
                logits_, nullptr, static_cast<float*>(samp_f32_.ptr) + static_cast<size_t>(s0) * m.vocab,
                samp_.n_bounds ? reinterpret_cast<const uint32_t*>(in + samp_.bounds) : nullptr,
                samp_.n_bounds ? reinterpret_cast<const int32_t*>(in + samp_.bounds_indptr) + s0 : nullptr,
                n, m.vocab, s));
        }
    }
}

void Executor::Growable::ensure(size_t bytes) {
    if (bytes <= cap) return;
    release();
    const size_t want = std::max<size_t>(bytes, 256);
    if (pinned) PIE_HIP_CHECK(hipHostMalloc(&ptr, want, hipHostMallocDefault));
    else PIE_HIP_CHECK(hipMalloc(&ptr, want));
    cap = want;
}

void Executor::Growable::release() {
    if (ptr) (void)(pinned ? hipHostFree(ptr) : hipFree(ptr));
    ptr = nullptr;
    cap = 0;
}

namespace {

// The reference's per-slot generator (Pcg32, driver/portable/src/sampler.cpp:31-57): PCG-XSH-RR
// 64/32, seeded in the canonical two steps on the default stream; a slot draws one uniform,
// the top 24 bits of the first output.
float pcg32_first_uniform(uint64_t seed) {
    const uint64_t inc = (0xda3e39cb94b95bdbULL << 1u) | 1u;
    uint64_t state = 0;
    state = state * 6364136223846793005ULL + inc;
    state += seed;
    state = state * 6364136223846793005ULL + inc;
    const uint64_t old = state;
    const uint32_t xorshifted = static_cast<uint32_t>(((old >> 18u) ^ old) >> 27u);
    const uint32_t rot = static_cast<uint32_t>(old >> 59u);
    const uint32_t r = (xorshifted >> rot) | (xorshifted << ((32u - rot) & 31u));
    return static_cast<float>(r >> 8) * (1.0f / 16777216.0f);
}

}  // namespace

// Prefill-shaped batches (every request brings at least 8 query rows, no custom masks) run
// their attention on the matrix cores: rows are cut into tiles of consecutive rows of one
// request.  Batches with single-row requests keep the per-row kernel, whose split-K spreads a
// long context over the machine.
void Executor::prepare_tiles(const BatchPlan& plan) {
    n_tiles_ = 0;
    const ModelConfig& m = model_.cfg();
    int cap = pie_hip_attn_prefill_tile_rows(m.q_heads, m.kv_heads);
    if (cap <= 0 || masked_ || page_size_ % 16 != 0 || (m.head_dim != 64 && m.head_dim != 128)) return;
    long long blocks = 0;
    for (int r = 0; r < plan.R; ++r) {
        const int n = plan.qo_indptr[r + 1] - plan.qo_indptr[r];
        if (n < 8) return;
        blocks += static_cast<long long>((n + cap - 1) / cap) * m.kv_heads;
    }
    // fewer than three full-size blocks per CU: halve the tiles (measured on a causal prompt of
    // 2048 tokens, 512 full-size blocks: 110 -> 100 us; of 3072 tokens, 768 blocks: 169 -> 179)
    if (blocks < 768) cap /= 2;
    tile_rows_ = cap;
    // Longest first: the kernel starts its blocks in tile order, and a long causal tile started
    // last would run on alone.
    std::vector<std::pair<int32_t, int32_t>> tiles;   // (first row, rows)
    for (int r = 0; r < plan.R; ++r)
        for (int t0 = plan.qo_indptr[r]; t0 < plan.qo_indptr[r + 1]; t0 += cap)
            tiles.emplace_back(t0, std::min(cap, plan.qo_indptr[r + 1] - t0));
    std::stable_sort(tiles.begin(), tiles.end(), [&](const auto& a, const auto& b) {
        return plan.row_kv_len[a.first + a.second - 1] > plan.row_kv_len[b.first + b.second - 1];
    });
    std::vector<int32_t> start, rows;
    for (const auto& tl : tiles) {
        start.push_back(tl.first);
        rows.push_back(tl.second);
    }
    const size_t n = start.size(), bytes = 8 * n;
    tile_in_host_.pinned = true;
    tile_in_host_.ensure(bytes);
    tile_in_dev_.ensure(bytes);
    auto* h = static_cast<int32_t*>(tile_in_host_.ptr);
    std::memcpy(h, start.data(), 4 * n);
    std::memcpy(h + n, rows.data(), 4 * n);
    PIE_HIP_CHECK(hipMemcpyAsync(tile_in_dev_.ptr, h, bytes, hipMemcpyHostToDevice, stream_));
    n_tiles_ = static_cast<int>(n);
}

// Custom attention masks: each row's BRLE runs become cumulative bounds, the device expands
// them into one visibility word per 16-token unit, and the layers' attention reads that.
void Executor::prepare_masks(const BatchPlan& plan) {
    const int N = plan.N;
    std::vector<int32_t> indptr(static_cast<size_t>(N) + 1, 0);
    std::vector<uint32_t> bounds;
    const bool user = static_cast<int>(plan.row_mask_runs.size()) == N;   // (absent: window only)
    for (int i = 0; i < N && user; ++i) {
        uint64_t acc = 0;
        for (uint32_t len : plan.row_mask_runs[i]) {
            acc = std::min<uint64_t>(acc + len, 0xFFFFFFFFull);
            bounds.push_back(static_cast<uint32_t>(acc));
        }
        indptr[i + 1] = static_cast<int32_t>(bounds.size());
    }
    if (!user) std::fill(indptr.begin(), indptr.end(), 0);
    const size_t off_bounds = align_up(4ull * (N + 1), 16);
    const size_t total = off_bounds + 4ull * std::max<size_t>(bounds.size(), 1);
    mask_in_host_.pinned = true;
    mask_in_host_.ensure(total);
    mask_in_dev_.ensure(total);
    mask_stride_ = std::max(1, (plan.max_kv_len + 15) / 16);
    mask_bitmap_.ensure(static_cast<size_t>(N) * mask_stride_ * sizeof(uint16_t));
    auto* h = static_cast<unsigned char*>(mask_in_host_.ptr);
    std::memcpy(h, indptr.data(), 4ull * (N + 1));
    if (!bounds.empty()) std::memcpy(h + off_bounds, bounds.data(), 4ull * bounds.size());
    PIE_HIP_CHECK(hipMemcpyAsync(mask_in_dev_.ptr, h, total, hipMemcpyHostToDevice, stream_));
    const auto* dv = static_cast<const unsigned char*>(mask_in_dev_.ptr);
    const Inputs lay = input_layout(N, static_cast<int>(plan.sample_rows.size()));   // this forward's staging layout
    const auto* row_len = reinterpret_cast<const int32_t*>(in_dev_ + lay.off_row_len);
    PIE_KERNEL(pie_hip_attn_mask_bitmap(reinterpret_cast<const uint32_t*>(dv + off_bounds),
                                        reinterpret_cast<const int32_t*>(dv), row_len,
                                        std::max(0, model_.cfg().sliding_window),
                                        static_cast<uint16_t*>(mask_bitmap_.ptr), N, mask_stride_, stream_));
}

// Host half of the sampler stage: per-slot parameter arrays, uniforms, payload ranges, BRLE
// bounds — staged in pinned memory and sent to the device ahead of the forward body.
void Executor::prepare_samplers(const BatchPlan& plan) {
    const int S = static_cast<int>(plan.sample_rows.size());
    const int V = cfg_.model.vocab;
    if (static_cast<int>(plan.slot_samplers.size()) != S)
        throw std::runtime_error("executor: one sampler per sampling slot expected");
    std::vector<int32_t> out_indptr(static_cast<size_t>(S) + 1, 0), bounds_indptr(static_cast<size_t>(S) + 1, 0);
    std::vector<uint32_t> bounds;
    for (int r = 0, s = 0; r < plan.R; ++r) {
        const auto& runs = plan.logit_mask_runs[r];
        for (; s < plan.sample_indptr[r + 1]; ++s) {
            uint64_t acc = 0;
            for (uint32_t len : runs) {
                acc = std::min<uint64_t>(acc + len, 0xFFFFFFFFull);
                bounds.push_back(static_cast<uint32_t>(acc));
            }
            bounds_indptr[s + 1] = static_cast<int32_t>(bounds.size());
        }
    }
    for (int s = 0; s < S; ++s) {
        const SlotSampler& sp = plan.slot_samplers[s];
        int n = 0;
        switch (sp.kind) {
            case PIE_SAMPLER_KIND_MULTINOMIAL: case PIE_SAMPLER_KIND_TOP_K: case PIE_SAMPLER_KIND_TOP_P:
            case PIE_SAMPLER_KIND_MIN_P: case PIE_SAMPLER_KIND_TOP_K_TOP_P: case PIE_SAMPLER_KIND_RAW_LOGITS:
                break;
            case PIE_SAMPLER_KIND_DIST:
                n = sp.top_k > 0 ? static_cast<int>(std::min<uint32_t>(sp.top_k, static_cast<uint32_t>(V))) : V;
                break;
            case PIE_SAMPLER_KIND_LOGPROB: case PIE_SAMPLER_KIND_LOGPROBS:
                n = static_cast<int>(sp.labels_end - sp.labels_begin);
                if (n == 0) throw std::runtime_error("sampler: Logprob slot has no labels");
                for (uint32_t i = sp.labels_begin; i < sp.labels_end; ++i)
                    if (plan.label_ids[i] >= static_cast<uint32_t>(V))
                        throw std::runtime_error("sampler: Logprob label id out of vocab");
                break;
            case PIE_SAMPLER_KIND_ENTROPY: n = 1; break;
            // the response has no field for it: the slot is accepted and yields nothing, as the
            // portable executor's per-slot switch leaves it (executor.cpp:1367-1392, default arm)
            case PIE_SAMPLER_KIND_EMBEDDING: break;
            default:
                throw std::runtime_error("sampler: unknown type " + std::to_string(static_cast<int>(sp.kind)));
        }
        out_indptr[s + 1] = out_indptr[s] + n;
    }
    const int payload = out_indptr[S];
    SampLayout L{};
    L.slots = S;
    L.payload = payload;
    L.n_bounds = static_cast<int>(bounds.size());
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes, 16); return at; };
    L.kind = take(4ull * S);
    L.temperature = take(4ull * S);
    L.top_k = take(4ull * S);
    L.top_p = take(4ull * S);
    L.min_p = take(4ull * S);
    L.uniform = take(4ull * S);
    L.out_indptr = take(4ull * (S + 1));
    L.labels = take(4ull * std::max(payload, 1));
    L.bounds_indptr = take(4ull * (S + 1));
    L.bounds = take(4ull * std::max<size_t>(bounds.size(), 1));
    L.total = o;
    o = 0;
    L.o_tokens = take(4ull * S);
    L.o_values = take(4ull * std::max(payload, 1));
    L.o_ids = take(4ull * std::max(payload, 1));
    L.o_total = o;
    samp_ = L;

    samp_in_host_.pinned = true;
    samp_out_host_.pinned = true;
    samp_in_host_.ensure(L.total);
    samp_in_dev_.ensure(L.total);
    samp_out_dev_.ensure(L.o_total);
    samp_out_host_.ensure(L.o_total);
    samp_f32_.ensure(static_cast<size_t>(S) * V * sizeof(float));
    samp_ws_.ensure(pie_hip_sample_workspace_bytes(S, V));

    auto* h = static_cast<unsigned char*>(samp_in_host_.ptr);
    std::memset(h, 0, L.total);
    auto* kind = reinterpret_cast<int32_t*>(h + L.kind);
    auto* temp = reinterpret_cast<float*>(h + L.temperature);
    auto* top_k = reinterpret_cast<uint32_t*>(h + L.top_k);
    auto* top_p = reinterpret_cast<float*>(h + L.top_p);
    auto* min_p = reinterpret_cast<float*>(h + L.min_p);
    auto* uni = reinterpret_cast<float*>(h + L.uniform);
    auto* labels = reinterpret_cast<uint32_t*>(h + L.labels);
    for (int s = 0; s < S; ++s) {
        const SlotSampler& sp = plan.slot_samplers[s];
        kind[s] = sp.kind;
        temp[s] = sp.temperature;
        top_k[s] = sp.top_k;
        top_p[s] = sp.top_p;
        min_p[s] = sp.min_p;
        // no caller seed: a process-wide counter, as the reference's default_rng_seed (:62-65)
        const uint64_t seed = sp.seed != 0 ? sp.seed : (0x9E3779B97F4A7C15ULL ^ unseeded_draws_++);
        uni[s] = pcg32_first_uniform(seed);
        for (uint32_t i = sp.labels_begin; i < sp.labels_end; ++i)
            labels[out_indptr[s] + (i - sp.labels_begin)] = plan.label_ids[i];
    }
    std::memcpy(h + L.out_indptr, out_indptr.data(), 4ull * (S + 1));
    std::memcpy(h + L.bounds_indptr, bounds_indptr.data(), 4ull * (S + 1));
    if (!bounds.empty()) std::memcpy(h + L.bounds, bounds.data(), 4ull * bounds.size());
    PIE_HIP_CHECK(hipMemcpyAsync(samp_in_dev_.ptr, h, L.total, hipMemcpyHostToDevice, stream_));
}

// Device half, queued behind the forward body: f32 rows (+ masks) unless the body gathered them
// chunk by chunk, one sampler block per slot, results into pinned memory.
void Executor::enqueue_samplers() {
    const int S = samp_.slots, V = cfg_.model.vocab;
    const auto* in = static_cast<const unsigned char*>(samp_in_dev_.ptr);
    auto* od = static_cast<unsigned char*>(samp_out_dev_.ptr);
    float* f32 = static_cast<float*>(samp_f32_.ptr);
    if (!samp_gather_in_body_) {
        PIE_KERNEL(pie_hip_sample_gather_logits(
            logits_, nullptr, f32, samp_.n_bounds ? reinterpret_cast<const uint32_t*>(in + samp_.bounds) : nullptr,
            samp_.n_bounds ? reinterpret_cast<const int32_t*>(in + samp_.bounds_indptr) : nullptr, S, V, stream_));
    }
    PIE_HIP_CHECK(hipMemsetAsync(od, 0, samp_.o_total, stream_));   // eager stage, never captured
    PIE_KERNEL(pie_hip_sample(
        f32, reinterpret_cast<const int32_t*>(in + samp_.kind), reinterpret_cast<const float*>(in + samp_.temperature),
        reinterpret_cast<const uint32_t*>(in + samp_.top_k), reinterpret_cast<const float*>(in + samp_.top_p),
        reinterpret_cast<const float*>(in + samp_.min_p), reinterpret_cast<const float*>(in + samp_.uniform),
        reinterpret_cast<const int32_t*>(in + samp_.out_indptr), reinterpret_cast<const uint32_t*>(in + samp_.labels),
        reinterpret_cast<uint32_t*>(od + samp_.o_tokens), reinterpret_cast<float*>(od + samp_.o_values),
        reinterpret_cast<uint32_t*>(od + samp_.o_ids), samp_ws_.ptr, samp_ws_.cap, S, V, stream_));
    PIE_HIP_CHECK(hipMemcpyAsync(samp_out_host_.ptr, od, samp_.o_total, hipMemcpyDeviceToHost, stream_));
}

// After the stream has drained: results out of pinned memory, RawLogits rows copied back.
void Executor::collect_samplers(const BatchPlan& plan, SampleOutputs& out) {
    const int S = samp_.slots, V = cfg_.model.vocab;
    const float* f32 = static_cast<const float*>(samp_f32_.ptr);
    const auto* oh = static_cast<const unsigned char*>(samp_out_host_.ptr);
    out.raw_logits.clear();
    size_t n_raw = 0;
    for (const SlotSampler& sp : plan.slot_samplers) n_raw += sp.kind == PIE_SAMPLER_KIND_RAW_LOGITS;
    out.raw_logits.resize(n_raw * static_cast<size_t>(V));
    size_t at = 0;
    for (int s = 0; s < S; ++s)
        if (plan.slot_samplers[s].kind == PIE_SAMPLER_KIND_RAW_LOGITS) {
            PIE_HIP_CHECK(hipMemcpy(out.raw_logits.data() + at, f32 + static_cast<size_t>(s) * V,
                                    static_cast<size_t>(V) * sizeof(float), hipMemcpyDeviceToHost));
            at += V;
        }
    const auto* tok = reinterpret_cast<const uint32_t*>(oh + samp_.o_tokens);
    out.tokens.assign(tok, tok + S);
    const auto* val = reinterpret_cast<const float*>(oh + samp_.o_values);
    out.values.assign(val, val + samp_.payload);
    const auto* ids = reinterpret_cast<const uint32_t*>(oh + samp_.o_ids);
    out.ids.assign(ids, ids + samp_.payload);
    const auto* ip = reinterpret_cast<const int32_t*>(static_cast<const unsigned char*>(samp_in_host_.ptr) + samp_.out_indptr);
    out.out_indptr.assign(ip, ip + S + 1);
}

// Captured graphs hold the old buffer's address: they are dropped with it.
void Executor::grow_outputs(size_t slots) {
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
    for (auto& kv : graphs_) (void)hipGraphExecDestroy(kv.second);
    graphs_.clear();
    const size_t cap = std::max(slots, 2 * out_cap_);
    (void)hipFree(out_tokens_);
    out_tokens_ = nullptr;
    (void)hipHostFree(out_host_);
    out_host_ = nullptr;
    out_cap_ = 0;
    out_tokens_ = dmalloc<uint32_t>(cap);
    PIE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&out_host_), cap * 4, hipHostMallocDefault));
    out_cap_ = cap;
}

void Executor::forward(const BatchPlan& plan, std::vector<uint32_t>& tokens_out,
                       ForwardTimings* t, SampleOutputs* samples) {
    const int N = plan.N, S = static_cast<int>(plan.sample_rows.size());
    if (N <= 0) throw std::runtime_error("executor: empty plan");
    if (N > max_tokens_) throw std::runtime_error("executor: batch exceeds max_forward_tokens");
    if (static_cast<int>(plan.page_indices.size()) > max_page_refs_)
        throw std::runtime_error("executor: batch exceeds the page reference capacity");
    // A request may put several samplers on one row, so the sampling slots can outnumber the
    // rows: the token buffers follow the slot count.
    if (static_cast<size_t>(S) > out_cap_) grow_outputs(static_cast<size_t>(S));

    auto t0 = clk::now();
    const Inputs in = input_layout(N, S);
    const size_t used = in.off_pages + plan.page_indices.size() * 4;
    if (used > in_.total) throw std::runtime_error("executor: staged inputs exceed their buffer");
    std::memcpy(in_host_ + in.off_tokens, plan.tokens.data(), static_cast<size_t>(N) * 4);
    std::memcpy(in_host_ + in.off_positions, plan.positions.data(), static_cast<size_t>(N) * 4);
    std::memcpy(in_host_ + in.off_slots, plan.kv_slots.data(), static_cast<size_t>(N) * 8);
    std::memcpy(in_host_ + in.off_row_begin, plan.row_page_begin.data(), static_cast<size_t>(N) * 4);
    std::memcpy(in_host_ + in.off_row_len, plan.row_kv_len.data(), static_cast<size_t>(N) * 4);
    if (S) std::memcpy(in_host_ + in.off_sample_rows, plan.sample_rows.data(), static_cast<size_t>(S) * 4);
    std::memcpy(in_host_ + in.off_pages, plan.page_indices.data(), plan.page_indices.size() * 4);
    PIE_HIP_CHECK(hipMemcpyAsync(in_dev_, in_host_, used, hipMemcpyHostToDevice, stream_));
    // a sliding window (driver/portable/src/plan.cpp:60-70: keys below p - W + 1 are hidden)
    // matters once some context is longer than the window; such batches take the masked kernels
    const int window = model_.cfg().sliding_window;
    masked_ = plan.has_user_masks || (window > 0 && plan.max_kv_len > window);
    if (masked_) prepare_masks(plan);
    prepare_tiles(plan);
    const bool sampling = !plan.all_greedy && S > 0;
    const int chunk = static_cast<int>(std::min<size_t>(max_tokens_, 2 * static_cast<size_t>(cfg_.batching.max_forward_requests)));
    samp_gather_in_body_ = false;
    if (sampling) {
        if (!samples) throw std::runtime_error("executor: a sampling plan needs a SampleOutputs");
        prepare_samplers(plan);
        samp_gather_in_body_ = S > chunk;   // logits_ keeps one chunk of rows only
    }
    if (t) t->h2d_us = us_since(t0);

    t0 = clk::now();
    n_page_refs_ = static_cast<int>(plan.page_indices.size());
    // A decode batch whose longest context is within an eighth of the mean: the attention launch
    // may then plan one round of equally long blocks (a graph is captured per answer).
    uniform_rows_ = false;
    if (plan.pure_decode && N >= 2 && !masked_) {
        long long total = 0;
        int longest = 0;
        for (int i = 0; i < N; ++i) {
            total += plan.row_kv_len[i];
            longest = std::max(longest, plan.row_kv_len[i]);
        }
        uniform_rows_ = 8LL * longest * N <= 9 * total;
    }
    // (4-bit blocks: the page expansion's extent changes from step to step, so no graph)
    const bool use_graph = cfg_.runtime.use_graphs && plan.pure_decode && !samp_gather_in_body_ && !masked_ &&
                           kv_format_ != PIE_HIP_KV_FP4_BLOCK;
    if (use_graph) {
        // The split grid depends on the context bound only through 512-token buckets.
        const int bucket = (plan.max_kv_len + 511) / 512 * 512;
        const auto key = std::make_tuple(N, S, bucket, uniform_rows_ ? 1 : 0);
        auto it = graphs_.find(key);
        if (it == graphs_.end()) {
            hipGraph_t graph = nullptr;
            PIE_HIP_CHECK(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal));
            try {
                body(N, S, bucket);
            } catch (...) {
                (void)hipStreamEndCapture(stream_, &graph);
                if (graph) (void)hipGraphDestroy(graph);
                throw;
            }
            PIE_HIP_CHECK(hipStreamEndCapture(stream_, &graph));
            hipGraphExec_t exec = nullptr;
            PIE_HIP_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
            PIE_HIP_CHECK(hipGraphDestroy(graph));
            it = graphs_.emplace(key, exec).first;
        }
        PIE_HIP_CHECK(hipGraphLaunch(it->second, stream_));
    } else {
        body(N, S, plan.max_kv_len);
    }
    if (S) PIE_HIP_CHECK(hipMemcpyAsync(out_host_, out_tokens_, static_cast<size_t>(S) * 4,
                                        hipMemcpyDeviceToHost, stream_));
    if (sampling) enqueue_samplers();
    if (t) t->launch_us = us_since(t0);

    t0 = clk::now();
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
    if (t) t->sync_us = us_since(t0);
    tokens_out.assign(out_host_, out_host_ + S);
    if (sampling) {
        collect_samplers(plan, *samples);
        tokens_out = samples->tokens;
    }
    const int cap = static_cast<int>(std::min<size_t>(max_tokens_, 2 * static_cast<size_t>(cfg_.batching.max_forward_requests)));
    last_logit_rows_ = S == 0 ? 0 : ((S - 1) % cap) + 1;
}

// A swap-pool slot holds a page's K (or V) bytes followed by its fp32 scales (scaled formats).
void Executor::copy_pages_d2h(const uint32_t* dev_srcs, const uint32_t* host_dsts, size_t n) {
    const size_t pb = page_bytes(), sb = scale_page_bytes();
    for (size_t i = 0; i < n; ++i)
        for (size_t l = 0; l < k_pool_.size(); ++l)
            for (int kv = 0; kv < 2; ++kv) {
                unsigned char* dst = swap_slot(static_cast<int>(l), kv, host_dsts[i]);
                const auto* pool = reinterpret_cast<const unsigned char*>(kv ? v_pool_[l] : k_pool_[l]);
                PIE_HIP_CHECK(hipMemcpyAsync(dst, pool + static_cast<size_t>(dev_srcs[i]) * pb, pb,
                                             hipMemcpyDeviceToHost, stream_));
                if (sb) {
                    const auto* sc = reinterpret_cast<const unsigned char*>(kv ? v_scale_pool_[l] : k_scale_pool_[l]);
                    PIE_HIP_CHECK(hipMemcpyAsync(dst + pb, sc + static_cast<size_t>(dev_srcs[i]) * sb, sb,
                                                 hipMemcpyDeviceToHost, stream_));
                }
            }
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
}

void Executor::copy_pages_h2d(const uint32_t* host_srcs, const uint32_t* dev_dsts, size_t n) {
    const size_t pb = page_bytes(), sb = scale_page_bytes();
    for (size_t i = 0; i < n; ++i)
        for (size_t l = 0; l < k_pool_.size(); ++l)
            for (int kv = 0; kv < 2; ++kv) {
                const unsigned char* src = swap_slot(static_cast<int>(l), kv, host_srcs[i]);
                auto* pool = reinterpret_cast<unsigned char*>(kv ? v_pool_[l] : k_pool_[l]);
                PIE_HIP_CHECK(hipMemcpyAsync(pool + static_cast<size_t>(dev_dsts[i]) * pb, src, pb,
                                             hipMemcpyHostToDevice, stream_));
                if (sb) {
                    auto* sc = reinterpret_cast<unsigned char*>(kv ? v_scale_pool_[l] : k_scale_pool_[l]);
                    PIE_HIP_CHECK(hipMemcpyAsync(sc + static_cast<size_t>(dev_dsts[i]) * sb, src + pb, sb,
                                                 hipMemcpyHostToDevice, stream_));
                }
            }
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
}

void Executor::copy_pages_h2h(const uint32_t* srcs, const uint32_t* dsts, size_t n) {
    const size_t pb = page_bytes() + scale_page_bytes();
    for (size_t i = 0; i < n; ++i)
        for (size_t l = 0; l < k_pool_.size(); ++l)
            for (int kv = 0; kv < 2; ++kv)
                std::memmove(swap_slot(static_cast<int>(l), kv, dsts[i]),
                             swap_slot(static_cast<int>(l), kv, srcs[i]), pb);
}

void Executor::copy_pages_d2d(const uint32_t* srcs, const uint32_t* dsts, size_t n) {
    if (n == 0) return;
    if (n > copy_ids_cap_) {
        if (copy_ids_) (void)hipFree(copy_ids_);
        copy_ids_ = dmalloc<uint32_t>(2 * n);
        copy_ids_cap_ = n;
    }
    PIE_HIP_CHECK(hipMemcpyAsync(copy_ids_, srcs, n * 4, hipMemcpyHostToDevice, stream_));
    PIE_HIP_CHECK(hipMemcpyAsync(copy_ids_ + copy_ids_cap_, dsts, n * 4, hipMemcpyHostToDevice, stream_));
    for (size_t i = 0; i < n; i += 65535) {
        const int cnt = static_cast<int>(std::min<size_t>(65535, n - i));
        for (size_t l = 0; l < k_pool_.size(); ++l) {
            PIE_KERNEL(pie_hip_copy_kv_pages(k_pool_[l], copy_ids_ + i, copy_ids_ + copy_ids_cap_ + i,
                                             cnt, page_bytes(), stream_));
            PIE_KERNEL(pie_hip_copy_kv_pages(v_pool_[l], copy_ids_ + i, copy_ids_ + copy_ids_cap_ + i,
                                             cnt, page_bytes(), stream_));
            if (scale_page_bytes()) {
                PIE_KERNEL(pie_hip_copy_kv_pages(k_scale_pool_[l], copy_ids_ + i, copy_ids_ + copy_ids_cap_ + i,
                                                 cnt, scale_page_bytes(), stream_));
                PIE_KERNEL(pie_hip_copy_kv_pages(v_scale_pool_[l], copy_ids_ + i, copy_ids_ + copy_ids_cap_ + i,
                                                 cnt, scale_page_bytes(), stream_));
            }
        }
    }
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
}

}  // namespace pie_hip_driver
