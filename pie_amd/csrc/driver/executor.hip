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

// Measured cost models (MI355X, microseconds): the skinny GEMM streams the weights once per 16
// rows at ~2.4 TB/s plus ~4 us per pass; the tiled GEMM walks K in 64-wide steps of ~1 us
// while its 128 x 128 tiles fit the machine (512 resident blocks), longer in proportion beyond.
bool tiled_gemm_is_faster(const Linear& w, int M) {
    if (w.K % 64 != 0 || M < 48) return false;
    const double skinny = ((M + 15) / 16) * (4.0 + static_cast<double>(w.data_bytes()) / 2.4e6);
    const double tiles = static_cast<double>((w.N + 127) / 128) * ((M + 127) / 128);
    const double gemm = (w.K / 64) * 0.97 * std::max(1.0, tiles / 512.0);
    return gemm < skinny;
}

// y = epilogue(rmsnorm?(act) · W^T) by the weight's storage format — the dispatcher role of
// gemm_act_x_w (driver/cuda/src/ops/gemm.cpp:1414-1583).  Up to four rows: the weight-streaming
// GEMV with the norm riding in its activation staging and SwiGLU in its epilogue.  More rows
// (norm as its own kernel into `norm_tmp`): the matrix-core skinny GEMM, which streams the
// weights once per 16 rows, or the tiled matrix-core GEMM where its cost model wins; shapes those do
// not take fall back to the GEMV path.
void linear_fused(const Linear& w, const uint16_t* act, const uint16_t* norm_w, float eps,
                  uint16_t* y, int M, int beta, int swiglu, uint16_t* norm_tmp, hipStream_t s) {
    const int fmt = fmt_code(w.kind);
    const int sbf = w.scale_bf16 ? 1 : 0;
    if (M > 4) {
        const uint16_t* a = act;
        if (norm_w) {
            PIE_KERNEL(pie_hip_rmsnorm(act, norm_w, norm_tmp, M, w.K, eps, s));
            a = norm_tmp;
        }
        if (tiled_gemm_is_faster(w, M)) {
            // compute-bound: the tiled GEMM (weights dequantised to bf16 while staged)
            const int sg = pie_hip_gemm_mfma(fmt, a, w.data, w.scale, sbf, w.group, y, M, w.N, w.K,
                                             beta, swiglu, s);
            if (sg == PIE_HIP_OK) return;
            if (sg != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(sg);
        }
        const int st = pie_hip_gemm_skinny(fmt, a, w.data, w.scale, sbf, w.group, y, M, w.N, w.K,
                                           beta, swiglu, s);
        if (st == PIE_HIP_OK) return;
        if (st != PIE_HIP_ERR_UNSUPPORTED) PIE_KERNEL(st);
        PIE_KERNEL(pie_hip_linear_fused(fmt, a, nullptr, eps, w.data, w.scale, sbf, w.group, y, M,
                                        w.N, w.K, beta, swiglu, s));
        return;
    }
    PIE_KERNEL(pie_hip_linear_fused(fmt, act, norm_w, eps, w.data, w.scale, sbf, w.group, y, M,
                                    w.N, w.K, beta, swiglu, s));
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
    alloc_kv();

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
    // Bound of the split-K partial buffers over every (rows, context) the planner can pick:
    // rows * splits <= 3072/hk + rows.
    attn_ws_bytes_ = (3072 / static_cast<size_t>(hk) + 1 + T) * hq * (d + 2) * sizeof(float);
    PIE_HIP_CHECK(hipMalloc(&attn_ws_, attn_ws_bytes_));

    in_ = input_layout(max_tokens_, max_tokens_);
    in_.total = align_up(in_.off_pages + static_cast<size_t>(max_page_refs_) * 4, 256);
    PIE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&in_host_), in_.total, hipHostMallocDefault));
    PIE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&in_dev_), in_.total));
    PIE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&out_host_), T * 4, hipHostMallocDefault));
}

Executor::~Executor() {
    if (stream_) (void)hipStreamSynchronize(stream_);
    for (auto& kv : graphs_) (void)hipGraphExecDestroy(kv.second);
    for (auto* p : k_pool_) (void)hipFree(p);
    for (auto* p : v_pool_) (void)hipFree(p);
    for (void* p : {static_cast<void*>(x_), static_cast<void*>(xn_), static_cast<void*>(qkv_),
                    static_cast<void*>(q_), static_cast<void*>(attn_), static_cast<void*>(gu_),
                    static_cast<void*>(act_), static_cast<void*>(xs_), static_cast<void*>(logits_),
                    static_cast<void*>(rope_tab_), static_cast<void*>(out_tokens_), attn_ws_,
                    static_cast<void*>(in_dev_), static_cast<void*>(copy_ids_),
                    static_cast<void*>(moe_y_), static_cast<void*>(moe_logits_),
                    static_cast<void*>(moe_idx_), static_cast<void*>(moe_w_),
                    static_cast<void*>(moe_offsets_), static_cast<void*>(moe_route_token_),
                    static_cast<void*>(moe_route_pos_)})
        if (p) (void)hipFree(p);
    if (in_host_) (void)hipHostFree(in_host_);
    if (out_host_) (void)hipHostFree(out_host_);
    if (stream_) (void)hipStreamDestroy(stream_);
}

size_t Executor::page_bytes() const {
    const ModelConfig& m = model_.cfg();
    return static_cast<size_t>(page_size_) * m.kv_heads * m.head_dim * 2;
}

// Allocate the pool; on out-of-memory halve the page count down to 64 pages
// (driver/portable/src/entry.cpp:327-348).
void Executor::alloc_kv() {
    const int L = model_.cfg().layers;
    for (;;) {
        const size_t bytes = page_bytes() * static_cast<size_t>(total_pages_);
        bool ok = true;
        for (int l = 0; l < L && ok; ++l) {
            void *k = nullptr, *v = nullptr;
            if (hipMalloc(&k, bytes) != hipSuccess) { ok = false; break; }
            k_pool_.push_back(static_cast<uint16_t*>(k));
            if (hipMalloc(&v, bytes) != hipSuccess) { ok = false; break; }
            v_pool_.push_back(static_cast<uint16_t*>(v));
        }
        if (ok) {
            // Pages start zeroed so slots no request has written hold finite values.
            for (int l = 0; l < L; ++l) {
                PIE_HIP_CHECK(hipMemsetAsync(k_pool_[l], 0, bytes, stream_));
                PIE_HIP_CHECK(hipMemsetAsync(v_pool_[l], 0, bytes, stream_));
            }
            PIE_HIP_CHECK(hipStreamSynchronize(stream_));
            return;
        }
        (void)hipGetLastError();
        for (auto* p : k_pool_) (void)hipFree(p);
        for (auto* p : v_pool_) (void)hipFree(p);
        k_pool_.clear();
        v_pool_.clear();
        if (total_pages_ <= 64) throw std::runtime_error("executor: cannot allocate the KV pool");
        total_pages_ = std::max(64, total_pages_ / 2);
    }
}

// x += sum_k w_k * down_e(swiglu(gate_up_e(norm(x)))) over each token's top-k experts
// (driver/portable/src/graph_common.cpp:237-345; kernel-by-kernel form
// driver/cuda/src/model/kimi_forward.cpp:662-714): norm, router GEMM, one routing kernel, two
// grouped expert GEMMs that read every touched expert once, one combine onto the residual.
void Executor::moe_block(const LayerWeights& w, int N, hipStream_t s) {
    const ModelConfig& m = model_.cfg();
    const int H = m.hidden, E = m.num_experts, K = m.top_k, Ie = m.expert_intermediate;
    const int fmt = fmt_code(w.wgu.kind);
    const int sbf = w.wgu.scale_bf16 ? 1 : 0;
    PIE_KERNEL(pie_hip_rmsnorm(x_, w.ffn_norm, xn_, N, H, m.rms_eps, s));
    linear_fused(w.router, xn_, nullptr, m.rms_eps, moe_logits_, N, 0, 0, nullptr, s);
    PIE_KERNEL(pie_hip_moe_route(moe_logits_, moe_idx_, moe_w_, moe_offsets_, moe_route_token_,
                                 moe_route_pos_, N, E, K, s));
    const int hint = std::max(1, std::min(N, 2 * ((N * K + E - 1) / E)));
    PIE_KERNEL(pie_hip_moe_grouped_gemm(fmt, xn_, moe_route_token_, moe_offsets_, E, hint, w.wgu.data,
                                        w.wgu.data_bytes() / E, w.wgu.scale, w.wgu.scale_bytes() / E,
                                        sbf, w.wgu.group, act_, 2 * Ie, H, 1, s));
    PIE_KERNEL(pie_hip_moe_grouped_gemm(fmt, act_, nullptr, moe_offsets_, E, hint, w.wdown.data,
                                        w.wdown.data_bytes() / E, w.wdown.scale,
                                        w.wdown.scale_bytes() / E, sbf, w.wdown.group, moe_y_, H, Ie,
                                        0, s));
    PIE_KERNEL(pie_hip_moe_combine(moe_y_, moe_route_pos_, moe_w_, x_, N, K, H, 1, s));
}

void Executor::body(int N, int S, int max_kv_len) {
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
    PIE_KERNEL(pie_hip_rope_table(positions, model_.inv_freq, rope_tab_, N, d, s));
    for (int l = 0; l < m.layers; ++l) {
        const LayerWeights& w = model_.layers[l];
        if (N <= 4 && m.rope_interleaved && !w.q_norm && (d & (d - 1)) == 0) {
            // decode rows of llama-type layers: rotation and KV write ride in the projection
            PIE_KERNEL(pie_hip_qkv_rope_fused(fmt_code(w.wqkv.kind), x_, w.attn_norm, m.rms_eps,
                                              w.wqkv.data, w.wqkv.scale, w.wqkv.scale_bf16 ? 1 : 0,
                                              w.wqkv.group, N, H, rope_tab_, slots, q_, k_pool_[l],
                                              v_pool_[l], hq, hk, d, s));
        } else {
            linear_fused(w.wqkv, x_, w.attn_norm, m.rms_eps, qkv_, N, 0, 0, xn_, s);
            PIE_KERNEL(pie_hip_qkv_rope_kvwrite(qkv_, q_, k_pool_[l], v_pool_[l], w.q_norm, w.k_norm,
                                                rope_tab_, slots, N, hq, hk, d, m.rope_interleaved,
                                                m.rms_eps, s));
        }
        PIE_KERNEL(pie_hip_attn_rows_paged(q_, k_pool_[l], v_pool_[l], attn_, nullptr, pages,
                                           row_begin, row_len, N, hq, hk, d, page_size_, -1.f,
                                           max_kv_len, attn_ws_, attn_ws_bytes_, s));
        linear_fused(w.wo, attn_, nullptr, m.rms_eps, x_, N, 1, 0, xn_, s);
        if (model_.is_moe()) {
            moe_block(w, N, s);
            continue;
        }
        linear_fused(w.wgu, x_, w.ffn_norm, m.rms_eps, act_, N, 0, 1, xn_, s);
        linear_fused(w.wdown, act_, nullptr, m.rms_eps, x_, N, 1, 0, xn_, s);
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
        linear_fused(head, xs_, model_.final_norm, m.rms_eps, logits_, n, 0, 0, xn_, s);
        PIE_KERNEL(pie_hip_argmax(logits_, out_tokens_ + s0, n, m.vocab, s));
    }
}

void Executor::forward(const BatchPlan& plan, std::vector<uint32_t>& tokens_out,
                       ForwardTimings* t) {
    const int N = plan.N, S = static_cast<int>(plan.sample_rows.size());
    if (N <= 0) throw std::runtime_error("executor: empty plan");
    if (N > max_tokens_) throw std::runtime_error("executor: batch exceeds max_forward_tokens");
    if (static_cast<int>(plan.page_indices.size()) > max_page_refs_)
        throw std::runtime_error("executor: batch exceeds the page reference capacity");

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
    if (t) t->h2d_us = us_since(t0);

    t0 = clk::now();
    const bool use_graph = cfg_.runtime.use_graphs && plan.pure_decode;
    if (use_graph) {
        // The split grid depends on the context bound only through 512-token buckets.
        const int bucket = (plan.max_kv_len + 511) / 512 * 512;
        const auto key = std::make_tuple(N, S, bucket);
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
    if (t) t->launch_us = us_since(t0);

    t0 = clk::now();
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
    if (t) t->sync_us = us_since(t0);
    tokens_out.assign(out_host_, out_host_ + S);
    const int cap = static_cast<int>(std::min<size_t>(max_tokens_, 2 * static_cast<size_t>(cfg_.batching.max_forward_requests)));
    last_logit_rows_ = S == 0 ? 0 : ((S - 1) % cap) + 1;
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
        }
    }
    PIE_HIP_CHECK(hipStreamSynchronize(stream_));
}

}  // namespace pie_hip_driver
