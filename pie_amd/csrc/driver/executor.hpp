// Forward-pass executor: owns the paged KV pool, the activation workspaces and the
// per-shape HIP graphs, and turns a BatchPlan into kernel launches.
//
// Op sequence per layer (bf16 activations, fp32 inside each op, one rounding per op —
// the rounding points of driver/cuda/src/model/llama_like.cpp:364-762; op order of
// driver/portable/src/graph_qwen3.cpp:225-829):
//   xn   = rmsnorm(x, attn_norm)
//   qkv  = xn · Wqkv^T                                  (weight-streaming GEMV)
//   q,K,V: optional qk-norm, RoPE, K/V written into their page slots
//   a    = paged attention(q, pages)                    (split-K over pages)
//   x    = x + a · Wo^T                                 (residual fused, one rounding)
//   xn   = rmsnorm(x, ffn_norm)
//   gu   = xn · Wgu^T ; h = silu(gate) * up ; x = x + h · Wdown^T
// tail: gather sampled rows -> final norm -> lm_head -> argmax (first index wins).
//
// Split into a host `prepare` (plan upload, outside any capture) and a device-only `body`
// that is captured into a HIP graph per (rows, sampled rows, context bucket) for pure decode,
// the prepare/body split of driver/cuda/src/executor/executor.hpp:42-75.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <tuple>
#include <vector>

#include "config.hpp"
#include "model.hpp"
#include "planner.hpp"

namespace pie_hip_driver {

struct ForwardTimings {
    uint32_t h2d_us = 0, launch_us = 0, sync_us = 0;
};

// What the non-greedy samplers of one forward pass produced, per sampling slot (slot order =
// BatchPlan::sample_rows).  Slot s's Distribution / Logprob(s) / Entropy payload is
// values / ids [out_indptr[s], out_indptr[s+1]); RawLogits slots own `vocab` floats each in
// raw_logits, in slot order.
struct SampleOutputs {
    std::vector<uint32_t> tokens;
    std::vector<float> values;
    std::vector<uint32_t> ids;
    std::vector<int32_t> out_indptr;
    std::vector<float> raw_logits;
};

class Executor {
  public:
    Executor(const DriverConfig& cfg, Model& model);
    ~Executor();
    Executor(const Executor&) = delete;
    Executor& operator=(const Executor&) = delete;

    // Runs one forward pass; greedy tokens for plan.sample_rows land in tokens_out.  A plan that
    // is not all-greedy also runs every slot's sampler on the device and fills `samples`
    // (required then); tokens_out then holds the samplers' tokens.
    void forward(const BatchPlan& plan, std::vector<uint32_t>& tokens_out, ForwardTimings* t,
                 SampleOutputs* samples = nullptr);

    // KV page copies inside the device pool (every layer, K and V).
    void copy_pages_d2d(const uint32_t* srcs, const uint32_t* dsts, size_t n);
    // Host swap pool (`[batching] cpu_pages` pinned pages per layer for K and for V,
    // driver/portable/src/host_swap_pool.cpp): device page -> host slot, back, host -> host.
    // Callers check the ids against total_pages() / cpu_pages() first.
    void copy_pages_d2h(const uint32_t* dev_srcs, const uint32_t* host_dsts, size_t n);
    void copy_pages_h2d(const uint32_t* host_srcs, const uint32_t* dev_dsts, size_t n);
    void copy_pages_h2h(const uint32_t* srcs, const uint32_t* dsts, size_t n);
    int cpu_pages() const { return cpu_pages_; }

    int total_pages() const { return total_pages_; }
    int page_size() const { return page_size_; }
    size_t page_bytes() const;         // K (or V) bytes of one page in the pool's storage format
    size_t scale_page_bytes() const;   // fp32 side scales of one page (0 without them)
    int kv_format() const { return kv_format_; }
    hipStream_t stream() const { return stream_; }
    int graphs_cached() const { return static_cast<int>(graphs_.size()); }
    // Logits [rows, vocab] bf16 of the last forward's (last chunk of) sampled rows; debug/test hook.
    const uint16_t* last_logits() const { return logits_; }
    // Row 0 of the last layer's intermediates after a forward (debug/test hook): "x" residual
    // stream, "q" rotated queries, "attn" attention output, "act" SwiGLU output.
    const uint16_t* debug_buffer(const std::string& what) const {
        if (what == "x") return x_;
        if (what == "q") return q_;
        if (what == "attn") return attn_;
        if (what == "act") return act_;
        return nullptr;
    }
    int last_logit_rows() const { return last_logit_rows_; }
    const uint16_t* kv_pool(bool k, int layer) const {
        if (layer < 0 || layer >= static_cast<int>(k_pool_.size())) return nullptr;
        return k ? k_pool_[layer] : v_pool_[layer];
    }

  private:
    void body(int N, int S, int max_kv_len);
    void grow_outputs(size_t slots);
    void prepare_masks(const BatchPlan& plan);
    void prepare_tiles(const BatchPlan& plan);
    void prepare_samplers(const BatchPlan& plan);
    void enqueue_samplers();
    void collect_samplers(const BatchPlan& plan, SampleOutputs& out);
    void moe_block(const LayerWeights& w, int N, const uint16_t* next_norm, hipStream_t s);
    static constexpr int kFusedRouteRows = 256;   // batches up to this size take pie_hip_moe_norm_route
    static constexpr size_t kMergeProjMaxBytes = 64 * 1024;   // partial results a merging output projection reads per block
    bool xn_holds_next_norm_ = false;             // (while a forward is being enqueued) xn_ = the coming layer's normalised rows
    void alloc_kv();
    void tune_linears();

    DriverConfig cfg_;
    Model& model_;
    hipStream_t stream_ = nullptr;
    int total_pages_ = 0, page_size_ = 0, max_tokens_ = 0, max_page_refs_ = 0;

    std::vector<uint16_t*> k_pool_, v_pool_;  // per layer [pages, ps, hk, d] (bf16 or one byte per element)
    int kv_format_ = 0;                        // PIE_HIP_KV_*
    std::vector<float*> k_scale_pool_, v_scale_pool_;   // per layer [pages, hk, ps] ([pages, hk, ps, d/16] for 4-bit blocks)
    // 4-bit block format: one bf16 pool pair of the whole pool's geometry, shared by the layers;
    // the pages a batch reads are expanded into it before each layer's attention
    uint16_t *kv_shadow_k_ = nullptr, *kv_shadow_v_ = nullptr;
    int n_page_refs_ = 0;                      // page list entries of the forward in flight
    uint16_t *k_rows_ = nullptr, *v_rows_ = nullptr;     // this step's rotated K / V rows before quantisation
    int64_t* iota_slots_ = nullptr;                      // 0, 1, 2, ...: row t of k_rows_ is "slot" t
    unsigned char* swap_pool_ = nullptr;       // pinned: [layer][K|V][cpu_pages] pages (+ their scales)
    int cpu_pages_ = 0;
    unsigned char* swap_slot(int layer, int kv, uint32_t slot) const {
        return swap_pool_ + ((static_cast<size_t>(layer) * 2 + kv) * cpu_pages_ + slot) *
                                (page_bytes() + scale_page_bytes());
    }
    // activations
    uint16_t *x_ = nullptr, *xn_ = nullptr, *qkv_ = nullptr, *q_ = nullptr, *attn_ = nullptr;
    uint16_t *gu_ = nullptr, *act_ = nullptr, *xs_ = nullptr, *logits_ = nullptr;
    // MoE: per-route outputs, router logits, routing tables (see moe_block)
    uint16_t *moe_y_ = nullptr, *moe_logits_ = nullptr;
    int32_t *moe_idx_ = nullptr, *moe_offsets_ = nullptr, *moe_route_token_ = nullptr,
            *moe_route_pos_ = nullptr;
    float* moe_w_ = nullptr;
    float* rope_tab_ = nullptr;
    uint32_t* out_tokens_ = nullptr;
    size_t out_cap_ = 0;   // sampling slots out_tokens_ / out_host_ hold
    void* attn_ws_ = nullptr;
    size_t attn_ws_bytes_ = 0;
    void* amax_ws_ = nullptr;      // (value, row) pairs of the lm_head GEMV's argmax stage
    size_t amax_ws_bytes_ = 0;
    void* gemm_ws_ = nullptr;      // split-K partial sums of the tiled GEMM
    size_t gemm_ws_bytes_ = 0;
    uint32_t* copy_ids_ = nullptr;  // staging for page-copy id lists
    size_t copy_ids_cap_ = 0;

    // staged inputs: one pinned host block mirrored by one device block
    struct Inputs {
        size_t off_tokens, off_positions, off_slots, off_row_begin, off_row_len, off_sample_rows,
            off_pages, total;
    };
    static Inputs input_layout(int N, int S);
    Inputs in_{};  // layout at capacity: sizes the staging buffers
    unsigned char* in_host_ = nullptr;
    unsigned char* in_dev_ = nullptr;
    uint32_t* out_host_ = nullptr;  // pinned

    // Sampler stage (allocated on first use, grown on demand; never touched by captured graphs
    // except the per-chunk logits gather of batches with more sampled rows than one chunk).
    struct Growable {
        void* ptr = nullptr;
        size_t cap = 0;
        bool pinned = false;
        void ensure(size_t bytes);
        void release();
    };
    // query-row tiles of the current forward for the matrix-core prefill attention (0 = per-row kernel)
    Growable tile_in_host_, tile_in_dev_;
    int n_tiles_ = 0, tile_rows_ = 0;
    // custom attention masks of the current forward (never part of a captured graph)
    Growable mask_in_host_, mask_in_dev_, mask_bitmap_;
    int mask_stride_ = 0;
    bool masked_ = false;
    Growable samp_f32_, samp_ws_, samp_in_dev_, samp_in_host_, samp_out_dev_, samp_out_host_;
    struct SampLayout {
        size_t kind, temperature, top_k, top_p, min_p, uniform, out_indptr, labels, bounds_indptr,
            bounds, total;
        size_t o_tokens, o_values, o_ids, o_total;
        int slots = 0, payload = 0, n_bounds = 0;
    } samp_{};
    bool samp_gather_in_body_ = false;
    uint64_t unseeded_draws_ = 0;

    std::map<std::tuple<int, int, int, int>, hipGraphExec_t> graphs_;   // (rows, sampling slots, context bucket, rows equally long)
    bool uniform_rows_ = false;   // this step's rows are about equally long (decode batches)
    int last_logit_rows_ = 0;
};

}  // namespace pie_hip_driver
