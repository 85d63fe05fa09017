// The `hip` driver flavour: request dispatch, response packing, the serve loop and the
// exported entry points.
//
//   serve loop / handler contract  driver/bridge/include/pie_bridge/inproc_server.hpp:35-96
//   method dispatch + status codes driver/portable/src/service/inproc_service.cpp:54-320
//   response CSR shape             driver/bridge/include/pie_bridge/response_builder.hpp:52-271
//   entry points                   driver/portable/src/entry.cpp:483-505, server/src/driver_ffi.rs:18-46
//   offline generation harness     driver/portable/src/executor/executor.cpp:1439-1597
#include <atomic>
#include <chrono>
#include <csignal>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "config.hpp"
#include "executor.hpp"
#include "model.hpp"
#include "pie_driver_abi.h"
#include "pie_hip_kernels.h"
#include "planner.hpp"
#include "snapshot.hpp"

using namespace pie_hip_driver;

namespace {

std::atomic<bool> g_stop{false};   // set by SIGINT / SIGTERM when the handlers are installed

using clk = std::chrono::steady_clock;
uint32_t us_since(clk::time_point t0) {
    return static_cast<uint32_t>(
        std::chrono::duration_cast<std::chrono::microseconds>(clk::now() - t0).count());
}

uint32_t method_of(const PieFrameDesc& f) {
    const PieRequestPayloadDesc& p = f.payload;
    switch (p.kind) {
        case PIE_REQ_FORWARD: return PIE_METHOD_FORWARD;
        case PIE_REQ_COPY:
            if (p.copy.dir > PIE_COPY_H2H) return PIE_METHOD_UNKNOWN;
            if (p.copy.resource == PIE_RESOURCE_KV) return PIE_METHOD_COPY_KV_D2H + p.copy.dir;
            if (p.copy.resource == PIE_RESOURCE_RS) return PIE_METHOD_COPY_RS_D2H + p.copy.dir;
            return PIE_METHOD_UNKNOWN;
        case PIE_REQ_ADAPTER:
            if (p.adapter.op == PIE_ADAPTER_GENERATE_AUDIO) return PIE_METHOD_GENERATE_AUDIO;
            if (p.adapter.op <= PIE_ADAPTER_ZO_UPDATE) return PIE_METHOD_ADAPTER_LOAD + p.adapter.op;
            return PIE_METHOD_UNKNOWN;
        case PIE_REQ_HEALTH: return PIE_METHOD_HEALTH;
        default: return PIE_METHOD_UNKNOWN;
    }
}

// Driver-owned storage behind a PieForwardResponseDesc; reused across calls.
struct ResponseStore {
    std::vector<uint32_t> tokens_indptr, tokens, dists_req_indptr, dists_kv_indptr,
        logits_req_indptr, logits_byte_indptr, logprobs_req_indptr, logprobs_val_indptr,
        entropies_indptr, spec_indptr, dists_ids;
    std::vector<float> dists_probs, logprobs_values, entropies;
    std::vector<uint8_t> logits_bytes;

    // Accepted tokens of one request from its slots' tokens: without drafts every slot's token;
    // with drafts the verifier walk — slot k predicts the token after draft k-1, the matching
    // prefix is accepted plus one bonus token (resolve_request_output,
    // driver/portable/src/executor/executor.cpp:204-248).
    static void resolve_tokens(const uint32_t* slot_tokens, int n_slots,
                               const std::vector<uint32_t>& drafts, std::vector<uint32_t>& out) {
        const int n_drafts = static_cast<int>(drafts.size());
        if (n_drafts == 0 || n_slots < n_drafts + 1) {
            out.insert(out.end(), slot_tokens, slot_tokens + n_slots);
            return;
        }
        for (int k = 0; k < n_drafts; ++k) {
            if (slot_tokens[k] != drafts[k]) {
                out.push_back(slot_tokens[k]);   // the model's own token replaces the rejected draft
                return;
            }
            out.push_back(drafts[k]);
        }
        out.push_back(slot_tokens[n_drafts]);
    }

    // Full response: per request, token slots -> tokens, Distribution -> dists, RawLogits ->
    // logits bytes (native f32), Logprob(s) -> logprobs, Entropy -> entropies, in slot order
    // (driver/portable/src/executor/executor.cpp:1343-1394; CSR shape of
    // driver/bridge/include/pie_bridge/response_builder.hpp:61-165).  `samples` == nullptr:
    // every slot is a greedy token slot.
    void build_full(const BatchPlan& plan, const std::vector<uint32_t>& slot_tokens,
                    const SampleOutputs* samples, int vocab, PieForwardResponseDesc& out) {
        const int R = plan.R;
        std::memset(&out, 0, sizeof(out));
        tokens_indptr.clear(); tokens.clear(); dists_req_indptr.clear(); dists_ids.clear();
        dists_probs.clear(); logits_req_indptr.clear(); logits_bytes.clear();
        logprobs_req_indptr.clear(); logprobs_values.clear(); entropies_indptr.clear();
        entropies.clear();
        dists_kv_indptr.assign(1, 0);
        logits_byte_indptr.assign(1, 0);
        logprobs_val_indptr.assign(1, 0);
        spec_indptr.assign(static_cast<size_t>(R) + 1, 0);
        size_t raw_at = 0;
        for (int r = 0; r < R; ++r) {
            tokens_indptr.push_back(static_cast<uint32_t>(tokens.size()));
            dists_req_indptr.push_back(static_cast<uint32_t>(dists_kv_indptr.size() - 1));
            logits_req_indptr.push_back(static_cast<uint32_t>(logits_byte_indptr.size() - 1));
            logprobs_req_indptr.push_back(static_cast<uint32_t>(logprobs_val_indptr.size() - 1));
            entropies_indptr.push_back(static_cast<uint32_t>(entropies.size()));
            const int s0 = plan.sample_indptr[r], s1 = plan.sample_indptr[r + 1];
            bool any_special = false;
            if (samples)
                for (int s = s0; s < s1; ++s) any_special |= !sampler_is_token_kind(plan.slot_samplers[s].kind);
            if (!any_special) {
                resolve_tokens(slot_tokens.data() + s0, s1 - s0, plan.draft_tokens[r], tokens);
                continue;
            }
            for (int s = s0; s < s1; ++s) {
                const int o0 = samples->out_indptr[s], o1 = samples->out_indptr[s + 1];
                switch (plan.slot_samplers[s].kind) {
                    case PIE_SAMPLER_KIND_DIST:
                        dists_ids.insert(dists_ids.end(), samples->ids.begin() + o0, samples->ids.begin() + o1);
                        dists_probs.insert(dists_probs.end(), samples->values.begin() + o0, samples->values.begin() + o1);
                        dists_kv_indptr.push_back(static_cast<uint32_t>(dists_ids.size()));
                        break;
                    case PIE_SAMPLER_KIND_RAW_LOGITS: {
                        const auto* b = reinterpret_cast<const uint8_t*>(samples->raw_logits.data() + raw_at);
                        logits_bytes.insert(logits_bytes.end(), b, b + static_cast<size_t>(vocab) * sizeof(float));
                        logits_byte_indptr.push_back(static_cast<uint32_t>(logits_bytes.size()));
                        break;
                    }
                    case PIE_SAMPLER_KIND_LOGPROB: case PIE_SAMPLER_KIND_LOGPROBS:
                        logprobs_values.insert(logprobs_values.end(), samples->values.begin() + o0, samples->values.begin() + o1);
                        logprobs_val_indptr.push_back(static_cast<uint32_t>(logprobs_values.size()));
                        break;
                    case PIE_SAMPLER_KIND_ENTROPY: entropies.push_back(samples->values[o0]); break;
                    case PIE_SAMPLER_KIND_EMBEDDING: break;   // no output
                    default: tokens.push_back(slot_tokens[s]); break;
                }
                if (plan.slot_samplers[s].kind == PIE_SAMPLER_KIND_RAW_LOGITS) raw_at += vocab;
            }
            // raw rows of requests without specials never exist: raw is itself a special kind
        }
        tokens_indptr.push_back(static_cast<uint32_t>(tokens.size()));
        dists_req_indptr.push_back(static_cast<uint32_t>(dists_kv_indptr.size() - 1));
        logits_req_indptr.push_back(static_cast<uint32_t>(logits_byte_indptr.size() - 1));
        logprobs_req_indptr.push_back(static_cast<uint32_t>(logprobs_val_indptr.size() - 1));
        entropies_indptr.push_back(static_cast<uint32_t>(entropies.size()));
        out.num_requests = static_cast<uint32_t>(R);
        out.tokens_indptr = {tokens_indptr.data(), tokens_indptr.size()};
        out.tokens = {tokens.data(), tokens.size()};
        out.dists_req_indptr = {dists_req_indptr.data(), dists_req_indptr.size()};
        out.dists_kv_indptr = {dists_kv_indptr.data(), dists_kv_indptr.size()};
        out.dists_ids = {dists_ids.data(), dists_ids.size()};
        out.dists_probs = {dists_probs.data(), dists_probs.size()};
        out.logits_req_indptr = {logits_req_indptr.data(), logits_req_indptr.size()};
        out.logits_byte_indptr = {logits_byte_indptr.data(), logits_byte_indptr.size()};
        out.logits_bytes = {logits_bytes.data(), logits_bytes.size()};
        out.logprobs_req_indptr = {logprobs_req_indptr.data(), logprobs_req_indptr.size()};
        out.logprobs_val_indptr = {logprobs_val_indptr.data(), logprobs_val_indptr.size()};
        out.logprobs_values = {logprobs_values.data(), logprobs_values.size()};
        out.entropies_indptr = {entropies_indptr.data(), entropies_indptr.size()};
        out.entropies = {entropies.data(), entropies.size()};
        out.spec_indptr = {spec_indptr.data(), spec_indptr.size()};
    }

    // R requests, every list empty except tokens (per-request CSR from sample_indptr).
    void build(int R, const std::vector<int32_t>& sample_indptr, const std::vector<uint32_t>& toks,
               PieForwardResponseDesc& out) {
        std::memset(&out, 0, sizeof(out));
        const size_t n1 = static_cast<size_t>(R) + 1;
        tokens_indptr.assign(n1, 0);
        for (int r = 0; r <= R && r < static_cast<int>(sample_indptr.size()); ++r)
            tokens_indptr[r] = static_cast<uint32_t>(sample_indptr[r]);
        tokens = toks;
        dists_req_indptr.assign(n1, 0);
        logits_req_indptr.assign(n1, 0);
        logprobs_req_indptr.assign(n1, 0);
        entropies_indptr.assign(n1, 0);
        spec_indptr.assign(n1, 0);
        dists_kv_indptr.assign(1, 0);      // second-level indptrs start with a leading 0
        logits_byte_indptr.assign(1, 0);
        logprobs_val_indptr.assign(1, 0);
        out.num_requests = static_cast<uint32_t>(R);
        out.tokens_indptr = {tokens_indptr.data(), tokens_indptr.size()};
        out.tokens = {tokens.data(), tokens.size()};
        out.dists_req_indptr = {dists_req_indptr.data(), dists_req_indptr.size()};
        out.dists_kv_indptr = {dists_kv_indptr.data(), dists_kv_indptr.size()};
        out.logits_req_indptr = {logits_req_indptr.data(), logits_req_indptr.size()};
        out.logits_byte_indptr = {logits_byte_indptr.data(), logits_byte_indptr.size()};
        out.logprobs_req_indptr = {logprobs_req_indptr.data(), logprobs_req_indptr.size()};
        out.logprobs_val_indptr = {logprobs_val_indptr.data(), logprobs_val_indptr.size()};
        out.entropies_indptr = {entropies_indptr.data(), entropies_indptr.size()};
        out.spec_indptr = {spec_indptr.data(), spec_indptr.size()};
    }
    // Failure shape: num_requests = 0, nothing else (driver/portable/src/executor/executor.cpp:1325-1341).
    static void build_failed(PieForwardResponseDesc& out) { std::memset(&out, 0, sizeof(out)); }
};

std::string json_escape(const std::string& s) {
    std::string o;
    for (char c : s) {
        if (c == '"' || c == '\\') { o.push_back('\\'); o.push_back(c); }
        else if (static_cast<unsigned char>(c) < 0x20) { char b[8]; std::snprintf(b, sizeof b, "\\u%04x", c); o += b; }
        else o.push_back(c);
    }
    return o;
}

}  // namespace

// TOML, then (with `[model] hf_path` / `snapshot_dir`) the snapshot's config.json for the shape.
static DriverConfig load_driver_config(const std::string& src) {
    DriverConfig c = load_config(src);
    if (!c.model.checkpoint_dir.empty()) {
        apply_hf_config(c.model, c.model.checkpoint_dir);
        finalize_config(c);
        if (c.runtime.snapshot_dir.empty()) c.runtime.snapshot_dir = c.model.checkpoint_dir;
    }
    return c;
}

struct PieHipDriver {
    DriverConfig cfg;
    Model model;
    std::unique_ptr<Executor> exec;
    std::string caps;
    ResponseStore store;
    std::vector<uint32_t> toks;
    SampleOutputs samples;
    std::string last_error;
    PieSamplerDesc gen_sampler{};   // decode-step sampler of the generation harness (kind 2, T 0 = greedy)
    bool gen_sampler_set = false;
    uint32_t gen_diverge = 0;   // generation harness: replica c starts decoding from (first token + c * this) % vocab

    explicit PieHipDriver(const DriverConfig& c) : cfg(c) {
        // the kernel library found at run time must be the one this driver was compiled against
        if (pie_hip_abi_version() != PIE_HIP_ABI_VERSION)
            throw std::runtime_error("libpie_hip_kernels.so has ABI version " + std::to_string(pie_hip_abi_version()) +
                                     ", this driver was built against " + std::to_string(PIE_HIP_ABI_VERSION));
        int ndev = 0;
        if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0)
            throw std::runtime_error("no HIP device is visible: this driver has no CPU path");
        hipStream_t s = nullptr;
        if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess)
            throw std::runtime_error("cannot create a HIP stream");
        try {
            if (cfg.model.checkpoint_dir.empty()) model.init_synthetic(cfg.model, s);
            else model.load_snapshot(cfg.model, s);
            if (cfg.runtime.tiled_weights) model.build_tiled_copies(s);
        } catch (...) {
            (void)hipStreamDestroy(s);
            throw;
        }
        (void)hipStreamDestroy(s);
        exec = std::make_unique<Executor>(cfg, model);
        build_caps();
    }

    // Capabilities handshake (driver/bridge/src/capabilities.rs:18-78; values as
    // driver/portable/src/entry.cpp:432-452).
    void build_caps() {
        const auto& m = cfg.model;
        const long long total_pages = exec->total_pages();
        const long long ps = exec->page_size();
        const unsigned long long umax = 4294967295ull;
        std::ostringstream j;
        j << "{\"total_pages\":" << total_pages << ",\"kv_page_size\":" << ps
          << ",\"swap_pool_size\":" << cfg.batching.cpu_pages
          << ",\"rs_cache_required\":false,\"rs_cache_slots\":0,\"rs_cache_slot_bytes\":0"
          << ",\"max_forward_tokens\":" << cfg.batching.max_forward_tokens
          << ",\"max_forward_requests\":" << cfg.batching.max_forward_requests
          << ",\"max_page_refs\":" << total_pages << ",\"max_logit_rows\":" << umax
          << ",\"max_prob_rows\":" << umax << ",\"max_custom_mask_bytes\":" << umax
          << ",\"max_sampler_rows\":" << umax << ",\"max_logprob_labels\":" << umax
          << ",\"arch_name\":\"" << json_escape(m.arch) << "\",\"vocab_size\":" << m.vocab
          << ",\"max_model_len\":" << total_pages * ps << ",\"activation_dtype\":\"bfloat16\""
          << ",\"snapshot_dir\":\"" << json_escape(cfg.runtime.snapshot_dir) << "\"}";
        caps = j.str();
    }

    void forward(const PieForwardRequestDesc& f, PieForwardResponseDesc& out) {
        const auto t_start = clk::now();
        // Empty batch: R empty per-request outputs (driver/portable/src/executor/executor.cpp:1310-1322).
        const int R = f.qo_indptr.len > 0 ? static_cast<int>(f.qo_indptr.len) - 1 : 0;
        if (f.token_ids.len == 0 || R <= 0) {
            store.build(R > 0 ? R : 0, std::vector<int32_t>(static_cast<size_t>(R > 0 ? R : 0) + 1, 0), {}, out);
            return;
        }
        try {
            auto t0 = clk::now();
            const BatchPlan plan = plan_forward(f, exec->page_size(), exec->total_pages());
            if (R > cfg.batching.max_forward_requests)
                throw std::runtime_error("forward: batch exceeds max_forward_requests");
            const uint32_t plan_us = us_since(t0);
            ForwardTimings ft;
            const bool sampling = !plan.all_greedy && !plan.sample_rows.empty();
            exec->forward(plan, toks, &ft, sampling ? &samples : nullptr);
            t0 = clk::now();
            store.build_full(plan, toks, sampling ? &samples : nullptr, cfg.model.vocab, out);
            out.probe_wire_parse_us = 0;
            out.probe_plan_us = plan_us;
            out.probe_h2d_us = ft.h2d_us;
            out.probe_kernel_launch_us = ft.launch_us;
            out.probe_sync_us = ft.sync_us;
            out.probe_response_build_us = us_since(t0);
            (void)t_start;
        } catch (const std::exception& e) {
            last_error = e.what();
            if (cfg.runtime.verbose) std::fprintf(stderr, "[pie-driver-hip] forward failed: %s\n", e.what());
            ResponseStore::build_failed(out);
        }
    }

    // Status codes and checks of driver/portable/src/service/inproc_service.cpp:82-203: a length
    // mismatch is a failure (5), host copies without a swap pool are unsupported (4), an id
    // outside its pool is out of range (3); pairs before a bad one have been copied.
    int copy(const PieCopyRequestDesc& c, uint32_t method) {
        if (c.srcs.len != c.dsts.len) return PIE_STATUS_FAILED;
        if (method >= PIE_METHOD_COPY_RS_D2H) return PIE_STATUS_UNSUPPORTED;  // no recurrent state
        const uint32_t dev = static_cast<uint32_t>(exec->total_pages());
        const uint32_t host = static_cast<uint32_t>(exec->cpu_pages());
        if (method != PIE_METHOD_COPY_KV_D2D && host == 0) return PIE_STATUS_UNSUPPORTED;
        const uint32_t src_cap = (method == PIE_METHOD_COPY_KV_D2H || method == PIE_METHOD_COPY_KV_D2D) ? dev : host;
        const uint32_t dst_cap = (method == PIE_METHOD_COPY_KV_H2D || method == PIE_METHOD_COPY_KV_D2D) ? dev : host;
        size_t good = 0;
        while (good < c.srcs.len && c.srcs.ptr[good] < src_cap && c.dsts.ptr[good] < dst_cap) ++good;
        switch (method) {
            case PIE_METHOD_COPY_KV_D2D:
                if (good != c.srcs.len) return PIE_STATUS_OUT_OF_RANGE;
                exec->copy_pages_d2d(c.srcs.ptr, c.dsts.ptr, c.srcs.len);
                return PIE_STATUS_OK;
            case PIE_METHOD_COPY_KV_D2H: exec->copy_pages_d2h(c.srcs.ptr, c.dsts.ptr, good); break;
            case PIE_METHOD_COPY_KV_H2D: exec->copy_pages_h2d(c.srcs.ptr, c.dsts.ptr, good); break;
            case PIE_METHOD_COPY_KV_H2H: exec->copy_pages_h2h(c.srcs.ptr, c.dsts.ptr, good); break;
            default: return PIE_STATUS_UNSUPPORTED;
        }
        return good == c.srcs.len ? PIE_STATUS_OK : PIE_STATUS_OUT_OF_RANGE;
    }

    void handle(const PieFrameDesc& frame, PieResponseFrameDesc& out) {
        std::memset(&out, 0, sizeof(out));
        out.driver_id = frame.driver_id;
        const uint32_t method = method_of(frame);
        if (method == PIE_METHOD_FORWARD) {
            out.payload.kind = PIE_RESP_FORWARD;
            forward(frame.payload.forward, out.payload.forward);
            return;
        }
        out.payload.kind = PIE_RESP_STATUS;
        int status;
        try {
            switch (method) {
                case PIE_METHOD_COPY_KV_D2H: case PIE_METHOD_COPY_KV_H2D: case PIE_METHOD_COPY_KV_D2D:
                case PIE_METHOD_COPY_KV_H2H: case PIE_METHOD_COPY_RS_D2H: case PIE_METHOD_COPY_RS_H2D:
                case PIE_METHOD_COPY_RS_D2D: case PIE_METHOD_COPY_RS_H2H:
                    status = copy(frame.payload.copy, method);
                    break;
                case PIE_METHOD_HEALTH: status = PIE_STATUS_OK; break;
                case PIE_METHOD_ADAPTER_LOAD: case PIE_METHOD_ADAPTER_SAVE:
                case PIE_METHOD_ADAPTER_ZO_INIT: case PIE_METHOD_ADAPTER_ZO_UPDATE:
                case PIE_METHOD_GENERATE_AUDIO:
                    status = PIE_STATUS_UNSUPPORTED;
                    break;
                default: status = PIE_STATUS_UNKNOWN_METHOD; break;
            }
        } catch (const std::exception& e) {
            last_error = e.what();
            status = PIE_STATUS_EXCEPTION;
        }
        out.payload.status.status = status;
    }
};

namespace {

void set_err(char* err, size_t cap, const std::string& msg) {
    if (err && cap) {
        std::snprintf(err, cap, "%s", msg.c_str());
    }
}

// Fills a forward frame over borrowed vectors (the harness plays the runtime's role).
struct FrameBuilder {
    std::vector<uint32_t> tokens, positions, pages, page_indptr, last_lens, qo_indptr, samp_idx,
        samp_indptr, sampler_indptr;
    std::vector<PieSamplerDesc> samplers;
    std::vector<uint64_t> ctx_ids;
    PieFrameDesc frame;
    void finish() {
        std::memset(&frame, 0, sizeof(frame));
        frame.payload.kind = PIE_REQ_FORWARD;
        PieForwardRequestDesc& f = frame.payload.forward;
        f.token_ids = {tokens.data(), tokens.size()};
        f.position_ids = {positions.data(), positions.size()};
        f.kv_page_indices = {pages.data(), pages.size()};
        f.kv_page_indptr = {page_indptr.data(), page_indptr.size()};
        f.kv_last_page_lens = {last_lens.data(), last_lens.size()};
        f.qo_indptr = {qo_indptr.data(), qo_indptr.size()};
        f.sampling_indices = {samp_idx.data(), samp_idx.size()};
        f.sampling_indptr = {samp_indptr.data(), samp_indptr.size()};
        f.samplers = {samplers.data(), samplers.size()};
        f.sampler_indptr = {sampler_indptr.data(), sampler_indptr.size()};
        f.context_ids = {ctx_ids.data(), ctx_ids.size()};
        f.single_token_mode = 1;
    }
};

PieSamplerDesc greedy_sampler() {
    // greedy arrives on the wire as TopP{temperature 0, p 1} (sdk/rust/inferlet/src/sample.rs:77-79)
    PieSamplerDesc s;
    std::memset(&s, 0, sizeof(s));
    s.kind = PIE_SAMPLER_KIND_TOP_P;
    s.temperature = 0.f;
    s.p = 1.f;
    return s;
}

}  // namespace

// Start-up warm-up ([runtime] warmup): the generation harness on a synthetic prompt of one full
// prefill chunk plus two decode steps.  Best effort: a pool too small for it skips it.
static void warm_up(PieHipDriver* d) {
    if (!d->cfg.runtime.warmup) return;
    const long long room = static_cast<long long>(d->exec->total_pages()) * d->exec->page_size() - 4;
    const int n = static_cast<int>(std::min<long long>(d->cfg.batching.max_forward_tokens, room));
    if (n <= 0) return;
    std::vector<uint32_t> prompt(n);
    for (int i = 0; i < n; ++i) prompt[i] = static_cast<uint32_t>(i % std::max(1, d->cfg.model.vocab));
    uint32_t out[3];
    double tm[4];
    char err[256];
    const int rc = pie_hip_driver_generate(d, prompt.data(), n, 3, 1, 0, out, tm, err, sizeof(err));
    if (rc != 0 && d->cfg.runtime.verbose) std::fprintf(stderr, "[pie-driver-hip] warm-up skipped: %s\n", err);
    d->last_error.clear();
}

extern "C" PieHipDriver* pie_hip_driver_create(const char* config_toml, char* err, size_t err_cap) {
    try {
        if (!config_toml) throw std::runtime_error("null config");
        PieHipDriver* d = new PieHipDriver(load_driver_config(config_toml));
        warm_up(d);
        return d;
    } catch (const std::exception& e) {
        set_err(err, err_cap, e.what());
        return nullptr;
    } catch (...) {
        set_err(err, err_cap, "unknown error");
        return nullptr;
    }
}

extern "C" void pie_hip_driver_destroy(PieHipDriver* d) { delete d; }

extern "C" const char* pie_hip_driver_capabilities(const PieHipDriver* d) {
    return d ? d->caps.c_str() : nullptr;
}

extern "C" int pie_hip_driver_handle(PieHipDriver* d, const PieFrameDesc* frame,
                                     PieResponseFrameDesc* out) {
    if (!d || !frame || !out) return -1;
    try {
        d->handle(*frame, *out);
    } catch (...) {  // handler exception -> status -1 (inproc_server.hpp:66-74)
        std::memset(out, 0, sizeof(*out));
        out->payload.kind = PIE_RESP_STATUS;
        out->payload.status.status = PIE_STATUS_EXCEPTION;
    }
    return 0;
}

extern "C" size_t pie_hip_driver_export_tensor(PieHipDriver* d, const char* name, void* dst,
                                               size_t cap) {
    if (!d || !name) return 0;
    if (std::string(name) == "debug.logits") {
        const size_t bytes = static_cast<size_t>(d->exec->last_logit_rows()) * d->cfg.model.vocab * 2;
        if (dst && bytes) {
            const size_t n = bytes < cap ? bytes : cap;
            if (hipMemcpy(dst, d->exec->last_logits(), n, hipMemcpyDeviceToHost) != hipSuccess) return 0;
        }
        return bytes;
    }
    const std::string nm(name);
    if (nm == "info.qk_rows_paired" || nm == "info.rope_interleaved") {   // one int32
        const int32_t v = nm == "info.qk_rows_paired" ? (d->model.qk_rows_paired() ? 1 : 0)
                                                      : d->cfg.model.rope_interleaved;
        if (dst && cap >= sizeof(v)) std::memcpy(dst, &v, sizeof(v));
        return sizeof(v);
    }
    if (nm == "info.tuned") {
        // the kernel each decoder linear runs per row count, as the start-up measurement left it:
        // int8 [4 linears (wqkv, wo, wgu, wdown)][129 row counts] of layer 0 (every layer holds the
        // same), -1 = the cost model decides, 0 GEMV, 1 skinny GEMM, 2 tiled GEMM, 3 tiled GEMM in K shares
        const auto& lw = d->model.layers.at(0);
        const Linear* lins[4] = {&lw.wqkv, &lw.wo, &lw.wgu, &lw.wdown};
        int8_t tab[4][129];
        for (int i = 0; i < 4; ++i)
            for (int m = 0; m <= 128; ++m) tab[i][m] = lins[i]->tuned[static_cast<size_t>(m)];
        if (dst && cap >= sizeof(tab)) std::memcpy(dst, tab, sizeof(tab));
        return sizeof(tab);
    }
    if (nm == "info.rope_mscale") {   // one float
        const float v = rope_mscale(d->cfg.model);
        if (dst && cap >= sizeof(v)) std::memcpy(dst, &v, sizeof(v));
        return sizeof(v);
    }
    if (nm.rfind("debug.", 0) == 0) {
        const uint16_t* buf = d->exec->debug_buffer(nm.substr(6));
        if (!buf) return 0;
        const auto& mc = d->cfg.model;
        const size_t elems = nm == "debug.x" ? mc.hidden
                             : nm == "debug.act" ? (mc.num_experts > 0 ? mc.expert_intermediate : mc.intermediate)
                                                 : static_cast<size_t>(mc.q_heads) * mc.head_dim;
        const size_t bytes = elems * 2;
        if (dst) {
            const size_t n = bytes < cap ? bytes : cap;
            if (hipMemcpy(dst, buf, n, hipMemcpyDeviceToHost) != hipSuccess) return 0;
        }
        return bytes;
    }
    if (nm.rfind("kv.k.", 0) == 0 || nm.rfind("kv.v.", 0) == 0) {
        const int l = std::atoi(nm.c_str() + 5);
        const uint16_t* pool = d->exec->kv_pool(nm[3] == 'k', l);
        if (!pool) return 0;
        const size_t bytes = d->exec->page_bytes() * static_cast<size_t>(d->exec->total_pages());
        if (dst) {
            const size_t n = bytes < cap ? bytes : cap;
            if (hipMemcpy(dst, pool, n, hipMemcpyDeviceToHost) != hipSuccess) return 0;
        }
        return bytes;
    }
    const auto& t = d->model.tensors();
    const auto it = t.find(name);
    if (it == t.end()) return 0;
    if (dst) {
        const size_t n = it->second.bytes < cap ? it->second.bytes : cap;
        if (hipMemcpy(dst, it->second.ptr, n, hipMemcpyDeviceToHost) != hipSuccess) return 0;
    }
    return it->second.bytes;
}

extern "C" void* pie_hip_driver_tensor_ptr(PieHipDriver* d, const char* name) {
    if (!d || !name) return nullptr;
    const auto& t = d->model.tensors();
    const auto it = t.find(name);
    return it == t.end() ? nullptr : it->second.ptr;
}

// Sampler the generation harness attaches to its decode steps (wire kind and fields; the seed
// is advanced per step and context).  Default: greedy.
extern "C" int pie_hip_driver_set_generate_sampler(PieHipDriver* d, int kind, float temperature,
                                                   uint32_t k, float p, uint32_t seed) {
    if (!d || kind < 0 || kind > PIE_SAMPLER_KIND_TOP_K_TOP_P) return -1;
    std::memset(&d->gen_sampler, 0, sizeof(d->gen_sampler));
    d->gen_sampler.kind = static_cast<uint8_t>(kind);
    d->gen_sampler.temperature = temperature;
    d->gen_sampler.k = k;
    d->gen_sampler.p = p;
    d->gen_sampler.seed = seed;
    d->gen_sampler_set = true;
    return 0;
}

// Replicas of the generation harness share the prompt; with stride > 0 replica c feeds
// (its last sampled token + c * stride) % vocab into every decode step, so the rows of a decode
// batch differ (distinct hidden states, distinct MoE routes) even where a synthetic model's greedy
// tokens coincide.  0: identical replicas.
extern "C" int pie_hip_driver_set_generate_divergence(PieHipDriver* d, uint32_t stride) {
    if (!d) return -1;
    d->gen_diverge = stride;
    return 0;
}

extern "C" int pie_hip_driver_generate(PieHipDriver* d, const uint32_t* prompt, int n_prompt,
                                       int max_new, int replicate, int warmup,
                                       uint32_t* out_tokens, double* timings_us, char* err,
                                       size_t err_cap) {
    if (!d || !prompt || n_prompt <= 0 || max_new <= 0 || replicate <= 0 || !out_tokens ||
        warmup < 0) {
        set_err(err, err_cap, "bad arguments");
        return -1;
    }
    try {
        const int ps = d->exec->page_size();
        const int pages_per_ctx = (n_prompt + max_new + ps - 1) / ps;
        if (static_cast<long long>(pages_per_ctx) * replicate > d->exec->total_pages())
            throw std::runtime_error("generate: needs " + std::to_string(pages_per_ctx * replicate) +
                                     " pages, pool has " + std::to_string(d->exec->total_pages()));
        if (replicate > d->cfg.batching.max_forward_requests)
            throw std::runtime_error("generate: replicate exceeds max_forward_requests");
        PieResponseFrameDesc resp;
        std::vector<uint32_t> last(replicate);
        const int chunk_cap = d->cfg.batching.max_forward_tokens;
        const auto t_prefill = clk::now();
        // Prefill: context 0 runs the prompt (contiguous page range), chunked to the token cap,
        // only the final chunk samples; the other contexts hold the same prompt, so their pages
        // are device-to-device copies of context 0's (the fork-by-copy path of Copy{D2D}).
        for (int c = 0; c < 1; ++c) {
            for (int t0 = 0; t0 < n_prompt; t0 += chunk_cap) {
                const int n = std::min(chunk_cap, n_prompt - t0);
                const int upto = t0 + n;  // tokens in the context after this chunk
                FrameBuilder fb;
                fb.tokens.assign(prompt + t0, prompt + upto);
                for (int i = t0; i < upto; ++i) fb.positions.push_back(static_cast<uint32_t>(i));
                const int np = (upto + ps - 1) / ps;
                for (int p = 0; p < np; ++p) fb.pages.push_back(static_cast<uint32_t>(c * pages_per_ctx + p));
                fb.page_indptr = {0u, static_cast<uint32_t>(np)};
                fb.last_lens = {static_cast<uint32_t>(upto - (np - 1) * ps)};
                fb.qo_indptr = {0u, static_cast<uint32_t>(n)};
                fb.ctx_ids = {static_cast<uint64_t>(c)};
                const bool final_chunk = upto == n_prompt;
                if (final_chunk) {
                    fb.samp_idx = {static_cast<uint32_t>(n - 1)};
                    fb.samp_indptr = {0u, 1u};
                    fb.samplers = {greedy_sampler()};
                    fb.sampler_indptr = {0u, 1u};
                } else {
                    fb.samp_indptr = {0u, 0u};
                    fb.sampler_indptr = {0u, 0u};
                }
                fb.finish();
                fb.frame.payload.forward.single_token_mode = 0;
                d->handle(fb.frame, resp);
                const PieForwardResponseDesc& fr = resp.payload.forward;
                if (fr.num_requests != 1) throw std::runtime_error("generate: prefill failed: " + d->last_error);
                if (final_chunk) {
                    if (fr.tokens.len != 1) throw std::runtime_error("generate: prefill returned no token");
                    last[c] = fr.tokens.ptr[0];
                    out_tokens[static_cast<size_t>(c) * max_new] = last[c];
                }
            }
        }
        if (replicate > 1) {
            const int np = (n_prompt + ps - 1) / ps;
            std::vector<uint32_t> srcs, dsts;
            for (int c = 1; c < replicate; ++c)
                for (int p = 0; p < np; ++p) {
                    srcs.push_back(static_cast<uint32_t>(p));
                    dsts.push_back(static_cast<uint32_t>(c * pages_per_ctx + p));
                }
            d->exec->copy_pages_d2d(srcs.data(), dsts.data(), srcs.size());
            for (int c = 1; c < replicate; ++c) {
                last[c] = last[0];
                out_tokens[static_cast<size_t>(c) * max_new] = last[0];
            }
        }
        const double prefill_us = us_since(t_prefill);
        // Decode: one multi-request single-token plan per step.
        hipEvent_t e0 = nullptr, e1 = nullptr;
        (void)hipEventCreate(&e0);
        (void)hipEventCreate(&e1);
        auto t_decode = clk::now();
        (void)hipEventRecord(e0, d->exec->stream());
        int timed_steps = 0;
        const uint64_t vocab = static_cast<uint64_t>(std::max(1, d->model.cfg().vocab));
        for (int s = 1; s < max_new; ++s) {
            if (s == warmup + 1 && warmup > 0) {  // restart the clocks after the warm-up steps
                (void)hipStreamSynchronize(d->exec->stream());
                t_decode = clk::now();
                (void)hipEventRecord(e0, d->exec->stream());
                timed_steps = 0;
            }
            ++timed_steps;
            const int pos = n_prompt + s - 1;  // position of the token fed in this step
            const int np = (pos + 1 + ps - 1) / ps;
            FrameBuilder fb;
            for (int c = 0; c < replicate; ++c) {
                fb.tokens.push_back(static_cast<uint32_t>((last[c] + static_cast<uint64_t>(c) * d->gen_diverge) % vocab));
                fb.positions.push_back(static_cast<uint32_t>(pos));
                for (int p = 0; p < np; ++p) fb.pages.push_back(static_cast<uint32_t>(c * pages_per_ctx + p));
                fb.last_lens.push_back(static_cast<uint32_t>(pos + 1 - (np - 1) * ps));
                fb.samp_idx.push_back(0u);
                PieSamplerDesc sd = d->gen_sampler_set ? d->gen_sampler : greedy_sampler();
                if (sd.seed != 0) sd.seed += static_cast<uint32_t>(s * replicate + c);   // a fresh draw per slot
                fb.samplers.push_back(sd);
                fb.ctx_ids.push_back(static_cast<uint64_t>(c));
            }
            for (int c = 0; c <= replicate; ++c) {
                fb.page_indptr.push_back(static_cast<uint32_t>(c * np));
                fb.qo_indptr.push_back(static_cast<uint32_t>(c));
                fb.samp_indptr.push_back(static_cast<uint32_t>(c));
                fb.sampler_indptr.push_back(static_cast<uint32_t>(c));
            }
            fb.finish();
            d->handle(fb.frame, resp);
            const PieForwardResponseDesc& fr = resp.payload.forward;
            if (fr.num_requests != static_cast<uint32_t>(replicate) || fr.tokens.len != static_cast<size_t>(replicate))
                throw std::runtime_error("generate: decode step failed: " + d->last_error);
            for (int c = 0; c < replicate; ++c) {
                last[c] = fr.tokens.ptr[c];
                out_tokens[static_cast<size_t>(c) * max_new + s] = last[c];
            }
        }
        (void)hipEventRecord(e1, d->exec->stream());
        (void)hipEventSynchronize(e1);
        float dev_ms = 0.f;
        (void)hipEventElapsedTime(&dev_ms, e0, e1);
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        if (timings_us) {
            timings_us[0] = prefill_us;
            timings_us[1] = us_since(t_decode);
            timings_us[2] = static_cast<double>(dev_ms) * 1e3;
            timings_us[3] = static_cast<double>(timed_steps);
        }
        return 0;
    } catch (const std::exception& e) {
        set_err(err, err_cap, e.what());
        return -2;
    } catch (...) {
        set_err(err, err_cap, "unknown error");
        return -3;
    }
}

// Every instance inside pie_driver_hip_run_inproc registers its stop flag on entry, before the
// model is loaded, so a stop requested while it loads is honoured as soon as it would start to
// serve; request_stop reaches every live instance of this flavour
// (driver/portable/src/entry.cpp:61-94, :483-505).
namespace {
std::mutex g_instances_mu;
std::vector<std::atomic<bool>*> g_instances;
struct InstanceStop {
    std::atomic<bool> flag{false};
    InstanceStop() {
        std::lock_guard<std::mutex> lk(g_instances_mu);
        g_instances.push_back(&flag);
    }
    ~InstanceStop() {
        std::lock_guard<std::mutex> lk(g_instances_mu);
        g_instances.erase(std::remove(g_instances.begin(), g_instances.end(), &flag), g_instances.end());
    }
};
}  // namespace

extern "C" void pie_driver_hip_request_stop(void) {
    std::lock_guard<std::mutex> lk(g_instances_mu);
    for (auto* f : g_instances) f->store(true, std::memory_order_release);
}

extern "C" int pie_driver_hip_run_inproc(int argc, char** argv, int install_signal_handlers,
                                         void (*ready_cb)(const char* caps_json, void* ctx),
                                         void* ready_ctx, PieInProcVTable vtable) {
    try {
        std::string config_path;
        for (int i = 1; i < argc; ++i) {
            const std::string a = argv[i] ? argv[i] : "";
            if ((a == "--config" || a == "-c") && i + 1 < argc) config_path = argv[++i];
            else if (a.rfind("--config=", 0) == 0) config_path = a.substr(9);
        }
        if (config_path.empty()) {
            std::fprintf(stderr, "[pie-driver-hip] missing --config <file.toml>\n");
            return -1;
        }
        if (!vtable.recv || !vtable.send_response) {
            std::fprintf(stderr, "[pie-driver-hip] incomplete vtable\n");
            return -1;
        }
        if (install_signal_handlers) {
            std::signal(SIGINT, [](int) { g_stop.store(true); });
            std::signal(SIGTERM, [](int) { g_stop.store(true); });
        }
        {
            // a signal of an earlier run is forgotten only when no instance is serving: a second
            // instance that starts during a reload must not erase a SIGINT / SIGTERM the first
            // has not seen yet
            std::lock_guard<std::mutex> lk(g_instances_mu);
            if (g_instances.empty()) g_stop.store(false, std::memory_order_release);
        }
        InstanceStop stop;
        PieHipDriver driver(load_driver_config(config_path));
        warm_up(&driver);
        if (ready_cb) ready_cb(driver.caps.c_str(), ready_ctx);
        if (driver.cfg.runtime.verbose) std::fprintf(stderr, "[pie-driver-hip] serving on in-process channel\n");
        PieResponseFrameDesc resp;
        while (!g_stop.load(std::memory_order_acquire) && !stop.flag.load(std::memory_order_acquire)) {
            const PieFrameDesc* req = nullptr;
            uint32_t req_id = 0;
            const int32_t rc = vtable.recv(vtable.ctx, &req, &req_id);
            if (rc != 0) break;  // -1 clean shutdown, anything else an error: stop either way
            if (!req) continue;
            try {
                driver.handle(*req, resp);
            } catch (...) {
                std::memset(&resp, 0, sizeof(resp));
                resp.driver_id = req->driver_id;
                resp.payload.kind = PIE_RESP_STATUS;
                resp.payload.status.status = PIE_STATUS_EXCEPTION;
            }
            vtable.send_response(vtable.ctx, req_id, &resp);
        }
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "[pie-driver-hip] fatal: %s\n", e.what());
        return -1;
    } catch (...) {
        std::fprintf(stderr, "[pie-driver-hip] fatal: unknown error\n");
        return -1;
    }
}

// Host-only snapshot hook: reads `<dir>/config.json` and the safetensors headers and writes a
// JSON summary {"arch", the shape fields, "tensors": {name: {"dtype", "shape", "bytes",
// "first_bytes": [up to 8 leading data bytes]}}} into out.  Returns its length, or -1 with the
// reader's message in err.  No GPU is touched.
extern "C" long long pie_hip_driver_snapshot_info(const char* dir, char* out, size_t out_cap,
                                                  char* err, size_t err_cap) {
    try {
        if (!dir || !out) throw std::runtime_error("null argument");
        ModelConfig m;
        apply_hf_config(m, dir);
        const Snapshot snap(dir);
        std::ostringstream j;
        j << "{\"arch\":\"" << m.arch << "\",\"hidden\":" << m.hidden << ",\"layers\":" << m.layers
          << ",\"q_heads\":" << m.q_heads << ",\"kv_heads\":" << m.kv_heads << ",\"head_dim\":" << m.head_dim
          << ",\"intermediate\":" << m.intermediate << ",\"vocab\":" << m.vocab
          << ",\"rms_eps\":" << m.rms_eps << ",\"rope_theta\":" << m.rope_theta
          << ",\"rope_factor\":" << m.rope_factor << ",\"tie_embeddings\":" << (m.tie_embeddings ? "true" : "false")
          << ",\"num_experts\":" << m.num_experts << ",\"top_k\":" << m.top_k
          << ",\"expert_intermediate\":" << m.expert_intermediate << ",\"tensors\":{";
        bool first = true;
        for (const auto& [name, t] : snap.tensors()) {
            j << (first ? "" : ",") << "\"" << json_escape(name) << "\":{\"dtype\":\"" << t.dtype << "\",\"shape\":[";
            for (size_t i = 0; i < t.shape.size(); ++i) j << (i ? "," : "") << t.shape[i];
            j << "],\"bytes\":" << t.bytes << ",\"first_bytes\":[";
            for (size_t i = 0; i < std::min<size_t>(8, t.bytes); ++i) j << (i ? "," : "") << static_cast<int>(t.data[i]);
            j << "]}";
            first = false;
        }
        j << "}}";
        const std::string text = j.str();
        if (text.size() + 1 > out_cap) throw std::runtime_error("output buffer too small");
        std::memcpy(out, text.c_str(), text.size() + 1);
        return static_cast<long long>(text.size());
    } catch (const std::exception& e) {
        set_err(err, err_cap, e.what());
        return -1;
    }
}

// Host-only planner hook: runs the planner on a forward request and copies the integer
// plan out, so that the page-table arithmetic can be checked bit-exactly without a GPU.
// out_i64 receives kv_slots[N]; out_i32 receives, back to back: positions[N],
// row_page_begin[N], row_kv_len[N], seq_len[R], sample_rows[S], sample_indptr[R+1], then
// {R, N, S, max_kv_len, pure_decode, all_greedy, has_user_masks}.  Returns the number of
// int32 values written, or -1 with the planner's message in err.
extern "C" long long pie_hip_driver_plan(const PieForwardRequestDesc* f, int page_size,
                                         int total_pages, long long* out_i64, int* out_i32,
                                         size_t out_i32_cap, char* err, size_t err_cap) {
    try {
        if (!f) throw std::runtime_error("null request");
        const BatchPlan p = plan_forward(*f, page_size, total_pages);
        const size_t S = p.sample_rows.size();
        const size_t need = 3 * static_cast<size_t>(p.N) + p.R + S + (p.R + 1) + 7;
        if (need > out_i32_cap) throw std::runtime_error("output buffer too small");
        size_t o = 0;
        for (int i = 0; i < p.N; ++i) out_i64[i] = p.kv_slots[i];
        for (int i = 0; i < p.N; ++i) out_i32[o++] = p.positions[i];
        for (int i = 0; i < p.N; ++i) out_i32[o++] = static_cast<int>(p.row_page_begin[i]);
        for (int i = 0; i < p.N; ++i) out_i32[o++] = p.row_kv_len[i];
        for (int r = 0; r < p.R; ++r) out_i32[o++] = p.seq_len[r];
        for (size_t i = 0; i < S; ++i) out_i32[o++] = p.sample_rows[i];
        for (int r = 0; r <= p.R; ++r) out_i32[o++] = p.sample_indptr[r];
        const int tail[7] = {p.R, p.N, static_cast<int>(S), p.max_kv_len, p.pure_decode ? 1 : 0,
                             p.all_greedy ? 1 : 0, p.has_user_masks ? 1 : 0};
        for (int v : tail) out_i32[o++] = v;
        return static_cast<long long>(o);
    } catch (const std::exception& e) {
        set_err(err, err_cap, e.what());
        return -1;
    }
}
