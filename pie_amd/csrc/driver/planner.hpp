// Forward-request planner: wire arrays -> the integer plan the kernels consume.
// Pure host C++ (no HIP), exercised bit-exactly against the oracle on the CPU.
//
// Follows the reference portable driver:
//   shape checks            driver/portable/src/plan.cpp:177-206
//   per-request plan        driver/portable/src/plan.cpp:224-470 (seq_len :247-249, page id
//                           bound :255-264, position bound :282-287, sampling rows :368-373)
//   physical slot           driver/portable/src/plan.hpp:36-45
//   synthesised causal mask driver/portable/src/plan.cpp:139-173
//   pure-decode / all-greedy driver/portable/src/executor/executor.cpp:537-543, :568-586
//   per-slot sampler params  driver/portable/src/plan.cpp:408-453 with the AoS -> SoA field
//                           mapping of driver/bridge/include/pie_bridge/view.hpp:441-496
//   logit masks, drafts     driver/portable/src/plan.cpp:379-406, :455-466
// The request count comes from qo_indptr (as the CUDA driver does,
// driver/cuda/src/executor/executor.cpp:2240); a non-empty context_ids must agree with it.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "pie_driver_abi.h"

namespace pie_hip_driver {

// One sampling slot's sampler, fields as the reference's SamplerParams
// (driver/portable/src/sampler.hpp:41-51) but with the wire kind.
struct SlotSampler {
    uint8_t kind = PIE_SAMPLER_KIND_TOP_P;
    float temperature = 0.f;
    uint32_t top_k = 0;       // TopK / TopKTopP: k; Dist: number of entries (0 = whole vocabulary)
    float top_p = 1.f;
    float min_p = 0.f;
    uint32_t seed = 0;        // 0 = no caller seed
    uint32_t labels_begin = 0, labels_end = 0;   // range in BatchPlan::label_ids
};

struct BatchPlan {
    int R = 0;  // requests
    int N = 0;  // token rows
    std::vector<uint32_t> tokens;      // [N]
    std::vector<int32_t> positions;    // [N]
    std::vector<int64_t> kv_slots;     // [N] page*page_size + slot of the token's own K/V
    std::vector<uint32_t> row_page_begin;  // [N] first entry of the row's page list
    std::vector<int32_t> row_kv_len;       // [N] keys visible to the row: min(seq_len, pos+1)
    std::vector<int32_t> seq_len;          // [R]
    std::vector<int32_t> qo_indptr;        // [R+1] token rows of each request
    std::vector<uint32_t> page_indices;    // copy of the wire list (uploaded as is)
    std::vector<int32_t> sample_rows;      // global token rows to sample, request-major
    std::vector<int32_t> sample_indptr;    // [R+1]
    std::vector<SlotSampler> slot_samplers;  // one per sample row
    std::vector<uint32_t> label_ids;         // Logprob / Logprobs labels of all slots
    std::vector<std::vector<uint32_t>> logit_mask_runs;  // [R] BRLE runs (empty = no constraint)
    std::vector<std::vector<uint32_t>> draft_tokens;     // [R] speculative drafts to verify
    std::vector<std::vector<uint32_t>> row_mask_runs;    // [N] when has_user_masks: BRLE runs per token row
    int max_kv_len = 0;
    bool pure_decode = false;  // every request has exactly one token row, no user masks
    bool all_greedy = false;   // every sampling slot is a token sampler with temperature ~ 0
    bool has_user_masks = false;
};

inline std::int64_t physical_idx(const uint32_t* page_indices, int indptr_off, int page_size,
                                 int pos) {
    const int page = static_cast<int>(page_indices[indptr_off + pos / page_size]);
    return static_cast<std::int64_t>(page) * page_size + pos % page_size;
}

// True when every per-token mask is the runtime-synthesised causal one: runs [0, pos+1].
inline bool masks_are_synthesised_causal(const PieForwardRequestDesc& f) {
    const size_t n = f.token_ids.len;
    if (f.masks.len == 0) return true;
    if (f.masks.len != n) return false;
    for (size_t i = 0; i < n; ++i) {
        const PieBrleDesc& m = f.masks.ptr[i];
        if (m.buffer.len != 2) return false;
        if (m.buffer.ptr[0] != 0u || m.buffer.ptr[1] != f.position_ids.ptr[i] + 1u) return false;
    }
    return true;
}

// Token-producing sampler kinds on the wire (Multinomial, TopK, TopP, MinP, TopKTopP).
inline bool sampler_is_token_kind(uint8_t kind) { return kind <= PIE_SAMPLER_KIND_TOP_K_TOP_P; }

// Wire sampler -> per-slot parameters; fields a variant does not carry take the neutral value.
inline SlotSampler slot_sampler_of(const PieSamplerDesc& s, std::vector<uint32_t>& label_ids) {
    SlotSampler o;
    o.kind = s.kind;
    o.temperature = s.temperature;
    o.seed = s.seed;
    switch (s.kind) {
        case PIE_SAMPLER_KIND_TOP_K: o.top_k = s.k; break;
        case PIE_SAMPLER_KIND_TOP_P: o.top_p = s.p; break;
        case PIE_SAMPLER_KIND_MIN_P: o.min_p = s.p; break;
        case PIE_SAMPLER_KIND_TOP_K_TOP_P: o.top_k = s.k; o.top_p = s.p; break;
        case PIE_SAMPLER_KIND_DIST: o.top_k = s.num_tokens; break;
        default: break;
    }
    o.labels_begin = static_cast<uint32_t>(label_ids.size());
    if (s.kind == PIE_SAMPLER_KIND_LOGPROB) label_ids.push_back(s.token_id);
    else if (s.kind == PIE_SAMPLER_KIND_LOGPROBS)
        label_ids.insert(label_ids.end(), s.token_ids.ptr, s.token_ids.ptr + s.token_ids.len);
    o.labels_end = static_cast<uint32_t>(label_ids.size());
    return o;
}

inline BatchPlan plan_forward(const PieForwardRequestDesc& f, int page_size, int total_pages) {
    BatchPlan p;
    if (f.qo_indptr.len < 2) throw std::runtime_error("plan: no requests in batch");
    const int R = static_cast<int>(f.qo_indptr.len) - 1;
    const size_t n_plus_1 = static_cast<size_t>(R) + 1;
    if (f.context_ids.len != 0 && f.context_ids.len != static_cast<size_t>(R))
        throw std::runtime_error("plan: context_ids length must equal num_requests");
    if (f.token_ids.len != f.position_ids.len)
        throw std::runtime_error("plan: token_ids/position_ids size mismatch");
    if (f.kv_page_indptr.len != n_plus_1)
        throw std::runtime_error("plan: kv_page_indptr length must be num_requests+1");
    if (f.kv_last_page_lens.len != static_cast<size_t>(R))
        throw std::runtime_error("plan: kv_last_page_lens length must equal num_requests");
    if (f.sampling_indptr.len != n_plus_1)
        throw std::runtime_error("plan: sampling_indptr length must be num_requests+1");
    if (f.sampler_indptr.len != n_plus_1)
        throw std::runtime_error("plan: request_num_samplers length mismatch");
    if (f.rs_slot_ids.len != 0 && f.rs_slot_ids.len != static_cast<size_t>(R))
        throw std::runtime_error("plan: rs_slot_ids length must equal num_requests");
    if (f.rs_slot_flags.len != 0 && f.rs_slot_flags.len != static_cast<size_t>(R))
        throw std::runtime_error("plan: rs_slot_flags length must equal num_requests");
    const int N = static_cast<int>(f.token_ids.len);
    if (static_cast<int>(f.qo_indptr.ptr[R]) != N || f.qo_indptr.ptr[0] != 0)
        throw std::runtime_error("plan: qo_indptr must span token_ids");
    if (f.kv_page_indptr.ptr[R] > f.kv_page_indices.len)
        throw std::runtime_error("plan: kv_page_indptr exceeds kv_page_indices");
    if (f.sampling_indptr.ptr[R] > f.sampling_indices.len)
        throw std::runtime_error("plan: sampling_indptr exceeds sampling_indices");
    if (f.sampler_indptr.ptr[R] > f.samplers.len)
        throw std::runtime_error("plan: sampler_indptr exceeds samplers");

    p.R = R;
    p.N = N;
    p.tokens.assign(f.token_ids.ptr, f.token_ids.ptr + N);
    p.positions.resize(N);
    p.kv_slots.resize(N);
    p.row_page_begin.resize(N);
    p.row_kv_len.resize(N);
    p.seq_len.resize(R);
    p.qo_indptr.assign(f.qo_indptr.ptr, f.qo_indptr.ptr + R + 1);
    p.page_indices.assign(f.kv_page_indices.ptr, f.kv_page_indices.ptr + f.kv_page_indices.len);
    p.sample_indptr.assign(1, 0);
    p.logit_mask_runs.resize(R);
    p.draft_tokens.resize(R);
    const bool has_logit_masks = f.logit_mask_indptr.len == n_plus_1;
    const bool has_drafts = f.spec_indptr.len == n_plus_1;
    if (has_logit_masks && f.logit_mask_indptr.ptr[R] > f.logit_masks.len)
        throw std::runtime_error("plan: logit_mask_indptr exceeds logit_masks");
    if (has_drafts && (f.spec_indptr.ptr[R] > f.spec_token_ids.len ||
                       f.spec_indptr.ptr[R] > f.spec_position_ids.len))
        throw std::runtime_error("plan: spec_indptr exceeds the draft arrays");
    p.has_user_masks = !masks_are_synthesised_causal(f);
    if (p.has_user_masks) {
        // one BRLE per token row over its keys [0, position]; no runs = plain causal
        // (driver/portable/src/plan.cpp:54-94, :296-334)
        if (f.masks.len != static_cast<size_t>(N))
            throw std::runtime_error("plan: custom attention masks must be one per token row");
        p.row_mask_runs.resize(N);
        for (int i = 0; i < N; ++i) {
            const PieBrleDesc& m = f.masks.ptr[i];
            p.row_mask_runs[i].assign(m.buffer.ptr, m.buffer.ptr + m.buffer.len);
        }
    }
    p.pure_decode = !p.has_user_masks;
    p.all_greedy = true;

    for (int r = 0; r < R; ++r) {
        const int qo_start = static_cast<int>(f.qo_indptr.ptr[r]);
        const int qo_end = static_cast<int>(f.qo_indptr.ptr[r + 1]);
        const int n_tok = qo_end - qo_start;
        if (n_tok <= 0) throw std::runtime_error("plan: request " + std::to_string(r) + " has zero tokens");
        if (n_tok != 1) p.pure_decode = false;
        const int pages_off = static_cast<int>(f.kv_page_indptr.ptr[r]);
        const int num_pages = static_cast<int>(f.kv_page_indptr.ptr[r + 1]) - pages_off;
        if (num_pages < 0) throw std::runtime_error("plan: kv_page_indptr must be non-decreasing");
        const int last_len = static_cast<int>(f.kv_last_page_lens.ptr[r]);
        if (last_len > page_size)
            throw std::runtime_error("plan: request " + std::to_string(r) + " last page length exceeds page size");
        const int seq_len = num_pages > 0 ? (num_pages - 1) * page_size + last_len : 0;
        if (seq_len <= 0) throw std::runtime_error("plan: request " + std::to_string(r) + " has empty KV state");
        p.seq_len[r] = seq_len;
        for (int pi = 0; pi < num_pages; ++pi) {
            const uint32_t pg = f.kv_page_indices.ptr[pages_off + pi];
            if (pg >= static_cast<uint32_t>(total_pages))
                throw std::runtime_error("plan: page id " + std::to_string(pg) + " out of bounds (total_pages=" +
                                         std::to_string(total_pages) + ")");
        }
        const int n_samplers = static_cast<int>(f.sampler_indptr.ptr[r + 1] - f.sampler_indptr.ptr[r]);
        const int s_start = static_cast<int>(f.sampling_indptr.ptr[r]);
        const int s_end = static_cast<int>(f.sampling_indptr.ptr[r + 1]);
        const int n_slots = s_end - s_start;
        const bool prefill_only = n_samplers == 0;
        if (n_slots < (prefill_only ? 0 : 1) || (prefill_only && n_slots != 0))
            throw std::runtime_error("plan: request " + std::to_string(r) + " has " + std::to_string(n_samplers) +
                                     " sampler slot(s) but " + std::to_string(n_slots) + " wire sampling indices");
        if (!prefill_only && n_samplers != n_slots && n_samplers != 1)
            throw std::runtime_error("plan: request " + std::to_string(r) + " sampler/slot count mismatch");
        for (int i = qo_start; i < qo_end; ++i) {
            const int pos = static_cast<int>(f.position_ids.ptr[i]);
            if (pos < 0 || pos >= seq_len)
                throw std::runtime_error("plan: request " + std::to_string(r) + " token at position " +
                                         std::to_string(pos) + " exceeds seq_len " + std::to_string(seq_len));
            p.positions[i] = pos;
            p.kv_slots[i] = physical_idx(f.kv_page_indices.ptr, pages_off, page_size, pos);
            p.row_page_begin[i] = static_cast<uint32_t>(pages_off);
            p.row_kv_len[i] = pos + 1 < seq_len ? pos + 1 : seq_len;
            if (p.row_kv_len[i] > p.max_kv_len) p.max_kv_len = p.row_kv_len[i];
        }
        for (int k = s_start; k < s_end; ++k) {
            const int rel = static_cast<int>(f.sampling_indices.ptr[k]);
            if (rel < 0 || rel >= n_tok)
                throw std::runtime_error("plan: request " + std::to_string(r) + " sampling_index " +
                                         std::to_string(rel) + " out of relative [0," + std::to_string(n_tok) + ")");
            p.sample_rows.push_back(qo_start + rel);
            const size_t si = f.sampler_indptr.ptr[r] + (n_samplers == n_slots ? static_cast<size_t>(k - s_start) : 0);
            const PieSamplerDesc& s = f.samplers.ptr[si];
            if (!sampler_is_token_kind(s.kind) || !(s.temperature <= 1e-5f)) p.all_greedy = false;
            p.slot_samplers.push_back(slot_sampler_of(s, p.label_ids));
        }
        if (has_drafts && !prefill_only) {
            // each draft is verified at the row holding its position; the extra slots reuse the
            // request's first sampler
            const uint32_t d0 = f.spec_indptr.ptr[r], d1 = f.spec_indptr.ptr[r + 1];
            for (uint32_t k = d0; k < d1; ++k) {
                const int draft_pos = static_cast<int>(f.spec_position_ids.ptr[k]);
                int idx = -1;
                for (int i = qo_start; i < qo_end; ++i)
                    if (static_cast<int>(f.position_ids.ptr[i]) == draft_pos) {
                        idx = i;
                        break;
                    }
                if (idx < 0)
                    throw std::runtime_error("plan: spec draft at position " + std::to_string(draft_pos) +
                                             " not found in request " + std::to_string(r) + "'s qo range");
                p.draft_tokens[r].push_back(f.spec_token_ids.ptr[k]);
                p.sample_rows.push_back(idx);
                const PieSamplerDesc& s = f.samplers.ptr[f.sampler_indptr.ptr[r]];
                if (!sampler_is_token_kind(s.kind) || !(s.temperature <= 1e-5f)) p.all_greedy = false;
                p.slot_samplers.push_back(slot_sampler_of(s, p.label_ids));
            }
        }
        if (has_logit_masks && !prefill_only) {
            for (uint32_t i = f.logit_mask_indptr.ptr[r]; i < f.logit_mask_indptr.ptr[r + 1]; ++i) {
                const PieBrleDesc& b = f.logit_masks.ptr[i];
                p.logit_mask_runs[r].insert(p.logit_mask_runs[r].end(), b.buffer.ptr,
                                            b.buffer.ptr + b.buffer.len);
            }
            if (!p.logit_mask_runs[r].empty()) p.all_greedy = false;
        }
        p.sample_indptr.push_back(static_cast<int32_t>(p.sample_rows.size()));
    }
    return p;
}

}  // namespace pie_hip_driver
