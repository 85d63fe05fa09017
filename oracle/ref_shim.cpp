// C entry points over the reference's OWN host sampler and BRLE decoder, compiled from the
// reference tree where it lies (never copied): driver/portable/src/sampler.cpp and
// driver/cuda/src/brle.cpp.  TEST INFRASTRUCTURE ONLY — built by oracle/build_ref.py into
// oracle/_ref/libpie_ref.so and used by tests to pin oracle/src/sampler.c and the BRLE
// restatements against the real thing.  Nothing here restates an algorithm: every function
// forwards to the reference's declaration in sampler.hpp / brle.hpp.
#include <cstdint>
#include <cstring>
#include <span>
#include <vector>

#include "brle.hpp"      // /root/reference/driver/cuda/src
#include "sampler.hpp"   // /root/reference/driver/portable/src

namespace ps = pie_portable_driver;

namespace {
// The oracle numbers the token samplers in wire order 0..4 (Multinomial, TopK, TopP, MinP,
// TopKTopP); the reference's enum is that plus one, with Distribution = 0.
ps::SamplerParams make_params(int kind, float temperature, uint32_t top_k, float top_p, float min_p,
                              uint32_t seed) {
    ps::SamplerParams p;
    p.type = static_cast<ps::SamplerType>(kind);
    p.temperature = temperature;
    p.top_k = top_k;
    p.top_p = top_p;
    p.min_p = min_p;
    p.seed = seed;
    return p;
}
}  // namespace

extern "C" {

// sample_token (sampler.cpp:345-409).  `type` is the reference's SamplerType value (1..5).
// Returns 0 and the token, or -1 when the reference throws.
int ref_sample_token(const float* logits, int vocab, int type, float temperature, uint32_t top_k,
                     float top_p, float min_p, uint32_t seed, uint32_t* token) {
    try {
        *token = ps::sample_token(logits, vocab, make_params(type, temperature, top_k, top_p, min_p, seed));
        return 0;
    } catch (...) {
        return -1;
    }
}

// sample_slot for Distribution (type 0): ids / vals must hold `vocab` entries; returns the count.
int ref_distribution(const float* logits, int vocab, float temperature, uint32_t k, uint32_t* ids,
                     float* vals) {
    try {
        ps::SlotOutput out;
        ps::sample_slot(logits, vocab, make_params(0, temperature, k, 1.0f, 0.0f, 1), out);
        std::memcpy(ids, out.dist_ids.data(), out.dist_ids.size() * sizeof(uint32_t));
        std::memcpy(vals, out.dist_vals.data(), out.dist_vals.size() * sizeof(float));
        return static_cast<int>(out.dist_ids.size());
    } catch (...) {
        return -1;
    }
}

// sample_slot for Logprob / Logprobs (types 8 / 9).
int ref_logprobs(const float* logits, int vocab, const uint32_t* labels, int n, float* out_lp) {
    try {
        ps::SamplerParams p = make_params(n == 1 ? 8 : 9, 1.0f, 0, 1.0f, 0.0f, 1);
        p.labels.assign(labels, labels + n);
        ps::SlotOutput out;
        ps::sample_slot(logits, vocab, p, out);
        std::memcpy(out_lp, out.logprobs.data(), out.logprobs.size() * sizeof(float));
        return static_cast<int>(out.logprobs.size());
    } catch (...) {
        return -1;
    }
}

// sample_slot for Entropy (type 10).
int ref_entropy(const float* logits, int vocab, float* h) {
    try {
        ps::SlotOutput out;
        ps::sample_slot(logits, vocab, make_params(10, 1.0f, 0, 1.0f, 0.0f, 1), out);
        *h = out.entropy;
        return out.has_entropy ? 0 : -1;
    } catch (...) {
        return -1;
    }
}

// sample_token_from_topk (the batch shortcut's host finalize, sampler.cpp:411-).
int ref_sample_token_from_topk(const int32_t* top_idx, const float* top_probs, int K, int type,
                               float temperature, uint32_t top_k, float top_p, float min_p, uint32_t seed,
                               uint64_t seed_xor, uint32_t* token) {
    try {
        *token = ps::sample_token_from_topk(top_idx, top_probs, K,
                                            make_params(type, temperature, top_k, top_p, min_p, seed), seed_xor);
        return 0;
    } catch (...) {
        return -1;
    }
}

void ref_apply_brle_logit_mask(float* logits, int vocab, const uint32_t* runs, size_t n_runs) {
    ps::apply_brle_logit_mask(logits, vocab, runs, n_runs);
}

// brle::is_pure_causal (driver/cuda/src/brle.cpp).  R requests; mask_indptr has tokens + 1 entries.
int ref_brle_is_pure_causal(const uint32_t* masks, size_t n_masks, const uint32_t* mask_indptr,
                            size_t n_mask_indptr, const uint32_t* qo_indptr, const uint32_t* kv_page_indptr,
                            const uint32_t* kv_last_page_lens, int R, int page_size) {
    namespace b = pie_cuda_driver::brle;
    try {
        return b::is_pure_causal({masks, n_masks}, {mask_indptr, n_mask_indptr},
                                 {qo_indptr, static_cast<size_t>(R + 1)},
                                 {kv_page_indptr, static_cast<size_t>(R + 1)},
                                 {kv_last_page_lens, static_cast<size_t>(R)}, page_size)
                   ? 1 : 0;
    } catch (...) {
        return -1;
    }
}

// brle::decode: the packed per-request bitmaps.  Call with packed = NULL for the sizes (returns
// packed bytes), then with buffers.  out_indptr holds R + 1 entries.  -1 when the reference throws.
long ref_brle_decode(const uint32_t* masks, size_t n_masks, const uint32_t* mask_indptr, size_t n_mask_indptr,
                     const uint32_t* qo_indptr, const uint32_t* kv_page_indptr, const uint32_t* kv_last_page_lens,
                     int R, int page_size, uint8_t* packed, int32_t* out_indptr, int* pure_causal) {
    namespace b = pie_cuda_driver::brle;
    try {
        const b::DecodedMasks d = b::decode({masks, n_masks}, {mask_indptr, n_mask_indptr},
                                            {qo_indptr, static_cast<size_t>(R + 1)},
                                            {kv_page_indptr, static_cast<size_t>(R + 1)},
                                            {kv_last_page_lens, static_cast<size_t>(R)}, page_size);
        if (packed) std::memcpy(packed, d.packed.data(), d.packed.size());
        if (out_indptr) std::memcpy(out_indptr, d.mask_indptr.data(), d.mask_indptr.size() * sizeof(int32_t));
        if (pure_causal) *pure_causal = d.pure_causal ? 1 : 0;
        return static_cast<long>(d.packed.size());
    } catch (...) {
        return -1;
    }
}

}  // extern "C"
