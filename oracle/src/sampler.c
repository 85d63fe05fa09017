/*
 * Oracle: the host sampler suite.  TEST INFRASTRUCTURE ONLY (see oracle_common.h).
 *
 * Follows driver/portable/src/sampler.cpp:
 *   - Pcg32 (:31-57): PCG-XSH-RR 64/32 with the canonical two-step seeding, default stream
 *     0xda3e39cb94b95bdb; next_uniform = top 24 bits / 2^24.
 *   - softmax_with_temperature (:69-87): max, e = expf((l - max) * (1 / max(T, 1e-5))), the sum
 *     of e accumulated in double in index order, p = e * float(1 / max(1e-30, sum)).
 *   - sample_token (:345-409): T <= 1e-5 -> first-index argmax; Multinomial walks the
 *     distribution in index order with a float running sum until u < acc (argmax of the
 *     probabilities when the walk ends without a hit); the filtered kinds take the entries with
 *     p > 0 in descending order of p, keep the first top_k of them (TopK, TopKTopP; 0 = all),
 *     then the shortest prefix whose float running sum reaches clamp(top_p, 0, 1) (TopP,
 *     TopKTopP; top_p >= 1 keeps all), or the entries with p >= min_p * p_max (MinP; none
 *     passing keeps all); total = double sum of the kept p; the token is the first kept entry
 *     whose float running sum exceeds u * float(total), the last kept entry if none does.
 *   - apply_brle_logit_mask (:169-198), run_distribution (:224-251), run_logprob(s) (:262-292),
 *     run_entropy (:294-306), log_softmax (:205-222, double sum of exp(double(l - max))).
 * The reference sorts with std::sort / std::partial_sort, which leave the order of equal
 * probabilities unspecified; here equal probabilities are ordered by ascending token id.
 *
 * orc_sample_token also reports `margin`: the smallest distance (in probability mass; relative
 * for the min-p threshold test) between any comparison that decided the outcome and its
 * flipping point, so a caller comparing against
 * an implementation with different float summation order can set near-boundary draws aside.
 *
 * Pinned by tests/test_oracle_sampler.py: the published PCG32 demo sequence (seed 42, stream
 * 54), scipy's softmax / log_softmax / entropy, argmax limits (T -> 0, top_k = 1, tiny top_p),
 * hand-worked top-p / min-p prefixes, sample frequencies against the probabilities
 * (chi-square), and the reference's BRLE known answers (driver/cuda/tests/test_brle.cpp).
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "oracle_api.h"

typedef struct {
    uint64_t state, inc;
} OrcPcg32;

static uint32_t pcg32_next(OrcPcg32* r) {
    const uint64_t old = r->state;
    r->state = old * 6364136223846793005ULL + r->inc;
    const uint32_t xorshifted = (uint32_t)(((old >> 18u) ^ old) >> 27u);
    const uint32_t rot = (uint32_t)(old >> 59u);
    return (xorshifted >> rot) | (xorshifted << ((32u - rot) & 31u));
}

static void pcg32_init(OrcPcg32* r, uint64_t seed, uint64_t stream) {
    r->state = 0;
    r->inc = (stream << 1u) | 1u;
    pcg32_next(r);
    r->state += seed;
    pcg32_next(r);
}

void orc_pcg32_sequence(uint64_t seed, uint64_t stream, uint32_t* out, int n) {
    OrcPcg32 r;
    pcg32_init(&r, seed, stream);
    for (int i = 0; i < n; ++i) out[i] = pcg32_next(&r);
}

float orc_pcg32_first_uniform(uint64_t seed) {
    OrcPcg32 r;
    pcg32_init(&r, seed, 0xda3e39cb94b95bdbULL);
    return (float)(pcg32_next(&r) >> 8) * (1.0f / 16777216.0f);
}

void orc_apply_brle_logit_mask(float* logits, int V, const uint32_t* runs, size_t n_runs) {
    if (n_runs == 0) return;
    int is_true = 0;
    int64_t pos = 0;
    for (size_t i = 0; i < n_runs && pos < V; ++i) {
        int64_t end = pos + (int64_t)runs[i];
        if (end > V) end = V;
        if (!is_true)
            for (int64_t v = pos; v < end; ++v) logits[v] = -INFINITY;
        pos = end;
        is_true = !is_true;
    }
    for (int64_t v = pos; v < V; ++v) logits[v] = -INFINITY;
}

void orc_softmax_temperature(const float* logits, int V, float temperature, float* probs) {
    float mx = logits[0];
    for (int v = 1; v < V; ++v)
        if (logits[v] > mx) mx = logits[v];
    const float inv_t = 1.0f / (temperature > 1e-5f ? temperature : 1e-5f);
    double sum = 0.0;
    for (int v = 0; v < V; ++v) {
        const float e = expf((logits[v] - mx) * inv_t);
        probs[v] = e;
        sum += e;
    }
    const float inv_sum = (float)(1.0 / (sum > 1e-30 ? sum : 1e-30));
    for (int v = 0; v < V; ++v) probs[v] *= inv_sum;
}

static uint32_t argmax_f32(const float* x, int V) {
    int best = 0;
    float bv = x[0];
    for (int v = 1; v < V; ++v)
        if (x[v] > bv) {
            bv = x[v];
            best = v;
        }
    return (uint32_t)best;
}

typedef struct {
    float p;
    uint32_t id;
} Cand;

static int cand_desc(const void* a, const void* b) {
    const Cand* x = (const Cand*)a;
    const Cand* y = (const Cand*)b;
    if (x->p > y->p) return -1;
    if (x->p < y->p) return 1;
    return x->id < y->id ? -1 : (x->id > y->id ? 1 : 0);
}

static void note(float* margin, double d) {
    if (d < 0) d = -d;
    if (d < *margin) *margin = (float)d;
}

/* kind: wire order (0 Multinomial, 1 TopK, 2 TopP, 3 MinP, 4 TopKTopP).  Returns 0, or -1 for a
 * kind that produces no token. */
int orc_sample_token(const float* logits, int V, int kind, float temperature, uint32_t top_k,
                     float top_p, float min_p, float u, uint32_t* token, float* margin) {
    float mg = INFINITY;
    if (kind < 0 || kind > 4) return -1;
    if (temperature <= 1e-5f) {
        *token = argmax_f32(logits, V);
        if (margin) *margin = mg;
        return 0;
    }
    float* probs = (float*)malloc((size_t)V * sizeof(float));
    orc_softmax_temperature(logits, V, temperature, probs);
    if (kind == 0) {
        float acc = 0.f;
        int hit = -1;
        for (int v = 0; v < V; ++v) {
            const float before = acc;
            acc += probs[v];
            if (u < acc) {
                hit = v;
                note(&mg, (double)acc - u);
                note(&mg, (double)u - before);
                break;
            }
        }
        if (hit < 0) {
            note(&mg, (double)u - acc);
            hit = (int)argmax_f32(probs, V);
        }
        *token = (uint32_t)hit;
        free(probs);
        if (margin) *margin = mg;
        return 0;
    }
    Cand* c = (Cand*)malloc((size_t)V * sizeof(Cand));
    size_t n = 0;
    for (int v = 0; v < V; ++v)
        if (probs[v] > 0.0f) {
            c[n].p = probs[v];
            c[n].id = (uint32_t)v;
            ++n;
        }
    free(probs);
    if (n == 0) {
        *token = 0;
        free(c);
        if (margin) *margin = 0.f;
        return 0;
    }
    qsort(c, n, sizeof(Cand), cand_desc);
    size_t keep = n;
    const int wants_k = kind == 1 || kind == 4, wants_p = kind == 2 || kind == 4, wants_m = kind == 3;
    if (wants_k && top_k != 0 && top_k < keep) keep = top_k;
    if (wants_p) {
        float thr = top_p < 0.f ? 0.f : (top_p > 1.f ? 1.f : top_p);
        if (thr < 1.0f) {
            float cum = 0.f;
            size_t cut = keep;
            for (size_t i = 0; i < keep; ++i) {
                const float before = cum;
                cum += c[i].p;
                if (cum >= thr) {
                    cut = i + 1;
                    note(&mg, (double)cum - thr);
                    if (i > 0) note(&mg, (double)thr - before);
                    break;
                }
            }
            if (cut == keep && cum < thr) note(&mg, (double)thr - cum);
            keep = cut;
        }
    }
    if (wants_m) {
        const float thr = min_p * c[0].p;
        size_t cut = 0;
        for (; cut < keep; ++cut)
            if (c[cut].p < thr) break;
        if (cut > 0) {
            /* p and thr are single float products on both sides: what matters is their
             * relative distance against a last-bit difference in p */
            note(&mg, ((double)c[cut - 1].p - thr) / c[cut - 1].p);
            if (cut < keep) note(&mg, ((double)thr - c[cut].p) / thr);
            keep = cut;
        }
    }
    double total = 0.0;
    for (size_t i = 0; i < keep; ++i) total += c[i].p;
    if (total <= 0.0) {
        *token = c[0].id;
    } else {
        const float x = u * (float)total;
        float acc = 0.f;
        uint32_t tok = c[keep - 1].id;
        int found = 0;
        for (size_t i = 0; i < keep; ++i) {
            const float before = acc;
            acc += c[i].p;
            if (x < acc) {
                tok = c[i].id;
                note(&mg, (double)acc - x);
                if (i > 0) note(&mg, (double)x - before);
                found = 1;
                break;
            }
        }
        if (!found) note(&mg, (double)x - acc);
        *token = tok;
    }
    free(c);
    if (margin) *margin = mg;
    return 0;
}

/* Distribution sampler: the k most probable tokens at `temperature`, descending (k = 0: the
 * whole vocabulary).  Returns the number of entries written. */
int orc_distribution(const float* logits, int V, float temperature, uint32_t k, uint32_t* ids,
                     float* vals) {
    float* probs = (float*)malloc((size_t)V * sizeof(float));
    orc_softmax_temperature(logits, V, temperature, probs);
    Cand* c = (Cand*)malloc((size_t)V * sizeof(Cand));
    for (int v = 0; v < V; ++v) {
        c[v].p = probs[v];
        c[v].id = (uint32_t)v;
    }
    qsort(c, (size_t)V, sizeof(Cand), cand_desc);
    const int n = (k > 0 && k < (uint32_t)V) ? (int)k : V;
    for (int i = 0; i < n; ++i) {
        ids[i] = c[i].id;
        vals[i] = c[i].p;
    }
    free(c);
    free(probs);
    return n;
}

static float lse_f32(const float* logits, int V, float* max_out) {
    float mx = logits[0];
    for (int v = 1; v < V; ++v)
        if (logits[v] > mx) mx = logits[v];
    double sum = 0.0;
    for (int v = 0; v < V; ++v) sum += exp((double)(logits[v] - mx));
    if (max_out) *max_out = mx;
    return mx + (float)log(sum > 1e-30 ? sum : 1e-30);
}

/* Logprob / Logprobs: log_softmax(logits)[label].  Returns -1 when a label is outside the
 * vocabulary (the reference throws). */
int orc_logprobs_at(const float* logits, int V, const uint32_t* labels, int n, float* out) {
    const float lse = lse_f32(logits, V, NULL);
    for (int i = 0; i < n; ++i) {
        if (labels[i] >= (uint32_t)V) return -1;
        out[i] = logits[labels[i]] - lse;
    }
    return 0;
}

float orc_entropy(const float* logits, int V) {
    const float lse = lse_f32(logits, V, NULL);
    double h = 0.0;
    for (int v = 0; v < V; ++v) {
        const float lp = logits[v] - lse;
        const double p = exp((double)lp);
        h -= p * lp;
    }
    return (float)h;
}
