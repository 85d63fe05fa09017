/*
 * Oracle: paged-KV attention and KV page writes.  TEST INFRASTRUCTURE ONLY
 * (see oracle_common.h).
 *
 * Follows the reference's hand-written paged kernels:
 *   decode (one query per request)  driver/cuda/src/ops/attention_naive_paged.cu:319-447
 *   prefill / mixed, causal limit   driver/cuda/src/ops/attention_naive_paged.cu:148-317
 *   KV page write                   driver/cuda/src/kernels/kv_paged.cu:28-80
 * KV pool layout [num_pages, page_size, num_kv_heads, head_dim] bf16
 * (driver/cuda/src/kv_cache.hpp:3-8); element address
 * ((page*page_size + slot)*hk + h)*d + j, the same address the portable driver's
 * per-slot rows give (driver/portable/src/kv_cache.hpp:5-17).
 *
 *   custom masks                    driver/portable/src/plan.cpp:54-94 (build_attn_mask_f16):
 *                                   key j is visible to a token at position p iff
 *                                   max(0, p - window + 1) <= j <= min(n_kv - 1, p) and, when
 *                                   the token carries BRLE runs, j lies in a true run (runs
 *                                   alternate false/true from position 0; a mask cannot unmask
 *                                   the future or reach past its last run)
 *
 * Pinned by tests/test_oracle_attention.py: dense numpy fp64 softmax attention over
 * the gathered rows, page-permutation invariance, forked-prefix equality, the LSE
 * definition, the zero-length case, the causal limit on small brute-force cases, and masked
 * rows against dense attention over the allowed keys only.
 */
#include <stdlib.h>
#include <string.h>

#include "oracle_common.h"

void orc_attn_rows_masked(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                          float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                          const uint32_t* row_begin, const int32_t* row_len, int rows, int hq,
                          int hk, int d, int ps, float sm_scale, int mode, const uint8_t* allow,
                          const int64_t* allow_off);

static int orc_kv_len(const uint32_t* indptr, const uint32_t* last_lens, int r, int ps) {
    const int pages = (int)(indptr[r + 1] - indptr[r]);
    /* attention_naive_paged.cu:349-352, with the empty page list made explicit */
    return pages > 0 ? (pages - 1) * ps + (int)last_lens[r] : 0;
}

/*
 * One query row (all hq heads) over the first `lim` keys of the page list starting at
 * page_indices[pg_lo].  mode 0: fp32 two-pass softmax in the reference's order
 * (attention_naive_paged.cu:362-447); mode 2: fp64.
 */
/* K / V element: bf16 pool, or (kv_f32) a pool of already dequantised f32 values — the
 * float(code) * scale of load_kv_scalar, attention_naive_paged.cu:56-112 */
static inline float orc_kv_at(const void* pages, int kv_f32, size_t idx) {
    return kv_f32 ? ((const float*)pages)[idx] : orc_bf16_to_f32(((const uint16_t*)pages)[idx]);
}

static void orc_attn_row(const uint16_t* q_row, const void* k_pages, const void* v_pages, int kv_f32,
                         float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                         uint32_t pg_lo, int lim, int hq, int hk, int d, int ps, float scale,
                         int mode, double* w, const uint8_t* allow) {
    const int gqa = hq / hk;
    for (int h = 0; h < hq; ++h) {
        const int kvh = h / gqa;
        const size_t qoff = (size_t)h * d;
        double row_max = -INFINITY;
        for (int j = 0; j < lim; ++j) {
            const uint32_t pid = page_indices[pg_lo + j / ps];
            const size_t koff = (((size_t)pid * ps + j % ps) * hk + kvh) * d;
            double dot;
            if (mode == 0) {
                float f = 0.f;
                for (int e = 0; e < d; ++e)
                    f += orc_bf16_to_f32(q_row[qoff + e]) * orc_kv_at(k_pages, kv_f32, koff + e);
                dot = (double)(f * scale);
            } else {
                double f = 0.0;
                for (int e = 0; e < d; ++e)
                    f += (double)orc_bf16_to_f32(q_row[qoff + e]) *
                         (double)orc_kv_at(k_pages, kv_f32, koff + e);
                dot = f * (double)scale;
            }
            if (allow && !allow[j]) dot = -INFINITY;
            w[j] = dot;
            if (dot > row_max) row_max = dot;
        }
        if (row_max == -INFINITY) {   /* no visible key: zero output, lse = -inf */
            for (int e = 0; e < d; ++e) {
                o_f32[qoff + e] = 0.f;
                if (o_bf16) o_bf16[qoff + e] = 0;
            }
            if (lse) lse[h] = -INFINITY;
            continue;
        }
        double z = 0.0;
        float zf = 0.f;
        for (int j = 0; j < lim; ++j) {
            if (mode == 0) {
                const float e = expf((float)w[j] - (float)row_max);
                w[j] = (double)e;
                zf += e;
            } else {
                w[j] = exp(w[j] - row_max);
                z += w[j];
            }
        }
        if (mode == 0) z = (double)zf;
        for (int e = 0; e < d; ++e) {
            double acc = 0.0;
            float accf = 0.f;
            for (int j = 0; j < lim; ++j) {
                const uint32_t pid = page_indices[pg_lo + j / ps];
                const size_t voff = (((size_t)pid * ps + j % ps) * hk + kvh) * d;
                const float v = orc_kv_at(v_pages, kv_f32, voff + e);
                if (mode == 0) accf = fmaf(v, (float)w[j], accf);
                else acc += (double)v * w[j];
            }
            if (mode == 0) acc = (double)accf;
            float out;
            if (mode == 0) out = z > 0.0 ? (float)acc * (1.0f / (float)z) : 0.f;
            else out = z > 0.0 ? (float)(acc / z) : 0.f;
            o_f32[qoff + e] = out;
            if (o_bf16) o_bf16[qoff + e] = orc_f32_to_bf16(out);
        }
        if (lse) lse[h] = z > 0.0 ? (float)(log(z) + row_max) : -INFINITY;
    }
}

/*
 * General paged attention: request r owns query rows qo_indptr[r]..qo_indptr[r+1];
 * query i of n_q sees kv positions j < kv_len - n_q + i + 1 (attention_naive_paged.cu:194-198).
 * Decode is the n_q = 1 case (qo_indptr = 0,1,2,...).
 * o_f32 [T,hq,d] unrounded, o_bf16 optional, lse optional [T,hq] (natural log).
 */
void orc_attn_paged(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                    float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* qo_indptr,
                    const uint32_t* page_indices, const uint32_t* page_indptr,
                    const uint32_t* last_lens, int R, int hq, int hk, int d, int ps,
                    float sm_scale, int mode) {
    const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)d);
#pragma omp parallel for schedule(dynamic)
    for (int r = 0; r < R; ++r) {
        const int kv_total = orc_kv_len(page_indptr, last_lens, r, ps);
        const int q_lo = (int)qo_indptr[r], n_q = (int)qo_indptr[r + 1] - q_lo;
        double* w = (double*)malloc(sizeof(double) * (size_t)(kv_total > 0 ? kv_total : 1));
        for (int qi = 0; qi < n_q; ++qi) {
            int lim = kv_total - n_q + qi + 1;
            if (lim > kv_total) lim = kv_total;
            if (lim < 0) lim = 0;
            const size_t row = (size_t)(q_lo + qi) * hq;
            orc_attn_row(q + row * d, k_pages, v_pages, 0, o_f32 + row * d,
                         o_bf16 ? o_bf16 + row * d : NULL, lse ? lse + row : NULL, page_indices,
                         page_indptr[r], lim, hq, hk, d, ps, scale, mode, w, NULL);
        }
        free(w);
    }
}

/*
 * Attention over explicit per-row extents: row r reads the page list from
 * page_indices[row_begin[r]] and sees its first row_len[r] keys
 * (visible keys = min(seq_len, position+1), driver/portable/src/plan.cpp:54-94).
 */
void orc_attn_rows(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                   float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                   const uint32_t* row_begin, const int32_t* row_len, int rows, int hq, int hk,
                   int d, int ps, float sm_scale, int mode) {
    orc_attn_rows_masked(q, k_pages, v_pages, o_f32, o_bf16, lse, page_indices, row_begin, row_len,
                         rows, hq, hk, d, ps, sm_scale, mode, NULL, NULL);
}

/* The same with per-row visibility: row r's key j is visible iff allow[allow_off[r] + j] != 0
 * (allow_off[r] < 0 or allow == NULL: every key below row_len[r]). */
void orc_attn_rows_masked(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                          float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                          const uint32_t* row_begin, const int32_t* row_len, int rows, int hq,
                          int hk, int d, int ps, float sm_scale, int mode, const uint8_t* allow,
                          const int64_t* allow_off) {
    const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)d);
#pragma omp parallel for schedule(dynamic)
    for (int r = 0; r < rows; ++r) {
        const int lim = row_len[r] > 0 ? row_len[r] : 0;
        double* w = (double*)malloc(sizeof(double) * (size_t)(lim > 0 ? lim : 1));
        const size_t row = (size_t)r * hq;
        orc_attn_row(q + row * d, k_pages, v_pages, 0, o_f32 + row * d,
                     o_bf16 ? o_bf16 + row * d : NULL, lse ? lse + row : NULL, page_indices,
                     row_begin[r], lim, hq, hk, d, ps, scale, mode, w,
                     (allow && allow_off && allow_off[r] >= 0) ? allow + allow_off[r] : NULL);
        free(w);
    }
}

/* Visibility of keys 0..n_kv-1 for a token at position `pos` (build_attn_mask_f16,
 * driver/portable/src/plan.cpp:54-94).  n_runs == 0: the causal window alone. */
void orc_brle_allow(const uint32_t* runs, size_t n_runs, int pos, int n_kv, int window,
                    uint8_t* out) {
    memset(out, 0, (size_t)(n_kv > 0 ? n_kv : 0));
    const int hi = pos < n_kv - 1 ? pos : n_kv - 1;
    int lo = window > 0 ? pos - window + 1 : 0;
    if (lo < 0) lo = 0;
    if (n_runs == 0) {
        for (int j = lo; j <= hi; ++j) out[j] = 1;
        return;
    }
    int is_true = 0;
    int64_t p = 0;
    for (size_t k = 0; k < n_runs && p <= hi; ++k) {
        int64_t end = p + (int64_t)runs[k];
        if (end > hi + 1) end = hi + 1;
        if (is_true)
            for (int64_t j = p > lo ? p : lo; j < end; ++j) out[j] = 1;
        p = end;
        is_true = !is_true;
    }
}

/*
 * Scatter this step's K/V rows [T, hk, d] into the pages.  The slot of token t of request
 * r comes from the page table alone: pre_kv_len = kv_len - n_new, abs = pre_kv_len + offset
 * (kv_paged.cu:49-59).
 */
void orc_kv_write(const uint16_t* k_curr, const uint16_t* v_curr, uint16_t* k_pages,
                  uint16_t* v_pages, const uint32_t* qo_indptr, const uint32_t* page_indices,
                  const uint32_t* page_indptr, const uint32_t* last_lens, int R, int hk, int d,
                  int ps) {
    const size_t row = (size_t)hk * d;
    for (int r = 0; r < R; ++r) {
        const int q_lo = (int)qo_indptr[r], n_new = (int)qo_indptr[r + 1] - q_lo;
        const int kv_total = orc_kv_len(page_indptr, last_lens, r, ps);
        for (int i = 0; i < n_new; ++i) {
            const int abs_pos = kv_total - n_new + i;
            const uint32_t pid = page_indices[page_indptr[r] + abs_pos / ps];
            const size_t dst = ((size_t)pid * ps + abs_pos % ps) * row;
            memcpy(k_pages + dst, k_curr + (size_t)(q_lo + i) * row, row * 2);
            memcpy(v_pages + dst, v_curr + (size_t)(q_lo + i) * row, row * 2);
        }
    }
}


/* orc_attn_rows_masked over pools of dequantised f32 values (one-byte KV-cache formats). */
void orc_attn_rows_f32kv(const uint16_t* q, const float* k_pages, const float* v_pages,
                         float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                         const uint32_t* row_begin, const int32_t* row_len, int rows, int hq,
                         int hk, int d, int ps, float sm_scale, int mode, const uint8_t* allow,
                         const int64_t* allow_off) {
    const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)d);
#pragma omp parallel for schedule(dynamic)
    for (int r = 0; r < rows; ++r) {
        const int lim = row_len[r] > 0 ? row_len[r] : 0;
        double* w = (double*)malloc(sizeof(double) * (size_t)(lim > 0 ? lim : 1));
        const size_t row = (size_t)r * hq;
        orc_attn_row(q + row * d, k_pages, v_pages, 1, o_f32 + row * d,
                     o_bf16 ? o_bf16 + row * d : NULL, lse ? lse + row : NULL, page_indices,
                     row_begin[r], lim, hq, hk, d, ps, scale, mode, w,
                     (allow && allow_off && allow_off[r] >= 0) ? allow + allow_off[r] : NULL);
        free(w);
    }
}

/*
 * KV-cache quantisation of `rows` (token, head) rows of d bf16 values
 * (driver/cuda/src/kernels/kv_paged.cu:155-297).
 *   fmt 1 (fp8_e4m3):            code = e4m3_satfinite(x); scales untouched
 *   fmt 2 (int8_per_token_head): scale = absmax/127 (1 when absmax == 0), inv = 1/scale,
 *                                code = clamp(rintf(x * inv), -128, 127)
 *   fmt 3 (fp8_per_token_head):  scale = absmax/448 (1 when 0), code = e4m3_satfinite(x * inv)
 *   fmt 4 (fp8_e5m2):            code = e5m2_satfinite(x); scales untouched
 *   fmt 5 (fp4_e2m1 / nvfp4):    per block of 16 elements scale = absmax/6 (1 when 0), code =
 *                                the nearest of +-{0, .5, 1, 1.5, 2, 3, 4, 6} to x * (1/scale), the
 *                                smaller magnitude on a tie, sign bit set for x < 0; two codes per
 *                                byte, the even element in the low nibble
 *                                (write_kv_fp4_block_kernel, kv_paged.cu:292-417).  codes is
 *                                [rows, (d+1)/2], scales [rows, ceil(d/16)], and dequant holds
 *                                bf16(level * scale) — the value the reference's attention reads
 *                                after dequant_fp4_pages_active_kernel (kv_paged.cu:496-531)
 * dequant (optional, f32): float(code) * scale, as the attention kernels read it.
 */
uint8_t orc_f32_to_fp8_e4m3(float f);
float orc_fp8_e4m3_to_f32(uint8_t v);

/* e5m2 byte -> f32: the byte is the high half of an IEEE binary16 (1-5-2). */
float orc_fp8_e5m2_to_f32(uint8_t v) {
    const int sign = v >> 7, e = (v >> 2) & 0x1F, m = v & 3;
    float r;
    if (e == 0) r = ldexpf((float)m, -16);                 /* subnormals: m * 2^-16 */
    else if (e == 31) r = m ? NAN : INFINITY;
    else r = ldexpf(1.f + (float)m / 4.f, e - 15);
    return sign ? -r : r;
}

/* f32 -> e5m2, round to nearest even, saturating to +-57344 (__NV_SATFINITE); NaN -> 0x7F.
 * Nearest of the two neighbouring codes, the even code on a tie — found by search over the 124
 * finite magnitudes, so the rule is the definition itself. */
uint8_t orc_f32_to_fp8_e5m2(float f) {
    if (f != f) return 0x7F;
    const uint8_t sign = signbit(f) ? 0x80 : 0;
    const float a = fabsf(f);
    if (a >= 57344.f) return (uint8_t)(sign | 0x7B);
    int best = 0;
    float best_err = a;
    for (int c = 1; c <= 0x7B; ++c) {
        const float err = fabsf(orc_fp8_e5m2_to_f32((uint8_t)c) - a);
        if (err < best_err || (err == best_err && (c & 1) == 0)) {
            best = c;
            best_err = err;
        }
    }
    return (uint8_t)(sign | best);
}

void orc_fp8_e5m2_decode(const uint8_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_fp8_e5m2_to_f32(src[i]);
}
void orc_fp8_e5m2_encode(const float* src, uint8_t* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_fp8_e5m2(src[i]);
}

float orc_fp4_e2m1_value(uint8_t code) {
    static const float levels[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
    const float v = levels[code & 7];
    return (code & 8) ? -v : v;
}
uint8_t orc_fp4_e2m1_quant(float x) {
    static const float levels[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
    const float ax = fabsf(x);
    int best = 0;
    float best_err = fabsf(ax - levels[0]);
    for (int i = 1; i < 8; ++i) {
        const float err = fabsf(ax - levels[i]);
        if (err < best_err) {
            best_err = err;
            best = i;
        }
    }
    return (uint8_t)((x < 0.f ? 8 : 0) | best);
}

static void orc_kv_quant_rows_fp4(const uint16_t* x, uint8_t* codes, float* scales, float* dequant,
                                  int rows, int d) {
    const int bs = 16, nb = (d + bs - 1) / bs, pd = (d + 1) / 2;
    for (int r = 0; r < rows; ++r) {
        const uint16_t* src = x + (size_t)r * d;
        uint8_t* dst = codes + (size_t)r * pd;
        for (int j = 0; j < pd; ++j) dst[j] = 0;
        for (int b = 0; b < nb; ++b) {
            const int lo = b * bs, hi = lo + bs < d ? lo + bs : d;
            float amax = 0.f;
            for (int j = lo; j < hi; ++j) amax = fmaxf(amax, fabsf(orc_bf16_to_f32(src[j])));
            const float scale = amax > 0.f ? amax / 6.f : 1.f;
            const float inv = 1.f / scale;
            if (scales) scales[(size_t)r * nb + b] = scale;
            for (int j = lo; j < hi; ++j) {
                const uint8_t c = orc_fp4_e2m1_quant(orc_bf16_to_f32(src[j]) * inv);
                dst[j / 2] |= (uint8_t)(c << ((j & 1) ? 4 : 0));
                if (dequant)
                    dequant[(size_t)r * d + j] = orc_bf16_to_f32(orc_f32_to_bf16(orc_fp4_e2m1_value(c) * scale));
            }
        }
    }
}

void orc_kv_quant_rows(const uint16_t* x, uint8_t* codes, float* scales, float* dequant, int rows,
                       int d, int fmt) {
    if (fmt == 5) {
        orc_kv_quant_rows_fp4(x, codes, scales, dequant, rows, d);
        return;
    }
    for (int r = 0; r < rows; ++r) {
        const uint16_t* src = x + (size_t)r * d;
        float scale = 1.f, inv = 1.f;
        if (fmt != 1 && fmt != 4) {
            float amax = 0.f;
            for (int j = 0; j < d; ++j) amax = fmaxf(amax, fabsf(orc_bf16_to_f32(src[j])));
            scale = amax > 0.f ? amax / (fmt == 2 ? 127.f : 448.f) : 1.f;
            inv = 1.f / scale;
            if (scales) scales[r] = scale;
        }
        for (int j = 0; j < d; ++j) {
            const float f = orc_bf16_to_f32(src[j]) * inv;
            float val;
            if (fmt == 2) {
                int qv = (int)rintf(f);
                qv = qv > 127 ? 127 : (qv < -128 ? -128 : qv);
                codes[(size_t)r * d + j] = (uint8_t)(int8_t)qv;
                val = (float)qv;
            } else if (fmt == 4) {
                const uint8_t c = orc_f32_to_fp8_e5m2(f);
                codes[(size_t)r * d + j] = c;
                val = orc_fp8_e5m2_to_f32(c);
            } else {
                const uint8_t c = orc_f32_to_fp8_e4m3(f);
                codes[(size_t)r * d + j] = c;
                val = orc_fp8_e4m3_to_f32(c);
            }
            if (dequant) dequant[(size_t)r * d + j] = val * scale;
        }
    }
}
