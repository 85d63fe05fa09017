/*
 * Body of the oracle's higher-precision forward passes; included by model_hp.c once per working
 * type with REAL, FN(name), HP_KV_F16 and HP_ACT_BF16_FOR_BF16_WEIGHTS defined.
 * TEST INFRASTRUCTURE ONLY (see oracle_common.h).
 *
 * Same graph as model.c (driver/portable/src/graph_qwen3.cpp:225-896), but nothing between ops
 * is rounded to bf16: the residual stream and every activation stay in REAL, as the portable
 * driver keeps them in F32 (graph_qwen3.cpp:85 get_rows -> F32, :287-291 mul_mat -> F32, :551
 * o_proj, :572 and :723 residual adds, none followed by a cast).
 */

/* Row n of a linear in its storage format -> REAL (exact products: int4/int8 code times scale,
 * e4m3 value times scale; bf16 as stored). */
static void FN(dequant_row)(const OrcModel* m, const OrcLinear* w, int quant, int n, int K, REAL* out) {
    switch (quant) {
        case 0: {
            const uint32_t* words = (const uint32_t*)w->data + (size_t)n * (K / 8);
            const uint16_t* sc = (const uint16_t*)w->scale + (size_t)n * (K / m->group);
            for (int k = 0; k < K; ++k) {
                const int nib = (int)((words[k >> 3] >> (4 * (k & 7))) & 0xFu);
                out[k] = (REAL)(nib - 8) * (REAL)orc_bf16_to_f32(sc[k / m->group]);
            }
            break;
        }
        case 1: {
            const int8_t* q = (const int8_t*)w->data + (size_t)n * K;
            const REAL s = (REAL)((const float*)w->scale)[n];
            for (int k = 0; k < K; ++k) out[k] = (REAL)q[k] * s;
            break;
        }
        case 2: {
            const uint8_t* q = (const uint8_t*)w->data + (size_t)n * K;
            const REAL s = (REAL)((const float*)w->scale)[n];
            for (int k = 0; k < K; ++k) out[k] = (REAL)orc_fp8_e4m3_to_f32(q[k]) * s;
            break;
        }
        default: {
            const uint16_t* q = (const uint16_t*)w->data + (size_t)n * K;
            for (int k = 0; k < K; ++k) out[k] = (REAL)orc_bf16_to_f32(q[k]);
            break;
        }
    }
}

/* y[M, N] (+)= act[M, K] . W[N, K]^T, sums in REAL. */
static void FN(linear)(const OrcModel* m, const OrcLinear* w, int quant, const REAL* act, REAL* y,
                       int M, int N, int K, int beta) {
    const REAL* a = act;
    REAL* rounded = NULL;
#if HP_ACT_BF16_FOR_BF16_WEIGHTS
    /* ggml's mul_mat converts the activations to the weights' dot-product type first; for bf16
     * weights that is bf16 (ggml-cpu type traits: vec_dot_type of BF16 is BF16). */
    if (quant == 3) {
        rounded = (REAL*)malloc(sizeof(REAL) * (size_t)M * K);
        for (size_t i = 0; i < (size_t)M * K; ++i) rounded[i] = (REAL)orc_round_bf16((float)act[i]);
        a = rounded;
    }
#endif
#pragma omp parallel
    {
        REAL* row = (REAL*)malloc(sizeof(REAL) * (size_t)K);
#pragma omp for schedule(static)
        for (int n = 0; n < N; ++n) {
            FN(dequant_row)(m, w, quant, n, K, row);
            for (int mi = 0; mi < M; ++mi) {
                const REAL* x = a + (size_t)mi * K;
                REAL s0 = 0, s1 = 0, s2 = 0, s3 = 0;
                int k = 0;
                for (; k + 3 < K; k += 4) {
                    s0 += x[k] * row[k];
                    s1 += x[k + 1] * row[k + 1];
                    s2 += x[k + 2] * row[k + 2];
                    s3 += x[k + 3] * row[k + 3];
                }
                for (; k < K; ++k) s0 += x[k] * row[k];
                const REAL dot = (s0 + s1) + (s2 + s3);
                REAL* o = y + (size_t)mi * N + n;
                *o = beta ? *o + dot : dot;
            }
        }
        free(row);
    }
    free(rounded);
}

/* y = x / sqrt(mean(x^2) + eps) * w  (ggml_rms_norm then norm_scale's multiply,
 * graph_qwen3.cpp:282-283, graph_common.cpp:217-228). */
static void FN(rmsnorm)(const REAL* x, const uint16_t* w, REAL* y, int rows, int H, float eps) {
    for (int r = 0; r < rows; ++r) {
        const REAL* xr = x + (size_t)r * H;
        double ss = 0.0;   /* ggml accumulates the sum of squares in double as well */
        for (int i = 0; i < H; ++i) ss += (double)xr[i] * (double)xr[i];
        const REAL inv = (REAL)(1.0 / sqrt(ss / (double)H + (double)eps));
        for (int i = 0; i < H; ++i) y[(size_t)r * H + i] = xr[i] * inv * (REAL)orc_bf16_to_f32(w[i]);
    }
}

static REAL FN(kv_store)(REAL v) {
#if HP_KV_F16
    return (REAL)orc_round_f16((float)v);   /* the pool is F16 (executor.cpp:351,359) */
#else
    return v;
#endif
}

/* Optional per-head RMSNorm, RoPE in either pairing, q to q_out, K / V into the pool slot. */
static void FN(rope_kvwrite)(const OrcModel* m, int l, const REAL* qkv, REAL* q_out, double* k_pool,
                             double* v_pool, const int32_t* positions, const int64_t* kv_slots,
                             int N) {
    const int d = m->head_dim, hq = m->q_heads, hk = m->kv_heads, half = d / 2;
    const size_t stride = (size_t)(hq + 2 * hk) * d;
    for (int n = 0; n < N; ++n)
        for (int head = 0; head < hq + 2 * hk; ++head) {
            const REAL* src = qkv + n * stride + (size_t)head * d;
            const int is_q = head < hq, is_k = !is_q && head < hq + hk;
            const int64_t slot = kv_slots[n];
            if (!is_q && slot < 0) continue;
            if (!is_q && !is_k) {
                double* dst = v_pool + ((size_t)slot * hk + (head - hq - hk)) * d;
                for (int i = 0; i < d; ++i) dst[i] = (double)FN(kv_store)(src[i]);
                continue;
            }
            const uint16_t* nw = !m->has_qk_norm ? NULL : (is_q ? m->q_norm[l] : m->k_norm[l]);
            REAL inv = 1;
            if (nw) {
                double ss = 0.0;
                for (int i = 0; i < d; ++i) ss += (double)src[i] * (double)src[i];
                inv = (REAL)(1.0 / sqrt(ss / (double)d + (double)m->rms_eps));
            }
            for (int i = 0; i < half; ++i) {
                const int ia = m->rope_interleaved ? 2 * i : i, ib = m->rope_interleaved ? 2 * i + 1 : i + half;
                REAL a = src[ia], b = src[ib];
                if (nw) {
                    a = a * inv * (REAL)orc_bf16_to_f32(nw[ia]);
                    b = b * inv * (REAL)orc_bf16_to_f32(nw[ib]);
                }
                const REAL ang = (REAL)positions[n] * (REAL)m->inv_freq[i];
                const REAL ms = m->rope_mscale > 0.f ? (REAL)m->rope_mscale : (REAL)1;
                const REAL c = (REAL)cos((double)ang) * ms, s = (REAL)sin((double)ang) * ms;
                const REAL ra = a * c - b * s, rb = b * c + a * s;
                if (is_q) {
                    REAL* dst = q_out + ((size_t)n * hq + head) * d;
                    dst[ia] = ra;
                    dst[ib] = rb;
                } else {
                    double* dst = k_pool + ((size_t)slot * hk + (head - hq)) * d;
                    dst[ia] = (double)FN(kv_store)(ra);
                    dst[ib] = (double)FN(kv_store)(rb);
                }
            }
        }
}

/* softmax(q.K^T / sqrt(d)) . V per row and head over the row's visible keys. */
static void FN(attention)(const OrcModel* m, const REAL* q, const double* k_pool, const double* v_pool,
                          REAL* out, const uint32_t* page_indices, const uint32_t* row_begin,
                          const int32_t* row_len, int N, int ps, const uint8_t* allow,
                          const int64_t* allow_off) {
    const int d = m->head_dim, hq = m->q_heads, hk = m->kv_heads, gqa = hq / hk;
    const REAL scale = (REAL)(1.0 / sqrt((double)d));
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int r = 0; r < N; ++r)
        for (int h = 0; h < hq; ++h) {
            const int n_kv = row_len[r], kvh = h / gqa;
            REAL* o = out + ((size_t)r * hq + h) * d;
            for (int j = 0; j < d; ++j) o[j] = 0;
            if (n_kv <= 0) continue;
            REAL* sc = (REAL*)malloc(sizeof(REAL) * (size_t)n_kv);
            const REAL* qh = q + ((size_t)r * hq + h) * d;
            REAL mx = -(REAL)INFINITY;
            for (int t = 0; t < n_kv; ++t) {
                if (allow && !allow[allow_off[r] + t]) {
                    sc[t] = -(REAL)INFINITY;
                    continue;
                }
                const size_t slot = (size_t)page_indices[row_begin[r] + t / ps] * ps + t % ps;
                const double* kr = k_pool + (slot * hk + kvh) * d;
                REAL dot = 0;
                for (int j = 0; j < d; ++j) dot += qh[j] * (REAL)kr[j];
                sc[t] = dot * scale;
                if (sc[t] > mx) mx = sc[t];
            }
            if (mx == -(REAL)INFINITY) {   /* no visible key: zeros */
                free(sc);
                continue;
            }
            REAL z = 0;
            for (int t = 0; t < n_kv; ++t) {
                sc[t] = sc[t] == -(REAL)INFINITY ? 0 : (REAL)exp((double)(sc[t] - mx));
                z += sc[t];
            }
            for (int t = 0; t < n_kv; ++t) {
                if (sc[t] == 0) continue;
                const size_t slot = (size_t)page_indices[row_begin[r] + t / ps] * ps + t % ps;
                const double* vr = v_pool + (slot * hk + kvh) * d;
                const REAL p = sc[t] / z;
                for (int j = 0; j < d; ++j) o[j] += p * (REAL)vr[j];
            }
            free(sc);
        }
}

/* x[t] += sum_k w_k * down_e(silu(gate_e xn) * up_e xn) over the token's top-k experts, weights
 * = softmax probabilities of the chosen experts divided by their sum (as they are under raw_topk); nothing rounded per route
 * (driver/portable/src/graph_common.cpp:237-345). */
static void FN(moe_ffn)(const OrcModel* m, int l, const REAL* xn, REAL* x, int N) {
    const int H = m->hidden, E = m->num_experts, K = m->top_k, Ie = m->expert_intermediate;
    OrcLinear router = {m->router[l], NULL};
    REAL* logits = (REAL*)malloc(sizeof(REAL) * (size_t)N * E);
    FN(linear)(m, &router, 3, xn, logits, N, E, H, 0);
    for (int t = 0; t < N; ++t) {
        REAL* p = logits + (size_t)t * E;
        REAL mx = p[0];
        for (int e = 1; e < E; ++e) mx = p[e] > mx ? p[e] : mx;
        REAL z = 0;
        for (int e = 0; e < E; ++e) {
            p[e] = (REAL)exp((double)(p[e] - mx));
            z += p[e];
        }
        for (int e = 0; e < E; ++e) p[e] /= z;
        int sel[64];
        REAL wsel[64], wsum = 0;
        for (int k = 0; k < K; ++k) {   /* strictly greater wins: the lowest index on ties */
            int best = -1;
            for (int e = 0; e < E; ++e) {
                int taken = 0;
                for (int j = 0; j < k; ++j) taken |= sel[j] == e;
                if (!taken && (best < 0 || p[e] > p[best])) best = e;
            }
            sel[k] = best;
            wsel[k] = p[best];
            wsum += p[best];
        }
        REAL* gu = (REAL*)malloc(sizeof(REAL) * (size_t)2 * Ie);
        REAL* act = (REAL*)malloc(sizeof(REAL) * (size_t)Ie);
        REAL* y = (REAL*)malloc(sizeof(REAL) * (size_t)H);
        for (int k = 0; k < K; ++k) {
            const int e = sel[k];
            OrcLinear wg, wd;
            const size_t nk_g = (size_t)e * 2 * Ie * H, nk_d = (size_t)e * H * Ie;
            switch (m->quant) {
                case 0:
                    wg.data = (const unsigned char*)m->wgu[l].data + nk_g / 2;
                    wg.scale = (const unsigned char*)m->wgu[l].scale + (size_t)e * 2 * Ie * (H / m->group) * 2;
                    wd.data = (const unsigned char*)m->wdown[l].data + nk_d / 2;
                    wd.scale = (const unsigned char*)m->wdown[l].scale + (size_t)e * H * (Ie / m->group) * 2;
                    break;
                case 1:
                case 2:
                    wg.data = (const unsigned char*)m->wgu[l].data + nk_g;
                    wg.scale = (const unsigned char*)m->wgu[l].scale + (size_t)e * 2 * Ie * 4;
                    wd.data = (const unsigned char*)m->wdown[l].data + nk_d;
                    wd.scale = (const unsigned char*)m->wdown[l].scale + (size_t)e * H * 4;
                    break;
                default:
                    wg.data = (const unsigned char*)m->wgu[l].data + nk_g * 2;
                    wd.data = (const unsigned char*)m->wdown[l].data + nk_d * 2;
                    wg.scale = wd.scale = NULL;
                    break;
            }
            FN(linear)(m, &wg, m->quant, xn + (size_t)t * H, gu, 1, 2 * Ie, H, 0);
            for (int i = 0; i < Ie; ++i) {
                const REAL g = gu[i];
                act[i] = g / (1 + (REAL)exp((double)-g)) * gu[Ie + i];
            }
            FN(linear)(m, &wd, m->quant, act, y, 1, H, Ie, 0);
            const REAL wk = m->raw_topk ? wsel[k] : wsel[k] / wsum;
            for (int i = 0; i < H; ++i) x[(size_t)t * H + i] += wk * y[i];
        }
        free(gu); free(act); free(y);
    }
    free(logits);
}

static void FN(forward)(const OrcModel* m, double* const* k_pool, double* const* v_pool,
                        const uint32_t* tokens, const int32_t* positions, const int64_t* kv_slots,
                        const uint32_t* row_begin, const int32_t* row_len,
                        const uint32_t* page_indices, int N, const uint32_t* sample_rows, int S,
                        int page_size, uint32_t* out_tokens, double* logits_out,
                        const uint8_t* allow, const int64_t* allow_off) {
    const int H = m->hidden, d = m->head_dim, hq = m->q_heads, hk = m->kv_heads;
    const int I = m->intermediate, V = m->vocab;
    const int qkv_dim = (hq + 2 * hk) * d;
    REAL* x = (REAL*)malloc(sizeof(REAL) * (size_t)N * H);
    REAL* xn = (REAL*)malloc(sizeof(REAL) * (size_t)N * H);
    REAL* qkv = (REAL*)malloc(sizeof(REAL) * (size_t)N * qkv_dim);
    REAL* q = (REAL*)malloc(sizeof(REAL) * (size_t)N * hq * d);
    REAL* attn = (REAL*)malloc(sizeof(REAL) * (size_t)N * hq * d);
    REAL* gu = (REAL*)malloc(sizeof(REAL) * (size_t)N * 2 * (I > 0 ? I : 1));
    REAL* act = (REAL*)malloc(sizeof(REAL) * (size_t)N * (I > 0 ? I : 1));
    for (int n = 0; n < N; ++n) {
        const size_t row = tokens[n] < (uint32_t)V ? tokens[n] : 0;
        for (int i = 0; i < H; ++i) x[(size_t)n * H + i] = (REAL)orc_bf16_to_f32(m->embed[row * H + i]);
    }
    for (int l = 0; l < m->layers; ++l) {
        FN(rmsnorm)(x, m->attn_norm[l], xn, N, H, m->rms_eps);
        FN(linear)(m, &m->wqkv[l], m->quant, xn, qkv, N, qkv_dim, H, 0);
        FN(rope_kvwrite)(m, l, qkv, q, k_pool[l], v_pool[l], positions, kv_slots, N);
        FN(attention)(m, q, k_pool[l], v_pool[l], attn, page_indices, row_begin, row_len, N, page_size,
                      allow, allow_off);
        FN(linear)(m, &m->wo[l], m->quant, attn, x, N, H, hq * d, 1);
        FN(rmsnorm)(x, m->ffn_norm[l], xn, N, H, m->rms_eps);
        if (m->num_experts > 0) {
            FN(moe_ffn)(m, l, xn, x, N);
        } else {
            FN(linear)(m, &m->wgu[l], m->quant, xn, gu, N, 2 * I, H, 0);
            for (int n = 0; n < N; ++n)
                for (int i = 0; i < I; ++i) {
                    const REAL g = gu[(size_t)n * 2 * I + i];
                    act[(size_t)n * I + i] = g / (1 + (REAL)exp((double)-g)) * gu[(size_t)n * 2 * I + I + i];
                }
            FN(linear)(m, &m->wdown[l], m->quant, act, x, N, H, I, 1);
        }
    }
    if (S > 0) {
        REAL* xs = (REAL*)malloc(sizeof(REAL) * (size_t)S * H);
        REAL* xsn = (REAL*)malloc(sizeof(REAL) * (size_t)S * H);
        REAL* lg = (REAL*)malloc(sizeof(REAL) * (size_t)S * V);
        for (int s = 0; s < S; ++s)
            memcpy(xs + (size_t)s * H, x + (size_t)(sample_rows[s] < (uint32_t)N ? sample_rows[s] : 0) * H,
                   sizeof(REAL) * (size_t)H);
        FN(rmsnorm)(xs, m->final_norm, xsn, S, H, m->rms_eps);
        OrcLinear head = {m->lm_head, NULL};
        FN(linear)(m, &head, 3, xsn, lg, S, V, H, 0);
        for (int s = 0; s < S; ++s) {
            int best = 0;
            for (int v = 1; v < V; ++v)
                if (lg[(size_t)s * V + v] > lg[(size_t)s * V + best]) best = v;   /* first index on ties */
            if (out_tokens) out_tokens[s] = (uint32_t)best;
            if (logits_out)
                for (int v = 0; v < V; ++v) logits_out[(size_t)s * V + v] = (double)lg[(size_t)s * V + v];
        }
        free(xs); free(xsn); free(lg);
    }
    free(x); free(xn); free(qkv); free(q); free(attn); free(gu); free(act);
}
