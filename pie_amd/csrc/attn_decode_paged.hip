// Paged-KV decode attention (one query token per request) for gfx950.
//
// Semantics: driver/cuda/src/ops/attention_naive_paged.cu:319-447 of the
// reference (softmax(q·K^T * scale)·V over the request's pages, fp32 maths,
// bf16 output, optional log-sum-exp), with the KV pool laid out
// [num_pages, page_size, num_kv_heads, head_dim] bf16
// (driver/cuda/src/kv_cache.hpp:3-8).  Prefix-shared (forked) pages need no
// special handling: several requests simply list the same physical page ids.
//
// HBM-bound design (every K and V byte of the context is read once):
//   * split-K over pages: grid = (splits, kv_head, request); a block of four waves
//     owns a run of 16-token units of one (request, kv head) and each wave walks
//     every fourth unit, so ragged contexts turn into many equal-sized blocks that
//     the dispatcher load-balances; blocks past a request's length exit at once;
//   * one wave load instruction covers whole 256-byte K (or V) rows: lane l reads
//     the 16 B piece (l % LPR) of token (l / LPR), LPR = head_dim/8, so every access
//     is a full, contiguous row and the GQA group's q heads share each K/V byte;
//   * q·k runs on v_dot2_f32_bf16; the LPR lanes of a token finish the dot product
//     with DPP row operations (no LDS, no ds_bpermute in the loop);
//   * each group of LPR lanes keeps its own online-softmax state (max, sum, 8
//     output dims per q head), so nothing crosses lane groups until the unit loop
//     ends; groups, then waves (through LDS), are merged once per block;
//   * the next unit's K and V rows are requested before the current unit is
//     reduced, so 2 x (K+V) = 16 KiB per wave is in flight;
//   * a second, tiny kernel merges the splits (skipped when there is one split).
#include <algorithm>
#include <cstdio>
#include <mutex>
#include <type_traits>

#include "common.hip.h"

namespace pie_hip {
namespace {

constexpr int kAttnBlock = 256;
constexpr int kAttnWaves = kAttnBlock / kWave;
constexpr int kUnitTokens = kAttnUnitTokens;

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
    return v + __int_as_float(t);
}
// Sum over the LPR (8 or 16) adjacent lanes that share a token; every lane gets the sum.
template <int LPR>
__device__ __forceinline__ float token_lanes_sum(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror
    if (LPR == 16) v = dpp_add<0x140>(v);  // row_mirror
    return v;
}

template <int D, int GQA, int KVF = kKvBf16>
struct UnitRegs {
    static constexpr int LPR = D / 8;
    static constexpr int TPI = kWave / LPR;          // tokens per load instruction
    static constexpr int IPU = kUnitTokens / TPI;    // load instructions per unit
    typename KvVec<KVF>::type k[IPU];
    typename KvVec<KVF>::type v[IPU];
    float ks[IPU], vs[IPU];   // one-byte formats: the (token, kv head) scales
    uint32_t mask;   // MASKED kernels: bit t = token t of the unit is visible
};

// part_o  [R, hq, nsplit, D] f32 (unnormalised), part_ml [R, hq, nsplit, 2] f32 (max, sum),
// both in units where scores were multiplied by scale*log2(e).
// MASKED: mask_bits [rows, mask_stride] u16, one word per 16-token unit (custom attention
// masks); hidden tokens are dropped like the slots past the context.
template <int D, int GQA, bool MASKED, int KVF = kKvBf16>
__global__ __launch_bounds__(kAttnBlock) void attn_decode_split_kernel(
    const uint16_t* __restrict__ q, const void* __restrict__ k_pages_raw,
    const void* __restrict__ v_pages_raw, const float* __restrict__ k_scales,
    const float* __restrict__ v_scales, const uint32_t* __restrict__ page_indices,
    const uint32_t* __restrict__ page_indptr, const uint32_t* __restrict__ last_lens,
    const uint32_t* __restrict__ row_begin, const int32_t* __restrict__ row_len,
    float* __restrict__ part_o, float* __restrict__ part_ml, uint16_t* __restrict__ o_direct,
    float* __restrict__ lse, const uint16_t* __restrict__ mask_bits, int mask_stride, int hq,
    int hk, int ps, int units_per_split, int nsplit, float scale_log2e) {
    using U = UnitRegs<D, GQA, KVF>;
    using KV = typename KvVec<KVF>::type;
    constexpr int LPR = U::LPR, TPI = U::TPI, IPU = U::IPU;
    constexpr int kElemBytes = KVF == kKvBf16 ? 2 : 1;
    const unsigned char* k_pages = static_cast<const unsigned char*>(k_pages_raw);
    const unsigned char* v_pages = static_cast<const unsigned char*>(v_pages_raw);
    const int kvh = blockIdx.x, split = blockIdx.y, r = blockIdx.z;  // kv heads of the same tokens are dispatched together
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform -> SGPR
    const int grp = lane / LPR, dl = lane % LPR;

    const RowExtent ext = row_extent(page_indptr, last_lens, row_begin, row_len, r, ps);
    const uint32_t pg_lo = ext.pg_lo;
    const int kv_len = ext.kv_len;
    const int nunits = (kv_len + kUnitTokens - 1) / kUnitTokens;
    const int u_begin = split * units_per_split;
    if (u_begin >= nunits) return;
    const int u_end = min(u_begin + units_per_split, nunits);

    // q for the GQA heads of this kv head: 8 dims per lane per head, as bf16 pairs.
    u32x4_t qv[GQA];
#pragma unroll
    for (int h = 0; h < GQA; ++h)
        qv[h] = *reinterpret_cast<const u32x4_t*>(
            q + (static_cast<size_t>(r) * hq + kvh * GQA + h) * D + dl * 8);

    const size_t row_stride = static_cast<size_t>(hk) * D;  // elements between tokens
    auto issue = [&](U& u, int unit) {
        const int tok0 = unit * kUnitTokens;
        const int page = tok0 / ps;
        const uint32_t pid = page_indices[pg_lo + page];
        const size_t slot0 = static_cast<size_t>(pid) * ps + (tok0 - page * ps);
        const size_t base = (slot0 * hk + kvh) * D + dl * 8;
#pragma unroll
        for (int i = 0; i < IPU; ++i) {
            const size_t off = (base + static_cast<size_t>(i * TPI + grp) * row_stride) * kElemBytes;
            u.k[i] = __builtin_nontemporal_load(reinterpret_cast<const KV*>(k_pages + off));
            u.v[i] = __builtin_nontemporal_load(reinterpret_cast<const KV*>(v_pages + off));
            if constexpr (KVF != kKvBf16) {
                // (a unit of tokens lies inside one page)
                const size_t th = kv_scale_index(pid, tok0 - page * ps + i * TPI + grp, kvh, hk, ps);
                u.ks[i] = k_scales ? k_scales[th] : 1.f;
                u.vs[i] = v_scales ? v_scales[th] : 1.f;
            }
        }
        if (MASKED) u.mask = mask_bits[static_cast<size_t>(r) * mask_stride + unit];
    };

    float m[GQA], l[GQA], o[GQA][8];
#pragma unroll
    for (int h = 0; h < GQA; ++h) {
        m[h] = -INFINITY;
        l[h] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[h][e] = 0.f;
    }

    auto compute = [&](U& u, int unit) {
        const int tok0 = unit * kUnitTokens;
        float s[IPU][GQA];
#pragma unroll
        for (int i = 0; i < IPU; ++i) {
            const u32x4_t kb = kv_decode_bf16<KVF>(u.k[i]);
            const float sc = KVF == kKvBf16 ? scale_log2e : scale_log2e * u.ks[i];
#pragma unroll
            for (int h = 0; h < GQA; ++h) {
                float p = 0.f;
                p = dot2_bf16(kb.x, qv[h].x, p);
                p = dot2_bf16(kb.y, qv[h].y, p);
                p = dot2_bf16(kb.z, qv[h].z, p);
                p = dot2_bf16(kb.w, qv[h].w, p);
                s[i][h] = token_lanes_sum<LPR>(p) * sc;
            }
        }
        if (tok0 + kUnitTokens > kv_len) {  // tail unit: drop slots past the context
#pragma unroll
            for (int i = 0; i < IPU; ++i) {
                if (tok0 + i * TPI + grp >= kv_len) {
#pragma unroll
                    for (int h = 0; h < GQA; ++h) s[i][h] = -INFINITY;
                    u.v[i] = KV{};
                    u.vs[i] = 0.f;
                }
            }
        }
        if (MASKED && u.mask != 0xFFFFu) {
#pragma unroll
            for (int i = 0; i < IPU; ++i) {
                if (!((u.mask >> (i * TPI + grp)) & 1u)) {
#pragma unroll
                    for (int h = 0; h < GQA; ++h) s[i][h] = -INFINITY;
                    u.v[i] = KV{};
                    u.vs[i] = 0.f;
                }
            }
        }
        float alpha[GQA];
        bool grew = false;
#pragma unroll
        for (int h = 0; h < GQA; ++h) {
            float mx = m[h];
#pragma unroll
            for (int i = 0; i < IPU; ++i) mx = fmaxf(mx, s[i][h]);
            const float safe = (mx == -INFINITY) ? 0.f : mx;
            alpha[h] = exp2f(m[h] - safe);
            grew |= (mx != m[h]);
            m[h] = mx;
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < IPU; ++i) {
                s[i][h] = exp2f(s[i][h] - safe);
                sum += s[i][h];
            }
            l[h] = l[h] * alpha[h] + sum;
        }
        if (__any(grew)) {
#pragma unroll
            for (int h = 0; h < GQA; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) o[h][e] *= alpha[h];
        }
#pragma unroll
        for (int i = 0; i < IPU; ++i) {
            float vf[8];
            kv_decode_f32<KVF>(u.v[i], vf);
#pragma unroll
            for (int h = 0; h < GQA; ++h) {
                const float pw = KVF == kKvBf16 ? s[i][h] : s[i][h] * u.vs[i];
#pragma unroll
                for (int e = 0; e < 8; ++e) o[h][e] = fmaf(pw, vf[e], o[h][e]);
            }
        }
    };

    // Two-deep pipeline over this wave's units (every fourth unit of the block's run).
    U ua, ub;
    const int first = u_begin + wv;
    const int last_valid = u_end - 1;
    if (first < u_end) {
        issue(ua, first);
        for (int u = first; u < u_end; u += 2 * kAttnWaves) {
            issue(ub, min(u + kAttnWaves, last_valid));
            compute(ua, u);
            issue(ua, min(u + 2 * kAttnWaves, last_valid));
            if (u + kAttnWaves < u_end) compute(ub, u + kAttnWaves);
        }
    }

    // Merge the lane groups of the wave (lanes with equal dl).
#pragma unroll
    for (int h = 0; h < GQA; ++h) {
        float mx = m[h];
#pragma unroll
        for (int off = LPR; off < kWave; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
        const float safe = (mx == -INFINITY) ? 0.f : mx;
        const float a = exp2f(m[h] - safe);
        float ls = l[h] * a;
#pragma unroll
        for (int off = LPR; off < kWave; off <<= 1) ls += __shfl_xor(ls, off, kWave);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float ov = o[h][e] * a;
#pragma unroll
            for (int off = LPR; off < kWave; off <<= 1) ov += __shfl_xor(ov, off, kWave);
            o[h][e] = ov;
        }
        m[h] = mx;
        l[h] = ls;
    }

    // Merge the four waves through LDS.
    __shared__ float sm_o[kAttnWaves][GQA][D];
    __shared__ float sm_m[kAttnWaves][GQA];
    __shared__ float sm_l[kAttnWaves][GQA];
    if (grp == 0) {
#pragma unroll
        for (int h = 0; h < GQA; ++h) {
#pragma unroll
            for (int e = 0; e < 8; ++e) sm_o[wv][h][dl * 8 + e] = o[h][e];
            if (dl == 0) {
                sm_m[wv][h] = m[h];
                sm_l[wv][h] = l[h];
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < GQA * D; idx += kAttnBlock) {
        const int h = idx / D, dd = idx - h * D;
        float mx = sm_m[0][h];
#pragma unroll
        for (int w = 1; w < kAttnWaves; ++w) mx = fmaxf(mx, sm_m[w][h]);
        const float safe = (mx == -INFINITY) ? 0.f : mx;
        float ov = 0.f, ls = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float a = exp2f(sm_m[w][h] - safe);
            ov += sm_o[w][h][dd] * a;
            ls += sm_l[w][h] * a;
        }
        const int head = kvh * GQA + h;
        const size_t rh = static_cast<size_t>(r) * hq + head;
        if (o_direct) {
            o_direct[rh * D + dd] = f32_to_bf16_bits(ls > 0.f ? ov / ls : 0.f);
            if (lse && dd == 0)
                lse[rh] = ls > 0.f ? (logf(ls) + mx * 0.6931471805599453f) : -INFINITY;
        } else {
            part_o[(rh * nsplit + split) * D + dd] = ov;
            if (dd == 0) {
                part_ml[(rh * nsplit + split) * 2 + 0] = mx;
                part_ml[(rh * nsplit + split) * 2 + 1] = ls;
            }
        }
    }
}

// ---- the same split on the matrix cores (bf16 pools, no custom mask) ------------------------
// One block = one (row, kv head, split) as above; each of the four waves walks every fourth
// 32-key step of the split on its own (own K/V loads, own LDS region, own online-softmax state;
// no block barrier inside the loop):
//   S^T[key, query] = K . Q^T      A = K fragment from the wave's LDS region (row = key, k = d; rows
//                                  padded to D + 8), B = the GQA query heads of the row in the
//                                  first GQA of 16 columns (the rest are zero)
//   O^T[d, query]  += V^T . P^T    A = V^T read transposed (ds_read_b64_tr_b16) from the V rows
//                                  in the wave's LDS region, B = P from registers
// The query sits on the lane%16 axis of both accumulators, so max / sum / rescale are per lane
// and cost two cross-lane steps per 32 keys instead of four per key and head.  The keys of a
// step leave the first product in the order [4g..4g+3, 16+4g..16+4g+3] per 16-lane group g —
// the rows the group's two transposing reads of a V^T fragment take (V rows padded to D + 16).
// Probabilities enter the second product as a bf16 pair (hi + lo), i.e. with 16 mantissa bits,
// so the result keeps the accuracy of the fp32 kernel above.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));
constexpr int kMStepKeys = 32;

template <int D, int GQA, int KVF = kKvBf16, bool MASKED = false, bool CHUNKS = false, int NW = kAttnWaves>
__global__ __launch_bounds__(NW * kWave, 2) void attn_decode_mfma_kernel(
    const uint16_t* __restrict__ q, const void* __restrict__ k_pages_raw,
    const void* __restrict__ v_pages_raw, const float* __restrict__ k_scales,
    const float* __restrict__ v_scales, const uint32_t* __restrict__ page_indices,
    const uint32_t* __restrict__ page_indptr, const uint32_t* __restrict__ last_lens,
    const uint32_t* __restrict__ row_begin, const int32_t* __restrict__ row_len,
    float* __restrict__ part_o, float* __restrict__ part_ml, uint16_t* __restrict__ o_direct,
    float* __restrict__ lse, const uint16_t* __restrict__ mask_bits, int mask_stride, int hq, int hk,
    int ps, int ps_shift, int units_per_split, int nsplit, float scale_log2e, int num_rows,
    int* __restrict__ row_pieces) {
    static_assert(!(CHUNKS && MASKED), "the chunked launch takes no custom masks");
    static_assert(CHUNKS || NW == kAttnWaves || NW == 2 * kAttnWaves, "the gridded launch has four or eight waves per block");
    constexpr int KS = D / 32;                 // k steps of the first product
    constexpr int DT = D / 16;                 // d tiles of the second product
    // One-byte pools: the codes become bf16 (exactly) on the way into the wave's LDS regions, the
    // per-(token, kv head) scales multiply the scores (K) and the probabilities (V) — the
    // arithmetic of the dot-product kernel above, float(code) * scale.
    constexpr bool Q8 = KVF != kKvBf16;
    constexpr int EB = Q8 ? 1 : 2;             // stored bytes per element
    constexpr int LPR = D * EB / 16;           // 16-byte pieces per stored K/V row
    constexpr int NK = kMStepKeys * LPR / kWave;   // K load instructions per step
    constexpr int PF = 2;                      // steps of K/V in flight per wave
    static_assert(GQA <= 16 && NK >= 1, "shape");
    const unsigned char* k_pages = static_cast<const unsigned char*>(k_pages_raw);
    const unsigned char* v_pages = static_cast<const unsigned char*>(v_pages_raw);
    constexpr int KSTRIDE = D + 8;             // bf16 elements per K row in LDS (padded: conflict-free reads)
    // V rows sit in LDS as they are stored (padded to D + 16: the four rows a transposing read
    // touches start eight banks apart); the V^T operand of the second product comes out of
    // ds_read_b64_tr_b16, which hands lane i of a 16-lane group element i of four 16-element rows
    constexpr int VSTRIDE = D + 16;
    // One-byte pools: rows of D codes padded to D + 16 bytes, the upper sixteen V rows 128 bytes
    // further (a 16-lane group's transposing read takes rows 4g.. and 16 + 4g..: without the
    // offset the two land on the same banks); a lane's 8-byte K fragment reads and the
    // transposing 8-byte V reads are then conflict-free per half wave.
    constexpr int STRIDE8 = D + 16, VUPPER8 = 128;
    constexpr int VREGION = Q8 ? (kMStepKeys * STRIDE8 + VUPPER8) / 2 : kMStepKeys * VSTRIDE;   // uint16 units
    constexpr int KREGION = Q8 ? kMStepKeys * STRIDE8 / 2 : kMStepKeys * KSTRIDE;
    static_assert(KREGION % 8 == 0, "a wave's V region starts on a 16-byte boundary");
    __shared__ __attribute__((aligned(16))) uint16_t kv_all[NW][KREGION + VREGION];   // per wave: K region, V region
    __shared__ float sm_m[CHUNKS ? 1 : NW][16];
    __shared__ float sm_l[CHUNKS ? 1 : NW][16];
    __shared__ __attribute__((aligned(16))) float sc_all[Q8 ? NW : 1][kWave];   // K | V scales of a step
    static_assert(sizeof(float) * GQA * D <= sizeof(uint16_t) * VREGION, "per-wave output fits its V region");

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int l16 = lane & 15, g = lane >> 4;

    // The (row, kv head, key range) in work.  One per block in the gridded launch; the chunked
    // launch walks a table of them (below).
    int kvh = 0, split = 0, r = 0, nunits = 0, k_begin = 0, k_end = 0;
    uint32_t pg_lo = 0;
    if constexpr (!CHUNKS) {
        kvh = blockIdx.x, split = blockIdx.y, r = blockIdx.z;
        const RowExtent ext = row_extent(page_indptr, last_lens, row_begin, row_len, r, ps);
        pg_lo = ext.pg_lo;
        const int kv_len = ext.kv_len;
        nunits = (kv_len + kUnitTokens - 1) / kUnitTokens;
        const int u_begin = split * units_per_split;
        if (u_begin >= nunits) {
            // (one split per row: a row without keys gets its zeros and its -inf here, no launch
            // of its own for that)
            if (o_direct && nunits == 0) {
                for (int idx = tid; idx < GQA * D; idx += NW * kWave) {
                    const int h = idx / D, dd = idx - h * D;
                    const size_t rh = static_cast<size_t>(r) * hq + kvh * GQA + h;
                    o_direct[rh * D + dd] = 0;
                    if (lse && dd == 0) lse[rh] = -INFINITY;
                }
            }
            return;
        }
        k_begin = u_begin * kUnitTokens;
        k_end = min(min(u_begin + units_per_split, nunits) * kUnitTokens, kv_len);
    }

    // Q^T fragment: column l16 = query head l16 of this kv head's group (zero beyond GQA)
    bf16x8_t qf[KS];
    auto load_q = [&]() {
        const bool valid = l16 < GQA;
        const uint16_t* qp = q + (static_cast<size_t>(r) * hq + kvh * GQA + (valid ? l16 : 0)) * D + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4_t v = *reinterpret_cast<const u32x4_t*>(qp + 32 * ks);
            if (!valid) v = u32x4_t{0u, 0u, 0u, 0u};
            qf[ks] = __builtin_bit_cast(bf16x8_t, v);
        }
    };
    if constexpr (!CHUNKS) load_q();

    uint16_t* Ks = kv_all[wv];
    uint16_t* Vs = Ks + KREGION;
    // K and V loads: whole rows, LPR adjacent lanes per key (kWave / LPR keys per instruction)
    constexpr int KPI = kWave / LPR;
    u32x4_t kreg[PF][NK], vreg[PF][NK];
    float sreg[PF];   // one-byte pools: lane < 32 holds the K scale of key `lane`, the others V's
    uint32_t mreg[PF];   // MASKED: the visibility words of the step's two 16-token units
    // A 32-key step starts on a multiple of 16 and touches at most two pages (page_size % 16 == 0);
    // their ids come through scalar loads.  Keys past the split repeat its last key (finite
    // data; their probabilities are zero).
    auto issue = [&](int slot, int j0, int kvh, uint32_t pg_lo, int k_end) {   // (the context of the keys requested, which in the chunked launch may be the next item's)
        const int ja = min(j0, k_end - 1);
        const int page_a = ps_shift >= 0 ? ja >> ps_shift : ja / ps;
        const int pa_end = (page_a + 1) * ps;
        const int jb = min(j0 + kMStepKeys - 1, k_end - 1);
        const uint32_t pid_a = __builtin_amdgcn_readfirstlane(page_indices[pg_lo + page_a]);
        const uint32_t pid_b = __builtin_amdgcn_readfirstlane(page_indices[pg_lo + page_a + (jb >= pa_end ? 1 : 0)]);
        auto row_th = [&](int key) {   // (token slot, kv head) index of a key of the step
            const int j = min(j0 + key, k_end - 1);
            const bool in_a = j < pa_end;
            const size_t slot_idx = static_cast<size_t>(in_a ? pid_a : pid_b) * ps + (j - (in_a ? pa_end - ps : pa_end));
            return slot_idx * hk + kvh;
        };
        auto row_sc = [&](int key) {   // the key's place in a scale pool
            const int j = min(j0 + key, k_end - 1);
            const bool in_a = j < pa_end;
            return kv_scale_index(in_a ? pid_a : pid_b, j - (in_a ? pa_end - ps : pa_end), kvh, hk, ps);
        };
#pragma unroll
        for (int i = 0; i < NK; ++i)
            kreg[slot][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(
                k_pages + row_th(lane / LPR + KPI * i) * (D * EB) + (lane % LPR) * 16));
#pragma unroll
        for (int i = 0; i < NK; ++i)
            vreg[slot][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(
                v_pages + row_th(lane / LPR + KPI * i) * (D * EB) + (lane % LPR) * 16));
        if constexpr (Q8) {
            const float* sp = lane < kMStepKeys ? k_scales : v_scales;
            sreg[slot] = sp ? sp[row_sc(lane & (kMStepKeys - 1))] : 1.f;
        }
        if constexpr (MASKED) {   // (the second unit may lie past the context: its keys are dropped anyway)
            const uint16_t* mrow = mask_bits + static_cast<size_t>(r) * mask_stride;
            const int u0 = j0 / kUnitTokens;
            mreg[slot] = static_cast<uint32_t>(mrow[u0]) | (static_cast<uint32_t>(mrow[min(u0 + 1, nunits - 1)]) << 16);
        }
    };
    // K and V rows into the wave's LDS regions as they are stored (one-byte codes become bf16 on
    // the way)
    auto stage = [&](int slot) {
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int row = lane / LPR + KPI * i;
            if constexpr (!Q8) {
                const int piece = (lane % LPR) * 8;
                uint16_t* kd = &Ks[row * KSTRIDE + piece];
                uint16_t* vd = &Vs[row * VSTRIDE + piece];
                *reinterpret_cast<u32x4_t*>(kd) = kreg[slot][i];
                *reinterpret_cast<u32x4_t*>(vd) = vreg[slot][i];
            } else {   // 16 codes, as stored
                unsigned char* kb = reinterpret_cast<unsigned char*>(Ks) + row * STRIDE8 + (lane % LPR) * 16;
                unsigned char* vb = reinterpret_cast<unsigned char*>(Vs) + row * STRIDE8 + (row >> 4) * VUPPER8 + (lane % LPR) * 16;
                *reinterpret_cast<u32x4_t*>(kb) = kreg[slot][i];
                *reinterpret_cast<u32x4_t*>(vb) = vreg[slot][i];
            }
        }
        if constexpr (Q8) sc_all[wv][lane] = sreg[slot];
    };

    f32x4_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float mx = -INFINITY, lsum = 0.f;

    // keys between two steps of one wave: the gridded launch deals a split's steps to its four
    // (or eight) waves in turn, a wave of the chunked launch walks its own kv head's keys alone
    constexpr int kStride = CHUNKS ? kMStepKeys : NW * kMStepKeys;

    // ---- chunked launch: the table of this block's items and the cursor of the K/V requests ----
    // An item is a (row, key range), worked on by all waves at once — wave w takes kv head w, so
    // the block as a whole reads whole token rows of the pool.  A wave's requests run PF steps
    // ahead of its arithmetic and cross from one item into the next, so it pays the wait for
    // its first keys once.
    constexpr int kMaxItems = 32;
    constexpr int QV = CHUNKS ? (GQA * D * 2 + 1023) / 1024 : 1;   // 1 KiB pieces of a q tile
    __shared__ int it_row[CHUNKS ? kMaxItems : 1], it_kb[CHUNKS ? kMaxItems : 1], it_ke[CHUNKS ? kMaxItems : 1],
        it_pg[CHUNKS ? kMaxItems : 1], it_slot[CHUNKS ? kMaxItems : 1];
    __shared__ int it_meta[CHUNKS ? 2 : 1];
    __shared__ __attribute__((aligned(16))) unsigned char q_next[CHUNKS ? NW : 1][CHUNKS ? QV * 1024 : 16];
    int n_items = 0, ci = 0, cj = 0, c_ke = 0;
    uint32_t c_pg = 0;
    auto cursor_load = [&]() {
        if (ci < n_items) {
            cj = __builtin_amdgcn_readfirstlane(it_kb[ci]);
            c_ke = __builtin_amdgcn_readfirstlane(it_ke[ci]);
            c_pg = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(it_pg[ci]));
        }
    };
    auto issue_cursor = [&](int slot) {
        if constexpr (CHUNKS) {
            if (ci < n_items) {
                issue(slot, cj, kvh, c_pg, c_ke);
                cj += kStride;
                if (cj >= c_ke) {
                    ++ci;
                    cursor_load();
                }
            }
        }
    };

    auto step = [&](int slot, int j0) {
        stage(slot);
        f32x4_t st[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
        // The fragments of a product are requested together, ahead of its first MFMA (left to
        // itself the compiler requests each next to its use to save registers, and the wave
        // then sits out one LDS round trip per fragment): all of them for one-byte pools (two
        // registers each), KG k-steps at a time for bf16 pools (four each).
        using KFrag = typename std::conditional<Q8, u32x2_t, u32x4_t>::type;
        constexpr int KG = Q8 ? KS : (KS < 2 ? KS : 2);
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += KG) {
            KFrag kc[KG][2];
#pragma unroll
            for (int ks = 0; ks < KG; ++ks)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    if constexpr (!Q8)
                        kc[ks][nt] = *reinterpret_cast<const u32x4_t*>(&Ks[(16 * nt + l16) * KSTRIDE + 32 * (k0 + ks) + 8 * g]);
                    else
                        kc[ks][nt] = *reinterpret_cast<const u32x2_t*>(
                            reinterpret_cast<const unsigned char*>(Ks) + (16 * nt + l16) * STRIDE8 + 32 * (k0 + ks) + 8 * g);
                }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < KG; ++ks)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    u32x4_t kf;
                    if constexpr (!Q8) kf = kc[ks][nt];
                    else kf = kv_decode_bf16<KVF>(kc[ks][nt]);   // 8 codes -> 8 bf16 (exact)
                    st[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kf), qf[k0 + ks], st[nt], 0, 0, 0);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
        // the first V^T fragments are requested here: they arrive while the softmax runs
        constexpr int VG = Q8 ? DT : (DT < 4 ? DT : 4);
        u32x4_t vc[VG];   // (one-byte pools use the first two words)
        auto vfetch = [&](int d0) {
#pragma unroll
            for (int dd = 0; dd < VG; ++dd) {
                const int dt = d0 + dd;
                if constexpr (!Q8) {
                    const uint16_t* va = &Vs[(4 * g + (l16 >> 2)) * VSTRIDE + 16 * dt + 4 * (l16 & 3)];
                    const bf16x4_t v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4_t*)(va));
                    const bf16x4_t v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                        (__attribute__((address_space(3))) bf16x4_t*)(va + 16 * VSTRIDE));
                    vc[dd] = __builtin_bit_cast(u32x4_t, __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7));
                } else {
                    const int rr = l16 >> 1;
                    const int vrow = rr < 4 ? 4 * g + rr : 12 + 4 * g + rr;
                    const unsigned char* va = reinterpret_cast<const unsigned char*>(Vs) + vrow * STRIDE8 + (vrow >> 4) * VUPPER8 +
                                              16 * dt + 8 * (l16 & 1);
                    const i32x2_t c = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2_t*)(va));
                    vc[dd] = u32x4_t{static_cast<uint32_t>(c.x), static_cast<uint32_t>(c.y), 0u, 0u};
                }
            }
        };
        vfetch(0);
        // (one-byte pools) the scales of this lane's keys, before the slot is refilled
        f32x4_t ksc[2], vsc[2];
        if constexpr (Q8) {
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                ksc[nt] = *reinterpret_cast<const f32x4_t*>(&sc_all[wv][16 * nt + 4 * g]);
                vsc[nt] = *reinterpret_cast<const f32x4_t*>(&sc_all[wv][kMStepKeys + 16 * nt + 4 * g]);
            }
        }
        const uint32_t vis = MASKED ? mreg[slot] : 0xFFFFFFFFu;   // bit 16nt + t: key t of unit nt visible
        if constexpr (CHUNKS) issue_cursor(slot);
        else if (j0 + PF * kStride < k_end) issue(slot, j0 + PF * kStride, kvh, pg_lo, k_end);

        // online softmax of query l16 over this lane's keys 16nt + 4g + r
        float sv[8];
        float m_new = mx;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int key = j0 + 16 * nt + 4 * g + rr;
                const float sc = Q8 ? scale_log2e * ksc[nt][rr] : scale_log2e;
                const bool seen = key < k_end && (!MASKED || ((vis >> (16 * nt + 4 * g + rr)) & 1u));
                const float v = seen ? st[nt][rr] * sc : -INFINITY;
                sv[4 * nt + rr] = v;
                m_new = fmaxf(m_new, v);
            }
        m_new = rows_max(m_new);
        const float safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = exp2f(mx - safe);
        mx = m_new;
        float sum = 0.f;
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            float p0 = exp2f(sv[e] - safe), p1 = exp2f(sv[e + 1] - safe);
            sum += p0 + p1;
            if constexpr (Q8) {   // V = float(code) * scale: the scale rides on the probability
                p0 *= vsc[e >> 2][e & 3];
                p1 *= vsc[e >> 2][(e & 3) + 1];
            }
            // p = hi + lo with both parts bf16: hi by truncation, lo = bf16(p - hi)
            const uint32_t b0 = __float_as_uint(p0) & 0xFFFF0000u, b1 = __float_as_uint(p1) & 0xFFFF0000u;
            hi[e >> 1] = (b0 >> 16) | b1;
            lo[e >> 1] = pack_bf16x2(p0 - __uint_as_float(b0), p1 - __uint_as_float(b1));
        }
        lsum = lsum * alpha + sum;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) acc[dt] *= alpha;
        }
        const bf16x8_t p_hi = __builtin_bit_cast(bf16x8_t, u32x4_t{hi[0], hi[1], hi[2], hi[3]});
        const bf16x8_t p_lo = __builtin_bit_cast(bf16x8_t, u32x4_t{lo[0], lo[1], lo[2], lo[3]});
        // V^T fragment of dimension 16 dt + l16: keys 4g..4g+3 and 16+4g..16+4g+3, the order of
        // the probabilities above.  bf16 pools: lane i of the group addresses 8 bytes of row
        // (i / 4) at column block (i % 4) and receives element i of each of the four rows, twice.
        // One-byte pools: the one-byte transposing read — lane i addresses 8 bytes of row (i / 2)
        // at column block (i % 2) and receives byte i of each of the eight rows.
#pragma unroll
        for (int d0 = 0; d0 < DT; d0 += VG) {
            if (d0 > 0) vfetch(d0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int dd = 0; dd < VG; ++dd) {
                bf16x8_t vf;
                if constexpr (!Q8) vf = __builtin_bit_cast(bf16x8_t, vc[dd]);
                else vf = __builtin_bit_cast(bf16x8_t, kv_decode_bf16<KVF>(u32x2_t{vc[dd].x, vc[dd].y}));
                acc[d0 + dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p_hi, acc[d0 + dd], 0, 0, 0);
                acc[d0 + dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p_lo, acc[d0 + dd], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // this wave's result into its own LDS region (as floats), then the four waves are merged
    // into slot pidx0 + h * pstride of the partial results (or, with one split, into the output)
    auto finish = [&](size_t pidx0, int pstride) {
        lsum += __shfl_xor(lsum, 16, kWave);
        lsum += __shfl_xor(lsum, 32, kWave);
        if constexpr (CHUNKS) {
            // (a wave owns its kv head: its partial result goes out as it stands)
            if (l16 < GQA) {
                const size_t pidx = pidx0 + static_cast<size_t>(l16) * pstride;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(&part_o[pidx * D + 16 * dt + 4 * g]) = acc[dt];
                if (g == 0) {
                    part_ml[pidx * 2 + 0] = mx;
                    part_ml[pidx * 2 + 1] = lsum;
                }
            }
            return;
        }
        float* so = reinterpret_cast<float*>(Vs);   // [GQA][D]
        if (l16 < GQA) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) so[l16 * D + 16 * dt + 4 * g + rr] = acc[dt][rr];
            if (g == 0) {
                sm_m[wv][l16] = mx;
                sm_l[wv][l16] = lsum;
            }
        }
        __syncthreads();
        for (int idx = tid; idx < GQA * D; idx += NW * kWave) {
            const int h = idx / D, dd = idx - h * D;
            float m_all = sm_m[0][h];
#pragma unroll
            for (int w = 1; w < NW; ++w) m_all = fmaxf(m_all, sm_m[w][h]);
            const float safe = (m_all == -INFINITY) ? 0.f : m_all;
            float ov = 0.f, ls = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float a = exp2f(sm_m[w][h] - safe);
                ov += reinterpret_cast<const float*>(kv_all[w] + KREGION)[h * D + dd] * a;
                ls += sm_l[w][h] * a;
            }
            const int head = kvh * GQA + h;
            const size_t rh = static_cast<size_t>(r) * hq + head;
            if (o_direct) {
                o_direct[rh * D + dd] = f32_to_bf16_bits(ls > 0.f ? ov / ls : 0.f);
                if (lse && dd == 0)
                    lse[rh] = ls > 0.f ? (logf(ls) + m_all * 0.6931471805599453f) : -INFINITY;
            } else {
                const size_t pidx = pidx0 + static_cast<size_t>(h) * pstride;
                part_o[pidx * D + dd] = ov;
                if (dd == 0) {
                    part_ml[pidx * 2 + 0] = m_all;
                    part_ml[pidx * 2 + 1] = ls;
                }
            }
        }
    };

    if constexpr (!CHUNKS) {
        const int first = k_begin + wv * kMStepKeys;
        if (first < k_end) issue(0, first, kvh, pg_lo, k_end);
        if (first + kStride < k_end) issue(1, first + kStride, kvh, pg_lo, k_end);
        for (int j0 = first; j0 < k_end; j0 += PF * kStride) {
            step(0, j0);
            if (j0 + kStride < k_end) step(1, j0 + kStride);
        }
        finish((static_cast<size_t>(r) * hq + kvh * GQA) * nsplit + split, nsplit);
    } else {
        // ---- The chunked launch.  The keys of all rows, in 16-token units, form one line; block
        // b takes units [b C, (b + 1) C) of it, C = the line's length over the grid, rounded up:
        // every block the same number of keys, whatever the rows' lengths, no block waits for a
        // slot, and the waves of a block (one per kv head) read the same tokens at the same
        // time, i.e. whole rows of the pool.  A chunk cuts the rows it covers into items; the
        // piece of row r inside chunk b goes to slot b + r of the partial results (along the
        // line either b or r grows from one piece to the next, so the slots are distinct and a
        // row's pieces are consecutive), which the merge kernel finds again from the same
        // arithmetic.
        const int R = num_rows, NB = gridDim.x, b = blockIdx.x;
        kvh = wv;
        int* row_pref = reinterpret_cast<int*>(&kv_all[0][0]);   // [R + 1] units before each row (set-up only: the first wave's regions are idle)
        int* row_pg = row_pref + kAttnBlock + 4;
        int* row_kl = row_pg + kAttnBlock;
        static_assert(sizeof(kv_all[0]) >= sizeof(int) * (3 * kAttnBlock + 4), "set-up tables fit a wave's regions");
        int pos = -1;
        for (;;) {
            if (wv == 0) {   // units per row and their prefix sums (again for every table: the regions held keys since)
                int carry = 0;
                for (int base = 0; base < R; base += kWave) {
                    const int rr = base + lane;
                    int n = 0;
                    if (rr < R) {
                        const RowExtent ext = row_extent(page_indptr, last_lens, row_begin, row_len, rr, ps);
                        n = (ext.kv_len + kUnitTokens - 1) / kUnitTokens;
                        row_pg[rr] = static_cast<int>(ext.pg_lo);
                        row_kl[rr] = ext.kv_len;
                    }
                    int x = n;
#pragma unroll
                    for (int off = 1; off < kWave; off <<= 1) {
                        const int y = __shfl_up(x, off, kWave);
                        if (lane >= off) x += y;
                    }
                    if (rr < R) row_pref[rr + 1] = carry + x;
                    carry += __shfl(x, kWave - 1, kWave);
                }
                if (lane == 0) row_pref[0] = 0;
            }
            __syncthreads();
            if (b == 0 && pos == -1) {   // for the merge: each row's first slot and number of pieces
                const int C = max((row_pref[R] + NB - 1) / NB, 1);
                for (int rr = tid; rr < R; rr += NW * kWave) {
                    const int lo = row_pref[rr], hi = row_pref[rr + 1];
                    const int b_lo = lo / C;
                    row_pieces[2 * rr] = b_lo + rr;
                    row_pieces[2 * rr + 1] = hi > lo ? (hi - 1) / C - b_lo + 1 : 0;
                }
            }
            if (tid == 0) {
                const int total = row_pref[R];
                const int C = (total + NB - 1) / NB;
                if (pos < 0) pos = b * C;
                const int chunk_end = min(total, (b + 1) * C);
                int x = pos, n = 0;
                while (x < chunk_end && n < kMaxItems) {
                    int lo = 0, hi = R;   // the row of line position x: pref[lo] <= x < pref[hi]
                    while (hi - lo > 1) {
                        const int mid = (lo + hi) >> 1;
                        if (row_pref[mid] <= x) lo = mid;
                        else hi = mid;
                    }
                    const int u0 = x - row_pref[lo];
                    const int take = min(row_pref[lo + 1] - x, chunk_end - x);
                    it_row[n] = lo;
                    it_kb[n] = u0 * kUnitTokens;
                    it_ke[n] = min((u0 + take) * kUnitTokens, row_kl[lo]);
                    it_pg[n] = row_pg[lo];
                    it_slot[n] = b + lo;
                    x += take;
                    ++n;
                }
                it_meta[0] = n;
                it_meta[1] = x < chunk_end ? x : -2;   // where the next table starts, if the chunk has more
            }
            __syncthreads();
            n_items = __builtin_amdgcn_readfirstlane(it_meta[0]);
            pos = __builtin_amdgcn_readfirstlane(it_meta[1]);
            if (n_items == 0) break;

            ci = 0;
            cursor_load();
            issue_cursor(0);
            issue_cursor(1);
            // The steps of all items in one sequence, alternating between the two slots of keys
            // in flight; between two steps, where an item ends: its partial result goes out, the
            // next one's q fragments come in.
            int item = 0, j0 = 0, slot_out = 0;
            auto begin_item = [&]() {
                r = __builtin_amdgcn_readfirstlane(it_row[item]);
                k_end = __builtin_amdgcn_readfirstlane(it_ke[item]);
                slot_out = __builtin_amdgcn_readfirstlane(it_slot[item]);
                j0 = __builtin_amdgcn_readfirstlane(it_kb[item]);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                mx = -INFINITY, lsum = 0.f;
                if (item == 0) {
                    load_q();
                } else {   // (parked in this wave's q_next during the item before)
                    const bool valid = l16 < GQA;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        u32x4_t v = *reinterpret_cast<const u32x4_t*>(&q_next[wv][((valid ? l16 : 0) * D + 32 * ks + 8 * g) * 2]);
                        if (!valid) v = u32x4_t{0u, 0u, 0u, 0u};
                        qf[ks] = __builtin_bit_cast(bf16x8_t, v);
                    }
                }
            };
            auto one_step = [&](int slot) {   // false once the table is worked off
                // during an item's last step the next item's q tile is fetched (whole 16-byte
                // pieces, lane by lane) and parked in LDS
                const bool last = j0 + kStride >= k_end;
                const bool fetch_q = last && item + 1 < n_items;
                u32x4_t qt[QV];
                if (fetch_q) {
                    const unsigned char* qsrc = reinterpret_cast<const unsigned char*>(
                        q + (static_cast<size_t>(it_row[item + 1]) * hq + kvh * GQA) * D);
#pragma unroll
                    for (int i = 0; i < QV; ++i)
                        qt[i] = *reinterpret_cast<const u32x4_t*>(qsrc + min(i * 1024 + lane * 16, GQA * D * 2 - 16));
                }
                step(slot, j0);
                if (fetch_q) {
#pragma unroll
                    for (int i = 0; i < QV; ++i) *reinterpret_cast<u32x4_t*>(&q_next[wv][i * 1024 + lane * 16]) = qt[i];
                }
                j0 += kStride;
                if (last) {
                    finish((static_cast<size_t>(slot_out) * hk + kvh) * GQA, 1);
                    if (++item >= n_items) return false;
                    begin_item();
                }
                return true;
            };
            begin_item();
            for (;;) {
                if (!one_step(0)) break;
                if (!one_step(1)) break;
            }
            if (pos < 0) break;
            __syncthreads();   // every wave is through with the table before it is rebuilt
        }
    }
}

// One block per (request, q head): combine the splits that exist for this request.  Two
// parallel phases instead of a serial walk over splits: (1) the (max, sum) pairs of all splits
// are loaded at once and reduced to per-split weights in LDS, (2) each thread sums its output
// dimension over splits with independent, unrolled loads.
constexpr int kMaxSplits = 1024;

template <int D>
__global__ __launch_bounds__(D) void attn_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const uint32_t* __restrict__ page_indptr, const uint32_t* __restrict__ last_lens,
    const uint32_t* __restrict__ row_begin, const int32_t* __restrict__ row_len,
    uint16_t* __restrict__ o, float* __restrict__ lse, int hq, int ps, int units_per_split,
    int nsplit) {
    __shared__ float s_w[kMaxSplits];
    __shared__ float s_red[2 * (D / kWave)];
    const int rh = blockIdx.x;
    const int r = rh / hq;
    const int dd = threadIdx.x;
    const int lane = dd & (kWave - 1), wv = dd / kWave;
    const float* ml = part_ml + static_cast<size_t>(rh) * nsplit * 2;
    const float* po = part_o + static_cast<size_t>(rh) * nsplit * D + dd;
    // Everything the block needs is requested at once — the row's extent, the (max, sum) pairs
    // and the first kPre partial outputs of every split slot, used or not (the workspace holds
    // nsplit slots per row; unused ones are masked below) — so the kernel waits for memory once
    // instead of three times in a row.
    constexpr int kPre = 24;
    float pre[kPre];
#pragma unroll
    for (int s = 0; s < kPre; ++s) pre[s] = s < nsplit ? po[static_cast<size_t>(s) * D] : 0.f;
    float2 mine_ml = make_float2(-INFINITY, 0.f);
    if (dd < nsplit) mine_ml = *reinterpret_cast<const float2*>(ml + 2 * dd);
    const int kv_len = row_extent(page_indptr, last_lens, row_begin, row_len, r, ps).kv_len;
    const int nunits = (kv_len + kUnitTokens - 1) / kUnitTokens;
    const int ns = min(nsplit, (nunits + units_per_split - 1) / units_per_split);

    float mloc = dd < ns ? mine_ml.x : -INFINITY;
    for (int s = dd + D; s < ns; s += D) mloc = fmaxf(mloc, ml[2 * s]);
    mloc = wave_max(mloc);
    if (lane == 0) s_red[wv] = mloc;
    __syncthreads();
    float mx = s_red[0];
#pragma unroll
    for (int w = 1; w < D / kWave; ++w) mx = fmaxf(mx, s_red[w]);
    const float safe = (mx == -INFINITY) ? 0.f : mx;
    float lloc = 0.f;
    if (dd < ns) {
        const float a = exp2f(mine_ml.x - safe);
        s_w[dd] = a;
        lloc = mine_ml.y * a;
    }
    for (int s = dd + D; s < ns; s += D) {
        const float a = exp2f(ml[2 * s] - safe);
        s_w[s] = a;
        lloc += ml[2 * s + 1] * a;
    }
    lloc = wave_sum(lloc);
    if (lane == 0) s_red[D / kWave + wv] = lloc;
    __syncthreads();
    float ls = 0.f;
#pragma unroll
    for (int w = 0; w < D / kWave; ++w) ls += s_red[D / kWave + w];

    // the sum over splits keeps its order: four interleaved accumulators over s = 0, 1, 2, ...
    float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
    int s = 0;
#pragma unroll
    for (int b = 0; b < kPre; b += 4) {
        if (b + 4 <= ns) {
            acc0 = fmaf(pre[b], s_w[b], acc0);
            acc1 = fmaf(pre[b + 1], s_w[b + 1], acc1);
            acc2 = fmaf(pre[b + 2], s_w[b + 2], acc2);
            acc3 = fmaf(pre[b + 3], s_w[b + 3], acc3);
            s = b + 4;
        }
    }
    for (; s + 4 <= ns; s += 4) {
        acc0 = fmaf(po[static_cast<size_t>(s) * D], s_w[s], acc0);
        acc1 = fmaf(po[static_cast<size_t>(s + 1) * D], s_w[s + 1], acc1);
        acc2 = fmaf(po[static_cast<size_t>(s + 2) * D], s_w[s + 2], acc2);
        acc3 = fmaf(po[static_cast<size_t>(s + 3) * D], s_w[s + 3], acc3);
    }
    // the last one to three splits, in order (s = ns rounded down to a multiple of four here)
#pragma unroll
    for (int b = 0; b < kPre; ++b)
        if (b >= s && b < ns) acc0 = fmaf(pre[b], s_w[b], acc0);
    for (int t = max(s, kPre); t < ns; ++t) acc0 = fmaf(po[static_cast<size_t>(t) * D], s_w[t], acc0);
    const float ov = (acc0 + acc1) + (acc2 + acc3);
    o[static_cast<size_t>(rh) * D + dd] = f32_to_bf16_bits(ls > 0.f ? ov / ls : 0.f);
    if (lse && dd == 0) lse[rh] = ls > 0.f ? (logf(ls) + mx * 0.6931471805599453f) : -INFINITY;
}

// Zero-length contexts never enter the split kernel; the single-split fast path needs their
// rows cleared (the merge kernel does it itself on the multi-split path).
template <int D>
__global__ void attn_decode_clear_empty_kernel(const uint32_t* __restrict__ page_indptr,
                                               const uint32_t* __restrict__ last_lens,
                                               const uint32_t* __restrict__ row_begin,
                                               const int32_t* __restrict__ row_len,
                                               uint16_t* __restrict__ o, float* __restrict__ lse,
                                               int hq, int ps) {
    const int rh = blockIdx.x;
    const int r = rh / hq;
    const int kv_len = row_extent(page_indptr, last_lens, row_begin, row_len, r, ps).kv_len;
    if (kv_len > 0) return;
    o[static_cast<size_t>(rh) * D + threadIdx.x] = 0;
    if (lse && threadIdx.x == 0) lse[rh] = -INFINITY;
}

// The merge of a chunked launch (attn_decode_mfma_kernel<..., CHUNKS = true>): one block per
// (row, q head).  A row's pieces sit in consecutive slots of the partial results — the piece of
// chunk b in slot b + row, a slot holding the row's q heads in order; the launch's first block
// left each row's first slot and number of pieces in row_pieces.
template <int D>
__global__ __launch_bounds__(D) void attn_decode_merge_chunks_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ row_pieces,
    uint16_t* __restrict__ o, float* __restrict__ lse, int hq) {
    const int rh = blockIdx.x;
    const int r = rh / hq, head = rh - r * hq;
    const int dd = threadIdx.x;
    const size_t slot0 = static_cast<size_t>(row_pieces[2 * r]);
    const int ns = row_pieces[2 * r + 1];
    const size_t out = static_cast<size_t>(rh) * D + dd;
    if (ns == 0) {
        o[out] = 0;
        if (lse && dd == 0) lse[rh] = -INFINITY;
        return;
    }
    const float* ml = part_ml + (slot0 * hq + head) * 2;
    const float* po = part_o + (slot0 * hq + head) * D + dd;
    const size_t ml_step = static_cast<size_t>(hq) * 2, po_step = static_cast<size_t>(hq) * D;
    // (a row is cut by few chunks: the first pieces are requested at once, ahead of the weights)
    constexpr int kPre = 4;
    float pre_o[kPre], pre_m[kPre], pre_l[kPre];
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
        const int ii = min(i, ns - 1);
        pre_o[i] = po[ii * po_step];
        pre_m[i] = ml[ii * ml_step];
        pre_l[i] = ml[ii * ml_step + 1];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < kPre; ++i)
        if (i < ns) mx = fmaxf(mx, pre_m[i]);
    for (int i = kPre; i < ns; ++i) mx = fmaxf(mx, ml[i * ml_step]);
    const float safe = (mx == -INFINITY) ? 0.f : mx;
    float ov = 0.f, ls = 0.f;
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
        if (i < ns) {
            const float a = exp2f(pre_m[i] - safe);
            ov = fmaf(pre_o[i], a, ov);
            ls = fmaf(pre_l[i], a, ls);
        }
    }
    for (int i = kPre; i < ns; ++i) {
        const float a = exp2f(ml[i * ml_step] - safe);
        ov = fmaf(po[i * po_step], a, ov);
        ls = fmaf(ml[i * ml_step + 1], a, ls);
    }
    o[out] = f32_to_bf16_bits(ls > 0.f ? ov / ls : 0.f);
    if (lse && dd == 0) lse[rh] = ls > 0.f ? (logf(ls) + mx * 0.6931471805599453f) : -INFINITY;
}

struct SplitPlan {
    int units_per_split;
    int nsplit;
    int waves = kAttnWaves;   // per block of the gridded launch (eight: whole rows by blocks of twice the width)
};

// pie_hip_attn_rows_paged_partials: the split launch alone, its partial results left in the
// workspace for a consumer that merges them itself (set around the one dispatch call)
thread_local bool t_defer_merge = false;
// pie_hip_attn_rows_paged_kvq_uniform: the caller knows the rows to be about equally long (set
// around the one dispatch call)
thread_local bool t_uniform_rows = false;

// Compute units of the current device (256 on an MI355X; that figure when no device answers).
int resident_attn_blocks() {
    constexpr int kMaxDev = 64;
    static std::mutex mu;
    static int cached[kMaxDev] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 0;
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 0;
        cached[dev] = cus;
    }
    return cached[dev];
}

// Same rule for the workspace query and the launch: aim for >= ~8 blocks per CU over the
// whole batch, never less than one unit per wave and per block.
SplitPlan plan_splits(int R, int hk, int max_kv_len, bool uniform = false) {
    const int max_units = (max_kv_len + kUnitTokens - 1) / kUnitTokens;
    if (max_units <= 0) return {1, 1};
    const long long rows = static_cast<long long>(R) * hk;
    // ~12 blocks per CU measured best on batch 64 x U[512, 8192] contexts (5.0 TB/s vs 4.4 at 8)
    const long long want_blocks = 3072;
    // a block should walk >= 512 tokens when that still leaves two blocks per CU (measured:
    // batch 64 x 1024..2048 tokens runs 8-25 % faster than with 128-token blocks); with few
    // rows, down to 128 tokens so the machine fills
    const long long min_ups = rows * ((max_units + 31) / 32) >= 512 ? 32 : 2 * kAttnWaves;
    long long want_split = (want_blocks + rows - 1) / rows;
    // Batches whose 512-token blocks would not fill two rounds of the resident grid (512 blocks of
    // four waves) take exactly one round: as many splits as put rows * splits at 512 (and not
    // under 448: a round that leaves an eighth of the slots empty is no gain).  A second, partial
    // round leaves most of the machine waiting for its last blocks (measured, 8B decode steps at
    // 2048 keys, batch 4 / 8 / 16: 2.34 / 2.61 / 3.15 -> 2.29 / 2.55 / 3.08 ms; 16 rows at 1024 keys
    // 2.84 -> 2.77; one and two rows plan as before).  Rows the caller knows to be about equally
    // long take the single round up to six rounds' worth of such blocks — then no block outlasts
    // the others, and with one split per row there is nothing to merge (batch 64 at 2048 / 512
    // keys 6.15 / 4.20 -> 5.74 / 3.87 ms, batch 32 at 1024 keys 3.49 -> 3.41, the MoE batch 10.19 ->
    // 10.03); with rows of unknown lengths a long one would run on alone.
    const int cus = resident_attn_blocks();
    const long long slots = 2LL * (cus > 0 ? cus : 256);   // resident blocks: two of four waves per CU
    // Equally long rows that fill at most half of those slots: one block of eight waves per (row,
    // kv head) with nothing to merge, when its waves walk at most a few steps (of 32 keys) more than
    // the waves of a plan that splits every row over the empty slots would.  Rows that fill half
    // the slots (32 rows of 8 kv heads, 64 rows of 4) always do: eight waves are then the same waves
    // in flight as two splits of four.  Fewer than 128 blocks leave most of the chip without key
    // requests in flight, and the longer walk costs more there.
    if (uniform && 2 * rows <= slots && rows >= 32 && rows * ((max_units + 31) / 32) < 6 * slots) {
        const long long ns = slots / rows;
        const long long steps_one = (max_units + 15) / 16, steps_split = (max_units + 8 * ns - 1) / (8 * ns);
        if (steps_one - steps_split <= (rows >= 128 ? 3 : 1)) return {max_units, 1, 2 * kAttnWaves};
    }
    if (rows * ((max_units + 31) / 32) < (uniform ? 6 * slots : slots + slots / 2) && rows <= slots) {
        const long long ns = slots / rows;
        // (equally long rows that fill more than half the slots: one split per row also where an
        // eighth or more of the slots stays empty, as long as the empty share times the rows'
        // length stays under what the second round and the merge of a split plan cost — 48 rows
        // of 8 kv heads at 512 / 2048 keys 3.85 / 5.33 -> 3.60 / 5.22 ms, 36 rows at 512 keys
        // 3.76 -> 3.51, at 2048 keys the splits stay: 4.72 against 5.02)
        const bool short_enough = uniform && ns == 1 && max_units * (slots - rows) <= 40 * slots;
        if (rows * ns >= slots - slots / 8 || short_enough) {
            long long u = (max_units + ns - 1) / ns;
            if (u < 2 * kAttnWaves) u = 2 * kAttnWaves;   // >= 2 units per wave amortises the merge
            if (u > max_units) u = max_units;
            return {static_cast<int>(u), static_cast<int>((max_units + u - 1) / u)};
        }
    }
    long long ups = (max_units + want_split - 1) / want_split;
    if (ups < min_ups) ups = min_ups;  // >= 2 units per wave amortises the merge
    if (ups > max_units) ups = max_units;
    if ((max_units + ups - 1) / ups > kMaxSplits) ups = (max_units + kMaxSplits - 1) / kMaxSplits;
    const int nsplit = static_cast<int>((max_units + ups - 1) / ups);
    return {static_cast<int>(ups), nsplit};
}

// The chunked launch (attn_decode_mfma_kernel<..., CHUNKS = true>): as many blocks as the device
// holds at once, every block the same share of the batch's keys.  Taken for one-byte pools when
// the gridded launch would queue blocks behind one another — its blocks then start and end at
// different times, each waits for its first keys on its own, and a third of the wave slots sit
// idle — and the batch fits the kernel's set-up.  Measured (MI355X, 64 rows of 512-8192 keys,
// 8 kv heads of 128): fp8 / int8 pools 121 / 124 -> 102 us (0.55 -> 0.67 of the HBM peak), a
// 64-row decode step of an 8B model over fp8 pools at 2048 keys 5.42 -> 5.03 ms.  bf16 pools keep
// the gridded launch: it already reads at the rate the chunked one reaches (5.6 TB/s), and the
// chunked launch measured slower there (186 -> 201 us, the same step 6.19 -> 6.64 ms).
struct ChunkPlan {
    bool use;
    int blocks;
    size_t slots;   // partial results: blocks + rows slots of hq heads each
};
ChunkPlan plan_chunks(int R, int hk, int max_kv_len, const SplitPlan& plan, bool one_byte_pool) {
    static const int forced = [] { const char* e = getenv("PIE_HIP_ATTN_CHUNKS"); return e ? atoi(e) : -1; }();   // measurement hook
    // a CU holds eight waves of the kernel (two per SIMD: its registers) = 8 / hk blocks of one
    // wave per kv head
    const int cus = resident_attn_blocks();
    const bool shape = hk == 1 || hk == 2 || hk == 4 || hk == 8;
    const int nb = shape ? cus * (8 / hk) : 0;
    const long long max_units = (max_kv_len + kUnitTokens - 1) / kUnitTokens;
    const bool fits = nb > 0 && R <= kAttnBlock && static_cast<long long>(R) * max_units < (1ll << 30);
    const bool queues = static_cast<long long>(R) * hk * plan.nsplit > 2 * cus;   // more blocks than the gridded launch has resident
    const bool use = fits && !t_defer_merge && (forced >= 0 ? forced != 0 : one_byte_pool && queues);
    return {use, nb, static_cast<size_t>(nb) + static_cast<size_t>(R)};
}

template <int D, int GQA, bool MASKED, int KVF = kKvBf16>
int launch_decode(const uint16_t* q, const void* k_pages, const void* v_pages,
                  const float* k_scales, const float* v_scales, uint16_t* o, float* lse, const uint32_t* page_indices, const uint32_t* page_indptr,
                  const uint32_t* last_lens, const uint32_t* row_begin, const int32_t* row_len,
                  int R, int hq, int hk, int ps, float sm_scale,
                  int max_kv_len, void* workspace, size_t workspace_bytes, const uint16_t* mask_bits,
                  int mask_stride, hipStream_t stream) {
    const SplitPlan plan = plan_splits(R, hk, max_kv_len, t_uniform_rows);
    const float scale_log2e = sm_scale * 1.4426950408889634f;
    {
        // The matrix-core kernel: bf16 and one-byte pools, rows with and without a custom mask.  Measured (MI355X, 8B / 30B-A3B
        // decode steps, four / eight query heads per kv head), matrix-core against dot-product
        // kernel: batch 1 1.808 / 1.860 ms, batch 8 2.68 / 2.80, batch 32 4.07 / 4.13, batch 64 at
        // 2048 keys 7.53 / 7.72, MoE batch 64 7.98 / 8.80; 64 rows of 512-8192 keys 5.61 / 4.96 TB/s.
        // PIE_HIP_ATTN_VALU = 1 / 0 forces one or the other (measurement hook).
        static const int forced = [] { const char* e = getenv("PIE_HIP_ATTN_VALU"); return e ? (atoi(e) ? 1 : 0) : -1; }();
        const bool mfma = forced >= 0 ? forced == 0 : true;
        if (mfma) {
            const int ps_shift = (ps & (ps - 1)) == 0 ? __builtin_ctz(static_cast<unsigned>(ps)) : -1;
            if constexpr (!MASKED) {
                const ChunkPlan cp = plan_chunks(R, hk, max_kv_len, plan, KVF != kKvBf16);
                if (cp.use) {
                    const size_t n_part = cp.slots * hq;
                    const size_t need = n_part * (D + 2) * sizeof(float) + static_cast<size_t>(R) * 2 * sizeof(int);
                    if (!workspace || workspace_bytes < need) return PIE_HIP_ERR_INVALID;
                    float* part_o = static_cast<float*>(workspace);
                    float* part_ml = part_o + n_part * D;
                    int* row_pieces = reinterpret_cast<int*>(part_ml + n_part * 2);
#define PIE_CHUNK_LAUNCH(NWAVES)                                                                                       \
    hipLaunchKernelGGL((attn_decode_mfma_kernel<D, GQA, KVF, false, true, NWAVES>), dim3(cp.blocks), dim3(NWAVES * kWave), \
                       0, stream, q, k_pages, v_pages, k_scales, v_scales, page_indices, page_indptr, last_lens,       \
                       row_begin, row_len, part_o, part_ml, nullptr, nullptr, nullptr, 0, hq, hk, ps, ps_shift, 0, 0,  \
                       scale_log2e, R, row_pieces)
                    if (hk == 8) PIE_CHUNK_LAUNCH(8);
                    else if (hk == 4) PIE_CHUNK_LAUNCH(4);
                    else if (hk == 2) PIE_CHUNK_LAUNCH(2);
                    else PIE_CHUNK_LAUNCH(1);
#undef PIE_CHUNK_LAUNCH
                    hipLaunchKernelGGL((attn_decode_merge_chunks_kernel<D>), dim3(R * hq), dim3(D), 0, stream, part_o,
                                       part_ml, row_pieces, o, lse, hq);
                    return launch_status();
                }
            }
            if constexpr (!MASKED) {
                if (plan.nsplit == 1 && plan.waves == 2 * kAttnWaves) {
                    hipLaunchKernelGGL((attn_decode_mfma_kernel<D, GQA, KVF, false, false, 2 * kAttnWaves>), dim3(hk, 1, R),
                                       dim3(2 * kAttnBlock), 0, stream, q, k_pages, v_pages, k_scales, v_scales,
                                       page_indices, page_indptr, last_lens, row_begin, row_len, nullptr, nullptr, o, lse,
                                       nullptr, 0, hq, hk, ps, ps_shift, plan.units_per_split, 1, scale_log2e, R, nullptr);
                    return launch_status();
                }
            }
            if (plan.nsplit == 1) {
                hipLaunchKernelGGL((attn_decode_mfma_kernel<D, GQA, KVF, MASKED>), dim3(hk, 1, R), dim3(kAttnBlock), 0,
                                   stream, q, k_pages, v_pages, k_scales, v_scales, page_indices, page_indptr,
                                   last_lens, row_begin, row_len,
                                   nullptr, nullptr, o, lse, mask_bits, mask_stride, hq, hk, ps, ps_shift,
                                   plan.units_per_split, 1, scale_log2e, R, nullptr);
                return launch_status();
            }
            const size_t n_part = static_cast<size_t>(R) * hq * plan.nsplit;
            const size_t need = n_part * (D + 2) * sizeof(float);
            if (!workspace || workspace_bytes < need) return PIE_HIP_ERR_INVALID;
            float* part_o = static_cast<float*>(workspace);
            float* part_ml = part_o + n_part * D;
            hipLaunchKernelGGL((attn_decode_mfma_kernel<D, GQA, KVF, MASKED>), dim3(hk, plan.nsplit, R), dim3(kAttnBlock), 0,
                               stream, q, k_pages, v_pages, k_scales, v_scales, page_indices, page_indptr,
                               last_lens, row_begin, row_len,
                               part_o, part_ml, nullptr, nullptr, mask_bits, mask_stride, hq, hk, ps, ps_shift,
                               plan.units_per_split, plan.nsplit, scale_log2e, R, nullptr);
            if (!t_defer_merge)
                hipLaunchKernelGGL((attn_decode_merge_kernel<D>), dim3(R * hq), dim3(D), 0, stream, part_o,
                                   part_ml, page_indptr, last_lens, row_begin, row_len, o, lse, hq, ps,
                                   plan.units_per_split, plan.nsplit);
            return launch_status();
        }
    }
    if (plan.nsplit == 1) {
        hipLaunchKernelGGL((attn_decode_clear_empty_kernel<D>), dim3(R * hq), dim3(D), 0, stream,
                           page_indptr, last_lens, row_begin, row_len, o, lse, hq, ps);
        hipLaunchKernelGGL((attn_decode_split_kernel<D, GQA, MASKED, KVF>), dim3(hk, 1, R),
                           dim3(kAttnBlock), 0, stream, q, k_pages, v_pages, k_scales, v_scales, page_indices,
                           page_indptr, last_lens, row_begin, row_len, nullptr, nullptr, o, lse,
                           mask_bits, mask_stride, hq, hk, ps, plan.units_per_split, 1, scale_log2e);
        return launch_status();
    }
    const size_t n_part = static_cast<size_t>(R) * hq * plan.nsplit;
    const size_t need = n_part * (D + 2) * sizeof(float);
    if (!workspace || workspace_bytes < need) return PIE_HIP_ERR_INVALID;
    float* part_o = static_cast<float*>(workspace);
    float* part_ml = part_o + n_part * D;
    hipLaunchKernelGGL((attn_decode_split_kernel<D, GQA, MASKED, KVF>), dim3(hk, plan.nsplit, R),
                       dim3(kAttnBlock), 0, stream, q, k_pages, v_pages, k_scales, v_scales, page_indices, page_indptr,
                       last_lens, row_begin, row_len, part_o, part_ml, nullptr, nullptr, mask_bits,
                       mask_stride, hq, hk, ps, plan.units_per_split, plan.nsplit, scale_log2e);
    if (!t_defer_merge)
        hipLaunchKernelGGL((attn_decode_merge_kernel<D>), dim3(R * hq), dim3(D), 0, stream, part_o,
                           part_ml, page_indptr, last_lens, row_begin, row_len, o, lse, hq, ps,
                           plan.units_per_split,
                           plan.nsplit);
    return launch_status();
}

}  // namespace
}  // namespace pie_hip

extern "C" size_t pie_hip_attn_decode_workspace_bytes(int num_requests, int num_q_heads,
                                                      int num_kv_heads, int head_dim,
                                                      int max_kv_len) {
    if (num_requests <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0) return 0;
    const pie_hip::SplitPlan plan = pie_hip::plan_splits(num_requests, num_kv_heads, max_kv_len);
    // (the plan for rows of unknown lengths and the one for rows known to be equally long:
    // whichever needs more)
    const int most_splits = std::max(plan.nsplit, pie_hip::plan_splits(num_requests, num_kv_heads, max_kv_len, true).nsplit);
    const size_t gridded = most_splits == 1 ? 0
                                            : static_cast<size_t>(num_requests) * num_q_heads * most_splits *
                                                  (head_dim + 2) * sizeof(float);
    // (the chunked launch's partial results, where a launch over one-byte pools without custom
    // masks would take it; bf16 pools and masked rows of the same shape keep the gridded launch)
    const pie_hip::ChunkPlan cp = pie_hip::plan_chunks(num_requests, num_kv_heads, max_kv_len, plan, true);
    const size_t chunked = cp.use ? cp.slots * num_q_heads * (head_dim + 2) * sizeof(float) +
                                        static_cast<size_t>(num_requests) * 2 * sizeof(int)
                                  : 0;
    return gridded > chunked ? gridded : chunked;
}

namespace pie_hip {
namespace {
int attn_dispatch(const uint16_t* q, const void* k_pages, const void* v_pages, uint16_t* o,
                  float* lse, const uint32_t* kv_page_indices, const uint32_t* kv_page_indptr,
                  const uint32_t* kv_last_page_lens, const uint32_t* row_begin,
                  const int32_t* row_len, int num_rows, int num_q_heads, int num_kv_heads,
                  int head_dim, int page_size, float sm_scale, int max_kv_len, void* workspace,
                  size_t workspace_bytes, void* stream, const uint16_t* mask_bits = nullptr,
                  int mask_stride = 0, int kv_format = PIE_HIP_KV_BF16, const float* k_scales = nullptr,
                  const float* v_scales = nullptr) {
    if (mask_bits && mask_stride < (max_kv_len + kUnitTokens - 1) / kUnitTokens) return PIE_HIP_ERR_INVALID;
    if (!q || !k_pages || !v_pages || !o || !kv_page_indices || num_rows <= 0 ||
        num_q_heads <= 0 || num_kv_heads <= 0 || page_size <= 0 || max_kv_len < 0)
        return PIE_HIP_ERR_INVALID;
    if (num_q_heads % num_kv_heads != 0 || page_size % kUnitTokens != 0)
        return PIE_HIP_ERR_UNSUPPORTED;
    if (num_rows > 65535 || num_kv_heads > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf(static_cast<float>(head_dim));
    const int gqa = num_q_heads / num_kv_heads;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // one-byte KV formats: per-(token, head) scales required for int8 and the scaled fp8 form,
    // absent for plain fp8 casts
    if (kv_format != PIE_HIP_KV_BF16) {
        const bool scaled = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD || kv_format == PIE_HIP_KV_FP8_PER_TOKEN_HEAD;
        if (kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2 && !scaled) return PIE_HIP_ERR_UNSUPPORTED;
        if (scaled != (k_scales != nullptr) || scaled != (v_scales != nullptr)) return PIE_HIP_ERR_INVALID;
    }
#define PIE_ATTN_CASE(DD, GG)                                                                  \
    if (head_dim == DD && gqa == GG) {                                                         \
        if (kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD && mask_bits)                          \
            return launch_decode<DD, GG, true, kKvInt8>(                                       \
                q, k_pages, v_pages, k_scales, v_scales, o, lse, kv_page_indices,              \
                kv_page_indptr, kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads,  \
                num_kv_heads, page_size, scale, max_kv_len, workspace, workspace_bytes,        \
                mask_bits, mask_stride, st);                                                   \
        if (kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD)                                       \
            return launch_decode<DD, GG, false, kKvInt8>(                                      \
                q, k_pages, v_pages, k_scales, v_scales, o, lse, kv_page_indices,              \
                kv_page_indptr, kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads,  \
                num_kv_heads, page_size, scale, max_kv_len, workspace, workspace_bytes,        \
                nullptr, 0, st);                                                               \
        if (kv_format == PIE_HIP_KV_FP8_E5M2 && mask_bits)                                     \
            return launch_decode<DD, GG, true, kKvBf8>(                                        \
                q, k_pages, v_pages, k_scales, v_scales, o, lse, kv_page_indices,              \
                kv_page_indptr, kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads,  \
                num_kv_heads, page_size, scale, max_kv_len, workspace, workspace_bytes,        \
                mask_bits, mask_stride, st);                                                   \
        if (kv_format == PIE_HIP_KV_FP8_E5M2)                                                  \
            return launch_decode<DD, GG, false, kKvBf8>(                                       \
                q, k_pages, v_pages, k_scales, v_scales, o, lse, kv_page_indices,              \
                kv_page_indptr, kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads,  \
                num_kv_heads, page_size, scale, max_kv_len, workspace, workspace_bytes,        \
                nullptr, 0, st);                                                               \
        if (kv_format != PIE_HIP_KV_BF16 && mask_bits)                                         \
            return launch_decode<DD, GG, true, kKvFp8>(                                        \
                q, k_pages, v_pages, k_scales, v_scales, o, lse, kv_page_indices,              \
                kv_page_indptr, kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads,  \
                num_kv_heads, page_size, scale, max_kv_len, workspace, workspace_bytes,        \
                mask_bits, mask_stride, st);                                                   \
        if (kv_format != PIE_HIP_KV_BF16)                                                      \
            return launch_decode<DD, GG, false, kKvFp8>(                                       \
                q, k_pages, v_pages, k_scales, v_scales, o, lse, kv_page_indices,              \
                kv_page_indptr, kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads,  \
                num_kv_heads, page_size, scale, max_kv_len, workspace, workspace_bytes,        \
                nullptr, 0, st);                                                               \
        if (mask_bits)                                                                         \
            return launch_decode<DD, GG, true>(                                                \
                q, k_pages, v_pages, nullptr, nullptr, o, lse, kv_page_indices, kv_page_indptr, \
                kv_last_page_lens, row_begin, row_len, num_rows, num_q_heads, num_kv_heads,    \
                page_size, scale, max_kv_len, workspace, workspace_bytes, mask_bits,           \
                mask_stride, st);                                                              \
        return launch_decode<DD, GG, false>(q, k_pages, v_pages, nullptr, nullptr, o, lse,     \
                                            kv_page_indices,                                   \
                                            kv_page_indptr, kv_last_page_lens, row_begin,      \
                                            row_len, num_rows, num_q_heads, num_kv_heads,      \
                                            page_size, scale, max_kv_len, workspace,           \
                                            workspace_bytes, nullptr, 0, st);                  \
    }
    PIE_ATTN_CASE(128, 1)
    PIE_ATTN_CASE(128, 2)
    PIE_ATTN_CASE(128, 4)
    PIE_ATTN_CASE(128, 8)
    PIE_ATTN_CASE(64, 1)
    PIE_ATTN_CASE(64, 2)
    PIE_ATTN_CASE(64, 4)
    PIE_ATTN_CASE(64, 8)
#undef PIE_ATTN_CASE
    return PIE_HIP_ERR_UNSUPPORTED;
}
}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_attn_decode_paged(const uint16_t* q, const uint16_t* k_pages,
                                         const uint16_t* v_pages, uint16_t* o, float* lse,
                                         const uint32_t* kv_page_indices,
                                         const uint32_t* kv_page_indptr,
                                         const uint32_t* kv_last_page_lens, int num_requests,
                                         int num_q_heads, int num_kv_heads, int head_dim,
                                         int page_size, float sm_scale, int max_kv_len,
                                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!kv_page_indptr || !kv_last_page_lens) return PIE_HIP_ERR_INVALID;
    return pie_hip::attn_dispatch(q, k_pages, v_pages, o, lse, kv_page_indices, kv_page_indptr,
                                  kv_last_page_lens, nullptr, nullptr, num_requests, num_q_heads,
                                  num_kv_heads, head_dim, page_size, sm_scale, max_kv_len,
                                  workspace, workspace_bytes, stream);
}

extern "C" int pie_hip_attn_rows_paged(const uint16_t* q, const uint16_t* k_pages,
                                       const uint16_t* v_pages, uint16_t* o, float* lse,
                                       const uint32_t* kv_page_indices,
                                       const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                       int num_rows, int num_q_heads, int num_kv_heads,
                                       int head_dim, int page_size, float sm_scale,
                                       int max_kv_len, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    if (!row_page_begin || !row_kv_len) return PIE_HIP_ERR_INVALID;
    return pie_hip::attn_dispatch(q, k_pages, v_pages, o, lse, kv_page_indices, nullptr, nullptr,
                                  row_page_begin, row_kv_len, num_rows, num_q_heads, num_kv_heads,
                                  head_dim, page_size, sm_scale, max_kv_len, workspace,
                                  workspace_bytes, stream);
}

extern "C" int pie_hip_attn_decode_is_chunked(int kv_format, int num_rows, int num_kv_heads, int max_kv_len) {
    if (num_rows <= 0 || num_kv_heads <= 0 || max_kv_len < 0) return 0;
    const pie_hip::SplitPlan plan = pie_hip::plan_splits(num_rows, num_kv_heads, max_kv_len);
    return pie_hip::plan_chunks(num_rows, num_kv_heads, max_kv_len, plan, kv_format != PIE_HIP_KV_BF16).use ? 1 : 0;
}

extern "C" int pie_hip_attn_decode_plan(int num_rows, int num_kv_heads, int max_kv_len, int* units_per_split,
                                        int* num_splits) {
    if (num_rows <= 0 || num_kv_heads <= 0 || max_kv_len < 0 || !units_per_split || !num_splits)
        return PIE_HIP_ERR_INVALID;
    const pie_hip::SplitPlan plan = pie_hip::plan_splits(num_rows, num_kv_heads, max_kv_len);
    *units_per_split = plan.units_per_split;
    *num_splits = plan.nsplit;
    return PIE_HIP_OK;
}

extern "C" int pie_hip_attn_rows_paged_partials(int kv_format, const uint16_t* q, const void* k_pages,
                                                const void* v_pages, const float* k_scales,
                                                const float* v_scales, const uint32_t* kv_page_indices,
                                                const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                                int num_rows, int num_q_heads, int num_kv_heads, int head_dim,
                                                int page_size, float sm_scale, int max_kv_len, void* workspace,
                                                size_t workspace_bytes, void* stream) {
    if (!row_page_begin || !row_kv_len || !workspace || num_rows <= 0 || num_kv_heads <= 0)
        return PIE_HIP_ERR_INVALID;
    if (pie_hip::plan_splits(num_rows, num_kv_heads, max_kv_len).nsplit < 2) return PIE_HIP_ERR_INVALID;
    // (the output pointer is only checked, never written: the partial results are the output)
    pie_hip::t_defer_merge = true;
    const int rc = pie_hip::attn_dispatch(q, k_pages, v_pages, static_cast<uint16_t*>(workspace), nullptr,
                                          kv_page_indices, nullptr, nullptr, row_page_begin, row_kv_len, num_rows,
                                          num_q_heads, num_kv_heads, head_dim, page_size, sm_scale, max_kv_len,
                                          workspace, workspace_bytes, stream, nullptr, 0, kv_format, k_scales,
                                          v_scales);
    pie_hip::t_defer_merge = false;
    return rc;
}

// ---------------------------------------------------------------------------------------------
// pie_hip_attn_rows_paged for callers that cannot allocate: the split partials live in a
// file-scope device array instead of a caller workspace.  Each GPU holds its own copy of the
// array at its own address; the address is looked up once per device and kept.
namespace pie_hip {
namespace {
constexpr size_t kStaticScratchBytes = PIE_HIP_ATTN_STATIC_SCRATCH_BYTES;
constexpr int kStaticScratchMaxDevices = 64;
}  // namespace
}  // namespace pie_hip

static __device__ __align__(256) unsigned char scratch[pie_hip::kStaticScratchBytes];

namespace pie_hip {
namespace {
std::mutex g_scratch_mu;
void* g_scratch_ptr[kStaticScratchMaxDevices] = {};

// The device-side address of `scratch` on the current device (nullptr on failure).
void* static_scratch_for_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticScratchMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_attn_rows_paged_static(const uint16_t* q, const uint16_t* k_pages,
                                              const uint16_t* v_pages, uint16_t* o, float* lse,
                                              const uint32_t* kv_page_indices,
                                              const uint32_t* row_page_begin,
                                              const int32_t* row_kv_len, int num_rows,
                                              int num_q_heads, int num_kv_heads, int head_dim,
                                              int page_size, float sm_scale, int max_kv_len,
                                              void* stream) {
    if (!row_page_begin || !row_kv_len) return PIE_HIP_ERR_INVALID;
    const size_t need = pie_hip_attn_decode_workspace_bytes(num_rows, num_q_heads, num_kv_heads,
                                                            head_dim, max_kv_len);
    if (need > pie_hip::kStaticScratchBytes) {
        fprintf(stderr,
                "pie_hip_attn_rows_paged_static: %d rows x %d heads over up to %d keys need %zu bytes of "
                "split partials, the built-in scratch holds %zu\n",
                num_rows, num_q_heads, max_kv_len, need, pie_hip::kStaticScratchBytes);
        return PIE_HIP_ERR_UNSUPPORTED;
    }
    void* ws = pie_hip::static_scratch_for_current_device();
    if (!ws) return PIE_HIP_ERR_LAUNCH;
    // Every partial slot the merge reads is written by the split kernel of the same call, so
    // nothing in the array has to start at zero.
    return pie_hip::attn_dispatch(q, k_pages, v_pages, o, lse, kv_page_indices, nullptr, nullptr,
                                  row_page_begin, row_kv_len, num_rows, num_q_heads, num_kv_heads,
                                  head_dim, page_size, sm_scale, max_kv_len, ws,
                                  pie_hip::kStaticScratchBytes, stream);
}

extern "C" int pie_hip_attn_rows_paged_kvq(int kv_format, const uint16_t* q, const void* k_pages,
                                           const void* v_pages, const float* k_scales,
                                           const float* v_scales, uint16_t* o, float* lse,
                                           const uint32_t* kv_page_indices,
                                           const uint32_t* row_page_begin,
                                           const int32_t* row_kv_len, int num_rows,
                                           int num_q_heads, int num_kv_heads, int head_dim,
                                           int page_size, float sm_scale, int max_kv_len,
                                           void* workspace, size_t workspace_bytes, void* stream) {
    if (!row_page_begin || !row_kv_len) return PIE_HIP_ERR_INVALID;
    return pie_hip::attn_dispatch(q, k_pages, v_pages, o, lse, kv_page_indices, nullptr, nullptr,
                                  row_page_begin, row_kv_len, num_rows, num_q_heads, num_kv_heads,
                                  head_dim, page_size, sm_scale, max_kv_len, workspace,
                                  workspace_bytes, stream, nullptr, 0, kv_format, k_scales, v_scales);
}

extern "C" int pie_hip_attn_rows_paged_kvq_uniform(int kv_format, const uint16_t* q, const void* k_pages,
                                                   const void* v_pages, const float* k_scales,
                                                   const float* v_scales, uint16_t* o, float* lse,
                                                   const uint32_t* kv_page_indices,
                                                   const uint32_t* row_page_begin,
                                                   const int32_t* row_kv_len, int num_rows,
                                                   int num_q_heads, int num_kv_heads, int head_dim,
                                                   int page_size, float sm_scale, int max_kv_len,
                                                   void* workspace, size_t workspace_bytes, void* stream) {
    pie_hip::t_uniform_rows = true;
    const int rc = pie_hip_attn_rows_paged_kvq(kv_format, q, k_pages, v_pages, k_scales, v_scales, o, lse,
                                               kv_page_indices, row_page_begin, row_kv_len, num_rows, num_q_heads,
                                               num_kv_heads, head_dim, page_size, sm_scale, max_kv_len, workspace,
                                               workspace_bytes, stream);
    pie_hip::t_uniform_rows = false;
    return rc;
}

extern "C" int pie_hip_attn_rows_paged_kvq_masked(int kv_format, const uint16_t* q, const void* k_pages,
                                                  const void* v_pages, const float* k_scales,
                                                  const float* v_scales, uint16_t* o, float* lse,
                                                  const uint32_t* kv_page_indices,
                                                  const uint32_t* row_page_begin,
                                                  const int32_t* row_kv_len, const uint16_t* mask_bitmap,
                                                  int mask_stride_units, int num_rows, int num_q_heads,
                                                  int num_kv_heads, int head_dim, int page_size,
                                                  float sm_scale, int max_kv_len, void* workspace,
                                                  size_t workspace_bytes, void* stream) {
    if (!row_page_begin || !row_kv_len || !mask_bitmap || mask_stride_units <= 0) return PIE_HIP_ERR_INVALID;
    return pie_hip::attn_dispatch(q, k_pages, v_pages, o, lse, kv_page_indices, nullptr, nullptr,
                                  row_page_begin, row_kv_len, num_rows, num_q_heads, num_kv_heads,
                                  head_dim, page_size, sm_scale, max_kv_len, workspace,
                                  workspace_bytes, stream, mask_bitmap, mask_stride_units, kv_format,
                                  k_scales, v_scales);
}

namespace pie_hip {
namespace {

// Writes this step's K / V rows [N, hk, d] bf16 into a one-byte pool at the tokens' slots:
// one wave per (token, kv head).  Per-(token, head) formats: scale = absmax / qmax (1 for an
// all-zero row), code = x * (1 / scale) rounded to nearest even and clamped (int8: [-128, 127];
// e4m3: saturating at 448); plain fp8: the saturating cast of x itself.  The arithmetic of
// write_kv_per_token_head_kernel / write_kv_fp8_per_tensor_kernel,
// driver/cuda/src/kernels/kv_paged.cu:155-297.
// f32 -> e5m2 byte, round to nearest even, saturating at the largest finite value (57344), as
// __nv_cvt_float_to_fp8(x, __NV_SATFINITE, __NV_E5M2) (driver/cuda/src/kernels/kv_paged.cu:181-184).
__device__ __forceinline__ unsigned char f32_to_e5m2_sat(float f) {
    const float c = fminf(fmaxf(f, -57344.f), 57344.f);
    return static_cast<unsigned char>(__builtin_amdgcn_cvt_pk_bf8_f32(c, c, 0, false) & 0xFF);
}

// Nearest of +-{0, .5, 1, 1.5, 2, 3, 4, 6}, the smaller magnitude on a tie, sign bit for x < 0
// (quant_fp4_e2m1, kv_paged.cu:309-323): the level index is the number of midpoints below |x|.
__device__ __forceinline__ unsigned f32_to_e2m1(float x) {
    const float ax = fabsf(x);
    const unsigned mag = (ax > 0.25f) + (ax > 0.75f) + (ax > 1.25f) + (ax > 1.75f) + (ax > 2.5f) + (ax > 3.5f) +
                         (ax > 5.f);
    return mag | (x < 0.f ? 8u : 0u);
}
__device__ __forceinline__ float e2m1_to_f32(unsigned code) {
    // magnitudes 0, .5, 1, 1.5 are code / 2; 2, 3, 4, 6 are (2 + (code & 1)) << ((code >> 1) - 2)
    const unsigned m = code & 7u;
    const float v = m < 4u ? 0.5f * static_cast<float>(m) : static_cast<float>((2u + (m & 1u)) << ((m >> 1) - 2u));
    return (code & 8u) ? -v : v;
}

// One-byte / 4-bit pools -> bf16 pools for the pages a batch reads: thread = eight consecutive
// elements of one (page, slot, kv head) row; the value is bf16(float(code) * scale)
// (dequant_*_pages_active_kernel, kv_paged.cu:419-531).
__global__ __launch_bounds__(256) void kv_dequant_pages_kernel(
    const unsigned char* __restrict__ k_pages, const unsigned char* __restrict__ v_pages,
    const float* __restrict__ k_scales, const float* __restrict__ v_scales,
    uint16_t* __restrict__ k_out, uint16_t* __restrict__ v_out, const uint32_t* __restrict__ page_ids,
    size_t total, int hk, int d, int ps, int kv_format) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int vecs = d / 8;                       // eight-element pieces per row
    const int piece = static_cast<int>(idx % vecs);
    size_t rest = idx / vecs;
    const int h = static_cast<int>(rest % hk);
    rest /= hk;
    const int slot = static_cast<int>(rest % ps);
    const size_t page = page_ids[rest / ps];
    const size_t th = (page * ps + slot) * hk + h;
    const size_t sc_at = kv_scale_index(page, slot, h, hk, ps);
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const unsigned char* src = which ? v_pages : k_pages;
        const float* scales = which ? v_scales : k_scales;
        float f[8];
        float scale = 1.f;
        if (kv_format == PIE_HIP_KV_FP4_BLOCK) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(src + th * (d / 2) + piece * 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = e2m1_to_f32((w >> (4 * e)) & 0xFu);
            scale = scales[sc_at * ((d + 15) / 16) + (piece >> 1)];
        } else {
            const u32x2_t w = *reinterpret_cast<const u32x2_t*>(src + th * d + piece * 8);
            if (kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD) kv_decode_f32<kKvInt8>(w, f);
            else if (kv_format == PIE_HIP_KV_FP8_E5M2) kv_decode_f32<kKvBf8>(w, f);
            else kv_decode_f32<kKvFp8>(w, f);
            if (scales) scale = scales[sc_at];
        }
        const u32x4_t out = {pack_bf16x2(f[0] * scale, f[1] * scale), pack_bf16x2(f[2] * scale, f[3] * scale),
                             pack_bf16x2(f[4] * scale, f[5] * scale), pack_bf16x2(f[6] * scale, f[7] * scale)};
        *reinterpret_cast<u32x4_t*>((which ? v_out : k_out) + th * d + piece * 8) = out;
    }
}

__global__ __launch_bounds__(256) void kv_write_quant_kernel(
    const uint16_t* __restrict__ k_src, const uint16_t* __restrict__ v_src,
    const int64_t* __restrict__ kv_slots, unsigned char* __restrict__ k_pages,
    unsigned char* __restrict__ v_pages, float* __restrict__ k_scales,
    float* __restrict__ v_scales, int n_rows, int hk, int d, int ps, int kv_format) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;   // (token, head)
    if (row >= n_rows) return;
    const int t = row / hk, h = row - t * hk;
    const int64_t slot = kv_slots[t];
    if (slot < 0) return;
    const size_t src = static_cast<size_t>(row) * d;
    const size_t th = static_cast<size_t>(slot) * hk + h;
    if (kv_format == PIE_HIP_KV_FP4_BLOCK) {
        // e2m1 codes, two per byte, one fp32 scale per block of 16 elements: a lane owns two
        // adjacent elements, eight lanes a block (write_kv_fp4_block_kernel, kv_paged.cu:325-417)
        const int nb = (d + 15) / 16, pd = d / 2;
        const size_t sc0 = kv_scale_index_of_slot(slot, h, hk, ps) * nb;
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            const uint16_t* x = which ? v_src : k_src;
            unsigned char* dst = (which ? v_pages : k_pages) + th * pd;
            float* sc = (which ? v_scales : k_scales) + sc0;
            for (int base = 0; base < d; base += 2 * kWave) {
                const int j0 = base + 2 * lane;
                const bool in = j0 < d;
                const float f0 = in ? bf16_bits_to_f32(x[src + j0]) : 0.f;
                const float f1 = in ? bf16_bits_to_f32(x[src + j0 + 1]) : 0.f;
                float amax = fmaxf(fabsf(f0), fabsf(f1));
                amax = fmaxf(amax, __shfl_xor(amax, 1, kWave));
                amax = fmaxf(amax, __shfl_xor(amax, 2, kWave));
                amax = fmaxf(amax, __shfl_xor(amax, 4, kWave));
                const float scale = amax > 0.f ? amax / 6.f : 1.f;
                const float inv = 1.f / scale;
                if (in) {
                    dst[j0 >> 1] = static_cast<unsigned char>(f32_to_e2m1(f0 * inv) | (f32_to_e2m1(f1 * inv) << 4));
                    if ((lane & 7) == 0) sc[j0 >> 4] = scale;
                }
            }
        }
        return;
    }
    const bool scaled = kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2;
    const size_t sc_at = scaled ? kv_scale_index_of_slot(slot, h, hk, ps) : 0;
    const float qmax = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD ? 127.f : 448.f;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const uint16_t* x = which ? v_src : k_src;
        unsigned char* dst = (which ? v_pages : k_pages) + th * d;
        float inv = 1.f;
        if (scaled) {
            float amax = 0.f;
            for (int j = lane; j < d; j += kWave) amax = fmaxf(amax, fabsf(bf16_bits_to_f32(x[src + j])));
            amax = wave_max(amax);
            const float scale = amax > 0.f ? amax / qmax : 1.f;
            inv = 1.f / scale;
            if (lane == 0) (which ? v_scales : k_scales)[sc_at] = scale;
        }
        for (int j = lane; j < d; j += kWave) {
            const float f = bf16_bits_to_f32(x[src + j]) * inv;
            if (kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD) {
                int qv = static_cast<int>(rintf(f));
                qv = qv > 127 ? 127 : (qv < -128 ? -128 : qv);
                dst[j] = static_cast<unsigned char>(static_cast<int8_t>(qv));
            } else if (kv_format == PIE_HIP_KV_FP8_E5M2) {
                dst[j] = f32_to_e5m2_sat(f);
            } else {
                const float c = fminf(fmaxf(f, -448.f), 448.f);
                dst[j] = static_cast<unsigned char>(__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xFF);
            }
        }
    }
}

// The same quantiser behind the RoPE stage: one wave per (token, head) of a packed q|k|v row
// rotates its head as qkv_rope_kvwrite_kernel does (optional per-head RMSNorm, both pairings),
// rounds to bf16 — the values the two-kernel path stages as rows — and, for K and V heads,
// quantises them from registers into the token's slot.  q heads go to q_out.
template <int ITER>   // pairs per lane: head_dim <= 128 * ITER
__global__ __launch_bounds__(64) void qkv_rope_kvwrite_quant_kernel(
    const uint16_t* __restrict__ packed, uint16_t* __restrict__ q_out,
    unsigned char* __restrict__ k_pages, unsigned char* __restrict__ v_pages,
    float* __restrict__ k_scales, float* __restrict__ v_scales,
    const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
    const float* __restrict__ rope_table, const int64_t* __restrict__ kv_slots, int hq, int hk,
    int d, int ps, int interleaved, float eps, int kv_format) {
    const int n = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int half = d / 2;
    const size_t stride = static_cast<size_t>(hq + 2 * hk) * d;
    const uint16_t* src = packed + n * stride + static_cast<size_t>(head) * d;
    const bool is_q = head < hq, is_k = !is_q && head < hq + hk;
    const int64_t slot = kv_slots[n];
    if (!is_q && slot < 0) return;  // token without a KV slot
    // this lane's pairs (ia, ib) and their bf16 values after the optional norm and rotation
    float va[ITER], vb[ITER];
    const uint16_t* nw = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
    float inv_rms = 1.f;
    if (nw) {
        float local = 0.f;
        for (int i = lane; i < d; i += kWave) {
            const float v = bf16_bits_to_f32(src[i]);
            local += v * v;
        }
        inv_rms = rsqrtf(wave_sum(local) / static_cast<float>(d) + eps);
    }
    const float* tab = rope_table + static_cast<size_t>(n) * d;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int i = lane + it * kWave;
        va[it] = vb[it] = 0.f;
        if (i < half) {
            // (interleaved = 2: q / k rows re-ordered at load, elements (2i, 2i+1) hold the
            // half-split pair (i, i+d/2) and go back to those positions; V rows are as stored)
            const int pin = (interleaved == 2 && !(is_q || is_k)) ? 0 : interleaved;
            const int ia = pin ? 2 * i : i, ib = pin ? 2 * i + 1 : i + half;
            const int oa = pin == 1 ? 2 * i : i, ob = pin == 1 ? 2 * i + 1 : i + half;
            float a = bf16_bits_to_f32(src[ia]), b = bf16_bits_to_f32(src[ib]);
            if (is_q || is_k) {
                if (nw) {
                    a = a * inv_rms * bf16_bits_to_f32(nw[oa]);
                    b = b * inv_rms * bf16_bits_to_f32(nw[ob]);
                }
                const float c = tab[i], sn = tab[i + half];
                const float ra = a * c - b * sn, rb = b * c + a * sn;
                a = bf16_bits_to_f32(f32_to_bf16_bits(ra));
                b = bf16_bits_to_f32(f32_to_bf16_bits(rb));
            }
            va[it] = a;
            vb[it] = b;
            if (is_q) {
                uint16_t* dst = q_out + (static_cast<size_t>(n) * hq + head) * d;
                dst[oa] = f32_to_bf16_bits(a);
                dst[ob] = f32_to_bf16_bits(b);
            }
        }
    }
    if (is_q) return;
    const int h = is_k ? head - hq : head - hq - hk;
    const size_t th = static_cast<size_t>(slot) * hk + h;
    unsigned char* dst = (is_k ? k_pages : v_pages) + th * d;
    const bool scaled = kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2;
    const float qmax = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD ? 127.f : 448.f;
    float inv = 1.f;
    if (scaled) {
        float amax = 0.f;
#pragma unroll
        for (int it = 0; it < ITER; ++it) amax = fmaxf(amax, fmaxf(fabsf(va[it]), fabsf(vb[it])));
        amax = wave_max(amax);
        const float scale = amax > 0.f ? amax / qmax : 1.f;
        inv = 1.f / scale;
        if (lane == 0) (is_k ? k_scales : v_scales)[kv_scale_index_of_slot(slot, h, hk, ps)] = scale;
    }
    auto code = [&](float x) {
        const float f = x * inv;
        if (kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD) {
            int qv = static_cast<int>(rintf(f));
            qv = qv > 127 ? 127 : (qv < -128 ? -128 : qv);
            return static_cast<unsigned char>(static_cast<int8_t>(qv));
        }
        if (kv_format == PIE_HIP_KV_FP8_E5M2) return f32_to_e5m2_sat(f);
        const float c = fminf(fmaxf(f, -448.f), 448.f);
        return static_cast<unsigned char>(__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xFF);
    };
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int i = lane + it * kWave;
        if (i < half) {
            const bool adjacent = interleaved == 1;
            dst[adjacent ? 2 * i : i] = code(va[it]);
            dst[adjacent ? 2 * i + 1 : i + half] = code(vb[it]);
        }
    }
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_qkv_rope_kvwrite_quant(int kv_format, const uint16_t* packed_qkv, uint16_t* q_out,
                                              void* k_pages, void* v_pages, float* k_scales,
                                              float* v_scales, const uint16_t* q_norm_weight,
                                              const uint16_t* k_norm_weight, const float* rope_table,
                                              const int64_t* kv_slots, int num_tokens, int num_q_heads,
                                              int num_kv_heads, int head_dim, int page_size,
                                              int interleaved, float eps, void* stream) {
    using namespace pie_hip;
    if (!packed_qkv || !q_out || !k_pages || !v_pages || !rope_table || !kv_slots || num_tokens <= 0 ||
        num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || page_size <= 0)
        return PIE_HIP_ERR_INVALID;
    if (!q_norm_weight != !k_norm_weight) return PIE_HIP_ERR_INVALID;
    const bool scaled = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD || kv_format == PIE_HIP_KV_FP8_PER_TOKEN_HEAD;
    if (kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2 && !scaled) return PIE_HIP_ERR_UNSUPPORTED;
    if (scaled && (!k_scales || !v_scales)) return PIE_HIP_ERR_INVALID;
    if (head_dim % 8 != 0 || head_dim > 256 || num_q_heads + 2 * num_kv_heads > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    const dim3 grid(num_tokens, num_q_heads + 2 * num_kv_heads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned char* kp = static_cast<unsigned char*>(k_pages);
    unsigned char* vp = static_cast<unsigned char*>(v_pages);
    if (head_dim <= 128)
        hipLaunchKernelGGL(qkv_rope_kvwrite_quant_kernel<1>, grid, dim3(64), 0, st, packed_qkv, q_out, kp, vp,
                           k_scales, v_scales, q_norm_weight, k_norm_weight, rope_table, kv_slots,
                           num_q_heads, num_kv_heads, head_dim, page_size, interleaved, eps, kv_format);
    else
        hipLaunchKernelGGL(qkv_rope_kvwrite_quant_kernel<2>, grid, dim3(64), 0, st, packed_qkv, q_out, kp, vp,
                           k_scales, v_scales, q_norm_weight, k_norm_weight, rope_table, kv_slots,
                           num_q_heads, num_kv_heads, head_dim, page_size, interleaved, eps, kv_format);
    return launch_status();
}

extern "C" int pie_hip_kv_write_quant(int kv_format, const uint16_t* k_rows, const uint16_t* v_rows,
                                      const int64_t* kv_slots, void* k_pages, void* v_pages,
                                      float* k_scales, float* v_scales, int num_tokens,
                                      int num_kv_heads, int head_dim, int page_size, void* stream) {
    using namespace pie_hip;
    if (!k_rows || !v_rows || !kv_slots || !k_pages || !v_pages || num_tokens < 0 || num_kv_heads <= 0 ||
        head_dim <= 0 || page_size <= 0)
        return PIE_HIP_ERR_INVALID;
    const bool scaled = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD || kv_format == PIE_HIP_KV_FP8_PER_TOKEN_HEAD ||
                        kv_format == PIE_HIP_KV_FP4_BLOCK;
    if (kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2 && !scaled) return PIE_HIP_ERR_UNSUPPORTED;
    if (scaled && (!k_scales || !v_scales)) return PIE_HIP_ERR_INVALID;
    if (kv_format == PIE_HIP_KV_FP4_BLOCK && head_dim % 16 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    if (num_tokens == 0) return PIE_HIP_OK;
    const int rows = num_tokens * num_kv_heads;
    hipLaunchKernelGGL(kv_write_quant_kernel, dim3((rows + 3) / 4), dim3(256), 0,
                       static_cast<hipStream_t>(stream), k_rows, v_rows, kv_slots,
                       static_cast<unsigned char*>(k_pages), static_cast<unsigned char*>(v_pages), k_scales,
                       v_scales, rows, num_kv_heads, head_dim, page_size, kv_format);
    return launch_status();
}

extern "C" int pie_hip_kv_dequant_pages(int kv_format, const void* k_pages, const void* v_pages,
                                        const float* k_scales, const float* v_scales, uint16_t* k_out,
                                        uint16_t* v_out, const uint32_t* page_ids, int num_pages,
                                        int num_kv_heads, int head_dim, int page_size, void* stream) {
    using namespace pie_hip;
    if (!k_pages || !v_pages || !k_out || !v_out || !page_ids || num_pages < 0 || num_kv_heads <= 0 ||
        head_dim <= 0 || page_size <= 0)
        return PIE_HIP_ERR_INVALID;
    const bool scaled = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD || kv_format == PIE_HIP_KV_FP8_PER_TOKEN_HEAD ||
                        kv_format == PIE_HIP_KV_FP4_BLOCK;
    if (kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2 && !scaled) return PIE_HIP_ERR_UNSUPPORTED;
    if (scaled != (k_scales != nullptr) || scaled != (v_scales != nullptr)) return PIE_HIP_ERR_INVALID;
    if (head_dim % 8 != 0 || (kv_format == PIE_HIP_KV_FP4_BLOCK && head_dim % 16 != 0)) return PIE_HIP_ERR_UNSUPPORTED;
    if (num_pages == 0) return PIE_HIP_OK;
    const size_t total = static_cast<size_t>(num_pages) * page_size * num_kv_heads * (head_dim / 8);
    if ((total + 255) / 256 > 0x7FFFFFFFull) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kv_dequant_pages_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const unsigned char*>(k_pages),
                       static_cast<const unsigned char*>(v_pages), k_scales, v_scales, k_out, v_out, page_ids,
                       total, num_kv_heads, head_dim, page_size, kv_format);
    return launch_status();
}

namespace pie_hip {
namespace {

// One thread per (row, 16-token unit): bit t = key 16*unit + t is visible to the row.
// bounds: per row the cumulative ends of its BRLE runs (run j covers [bounds[j-1], bounds[j])
// and is a visible run when j is odd); a row without runs sees its whole causal window.
__global__ __launch_bounds__(256) void attn_mask_bitmap_kernel(
    const uint32_t* __restrict__ bounds, const int32_t* __restrict__ bounds_indptr,
    const int32_t* __restrict__ row_kv_len, int window, uint16_t* __restrict__ bitmap, int rows,
    int stride) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * stride) return;
    const int r = idx / stride, unit = idx - r * stride;
    const int kv_len = row_kv_len[r];                      // visible keys end at the row's position
    const int lo = window > 0 ? max(0, kv_len - window) : 0;
    const int b0 = bounds_indptr[r], b1 = bounds_indptr[r + 1];
    uint32_t word = 0u;
    for (int t = 0; t < kUnitTokens; ++t) {
        const int j = unit * kUnitTokens + t;
        bool vis = j < kv_len && j >= lo;
        if (vis && b1 > b0) {
            int a = b0, b = b1;   // first run whose end is past j
            while (a < b) {
                const int mid = (a + b) >> 1;
                if (bounds[mid] > static_cast<uint32_t>(j)) b = mid;
                else a = mid + 1;
            }
            vis = a < b1 && ((a - b0) & 1);
        }
        word |= static_cast<uint32_t>(vis) << t;
    }
    bitmap[idx] = static_cast<uint16_t>(word);
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_attn_mask_bitmap(const uint32_t* run_bounds, const int32_t* run_bounds_indptr,
                                        const int32_t* row_kv_len, int window, uint16_t* bitmap,
                                        int num_rows, int stride_units, void* stream) {
    using namespace pie_hip;
    if (!run_bounds_indptr || !row_kv_len || !bitmap || num_rows <= 0 || stride_units <= 0)
        return PIE_HIP_ERR_INVALID;
    const long long n = static_cast<long long>(num_rows) * stride_units;
    if (n > 0x7FFFFFFFll) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(attn_mask_bitmap_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), run_bounds, run_bounds_indptr, row_kv_len,
                       window, bitmap, num_rows, stride_units);
    return launch_status();
}

extern "C" int pie_hip_attn_rows_paged_masked(const uint16_t* q, const uint16_t* k_pages,
                                              const uint16_t* v_pages, uint16_t* o, float* lse,
                                              const uint32_t* kv_page_indices,
                                              const uint32_t* row_page_begin,
                                              const int32_t* row_kv_len, const uint16_t* mask_bitmap,
                                              int mask_stride_units, int num_rows, int num_q_heads,
                                              int num_kv_heads, int head_dim, int page_size,
                                              float sm_scale, int max_kv_len, void* workspace,
                                              size_t workspace_bytes, void* stream) {
    if (!row_page_begin || !row_kv_len || !mask_bitmap) return PIE_HIP_ERR_INVALID;
    return pie_hip::attn_dispatch(q, k_pages, v_pages, o, lse, kv_page_indices, nullptr, nullptr,
                                  row_page_begin, row_kv_len, num_rows, num_q_heads, num_kv_heads,
                                  head_dim, page_size, sm_scale, max_kv_len, workspace,
                                  workspace_bytes, stream, mask_bitmap, mask_stride_units);
}

