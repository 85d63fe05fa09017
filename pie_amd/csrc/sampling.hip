// Sampling on the device for gfx950: everything the forward response needs beyond greedy argmax.
//
//   pie_hip_sample_gather_logits: the sampled rows of the bf16 logits widened to f32, with each
//   request's BRLE logit mask applied (apply_brle_logit_mask, driver/portable/src/sampler.cpp:
//   169-198: runs alternate false/true starting with false, everything past the last run is
//   masked, no runs = no constraint).
//
//   pie_hip_sample: one block per sampling slot, the arithmetic of sample_slot / sample_token
//   (driver/portable/src/sampler.cpp:308-409) and of the special samplers (:224-306):
//     token kinds   T <= 1e-5: first-index argmax.  Otherwise p = softmax(logits / T) with the
//                   normaliser summed in double; Multinomial walks p in index order until the
//                   running sum exceeds u; TopK / TopP / MinP / TopKTopP order the entries with
//                   p > 0 by descending p (equal p: ascending id), keep the first top_k, then
//                   the shortest prefix whose running sum reaches top_p, or the entries with
//                   p >= min_p * p_max, and pick the first kept entry whose running sum exceeds
//                   u * total.  u is the slot's uniform draw, made on the host (PCG32).
//     Distribution  the top_k (0 = all) entries of softmax(logits / T), descending.
//     Logprob(s)    logits[label] - logsumexp(logits), the sum of exp in double.
//     Entropy       -sum p * log p over the same log-softmax, in double.
//   The reference walks its running sums sequentially in float; here each wave scans 64 entries
//   at a time in double and compares the float-rounded value, so a draw within float rounding of
//   a boundary may land on the neighbouring token.
//
//   With at most sixteen slots over a wide vocabulary the row-wide passes (maximum, exponentials
//   and their sum, normalisation and candidate statistics, the candidates' compaction) run first
//   over up to 32 blocks per slot, four short launches; the one block per slot then starts from
//   their results.  Partial results are combined in part order, so a call's output does not
//   depend on how the blocks were scheduled.
//
//   The descending order comes from a block-wide LSD radix sort (8-bit digits, 4 passes over
//   the non-negative float bit patterns): each wave owns a contiguous segment, ranks its 64
//   keys per step by matching digits across the wave (8 ballots), and scatters stably, so
//   equal keys keep ascending ids.
#include <algorithm>
#include <cstdlib>

#include "common.hip.h"

namespace pie_hip {
namespace {

constexpr int kSampBlock = 1024;
constexpr int kSampWaves = kSampBlock / kWave;   // 16
constexpr int kDigits = 256;
// A single block walks a whole vocabulary row: every pass requests kLoads values per thread
// before it uses the first, or it would pay one memory latency per element.
constexpr int kLoads = 32;

struct SampleArgs {
    const float* logits;        // [S, V]
    const int32_t* kind;        // wire sampler kinds
    const float* temperature;
    const uint32_t* top_k;
    const float* top_p;
    const float* min_p;
    const float* uniform;
    const int32_t* out_indptr;  // [S + 1] ranges in values / ids / labels
    const uint32_t* labels;
    uint32_t* tokens;           // [S]
    float* values;
    uint32_t* ids;
    uint32_t* key_a;            // [S, V] each
    uint32_t* key_b;
    uint32_t* id_a;
    uint32_t* id_b;
    int V;
    int parts;                  // > 0: the front-end kernels below have run with this many parts per slot
};

// Candidate thresholds t_j = p_max * 2^(-3j), j = 1..kLevels: how many entries, and how much
// probability mass, lie at or above each (mass in float: a guide for picking a level, not a
// result).
constexpr int kLevels = 8;
constexpr uint32_t kLevelStep = 3u << 23;   // three binades in the float bit pattern

struct BlockShared {
    uint32_t lcnt[kSampWaves][kLevels];
    float lmass[kSampWaves][kLevels];
    uint32_t cnt[kSampWaves][kDigits];
    double f64[kSampWaves];
    float f32[kSampWaves];
    int i32[kSampWaves];
    uint32_t u32[kSampWaves];
};

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Sum over the block in a fixed order (same value in every thread).
__device__ double block_sum_f64(double v, BlockShared& sh, int lane, int wv) {
    v = wave_sum_f64(v);
    if (lane == 0) sh.f64[wv] = v;
    __syncthreads();
    double t = 0.0;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) t += sh.f64[w];
    __syncthreads();
    return t;
}

__device__ int block_sum_i32(int v, BlockShared& sh, int lane, int wv) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    if (lane == 0) sh.i32[wv] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) t += sh.i32[w];
    __syncthreads();
    return t;
}

__device__ uint32_t block_excl_scan_u32(uint32_t v, BlockShared& sh, int lane, int wv) {
    uint32_t incl = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t o = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += o;
    }
    if (lane == kWave - 1) sh.u32[wv] = incl;
    __syncthreads();
    uint32_t base = 0;
    for (int w = 0; w < wv; ++w) base += sh.u32[w];
    __syncthreads();
    return base + incl - v;
}

// (max, first index of the max) of a row; NaNs never win.
__device__ void block_argmax(const float* row, int V, BlockShared& sh, int tid, int lane, int wv,
                             float& mx_out, int& idx_out) {
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int v0 = tid; v0 < V; v0 += kSampBlock * kLoads) {
        float x[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            x[j] = v < V ? row[v] : -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            if (v < V && (x[j] > bv || (bi == 0x7FFFFFFF && x[j] == bv))) {
                bv = x[j];
                bi = v;
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (lane == 0) {
        sh.f32[wv] = bv;
        sh.i32[wv] = bi;
    }
    __syncthreads();
    bv = sh.f32[0];
    bi = sh.i32[0];
#pragma unroll
    for (int w = 1; w < kSampWaves; ++w) {
        const float ov = sh.f32[w];
        const int oi = sh.i32[w];
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    __syncthreads();
    mx_out = bv;
    idx_out = bi == 0x7FFFFFFF ? 0 : bi;
}

// Lanes of the wave holding the same digit as this lane (invalid lanes match nobody).
__device__ __forceinline__ uint64_t match_digit(uint32_t d, bool valid) {
    uint64_t m = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const bool bit = (d >> b) & 1u;
        const uint64_t bal = __ballot(bit);
        m &= bit ? bal : ~bal;
    }
    return m;
}

// One stable LSD pass, descending in the digit.  ids == nullptr: the input ids are 0..n-1.
__device__ void radix_pass(const uint32_t* __restrict__ kin, const uint32_t* __restrict__ iin,
                           uint32_t* __restrict__ kout, uint32_t* __restrict__ iout, int n,
                           int shift, BlockShared& sh, int tid, int lane, int wv) {
    for (int e = tid; e < kSampWaves * kDigits; e += kSampBlock) (&sh.cnt[0][0])[e] = 0;
    __syncthreads();
    const int seg = ((n + kSampBlock - 1) / kSampBlock) * kWave;   // per wave, a multiple of 64
    const int lo = wv * seg, hi = min(n, lo + seg);
    constexpr int kSteps = 16;   // 64-key steps whose loads are requested together
    for (int i0 = lo; i0 < hi; i0 += kWave * kSteps) {
        uint32_t keys[kSteps];
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const int i = i0 + j * kWave + lane;
            keys[j] = i < hi ? kin[i] : 0u;
        }
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const bool valid = i0 + j * kWave + lane < hi;
            const uint32_t d = 255u - ((keys[j] >> shift) & 255u);
            const uint64_t m = match_digit(d, valid);
            if (valid && lane == __ffsll(static_cast<long long>(m)) - 1) sh.cnt[wv][d] += __popcll(m);
        }
    }
    __syncthreads();
    {   // exclusive offsets in (digit, wave) order: thread t owns digit t/4, waves 4*(t%4)..+3
        const int d = tid >> 2, w0 = (tid & 3) * 4;
        const uint32_t c0 = sh.cnt[w0][d], c1 = sh.cnt[w0 + 1][d], c2 = sh.cnt[w0 + 2][d],
                       c3 = sh.cnt[w0 + 3][d];
        const uint32_t ex = block_excl_scan_u32(c0 + c1 + c2 + c3, sh, lane, wv);
        sh.cnt[w0][d] = ex;
        sh.cnt[w0 + 1][d] = ex + c0;
        sh.cnt[w0 + 2][d] = ex + c0 + c1;
        sh.cnt[w0 + 3][d] = ex + c0 + c1 + c2;
    }
    __syncthreads();
    for (int i0 = lo; i0 < hi; i0 += kWave * kSteps) {
        uint32_t keys[kSteps], idv[kSteps];
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const int i = i0 + j * kWave + lane;
            keys[j] = i < hi ? kin[i] : 0u;
            idv[j] = i < hi ? (iin ? iin[i] : static_cast<uint32_t>(i)) : 0u;
        }
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const bool valid = i0 + j * kWave + lane < hi;
            const uint32_t d = 255u - ((keys[j] >> shift) & 255u);
            const uint64_t m = match_digit(d, valid);
            const uint32_t base = valid ? sh.cnt[wv][d] : 0u;
            const uint32_t rank = __popcll(m & ((1ull << lane) - 1ull));
            if (valid) {
                kout[base + rank] = keys[j];
                iout[base + rank] = idv[j];
                if (rank == 0) sh.cnt[wv][d] = base + __popcll(m);   // after every peer read `base`
            }
        }
    }
    __syncthreads();
}

// Sorted (descending key, ascending position) result in (key_a, id_a).  have_ids: id_a holds the
// entries' ids (in ascending order for equal keys to come out by ascending id); else ids 0..n-1.
__device__ void sort_desc(uint32_t* key_a, uint32_t* key_b, uint32_t* id_a, uint32_t* id_b, int n,
                          bool have_ids, BlockShared& sh, int tid, int lane, int wv) {
    radix_pass(key_a, have_ids ? id_a : nullptr, key_b, id_b, n, 0, sh, tid, lane, wv);
    radix_pass(key_b, id_b, key_a, id_a, n, 8, sh, tid, lane, wv);
    radix_pass(key_a, id_a, key_b, id_b, n, 16, sh, tid, lane, wv);
    radix_pass(key_b, id_b, key_a, id_a, n, 24, sh, tid, lane, wv);
}

// First i < limit whose running sum s_i = p_0 + ... + p_i satisfies
//   kReach:   float(s_i) >= thr                 (top-p prefix)
//   kExceed:  thr < float(s_i)                  (multinomial walk)
//   kExceedScaled: thr * float(total) < float(s_i), total = s_{limit-1}   (categorical draw)
// `limit` when there is none.  Block-uniform result.
enum { kReach = 0, kExceed = 1, kExceedScaled = 2 };
// (from_lo, from_hi, from_base): a sub-range already known to hold the answer and the sum of
// everything before it — the walk then starts there instead of at the whole range (kExceed only).
template <int MODE>
__device__ int find_first(const uint32_t* __restrict__ pbits, int limit, float thr, BlockShared& sh,
                          int lane, int wv, double* total_out, int from_lo = -1, int from_hi = 0,
                          double from_base = 0.0) {
    // Narrow the range 16-fold per level: every wave sums one sub-range (coalesced, batched
    // loads), the first sub-range whose end satisfies the rule holds the answer; the last
    // <= 64 entries are scanned by lane.  Sums are double; only the compared value is rounded.
    int lo = 0, hi = limit;
    double base = 0.0;
    float x = thr;
    bool top = true;
    if (from_lo >= 0) {
        lo = from_lo;
        hi = from_hi;
        base = from_base;
        top = false;
    }
    while (top || hi - lo > kWave) {
        const int span = hi - lo;
        const int sub = ((span + kSampWaves * kWave - 1) / (kSampWaves * kWave)) * kWave;
        const int wlo = min(hi, lo + wv * sub), whi = min(hi, wlo + sub);
        double s = 0.0;
        for (int i0 = wlo + lane; i0 < whi; i0 += kWave * kLoads) {
            uint32_t b[kLoads];
#pragma unroll
            for (int j = 0; j < kLoads; ++j) b[j] = i0 + j * kWave < whi ? pbits[i0 + j * kWave] : 0u;
#pragma unroll
            for (int j = 0; j < kLoads; ++j) s += static_cast<double>(__uint_as_float(b[j]));
        }
        s = wave_sum_f64(s);
        if (lane == 0) sh.f64[wv] = s;
        __syncthreads();
        if (top) {
            double total = 0.0;
#pragma unroll
            for (int w = 0; w < kSampWaves; ++w) total += sh.f64[w];
            *total_out = total;
            if (MODE == kExceedScaled) x = thr * static_cast<float>(total);
        }
        int pick = -1, last_mass = -1;
        double before = base, run = base, before_last = base;
#pragma unroll
        for (int w = 0; w < kSampWaves; ++w) {
            if (sh.f64[w] > 0.0) {
                last_mass = w;
                before_last = run;
            }
            run += sh.f64[w];
            const float cum = static_cast<float>(run);
            const bool hit = MODE == kReach ? cum >= x : x < cum;
            if (hit && pick < 0) pick = w;
            if (pick < 0) before = run;
        }
        __syncthreads();
        if (pick < 0) {
            if (top) return limit;      // the rule is never met
            // The level above found the crossing inside this range and this level's
            // re-associated sums disagree in the last bit: the answer is the range's last entry
            // with a positive probability (never an entry the softmax or a logit mask zeroed),
            // so carry on inside the last sub-range that holds any mass.
            pick = last_mass;
            before = before_last;
            if (pick < 0) return hi - 1;   // (a range without mass is never chosen by the level above)
        }
        base = before;
        lo = min(hi, lo + pick * sub);
        hi = min(hi, lo + sub);
        top = false;
    }
    const int i = lo + lane;
    double incl = i < hi ? static_cast<double>(__uint_as_float(pbits[i])) : 0.0;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const double o = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += o;
    }
    const float cum = static_cast<float>(base + incl);
    const uint64_t b = __ballot(i < hi && (MODE == kReach ? cum >= x : x < cum));
    if (b) return lo + __ffsll(static_cast<long long>(b)) - 1;
    // same disagreement in the last 64 entries: the last one with a positive probability
    const uint64_t pos = __ballot(i < hi && __uint_as_float(pbits[min(i, hi - 1)]) > 0.0f);
    return pos ? lo + 63 - __clzll(static_cast<long long>(pos)) : hi - 1;
}

// p = softmax(row / T) as float bit patterns in `out`.  Also: the number of entries with p > 0,
// their sum, the largest p, and (HIST) a histogram of count and mass over the buckets.
struct SoftmaxStats {
    int n_pos;
    double total;
    uint32_t max_bits;
};
template <bool HIST>
__device__ SoftmaxStats softmax_to_bits(const float* row, int V, float mx, float temperature,
                                        uint32_t* out, BlockShared& sh, int tid, int lane, int wv) {
    const float inv_t = 1.0f / fmaxf(temperature, 1e-5f);
    double s = 0.0;
    for (int v0 = tid; v0 < V; v0 += kSampBlock * kLoads) {
        float x[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            x[j] = v < V ? row[v] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            if (v < V) {
                const float e = expf((x[j] - mx) * inv_t);
                out[v] = __float_as_uint(e);
                s += static_cast<double>(e);
            }
        }
    }
    const double sum = block_sum_f64(s, sh, lane, wv);
    const float inv_sum = static_cast<float>(1.0 / fmax(1e-30, sum));
    int pos = 0;
    double ps = 0.0;
    uint32_t mb = 0u;
    // p_max = e_max * inv_sum with e_max = expf(0) = 1 (the row maximum), known before the pass
    const uint32_t top_bits = __float_as_uint(inv_sum);
    uint32_t lc[kLevels];
    float lm[kLevels];
#pragma unroll
    for (int j = 0; j < kLevels; ++j) {
        lc[j] = 0u;
        lm[j] = 0.f;
    }
    for (int v0 = tid; v0 < V; v0 += kSampBlock * kLoads) {
        uint32_t eb[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            eb[j] = v < V ? out[v] : 0u;
        }
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            if (v >= V) continue;
            const float p = __uint_as_float(eb[j]) * inv_sum;
            const uint32_t bits = __float_as_uint(p);
            out[v] = bits;
            if (p > 0.0f) {
                ++pos;
                ps += static_cast<double>(p);
                mb = max(mb, bits);
                if (HIST) {
#pragma unroll
                    for (int j = 0; j < kLevels; ++j) {
                        const bool in = bits + (j + 1) * kLevelStep >= top_bits;
                        lc[j] += in;
                        lm[j] += in ? p : 0.f;
                    }
                }
            }
        }
    }
    SoftmaxStats st;
    st.n_pos = block_sum_i32(pos, sh, lane, wv);
    st.total = block_sum_f64(ps, sh, lane, wv);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mb = max(mb, static_cast<uint32_t>(__shfl_xor(mb, off, kWave)));
    if (lane == 0) sh.u32[wv] = mb;
    __syncthreads();
    mb = 0u;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) mb = max(mb, sh.u32[w]);
    __syncthreads();
    st.max_bits = mb;
    if (HIST) {
#pragma unroll
        for (int j = 0; j < kLevels; ++j) {
            uint32_t c = lc[j];
            float m = lm[j];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                c += __shfl_xor(c, off, kWave);
                m += __shfl_xor(m, off, kWave);
            }
            if (lane == 0) {
                sh.lcnt[wv][j] = c;
                sh.lmass[wv][j] = m;
            }
        }
        __syncthreads();
    }
    return st;
}

// Entries with bits >= floor_bits, in index order, into (kout, iout); returns how many.
__device__ int compact_ge(const uint32_t* __restrict__ kin, uint32_t floor_bits,
                          uint32_t* __restrict__ kout, uint32_t* __restrict__ iout, int n,
                          BlockShared& sh, int lane, int wv) {
    const int seg = ((n + kSampBlock - 1) / kSampBlock) * kWave;
    const int lo = min(n, wv * seg), hi = min(n, lo + seg);
    constexpr int kSteps = 16;
    int c = 0;
    for (int i0 = lo; i0 < hi; i0 += kWave * kSteps) {
        uint32_t keys[kSteps];
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const int i = i0 + j * kWave + lane;
            keys[j] = i < hi ? kin[i] : 0u;
        }
#pragma unroll
        for (int j = 0; j < kSteps; ++j)
            c += __popcll(__ballot(i0 + j * kWave + lane < hi && keys[j] >= floor_bits));
    }
    if (lane == 0) sh.i32[wv] = c;
    __syncthreads();
    int base = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) {
        if (w < wv) base += sh.i32[w];
        total += sh.i32[w];
    }
    __syncthreads();
    for (int i0 = lo; i0 < hi; i0 += kWave * kSteps) {
        uint32_t keys[kSteps];
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const int i = i0 + j * kWave + lane;
            keys[j] = i < hi ? kin[i] : 0u;
        }
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const int i = i0 + j * kWave + lane;
            const bool take = i < hi && keys[j] >= floor_bits;
            const uint64_t b = __ballot(take);
            if (take) {
                const int at = base + __popcll(b & ((1ull << lane) - 1ull));
                kout[at] = keys[j];
                iout[at] = static_cast<uint32_t>(i);
            }
            base += __popcll(b);
        }
    }
    __syncthreads();
    return total;
}

__device__ float log_sum_exp(const float* row, int V, float mx, BlockShared& sh, int tid, int lane,
                             int wv) {
    double s = 0.0;
    for (int v0 = tid; v0 < V; v0 += kSampBlock * kLoads) {
        float x[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int v = v0 + j * kSampBlock;
            x[j] = v < V ? row[v] : -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < kLoads; ++j)
            if (v0 + j * kSampBlock < V) s += exp(static_cast<double>(x[j] - mx));
    }
    const double sum = block_sum_f64(s, sh, lane, wv);
    return mx + static_cast<float>(log(fmax(1e-30, sum)));
}

// What the draw can touch is a head of the descending order: the first top_k entries, the
// prefix reaching top_p, the entries above the min-p threshold, or (nothing restricting)
// the prefix whose mass exceeds u * total.  Any set {p >= t} containing that head gives
// the same result as the whole vocabulary, so only such a set is compacted and sorted;
// t is the first of the levels p_max * 2^(-3j) that covers the need (exact for min-p).
struct DrawNeed {
    int need_count;
    float need_mass;
    uint32_t floor_bits;   // nonzero: the exact lower bound of the kept entries (min-p)
    bool keep_all, wants_k, wants_p;
    float thr_p;
};
__device__ __forceinline__ DrawNeed draw_need(const SampleArgs& a, int s, int kind, const SoftmaxStats& st, float u) {
    DrawNeed d;
    d.wants_k = kind == PIE_HIP_SAMPLER_TOP_K || kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
    d.wants_p = kind == PIE_HIP_SAMPLER_TOP_P || kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
    const uint32_t top_k = a.top_k[s];
    d.thr_p = fminf(fmaxf(a.top_p[s], 0.0f), 1.0f);
    const float thr_m = a.min_p[s] * __uint_as_float(st.max_bits);
    d.need_count = 0;
    d.need_mass = 0.f;
    d.floor_bits = 0u;
    d.keep_all = false;
    if (d.wants_k && top_k != 0u) d.need_count = static_cast<int>(min(top_k, static_cast<uint32_t>(st.n_pos)));
    else if (d.wants_p && d.thr_p < 1.0f) d.need_mass = d.thr_p;
    else if (kind == PIE_HIP_SAMPLER_MIN_P && thr_m > 0.0f && thr_m <= __uint_as_float(st.max_bits))
        d.floor_bits = __float_as_uint(thr_m);
    else {
        d.keep_all = true;
        d.need_mass = u * static_cast<float>(st.total);
    }
    return d;
}
// the first level whose candidates cover the need; 1 (every positive entry) when none does
__device__ __forceinline__ uint32_t level_floor(const DrawNeed& d, uint32_t top_bits, const uint32_t* cc, const float* cm) {
    if (d.floor_bits) return d.floor_bits;
    for (int j = 0; j < kLevels; ++j) {
        const bool enough = d.need_count > 0 ? cc[j] >= static_cast<uint32_t>(d.need_count)
                                             : cm[j] >= d.need_mass + 1e-4f;
        if (enough && top_bits > (j + 1) * kLevelStep) return top_bits - (j + 1) * kLevelStep;
    }
    return 1u;
}
__device__ __forceinline__ bool sorts_candidates(int kind) {
    return kind == PIE_HIP_SAMPLER_TOP_K || kind == PIE_HIP_SAMPLER_TOP_P || kind == PIE_HIP_SAMPLER_MIN_P ||
           kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
}

// ---- front end over many blocks ----------------------------------------------------------------
// One block per slot walks a 128 k row four times from a single CU (80-145 us).  With few slots the
// row-wide passes — maximum, exponentials and their sum, normalisation with the candidate
// statistics — are cut into `parts` contiguous segments, one block each, in three launches; the
// per-part results are combined in part order (a fixed order: the same inputs give the same bits
// every time), and sample_kernel starts from the normalised probabilities — for the kinds that
// sort a candidate set, from the candidates too: each part compacts its own, in index order, to the
// head of its segment of (key_b, id_b).  A slot's part records sit at the head of its id_a region,
// which nothing else uses before sample_kernel has read them.
constexpr int kFrontBlock = 256;
constexpr int kFrontWaves = kFrontBlock / kWave;
constexpr int kFrontLoads = 8;
constexpr int kMaxParts = 32;
struct FrontPart {
    float mx;
    int amax;
    int n_pos;
    uint32_t max_bits;
    double sum;       // of the part's exponentials
    double ps;        // of its normalised probabilities
    uint32_t lc[kLevels];
    float lm[kLevels];
    int cnt;          // candidates this part put at the head of its segment of (key_b, id_b); -1: none made
    uint32_t t_bits;  // the threshold they were taken at
    uint32_t pad[2];
};
static_assert(sizeof(FrontPart) == 112, "part record layout");

__device__ __forceinline__ FrontPart* front_parts(const SampleArgs& a, int s) {
    return reinterpret_cast<FrontPart*>(a.id_a + static_cast<size_t>(s) * a.V);
}
__device__ __forceinline__ void front_segment(int V, int parts, int part, int& lo, int& hi) {
    const int seg = ((V + parts - 1) / parts + kFrontBlock - 1) / kFrontBlock * kFrontBlock;
    lo = min(V, part * seg);
    hi = min(V, lo + seg);
}
// (max, first index) over all parts of a slot, as block_argmax orders them
__device__ __forceinline__ void front_max(const FrontPart* fp, int parts, float& mx, int& amax) {
    mx = fp[0].mx;
    amax = fp[0].amax;
    for (int b = 1; b < parts; ++b) {
        const float ov = fp[b].mx;
        const int oi = fp[b].amax;
        if (ov > mx || (ov == mx && oi < amax)) {
            mx = ov;
            amax = oi;
        }
    }
}

__global__ __launch_bounds__(kFrontBlock) void sample_front_max_kernel(SampleArgs a) {
    __shared__ float s_v[kFrontWaves];
    __shared__ int s_i[kFrontWaves];
    const int part = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const float* row = a.logits + static_cast<size_t>(s) * a.V;
    int lo, hi;
    front_segment(a.V, a.parts, part, lo, hi);
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int v0 = lo + tid; v0 < hi; v0 += kFrontBlock * kFrontLoads) {
        float x[kFrontLoads];
#pragma unroll
        for (int j = 0; j < kFrontLoads; ++j) {
            const int v = v0 + j * kFrontBlock;
            x[j] = v < hi ? row[v] : -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < kFrontLoads; ++j) {
            const int v = v0 + j * kFrontBlock;
            if (v < hi && (x[j] > bv || (bi == 0x7FFFFFFF && x[j] == bv))) {
                bv = x[j];
                bi = v;
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (lane == 0) {
        s_v[wv] = bv;
        s_i[wv] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kFrontWaves; ++w)
            if (s_v[w] > bv || (s_v[w] == bv && s_i[w] < bi)) {
                bv = s_v[w];
                bi = s_i[w];
            }
        FrontPart* fp = front_parts(a, s) + part;
        fp->mx = bv;
        fp->amax = bi;
    }
}

__device__ __forceinline__ double front_block_sum_f64(double v, double* sh, int lane, int wv) {
    v = wave_sum_f64(v);
    if (lane == 0) sh[wv] = v;
    __syncthreads();
    double t = 0.0;
#pragma unroll
    for (int w = 0; w < kFrontWaves; ++w) t += sh[w];
    __syncthreads();
    return t;
}

// e = expf((x - max) / T) into key_a, the part's sum of e in double
__global__ __launch_bounds__(kFrontBlock) void sample_front_exp_kernel(SampleArgs a) {
    __shared__ double s_d[kFrontWaves];
    const int part = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const float* row = a.logits + static_cast<size_t>(s) * a.V;
    uint32_t* out = a.key_a + static_cast<size_t>(s) * a.V;
    FrontPart* fp = front_parts(a, s);
    float mx;
    int amax;
    front_max(fp, a.parts, mx, amax);
    const float inv_t = 1.0f / fmaxf(a.temperature[s], 1e-5f);
    int lo, hi;
    front_segment(a.V, a.parts, part, lo, hi);
    double acc = 0.0;
    for (int v0 = lo + tid; v0 < hi; v0 += kFrontBlock * kFrontLoads) {
        float x[kFrontLoads];
#pragma unroll
        for (int j = 0; j < kFrontLoads; ++j) {
            const int v = v0 + j * kFrontBlock;
            x[j] = v < hi ? row[v] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < kFrontLoads; ++j) {
            const int v = v0 + j * kFrontBlock;
            if (v < hi) {
                const float e = expf((x[j] - mx) * inv_t);
                out[v] = __float_as_uint(e);
                acc += static_cast<double>(e);
            }
        }
    }
    const double sum = front_block_sum_f64(acc, s_d, lane, wv);
    if (tid == 0) fp[part].sum = sum;
}

// p = e / sum in place, and the part's share of softmax_to_bits' statistics
__global__ __launch_bounds__(kFrontBlock) void sample_front_norm_kernel(SampleArgs a) {
    __shared__ double s_d[kFrontWaves];
    __shared__ uint32_t s_u[kFrontWaves][2 + kLevels];
    __shared__ float s_f[kFrontWaves][kLevels];
    const int part = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    uint32_t* out = a.key_a + static_cast<size_t>(s) * a.V;
    FrontPart* fp = front_parts(a, s);
    double sum = 0.0;
    for (int b = 0; b < a.parts; ++b) sum += fp[b].sum;
    const float inv_sum = static_cast<float>(1.0 / fmax(1e-30, sum));
    const uint32_t top_bits = __float_as_uint(inv_sum);   // p_max = expf(0) * inv_sum
    int lo, hi;
    front_segment(a.V, a.parts, part, lo, hi);
    int pos = 0;
    double ps = 0.0;
    uint32_t mb = 0u;
    uint32_t lc[kLevels];
    float lm[kLevels];
#pragma unroll
    for (int j = 0; j < kLevels; ++j) {
        lc[j] = 0u;
        lm[j] = 0.f;
    }
    for (int v0 = lo + tid; v0 < hi; v0 += kFrontBlock * kFrontLoads) {
        uint32_t eb[kFrontLoads];
#pragma unroll
        for (int j = 0; j < kFrontLoads; ++j) {
            const int v = v0 + j * kFrontBlock;
            eb[j] = v < hi ? out[v] : 0u;
        }
#pragma unroll
        for (int j = 0; j < kFrontLoads; ++j) {
            const int v = v0 + j * kFrontBlock;
            if (v >= hi) continue;
            const float p = __uint_as_float(eb[j]) * inv_sum;
            const uint32_t bits = __float_as_uint(p);
            out[v] = bits;
            if (p > 0.0f) {
                ++pos;
                ps += static_cast<double>(p);
                mb = max(mb, bits);
#pragma unroll
                for (int l = 0; l < kLevels; ++l) {
                    const bool in = bits + (l + 1) * kLevelStep >= top_bits;
                    lc[l] += in;
                    lm[l] += in ? p : 0.f;
                }
            }
        }
    }
    const double ps_all = front_block_sum_f64(ps, s_d, lane, wv);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        pos += __shfl_xor(pos, off, kWave);
        mb = max(mb, static_cast<uint32_t>(__shfl_xor(mb, off, kWave)));
#pragma unroll
        for (int l = 0; l < kLevels; ++l) {
            lc[l] += __shfl_xor(lc[l], off, kWave);
            lm[l] += __shfl_xor(lm[l], off, kWave);
        }
    }
    if (lane == 0) {
        s_u[wv][0] = static_cast<uint32_t>(pos);
        s_u[wv][1] = mb;
#pragma unroll
        for (int l = 0; l < kLevels; ++l) {
            s_u[wv][2 + l] = lc[l];
            s_f[wv][l] = lm[l];
        }
    }
    __syncthreads();
    if (tid == 0) {
        FrontPart& o = fp[part];
        int n = 0;
        uint32_t m = 0u;
        for (int w = 0; w < kFrontWaves; ++w) {
            n += static_cast<int>(s_u[w][0]);
            m = max(m, s_u[w][1]);
        }
        o.n_pos = n;
        o.max_bits = m;
        o.ps = ps_all;
        o.cnt = -1;
        for (int l = 0; l < kLevels; ++l) {
            uint32_t c = 0u;
            float f = 0.f;
            for (int w = 0; w < kFrontWaves; ++w) {
                c += s_u[w][2 + l];
                f += s_f[w][l];
            }
            o.lc[l] = c;
            o.lm[l] = f;
        }
    }
}

// The part's entries with p >= t, in index order, to (key_b, id_b)[lo ..): t is the level every
// block of the slot derives from the combined statistics, exactly as sample_kernel would.
__global__ __launch_bounds__(kFrontBlock) void sample_front_compact_kernel(SampleArgs a) {
    __shared__ FrontPart s_parts[kMaxParts];
    __shared__ int s_cnt[kFrontWaves];
    const int part = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int kind = a.kind[s];
    if (!sorts_candidates(kind) || a.temperature[s] <= 1e-5f) return;
    const int V = a.V;
    FrontPart* gp = front_parts(a, s);
    {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(gp);
        uint32_t* dst = reinterpret_cast<uint32_t*>(s_parts);
        const int words = a.parts * static_cast<int>(sizeof(FrontPart) / 4);
        for (int i = tid; i < words; i += kFrontBlock) dst[i] = src[i];
    }
    __syncthreads();
    SoftmaxStats st{0, 0.0, 0u};
    uint32_t cc[kLevels];
    float cm[kLevels];
#pragma unroll
    for (int l = 0; l < kLevels; ++l) {
        cc[l] = 0u;
        cm[l] = 0.f;
    }
    for (int b = 0; b < a.parts; ++b) {
        st.n_pos += s_parts[b].n_pos;
        st.total += s_parts[b].ps;
        st.max_bits = max(st.max_bits, s_parts[b].max_bits);
#pragma unroll
        for (int l = 0; l < kLevels; ++l) {
            cc[l] += s_parts[b].lc[l];
            cm[l] += s_parts[b].lm[l];
        }
    }
    if (st.n_pos == 0) return;
    const DrawNeed need = draw_need(a, s, kind, st, a.uniform[s]);
    const uint32_t t_bits = level_floor(need, st.max_bits, cc, cm);
    const uint32_t* kin = a.key_a + static_cast<size_t>(s) * V;
    uint32_t* kout = a.key_b + static_cast<size_t>(s) * V;
    uint32_t* iout = a.id_b + static_cast<size_t>(s) * V;
    int lo, hi;
    front_segment(V, a.parts, part, lo, hi);
    // each wave a contiguous quarter of the segment, so that the order is the index order
    const int sub = ((hi - lo + kFrontBlock - 1) / kFrontBlock) * kWave;
    const int wlo = min(hi, lo + wv * sub), whi = min(hi, wlo + sub);
    int c = 0;
    for (int i0 = wlo; i0 < whi; i0 += kWave) {
        const int i = i0 + lane;
        c += __popcll(__ballot(i < whi && kin[i] >= t_bits));
    }
    if (lane == 0) s_cnt[wv] = c;
    __syncthreads();
    int base = lo, total = 0;
#pragma unroll
    for (int w = 0; w < kFrontWaves; ++w) {
        if (w < wv) base += s_cnt[w];
        total += s_cnt[w];
    }
    for (int i0 = wlo; i0 < whi; i0 += kWave) {
        const int i = i0 + lane;
        const uint32_t key = i < whi ? kin[i] : 0u;
        const bool take = i < whi && key >= t_bits;
        const uint64_t bm = __ballot(take);
        if (take) {
            const int at = base + __popcll(bm & ((1ull << lane) - 1ull));
            kout[at] = key;
            iout[at] = static_cast<uint32_t>(i);
        }
        base += __popcll(bm);
    }
    if (tid == 0) {
        gp[part].cnt = total;
        gp[part].t_bits = t_bits;
    }
}

__global__ __launch_bounds__(kSampBlock) void sample_kernel(SampleArgs a) {
    __shared__ BlockShared sh;
    const int s = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int V = a.V;
    const float* row = a.logits + static_cast<size_t>(s) * V;
    const int kind = a.kind[s];
    if (kind == PIE_HIP_SAMPLER_RAW_LOGITS) return;   // the caller reads the f32 row itself
    if (kind == PIE_HIP_SAMPLER_EMBEDDING) return;    // no output for this slot
    float mx;
    int amax;
    const bool front = a.parts > 0;
    SoftmaxStats fst{0, 0.0, 0u};
    __shared__ FrontPart s_parts[kMaxParts];
    if (front) {
        // the part records through LDS: every thread then combines the same values in the same order
        {
            const uint32_t* src = reinterpret_cast<const uint32_t*>(front_parts(a, s));
            uint32_t* dst = reinterpret_cast<uint32_t*>(s_parts);
            const int words = a.parts * static_cast<int>(sizeof(FrontPart) / 4);
            for (int i = tid; i < words; i += kSampBlock) dst[i] = src[i];
        }
        __syncthreads();
        const FrontPart* fp = s_parts;
        front_max(fp, a.parts, mx, amax);
        for (int b = 0; b < a.parts; ++b) {
            fst.n_pos += fp[b].n_pos;
            fst.total += fp[b].ps;
            fst.max_bits = max(fst.max_bits, fp[b].max_bits);
        }
        if (tid < kSampWaves * kLevels) {
            const int w = tid / kLevels, l = tid % kLevels;
            uint32_t c = 0u;
            float f = 0.f;
            if (w == 0)
                for (int b = 0; b < a.parts; ++b) {
                    c += fp[b].lc[l];
                    f += fp[b].lm[l];
                }
            sh.lcnt[w][l] = c;
            sh.lmass[w][l] = f;
        }
        __syncthreads();
    } else {
        block_argmax(row, V, sh, tid, lane, wv, mx, amax);
    }
    const int o0 = a.out_indptr[s], o1 = a.out_indptr[s + 1];

    if (kind == PIE_HIP_SAMPLER_LOGPROB || kind == PIE_HIP_SAMPLER_LOGPROBS) {
        const float lse = log_sum_exp(row, V, mx, sh, tid, lane, wv);
        for (int i = o0 + tid; i < o1; i += kSampBlock) a.values[i] = row[a.labels[i]] - lse;
        return;
    }
    if (kind == PIE_HIP_SAMPLER_ENTROPY) {
        const float lse = log_sum_exp(row, V, mx, sh, tid, lane, wv);
        double h = 0.0;
        for (int v0 = tid; v0 < V; v0 += kSampBlock * kLoads) {
            float x[kLoads];
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                const int v = v0 + j * kSampBlock;
                x[j] = v < V ? row[v] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < kLoads; ++j)
                if (v0 + j * kSampBlock < V) {
                    const float lp = x[j] - lse;
                    h -= exp(static_cast<double>(lp)) * static_cast<double>(lp);
                }
        }
        const double H = block_sum_f64(h, sh, lane, wv);
        if (tid == 0 && o1 > o0) a.values[o0] = static_cast<float>(H);
        return;
    }

    uint32_t* ka = a.key_a + static_cast<size_t>(s) * V;
    uint32_t* kb = a.key_b + static_cast<size_t>(s) * V;
    uint32_t* ia = a.id_a + static_cast<size_t>(s) * V;
    uint32_t* ib = a.id_b + static_cast<size_t>(s) * V;
    const float temperature = a.temperature[s];

    if (kind == PIE_HIP_SAMPLER_DIST) {
        if (!front) softmax_to_bits<false>(row, V, mx, temperature, ka, sh, tid, lane, wv);
        sort_desc(ka, kb, ia, ib, V, false, sh, tid, lane, wv);
        const int k = min(o1 - o0, V);
        for (int i = tid; i < k; i += kSampBlock) {
            a.values[o0 + i] = __uint_as_float(ka[i]);
            a.ids[o0 + i] = ia[i];
        }
        return;
    }

    // token-producing kinds
    if (temperature <= 1e-5f) {
        if (tid == 0) a.tokens[s] = static_cast<uint32_t>(amax);
        return;
    }
    const float u = a.uniform[s];
    double total;
    if (kind == PIE_HIP_SAMPLER_MULTINOMIAL) {
        if (!front) softmax_to_bits<false>(row, V, mx, temperature, ka, sh, tid, lane, wv);
        int tok = V;
        if (front) {
            // the walk's own rule applied to the parts' sums — the first part whose end exceeds u
            // holds the token — then the walk inside that part only
            const FrontPart* fp = s_parts;
            double run = 0.0, before = 0.0;
            int pick = -1;
            for (int b = 0; b < a.parts; ++b) {
                run += fp[b].ps;
                if (pick < 0) {
                    if (u < static_cast<float>(run)) pick = b;
                    else before = run;
                }
            }
            if (pick >= 0) {
                int plo, phi;
                front_segment(V, a.parts, pick, plo, phi);
                tok = find_first<kExceed>(ka, V, u, sh, lane, wv, &total, plo, phi, before);
            }
        } else {
            tok = find_first<kExceed>(ka, V, u, sh, lane, wv, &total);
        }
        if (tid == 0) a.tokens[s] = static_cast<uint32_t>(tok < V ? tok : amax);
        return;
    }
    const SoftmaxStats st = front ? fst : softmax_to_bits<true>(row, V, mx, temperature, ka, sh, tid, lane, wv);
    const int n_pos = st.n_pos;
    if (n_pos == 0) {
        if (tid == 0) a.tokens[s] = 0u;
        return;
    }
    const DrawNeed need = draw_need(a, s, kind, st, u);
    const int need_count = need.need_count;
    const float need_mass = need.need_mass, thr_p = need.thr_p;
    const bool keep_all = need.keep_all, wants_p = need.wants_p;
    for (int attempt = 0; attempt < 2; ++attempt) {
        uint32_t *ck = kb, *ci = ib;   // where the sorted candidates end up
        int m;
        if (attempt == 0 && front && s_parts[0].cnt >= 0) {
            // the parts' candidate lists (each at the head of its segment of (key_b, id_b)) end to
            // end into (key_a, id_a): the order compact_ge gives
            m = 0;
            for (int b = 0; b < a.parts; ++b) {
                int plo, phi;
                front_segment(V, a.parts, b, plo, phi);
                const int cb = s_parts[b].cnt;
                for (int i = tid; i < cb; i += kSampBlock) {
                    ka[m + i] = kb[plo + i];
                    ia[m + i] = ib[plo + i];
                }
                m += cb;
            }
            __syncthreads();
            sort_desc(ka, kb, ia, ib, m, true, sh, tid, lane, wv);
            ck = ka;
            ci = ia;
        } else {
            uint32_t t_bits = 1u;     // every positive entry
            if (attempt == 0) {
                // the first level whose candidates cover the need (every thread computes the same)
                uint32_t cc[kLevels];
                float cm[kLevels];
#pragma unroll
                for (int j = 0; j < kLevels; ++j) {
                    cc[j] = 0u;
                    cm[j] = 0.f;
#pragma unroll
                    for (int w = 0; w < kSampWaves; ++w) {
                        cc[j] += sh.lcnt[w][j];
                        cm[j] += sh.lmass[w][j];
                    }
                }
                t_bits = level_floor(need, st.max_bits, cc, cm);
            } else if (need.floor_bits) {
                t_bits = need.floor_bits;
            }
            m = compact_ge(ka, t_bits, kb, ib, V, sh, lane, wv);
            sort_desc(kb, ka, ib, ia, m, true, sh, tid, lane, wv);   // note: overwrites ka
        }
        const bool whole = m == n_pos;
        bool ok = true;
        uint32_t tok = 0u;
        if (keep_all) {
            const int i = find_first<kExceed>(ck, m, need_mass, sh, lane, wv, &total);
            ok = i < m || whole;
            tok = ci[i < m ? i : m - 1];
        } else {
            int keep = m;
            if (need_count > 0) keep = min(need_count, m);
            if (wants_p && thr_p < 1.0f) {
                const int i = find_first<kReach>(ck, keep, thr_p, sh, lane, wv, &total);
                if (i < keep) keep = i + 1;
                else ok = whole || need_count > 0;   // the prefix must end inside the candidates
            }
            const int i = find_first<kExceedScaled>(ck, keep, u, sh, lane, wv, &total);
            tok = total <= 0.0 ? ci[0] : ci[i < keep ? i : keep - 1];
        }
        if (ok || attempt == 1) {
            if (tid == 0) a.tokens[s] = tok;
            return;
        }
        // the histogram's float masses misjudged the head: rebuild p (the sort used its buffer)
        // and take every positive entry
        softmax_to_bits<false>(row, V, mx, temperature, ka, sh, tid, lane, wv);
    }
}

// Sampled rows of the bf16 logits -> f32, BRLE logit mask applied.  bounds: per slot, the
// cumulative ends of its runs (run j covers [bounds[j-1], bounds[j]) and allows its tokens
// when j is odd); a slot without runs is unconstrained.
__global__ __launch_bounds__(256) void sample_gather_kernel(
    const uint16_t* __restrict__ logits, const int32_t* __restrict__ rows, float* __restrict__ out,
    const uint32_t* __restrict__ bounds, const int32_t* __restrict__ bounds_indptr, int V) {
    const int s = blockIdx.y;
    const int v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= V) return;
    const size_t src_row = rows ? static_cast<size_t>(rows[s]) : static_cast<size_t>(s);
    float x = bf16_bits_to_f32(logits[src_row * V + v]);
    if (bounds_indptr) {
        const int b0 = bounds_indptr[s], b1 = bounds_indptr[s + 1];
        if (b1 > b0) {
            int lo = b0, hi = b1;   // first run index whose end is past v
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (bounds[mid] > static_cast<uint32_t>(v)) hi = mid;
                else lo = mid + 1;
            }
            const int run = lo - b0;
            if (lo == b1 || (run & 1) == 0) x = -INFINITY;
        }
    }
    out[static_cast<size_t>(s) * V + v] = x;
}

}  // namespace
}  // namespace pie_hip

extern "C" size_t pie_hip_sample_workspace_bytes(int num_slots, int vocab) {
    if (num_slots <= 0 || vocab <= 0) return 0;
    return static_cast<size_t>(num_slots) * vocab * 4 * sizeof(uint32_t);
}

extern "C" int pie_hip_sample_gather_logits(const uint16_t* logits_bf16, const int32_t* rows,
                                            float* out_f32, const uint32_t* mask_bounds,
                                            const int32_t* mask_bounds_indptr, int num_slots,
                                            int vocab, void* stream) {
    using namespace pie_hip;
    if (!logits_bf16 || !out_f32 || num_slots <= 0 || vocab <= 0) return PIE_HIP_ERR_INVALID;
    if (num_slots > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    if (mask_bounds_indptr && !mask_bounds) mask_bounds_indptr = nullptr;
    hipLaunchKernelGGL(sample_gather_kernel, dim3((vocab + 255) / 256, num_slots), dim3(256), 0,
                       static_cast<hipStream_t>(stream), logits_bf16, rows, out_f32, mask_bounds,
                       mask_bounds_indptr, vocab);
    return launch_status();
}

extern "C" int pie_hip_sample(const float* logits_f32, const int32_t* kind, const float* temperature,
                              const uint32_t* top_k, const float* top_p, const float* min_p,
                              const float* uniform, const int32_t* out_indptr,
                              const uint32_t* labels, uint32_t* tokens, float* values,
                              uint32_t* ids, void* workspace, size_t workspace_bytes,
                              int num_slots, int vocab, void* stream) {
    using namespace pie_hip;
    if (!logits_f32 || !kind || !temperature || !top_k || !top_p || !min_p || !uniform ||
        !out_indptr || !tokens || num_slots <= 0 || vocab <= 0)
        return PIE_HIP_ERR_INVALID;
    if (vocab > (1 << 24)) return PIE_HIP_ERR_UNSUPPORTED;
    const size_t need = pie_hip_sample_workspace_bytes(num_slots, vocab);
    if (!workspace || workspace_bytes < need) return PIE_HIP_ERR_INVALID;
    SampleArgs a;
    a.logits = logits_f32;
    a.kind = kind;
    a.temperature = temperature;
    a.top_k = top_k;
    a.top_p = top_p;
    a.min_p = min_p;
    a.uniform = uniform;
    a.out_indptr = out_indptr;
    a.labels = labels;
    a.tokens = tokens;
    a.values = values;
    a.ids = ids;
    const size_t n = static_cast<size_t>(num_slots) * vocab;
    a.key_a = static_cast<uint32_t*>(workspace);
    a.key_b = a.key_a + n;
    a.id_a = a.key_b + n;
    a.id_b = a.id_a + n;
    a.V = vocab;
    // Few slots over a wide vocabulary: the row-wide passes run over many blocks first
    // (PIE_HIP_SAMPLE_PARTS = n forces the part count, 0 the single-block path: measurement hook).
    static const int forced_parts = [] { const char* e = getenv("PIE_HIP_SAMPLE_PARTS"); return e ? atoi(e) : -1; }();
    int parts = 0;
    // (measured at a 128 k vocabulary, peaked rows: 1 / 8 slots 40-60 us less per call for the kinds
    // that sort candidates, 20-40 us less for the multinomial walk; at 64 slots the four launches
    // cost more than one block per slot, which fills a quarter of the machine by itself)
    if (vocab >= 16384 && num_slots <= 16) parts = std::min(kMaxParts, 256 / num_slots);
    if (forced_parts >= 0) parts = std::min(forced_parts, kMaxParts);
    if (parts == 1 || static_cast<size_t>(parts) * sizeof(FrontPart) > static_cast<size_t>(vocab) * 4) parts = 0;
    // a slot's part records hold doubles at byte 4 * slot * vocab of the id_a region: keep them
    // 8-byte aligned (an odd vocabulary takes the single-block path)
    if (vocab % 2 != 0 && num_slots > 1) parts = 0;
    a.parts = parts;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (parts > 0) {
        const dim3 grid(parts, num_slots);
        hipLaunchKernelGGL(sample_front_max_kernel, grid, dim3(kFrontBlock), 0, st, a);
        hipLaunchKernelGGL(sample_front_exp_kernel, grid, dim3(kFrontBlock), 0, st, a);
        hipLaunchKernelGGL(sample_front_norm_kernel, grid, dim3(kFrontBlock), 0, st, a);
        hipLaunchKernelGGL(sample_front_compact_kernel, grid, dim3(kFrontBlock), 0, st, a);
    }
    hipLaunchKernelGGL(sample_kernel, dim3(num_slots), dim3(kSampBlock), 0, st, a);
    return launch_status();
}
