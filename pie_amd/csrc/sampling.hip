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
//   The descending order comes from a block-wide LSD radix sort (8-bit digits, 4 passes over
//   the non-negative float bit patterns): each wave owns a contiguous segment, ranks its 64
//   keys per step by matching digits across the wave (8 ballots), and scatters stably, so
//   equal keys keep ascending ids.
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
template <int MODE>
__device__ int find_first(const uint32_t* __restrict__ pbits, int limit, float thr, BlockShared& sh,
                          int lane, int wv, double* total_out) {
    // Narrow the range 16-fold per level: every wave sums one sub-range (coalesced, batched
    // loads), the first sub-range whose end satisfies the rule holds the answer; the last
    // <= 64 entries are scanned by lane.  Sums are double; only the compared value is rounded.
    int lo = 0, hi = limit;
    double base = 0.0;
    float x = thr;
    bool top = true;
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
        int pick = -1;
        double before = base, run = base;
#pragma unroll
        for (int w = 0; w < kSampWaves; ++w) {
            run += sh.f64[w];
            const float cum = static_cast<float>(run);
            const bool hit = MODE == kReach ? cum >= x : x < cum;
            if (hit && pick < 0) pick = w;
            if (pick < 0) before = run;
        }
        __syncthreads();
        if (pick < 0) {
            if (top) return limit;      // the rule is never met
            return hi - 1;              // (re-associated sums disagreeing in the last bit)
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
    return b ? lo + __ffsll(static_cast<long long>(b)) - 1 : hi - 1;
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
    block_argmax(row, V, sh, tid, lane, wv, mx, amax);
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
        softmax_to_bits<false>(row, V, mx, temperature, ka, sh, tid, lane, wv);
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
        softmax_to_bits<false>(row, V, mx, temperature, ka, sh, tid, lane, wv);
        const int tok = find_first<kExceed>(ka, V, u, sh, lane, wv, &total);
        if (tid == 0) a.tokens[s] = static_cast<uint32_t>(tok < V ? tok : amax);
        return;
    }
    const SoftmaxStats st = softmax_to_bits<true>(row, V, mx, temperature, ka, sh, tid, lane, wv);
    const int n_pos = st.n_pos;
    if (n_pos == 0) {
        if (tid == 0) a.tokens[s] = 0u;
        return;
    }
    // What the draw can touch is a head of the descending order: the first top_k entries, the
    // prefix reaching top_p, the entries above the min-p threshold, or (nothing restricting)
    // the prefix whose mass exceeds u * total.  Any set {p >= t} containing that head gives
    // the same result as the whole vocabulary, so only such a set is compacted and sorted;
    // t is the first of the levels p_max * 2^(-3j) that covers the need (exact for min-p).
    const bool wants_k = kind == PIE_HIP_SAMPLER_TOP_K || kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
    const bool wants_p = kind == PIE_HIP_SAMPLER_TOP_P || kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
    const uint32_t top_k = a.top_k[s];
    const float thr_p = fminf(fmaxf(a.top_p[s], 0.0f), 1.0f);
    const float thr_m = a.min_p[s] * __uint_as_float(st.max_bits);
    int need_count = 0;
    float need_mass = 0.f;
    uint32_t floor_bits = 0u;     // nonzero: the exact lower bound of the kept entries (min-p)
    bool keep_all = false;
    if (wants_k && top_k != 0u) need_count = static_cast<int>(min(top_k, static_cast<uint32_t>(n_pos)));
    else if (wants_p && thr_p < 1.0f) need_mass = thr_p;
    else if (kind == PIE_HIP_SAMPLER_MIN_P && thr_m > 0.0f && thr_m <= __uint_as_float(st.max_bits))
        floor_bits = __float_as_uint(thr_m);
    else {
        keep_all = true;
        need_mass = u * static_cast<float>(st.total);
    }
    for (int attempt = 0; attempt < 2; ++attempt) {
        uint32_t t_bits = 1u;     // every positive entry
        if (floor_bits) t_bits = floor_bits;
        else if (attempt == 0) {
            // the first level whose candidates cover the need (every thread computes the same)
            const uint32_t top_bits = st.max_bits;
            for (int j = 0; j < kLevels; ++j) {
                uint32_t cc = 0u;
                float cm = 0.f;
#pragma unroll
                for (int w = 0; w < kSampWaves; ++w) {
                    cc += sh.lcnt[w][j];
                    cm += sh.lmass[w][j];
                }
                const bool enough = need_count > 0 ? cc >= static_cast<uint32_t>(need_count)
                                                   : cm >= need_mass + 1e-4f;
                if (enough && top_bits > (j + 1) * kLevelStep) {
                    t_bits = top_bits - (j + 1) * kLevelStep;
                    break;
                }
            }
        }
        const int m = compact_ge(ka, t_bits, kb, ib, V, sh, lane, wv);
        const bool whole = m == n_pos;
        sort_desc(kb, ka, ib, ia, m, true, sh, tid, lane, wv);   // note: overwrites ka
        bool ok = true;
        uint32_t tok = 0u;
        if (keep_all) {
            const int i = find_first<kExceed>(kb, m, need_mass, sh, lane, wv, &total);
            ok = i < m || whole;
            tok = ib[i < m ? i : m - 1];
        } else {
            int keep = m;
            if (need_count > 0) keep = min(need_count, m);
            if (wants_p && thr_p < 1.0f) {
                const int i = find_first<kReach>(kb, keep, thr_p, sh, lane, wv, &total);
                if (i < keep) keep = i + 1;
                else ok = whole || need_count > 0;   // the prefix must end inside the candidates
            }
            const int i = find_first<kExceedScaled>(kb, keep, u, sh, lane, wv, &total);
            tok = total <= 0.0 ? ib[0] : ib[i < keep ? i : keep - 1];
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
    hipLaunchKernelGGL(sample_kernel, dim3(num_slots), dim3(kSampBlock), 0,
                       static_cast<hipStream_t>(stream), a);
    return launch_status();
}
