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

struct BlockShared {
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
    for (int v = tid; v < V; v += kSampBlock) {
        const float x = row[v];
        if (x > bv || (bi == 0x7FFFFFFF && x == bv)) {
            bv = x;
            bi = v;
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
    for (int i0 = lo; i0 < hi; i0 += kWave) {
        const int i = i0 + lane;
        const bool valid = i < hi;
        const uint32_t key = valid ? kin[i] : 0u;
        const uint32_t d = 255u - ((key >> shift) & 255u);
        const uint64_t m = match_digit(d, valid);
        if (valid && lane == __ffsll(static_cast<long long>(m)) - 1) sh.cnt[wv][d] += __popcll(m);
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
    for (int i0 = lo; i0 < hi; i0 += kWave) {
        const int i = i0 + lane;
        const bool valid = i < hi;
        const uint32_t key = valid ? kin[i] : 0u;
        const uint32_t id = valid ? (iin ? iin[i] : static_cast<uint32_t>(i)) : 0u;
        const uint32_t d = 255u - ((key >> shift) & 255u);
        const uint64_t m = match_digit(d, valid);
        const uint32_t base = valid ? sh.cnt[wv][d] : 0u;
        const uint32_t rank = __popcll(m & ((1ull << lane) - 1ull));
        if (valid) {
            kout[base + rank] = key;
            iout[base + rank] = id;
            if (rank == 0) sh.cnt[wv][d] = base + __popcll(m);   // after every peer read `base`
        }
    }
    __syncthreads();
}

// Sorted (descending key, ascending id) result in (key_a, id_a).
__device__ void sort_desc(uint32_t* key_a, uint32_t* key_b, uint32_t* id_a, uint32_t* id_b, int n,
                          BlockShared& sh, int tid, int lane, int wv) {
    radix_pass(key_a, nullptr, key_b, id_b, n, 0, sh, tid, lane, wv);
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
    const int seg = ((limit + kSampBlock - 1) / kSampBlock) * kWave;
    const int lo = min(limit, wv * seg), hi = min(limit, lo + seg);
    double s = 0.0;
    for (int i = lo + lane; i < hi; i += kWave) s += static_cast<double>(__uint_as_float(pbits[i]));
    s = wave_sum_f64(s);
    if (lane == 0) sh.f64[wv] = s;
    __syncthreads();
    double base = 0.0, total = 0.0;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) {
        if (w < wv) base += sh.f64[w];
        total += sh.f64[w];
    }
    const float x = MODE == kExceedScaled ? thr * static_cast<float>(total) : thr;
    int cand = limit;
    double acc = base;
    for (int i0 = lo; i0 < hi; i0 += kWave) {
        const int i = i0 + lane;
        double incl = i < hi ? static_cast<double>(__uint_as_float(pbits[i])) : 0.0;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const double o = __shfl_up(incl, off, kWave);
            if (lane >= off) incl += o;
        }
        const float cum = static_cast<float>(acc + incl);
        const bool hit = i < hi && (MODE == kReach ? cum >= x : x < cum);
        const uint64_t b = __ballot(hit);
        if (b) {
            cand = i0 + __ffsll(static_cast<long long>(b)) - 1;
            break;
        }
        acc += __shfl(incl, kWave - 1, kWave);
    }
    if (lane == 0) sh.i32[wv] = cand;
    __syncthreads();
    int r = limit;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) r = min(r, sh.i32[w]);
    __syncthreads();
    *total_out = total;
    return r;
}

// p = softmax(row / T) as float bit patterns in `out`; returns the number of entries with p > 0.
__device__ int softmax_to_bits(const float* row, int V, float mx, float temperature, uint32_t* out,
                               BlockShared& sh, int tid, int lane, int wv) {
    const float inv_t = 1.0f / fmaxf(temperature, 1e-5f);
    double s = 0.0;
    for (int v = tid; v < V; v += kSampBlock) {
        const float e = expf((row[v] - mx) * inv_t);
        out[v] = __float_as_uint(e);
        s += static_cast<double>(e);
    }
    const double sum = block_sum_f64(s, sh, lane, wv);
    const float inv_sum = static_cast<float>(1.0 / fmax(1e-30, sum));
    int pos = 0;
    for (int v = tid; v < V; v += kSampBlock) {
        const float p = __uint_as_float(out[v]) * inv_sum;
        out[v] = __float_as_uint(p);
        pos += p > 0.0f;
    }
    return block_sum_i32(pos, sh, lane, wv);
}

__device__ float log_sum_exp(const float* row, int V, float mx, BlockShared& sh, int tid, int lane,
                             int wv) {
    double s = 0.0;
    for (int v = tid; v < V; v += kSampBlock) s += exp(static_cast<double>(row[v] - mx));
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
        for (int v = tid; v < V; v += kSampBlock) {
            const float lp = row[v] - lse;
            h -= exp(static_cast<double>(lp)) * static_cast<double>(lp);
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
        softmax_to_bits(row, V, mx, temperature, ka, sh, tid, lane, wv);
        __syncthreads();
        sort_desc(ka, kb, ia, ib, V, sh, tid, lane, wv);
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
    const int n_pos = softmax_to_bits(row, V, mx, temperature, ka, sh, tid, lane, wv);
    __syncthreads();
    const float u = a.uniform[s];
    double total;
    if (kind == PIE_HIP_SAMPLER_MULTINOMIAL) {
        const int tok = find_first<kExceed>(ka, V, u, sh, lane, wv, &total);
        if (tid == 0) a.tokens[s] = static_cast<uint32_t>(tok < V ? tok : amax);
        return;
    }
    if (n_pos == 0) {
        if (tid == 0) a.tokens[s] = 0u;
        return;
    }
    sort_desc(ka, kb, ia, ib, V, sh, tid, lane, wv);
    int keep = n_pos;
    const bool wants_k = kind == PIE_HIP_SAMPLER_TOP_K || kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
    const bool wants_p = kind == PIE_HIP_SAMPLER_TOP_P || kind == PIE_HIP_SAMPLER_TOP_K_TOP_P;
    if (wants_k) {
        const uint32_t k = a.top_k[s];
        if (k != 0u && k < static_cast<uint32_t>(keep)) keep = static_cast<int>(k);
    }
    if (wants_p) {
        const float thr = fminf(fmaxf(a.top_p[s], 0.0f), 1.0f);
        if (thr < 1.0f) {
            const int i = find_first<kReach>(ka, keep, thr, sh, lane, wv, &total);
            if (i < keep) keep = i + 1;
        }
    }
    if (kind == PIE_HIP_SAMPLER_MIN_P) {
        const float thr = a.min_p[s] * __uint_as_float(ka[0]);
        int c = 0;
        for (int i = tid; i < keep; i += kSampBlock) c += __uint_as_float(ka[i]) >= thr;
        const int cut = block_sum_i32(c, sh, lane, wv);   // sorted: the passing entries are a prefix
        if (cut > 0) keep = cut;
    }
    const int i = find_first<kExceedScaled>(ka, keep, u, sh, lane, wv, &total);
    uint32_t tok;
    if (total <= 0.0) tok = ia[0];
    else tok = ia[i < keep ? i : keep - 1];
    if (tid == 0) a.tokens[s] = tok;
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
