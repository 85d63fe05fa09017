// MoE routing and combine for gfx950.
//
//   pie_hip_moe_route: per token softmax over the router logits, top-k by repeated argmax with
//   exclusion (lowest expert index wins ties), renormalised weights — the arithmetic of
//   topk_softmax_bf16_kernel (driver/cuda/src/kernels/topk_softmax.cu:19-86; graph form
//   driver/portable/src/graph_common.cpp:262-283) — followed by a one-block kernel that builds the grouped layout
//   the expert GEMM consumes: routes counting-sorted by expert (offsets per expert, the token of
//   each sorted route, the sorted position of each (token, k) route).  The reference instead
//   launches one GEMV per route (driver/cuda/src/model/kimi_forward.cpp:662-714).
//
//   pie_hip_moe_combine: out[t] (+)= sum_k w[t, k] * y_route[pos[t, k]] in top-k order, fp32,
//   one rounding (token_batched_weighted_sum[_add]_bf16_kernel,
//   driver/cuda/src/kernels/moe_dispatch.cu:152-196).
#include "common.hip.h"

namespace pie_hip {
namespace {

constexpr int kRouteThreads = 1024;
constexpr int kMaxExperts = 512;   // the reference's MAX_EXPERTS (topk_softmax.cu:14)
constexpr int kMaxTopK = 16;       // the reference's combine unroll bound (moe_dispatch.cu:128)
constexpr int kPerLane = kMaxExperts / kWave;

// (value, index) max with ties to the lower index, across the wave: four DPP steps inside a
// 16-lane row, two row swaps across rows (no LDS permutes; the result does not depend on the
// order of the steps).
template <int CTRL>
__device__ __forceinline__ void argmax_dpp_step(float& v, int& i) {
    const float ov = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, false));
    const int oi = __builtin_amdgcn_update_dpp(i, i, CTRL, 0xF, 0xF, false);
    const bool take = ov > v || (ov == v && oi < i);
    v = take ? ov : v;
    i = take ? oi : i;
}
__device__ __forceinline__ void argmax_pick(float& v, int& i, float v0, int i0, float v1, int i1) {
    const bool first = v0 > v1 || (v0 == v1 && i0 < i1);
    v = first ? v0 : v1;
    i = first ? i0 : i1;
}
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
    argmax_dpp_step<0xB1>(v, i);    // quad_perm [1,0,3,2]
    argmax_dpp_step<0x4E>(v, i);    // quad_perm [2,3,0,1]
    argmax_dpp_step<0x141>(v, i);   // row_half_mirror
    argmax_dpp_step<0x140>(v, i);   // row_mirror: every lane holds its row's winner
    const auto v16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const auto i16 = __builtin_amdgcn_permlane16_swap(static_cast<unsigned>(i), static_cast<unsigned>(i), false, false);
    argmax_pick(v, i, __uint_as_float(v16[0]), static_cast<int>(i16[0]), __uint_as_float(v16[1]), static_cast<int>(i16[1]));
    const auto v32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const auto i32 = __builtin_amdgcn_permlane32_swap(static_cast<unsigned>(i), static_cast<unsigned>(i), false, false);
    argmax_pick(v, i, __uint_as_float(v32[0]), static_cast<int>(i32[0]), __uint_as_float(v32[1]), static_cast<int>(i32[1]));
}

// One wave: softmax over one token's experts, top-k with exclusion, renormalise (`renorm`; without
// it the chosen experts keep their softmax probabilities, driver/portable/src/graph_common.cpp:279-283).
// logit(e) returns expert e's router logit (a bf16 value widened to float).
template <class Logit>
__device__ __forceinline__ void topk_of_token(Logit logit, int lane, int t, int32_t* __restrict__ topk_idx,
                                              float* __restrict__ topk_w, int E, int K, int renorm) {
    // (entries j >= nper hold no expert: the passes below skip them)
    const int nper = (E + kWave - 1) / kWave;
    float p[kPerLane];
    float mx = -3.4e38f;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
        const int e = lane + kWave * j;
        p[j] = e < E ? logit(e) : -3.4e38f;
        mx = fmaxf(mx, p[j]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
        const int e = lane + kWave * j;
        float ex = 0.f;
        if (j < nper) ex = e < E ? expf(p[j] - mx) : 0.f;   // (a wave-uniform test)
        p[j] = ex;
        sum += ex;
    }
    sum = wave_sum(sum);
    const float inv_z = 1.f / sum;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) p[j] = (lane + kWave * j < E) ? p[j] * inv_z : -2.f;
    float w_sum = 0.f, my_w = 0.f;   // lane k keeps the k-th weight
    int my_e = 0;
    for (int k = 0; k < K; ++k) {
        float bv = -1.f;
        int bi = kMaxExperts;
#pragma unroll
        for (int j = 0; j < kPerLane; ++j)
            if (j < nper && p[j] > bv) {
                bv = p[j];
                bi = lane + kWave * j;
            }
        wave_argmax(bv, bi);
        bi = min(bi, E - 1);   // only reachable with NaN logits; keeps every index in range
#pragma unroll
        for (int j = 0; j < kPerLane; ++j)
            if (j < nper && bi == lane + kWave * j) p[j] = -1.f;   // exclude on the next pass
        w_sum += bv;
        if (lane == k) {
            my_w = bv;
            my_e = bi;
        }
    }
    const float inv_w = 1.f / w_sum;
    if (lane < K) {
        topk_idx[static_cast<size_t>(t) * K + lane] = my_e;
        topk_w[static_cast<size_t>(t) * K + lane] = renorm ? my_w * inv_w : my_w;
    }
}

// One wave per token.
__global__ __launch_bounds__(256) void moe_topk_kernel(const uint16_t* __restrict__ logits,
                                                       int32_t* __restrict__ topk_idx,
                                                       float* __restrict__ topk_w, int N, int E, int K,
                                                       int renorm) {
    const int lane = threadIdx.x & (kWave - 1);
    const int t = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (t >= N) return;
    const uint16_t* row = logits + static_cast<size_t>(t) * E;
    topk_of_token([&](int e) { return bf16_bits_to_f32(row[e]); }, lane, t, topk_idx, topk_w, E, K, renorm);
}

// A decode batch's way into the MoE block, one block of sixteen waves per token: RMSNorm of the
// token's row by the first four waves (the arithmetic and thread assignment of rmsnorm_kernel: the
// stored row is the one pie_hip_rmsnorm stores, bit for bit), the router logits as bf16(fp32 dot
// product) of that row with the experts' router rows — a wave takes eight experts at a time with
// all their 16-byte pieces of 1024 k-values in flight, so 128 experts are one pass — and the
// top-k of topk_of_token by the first wave.  The router matrix is read through the L2 by every
// token (E * H * 2 bytes each): for batches of up to a few hundred rows that is cheaper than a
// norm launch, a GEMM launch and a top-k launch.  The fp32 sums run in this kernel's own order (a
// lane's pieces in ascending k, then the wave's butterfly), like every other product of the library.
constexpr int kNormRouteThreads = 1024;
constexpr int kNormThreads = 256;     // rmsnorm_kernel's block
constexpr int kNormRouteMaxVec = 4;   // rows of up to 256 * 8 * 4 = 8192 values
__global__ __launch_bounds__(kNormRouteThreads) void moe_norm_route_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ norm_w, const uint16_t* __restrict__ router,
    uint16_t* __restrict__ xn, uint16_t* __restrict__ logits_out, int32_t* __restrict__ topk_idx,
    float* __restrict__ topk_w, int H, int E, int K, float eps, int renorm) {
    extern __shared__ __align__(16) unsigned char smem[];
    u32x4_t* row_lds = reinterpret_cast<u32x4_t*>(smem);            // [H / 8]
    float* logit_lds = reinterpret_cast<float*>(row_lds + H / 8);   // [E]
    __shared__ float red[4];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int t = blockIdx.x;
    const size_t base = static_cast<size_t>(t) * H;
    const int nvec = H / 8;
    u32x4_t cache[kNormRouteMaxVec];
    float local = 0.f;
    if (tid < kNormThreads) {
#pragma unroll
        for (int c = 0; c < kNormRouteMaxVec; ++c) {
            const int v = tid + c * kNormThreads;
            if (v < nvec) {
                cache[c] = *reinterpret_cast<const u32x4_t*>(x + base + v * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lo = bf16_lo(cache[c][i]), hi = bf16_hi(cache[c][i]);
                    local += lo * lo + hi * hi;
                }
            }
        }
        // (rmsnorm_kernel's block_sum)
        local = wave_sum(local);
        if (lane == 0) red[wv] = local;
    }
    __syncthreads();
    if (tid < kNormThreads) {
        float total = 0.f;
#pragma unroll
        for (int i = 0; i < kNormThreads / kWave; ++i) total += red[i];
        const float inv_rms = rsqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
        for (int c = 0; c < kNormRouteMaxVec; ++c) {
            const int v = tid + c * kNormThreads;
            if (v < nvec) {
                const u32x4_t ww = *reinterpret_cast<const u32x4_t*>(norm_w + v * 8);
                u32x4_t o;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    o[i] = pack_bf16x2(bf16_lo(cache[c][i]) * inv_rms * bf16_lo(ww[i]),
                                       bf16_hi(cache[c][i]) * inv_rms * bf16_hi(ww[i]));
                *reinterpret_cast<u32x4_t*>(xn + base + v * 8) = o;
                row_lds[v] = o;
            }
        }
    }
    __syncthreads();
    constexpr int kWaves = kNormRouteThreads / kWave, kAt = 8;
    // (the blocks of a batch run in step: each starts at another group of experts, or all of them
    // ask the same L2 channel for the same lines at the same time)
    const int wrot = (wv + t * 5) % kWaves;
    for (int e0 = wrot * kAt; e0 < E; e0 += kWaves * kAt) {
        float acc[kAt];
#pragma unroll
        for (int j = 0; j < kAt; ++j) acc[j] = 0.f;
        // two 512-value steps per trip: sixteen loads in flight per lane
        for (int v0 = lane; v0 < nvec; v0 += 2 * kWave) {
            const int v1 = v0 + kWave;
            const bool two = v1 < nvec;
            u32x4_t w0[kAt], w1[kAt];
#pragma unroll
            for (int j = 0; j < kAt; ++j) {
                const uint16_t* row = router + static_cast<size_t>(min(e0 + j, E - 1)) * H;
                w0[j] = *reinterpret_cast<const u32x4_t*>(row + v0 * 8);
                w1[j] = *reinterpret_cast<const u32x4_t*>(row + (two ? v1 : v0) * 8);
            }
            const u32x4_t a0 = row_lds[v0];
            const u32x4_t a1 = two ? row_lds[v1] : u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
            for (int j = 0; j < kAt; ++j) {
                acc[j] = dot2_bf16(a0.x, w0[j].x, acc[j]);
                acc[j] = dot2_bf16(a0.y, w0[j].y, acc[j]);
                acc[j] = dot2_bf16(a0.z, w0[j].z, acc[j]);
                acc[j] = dot2_bf16(a0.w, w0[j].w, acc[j]);
                acc[j] = dot2_bf16(a1.x, w1[j].x, acc[j]);
                acc[j] = dot2_bf16(a1.y, w1[j].y, acc[j]);
                acc[j] = dot2_bf16(a1.z, w1[j].z, acc[j]);
                acc[j] = dot2_bf16(a1.w, w1[j].w, acc[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < kAt; ++j) {
            const float s = wave_sum_dpp(acc[j]);
            if (lane == 0 && e0 + j < E) {
                const uint16_t b = f32_to_bf16_bits(s);
                logit_lds[e0 + j] = bf16_bits_to_f32(b);
                if (logits_out) logits_out[static_cast<size_t>(t) * E + e0 + j] = b;
            }
        }
    }
    __syncthreads();
    // Top-k by rank instead of k dependent argmax passes of one wave (a chain of ~800
    // instructions, 3 us): the first wave turns the logits into the probabilities of
    // topk_of_token (same operations, same order), every thread then counts, for one expert and a
    // share of the others, how many precede it — larger probability, or equal and a lower index:
    // the order in which the argmax passes pick — and the experts of rank < k are the choice, in
    // rank order.  Bit-identical to topk_of_token for finite logits.
    float* prob_lds = logit_lds;                                    // (overwritten in place)
    int* rank_lds = reinterpret_cast<int*>(logit_lds + E);          // [E]
    float* sel_w = reinterpret_cast<float*>(rank_lds + E);          // [kMaxTopK]
    int* sel_e = reinterpret_cast<int*>(sel_w + kMaxTopK);          // [kMaxTopK]
    if (wv == 0) {
        const int nper = (E + kWave - 1) / kWave;
        float p[kPerLane];
        float mx = -3.4e38f;
#pragma unroll
        for (int j = 0; j < kPerLane; ++j) {
            const int e = lane + kWave * j;
            p[j] = e < E ? logit_lds[e] : -3.4e38f;
            mx = fmaxf(mx, p[j]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < kPerLane; ++j) {
            const int e = lane + kWave * j;
            float ex = 0.f;
            if (j < nper) ex = e < E ? expf(p[j] - mx) : 0.f;
            p[j] = ex;
            sum += ex;
        }
        sum = wave_sum(sum);
        const float inv_z = 1.f / sum;
#pragma unroll
        for (int j = 0; j < kPerLane; ++j) {
            const int e = lane + kWave * j;
            if (e < E) prob_lds[e] = p[j] * inv_z;
        }
    }
    for (int e = tid; e < E; e += kNormRouteThreads) rank_lds[e] = 0;
    __syncthreads();
    {
        // thread (e, share): kShares threads per expert, each over every kShares-th rival
        const int shares = max(1, kNormRouteThreads / E);            // 8 for 128 experts
        for (int e = tid / shares; e < E; e += kNormRouteThreads / shares) {
            const int sh = tid % shares;
            const float pe = prob_lds[e];
            int before = 0;
            for (int o = sh; o < E; o += shares) {
                const float po = prob_lds[o];
                before += (po > pe || (po == pe && o < e)) ? 1 : 0;
            }
            if (before) atomicAdd(&rank_lds[e], before);
        }
    }
    __syncthreads();
    for (int e = tid; e < E; e += kNormRouteThreads) {
        const int r = rank_lds[e];
        if (r < K) {
            sel_w[r] = prob_lds[e];
            sel_e[r] = e;
        }
    }
    __syncthreads();
    if (tid < K) {
        float w_sum = 0.f;
        for (int k = 0; k < K; ++k) w_sum += sel_w[k];   // (the passes' order)
        const float inv_w = 1.f / w_sum;
        topk_idx[static_cast<size_t>(t) * K + tid] = sel_e[tid];
        topk_w[static_cast<size_t>(t) * K + tid] = renorm ? sel_w[tid] * inv_w : sel_w[tid];
    }
}

// One block: rank of every route inside its expert, expert offsets, sorted positions.
__global__ __launch_bounds__(kRouteThreads) void moe_sort_kernel(
    const int32_t* __restrict__ topk_idx, int32_t* __restrict__ expert_offsets,
    int32_t* __restrict__ route_token, int32_t* __restrict__ route_pos, int N, int E, int K) {
    __shared__ int cnt[kMaxExperts];
    __shared__ int base[kMaxExperts + 1];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    for (int e = tid; e < E; e += kRouteThreads) cnt[e] = 0;
    __syncthreads();
    const int R = N * K;
    for (int r = tid; r < R; r += kRouteThreads) route_pos[r] = atomicAdd(&cnt[topk_idx[r]], 1);
    __syncthreads();
    if (wv == 0) {
        // exclusive scan of cnt[0..E): each lane owns a run of consecutive experts
        const int per = (E + kWave - 1) / kWave;
        int run = 0;
        for (int i = 0; i < per; ++i) {
            const int e = lane * per + i;
            if (e < E) run += cnt[e];
        }
        int incl = run;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int o = __shfl_up(incl, off, kWave);
            if (lane >= off) incl += o;
        }
        int acc = incl - run;
        for (int i = 0; i < per; ++i) {
            const int e = lane * per + i;
            if (e < E) {
                base[e] = acc;
                acc += cnt[e];
            }
        }
        if (lane == kWave - 1) base[E] = incl;
    }
    __syncthreads();
    for (int e = tid; e <= E; e += kRouteThreads) expert_offsets[e] = base[e];
    for (int r = tid; r < R; r += kRouteThreads) {
        const int pos = base[topk_idx[r]] + route_pos[r];
        route_pos[r] = pos;
        route_token[pos] = r / K;
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(
    const uint16_t* __restrict__ y_routes, const int32_t* __restrict__ route_pos,
    const float* __restrict__ topk_w, uint16_t* __restrict__ out, int K, int H, int add) {
    const int t = blockIdx.y;
    const int h = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (h >= H) return;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < K; ++k) {
        const int pos = route_pos[static_cast<size_t>(t) * K + k];
        const float w = topk_w[static_cast<size_t>(t) * K + k];
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(y_routes + static_cast<size_t>(pos) * H + h);
        acc[0] = fmaf(w, bf16_lo(v.x), acc[0]);
        acc[1] = fmaf(w, bf16_hi(v.x), acc[1]);
        acc[2] = fmaf(w, bf16_lo(v.y), acc[2]);
        acc[3] = fmaf(w, bf16_hi(v.y), acc[3]);
        acc[4] = fmaf(w, bf16_lo(v.z), acc[4]);
        acc[5] = fmaf(w, bf16_hi(v.z), acc[5]);
        acc[6] = fmaf(w, bf16_lo(v.w), acc[6]);
        acc[7] = fmaf(w, bf16_hi(v.w), acc[7]);
    }
    u32x4_t* o = reinterpret_cast<u32x4_t*>(out + static_cast<size_t>(t) * H + h);
    if (add) {
        const u32x4_t p = *o;
        acc[0] += bf16_lo(p.x);
        acc[1] += bf16_hi(p.x);
        acc[2] += bf16_lo(p.y);
        acc[3] += bf16_hi(p.y);
        acc[4] += bf16_lo(p.z);
        acc[5] += bf16_hi(p.z);
        acc[6] += bf16_lo(p.w);
        acc[7] += bf16_hi(p.w);
    }
    *o = u32x4_t{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]),
                 pack_bf16x2(acc[4], acc[5]), pack_bf16x2(acc[6], acc[7])};
}

// The combine with the residual add (moe_combine_kernel, add = 1) and, on the row it has just
// stored, the RMSNorm in front of the next layer's projections (rmsnorm_kernel's arithmetic on the
// rounded row): one block per token, both results bit-identical to the two separate launches.
__global__ __launch_bounds__(256) void moe_combine_norm_kernel(
    const uint16_t* __restrict__ y_routes, const int32_t* __restrict__ route_pos,
    const float* __restrict__ topk_w, uint16_t* __restrict__ out, const uint16_t* __restrict__ norm_w,
    uint16_t* __restrict__ xn, int K, int H, float eps) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int nvec = H / 8;
    const size_t base = static_cast<size_t>(t) * H;
    u32x4_t cache[kNormRouteMaxVec];
    float local = 0.f;
#pragma unroll
    for (int c = 0; c < kNormRouteMaxVec; ++c) {
        const int v = tid + c * 256;
        if (v < nvec) {
            const int h = v * 8;
            float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < K; ++k) {
                const int pos = route_pos[static_cast<size_t>(t) * K + k];
                const float w = topk_w[static_cast<size_t>(t) * K + k];
                const u32x4_t yv = *reinterpret_cast<const u32x4_t*>(y_routes + static_cast<size_t>(pos) * H + h);
                acc[0] = fmaf(w, bf16_lo(yv.x), acc[0]);
                acc[1] = fmaf(w, bf16_hi(yv.x), acc[1]);
                acc[2] = fmaf(w, bf16_lo(yv.y), acc[2]);
                acc[3] = fmaf(w, bf16_hi(yv.y), acc[3]);
                acc[4] = fmaf(w, bf16_lo(yv.z), acc[4]);
                acc[5] = fmaf(w, bf16_hi(yv.z), acc[5]);
                acc[6] = fmaf(w, bf16_lo(yv.w), acc[6]);
                acc[7] = fmaf(w, bf16_hi(yv.w), acc[7]);
            }
            u32x4_t* o = reinterpret_cast<u32x4_t*>(out + base + h);
            const u32x4_t p = *o;
            acc[0] += bf16_lo(p.x);
            acc[1] += bf16_hi(p.x);
            acc[2] += bf16_lo(p.y);
            acc[3] += bf16_hi(p.y);
            acc[4] += bf16_lo(p.z);
            acc[5] += bf16_hi(p.z);
            acc[6] += bf16_lo(p.w);
            acc[7] += bf16_hi(p.w);
            const u32x4_t r = u32x4_t{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]),
                                      pack_bf16x2(acc[4], acc[5]), pack_bf16x2(acc[6], acc[7])};
            *o = r;
            cache[c] = r;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = bf16_lo(r[i]), hi = bf16_hi(r[i]);
                local += lo * lo + hi * hi;
            }
        }
    }
    local = wave_sum(local);
    if (lane == 0) red[wv] = local;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) total += red[i];
    const float inv_rms = rsqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
    for (int c = 0; c < kNormRouteMaxVec; ++c) {
        const int v = tid + c * 256;
        if (v < nvec) {
            const u32x4_t ww = *reinterpret_cast<const u32x4_t*>(norm_w + v * 8);
            u32x4_t o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o[i] = pack_bf16x2(bf16_lo(cache[c][i]) * inv_rms * bf16_lo(ww[i]),
                                   bf16_hi(cache[c][i]) * inv_rms * bf16_hi(ww[i]));
            *reinterpret_cast<u32x4_t*>(xn + base + v * 8) = o;
        }
    }
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_moe_norm_route(const uint16_t* x_bf16, const uint16_t* norm_weight_bf16, float eps,
                                      const uint16_t* router_bf16, uint16_t* norm_out_bf16,
                                      uint16_t* router_logits_bf16, int32_t* topk_idx, float* topk_weight,
                                      int32_t* expert_offsets, int32_t* route_token, int32_t* route_pos,
                                      int num_tokens, int hidden, int num_experts, int top_k, int renormalize,
                                      void* stream) {
    using namespace pie_hip;
    if (!x_bf16 || !norm_weight_bf16 || !router_bf16 || !norm_out_bf16 || !topk_idx || !topk_weight ||
        !expert_offsets || !route_token || !route_pos || num_tokens <= 0 || hidden <= 0)
        return PIE_HIP_ERR_INVALID;
    if (num_experts <= 0 || num_experts > kMaxExperts || top_k <= 0 || top_k > kMaxTopK || top_k > num_experts ||
        hidden % 8 != 0 || hidden > kNormThreads * 8 * kNormRouteMaxVec)
        return PIE_HIP_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t smem = static_cast<size_t>(hidden) * 2 + static_cast<size_t>(num_experts) * 2 * sizeof(float) +
                        kMaxTopK * 2 * sizeof(float);
    hipLaunchKernelGGL(moe_norm_route_kernel, dim3(num_tokens), dim3(kNormRouteThreads), smem, st, x_bf16,
                       norm_weight_bf16, router_bf16, norm_out_bf16, router_logits_bf16, topk_idx, topk_weight,
                       hidden, num_experts, top_k, eps, renormalize ? 1 : 0);
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(kRouteThreads), 0, st, topk_idx, expert_offsets,
                       route_token, route_pos, num_tokens, num_experts, top_k);
    return launch_status();
}

extern "C" int pie_hip_moe_combine_norm(const uint16_t* y_routes_bf16, const int32_t* route_pos,
                                        const float* topk_weight, uint16_t* out_bf16,
                                        const uint16_t* norm_weight_bf16, float eps, uint16_t* norm_out_bf16,
                                        int num_tokens, int top_k, int hidden, void* stream) {
    using namespace pie_hip;
    if (!y_routes_bf16 || !route_pos || !topk_weight || !out_bf16 || !norm_weight_bf16 || !norm_out_bf16 ||
        num_tokens <= 0)
        return PIE_HIP_ERR_INVALID;
    if (hidden <= 0 || hidden % 8 != 0 || hidden > 256 * 8 * kNormRouteMaxVec || top_k <= 0 || top_k > kMaxTopK)
        return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(moe_combine_norm_kernel, dim3(num_tokens), dim3(256), 0, static_cast<hipStream_t>(stream),
                       y_routes_bf16, route_pos, topk_weight, out_bf16, norm_weight_bf16, norm_out_bf16, top_k,
                       hidden, eps);
    return launch_status();
}

extern "C" int pie_hip_moe_route(const uint16_t* router_logits_bf16, int32_t* topk_idx,
                                 float* topk_weight, int32_t* expert_offsets,
                                 int32_t* route_token, int32_t* route_pos, int num_tokens,
                                 int num_experts, int top_k, void* stream) {
    return pie_hip_moe_route_opt(router_logits_bf16, topk_idx, topk_weight, expert_offsets, route_token,
                                 route_pos, num_tokens, num_experts, top_k, 1, stream);
}

extern "C" int pie_hip_moe_route_opt(const uint16_t* router_logits_bf16, int32_t* topk_idx,
                                     float* topk_weight, int32_t* expert_offsets,
                                     int32_t* route_token, int32_t* route_pos, int num_tokens,
                                     int num_experts, int top_k, int renormalize, void* stream) {
    using namespace pie_hip;
    if (!router_logits_bf16 || !topk_idx || !topk_weight || !expert_offsets || !route_token ||
        !route_pos || num_tokens <= 0)
        return PIE_HIP_ERR_INVALID;
    if (num_experts <= 0 || num_experts > kMaxExperts || top_k <= 0 || top_k > kMaxTopK ||
        top_k > num_experts)
        return PIE_HIP_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(moe_topk_kernel, dim3((num_tokens + 3) / 4), dim3(256), 0, st,
                       router_logits_bf16, topk_idx, topk_weight, num_tokens, num_experts, top_k,
                       renormalize ? 1 : 0);
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(kRouteThreads), 0, st, topk_idx, expert_offsets,
                       route_token, route_pos, num_tokens, num_experts, top_k);
    return launch_status();
}

extern "C" int pie_hip_moe_combine(const uint16_t* y_routes_bf16, const int32_t* route_pos,
                                   const float* topk_weight, uint16_t* out_bf16, int num_tokens,
                                   int top_k, int hidden, int add, void* stream) {
    using namespace pie_hip;
    if (!y_routes_bf16 || !route_pos || !topk_weight || !out_bf16 || num_tokens <= 0)
        return PIE_HIP_ERR_INVALID;
    if (hidden <= 0 || hidden % 8 != 0 || top_k <= 0 || top_k > kMaxTopK) return PIE_HIP_ERR_UNSUPPORTED;
    const dim3 grid((hidden / 8 + 255) / 256, num_tokens);
    hipLaunchKernelGGL(moe_combine_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                       y_routes_bf16, route_pos, topk_weight, out_bf16, top_k, hidden, add ? 1 : 0);
    return launch_status();
}
