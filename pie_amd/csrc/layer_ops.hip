// The small per-layer kernels of the llama-like decoder: embedding gather, RMSNorm
// (plain and residual-add fused), RoPE table, fused per-head qk-norm + RoPE + KV page
// write, SwiGLU, argmax and KV page copies.  All are HBM/latency bound; each moves
// every byte once with 16-byte accesses where the layout allows and keeps the
// reference's rounding points (fp32 maths inside an op, one bf16 rounding at its
// output), see the driver/cuda/src/kernels citations on each kernel.
#include "common.hip.h"

namespace pie_hip {
namespace {

__device__ __forceinline__ float block_sum(float v, float* smem) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    const int nw = (blockDim.x + kWave - 1) / kWave;
    __syncthreads();
    if (lane == 0) smem[wv] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += smem[i];
    return t;
}

// y[n,:] = E[token[n],:]; out-of-vocab ids read row 0 (driver/cuda/src/kernels/embed.cu:8-23).
__global__ void embed_kernel(const uint32_t* __restrict__ tokens, const u32x4_t* __restrict__ table,
                             u32x4_t* __restrict__ y, int hidden_v4, int vocab) {
    const int n = blockIdx.x;
    const uint32_t t = tokens[n];
    const size_t row = t < static_cast<uint32_t>(vocab) ? t : 0;
    for (int i = threadIdx.x; i < hidden_v4; i += blockDim.x)
        y[static_cast<size_t>(n) * hidden_v4 + i] = table[row * hidden_v4 + i];
}

// RMSNorm, optionally fused with the residual add that precedes it:
//   FUSE: h = bf16(h + r) is stored back, the norm reads the rounded h
//         (driver/cuda/src/kernels/rmsnorm.cu:56-98);
//   else: y = bf16(x * rsqrt(mean(x^2) + eps) * w)  (rmsnorm.cu:14-54).
// One block per row, 8 elements per thread per step, row cached in registers for H <= 8192.
template <bool FUSE>
__global__ __launch_bounds__(256) void rmsnorm_kernel(uint16_t* __restrict__ x,
                                                      const uint16_t* __restrict__ residual,
                                                      const uint16_t* __restrict__ w,
                                                      uint16_t* __restrict__ y, int H, float eps) {
    __shared__ float red[4];
    const size_t base = static_cast<size_t>(blockIdx.x) * H;
    constexpr int kMaxVec = 4;  // 256 threads * 8 * 4 = 8192 columns in registers
    u32x4_t cache[kMaxVec];
    float local = 0.f;
    const int nvec = H / 8;
    auto load_vec = [&](int v) {
        u32x4_t a = *reinterpret_cast<const u32x4_t*>(x + base + v * 8);
        if (FUSE) {
            const u32x4_t r = *reinterpret_cast<const u32x4_t*>(residual + base + v * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                a[i] = pack_bf16x2(bf16_lo(a[i]) + bf16_lo(r[i]), bf16_hi(a[i]) + bf16_hi(r[i]));
            *reinterpret_cast<u32x4_t*>(x + base + v * 8) = a;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = bf16_lo(a[i]), hi = bf16_hi(a[i]);
            local += lo * lo + hi * hi;
        }
        return a;
    };
    // (the norm weights are requested with the row, ahead of the block-wide sum: one wait for
    // memory instead of two in a row)
    u32x4_t wcache[kMaxVec];
#pragma unroll
    for (int c = 0; c < kMaxVec; ++c) {
        const int v = threadIdx.x + c * 256;
        if (v < nvec) wcache[c] = *reinterpret_cast<const u32x4_t*>(w + v * 8);
    }
#pragma unroll
    for (int c = 0; c < kMaxVec; ++c) {
        const int v = threadIdx.x + c * 256;
        if (v < nvec) cache[c] = load_vec(v);
    }
    for (int v = threadIdx.x + kMaxVec * 256; v < nvec; v += 256) load_vec(v);
    const float total = block_sum(local, red);
    const float inv_rms = rsqrtf(total / static_cast<float>(H) + eps);
    auto store_vec = [&](int v, const u32x4_t a, const u32x4_t ww) {
        u32x4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            o[i] = pack_bf16x2(bf16_lo(a[i]) * inv_rms * bf16_lo(ww[i]),
                               bf16_hi(a[i]) * inv_rms * bf16_hi(ww[i]));
        *reinterpret_cast<u32x4_t*>(y + base + v * 8) = o;
    };
#pragma unroll
    for (int c = 0; c < kMaxVec; ++c) {
        const int v = threadIdx.x + c * 256;
        if (v < nvec) store_vec(v, cache[c], wcache[c]);
    }
    for (int v = threadIdx.x + kMaxVec * 256; v < nvec; v += 256)
        store_vec(v, *reinterpret_cast<const u32x4_t*>(x + base + v * 8), *reinterpret_cast<const u32x4_t*>(w + v * 8));
}

// table[n, i] = cos(pos_n * inv_freq[i]), table[n, i + d/2] = sin(...), i < d/2: the
// per-forward cos/sin rows every layer reuses (rope_standard_table_kernel,
// driver/cuda/src/kernels/rope.cu:35-53).  inv_freq comes from the host so that any
// frequency scaling (llama3 bands, YaRN) is a host-side table, not kernel code.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq, float* __restrict__ table,
                                  int d, float mscale) {
    const int n = blockIdx.x, half = d / 2;
    const float pos = static_cast<float>(positions[n]);
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const float ang = pos * inv_freq[i];
        float s, c;
        sincosf(ang, &s, &c);
        // (YaRN's attention factor rides on cos and sin, driver/cuda/src/kernels/rope.cu:531-535;
        // 1 otherwise, which changes no bit)
        table[static_cast<size_t>(n) * d + i] = c * mscale;
        table[static_cast<size_t>(n) * d + i + half] = s * mscale;
    }
}

// One wave per (token, head) of a packed QKV row [N, (hq + 2*hk) * d]:
//   q heads: optional per-head RMSNorm (fp32, unrounded), RoPE, bf16 -> q_out[N, hq, d];
//   k heads: same, written straight into the KV page slot kv_slots[n];
//   v heads: copied into the slot.
// One bf16 rounding at the store (qkv_decode_qk_norm_rope_write_kv_kernel,
// driver/cuda/src/kernels/split_packed.cu:62-178; slot addressing :116-138 NHD).  The slot
// (page*page_size + offset) is computed by the host planner from the page table, so the
// same kernel serves decode and prefill rows.  interleaved = 0 pairs (i, i+d/2), 1 pairs
// (2i, 2i+1) (driver/cuda/src/kernels/rope.cu:14-33); 2: the projection's q / k rows were
// re-ordered at load so that elements (2i, 2i+1) of its output hold the half-split pair
// (i, i+d/2) — rotated as that pair and written to positions i and i+d/2, so q_out and the
// pool hold exactly what interleaved = 0 gives over the original row order.
__global__ __launch_bounds__(64) void qkv_rope_kvwrite_kernel(
    const uint16_t* __restrict__ packed, uint16_t* __restrict__ q_out,
    uint16_t* __restrict__ k_pages, uint16_t* __restrict__ v_pages,
    const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
    const float* __restrict__ rope_table, const int64_t* __restrict__ kv_slots, int hq, int hk,
    int d, int interleaved, float eps) {
    const int n = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int half = d / 2;
    const size_t stride = static_cast<size_t>(hq + 2 * hk) * d;
    const uint16_t* src = packed + n * stride + static_cast<size_t>(head) * d;
    const bool is_q = head < hq, is_k = !is_q && head < hq + hk;
    const int64_t slot = kv_slots[n];
    if (!is_q && slot < 0) return;  // token without a KV slot
    if (!is_q && !is_k) {
        uint16_t* dst = v_pages + (static_cast<size_t>(slot) * hk + (head - hq - hk)) * d;
        for (int i = lane; i < d / 8; i += kWave)
            reinterpret_cast<u32x4_t*>(dst)[i] = reinterpret_cast<const u32x4_t*>(src)[i];
        return;
    }
    const uint16_t* nw = is_q ? q_norm_w : k_norm_w;
    float inv_rms = 1.f;
    if (nw) {
        float local = 0.f;
        for (int i = lane; i < d; i += kWave) {
            const float v = bf16_bits_to_f32(src[i]);
            local += v * v;
        }
        inv_rms = rsqrtf(wave_sum(local) / static_cast<float>(d) + eps);
    }
    uint16_t* dst = is_q ? q_out + (static_cast<size_t>(n) * hq + head) * d
                         : k_pages + (static_cast<size_t>(slot) * hk + (head - hq)) * d;
    const float* tab = rope_table + static_cast<size_t>(n) * d;
    for (int i = lane; i < half; i += kWave) {
        // where pair i sits in the projection's row, and where it goes
        const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
        const int oa = interleaved == 1 ? 2 * i : i, ob = interleaved == 1 ? 2 * i + 1 : i + half;
        float a = bf16_bits_to_f32(src[ia]), b = bf16_bits_to_f32(src[ib]);
        if (nw) {
            a = a * inv_rms * bf16_bits_to_f32(nw[oa]);
            b = b * inv_rms * bf16_bits_to_f32(nw[ob]);
        }
        const float c = tab[i], s = tab[i + half];
        dst[oa] = f32_to_bf16_bits(a * c - b * s);
        dst[ob] = f32_to_bf16_bits(b * c + a * s);
    }
}

// y[n, i] = bf16( silu(g) * u ), g = gu[n, i], u = gu[n, I + i] over a fused gate/up row
// [N, 2I] (swiglu_bf16_kernel, driver/cuda/src/kernels/swiglu.cu:9-22; fused-row form
// chunked_swiglu, swiglu.hpp:82).  8 elements per thread.
__global__ void swiglu_kernel(const uint16_t* __restrict__ gu, uint16_t* __restrict__ y, int I,
                              size_t total_vec) {
    const size_t v = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (v >= total_vec) return;
    const int vec_per_row = I / 8;
    const size_t n = v / vec_per_row;
    const int i = static_cast<int>(v - n * vec_per_row) * 8;
    const u32x4_t g = *reinterpret_cast<const u32x4_t*>(gu + n * 2 * I + i);
    const u32x4_t u = *reinterpret_cast<const u32x4_t*>(gu + n * 2 * I + I + i);
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float g0 = bf16_lo(g[j]), g1 = bf16_hi(g[j]);
        o[j] = pack_bf16x2(g0 / (1.f + expf(-g0)) * bf16_lo(u[j]),
                           g1 / (1.f + expf(-g1)) * bf16_hi(u[j]));
    }
    *reinterpret_cast<u32x4_t*>(y + n * I + i) = o;
}

// Row argmax over bf16 logits; ties -> lowest index; NaN never wins
// (argmax_bf16_kernel, driver/cuda/src/kernels/argmax.cu:36-80).
__device__ __forceinline__ void argmax_update(float v, int idx, float& bv, int& bi) {
    if (v > bv || (v == bv && idx < bi)) {
        bv = v;
        bi = idx;
    }
}
__global__ __launch_bounds__(1024) void argmax_kernel(const uint16_t* __restrict__ logits,
                                                      uint32_t* __restrict__ out, int V) {
    __shared__ float svals[16];
    __shared__ int sidx[16];
    const uint16_t* row = logits + static_cast<size_t>(blockIdx.x) * V;
    float bv = -INFINITY;
    int bi = 0;
    const int nvec = V / 8;
    for (int v = threadIdx.x; v < nvec; v += blockDim.x) {
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(row + v * 8);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            argmax_update(bf16_lo(a[j]), v * 8 + 2 * j, bv, bi);
            argmax_update(bf16_hi(a[j]), v * 8 + 2 * j + 1, bv, bi);
        }
    }
    for (int i = nvec * 8 + threadIdx.x; i < V; i += blockDim.x)
        argmax_update(bf16_bits_to_f32(row[i]), i, bv, bi);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        argmax_update(ov, oi, bv, bi);
    }
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    if (lane == 0) {
        svals[wv] = bv;
        sidx[wv] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nw = (blockDim.x + kWave - 1) / kWave;
        for (int i = 1; i < nw; ++i) argmax_update(svals[i], sidx[i], bv, bi);
        out[blockIdx.x] = static_cast<uint32_t>(bi);
    }
}

// Device-to-device KV page copies (fork of a partially filled tail page):
// page dsts[i] <- page srcs[i], `page_vec` 16-byte vectors each
// (driver/portable/src/service/inproc_service.cpp:149-172).
__global__ void copy_pages_kernel(u32x4_t* __restrict__ pool, const uint32_t* __restrict__ srcs,
                                  const uint32_t* __restrict__ dsts, size_t page_vec) {
    const size_t s = srcs[blockIdx.y], dpg = dsts[blockIdx.y];
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < page_vec;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        pool[dpg * page_vec + i] = pool[s * page_vec + i];
}

}  // namespace
}  // namespace pie_hip

using namespace pie_hip;

extern "C" int pie_hip_embed(const uint32_t* token_ids, const uint16_t* table_bf16,
                             uint16_t* y_bf16, int num_tokens, int hidden, int vocab,
                             void* stream) {
    if (!token_ids || !table_bf16 || !y_bf16 || num_tokens <= 0 || hidden <= 0 || vocab <= 0)
        return PIE_HIP_ERR_INVALID;
    if (hidden % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(embed_kernel, dim3(num_tokens), dim3(256), 0,
                       static_cast<hipStream_t>(stream), token_ids,
                       reinterpret_cast<const u32x4_t*>(table_bf16),
                       reinterpret_cast<u32x4_t*>(y_bf16), hidden / 8, vocab);
    return launch_status();
}

extern "C" int pie_hip_rmsnorm(const uint16_t* x_bf16, const uint16_t* weight_bf16,
                               uint16_t* y_bf16, int rows, int hidden, float eps, void* stream) {
    if (!x_bf16 || !weight_bf16 || !y_bf16 || rows <= 0 || hidden <= 0) return PIE_HIP_ERR_INVALID;
    if (hidden % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(rmsnorm_kernel<false>, dim3(rows), dim3(256), 0,
                       static_cast<hipStream_t>(stream), const_cast<uint16_t*>(x_bf16), nullptr,
                       weight_bf16, y_bf16, hidden, eps);
    return launch_status();
}

extern "C" int pie_hip_residual_rmsnorm(uint16_t* hidden_bf16, const uint16_t* residual_bf16,
                                        const uint16_t* weight_bf16, uint16_t* norm_out_bf16,
                                        int rows, int hidden, float eps, void* stream) {
    if (!hidden_bf16 || !residual_bf16 || !weight_bf16 || !norm_out_bf16 || rows <= 0 ||
        hidden <= 0)
        return PIE_HIP_ERR_INVALID;
    if (hidden % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(rmsnorm_kernel<true>, dim3(rows), dim3(256), 0,
                       static_cast<hipStream_t>(stream), hidden_bf16, residual_bf16, weight_bf16,
                       norm_out_bf16, hidden, eps);
    return launch_status();
}

extern "C" int pie_hip_rope_table(const int32_t* positions, const float* inv_freq, float* table,
                                  int num_tokens, int head_dim, void* stream) {
    if (!positions || !inv_freq || !table || num_tokens <= 0 || head_dim <= 0)
        return PIE_HIP_ERR_INVALID;
    if (head_dim % 2 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(rope_table_kernel, dim3(num_tokens), dim3(64), 0,
                       static_cast<hipStream_t>(stream), positions, inv_freq, table, head_dim, 1.0f);
    return launch_status();
}

extern "C" int pie_hip_rope_table_scaled(const int32_t* positions, const float* inv_freq, float* table,
                                         int num_tokens, int head_dim, float mscale, void* stream) {
    if (!positions || !inv_freq || !table || num_tokens <= 0 || head_dim <= 0 || !(mscale > 0.f))
        return PIE_HIP_ERR_INVALID;
    if (head_dim % 2 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(rope_table_kernel, dim3(num_tokens), dim3(64), 0,
                       static_cast<hipStream_t>(stream), positions, inv_freq, table, head_dim, mscale);
    return launch_status();
}

extern "C" int pie_hip_qkv_rope_kvwrite(const uint16_t* packed_qkv, uint16_t* q_out,
                                        uint16_t* k_pages, uint16_t* v_pages,
                                        const uint16_t* q_norm_weight,
                                        const uint16_t* k_norm_weight, const float* rope_table,
                                        const int64_t* kv_slots, int num_tokens, int num_q_heads,
                                        int num_kv_heads, int head_dim, int interleaved, float eps,
                                        void* stream) {
    if (!packed_qkv || !q_out || !k_pages || !v_pages || !rope_table || !kv_slots ||
        num_tokens <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0)
        return PIE_HIP_ERR_INVALID;
    if (!q_norm_weight != !k_norm_weight) return PIE_HIP_ERR_INVALID;
    if (head_dim % 8 != 0 || num_q_heads + 2 * num_kv_heads > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(qkv_rope_kvwrite_kernel, dim3(num_tokens, num_q_heads + 2 * num_kv_heads),
                       dim3(64), 0, static_cast<hipStream_t>(stream), packed_qkv, q_out, k_pages,
                       v_pages, q_norm_weight, k_norm_weight, rope_table, kv_slots, num_q_heads,
                       num_kv_heads, head_dim, interleaved, eps);
    return launch_status();
}

extern "C" int pie_hip_swiglu(const uint16_t* gate_up_bf16, uint16_t* y_bf16, int num_tokens,
                              int intermediate, void* stream) {
    if (!gate_up_bf16 || !y_bf16 || num_tokens <= 0 || intermediate <= 0)
        return PIE_HIP_ERR_INVALID;
    if (intermediate % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    const size_t total = static_cast<size_t>(num_tokens) * (intermediate / 8);
    hipLaunchKernelGGL(swiglu_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256),
                       0, static_cast<hipStream_t>(stream), gate_up_bf16, y_bf16, intermediate,
                       total);
    return launch_status();
}

extern "C" int pie_hip_argmax(const uint16_t* logits_bf16, uint32_t* out_idx, int rows, int vocab,
                              void* stream) {
    if (!logits_bf16 || !out_idx || rows <= 0 || vocab <= 0) return PIE_HIP_ERR_INVALID;
    if (vocab % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;  // keeps every row 16-byte aligned
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       logits_bf16, out_idx, vocab);
    return launch_status();
}

extern "C" int pie_hip_copy_kv_pages(void* pool, const uint32_t* src_pages,
                                     const uint32_t* dst_pages, int num_copies, size_t page_bytes,
                                     void* stream) {
    if (!pool || !src_pages || !dst_pages || num_copies < 0 || page_bytes == 0)
        return PIE_HIP_ERR_INVALID;
    if (num_copies == 0) return PIE_HIP_OK;
    if (page_bytes % 16 != 0 || num_copies > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    const size_t page_vec = page_bytes / 16;
    unsigned gx = static_cast<unsigned>((page_vec + 255) / 256);
    if (gx > 64) gx = 64;
    hipLaunchKernelGGL(copy_pages_kernel, dim3(gx, num_copies), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<u32x4_t*>(pool), src_pages,
                       dst_pages, page_vec);
    return launch_status();
}
