// Shared device helpers for the gfx950 kernels: bf16 bit handling, wave64
// reductions, status codes. Everything here is wave64 / CDNA4 specific.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pie_hip_kernels.h"

namespace pie_hip {

constexpr int kWave = 64;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// bf16 stored as raw uint16_t in memory.
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }

// Round-to-nearest-even f32 -> bf16 bits (NaN stays NaN). The compiler lowers
// the __bf16 cast to the native gfx950 conversion instruction.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    // one v_cvt_pk_bf16_f32 (round to nearest even, as the scalar conversion)
    typedef __bf16 bf16x2_pk_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_pk_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_pk_t{lo, hi}, bf16x2_pk_t));
}

// acc += a.lo*b.lo + a.hi*b.hi with bf16 inputs and an fp32 accumulator.
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), acc, false);
}

// (a & mask) | bits in one VALU op.  On gfx9-family encodings a three-source VALU op may
// read one scalar operand and no literal, so the mask rides in an SGPR and `bits` in a VGPR;
// written as asm because the compiler otherwise splits it into v_and + v_or.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask_sgpr, uint32_t bits_vgpr) {
    uint32_t d;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask_sgpr), "v"(bits_vgpr));
    return d;
}

template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ float dpp_add_f32(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, BANK_MASK, true);
    return v + __int_as_float(t);
}

// Wave64 sum on the DPP network (no LDS traffic): butterflies inside each row of 16 lanes,
// then the two row-broadcast steps; lane 63 holds the total, which readlane makes uniform.
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v = dpp_add_f32<0xB1>(v);             // quad_perm [1,0,3,2]
    v = dpp_add_f32<0x4E>(v);             // quad_perm [2,3,0,1]
    v = dpp_add_f32<0x141>(v);            // row_half_mirror
    v = dpp_add_f32<0x140>(v);            // row_mirror: every lane holds its row's sum
    v = dpp_add_f32<0x142, 0xA, 0xF>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add_f32<0x143, 0xC, 0xF>(v);  // row_bcast:31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

template <int CTRL>
__device__ __forceinline__ float dpp_mov_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Wave64 sums of NV (2 or 4) values at once: lane i < NV ends with the total of v[i] (every
// lane ends with the total of value `lane' & (NV - 1)`, lane' = lane with its low two bits
// flipped in odd quads).  The first log2(NV) butterfly steps halve the number of values a lane
// carries instead of adding NV separate butterflies: each lane keeps the values whose index
// bit matches its lane bit and sends the others to its partner.  Odd quads use the mirrored
// assignment so that the two mirror steps (lane ^ 7, lane ^ 15) pair lanes that carry the same
// value; rows are folded with the 16- and 32-lane swaps.  Every value is added over the same
// tree as wave_sum_dpp uses, so the totals are bit-identical to NV separate wave_sum_dpp calls.
template <int NV>
__device__ __forceinline__ float wave_sum_multi(const float* v, int lane) {
    static_assert(NV == 2 || NV == 4, "two or four values");
    const int lp = (lane & 4) ? lane ^ 3 : lane;
    const bool b0 = lp & 1;
    float x;
    if (NV == 4) {
        const float a = (b0 ? v[1] : v[0]) + dpp_mov_f32<0xB1>(b0 ? v[0] : v[1]);   // lane ^ 1
        const float b = (b0 ? v[3] : v[2]) + dpp_mov_f32<0xB1>(b0 ? v[2] : v[3]);
        const bool b1 = lp & 2;
        x = (b1 ? b : a) + dpp_mov_f32<0x4E>(b1 ? a : b);                           // lane ^ 2
    } else {
        x = (b0 ? v[1] : v[0]) + dpp_mov_f32<0xB1>(b0 ? v[0] : v[1]);
        x = dpp_add_f32<0x4E>(x);
    }
    x = dpp_add_f32<0x141>(x);   // row_half_mirror (lane ^ 7)
    x = dpp_add_f32<0x140>(x);   // row_mirror (lane ^ 15)
    const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);   // rows 0+1, 2+3
    const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r32[0]) + __uint_as_float(r32[1]);
}

// max over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one value per 16-lane row) with the row
// swaps instead of two LDS permutes: exact, so identical to the shuffle form
__device__ __forceinline__ float rows_max(float x) {
    const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r16[0]), __uint_as_float(r16[1]));
    const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r32[0]), __uint_as_float(r32[1]));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Decode attention splits a row's keys in units of this many tokens (the partial results of the
// splits are merged by attn_decode_merge_kernel or by the output projection's prologue).
constexpr int kAttnUnitTokens = 16;

// A query row's KV extent comes either from the wire arrays of a decode batch
// (kv_page_indptr / kv_last_page_lens) or, when `row_len` is given, from explicit per-row
// (first page-list entry, visible key count) pairs that a planner derived.
struct RowExtent {
    uint32_t pg_lo;
    int kv_len;
};
__device__ __forceinline__ RowExtent row_extent(const uint32_t* __restrict__ page_indptr,
                                                const uint32_t* __restrict__ last_lens,
                                                const uint32_t* __restrict__ row_begin,
                                                const int32_t* __restrict__ row_len, int r,
                                                int ps) {
    if (row_len) return {row_begin[r], row_len[r]};
    const uint32_t lo = page_indptr[r];
    const int npages = static_cast<int>(page_indptr[r + 1] - lo);
    return {lo, npages > 0 ? (npages - 1) * ps + static_cast<int>(last_lens[r]) : 0};
}

// KV storage of the pool (driver/cuda/src/kv_cache_format.hpp:11-17): bf16; one-byte e4m3 with
// optional fp32 scales per (token, kv head) — "fp8_e4m3" stores casts, "fp8_per_token_head"
// stores x / scale; int8 with such scales; one-byte e5m2 casts ("fp8_e5m2").  A lane still owns 8 elements of a row: 16 bytes of
// bf16 or 8 bytes of a one-byte format.  Values are decoded as the reference's load_kv_scalar
// does (driver/cuda/src/ops/attention_naive_paged.cu:56-112): float(code) * scale.
constexpr int kKvBf16 = 0, kKvFp8 = 1, kKvInt8 = 2, kKvBf8 = 3;   // (kKvBf8: e5m2 casts, "fp8_e5m2")

// Scale pools are laid out [pages, kv heads, page_size]: the scales a (page, head) block of an
// attention launch reads are contiguous (64 bytes for 16 tokens), where [pages, page_size,
// kv heads] spread them over one 32-byte sector per token that every head's block fetches
// again.  A page's scales stay one contiguous run, so page copies move them like the codes.
__device__ __forceinline__ size_t kv_scale_index(size_t page, int in_page, int head, int hk, int ps) {
    return (page * hk + head) * ps + in_page;
}
__device__ __forceinline__ size_t kv_scale_index_of_slot(int64_t slot, int head, int hk, int ps) {
    const uint64_t page = static_cast<uint64_t>(slot) < 0x80000000ull
                              ? static_cast<uint32_t>(slot) / static_cast<uint32_t>(ps)
                              : static_cast<uint64_t>(slot) / static_cast<uint32_t>(ps);
    return kv_scale_index(page, static_cast<int>(static_cast<uint64_t>(slot) - page * ps), head, hk, ps);
}

template <int KVF>
struct KvVec {
    using type = u32x4_t;
};
template <>
struct KvVec<kKvFp8> {
    using type = u32x2_t;
};
template <>
struct KvVec<kKvInt8> {
    using type = u32x2_t;
};
template <>
struct KvVec<kKvBf8> {
    using type = u32x2_t;
};

__device__ __forceinline__ uint32_t kv_pack_trunc(float lo, float hi) {
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}
// 8 stored elements -> 8 floats / 4 bf16 pairs (every code is exact in bf16)
template <int KVF>
__device__ __forceinline__ void kv_decode_f32(const typename KvVec<KVF>::type r, float* f) {
    if constexpr (KVF == kKvBf16) {
        f[0] = bf16_lo(r.x); f[1] = bf16_hi(r.x); f[2] = bf16_lo(r.y); f[3] = bf16_hi(r.y);
        f[4] = bf16_lo(r.z); f[5] = bf16_hi(r.z); f[6] = bf16_lo(r.w); f[7] = bf16_hi(r.w);
    } else if constexpr (KVF == kKvFp8) {
        typedef float f32x2_t __attribute__((ext_vector_type(2)));
        const f32x2_t a = __builtin_amdgcn_cvt_pk_f32_fp8(r.x, false), b = __builtin_amdgcn_cvt_pk_f32_fp8(r.x, true);
        const f32x2_t c = __builtin_amdgcn_cvt_pk_f32_fp8(r.y, false), d = __builtin_amdgcn_cvt_pk_f32_fp8(r.y, true);
        f[0] = a.x; f[1] = a.y; f[2] = b.x; f[3] = b.y; f[4] = c.x; f[5] = c.y; f[6] = d.x; f[7] = d.y;
    } else if constexpr (KVF == kKvBf8) {
        typedef float f32x2_t __attribute__((ext_vector_type(2)));
        const f32x2_t a = __builtin_amdgcn_cvt_pk_f32_bf8(r.x, false), b = __builtin_amdgcn_cvt_pk_f32_bf8(r.x, true);
        const f32x2_t c = __builtin_amdgcn_cvt_pk_f32_bf8(r.y, false), d = __builtin_amdgcn_cvt_pk_f32_bf8(r.y, true);
        f[0] = a.x; f[1] = a.y; f[2] = b.x; f[3] = b.y; f[4] = c.x; f[5] = c.y; f[6] = d.x; f[7] = d.y;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            f[e] = static_cast<float>(static_cast<int8_t>(r.x >> (8 * e)));
            f[4 + e] = static_cast<float>(static_cast<int8_t>(r.y >> (8 * e)));
        }
    }
}
template <int KVF>
__device__ __forceinline__ u32x4_t kv_decode_bf16(const typename KvVec<KVF>::type r) {
    if constexpr (KVF == kKvBf16) {
        return r;
    } else if constexpr (KVF == kKvFp8 || KVF == kKvBf8) {
        // two codes -> a bf16 pair in one instruction (scale 1: every code is exact in bf16)
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
#define PIE_KV_TWO(w, hi)                                                                                       \
    (KVF == kKvFp8 ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((w), 1.0f, (hi))) \
                   : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8((w), 1.0f, (hi))))
        return u32x4_t{PIE_KV_TWO(r.x, false), PIE_KV_TWO(r.x, true), PIE_KV_TWO(r.y, false), PIE_KV_TWO(r.y, true)};
#undef PIE_KV_TWO
    } else {
        float f[8];
        kv_decode_f32<KVF>(r, f);
        return u32x4_t{kv_pack_trunc(f[0], f[1]), kv_pack_trunc(f[2], f[3]), kv_pack_trunc(f[4], f[5]),
                       kv_pack_trunc(f[6], f[7])};
    }
}

// 8 stored elements of each of two rows -> the 8 pairs (bf16(a_e), bf16(b_e)), a_e in the low half
template <int KVF>
__device__ __forceinline__ void kv_decode_bf16_pairs(const typename KvVec<KVF>::type a,
                                                     const typename KvVec<KVF>::type b, uint32_t* out) {
    static_assert(KVF != kKvBf16, "one-byte formats only");
    if constexpr (KVF == kKvFp8 || KVF == kKvBf8) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            // bytes (a0, b0, a1, b1) and (a2, b2, a3, b3) of this word, then two codes per conversion
            const uint32_t m0 = __builtin_amdgcn_perm(b[w], a[w], 0x05010400u);
            const uint32_t m1 = __builtin_amdgcn_perm(b[w], a[w], 0x07030602u);
            if constexpr (KVF == kKvFp8) {
                out[4 * w + 0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(m0, 1.0f, false));
                out[4 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(m0, 1.0f, true));
                out[4 * w + 2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(m1, 1.0f, false));
                out[4 * w + 3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(m1, 1.0f, true));
            } else {
                out[4 * w + 0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(m0, 1.0f, false));
                out[4 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(m0, 1.0f, true));
                out[4 * w + 2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(m1, 1.0f, false));
                out[4 * w + 3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(m1, 1.0f, true));
            }
        }
    } else {
        float fa[8], fb[8];
        kv_decode_f32<KVF>(a, fa);
        kv_decode_f32<KVF>(b, fb);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = kv_pack_trunc(fa[e], fb[e]);
    }
}

inline int launch_status() {
    return hipGetLastError() == hipSuccess ? PIE_HIP_OK : PIE_HIP_ERR_LAUNCH;
}

}  // namespace pie_hip
