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
    return static_cast<uint32_t>(f32_to_bf16_bits(lo)) |
           (static_cast<uint32_t>(f32_to_bf16_bits(hi)) << 16);
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

inline int launch_status() {
    return hipGetLastError() == hipSuccess ? PIE_HIP_OK : PIE_HIP_ERR_LAUNCH;
}

}  // namespace pie_hip
