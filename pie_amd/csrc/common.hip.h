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
