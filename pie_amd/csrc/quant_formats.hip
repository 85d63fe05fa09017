// Weight-format kernels: integer unpack and dequantisation of the quantised
// layouts the forward pass consumes.  These are cold (load-time / test) kernels;
// they exist so that the integer side of every format has a bit-exact device
// statement that tests can compare with the CPU oracle.
#include "common.hip.h"

namespace pie_hip {
namespace {

// One thread per packed word: 8 int8 outputs, written as one 8-byte store.
// Reference nibble order: driver/cuda/src/kernels/dequant_wna16.cu:31-36.
__global__ void unpack_w4_kernel(const uint32_t* __restrict__ packed, int8_t* __restrict__ q,
                                 size_t nwords) {
    const size_t w = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (w >= nwords) return;
    const uint32_t word = packed[w];
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        lo |= static_cast<uint32_t>(static_cast<uint8_t>(static_cast<int>((word >> (4 * j)) & 0xF) - 8)) << (8 * j);
        hi |= static_cast<uint32_t>(static_cast<uint8_t>(static_cast<int>((word >> (4 * (j + 4))) & 0xF) - 8)) << (8 * j);
    }
    reinterpret_cast<u32x2_t*>(q)[w] = u32x2_t{lo, hi};
}

// Reference: dequant_wna16_int4b8_kernel, driver/cuda/src/kernels/dequant_wna16.cu:11-38.
__global__ void dequant_w4a16_kernel(const uint32_t* __restrict__ packed,
                                     const uint16_t* __restrict__ scale,
                                     uint16_t* __restrict__ out, int out_dim, int in_dim,
                                     int group) {
    const int words_per_row = in_dim / 8;
    const size_t w = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (w >= static_cast<size_t>(out_dim) * words_per_row) return;
    const int row = static_cast<int>(w / words_per_row);
    const int wc = static_cast<int>(w - static_cast<size_t>(row) * words_per_row);
    const uint32_t word = packed[w];
    const uint16_t* rs = scale + static_cast<size_t>(row) * (in_dim / group);
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int k0 = wc * 8 + 2 * j;
        const float q0 = static_cast<float>(static_cast<int>((word >> (8 * j)) & 0xF) - 8);
        const float q1 = static_cast<float>(static_cast<int>((word >> (8 * j + 4)) & 0xF) - 8);
        o[j] = pack_bf16x2(q0 * bf16_bits_to_f32(rs[k0 / group]),
                           q1 * bf16_bits_to_f32(rs[(k0 + 1) / group]));
    }
    reinterpret_cast<u32x4_t*>(out)[w] = o;
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_abi_version(void) { return 1; }

extern "C" int pie_hip_unpack_w4(const uint32_t* packed, int8_t* q, int out_dim, int in_dim,
                                 void* stream) {
    if (!packed || !q || out_dim <= 0 || in_dim <= 0) return PIE_HIP_ERR_INVALID;
    if (in_dim % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    const size_t nwords = static_cast<size_t>(out_dim) * (in_dim / 8);
    const int block = 256;
    const unsigned grid = static_cast<unsigned>((nwords + block - 1) / block);
    hipLaunchKernelGGL(pie_hip::unpack_w4_kernel, dim3(grid), dim3(block), 0,
                       static_cast<hipStream_t>(stream), packed, q, nwords);
    return pie_hip::launch_status();
}

extern "C" int pie_hip_dequant_w4a16(const uint32_t* packed, const uint16_t* scale_bf16,
                                     uint16_t* out_bf16, int out_dim, int in_dim,
                                     int group_size, void* stream) {
    if (!packed || !scale_bf16 || !out_bf16 || out_dim <= 0 || in_dim <= 0 || group_size <= 0)
        return PIE_HIP_ERR_INVALID;
    if (in_dim % 8 != 0 || in_dim % group_size != 0) return PIE_HIP_ERR_UNSUPPORTED;
    const size_t nwords = static_cast<size_t>(out_dim) * (in_dim / 8);
    const int block = 256;
    const unsigned grid = static_cast<unsigned>((nwords + block - 1) / block);
    hipLaunchKernelGGL(pie_hip::dequant_w4a16_kernel, dim3(grid), dim3(block), 0,
                       static_cast<hipStream_t>(stream), packed, scale_bf16, out_bf16, out_dim,
                       in_dim, group_size);
    return pie_hip::launch_status();
}
