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


__device__ __forceinline__ float block_max_256(float v, float* smem) {
    v = wave_max(v);
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    if (lane == 0) smem[wv] = v;
    __syncthreads();
    const float m = fmaxf(fmaxf(smem[0], smem[1]), fmaxf(smem[2], smem[3]));
    __syncthreads();
    return m;
}

// One block per row: absmax, scale_inv = absmax/127 (1 for an all-zero row),
// q = clamp(rintf(w * (127/absmax)), -128, 127); rintf rounds half to even.
// Reference: quant_int8_per_channel_kernel, driver/cuda/src/kernels/quant_bf16_to_fp8.cu:273-323.
__global__ __launch_bounds__(256) void quant_int8_row_kernel(const uint16_t* __restrict__ w,
                                                             int8_t* __restrict__ q,
                                                             float* __restrict__ scale_inv,
                                                             int cols) {
    __shared__ float red[4];
    const size_t off = static_cast<size_t>(blockIdx.x) * cols;
    float local = 0.f;
    for (int j = threadIdx.x; j < cols; j += 256) local = fmaxf(local, fabsf(bf16_bits_to_f32(w[off + j])));
    const float row_max = block_max_256(local, red);
    const float inv = row_max > 0.f ? 127.f / row_max : 1.f;
    if (threadIdx.x == 0) scale_inv[blockIdx.x] = row_max > 0.f ? row_max / 127.f : 1.f;
    for (int j = threadIdx.x; j < cols; j += 256) {
        int v = static_cast<int>(rintf(bf16_bits_to_f32(w[off + j]) * inv));
        v = v > 127 ? 127 : (v < -128 ? -128 : v);
        q[off + j] = static_cast<int8_t>(v);
    }
}

// f32 -> OCP e4m3fn byte, round to nearest even, saturating at +-448 (the hardware
// conversion saturates when the clamp bit is set; inputs are pre-clamped here).
__device__ __forceinline__ uint8_t f32_to_e4m3(float f) {
    f = fminf(fmaxf(f, -448.f), 448.f);
    const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false);
    return static_cast<uint8_t>(packed & 0xFF);
}

// Reference: quant_per_channel_kernel, driver/cuda/src/kernels/quant_bf16_to_fp8.cu:181-226.
__global__ __launch_bounds__(256) void quant_fp8_row_kernel(const uint16_t* __restrict__ w,
                                                            uint8_t* __restrict__ q,
                                                            float* __restrict__ scale_inv,
                                                            int cols) {
    __shared__ float red[4];
    const size_t off = static_cast<size_t>(blockIdx.x) * cols;
    float local = 0.f;
    for (int j = threadIdx.x; j < cols; j += 256) local = fmaxf(local, fabsf(bf16_bits_to_f32(w[off + j])));
    const float row_max = block_max_256(local, red);
    const float inv = row_max > 0.f ? 448.f / row_max : 1.f;
    if (threadIdx.x == 0) scale_inv[blockIdx.x] = row_max > 0.f ? row_max / 448.f : 1.f;
    for (int j = threadIdx.x; j < cols; j += 256)
        q[off + j] = f32_to_e4m3(bf16_bits_to_f32(w[off + j]) * inv);
}

// Symmetric group-wise int4: one thread per (row, group): s = bf16(absmax/7) (1 for a zero
// group), nibble = clamp(rintf(w / s), -8, 7) + 8, packed 8 per u32, nibble j = element 8w+j
// (the int4b8 layout of driver/cuda/src/kernels/dequant_wna16.cu:11-38; the reference ships
// no bf16->int4 quantiser, so this rounding rule is this library's own).
__global__ void quant_int4b8_group_kernel(const uint16_t* __restrict__ w,
                                          uint32_t* __restrict__ packed,
                                          uint16_t* __restrict__ scale, int rows, int cols,
                                          int group) {
    const size_t gid = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    const int groups = cols / group;
    if (gid >= static_cast<size_t>(rows) * groups) return;
    const size_t row = gid / groups;
    const int g = static_cast<int>(gid - row * groups);
    const uint16_t* src = w + row * cols + static_cast<size_t>(g) * group;
    float absmax = 0.f;
    for (int j = 0; j < group; ++j) absmax = fmaxf(absmax, fabsf(bf16_bits_to_f32(src[j])));
    const uint16_t sb = absmax > 0.f ? f32_to_bf16_bits(absmax / 7.f) : 0x3F80;
    const float s = bf16_bits_to_f32(sb);
    scale[gid] = sb;
    uint32_t* dst = packed + row * (cols / 8) + static_cast<size_t>(g) * (group / 8);
    for (int wd = 0; wd < group / 8; ++wd) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            int v = static_cast<int>(rintf(bf16_bits_to_f32(src[wd * 8 + j]) / s));
            v = v > 7 ? 7 : (v < -8 ? -8 : v);
            word |= static_cast<uint32_t>(v + 8) << (4 * j);
        }
        dst[wd] = word;
    }
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_abi_version(void) { return PIE_HIP_ABI_VERSION; }

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

extern "C" int pie_hip_quant_int8_per_channel(const uint16_t* w_bf16, int8_t* q,
                                              float* scale_inv, int rows, int cols,
                                              void* stream) {
    if (!w_bf16 || !q || !scale_inv || rows <= 0 || cols <= 0) return PIE_HIP_ERR_INVALID;
    hipLaunchKernelGGL(pie_hip::quant_int8_row_kernel, dim3(rows), dim3(256), 0,
                       static_cast<hipStream_t>(stream), w_bf16, q, scale_inv, cols);
    return pie_hip::launch_status();
}

extern "C" int pie_hip_quant_fp8_per_channel(const uint16_t* w_bf16, uint8_t* q_e4m3,
                                             float* scale_inv, int rows, int cols,
                                             void* stream) {
    if (!w_bf16 || !q_e4m3 || !scale_inv || rows <= 0 || cols <= 0) return PIE_HIP_ERR_INVALID;
    hipLaunchKernelGGL(pie_hip::quant_fp8_row_kernel, dim3(rows), dim3(256), 0,
                       static_cast<hipStream_t>(stream), w_bf16, q_e4m3, scale_inv, cols);
    return pie_hip::launch_status();
}

extern "C" int pie_hip_quant_int4b8_group(const uint16_t* w_bf16, uint32_t* packed,
                                          uint16_t* scale_bf16, int rows, int cols,
                                          int group_size, void* stream) {
    if (!w_bf16 || !packed || !scale_bf16 || rows <= 0 || cols <= 0 || group_size <= 0)
        return PIE_HIP_ERR_INVALID;
    if (group_size % 8 != 0 || cols % group_size != 0) return PIE_HIP_ERR_UNSUPPORTED;
    const size_t n = static_cast<size_t>(rows) * (cols / group_size);
    hipLaunchKernelGGL(pie_hip::quant_int4b8_group_kernel,
                       dim3(static_cast<unsigned>((n + 127) / 128)), dim3(128), 0,
                       static_cast<hipStream_t>(stream), w_bf16, packed, scale_bf16, rows, cols,
                       group_size);
    return pie_hip::launch_status();
}
