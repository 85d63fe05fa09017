// Tiled weight-only GEMM on the matrix cores for prefill and large batches (gfx950):
//   y[M, N] = epilogue( act[M, K] · W[N, K]^T ),  W in int4b8 / int8 / fp8-e4m3 / bf16.
//
// The compute-bound sibling of the weight-streaming GEMV and the skinny GEMM: the role of the
// reference's large-M paths — dequantise to bf16 then a bf16 tensor-core GEMM
// (driver/cuda/src/ops/gemm.cpp:1213-1236, :1257-1264 for fp8) and Marlin for W4A16
// (driver/cuda/third_party/marlin/marlin_wrapper.hpp:39-51).  Evaluation order: weights become
// bf16 while they are staged (int4: bf16((nibble-8) * group_scale), the exact value of
// dequant_wna16_int4b8_to_bf16, driver/cuda/src/kernels/dequant_wna16.cu:11-38; int8/fp8: the
// integer / e4m3 value itself, exact in bf16, with the row scale applied to the fp32 sum),
// bf16 x bf16 products, fp32 accumulation, one rounding at the end.
//
// Tiling: a 128 x 128 output tile per block of four waves, each wave a 64 x 64 quadrant held as
// 4 x 4 accumulators of v_mfma_f32_16x16x32_bf16; K advances 64 at a time through two LDS
// buffers (global loads of tile t+1 are in flight while tile t is multiplied; one barrier per
// step).  LDS rows are padded to 144 bytes so the 16 rows an operand read touches fall in
// distinct banks.  Activations are the MFMA A operand, weights the B operand: an accumulator
// lane holds one weight row n (column of y) for four consecutive activation rows, so row scales
// are per-lane scalars and the SwiGLU partner (gate_i, up_i interleaved) is the neighbouring lane.
#include "common.hip.h"

namespace pie_hip {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kThreads = 256;
constexpr int kVecPerRow = BK / 8;           // 16-byte vectors per tile row
constexpr int kRowStride = kVecPerRow + 1;   // padded
constexpr int kTileVecs = BM * kRowStride;   // per operand per buffer

struct GemmArgs {
    const uint16_t* act;
    const unsigned char* w;
    const unsigned char* scale;
    uint16_t* y;
    int M, N, K, g_shift, beta, swiglu, scale_is_bf16;
};

__device__ __forceinline__ uint32_t pack_trunc(float lo, float hi) {
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

// ---- weight staging: global -> registers (raw) -> bf16 vectors in LDS --------------------
// Every format hands each thread the raw bytes of 32 (int4/int8/fp8) or 32 (bf16: 4 x 8)
// weights of one tile row per K step.
struct GInt4 {
    static constexpr int kRawVecs = 1;   // 16 bytes = 32 nibbles of row t/2, k half t%2
    static constexpr bool kRowScale = false;
    static __device__ __forceinline__ void load(const GemmArgs& a, int n, int k0, int tid, u32x4_t* raw,
                                                float& gs) {
        const int half = tid & 1;
        const unsigned char* p = a.w + (static_cast<size_t>(n) * a.K + k0 + half * 32) / 2;
        raw[0] = *reinterpret_cast<const u32x4_t*>(p);
        const uint16_t* sc = reinterpret_cast<const uint16_t*>(a.scale);
        gs = bf16_bits_to_f32(sc[static_cast<size_t>(n) * (a.K >> a.g_shift) + ((k0 + half * 32) >> a.g_shift)]);
    }
    static __device__ __forceinline__ void store(u32x4_t* row, int tid, const u32x4_t* raw, float gs) {
        const int half = tid & 1;
        const float off = -136.f * gs;
        uint32_t k128 = 0x43004300u;
        asm volatile("" : "+v"(k128));
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint32_t v = raw[0][s];
            uint32_t pr[4];   // pr[j] = (128 + nib_j, 128 + nib_{j+4}) as bf16 pair
#pragma unroll
            for (int j = 0; j < 4; ++j) pr[j] = and_or(v >> (4 * j), 0x000F000Fu, k128);
            float f[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                f[j] = fmaf(bf16_lo(pr[j]), gs, off);       // exact: (nib - 8) * scale
                f[j + 4] = fmaf(bf16_hi(pr[j]), gs, off);
            }
            row[half * 4 + s] = u32x4_t{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]),
                                        pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
        }
    }
};
struct GFp8 {
    static constexpr int kRawVecs = 2;   // 32 bytes of row t/2, k half t%2
    static constexpr bool kRowScale = true;
    static __device__ __forceinline__ void load(const GemmArgs& a, int n, int k0, int tid, u32x4_t* raw,
                                                float&) {
        const unsigned char* p = a.w + static_cast<size_t>(n) * a.K + k0 + (tid & 1) * 32;
        raw[0] = *reinterpret_cast<const u32x4_t*>(p);
        raw[1] = *reinterpret_cast<const u32x4_t*>(p + 16);
    }
    static __device__ __forceinline__ uint32_t cv(uint32_t w, bool hi) {
        const f32x2_t f = hi ? __builtin_amdgcn_cvt_pk_f32_fp8(w, true) : __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
        return pack_trunc(f.x, f.y);
    }
    static __device__ __forceinline__ void store(u32x4_t* row, int tid, const u32x4_t* raw, float) {
        const int half = tid & 1;
#pragma unroll
        for (int v = 0; v < 2; ++v)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t a = raw[v][2 * s], b = raw[v][2 * s + 1];
                row[half * 4 + v * 2 + s] = u32x4_t{cv(a, false), cv(a, true), cv(b, false), cv(b, true)};
            }
    }
};
struct GInt8 {
    static constexpr int kRawVecs = 2;
    static constexpr bool kRowScale = true;
    static __device__ __forceinline__ void load(const GemmArgs& a, int n, int k0, int tid, u32x4_t* raw,
                                                float& gs) {
        GFp8::load(a, n, k0, tid, raw, gs);
    }
    static __device__ __forceinline__ uint32_t two(uint32_t u, int sh) {
        // signed bytes -> exact bf16 pair: (byte ^ 0x80) - 128
        const float lo = static_cast<float>((u >> sh) & 0xFFu) - 128.f;
        const float hi = static_cast<float>((u >> (sh + 8)) & 0xFFu) - 128.f;
        return pack_trunc(lo, hi);
    }
    static __device__ __forceinline__ void store(u32x4_t* row, int tid, const u32x4_t* raw, float) {
        const int half = tid & 1;
#pragma unroll
        for (int v = 0; v < 2; ++v)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t a = raw[v][2 * s] ^ 0x80808080u, b = raw[v][2 * s + 1] ^ 0x80808080u;
                row[half * 4 + v * 2 + s] = u32x4_t{two(a, 0), two(a, 16), two(b, 0), two(b, 16)};
            }
    }
};
struct GBf16 {
    static constexpr int kRawVecs = 4;   // 64 bytes of row t/2, k half t%2
    static constexpr bool kRowScale = false;
    static __device__ __forceinline__ void load(const GemmArgs& a, int n, int k0, int tid, u32x4_t* raw,
                                                float&) {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(a.w) + static_cast<size_t>(n) * a.K + k0 + (tid & 1) * 32;
#pragma unroll
        for (int v = 0; v < 4; ++v) raw[v] = *reinterpret_cast<const u32x4_t*>(p + 8 * v);
    }
    static __device__ __forceinline__ void store(u32x4_t* row, int tid, const u32x4_t* raw, float) {
        const int half = tid & 1;
#pragma unroll
        for (int v = 0; v < 4; ++v) row[half * 4 + v] = raw[v];
    }
};

template <class F>
__global__ __launch_bounds__(kThreads) void gemm_mfma_kernel(const GemmArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    u32x4_t* lds = reinterpret_cast<u32x4_t*>(smem);   // [2 buffers][A tile | B tile]
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int j = lane & 15, q = lane >> 4;
    const int wm = wv >> 1, wn = wv & 1;
    const int M = a.M, N = a.N, K = a.K;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;

    // staging roles: activations — 4 vectors per thread (row tid/8 + 32u, vector tid%8);
    // weights — the 32 k-values (tid%2) of tile row tid/2
    const int arow = tid >> 3, avec = tid & 7;
    const uint16_t* aptr[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        aptr[u] = a.act + static_cast<size_t>(min(m0 + arow + 32 * u, M - 1)) * K + avec * 8;
    const int wrow = tid >> 1;
    const int wn_glob = min(n0 + wrow, N - 1);

    f32x4_t acc[4][4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t areg[4], wreg[F::kRawVecs];
    float gs = 1.f;
    auto gload = [&](int k0) {
#pragma unroll
        for (int u = 0; u < 4; ++u) areg[u] = *reinterpret_cast<const u32x4_t*>(aptr[u] + k0);
        F::load(a, wn_glob, k0, tid, wreg, gs);
    };
    auto lstore = [&](int buf) {
        u32x4_t* A = lds + buf * 2 * kTileVecs;
        u32x4_t* B = A + kTileVecs;
#pragma unroll
        for (int u = 0; u < 4; ++u) A[(arow + 32 * u) * kRowStride + avec] = areg[u];
        F::store(B + wrow * kRowStride, tid, wreg, gs);
    };

    const int nk = K / BK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        gload(min(kt + 1, nk - 1) * BK);   // next tile travels while this one is multiplied
        const u32x4_t* A = lds + buf * 2 * kTileVecs + (wm * 64 + j) * kRowStride + q;
        const u32x4_t* B = lds + buf * 2 * kTileVecs + kTileVecs + (wn * 64 + j) * kRowStride + q;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            bf16x8_t af[4], bfr[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                af[t] = __builtin_bit_cast(bf16x8_t, A[t * 16 * kRowStride + ks * 4]);
                bfr[t] = __builtin_bit_cast(bf16x8_t, B[t * 16 * kRowStride + ks * 4]);
            }
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int nt = 0; nt < 4; ++nt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt], bfr[nt], acc[mt][nt], 0, 0, 0);
        }
        lstore(buf ^ 1);   // the other buffer was released by the barrier of the previous step
        __syncthreads();
    }

    // ---- epilogue: lane holds column n for rows 4q + r of each 16 x 16 tile ----
    const int nout = a.swiglu ? N / 2 : N;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
        const int n = n0 + wn * 64 + nt * 16 + j;
        float rs = 1.f;
        if (F::kRowScale) {
            const int nc = min(n, N - 1);
            rs = a.scale_is_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(a.scale)[nc])
                                 : reinterpret_cast<const float*>(a.scale)[nc];
        }
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wm * 64 + mt * 16 + 4 * q + r;
                float v = acc[mt][nt][r] * rs;
                const bool ok = m < M && n < N;
                if (a.swiglu) {
                    const float gb = bf16_bits_to_f32(f32_to_bf16_bits(v));
                    const float other = __int_as_float(__builtin_amdgcn_update_dpp(
                        0, __float_as_int(gb), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
                    if ((j & 1) == 0 && ok) {
                        const float silu = gb / (1.f + expf(-gb));
                        a.y[static_cast<size_t>(m) * nout + n / 2] = f32_to_bf16_bits(silu * other);
                    }
                } else if (ok) {
                    const size_t o = static_cast<size_t>(m) * nout + n;
                    if (a.beta) v += bf16_bits_to_f32(a.y[o]);
                    a.y[o] = f32_to_bf16_bits(v);
                }
            }
    }
}

template <class F>
int launch_gemm(const GemmArgs& a, hipStream_t stream) {
    constexpr size_t smem = static_cast<size_t>(2) * 2 * kTileVecs * sizeof(u32x4_t);
    static const hipError_t attr =
        hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mfma_kernel<F>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (attr != hipSuccess) return PIE_HIP_ERR_LAUNCH;
    const dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM);
    if (grid.y > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(gemm_mfma_kernel<F>, grid, dim3(kThreads), smem, stream, a);
    return launch_status();
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_gemm_mfma(int format, const uint16_t* act_bf16, const void* weight,
                                 const void* scale, int scale_is_bf16, int group_size,
                                 uint16_t* y_bf16, int M, int N, int K, int beta, int swiglu,
                                 void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !weight || !y_bf16 || M <= 0 || N <= 0 || K <= 0) return PIE_HIP_ERR_INVALID;
    if (format != PIE_HIP_FMT_BF16 && !scale) return PIE_HIP_ERR_INVALID;
    if (K % BK != 0) return PIE_HIP_ERR_UNSUPPORTED;
    if (swiglu && (N % 2 != 0 || beta)) return PIE_HIP_ERR_INVALID;
    GemmArgs a{};
    a.act = act_bf16;
    a.w = static_cast<const unsigned char*>(weight);
    a.scale = static_cast<const unsigned char*>(scale);
    a.y = y_bf16;
    a.M = M;
    a.N = N;
    a.K = K;
    a.beta = beta;
    a.swiglu = swiglu ? 1 : 0;
    a.scale_is_bf16 = scale_is_bf16;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (format) {
        case PIE_HIP_FMT_INT4B8:
            // a 32-value run of one row must lie inside one scale group
            if (group_size < 32 || (group_size & (group_size - 1)) != 0 || K % group_size != 0)
                return PIE_HIP_ERR_UNSUPPORTED;
            a.g_shift = __builtin_ctz(static_cast<unsigned>(group_size));
            return launch_gemm<GInt4>(a, st);
        case PIE_HIP_FMT_INT8: return launch_gemm<GInt8>(a, st);
        case PIE_HIP_FMT_FP8: return launch_gemm<GFp8>(a, st);
        case PIE_HIP_FMT_BF16: return launch_gemm<GBf16>(a, st);
        default: return PIE_HIP_ERR_INVALID;
    }
}
