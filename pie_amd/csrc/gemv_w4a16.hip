// Weight-only int4 (W4A16, "int4b8") GEMV / skinny GEMM for decode on gfx950.
//
// Contract: driver/cuda/src/kernels/dequant_wna16.cu:11-38 (format) and :96-110
// (fused decode dot product) of the reference; replaces its Marlin call for
// small M (driver/cuda/third_party/marlin/marlin_wrapper.hpp:39-51).
//
// HBM-bound design (N*K/2 weight bytes dominate):
//   * the grid is sized to the machine, not to the problem: `waves_per_simd`
//     resident waves on each of the 1024 SIMDs, every wave owning one contiguous,
//     balanced slice of the output rows, so all CUs start and finish together;
//   * a wave walks its slice R rows at a time; every lane streams 16-byte
//     (32-weight) pieces of each row, so one wave instruction covers 1 KiB of a
//     row, fully coalesced.  Loads are branch-free and issued one work unit
//     (R rows x 2048 columns) ahead of the arithmetic, so 2R independent 16 B
//     loads per lane are in flight while the previous unit is being reduced;
//   * the first unit is requested before the activation row is staged, so the
//     HBM latency of the weights overlaps the LDS staging;
//   * the activation row is staged once per block into LDS, already permuted
//     into the (k, k+4) bf16 pairs that one `v_and_or_b32` produces from a packed
//     word, laid out so a lane's four 16 B LDS reads are conflict free;
//   * nibbles become bf16 by OR-ing the exponent of 128.0 onto them
//     ((w >> 4j) & 0x000F000F) | 0x43004300 = (128+n_j, 128+n_{j+4}); the dot
//     product runs on v_dot2_f32_bf16 with an fp32 accumulator that starts at
//     -136 * sum(x) so the result is sum x*(n-8) exactly as the format defines;
//   * the bf16 group scale multiplies each lane's 32-weight partial sum (a lane
//     never straddles a group because G % 32 == 0);
//   * a wave64 butterfly finishes the row.
#include "common.hip.h"

namespace pie_hip {
namespace {

constexpr int kBlock = 256;  // 4 waves: one per SIMD of a CU
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kChunkK = kWave * 32;  // weights covered by one wave-wide 16 B load
constexpr int kNumCU = 256;

constexpr uint32_t kNibblePairMask = 0x000F000Fu;
constexpr uint32_t kBf16x2_128 = 0x43004300u;  // (128.0bf16, 128.0bf16)

template <int R>
struct Unit {
    u32x4_t w[R];
    uint16_t s[R];
    uint16_t prev;  // y value this lane may add to (lane = r*M + m), for beta = 1
};

template <int R, int M>
__global__ __launch_bounds__(kBlock) void gemv_w4a16_kernel(
    const uint16_t* __restrict__ act, const u32x4_t* __restrict__ packed,
    const uint16_t* __restrict__ scale, uint16_t* __restrict__ y, int N, int K, int G,
    int beta) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform -> SGPR
    const int nchunks = (K + kChunkK - 1) / kChunkK;
    const int nwords = K / 8;
    const int padded_words = nchunks * 256;
    const int row_stride_v4 = K / 32;
    const int groups_per_row = K / G;

    u32x4_t* lds_x = reinterpret_cast<u32x4_t*>(smem);                   // [M][nchunks*4*64]
    float* lds_sx = reinterpret_cast<float*>(lds_x + M * padded_words);  // [M][nchunks*64]

    // Balanced contiguous row slice of this wave.
    const long long total_waves = static_cast<long long>(gridDim.x) * kWavesPerBlock;
    const long long wg = static_cast<long long>(blockIdx.x) * kWavesPerBlock + wv;
    const int row_begin = static_cast<int>(wg * N / total_waves);
    const int row_end = static_cast<int>((wg + 1) * N / total_waves);
    const int ngroups = (row_end - row_begin + R - 1) / R;
    const int nunits = ngroups * nchunks;

    // Branch-free loads: lanes past K re-read lane 0's piece and are masked by a zero scale;
    // rows past the slice re-read its last row and are dropped at the store.
    auto issue = [&](Unit<R>& u, int g, int c) {
        const int kbase = c * kChunkK + lane * 32;
        const bool valid = kbase < K;
        const int piece = valid ? c * kWave + lane : 0;
        const int sgrp = valid ? kbase / G : 0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = min(row_begin + g * R + r, row_end - 1);
            u.w[r] = __builtin_nontemporal_load(packed + static_cast<size_t>(row) * row_stride_v4 +
                                                piece);
            u.s[r] = scale[static_cast<size_t>(row) * groups_per_row + sgrp];
        }
        // Every unit prefetches the output element its lane would finish, so the residual
        // add never stalls the pipeline (only the last chunk's value is used).
        const int lr = lane < R * M ? lane / M : 0;
        const int lm = lane < R * M ? lane % M : 0;
        u.prev = y[static_cast<size_t>(lm) * N + min(row_begin + g * R + lr, row_end - 1)];
    };

    Unit<R> ua, ub;
    if (nunits > 0) issue(ua, 0, 0);

    // Stage activations: word w (8 consecutive k) -> pairs (0,4)(1,5)(2,6)(3,7).
    for (int w = tid; w < M * padded_words; w += kBlock) {
        const int m = w / padded_words;
        const int wi = w - m * padded_words;
        u32x4_t p = {0u, 0u, 0u, 0u};
        if (wi < nwords) {
            const u32x4_t v =
                *reinterpret_cast<const u32x4_t*>(act + static_cast<size_t>(m) * K + wi * 8);
            p.x = (v.x & 0xFFFFu) | (v.z << 16);
            p.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
            p.z = (v.y & 0xFFFFu) | (v.w << 16);
            p.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
        }
        const int c = wi >> 8;
        const int l = (wi & 255) >> 2;
        const int i = wi & 3;
        lds_x[m * padded_words + (c * 4 + i) * kWave + l] = p;
    }
    __syncthreads();
    // Per-(chunk, lane) sum of the 32 activations the lane will multiply.
    for (int j = tid; j < M * nchunks * kWave; j += kBlock) {
        const int m = j / (nchunks * kWave);
        const int cl = j - m * (nchunks * kWave);
        const int c = cl / kWave;
        const int l = cl - c * kWave;
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32x4_t p = lds_x[m * padded_words + (c * 4 + i) * kWave + l];
            s += bf16_lo(p.x) + bf16_hi(p.x) + bf16_lo(p.y) + bf16_hi(p.y) + bf16_lo(p.z) +
                 bf16_hi(p.z) + bf16_lo(p.w) + bf16_hi(p.w);
        }
        lds_sx[j] = s;
    }
    __syncthreads();

    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.f;

    auto compute = [&](const Unit<R>& u, int g, int c) {
        const bool valid = c * kChunkK + lane * 32 < K;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            uint32_t wu[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = u.w[r][i];
                wu[4 * i + 0] = (w & kNibblePairMask) | kBf16x2_128;
                wu[4 * i + 1] = ((w >> 4) & kNibblePairMask) | kBf16x2_128;
                wu[4 * i + 2] = ((w >> 8) & kNibblePairMask) | kBf16x2_128;
                wu[4 * i + 3] = ((w >> 12) & kNibblePairMask) | kBf16x2_128;
            }
            const float s = valid ? bf16_bits_to_f32(u.s[r]) : 0.f;
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float p = -136.f * lds_sx[(m * nchunks + c) * kWave + lane];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32x4_t xv = lds_x[m * padded_words + (c * 4 + i) * kWave + lane];
                    p = dot2_bf16(xv.x, wu[4 * i + 0], p);
                    p = dot2_bf16(xv.y, wu[4 * i + 1], p);
                    p = dot2_bf16(xv.z, wu[4 * i + 2], p);
                    p = dot2_bf16(xv.w, wu[4 * i + 3], p);
                }
                acc[r][m] = fmaf(s, p, acc[r][m]);
            }
        }
        if (c == nchunks - 1) {
            float mine = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const float v = wave_sum(acc[r][m]);
                    acc[r][m] = 0.f;
                    if (lane == r * M + m) mine = v;
                }
            }
            const int row = row_begin + g * R + lane / M;
            if (lane < R * M && row < row_end) {
                const float prev = beta ? bf16_bits_to_f32(u.prev) : 0.f;
                y[static_cast<size_t>(lane % M) * N + row] = f32_to_bf16_bits(mine + prev);
            }
        }
    };

    // Two-deep software pipeline over (row group, chunk) units.  Loads are issued
    // unconditionally (past the end they re-request the last unit) so the wait
    // before each compute only covers the unit it consumes.
    const int last_g = ngroups - 1, last_c = nchunks - 1;
    auto advance = [&](int& gg, int& cc) {
        if (gg == last_g && cc == last_c) return;
        if (++cc == nchunks) { cc = 0; ++gg; }
    };
    int g = 0, c = 0;  // coordinates of the unit held in `ua`
    for (int u = 0; u < nunits; u += 2) {
        int g1 = g, c1 = c;
        advance(g1, c1);
        int g2 = g1, c2 = c1;
        advance(g2, c2);
        issue(ub, g1, c1);
        compute(ua, g, c);
        issue(ua, g2, c2);
        if (u + 1 < nunits) compute(ub, g1, c1);
        g = g2;
        c = c2;
    }
}

template <int R, int M>
int launch(const uint16_t* act, const uint32_t* packed, const uint16_t* scale, uint16_t* y,
           int N, int K, int G, int beta, int waves_per_simd, hipStream_t stream) {
    const int nchunks = (K + kChunkK - 1) / kChunkK;
    const size_t smem = static_cast<size_t>(M) * nchunks * (256 * 16 + kWave * 4);
    if (smem > 64 * 1024) return PIE_HIP_ERR_UNSUPPORTED;
    int grid = kNumCU * waves_per_simd;
    const int max_grid = (N + kWavesPerBlock - 1) / kWavesPerBlock;  // >= 1 row per wave
    if (grid > max_grid) grid = max_grid;
    hipLaunchKernelGGL((gemv_w4a16_kernel<R, M>), dim3(grid), dim3(kBlock), smem, stream, act,
                       reinterpret_cast<const u32x4_t*>(packed), scale, y, N, K, G, beta);
    return launch_status();
}

template <int R>
int launch_m(int M, const uint16_t* act, const uint32_t* packed, const uint16_t* scale,
             uint16_t* y, int N, int K, int G, int beta, int wps, hipStream_t stream) {
    switch (M) {
        case 1: return launch<R, 1>(act, packed, scale, y, N, K, G, beta, wps, stream);
        case 2: return launch<R, 2>(act, packed, scale, y, N, K, G, beta, wps, stream);
        case 3: return launch<R, 3>(act, packed, scale, y, N, K, G, beta, wps, stream);
        case 4: return launch<R, 4>(act, packed, scale, y, N, K, G, beta, wps, stream);
        default: return PIE_HIP_ERR_UNSUPPORTED;
    }
}

}  // namespace

// rows_per_wave (R) in {1,2,3,4}; waves_per_simd in 1..8.  0 = pick.
int gemv_w4a16_dispatch(const uint16_t* act, const uint32_t* packed, const uint16_t* scale,
                        uint16_t* y, int M, int N, int K, int G, int beta, int rows_per_wave,
                        int waves_per_simd, hipStream_t stream) {
    if (!act || !packed || !scale || !y || M <= 0 || N <= 0 || K <= 0 || G <= 0)
        return PIE_HIP_ERR_INVALID;
    if (K % 32 != 0 || G % 32 != 0 || K % G != 0) return PIE_HIP_ERR_UNSUPPORTED;
    // Measured on MI355X: two resident waves per SIMD, each walking its slice four rows
    // at a time (fewer when the slice is shorter), is within a few percent of the best
    // (rows, waves) pair for every decode shape of an 8B-class model.
    if (waves_per_simd <= 0) waves_per_simd = 2;
    if (waves_per_simd > 8) return PIE_HIP_ERR_INVALID;
    if (rows_per_wave <= 0) {
        const long long per_wave =
            N / (static_cast<long long>(kNumCU) * kWavesPerBlock * waves_per_simd);
        rows_per_wave = per_wave >= 4 ? 4 : (per_wave >= 3 ? 3 : (per_wave >= 2 ? 2 : 1));
    }
    // M > 4 re-reads the weights per group of four activation rows.
    for (int m0 = 0; m0 < M; m0 += 4) {
        const int mm = (M - m0) < 4 ? (M - m0) : 4;
        const uint16_t* a = act + static_cast<size_t>(m0) * K;
        uint16_t* yo = y + static_cast<size_t>(m0) * N;
        int st;
        switch (rows_per_wave) {
            case 1: st = launch_m<1>(mm, a, packed, scale, yo, N, K, G, beta, waves_per_simd, stream); break;
            case 2: st = launch_m<2>(mm, a, packed, scale, yo, N, K, G, beta, waves_per_simd, stream); break;
            case 3: st = launch_m<3>(mm, a, packed, scale, yo, N, K, G, beta, waves_per_simd, stream); break;
            case 4: st = launch_m<4>(mm, a, packed, scale, yo, N, K, G, beta, waves_per_simd, stream); break;
            default: return PIE_HIP_ERR_INVALID;
        }
        if (st != PIE_HIP_OK) return st;
    }
    return PIE_HIP_OK;
}

}  // namespace pie_hip

extern "C" int pie_hip_gemv_w4a16(const uint16_t* act_bf16, const uint32_t* packed,
                                  const uint16_t* scale_bf16, uint16_t* y_bf16, int M, int N,
                                  int K, int group_size, int beta, void* stream) {
    if (M > 32) return PIE_HIP_ERR_UNSUPPORTED;
    return pie_hip::gemv_w4a16_dispatch(act_bf16, packed, scale_bf16, y_bf16, M, N, K,
                                        group_size, beta, 0, 0,
                                        static_cast<hipStream_t>(stream));
}

// Tuning hook: same contract with explicit rows-per-wave / waves-per-SIMD.
extern "C" int pie_hip_gemv_w4a16_tuned(const uint16_t* act_bf16, const uint32_t* packed,
                                        const uint16_t* scale_bf16, uint16_t* y_bf16, int M,
                                        int N, int K, int group_size, int beta,
                                        int rows_per_wave, int waves_per_simd, void* stream) {
    return pie_hip::gemv_w4a16_dispatch(act_bf16, packed, scale_bf16, y_bf16, M, N, K,
                                        group_size, beta, rows_per_wave, waves_per_simd,
                                        static_cast<hipStream_t>(stream));
}
