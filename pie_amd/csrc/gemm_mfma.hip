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
// Tiling: a 128 x 128 output tile per block of four waves or, for large M, 256 x 128 per block of
// eight (two per SIMD), each wave a 64 x 64 quadrant held as 4 x 4 accumulators of
// v_mfma_f32_16x16x32_bf16; K advances 64 at a time.
//   * activations (and bf16 weights) travel global -> LDS directly (global_load_lds_dwordx4,
//     no registers) into a ring of three stages, issued two K steps ahead; every wave waits
//     for its own transfers with an explicit vmcnt and the block meets at one barrier per step;
//   * quantised weights travel through registers, three K steps ahead (a tile row is only
//     8-32 bytes per thread: two or four threads share a row, every wave stages its share), are
//     decoded to bf16 and written to a double-buffered LDS tile one step before use; the rows of
//     eight consecutive lanes are two apart, so one LDS write cycle touches eight bank groups;
//   * LDS tiles are unpadded and XOR-swizzled in 16-byte granules (granule g of row r sits at
//     g ^ ((r >> 1) & 7)) so that the 16 rows an MFMA operand read touches fall in distinct
//     banks while a direct-to-LDS transfer still writes 1 KiB contiguous per wave;
//   * activations are the MFMA A operand, weights the B operand: an accumulator lane holds one
//     weight row n (column of y) for four consecutive activation rows, so row scales are
//     per-lane scalars and the SwiGLU partner (gate_i, up_i interleaved) is the neighbour lane.
#include "common.hip.h"

#include <type_traits>

namespace pie_hip {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kThreads = 256;
constexpr int kTileVecs = BM * (BK / 8);   // 16-byte vectors per bf16 tile (16 KiB)
constexpr int kStages = 3;
constexpr int kMaxMT = 8;   // 16-row activation tiles per wave, at most

#define PIE_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

struct GemmArgs {
    const uint16_t* act;
    const unsigned char* w;
    const unsigned char* scale;
    uint16_t* y;
    int M, N, K, g_shift, beta, swiglu, scale_is_bf16;
    float* partial;   // split-K: fp32 [gridDim.z][M][N] partial sums (row scale applied), else null
};

__device__ __forceinline__ uint32_t pack_trunc(float lo, float hi) {
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

// position of granule g of tile row r (in 16-byte vectors)
__device__ __forceinline__ int swz(int r, int g) { return r * 8 + (g ^ ((r >> 1) & 7)); }

// ---- quantised weight staging: global -> registers (raw) -> bf16 vectors in LDS ------------
// TPR threads share a tile row of one K step: part p of a row holds its k-values
// [p * 64 / TPR, (p + 1) * 64 / TPR) — 32 per thread with four waves, 16 with eight.
template <int TPR>
struct GInt4T {
    static constexpr int kWords = 8 / TPR;   // 32-bit words (8 nibbles each) per thread
    static constexpr int kLoads = 2;         // vector-memory operations per thread per K step
    static constexpr int kValuPerMfma = 4;   // decode instructions placed behind each MFMA of the 256-row tile
    static constexpr bool kRowScale = false, kDirect = false;
    struct Raw {
        uint32_t v[kWords];
        uint16_t gs;
    };
    static __device__ __forceinline__ Raw load(const GemmArgs& a, int n, int k0, int part) {
        Raw r;
        const int kk = k0 + part * (64 / TPR);
        const unsigned char* p = a.w + (static_cast<size_t>(n) * a.K + kk) / 2;
        if constexpr (kWords == 4) {
            const u32x4_t t = *reinterpret_cast<const u32x4_t*>(p);
            r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
        } else {
            const u32x2_t t = *reinterpret_cast<const u32x2_t*>(p);
            r.v[0] = t.x; r.v[1] = t.y;
        }
        r.gs = reinterpret_cast<const uint16_t*>(a.scale)[static_cast<size_t>(n) * (a.K >> a.g_shift) + (kk >> a.g_shift)];
        return r;
    }
    static __device__ __forceinline__ void store(u32x4_t* tile, int row, int part, const Raw& r, uint32_t k128) {
        const float gs = bf16_bits_to_f32(r.gs);
        const float off = -136.f * gs;
#pragma unroll
        for (int s = 0; s < kWords; ++s) {
            const uint32_t v = r.v[s];
            uint32_t pr[4];   // pr[j] = (128 + nib_j, 128 + nib_{j+4}) as a bf16 pair
#pragma unroll
            for (int j = 0; j < 4; ++j) pr[j] = and_or(v >> (4 * j), 0x000F000Fu, k128);
            float f[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                f[j] = fmaf(bf16_lo(pr[j]), gs, off);       // exact: (nib - 8) * scale
                f[j + 4] = fmaf(bf16_hi(pr[j]), gs, off);
            }
            tile[swz(row, part * kWords + s)] = u32x4_t{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]),
                                                       pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
        }
    }
};
template <int TPR>
struct GFp8T {
    static constexpr int kVecs = 4 / TPR;    // 16-byte vectors (16 codes each) per thread
    static constexpr int kLoads = kVecs, kValuPerMfma = 1;
    static constexpr bool kRowScale = true, kDirect = false;
    struct Raw {
        u32x4_t v[kVecs];
    };
    static __device__ __forceinline__ Raw load(const GemmArgs& a, int n, int k0, int part) {
        Raw r;
        const unsigned char* p = a.w + static_cast<size_t>(n) * a.K + k0 + part * (64 / TPR);
#pragma unroll
        for (int v = 0; v < kVecs; ++v) r.v[v] = *reinterpret_cast<const u32x4_t*>(p + 16 * v);
        return r;
    }
    static __device__ __forceinline__ uint32_t cv(uint32_t w, bool hi) {
        const f32x2_t f = hi ? __builtin_amdgcn_cvt_pk_f32_fp8(w, true) : __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
        return pack_trunc(f.x, f.y);
    }
    static __device__ __forceinline__ void store(u32x4_t* tile, int row, int part, const Raw& r, uint32_t) {
#pragma unroll
        for (int v = 0; v < kVecs; ++v)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t a = r.v[v][2 * s], b = r.v[v][2 * s + 1];
                tile[swz(row, part * 2 * kVecs + v * 2 + s)] = u32x4_t{cv(a, false), cv(a, true), cv(b, false), cv(b, true)};
            }
    }
};
template <int TPR>
struct GInt8T {
    static constexpr int kVecs = 4 / TPR;
    static constexpr int kLoads = kVecs, kValuPerMfma = 2;
    static constexpr bool kRowScale = true, kDirect = false;
    using Raw = typename GFp8T<TPR>::Raw;
    static __device__ __forceinline__ Raw load(const GemmArgs& a, int n, int k0, int part) {
        return GFp8T<TPR>::load(a, n, k0, part);
    }
    static __device__ __forceinline__ uint32_t two(uint32_t u, int sh) {
        // signed bytes -> exact bf16 pair: (byte ^ 0x80) - 128
        const float lo = static_cast<float>((u >> sh) & 0xFFu) - 128.f;
        const float hi = static_cast<float>((u >> (sh + 8)) & 0xFFu) - 128.f;
        return pack_trunc(lo, hi);
    }
    static __device__ __forceinline__ void store(u32x4_t* tile, int row, int part, const Raw& r, uint32_t) {
#pragma unroll
        for (int v = 0; v < kVecs; ++v)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t a = r.v[v][2 * s] ^ 0x80808080u, b = r.v[v][2 * s + 1] ^ 0x80808080u;
                tile[swz(row, part * 2 * kVecs + v * 2 + s)] = u32x4_t{two(a, 0), two(a, 16), two(b, 0), two(b, 16)};
            }
    }
};
// (the format tags the launchers take; the kernel picks the TPR form for its wave count)
struct GInt4 {
    template <int TPR> using Staged = GInt4T<TPR>;
    static constexpr bool kDirect = false, kRowScale = false;
};
struct GFp8 {
    template <int TPR> using Staged = GFp8T<TPR>;
    static constexpr bool kDirect = false, kRowScale = true;
};
struct GInt8 {
    template <int TPR> using Staged = GInt8T<TPR>;
    static constexpr bool kDirect = false, kRowScale = true;
};
struct GBf16T {
    static constexpr int kLoads = 4, kValuPerMfma = 0;   // direct-to-LDS transfers per wave per K step
    static constexpr bool kRowScale = false, kDirect = true;
    struct Raw {};
    static __device__ __forceinline__ Raw load(const GemmArgs&, int, int, int) { return {}; }
    static __device__ __forceinline__ void store(u32x4_t*, int, int, const Raw&, uint32_t) {}
};
struct GBf16 {
    template <int TPR> using Staged = GBf16T;
    static constexpr bool kDirect = true, kRowScale = false;
};

// s_waitcnt with vmcnt(n) (n < 16) and lgkmcnt(0), expcnt untouched (gfx9 encoding)
#define PIE_WAIT_VM_LGKM0(n) __builtin_amdgcn_s_waitcnt(0x0070 | (n))

// MT: 16-row activation tiles per wave (4: 64 x 64 per wave; 2: 32 x 64 for small batches).
// NW: waves per block, 4 (2 x 2 quadrants) or 8 (4 x 2: two waves per SIMD, so one wave's
// barrier and operand-read waits sit in the other's MFMAs).
template <class Base, int MT_, int NW_ = 4>
struct Shape {
    using Format = Base;
    static constexpr int kMT = MT_, kNW = NW_;
};

template <class SH>
__global__ __launch_bounds__(SH::kNW* kWave) void gemm_mfma_kernel(const GemmArgs a) {
    constexpr int MT = SH::kMT, NW = SH::kNW;
    constexpr int TPR = NW / 2;                  // threads that share a staged weight row
    using F = typename SH::Format::template Staged<TPR>;
    constexpr int BMv = 16 * MT * (NW / 2);      // activation rows per block
    constexpr int TB = 16 / NW;                  // direct weight transfers per wave and K step
    constexpr int kATileVecs = BMv * (BK / 8);   // 16-byte vectors per activation stage
    extern __shared__ __align__(16) unsigned char smem[];
    u32x4_t* lds_a = reinterpret_cast<u32x4_t*>(smem);            // [kStages][A tile]
    u32x4_t* lds_b = lds_a + kStages * kATileVecs;                // direct: [kStages][tile]; else [2][tile]
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int j = lane & 15, q = lane >> 4;
    const int wm = wv >> 1, wn = wv & 1;
    const int M = a.M, N = a.N, K = a.K;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BMv;
    // split-K: block z owns the K steps [kbeg, kbeg + nk) (the host makes every share non-empty)
    const int nk_all = K / BK;
    const int per_split = (nk_all + static_cast<int>(gridDim.z) - 1) / static_cast<int>(gridDim.z);
    const int kbeg = blockIdx.z * per_split;
    const int nk = min(per_split, nk_all - kbeg);

    // direct transfers: wave w moves the 1 KiB chunks ci = 4u + w (8 tile rows each); lane p
    // lands at chunk position p = (row ci*8 + p/8, slot p%8), which holds granule slot ^ key(row)
    const uint16_t* aptr[kMaxMT];   // (fixed bounds: arrays sized by the template value kept the
                                    // host side from emitting the kernel stubs)
    const uint16_t* bptr[4];
#pragma unroll
    for (int u = 0; u < (MT > 4 ? MT : 4); ++u) {
        const int r = (u * NW + wv) * 8 + (lane >> 3);
        const int g = (lane & 7) ^ ((r >> 1) & 7);
        if (u < MT) aptr[u] = a.act + static_cast<size_t>(min(m0 + r, M - 1)) * K + g * 8;
        if (u < TB)
            bptr[u] = reinterpret_cast<const uint16_t*>(a.w) + static_cast<size_t>(min(n0 + r, N - 1)) * K + g * 8;
    }
    auto issue_direct = [&](int kt) {
        const int k0 = (kbeg + min(kt, nk - 1)) * BK;
        const int st = kt % kStages;
        if (F::kDirect) {
#pragma unroll
            for (int u = 0; u < TB; ++u)
                __builtin_amdgcn_global_load_lds(bptr[u] + k0, PIE_LDS_PTR(lds_b + st * kTileVecs + (u * NW + wv) * 64), 16, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < MT; ++u)
            __builtin_amdgcn_global_load_lds(aptr[u] + k0, PIE_LDS_PTR(lds_a + st * kATileVecs + (u * NW + wv) * 64), 16, 0, 0);
    };
    // quantised weights: TPR threads per tile row, every wave stages 128 / NW rows.  Within
    // eight consecutive lanes (one LDS write cycle) the rows are 2 apart, so that their swizzle
    // keys differ and the eight 16-byte granules fall in eight different bank groups.
    constexpr bool stager = true;
    const int wpart = lane & (TPR - 1);
    const int wrow = TPR == 2 ? wv * 32 + ((lane >> 4) & 3) * 8 + ((lane >> 3) & 1) + ((lane >> 1) & 3) * 2
                              : wv * 16 + ((lane >> 4) & 3) * 4 + ((lane >> 2) & 1) * 2 + ((lane >> 3) & 1);
    const int wn_glob = min(n0 + wrow, N - 1);
    auto load_w = [&](int kt) { return F::load(a, wn_glob, (kbeg + min(kt, nk - 1)) * BK, wpart); };

    uint32_t magic = 0x43004300u;   // (128.0, 128.0) as a bf16 pair, opaque to the compiler
    asm volatile("" : "+v"(magic));
    f32x4_t acc[kMaxMT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // prologue: activations of steps 0 and 1 in flight, weights of steps 0..2 in registers,
    // the bf16 tile of step 0 written
    typename F::Raw rr[kStages];
    issue_direct(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kStages; ++i)
        if (stager) rr[i] = load_w(i);
    __builtin_amdgcn_sched_barrier(0);
    issue_direct(1);
    __builtin_amdgcn_sched_barrier(0);
    if (!F::kDirect && stager) F::store(lds_b, wrow, wpart, rr[0], magic);

    // The loop body is unrolled three times so that ring slots (LDS stage, register set) are
    // compile-time constants: a register rotation would have to wait for the newest load.
    // Whole triples of K steps run without a branch, so that one scheduling region holds a
    // step's MFMAs, its operand reads and the decode of the next step's weights; the region's
    // group barriers then spread the vector-ALU work and the LDS traffic between the MFMAs (a
    // block is one wave per SIMD: nothing else would fill the matrix pipe's shadow).
    auto step = [&](const int i, const int kt, auto tail) {
        constexpr bool kTail = decltype(tail)::value;
        // Transfers of step kt are complete when at most the operations issued after them
        // are outstanding: the previous iteration's weight loads and its 4 (8) transfers.
        __builtin_amdgcn_sched_barrier(0);
        if (F::kDirect) PIE_WAIT_VM_LGKM0(TB + MT);
        else PIE_WAIT_VM_LGKM0(MT + F::kLoads);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        rr[i] = load_w(kt + kStages);   // slot i held step kt, already written to LDS
        __builtin_amdgcn_sched_barrier(0);
        issue_direct(kt + 2);           // into the stage step kt - 1 was read from
        __builtin_amdgcn_sched_barrier(0);

        if (!kTail || kt < nk) {
            const u32x4_t* A = lds_a + i * kATileVecs + (wm * 16 * MT + j) * 8;
            const u32x4_t* B = lds_b + (F::kDirect ? i : (kt & 1)) * kTileVecs + (wn * 64 + j) * 8;
            const int key = j >> 1;   // swizzle key of rows base16 + j
            bf16x8_t af[BK / 32][kMaxMT], bfr[BK / 32][4];
#pragma unroll
            for (int ks = 0; ks < BK / 32; ++ks) {
                const int slot = (ks * 4 + q) ^ key;
#pragma unroll
                for (int t = 0; t < MT; ++t) af[ks][t] = __builtin_bit_cast(bf16x8_t, A[t * 16 * 8 + slot]);
#pragma unroll
                for (int t = 0; t < 4; ++t) bfr[ks][t] = __builtin_bit_cast(bf16x8_t, B[t * 16 * 8 + slot]);
            }
#pragma unroll
            for (int ks = 0; ks < BK / 32; ++ks)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int nt = 0; nt < 4; ++nt)
                        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[ks][mt], bfr[ks][nt], acc[mt][nt], 0, 0, 0);
        }
        // next step's weights -> bf16 tile (the other buffer; its readers passed the barrier)
        if (!F::kDirect) F::store(lds_b + ((kt + 1) & 1) * kTileVecs, wrow, wpart, rr[(i + 1) % kStages], magic);
        if (!kTail) {
            // order of the region: the first K half's operand reads, then per MFMA a few vector-ALU
            // instructions of the decode; the second half's reads ride in the first MFMAs' shadow,
            // the decoded tile's four LDS writes in the last ones'
            constexpr int kMfma = MT * 4;
            __builtin_amdgcn_sched_group_barrier(0x100, MT + 4, 0);
#pragma unroll
            for (int u = 0; u < kMfma; ++u) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (u < MT + 4) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if (!F::kDirect) __builtin_amdgcn_sched_group_barrier(0x002, F::kValuPerMfma, 0);
            }
#pragma unroll
            for (int u = 0; u < kMfma; ++u) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (!F::kDirect) __builtin_amdgcn_sched_group_barrier(0x002, F::kValuPerMfma, 0);
                if (!F::kDirect && u >= kMfma - 8 && (u & 1)) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
        }
    };
    int kt0 = 0;
    for (; kt0 + kStages <= nk; kt0 += kStages) {
#pragma unroll
        for (int i = 0; i < kStages; ++i) step(i, kt0 + i, std::false_type{});
    }
    if (kt0 < nk) {
#pragma unroll
        for (int i = 0; i < kStages; ++i) step(i, kt0 + i, std::true_type{});
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
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wm * 16 * MT + mt * 16 + 4 * q + r;
                float v = acc[mt][nt][r] * rs;
                const bool ok = m < M && n < N;
                if (a.partial) {
                    if (ok) a.partial[(static_cast<size_t>(blockIdx.z) * M + m) * N + n] = v;
                } else if (a.swiglu) {
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

// Sums the split-K partials and applies the epilogue the single-pass kernel would have applied
// (residual add, or SwiGLU over adjacent (gate, up) columns with both rounded to bf16 first).
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* partial, uint16_t* y,
                                                                 int M, int N, int splits, int beta,
                                                                 int swiglu) {
    const int nout = swiglu ? N / 2 : N;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<size_t>(M) * nout) return;
    const int m = static_cast<int>(idx / nout), c = static_cast<int>(idx % nout);
    const size_t plane = static_cast<size_t>(M) * N;
    if (swiglu) {
        const float* p = partial + static_cast<size_t>(m) * N + 2 * c;
        float g = 0.f, u = 0.f;
        for (int z = 0; z < splits; ++z) {
            g += p[z * plane];
            u += p[z * plane + 1];
        }
        const float gb = bf16_bits_to_f32(f32_to_bf16_bits(g));
        const float ub = bf16_bits_to_f32(f32_to_bf16_bits(u));
        const float silu = gb / (1.f + expf(-gb));
        y[idx] = f32_to_bf16_bits(silu * ub);
    } else {
        const float* p = partial + static_cast<size_t>(m) * N + c;
        float v = 0.f;
        for (int z = 0; z < splits; ++z) v += p[z * plane];
        if (beta) v += bf16_bits_to_f32(y[idx]);
        y[idx] = f32_to_bf16_bits(v);
    }
}

template <class F, int MT, int NW = 4>
int launch_gemm_mt(const GemmArgs& a, int splits, hipStream_t stream) {
    constexpr int BMv = 16 * MT * (NW / 2);
    constexpr size_t smem = (static_cast<size_t>(kStages) * BMv * (BK / 8) +
                             static_cast<size_t>(F::kDirect ? kStages : 2) * kTileVecs) * sizeof(u32x4_t);
    static const hipError_t attr =
        hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mfma_kernel<Shape<F, MT, NW>>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (attr != hipSuccess) return PIE_HIP_ERR_LAUNCH;
    const dim3 grid((a.N + BN - 1) / BN, (a.M + BMv - 1) / BMv, splits);
    if (grid.y > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gemm_mfma_kernel<Shape<F, MT, NW>>), grid, dim3(NW * kWave), smem, stream, a);
    return launch_status();
}

// Blocks are eight waves, two per SIMD, so that one wave's barrier and operand-read waits sit
// in another's MFMAs: 256 x 128 tiles (64 x 64 per wave) or 128 x 128 (32 x 64 per wave).
// Measured at M = 2048 (MI355X): int4 805-905 TFLOP/s against 690-755 with 128 x 128 tiles on
// four waves, fp8 830-960 against 690-860, bf16 1020-1170 against 670-920 (the 256-row tile on
// four waves of 128 x 64 reached 790-930 for bf16 and nothing for the quantised formats); at
// M = 128 / 512 on the shapes that fill one round of blocks the 128-row tile went from 57-187
// to 46-151 us with eight waves.  A 256-row tile takes 1.85x the time of a 128-row one for
// twice the work; it is taken when its rounds of 256 blocks cost less.  Batches of up to 64
// rows take 64 x 128 tiles (16 x 64 per wave: 38-119 us against 44-136 on four waves).
// PIE_HIP_GEMM_MT=4|8 forces the 128- / 256-row shape (measurement hook).
template <class F>
int launch_gemm(const GemmArgs& a, hipStream_t stream) {
    static const int forced = [] { const char* e = getenv("PIE_HIP_GEMM_MT"); return e ? atoi(e) : 0; }();
    if (a.M <= 64 && !forced) return launch_gemm_mt<F, 1, 8>(a, 1, stream);   // 64-row block tiles (16 x 64 per wave)
    const long long nt = (a.N + BN - 1) / BN;
    const long long t4 = nt * ((a.M + 127) / 128), t8 = nt * ((a.M + 255) / 256);
    const double c4 = static_cast<double>((t4 + 255) / 256), c8 = 1.85 * static_cast<double>((t8 + 255) / 256);
    const bool tall = forced ? forced == 8 : (a.M > 128 && c8 < c4);
    return tall ? launch_gemm_mt<F, 4, 8>(a, 1, stream) : launch_gemm_mt<F, 2, 8>(a, 1, stream);
}

// Few output tiles (M up to 128 rows of a decode batch): a block per (tile, K share) so that
// the machine is full and each block's serial K loop is short; fp32 partials meet in a second
// kernel.  Returns the number of K shares for a shape, 1 = not worth splitting.
int splitk_shares(int M, int N, int K) {
    if (M > 128) return 1;
    const long long tiles = static_cast<long long>((N + BN - 1) / BN) * (M > 64 ? (M + 127) / 128 : 1);
    const int nk_all = K / BK;
    long long want = 1024 / tiles;
    if (want > 16) want = 16;
    if (want > nk_all / 4) want = nk_all / 4;
    if (want < 2) return 1;
    const int per = (nk_all + static_cast<int>(want) - 1) / static_cast<int>(want);
    return (nk_all + per - 1) / per;   // every share non-empty
}

template <class F>
int launch_gemm_splitk(GemmArgs a, int splits, float* ws, hipStream_t stream) {
    const int beta = a.beta, swiglu = a.swiglu;
    a.partial = ws;
    a.beta = 0;
    a.swiglu = 0;
    const int st = a.M <= 64 ? launch_gemm_mt<F, 1, 8>(a, splits, stream) : launch_gemm_mt<F, 2, 8>(a, splits, stream);
    if (st != PIE_HIP_OK) return st;
    const size_t outs = static_cast<size_t>(a.M) * (swiglu ? a.N / 2 : a.N);
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3(static_cast<unsigned>((outs + 255) / 256)), dim3(256), 0,
                       stream, ws, a.y, a.M, a.N, splits, beta, swiglu);
    return launch_status();
}

}  // namespace
}  // namespace pie_hip

namespace pie_hip {
namespace {
int gemm_entry(int format, const uint16_t* act_bf16, const void* weight, const void* scale,
               int scale_is_bf16, int group_size, uint16_t* y_bf16, int M, int N, int K, int beta,
               int swiglu, void* workspace, size_t workspace_bytes, void* stream) {
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
    if (format == PIE_HIP_FMT_INT4B8) {
        // a 32-value run of one row must lie inside one scale group
        if (group_size < 32 || (group_size & (group_size - 1)) != 0 || K % group_size != 0)
            return PIE_HIP_ERR_UNSUPPORTED;
        a.g_shift = __builtin_ctz(static_cast<unsigned>(group_size));
    }
    const int splits = workspace ? splitk_shares(M, N, K) : 1;
    if (splits > 1) {
        if (workspace_bytes < static_cast<size_t>(splits) * M * N * sizeof(float)) return PIE_HIP_ERR_INVALID;
        float* ws = static_cast<float*>(workspace);
        switch (format) {
            case PIE_HIP_FMT_INT4B8: return launch_gemm_splitk<GInt4>(a, splits, ws, st);
            case PIE_HIP_FMT_INT8: return launch_gemm_splitk<GInt8>(a, splits, ws, st);
            case PIE_HIP_FMT_FP8: return launch_gemm_splitk<GFp8>(a, splits, ws, st);
            case PIE_HIP_FMT_BF16: return launch_gemm_splitk<GBf16>(a, splits, ws, st);
            default: return PIE_HIP_ERR_INVALID;
        }
    }
    switch (format) {
        case PIE_HIP_FMT_INT4B8: return launch_gemm<GInt4>(a, st);
        case PIE_HIP_FMT_INT8: return launch_gemm<GInt8>(a, st);
        case PIE_HIP_FMT_FP8: return launch_gemm<GFp8>(a, st);
        case PIE_HIP_FMT_BF16: return launch_gemm<GBf16>(a, st);
        default: return PIE_HIP_ERR_INVALID;
    }
}
}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_gemm_mfma(int format, const uint16_t* act_bf16, const void* weight,
                                 const void* scale, int scale_is_bf16, int group_size,
                                 uint16_t* y_bf16, int M, int N, int K, int beta, int swiglu,
                                 void* stream) {
    return pie_hip::gemm_entry(format, act_bf16, weight, scale, scale_is_bf16, group_size, y_bf16, M, N,
                               K, beta, swiglu, nullptr, 0, stream);
}

extern "C" size_t pie_hip_gemm_mfma_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % pie_hip::BK != 0) return 0;
    const int splits = pie_hip::splitk_shares(M, N, K);
    return splits > 1 ? static_cast<size_t>(splits) * M * N * sizeof(float) : 0;
}

extern "C" int pie_hip_gemm_mfma_splitk(int format, const uint16_t* act_bf16, const void* weight,
                                        const void* scale, int scale_is_bf16, int group_size,
                                        uint16_t* y_bf16, int M, int N, int K, int beta, int swiglu,
                                        void* workspace, size_t workspace_bytes, void* stream) {
    return pie_hip::gemm_entry(format, act_bf16, weight, scale, scale_is_bf16, group_size, y_bf16, M, N,
                               K, beta, swiglu, workspace, workspace_bytes, stream);
}
