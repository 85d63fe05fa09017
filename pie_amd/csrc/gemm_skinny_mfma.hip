// Skinny / grouped weight-only GEMM on the matrix cores (v_mfma_f32_16x16x32_bf16) for
// gfx950: y[m, n] = sum_k act[m, k] * w(n, k) for a handful to a few dozen activation rows,
// and the MoE grouped form (one small-M problem per expert, rows gathered by route).
//
// Same contracts as the weight-streaming GEMV (formats, fused evaluation order, fp32
// accumulation); it replaces re-streaming the weights once per four activation rows with one
// pass over the weights per 16 rows.  Reference roles: Marlin W4A16 for small/medium M
// (driver/cuda/third_party/marlin/marlin_wrapper.hpp:39-51), the per-route MoE decode GEMVs
// (driver/cuda/src/kernels/dequant_wna16.cu:59-169, grid = routes x rows, which re-read an
// expert's weights once per route) and the grouped GEMM (driver/cuda/src/ops/gemm.hpp:189-198).
//
// Design — still HBM-bound, the weights are the traffic:
//   * weights never touch LDS.  Each lane loads 16 bytes of ONE weight row straight into the
//     MFMA B-operand layout (column n = lane % 16, k-block = lane / 16) and decodes them in
//     registers (int4 -> bf16 by OR-ing the exponent of 128.0 onto nibble pairs; int8/fp8 ->
//     bf16 exactly through the conversion instructions); one 16-byte load feeds 4 / 2 / 1 MFMA
//     steps.  Weight loads run a ring of PW blocks ahead of the MFMAs and nothing else uses the
//     vector-memory counter inside the stream, so the waits stay partial;
//   * activations are the A operand (row m = lane % 16): a tile of 16 rows x CK k-values sits in
//     LDS (rows padded by one 16-byte vector so the 16 rows a read touches hit different banks),
//     already in the element order the weight decode produces, staged once per K chunk and
//     reused by all NG tiles of 16 weight rows the block owns;
//   * with activations as A and weights as B, the accumulator lane holding outputs of column n
//     is the lane that loaded row n's weights: int4 group scales and int8/fp8 row scales are
//     per-lane scalars.  The offset-binary bias (-136 / -128 times the sum of the activations)
//     needs sum_k x[m, k] in the accumulator layout — one more MFMA against a tile of ones,
//     done once per K block and reused for every weight tile;
//   * the KP waves of a block split K (wave w takes 16-byte blocks b = KP*g + w, so together they
//     read KP*64 contiguous bytes of each weight row per step); partial sums meet in LDS once;
//   * epilogue: row scale, residual add, or SwiGLU over adjacent (gate, up) columns exchanged
//     with one DPP move.
#include "common.hip.h"

namespace pie_hip {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_hi16(float lo, float hi) {
    // bf16 pair by truncation (exact for values with <= 8 significant bits)
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

// ---- formats: K per 16-byte load (per lane), MFMA steps per load, decode of step s --------
struct SkInt4 {
    static constexpr int kPerLane = 32, kSteps = 4, kBytesPer2K = 1;
    static constexpr float kBias = -136.f;
    static constexpr bool kGroupScale = true;
    // (128.0bf16, 128.0bf16) held in a VGPR for and_or: made once per kernel, opaque to the compiler
    static __device__ __forceinline__ uint32_t magic() {
        uint32_t k128 = 0x43004300u;
        asm volatile("" : "+v"(k128));
        return k128;
    }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int s, uint32_t k128) {
        const uint32_t v = w[s];
        return u32x4_t{and_or(v, 0x000F000Fu, k128), and_or(v >> 4, 0x000F000Fu, k128),
                       and_or(v >> 8, 0x000F000Fu, k128), and_or(v >> 12, 0x000F000Fu, k128)};
    }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int s) {
        uint32_t k128 = 0x43004300u;
        asm volatile("" : "+v"(k128));
        const uint32_t v = w[s];
        return u32x4_t{and_or(v, 0x000F000Fu, k128), and_or(v >> 4, 0x000F000Fu, k128),
                       and_or(v >> 8, 0x000F000Fu, k128), and_or(v >> 12, 0x000F000Fu, k128)};
    }
    // activations of one 8-block in the order decode() yields weights: (0,4)(1,5)(2,6)(3,7)
    static __device__ __forceinline__ u32x4_t order(const u32x4_t v) {
        return u32x4_t{__builtin_amdgcn_perm(v.z, v.x, 0x05040100u),
                       __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                       __builtin_amdgcn_perm(v.w, v.y, 0x05040100u),
                       __builtin_amdgcn_perm(v.w, v.y, 0x07060302u)};
    }
};
struct SkFp8 {
    static constexpr int kPerLane = 16, kSteps = 2, kBytesPer2K = 2;
    static constexpr float kBias = 0.f;
    static constexpr bool kGroupScale = false;
    static __device__ __forceinline__ uint32_t magic() { return 0u; }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int s, uint32_t) { return decode(w, s); }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int s) {
        const uint32_t a = w[2 * s], b = w[2 * s + 1];
        const f32x2_t a0 = __builtin_amdgcn_cvt_pk_f32_fp8(a, false);
        const f32x2_t a1 = __builtin_amdgcn_cvt_pk_f32_fp8(a, true);
        const f32x2_t b0 = __builtin_amdgcn_cvt_pk_f32_fp8(b, false);
        const f32x2_t b1 = __builtin_amdgcn_cvt_pk_f32_fp8(b, true);
        return u32x4_t{pack_hi16(a0.x, a0.y), pack_hi16(a1.x, a1.y), pack_hi16(b0.x, b0.y),
                       pack_hi16(b1.x, b1.y)};
    }
    static __device__ __forceinline__ u32x4_t order(const u32x4_t v) { return v; }
};
struct SkInt8 {
    static constexpr int kPerLane = 16, kSteps = 2, kBytesPer2K = 2;
    static constexpr float kBias = -128.f;
    static constexpr bool kGroupScale = false;
    static __device__ __forceinline__ uint32_t two(uint32_t u, int lo_shift) {
        return pack_hi16(static_cast<float>((u >> lo_shift) & 0xFFu),
                         static_cast<float>((u >> (lo_shift + 8)) & 0xFFu));
    }
    static __device__ __forceinline__ uint32_t magic() { return 0u; }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int s, uint32_t) { return decode(w, s); }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int s) {
        const uint32_t a = w[2 * s] ^ 0x80808080u, b = w[2 * s + 1] ^ 0x80808080u;
        return u32x4_t{two(a, 0), two(a, 16), two(b, 0), two(b, 16)};
    }
    static __device__ __forceinline__ u32x4_t order(const u32x4_t v) { return v; }
};
struct SkBf16 {
    static constexpr int kPerLane = 8, kSteps = 1, kBytesPer2K = 4;
    static constexpr float kBias = 0.f;
    static constexpr bool kGroupScale = false;
    static __device__ __forceinline__ uint32_t magic() { return 0u; }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int, uint32_t) { return w; }
    static __device__ __forceinline__ u32x4_t decode(const u32x4_t w, int) { return w; }
    static __device__ __forceinline__ u32x4_t order(const u32x4_t v) { return v; }
};

struct SkinnyArgs {
    const uint16_t* act;        // bf16 [*, K]
    const int32_t* act_rows;    // gather: activation row of each problem row, or null
    const unsigned char* w;     // weights of problem 0, row-major [N, K] in the format
    const unsigned char* scale; // int4: bf16 [N, K/G]; int8/fp8: row scale [N]; bf16: null
    uint16_t* y;                // [rows, N] (or [rows, N/2] with swiglu)
    const int32_t* offsets;     // grouped: [P+1] first row of each problem; null: one problem
    int M;                      // rows when offsets == null
    int N, K, G, g_shift, beta, swiglu, scale_is_bf16;
    int m_split;                // dense only: blockIdx.y = 16-row pass
    int tiled;                  // weights (and int4 group scales) in the tile-major layout
    size_t w_stride, scale_stride;  // bytes between problems
    // q|k|v epilogue of the wave-private form (rope_table != null): rows of W are the q, k and
    // v heads; adjacent output pairs of q and k heads are rotated, q goes to y [rows, hq*d], k
    // and v to slot kv_slots[row] of the page pools
    const float* rope_table;    // [rows, d]: cos (d/2) then sin (d/2) per row
    const int64_t* kv_slots;    // [rows]; negative: the row writes no K/V
    uint16_t* k_pages;
    uint16_t* v_pages;
    int hq, hk, d;
    int half_out;   // q / k rows re-ordered at load: pair (2i, 2i+1) goes to positions (i, i + d/2)
};

constexpr int gcd_c(int a, int b) { return b == 0 ? a : gcd_c(b, a % b); }

template <int WL>
struct WSlot {
    u32x4_t w[WL];
    uint16_t gs[WL];
};

// KP waves split K; CK k-values of activations per LDS chunk; NG tiles of 16 weight rows per
// block; PW ring slots of WL adjacent 16-byte weight blocks in flight per lane (WL = 2: a
// wave's two loads of a step cover whole 128-byte lines of each of its 16 rows).
template <class F, int KP, int CK, int NG, int PW, int WL, bool TILED>
__global__ __launch_bounds__(KP* kWave) void skinny_kernel(const SkinnyArgs a) {
    constexpr int KPL = F::kPerLane, S = F::kSteps;
    constexpr int LK = 4 * KPL;               // k covered by one wave-wide 16-byte load
    constexpr int GC = CK / (KP * LK * WL);   // steps per wave per full chunk
    constexpr int STRIDE = CK / 8 + 1;        // 16-byte vectors per staged activation row
    constexpr int NT = KP * kWave;
    constexpr bool kBiased = F::kBias != 0.f;
    constexpr bool kRowBias = kBiased && !F::kGroupScale;
    static_assert(GC >= 1 && (GC < PW || GC % PW == 0), "ring must tile a chunk");
    static_assert(!F::kGroupScale || GC <= PW, "per-block activation sums are kept per step of a tile");
    extern __shared__ __align__(16) unsigned char smem[];
    u32x4_t* lds_a = reinterpret_cast<u32x4_t*>(smem);
    float* red = reinterpret_cast<float*>(smem);
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int j = lane & 15, q = lane >> 4;
    const int N = a.N, K = a.K;
    // blockIdx.y: the problem (expert) of a grouped launch, or — dense launches of small
    // matrices — the 16-row pass, so that the passes run side by side instead of in a loop
    const int p = a.offsets ? blockIdx.y : 0;
    const int r0 = a.offsets ? a.offsets[p] : (a.m_split ? blockIdx.y * 16 : 0);
    const int r1 = a.offsets ? a.offsets[p + 1] : (a.m_split ? min(a.M, r0 + 16) : a.M);
    if (r1 <= r0) return;

    const int T = (N + 15) / 16;
    const int tile0 = blockIdx.x * NG;
    const size_t row_bytes = static_cast<size_t>(K) * F::kBytesPer2K / 2;
    const unsigned char* wbase = a.w + static_cast<size_t>(p) * a.w_stride;
    const unsigned char* sbase = a.scale ? a.scale + static_cast<size_t>(p) * a.scale_stride : nullptr;
    const uint16_t* gsbase = reinterpret_cast<const uint16_t*>(sbase);
    const int blk_shift = a.g_shift - (F::kGroupScale ? 7 : 0);   // 16-byte blocks per scale group, log2
    // Weight addressing.  Row-major [N, K]: lane (j, q) reads 16 bytes of row 16*tile + j at byte
    // 64*b + 16*q of the row.  Tile-major: the same 16 bytes sit at ((tile*nb + b)*64 + lane)*16,
    // so one wave load is 1 KiB contiguous and consecutive b are consecutive KiB.
    const int nb = K / LK;                      // 16-byte blocks along K per lane quad
    const int groups = F::kGroupScale ? K >> a.g_shift : 0;
    constexpr size_t bstride = TILED ? 1024 : static_cast<size_t>(LK) * F::kBytesPer2K / 2;
    constexpr int gstride = TILED ? 16 : 1;     // int4 scales: tile-major [tile][group][16 rows]
    // tile-major: everything but the lane's own 16 bytes (2 bytes of a scale row) is uniform
    // over the wave, so the addresses are scalar bases plus one constant vector offset
    const unsigned char* wptr[NG];
    int nrow[NG];                               // (scale row offset)
    const unsigned lane16 = TILED ? static_cast<unsigned>(lane) * 16u : 0u;
    const unsigned j2 = TILED ? static_cast<unsigned>(j) : 0u;
    float row_scale[NG];
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int tile = min(tile0 + i, T - 1);
        const int n = min(tile * 16 + j, N - 1);
        nrow[i] = TILED ? tile * 16 * groups : n * groups;   // offset of the row's first group scale
        wptr[i] = TILED ? wbase + static_cast<size_t>(tile) * nb * 1024
                        : wbase + static_cast<size_t>(n) * row_bytes + static_cast<size_t>(q) * KPL * F::kBytesPer2K / 2;
        row_scale[i] = 1.f;
        if (!F::kGroupScale && sbase)
            row_scale[i] = a.scale_is_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(sbase)[n])
                                           : reinterpret_cast<const float*>(sbase)[n];
    }
    const int nchunks = (K + CK - 1) / CK;
    const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, u32x4_t{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};

    auto load_w = [&](int c, const unsigned char* wp, int n, int g) {
        WSlot<WL> sl;
        const int b0 = c * (CK / LK) + (KP * g + wv) * WL;
#pragma unroll
        for (int h = 0; h < WL; ++h) {
            const int b = min(b0 + h, nb - 1);
            sl.w[h] = *reinterpret_cast<const u32x4_t*>(wp + static_cast<size_t>(b) * bstride + lane16);
            sl.gs[h] = F::kGroupScale ? (gsbase + static_cast<size_t>(n) + static_cast<size_t>(b >> blk_shift) * gstride)[j2] : uint16_t(0);
        }
        return sl;
    };

    // staging: TPR threads per activation row, SV 16-byte vectors per thread per chunk, held in
    // registers from one chunk's compute to the next chunk's LDS write
    constexpr int TPR = NT / 16, SV = (CK / 8) / TPR;
    const int sm = tid / TPR, sv = tid % TPR;

    for (int mt0 = r0; mt0 < r1; mt0 += 16) {
        // rows past the problem repeat its last row and are never stored.  A pass of at most four
        // (eight) rows stages four (eight): the other rows of the MFMA operand read those again,
        // their accumulator rows are never stored, and the staging traffic — every tile group
        // fetches the activations again, for an expert with a handful of routes they are as many
        // bytes as a block's weights — falls to a quarter (half).
        const int rmask = r1 - mt0 <= 4 ? 3 : r1 - mt0 <= 8 ? 7 : 15;
        const int jr = j & rmask;
        const bool stager = sm <= rmask;
        const int srow = min(mt0 + sm, r1 - 1);
        const uint16_t* arow = a.act + static_cast<size_t>(a.act_rows ? a.act_rows[srow] : srow) * K;
        u32x4_t stg[SV];
        auto stage_load = [&](int c) {
            const int cc = min(c, nchunks - 1);
            const int nvec = min(CK, K - cc * CK) / 8;
            if (stager) {
#pragma unroll
                for (int u = 0; u < SV; ++u)
                    stg[u] = *reinterpret_cast<const u32x4_t*>(arow + cc * CK + min(u * TPR + sv, nvec - 1) * 8);
            }
        };
        auto stage_store = [&](int c) {
            const int nvec = min(CK, K - min(c, nchunks - 1) * CK) / 8;
#pragma unroll
            for (int u = 0; u < SV; ++u)
                if (stager && u * TPR + sv < nvec) lds_a[sm * STRIDE + u * TPR + sv] = TILED ? stg[u] : F::order(stg[u]);   // (tile-major int4 codes sit in k order)
        };

        constexpr int NSX = F::kGroupScale ? GC * WL : 1;
        f32x4_t acc[NG], sxs[NSX], sxt = zero4;
#pragma unroll
        for (int i = 0; i < NG; ++i) acc[i] = zero4;
#pragma unroll
        for (int i = 0; i < NSX; ++i) sxs[i] = zero4;

        // the ring holds the next PW steps of the sequence (chunk, tile, g), g fastest
        WSlot<WL> ring[PW];
#pragma unroll
        for (int l = 0; l < PW; ++l) {
            const int t = l / GC;
            ring[l] = load_w(t / NG, wptr[t % NG], nrow[t % NG], l % GC);
        }
        stage_load(0);
        __syncthreads();  // the previous pass's reduction is consumed
        stage_store(0);

        auto step = [&](const WSlot<WL>& cur, int ng, int g) {
#pragma unroll
            for (int h = 0; h < WL; ++h) {
                const int vbase = ((KP * g + wv) * WL + h) * (LK / 8) + q * S;
                const int sxi = F::kGroupScale ? g * WL + h : 0;
                bf16x8_t ax[S];
#pragma unroll
                for (int s = 0; s < S; ++s) ax[s] = __builtin_bit_cast(bf16x8_t, lds_a[jr * STRIDE + vbase + s]);
                f32x4_t part = zero4;
#pragma unroll
                for (int s = 0; s < S; ++s) {
                    const bf16x8_t bw = __builtin_bit_cast(bf16x8_t, F::decode(cur.w[h], s));
                    if (kBiased && ng == 0) {
                        if (F::kGroupScale)
                            sxs[sxi] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[s], ones, s == 0 ? zero4 : sxs[sxi], 0, 0, 0);
                        else
                            sxt = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[s], ones, sxt, 0, 0, 0);
                    }
                    if (F::kGroupScale)
                        part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[s], bw, part, 0, 0, 0);
                    else
                        acc[ng] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[s], bw, acc[ng], 0, 0, 0);
                }
                if (F::kGroupScale) {
                    // a 16-byte block per lane quad = 128 k inside one scale group; the block's
                    // activation sums are kept already multiplied by the offset-binary bias
                    if (ng == 0) sxs[sxi] = sxs[sxi] * F::kBias;
                    const float sc = bf16_bits_to_f32(cur.gs[h]);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[ng][r] = fmaf(sc, part[r] + sxs[sxi][r], acc[ng][r]);
                }
            }
        };

        // CU chunks per trip of the chunk loop keep ring slots compile-time constants; the
        // chunk count is padded up to a multiple (a padded chunk has no steps, its loads are
        // clamped repeats)
        constexpr int CU = (GC >= PW) ? 1 : PW / gcd_c(PW, NG * GC);
        for (int c0 = 0; c0 < nchunks; c0 += CU) {
#pragma unroll
            for (int cu = 0; cu < CU; ++cu) {
                const int c = c0 + cu;
                __syncthreads();      // chunk c is staged
                stage_load(c + 1);    // next chunk's activations travel while this one is consumed
                const int gc_here = max(0, min(GC, (nb - c * (CK / LK)) / (KP * WL)));

#pragma unroll
                for (int ng = 0; ng < NG; ++ng) {
                    if constexpr (GC >= PW) {
                        for (int g0 = 0; g0 < GC; g0 += PW) {
#pragma unroll
                            for (int i = 0; i < PW; ++i) {
                                const int g = g0 + i;
                                const WSlot<WL> cur = ring[i];
                                // refill with the step PW ahead: same tile, or the next on wrap
                                int gn = g + PW;
                                const bool wrap = gn >= GC;
                                gn = wrap ? gn - GC : gn;
                                const int ngn = (ng + 1 < NG) ? ng + 1 : 0;
                                const unsigned char* wpn = wrap ? wptr[ngn] : wptr[ng];
                                const int nn = wrap ? nrow[ngn] : nrow[ng];
                                const int cn = (wrap && ng + 1 == NG) ? c + 1 : c;
                                ring[i] = load_w(cn, wpn, nn, gn);
                                if (g < gc_here) step(cur, ng, F::kGroupScale ? i : g);
                            }
                        }
                    } else {
#pragma unroll
                        for (int g = 0; g < GC; ++g) {
                            const int lin = (cu * NG + ng) * GC + g;
                            const int slot = lin % PW;
                            const WSlot<WL> cur = ring[slot];
                            const int tn = (lin + PW) / GC;
                            ring[slot] = load_w(c0 + tn / NG, wptr[tn % NG], nrow[tn % NG], (lin + PW) % GC);
                            if (g < gc_here) step(cur, ng, g);
                        }
                    }
                }
                __syncthreads();      // every wave is done with chunk c
                stage_store(c + 1);   // (after the last chunk: a harmless rewrite)
            }
        }

        // ---- meet the KP waves' partial sums; wave w finishes accumulator row r = w % 4 ----
        __syncthreads();  // every wave is done with the staged activations
        constexpr int kItems = NG + (kRowBias ? 1 : 0);
        float* mine = red + static_cast<size_t>(wv) * kItems * 4 * kWave;
#pragma unroll
        for (int i = 0; i < NG; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[(i * 4 + r) * kWave + lane] = acc[i][r];
        if (kRowBias) {
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[(NG * 4 + r) * kWave + lane] = sxt[r];
        }
        __syncthreads();
        const int rr = wv & 3;
        auto total = [&](int item) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < KP; ++w)
                v += red[((static_cast<size_t>(w) * kItems + item) * 4 + rr) * kWave + lane];
            return v;
        };
        const int nout = a.swiglu ? N / 2 : N;
        const int m = mt0 + 4 * q + rr;
        const float bias = kRowBias ? F::kBias * total(NG) : 0.f;
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            if (KP > 4 && (i & 1) != (wv >> 2) && NG > 1) continue;   // 8 waves: split the tiles
            if (KP > 4 && NG == 1 && wv >= 4) continue;
            const int n = (tile0 + i) * 16 + j;
            const bool ok = m < r1 && n < N;
            float v = (total(i) + bias) * row_scale[i];
            if (a.swiglu) {
                // columns (2i, 2i+1) = (gate_i, up_i) sit in adjacent lanes
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

// ---- wave-private form (tile-major weights) -------------------------------------------------
// The form above shares each staged activation chunk among the waves of a block and pays two
// block barriers per chunk; with four waves splitting K that also caps a CU at a few waves.
// Here a wave owns its work outright: NG tiles of 16 weight rows times one contiguous K slice,
// its own LDS region for the activations of that slice (256 k-values at a time, loaded one
// chunk ahead into registers), its own ring of weight loads.  Nothing synchronises inside the
// K loop; the KP = 1 << kp_shift waves that share a tile group meet once, in LDS, at the end.
// A block is kSwWaves waves = kSwWaves / KP tile groups.
constexpr int kSwWaves = 8;
constexpr int kSwChunk = 256;                       // k-values per staged chunk
constexpr int kSwStride = kSwChunk / 8 + 1;         // 16-byte vectors per staged row (padded)
constexpr int kSwRegion = 16 * kSwStride;           // vectors per wave region

struct WOne {
    u32x4_t w;
    uint16_t gs;
};

// MT row tiles of 16 per pass: a decoded weight fragment then feeds MT MFMAs, so a batch of 17
// to 64 rows decodes the weights half as often.  The staged chunk shrinks by MT (the region and
// the staging registers keep their size), so MT = 2 is the limit for int4 (one 128-k block).
// Eight tiles per wave take the 128-k chunk with 16-row passes too: half the staging registers
// pay for the second four accumulators and weight pointers.
template <int MT, int NG>
struct SwGeom {
    static constexpr int chunk = kSwChunk / (MT == 1 && NG == 8 ? 2 : MT);   // k-values per staged chunk
    static constexpr int stride = chunk / 8 + 1;        // 16-byte vectors per staged row (padded)
    static constexpr int staged = 16 * MT * stride;     // vectors of a staged chunk
    static constexpr int meet = (NG + 1) * kWave;       // vectors of a row tile's partial sums (+ the row-bias sums)
    static constexpr int region = staged > meet ? staged : meet;   // vectors per wave region
};

template <class F, int NG, int MT, bool GROUPED = false>
__global__ __launch_bounds__(kSwWaves* kWave, NG == 1 && MT == 1 ? 4 : 2) void skinny_wave_kernel(const SkinnyArgs a, const int kp_shift) {
    constexpr int KPL = F::kPerLane, S = F::kSteps;
    constexpr int LK = 4 * KPL;                     // k covered by one wave-wide 16-byte load (a block)
    constexpr int CHUNK = SwGeom<MT, NG>::chunk, STRIDE = SwGeom<MT, NG>::stride, REGION = SwGeom<MT, NG>::region;
    constexpr int CB = CHUNK / LK;                  // blocks per chunk
    constexpr int NS = NG * CB;                     // steps per chunk, tile-major order
    constexpr int PF = NS < 8 ? NS : 8;             // weight loads in flight per lane (deeper rings cost the occupancy that pays more)
    constexpr int CU = NS >= PF ? 1 : PF / NS;      // chunks per trip: ring slots stay compile-time
    constexpr int VPR = CHUNK / 8;                  // staged vectors per row
    constexpr int RPL = kWave / VPR;                // rows one wave-wide staging load covers
    constexpr int SV = 16 * MT / RPL;               // staged vectors per lane and chunk
    constexpr int ROWS = 16 * MT;                   // rows per pass
    constexpr bool kBiased = F::kBias != 0.f;
    constexpr bool kRowBias = kBiased && !F::kGroupScale;
    static_assert(CB >= 1 && (NS % PF == 0 || PF % NS == 0) && (SV == 8 || SV == 4), "ring and staging shapes");
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int j = lane & 15, q = lane >> 4;
    u32x4_t* lds_a = reinterpret_cast<u32x4_t*>(smem) + wv * REGION;
    float* red = reinterpret_cast<float*>(smem);
    constexpr int kRegionF = REGION * 4;
    static_assert((NG + (kRowBias ? 1 : 0)) * 4 * kWave <= kRegionF, "a wave's partial sums of one row tile fit its region");
    const int KP = 1 << kp_shift;
    const int ks = wv & (KP - 1);
    const int N = a.N, K = a.K;
    // (GROUPED: blockIdx.y is the problem — an expert — with its rows offsets[p] .. offsets[p + 1],
    // its weights and scales one stride further, its activation rows gathered by route.  A compile-
    // time case: every scalar instruction ahead of the first weight request delays it, four waves
    // per SIMD walk this prologue at once)
    const int p = GROUPED ? blockIdx.y : 0;
    const int r0 = GROUPED ? a.offsets[p] : (a.m_split ? blockIdx.y * ROWS : 0);
    const int r1 = GROUPED ? a.offsets[p + 1] : (a.m_split ? min(a.M, r0 + ROWS) : a.M);
    if (r1 <= r0) return;

    const int T = (N + 15) / 16;
    const int tile0 = (blockIdx.x * (kSwWaves >> kp_shift) + (wv >> kp_shift)) * NG;
    const unsigned char* wbase = GROUPED ? a.w + static_cast<size_t>(p) * a.w_stride : a.w;
    const unsigned char* sbase = GROUPED && a.scale ? a.scale + static_cast<size_t>(p) * a.scale_stride : a.scale;
    const uint16_t* gsbase = reinterpret_cast<const uint16_t*>(sbase);
    const int blk_shift = a.g_shift - (F::kGroupScale ? 7 : 0);
    const int nb = K / LK;
    const int groups = F::kGroupScale ? K >> a.g_shift : 0;
    // this wave's K slice, in whole chunks
    const int nch_all = nb / CB;                    // the launcher takes whole chunks only
    const int per = (nch_all + KP - 1) >> kp_shift;
    const int ch_lo = ks * per;
    const int nch = max(0, min(nch_all, ch_lo + per) - ch_lo);
    const int b_lo = ch_lo * CB;

    const unsigned char* wt[NG];
    const uint16_t* st[NG];
    float row_scale[NG];
    // (one 64-bit product for the wave's first tile; the others are 32-bit steps from it)
    const int tfirst = min(tile0, T - 1);
    const unsigned char* wt0 = wbase + static_cast<size_t>(tfirst) * nb * 1024;
    const uint16_t* st0 = gsbase + static_cast<size_t>(tfirst) * 16 * groups;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int tile = min(tile0 + i, T - 1);
        wt[i] = wt0 + static_cast<unsigned>(tile - tfirst) * static_cast<unsigned>(nb * 1024);
        st[i] = st0 + static_cast<unsigned>(tile - tfirst) * static_cast<unsigned>(16 * groups);
        row_scale[i] = 1.f;
        const int n = min(tile * 16 + j, N - 1);
        if (!F::kGroupScale && sbase)
            row_scale[i] = a.scale_is_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(sbase)[n])
                                           : reinterpret_cast<const float*>(sbase)[n];
    }
    const unsigned lane16 = static_cast<unsigned>(lane) * 16u;
    const uint32_t magic = F::magic();
    const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, u32x4_t{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};

    // step `lin` of chunk c: block lin / NG of the chunk, tile lin % NG — block-major, so the
    // activation fragments of a block are read from LDS once and serve all NG tiles
    // (the ring runs ahead of the arithmetic, so its last trips reach past the wave's K slice:
    // those requests repeat the slice's own last block — a cache hit — instead of fetching the
    // neighbour's blocks a second time)
    const int b_last = max(b_lo, min(nb, b_lo + nch * CB) - 1);
    // Group scales: one load per block for all NG tiles — lane 16 i + j fetches tile i's scale of
    // weight row j — carried in the ring slot of the block's first tile; a tile's step reads its
    // value across the wave.  (A load per tile and step made a third of the kernel's vector-memory
    // instructions, and those, not the bytes, are what a CU's address unit runs out of.)
    // (eight tiles: two such loads per block, with the slots of tiles 0 and 4)
    constexpr int NGS = (NG + 3) / 4;
    const uint16_t* gsp[NGS];
#pragma unroll
    for (int h = 0; h < NGS; ++h) {
        gsp[h] = st[min(4 * h, NG - 1)];
#pragma unroll
        for (int i = 1; i < 4; ++i)
            if (4 * h + i < NG) gsp[h] = (lane >> 4) == i ? st[4 * h + i] : gsp[h];
        if (4 * h + (lane >> 4) >= NG) gsp[h] = st[NG - 1];
    }
    auto load_w = [&](int c, int lin) {
        const int b = min(b_lo + c * CB + lin / NG, b_last);
        WOne sl;
        sl.w = *reinterpret_cast<const u32x4_t*>(wt[lin % NG] + static_cast<size_t>(b) * 1024 + lane16);
        sl.gs = F::kGroupScale && lin % NG % 4 == 0 ? (gsp[lin % NG / 4] + static_cast<size_t>(b >> blk_shift) * 16)[j] : uint16_t(0);
        return sl;
    };

    // staging: a wave-wide load covers whole chunk rows (VPR vectors each) of RPL activation rows
    const int srow = lane / VPR, svec = lane % VPR;

    for (int mt0 = r0; mt0 < r1; mt0 += ROWS) {
        // a pass of at most eight rows stages eight: the activations are re-read by every tile
        // group, so their traffic matters as much as the weights'.  Accumulator rows 8..15 then
        // repeat rows 0..7 and are never stored.
        // (four rows for passes of at most four: a decode batch of three or four requests)
        const int rstage = MT == 1 ? (r1 - mt0 <= 4 ? 4 : r1 - mt0 <= 8 ? 8 : 16) : 16 * MT;
        const int jr = MT == 1 ? (j & (rstage - 1)) : j;
        int arow[SV];   // rows past the problem repeat its last row and are never stored
#pragma unroll
        for (int u = 0; u < SV; ++u) {
            arow[u] = min(mt0 + srow + RPL * u, r1 - 1);
            if (GROUPED && a.act_rows) arow[u] = a.act_rows[arow[u]];
        }
        u32x4_t stg[SV];
        auto stage_load = [&](int c) {
            const int k0 = min((b_lo + min(c, max(nch - 1, 0)) * CB) * LK + svec * 8, K - 8);   // (past the slice: its last chunk again)
#pragma unroll
            for (int u = 0; u < SV; ++u)
                if (RPL * u < rstage)
                    stg[u] = *reinterpret_cast<const u32x4_t*>(a.act + static_cast<size_t>(arow[u]) * K + k0);
        };
        auto stage_store = [&]() {
#pragma unroll
            for (int u = 0; u < SV; ++u)
                if (RPL * u < rstage) lds_a[(srow + RPL * u) * STRIDE + svec] = stg[u];
        };

        f32x4_t acc[MT][NG], sxt[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            sxt[t] = zero4;
#pragma unroll
            for (int i = 0; i < NG; ++i) acc[t][i] = zero4;
        }

        // (the activations first: loads return in order, so staged behind the weight ring they
        // would reach LDS only after the last of its eight loads has come back from HBM)
        WOne ring[PF];
        stage_load(0);
#pragma unroll
        for (int l = 0; l < PF; ++l) ring[l] = load_w(l / NS, l % NS);
        stage_store();

        // The fragments of the current block (read at its first tile) and, for group-scaled
        // biased codes, bias * (the block's activation sums): the sums come from MFMAs against
        // ones and enter every tile's product as its initial accumulator.
        bf16x8_t ax[MT][S];
        f32x4_t sxb[MT];
        int gsb = 0;   // the current block's scales, tile i's in lanes 16 i .. 16 i + 15
        auto step = [&](const WOne& cur, int ng, int blk) {
            if (ng % 4 == 0) gsb = cur.gs;
            if (ng == 0) {
                const int vbase = blk * (LK / 8) + q * S;
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int s = 0; s < S; ++s)
                        ax[t][s] = __builtin_bit_cast(bf16x8_t, lds_a[(t * 16 + jr) * STRIDE + vbase + s]);
                if (kBiased) {
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        if (F::kGroupScale) {
                            f32x4_t sx = zero4;
#pragma unroll
                            for (int s = 0; s < S; ++s) sx = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[t][s], ones, sx, 0, 0, 0);
                            sxb[t] = sx * F::kBias;
                        } else {
#pragma unroll
                            for (int s = 0; s < S; ++s) sxt[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[t][s], ones, sxt[t], 0, 0, 0);
                        }
                    }
                }
            }
            f32x4_t part[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) part[t] = F::kGroupScale && kBiased ? sxb[t] : zero4;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const bf16x8_t bw = __builtin_bit_cast(bf16x8_t, F::decode(cur.w, s, magic));
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    if (F::kGroupScale)
                        part[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[t][s], bw, part[t], 0, 0, 0);
                    else
                        acc[t][ng] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[t][s], bw, acc[t][ng], 0, 0, 0);
                }
            }
            if (F::kGroupScale) {
                const float sc = bf16_bits_to_f32(static_cast<uint16_t>(
                    ng == 0 && NG == 1 ? gsb : __builtin_amdgcn_ds_bpermute((ng % 4 * 16 + j) * 4, gsb)));
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[t][ng][r] = fmaf(sc, part[t][r], acc[t][ng][r]);
            }
        };

        for (int c0 = 0; c0 < nch; c0 += CU) {
            // Issue priority falls with progress: the SIMD's arbiter serves its oldest wave
            // first, so of the two (or four) waves that share a SIMD one would finish its K slice
            // well ahead and then idle at the barrier below; a wave that has fallen behind
            // outranks its neighbours until it has caught up.
            {
                const int quarter = (c0 * 4) / nch;
                if (quarter == 0) __builtin_amdgcn_s_setprio(3);
                else if (quarter == 1) __builtin_amdgcn_s_setprio(2);
                else if (quarter == 2) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
            }
#pragma unroll
            for (int cu = 0; cu < CU; ++cu) {
                const int c = c0 + cu;
                stage_load(c + 1);   // (past the slice: a clamped, unused repeat)
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int lin = 0; lin < NS; ++lin) {
                    const int slot = (cu * NS + lin) % PF;
                    // consume the slot, then refill it (a ring ahead of its next use).  In this
                    // order the old and the new value never live at once, so the slot keeps its
                    // registers around the loop; refilling first makes the compiler copy the ring
                    // at the loop end, which waits for every load in flight.  The scheduling
                    // barriers keep the order (left alone, the scheduler also gathers all loads
                    // of a chunk behind all of its arithmetic).
                    step(ring[slot], lin % NG, lin / NG);   // K is whole chunks: no step is partial
                    __builtin_amdgcn_sched_barrier(0);
                    ring[slot] = load_w(c + (lin + PF) / NS, (lin + PF) % NS);
                    __builtin_amdgcn_sched_barrier(0);
                }
                stage_store();
            }
        }

        // ---- the KP waves of a tile group meet, one row tile at a time; work item (tile i,
        // accumulator row rr) ----
        const int nout = a.swiglu ? N / 2 : N;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
        // (a wave's partial sums go to its own staging region, which no other wave reads before
        // the barrier below: only the second row tile has to wait for the readers of the first)
        if (t > 0) __syncthreads();
        float* mine = red + static_cast<size_t>(wv) * kRegionF;
#pragma unroll
        for (int i = 0; i < NG; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[(i * 4 + r) * kWave + lane] = acc[t][i][r];
        if (kRowBias) {
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[(NG * 4 + r) * kWave + lane] = sxt[t][r];
        }
        __syncthreads();
        const float* grp = red + static_cast<size_t>(wv - ks) * kRegionF;
        auto total = [&](int item, int rr) {
            float v = 0.f;
            for (int w = 0; w < KP; ++w) v += grp[static_cast<size_t>(w) * kRegionF + (item * 4 + rr) * kWave + lane];
            return v;
        };
        for (int id = ks; id < NG * 4; id += KP) {
            const int i = id >> 2, rr = id & 3;
            const int m = mt0 + 16 * t + 4 * q + rr;
            const float bias = kRowBias ? F::kBias * total(NG, rr) : 0.f;
            float rs = row_scale[0];
#pragma unroll
            for (int t = 1; t < NG; ++t) rs = i == t ? row_scale[t] : rs;
            const int n = (tile0 + i) * 16 + j;
            const bool ok = m < r1 && n < N;
            float v = (total(i, rr) + bias) * rs;
            if (a.rope_table) {
                // the projection's bf16 values, then the rotation of qkv_rope_kvwrite_kernel with
                // the same operations and rounding; columns (n, n + 1) sit in adjacent lanes
                const float gb = bf16_bits_to_f32(f32_to_bf16_bits(v));
                const float ub = __int_as_float(__builtin_amdgcn_update_dpp(
                    0, __float_as_int(gb), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
                if ((j & 1) == 0 && ok) {
                    const int dsh = __builtin_ctz(static_cast<unsigned>(a.d));   // head_dim is a power of two
                    const int head = n >> dsh, dd = n & (a.d - 1);
                    const int64_t slot = a.kv_slots[m];
                    if (head < a.hq + a.hk) {
                        const float* tab = a.rope_table + static_cast<size_t>(m) * a.d + (dd >> 1);
                        const float c = tab[0], sn = tab[a.d >> 1];
                        const uint32_t out = pack_bf16x2(gb * c - ub * sn, ub * c + gb * sn);
                        uint16_t* dst = head < a.hq ? a.y + (static_cast<size_t>(m) * a.hq + head) * a.d
                                                    : a.k_pages + (static_cast<size_t>(slot) * a.hk + (head - a.hq)) * a.d;
                        if (head < a.hq || slot >= 0) {
                            if (a.half_out) {
                                dst[dd >> 1] = static_cast<uint16_t>(out & 0xFFFFu);
                                dst[(dd >> 1) + (a.d >> 1)] = static_cast<uint16_t>(out >> 16);
                            } else {
                                *reinterpret_cast<uint32_t*>(dst + dd) = out;
                            }
                        }
                    } else if (slot >= 0) {
                        *reinterpret_cast<uint32_t*>(a.v_pages + (static_cast<size_t>(slot) * a.hk + (head - a.hq - a.hk)) * a.d + dd) =
                            pack_bf16x2(gb, ub);
                    }
                }
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
        __syncthreads();   // the regions go back to staging
    }
}

template <class F, int NG, int MT, bool GROUPED = false>
int launch_wave_cfg(const SkinnyArgs& a, int problems, int kp_shift, hipStream_t stream) {
    constexpr size_t smem = static_cast<size_t>(kSwWaves) * SwGeom<MT, NG>::region * 16;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&skinny_wave_kernel<F, NG, MT, GROUPED>),
        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (attr != hipSuccess) return PIE_HIP_ERR_LAUNCH;
    const int tgroups = ((a.N + 15) / 16 + NG - 1) / NG;
    const int per_block = kSwWaves >> kp_shift;
    const dim3 grid((tgroups + per_block - 1) / per_block, a.m_split ? (a.M + 16 * MT - 1) / (16 * MT) : problems);
    hipLaunchKernelGGL((skinny_wave_kernel<F, NG, MT, GROUPED>), grid, dim3(kSwWaves * kWave), smem, stream, a, kp_shift);
    return launch_status();
}

// Tiles per wave and K split: the most tiles per wave (activation staging and the bias MFMAs
// are paid once per chunk, whatever the tile count) that still gives the machine about eight
// waves per CU.
template <class F, int MT>
int launch_wave_mt(const SkinnyArgs& a, int problems, hipStream_t stream) {
    constexpr int LK = 4 * F::kPerLane;
    const long mult = a.m_split ? (a.M + 16 * MT - 1) / (16 * MT) : problems;
    const long tiles = (a.N + 15) / 16;
    static const int force_ng = [] { const char* e = getenv("PIE_SKINNY_NG"); return e ? atoi(e) : 0; }();
    static const int force_kp = [] { const char* e = getenv("PIE_SKINNY_KP"); return e ? atoi(e) : -1; }();
    // a CU holds one block of eight waves (two with one tile per wave: fewer registers).  Take
    // the most tiles per wave whose K split still puts >= 1100 waves on the machine without
    // going past what is resident at once (a second round of blocks costs more than idle CUs).
    // (eight tiles per wave — half the staged activation bytes per weight byte — for group-scaled
    // int4: gate|up of an 8B model at 64 rows 34.3 -> 30.4 us.  With 16-row passes over 256-k chunks
    // the kernel needed more registers than a wave has and started its loads 6 us late: there it
    // takes 128-k chunks)
    constexpr bool kEight = F::kGroupScale;
    int ng = 1, kp_shift = 0;
    for (int cand = kEight ? 8 : 4; cand >= 1; cand >>= 1) {
        const int cb = (cand == 8 ? SwGeom<MT, 8>::chunk : SwGeom<MT, 4>::chunk) / LK;
        const int nch_all = (a.K / LK + cb - 1) / cb;
        const long groups = (tiles + cand - 1) / cand * mult;
        const long cap = 256L * (cand == 1 && MT == 1 ? 16 : 8);
        int sh = 0;
        while (sh < 3 && (groups << (sh + 1)) <= cap && (2 << sh) <= nch_all) ++sh;
        // (eight tiles only where four waves or fewer share a tile group: over an eighth of K the
        // loop is too short for its prologue and the eight-wave meeting — gate|up at 16 rows 16.4 us
        // with four tiles, 17.9 with eight; at 32 rows, two passes side by side, 25.0 against 20.4)
        if (cand == 8 && sh > 2) continue;
        if ((groups << sh) >= 1100 || cand == 1) {
            ng = cand;
            kp_shift = sh;
            break;
        }
    }
    if (force_ng) ng = force_ng;
    if (force_kp >= 0) kp_shift = force_kp;
    if constexpr (kEight)
        if (ng == 8) return launch_wave_cfg<F, 8, MT>(a, problems, kp_shift, stream);
    switch (ng) {
        case 8:
        case 4: return launch_wave_cfg<F, 4, MT>(a, problems, kp_shift, stream);
        case 2: return launch_wave_cfg<F, 2, MT>(a, problems, kp_shift, stream);
        default: return launch_wave_cfg<F, 1, MT>(a, problems, kp_shift, stream);
    }
}

template <class F>
int launch_wave(const SkinnyArgs& a, int problems, hipStream_t stream) {
    static const int force_mt = [] { const char* e = getenv("PIE_SKINNY_MT"); return e ? atoi(e) : 0; }();
    // dense launches of more than 32 rows: 32-row passes (measured on the 8B shapes: a 48 / 64
    // row decode step 4.63 / 4.88 -> 4.26 / 4.61 ms; at 17..32 rows the shorter chunks cost
    // more than the second pass saves, 3.40 -> 3.47 ms)
    const bool two = force_mt ? force_mt == 2 : (!a.offsets && a.M > 32);
    if (two && a.K % SwGeom<2, 4>::chunk == 0) return launch_wave_mt<F, 2>(a, problems, stream);
    return launch_wave_mt<F, 1>(a, problems, stream);
}

template <class F, int KP, int CK, int NG, int PW, int WL, bool TILED>
int launch_cfg_t(const SkinnyArgs& a, int problems, hipStream_t stream) {
    constexpr bool kRowBias = F::kBias != 0.f && !F::kGroupScale;
    constexpr size_t kStage = static_cast<size_t>(16) * (CK / 8 + 1) * 16;
    constexpr size_t kRed = static_cast<size_t>(KP) * (NG + (kRowBias ? 1 : 0)) * 4 * kWave * sizeof(float);
    constexpr size_t smem = kStage > kRed ? kStage : kRed;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&skinny_kernel<F, KP, CK, NG, PW, WL, TILED>),
        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (attr != hipSuccess) return PIE_HIP_ERR_LAUNCH;
    const int tiles = (a.N + 15) / 16;
    const dim3 grid((tiles + NG - 1) / NG, a.m_split ? (a.M + 15) / 16 : problems);
    hipLaunchKernelGGL((skinny_kernel<F, KP, CK, NG, PW, WL, TILED>), grid, dim3(KP * kWave), smem, stream, a);
    return launch_status();
}

template <class F, int KP, int CK, int NG, int PW, int WL>
int launch_cfg(const SkinnyArgs& a, int problems, hipStream_t stream) {
    return a.tiled ? launch_cfg_t<F, KP, CK, NG, PW, WL, true>(a, problems, stream)
                   : launch_cfg_t<F, KP, CK, NG, PW, WL, false>(a, problems, stream);
}

template <class F>
int launch_skinny(SkinnyArgs a, int problems, hipStream_t stream) {
    constexpr int LK = 4 * F::kPerLane;
    constexpr int CK = 1024;
    if (a.K <= 0 || a.N <= 0 || a.K % (4 * LK) != 0) return PIE_HIP_ERR_UNSUPPORTED;
    if (F::kGroupScale) {
        // group = 128 * 2^i k-values: a 16-byte block per lane quad never straddles two groups
        if (a.G < LK || (a.G & (a.G - 1)) != 0 || a.K % a.G != 0) return PIE_HIP_ERR_UNSUPPORTED;
        a.g_shift = __builtin_ctz(static_cast<unsigned>(a.G));
    }
    if (a.swiglu && (a.N % 2 != 0 || a.beta)) return PIE_HIP_ERR_INVALID;
    if (problems > 65535) return PIE_HIP_ERR_UNSUPPORTED;
    // Dense matrices with more than one 16-row pass: one block per (tile group, pass) instead
    // of a pass loop inside the block.  The passes then read the same weights at about the same
    // time, so all but one of them hit L2 / the 256 MB MALL (measured: batch-64 decode 9.9 ->
    // 9.0 ms per step); beyond the MALL size the loop form keeps HBM traffic at one pass.
    if (!a.offsets && a.M > 16 && a.M <= 16 * 65535 &&
        static_cast<size_t>(a.N) * a.K * F::kBytesPer2K / 2 <= (size_t(256) << 20))
        a.m_split = 1;
    // tiles of 16 weight rows per block: as many as still leave two blocks per CU; with few
    // tiles, eight waves split K instead of four.  Paired loads (whole 128-byte lines per row
    // and wave) when K allows.
    const long tiles = static_cast<long>((a.N + 15) / 16) * (a.m_split ? (a.M + 15) / 16 : problems);
    constexpr int W8 = (CK / (8 * LK) >= 2) ? 2 : 1;   // loads per step with eight waves
    static const bool old_form = getenv("PIE_SKINNY_OLD") != nullptr;
    // dense tile-major launches take the wave-private form (measured, 8B decode steps of 8 / 16 /
    // 32 / 64 rows: 2.43 / 2.78 / 3.42 / 5.18 ms against 2.75 / 2.95 / 4.07 / 5.64); the grouped
    // MoE launches stay with the block-shared form, whose eight tiles per staged chunk halve the
    // activation traffic (30B-A3B, 64 rows: 7.9 against 11.0 ms per step) — except over a short K, below
    if (a.rope_table) return launch_wave<F>(a, problems, stream);   // (entry point checked K)
    if (a.tiled && !a.offsets && !old_form && a.K % kSwChunk == 0) return launch_wave<F>(a, problems, stream);
    // grouped launches over a short K (an expert's down projection: K = 768): one tile per wave over
    // the whole K, no waves to meet — 43.4 against 47.9 us for the 128 experts of a 30B-A3B layer;
    // at K = 2048 (gate|up) the block-shared form keeps its lead, 74.1 against 75.8 us
    if (a.tiled && a.offsets && !old_form && a.K <= 1024 && a.K % kSwChunk == 0)
        return launch_wave_cfg<F, 1, 1, true>(a, problems, 0, stream);
    if (a.K % (8 * LK) == 0) {
        if (tiles / 8 >= 448) return launch_cfg<F, 4, CK, 8, 4, 2>(a, problems, stream);
        if (tiles / 4 >= 448) return launch_cfg<F, 4, CK, 4, 4, 2>(a, problems, stream);
        if (tiles / 2 >= 448) return launch_cfg<F, 4, CK, 2, 4, 2>(a, problems, stream);
        if (a.K % (8 * LK * W8) == 0) return launch_cfg<F, 8, CK, 1, 4, W8>(a, problems, stream);
    }
    if (tiles / 4 >= 448) return launch_cfg<F, 4, CK, 4, 4, 1>(a, problems, stream);
    return launch_cfg<F, 4, CK, 1, 4, 1>(a, problems, stream);
}

// Tile-major weight layout: the 16 bytes lane (j, q) of a wave loads for tile t (rows 16t..16t+15)
// and K block b — byte 64 b + 16 q of row 16 t + j — move to ((t*nb + b)*64 + 16 q + j)*16, so a
// wave's load is 1 KiB contiguous.  One thread per 16-byte block of the destination; rows past N
// are zero.
// int4 (`nibble_pairs`): the eight codes of a 32-bit word also change places — codes 2i and 2i + 1
// go to nibbles i and i + 4 — so that the decode's (nibble i, nibble i + 4) pairs come out in k
// order and the activations are staged as they are stored.
__device__ __forceinline__ uint32_t pair_nibbles(uint32_t v) {
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r |= ((v >> (8 * i)) & 0xFu) << (4 * i);
        r |= ((v >> (8 * i + 4)) & 0xFu) << (4 * i + 16);
    }
    return r;
}
__global__ __launch_bounds__(256) void repack_tiles_kernel(const u32x4_t* __restrict__ src,
                                                           u32x4_t* __restrict__ dst, int N, int nb,
                                                           size_t total, int nibble_pairs) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int lane = static_cast<int>(idx & 63);
    const size_t tb = idx >> 6;
    const int b = static_cast<int>(tb % nb);
    const size_t tile = tb / nb;
    const size_t n = tile * 16 + (lane & 15);
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (n < static_cast<size_t>(N)) v = src[n * (static_cast<size_t>(nb) * 4) + b * 4 + (lane >> 4)];
    if (nibble_pairs) v = u32x4_t{pair_nibbles(v.x), pair_nibbles(v.y), pair_nibbles(v.z), pair_nibbles(v.w)};
    dst[idx] = v;
}
// int4 group scales [N, groups] -> [tile][group][16 rows]
__global__ __launch_bounds__(256) void repack_scale_tiles_kernel(const uint16_t* __restrict__ src,
                                                                 uint16_t* __restrict__ dst, int N,
                                                                 int groups, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int j = static_cast<int>(idx & 15);
    const size_t tg = idx >> 4;
    const int g = static_cast<int>(tg % groups);
    const size_t n = (tg / groups) * 16 + j;
    dst[idx] = n < static_cast<size_t>(N) ? src[n * groups + g] : uint16_t(0);
}

int dispatch_skinny(int format, const SkinnyArgs& a, int problems, hipStream_t st) {
    switch (format) {
        case PIE_HIP_FMT_INT4B8: return launch_skinny<SkInt4>(a, problems, st);
        case PIE_HIP_FMT_INT8: return launch_skinny<SkInt8>(a, problems, st);
        case PIE_HIP_FMT_FP8: return launch_skinny<SkFp8>(a, problems, st);
        case PIE_HIP_FMT_BF16: return launch_skinny<SkBf16>(a, problems, st);
        default: return PIE_HIP_ERR_INVALID;
    }
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_gemm_skinny(int format, const uint16_t* act_bf16, const void* weight,
                                   const void* scale, int scale_is_bf16, int group_size,
                                   uint16_t* y_bf16, int M, int N, int K, int beta, int swiglu,
                                   void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !weight || !y_bf16 || M <= 0) return PIE_HIP_ERR_INVALID;
    if (format != PIE_HIP_FMT_BF16 && !scale) return PIE_HIP_ERR_INVALID;
    SkinnyArgs a{};
    a.act = act_bf16;
    a.w = static_cast<const unsigned char*>(weight);
    a.scale = static_cast<const unsigned char*>(scale);
    a.y = y_bf16;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = group_size;
    a.beta = beta;
    a.swiglu = swiglu ? 1 : 0;
    a.scale_is_bf16 = scale_is_bf16;
    return dispatch_skinny(format, a, 1, static_cast<hipStream_t>(stream));
}

extern "C" int pie_hip_moe_grouped_gemm(int format, const uint16_t* act_bf16,
                                        const int32_t* route_act_rows,
                                        const int32_t* expert_offsets, int num_experts,
                                        int max_rows_per_expert, const void* weights,
                                        size_t weight_stride_bytes, const void* scales,
                                        size_t scale_stride_bytes, int scale_is_bf16,
                                        int group_size, uint16_t* y_bf16, int N, int K, int swiglu,
                                        void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !expert_offsets || !weights || !y_bf16 || num_experts <= 0 ||
        max_rows_per_expert <= 0)
        return PIE_HIP_ERR_INVALID;
    if (format != PIE_HIP_FMT_BF16 && !scales) return PIE_HIP_ERR_INVALID;
    SkinnyArgs a{};
    a.act = act_bf16;
    a.act_rows = route_act_rows;
    a.w = static_cast<const unsigned char*>(weights);
    a.scale = static_cast<const unsigned char*>(scales);
    a.y = y_bf16;
    a.offsets = expert_offsets;
    a.N = N;
    a.K = K;
    a.G = group_size;
    a.swiglu = swiglu ? 1 : 0;
    a.scale_is_bf16 = scale_is_bf16;
    a.w_stride = weight_stride_bytes;
    a.scale_stride = scale_stride_bytes;
    return dispatch_skinny(format, a, num_experts, static_cast<hipStream_t>(stream));
}

// ---- the same two entry points over weights in the tile-major layout ----------------------
extern "C" int pie_hip_gemm_skinny_tiled(int format, const uint16_t* act_bf16, const void* weight,
                                   const void* scale, int scale_is_bf16, int group_size,
                                   uint16_t* y_bf16, int M, int N, int K, int beta, int swiglu,
                                   void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !weight || !y_bf16 || M <= 0) return PIE_HIP_ERR_INVALID;
    if (format != PIE_HIP_FMT_BF16 && !scale) return PIE_HIP_ERR_INVALID;
    SkinnyArgs a{};
    a.act = act_bf16;
    a.w = static_cast<const unsigned char*>(weight);
    a.scale = static_cast<const unsigned char*>(scale);
    a.y = y_bf16;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = group_size;
    a.beta = beta;
    a.swiglu = swiglu ? 1 : 0;
    a.scale_is_bf16 = scale_is_bf16;
    a.tiled = 1;
    return dispatch_skinny(format, a, 1, static_cast<hipStream_t>(stream));
}

// q|k|v projection over tile-major weights with RoPE and the KV write in the epilogue (more rows
// than the GEMV form takes): values of pie_hip_gemm_skinny_tiled followed by
// pie_hip_qkv_rope_kvwrite with interleaved = pairing (1 or 2) and no q/k norm.
extern "C" int pie_hip_qkv_rope_skinny_tiled(int format, const uint16_t* act_bf16, const void* weight,
                                             const void* scale, int scale_is_bf16, int group_size,
                                             int M, int K, const float* rope_table,
                                             const int64_t* kv_slots, uint16_t* q_out,
                                             uint16_t* k_pages, uint16_t* v_pages, int num_q_heads,
                                             int num_kv_heads, int head_dim, int pairing, void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !weight || !rope_table || !kv_slots || !q_out || !k_pages || !v_pages || M <= 0 ||
        num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || (pairing != 1 && pairing != 2))
        return PIE_HIP_ERR_INVALID;
    if (format != PIE_HIP_FMT_BF16 && !scale) return PIE_HIP_ERR_INVALID;
    if ((head_dim & (head_dim - 1)) != 0 || head_dim % 16 != 0 || K % kSwChunk != 0) return PIE_HIP_ERR_UNSUPPORTED;
    SkinnyArgs a{};
    a.act = act_bf16;
    a.w = static_cast<const unsigned char*>(weight);
    a.scale = static_cast<const unsigned char*>(scale);
    a.y = q_out;
    a.M = M;
    a.N = (num_q_heads + 2 * num_kv_heads) * head_dim;
    a.K = K;
    a.G = group_size;
    a.scale_is_bf16 = scale_is_bf16;
    a.tiled = 1;
    a.rope_table = rope_table;
    a.kv_slots = kv_slots;
    a.k_pages = k_pages;
    a.v_pages = v_pages;
    a.hq = num_q_heads;
    a.hk = num_kv_heads;
    a.d = head_dim;
    a.half_out = pairing == 2;
    return dispatch_skinny(format, a, 1, static_cast<hipStream_t>(stream));
}

extern "C" int pie_hip_moe_grouped_gemm_tiled(int format, const uint16_t* act_bf16,
                                        const int32_t* route_act_rows,
                                        const int32_t* expert_offsets, int num_experts,
                                        int max_rows_per_expert, const void* weights,
                                        size_t weight_stride_bytes, const void* scales,
                                        size_t scale_stride_bytes, int scale_is_bf16,
                                        int group_size, uint16_t* y_bf16, int N, int K, int swiglu,
                                        void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !expert_offsets || !weights || !y_bf16 || num_experts <= 0 ||
        max_rows_per_expert <= 0)
        return PIE_HIP_ERR_INVALID;
    if (format != PIE_HIP_FMT_BF16 && !scales) return PIE_HIP_ERR_INVALID;
    SkinnyArgs a{};
    a.act = act_bf16;
    a.act_rows = route_act_rows;
    a.w = static_cast<const unsigned char*>(weights);
    a.scale = static_cast<const unsigned char*>(scales);
    a.y = y_bf16;
    a.offsets = expert_offsets;
    a.N = N;
    a.K = K;
    a.G = group_size;
    a.swiglu = swiglu ? 1 : 0;
    a.scale_is_bf16 = scale_is_bf16;
    a.tiled = 1;
    a.w_stride = weight_stride_bytes;
    a.scale_stride = scale_stride_bytes;
    return dispatch_skinny(format, a, num_experts, static_cast<hipStream_t>(stream));
}

namespace {
int repack_tiles(const void* src, void* dst, int N, size_t row_bytes, void* stream, int nibble_pairs) {
    if (!src || !dst || N <= 0 || row_bytes == 0) return PIE_HIP_ERR_INVALID;
    if (row_bytes % 64 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    const int nb = static_cast<int>(row_bytes / 64);
    const size_t total = static_cast<size_t>((N + 15) / 16) * nb * 64;
    if ((total + 255) / 256 > 0x7FFFFFFFull) return PIE_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(pie_hip::repack_tiles_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256),
                       0, static_cast<hipStream_t>(stream), static_cast<const pie_hip::u32x4_t*>(src),
                       static_cast<pie_hip::u32x4_t*>(dst), N, nb, total, nibble_pairs);
    return pie_hip::launch_status();
}
}  // namespace

extern "C" int pie_hip_repack_mfma_tiles(const void* src, void* dst, int N, size_t row_bytes,
                                         void* stream) {
    return repack_tiles(src, dst, N, row_bytes, stream, 0);
}

extern "C" int pie_hip_repack_mfma_tiles_int4(const void* src, void* dst, int N, size_t row_bytes,
                                              void* stream) {
    return repack_tiles(src, dst, N, row_bytes, stream, 1);
}

extern "C" int pie_hip_repack_scale_tiles(const uint16_t* src, uint16_t* dst, int N, int groups,
                                          void* stream) {
    if (!src || !dst || N <= 0 || groups <= 0) return PIE_HIP_ERR_INVALID;
    const size_t total = static_cast<size_t>((N + 15) / 16) * groups * 16;
    hipLaunchKernelGGL(pie_hip::repack_scale_tiles_kernel, dim3(static_cast<unsigned>((total + 255) / 256)),
                       dim3(256), 0, static_cast<hipStream_t>(stream), src, dst, N, groups, total);
    return pie_hip::launch_status();
}
