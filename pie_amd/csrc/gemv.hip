// Weight-streaming GEMV / skinny GEMM for decode on gfx950, one kernel template
// for every weight storage format of the forward pass:
//
//   int4b8  W4A16, group scales    driver/cuda/src/kernels/dequant_wna16.cu:11-38, :96-110
//   int8    W8A16, per-row scale   driver/cuda/src/kernels/argmax.cu:846-854 (fused order:
//                                  scale applied once after the fp32 sum)
//   fp8     e4m3fn, per-row scale  driver/cuda/src/kernels/dequant_fp8.cu:25-39
//   bf16    plain                  gemm_act_x_w bf16 path, driver/cuda/src/ops/gemm.hpp:152-160
//
// y[m, n] = bf16( beta*y[m, n] + sum_k act[m, k] * w(n, k) ), fp32 accumulation.
//
// HBM-bound design (the N*K weight bytes dominate):
//   * the grid is sized to the machine, not to the problem: `waves_per_simd`
//     resident waves on each of the 1024 SIMDs, every wave owning one contiguous,
//     balanced slice of the output rows, so all CUs start and finish together;
//   * a wave walks its slice R rows at a time; every lane streams 16-byte pieces of
//     each row, so one wave instruction covers 1 KiB of a row, fully coalesced.
//     Loads are branch-free and run a ring of two work units (R rows x one 1 KiB chunk)
//     ahead of the arithmetic, so 2R independent 16 B loads per lane are in flight
//     while the previous unit is being reduced;
//   * the first units are requested before the activation row is staged, so the
//     HBM latency of the weights overlaps the LDS staging; the activations themselves
//     are requested even earlier (vector memory operations return in order);
//   * activations are staged once per block into LDS in exactly the order the
//     format's in-register decode produces weights, laid out so a lane's 16 B LDS
//     reads are conflict free;
//   * int4: nibbles become bf16 by OR-ing the exponent of 128.0 onto them,
//     ((w >> 4j) & 0x000F000F) | 0x43004300 = (128+n_j, 128+n_{j+4}), and the dot
//     product runs on v_dot2_f32_bf16 from an accumulator preset to -136*sum(x),
//     which makes the result sum x*(n-8) exactly as the format defines; the bf16
//     group scale multiplies each lane's 32-weight partial sum;
//   * int8: bytes are flipped to offset binary (w ^ 0x80808080) so the byte->f32
//     conversion instruction decodes them, with -128*sum(x) preset the same way;
//   * fp8: the packed e4m3 -> f32 conversion instruction decodes two weights each;
//   * bf16: weights feed v_dot2_f32_bf16 directly;
//   * a wave64 butterfly finishes the row (one shared butterfly for the 2-4 rows of a
//     step when there is a single activation row); the lane that stores an output has
//     prefetched the residual / row scale it needs with the unit's loads.
#include <type_traits>
#include <hip/hip_ext.h>

#include "common.hip.h"

namespace pie_hip {
namespace {

constexpr int kBlock = 512;  // 8 waves: two per SIMD of a CU, so one block's prologue serves the whole CU
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kNumCU = 256;
constexpr int kUnits = 2;   // work units in flight per wave

typedef float f32x2_t __attribute__((ext_vector_type(2)));

// ---- weight formats ---------------------------------------------------------
// WPP: weights in one 16-byte piece.  XV: 16-byte LDS vectors of staged activations
// a lane reads per piece.  stage(): the XV vectors for the piece starting at k0, from
// the bf16 activation row.  dot(): p += sum over the piece of x*w(raw).  sum_x():
// the sum of the staged activations of a piece (only when kBias != 0).

// Reads activations for staging; with `norm_w` set it applies the RMSNorm that precedes the
// projection on the fly: bf16(x * inv_rms * w), the value and the single rounding of
// rmsnorm_bf16_kernel (driver/cuda/src/kernels/rmsnorm.cu:47-52), so fusing the norm into the
// GEMV leaves every bit of the result unchanged.
struct ActLoader {
    const uint16_t* row;
    const uint16_t* norm_w;
    float inv_rms;
    __device__ __forceinline__ uint32_t norm2(uint32_t x, uint32_t w) const {
        return pack_bf16x2(bf16_lo(x) * inv_rms * bf16_lo(w), bf16_hi(x) * inv_rms * bf16_hi(w));
    }
    __device__ __forceinline__ u32x4_t load8(int k) const {
        u32x4_t v = *reinterpret_cast<const u32x4_t*>(row + k);
        if (norm_w) {
            const u32x4_t w = *reinterpret_cast<const u32x4_t*>(norm_w + k);
            v = u32x4_t{norm2(v.x, w.x), norm2(v.y, w.y), norm2(v.z, w.z), norm2(v.w, w.w)};
        }
        return v;
    }
    __device__ __forceinline__ u32x2_t load4(int k) const {
        u32x2_t v = *reinterpret_cast<const u32x2_t*>(row + k);
        if (norm_w) {
            const u32x2_t w = *reinterpret_cast<const u32x2_t*>(norm_w + k);
            v = u32x2_t{norm2(v.x, w.x), norm2(v.y, w.y)};
        }
        return v;
    }
};

struct FmtInt4 {
    static constexpr int WPP = 32, XV = 4;
    static constexpr bool kGroupScale = true, kRowScale = false;
    static constexpr float kBias = -136.f;
    // vector i holds word i's 8 activations as pairs (0,4)(1,5)(2,6)(3,7)
    static __device__ __forceinline__ u32x4_t stage(const ActLoader& ld, int k0, int i) {
        const u32x4_t v = ld.load8(k0 + 8 * i);
        u32x4_t p;
        p.x = (v.x & 0xFFFFu) | (v.z << 16);
        p.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
        p.z = (v.y & 0xFFFFu) | (v.w << 16);
        p.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
        return p;
    }
    static __device__ __forceinline__ float sum_x(const u32x4_t* xs) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < XV; ++i)
            s += bf16_lo(xs[i].x) + bf16_hi(xs[i].x) + bf16_lo(xs[i].y) + bf16_hi(xs[i].y) +
                 bf16_lo(xs[i].z) + bf16_hi(xs[i].z) + bf16_lo(xs[i].w) + bf16_hi(xs[i].w);
        return s;
    }
    // the same staging from a register: v = activations 8*sv .. 8*sv + 7 of a row
    static __device__ __forceinline__ void stage_vec(u32x4_t* xrow, int sv, const u32x4_t v) {
        const int c = sv >> 8, l = (sv & 255) >> 2, i = sv & 3;
        u32x4_t p;
        p.x = (v.x & 0xFFFFu) | (v.z << 16);
        p.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
        p.z = (v.y & 0xFFFFu) | (v.w << 16);
        p.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
        xrow[(c * XV + i) * kWave + l] = p;
    }
    static __device__ __forceinline__ float dot(const u32x4_t w, const u32x4_t* xs, float p) {
        const uint32_t kMask = 0x000F000Fu;
        uint32_t k128 = 0x43004300u;  // (128.0bf16, 128.0bf16), kept in a VGPR for and_or
        asm volatile("" : "+v"(k128));
        // all sixteen pairs first, then the dot products: a dot product issued right behind the
        // instruction that made its operand costs a wait state
        uint32_t t[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t v = w[i];
            t[4 * i + 0] = and_or(v, kMask, k128);
            t[4 * i + 1] = and_or(v >> 4, kMask, k128);
            t[4 * i + 2] = and_or(v >> 8, kMask, k128);
            t[4 * i + 3] = and_or(v >> 12, kMask, k128);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p = dot2_bf16(xs[i].x, t[4 * i + 0], p);
            p = dot2_bf16(xs[i].y, t[4 * i + 1], p);
            p = dot2_bf16(xs[i].z, t[4 * i + 2], p);
            p = dot2_bf16(xs[i].w, t[4 * i + 3], p);
        }
        return p;
    }
};

struct FmtBf16 {
    static constexpr int WPP = 8, XV = 1;
    static constexpr bool kGroupScale = false, kRowScale = false;
    static constexpr float kBias = 0.f;
    static __device__ __forceinline__ u32x4_t stage(const ActLoader& ld, int k0, int) {
        return ld.load8(k0);
    }
    static __device__ __forceinline__ float sum_x(const u32x4_t*) { return 0.f; }
    static __device__ __forceinline__ void stage_vec(u32x4_t* xrow, int sv, const u32x4_t v) {
        xrow[sv] = v;   // (chunk sv / 64, lane sv % 64)
    }
    static __device__ __forceinline__ float dot(const u32x4_t w, const u32x4_t* xs, float p) {
        p = dot2_bf16(xs[0].x, w.x, p);
        p = dot2_bf16(xs[0].y, w.y, p);
        p = dot2_bf16(xs[0].z, w.z, p);
        p = dot2_bf16(xs[0].w, w.w, p);
        return p;
    }
};

// 16 weights per piece, activations staged as f32 in natural order.
struct FmtF32Act {
    static constexpr int WPP = 16, XV = 4;
    static __device__ __forceinline__ u32x4_t stage(const ActLoader& ld, int k0, int i) {
        const u32x2_t v = ld.load4(k0 + 4 * i);
        return u32x4_t{v.x << 16, v.x & 0xFFFF0000u, v.y << 16, v.y & 0xFFFF0000u};
    }
    static __device__ __forceinline__ float sum_x(const u32x4_t* xs) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < XV; ++i)
            s += __uint_as_float(xs[i].x) + __uint_as_float(xs[i].y) + __uint_as_float(xs[i].z) +
                 __uint_as_float(xs[i].w);
        return s;
    }
    static __device__ __forceinline__ void stage_vec(u32x4_t* xrow, int sv, const u32x4_t v) {
        const int c = sv >> 7, l = (sv & 127) >> 1, h = sv & 1;
        xrow[(c * XV + 2 * h) * kWave + l] = u32x4_t{v.x << 16, v.x & 0xFFFF0000u, v.y << 16, v.y & 0xFFFF0000u};
        xrow[(c * XV + 2 * h + 1) * kWave + l] = u32x4_t{v.z << 16, v.z & 0xFFFF0000u, v.w << 16, v.w & 0xFFFF0000u};
    }
};

// Row scale stored as f32 (SB = false) or bf16 (SB = true).
template <bool SB>
struct RowScale {
    static __device__ __forceinline__ float load(const void* p, int row) {
        if (SB) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[row]);
        return static_cast<const float*>(p)[row];
    }
};

template <bool SB>
struct FmtInt8 : FmtF32Act, RowScale<SB> {
    static constexpr bool kGroupScale = false, kRowScale = true;
    static constexpr float kBias = -128.f;
    static __device__ __forceinline__ float dot(const u32x4_t w, const u32x4_t* xs, float p) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t u = w[i] ^ 0x80808080u;  // int8 -> offset binary
            p = fmaf(__uint_as_float(xs[i].x), static_cast<float>(u & 0xFFu), p);
            p = fmaf(__uint_as_float(xs[i].y), static_cast<float>((u >> 8) & 0xFFu), p);
            p = fmaf(__uint_as_float(xs[i].z), static_cast<float>((u >> 16) & 0xFFu), p);
            p = fmaf(__uint_as_float(xs[i].w), static_cast<float>(u >> 24), p);
        }
        return p;
    }
};

template <bool SB>
struct FmtFp8 : FmtF32Act, RowScale<SB> {
    static constexpr bool kGroupScale = false, kRowScale = true;
    static constexpr float kBias = 0.f;
    static __device__ __forceinline__ float dot(const u32x4_t w, const u32x4_t* xs, float p) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[i], false);
            const f32x2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[i], true);
            p = fmaf(__uint_as_float(xs[i].x), lo.x, p);
            p = fmaf(__uint_as_float(xs[i].y), lo.y, p);
            p = fmaf(__uint_as_float(xs[i].z), hi.x, p);
            p = fmaf(__uint_as_float(xs[i].w), hi.y, p);
        }
        return p;
    }
};

template <int R>
struct Unit {
    u32x4_t w[R];
    uint16_t gs[R];  // group scale (int4), one load per row ...
    uint16_t gsv;    // ... or one load for the unit: lane l holds (row l / gpc, group l % gpc of the chunk)
    uint16_t prev;   // y element this lane may add to (lane = r*M + m), for beta = 1
    float rs;        // row scale for that lane's row (int8 / fp8)
    float rs2;       // swiglu epilogue: row scale of the pair's second (up) row
    float rc, rsn;   // qkv epilogue: cos / sin of this lane's (token, pair)
    int slot;        // qkv epilogue: KV slot of this lane's token (< 0: none)
};

struct GemvArgs {
    const uint16_t* act;
    const u32x4_t* w;
    const uint16_t* gscale;  // bf16 [N, K/G]        (int4)
    const void* rscale;      // f32 or bf16 [N]      (int8 / fp8)
    uint16_t* y;
    int N, K, G, beta;
    const uint16_t* norm_w;  // bf16 [K] or null: RMSNorm applied to act while staging
    float eps;
    int swiglu;  // 1: rows are (gate_i, up_i) pairs; y[m, i] = silu(bf16 g) * bf16 u, y is [M, N/2]
    // qkv epilogue (rope_table != null): rows are the fused q | k | v projection; pairs
    // (2i, 2i+1) of a q / k head are rotated (interleaved RoPE), q goes to y = q_out
    // [M, hq*d], k and v to the token's slot of the paged pools
    const float* rope_table;  // f32 [M, d]: cos at [i], sin at [d/2 + i]
    const int64_t* kv_slots;  // [M], < 0: no KV slot
    uint16_t* k_pages;
    uint16_t* v_pages;
    int hq, hk, d;
    int g_shift;  // log2(G) when G is a power of two, else -1 (set by dispatch)
    // qkv epilogue: 1 when the q / k rows were re-ordered at load so that rows (2i, 2i+1) of a
    // head hold the half-split pair (i, i + d/2); the rotated pair goes back to those positions
    int half_out;
    // lm_head form: when set, every lane that finishes outputs also keeps the largest bf16 value
    // it stored and its row; slot (m, wave * R + r) of amax_part receives the pair (value bits in
    // the high word, row in the low word), for a second small kernel to reduce
    unsigned long long* amax_part;
    // a wave's row slice (set by launch): the first slice_r waves take slice_q + 1 rows (or row
    // pairs), the others slice_q
    int slice_q, slice_r;
    int groups_per_row;   // K / G (int4), set by launch
    // Output projection of a decode step with the attention's split merge in its prologue
    // (mg_part_o != null, act unused): the activation row m is the merged, normalised and
    // bf16-rounded attention output of row m, computed from the split kernel's partial results
    // exactly as attn_decode_merge_kernel computes it.  K = mg_hq * mg_d.
    const float* mg_part_o;      // [M, hq, nsplit, d] f32
    const float* mg_part_ml;     // [M, hq, nsplit, 2] f32 (max, sum)
    const int32_t* mg_row_len;   // visible keys per row
    int mg_nsplit, mg_units_per_split, mg_hq, mg_d;
};

// attn_decode_merge_kernel's arithmetic for the eight output dimensions d0 .. d0 + 7 of one
// (row, head), from values already in registers: po[s][0..7] the partial outputs and ml[s] the
// (max, sum) pair of split s, ns the splits the row really has (<= NSP <= 8).  Same operations in
// the same order — the weights exp2(m_s - max), the normaliser in the order of that kernel's
// wave reduction (lanes s and s + 4 first, then + 2, then + 1), four interleaved accumulators
// over the splits, one division — so the packed result is what that kernel stores, bit for bit.
template <int NSP>
__device__ __forceinline__ u32x4_t merge_splits(const f32x4_t (&po)[NSP][2], const f32x2_t (&ml)[NSP], int ns) {
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < NSP; ++s) mx = s < ns ? fmaxf(mx, ml[s][0]) : mx;
    const float safe = (mx == -INFINITY) ? 0.f : mx;
    float w[8], lv[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        w[s] = 0.f;
        lv[s] = 0.f;
        if (s < NSP) {
            if (s < ns) {
                w[s] = exp2f(ml[s][0] - safe);
                lv[s] = ml[s][1] * w[s];
            }
        }
    }
    const float ls = ((lv[0] + lv[4]) + (lv[2] + lv[6])) + ((lv[1] + lv[5]) + (lv[3] + lv[7]));
    float out[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
        int done = 0;
#pragma unroll
        for (int b = 0; b + 4 <= NSP; b += 4) {
            if (b + 4 <= ns) {
                acc0 = fmaf(po[b][e >> 2][e & 3], w[b], acc0);
                acc1 = fmaf(po[b + 1][e >> 2][e & 3], w[b + 1], acc1);
                acc2 = fmaf(po[b + 2][e >> 2][e & 3], w[b + 2], acc2);
                acc3 = fmaf(po[b + 3][e >> 2][e & 3], w[b + 3], acc3);
                done = b + 4;
            }
        }
#pragma unroll
        for (int b = 0; b < NSP; ++b)
            if (b >= done && b < ns) acc0 = fmaf(po[b][e >> 2][e & 3], w[b], acc0);
        const float ov = (acc0 + acc1) + (acc2 + acc3);
        out[e] = ls > 0.f ? ov / ls : 0.f;
    }
    return u32x4_t{pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3]), pack_bf16x2(out[4], out[5]),
                   pack_bf16x2(out[6], out[7])};
}

// ROPE: the q|k|v epilogue (rotation + KV write); its per-lane cos / sin / slot ride with every
// unit's loads like the residual does, so the epilogue itself issues no loads.
// GS1: the unit's int4 group scales come with one load (see issue()).  PJ: activation vectors
// (8 values) a thread holds per row in the register prologue — 1 covers K <= 4096, the other
// value min(4, 8 / M); a vector-memory instruction costs the CU's address unit sixteen cycles whatever
// it fetches and every instruction ahead of the first weight request delays it, so short rows
// get a prologue with no idle trips.
// MG: 0, or the most splits (4 or 8) of the attention-merge prologue (PJ = 1, no norm, no RoPE).
template <class F, int R, int M, bool ROPE, bool GS1, int PJ, int MG = 0>
__global__ __launch_bounds__(kBlock) void gemv_kernel(const GemvArgs a) {
    constexpr int WPP = F::WPP, XV = F::XV;
    constexpr int kChunkK = kWave * WPP;  // weights covered by one wave-wide 16 B load
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform -> SGPR
    const int N = a.N, K = a.K;
    const int nchunks = (K + kChunkK - 1) / kChunkK;
    const int vec_per_m = nchunks * XV * kWave;
    const int row_stride_v4 = K / WPP;
    const int groups_per_row = a.groups_per_row;

    u32x4_t* lds_x = reinterpret_cast<u32x4_t*>(smem);               // [M][nchunks][XV][64]
    float* lds_sx = reinterpret_cast<float*>(lds_x + M * vec_per_m);  // [M][nchunks][64]

    // Balanced contiguous row slice of this wave.
    const long long total_waves = static_cast<long long>(gridDim.x) * kWavesPerBlock;
    const long long wg = static_cast<long long>(blockIdx.x) * kWavesPerBlock + wv;
    // (slices fall on even rows for the swiglu epilogue, which pairs rows 2i and 2i+1)
    const bool pairs = a.swiglu || ROPE;
    const int gran = pairs ? 2 : 1;
    const int wgi = static_cast<int>(wg);
    const int row_begin = (wgi * a.slice_q + min(wgi, a.slice_r)) * gran;
    const int row_end = row_begin + (a.slice_q + (wgi < a.slice_r ? 1 : 0)) * gran;
    const int ngroups = (row_end - row_begin + R - 1) / R;
    const int nunits = ngroups * nchunks;

    // Branch-free loads: lanes past K re-read lane 0's piece and are masked out in compute;
    // rows past the slice re-read its last row and are dropped at the store.
    // (`live` false: a unit past the end of the slice; every lane then re-reads one 16-byte
    // piece, so the request costs a single cache line)
    // int4 group scales: when the R rows' groups of one chunk fit a wave (gpc groups per chunk and
    // row, R * gpc <= 64) one load fetches them all and the lanes pick theirs with a lane
    // permute — a vector-memory instruction occupies the CU's address unit for sixteen cycles
    // whatever it fetches, and the eight waves of a CU issue their first units at the same time
    constexpr bool one_gs = GS1 && F::kGroupScale;
    const int gpc_shift = one_gs ? __builtin_ctz(static_cast<unsigned>(kChunkK)) - a.g_shift : 0;
    auto issue = [&](Unit<R>& u, int g, int c, bool live) {
        const int kbase = c * kChunkK + lane * WPP;
        const bool valid = kbase < K;
        const int piece = (valid && live) ? c * kWave + lane : 0;
        int gidx = 0;   // scale group of this lane's piece
        if constexpr (F::kGroupScale)
            gidx = (valid && live) ? (a.g_shift >= 0 ? kbase >> a.g_shift : kbase / a.G) : 0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = live ? min(row_begin + g * R + r, row_end - 1) : row_begin;
            u.w[r] = __builtin_nontemporal_load(a.w + static_cast<size_t>(row) * row_stride_v4 +
                                                piece);
            if constexpr (F::kGroupScale && !one_gs)
                u.gs[r] = a.gscale[static_cast<size_t>(row) * groups_per_row + gidx];
        }
        if constexpr (one_gs) {
            {
                const int lr = min(lane >> gpc_shift, R - 1);
                const int row = live ? min(row_begin + g * R + lr, row_end - 1) : row_begin;
                const int grp = live ? min(((c * kChunkK) >> a.g_shift) + (lane & ((1 << gpc_shift) - 1)), groups_per_row - 1) : 0;
                u.gsv = a.gscale[static_cast<size_t>(row) * groups_per_row + grp];
            }
        }
        // Every unit prefetches what the lane that finishes an output needs, so the
        // epilogue never stalls the pipeline (only the last chunk's values are used).
        // (branch-free on purpose: a branch around loads would merge the outstanding-load state
        // of both arms and force the next wait to drain the whole pipeline)
        const int per = pairs ? (R / 2) * M : R * M;
        const int li = lane < per ? lane / M : 0;
        const int lm = lane < per ? lane % M : 0;
        // (a wave whose slice is empty has no live unit: row_end - 1 may be -1 there)
        const int lrow = !live ? row_begin
                         : pairs ? min(row_begin + g * R + 2 * li, row_end - 2)
                                 : min(row_begin + g * R + li, row_end - 1);
        u.prev = a.y[pairs ? 0 : static_cast<size_t>(lm) * N + lrow];
        if constexpr (F::kRowScale) {
            u.rs = F::load(a.rscale, lrow);
            u.rs2 = F::load(a.rscale, min(lrow + 1, N - 1));
        }
        if constexpr (ROPE) {
            const int dd = lrow & (a.d - 1);   // head_dim is a power of two here
            const float* tab = a.rope_table + static_cast<size_t>(lm) * a.d + (dd >> 1);
            u.rc = tab[0];
            u.rsn = tab[a.d >> 1];
            u.slot = static_cast<int>(a.kv_slots[lm]);
        }
    };

    // kUnits work units are requested before the activations are staged and stay in flight
    // from then on.  (Measured: deeper rings than two lose on every decode shape of an 8B
    // model, 1.84 / 1.94 / 2.03 ms per decode step for 2 / 3 / 4 units.)
    float best_v = -INFINITY;   // lm_head form: largest output of this lane so far, and its row
    int best_i = 0x7FFFFFFF;
    Unit<R> un[kUnits];
    int ug[kUnits], uc[kUnits];
    int next_g = 0, next_c = 0, issued = 0;
    auto issue_next = [&](Unit<R>& u, int& og, int& oc) {
        og = next_g;
        oc = next_c;
        issue(u, next_g, next_c, issued < nunits);
        ++issued;
        if (++next_c == nchunks) {
            next_c = 0;
            ++next_g;
        }
    };
    // Activation rows short enough to sit in registers (8 vectors of 16 bytes per thread) are
    // requested before the weights: memory operations return in order, so a prologue that
    // loads activations after the first weight requests starts only when those have arrived
    // from HBM.  Longer rows keep the two-pass prologue below.
    constexpr int kPreJ = PJ > 0 ? PJ : 1;
    const int nv = K / 8, nvp = nchunks * (kChunkK / 8);   // real / padded source vectors per row
    constexpr bool pre = PJ > 0;   // (the launch picks PJ so that the row fits: nvp <= PJ * kBlock)
    float inv_rms[M];
#pragma unroll
    for (int m = 0; m < M; ++m) inv_rms[m] = 1.f;
    if constexpr (pre) {
        u32x4_t xr[kPreJ * M], nw[kPreJ];
        constexpr int NSP = MG > 0 ? MG : 1;
        f32x4_t mg_po[M][NSP][2];
        f32x2_t mg_ml[M][NSP];
        int mg_ns[M];
        if constexpr (MG > 0) {
            // every split slot of the row is requested, used or not (slots past the row's own
            // splits repeat its last configured slot and never enter the arithmetic)
            static_assert(PJ == 1 && !ROPE, "merge prologue: one vector per thread");
            const int svc = min(tid, nv - 1);
            const int dsh = __builtin_ctz(static_cast<unsigned>(a.mg_d));   // head_dim is a power of two here
            const int head = (svc * 8) >> dsh, d0 = (svc * 8) & (a.mg_d - 1);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const size_t rh = static_cast<size_t>(m) * a.mg_hq + head;
#pragma unroll
                for (int s = 0; s < NSP; ++s) {
                    const size_t slot = rh * a.mg_nsplit + min(s, a.mg_nsplit - 1);
                    const float* p = a.mg_part_o + (slot << dsh) + d0;
                    mg_po[m][s][0] = *reinterpret_cast<const f32x4_t*>(p);
                    mg_po[m][s][1] = *reinterpret_cast<const f32x4_t*>(p + 4);
                    mg_ml[m][s] = *reinterpret_cast<const f32x2_t*>(a.mg_part_ml + slot * 2);
                }
                const int kv_len = a.mg_row_len[m];
                const int nunits = (kv_len + kAttnUnitTokens - 1) / kAttnUnitTokens;
                mg_ns[m] = min(a.mg_nsplit, (nunits + a.mg_units_per_split - 1) / a.mg_units_per_split);
            }
        } else {
#pragma unroll
        for (int jj = 0; jj < kPreJ; ++jj) {
            const int sv = tid + jj * kBlock;
            const int svc = min(sv, nv - 1);
#pragma unroll
            for (int m = 0; m < M; ++m)   // (lanes past the row hold a repeat until the masking below)
                xr[jj * M + m] = *reinterpret_cast<const u32x4_t*>(a.act + static_cast<size_t>(m) * K + svc * 8);
            if (a.norm_w) nw[jj] = *reinterpret_cast<const u32x4_t*>(a.norm_w + svc * 8);
        }
        }
        // (the scheduling barriers keep every use of the activations behind the first weight
        // requests: left alone, the compiler masks the vectors right after their loads and so waits
        // for the activations before it has asked for a single weight)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kUnits; ++i) issue_next(un[i], ug[i], uc[i]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MG > 0) {
#pragma unroll
            for (int m = 0; m < M; ++m) xr[m] = merge_splits<NSP>(mg_po[m], mg_ml[m], mg_ns[m]);
        }
#pragma unroll
        for (int jj = 0; jj < kPreJ; ++jj) {
            const bool in_row = tid + jj * kBlock < nv;
#pragma unroll
            for (int m = 0; m < M; ++m)
                xr[jj * M + m] = in_row ? xr[jj * M + m] : u32x4_t{0u, 0u, 0u, 0u};
        }
        // ---- activations from registers (requested before the weights) ----
        if (a.norm_w) {
            float* red = lds_sx;  // free until the sums are written below
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float local = 0.f;
#pragma unroll
                for (int jj = 0; jj < kPreJ; ++jj) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float lo = bf16_lo(xr[jj * M + m][i]), hi = bf16_hi(xr[jj * M + m][i]);
                        local += lo * lo + hi * hi;
                    }
                }
                local = wave_sum_dpp(local);
                if (lane == 0) red[m * kWavesPerBlock + wv] = local;
            }
            __syncthreads();
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float t = 0.f;
#pragma unroll
                for (int w = 0; w < kWavesPerBlock; ++w) t += red[m * kWavesPerBlock + w];
                inv_rms[m] = rsqrtf(t / static_cast<float>(K) + a.eps);
            }
            __syncthreads();
        }
#pragma unroll
        for (int jj = 0; jj < kPreJ; ++jj) {
            const int sv = tid + jj * kBlock;
            if (sv < nvp) {
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    u32x4_t v = xr[jj * M + m];
                    if (a.norm_w) {
                        const ActLoader ld{nullptr, a.norm_w, inv_rms[m]};
                        v = u32x4_t{ld.norm2(v.x, nw[jj].x), ld.norm2(v.y, nw[jj].y),
                                    ld.norm2(v.z, nw[jj].z), ld.norm2(v.w, nw[jj].w)};
                    }
                    F::stage_vec(lds_x + m * vec_per_m, sv, v);
                    if (F::kBias != 0.f) {
                        // the WPP / 8 neighbouring lanes that hold one piece's activations add
                        // their sums (a piece never straddles a quad)
                        float sx = bf16_lo(v.x) + bf16_hi(v.x) + bf16_lo(v.y) + bf16_hi(v.y) +
                                   bf16_lo(v.z) + bf16_hi(v.z) + bf16_lo(v.w) + bf16_hi(v.w);
                        constexpr int kPer = WPP / 8;   // 4 (int4) or 2 (byte formats)
                        sx = dpp_add_f32<0xB1>(sx);                      // quad_perm [1,0,3,2]
                        if (kPer == 4) sx = dpp_add_f32<0x4E>(sx);       // quad_perm [2,3,0,1]
                        const int piece = sv / kPer;   // = chunk * 64 + lane
                        if ((sv & (kPer - 1)) == 0) lds_sx[m * nchunks * kWave + piece] = sx;
                    }
                }
            }
        }
        __syncthreads();
    } else {
#pragma unroll
    for (int i = 0; i < kUnits; ++i) issue_next(un[i], ug[i], uc[i]);
    // Optional fused RMSNorm: sum of squares of each activation row (fp32), block-reduced.
    if (a.norm_w) {
        float* red = lds_sx;  // free until the sum_x pass below
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float local = 0.f;
            for (int v = tid; v < K / 8; v += kBlock) {
                const u32x4_t t =
                    *reinterpret_cast<const u32x4_t*>(a.act + static_cast<size_t>(m) * K + v * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lo = bf16_lo(t[i]), hi = bf16_hi(t[i]);
                    local += lo * lo + hi * hi;
                }
            }
            local = wave_sum_dpp(local);
            if (lane == 0) red[m * kWavesPerBlock + wv] = local;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float t = 0.f;
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) t += red[m * kWavesPerBlock + w];
            inv_rms[m] = rsqrtf(t / static_cast<float>(K) + a.eps);
        }
        __syncthreads();
    }

    // Stage activations in the format's decode order.
    for (int v = tid; v < M * vec_per_m; v += kBlock) {
        const int m = v / vec_per_m;
        const int rem = v - m * vec_per_m;
        const int c = rem / (XV * kWave);
        const int i = (rem / kWave) % XV;
        const int l = rem % kWave;
        const int k0 = c * kChunkK + l * WPP;
        u32x4_t p = {0u, 0u, 0u, 0u};
        if (k0 < K) {
            float ir = inv_rms[0];
#pragma unroll
            for (int mm = 1; mm < M; ++mm) ir = (m == mm) ? inv_rms[mm] : ir;
            p = F::stage(ActLoader{a.act + static_cast<size_t>(m) * K, a.norm_w, ir}, k0, i);
        }
        lds_x[v] = p;
    }
    __syncthreads();
    if (F::kBias != 0.f) {
        // Per-(chunk, lane) sum of the activations the lane will multiply.
        for (int j = tid; j < M * nchunks * kWave; j += kBlock) {
            const int m = j / (nchunks * kWave);
            const int cl = j - m * (nchunks * kWave);
            const int c = cl / kWave;
            const int l = cl - c * kWave;
            u32x4_t xs[XV];
#pragma unroll
            for (int i = 0; i < XV; ++i) xs[i] = lds_x[m * vec_per_m + (c * XV + i) * kWave + l];
            lds_sx[j] = F::sum_x(xs);
        }
        __syncthreads();
    }
    }

    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.f;

    auto compute = [&](const Unit<R>& u, int g, int c) {
        const bool valid = c * kChunkK + lane * WPP < K;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            u32x4_t xs[XV];
#pragma unroll
            for (int i = 0; i < XV; ++i) xs[i] = lds_x[m * vec_per_m + (c * XV + i) * kWave + lane];
            const float p0 =
                F::kBias != 0.f ? F::kBias * lds_sx[(m * nchunks + c) * kWave + lane] : 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float p = F::dot(u.w[r], xs, p0);
                if constexpr (F::kGroupScale) {
                    uint16_t gsr = u.gs[r];
                    if constexpr (one_gs)
                        gsr = static_cast<uint16_t>(__builtin_amdgcn_ds_bpermute(
                            ((r << gpc_shift) + ((lane * WPP) >> a.g_shift)) * 4, static_cast<int>(u.gsv)));
                    const float s = valid ? bf16_bits_to_f32(gsr) : 0.f;
                    acc[r][m] = fmaf(s, p, acc[r][m]);
                } else {
                    acc[r][m] += valid ? p : 0.f;
                }
            }
        }
        if (c == nchunks - 1) {
            // One activation row and 2-4 weight rows (single-sequence decode): the R sums are
            // reduced together and lane r holds row r's total.  Otherwise one butterfly each.
            constexpr bool kMulti = M == 1 && R >= 2;
            float tot[R][M];
            float multi = 0.f;
            if constexpr (kMulti) {
                const float vals[4] = {acc[0][0], acc[1][0], R > 2 ? acc[R > 2 ? 2 : 0][0] : 0.f,
                                       R > 3 ? acc[R > 3 ? 3 : 0][0] : 0.f};
                multi = wave_sum_multi<(R > 2 ? 4 : 2)>(vals, lane);
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][0] = 0.f;
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int m = 0; m < M; ++m) {
                        tot[r][m] = wave_sum_dpp(acc[r][m]);
                        acc[r][m] = 0.f;
                    }
                }
            }
            if (pairs) {
                if constexpr (R % 2 == 0) {
                    // lane p*M + m finishes pair p: g and u are rounded to bf16 first, as the
                    // unfused projection would store them (swiglu.cu:18-21 reads bf16 inputs)
                    float gv = 0.f, uv = 0.f;
                    if constexpr (kMulti) {
                        gv = dpp_mov_f32<0x88>(multi);   // quad_perm [0,2,0,2]: lane p <- lane 2p
                        uv = dpp_mov_f32<0xDD>(multi);   // quad_perm [1,3,1,3]: lane p <- lane 2p + 1
                    } else {
#pragma unroll
                        for (int pr = 0; pr < R / 2; ++pr) {
#pragma unroll
                            for (int m = 0; m < M; ++m) {
                                if (lane == pr * M + m) {
                                    gv = tot[2 * pr][m];
                                    uv = tot[2 * pr + 1][m];
                                }
                            }
                        }
                    }
                    const int row = row_begin + g * R + 2 * (lane / M);
                    if (lane < (R / 2) * M && row < row_end) {
                        if constexpr (F::kRowScale) {
                            gv *= u.rs;
                            uv *= u.rs2;
                        }
                        const float gb = bf16_bits_to_f32(f32_to_bf16_bits(gv));
                        const float ub = bf16_bits_to_f32(f32_to_bf16_bits(uv));
                        const int m = lane % M;
                        if (!ROPE) {
                            const float silu = gb / (1.f + expf(-gb));
                            a.y[static_cast<size_t>(m) * (N / 2) + row / 2] = f32_to_bf16_bits(silu * ub);
                        } else {
                            // the projection's bf16 values, then the rotation of
                            // qkv_rope_kvwrite_kernel with the same operations and rounding
                            const int head = row >> __builtin_ctz(static_cast<unsigned>(a.d));   // (power of two)
                            const int dd = row & (a.d - 1);
                            const int slot = u.slot;
                            if (head < a.hq + a.hk) {
                                const float c = u.rc, sn = u.rsn;
                                const uint32_t out = pack_bf16x2(gb * c - ub * sn, ub * c + gb * sn);
                                uint16_t* dst = head < a.hq
                                                    ? a.y + (static_cast<size_t>(m) * a.hq + head) * a.d
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
                    }
                }
            } else {
                float mine = 0.f;
                if constexpr (kMulti) {
                    mine = multi;
                } else {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
#pragma unroll
                        for (int m = 0; m < M; ++m) {
                            if (lane == r * M + m) mine = tot[r][m];
                        }
                    }
                }
                const int row = row_begin + g * R + lane / M;
                if (lane < R * M && row < row_end) {
                    if constexpr (F::kRowScale) mine *= u.rs;
                    const float prev = a.beta ? bf16_bits_to_f32(u.prev) : 0.f;
                    const uint16_t out = f32_to_bf16_bits(mine + prev);
                    a.y[static_cast<size_t>(lane % M) * N + row] = out;
                    // (rows ascend inside a lane: a strict comparison keeps the first of equals;
                    // a NaN never compares greater)
                    const float ov = bf16_bits_to_f32(out);
                    if (ov > best_v) {
                        best_v = ov;
                        best_i = row;
                    }
                }
            }
        }
    };

    // Ring of kUnits units: a unit's registers are requested again as soon as it has been
    // reduced.  Loads are issued unconditionally so the wait before each compute only covers
    // the unit it consumes.
    for (int u = 0; u < nunits; u += kUnits) {
        // Issue priority falls with progress.  The SIMD's arbiter serves its oldest wave first,
        // so of a CU's two blocks the one dispatched first would finish well ahead of the other
        // and leave its wave slots idle for the last third of the launch; a wave that has
        // fallen behind its SIMD neighbour now outranks it until it has caught up.
        {
            const int quarter = (u * 4) / nunits;
            if (quarter == 0) __builtin_amdgcn_s_setprio(3);
            else if (quarter == 1) __builtin_amdgcn_s_setprio(2);
            else if (quarter == 2) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
        }
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
            if (u + i < nunits) compute(un[i], ug[i], uc[i]);
            issue_next(un[i], ug[i], uc[i]);
        }
    }
    if (!ROPE && a.amax_part && lane < R * M)
        a.amax_part[static_cast<size_t>(lane % M) * (total_waves * R) + wg * R + lane / M] =
            (static_cast<unsigned long long>(__float_as_uint(best_v)) << 32) | static_cast<unsigned>(best_i);
}

// Second stage of the lm_head form: one block per activation row reduces the per-lane
// (value, row) pairs; the largest value wins, the lowest row among equals, NaN never
// (argmax_bf16_kernel, driver/cuda/src/kernels/argmax.cu:36-80).
constexpr int kPairThreads = 1024;
__global__ __launch_bounds__(kPairThreads) void argmax_pairs_kernel(const unsigned long long* __restrict__ part,
                                                                    int count, uint32_t* __restrict__ out) {
    __shared__ float sv[kPairThreads / kWave];
    __shared__ int si[kPairThreads / kWave];
    const unsigned long long* row = part + static_cast<size_t>(blockIdx.x) * count;
    float bv = -INFINITY;
    int bi = 0;
    auto upd = [&](float v, int i) {
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    };
    // eight loads in flight per thread (the pairs of a row are a few thousand)
    for (int i0 = threadIdx.x; i0 < count; i0 += 8 * kPairThreads) {
        unsigned long long e[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * kPairThreads;
            e[u] = i < count ? row[i] : (static_cast<unsigned long long>(0xFF800000u) << 32) | 0x7FFFFFFFull;   // (-inf, no row)
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            upd(__uint_as_float(static_cast<uint32_t>(e[u] >> 32)), static_cast<int>(e[u] & 0xFFFFFFFFull));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        upd(ov, oi);
    }
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    if (lane == 0) {
        sv[wv] = bv;
        si[wv] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kPairThreads / kWave; ++w) upd(sv[w], si[w]);
        out[blockIdx.x] = static_cast<uint32_t>(bi == 0x7FFFFFFF ? 0 : bi);
    }
}

// Event pair that brackets the kernel of a pie_hip_gemv_w4a16_timed call (set and cleared inside
// that call).
thread_local hipEvent_t t_start_event = nullptr;
thread_local hipEvent_t t_stop_event = nullptr;

// Blocks of a launch: the machine-sized grid, but at least one row (or row pair) per wave.
int gemv_grid(int N, bool pairs, int waves_per_simd) {
    int grid = kNumCU * 4 * waves_per_simd / kWavesPerBlock;
    if (grid < 1) grid = 1;
    const int max_grid = (N / (pairs ? 2 : 1) + kWavesPerBlock - 1) / kWavesPerBlock;
    return grid > max_grid ? max_grid : grid;
}

template <class F, int R, int M>
int launch(const GemvArgs& a_in, int waves_per_simd, hipStream_t stream) {
    constexpr int kChunkK = kWave * F::WPP;
    const int nchunks = (a_in.K + kChunkK - 1) / kChunkK;
    const size_t smem = static_cast<size_t>(M) * nchunks * kWave * (F::XV * 16 + 4);
    if (smem > 64 * 1024) return PIE_HIP_ERR_UNSUPPORTED;
    const int grid = gemv_grid(a_in.N, a_in.swiglu || a_in.rope_table, waves_per_simd);
    GemvArgs a = a_in;
    const int units = a.N / ((a.swiglu || a.rope_table) ? 2 : 1), waves = grid * kWavesPerBlock;
    a.slice_q = units / waves;
    a.slice_r = units % waves;
    a.groups_per_row = F::kGroupScale && a.G > 0 ? a.K / a.G : 0;
    // (group scales with one load per unit: the R rows' groups of a chunk fit one wave)
    const bool gs1 = F::kGroupScale && a.g_shift >= 0 && a.g_shift <= __builtin_ctz(static_cast<unsigned>(kChunkK)) &&
                     (R << (__builtin_ctz(static_cast<unsigned>(kChunkK)) - a.g_shift)) <= kWave;
    constexpr int kLongJ = 8 / M < 4 ? 8 / M : 4;   // (the register prologue's reach: rows of up to 4096 * kLongJ values)
    const int nvp = nchunks * (kChunkK / 8);
    const bool short_row = nvp <= kBlock;
    if (a.mg_part_o && (!short_row || a.rope_table || a.norm_w || a.mg_nsplit > 8 || M * (a.mg_nsplit <= 4 ? 4 : 8) > 8))
        return PIE_HIP_ERR_UNSUPPORTED;
    auto go_j = [&](auto rope, auto one, auto pj) {
        constexpr bool kRope = decltype(rope)::value, kOne = decltype(one)::value;
        constexpr int kPj = decltype(pj)::value;
        if constexpr (!kRope && kPj == 1 && M <= 2) {
            // (the partial results sit in registers across the first weight requests: eight
            // splits of one row, or four of two)
            if (a.mg_part_o) {
                if (a.mg_nsplit <= 4)
                    hipLaunchKernelGGL((gemv_kernel<F, R, M, false, kOne, 1, 4>), dim3(grid), dim3(kBlock), smem, stream, a);
                else if constexpr (M == 1)
                    hipLaunchKernelGGL((gemv_kernel<F, R, M, false, kOne, 1, 8>), dim3(grid), dim3(kBlock), smem, stream, a);
                return;
            }
        }
        if (!kRope && t_start_event && t_stop_event) {
            hipExtLaunchKernelGGL((gemv_kernel<F, R, M, kRope, kOne, kPj>), dim3(grid), dim3(kBlock),
                                  static_cast<uint32_t>(smem), stream, t_start_event, t_stop_event, 0, a);
            t_start_event = t_stop_event = nullptr;
        } else {
            hipLaunchKernelGGL((gemv_kernel<F, R, M, kRope, kOne, kPj>), dim3(grid), dim3(kBlock), smem, stream, a);
        }
    };
    auto go = [&](auto rope, auto one) {
        if (short_row) {
            go_j(rope, one, std::integral_constant<int, 1>{});
        } else if (nvp <= kLongJ * kBlock) {
            go_j(rope, one, std::integral_constant<int, kLongJ>{});
        } else {
            go_j(rope, one, std::integral_constant<int, 0>{});   // (the two-pass prologue through LDS)
        }
    };
    if (a.rope_table) {
        if constexpr (R % 2 == 0) {
            if constexpr (F::kGroupScale) {
                if (gs1) go(std::true_type{}, std::true_type{});
                else go(std::true_type{}, std::false_type{});
            } else {
                go(std::true_type{}, std::false_type{});
            }
        } else {
            return PIE_HIP_ERR_INVALID;
        }
    } else {
        if constexpr (F::kGroupScale) {
            if (gs1) go(std::false_type{}, std::true_type{});
            else go(std::false_type{}, std::false_type{});
        } else {
            go(std::false_type{}, std::false_type{});
        }
    }
    return launch_status();
}

template <class F, int R>
int launch_m(int M, const GemvArgs& a, int wps, hipStream_t stream) {
    switch (M) {
        case 1: return launch<F, R, 1>(a, wps, stream);
        case 2: return launch<F, R, 2>(a, wps, stream);
        case 3: return launch<F, R, 3>(a, wps, stream);
        case 4: return launch<F, R, 4>(a, wps, stream);
        default: return PIE_HIP_ERR_UNSUPPORTED;
    }
}

// rows_per_wave (R) in {1,2,3,4}; waves_per_simd in 1..8.  0 = pick.
template <class F>
int dispatch(GemvArgs a, int M, int rows_per_wave, int waves_per_simd, hipStream_t stream) {
    if ((!a.act && !a.mg_part_o) || !a.w || !a.y || M <= 0 || a.N <= 0 || a.K <= 0) return PIE_HIP_ERR_INVALID;
    if (a.K % F::WPP != 0) return PIE_HIP_ERR_UNSUPPORTED;
    if (a.norm_w && a.K % 8 != 0) return PIE_HIP_ERR_UNSUPPORTED;
    if (a.swiglu && (a.N % 2 != 0 || a.beta)) return PIE_HIP_ERR_INVALID;
    // Measured on MI355X: two resident waves per SIMD, each walking its slice four rows
    // at a time (fewer when the slice is shorter), is within a few percent of the best
    // (rows, waves) pair for every decode shape of an 8B-class model.
    a.g_shift = (a.G > 0 && (a.G & (a.G - 1)) == 0) ? __builtin_ctz(static_cast<unsigned>(a.G)) : -1;
    if (waves_per_simd <= 0) waves_per_simd = 2;
    if (waves_per_simd > 8) return PIE_HIP_ERR_INVALID;
    if (rows_per_wave <= 0) {
        const long long per_wave =
            a.N / (static_cast<long long>(kNumCU) * 4 * waves_per_simd);
        rows_per_wave = per_wave >= 4 ? 4 : (per_wave >= 3 ? 3 : (per_wave >= 2 ? 2 : 1));
    }
    if ((a.swiglu || a.rope_table) && rows_per_wave % 2 != 0) rows_per_wave = rows_per_wave == 3 ? 4 : 2;
    // Up to four activation rows share one pass over the weights (fewer when their staged
    // copies would not fit in 64 KiB of LDS); larger M re-reads the weights per group.
    constexpr int kChunkK = kWave * F::WPP;
    const size_t per_m = static_cast<size_t>((a.K + kChunkK - 1) / kChunkK) * kWave * (F::XV * 16 + 4);
    if (per_m > 64 * 1024) return PIE_HIP_ERR_UNSUPPORTED;
    int mcap = static_cast<int>(64 * 1024 / per_m);
    if (mcap > 4) mcap = 4;
    if (a.mg_part_o && M > mcap) return PIE_HIP_ERR_UNSUPPORTED;   // (the merge prologue indexes rows from 0)
    const uint16_t* act = a.act;
    uint16_t* y = a.y;
    const float* rope_table = a.rope_table;
    const int64_t* kv_slots = a.kv_slots;
    unsigned long long* amax_part = a.amax_part;
    const size_t amax_per_m = static_cast<size_t>(gemv_grid(a.N, a.swiglu || a.rope_table, waves_per_simd)) *
                              kWavesPerBlock * rows_per_wave;
    for (int m0 = 0; m0 < M; m0 += mcap) {
        if (amax_part) a.amax_part = amax_part + m0 * amax_per_m;
        const int mm = (M - m0) < mcap ? (M - m0) : mcap;
        a.act = act + static_cast<size_t>(m0) * a.K;
        a.y = y + static_cast<size_t>(m0) * (a.rope_table ? a.hq * a.d : (a.swiglu ? a.N / 2 : a.N));
        if (rope_table) {
            a.rope_table = rope_table + static_cast<size_t>(m0) * a.d;
            a.kv_slots = kv_slots + m0;
        }
        int st;
        switch (rows_per_wave) {
            case 1: st = launch_m<F, 1>(mm, a, waves_per_simd, stream); break;
            case 2: st = launch_m<F, 2>(mm, a, waves_per_simd, stream); break;
            case 3: st = launch_m<F, 3>(mm, a, waves_per_simd, stream); break;
            case 4: st = launch_m<F, 4>(mm, a, waves_per_simd, stream); break;
            default: return PIE_HIP_ERR_INVALID;
        }
        if (st != PIE_HIP_OK) return st;
    }
    return PIE_HIP_OK;
}

}  // namespace
}  // namespace pie_hip

using pie_hip::GemvArgs;


extern "C" int pie_hip_gemv_w4a16_tuned(const uint16_t* act_bf16, const uint32_t* packed,
                                        const uint16_t* scale_bf16, uint16_t* y_bf16, int M,
                                        int N, int K, int group_size, int beta,
                                        int rows_per_wave, int waves_per_simd, void* stream) {
    if (!scale_bf16 || group_size <= 0) return PIE_HIP_ERR_INVALID;
    if (group_size % 32 != 0 || K % group_size != 0) return PIE_HIP_ERR_UNSUPPORTED;
    GemvArgs a{act_bf16, reinterpret_cast<const pie_hip::u32x4_t*>(packed), scale_bf16, nullptr,
               y_bf16, N, K, group_size, beta};
    return pie_hip::dispatch<pie_hip::FmtInt4>(a, M, rows_per_wave, waves_per_simd,
                                               static_cast<hipStream_t>(stream));
}

extern "C" int pie_hip_gemv_w4a16(const uint16_t* act_bf16, const uint32_t* packed,
                                  const uint16_t* scale_bf16, uint16_t* y_bf16, int M, int N,
                                  int K, int group_size, int beta, void* stream) {
    return pie_hip_gemv_w4a16_tuned(act_bf16, packed, scale_bf16, y_bf16, M, N, K, group_size,
                                    beta, 0, 0, stream);
}

// The same launch bracketed by the caller's two events (measurement): the events travel with
// this one call — nothing is remembered between calls.
extern "C" int pie_hip_gemv_w4a16_timed(const uint16_t* act_bf16, const uint32_t* packed,
                                        const uint16_t* scale_bf16, uint16_t* y_bf16, int M, int N,
                                        int K, int group_size, int beta, void* start_event,
                                        void* stop_event, void* stream) {
    if (!start_event || !stop_event || M > 4) return PIE_HIP_ERR_INVALID;   // one kernel per call
    pie_hip::t_start_event = static_cast<hipEvent_t>(start_event);
    pie_hip::t_stop_event = static_cast<hipEvent_t>(stop_event);
    const int rc = pie_hip_gemv_w4a16_tuned(act_bf16, packed, scale_bf16, y_bf16, M, N, K, group_size,
                                            beta, 0, 0, stream);
    pie_hip::t_start_event = pie_hip::t_stop_event = nullptr;
    return rc;
}

extern "C" int pie_hip_gemv_w8a16(const uint16_t* act_bf16, const int8_t* w_int8,
                                  const float* scale_inv_f32, const uint16_t* scale_inv_bf16,
                                  uint16_t* y_bf16, int M, int N, int K, int beta, void* stream) {
    if (!scale_inv_f32 == !scale_inv_bf16) return PIE_HIP_ERR_INVALID;  // exactly one
    GemvArgs a{act_bf16, reinterpret_cast<const pie_hip::u32x4_t*>(w_int8), nullptr,
               scale_inv_f32 ? static_cast<const void*>(scale_inv_f32) : scale_inv_bf16, y_bf16,
               N, K, 0, beta};
    hipStream_t st = static_cast<hipStream_t>(stream);
    return scale_inv_f32 ? pie_hip::dispatch<pie_hip::FmtInt8<false>>(a, M, 0, 0, st)
                         : pie_hip::dispatch<pie_hip::FmtInt8<true>>(a, M, 0, 0, st);
}

extern "C" int pie_hip_gemv_fp8(const uint16_t* act_bf16, const uint8_t* w_e4m3,
                                const float* scale_inv_f32, const uint16_t* scale_inv_bf16,
                                uint16_t* y_bf16, int M, int N, int K, int beta, void* stream) {
    if (!scale_inv_f32 == !scale_inv_bf16) return PIE_HIP_ERR_INVALID;
    GemvArgs a{act_bf16, reinterpret_cast<const pie_hip::u32x4_t*>(w_e4m3), nullptr,
               scale_inv_f32 ? static_cast<const void*>(scale_inv_f32) : scale_inv_bf16, y_bf16,
               N, K, 0, beta};
    hipStream_t st = static_cast<hipStream_t>(stream);
    return scale_inv_f32 ? pie_hip::dispatch<pie_hip::FmtFp8<false>>(a, M, 0, 0, st)
                         : pie_hip::dispatch<pie_hip::FmtFp8<true>>(a, M, 0, 0, st);
}

extern "C" int pie_hip_gemv_bf16(const uint16_t* act_bf16, const uint16_t* w_bf16,
                                 uint16_t* y_bf16, int M, int N, int K, int beta, void* stream) {
    GemvArgs a{act_bf16, reinterpret_cast<const pie_hip::u32x4_t*>(w_bf16), nullptr, nullptr,
               y_bf16, N, K, 0, beta};
    return pie_hip::dispatch<pie_hip::FmtBf16>(a, M, 0, 0, static_cast<hipStream_t>(stream));
}

// lm_head with the greedy token in its wake: the bf16 GEMV (final RMSNorm riding in its
// activation staging) writes the logits and per-lane (largest value, row) pairs; a one-block-per-
// row kernel reduces the pairs.  Replaces the GEMV followed by a pass over the whole logits row
// (lm_head_gemv_argmax_bf16, driver/cuda/src/kernels/argmax.cu:795-935: the same two stages).
extern "C" size_t pie_hip_lm_head_argmax_workspace_bytes(int M, int V) {
    if (M <= 0 || M > 4 || V <= 0) return 0;
    return static_cast<size_t>(M) * pie_hip::gemv_grid(V, false, 2) * pie_hip::kWavesPerBlock * 4 * sizeof(unsigned long long);
}

extern "C" int pie_hip_lm_head_argmax(const uint16_t* act_bf16, const uint16_t* norm_weight_bf16, float eps,
                                      const uint16_t* w_bf16, uint16_t* logits_bf16, uint32_t* out_tokens,
                                      int M, int V, int H, void* workspace, size_t workspace_bytes,
                                      void* stream) {
    using namespace pie_hip;
    if (!act_bf16 || !w_bf16 || !logits_bf16 || !out_tokens || !workspace || M <= 0 || V <= 0 || H <= 0)
        return PIE_HIP_ERR_INVALID;
    if (M > 4 || V < 4 * kWavesPerBlock) return PIE_HIP_ERR_UNSUPPORTED;   // one weight pass, four rows per wave
    const size_t need = pie_hip_lm_head_argmax_workspace_bytes(M, V);
    if (workspace_bytes < need) return PIE_HIP_ERR_INVALID;
    GemvArgs a{act_bf16, reinterpret_cast<const u32x4_t*>(w_bf16), nullptr, nullptr, logits_bf16, V, H, 0, 0,
               norm_weight_bf16, eps, 0};
    a.amax_part = static_cast<unsigned long long*>(workspace);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int rc = dispatch<FmtBf16>(a, M, 4, 2, st);
    if (rc != PIE_HIP_OK) return rc;
    const int count = gemv_grid(V, false, 2) * kWavesPerBlock * 4;
    hipLaunchKernelGGL(argmax_pairs_kernel, dim3(M), dim3(kPairThreads), 0, st,
                       static_cast<const unsigned long long*>(workspace), count, out_tokens);
    return launch_status();
}

// One entry point for the fused forms the decoder layer uses: optional RMSNorm of the
// activations while they are staged, optional SwiGLU over (gate, up) row pairs in the epilogue.
extern "C" int pie_hip_linear_fused(int format, const uint16_t* act_bf16,
                                    const uint16_t* norm_weight_bf16, float eps,
                                    const void* weight, const void* scale, int scale_is_bf16,
                                    int group_size, uint16_t* y_bf16, int M, int N, int K,
                                    int beta, int swiglu, void* stream) {
    using namespace pie_hip;
    GemvArgs a{act_bf16, static_cast<const u32x4_t*>(weight), nullptr, nullptr, y_bf16, N, K,
               group_size, beta, norm_weight_bf16, eps, swiglu ? 1 : 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (format) {
        case PIE_HIP_FMT_INT4B8:
            if (!scale || group_size <= 0) return PIE_HIP_ERR_INVALID;
            if (group_size % 32 != 0 || K % group_size != 0) return PIE_HIP_ERR_UNSUPPORTED;
            a.gscale = static_cast<const uint16_t*>(scale);
            return dispatch<FmtInt4>(a, M, 0, 0, st);
        case PIE_HIP_FMT_INT8:
            if (!scale) return PIE_HIP_ERR_INVALID;
            a.rscale = scale;
            return scale_is_bf16 ? dispatch<FmtInt8<true>>(a, M, 0, 0, st)
                                 : dispatch<FmtInt8<false>>(a, M, 0, 0, st);
        case PIE_HIP_FMT_FP8:
            if (!scale) return PIE_HIP_ERR_INVALID;
            a.rscale = scale;
            return scale_is_bf16 ? dispatch<FmtFp8<true>>(a, M, 0, 0, st)
                                 : dispatch<FmtFp8<false>>(a, M, 0, 0, st);
        case PIE_HIP_FMT_BF16:
            return dispatch<FmtBf16>(a, M, 0, 0, st);
        default:
            return PIE_HIP_ERR_INVALID;
    }
}

namespace pie_hip {
namespace {
template <class F>
bool merge_shape_ok(int M, int K, int num_splits) {
    constexpr int kChunkK = kWave * F::WPP;
    if (K % F::WPP != 0) return false;
    const int nchunks = (K + kChunkK - 1) / kChunkK;
    if (nchunks * (kChunkK / 8) > kBlock) return false;                                   // one vector per thread
    if (static_cast<size_t>(M) * nchunks * kWave * (F::XV * 16 + 4) > 64 * 1024) return false;   // staged rows in LDS
    return num_splits >= 2 && num_splits <= 8 && M * (num_splits <= 4 ? 4 : 8) <= 8;
}
}  // namespace
}  // namespace pie_hip

// Whether pie_hip_linear_attn_merge takes the shape (1) or answers PIE_HIP_ERR_UNSUPPORTED (0).
extern "C" int pie_hip_linear_attn_merge_supported(int format, int M, int num_splits, int num_q_heads,
                                                   int head_dim, int group_size) {
    using namespace pie_hip;
    if (M <= 0 || num_q_heads <= 0 || head_dim < 8 || (head_dim & (head_dim - 1)) != 0) return 0;
    const int K = num_q_heads * head_dim;
    switch (format) {
        case PIE_HIP_FMT_INT4B8:
            return group_size > 0 && group_size % 32 == 0 && K % group_size == 0 && merge_shape_ok<FmtInt4>(M, K, num_splits);
        case PIE_HIP_FMT_INT8: return merge_shape_ok<FmtInt8<true>>(M, K, num_splits);
        case PIE_HIP_FMT_FP8: return merge_shape_ok<FmtFp8<true>>(M, K, num_splits);
        case PIE_HIP_FMT_BF16: return merge_shape_ok<FmtBf16>(M, K, num_splits);
        default: return 0;
    }
}

// The attention output projection of a decode step with the split merge of the attention in its
// prologue: y (+)= merge(partials) . W^T, the merged rows bit-identical to attn_decode_merge_kernel's.
extern "C" int pie_hip_linear_attn_merge(int format, const void* attn_workspace, int num_splits,
                                         int units_per_split, const int32_t* row_kv_len, int num_q_heads,
                                         int head_dim, const void* weight, const void* scale, int scale_is_bf16,
                                         int group_size, uint16_t* y_bf16, int M, int N, int beta, void* stream) {
    using namespace pie_hip;
    if (!attn_workspace || !row_kv_len || num_splits < 2 || units_per_split <= 0 || num_q_heads <= 0 ||
        head_dim <= 0 || M <= 0)
        return PIE_HIP_ERR_INVALID;
    if ((head_dim & (head_dim - 1)) != 0 || head_dim < 8) return PIE_HIP_ERR_UNSUPPORTED;
    const int K = num_q_heads * head_dim;
    GemvArgs a{nullptr, static_cast<const u32x4_t*>(weight), nullptr, nullptr, y_bf16, N, K, group_size, beta};
    // the workspace layout of the split launch: partial outputs, then the (max, sum) pairs
    const size_t n_part = static_cast<size_t>(M) * num_q_heads * num_splits;
    a.mg_part_o = static_cast<const float*>(attn_workspace);
    a.mg_part_ml = a.mg_part_o + n_part * head_dim;
    a.mg_row_len = row_kv_len;
    a.mg_nsplit = num_splits;
    a.mg_units_per_split = units_per_split;
    a.mg_hq = num_q_heads;
    a.mg_d = head_dim;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (format) {
        case PIE_HIP_FMT_INT4B8:
            if (!scale || group_size <= 0) return PIE_HIP_ERR_INVALID;
            if (group_size % 32 != 0 || K % group_size != 0) return PIE_HIP_ERR_UNSUPPORTED;
            a.gscale = static_cast<const uint16_t*>(scale);
            return dispatch<FmtInt4>(a, M, 0, 0, st);
        case PIE_HIP_FMT_INT8:
            if (!scale) return PIE_HIP_ERR_INVALID;
            a.rscale = scale;
            return scale_is_bf16 ? dispatch<FmtInt8<true>>(a, M, 0, 0, st)
                                 : dispatch<FmtInt8<false>>(a, M, 0, 0, st);
        case PIE_HIP_FMT_FP8:
            if (!scale) return PIE_HIP_ERR_INVALID;
            a.rscale = scale;
            return scale_is_bf16 ? dispatch<FmtFp8<true>>(a, M, 0, 0, st)
                                 : dispatch<FmtFp8<false>>(a, M, 0, 0, st);
        case PIE_HIP_FMT_BF16:
            return dispatch<FmtBf16>(a, M, 0, 0, st);
        default:
            return PIE_HIP_ERR_INVALID;
    }
}

// The fused q|k|v projection of a decode step with the rotation and the KV-cache write in its
// epilogue (no per-head q/k norm): replaces the projection followed by qkv_rope_kvwrite_kernel
// with identical values.  pairing 1: adjacent pairs (2i, 2i+1); 2: weight rows re-ordered at load
// so that rows (2i, 2i+1) of a q / k head are the half-split pair (i, i + d/2), written back to
// those positions.
extern "C" int pie_hip_qkv_rope_fused(int format, const uint16_t* act_bf16,
                                      const uint16_t* norm_weight_bf16, float eps,
                                      const void* weight, const void* scale, int scale_is_bf16,
                                      int group_size, int M, int K, const float* rope_table,
                                      const int64_t* kv_slots, uint16_t* q_out, uint16_t* k_pages,
                                      uint16_t* v_pages, int num_q_heads, int num_kv_heads,
                                      int head_dim, int pairing, void* stream) {
    using namespace pie_hip;
    if (!rope_table || !kv_slots || !q_out || !k_pages || !v_pages || num_q_heads <= 0 ||
        num_kv_heads <= 0 || head_dim <= 0 || (pairing != 1 && pairing != 2))
        return PIE_HIP_ERR_INVALID;
    if (head_dim < 2 || (head_dim & (head_dim - 1)) != 0) return PIE_HIP_ERR_UNSUPPORTED;
    const int N = (num_q_heads + 2 * num_kv_heads) * head_dim;
    GemvArgs a{act_bf16, static_cast<const u32x4_t*>(weight), nullptr, nullptr, q_out, N, K,
               group_size, 0, norm_weight_bf16, eps, 0, rope_table, kv_slots, k_pages, v_pages,
               num_q_heads, num_kv_heads, head_dim};
    a.half_out = pairing == 2;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (format) {
        case PIE_HIP_FMT_INT4B8:
            if (!scale || group_size <= 0) return PIE_HIP_ERR_INVALID;
            if (group_size % 32 != 0 || K % group_size != 0) return PIE_HIP_ERR_UNSUPPORTED;
            a.gscale = static_cast<const uint16_t*>(scale);
            return dispatch<FmtInt4>(a, M, 0, 0, st);
        case PIE_HIP_FMT_INT8:
            if (!scale) return PIE_HIP_ERR_INVALID;
            a.rscale = scale;
            return scale_is_bf16 ? dispatch<FmtInt8<true>>(a, M, 0, 0, st)
                                 : dispatch<FmtInt8<false>>(a, M, 0, 0, st);
        case PIE_HIP_FMT_FP8:
            if (!scale) return PIE_HIP_ERR_INVALID;
            a.rscale = scale;
            return scale_is_bf16 ? dispatch<FmtFp8<true>>(a, M, 0, 0, st)
                                 : dispatch<FmtFp8<false>>(a, M, 0, 0, st);
        case PIE_HIP_FMT_BF16:
            return dispatch<FmtBf16>(a, M, 0, 0, st);
        default:
            return PIE_HIP_ERR_INVALID;
    }
}
