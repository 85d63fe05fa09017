// Prefill attention over paged KV on the matrix cores (gfx950, v_mfma_f32_16x16x32_bf16).
//
//   o[row, h, :] = softmax_j( q[row, h, :] . K[j, kvh, :] * scale ) . V[j, kvh, :],  j < row_kv_len[row]
// for tiles of consecutive query rows that share one page list (the tokens of one prefill
// chunk): same result contract as pie_hip_attn_rows_paged, i.e. the causal prefill branch of
// the reference's paged kernel (driver/cuda/src/ops/attention_naive_paged.cu:148-317) and of
// build_request_flash_attn (driver/portable/src/graph_common.cpp:347-396).
//
// One block (4 waves) = one tile x one kv head = 128 (token, q head) rows, 32 per wave as two
// 16-row MFMA tiles.  Keys advance 32 at a time:
//   S^T[key, query]  = K . Q^T     A = K fragment from LDS (row = key, k = d),  B = Q fragment kept
//                                  in registers (col = query, k = d)
//   O^T[d, query]   += V^T . P^T   A = V^T fragment from LDS (row = d, k = key), B = P in registers
// Both products put the query on the lane%16 axis, so the online-softmax state (max, sum,
// rescale) is per lane and the probabilities leave the first product already in the register
// layout the second one consumes — with the 32 keys of a step in the order
// [4g..4g+3, 16+4g..16+4g+3] per 16-lane group g, which is the order V^T is laid out in LDS.
// K rows are padded to 272 B and V^T rows to 80 B: every 16-byte operand read of 16 lanes
// touches 64 distinct banks.  The next step's K/V are requested from HBM before the current
// step is multiplied.  Probabilities enter the second product as a hi + lo pair of bf16 values
// (fp32 accumulators), and the normaliser sums the unrounded values.
#include "common.hip.h"

#include <type_traits>

namespace pie_hip {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int kTileWaves = 4;
constexpr int kTileThreads = kTileWaves * kWave;
constexpr int kStepKeys = 32;
constexpr int kBlockRows = 128;           // (token, head) rows per block
constexpr int kVtStride = kStepKeys + 8;  // bf16 elements per V^T row (80 B)

// slot of key kappa (0..31) inside a V^T row
__device__ __forceinline__ int vt_slot(int kappa) {
    return kappa < 16 ? 8 * (kappa >> 2) + (kappa & 3) : 8 * ((kappa - 16) >> 2) + 4 + (kappa & 3);
}

// QT: 16-row MFMA tiles per wave (2: 128 rows per block, K/V fragments read once per two tiles;
// 1: 64 rows per block, twice the blocks for small batches).
// KVF: one-byte pools (the codes become bf16 — exactly — on the way into the LDS tiles, one
// 16-code piece per thread and matrix; the step's per-(token, kv head) scales sit in LDS and
// multiply the scores (K) and the probabilities (V): float(code) * scale as in the row kernels).
template <int D, int GQA, int QT, int KVF = kKvBf16>
__global__ __launch_bounds__(kTileThreads, 2) void attn_prefill_tile_kernel(
    const uint16_t* __restrict__ q, const void* __restrict__ k_pages_raw,
    const void* __restrict__ v_pages_raw, const float* __restrict__ k_scales,
    const float* __restrict__ v_scales, uint16_t* __restrict__ o,
    const uint32_t* __restrict__ page_indices, const uint32_t* __restrict__ row_begin,
    const int32_t* __restrict__ row_len, const int32_t* __restrict__ tile_start,
    const int32_t* __restrict__ tile_rows, int hq, int hk, int ps, float scale_log2e) {
    constexpr int TQ = 32 * QT * kTileWaves / (2 * GQA);   // query tokens per tile: 64 QT / GQA
    constexpr int KS = D / 32;             // k steps of the first product
    constexpr int DT = D / 16;             // d tiles of the second product
    constexpr int LPR = D / 8;             // 16-byte pieces per K/V row
    constexpr int KSTRIDE = D + 8;         // bf16 elements per K row in LDS
    constexpr bool Q8 = KVF != kKvBf16;
    constexpr int LPRQ = D / 16;           // 16-code pieces per one-byte row
    constexpr int PIECES = Q8 ? 1 : kStepKeys * LPR / kTileThreads;   // 16-byte pieces per thread per matrix
    static_assert(PIECES >= 1 && (PIECES % 2 == 0 || PIECES == 1), "piece mapping");
    static_assert(kStepKeys * LPRQ <= kTileThreads, "one-byte pieces fit one per thread");
    const uint16_t* k_pages = static_cast<const uint16_t*>(k_pages_raw);
    const uint16_t* v_pages = static_cast<const uint16_t*>(v_pages_raw);
    const unsigned char* k_bytes = static_cast<const unsigned char*>(k_pages_raw);
    const unsigned char* v_bytes = static_cast<const unsigned char*>(v_pages_raw);
    // two LDS buffers: a step's tiles are written while the previous step's are read, one
    // barrier per step
    __shared__ __attribute__((aligned(16))) float s_sc_all[2][Q8 ? 2 * kStepKeys : 1];   // K | V scales of a step

    __shared__ __attribute__((aligned(16))) uint16_t Ks_all[2][kStepKeys * KSTRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t Vt_all[2][D * kVtStride];
    __shared__ int s_kmax;

    // Blocks start in the order of their linear index: tile-major, the kv heads of a tile side by
    // side.  A caller that lists its tiles longest first therefore gets the long causal tiles
    // started first and the short ones handed to the slots that free up — the longest-first rule,
    // which for a causal prompt of more tiles than slots comes within a step of an even split
    // (measured, 32 q / 8 kv heads of 128: 3072 tokens 242 -> 169 us, 4096 tokens 355 -> 278, 8192
    // tokens 1072 -> 934).
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;
    const int tile = lin / hk;
    const int kvh = lin - tile * hk;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int l16 = lane & 15, g = lane >> 4;
    const int s0 = tile_start[tile], n_rows = tile_rows[tile];
    const uint32_t pg_lo = row_begin[s0];

    if (tid == 0) s_kmax = 0;
    __syncthreads();
    if (tid < n_rows) atomicMax(&s_kmax, row_len[s0 + tid]);
    __syncthreads();
    const int kmax = s_kmax;

    // this lane's two query rows (one per 16-row tile of the wave)
    int my_len[QT], my_row[QT], my_head[QT];
    bf16x8_t qf[QT][KS];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int m = wv * 16 * QT + qt * 16 + l16;
        const int h = m / TQ, t = m % TQ;
        const bool valid = t < n_rows;
        my_row[qt] = s0 + (valid ? t : 0);
        my_head[qt] = kvh * GQA + h;
        my_len[qt] = valid ? row_len[my_row[qt]] : 0;
        const uint16_t* qp = q + (static_cast<size_t>(my_row[qt]) * hq + my_head[qt]) * D + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4_t v = *reinterpret_cast<const u32x4_t*>(qp + 32 * ks);
            if (!valid) v = u32x4_t{0u, 0u, 0u, 0u};
            qf[qt][ks] = __builtin_bit_cast(bf16x8_t, v);
        }
    }

    // the shortest causal extent among this wave's rows: steps below it need no masking
    int min_len_v = my_len[0];
#pragma unroll
    for (int qt = 1; qt < QT; ++qt) min_len_v = min(min_len_v, my_len[qt]);
#pragma unroll
    for (int sh = 1; sh < kWave; sh <<= 1) min_len_v = min(min_len_v, __shfl_xor(min_len_v, sh, kWave));
    const int min_len = __builtin_amdgcn_readfirstlane(min_len_v);

    // K/V staging: thread -> (key pair kp, 16-byte piece dc) so that two adjacent keys of one
    // piece meet in one thread (their V values pack into 4-byte LDS writes)
    constexpr int PAIRS = kStepKeys / 2;
    constexpr int PF = 2;   // steps of K/V in flight
    u32x4_t kreg[PF][PIECES], vreg[PF][PIECES];
    float sreg[PF];   // one-byte pools: thread t < 32 holds the K scale of key t, t < 64 V's
    auto piece_of = [&](int u, int& key, int& dc) {
        if constexpr (Q8) {   // thread -> (key, 16-code piece); threads past the tile idle
            key = tid % kStepKeys;
            dc = tid / kStepKeys;
            return;
        }
        if (PIECES == 1) {   // D = 64: one piece per thread
            key = tid % kStepKeys;
            dc = tid / kStepKeys;
            return;
        }
        // pieces of one thread: (pair, dc) pairs p = tid + kTileThreads * (u / 2); key = 2 * pair + (u & 1)
        const int p = tid + kTileThreads * (u >> 1);
        const int pair = p % PAIRS;
        dc = p / PAIRS;
        key = 2 * pair + (u & 1);
    };
    // a 32-key step touches at most two pages (page_size % 16 == 0): their ids come through
    // scalar loads, so the vector-memory queue holds K/V loads only, in step order
    auto issue = [&](int slot, int j0) {
        const int ja = min(j0, kmax - 1), jb = min(j0 + kStepKeys - 1, kmax - 1);
        // (the step's first page by one scalar division; a key is in it or in the next one — no
        // division per lane, which was a fifth of the step's instructions)
        const int page_a = ja / ps;
        const int pa_end = (page_a + 1) * ps;
        const uint32_t pid_a = __builtin_amdgcn_readfirstlane(page_indices[pg_lo + page_a]);
        const uint32_t pid_b = __builtin_amdgcn_readfirstlane(page_indices[pg_lo + page_a + (jb >= pa_end ? 1 : 0)]);
        auto token_head = [&](int key) {
            const int j = min(j0 + key, kmax - 1);
            const bool in_a = j < pa_end;
            return (static_cast<size_t>(in_a ? pid_a : pid_b) * ps + (j - (in_a ? pa_end - ps : pa_end))) * hk + kvh;
        };
        auto token_sc = [&](int key) {   // the key's place in a scale pool
            const int j = min(j0 + key, kmax - 1);
            const bool in_a = j < pa_end;
            return kv_scale_index(in_a ? pid_a : pid_b, j - (in_a ? pa_end - ps : pa_end), kvh, hk, ps);
        };
        if constexpr (Q8) {
            int key, dc;
            piece_of(0, key, dc);
            if (dc < LPRQ) {
                const size_t off = token_head(key) * D + dc * 16;
                kreg[slot][0] = *reinterpret_cast<const u32x4_t*>(k_bytes + off);
                vreg[slot][0] = *reinterpret_cast<const u32x4_t*>(v_bytes + off);
            }
            if (tid < 2 * kStepKeys) {
                const float* sp = tid < kStepKeys ? k_scales : v_scales;
                sreg[slot] = sp ? sp[token_sc(tid % kStepKeys)] : 1.f;
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            int key, dc;
            piece_of(u, key, dc);
            const size_t off = token_head(key) * D + dc * 8;
            kreg[slot][u] = *reinterpret_cast<const u32x4_t*>(k_pages + off);
            vreg[slot][u] = *reinterpret_cast<const u32x4_t*>(v_pages + off);
        }
    };
    auto stage = [&](int slot) {   // register slot = LDS buffer
        uint16_t* Ks = Ks_all[slot];
        uint16_t* Vt = Vt_all[slot];
        float* s_sc = s_sc_all[slot];
        if constexpr (Q8) {
            int key, dc;
            piece_of(0, key, dc);
            if (dc < LPRQ) {
                const u32x4_t kw = kreg[slot][0], vw = vreg[slot][0];
                uint16_t* kd = &Ks[key * KSTRIDE + dc * 16];
                *reinterpret_cast<u32x4_t*>(kd) = kv_decode_bf16<KVF>(u32x2_t{kw.x, kw.y});
                *reinterpret_cast<u32x4_t*>(kd + 8) = kv_decode_bf16<KVF>(u32x2_t{kw.z, kw.w});
                const int col = vt_slot(key);
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    float f[8];
                    kv_decode_f32<KVF>(u32x2_t{vw[2 * h], vw[2 * h + 1]}, f);
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        Vt[(dc * 16 + 8 * h + e) * kVtStride + col] = static_cast<uint16_t>(__float_as_uint(f[e]) >> 16);
                }
            }
            if (tid < 2 * kStepKeys) s_sc[tid] = sreg[slot];
            return;
        }
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            int key, dc;
            piece_of(u, key, dc);
            *reinterpret_cast<u32x4_t*>(&Ks[key * KSTRIDE + dc * 8]) = kreg[slot][u];
        }
#pragma unroll
        for (int u = 0; u + 1 < PIECES || (PIECES == 1 && u == 0); u += 2) {
            int key, dc;
            piece_of(u, key, dc);
            const int col = vt_slot(key);
            if constexpr (PIECES == 1) {
                const uint32_t w[4] = {vreg[slot][0].x, vreg[slot][0].y, vreg[slot][0].z, vreg[slot][0].w};
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    Vt[(dc * 8 + e) * kVtStride + col] = static_cast<uint16_t>(w[e >> 1] >> (16 * (e & 1)));
            } else {
                const uint32_t a[4] = {vreg[slot][u].x, vreg[slot][u].y, vreg[slot][u].z, vreg[slot][u].w};
                const uint32_t b[4] = {vreg[slot][u + 1].x, vreg[slot][u + 1].y, vreg[slot][u + 1].z, vreg[slot][u + 1].w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint32_t lo = (a[e >> 1] >> (16 * (e & 1))) & 0xFFFFu;
                    const uint32_t hi = (b[e >> 1] >> (16 * (e & 1))) & 0xFFFFu;
                    *reinterpret_cast<uint32_t*>(&Vt[(dc * 8 + e) * kVtStride + col]) = lo | (hi << 16);
                }
            }
        }
    };

    f32x4_t acc[QT][DT];
    float mx[QT], lsum[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        mx[qt] = -INFINITY;
        lsum[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[qt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // Step j reads buffer j % 2.  On entry its tiles are staged and the block has met; the
    // step first stages step j + 1 from the other register slot into the other buffer (whose
    // readers passed the last barrier), then refills that slot with step j + 3.
    auto step = [&](int slot, int j0) {
        const uint16_t* Ks = Ks_all[slot];
        const uint16_t* Vt = Vt_all[slot];
        const float* s_sc = s_sc_all[slot];
        if (j0 + kStepKeys < kmax) stage(slot ^ 1);
        if (j0 + 3 * kStepKeys < kmax) issue(slot ^ 1, j0 + 3 * kStepKeys);   // (slot ^ 1 held step j + 1)
        // (one-byte pools) the scales of this lane's keys 16nt + 4g + r
        f32x4_t ksc[2], vsc[2];
        if constexpr (Q8) {
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                ksc[nt] = *reinterpret_cast<const f32x4_t*>(&s_sc[16 * nt + 4 * g]);
                vsc[nt] = *reinterpret_cast<const f32x4_t*>(&s_sc[kStepKeys + 16 * nt + 4 * g]);
            }
        }
        // S^T = K . Q^T for both query tiles
        f32x4_t st[QT][2];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) st[qt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                const bf16x8_t kf = __builtin_bit_cast(
                    bf16x8_t, *reinterpret_cast<const u32x4_t*>(&Ks[(16 * nt + l16) * KSTRIDE + 32 * ks + 8 * g]));
#pragma unroll
                for (int qt = 0; qt < QT; ++qt)
                    st[qt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qt][ks], st[qt][nt], 0, 0, 0);
            }
        }
        // online softmax per query (= per lane%16); the 8 keys of this lane: 16nt + 4g + r.
        // bf16 pools keep the running maximum in raw score units and fold the softmax scale into
        // the exponent's fma; steps wholly inside every row's causal extent skip the masking
        // (a wave-uniform branch); exponentials are the bare v_exp_f32 (arguments <= 0).
        bf16x8_t pf_hi[QT], pf_lo[QT];
        auto softmax = [&](auto masked_tag) {
            constexpr bool kMask = decltype(masked_tag)::value;
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
                float s[8];
                float m_new = mx[qt];
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float v = st[qt][nt][r];
                        if constexpr (Q8) v *= scale_log2e * ksc[nt][r];
                        if constexpr (kMask) v = j0 + 16 * nt + 4 * g + r < my_len[qt] ? v : -INFINITY;
                        s[4 * nt + r] = v;
                        m_new = fmaxf(m_new, v);
                    }
                m_new = rows_max(m_new);
                const float safe = m_new == -INFINITY ? 0.f : m_new;
                const float c = Q8 ? 1.f : scale_log2e;   // (one-byte pools: already in the scores)
                const float off = -safe * c;
                const float alpha = __builtin_amdgcn_exp2f(fmaf(mx[qt], c, off));
                mx[qt] = m_new;
                // The weights reach the second product as hi + lo with both parts bf16 (hi by
                // truncation, lo = bf16(p - hi)): 16 significant bits, so P . V keeps the accuracy
                // of fp32 weights (the reference multiplies fp32 probabilities,
                // driver/cuda/src/ops/attention_naive_paged.cu:148-317), and the normaliser sums
                // the unrounded values, as the decode kernel does.
                float sum = 0.f;
                uint32_t hi[4], lo[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    float p0 = __builtin_amdgcn_exp2f(fmaf(s[e], c, off));
                    float p1 = __builtin_amdgcn_exp2f(fmaf(s[e + 1], c, off));
                    sum += p0 + p1;
                    if constexpr (Q8) {   // V = float(code) * scale: the scale rides on the weight
                        p0 *= vsc[e >> 2][e & 3];
                        p1 *= vsc[e >> 2][(e & 3) + 1];
                    }
                    const uint32_t u0 = __float_as_uint(p0), u1 = __float_as_uint(p1);
                    hi[e >> 1] = __builtin_amdgcn_perm(u1, u0, 0x07060302u);
                    lo[e >> 1] = pack_bf16x2(p0 - __uint_as_float(u0 & 0xFFFF0000u),
                                             p1 - __uint_as_float(u1 & 0xFFFF0000u));
                }
                pf_hi[qt] = __builtin_bit_cast(bf16x8_t, u32x4_t{hi[0], hi[1], hi[2], hi[3]});
                pf_lo[qt] = __builtin_bit_cast(bf16x8_t, u32x4_t{lo[0], lo[1], lo[2], lo[3]});
                lsum[qt] = lsum[qt] * alpha + sum;
                if (alpha != 1.0f) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) acc[qt][dt] *= alpha;
                }
            }
        };
        if (j0 + kStepKeys <= min_len) softmax(std::false_type{});
        else softmax(std::true_type{});
        // O^T += V^T . P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16x8_t vf = __builtin_bit_cast(
                bf16x8_t, *reinterpret_cast<const u32x4_t*>(&Vt[(16 * dt + l16) * kVtStride + 8 * g]));
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
                acc[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_hi[qt], acc[qt][dt], 0, 0, 0);
                acc[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_lo[qt], acc[qt][dt], 0, 0, 0);
            }
        }
        __syncthreads();   // step j + 1 is staged, step j read
    };

    if (kmax > 0) issue(0, 0);
    if (kmax > kStepKeys) issue(1, kStepKeys);
    if (kmax > 0) stage(0);
    if (kmax > 2 * kStepKeys) issue(0, 2 * kStepKeys);
    __syncthreads();
    for (int j0 = 0; j0 < kmax; j0 += PF * kStepKeys) {   // unrolled by PF: compile-time register slots
        step(0, j0);
        if (j0 + kStepKeys < kmax) step(1, j0 + kStepKeys);
    }

    // normalise and store: this lane holds, for its query, d = 16 dt + 4 g + r
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float l = lsum[qt];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        const int m = wv * 16 * QT + qt * 16 + l16;
        if (m % TQ >= n_rows) continue;
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        uint16_t* op = o + (static_cast<size_t>(my_row[qt]) * hq + my_head[qt]) * D + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const f32x4_t a = acc[qt][dt];
            const u32x2_t w = {pack_bf16x2(a[0] * inv, a[1] * inv), pack_bf16x2(a[2] * inv, a[3] * inv)};
            *reinterpret_cast<u32x2_t*>(op + 16 * dt) = w;
        }
    }
}

template <int D, int GQA, int QT>
int launch_tiles(int kv_format, const uint16_t* q, const void* k_pages, const void* v_pages,
                 const float* k_scales, const float* v_scales, uint16_t* o,
                 const uint32_t* page_indices, const uint32_t* row_begin, const int32_t* row_len,
                 const int32_t* tile_start, const int32_t* tile_rows, int num_tiles, int hq, int hk,
                 int ps, float scale, hipStream_t stream) {
    const dim3 grid(num_tiles, hk);
    const float sl = scale * 1.4426950408889634f;
    if (kv_format == PIE_HIP_KV_BF16)
        hipLaunchKernelGGL((attn_prefill_tile_kernel<D, GQA, QT, kKvBf16>), grid, dim3(kTileThreads), 0, stream, q,
                           k_pages, v_pages, k_scales, v_scales, o, page_indices, row_begin, row_len,
                           tile_start, tile_rows, hq, hk, ps, sl);
    else if (kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD)
        hipLaunchKernelGGL((attn_prefill_tile_kernel<D, GQA, QT, kKvInt8>), grid, dim3(kTileThreads), 0, stream, q,
                           k_pages, v_pages, k_scales, v_scales, o, page_indices, row_begin, row_len,
                           tile_start, tile_rows, hq, hk, ps, sl);
    else if (kv_format == PIE_HIP_KV_FP8_E5M2)
        hipLaunchKernelGGL((attn_prefill_tile_kernel<D, GQA, QT, kKvBf8>), grid, dim3(kTileThreads), 0, stream, q,
                           k_pages, v_pages, k_scales, v_scales, o, page_indices, row_begin, row_len,
                           tile_start, tile_rows, hq, hk, ps, sl);
    else
        hipLaunchKernelGGL((attn_prefill_tile_kernel<D, GQA, QT, kKvFp8>), grid, dim3(kTileThreads), 0, stream, q,
                           k_pages, v_pages, k_scales, v_scales, o, page_indices, row_begin, row_len,
                           tile_start, tile_rows, hq, hk, ps, sl);
    return launch_status();
}

}  // namespace
}  // namespace pie_hip

extern "C" int pie_hip_attn_prefill_tile_rows(int num_q_heads, int num_kv_heads) {
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0) return 0;
    const int gqa = num_q_heads / num_kv_heads;
    if (gqa != 1 && gqa != 2 && gqa != 4 && gqa != 8) return 0;
    return pie_hip::kBlockRows / gqa;
}

extern "C" int pie_hip_attn_prefill_tiles_kvq(int kv_format, const uint16_t* q, const void* k_pages,
                                              const void* v_pages, const float* k_scales,
                                              const float* v_scales, uint16_t* o,
                                              const uint32_t* kv_page_indices,
                                              const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                              const int32_t* tile_row_start, const int32_t* tile_num_rows,
                                              int num_tiles, int rows_per_tile, int num_q_heads,
                                              int num_kv_heads, int head_dim, int page_size,
                                              float sm_scale, void* stream) {
    using namespace pie_hip;
    if (!q || !k_pages || !v_pages || !o || !kv_page_indices || !row_page_begin || !row_kv_len ||
        !tile_row_start || !tile_num_rows || num_tiles <= 0 || page_size <= 0)
        return PIE_HIP_ERR_INVALID;
    {
        const bool scaled = kv_format == PIE_HIP_KV_INT8_PER_TOKEN_HEAD || kv_format == PIE_HIP_KV_FP8_PER_TOKEN_HEAD;
        if (kv_format != PIE_HIP_KV_BF16 && kv_format != PIE_HIP_KV_FP8_E4M3 && kv_format != PIE_HIP_KV_FP8_E5M2 && !scaled)
            return PIE_HIP_ERR_UNSUPPORTED;
        if (scaled != (k_scales != nullptr) || scaled != (v_scales != nullptr)) return PIE_HIP_ERR_INVALID;
    }
    const int cap = pie_hip_attn_prefill_tile_rows(num_q_heads, num_kv_heads);
    if (cap == 0 || page_size % 16 != 0 || num_tiles > 0x7FFFFFFF / 2 || num_kv_heads > 65535)
        return PIE_HIP_ERR_UNSUPPORTED;
    if (rows_per_tile != cap && rows_per_tile * 2 != cap) return PIE_HIP_ERR_UNSUPPORTED;
    const bool big = rows_per_tile == cap;
    const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf(static_cast<float>(head_dim));
    const int gqa = num_q_heads / num_kv_heads;
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PIE_TILE_CASE(DD, GG)                                                                       \
    if (head_dim == DD && gqa == GG)                                                                \
        return big ? launch_tiles<DD, GG, 2>(kv_format, q, k_pages, v_pages, k_scales, v_scales, o, \
                                             kv_page_indices, row_page_begin, row_kv_len,           \
                                             tile_row_start, tile_num_rows, num_tiles, num_q_heads, \
                                             num_kv_heads, page_size, scale, st)                    \
                   : launch_tiles<DD, GG, 1>(kv_format, q, k_pages, v_pages, k_scales, v_scales, o, \
                                             kv_page_indices, row_page_begin, row_kv_len,           \
                                             tile_row_start, tile_num_rows, num_tiles, num_q_heads, \
                                             num_kv_heads, page_size, scale, st);
    PIE_TILE_CASE(128, 1)
    PIE_TILE_CASE(128, 2)
    PIE_TILE_CASE(128, 4)
    PIE_TILE_CASE(128, 8)
    PIE_TILE_CASE(64, 1)
    PIE_TILE_CASE(64, 2)
    PIE_TILE_CASE(64, 4)
    PIE_TILE_CASE(64, 8)
#undef PIE_TILE_CASE
    return PIE_HIP_ERR_UNSUPPORTED;
}

extern "C" int pie_hip_attn_prefill_tiles(const uint16_t* q, const uint16_t* k_pages,
                                          const uint16_t* v_pages, uint16_t* o,
                                          const uint32_t* kv_page_indices,
                                          const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                          const int32_t* tile_row_start, const int32_t* tile_num_rows,
                                          int num_tiles, int rows_per_tile, int num_q_heads,
                                          int num_kv_heads, int head_dim, int page_size,
                                          float sm_scale, void* stream) {
    return pie_hip_attn_prefill_tiles_kvq(PIE_HIP_KV_BF16, q, k_pages, v_pages, nullptr, nullptr, o,
                                          kv_page_indices, row_page_begin, row_kv_len, tile_row_start,
                                          tile_num_rows, num_tiles, rows_per_tile, num_q_heads,
                                          num_kv_heads, head_dim, page_size, sm_scale, stream);
}
