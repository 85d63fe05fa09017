"""CPU oracle for the Pie driver forward-pass kernels — TEST INFRASTRUCTURE ONLY.

A ctypes front end over `oracle/src/*.c` (a plain-C restatement of the
reference's arithmetic; each C function cites the reference lines it follows).
Only `tests/`, `__graft_entry__.smoke()` and `bench.py`'s `cpu_baseline` leg may
import this package, and only as the checker / reported CPU baseline.  The
product (`pie_amd/`) must never import it.

bf16 tensors travel as `numpy.uint16` arrays of raw bits.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libpie_oracle.so"
_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            from . import build as _build

            _build.build()
        _lib = C.CDLL(str(_LIB_PATH))
    return _lib


# ---------------------------------------------------------------- bf16 helpers
def f32_to_bf16(x) -> np.ndarray:
    """Round-to-nearest-even float32 -> bf16 bits (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(b) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# ---------------------------------------------------------------- W4A16
def unpack_w4(packed: np.ndarray, out_dim: int, in_dim: int) -> np.ndarray:
    packed = _c(packed, np.uint32)
    q = np.empty((out_dim, in_dim), np.int8)
    lib().orc_unpack_w4(_p(packed), _p(q), C.c_int(out_dim), C.c_int(in_dim))
    return q


def pack_w4(q: np.ndarray) -> np.ndarray:
    q = _c(q, np.int8)
    out_dim, in_dim = q.shape
    packed = np.empty((out_dim, in_dim // 8), np.uint32)
    lib().orc_pack_w4(_p(q), _p(packed), C.c_int(out_dim), C.c_int(in_dim))
    return packed


def dequant_w4a16(packed, scale_bf16, out_dim: int, in_dim: int, group: int) -> np.ndarray:
    packed = _c(packed, np.uint32)
    scale_bf16 = _c(scale_bf16, np.uint16)
    out = np.empty((out_dim, in_dim), np.uint16)
    lib().orc_dequant_w4a16(_p(packed), _p(scale_bf16), _p(out), C.c_int(out_dim),
                            C.c_int(in_dim), C.c_int(group))
    return out


def gemm_w4a16(act_bf16, packed, scale_bf16, group: int, mode: int = 0, y_in=None,
               want_abs: bool = False):
    """Returns (y_f32[M,N], y_bf16[M,N]) (+ abs_sum[M,N] float64 if want_abs)."""
    act = _c(act_bf16, np.uint16)
    M, K = act.shape
    packed = _c(packed, np.uint32)
    N = packed.shape[0]
    scale = _c(scale_bf16, np.uint16)
    y32 = np.empty((M, N), np.float32)
    y16 = np.empty((M, N), np.uint16)
    ab = np.empty((M, N), np.float64) if want_abs else None
    yin = None if y_in is None else _c(y_in, np.uint16)
    lib().orc_gemm_w4a16(_p(act), _p(packed), _p(scale), _p(yin), _p(y32), _p(y16), _p(ab),
                         C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(group),
                         C.c_int(0 if y_in is None else 1), C.c_int(mode))
    return (y32, y16, ab) if want_abs else (y32, y16)


# ---------------------------------------------------------------- int8 per channel
def quant_int8_per_channel(w_bf16):
    w = _c(w_bf16, np.uint16)
    rows, cols = w.shape
    q = np.empty((rows, cols), np.int8)
    s = np.empty((rows,), np.float32)
    lib().orc_quant_int8_per_channel(_p(w), _p(q), _p(s), C.c_int(rows), C.c_int(cols))
    return q, s


def dequant_int8_per_channel(q, scale_inv):
    q = _c(q, np.int8)
    s = _c(scale_inv, np.float32)
    rows, cols = q.shape
    out = np.empty((rows, cols), np.uint16)
    lib().orc_dequant_int8_per_channel(_p(q), _p(s), _p(out), C.c_int(rows), C.c_int(cols))
    return out


def gemm_w8a16(act_bf16, q, scale_inv, mode: int = 0, y_in=None, want_abs: bool = False):
    act = _c(act_bf16, np.uint16)
    M, K = act.shape
    q = _c(q, np.int8)
    N = q.shape[0]
    s = _c(scale_inv, np.float32)
    y32 = np.empty((M, N), np.float32)
    y16 = np.empty((M, N), np.uint16)
    ab = np.empty((M, N), np.float64) if want_abs else None
    yin = None if y_in is None else _c(y_in, np.uint16)
    lib().orc_gemm_w8a16(_p(act), _p(q), _p(s), _p(yin), _p(y32), _p(y16), _p(ab), C.c_int(M),
                         C.c_int(N), C.c_int(K), C.c_int(0 if y_in is None else 1),
                         C.c_int(mode))
    return (y32, y16, ab) if want_abs else (y32, y16)


# ---------------------------------------------------------------- paged attention
def attn_paged(q_bf16, k_pages, v_pages, qo_indptr, page_indices, page_indptr, last_lens,
               hq: int, hk: int, d: int, ps: int, sm_scale: float = -1.0, mode: int = 0):
    """General paged attention (decode = one query row per request).
    Returns (o_f32[T,hq,d], o_bf16[T,hq,d], lse[T,hq])."""
    q = _c(q_bf16, np.uint16)
    T = q.shape[0]
    kp = _c(k_pages, np.uint16)
    vp = _c(v_pages, np.uint16)
    qo = _c(qo_indptr, np.uint32)
    pi = _c(page_indices, np.uint32)
    pp = _c(page_indptr, np.uint32)
    ll = _c(last_lens, np.uint32)
    R = len(ll)
    o32 = np.zeros((T, hq, d), np.float32)
    o16 = np.zeros((T, hq, d), np.uint16)
    lse = np.zeros((T, hq), np.float32)
    lib().orc_attn_paged(_p(q), _p(kp), _p(vp), _p(o32), _p(o16), _p(lse), _p(qo), _p(pi), _p(pp),
                         _p(ll), C.c_int(R), C.c_int(hq), C.c_int(hk), C.c_int(d), C.c_int(ps),
                         C.c_float(sm_scale), C.c_int(mode))
    return o32, o16, lse


def attn_decode_paged(q_bf16, k_pages, v_pages, page_indices, page_indptr, last_lens, hq, hk, d,
                      ps, sm_scale: float = -1.0, mode: int = 0):
    R = len(last_lens)
    return attn_paged(q_bf16, k_pages, v_pages, np.arange(R + 1, dtype=np.uint32), page_indices,
                      page_indptr, last_lens, hq, hk, d, ps, sm_scale, mode)


def kv_write(k_curr, v_curr, k_pages, v_pages, qo_indptr, page_indices, page_indptr, last_lens,
             hk: int, d: int, ps: int):
    """In-place scatter of this step's K/V rows into the (uint16) page pools."""
    kc = _c(k_curr, np.uint16)
    vc = _c(v_curr, np.uint16)
    assert k_pages.dtype == np.uint16 and k_pages.flags.c_contiguous
    assert v_pages.dtype == np.uint16 and v_pages.flags.c_contiguous
    qo = _c(qo_indptr, np.uint32)
    pi = _c(page_indices, np.uint32)
    pp = _c(page_indptr, np.uint32)
    ll = _c(last_lens, np.uint32)
    lib().orc_kv_write(_p(kc), _p(vc), _p(k_pages), _p(v_pages), _p(qo), _p(pi), _p(pp), _p(ll),
                       C.c_int(len(ll)), C.c_int(hk), C.c_int(d), C.c_int(ps))


# ---------------------------------------------------------------- per-layer ops
def embed(tokens, table_bf16, vocab=None):
    t = _c(tokens, np.uint32)
    tab = _c(table_bf16, np.uint16)
    V, H = tab.shape
    y = np.empty((len(t), H), np.uint16)
    lib().orc_embed(_p(t), _p(tab), _p(y), C.c_int(len(t)), C.c_int(H), C.c_int(vocab or V))
    return y


def rmsnorm(x_bf16, w_bf16, eps, residual=None):
    """Returns y (and the updated x when a residual is given)."""
    x = np.array(x_bf16, dtype=np.uint16, order="C", copy=True)
    rows, H = x.shape
    w = _c(w_bf16, np.uint16)
    r = None if residual is None else _c(residual, np.uint16)
    y = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(r), _p(w), _p(y), C.c_int(rows), C.c_int(H), C.c_float(eps))
    return y if residual is None else (y, x)


def rope_inv_freq(d, theta, factor=0.0, low_freq_factor=1.0, high_freq_factor=4.0,
                  original_max_pos=8192):
    out = np.empty((d // 2,), np.float32)
    lib().orc_rope_inv_freq(_p(out), C.c_int(d), C.c_float(theta), C.c_float(factor),
                            C.c_float(low_freq_factor), C.c_float(high_freq_factor),
                            C.c_int(original_max_pos))
    return out


def rope_inv_freq_yarn(d, theta, factor, beta_fast=32.0, beta_slow=1.0, original_max_pos=4096):
    out = np.empty((d // 2,), np.float32)
    lib().orc_rope_inv_freq_yarn(_p(out), C.c_int(d), C.c_float(theta), C.c_float(factor), C.c_float(beta_fast),
                                 C.c_float(beta_slow), C.c_int(original_max_pos))
    return out


def rope_table(positions, inv_freq, d):
    pos = _c(positions, np.int32)
    f = _c(inv_freq, np.float32)
    tab = np.empty((len(pos), d), np.float32)
    lib().orc_rope_table(_p(pos), _p(f), _p(tab), C.c_int(len(pos)), C.c_int(d))
    return tab


def qkv_rope_kvwrite(packed, k_pages, v_pages, table, kv_slots, hq, hk, d, interleaved,
                     q_norm_w=None, k_norm_w=None, eps=1e-6):
    """Returns q_out; k_pages / v_pages (uint16, C-contiguous) are updated in place."""
    pk = _c(packed, np.uint16)
    N = pk.shape[0]
    q_out = np.zeros((N, hq, d), np.uint16)
    tab = _c(table, np.float32)
    sl = _c(kv_slots, np.int64)
    assert k_pages.dtype == np.uint16 and k_pages.flags.c_contiguous
    assert v_pages.dtype == np.uint16 and v_pages.flags.c_contiguous
    qn = None if q_norm_w is None else _c(q_norm_w, np.uint16)
    kn = None if k_norm_w is None else _c(k_norm_w, np.uint16)
    lib().orc_qkv_rope_kvwrite(_p(pk), _p(q_out), _p(k_pages), _p(v_pages), _p(qn), _p(kn), _p(tab),
                               _p(sl), C.c_int(N), C.c_int(hq), C.c_int(hk), C.c_int(d),
                               C.c_int(interleaved), C.c_float(eps))
    return q_out


def swiglu(gate_up_bf16):
    gu = _c(gate_up_bf16, np.uint16)
    N, two_i = gu.shape
    y = np.empty((N, two_i // 2), np.uint16)
    lib().orc_swiglu(_p(gu), _p(y), C.c_int(N), C.c_int(two_i // 2))
    return y


def argmax_bf16(logits_bf16):
    lg = _c(logits_bf16, np.uint16)
    rows, V = lg.shape
    out = np.empty((rows,), np.uint32)
    lib().orc_argmax_bf16(_p(lg), _p(out), C.c_int(rows), C.c_int(V))
    return out


def gemm_bf16(act_bf16, w_bf16, mode: int = 0, y_in=None, want_abs: bool = False):
    act = _c(act_bf16, np.uint16)
    M, K = act.shape
    w = _c(w_bf16, np.uint16)
    N = w.shape[0]
    y32 = np.empty((M, N), np.float32)
    y16 = np.empty((M, N), np.uint16)
    ab = np.empty((M, N), np.float64) if want_abs else None
    yin = None if y_in is None else _c(y_in, np.uint16)
    lib().orc_gemm_bf16(_p(act), _p(w), _p(yin), _p(y32), _p(y16), _p(ab), C.c_int(M), C.c_int(N),
                        C.c_int(K), C.c_int(0 if y_in is None else 1), C.c_int(mode))
    return (y32, y16, ab) if want_abs else (y32, y16)


# ---------------------------------------------------------------- fp8 e4m3fn per channel
def fp8_decode(b) -> np.ndarray:
    b = _c(b, np.uint8)
    out = np.empty(b.shape, np.float32)
    lib().orc_fp8_decode(_p(b), _p(out), C.c_size_t(b.size))
    return out


def quant_fp8_per_channel(w_bf16):
    w = _c(w_bf16, np.uint16)
    rows, cols = w.shape
    q = np.empty((rows, cols), np.uint8)
    s = np.empty((rows,), np.float32)
    lib().orc_quant_fp8_per_channel(_p(w), _p(q), _p(s), C.c_int(rows), C.c_int(cols))
    return q, s


def gemm_fp8(act_bf16, q, scale_inv, mode: int = 0, y_in=None, want_abs: bool = False):
    act = _c(act_bf16, np.uint16)
    M, K = act.shape
    q = _c(q, np.uint8)
    N = q.shape[0]
    s = _c(scale_inv, np.float32)
    y32 = np.empty((M, N), np.float32)
    y16 = np.empty((M, N), np.uint16)
    ab = np.empty((M, N), np.float64) if want_abs else None
    yin = None if y_in is None else _c(y_in, np.uint16)
    lib().orc_gemm_fp8(_p(act), _p(q), _p(s), _p(yin), _p(y32), _p(y16), _p(ab), C.c_int(M),
                       C.c_int(N), C.c_int(K), C.c_int(0 if y_in is None else 1), C.c_int(mode))
    return (y32, y16, ab) if want_abs else (y32, y16)


def topk_softmax(logits_bf16, top_k: int, renorm: bool = True):
    """(idx int32 [N, k], weights f32 [N, k]) — driver/cuda/src/kernels/topk_softmax.cu:19-86;
    renorm=False leaves the chosen experts' probabilities undivided (norm_topk = false,
    driver/portable/src/graph_common.cpp:279-283)."""
    lg = _c(logits_bf16, np.uint16)
    N, E = lg.shape
    idx = np.empty((N, top_k), np.int32)
    w = np.empty((N, top_k), np.float32)
    lib().orc_topk_softmax_opt(_p(lg), _p(idx), _p(w), C.c_int(N), C.c_int(E), C.c_int(top_k), C.c_int(1 if renorm else 0))
    return idx, w


def moe_combine(y_routes_bf16, topk_w, out_bf16=None):
    """out[t] (+)= sum_k w[t,k] * y_routes[t*k + k] (driver/cuda/src/kernels/moe_dispatch.cu:152-196).
    y_routes: [N*k, H] in (token, k) order; `out_bf16` given = accumulate onto it."""
    w = _c(topk_w, np.float32)
    N, K = w.shape
    yr = _c(y_routes_bf16, np.uint16)
    H = yr.shape[1]
    add = out_bf16 is not None
    out = np.array(out_bf16, np.uint16, copy=True) if add else np.zeros((N, H), np.uint16)
    out = np.ascontiguousarray(out)
    lib().orc_moe_combine(_p(yr), _p(w), _p(out), C.c_int(N), C.c_int(K), C.c_int(H), C.c_int(int(add)))
    return out


def brle_allow(runs, pos: int, n_kv: int, window: int = 0) -> np.ndarray:
    """uint8 [n_kv]: keys visible to a token at `pos` carrying the BRLE `runs`
    (build_attn_mask_f16, driver/portable/src/plan.cpp:54-94)."""
    r = _c(np.asarray(runs, np.uint32), np.uint32)
    out = np.zeros(max(n_kv, 1), np.uint8)
    lib().orc_brle_allow(_p(r), C.c_size_t(r.size), C.c_int(pos), C.c_int(n_kv), C.c_int(window), _p(out))
    return out[:n_kv]


KV_FORMATS = {"bf16": 0, "fp8_e4m3": 1, "int8_per_token_head": 2, "fp8_per_token_head": 3, "fp8_e5m2": 4,
              "fp4_e2m1": 5, "nvfp4": 5}


def kv_quant_rows(x_bf16, fmt: str):
    """KV-cache quantisation of (token, head) rows [rows, d] bf16
    (driver/cuda/src/kernels/kv_paged.cu:155-297).  Returns (codes u8 [rows, d], scales f32 [rows]
    or None for fp8_e4m3, dequantised f32 [rows, d] = float(code) * scale)."""
    x = _c(x_bf16, np.uint16)
    rows, d = x.shape
    if KV_FORMATS[fmt] == 5:
        # 4-bit e2m1 codes, two per byte, and one scale per block of 16 elements; the dequantised
        # values are bf16(level * scale) as the reference's attention reads them
        codes = np.zeros((rows, (d + 1) // 2), np.uint8)
        scales = np.ones((rows, (d + 15) // 16), np.float32)
        deq = np.zeros((rows, d), np.float32)
        lib().orc_kv_quant_rows(_p(x), _p(codes), _p(scales), _p(deq), C.c_int(rows), C.c_int(d), C.c_int(5))
        return codes, scales, deq
    codes = np.zeros((rows, d), np.uint8)
    scales = np.ones(rows, np.float32)
    deq = np.zeros((rows, d), np.float32)
    lib().orc_kv_quant_rows(_p(x), _p(codes), _p(scales), _p(deq), C.c_int(rows), C.c_int(d),
                            C.c_int(KV_FORMATS[fmt]))
    return codes, (None if fmt in ("fp8_e4m3", "fp8_e5m2") else scales), deq


def attn_rows_f32kv(q_bf16, k_pages_f32, v_pages_f32, page_indices, row_begin, row_len, hq, hk, d, ps,
                    sm_scale=-1.0, mode=2):
    """attn_rows over pools of dequantised f32 K / V values (one-byte KV-cache formats)."""
    q = _c(q_bf16, np.uint16)
    rows = q.shape[0]
    kp, vp_ = _c(k_pages_f32, np.float32), _c(v_pages_f32, np.float32)
    pi = _c(np.asarray(page_indices, np.uint32), np.uint32)
    rb = _c(np.asarray(row_begin, np.uint32), np.uint32)
    rl = _c(np.asarray(row_len, np.int32), np.int32)
    o32 = np.zeros((rows, hq, d), np.float32)
    o16 = np.zeros((rows, hq, d), np.uint16)
    lse = np.zeros((rows, hq), np.float32)
    lib().orc_attn_rows_f32kv(_p(q), _p(kp), _p(vp_), _p(o32), _p(o16), _p(lse), _p(pi), _p(rb), _p(rl),
                              C.c_int(rows), C.c_int(hq), C.c_int(hk), C.c_int(d), C.c_int(ps),
                              C.c_float(sm_scale), C.c_int(mode), None, None)
    return o32, o16, lse


def attn_rows_masked(q_bf16, k_pages, v_pages, page_indices, row_begin, row_len, hq, hk, d, ps,
                     allow_rows, sm_scale=-1.0, mode=2):
    """Per-row extents with per-row visibility: allow_rows[r] is None or a uint8 array over the
    row's keys.  Returns (o_f32, o_bf16, lse)."""
    q = _c(q_bf16, np.uint16)
    rows = q.shape[0]
    kp, vp_ = _c(k_pages, np.uint16), _c(v_pages, np.uint16)
    pi = _c(np.asarray(page_indices, np.uint32), np.uint32)
    rb = _c(np.asarray(row_begin, np.uint32), np.uint32)
    rl = _c(np.asarray(row_len, np.int32), np.int32)
    offs, chunks, at = [], [], 0
    for r in range(rows):
        if allow_rows[r] is None:
            offs.append(-1)
        else:
            a = np.asarray(allow_rows[r], np.uint8)
            assert a.size >= rl[r]
            chunks.append(a)
            offs.append(at)
            at += a.size
    allow = _c(np.concatenate(chunks) if chunks else np.zeros(1, np.uint8), np.uint8)
    off = _c(np.asarray(offs, np.int64), np.int64)
    o32 = np.zeros((rows, hq, d), np.float32)
    o16 = np.zeros((rows, hq, d), np.uint16)
    lse = np.zeros((rows, hq), np.float32)
    lib().orc_attn_rows_masked(_p(q), _p(kp), _p(vp_), _p(o32), _p(o16), _p(lse), _p(pi), _p(rb), _p(rl),
                               C.c_int(rows), C.c_int(hq), C.c_int(hk), C.c_int(d), C.c_int(ps),
                               C.c_float(sm_scale), C.c_int(mode), _p(allow), _p(off))
    return o32, o16, lse


# ---------------------------------------------------------------- samplers
SAMPLER_KINDS = {"multinomial": 0, "top_k": 1, "top_p": 2, "min_p": 3, "top_k_top_p": 4,
                 "dist": 6, "raw_logits": 7, "logprob": 8, "logprobs": 9, "entropy": 10}


def pcg32_sequence(seed: int, stream: int, n: int) -> np.ndarray:
    """n outputs of PCG32 seeded like Pcg32(seed, stream) (driver/portable/src/sampler.cpp:31-57)."""
    out = np.empty(n, np.uint32)
    lib().orc_pcg32_sequence(C.c_uint64(seed), C.c_uint64(stream), _p(out), C.c_int(n))
    return out


def pcg32_first_uniform(seed: int) -> float:
    """The uniform a slot with wire seed `seed` draws: first output of the default stream."""
    f = lib().orc_pcg32_first_uniform
    f.restype = C.c_float
    return float(f(C.c_uint64(seed)))


def apply_brle_logit_mask(logits_f32, runs) -> np.ndarray:
    lg = np.array(logits_f32, np.float32, copy=True)
    r = _c(np.asarray(runs, np.uint32), np.uint32)
    lib().orc_apply_brle_logit_mask(_p(lg), C.c_int(lg.shape[-1]), _p(r), C.c_size_t(r.size))
    return lg


def softmax_temperature(logits_f32, temperature: float) -> np.ndarray:
    lg = _c(logits_f32, np.float32)
    out = np.empty_like(lg)
    lib().orc_softmax_temperature(_p(lg), C.c_int(lg.size), C.c_float(temperature), _p(out))
    return out


def sample_token(logits_f32, kind, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, u=None, seed=0):
    """(token, margin) of one slot (sample_token, driver/portable/src/sampler.cpp:345-409).
    `u` overrides the uniform the seed would draw."""
    lg = _c(logits_f32, np.float32)
    k = SAMPLER_KINDS[kind] if isinstance(kind, str) else int(kind)
    if u is None:
        u = pcg32_first_uniform(seed)
    tok = C.c_uint32(0)
    mg = C.c_float(0)
    rc = lib().orc_sample_token(_p(lg), C.c_int(lg.size), C.c_int(k), C.c_float(temperature),
                                C.c_uint32(top_k), C.c_float(top_p), C.c_float(min_p), C.c_float(u),
                                C.byref(tok), C.byref(mg))
    if rc != 0:
        raise ValueError("sampler kind produces no token")
    return int(tok.value), float(mg.value)


def distribution(logits_f32, temperature: float, k: int):
    lg = _c(logits_f32, np.float32)
    ids = np.empty(lg.size, np.uint32)
    vals = np.empty(lg.size, np.float32)
    n = lib().orc_distribution(_p(lg), C.c_int(lg.size), C.c_float(temperature), C.c_uint32(k),
                               _p(ids), _p(vals))
    return ids[:n].copy(), vals[:n].copy()


def logprobs_at(logits_f32, labels) -> np.ndarray:
    lg = _c(logits_f32, np.float32)
    lb = _c(np.asarray(labels, np.uint32), np.uint32)
    out = np.empty(lb.size, np.float32)
    if lib().orc_logprobs_at(_p(lg), C.c_int(lg.size), _p(lb), C.c_int(lb.size), _p(out)) != 0:
        raise ValueError("label outside the vocabulary")
    return out


def entropy(logits_f32) -> float:
    lg = _c(logits_f32, np.float32)
    f = lib().orc_entropy
    f.restype = C.c_float
    return float(f(_p(lg), C.c_int(lg.size)))
