"""Python mirror of the reference driver's kernel-launcher interface.

Each function takes torch-ROCm device tensors, checks shapes/dtypes on the host
(the kernels trust their arguments), and calls the C ABI of
`libpie_hip_kernels.so` on torch's current stream.  Names follow the reference's
`launch_*` / `gemm_act_x_w` vocabulary (driver/cuda/src/kernels, driver/cuda/src/ops).
Nothing here computes: without the HIP library these functions raise.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import torch

from ._lib import kernels

STATUS = {0: "ok", 1: "invalid argument", 2: "unsupported shape", 3: "launch error"}


class KernelError(RuntimeError):
    pass


def _check(status: int, what: str) -> None:
    if status != 0:
        raise KernelError(f"{what}: {STATUS.get(status, status)}")


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _dev(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


# ---------------------------------------------------------------- weight views
@dataclass
class WeightView:
    """A [N, K] linear weight in one of the reference's storage formats
    (`WeightView`, driver/cuda/src/ops/gemm.hpp).

    kind "int4b8": `data` int32/uint32 [N, K/8], `scale` bf16 [N, K/group]
    kind "int8":   `data` int8 [N, K], `scale` f32 or bf16 [N] (= absmax/127)
    kind "fp8":    `data` uint8 (e4m3fn) [N, K], `scale` f32 or bf16 [N]
    kind "bf16":   `data` bf16 [N, K]
    """

    kind: str
    data: torch.Tensor
    scale: Optional[torch.Tensor] = None
    group_size: int = 0
    N: int = 0
    K: int = 0


def int4b8_view(packed: torch.Tensor, scale: torch.Tensor, group_size: int) -> WeightView:
    if packed.dtype == torch.int32:
        pass
    elif packed.dtype != torch.uint32:
        raise KernelError("packed int4 weights must be int32/uint32")
    N, words = packed.shape
    return WeightView("int4b8", packed, scale, group_size, N, words * 8)


# ---------------------------------------------------------------- W4A16
def unpack_w4(packed: torch.Tensor) -> torch.Tensor:
    """int8 [N, K] of (nibble - 8); nibble j of a word is element 8*w + j."""
    N, words = packed.shape
    q = torch.empty((N, words * 8), dtype=torch.int8, device=packed.device)
    _check(kernels().pie_hip_unpack_w4(_ptr(packed), _ptr(q), N, words * 8, _stream()),
           "pie_hip_unpack_w4")
    return q


def dequant_wna16_int4b8_to_bf16(packed: torch.Tensor, scale: torch.Tensor,
                                 group_size: int) -> torch.Tensor:
    _dev(scale, torch.bfloat16, "scale")
    N, words = packed.shape
    K = words * 8
    if scale.shape != (N, K // group_size):
        raise KernelError(f"scale shape {tuple(scale.shape)} != {(N, K // group_size)}")
    out = torch.empty((N, K), dtype=torch.bfloat16, device=packed.device)
    _check(kernels().pie_hip_dequant_w4a16(_ptr(packed), _ptr(scale), _ptr(out), N, K,
                                           group_size, _stream()), "pie_hip_dequant_w4a16")
    return out


def gemv_w4a16(act: torch.Tensor, w: WeightView, y: Optional[torch.Tensor] = None,
               beta: int = 0, rows_per_wave: int = 0, waves_per_simd: int = 0) -> torch.Tensor:
    """y[M,N] = act[M,K] · dequant(W)[N,K]^T (+ y if beta), M <= 32."""
    _dev(act, torch.bfloat16, "act")
    _dev(w.scale, torch.bfloat16, "scale")
    M, K = act.shape
    if K != w.K:
        raise KernelError(f"act K={K} != weight K={w.K}")
    if tuple(w.scale.shape) != (w.N, K // w.group_size):
        raise KernelError("scale shape does not match [N, K/group]")
    if y is None:
        if beta:
            raise KernelError("beta=1 needs an existing y")
        y = torch.empty((M, w.N), dtype=torch.bfloat16, device=act.device)
    _dev(y, torch.bfloat16, "y")
    if tuple(y.shape) != (M, w.N):
        raise KernelError("y shape mismatch")
    lib = kernels()
    if rows_per_wave or waves_per_simd:
        st = lib.pie_hip_gemv_w4a16_tuned(_ptr(act), _ptr(w.data), _ptr(w.scale), _ptr(y), M,
                                          w.N, K, w.group_size, beta, rows_per_wave,
                                          waves_per_simd, _stream())
    else:
        st = lib.pie_hip_gemv_w4a16(_ptr(act), _ptr(w.data), _ptr(w.scale), _ptr(y), M, w.N, K,
                                    w.group_size, beta, _stream())
    _check(st, "pie_hip_gemv_w4a16")
    return y


# ---------------------------------------------------------------- paged decode attention
def attn_decode_workspace_bytes(R: int, hq: int, hk: int, d: int, max_kv_len: int) -> int:
    lib = kernels()
    lib.pie_hip_attn_decode_workspace_bytes.restype = C.c_size_t
    return int(lib.pie_hip_attn_decode_workspace_bytes(R, hq, hk, d, max_kv_len))


def attention_paged_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                           kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                           kv_last_page_lens: torch.Tensor, max_kv_len: int,
                           sm_scale: float = -1.0, o: Optional[torch.Tensor] = None,
                           lse: Optional[torch.Tensor] = None,
                           workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """o[R,hq,d] for one query token per request (launch_attention_naive_paged_decode,
    driver/cuda/src/ops/attention_naive_paged.hpp:57-69).  Page-table tensors are int32
    device tensors holding the wire u32 values."""
    _dev(q, torch.bfloat16, "q")
    _dev(k_pages, torch.bfloat16, "k_pages")
    _dev(v_pages, torch.bfloat16, "v_pages")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_lens", kv_last_page_lens)):
        _dev(t, torch.int32, name)
    R, hq, d = q.shape
    num_pages, ps, hk, d2 = k_pages.shape
    if d2 != d or v_pages.shape != k_pages.shape:
        raise KernelError("k_pages/v_pages must be [pages, page_size, hk, d] with q's d")
    if kv_page_indptr.numel() != R + 1 or kv_last_page_lens.numel() != R:
        raise KernelError("page table arrays do not match the request count")
    if o is None:
        o = torch.empty_like(q)
    _dev(o, torch.bfloat16, "o")
    if lse is not None:
        _dev(lse, torch.float32, "lse")
    need = attn_decode_workspace_bytes(R, hq, hk, d, max_kv_len)
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    wbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    st = kernels().pie_hip_attn_decode_paged(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(o), _ptr(lse), _ptr(kv_page_indices),
        _ptr(kv_page_indptr), _ptr(kv_last_page_lens), R, hq, hk, d, ps, C.c_float(sm_scale),
        max_kv_len, _ptr(workspace), C.c_size_t(wbytes), _stream())
    _check(st, "pie_hip_attn_decode_paged")
    return o


# ---------------------------------------------------------------- other weight formats
def _row_scale_args(scale: torch.Tensor):
    if scale.dtype == torch.float32:
        return _ptr(scale), _ptr(None)
    if scale.dtype == torch.bfloat16:
        return _ptr(None), _ptr(scale)
    raise KernelError("row scale must be float32 or bfloat16")


def _gemv_out(act, N, y, beta):
    M = act.shape[0]
    if y is None:
        if beta:
            raise KernelError("beta=1 needs an existing y")
        y = torch.empty((M, N), dtype=torch.bfloat16, device=act.device)
    _dev(y, torch.bfloat16, "y")
    if tuple(y.shape) != (M, N):
        raise KernelError("y shape mismatch")
    return y


def gemv_w8a16(act, q_int8, scale_inv, y=None, beta=0):
    """y = (act · q^T) * scale_inv[n]; q int8 [N,K], scale_inv f32 or bf16 [N]."""
    _dev(act, torch.bfloat16, "act")
    _dev(q_int8, torch.int8, "q_int8")
    N, K = q_int8.shape
    if act.shape[1] != K or scale_inv.numel() != N or not scale_inv.is_contiguous():
        raise KernelError("shape mismatch")
    y = _gemv_out(act, N, y, beta)
    sf, sb = _row_scale_args(scale_inv)
    _check(kernels().pie_hip_gemv_w8a16(_ptr(act), _ptr(q_int8), sf, sb, _ptr(y), act.shape[0], N,
                                        K, beta, _stream()), "pie_hip_gemv_w8a16")
    return y


def gemv_fp8(act, w_e4m3, scale_inv, y=None, beta=0):
    """y = (act · fp8(w)^T) * scale_inv[n]; w uint8 holding OCP e4m3fn bytes [N,K]."""
    _dev(act, torch.bfloat16, "act")
    _dev(w_e4m3, torch.uint8, "w_e4m3")
    N, K = w_e4m3.shape
    if act.shape[1] != K or scale_inv.numel() != N or not scale_inv.is_contiguous():
        raise KernelError("shape mismatch")
    y = _gemv_out(act, N, y, beta)
    sf, sb = _row_scale_args(scale_inv)
    _check(kernels().pie_hip_gemv_fp8(_ptr(act), _ptr(w_e4m3), sf, sb, _ptr(y), act.shape[0], N, K,
                                      beta, _stream()), "pie_hip_gemv_fp8")
    return y


def gemv_bf16(act, w, y=None, beta=0):
    _dev(act, torch.bfloat16, "act")
    _dev(w, torch.bfloat16, "w")
    N, K = w.shape
    if act.shape[1] != K:
        raise KernelError("shape mismatch")
    y = _gemv_out(act, N, y, beta)
    _check(kernels().pie_hip_gemv_bf16(_ptr(act), _ptr(w), _ptr(y), act.shape[0], N, K, beta,
                                       _stream()), "pie_hip_gemv_bf16")
    return y


# ---------------------------------------------------------------- per-layer kernels
def embed_bf16(token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    _dev(token_ids, torch.int32, "token_ids")
    _dev(table, torch.bfloat16, "table")
    V, H = table.shape
    y = torch.empty((token_ids.numel(), H), dtype=torch.bfloat16, device=table.device)
    _check(kernels().pie_hip_embed(_ptr(token_ids), _ptr(table), _ptr(y), token_ids.numel(), H, V,
                                   _stream()), "pie_hip_embed")
    return y


def rmsnorm_bf16(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    _dev(x, torch.bfloat16, "x")
    _dev(weight, torch.bfloat16, "weight")
    rows, H = x.shape
    y = torch.empty_like(x)
    _check(kernels().pie_hip_rmsnorm(_ptr(x), _ptr(weight), _ptr(y), rows, H, C.c_float(eps),
                                     _stream()), "pie_hip_rmsnorm")
    return y


def residual_add_rmsnorm_bf16(hidden: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                              eps: float) -> torch.Tensor:
    """hidden += residual (in place, rounded to bf16); returns rmsnorm(hidden)."""
    for n, t in (("hidden", hidden), ("residual", residual), ("weight", weight)):
        _dev(t, torch.bfloat16, n)
    rows, H = hidden.shape
    y = torch.empty_like(hidden)
    _check(kernels().pie_hip_residual_rmsnorm(_ptr(hidden), _ptr(residual), _ptr(weight), _ptr(y),
                                              rows, H, C.c_float(eps), _stream()),
           "pie_hip_residual_rmsnorm")
    return y


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, head_dim: int) -> torch.Tensor:
    _dev(positions, torch.int32, "positions")
    _dev(inv_freq, torch.float32, "inv_freq")
    if inv_freq.numel() != head_dim // 2:
        raise KernelError("inv_freq must have head_dim/2 entries")
    tab = torch.empty((positions.numel(), head_dim), dtype=torch.float32, device=positions.device)
    _check(kernels().pie_hip_rope_table(_ptr(positions), _ptr(inv_freq), _ptr(tab),
                                        positions.numel(), head_dim, _stream()),
           "pie_hip_rope_table")
    return tab


def qkv_rope_kvwrite(packed, k_pages, v_pages, table, kv_slots, hq, hk, d, interleaved,
                     q_norm_w=None, k_norm_w=None, eps=1e-6):
    _dev(packed, torch.bfloat16, "packed")
    _dev(k_pages, torch.bfloat16, "k_pages")
    _dev(v_pages, torch.bfloat16, "v_pages")
    _dev(table, torch.float32, "rope_table")
    _dev(kv_slots, torch.int64, "kv_slots")
    N = packed.shape[0]
    if packed.shape[1] != (hq + 2 * hk) * d or tuple(table.shape) != (N, d) or kv_slots.numel() != N:
        raise KernelError("shape mismatch")
    total_slots = k_pages.numel() // (hk * d)
    if N and int(kv_slots.max()) >= total_slots:
        raise KernelError("kv slot out of range")
    q_out = torch.empty((N, hq, d), dtype=torch.bfloat16, device=packed.device)
    _check(kernels().pie_hip_qkv_rope_kvwrite(
        _ptr(packed), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _ptr(q_norm_w), _ptr(k_norm_w),
        _ptr(table), _ptr(kv_slots), N, hq, hk, d, int(interleaved), C.c_float(eps), _stream()),
        "pie_hip_qkv_rope_kvwrite")
    return q_out


def swiglu_bf16(gate_up: torch.Tensor) -> torch.Tensor:
    _dev(gate_up, torch.bfloat16, "gate_up")
    N, two_i = gate_up.shape
    y = torch.empty((N, two_i // 2), dtype=torch.bfloat16, device=gate_up.device)
    _check(kernels().pie_hip_swiglu(_ptr(gate_up), _ptr(y), N, two_i // 2, _stream()),
           "pie_hip_swiglu")
    return y


def argmax_bf16(logits: torch.Tensor) -> torch.Tensor:
    _dev(logits, torch.bfloat16, "logits")
    rows, V = logits.shape
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    _check(kernels().pie_hip_argmax(_ptr(logits), _ptr(out), rows, V, _stream()), "pie_hip_argmax")
    return out


def lm_head_argmax(act: torch.Tensor, w: torch.Tensor, norm_weight: Optional[torch.Tensor] = None,
                   eps: float = 1e-5):
    """bf16 lm_head GEMV with the greedy token in its wake (up to four rows).  Returns
    (logits [M, V] bf16, tokens [M] int32)."""
    _dev(act, torch.bfloat16, "act")
    _dev(w, torch.bfloat16, "w")
    M, H = act.shape
    V = w.shape[0]
    if w.shape[1] != H:
        raise KernelError("shape mismatch")
    lib = kernels()
    lib.pie_hip_lm_head_argmax_workspace_bytes.restype = C.c_size_t
    need = int(lib.pie_hip_lm_head_argmax_workspace_bytes(M, V))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=act.device)
    logits = torch.empty((M, V), dtype=torch.bfloat16, device=act.device)
    toks = torch.empty(M, dtype=torch.int32, device=act.device)
    _check(lib.pie_hip_lm_head_argmax(_ptr(act), _ptr(norm_weight), C.c_float(eps), _ptr(w), _ptr(logits),
                                      _ptr(toks), M, V, H, _ptr(ws), C.c_size_t(need), _stream()),
           "pie_hip_lm_head_argmax")
    return logits, toks


def copy_kv_pages(pool: torch.Tensor, srcs: torch.Tensor, dsts: torch.Tensor) -> None:
    """pool[dsts[i]] <- pool[srcs[i]] over the leading (page) dimension."""
    _dev(srcs, torch.int32, "srcs")
    _dev(dsts, torch.int32, "dsts")
    if not pool.is_contiguous() or srcs.numel() != dsts.numel():
        raise KernelError("bad copy arguments")
    n_pages = pool.shape[0]
    if srcs.numel() and (int(srcs.max()) >= n_pages or int(dsts.max()) >= n_pages):
        raise KernelError("page id out of range")
    page_bytes = pool[0].numel() * pool.element_size()
    _check(kernels().pie_hip_copy_kv_pages(_ptr(pool), _ptr(srcs), _ptr(dsts), srcs.numel(),
                                           C.c_size_t(page_bytes), _stream()),
           "pie_hip_copy_kv_pages")


FMT = {"int4b8": 0, "int8": 1, "fp8": 2, "bf16": 3}


def linear_fused(act: torch.Tensor, w: WeightView, norm_weight: Optional[torch.Tensor] = None,
                 eps: float = 1e-5, y: Optional[torch.Tensor] = None, beta: int = 0,
                 swiglu: bool = False) -> torch.Tensor:
    """y = epilogue(rmsnorm?(act) · W^T): optional RMSNorm fused into the activation staging,
    optional SwiGLU over interleaved (gate_i, up_i) weight rows (then y is [M, N/2])."""
    _dev(act, torch.bfloat16, "act")
    M, K = act.shape
    if K != w.K:
        raise KernelError("act K != weight K")
    if norm_weight is not None:
        _dev(norm_weight, torch.bfloat16, "norm_weight")
        if norm_weight.numel() != K:
            raise KernelError("norm weight must have K entries")
    n_out = w.N // 2 if swiglu else w.N
    if y is None:
        if beta:
            raise KernelError("beta=1 needs an existing y")
        y = torch.empty((M, n_out), dtype=torch.bfloat16, device=act.device)
    _dev(y, torch.bfloat16, "y")
    if tuple(y.shape) != (M, n_out):
        raise KernelError("y shape mismatch")
    scale_is_bf16 = int(w.scale is not None and w.scale.dtype == torch.bfloat16)
    st = kernels().pie_hip_linear_fused(FMT[w.kind], _ptr(act), _ptr(norm_weight), C.c_float(eps),
                                        _ptr(w.data), _ptr(w.scale), scale_is_bf16, w.group_size,
                                        _ptr(y), M, w.N, K, beta, int(swiglu), _stream())
    _check(st, "pie_hip_linear_fused")
    return y


def repack_mfma_tiles(w: WeightView) -> WeightView:
    """The weight (and int4 group scales) in the skinny GEMM's tile-major layout: a WeightView
    whose kind carries the suffix '+tiled' for gemm_skinny / moe_grouped_gemm."""
    rows = w.data.shape[0] if w.data.dim() == 2 else w.data.shape[0] * w.data.shape[1]
    flat = w.data.reshape(rows, -1).contiguous()
    row_bytes = flat.shape[1] * flat.element_size()
    dst = torch.empty(((rows + 15) // 16 * 16, flat.shape[1]), dtype=flat.dtype, device=flat.device)
    # (int4: the codes of every 32-bit word are also put in the order the kernels decode them in)
    repack = kernels().pie_hip_repack_mfma_tiles_int4 if w.kind == "int4b8" else kernels().pie_hip_repack_mfma_tiles
    _check(repack(_ptr(flat), _ptr(dst), rows, C.c_size_t(row_bytes), _stream()), "pie_hip_repack_mfma_tiles")
    scale = w.scale
    if w.kind == "int4b8":
        sf = w.scale.reshape(rows, -1).contiguous()
        _dev(sf, torch.bfloat16, "scale")
        scale = torch.empty(((rows + 15) // 16 * 16, sf.shape[1]), dtype=torch.bfloat16, device=sf.device)
        _check(kernels().pie_hip_repack_scale_tiles(_ptr(sf), _ptr(scale), rows, sf.shape[1], _stream()),
               "pie_hip_repack_scale_tiles")
    return WeightView(w.kind + "+tiled", dst, scale, w.group_size, w.N, w.K)


def gemm_skinny(act: torch.Tensor, w: WeightView, y: Optional[torch.Tensor] = None, beta: int = 0,
                swiglu: bool = False) -> torch.Tensor:
    """Matrix-core weight-only GEMM for a handful to a few dozen activation rows (same contract as
    `linear_fused` without the norm).  A WeightView from repack_mfma_tiles runs the tile-major
    entry point."""
    _dev(act, torch.bfloat16, "act")
    M, K = act.shape
    if K != w.K:
        raise KernelError("act K != weight K")
    n_out = w.N // 2 if swiglu else w.N
    if y is None:
        if beta:
            raise KernelError("beta=1 needs an existing y")
        y = torch.empty((M, n_out), dtype=torch.bfloat16, device=act.device)
    _dev(y, torch.bfloat16, "y")
    if tuple(y.shape) != (M, n_out):
        raise KernelError("y shape mismatch")
    scale_is_bf16 = int(w.scale is not None and w.scale.dtype == torch.bfloat16)
    tiled = w.kind.endswith("+tiled")
    fn = kernels().pie_hip_gemm_skinny_tiled if tiled else kernels().pie_hip_gemm_skinny
    st = fn(FMT[w.kind.split("+")[0]], _ptr(act), _ptr(w.data), _ptr(w.scale), scale_is_bf16, w.group_size,
            _ptr(y), M, w.N, K, beta, int(swiglu), _stream())
    _check(st, "pie_hip_gemm_skinny")
    return y


def moe_grouped_gemm(act: torch.Tensor, route_act_rows: Optional[torch.Tensor],
                     expert_offsets: torch.Tensor, kind: str, weights: torch.Tensor,
                     scales: Optional[torch.Tensor], N: int, K: int, rows_hint: int,
                     group_size: int = 0, swiglu: bool = False,
                     y: Optional[torch.Tensor] = None, num_routes: Optional[int] = None,
                     tiled: bool = False) -> torch.Tensor:
    """One skinny GEMM per expert in a single launch.  `weights` is [E, N, K] in the format's
    element type (int4b8: [E, N, K/8] words), `scales` [E, N] (int4b8: [E, N, K/G]);
    `expert_offsets` int32 [E+1] are the first route row of each expert (routes sorted by expert);
    `route_act_rows` int32 [routes] names each route's activation row (None: route r reads
    act[r])."""
    _dev(act, torch.bfloat16, "act")
    _dev(expert_offsets, torch.int32, "expert_offsets")
    E = expert_offsets.numel() - 1
    if weights.shape[0] != E:
        raise KernelError("weights must have one [N, K] block per expert")
    if route_act_rows is not None:
        _dev(route_act_rows, torch.int32, "route_act_rows")
        routes = route_act_rows.numel()
    else:
        routes = act.shape[0] if num_routes is None else num_routes
    if act.shape[1] != K:
        raise KernelError("act K mismatch")
    if not weights.is_contiguous() or (scales is not None and not scales.is_contiguous()):
        raise KernelError("weights/scales must be contiguous")
    n_out = N // 2 if swiglu else N
    if y is None:
        y = torch.empty((routes, n_out), dtype=torch.bfloat16, device=act.device)
    _dev(y, torch.bfloat16, "y")
    if tuple(y.shape) != (routes, n_out):
        raise KernelError("y shape mismatch")
    wstride = weights[0].numel() * weights.element_size()
    sstride = 0 if scales is None else scales[0].numel() * scales.element_size()
    scale_is_bf16 = int(scales is not None and scales.dtype == torch.bfloat16)
    fn = kernels().pie_hip_moe_grouped_gemm_tiled if tiled else kernels().pie_hip_moe_grouped_gemm
    st = fn(
        FMT[kind], _ptr(act), _ptr(route_act_rows), _ptr(expert_offsets), E, int(rows_hint),
        _ptr(weights), C.c_size_t(wstride), _ptr(scales), C.c_size_t(sstride), scale_is_bf16,
        group_size, _ptr(y), N, K, int(swiglu), _stream())
    _check(st, "pie_hip_moe_grouped_gemm")
    return y


def moe_route(router_logits: torch.Tensor, top_k: int, renormalize: bool = True):
    """Softmax -> top-k -> renormalise per token (renormalize=False: the chosen experts keep their
    softmax probabilities), plus the expert-sorted route layout.
    Returns (topk_idx [T,k] int32, topk_w [T,k] f32, expert_offsets [E+1] int32,
    route_token [T*k] int32, route_pos [T*k] int32)."""
    _dev(router_logits, torch.bfloat16, "router_logits")
    T, E = router_logits.shape
    d = router_logits.device
    idx = torch.empty((T, top_k), dtype=torch.int32, device=d)
    w = torch.empty((T, top_k), dtype=torch.float32, device=d)
    offs = torch.empty(E + 1, dtype=torch.int32, device=d)
    rtok = torch.empty(T * top_k, dtype=torch.int32, device=d)
    rpos = torch.empty(T * top_k, dtype=torch.int32, device=d)
    _check(kernels().pie_hip_moe_route_opt(_ptr(router_logits), _ptr(idx), _ptr(w), _ptr(offs), _ptr(rtok),
                                           _ptr(rpos), T, E, top_k, int(renormalize), _stream()),
           "pie_hip_moe_route_opt")
    return idx, w, offs, rtok, rpos


def moe_combine(y_routes: torch.Tensor, route_pos: torch.Tensor, topk_w: torch.Tensor,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] (+)= sum_k w[t,k] * y_routes[route_pos[t,k]]; `out` given = accumulate onto it."""
    _dev(y_routes, torch.bfloat16, "y_routes")
    _dev(route_pos, torch.int32, "route_pos")
    _dev(topk_w, torch.float32, "topk_w")
    T, K = topk_w.shape
    H = y_routes.shape[1]
    add = out is not None
    if out is None:
        out = torch.empty((T, H), dtype=torch.bfloat16, device=y_routes.device)
    _dev(out, torch.bfloat16, "out")
    _check(kernels().pie_hip_moe_combine(_ptr(y_routes), _ptr(route_pos), _ptr(topk_w), _ptr(out), T, K,
                                         H, int(add), _stream()), "pie_hip_moe_combine")
    return out


def moe_combine_norm(y_routes: torch.Tensor, route_pos: torch.Tensor, topk_w: torch.Tensor,
                     out: torch.Tensor, norm_weight: torch.Tensor, eps: float) -> torch.Tensor:
    """moe_combine onto `out` (in place) and the RMSNorm of the updated rows in one launch;
    returns the normalised rows."""
    for n, t, dt in (("y_routes", y_routes, torch.bfloat16), ("route_pos", route_pos, torch.int32),
                     ("topk_w", topk_w, torch.float32), ("out", out, torch.bfloat16),
                     ("norm_weight", norm_weight, torch.bfloat16)):
        _dev(t, dt, n)
    T, K = topk_w.shape
    H = y_routes.shape[1]
    if tuple(out.shape) != (T, H) or norm_weight.numel() != H:
        raise KernelError("shape mismatch")
    xn = torch.empty_like(out)
    _check(kernels().pie_hip_moe_combine_norm(_ptr(y_routes), _ptr(route_pos), _ptr(topk_w), _ptr(out),
                                              _ptr(norm_weight), C.c_float(eps), _ptr(xn), T, K, H, _stream()),
           "pie_hip_moe_combine_norm")
    return xn


def moe_norm_route(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, router: torch.Tensor, top_k: int,
                   renormalize: bool = True):
    """RMSNorm of the rows, router logits, softmax -> top-k and the expert-sorted layout for a
    decode batch.  Returns (xn [T,H], logits [T,E] bf16, topk_idx, topk_w, expert_offsets,
    route_token, route_pos) as `moe_route` does."""
    _dev(x, torch.bfloat16, "x")
    _dev(norm_weight, torch.bfloat16, "norm_weight")
    _dev(router, torch.bfloat16, "router")
    T, H = x.shape
    E = router.shape[0]
    if router.shape[1] != H or norm_weight.numel() != H:
        raise KernelError("shape mismatch")
    d = x.device
    xn = torch.empty_like(x)
    logits = torch.empty((T, E), dtype=torch.bfloat16, device=d)
    idx = torch.empty((T, top_k), dtype=torch.int32, device=d)
    w = torch.empty((T, top_k), dtype=torch.float32, device=d)
    offs = torch.empty(E + 1, dtype=torch.int32, device=d)
    rtok = torch.empty(T * top_k, dtype=torch.int32, device=d)
    rpos = torch.empty(T * top_k, dtype=torch.int32, device=d)
    _check(kernels().pie_hip_moe_norm_route(_ptr(x), _ptr(norm_weight), C.c_float(eps), _ptr(router), _ptr(xn),
                                            _ptr(logits), _ptr(idx), _ptr(w), _ptr(offs), _ptr(rtok), _ptr(rpos),
                                            T, H, E, top_k, int(renormalize), _stream()),
           "pie_hip_moe_norm_route")
    return xn, logits, idx, w, offs, rtok, rpos


def gemm_mfma(act: torch.Tensor, w: WeightView, y: Optional[torch.Tensor] = None, beta: int = 0,
              swiglu: bool = False, split_k: bool = False,
              workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Tiled matrix-core GEMM for large M (weights dequantised to bf16 while staged).
    split_k: the decode-batch form (K shares + fp32 partials in `workspace`, allocated here
    when not given)."""
    _dev(act, torch.bfloat16, "act")
    M, K = act.shape
    if K != w.K:
        raise KernelError("act K != weight K")
    n_out = w.N // 2 if swiglu else w.N
    if y is None:
        if beta:
            raise KernelError("beta=1 needs an existing y")
        y = torch.empty((M, n_out), dtype=torch.bfloat16, device=act.device)
    _dev(y, torch.bfloat16, "y")
    if tuple(y.shape) != (M, n_out):
        raise KernelError("y shape mismatch")
    scale_is_bf16 = int(w.scale is not None and w.scale.dtype == torch.bfloat16)
    lib = kernels()
    if split_k:
        lib.pie_hip_gemm_mfma_workspace_bytes.restype = C.c_size_t
        need = int(lib.pie_hip_gemm_mfma_workspace_bytes(M, w.N, K))
        if need:
            if workspace is None:
                workspace = torch.empty(need, dtype=torch.uint8, device=act.device)
            if workspace.numel() * workspace.element_size() < need:
                raise KernelError("workspace too small")
            st = lib.pie_hip_gemm_mfma_splitk(FMT[w.kind], _ptr(act), _ptr(w.data), _ptr(w.scale),
                                              scale_is_bf16, w.group_size, _ptr(y), M, w.N, K, beta,
                                              int(swiglu), _ptr(workspace), C.c_size_t(need), _stream())
            _check(st, "pie_hip_gemm_mfma_splitk")
            return y
    st = lib.pie_hip_gemm_mfma(FMT[w.kind], _ptr(act), _ptr(w.data), _ptr(w.scale),
                               scale_is_bf16, w.group_size, _ptr(y), M, w.N, K, beta,
                               int(swiglu), _stream())
    _check(st, "pie_hip_gemm_mfma")
    return y


def gemm_mfma_workspace_bytes(M: int, N: int, K: int) -> int:
    lib = kernels()
    lib.pie_hip_gemm_mfma_workspace_bytes.restype = C.c_size_t
    return int(lib.pie_hip_gemm_mfma_workspace_bytes(M, N, K))


def pair_qk_rows(w: WeightView, hq: int, hk: int, d: int) -> WeightView:
    """The load-time row order of a fused q|k|v weight whose RoPE pairs are (i, i + d/2): inside
    every q and k head, row 2i <- row i and row 2i+1 <- row i + d/2 (data and scales together;
    V rows stay).  The fused epilogues with pairing = 2 undo it at the store."""
    half = d // 2
    head = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1)
    idx = torch.cat([head + h * d for h in range(hq + hk)] +
                    [torch.arange((hq + hk) * d, (hq + 2 * hk) * d)]).to(w.data.device)
    data = w.data.reshape(w.N, -1)[idx].reshape(w.data.shape).contiguous()
    scale = None if w.scale is None else w.scale.reshape(w.N, -1)[idx].reshape(w.scale.shape).contiguous()
    return WeightView(w.kind, data, scale, w.group_size, w.N, w.K)


def qkv_rope_fused(act: torch.Tensor, w: WeightView, table: torch.Tensor, kv_slots: torch.Tensor,
                   k_pages: torch.Tensor, v_pages: torch.Tensor, hq: int, hk: int, d: int,
                   norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-5,
                   pairing: int = 1) -> torch.Tensor:
    """Fused q|k|v projection + RoPE + KV-cache write (decode rows).  Returns q [M, hq, d]; k / v
    land in their slots of the pools.  pairing 1: adjacent pairs; 2: half-split pairs over
    weights whose q / k rows were re-ordered with `pair_qk_rows`."""
    _dev(act, torch.bfloat16, "act")
    _dev(table, torch.float32, "rope_table")
    _dev(kv_slots, torch.int64, "kv_slots")
    _dev(k_pages, torch.bfloat16, "k_pages")
    _dev(v_pages, torch.bfloat16, "v_pages")
    M, K = act.shape
    if K != w.K or w.N != (hq + 2 * hk) * d or tuple(table.shape) != (M, d) or kv_slots.numel() != M:
        raise KernelError("shape mismatch")
    if M and int(kv_slots.max()) >= k_pages.numel() // (hk * d):
        raise KernelError("kv slot out of range")
    q_out = torch.empty((M, hq, d), dtype=torch.bfloat16, device=act.device)
    scale_is_bf16 = int(w.scale is not None and w.scale.dtype == torch.bfloat16)
    _check(kernels().pie_hip_qkv_rope_fused(
        FMT[w.kind], _ptr(act), _ptr(norm_weight), C.c_float(eps), _ptr(w.data), _ptr(w.scale),
        scale_is_bf16, w.group_size, M, K, _ptr(table), _ptr(kv_slots), _ptr(q_out), _ptr(k_pages),
        _ptr(v_pages), hq, hk, d, pairing, _stream()), "pie_hip_qkv_rope_fused")
    return q_out


def qkv_rope_skinny_tiled(act: torch.Tensor, w: WeightView, table: torch.Tensor, kv_slots: torch.Tensor,
                          k_pages: torch.Tensor, v_pages: torch.Tensor, hq: int, hk: int, d: int,
                          pairing: int = 1) -> torch.Tensor:
    """q|k|v projection over tile-major weights + RoPE + KV-cache write for a decode batch (act
    already normalised).  Returns q [M, hq, d]; k / v land in their slots.  pairing as for
    `qkv_rope_fused`."""
    _dev(act, torch.bfloat16, "act")
    _dev(table, torch.float32, "rope_table")
    _dev(kv_slots, torch.int64, "kv_slots")
    _dev(k_pages, torch.bfloat16, "k_pages")
    _dev(v_pages, torch.bfloat16, "v_pages")
    if not w.kind.endswith("+tiled"):
        raise KernelError("tile-major weights expected (repack_mfma_tiles)")
    M, K = act.shape
    if K != w.K or w.N != (hq + 2 * hk) * d or tuple(table.shape) != (M, d) or kv_slots.numel() != M:
        raise KernelError("shape mismatch")
    if M and int(kv_slots.max()) >= k_pages.numel() // (hk * d):
        raise KernelError("kv slot out of range")
    q_out = torch.empty((M, hq, d), dtype=torch.bfloat16, device=act.device)
    scale_is_bf16 = int(w.scale is not None and w.scale.dtype == torch.bfloat16)
    _check(kernels().pie_hip_qkv_rope_skinny_tiled(
        FMT[w.kind[:-len("+tiled")]], _ptr(act), _ptr(w.data), _ptr(w.scale), scale_is_bf16, w.group_size,
        M, K, _ptr(table), _ptr(kv_slots), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), hq, hk, d,
        pairing, _stream()), "pie_hip_qkv_rope_skinny_tiled")
    return q_out


# ---------------------------------------------------------------- sampling
SAMPLER_KINDS = {"multinomial": 0, "top_k": 1, "top_p": 2, "min_p": 3, "top_k_top_p": 4,
                 "dist": 6, "raw_logits": 7, "logprob": 8, "logprobs": 9, "entropy": 10}


def brle_bounds(runs_per_slot, device) -> tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Cumulative run ends (u32, saturating) + per-slot offsets for `sample_gather_logits`."""
    if runs_per_slot is None or not any(len(r) for r in runs_per_slot):
        return None, None
    bounds, indptr = [], [0]
    for runs in runs_per_slot:
        acc = 0
        for r in runs:
            acc = min(acc + int(r), 0xFFFFFFFF)
            bounds.append(acc)
        indptr.append(len(bounds))
    import numpy as np
    b = torch.from_numpy(np.asarray(bounds, np.uint32).view(np.int32)).to(device)
    return b, torch.tensor(indptr, dtype=torch.int32, device=device)


def sample_gather_logits(logits: torch.Tensor, rows: Optional[torch.Tensor] = None,
                         mask_runs=None) -> torch.Tensor:
    """f32 copies of the sampled logits rows with per-slot BRLE logit masks applied
    (apply_brle_logit_mask, driver/portable/src/sampler.cpp:169-198)."""
    _dev(logits, torch.bfloat16, "logits")
    V = logits.shape[1]
    S = logits.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _dev(rows, torch.int32, "rows")
    bounds, indptr = brle_bounds(mask_runs, logits.device)
    if mask_runs is not None and len(mask_runs) != S:
        raise KernelError("one run list per slot expected")
    out = torch.empty((S, V), dtype=torch.float32, device=logits.device)
    _check(kernels().pie_hip_sample_gather_logits(_ptr(logits), _ptr(rows), _ptr(out), _ptr(bounds),
                                                  _ptr(indptr), S, V, _stream()),
           "pie_hip_sample_gather_logits")
    return out


def sample(logits_f32: torch.Tensor, kinds, temperature, top_k, top_p, min_p, uniform,
           out_counts=None, labels=None):
    """Runs every slot's sampler (sample_slot, driver/portable/src/sampler.cpp:308-343).
    Per-slot python lists in; returns (tokens u32 [S], values f32, ids u32, out_indptr) where
    slot s's dist / logprob / entropy payload is values[out_indptr[s]:out_indptr[s+1]]."""
    import numpy as np

    _dev(logits_f32, torch.float32, "logits_f32")
    S, V = logits_f32.shape
    dev = logits_f32.device
    kinds = [SAMPLER_KINDS[k] if isinstance(k, str) else int(k) for k in kinds]
    counts = list(out_counts) if out_counts is not None else [0] * S
    indptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    total = int(indptr[-1])
    lab = np.zeros(max(total, 1), np.uint32)
    if labels is not None:
        for s in range(S):
            if labels[s] is not None and len(labels[s]):
                if max(labels[s]) >= V:
                    raise KernelError("label outside the vocabulary")
                lab[indptr[s]:indptr[s + 1]] = labels[s]
    t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(np.asarray(a, dt))).to(dev)
    kind_t, temp_t = t(kinds, np.int32), t(temperature, np.float32)
    topk_t = t(np.asarray(top_k, np.uint32).view(np.int32), np.int32)
    topp_t, minp_t, u_t = t(top_p, np.float32), t(min_p, np.float32), t(uniform, np.float32)
    indptr_t = t(indptr, np.int32)
    lab_t = t(lab.view(np.int32), np.int32)
    tokens = torch.zeros(S, dtype=torch.int32, device=dev)
    values = torch.zeros(max(total, 1), dtype=torch.float32, device=dev)
    ids = torch.zeros(max(total, 1), dtype=torch.int32, device=dev)
    k = kernels()
    k.pie_hip_sample_workspace_bytes.restype = C.c_size_t
    need = int(k.pie_hip_sample_workspace_bytes(S, V))
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    _check(k.pie_hip_sample(_ptr(logits_f32), _ptr(kind_t), _ptr(temp_t), _ptr(topk_t), _ptr(topp_t),
                            _ptr(minp_t), _ptr(u_t), _ptr(indptr_t), _ptr(lab_t), _ptr(tokens),
                            _ptr(values), _ptr(ids), _ptr(ws), C.c_size_t(need), S, V, _stream()),
           "pie_hip_sample")
    return tokens, values, ids, indptr


# ---------------------------------------------------------------- per-row attention (prefill / mixed)
def attn_mask_bitmap(mask_runs, row_kv_len: torch.Tensor, max_kv_len: int, window: int = 0):
    """u16 [rows, ceil(max_kv_len/16)] visibility words from per-row BRLE runs
    (build_attn_mask_f16, driver/portable/src/plan.cpp:54-94).  Returns (bitmap, stride)."""
    _dev(row_kv_len, torch.int32, "row_kv_len")
    rows = row_kv_len.numel()
    if len(mask_runs) != rows:
        raise KernelError("one run list per row expected")
    bounds, indptr = brle_bounds(mask_runs, row_kv_len.device)
    if indptr is None:
        indptr = torch.zeros(rows + 1, dtype=torch.int32, device=row_kv_len.device)
        bounds = torch.zeros(1, dtype=torch.int32, device=row_kv_len.device)
    stride = max(1, (max_kv_len + 15) // 16)
    bitmap = torch.empty((rows, stride), dtype=torch.int16, device=row_kv_len.device)
    _check(kernels().pie_hip_attn_mask_bitmap(_ptr(bounds), _ptr(indptr), _ptr(row_kv_len), window,
                                              _ptr(bitmap), rows, stride, _stream()),
           "pie_hip_attn_mask_bitmap")
    return bitmap, stride


def attention_rows_paged(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                         kv_page_indices: torch.Tensor, row_page_begin: torch.Tensor,
                         row_kv_len: torch.Tensor, max_kv_len: int, mask_runs=None, window: int = 0,
                         lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """o[rows, hq, d]: query row r over the first row_kv_len[r] keys of the page list starting at
    kv_page_indices[row_page_begin[r]]; with `mask_runs` (per-row BRLE) or `window`, over the
    visible keys only."""
    _dev(q, torch.bfloat16, "q")
    _dev(k_pages, torch.bfloat16, "k_pages")
    for name, t in (("kv_page_indices", kv_page_indices), ("row_page_begin", row_page_begin),
                    ("row_kv_len", row_kv_len)):
        _dev(t, torch.int32, name)
    rows, hq, d = q.shape
    _, ps, hk, _ = k_pages.shape
    o = torch.empty_like(q)
    need = attn_decode_workspace_bytes(rows, hq, hk, d, max_kv_len)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    k = kernels()
    if mask_runs is None and window <= 0:
        st = k.pie_hip_attn_rows_paged(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(o), _ptr(lse),
                                       _ptr(kv_page_indices), _ptr(row_page_begin), _ptr(row_kv_len),
                                       rows, hq, hk, d, ps, C.c_float(-1.0), max_kv_len, _ptr(ws),
                                       C.c_size_t(need), _stream())
        _check(st, "pie_hip_attn_rows_paged")
        return o
    bitmap, stride = attn_mask_bitmap(mask_runs if mask_runs is not None else [[]] * rows,
                                      row_kv_len, max_kv_len, window)
    st = k.pie_hip_attn_rows_paged_masked(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(o), _ptr(lse),
                                          _ptr(kv_page_indices), _ptr(row_page_begin),
                                          _ptr(row_kv_len), _ptr(bitmap), stride, rows, hq, hk, d, ps,
                                          C.c_float(-1.0), max_kv_len, _ptr(ws), C.c_size_t(need),
                                          _stream())
    _check(st, "pie_hip_attn_rows_paged_masked")
    return o


def attn_decode_plan(rows: int, hk: int, max_kv_len: int):
    """(units_per_split, num_splits) of a decode attention launch."""
    ups, ns = C.c_int(0), C.c_int(0)
    _check(kernels().pie_hip_attn_decode_plan(rows, hk, max_kv_len, C.byref(ups), C.byref(ns)),
           "pie_hip_attn_decode_plan")
    return ups.value, ns.value


def attn_decode_is_chunked(fmt: str, rows: int, hk: int, max_kv_len: int) -> bool:
    """Whether a decode attention launch of this shape over pools of `fmt` takes the chunked form."""
    code = 0 if fmt == "bf16" else KV_FORMATS[fmt]
    return bool(kernels().pie_hip_attn_decode_is_chunked(code, rows, hk, max_kv_len))


def attention_rows_paged_partials(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                                  kv_page_indices: torch.Tensor, row_page_begin: torch.Tensor,
                                  row_kv_len: torch.Tensor, max_kv_len: int, fmt: str = "bf16",
                                  k_scales: Optional[torch.Tensor] = None,
                                  v_scales: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The split launch of `attention_rows_paged` (or `_kvq`) alone: returns the workspace holding
    the splits' partial results, for `linear_attn_merge`."""
    _dev(q, torch.bfloat16, "q")
    for name, t in (("kv_page_indices", kv_page_indices), ("row_page_begin", row_page_begin),
                    ("row_kv_len", row_kv_len)):
        _dev(t, torch.int32, name)
    rows, hq, d = q.shape
    _, ps, hk, _ = k_pages.shape
    need = attn_decode_workspace_bytes(rows, hq, hk, d, max_kv_len)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    st = kernels().pie_hip_attn_rows_paged_partials(
        KV_FORMATS[fmt], _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(k_scales), _ptr(v_scales),
        _ptr(kv_page_indices), _ptr(row_page_begin), _ptr(row_kv_len), rows, hq, hk, d, ps, C.c_float(-1.0),
        max_kv_len, _ptr(ws), C.c_size_t(need), _stream())
    _check(st, "pie_hip_attn_rows_paged_partials")
    return ws


def linear_attn_merge(ws: torch.Tensor, num_splits: int, units_per_split: int, row_kv_len: torch.Tensor,
                      hq: int, d: int, w: WeightView, y: Optional[torch.Tensor] = None,
                      beta: int = 0) -> torch.Tensor:
    """The output projection over the merged attention rows, merge included (one launch)."""
    _dev(row_kv_len, torch.int32, "row_kv_len")
    M = row_kv_len.numel()
    if w.K != hq * d:
        raise KernelError("weight K != hq * d")
    if y is None:
        if beta:
            raise KernelError("beta=1 needs an existing y")
        y = torch.empty((M, w.N), dtype=torch.bfloat16, device=ws.device)
    _dev(y, torch.bfloat16, "y")
    scale_is_bf16 = int(w.scale is not None and w.scale.dtype == torch.bfloat16)
    st = kernels().pie_hip_linear_attn_merge(FMT[w.kind], _ptr(ws), num_splits, units_per_split, _ptr(row_kv_len),
                                             hq, d, _ptr(w.data), _ptr(w.scale), scale_is_bf16, w.group_size,
                                             _ptr(y), M, w.N, beta, _stream())
    _check(st, "pie_hip_linear_attn_merge")
    return y


ATTN_STATIC_SCRATCH_BYTES = 16 << 20


def attention_rows_paged_static(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                                kv_page_indices: torch.Tensor, row_page_begin: torch.Tensor,
                                row_kv_len: torch.Tensor, max_kv_len: int, o: torch.Tensor,
                                lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`attention_rows_paged` through the entry point that allocates nothing: the caller brings
    the output `o`, the split partials live in the library's built-in per-GPU scratch array
    (ATTN_STATIC_SCRATCH_BYTES; larger batches raise).  No tensor is created here."""
    _dev(q, torch.bfloat16, "q")
    _dev(k_pages, torch.bfloat16, "k_pages")
    _dev(o, torch.bfloat16, "o")
    for name, t in (("kv_page_indices", kv_page_indices), ("row_page_begin", row_page_begin),
                    ("row_kv_len", row_kv_len)):
        _dev(t, torch.int32, name)
    rows, hq, d = q.shape
    _, ps, hk, _ = k_pages.shape
    if o.shape != q.shape:
        raise KernelError("o must have q's shape")
    st = kernels().pie_hip_attn_rows_paged_static(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(o), _ptr(lse), _ptr(kv_page_indices),
        _ptr(row_page_begin), _ptr(row_kv_len), rows, hq, hk, d, ps, C.c_float(-1.0), max_kv_len,
        _stream())
    _check(st, "pie_hip_attn_rows_paged_static")
    return o


def attn_prefill_tile_rows(hq: int, hk: int) -> int:
    """Most query rows one tile of `attention_prefill_tiles` may hold (0: unsupported head ratio)."""
    return int(kernels().pie_hip_attn_prefill_tile_rows(hq, hk))


def attention_prefill_tiles(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                            kv_page_indices: torch.Tensor, row_page_begin: torch.Tensor,
                            row_kv_len: torch.Tensor, tile_row_start: torch.Tensor,
                            tile_num_rows: torch.Tensor, rows_per_tile: Optional[int] = None) -> torch.Tensor:
    """Matrix-core prefill attention over tiles of consecutive rows that share a page list.
    rows_per_tile: `attn_prefill_tile_rows(hq, hk)` (default) or half of it."""
    _dev(q, torch.bfloat16, "q")
    _dev(k_pages, torch.bfloat16, "k_pages")
    for name, t in (("kv_page_indices", kv_page_indices), ("row_page_begin", row_page_begin),
                    ("row_kv_len", row_kv_len), ("tile_row_start", tile_row_start),
                    ("tile_num_rows", tile_num_rows)):
        _dev(t, torch.int32, name)
    rows, hq, d = q.shape
    _, ps, hk, _ = k_pages.shape
    o = torch.zeros_like(q)
    st = kernels().pie_hip_attn_prefill_tiles(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(o),
                                              _ptr(kv_page_indices), _ptr(row_page_begin),
                                              _ptr(row_kv_len), _ptr(tile_row_start), _ptr(tile_num_rows),
                                              tile_row_start.numel(),
                                              rows_per_tile or attn_prefill_tile_rows(hq, hk), hq, hk, d,
                                              ps, C.c_float(-1.0), _stream())
    _check(st, "pie_hip_attn_prefill_tiles")
    return o


KV_FORMATS = {"bf16": 0, "fp8_e4m3": 1, "int8_per_token_head": 2, "fp8_per_token_head": 3, "fp8_e5m2": 4,
              "fp4_e2m1": 5, "nvfp4": 5}


def attention_prefill_tiles_kvq(fmt: str, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                                k_scales: Optional[torch.Tensor], v_scales: Optional[torch.Tensor],
                                kv_page_indices: torch.Tensor, row_page_begin: torch.Tensor,
                                row_kv_len: torch.Tensor, tile_row_start: torch.Tensor,
                                tile_num_rows: torch.Tensor, rows_per_tile: Optional[int] = None) -> torch.Tensor:
    """`attention_prefill_tiles` over one-byte pools [pages, ps, hk, d] (+ f32 scales [pages, hk, ps])."""
    _dev(q, torch.bfloat16, "q")
    for name, t in (("kv_page_indices", kv_page_indices), ("row_page_begin", row_page_begin),
                    ("row_kv_len", row_kv_len), ("tile_row_start", tile_row_start),
                    ("tile_num_rows", tile_num_rows)):
        _dev(t, torch.int32, name)
    for t in (k_pages, v_pages):
        if t.element_size() != 1 or not t.is_contiguous():
            raise KernelError("pools must be contiguous one-byte [pages, ps, hk, d]")
    rows, hq, d = q.shape
    _, ps, hk, _ = k_pages.shape
    o = torch.zeros_like(q)
    st = kernels().pie_hip_attn_prefill_tiles_kvq(
        KV_FORMATS[fmt], _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(k_scales), _ptr(v_scales), _ptr(o),
        _ptr(kv_page_indices), _ptr(row_page_begin), _ptr(row_kv_len), _ptr(tile_row_start),
        _ptr(tile_num_rows), tile_row_start.numel(), rows_per_tile or attn_prefill_tile_rows(hq, hk), hq, hk,
        d, ps, C.c_float(-1.0), _stream())
    _check(st, "pie_hip_attn_prefill_tiles_kvq")
    return o


def kv_write_quant(fmt: str, k_rows: torch.Tensor, v_rows: torch.Tensor, kv_slots: torch.Tensor,
                   k_pages: torch.Tensor, v_pages: torch.Tensor,
                   k_scales: Optional[torch.Tensor] = None,
                   v_scales: Optional[torch.Tensor] = None) -> None:
    """Quantising KV write of rows [N, hk, d] bf16 into one-byte pools [pages, ps, hk, d]
    (+ f32 scales [pages, hk, ps] for the per-token-head formats)."""
    _dev(k_rows, torch.bfloat16, "k_rows")
    _dev(v_rows, torch.bfloat16, "v_rows")
    _dev(kv_slots, torch.int64, "kv_slots")
    N, hk, d = k_rows.shape
    if tuple(v_rows.shape) != (N, hk, d) or kv_slots.numel() != N:
        raise KernelError("shape mismatch")
    fp4 = KV_FORMATS[fmt] == 5          # two codes per byte, one scale per 16 elements
    dstore = d // 2 if fp4 else d
    for t in (k_pages, v_pages):
        if t.element_size() != 1 or not t.is_contiguous() or t.shape[-2:] != (hk, dstore):
            raise KernelError("pools must be contiguous one-byte [pages, ps, hk, d] (d/2 for the 4-bit format)")
    if N and int(kv_slots.max()) >= k_pages.numel() // (hk * dstore):
        raise KernelError("kv slot out of range")
    for sc in (k_scales, v_scales):
        if sc is not None:
            _dev(sc, torch.float32, "scales")
            if sc.numel() != k_pages.numel() // dstore * (d // 16 if fp4 else 1):
                raise KernelError("scales must be [pages, hk, ps] ([pages, hk, ps, d/16] for the 4-bit format)")
    _check(kernels().pie_hip_kv_write_quant(KV_FORMATS[fmt], _ptr(k_rows), _ptr(v_rows), _ptr(kv_slots),
                                            _ptr(k_pages), _ptr(v_pages), _ptr(k_scales), _ptr(v_scales),
                                            N, hk, d, k_pages.shape[1], _stream()), "pie_hip_kv_write_quant")


def kv_dequant_pages(fmt: str, k_pages: torch.Tensor, v_pages: torch.Tensor, k_scales: Optional[torch.Tensor],
                     v_scales: Optional[torch.Tensor], k_out: torch.Tensor, v_out: torch.Tensor,
                     page_ids: torch.Tensor) -> None:
    """Expand the named pages of a one-byte / 4-bit pool into bf16 pools [pages, ps, hk, d]."""
    _dev(k_out, torch.bfloat16, "k_out")
    _dev(v_out, torch.bfloat16, "v_out")
    _dev(page_ids, torch.int32, "page_ids")
    pages, ps, hk, d = k_out.shape
    if tuple(v_out.shape) != (pages, ps, hk, d) or k_pages.shape[0] != pages:
        raise KernelError("shape mismatch")
    if page_ids.numel() and int(page_ids.max()) >= pages:
        raise KernelError("page id out of range")
    _check(kernels().pie_hip_kv_dequant_pages(KV_FORMATS[fmt], _ptr(k_pages), _ptr(v_pages), _ptr(k_scales),
                                              _ptr(v_scales), _ptr(k_out), _ptr(v_out), _ptr(page_ids),
                                              page_ids.numel(), hk, d, ps, _stream()), "pie_hip_kv_dequant_pages")


def qkv_rope_kvwrite_quant(fmt: str, packed: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                           k_scales: Optional[torch.Tensor], v_scales: Optional[torch.Tensor],
                           table: torch.Tensor, kv_slots: torch.Tensor, hq: int, hk: int, d: int,
                           interleaved: bool, q_norm_w=None, k_norm_w=None, eps: float = 1e-6) -> torch.Tensor:
    """RoPE (+ optional per-head q/k norm) and the quantising KV write in one launch over packed
    q|k|v rows [N, (hq + 2 hk) d]; returns q [N, hq, d]."""
    _dev(packed, torch.bfloat16, "packed")
    _dev(table, torch.float32, "rope_table")
    _dev(kv_slots, torch.int64, "kv_slots")
    N = packed.shape[0]
    if packed.shape[1] != (hq + 2 * hk) * d or tuple(table.shape) != (N, d) or kv_slots.numel() != N:
        raise KernelError("shape mismatch")
    for t in (k_pages, v_pages):
        if t.element_size() != 1 or not t.is_contiguous() or t.shape[-2:] != (hk, d):
            raise KernelError("pools must be contiguous one-byte [pages, ps, hk, d]")
    if N and int(kv_slots.max()) >= k_pages.numel() // (hk * d):
        raise KernelError("kv slot out of range")
    for sc in (k_scales, v_scales):
        if sc is not None:
            _dev(sc, torch.float32, "scales")
            if sc.numel() != k_pages.numel() // d:
                raise KernelError("scales must be [pages, hk, ps]")
    q_out = torch.empty((N, hq, d), dtype=torch.bfloat16, device=packed.device)
    _check(kernels().pie_hip_qkv_rope_kvwrite_quant(
        KV_FORMATS[fmt], _ptr(packed), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _ptr(k_scales),
        _ptr(v_scales), _ptr(q_norm_w), _ptr(k_norm_w), _ptr(table), _ptr(kv_slots), N, hq, hk, d,
        k_pages.shape[1], int(interleaved), C.c_float(eps), _stream()), "pie_hip_qkv_rope_kvwrite_quant")
    return q_out


def attention_rows_paged_kvq(fmt: str, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                             k_scales: Optional[torch.Tensor], v_scales: Optional[torch.Tensor],
                             kv_page_indices: torch.Tensor, row_page_begin: torch.Tensor,
                             row_kv_len: torch.Tensor, lse: bool = False,
                             max_kv_len: Optional[int] = None, o: Optional[torch.Tensor] = None,
                             workspace: Optional[torch.Tensor] = None, uniform: bool = False):
    """Per-row paged attention over a one-byte KV pool (fmt "bf16": a bf16 pool, no scales).
    q [rows, hq, d] bf16.  With max_kv_len, o and workspace given the call neither synchronises
    nor allocates (graph capture); the extents are then the caller's responsibility.  uniform:
    the rows are known to be about equally long (pie_hip_attn_rows_paged_kvq_uniform)."""
    _dev(q, torch.bfloat16, "q")
    rows, hq, d = q.shape
    ps, hk = k_pages.shape[1], k_pages.shape[2]
    if fmt != "bf16" and (k_pages.element_size() != 1 or v_pages.element_size() != 1):
        raise KernelError("one-byte pools expected")
    _dev(kv_page_indices, torch.int32, "kv_page_indices")
    _dev(row_page_begin, torch.int32, "row_page_begin")
    _dev(row_kv_len, torch.int32, "row_kv_len")
    if rows == 0:
        return torch.empty_like(q), None
    if max_kv_len is None:
        max_kv = int(row_kv_len.max())
        npages = (row_kv_len.to(torch.int64) + ps - 1) // ps
        if int((row_page_begin.to(torch.int64) + npages).max()) > kv_page_indices.numel():
            raise KernelError("row extent runs past the page list")
        if kv_page_indices.numel() and int(kv_page_indices.max()) >= k_pages.shape[0]:
            raise KernelError("page id out of range")
    else:
        max_kv = int(max_kv_len)
    if o is None:
        o = torch.empty_like(q)
    lse_t = torch.empty((rows, hq), dtype=torch.float32, device=q.device) if lse else None
    lib = kernels()
    lib.pie_hip_attn_decode_workspace_bytes.restype = C.c_size_t
    need = int(lib.pie_hip_attn_decode_workspace_bytes(rows, hq, hk, d, max_kv))
    ws = workspace if workspace is not None else torch.empty(max(need, 1), dtype=torch.uint8, device=q.device)
    if ws.numel() < need:
        raise KernelError("workspace too small")
    fn = lib.pie_hip_attn_rows_paged_kvq_uniform if uniform else lib.pie_hip_attn_rows_paged_kvq
    _check(fn(KV_FORMATS[fmt], _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(k_scales), _ptr(v_scales), _ptr(o),
              _ptr(lse_t), _ptr(kv_page_indices), _ptr(row_page_begin), _ptr(row_kv_len), rows, hq, hk, d, ps,
              C.c_float(-1.0), max_kv, _ptr(ws), C.c_size_t(need), _stream()), "pie_hip_attn_rows_paged_kvq")
    return o, lse_t
