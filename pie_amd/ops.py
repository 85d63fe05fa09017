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
