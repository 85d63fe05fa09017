"""Helpers shared by the GPU tests: numpy <-> device tensors with bf16 as raw uint16 bits."""
import numpy as np


def dev(arr, device, dtype=None):
    import torch

    a = np.ascontiguousarray(arr)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    t = torch.from_numpy(a).to(device)
    return t.view(dtype) if dtype is not None else t


def bits(t):
    import torch

    if t.dtype == torch.bfloat16:
        return t.view(torch.uint16).cpu().numpy()
    return t.cpu().numpy()


def ulp_diff(a_bits, b_bits):
    """Distance in bf16 representable steps (sign-magnitude aware)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))
