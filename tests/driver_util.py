"""Helpers for driver-level tests: TOML configs for tiny models, and an oracle model built
from the tensors the driver exports (so both sides hold bit-identical weights)."""
import numpy as np


def toml_config(arch="llama3", hidden=512, layers=2, q_heads=8, kv_heads=2, head_dim=64,
                intermediate=1024, vocab=2048, quant="int4b8", group_size=128, scale_dtype="bf16",
                page_size=16, total_pages=64, max_forward_tokens=256, max_forward_requests=16,
                rope_theta=500000.0, rope_factor=0.0, tie=False, seed=1234, use_graphs=True,
                rms_eps=1e-5, num_experts=0, top_k=0, expert_intermediate=0, router_std=0.0,
                cpu_pages=0, kv_cache_dtype="auto", warmup=True, rope_interleaved=None, sliding_window=0, model_extra="",
                tune_linears=True, attn_merge_proj=True):
    moe = "" if not num_experts else (f"num_experts = {num_experts}\ntop_k = {top_k}\n"
                                      f"expert_intermediate = {expert_intermediate}\n"
                                      f"router_std = {router_std}\n")
    if rope_interleaved is not None:   # default: half-split pairs, as checkpoints use
        moe += f"rope_interleaved = {'true' if rope_interleaved else 'false'}\n"
    if sliding_window:
        moe += f"sliding_window = {sliding_window}\n"
    moe += model_extra   # further [model] lines, verbatim
    return f"""
[model]
arch = "{arch}"
hidden = {hidden}
layers = {layers}
q_heads = {q_heads}
kv_heads = {kv_heads}
head_dim = {head_dim}
intermediate = {intermediate}
vocab = {vocab}
quant = "{quant}"
group_size = {group_size}
scale_dtype = "{scale_dtype}"
rope_theta = {rope_theta}
rope_factor = {rope_factor}
rms_eps = {rms_eps}
tie_embeddings = {"true" if tie else "false"}
seed = {seed}
{moe}
[batching]
kv_page_size = {page_size}
total_pages = {total_pages}
max_forward_tokens = {max_forward_tokens}
max_forward_requests = {max_forward_requests}
cpu_pages = {cpu_pages}
kv_cache_dtype = "{kv_cache_dtype}"

[runtime]
use_graphs = {"true" if use_graphs else "false"}
warmup = {"true" if warmup else "false"}
tune_linears = {"true" if tune_linears else "false"}
attn_merge_proj = {"true" if attn_merge_proj else "false"}
verbose = true
"""


def oracle_model_from_driver(drv, cfg: dict):
    """cfg: the keyword arguments given to toml_config (defaults filled in)."""
    from oracle.model import model_from_driver

    return model_from_driver(drv, cfg)


def full_cfg(**kw):
    import inspect

    sig = inspect.signature(toml_config)
    cfg = {k: v.default for k, v in sig.parameters.items()}
    cfg.update(kw)
    return cfg


def cosine(a, b):
    a = a.astype(np.float64)
    b = b.astype(np.float64)
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b) + 1e-30))
