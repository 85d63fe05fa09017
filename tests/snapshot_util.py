"""Writes tiny Hugging Face style snapshots (config.json + safetensors) for the loader tests and
returns the tensors the driver should end up holding, computed independently with the oracle's
quantisers."""
import json
import os

import numpy as np


def hf_config(arch, hidden, layers, q_heads, kv_heads, head_dim, intermediate, vocab, rms_eps=1e-6,
              rope_theta=10000.0, tie=False, num_experts=0, top_k=0, expert_intermediate=0,
              rope_scaling=None):
    c = dict(model_type={"llama3": "llama", "qwen3": "qwen3", "qwen3_moe": "qwen3_moe"}[arch],
             architectures=["X"], hidden_size=hidden, num_hidden_layers=layers,
             num_attention_heads=q_heads, num_key_value_heads=kv_heads, head_dim=head_dim,
             intermediate_size=intermediate, vocab_size=vocab, rms_norm_eps=rms_eps,
             rope_theta=rope_theta, tie_word_embeddings=tie, torch_dtype="bfloat16")
    if num_experts:
        c.update(num_experts=num_experts, num_experts_per_tok=top_k,
                 moe_intermediate_size=expert_intermediate, norm_topk_prob=True)
    if rope_scaling:
        c["rope_scaling"] = rope_scaling
    return c


def write_snapshot(directory, oracle, rng, cfg: dict, dtype="bf16", packed_int4_group=0, files=2):
    """cfg: arch, hidden, layers, q_heads, kv_heads, head_dim, intermediate, vocab (+ MoE keys).
    Returns {hf_name: float32 array of the values as stored (after the dtype's rounding)}."""
    import torch
    from safetensors.torch import save_file

    os.makedirs(directory, exist_ok=True)
    H, L, hq, hk, d, I, V = (cfg[k] for k in ("hidden", "layers", "q_heads", "kv_heads", "head_dim",
                                              "intermediate", "vocab"))
    E, Ie = cfg.get("num_experts", 0), cfg.get("expert_intermediate", 0)
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype]
    t = {}

    def add(name, shape, std=None, lo=None):
        a = rng.uniform(0.8, 1.2, shape) if lo is not None else rng.standard_normal(shape) * std
        t[name] = torch.from_numpy(np.asarray(a, np.float32)).to(tdt)

    add("model.embed_tokens.weight", (V, H), std=0.5)
    if not cfg.get("tie", False):
        add("lm_head.weight", (V, H), std=0.05)
    add("model.norm.weight", (H,), lo=True)
    for l in range(L):
        p = f"model.layers.{l}."
        add(p + "input_layernorm.weight", (H,), lo=True)
        add(p + "post_attention_layernorm.weight", (H,), lo=True)
        if cfg["arch"] != "llama3":
            add(p + "self_attn.q_norm.weight", (d,), lo=True)
            add(p + "self_attn.k_norm.weight", (d,), lo=True)
        add(p + "self_attn.q_proj.weight", (hq * d, H), std=0.7 / np.sqrt(H))
        add(p + "self_attn.k_proj.weight", (hk * d, H), std=0.7 / np.sqrt(H))
        add(p + "self_attn.v_proj.weight", (hk * d, H), std=0.7 / np.sqrt(H))
        add(p + "self_attn.o_proj.weight", (H, hq * d), std=0.7 / np.sqrt(hq * d))
        if E:
            add(p + "mlp.gate.weight", (E, H), std=4.0 / np.sqrt(H))
            for e in range(E):
                add(p + f"mlp.experts.{e}.gate_proj.weight", (Ie, H), std=0.7 / np.sqrt(H))
                add(p + f"mlp.experts.{e}.up_proj.weight", (Ie, H), std=0.7 / np.sqrt(H))
                add(p + f"mlp.experts.{e}.down_proj.weight", (H, Ie), std=0.7 / np.sqrt(Ie))
        else:
            add(p + "mlp.gate_proj.weight", (I, H), std=0.7 / np.sqrt(H))
            add(p + "mlp.up_proj.weight", (I, H), std=0.7 / np.sqrt(H))
            add(p + "mlp.down_proj.weight", (H, I), std=0.7 / np.sqrt(I))
    stored = {k: v.to(torch.float32).numpy().copy() for k, v in t.items()}
    if packed_int4_group:
        # compressed-tensors pack-quantized layout: weight_packed int32 [N, K/8] (nibble j of a
        # word = element 8w+j, value+8), weight_scale [N, K/G]
        G = packed_int4_group
        for name in [n for n in t if n.endswith("_proj.weight")]:
            w = oracle.f32_to_bf16(stored[name])
            n, k = w.shape
            wf = oracle.bf16_to_f32(w).reshape(n, k // G, G)
            s = oracle.f32_to_bf16(np.abs(wf).max(axis=2) / 7.0)
            q = np.clip(np.rint(wf / oracle.bf16_to_f32(s)[:, :, None]), -8, 7).astype(np.int8)
            packed = oracle.pack_w4(q.reshape(n, k)).view(np.int32)
            del t[name]
            base = name[:-len(".weight")]
            t[base + ".weight_packed"] = torch.from_numpy(packed.copy())
            t[base + ".weight_scale"] = torch.from_numpy(s.view(np.int16).copy()).view(torch.bfloat16)
    names = sorted(t)
    per = (len(names) + files - 1) // files
    for i in range(files):
        part = {n: t[n].contiguous() for n in names[i * per:(i + 1) * per]}
        if part:
            save_file(part, os.path.join(directory, f"model-{i + 1:05d}-of-{files:05d}.safetensors"))
    hc = hf_config(cfg["arch"], H, L, hq, hk, d, I, V, tie=cfg.get("tie", False), num_experts=E,
                   top_k=cfg.get("top_k", 0), expert_intermediate=Ie,
                   rms_eps=cfg.get("rms_eps", 1e-6), rope_theta=cfg.get("rope_theta", 10000.0),
                   rope_scaling=cfg.get("rope_scaling"))
    with open(os.path.join(directory, "config.json"), "w") as f:
        json.dump(hc, f)
    return stored


def expected_tensors(oracle, stored: dict, cfg: dict, quant: str, group: int, scale_dtype="bf16"):
    """The canonical tensor dict (oracle naming: q|k|v rows fused, gate rows then up rows,
    experts stacked) the driver should hold after loading `stored` with `quant`."""
    L = cfg["layers"]
    E = cfg.get("num_experts", 0)
    bf = lambda a: oracle.f32_to_bf16(np.asarray(a, np.float32))
    t = {"embed": bf(stored["model.embed_tokens.weight"]), "final_norm": bf(stored["model.norm.weight"])}
    t["lm_head"] = t["embed"] if "lm_head.weight" not in stored else bf(stored["lm_head.weight"])

    def lin(prefix, w_bf16):
        n, k = w_bf16.shape
        if quant == "bf16":
            t[prefix + ".data"] = w_bf16
        elif quant == "int8":
            q, s = oracle.quant_int8_per_channel(w_bf16)
            t[prefix + ".data"] = q
            t[prefix + ".scale"] = oracle.f32_to_bf16(s) if scale_dtype == "bf16" else s
        elif quant == "fp8":
            q, s = oracle.quant_fp8_per_channel(w_bf16)
            t[prefix + ".data"] = q
            t[prefix + ".scale"] = oracle.f32_to_bf16(s) if scale_dtype == "bf16" else s
        else:
            wf = oracle.bf16_to_f32(w_bf16).reshape(n, k // group, group)
            s = oracle.f32_to_bf16(np.abs(wf).max(axis=2) / 7.0)
            q = np.clip(np.rint(wf / oracle.bf16_to_f32(s)[:, :, None]), -8, 7).astype(np.int8)
            t[prefix + ".data"] = oracle.pack_w4(q.reshape(n, k))
            t[prefix + ".scale"] = s

    for l in range(L):
        p, hf = f"layers.{l}.", f"model.layers.{l}."
        t[p + "attn_norm"] = bf(stored[hf + "input_layernorm.weight"])
        t[p + "ffn_norm"] = bf(stored[hf + "post_attention_layernorm.weight"])
        if cfg["arch"] != "llama3":
            t[p + "q_norm"] = bf(stored[hf + "self_attn.q_norm.weight"])
            t[p + "k_norm"] = bf(stored[hf + "self_attn.k_norm.weight"])
        a = hf + "self_attn."
        lin(p + "wqkv", bf(np.concatenate([stored[a + "q_proj.weight"], stored[a + "k_proj.weight"],
                                           stored[a + "v_proj.weight"]])))
        lin(p + "wo", bf(stored[a + "o_proj.weight"]))
        if E:
            t[p + "router"] = bf(stored[hf + "mlp.gate.weight"])
            ex = [hf + f"mlp.experts.{e}." for e in range(E)]
            lin(p + "wgu", bf(np.concatenate([np.concatenate([stored[x + "gate_proj.weight"],
                                                              stored[x + "up_proj.weight"]]) for x in ex])))
            lin(p + "wdown", bf(np.concatenate([stored[x + "down_proj.weight"] for x in ex])))
        else:
            m = hf + "mlp."
            lin(p + "wgu", bf(np.concatenate([stored[m + "gate_proj.weight"], stored[m + "up_proj.weight"]])))
            lin(p + "wdown", bf(stored[m + "down_proj.weight"]))
    return t
