"""Pin for the oracle's model forward (CPU only): an independent numpy fp64 llama-like
transformer with a dense (unpaged) KV cache, on a tiny random model.  The oracle rounds every
inter-op activation to bf16; agreement is therefore toleranced: logits cosine >= 0.9999 (the
reference's own parity bar, driver/cuda/tests/parity_qwen3.py:160-181) and the same greedy
tokens wherever the fp64 top-2 gap is not a near-tie."""
import numpy as np
import pytest


def make_tensors(oracle, rng, cfg):
    H, d, hq, hk, I, V, L = (cfg[k] for k in ("hidden", "head_dim", "q_heads", "kv_heads",
                                              "intermediate", "vocab", "layers"))
    bf = lambda x: oracle.f32_to_bf16(np.asarray(x, np.float32))
    t = {"embed": bf(rng.standard_normal((V, H)) * 0.5), "lm_head": bf(rng.standard_normal((V, H)) * 0.05),
         "final_norm": bf(rng.uniform(0.8, 1.2, H)),
         "inv_freq": oracle.rope_inv_freq(d, 10000.0)}
    for l in range(L):
        p = f"layers.{l}."
        t[p + "attn_norm"] = bf(rng.uniform(0.8, 1.2, H))
        t[p + "ffn_norm"] = bf(rng.uniform(0.8, 1.2, H))
        if cfg["qk_norm"]:
            t[p + "q_norm"] = bf(rng.uniform(0.8, 1.2, d))
            t[p + "k_norm"] = bf(rng.uniform(0.8, 1.2, d))
        E, Ie = cfg.get("num_experts", 0), cfg.get("expert_intermediate", 0)
        shapes = dict(wqkv=((hq + 2 * hk) * d, H), wo=(H, hq * d), wgu=(2 * I, H), wdown=(H, I))
        if E:
            # experts stacked along the rows: per expert gate rows then up rows / down rows
            t[p + "router"] = bf(rng.standard_normal((E, H)) * (4.0 / np.sqrt(H)))
            shapes.update(wgu=(E * 2 * Ie, H), wdown=(E * H, Ie))
        for name, (n, k) in shapes.items():
            w = bf(rng.standard_normal((n, k)) * (0.7 / np.sqrt(k)))
            if cfg["quant"] == "bf16":
                t[p + name + ".data"] = w
            elif cfg["quant"] == "int8":
                q, s = oracle.quant_int8_per_channel(w)
                t[p + name + ".data"], t[p + name + ".scale"] = q, s
            elif cfg["quant"] == "int4b8":
                G = cfg["group_size"]
                wf = oracle.bf16_to_f32(w).reshape(n, k // G, G)
                s = oracle.f32_to_bf16(np.abs(wf).max(axis=2) / 7.0)
                q = np.clip(np.rint(wf / oracle.bf16_to_f32(s)[:, :, None]), -8, 7).astype(np.int8)
                t[p + name + ".data"] = oracle.pack_w4(q.reshape(n, k))
                t[p + name + ".scale"] = s
    return t


def dequant(oracle, cfg, t, prefix, n, k):
    data = t[prefix + ".data"]
    if cfg["quant"] == "bf16":
        return oracle.bf16_to_f32(data).astype(np.float64)
    if cfg["quant"] == "int8":
        return data.astype(np.float64) * t[prefix + ".scale"].astype(np.float64)[:, None]
    q = oracle.unpack_w4(data, n, k).astype(np.float64)
    s = np.repeat(oracle.bf16_to_f32(t[prefix + ".scale"]).astype(np.float64), cfg["group_size"], axis=1)
    return q * s


class DenseRef:
    """fp64 llama-like decoder with a plain list KV cache (no pages, no rounding)."""

    def __init__(self, oracle, cfg, t):
        self.o, self.cfg, self.t = oracle, cfg, t
        self.f = lambda name: oracle.bf16_to_f32(t[name]).astype(np.float64)
        self.k = [[] for _ in range(cfg["layers"])]
        self.v = [[] for _ in range(cfg["layers"])]

    def norm(self, x, w):
        return x / np.sqrt((x ** 2).mean() + self.cfg["rms_eps"]) * w

    def rope(self, x, pos):
        d = self.cfg["head_dim"]
        ang = pos * self.t["inv_freq"].astype(np.float64)
        c, s = np.cos(ang), np.sin(ang)
        if self.cfg["rope_interleaved"]:
            a, b = x[0::2], x[1::2]
            out = np.empty(d)
            out[0::2], out[1::2] = a * c - b * s, b * c + a * s
            return out
        a, b = x[:d // 2], x[d // 2:]
        return np.concatenate([a * c - b * s, b * c + a * s])

    def step(self, tok, pos):
        cfg = self.cfg
        H, d, hq, hk, I = (cfg[k] for k in ("hidden", "head_dim", "q_heads", "kv_heads", "intermediate"))
        x = self.f("embed")[tok]
        for l in range(cfg["layers"]):
            p = f"layers.{l}."
            xn = self.norm(x, self.f(p + "attn_norm"))
            qkv = dequant(self.o, cfg, self.t, p + "wqkv", (hq + 2 * hk) * d, H) @ xn
            q = qkv[:hq * d].reshape(hq, d)
            k = qkv[hq * d:(hq + hk) * d].reshape(hk, d)
            v = qkv[(hq + hk) * d:].reshape(hk, d)
            if cfg["qk_norm"]:
                q = np.stack([self.norm(h, self.f(p + "q_norm")) for h in q])
                k = np.stack([self.norm(h, self.f(p + "k_norm")) for h in k])
            q = np.stack([self.rope(h, pos) for h in q])
            k = np.stack([self.rope(h, pos) for h in k])
            self.k[l].append(k)
            self.v[l].append(v)
            K, V = np.stack(self.k[l]), np.stack(self.v[l])  # [T, hk, d]
            out = np.zeros((hq, d))
            for h in range(hq):
                kv = h // (hq // hk)
                s = K[:, kv] @ q[h] / np.sqrt(d)
                w = np.exp(s - s.max())
                out[h] = (w / w.sum()) @ V[:, kv]
            x = x + dequant(self.o, cfg, self.t, p + "wo", H, hq * d) @ out.reshape(-1)
            xn = self.norm(x, self.f(p + "ffn_norm"))
            E = cfg.get("num_experts", 0)
            if E:
                x = x + self.moe(p, xn)
                continue
            gu = dequant(self.o, cfg, self.t, p + "wgu", 2 * I, H) @ xn
            g, u = gu[:I], gu[I:]
            x = x + dequant(self.o, cfg, self.t, p + "wdown", H, I) @ (g / (1 + np.exp(-g)) * u)
        return self.f("lm_head") @ self.norm(x, self.f("final_norm"))

    def moe(self, p, xn):
        """softmax router -> top-k (ties to the lowest index) -> renormalise -> weighted sum of
        the selected experts' SwiGLU FFNs (driver/portable/src/graph_common.cpp:237-345)."""
        cfg = self.cfg
        H, E, K, Ie = cfg["hidden"], cfg["num_experts"], cfg["top_k"], cfg["expert_intermediate"]
        logits = self.f(p + "router") @ xn
        pr = np.exp(logits - logits.max())
        pr /= pr.sum()
        sel = np.argsort(-pr, kind="stable")[:K]
        self.min_gap = min(getattr(self, "min_gap", 1.0), float(pr[sel[-1]] - np.sort(pr)[-K - 1]))
        w = pr[sel] / pr[sel].sum()
        wgu = dequant(self.o, cfg, self.t, p + "wgu", E * 2 * Ie, H).reshape(E, 2 * Ie, H)
        wdn = dequant(self.o, cfg, self.t, p + "wdown", E * H, Ie).reshape(E, H, Ie)
        out = np.zeros(H)
        for e, we in zip(sel, w):
            gu = wgu[e] @ xn
            g, u = gu[:Ie], gu[Ie:]
            out += we * (wdn[e] @ (g / (1 + np.exp(-g)) * u))
        return out


@pytest.mark.parametrize("quant,qk_norm,interleaved", [("bf16", False, 1), ("int8", False, 1),
                                                       ("int4b8", True, 0)])
def test_oracle_forward_matches_dense_fp64(oracle, quant, qk_norm, interleaved):
    from oracle.model import OracleModel

    cfg = dict(hidden=128, layers=2, q_heads=4, kv_heads=2, head_dim=32, intermediate=256, vocab=300,
               rms_eps=1e-5, rope_interleaved=interleaved, qk_norm=qk_norm, quant=quant,
               group_size=64, page_size=4, total_pages=16)
    rng = np.random.default_rng(100)
    t = make_tensors(oracle, rng, cfg)
    om = OracleModel(cfg, t)
    ref = DenseRef(oracle, cfg, t)
    prompt = rng.integers(0, cfg["vocab"], 7)
    # prefill through scattered pages, sampling every prompt row
    pages = [9, 2, 5, 11]
    toks, logits, plan = om.forward(prompt, np.arange(7), pages[:2], [0, 2], [3], [0, 7],
                                    sampling_indices=np.arange(7), sampling_indptr=[0, 7],
                                    want_logits=True)
    ref_logits = [ref.step(int(tk), i) for i, tk in enumerate(prompt)]
    checked = 0
    for i in range(7):
        lo = oracle.bf16_to_f32(logits[i]).astype(np.float64)
        cos = lo @ ref_logits[i] / (np.linalg.norm(lo) * np.linalg.norm(ref_logits[i]))
        assert cos >= 0.9999, (i, cos)
        top2 = np.sort(ref_logits[i])[-2:]
        if top2[1] - top2[0] > 0.02 * abs(top2[1]):
            assert int(toks[i]) == int(np.argmax(ref_logits[i]))
            checked += 1
    # decode steps continue on the same pages (grows into page index 2 and 3)
    tok = int(toks[-1])
    for s in range(7, 14):
        npg = s // 4 + 1
        t1, lg, _ = om.forward([tok], [s], pages[:npg], [0, npg], [s + 1 - (npg - 1) * 4], [0, 1],
                               want_logits=True)
        rl = ref.step(tok, s)
        lo = oracle.bf16_to_f32(lg[0]).astype(np.float64)
        assert lo @ rl / (np.linalg.norm(lo) * np.linalg.norm(rl)) >= 0.9999
        top2 = np.sort(rl)[-2:]
        if top2[1] - top2[0] > 0.02 * abs(top2[1]):
            assert int(t1[0]) == int(np.argmax(rl))
            checked += 1
        tok = int(t1[0])
    assert checked >= 8


def test_oracle_generate_equals_stepwise_forward(oracle):
    from oracle.model import OracleModel

    cfg = dict(hidden=64, layers=1, q_heads=2, kv_heads=1, head_dim=32, intermediate=64, vocab=50,
               rms_eps=1e-5, rope_interleaved=1, qk_norm=False, quant="bf16", group_size=32,
               page_size=4, total_pages=16)
    rng = np.random.default_rng(101)
    t = make_tensors(oracle, rng, cfg)
    a = OracleModel(cfg, t).generate(rng.integers(0, 50, 5).tolist() + [], 6, replicate=2)
    assert a.shape == (2, 6) and np.array_equal(a[0], a[1])
