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
            elif cfg["quant"] == "fp8":
                q, s = oracle.quant_fp8_per_channel(w)
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
    if cfg["quant"] == "fp8":
        import torch
        vals = torch.from_numpy(np.ascontiguousarray(data)).view(torch.float8_e4m3fn).to(torch.float64).numpy()
        return vals * t[prefix + ".scale"].astype(np.float64)[:, None]
    q = oracle.unpack_w4(data, n, k).astype(np.float64)
    s = np.repeat(oracle.bf16_to_f32(t[prefix + ".scale"]).astype(np.float64), cfg["group_size"], axis=1)
    return q * s


class DenseRef:
    """fp64 llama-like decoder with a plain list KV cache (no pages, no rounding)."""

    def __init__(self, oracle, cfg, t, kv_format=None):
        self.o, self.cfg, self.t = oracle, cfg, t
        self.kv_format = kv_format   # None, "fp8_e4m3", "int8_per_token_head", "fp8_per_token_head"
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

    def kv_qdq(self, x):
        """What a one-byte pool gives back for a [heads, d] block: per (token, head)
        scale = absmax / qmax, code = round(x / scale), value = code * scale
        (driver/cuda/src/kernels/kv_paged.cu:155-297) — an independent numpy / torch evaluation."""
        import torch

        if self.kv_format is None:
            return x
        x = x.astype(np.float32)
        e4m3 = lambda a: torch.from_numpy(np.clip(a, -448.0, 448.0).astype(np.float32)).to(
            torch.float8_e4m3fn).to(torch.float32).numpy()
        if self.kv_format == "fp8_e4m3":
            return e4m3(x).astype(np.float64)
        qmax = np.float32(127.0 if self.kv_format == "int8_per_token_head" else 448.0)
        amax = np.abs(x).max(axis=-1, keepdims=True)
        scale = np.where(amax > 0, amax / qmax, np.float32(1.0)).astype(np.float32)
        y = x * (np.float32(1.0) / scale)
        code = np.clip(np.rint(y), -128, 127) if self.kv_format == "int8_per_token_head" else e4m3(y)
        return (code.astype(np.float32) * scale).astype(np.float64)

    def step(self, tok, pos, allow=None):
        """allow: optional boolean array over the keys 0..pos (custom attention mask)."""
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
            self.k[l].append(self.kv_qdq(k))
            self.v[l].append(self.kv_qdq(v))
            K, V = np.stack(self.k[l]), np.stack(self.v[l])  # [T, hk, d]
            out = np.zeros((hq, d))
            vis = np.ones(len(K), bool) if allow is None else np.asarray(allow, bool)
            for h in range(hq):
                if not vis.any():
                    break
                kv = h // (hq // hk)
                s = K[vis, kv] @ q[h] / np.sqrt(d)
                w = np.exp(s - s.max())
                out[h] = (w / w.sum()) @ V[vis, kv]
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


def test_f16_rounding_matches_numpy(oracle):
    """The F16 rounding the portable-faithful mode applies at the KV write, against numpy's
    float16: random values over the whole range, subnormals, ties and the overflow edge."""
    import ctypes as C

    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(4000) * 10.0 ** rng.integers(-9, 5, 4000),
                        [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25,
                         2.0 ** -14, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 5.96e-8, 6.1e-5]]).astype(np.float32)
    out = np.empty_like(x)
    oracle.lib().orc_round_f16_array(C.c_void_p(x.ctypes.data), C.c_void_p(out.ctypes.data), C.c_size_t(x.size))
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def _run_both(oracle, om, ref, prompt, pages, ps, steps, forward, masks=None):
    """Prefill `prompt` through scattered pages (every row sampled), then `steps` decode steps;
    `forward(args, masks)` -> logits [rows, V] as float64.  Yields (logits, reference logits)."""
    n = len(prompt)
    npg = (n + ps - 1) // ps
    args = dict(token_ids=prompt, position_ids=np.arange(n), kv_page_indices=pages[:npg], kv_page_indptr=[0, npg],
                kv_last_page_lens=[n - (npg - 1) * ps], qo_indptr=[0, n], sampling_indices=np.arange(n),
                sampling_indptr=[0, n])
    m = None if masks is None else [masks(i) for i in range(n)]
    lg = forward(args, m)
    for i, tk in enumerate(prompt):
        allow = None if masks is None else oracle.brle_allow(masks(i), i, i + 1, 0).astype(bool)
        yield lg[i], ref.step(int(tk), i, allow)
    tok = int(np.argmax(lg[-1]))
    for s in range(n, n + steps):
        npg = s // ps + 1
        args = dict(token_ids=[tok], position_ids=[s], kv_page_indices=pages[:npg], kv_page_indptr=[0, npg],
                    kv_last_page_lens=[s + 1 - (npg - 1) * ps], qo_indptr=[0, 1])
        lg = forward(args, None if masks is None else [masks(s)])
        allow = None if masks is None else oracle.brle_allow(masks(s), s, s + 1, 0).astype(bool)
        rl = ref.step(tok, s, allow)
        yield lg[0], rl
        tok = int(np.argmax(rl))


CFG_HP = dict(hidden=128, layers=3, q_heads=4, kv_heads=2, head_dim=32, intermediate=256, vocab=300,
              rms_eps=1e-5, group_size=64, page_size=4, total_pages=16)


@pytest.mark.parametrize("quant,qk_norm,interleaved", [("bf16", False, 0), ("int8", False, 1), ("int4b8", True, 0),
                                                       ("fp8", True, 1)])
def test_truth_mode_equals_dense_fp64(oracle, quant, qk_norm, interleaved):
    """Mode "f64" (double throughout) is the independent numpy transformer to summation-order
    accuracy: 1e-9 of the largest logit, on prefill rows and decode steps over scattered pages."""
    from oracle.model import OracleModel

    cfg = dict(CFG_HP, rope_interleaved=interleaved, qk_norm=qk_norm, quant=quant)
    rng = np.random.default_rng(200)
    t = make_tensors(oracle, rng, cfg)
    om, ref = OracleModel(cfg, t), DenseRef(oracle, cfg, t)
    fwd = lambda args, m: om.forward_hp("f64", **args, masks=m)[1]
    n = 0
    for lg, rl in _run_both(oracle, om, ref, rng.integers(0, cfg["vocab"], 9), [9, 2, 5, 11, 7], 4, 6, fwd):
        assert np.max(np.abs(lg - rl)) <= 1e-9 * np.max(np.abs(rl))
        n += 1
    assert n == 15


@pytest.mark.parametrize("quant,qk_norm", [("bf16", False), ("int4b8", True)])
def test_portable_mode_is_f32_with_an_f16_pool(oracle, quant, qk_norm):
    """Mode "P": F32 activations and F16 K/V.  Against the fp64 transformer its logits differ by
    the F16 rounding of the pool (2^-11 per element) and, for bf16 weights, the bf16 rounding of
    the activations that meet them: relative error <= 1 %, far inside the mode-C error, and not
    bit-equal to the truth (the roundings are really applied)."""
    from oracle.model import OracleModel

    cfg = dict(CFG_HP, rope_interleaved=0, qk_norm=qk_norm, quant=quant)
    rng = np.random.default_rng(201)
    t = make_tensors(oracle, rng, cfg)
    om, ref = OracleModel(cfg, t), DenseRef(oracle, cfg, t)
    fwd = lambda args, m: om.forward_hp("P", **args, masks=m)[1]
    worst = 0.0
    for lg, rl in _run_both(oracle, om, ref, rng.integers(0, cfg["vocab"], 9), [9, 2, 5, 11, 7], 4, 6, fwd):
        cos = lg @ rl / (np.linalg.norm(lg) * np.linalg.norm(rl))
        assert cos >= 0.99999
        worst = max(worst, np.max(np.abs(lg - rl)) / np.max(np.abs(rl)))
    assert 1e-7 < worst <= 1e-2
    # the pool holds F16 values
    k, _ = om.hp_pools("P")
    used = k[0][9]
    assert np.array_equal(used.astype(np.float16).astype(np.float64), used) and np.any(used != 0)


def test_mode_c_error_is_bf16_sized_against_truth(oracle):
    """Mode C (bf16 between ops) against mode "f64" on the same weights: the deviation has the
    size of bf16 rounding noise (1 - cosine about 1e-5 at three layers), mode P's is an order
    smaller — the three modes order as they should."""
    from oracle.model import OracleModel

    cfg = dict(CFG_HP, rope_interleaved=0, qk_norm=False, quant="int4b8")
    rng = np.random.default_rng(202)
    t = make_tensors(oracle, rng, cfg)
    om = OracleModel(cfg, t)
    prompt = rng.integers(0, cfg["vocab"], 11)
    args = dict(token_ids=prompt, position_ids=np.arange(11), kv_page_indices=[3, 8, 1], kv_page_indptr=[0, 3],
                kv_last_page_lens=[3], qo_indptr=[0, 11], sampling_indices=np.arange(11), sampling_indptr=[0, 11])
    _, lc, _ = om.forward(**args, want_logits=True)
    lc = oracle.bf16_to_f32(lc).astype(np.float64)
    lp, lt = om.forward_hp("P", **args)[1], om.forward_hp("f64", **args)[1]
    dev = lambda a: 1.0 - np.sum(a * lt, axis=1) / (np.linalg.norm(a, axis=1) * np.linalg.norm(lt, axis=1))
    # (mode P's share is the bf16 rounding of the activations that meet the bf16 lm_head)
    assert np.all(dev(lc) < 1e-4) and np.all(dev(lp) < 5e-6) and dev(lc).mean() > 5 * dev(lp).mean()


@pytest.mark.parametrize("kv_format", ["fp8_e4m3", "int8_per_token_head", "fp8_per_token_head"])
def test_oracle_forward_over_one_byte_pools_matches_dense_fp64(oracle, kv_format):
    """orc_llama_forward_kvq (K / V quantised per (token, head) at the write, read back as
    code * scale) against the fp64 transformer doing the same with an independent numpy / torch
    quantiser.  The oracle quantises bf16-rounded rows, the reference unrounded ones, so a value
    at a rounding boundary may land one code apart: cosine >= 0.999, and clearly apart from the
    unquantised model (the quantisation really happens)."""
    from oracle.model import OracleModel

    cfg = dict(CFG_HP, rope_interleaved=0, qk_norm=False, quant="int8", kv_cache_dtype=kv_format)
    rng = np.random.default_rng(203)
    t = make_tensors(oracle, rng, cfg)
    om = OracleModel(cfg, t)
    ref, plain = DenseRef(oracle, cfg, t, kv_format=kv_format), DenseRef(oracle, cfg, t)
    fwd = lambda args, m: oracle.bf16_to_f32(om.forward(**args, want_logits=True, masks=m)[1]).astype(np.float64)
    prompt = rng.integers(0, cfg["vocab"], 9)
    cos = lambda a, b: a @ b / (np.linalg.norm(a) * np.linalg.norm(b))
    pages = [9, 2, 5, 11, 7]
    for i, (lg, rl) in enumerate(_run_both(oracle, om, ref, prompt, pages, 4, 6, fwd)):
        assert cos(lg, rl) >= 0.999, (i, cos(lg, rl))
        if i < 9:
            plain.step(int(prompt[i]), i)
    # Layer 0's pool (same inputs on both sides up to the bf16 rounding of the rotated rows): the
    # oracle's slots hold the independent quantiser's values to within one code step, at the
    # tokens' own slots, and differ from the unquantised rows by quantisation noise of that size.
    T = 9
    got_k = np.stack([om.k_f32[0][pages[t // 4], t % 4] for t in range(T)]).astype(np.float64)
    got_v = np.stack([om.v_f32[0][pages[t // 4], t % 4] for t in range(T)]).astype(np.float64)
    for got, want, raw in ((got_k, np.stack(ref.k[0][:T]), np.stack(plain.k[0])),
                           (got_v, np.stack(ref.v[0][:T]), np.stack(plain.v[0]))):
        amax = np.abs(raw).max(axis=-1, keepdims=True)
        if kv_format == "int8_per_token_head":
            step = np.broadcast_to(amax / 127.0, raw.shape)
        else:   # e4m3: three mantissa bits -> one step is 2^-3 of the value's binade
            ref_mag = np.abs(raw) if kv_format == "fp8_e4m3" else np.abs(raw) / amax * 448.0
            unit = amax / 448.0 if kv_format == "fp8_per_token_head" else 1.0
            step = 2.0 ** (np.floor(np.log2(np.maximum(ref_mag, 2.0 ** -6))) - 3) * unit
        # (+ the bf16 noise of the oracle's own rows, which matters for elements near zero)
        assert np.all(np.abs(got - want) <= 1.05 * step + 2.0 ** -7 * amax)
        noise = np.abs(got - raw) / (step + 2.0 ** -7 * amax)
        assert 0.1 < noise.mean() < 0.6 and noise.max() <= 1.6   # (unquantised rows: 0.03 - 0.06)


@pytest.mark.parametrize("mode", ["C", "f64"])
def test_oracle_forward_with_custom_masks_matches_dense_fp64(oracle, mode):
    """The `masks=` path of the forward (BRLE runs -> per-row key visibility -> masked attention)
    against the fp64 transformer attending to the same visible keys, prefill rows and decode."""
    from oracle.model import OracleModel

    cfg = dict(CFG_HP, rope_interleaved=1, qk_norm=True, quant="bf16")
    rng = np.random.default_rng(204)
    t = make_tensors(oracle, rng, cfg)
    om, ref, plain = OracleModel(cfg, t), DenseRef(oracle, cfg, t), DenseRef(oracle, cfg, t)
    # row i: runs alternate hidden / visible from key 0; rows 0 and 5 keep the plain causal mask
    table = {1: [0, 1, 1], 2: [1, 2], 3: [2, 1, 1, 9], 4: [0, 2, 2, 1], 6: [3, 4], 7: [0, 1, 6, 1], 8: [1, 1, 1, 1, 1, 9],
             9: [4, 6], 10: [0, 3, 7, 1], 11: [9, 3]}
    masks = lambda i: table.get(i, [])
    if mode == "C":
        fwd = lambda args, m: oracle.bf16_to_f32(om.forward(**args, want_logits=True, masks=m)[1]).astype(np.float64)
    else:
        fwd = lambda args, m: om.forward_hp("f64", **args, masks=m)[1]
    prompt = rng.integers(0, cfg["vocab"], 9)
    differs = 0
    for i, (lg, rl) in enumerate(_run_both(oracle, om, ref, prompt, [9, 2, 5, 11, 7], 4, 3, fwd, masks=masks)):
        if mode == "C":
            assert lg @ rl / (np.linalg.norm(lg) * np.linalg.norm(rl)) >= 0.9999, i
        else:
            assert np.max(np.abs(lg - rl)) <= 1e-9 * np.max(np.abs(rl)), i
        if i < 9:
            pl = plain.step(int(prompt[i]), i)
            differs += np.max(np.abs(pl - rl)) > 1e-3 * np.max(np.abs(rl))
    assert differs >= 5   # the masks change the result on the masked rows
