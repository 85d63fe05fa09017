"""Oracle: llama-like decoder forward over a paged KV cache (ctypes front end of
oracle/src/model.c) plus a greedy generation loop shaped like the reference's offline
harness (driver/portable/src/executor/executor.cpp:1439-1597).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import bf16_to_f32, lib
from .planner import plan_forward

QUANT_CODE = {"int4b8": 0, "int8": 1, "fp8": 2, "bf16": 3}


class _Linear(C.Structure):
    _fields_ = [("data", C.c_void_p), ("scale", C.c_void_p)]


class _Model(C.Structure):
    _fields_ = [("hidden", C.c_int), ("layers", C.c_int), ("q_heads", C.c_int),
                ("kv_heads", C.c_int), ("head_dim", C.c_int), ("intermediate", C.c_int),
                ("vocab", C.c_int), ("rms_eps", C.c_float), ("rope_interleaved", C.c_int),
                ("has_qk_norm", C.c_int), ("quant", C.c_int), ("group", C.c_int),
                ("embed", C.c_void_p), ("lm_head", C.c_void_p), ("final_norm", C.c_void_p),
                ("inv_freq", C.c_void_p),
                ("attn_norm", C.POINTER(C.c_void_p)), ("ffn_norm", C.POINTER(C.c_void_p)),
                ("q_norm", C.POINTER(C.c_void_p)), ("k_norm", C.POINTER(C.c_void_p)),
                ("wqkv", C.POINTER(_Linear)), ("wo", C.POINTER(_Linear)),
                ("wgu", C.POINTER(_Linear)), ("wdown", C.POINTER(_Linear)),
                ("num_experts", C.c_int), ("top_k", C.c_int), ("expert_intermediate", C.c_int),
                ("router", C.POINTER(C.c_void_p)), ("rope_mscale", C.c_float), ("raw_topk", C.c_int)]


class OracleModel:
    """`cfg`: dict with hidden, layers, q_heads, kv_heads, head_dim, intermediate, vocab,
    rms_eps, rope_interleaved, qk_norm, quant, group_size, page_size, total_pages; for MoE also
    num_experts, top_k, expert_intermediate (then `layers.l.wgu` / `.wdown` hold the experts
    stacked along the rows, gate rows before up rows inside each expert, and `layers.l.router`
    is bf16 [E, H]).
    `tensors`: name -> numpy array, names as the driver exports them; row scales of int8/fp8
    may be bf16 bits (uint16) and are widened to f32 here."""

    def __init__(self, cfg: dict, tensors: dict):
        self.cfg = dict(cfg)
        L = cfg["layers"]
        self._keep = []

        def ptr(a):
            a = np.ascontiguousarray(a)
            self._keep.append(a)
            return a.ctypes.data

        def lin(prefix):
            data = tensors[prefix + ".data"]
            sc = tensors.get(prefix + ".scale")
            if sc is not None and cfg["quant"] in ("int8", "fp8") and sc.dtype == np.uint16:
                sc = bf16_to_f32(sc)
            return _Linear(ptr(data), ptr(sc) if sc is not None else None)

        m = _Model()
        for k in ("hidden", "layers", "q_heads", "kv_heads", "head_dim", "intermediate", "vocab"):
            setattr(m, k, int(cfg[k]))
        m.rms_eps = float(cfg["rms_eps"])
        m.rope_interleaved = int(cfg["rope_interleaved"])
        m.has_qk_norm = int(bool(cfg.get("qk_norm", False)))
        m.quant = QUANT_CODE[cfg["quant"]]
        m.group = int(cfg.get("group_size", 128))
        m.embed = ptr(tensors["embed"])
        m.lm_head = ptr(tensors["lm_head"])
        m.final_norm = ptr(tensors["final_norm"])
        m.inv_freq = ptr(np.asarray(tensors["inv_freq"], np.float32))

        def parr(names):
            arr = (C.c_void_p * L)(*[ptr(tensors[n]) if n in tensors else None for n in names])
            self._keep.append(arr)
            return C.cast(arr, C.POINTER(C.c_void_p))

        def larr(suffix):
            arr = (_Linear * L)(*[lin(f"layers.{l}.{suffix}") for l in range(L)])
            self._keep.append(arr)
            return C.cast(arr, C.POINTER(_Linear))

        m.attn_norm = parr([f"layers.{l}.attn_norm" for l in range(L)])
        m.ffn_norm = parr([f"layers.{l}.ffn_norm" for l in range(L)])
        m.q_norm = parr([f"layers.{l}.q_norm" for l in range(L)])
        m.k_norm = parr([f"layers.{l}.k_norm" for l in range(L)])
        m.wqkv, m.wo, m.wgu, m.wdown = larr("wqkv"), larr("wo"), larr("wgu"), larr("wdown")
        m.num_experts = int(cfg.get("num_experts", 0))
        m.top_k = int(cfg.get("top_k", 0))
        m.expert_intermediate = int(cfg.get("expert_intermediate", 0))
        if m.num_experts:
            m.router = parr([f"layers.{l}.router" for l in range(L)])
        m.rope_mscale = float(cfg.get("rope_mscale", 1.0))
        m.raw_topk = 0 if cfg.get("norm_topk", True) else 1
        self._m = m
        ps, tp = cfg["page_size"], cfg["total_pages"]
        shape = (tp, ps, cfg["kv_heads"], cfg["head_dim"])
        self.k_pages = [np.zeros(shape, np.uint16) for _ in range(L)]
        self.v_pages = [np.zeros(shape, np.uint16) for _ in range(L)]
        self._kp = (C.c_void_p * L)(*[a.ctypes.data for a in self.k_pages])
        self._vp = (C.c_void_p * L)(*[a.ctypes.data for a in self.v_pages])
        # one-byte KV-cache formats: pools of the dequantised values the attention reads back
        from oracle import KV_FORMATS
        kv_dtype = cfg.get("kv_cache_dtype", "bf16")
        self.kv_format = KV_FORMATS["bf16" if kv_dtype in ("auto", "bfloat16") else kv_dtype]
        if self.kv_format:
            self.k_f32 = [np.zeros(shape, np.float32) for _ in range(L)]
            self.v_f32 = [np.zeros(shape, np.float32) for _ in range(L)]
            self._kf = (C.c_void_p * L)(*[a.ctypes.data for a in self.k_f32])
            self._vf = (C.c_void_p * L)(*[a.ctypes.data for a in self.v_f32])

    def forward(self, token_ids, position_ids, kv_page_indices, kv_page_indptr, kv_last_page_lens,
                qo_indptr, sampling_indices=None, sampling_indptr=None, want_logits=False,
                masks=None, window: int = 0):
        """One forward pass; returns (tokens per sampled row, logits bf16 bits or None, plan).
        masks: optional per-token BRLE run lists (custom attention masks,
        driver/portable/src/plan.cpp:54-94); an empty list = plain causal."""
        R = len(qo_indptr) - 1
        if sampling_indices is None:
            qo = np.asarray(qo_indptr, np.int64)
            sampling_indices = qo[1:] - qo[:-1] - 1
            sampling_indptr = np.arange(R + 1)
        p = plan_forward(token_ids, position_ids, kv_page_indices, kv_page_indptr,
                         kv_last_page_lens, qo_indptr, sampling_indices, sampling_indptr,
                         self.cfg["page_size"], self.cfg["total_pages"])
        N, S = p["N"], len(p["sample_rows"])
        tok = np.ascontiguousarray(np.asarray(token_ids, np.uint32))
        pos = np.ascontiguousarray(np.asarray(p["positions"], np.int32))
        slots = np.ascontiguousarray(np.asarray(p["kv_slots"], np.int64))
        rb = np.ascontiguousarray(np.asarray(p["row_page_begin"], np.uint32))
        rl = np.ascontiguousarray(np.asarray(p["row_kv_len"], np.int32))
        pages = np.ascontiguousarray(np.asarray(kv_page_indices, np.uint32))
        sr = np.ascontiguousarray(np.asarray(p["sample_rows"], np.uint32))
        out = np.zeros(max(S, 1), np.uint32)
        logits = np.zeros((max(S, 1), self.cfg["vocab"]), np.uint16) if want_logits else None
        vp = lambda a: C.c_void_p(a.ctypes.data)
        allow = allow_off = None
        if masks is not None:
            from oracle import brle_allow
            offs, chunks, at = [], [], 0
            for i in range(N):
                chunks.append(brle_allow(masks[i], int(pos[i]), int(rl[i]), window))
                offs.append(at)
                at += int(rl[i])
            allow = np.ascontiguousarray(np.concatenate(chunks) if chunks else np.zeros(1, np.uint8))
            allow_off = np.ascontiguousarray(np.asarray(offs, np.int64))
        lib().orc_router_gap_reset()
        try:
            return self._forward_call(tok, pos, slots, rb, rl, pages, N, sr, S, out, logits, want_logits,
                                      masks, allow, allow_off, p)
        finally:
            lib().orc_router_gap_get.restype = C.c_float
            self._router_gap = float(lib().orc_router_gap_get())
            rows = np.zeros(max(N, 1), np.float32)
            lib().orc_router_gap_rows(C.c_void_p(rows.ctypes.data), C.c_int(N))
            self._router_row_gaps = rows[:N]

    def _forward_call(self, tok, pos, slots, rb, rl, pages, N, sr, S, out, logits, want_logits, masks,
                      allow, allow_off, p):
        vp = lambda a: C.c_void_p(a.ctypes.data)
        if self.kv_format:
            lib().orc_llama_forward_kvq(C.byref(self._m), C.c_int(self.kv_format), self._kf, self._vf,
                                        vp(tok), vp(pos), vp(slots), vp(rb), vp(rl), vp(pages), C.c_int(N),
                                        vp(sr), C.c_int(S), C.c_int(self.cfg["page_size"]), vp(out),
                                        vp(logits) if want_logits else None,
                                        vp(allow) if allow is not None else None,
                                        vp(allow_off) if allow_off is not None else None)
            return out[:S], (logits[:S] if want_logits else None), p
        lib().orc_llama_forward(C.byref(self._m), self._kp, self._vp, vp(tok), vp(pos), vp(slots),
                                vp(rb), vp(rl), vp(pages), C.c_int(N), vp(sr), C.c_int(S),
                                C.c_int(self.cfg["page_size"]), vp(out),
                                vp(logits) if want_logits else None,
                                vp(allow) if allow is not None else None,
                                vp(allow_off) if allow_off is not None else None)
        return out[:S], (logits[:S] if want_logits else None), p

    # ---- higher-precision evaluations of the same graph (oracle/src/model_hp.c) ----
    HP_MODES = {"P": 1, "f64": 2}

    def hp_pools(self, mode: str):
        """The KV pools of a higher-precision mode: two lists of float64 arrays
        [pages, page_size, hk, d], created zeroed on first use."""
        if not hasattr(self, "_hp"):
            self._hp = {}
        if mode not in self._hp:
            cfg = self.cfg
            shape = (cfg["total_pages"], cfg["page_size"], cfg["kv_heads"], cfg["head_dim"])
            k = [np.zeros(shape, np.float64) for _ in range(cfg["layers"])]
            v = [np.zeros(shape, np.float64) for _ in range(cfg["layers"])]
            self._hp[mode] = (k, v, (C.c_void_p * len(k))(*[a.ctypes.data for a in k]),
                              (C.c_void_p * len(v))(*[a.ctypes.data for a in v]))
        return self._hp[mode][0], self._hp[mode][1]

    def seed_hp_pools(self, mode: str, pages=None):
        """Copies the bf16 pools' current contents (all pages, or the listed ones) into the
        pools of `mode`, so that a higher-precision step starts from the same KV state."""
        k, v = self.hp_pools(mode)
        sel = slice(None) if pages is None else np.asarray(pages, np.int64)
        for l in range(self.cfg["layers"]):
            k[l][sel] = bf16_to_f32(self.k_pages[l][sel])
            v[l][sel] = bf16_to_f32(self.v_pages[l][sel])

    def forward_hp(self, mode: str, token_ids, position_ids, kv_page_indices, kv_page_indptr,
                   kv_last_page_lens, qo_indptr, sampling_indices=None, sampling_indptr=None,
                   masks=None, window: int = 0):
        """The forward pass without the bf16 rounding points: mode "P" = F32 activations and an
        F16 KV pool (the portable driver's rounding points), "f64" = double throughout (truth).
        Uses and updates the pools of hp_pools(mode).  Returns (tokens, logits float64 [S, V],
        plan)."""
        R = len(qo_indptr) - 1
        if sampling_indices is None:
            qo = np.asarray(qo_indptr, np.int64)
            sampling_indices = qo[1:] - qo[:-1] - 1
            sampling_indptr = np.arange(R + 1)
        p = plan_forward(token_ids, position_ids, kv_page_indices, kv_page_indptr,
                         kv_last_page_lens, qo_indptr, sampling_indices, sampling_indptr,
                         self.cfg["page_size"], self.cfg["total_pages"])
        N, S = p["N"], len(p["sample_rows"])
        c = lambda a, dt: np.ascontiguousarray(np.asarray(a, dt))
        tok, pos = c(token_ids, np.uint32), c(p["positions"], np.int32)
        slots, rb, rl = c(p["kv_slots"], np.int64), c(p["row_page_begin"], np.uint32), c(p["row_kv_len"], np.int32)
        pages, sr = c(kv_page_indices, np.uint32), c(p["sample_rows"], np.uint32)
        out = np.zeros(max(S, 1), np.uint32)
        logits = np.zeros((max(S, 1), self.cfg["vocab"]), np.float64)
        allow = allow_off = None
        if masks is not None:
            from oracle import brle_allow
            offs, chunks, at = [], [], 0
            for i in range(N):
                chunks.append(brle_allow(masks[i], int(pos[i]), int(rl[i]), window))
                offs.append(at)
                at += int(rl[i])
            allow = c(np.concatenate(chunks) if chunks else np.zeros(1, np.uint8), np.uint8)
            allow_off = c(offs, np.int64)
        self.hp_pools(mode)
        _, _, kp, vp_ = self._hp[mode]
        vp = lambda a: C.c_void_p(a.ctypes.data) if a is not None else None
        lib().orc_llama_forward_hp(C.byref(self._m), C.c_int(self.HP_MODES[mode]), kp, vp_, vp(tok), vp(pos),
                                   vp(slots), vp(rb), vp(rl), vp(pages), C.c_int(N), vp(sr), C.c_int(S),
                                   C.c_int(self.cfg["page_size"]), vp(out), vp(logits), vp(allow),
                                   vp(allow_off))
        return out[:S], logits[:S], p

    def router_gap(self) -> float:
        """Smallest gap between the last chosen and the first rejected router logit, relative to
        the token's largest logit magnitude, in the most recent forward (huge for dense models):
        near bf16 resolution, another summation order may route a token to another expert."""
        return self._router_gap

    def router_row_gaps(self) -> np.ndarray:
        """router_gap() per row of the most recent forward (minimum over its layers)."""
        return self._router_row_gaps

    def generate(self, prompt, max_new: int, replicate: int = 1, want_logits=False):
        """Greedy generation of `replicate` copies of one prompt (see generate_ragged).  Returns
        tokens [replicate, max_new] (and the per-step logits of context 0 when asked)."""
        out = self.generate_ragged([prompt] * replicate, max_new, want_logits=want_logits)
        if want_logits:
            return out[0], [step[0] for step in out[1]]
        return out

    def generate_ragged(self, prompts, max_new: int, want_logits=False):
        """Greedy generation of several contexts with their own prompts (any lengths) over
        contiguous page ranges: one prefill per context, then one multi-request decode forward
        per step in which every request sits at its own position with its own page count —
        the loop of the reference's offline harness
        (driver/portable/src/executor/executor.cpp:1439-1597) over a ragged batch.  Returns tokens
        [R, max_new] and, when asked, trace[step][r] = logits (bf16 bits) of context r;
        `prefill_router_gaps[r]` holds router_gap() of context r's prefill, `last_router_gaps` the
        smallest of those followed by the gap of each decode step, `step_router_row_gaps[s][r]`
        the gap of request r's own rows in step s (step 0 = its prefill)."""
        ps = self.cfg["page_size"]
        R = len(prompts)
        lens = [len(p) for p in prompts]
        ppc = (max(lens) + max_new + ps - 1) // ps
        toks = np.zeros((R, max_new), np.uint32)
        trace = [[None] * R for _ in range(max_new)]
        self.prefill_router_gaps = []
        for c, prompt in enumerate(prompts):
            n = lens[c]
            npg = (n + ps - 1) // ps
            t, lg, _ = self.forward(prompt, np.arange(n), np.arange(npg) + c * ppc, [0, npg],
                                    [n - (npg - 1) * ps], [0, n], want_logits=want_logits)
            toks[c, 0] = t[0]
            self.prefill_router_gaps.append(self.router_gap())
            if want_logits:
                trace[0][c] = lg[0]
        self.last_router_gaps = [min(self.prefill_router_gaps)]
        self.step_router_row_gaps = [np.asarray(self.prefill_router_gaps, np.float32)]   # [step][request]
        for s in range(1, max_new):
            pos = [n + s - 1 for n in lens]
            npg = [(p + 1 + ps - 1) // ps for p in pos]
            pages = np.concatenate([np.arange(g) + c * ppc for c, g in enumerate(npg)])
            t, lg, _ = self.forward(toks[:, s - 1], pos, pages, np.concatenate([[0], np.cumsum(npg)]),
                                    [p + 1 - (g - 1) * ps for p, g in zip(pos, npg)],
                                    np.arange(R + 1), want_logits=want_logits)
            toks[:, s] = t
            self.last_router_gaps.append(self.router_gap())
            self.step_router_row_gaps.append(self.router_row_gaps().copy())
            if want_logits:
                for c in range(R):
                    trace[s][c] = lg[c]
        return (toks, trace) if want_logits else toks


_DATA_DTYPE = {"int4b8": np.uint32, "int8": np.int8, "fp8": np.uint8, "bf16": np.uint16}


def model_from_driver(drv, cfg: dict):
    """Builds an OracleModel holding bit-identical copies of the weights a `pie_amd.driver.Driver`
    keeps on the GPU (copied out through its export hook).  `cfg` carries arch, hidden, layers,
    q_heads, kv_heads, head_dim, intermediate, vocab, quant, group_size, scale_dtype, rms_eps,
    page_size, total_pages.  Returns (model, tensors)."""
    L, quant = cfg["layers"], cfg["quant"]
    t = {}
    # the driver may keep the q / k rows of wqkv re-ordered (rows (2i, 2i+1) of a head = the
    # half-split pair (i, i + d/2)); the oracle uses the checkpoint's row order
    paired = drv.export_tensor("info.qk_rows_paired", np.int32)
    paired = bool(paired is not None and paired[0])
    interleaved = drv.export_tensor("info.rope_interleaved", np.int32)
    interleaved = int(interleaved[0]) if interleaved is not None else 0
    d_, hq_, hk_ = cfg["head_dim"], cfg["q_heads"], cfg["kv_heads"]
    inv_pair = np.arange((hq_ + 2 * hk_) * d_)
    if paired:
        # stored row h*d + 2i = original row h*d + i, stored row h*d + 2i + 1 = original h*d + d/2 + i
        head = np.empty(d_, np.int64)
        head[:d_ // 2] = 2 * np.arange(d_ // 2)
        head[d_ // 2:] = 2 * np.arange(d_ // 2) + 1
        for h in range(hq_ + hk_):
            inv_pair[h * d_:(h + 1) * d_] = h * d_ + head
    for name in ("embed", "lm_head", "final_norm"):
        t[name] = drv.export_tensor(name, np.uint16)
    t["inv_freq"] = drv.export_tensor("inv_freq", np.float32)
    scale_dt = np.uint16 if (quant == "int4b8" or cfg.get("scale_dtype", "bf16") == "bf16") else np.float32
    for l in range(L):
        p = f"layers.{l}."
        for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm"):
            a = drv.export_tensor(p + n, np.uint16)
            if a is not None:
                t[p + n] = a
        E = int(cfg.get("num_experts", 0)) if cfg["arch"] == "qwen3_moe" else 0
        if E:
            t[p + "router"] = drv.export_tensor(p + "router", np.uint16)
        for w in ("wqkv", "wo", "wgu", "wdown"):
            data = drv.export_tensor(p + w + ".data", _DATA_DTYPE[quant])
            sc = drv.export_tensor(p + w + ".scale", scale_dt)
            if w == "wgu":
                # the driver stores gate/up rows interleaved (gate_0, up_0, ...) — per expert for
                # MoE; the oracle uses the canonical order (all gate rows, then all up rows)
                n = 2 * (cfg["expert_intermediate"] if E else cfg["intermediate"])
                blocks = max(E, 1)

                def canon(a):
                    a = a.reshape(blocks, n, -1)
                    return np.concatenate([a[:, 0::2], a[:, 1::2]], axis=1).reshape(-1)
                data = canon(data)
                if sc is not None:
                    sc = canon(sc)
            if w == "wqkv" and paired:
                rows = len(inv_pair)
                data = data.reshape(rows, -1)[inv_pair].reshape(-1)
                if sc is not None:
                    sc = sc.reshape(rows, -1)[inv_pair].reshape(-1)
            t[p + w + ".data"] = data
            if sc is not None:
                t[p + w + ".scale"] = sc
    ocfg = dict(hidden=cfg["hidden"], layers=L, q_heads=cfg["q_heads"], kv_heads=cfg["kv_heads"],
                head_dim=cfg["head_dim"], intermediate=cfg["intermediate"], vocab=cfg["vocab"],
                rms_eps=cfg.get("rms_eps", 1e-5), rope_interleaved=interleaved,
                qk_norm=cfg["arch"] != "llama3", quant=quant, group_size=cfg.get("group_size", 128),
                page_size=cfg["page_size"], total_pages=cfg["total_pages"])
    ms = drv.export_tensor("info.rope_mscale", np.float32)
    ocfg["rope_mscale"] = float(ms[0]) if ms is not None else 1.0
    if cfg["arch"] == "qwen3_moe":
        ocfg.update(num_experts=cfg["num_experts"], top_k=cfg["top_k"],
                    expert_intermediate=cfg["expert_intermediate"], intermediate=0,
                    norm_topk="norm_topk = false" not in cfg.get("model_extra", ""))
    return OracleModel(ocfg, t), t
