#!/usr/bin/env python3
"""Decode benchmark of the MI355X Pie driver on its headline workload.

Workload (BASELINE.json configs[3], the configuration the metric's target is quoted on and
the largest single-GPU one): Llama-3-8B-shaped decoder, random-init N(0, 0.02) weights
quantised to W4A16 (int4b8, group 128), bf16 embeddings / lm_head, page size 16; prefill a
2048-token random prompt, then greedy decode at batch 1.  A "step" is one decode forward pass
through the driver boundary (frame -> planner -> kernels -> argmax -> response), so
`value` is whole-job decode tokens/s with weights and KV resident in HBM.

Also reported on the same JSON line:
  roofline     the dominant kernel (the weight-streaming W4A16 GEMV) over every decoder
               linear of the model: algorithmic bytes / kernel duration, each launch bracketed
               by HIP events on its own stream, against the 8 TB/s HBM peak;
  cpu_baseline the CPU oracle (a port of the reference's forward pass) timed on this box's
               host cores on a bounded sample of the same decode steps, and its tokens
               compared with the GPU's;
  extra        per-shape GEMV figures, the paged decode-attention kernel on BASELINE's
               attention config (batch 64, contexts U[512, 8192], 25% forked prefix), and the
               lm_head GEMV.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0

MODEL = dict(arch="llama3", hidden=4096, layers=32, q_heads=32, kv_heads=8, head_dim=128,
             intermediate=14336, vocab=128256, rope_theta=500000.0, quant="int4b8", group_size=128)

# Other BASELINE configurations, selectable with --model (no roofline / CPU leg on these lines):
# configs[0] Llama-3.2-1B-shaped int8 per-channel, configs[4] Qwen3-30B-A3B-shaped fp8 MoE.
OTHER_MODELS = {
    "llama1b-int8": (dict(arch="llama3", hidden=2048, layers=16, q_heads=32, kv_heads=8, head_dim=64,
                          intermediate=8192, vocab=128256, rope_theta=500000.0, quant="int8",
                          scale_dtype="bf16", tie_embeddings=True),
                     "Llama-3.2-1B-shaped W8A16 (int8 per-channel, bf16 scales) greedy decode"),
    "qwen3-30b-a3b-fp8": (dict(arch="qwen3_moe", hidden=2048, layers=48, q_heads=32, kv_heads=4,
                               head_dim=128, intermediate=0, vocab=151936, rope_theta=1000000.0,
                               quant="fp8", scale_dtype="bf16", num_experts=128, top_k=8,
                               expert_intermediate=768, router_std=0.0221, embed_std=16.0),
                          "Qwen3-30B-A3B-shaped MoE (128 experts, top-8, fp8 e4m3 experts with bf16 "
                          "row scales) greedy decode"),
}


def toml(model: dict, page_size: int, total_pages: int, max_tokens: int, max_requests: int,
         kv_cache_dtype: str = "auto") -> str:
    lines = ["[model]"]
    for k, v in model.items():
        if isinstance(v, bool):
            lines.append(f"{k} = {'true' if v else 'false'}")
        else:
            lines.append(f'{k} = "{v}"' if isinstance(v, str) else f"{k} = {v}")
    lines += ["[batching]", f"kv_page_size = {page_size}", f"total_pages = {total_pages}",
              f"max_forward_tokens = {max_tokens}", f"max_forward_requests = {max_requests}",
              f'kv_cache_dtype = "{kv_cache_dtype}"', "[runtime]", "use_graphs = true"]
    return "\n".join(lines) + "\n"


class Hip:
    """The few HIP runtime calls the measurement needs (events bracketing single kernels)."""

    def __init__(self):
        self.lib = C.CDLL("libamdhip64.so")
        self.lib.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.lib.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.lib.hipEventDestroy.argtypes = [C.c_void_p]
        self.lib.hipDeviceSynchronize.argtypes = []

    def event(self) -> C.c_void_p:
        e = C.c_void_p()
        if self.lib.hipEventCreate(C.byref(e)) != 0:
            raise RuntimeError("hipEventCreate failed")
        return e

    def elapsed_ms(self, a, b) -> float:
        ms = C.c_float()
        if self.lib.hipEventElapsedTime(C.byref(ms), a, b) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        return float(ms.value)

    def sync(self):
        if self.lib.hipDeviceSynchronize() != 0:
            raise RuntimeError("hipDeviceSynchronize failed")


def gemv_roofline(drv, hip, model, reps: int):
    """Every int4 decoder linear of the model, M = 1, each kernel bracketed by its own events.
    Walking all layers streams 3.6 GB per pass, far beyond the last-level cache, so every launch
    reads its weights from HBM as it does inside a decode step."""
    import torch

    from pie_amd._lib import kernels

    k = kernels()
    H, d, hq, hk, I, G = (model[x] for x in ("hidden", "head_dim", "q_heads", "kv_heads",
                                             "intermediate", "group_size"))
    shapes = {"wqkv": ((hq + 2 * hk) * d, H), "wo": (H, hq * d), "wgu": (2 * I, H), "wdown": (H, I)}
    dev = torch.device("cuda:0")
    acts = {K: torch.randn(1, K, device=dev).bfloat16() for K in {s[1] for s in shapes.values()}}
    outs = {N: torch.zeros(1, N, device=dev, dtype=torch.bfloat16) for N in {s[0] for s in shapes.values()}}
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    per_shape = {n: [0.0, 0] for n in shapes}
    events = []
    for rep in range(reps + 1):  # first pass warms code objects and is dropped
        for l in range(model["layers"]):
            for name, (N, K) in shapes.items():
                e0, e1 = hip.event(), hip.event()
                st = k.pie_hip_gemv_w4a16_timed(C.c_void_p(acts[K].data_ptr()),
                                                C.c_void_p(drv.tensor_ptr(f"layers.{l}.{name}.data")),
                                                C.c_void_p(drv.tensor_ptr(f"layers.{l}.{name}.scale")),
                                                C.c_void_p(outs[N].data_ptr()), 1, N, K, G, 0, e0, e1, stream)
                if st != 0:
                    raise RuntimeError(f"pie_hip_gemv_w4a16_timed status {st}")
                if rep > 0:
                    events.append((name, e0, e1))
    hip.sync()
    for name, e0, e1 in events:
        per_shape[name][0] += hip.elapsed_ms(e0, e1) * 1e-3
        per_shape[name][1] += 1
    def alg_bytes(N, K):
        return N * K // 2 + N * (K // G) * 2 + K * 2 + N * 2
    tot_t = sum(v[0] for v in per_shape.values())
    tot_b = sum(alg_bytes(*shapes[n]) * v[1] for n, v in per_shape.items())
    launches = sum(v[1] for v in per_shape.values())
    detail = {n: dict(N=shapes[n][0], K=shapes[n][1], us=round(v[0] / v[1] * 1e6, 2),
                      gbps=round(alg_bytes(*shapes[n]) / (v[0] / v[1]) / 1e9, 1))
              for n, v in per_shape.items()}
    return dict(achieved=tot_b / tot_t / 1e9, avg_us=tot_t / launches * 1e6,
                bytes_per_launch=tot_b / launches, launches=launches, detail=detail)


def time_graph(fn, n_launch: int, reps: int = 5) -> float:
    """Average seconds per launch of fn() replayed from a HIP graph on torch's stream."""
    import torch

    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        for _ in range(2):
            fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(n_launch):
            fn()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / (reps * n_launch)


def attention_case():
    """BASELINE's attention config as device tensors plus one launcher per KV storage:
    32 q / 8 kv heads of 128, page 16, 64 requests with contexts uniform in [512, 8192], block
    tables a random permutation of the pool, 16 of the 64 sharing a forked 1024-token prefix."""
    import torch

    from pie_amd import ops

    dev = torch.device("cuda:0")
    hq, hk, d, ps, R = 32, 8, 128, 16, 64
    rng = np.random.default_rng(3)
    ctx = rng.integers(512, 8193, size=R)
    ctx[:16] = np.maximum(ctx[:16], 1024)
    npg = (ctx + ps - 1) // ps
    shared = 1024 // ps
    total = int(npg.sum() - 15 * shared) + 8
    perm = rng.permutation(total).astype(np.int32)
    idx, indptr, last = [], [0], []
    nxt, prefix = shared, perm[:shared]
    for r in range(R):
        n = int(npg[r])
        if r < 16:
            pages = np.concatenate([prefix, perm[nxt:nxt + n - shared]])
            nxt += n - shared
        else:
            pages = perm[nxt:nxt + n]
            nxt += n
        idx.append(pages)
        indptr.append(indptr[-1] + n)
        last.append(int(ctx[r]) - (n - 1) * ps)
    kp = torch.randn(total, ps, hk, d, device=dev).bfloat16()
    vp = torch.randn(total, ps, hk, d, device=dev).bfloat16()
    q = torch.randn(R, hq, d, device=dev).bfloat16()
    pi = torch.from_numpy(np.concatenate(idx)).to(dev)
    pp = torch.tensor(indptr, dtype=torch.int32, device=dev)
    ll = torch.tensor(last, dtype=torch.int32, device=dev)
    maxlen = int(ctx.max())
    need = ops.attn_decode_workspace_bytes(R, hq, hk, d, maxlen)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    o = torch.empty_like(q)
    alg = int(ctx.sum()) * 2 * hk * d * 2 + R * hq * d * 2 * 2
    dedup = alg - 15 * 1024 * 2 * hk * d * 2
    launch = {"bf16": lambda: ops.attention_paged_decode(q, kp, vp, pi, pp, ll, maxlen, o=o, workspace=ws)}
    # the same batch over one-byte pools (codes + fp32 scales per (token, head))
    rb = torch.tensor(indptr[:-1], dtype=torch.int32, device=dev)
    rl = torch.from_numpy(ctx.astype(np.int32)).to(dev)
    keep = []
    for fmt in ("fp8_per_token_head", "int8_per_token_head"):
        k8 = torch.randint(0, 120, (total, ps, hk, d), dtype=torch.uint8, device=dev)
        v8 = torch.randint(0, 120, (total, ps, hk, d), dtype=torch.uint8, device=dev)
        ks = torch.rand(total, hk, ps, device=dev) * 0.01 + 0.001
        vs = torch.rand(total, hk, ps, device=dev) * 0.01 + 0.001
        keep.append((k8, v8, ks, vs))
        launch[fmt] = (lambda fmt=fmt, k8=k8, v8=v8, ks=ks, vs=vs:
                       ops.attention_rows_paged_kvq(fmt, q, k8, v8, ks, vs, pi, rb, rl, max_kv_len=maxlen,
                                                    o=o, workspace=ws))
    algq = int(ctx.sum()) * 2 * hk * (d + 4) + R * hq * d * 2 * 2
    return dict(launch=launch, alg=alg, dedup=dedup, alg_one_byte=algq, keep=keep)


def attention_extra():
    """Paged decode attention on BASELINE's attention config, timed from a HIP graph."""
    case = attention_case()
    t = time_graph(case["launch"]["bf16"], 10)
    one_byte = {}
    for fmt in ("fp8_per_token_head", "int8_per_token_head"):
        case["launch"][fmt]()
        tq = time_graph(case["launch"][fmt], 10)
        algq = case["alg_one_byte"]
        one_byte[fmt] = dict(us=round(tq * 1e6, 1), algorithmic_bytes=algq, gbps=round(algq / tq / 1e9, 1),
                             frac_of_hbm_peak=round(algq / tq / 1e9 / HBM_PEAK_GBPS, 4))
    alg = case["alg"]
    return dict(workload="decode attention 32q/8kv d128 page16 batch64 ctx U[512,8192] 25% forked 1024 prefix",
                us=round(t * 1e6, 1), algorithmic_bytes=alg, gbps=round(alg / t / 1e9, 1),
                frac_of_hbm_peak=round(alg / t / 1e9 / HBM_PEAK_GBPS, 4),
                dedup_bytes=case["dedup"], note="split kernel + merge kernel per call", one_byte_kv=one_byte)


def attention_workload():
    """What a `rocprofv3` run over the attention config needs: four 256 MiB device copies (the
    scale of the FETCH_SIZE / WRITE_SIZE counters), then 12 eager launches of the decode
    attention over the bf16 pool and 12 over each one-byte pool."""
    import torch

    dev = torch.device("cuda:0")
    src = torch.empty(256 * 1024 * 1024 // 4, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    for _ in range(4):
        dst.copy_(src)
    torch.cuda.synchronize()
    case = attention_case()
    for name, fn in case["launch"].items():
        for _ in range(12):
            fn()
        torch.cuda.synchronize()
    print(json.dumps({"attention_workload": "4 x 256 MiB copy, 12 launches of the batch-64 decode attention per "
                                            "KV storage (bf16, fp8_per_token_head, int8_per_token_head)",
                      "algorithmic_bytes_bf16": case["alg"], "deduplicated_bytes_bf16": case["dedup"],
                      "algorithmic_bytes_one_byte": case["alg_one_byte"]}))


def w4a16_sweep_extra():
    """The W4A16 GEMM sweep of BASELINE's second config: (K, N) x M, int4b8 group 128.  Each
    (shape, M) is timed from a HIP graph that walks a ring of weight copies larger than the
    256 MB last-level cache, so every launch streams its weights from HBM.  M <= 4 runs the GEMV,
    above that the faster of the skinny and the tiled matrix-core GEMM (both reported); the skinny
    GEMM reads tile-major copies of the weights, as the driver's decoder linears do."""
    import torch

    from pie_amd import ops

    dev = torch.device("cuda:0")
    G = 128
    out = {}
    for K, N in ((4096, 4096), (4096, 14336), (14336, 4096)):
        wbytes = N * K // 2 + N * (K // G) * 2
        ncopy = max(2, -(-600_000_000 // wbytes))
        ring = [ops.int4b8_view(torch.randint(-2**31, 2**31 - 1, (N, K // 8), dtype=torch.int32, device=dev),
                                (torch.rand(N, K // G, device=dev) * 0.015 + 0.005).bfloat16(), G)
                for _ in range(ncopy)]
        tiled_ring = [ops.repack_mfma_tiles(w) for w in ring]
        for M in (1, 8, 32, 128, 2048):
            act = torch.randn(M, K, device=dev).bfloat16()
            y = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            it = iter(range(10**9))
            alg = wbytes + M * K * 2 + M * N * 2
            kernels = {"gemv": ops.linear_fused} if M <= 4 else {}
            if 4 < M <= 128:
                kernels["skinny"] = ops.gemm_skinny
            if M >= 48:
                kernels["tiled"] = ops.gemm_mfma
            res = {}
            for name, fn in kernels.items():
                src = tiled_ring if name == "skinny" else ring
                t = time_graph(lambda: fn(act, src[next(it) % ncopy], y=y), ncopy, reps=3)
                res[name] = dict(us=round(t * 1e6, 1), gbps=round(alg / t / 1e9, 1),
                                 tflops=round(2.0 * M * N * K / t / 1e12, 1))
            out[f"K{K}_N{N}_M{M}"] = res
        del ring, tiled_ring
        torch.cuda.empty_cache()
    return out


def other_configs_extra(drvmod):
    """Decode throughput of the other BASELINE decode configurations, each through its own driver
    instance (created after the headline driver is closed): the 8B W4A16 model at batch 16 and 64
    after 2048-token prefills, the 1B int8 model at batch 1 (128-token prompt, 64 steps) and the
    30B-A3B fp8 MoE at batch 64 over 1024-token contexts."""
    import torch

    out = {}
    cases = [("llama8b_w4a16_batch16_ctx2048", MODEL, 16, 2048, 32, 4),
             ("llama8b_w4a16_batch64_ctx2048", MODEL, 64, 2048, 32, 4),
             ("llama1b_int8_batch1_prompt128", OTHER_MODELS["llama1b-int8"][0], 1, 128, 64, 8),
             ("qwen3_30b_a3b_fp8_batch64_ctx1024", OTHER_MODELS["qwen3-30b-a3b-fp8"][0], 64, 1024, 32, 4)]
    for name, model, batch, n_prompt, steps, warm in cases:
        page_size = 16
        max_new = warm + steps + 1
        pages = (n_prompt + max_new + page_size - 1) // page_size * batch + 8
        rng = np.random.default_rng(4096 + batch)
        prompt = rng.integers(0, model["vocab"], n_prompt)
        t0 = time.perf_counter()
        drv = drvmod.Driver(toml(model, page_size, pages, 2048, max(16, batch)))
        t_init = time.perf_counter() - t0
        try:
            drv.set_generate_divergence(7919)   # distinct rows in the decode batch (distinct MoE routes)
            _, tm = drv.generate(prompt, max_new, replicate=batch, warmup=warm)
        finally:
            drv.close()
        torch.cuda.empty_cache()
        wall = tm["decode_wall_us"] * 1e-6
        out[name] = dict(tokens_per_s=round(batch * tm["decode_steps"] / wall, 1),
                         ms_per_step=round(wall / tm["decode_steps"] * 1e3, 4), steps=tm["decode_steps"],
                         warmup=warm, init_s=round(t_init, 2), prefill_s=round(tm["prefill_us"] * 1e-6, 3))
    return out


def lm_head_extra(drv, model):
    import torch

    from pie_amd._lib import kernels

    k = kernels()
    dev = torch.device("cuda:0")
    V, H = model["vocab"], model["hidden"]
    x = torch.randn(1, H, device=dev).bfloat16()
    y = torch.empty(1, V, device=dev, dtype=torch.bfloat16)
    w = drv.tensor_ptr("lm_head")
    fn = lambda: k.pie_hip_gemv_bf16(C.c_void_p(x.data_ptr()), C.c_void_p(w), C.c_void_p(y.data_ptr()),
                                     1, V, H, 0, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    t = time_graph(fn, 4)
    b = V * H * 2 + H * 2 + V * 2
    return dict(workload="bf16 lm_head GEMV [128256 x 4096]", us=round(t * 1e6, 1),
                gbps=round(b / t / 1e9, 1), frac_of_hbm_peak=round(b / t / 1e9 / HBM_PEAK_GBPS, 4),
                note="1 GB per call: larger than L2, smaller than the 256 MB last-level cache x4")


def cpu_baseline(drv, model, page_size, total_pages, n_prompt, gpu_tokens, budget_s: float):
    """The CPU oracle on the same decode steps: weights and the prefilled KV pools are copied
    from the GPU, then the oracle decodes from the first post-prompt position."""
    from oracle.model import model_from_driver

    cfg = dict(model, page_size=page_size, total_pages=total_pages, scale_dtype="bf16", rms_eps=1e-5)
    om, _ = model_from_driver(drv, cfg)
    for l in range(model["layers"]):
        om.k_pages[l][...] = drv.export_tensor(f"kv.k.{l}", np.uint16).reshape(om.k_pages[l].shape)
        om.v_pages[l][...] = drv.export_tensor(f"kv.v.{l}", np.uint16).reshape(om.v_pages[l].shape)
    import oracle

    from pie_amd import driver as drvmod

    # The same steps in double precision (the value both implementations approximate), from the
    # same prefilled pages: separates rounding noise shared by both from a defect in either.
    truth_steps = 4
    om.seed_hp_pools("f64", pages=np.arange((n_prompt + page_size - 1) // page_size))
    dev_gpu_truth, dev_orc_truth = [], []
    steps, matched, near_ties, t_total = 0, 0, 0, 0.0
    margins = []   # per mismatch: how far below its own choice the oracle ranks the GPU's token
    cosines, noise_rel_top, replay_diff = [], [], 0
    tok = int(gpu_tokens[0])
    V = model["vocab"]
    while steps < len(gpu_tokens) - 1 and (steps < 2 or t_total < budget_s):
        pos = n_prompt + steps
        npg = (pos + 1 + page_size - 1) // page_size
        last = pos + 1 - (npg - 1) * page_size
        # the same step through the boundary once more, for its logits (the KV slot of `pos` is
        # rewritten with the values it already holds: same token, same context)
        res = drv.forward(drvmod.ForwardFrame([tok], [pos], np.arange(npg), [0, npg], [last], [0, 1]))
        g = oracle.bf16_to_f32(drv.export_tensor("debug.logits", np.uint16).reshape(-1, V)[0]).astype(np.float64)
        t0 = time.perf_counter()
        out, logits, _ = om.forward([tok], [pos], np.arange(npg), [0, npg], [last], [0, 1], want_logits=True)
        t_total += time.perf_counter() - t0
        steps += 1
        lg = oracle.bf16_to_f32(np.asarray(logits).reshape(-1)).astype(np.float64)
        cosines.append(float(g @ lg / (np.linalg.norm(g) * np.linalg.norm(lg) + 1e-30)))
        if steps <= truth_steps:   # (untimed)
            _, lt, _ = om.forward_hp("f64", [tok], [pos], np.arange(npg), [0, npg], [last], [0, 1])
            lt = lt[0]
            one_minus_cos = lambda a: float(1.0 - a @ lt / (np.linalg.norm(a) * np.linalg.norm(lt) + 1e-30))
            dev_gpu_truth.append(one_minus_cos(g))
            dev_orc_truth.append(one_minus_cos(lg))
        top = float(lg[int(out[0])])
        dev_rms = float(np.sqrt(np.mean((g - lg) ** 2)))   # rms logit deviation of this step
        noise_rel_top.append(dev_rms / max(abs(top), 1e-30))
        replay_diff += int(int(res.tokens[0]) != int(gpu_tokens[steps]))   # (expected 0: same step, same kernels)
        if int(out[0]) == int(gpu_tokens[steps]):
            matched += 1
        else:
            # a mismatch counts as a near-tie where the oracle's margin for its own token over the
            # GPU's is within three times the rms deviation between the two logit vectors of
            # this step (two independent errors of that size close such a gap)
            margin = top - float(lg[int(gpu_tokens[steps])])
            near_ties += int(margin <= 3.0 * dev_rms)
            margins.append(round(margin / max(abs(top), 1e-30), 5))
        tok = int(gpu_tokens[steps])  # teacher-forced: every step is compared on the same context
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return dict(value=steps / t_total, unit="tokens/s", cores=cores, kind="port",
                sample=f"{steps} batch-1 decode steps of the same model at context {n_prompt}+, "
                       "oracle (C restatement of the reference forward pass, OpenMP over rows) "
                       "fed the GPU's weights and prefilled KV pages; every compared step is also replayed "
                       "through the driver boundary for its logits",
                greedy_tokens_matched=matched, greedy_tokens_compared=steps,
                mismatches_at_oracle_near_ties=near_ties,
                mismatch_margins_rel_to_top_logit=margins,
                logit_cosine_min=round(min(cosines), 6), logit_cosine_mean=round(float(np.mean(cosines)), 6),
                logit_rms_deviation_rel_to_top_logit=round(float(np.mean(noise_rel_top)), 5),
                replayed_steps_with_another_token=replay_diff,
                one_minus_cosine_vs_double_precision=dict(
                    note=f"first {len(dev_gpu_truth)} compared steps re-evaluated in double precision from the "
                         "same prefilled pages (untimed): distance of the GPU's and of the oracle's logits "
                         "from that truth",
                    gpu=[float(f"{v:.3e}") for v in dev_gpu_truth],
                    oracle=[float(f"{v:.3e}") for v in dev_orc_truth]))


def gemv_traffic_bytes_per_launch():
    """HBM bytes per GEMV launch (average of the model's four int4 linears at M = 1) as the
    committed `rocprofv3 --pmc` summary states them, or None when that file is missing or holds
    no such line.  The summary is rewritten whenever the kernel is profiled again, so this figure
    cannot outlive the kernel it was measured on unnoticed: the summary names the library build
    it profiled."""
    import re

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "gemv_w4a16_m1_hbm_traffic_pmc.md")
    try:
        m = re.search(r"^traffic_bytes_per_launch:\s*([0-9_]+)", open(path).read(), re.M)
    except OSError:
        return None
    return int(m.group(1).replace("_", "")) if m else None


def pmc_workload():
    import torch

    from pie_amd import ops

    dev = torch.device("cuda:0")
    src = torch.empty(256 * 1024 * 1024 // 4, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    for _ in range(4):
        dst.copy_(src)
    torch.cuda.synchronize()
    H, I, G = MODEL["hidden"], MODEL["intermediate"], MODEL["group_size"]
    qkv = (MODEL["q_heads"] + 2 * MODEL["kv_heads"]) * MODEL["head_dim"]
    for (N, K) in [(qkv, H), (H, H), (2 * I, H), (H, I)]:
        ws = [ops.int4b8_view(torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev),
                              (torch.rand(N, K // G, device=dev) * 0.015 + 0.005).bfloat16(), G)
              for _ in range(6)]
        act = torch.randn(1, K, device=dev).bfloat16()
        y = torch.empty(1, N, device=dev, dtype=torch.bfloat16)
        for i in range(12):
            ops.linear_fused(act, ws[i % 6], y=y)
        torch.cuda.synchronize()
        if N == 2 * I:
            # the same matrices in the tile-major layout under the skinny GEMM at 16 rows
            tiled = [ops.repack_mfma_tiles(w) for w in ws]
            act16 = torch.randn(16, K, device=dev).bfloat16()
            y16 = torch.empty(16, N, device=dev, dtype=torch.bfloat16)
            for i in range(12):
                ops.gemm_skinny(act16, tiled[i % 6], y=y16)
            torch.cuda.synchronize()
            del tiled
        del ws
    print(json.dumps({"pmc_workload": "4 x 256 MiB copy, 12 launches of each int4 GEMV shape at M=1, "
                                      "12 launches of the skinny GEMM at M=16 on the gate|up shape"}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--kv-cache-dtype", default="auto",
                    choices=["auto", "bf16", "fp8_e4m3", "fp8_e5m2", "int8_per_token_head", "fp8_per_token_head", "nvfp4"],
                    help="KV-cache storage of the driver under test (the headline run keeps bf16)")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--model", default="llama8b-w4a16", choices=["llama8b-w4a16", *OTHER_MODELS])
    ap.add_argument("--sampler", default="greedy", choices=["greedy", "top_p", "top_k", "min_p", "multinomial"],
                    help="decode-step sampler (default greedy = the headline workload); the others run "
                         "the device samplers at temperature 0.8 (top_p 0.95 / top_k 50 / min_p 0.05)")
    ap.add_argument("--attention-workload", action="store_true",
                    help="only launch the batch-64 decode attention of BASELINE's attention config (and a "
                         "256 MiB copy as the counters' scale), for `rocprofv3` kernel traces and --pmc runs")
    ap.add_argument("--pmc-workload", action="store_true",
                    help="only launch what a `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE` run needs: a "
                         "256 MiB device copy (the counter's scale) and the four int4 GEMV shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this driver path is built and measured on one GPU; "
              f"--gpus {args.gpus} is not supported (run with --gpus 1).", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from pie_amd import driver as drvmod

    if args.pmc_workload:
        pmc_workload()
        return
    if args.attention_workload:
        attention_workload()
        return
    page_size = 16
    max_new = args.warmup + args.steps + 1
    pages_per_ctx = (args.prompt + max_new + page_size - 1) // page_size
    total_pages = pages_per_ctx * args.batch + 8
    model, label = (MODEL, None) if args.model == "llama8b-w4a16" else OTHER_MODELS[args.model]
    cfg_text = toml(model, page_size, total_pages, 2048, max(16, args.batch), args.kv_cache_dtype)
    hip = Hip()
    rng = np.random.default_rng(2048)
    prompt = rng.integers(0, model["vocab"], args.prompt)

    t0 = time.perf_counter()
    drv = drvmod.Driver(cfg_text)
    t_init = time.perf_counter() - t0

    if args.sampler != "greedy":
        kind, k, p = {"multinomial": (0, 0, 1.0), "top_k": (1, 50, 1.0), "top_p": (2, 0, 0.95),
                      "min_p": (3, 0, 0.05)}[args.sampler]
        drv.set_generate_sampler(kind, 0.8, k, p, seed=12345)
        label = (label or "Llama-3-8B-shaped W4A16 (int4b8 group 128) decode") + f", {args.sampler} sampling at T=0.8"
    torch.cuda.synchronize()
    if args.batch > 1:
        drv.set_generate_divergence(7919)   # distinct rows in the decode batch (distinct MoE routes)
    tokens, tm = drv.generate(prompt, max_new, replicate=args.batch, warmup=args.warmup)
    steps = tm["decode_steps"]
    assert steps == args.steps, (steps, args.steps)
    wall_s = tm["decode_wall_us"] * 1e-6
    value = args.batch * steps / wall_s
    if label is not None:
        drv.close()
        print(json.dumps({
            "metric": "decode tokens/sec @1 GPU + quant-GEMV/attention HBM GB/s as % of 8 TB/s",
            "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
            "warmup": args.warmup, "ms_per_step": round(wall_s / steps * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
            "data": "synthetic",
            "config": {"workload": f"{label}, batch {args.batch}, after a {args.prompt}-token "
                                   "prefill, page size 16", "batch": args.batch,
                       "prompt_tokens": args.prompt, "page_size": page_size},
            "roofline": None, "cpu_baseline": None,
            "extra": {"init_s": round(t_init, 2), "prefill_s": round(tm["prefill_us"] * 1e-6, 3),
                      "decode_device_ms_per_step": round(tm["decode_device_us"] * 1e-3 / steps, 4)}}))
        return

    roof = gemv_roofline(drv, hip, MODEL, reps=2)
    extra = {"gemv_w4a16_shapes": roof["detail"], "init_s": round(t_init, 2),
             "prefill_s": round(tm["prefill_us"] * 1e-6, 3),
             "decode_device_ms_per_step": round(tm["decode_device_us"] * 1e-3 / steps, 4)}
    if not args.no_extra:
        extra["decode_attention"] = attention_extra()
        extra["lm_head"] = lm_head_extra(drv, MODEL)
        extra["w4a16_gemm_sweep"] = w4a16_sweep_extra()
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(drv, MODEL, page_size, total_pages, args.prompt, tokens[0], args.cpu_seconds)
    drv.close()
    if not args.no_extra:
        torch.cuda.empty_cache()
        extra["other_configs"] = other_configs_extra(drvmod)

    out = {
        "metric": "decode tokens/sec @1 GPU + quant-GEMV/attention HBM GB/s as % of 8 TB/s",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": args.warmup, "ms_per_step": round(wall_s / steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Llama-3-8B-shaped W4A16 (int4b8 group 128) greedy decode, "
                               f"batch {args.batch}, after a {args.prompt}-token prefill, page size 16",
                   "batch": args.batch, "prompt_tokens": args.prompt, "page_size": page_size,
                   "weights": "int4b8 group 128, bf16 scales; bf16 embed/lm_head; fp32 accumulation"},
        "roofline": {"bound": "hbm", "kernel": "gemv_kernel<FmtInt4> (W4A16 weight-streaming GEMV, M=1)",
                     "achieved": round(roof["achieved"], 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(roof["achieved"] / HBM_PEAK_GBPS, 4),
                     "traffic": gemv_traffic_bytes_per_launch(),
                     "avg_launch_us": round(roof["avg_us"], 2),
                     "algorithmic_bytes_per_launch": int(roof["bytes_per_launch"]),
                     "launches_timed": roof["launches"]},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
