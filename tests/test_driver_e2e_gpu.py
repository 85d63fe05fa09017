"""End-to-end GPU parity: the driver (boundary -> planner -> kernels -> response) against the
oracle model on bit-identical weights.  Greedy tokens must match wherever the oracle's top-2
logit gap exceeds bf16 resolution (near-ties are flagged, not hidden); logits agree to cosine
>= 0.9999, the tolerance precedent of driver/cuda/tests/parity_qwen3.py:160-181."""
import numpy as np
import pytest

from driver_util import cosine, full_cfg, oracle_model_from_driver, toml_config

pytestmark = pytest.mark.gpu


def ragged_prompts(rng, vocab, n_prompt, count):
    """`count` distinct prompts of different lengths (the first `n_prompt` long, the others
    shorter or longer by a few tokens, crossing page boundaries at different steps; for large
    batches, lengths drawn from 1 .. 3 * n_prompt)."""
    if count > 8:
        lens = [n_prompt] + [int(n) for n in rng.integers(1, 3 * n_prompt + 1, count - 1)]
    else:
        lens = [max(1, n_prompt + ((-1) ** c) * (3 * c + (c // 2))) for c in range(count)]
    return [rng.integers(0, vocab, n) for n in lens]


def teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, max_new, **bars):
    """Feed the oracle's tokens to the GPU step by step — every context with its own prompt, its
    own length and so its own position and page count in each decode batch — and compare the
    token and the logits of EVERY request of every step.  Returns (oracle tokens, near-ties,
    checks)."""
    ps, V = cfg["page_size"], cfg["vocab"]
    R = len(prompts)
    lens = [len(p) for p in prompts]
    ppc = (max(lens) + max_new + ps - 1) // ps
    otoks, otrace = om.generate_ragged(prompts, max_new, want_logits=True)
    near_ties = checks = 0
    for c, prompt in enumerate(prompts):   # prefill each context
        n = lens[c]
        npg = (n + ps - 1) // ps
        fr = drvmod.ForwardFrame(prompt, np.arange(n), np.arange(npg) + c * ppc, [0, npg],
                                 [n - (npg - 1) * ps], [0, n])
        res = d.forward(fr)
        assert res.num_requests == 1 and len(res.tokens) == 1
        lg = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[0]
        near_ties += check_step(oracle, lg, otrace[0][c], res.tokens[0], otoks[c, 0],
                                router_gap=om.prefill_router_gaps[c], **bars)
        checks += 1
    # A request's logits depend on the routing of its own rows only, now and in the steps that
    # wrote its KV history: the margin that matters is the smallest over the request's past.
    gap_so_far = np.asarray(om.step_router_row_gaps[0], np.float64).copy()
    for s in range(1, max_new):
        pos = [n + s - 1 for n in lens]
        npg = [(p + 1 + ps - 1) // ps for p in pos]
        pages = np.concatenate([np.arange(g) + c * ppc for c, g in enumerate(npg)])
        fr = drvmod.ForwardFrame(otoks[:, s - 1], pos, pages, np.concatenate([[0], np.cumsum(npg)]),
                                 [p + 1 - (g - 1) * ps for p, g in zip(pos, npg)], np.arange(R + 1))
        res = d.forward(fr)
        assert res.num_requests == R and res.tokens_indptr == list(range(R + 1))
        lg = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
        gap_so_far = np.minimum(gap_so_far, om.step_router_row_gaps[s])
        for c in range(R):
            near_ties += check_step(oracle, lg[c], otrace[s][c], res.tokens[c], otoks[c, s],
                                    router_gap=gap_so_far[c], **bars)
            checks += 1
    return otoks, near_ties, checks


def check_step(oracle, gpu_logit_bits, orc_logit_bits, gpu_tok, orc_tok, cos_min=0.9999, rel=0.02,
               tie=2.0 ** -6, router_gap=float("inf")):
    g = oracle.bf16_to_f32(gpu_logit_bits)
    o = oracle.bf16_to_f32(orc_logit_bits)
    # MoE: where the oracle's router logits separate the last chosen expert from the first
    # rejected one by no more than two bf16 steps of the row's largest logit, another fp32
    # summation order upstream may route a token of this forward to another expert.  Such a step
    # counts as a near-tie and is held to a looser logit bar (one expert of top_k swapped for its
    # neighbour), never skipped.
    router_tie = router_gap <= 2.0 ** -7
    if router_tie:
        cos_min, rel = min(cos_min, 0.995), max(rel, 0.15)
    assert cosine(g, o) >= cos_min
    assert np.max(np.abs(g - o)) <= rel * np.max(np.abs(o)) + 1e-3
    top2 = np.sort(o)[-2:]
    # a near-tie: the oracle's two best logits are closer than the measured noise between the two
    # logit vectors can bridge — four times the rms deviation of this very row (the difference of
    # two entries' deviations has sqrt(2) of it: 2.8 sigma) — and never more than `tie` of the best
    # logit (2^-6 = two bf16 steps in the worst case), the bound that stood alone before
    noise = 4.0 * float(np.sqrt(np.mean((g - o) ** 2)))
    margin = min(tie * abs(top2[1]), noise) + 1e-6
    near_tie = router_tie or (top2[1] - top2[0]) <= margin
    if not near_tie:
        assert int(gpu_tok) == int(orc_tok)
    elif not router_tie:
        # a near-tie is not skipped: the token must be one of the tied candidates, i.e. a token
        # whose oracle logit is within `tie` of the oracle's best (the two entries' own deviations
        # can exceed the row's rms several times)
        assert o[int(gpu_tok)] >= top2[1] - (tie * abs(top2[1]) + 1e-6)
    # the token the driver returns is the argmax of its own logits, first index on ties
    assert int(gpu_tok) == int(np.argmax(g))
    return int(near_tie)


@pytest.mark.parametrize("kw", [
    dict(quant="int4b8"),
    dict(quant="int8", scale_dtype="bf16"),
    dict(quant="int8", scale_dtype="f32", tie=True),
    dict(quant="fp8"),
    dict(quant="bf16"),
    dict(arch="qwen3", quant="int4b8", head_dim=128, q_heads=4, kv_heads=1, rope_theta=1e6),
    dict(quant="int4b8", head_dim=128, q_heads=8, kv_heads=2, hidden=1024, rope_factor=8.0),
    dict(quant="int4b8", page_size=32, use_graphs=False),
    dict(quant="int4b8", rope_interleaved=True),
    dict(quant="bf16", rope_interleaved=True, use_graphs=False),
    # a down projection whose rows are past the GEMV's staged-activation limit for one-byte
    # weights (16 384 values): single-row decode steps take the matrix-core route for it
    dict(quant="int8", scale_dtype="bf16", intermediate=16384),
    dict(arch="qwen3_moe", quant="fp8", head_dim=128, q_heads=4, kv_heads=1, num_experts=8, top_k=2,
         expert_intermediate=256, router_std=0.2, intermediate=0),
    dict(arch="qwen3_moe", quant="int4b8", head_dim=128, q_heads=4, kv_heads=1, num_experts=16,
         top_k=4, expert_intermediate=512, router_std=0.2, intermediate=0),
    dict(arch="qwen3_moe", quant="bf16", head_dim=64, q_heads=8, kv_heads=2, num_experts=6, top_k=3,
         expert_intermediate=128, router_std=0.2, intermediate=0, use_graphs=False),
], ids=lambda k: "-".join(f"{a}={b}" for a, b in k.items()))
def test_greedy_generation_matches_oracle(gpu, oracle, kw):
    from pie_amd import driver as drvmod

    cfg = full_cfg(**kw)
    rng = np.random.default_rng(90)
    prompts = ragged_prompts(rng, cfg["vocab"], 21, 3)
    with drvmod.Driver(toml_config(**kw)) as d:
        caps = d.capabilities()
        assert caps["kv_page_size"] == cfg["page_size"] and caps["vocab_size"] == cfg["vocab"]
        om, _ = oracle_model_from_driver(d, cfg)
        otoks, near, checks = teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, 10)
        # (2048 nearly flat logits: about a third of the rows have a runner-up within two bf16
        # steps of the best; those rows are held to "one of the tied candidates" by check_step)
        # (MoE: a request also counts as near-tie once any token of its history had a router
        # margin at bf16 resolution; those steps are held to the looser bar, never skipped)
        print(f"near-ties {near} of {checks}")
        # (measured 0 - 6 of 30 on the dense models; the old 2^-6 bound alone gave about a third)
        assert checks == 30 and (near <= checks // 4 or cfg["num_experts"])
    # free-running generation through the driver's own harness reproduces the oracle's
    # sequence (up to the first near-tie, if any)
    with drvmod.Driver(toml_config(**kw)) as d:
        gtoks, tm = d.generate(prompts[0], 10, replicate=2)
        assert tm["decode_steps"] == 9 and tm["decode_device_us"] > 0
        if near == 0:
            assert np.array_equal(gtoks[0], otoks[0])
        assert np.array_equal(gtoks[0], gtoks[1])


@pytest.mark.parametrize("quant", ["int4b8", "fp8"])
def test_long_prefill_through_the_tiled_gemm(gpu, oracle, quant):
    """A 230-token prompt (two chunks under max_forward_tokens=208: 208 rows through the tiled
    matrix-core GEMM, 22 through the skinny one), then decode; logits and tokens against the
    oracle."""
    from pie_amd import driver as drvmod

    kw = dict(quant=quant, max_forward_tokens=208, total_pages=32)
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(93)
    prompt = rng.integers(0, cfg["vocab"], 230)
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        otoks, otrace = om.generate(prompt, 4, 1, want_logits=True)
        gtoks, _ = d.generate(prompt, 4, replicate=1)
        lg = d.export_tensor("debug.logits", np.uint16).reshape(-1, cfg["vocab"])[0]
        check_step(oracle, lg, otrace[3], gtoks[0, 3], otoks[0, 3]) if np.array_equal(gtoks[0, :3], otoks[0, :3]) else None
        # the first token comes straight out of the prefill
        o0 = oracle.bf16_to_f32(otrace[0])
        top2 = np.sort(o0)[-2:]
        if top2[1] - top2[0] > 2.0 ** -6 * abs(top2[1]) + 1e-6:
            assert int(gtoks[0, 0]) == int(otoks[0, 0])


def test_mixed_batch_prefill_plus_decode_and_kv_copy(gpu, oracle):
    """A decode request and a chunked prefill in one forward, then a forked context whose
    partially filled tail page is duplicated with Copy D2D."""
    from pie_amd import driver as drvmod

    kw = dict(quant="int4b8")
    cfg = full_cfg(**kw)
    ps = cfg["page_size"]
    rng = np.random.default_rng(91)
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        a = rng.integers(0, cfg["vocab"], 20)   # context A: pages 0,1
        b = rng.integers(0, cfg["vocab"], 9)    # context B: page 4
        fa = dict(token_ids=a, position_ids=np.arange(20), kv_page_indices=[0, 1],
                  kv_page_indptr=[0, 2], kv_last_page_lens=[4], qo_indptr=[0, 20])
        V = cfg["vocab"]

        def same(res, frame_args):
            """Tokens equal the oracle's unless its top-2 logits are a near-tie; logits close."""
            otok, olog, _ = om.forward(**frame_args, want_logits=True)
            glog = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
            assert len(res.tokens) == len(otok)
            for i in range(len(otok)):
                check_step(oracle, glog[i], olog[i], res.tokens[i], otok[i])
            return otok

        ra = d.forward(drvmod.ForwardFrame(**fa))
        same(ra, fa)
        # mixed: A decodes one token (position 20) while B prefills 9 tokens
        mixed = dict(token_ids=np.concatenate([[ra.tokens[0]], b]),
                     position_ids=np.concatenate([[20], np.arange(9)]),
                     kv_page_indices=[0, 1, 4], kv_page_indptr=[0, 2, 3], kv_last_page_lens=[5, 9],
                     qo_indptr=[0, 1, 10])
        rm = d.forward(drvmod.ForwardFrame(**mixed))
        assert rm.num_requests == 2
        same(rm, mixed)
        # fork A: share full page 0, copy tail page 1 -> page 7 (device-to-device)
        resp = d.handle(drvmod.copy_frame(2, [1], [7]))
        assert resp.payload.kind == drvmod.RESP_STATUS and resp.payload.status.status == 0
        for pool_k, pool_v in zip(om.k_pages, om.v_pages):
            pool_k[7] = pool_k[1]
            pool_v[7] = pool_v[1]
        fork = dict(token_ids=[rm.tokens[0], 77], position_ids=[21, 21],
                    kv_page_indices=[0, 1, 0, 7], kv_page_indptr=[0, 2, 4],
                    kv_last_page_lens=[6, 6], qo_indptr=[0, 1, 2])
        rf = d.forward(drvmod.ForwardFrame(**fork))
        same(rf, fork)
        # status codes of the copy path (driver/portable/src/service/inproc_service.cpp:82-203)
        assert d.handle(drvmod.copy_frame(2, [1], [999])).payload.status.status == 3
        assert d.handle(drvmod.copy_frame(2, [1, 2], [3])).payload.status.status == 5
        assert d.handle(drvmod.copy_frame(0, [1], [0])).payload.status.status == 4
        assert d.handle(drvmod.copy_frame(2, [1], [3], resource=1)).payload.status.status == 4
        health = drvmod.FrameDesc()
        health.payload.kind = drvmod.REQ_HEALTH
        assert d.handle(health).payload.status.status == 0
        bad = drvmod.FrameDesc()
        bad.payload.kind = 77
        assert d.handle(bad).payload.status.status == 2


def test_more_sampling_slots_than_rows(gpu):
    """A request may name the same row in many sampling slots (several samplers on one row, as
    the reference's planner allows, driver/portable/src/plan.cpp:224-470): the slot count then
    exceeds max_forward_tokens.  Every slot gets its row's greedy token, graphs and later
    ordinary batches keep working after the token buffers have grown."""
    from pie_amd import driver as drvmod

    kw = dict(quant="int4b8", max_forward_tokens=32, max_forward_requests=4)
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(95)
    prompt = rng.integers(0, cfg["vocab"], 9)
    with drvmod.Driver(toml_config(**kw)) as d:
        base = dict(token_ids=prompt, position_ids=np.arange(9), kv_page_indices=[2], kv_page_indptr=[0, 1],
                    kv_last_page_lens=[9], qo_indptr=[0, 9])
        plain = d.forward(drvmod.ForwardFrame(**base))
        # one decode step first, so a graph is cached before the buffers grow
        step = dict(token_ids=[plain.tokens[0]], position_ids=[9], kv_page_indices=[2], kv_page_indptr=[0, 1],
                    kv_last_page_lens=[10], qo_indptr=[0, 1])
        t_before = d.forward(drvmod.ForwardFrame(**step)).tokens
        slots = np.concatenate([np.full(70, 8), np.arange(9), np.full(21, 3)])   # 100 slots on 9 rows
        res = d.forward(drvmod.ForwardFrame(**base, sampling_indices=slots, sampling_indptr=[0, len(slots)]))
        assert res.num_requests == 1 and len(res.tokens) == len(slots)
        for i, row in enumerate(slots):
            assert res.tokens[i] == res.tokens[70 + row]          # same row, same token
        assert res.tokens[0] == plain.tokens[0]
        assert d.forward(drvmod.ForwardFrame(**step)).tokens == t_before   # the graph was rebuilt


def test_forward_failures_return_empty_response(gpu):
    from pie_amd import driver as drvmod

    with drvmod.Driver(toml_config()) as d:
        ok = dict(token_ids=[1], position_ids=[0], kv_page_indices=[0], kv_page_indptr=[0, 1],
                  kv_last_page_lens=[1], qo_indptr=[0, 1])
        # out-of-range page id, position past the context, a sampler kind that does not exist,
        # attention masks that are not one per token row
        for bad in (dict(kv_page_indices=[9999]), dict(position_ids=[5]),
                    dict(samplers=[dict(kind=11, temperature=0.8)], sampling_indices=[0],
                         sampling_indptr=[0, 1], sampler_indptr=[0, 1]),
                    dict(masks=[[0, 1], [0, 1]])):
            args = dict(ok)
            args.update(bad)
            res = d.forward(drvmod.ForwardFrame(**args))
            assert res.kind == drvmod.RESP_FORWARD and res.num_requests == 0 and res.tokens == []
        # empty batch: R empty per-request outputs
        res = d.forward(drvmod.ForwardFrame([], [], [], [0, 0, 0], [0, 0], [0, 0, 0],
                                            sampling_indices=[], sampling_indptr=[0, 0, 0],
                                            samplers=[], sampler_indptr=[0, 0, 0]))
        assert res.num_requests == 2 and res.tokens_indptr == [0, 0, 0]
        assert res.other_indptr_lens["dists_req_indptr"] == 3
        assert res.other_indptr_lens["dists_kv_indptr"] == 1
        # the driver still works afterwards
        assert d.forward(drvmod.ForwardFrame(**ok)).num_requests == 1


def test_run_inproc_serve_loop(gpu, tmp_path):
    """The exported serve loop: ready callback with capabilities, recv/send_response alternation,
    clean shutdown on recv = -1 — with Python callbacks playing the runtime."""
    import ctypes as C
    import json
    import threading

    from pie_amd import driver as drvmod

    cfg_path = tmp_path / "driver.toml"
    cfg_path.write_text(toml_config())
    frames = [drvmod.ForwardFrame([5], [0], [3], [0, 1], [1], [0, 1]),
              drvmod.ForwardFrame([6], [1], [3], [0, 1], [2], [0, 1])]
    health = drvmod.FrameDesc()
    health.payload.kind = drvmod.REQ_HEALTH
    queue = [frames[0].frame, health, frames[1].frame]
    got, caps = [], []
    state = dict(i=0)

    def recv(ctx, out_req, out_id):
        if state["i"] >= len(queue):
            return -1
        out_req[0] = C.pointer(queue[state["i"]])
        out_id[0] = 100 + state["i"]
        state["i"] += 1
        return 0

    def send(ctx, req_id, resp):
        r = resp.contents
        if r.payload.kind == drvmod.RESP_FORWARD:
            got.append((req_id, "fwd", r.payload.forward.num_requests,
                        [r.payload.forward.tokens.ptr[i] for i in range(r.payload.forward.tokens.len)]))
        else:
            got.append((req_id, "status", r.payload.status.status))

    vt = drvmod.InProcVTable(drvmod.RECV_FN(recv), drvmod.SEND_FN(send), None)
    ready = drvmod.READY_FN(lambda js, ctx: caps.append(json.loads(js.decode())))
    argv = (C.c_char_p * 3)(b"pie-driver-hip", b"--config", str(cfg_path).encode())
    rc = []
    th = threading.Thread(target=lambda: rc.append(
        drvmod.lib().pie_driver_hip_run_inproc(3, argv, 0, ready, None, vt)))
    th.start()
    th.join(timeout=120)
    assert not th.is_alive() and rc == [0]
    assert len(caps) == 1 and caps[0]["total_pages"] == 64 and caps[0]["arch_name"] == "llama3"
    assert [g[0] for g in got] == [100, 101, 102]
    assert got[0][1] == "fwd" and got[0][2] == 1 and len(got[0][3]) == 1
    assert got[1] == (101, "status", 0)
    assert got[2][1] == "fwd" and got[2][2] == 1
    # a missing config is an error return, not a crash
    argv2 = (C.c_char_p * 1)(b"pie-driver-hip")
    assert drvmod.lib().pie_driver_hip_run_inproc(1, argv2, 0, ready, None, vt) == -1


def _run_inproc_thread(drvmod, cfg_path, recv, send, on_ready):
    import ctypes as C
    import threading

    vt = drvmod.InProcVTable(drvmod.RECV_FN(recv), drvmod.SEND_FN(send), None)
    ready = drvmod.READY_FN(on_ready)
    argv = (C.c_char_p * 3)(b"pie-driver-hip", b"--config", str(cfg_path).encode())
    rc = []
    th = threading.Thread(target=lambda: rc.append(
        drvmod.lib().pie_driver_hip_run_inproc(3, argv, 0, ready, None, vt)))
    th.keep = (vt, ready, argv)   # the callbacks must outlive the call
    th.start()
    return th, rc


def test_request_stop_from_another_thread_ends_a_waiting_serve_loop(gpu, tmp_path):
    """pie_driver_hip_request_stop from a second thread while the loop waits in recv (a vtable
    whose recv times out with "nothing yet"): the loop returns 0 after the recv in progress,
    having answered what it was given before."""
    import ctypes as C
    import threading
    import time

    from pie_amd import driver as drvmod

    cfg_path = tmp_path / "driver.toml"
    cfg_path.write_text(toml_config())
    frame = drvmod.ForwardFrame([5], [0], [3], [0, 1], [1], [0, 1])
    pending, got, is_ready, polls = [frame.frame], [], threading.Event(), [0]

    def recv(ctx, out_req, out_id):
        if pending:
            out_req[0] = C.pointer(pending.pop(0))
            out_id[0] = 7
            return 0
        polls[0] += 1
        time.sleep(0.02)          # nothing yet: a null frame with status 0
        out_req[0] = None
        return 0

    def send(ctx, req_id, resp):
        got.append((req_id, resp.contents.payload.forward.num_requests))

    th, rc = _run_inproc_thread(drvmod, cfg_path, recv, send, lambda js, ctx: is_ready.set())
    assert is_ready.wait(timeout=120)
    while not got or polls[0] < 3:   # the request is answered and the loop is idling in recv
        time.sleep(0.01)
        assert th.is_alive()
    drvmod.lib().pie_driver_hip_request_stop()
    th.join(timeout=30)
    assert not th.is_alive() and rc == [0] and got == [(7, 1)]


def test_request_stop_during_model_load_is_not_lost(gpu, tmp_path):
    """A stop requested while the instance is still loading its model: the instance registers
    for stops before it loads, so it returns 0 after the ready handshake without a single recv."""
    import threading
    import time

    from pie_amd import driver as drvmod

    cfg_path = tmp_path / "driver.toml"
    # big enough that loading takes a moment: 8 layers of a 2048-wide model
    cfg_path.write_text(toml_config(hidden=2048, layers=8, q_heads=16, kv_heads=4, head_dim=128, intermediate=8192,
                                    vocab=32000))
    is_ready, recvs = threading.Event(), [0]

    def recv(ctx, out_req, out_id):
        recvs[0] += 1
        return -1

    th, rc = _run_inproc_thread(drvmod, cfg_path, recv, lambda *a: None, lambda js, ctx: is_ready.set())
    # stops in a tight loop from the moment the thread starts: the first one that finds the
    # instance registered arrives microseconds after its entry, long before the model is loaded
    stop = drvmod.lib().pie_driver_hip_request_stop
    t_end = time.time() + 120
    while th.is_alive() and time.time() < t_end:
        stop()
    th.join(timeout=1)
    assert not th.is_alive() and rc == [0]
    assert is_ready.is_set() and recvs[0] == 0


def test_custom_attention_masks_match_oracle(gpu, oracle):
    """Prefill and a decode step under per-token BRLE attention masks
    (build_attn_mask_f16, driver/portable/src/plan.cpp:54-94) against the oracle model."""
    from pie_amd import driver as drvmod

    kw = dict(quant="int8")
    cfg = full_cfg(**kw)
    V, ps = cfg["vocab"], cfg["page_size"]
    rng = np.random.default_rng(93)
    n = 45
    prompt = rng.integers(0, V, n)
    masks = []
    for i in range(n):
        if i % 4 == 0:
            masks.append([])                              # no runs: plain causal
        elif i % 4 == 1:
            masks.append([0, i + 1])                      # the synthesised causal shape
        else:
            a = int(rng.integers(0, i + 1))
            b = int(rng.integers(1, 8))
            masks.append([a, b, int(rng.integers(0, 5)), n])   # a hole pattern, clipped at i
    masks[7] = [0, 1, 100]                                # only key 0
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        npg = (n + ps - 1) // ps
        args = dict(token_ids=prompt, position_ids=np.arange(n), kv_page_indices=np.arange(npg),
                    kv_page_indptr=[0, npg], kv_last_page_lens=[n - (npg - 1) * ps], qo_indptr=[0, n],
                    sampling_indices=[n - 1, 7, 20], sampling_indptr=[0, 3])
        res = d.forward(drvmod.ForwardFrame(**args, masks=masks))
        assert res.num_requests == 1 and len(res.tokens) == 3
        otok, olog, _ = om.forward(**args, masks=masks, want_logits=True)
        glog = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
        for i in range(3):
            check_step(oracle, glog[i], olog[i], res.tokens[i], otok[i])
        masked_row7 = olog[1].copy()
        # a decode step that hides the first half of the context
        step = dict(token_ids=[int(res.tokens[0])], position_ids=[n], kv_page_indices=np.arange(npg),
                    kv_page_indptr=[0, npg], kv_last_page_lens=[n + 1 - (npg - 1) * ps], qo_indptr=[0, 1])
        m = [[n // 2, n]]
        res = d.forward(drvmod.ForwardFrame(**step, masks=m))
        otok, olog, _ = om.forward(**step, masks=m, want_logits=True)
        glog = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
        check_step(oracle, glog[0], olog[0], res.tokens[0], otok[0])
        # the masks matter: without them the oracle gives different logits on a masked row
        # (last: this run overwrites the oracle's KV pool)
        _, plain, _ = om.forward(**args, want_logits=True)
        assert cosine(oracle.bf16_to_f32(plain[1]), oracle.bf16_to_f32(masked_row7)) < 0.999


def test_host_swap_pool_round_trip(gpu, oracle):
    """Copy D2H / H2H / H2D of KV pages through the pinned swap pool
    (driver/portable/src/service/inproc_service.cpp:82-203): a context swapped out and back into
    other device pages decodes bit-identically; status codes of the error cases."""
    from pie_amd import driver as drvmod

    cfg = full_cfg(cpu_pages=4)
    ps, V = cfg["page_size"], cfg["vocab"]
    rng = np.random.default_rng(95)
    prompt = rng.integers(0, V, 27)          # pages 0 and 1
    with drvmod.Driver(toml_config(cpu_pages=4)) as d:
        assert d.capabilities()["swap_pool_size"] == 4
        t0 = d.forward(drvmod.ForwardFrame(prompt, np.arange(27), [0, 1], [0, 2], [11], [0, 27])).tokens[0]
        step = lambda pages: d.forward(drvmod.ForwardFrame([t0], [27], pages, [0, 2], [12], [0, 1]))
        status = lambda fr: d.handle(fr).payload.status.status
        assert status(drvmod.copy_frame(0, [0, 1], [2, 3])) == 0          # device 0,1 -> host 2,3
        assert status(drvmod.copy_frame(3, [2, 3], [0, 1])) == 0          # host 2,3 -> host 0,1
        assert status(drvmod.copy_frame(1, [0, 1], [5, 6])) == 0          # host 0,1 -> device 5,6
        a = step([0, 1])
        la = d.export_tensor("debug.logits", np.uint16)[:V].copy()
        # undo the decode write on the copy's source... the copies were taken before it: decode on them
        b = step([5, 6])
        lb = d.export_tensor("debug.logits", np.uint16)[:V].copy()
        assert a.tokens == b.tokens and np.array_equal(la, lb)
        assert status(drvmod.copy_frame(0, [0], [4])) == 3                # host slot out of range
        assert status(drvmod.copy_frame(1, [0], [9999])) == 3             # device page out of range
        assert status(drvmod.copy_frame(3, [0, 1], [2])) == 5             # length mismatch
    with drvmod.Driver(toml_config()) as d:                                # no pool
        for direction in (0, 1, 3):
            assert d.handle(drvmod.copy_frame(direction, [0], [0])).payload.status.status == 4


KV_FORMATS = ["fp8_e4m3", "int8_per_token_head", "fp8_per_token_head", "fp8_e5m2", "nvfp4", "fp4_e2m1"]


@pytest.mark.parametrize("kv_dtype", KV_FORMATS)
@pytest.mark.parametrize("kw", [dict(quant="int4b8"),
                                dict(arch="qwen3", quant="fp8", head_dim=128, q_heads=4, kv_heads=1,
                                     rope_theta=1e6, page_size=32)],
                         ids=["llama3", "qwen3"])
def test_generation_with_one_byte_kv_cache_matches_oracle(gpu, oracle, kw, kv_dtype):
    """[batching] kv_cache_dtype: K / V rows quantised at the write (kv_paged.cu:155-297) and
    read back as float(code) * scale; the oracle model does the same arithmetic on the CPU.
    Prefill (per-row attention over the one-byte pool), batched decode, graphs on.

    Bars: a 3-bit mantissa turns a one-bf16-step difference between the two implementations'
    K / V rows (summation order) into a whole code step (6-12 % of the element) wherever the
    value sits at a rounding boundary, so the logits agree less tightly than with a bf16 pool:
    cosine >= 0.998, 10 % of the largest logit, tokens compared where the oracle's top-2 gap
    exceeds 2^-4.  The arithmetic itself is pinned bit-exactly (write) and to the bf16-pool
    tolerance (attention over identical codes) in test_kv_quant_gpu.py."""
    from pie_amd import driver as drvmod

    kw = dict(kw, kv_cache_dtype=kv_dtype)
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(97)
    prompts = ragged_prompts(rng, cfg["vocab"], 37, 2)
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        # (e5m2 keeps two mantissa bits: a code step is twice as coarse, 12-25 % of the element,
        # so 1 - cosine — quadratic in the deviation — gets four times e4m3's allowance)
        # (the 4-bit block format keeps one mantissa bit: a code step is 25-50 % of the element;
        # another factor of four on 1 - cosine.  Its pages are expanded to bf16 before the
        # attention, as the reference does, and the oracle reads the same bf16(level * scale).)
        bars = dict(cos_min=0.992, rel=0.2, tie=2.0 ** -3) if kv_dtype == "fp8_e5m2" else \
            dict(cos_min=0.968, rel=0.4, tie=2.0 ** -2) if kv_dtype in ("nvfp4", "fp4_e2m1") else \
            dict(cos_min=0.998, rel=0.1, tie=2.0 ** -4)
        otoks, near, checks = teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, 8, **bars)
        # (the tiny model's logits are flat: most steps are near-ties at 2^-4, all of them at the
        # 4-bit format's 2^-2 — there every token is still held to the tied candidates)
        print(f"near-ties {near} of {checks} ({kv_dtype})")
        assert checks == 16 and (near <= (12 if kv_dtype == "fp8_e5m2" else 8) or kv_dtype in ("nvfp4", "fp4_e2m1"))
    with drvmod.Driver(toml_config(**kw)) as d:
        gtoks, _ = d.generate(prompts[0], 8, replicate=2)
        if near == 0:
            assert np.array_equal(gtoks[0], otoks[0])
        assert np.array_equal(gtoks[0], gtoks[1])


@pytest.mark.parametrize("kv_dtype", ["int8_per_token_head", "fp8_e4m3", "nvfp4"])
def test_page_copies_carry_one_byte_pages_and_their_scales(gpu, oracle, kv_dtype):
    """Device-to-device copies and the host swap pool move a page's codes and (per-token-head
    formats) its scales: a context copied to other pages decodes bit-identically."""
    from pie_amd import driver as drvmod

    kw = dict(cpu_pages=4, kv_cache_dtype=kv_dtype)
    cfg = full_cfg(**kw)
    V = cfg["vocab"]
    rng = np.random.default_rng(98)
    prompt = rng.integers(0, V, 27)          # pages 0 and 1
    with drvmod.Driver(toml_config(**kw)) as d:
        t0 = d.forward(drvmod.ForwardFrame(prompt, np.arange(27), [0, 1], [0, 2], [11], [0, 27])).tokens[0]
        step = lambda pages: d.forward(drvmod.ForwardFrame([t0], [27], pages, [0, 2], [12], [0, 1]))
        status = lambda fr: d.handle(fr).payload.status.status
        assert status(drvmod.copy_frame(2, [0, 1], [7, 8])) == 0          # device -> device
        assert status(drvmod.copy_frame(0, [0, 1], [2, 3])) == 0          # device -> host
        assert status(drvmod.copy_frame(3, [2, 3], [0, 1])) == 0          # host -> host
        assert status(drvmod.copy_frame(1, [0, 1], [5, 6])) == 0          # host -> device
        outs = []
        for pages in ([0, 1], [7, 8], [5, 6]):
            r = step(pages)
            outs.append((r.tokens, d.export_tensor("debug.logits", np.uint16)[:V].copy()))
        for tk, lg in outs[1:]:
            assert tk == outs[0][0] and np.array_equal(lg, outs[0][1])


@pytest.mark.parametrize("kv", ["fp8_per_token_head", "int8_per_token_head", "nvfp4"])
def test_custom_masks_over_a_one_byte_kv_cache_match_oracle(gpu, oracle, kv):
    """Per-token BRLE masks with one-byte KV pools: prefill rows and a decode step against the
    oracle model reading the same quantised values (the bars of the one-byte generation test)."""
    from pie_amd import driver as drvmod

    kw = dict(quant="int8", kv_cache_dtype=kv)
    cfg = full_cfg(**kw)
    V, ps = cfg["vocab"], cfg["page_size"]
    rng = np.random.default_rng(97)
    n = 37
    prompt = rng.integers(0, V, n)
    masks = []
    for i in range(n):
        if i % 3 == 0:
            masks.append([])                              # plain causal
        else:
            a = int(rng.integers(0, i + 1))
            masks.append([a, int(rng.integers(1, 8)), int(rng.integers(0, 5)), n])
    masks[5] = [0, 1, 100]                                # only key 0
    bars = dict(cos_min=0.968, rel=0.4, tie=2.0 ** -2) if kv == "nvfp4" else dict(cos_min=0.998, rel=0.1, tie=2.0 ** -4)
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        npg = (n + ps - 1) // ps
        args = dict(token_ids=prompt, position_ids=np.arange(n), kv_page_indices=np.arange(npg),
                    kv_page_indptr=[0, npg], kv_last_page_lens=[n - (npg - 1) * ps], qo_indptr=[0, n],
                    sampling_indices=[n - 1, 5, 20], sampling_indptr=[0, 3])
        res = d.forward(drvmod.ForwardFrame(**args, masks=masks))
        assert res.num_requests == 1 and len(res.tokens) == 3
        otok, olog, _ = om.forward(**args, masks=masks, want_logits=True)
        glog = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
        for i in range(3):
            check_step(oracle, glog[i], olog[i], res.tokens[i], otok[i], **bars)
        step = dict(token_ids=[int(otok[0])], position_ids=[n], kv_page_indices=np.arange(npg),
                    kv_page_indptr=[0, npg], kv_last_page_lens=[n + 1 - (npg - 1) * ps], qo_indptr=[0, 1])
        m = [[n // 2, n]]
        res = d.forward(drvmod.ForwardFrame(**step, masks=m))
        otok2, olog2, _ = om.forward(**step, masks=m, want_logits=True)
        glog2 = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
        check_step(oracle, glog2[0], olog2[0], res.tokens[0], otok2[0], **bars)
        # the mask matters: the unmasked step gives other logits
        res3 = d.forward(drvmod.ForwardFrame(**step))
        glog3 = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)
        assert cosine(oracle.bf16_to_f32(glog3[0]), oracle.bf16_to_f32(glog2[0])) < 0.9999


def test_unknown_kv_cache_dtypes_are_refused(gpu):
    from pie_amd import driver as drvmod

    for bad, msg in (("mxfp4", "invalid kv_cache_dtype"), ("turboquant", "invalid kv_cache_dtype")):
        with pytest.raises(Exception, match=msg):
            drvmod.Driver(toml_config(kv_cache_dtype=bad))


def test_raw_router_probabilities_match_oracle(gpu, oracle):
    """norm_topk = false (config.json norm_topk_prob): the chosen experts keep their softmax
    probabilities (driver/portable/src/graph_common.cpp:279-283 divides by their sum only under
    norm_topk).  Teacher-forced steps against the oracle run the same way, and the setting
    changes the logits."""
    from pie_amd import driver as drvmod

    kw = dict(arch="qwen3_moe", quant="bf16", head_dim=64, q_heads=8, kv_heads=2, num_experts=6, top_k=3,
              expert_intermediate=128, router_std=0.2, intermediate=0, model_extra="norm_topk = false\n")
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(97)
    prompts = ragged_prompts(rng, cfg["vocab"], 19, 2)
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        _, _, checks = teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, 6)
        assert checks == 12
        d.generate(prompts[0], 1, replicate=1)
        raw = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16)).astype(np.float64).ravel()
    with drvmod.Driver(toml_config(**dict(kw, model_extra=""))) as d:
        d.generate(prompts[0], 1, replicate=1)
        normed = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16)).astype(np.float64).ravel()
    assert raw.shape == normed.shape and not np.array_equal(raw, normed)


@pytest.mark.parametrize("kw", [dict(quant="int4b8"), dict(arch="qwen3", quant="bf16", head_dim=128, q_heads=4,
                                                           kv_heads=1, rope_theta=1e6)],
                         ids=["llama3-int4b8", "qwen3-bf16"])
def test_last_layer_intermediates_match_oracle(gpu, oracle, kw):
    """Beyond the logits: row 0 of the last layer's rotated queries, attention output, SwiGLU
    output and residual stream of a decode step against the oracle's (`orc_debug_capture`).
    Each is a bf16 vector a few rounding points downstream of identical inputs: cosine >= 0.9999
    and at most a few bf16 steps apart anywhere."""
    import ctypes as C
    from pie_amd import driver as drvmod

    cfg = full_cfg(**kw)
    ps = cfg["page_size"]
    rng = np.random.default_rng(95)
    prompt = rng.integers(0, cfg["vocab"], 19)
    H, I, QD = cfg["hidden"], cfg["intermediate"], cfg["q_heads"] * cfg["head_dim"]
    # (the attention rows are stored: no merge inside the output projection)
    with drvmod.Driver(toml_config(**kw, attn_merge_proj=False)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        n, npg = len(prompt), (len(prompt) + ps - 1) // ps
        fr = (prompt, np.arange(n), np.arange(npg), [0, npg], [n - (npg - 1) * ps], [0, n])
        tok = int(d.forward(drvmod.ForwardFrame(*fr)).tokens[0])
        assert int(om.forward(*fr)[0][0]) == tok
        step = ([tok], [n], np.arange(npg + 1)[: (n + ps) // ps], [0, (n + ps) // ps], [n + 1 - ((n + ps) // ps - 1) * ps], [0, 1])
        d.forward(drvmod.ForwardFrame(*step))
        got = {k: d.export_tensor("debug." + k, np.uint16) for k in ("q", "attn", "act", "x")}
        cap = dict(q=np.zeros(QD, np.uint16), attn=np.zeros(QD, np.uint16), act=np.zeros(I, np.uint16),
                   x=np.zeros(H, np.uint16))
        lib = oracle.lib()
        lib.orc_debug_capture(*[C.c_void_p(cap[k].ctypes.data) for k in ("q", "attn", "act", "x")])
        try:
            om.forward(*step)
        finally:
            lib.orc_debug_capture(None, None, None, None)
    for k in ("q", "attn", "act", "x"):
        g, o = oracle.bf16_to_f32(got[k][: len(cap[k])]), oracle.bf16_to_f32(cap[k])
        assert len(got[k]) == len(cap[k]) and np.any(o != 0), k
        assert cosine(g, o) >= 0.9999, (k, cosine(g, o))
        assert np.max(np.abs(g - o)) <= 2.0 ** -5 * np.max(np.abs(o)) + 1e-3, k


@pytest.mark.parametrize("kw", [dict(quant="int4b8"), dict(quant="int8", kv_cache_dtype="fp8_per_token_head"),
                                dict(arch="qwen3", quant="bf16", head_dim=128, q_heads=4, kv_heads=1, rope_theta=1e6)],
                         ids=["llama3-int4b8", "llama3-int8-fp8kv", "qwen3-bf16"])
def test_output_projection_that_merges_the_attention_splits_changes_no_bit(gpu, kw):
    """[runtime] attn_merge_proj: decode steps of one and of two rows give the same logits, bit for
    bit, with the merge inside the output projection (the default) and as a launch of its own."""
    from pie_amd import driver as drvmod

    cfg = full_cfg(**kw)
    ps = cfg["page_size"]
    rng = np.random.default_rng(96)
    prompts = [rng.integers(0, cfg["vocab"], n) for n in (37, 21)]
    logits = {}
    for merge in (True, False):
        rows = []
        with drvmod.Driver(toml_config(**kw, attn_merge_proj=merge, tune_linears=False)) as d:
            V = cfg["vocab"]
            pages, lens, toks = [], [], []
            nxt = 0
            for p in prompts:     # prefill one request at a time
                n, npg = len(p), (len(p) + ps - 1) // ps
                pg = np.arange(nxt, nxt + npg + 1)       # one spare page for the decode steps
                nxt += npg + 1
                t = int(d.forward(drvmod.ForwardFrame(p, np.arange(n), pg[:npg], [0, npg], [n - (npg - 1) * ps],
                                                      [0, n])).tokens[0])
                pages.append(pg)
                lens.append(n)
                toks.append(t)
            for nreq in (1, 2):   # a decode step of one row, then of two
                for _ in range(3):
                    tk, pos, pgl, indptr, last = [], [], [], [0], []
                    for r in range(nreq):
                        n = lens[r]
                        npg = (n + 1 + ps - 1) // ps
                        tk.append(toks[r]); pos.append(n)
                        pgl.extend(pages[r][:npg]); indptr.append(len(pgl)); last.append(n + 1 - (npg - 1) * ps)
                    out = d.forward(drvmod.ForwardFrame(tk, pos, pgl, indptr, last, list(range(nreq + 1))))
                    rows.append(d.export_tensor("debug.logits", np.uint16)[: nreq * V].copy())
                    for r in range(nreq):
                        toks[r] = int(out.tokens[r]); lens[r] += 1
        logits[merge] = rows
    assert len(logits[True]) == 6
    for a, b in zip(logits[True], logits[False]):
        assert np.any(a != 0) and np.array_equal(a, b)


@pytest.mark.parametrize("kw", [dict(quant="int4b8"), dict(quant="fp8"),
                                dict(arch="qwen3", quant="int4b8", head_dim=128, q_heads=4, kv_heads=1,
                                     rope_theta=1e6)], ids=["llama3-int4b8", "llama3-fp8", "qwen3-int4b8"])
@pytest.mark.parametrize("replicate", [3, 4, 7])
def test_small_decode_batches_match_oracle(gpu, oracle, kw, replicate):
    """Three, four and seven contexts with their own prompts and lengths: the rows where each
    linear is sent to the GEMV or to the skinny GEMM by cost (and the q|k|v epilogue changes
    kernels) against the oracle, every request of every step."""
    from pie_amd import driver as drvmod

    cfg = full_cfg(**kw)
    rng = np.random.default_rng(96)
    prompts = ragged_prompts(rng, cfg["vocab"], 13, replicate)
    with drvmod.Driver(toml_config(**kw, total_pages=96)) as d:
        om, _ = oracle_model_from_driver(d, dict(cfg, total_pages=96))
        _, near, checks = teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, 6)
        print(f"near-ties {near} of {checks}")
        assert checks == 6 * replicate and near <= checks // 5


@pytest.mark.parametrize("kw", [
    dict(quant="int4b8"),
    dict(quant="int4b8", kv_cache_dtype="fp8_per_token_head"),
    dict(arch="qwen3_moe", quant="fp8", head_dim=128, q_heads=8, kv_heads=1, num_experts=16, top_k=4,
         expert_intermediate=256, router_std=0.2, intermediate=0),
    dict(arch="qwen3_moe", quant="fp8", head_dim=128, q_heads=8, kv_heads=1, num_experts=16, top_k=4,
         expert_intermediate=256, router_std=0.2, intermediate=0, kv_cache_dtype="int8_per_token_head"),
], ids=["llama3-int4b8", "llama3-int4b8-fp8kv", "moe-fp8", "moe-fp8-int8kv"])
@pytest.mark.parametrize("count", [16, 64])
def test_decode_batches_of_16_and_64_distinct_requests(gpu, oracle, kw, count):
    """Decode batches of 16 and 64 requests, every request with its own prompt and context length
    (1 to 39 tokens at the first step): the 16-row skinny GEMM passes (one, and four side by
    side), the matrix-core decode attention over ragged contexts, the grouped expert GEMMs with
    64 x top-k routes — every request of every step against the oracle."""
    from pie_amd import driver as drvmod

    kw = dict(kw, total_pages=4 * count + 8, max_forward_requests=count, max_forward_tokens=128)
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(1000 + count)
    prompts = ragged_prompts(rng, cfg["vocab"], 13, count)
    bars = dict(cos_min=0.998, rel=0.1, tie=2.0 ** -4) if kw.get("kv_cache_dtype") else {}
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        _, near, checks = teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, 4, **bars)
        assert checks == 4 * count
        print(f"near-ties {near} of {checks}")
        # (one-byte KV pools: the quantisation noise is the margin, most steps count as near-ties
        # and are held to the tied candidates)
        if not cfg["num_experts"] and not kw.get("kv_cache_dtype"):
            assert near <= checks // 8


@pytest.mark.parametrize("kw", [dict(quant="int4b8"), dict(quant="bf16", kv_cache_dtype="int8_per_token_head"),
                                dict(arch="qwen3", quant="int8", head_dim=128, q_heads=4, kv_heads=1)],
                         ids=["llama3", "llama3-int8kv", "qwen3"])
def test_sliding_window_models_match_oracle(gpu, oracle, kw):
    """[model] sliding_window = W (Mistral-type checkpoints): a query at position p sees keys
    p - W + 1 .. p (driver/portable/src/plan.cpp:60-70).  Prefill rows and decode steps past the
    window against the oracle with the same window, and the window really hides the old keys
    (the logits differ from the full-context model's)."""
    from pie_amd import driver as drvmod

    W = 24
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(1200)
    prompt = rng.integers(0, cfg["vocab"], 41)
    ps, V = cfg["page_size"], cfg["vocab"]
    bars = dict(cos_min=0.998, rel=0.1, tie=2.0 ** -4) if kw.get("kv_cache_dtype") else {}
    # (the two drivers are compared bit for bit below: both dispatch by the cost model, not by their
    # own start-up measurements)
    with drvmod.Driver(toml_config(**kw, sliding_window=W, tune_linears=False)) as d, \
            drvmod.Driver(toml_config(**kw, tune_linears=False)) as full:
        om, _ = oracle_model_from_driver(d, cfg)
        n = len(prompt)
        npg = (n + ps - 1) // ps
        args = dict(token_ids=prompt, position_ids=np.arange(n), kv_page_indices=np.arange(npg), kv_page_indptr=[0, npg],
                    kv_last_page_lens=[n - (npg - 1) * ps], qo_indptr=[0, n], sampling_indices=[20, 30, n - 1],
                    sampling_indptr=[0, 3])
        res = d.forward(drvmod.ForwardFrame(**args))
        glog = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:3].copy()
        otok, olog, _ = om.forward(**args, want_logits=True, masks=[[]] * n, window=W)
        for i in range(3):
            check_step(oracle, glog[i], olog[i], res.tokens[i], otok[i], **bars)
        full.forward(drvmod.ForwardFrame(**args))
        flog = full.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:3]
        assert np.array_equal(flog[0], glog[0])                  # position 20: inside the window
        assert cosine(oracle.bf16_to_f32(flog[2]), oracle.bf16_to_f32(glog[2])) < 0.9999   # position 40: clipped
        tok = int(otok[2])
        for s in range(n, n + 4):
            npg = s // ps + 1
            step = dict(token_ids=[tok], position_ids=[s], kv_page_indices=np.arange(npg), kv_page_indptr=[0, npg],
                        kv_last_page_lens=[s + 1 - (npg - 1) * ps], qo_indptr=[0, 1])
            res = d.forward(drvmod.ForwardFrame(**step))
            lg = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[0]
            ot, ol, _ = om.forward(**step, want_logits=True, masks=[[]], window=W)
            check_step(oracle, lg, ol[0], res.tokens[0], ot[0], **bars)
            tok = int(ot[0])


def test_yarn_scaled_model_matches_oracle(gpu, oracle):
    """[model] rope_scaling = "yarn": the driver's frequency table equals the oracle's YaRN table,
    cos / sin carry the attention factor 0.1 ln(factor) + 1, and generation past the original
    context matches the oracle model (which rotates with the same table and factor)."""
    from pie_amd import driver as drvmod

    extra = 'rope_scaling = "yarn"\nrope_beta_fast = 8.0\nrope_beta_slow = 1.0\n'
    kw = dict(arch="qwen3", quant="int8", head_dim=128, q_heads=4, kv_heads=1, rope_theta=10000.0, rope_factor=4.0)
    cfg = full_cfg(**kw)
    rng = np.random.default_rng(1300)
    with drvmod.Driver(toml_config(**kw, model_extra=extra + "rope_original_max_pos = 16\n")) as d, \
            drvmod.Driver(toml_config(**dict(kw, rope_factor=0.0))) as plain:
        want = oracle.rope_inv_freq_yarn(128, 10000.0, 4.0, 8.0, 1.0, 16)
        got = d.export_tensor("inv_freq", np.float32)
        assert np.allclose(got, want, rtol=2e-6) and not np.allclose(got, plain.export_tensor("inv_freq", np.float32))
        ms = d.export_tensor("info.rope_mscale", np.float32)[0]
        assert abs(ms - (0.1 * np.log(4.0) + 1.0)) < 1e-6 and plain.export_tensor("info.rope_mscale", np.float32)[0] == 1.0
        om, _ = oracle_model_from_driver(d, cfg)
        assert om.cfg["rope_mscale"] == ms
        prompts = ragged_prompts(rng, cfg["vocab"], 40, 2)     # contexts beyond the original 16 positions
        _, near, checks = teacher_forced_compare(oracle, drvmod, d, om, cfg, prompts, 5)
        print(f"near-ties {near} of {checks}")
        assert checks == 10 and near <= 4


def test_start_up_warm_up_changes_no_result(gpu):
    """[runtime] warmup runs a synthetic chunk over unowned pages at start-up: with it on or off
    the same request gives the same tokens and the same logits, bit for bit (with the kernel per
    linear fixed by the cost model: the start-up measurement may pick another, see the next test)."""
    from pie_amd import driver as drvmod

    rng = np.random.default_rng(98)
    prompt = rng.integers(0, 2048, 23)
    outs = []
    for warm in (True, False):
        with drvmod.Driver(toml_config(warmup=warm, tune_linears=False)) as d:
            toks, _ = d.generate(prompt, 6, replicate=2)
            outs.append((toks.copy(), d.export_tensor("debug.logits", np.uint16).copy()))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])


def test_start_up_kernel_measurement_keeps_results_within_rounding(gpu, oracle):
    """[runtime] tune_linears times each decoder linear's candidate kernels at start-up and may route
    a row count to another kernel than the cost model: the kernels sum in different orders, so the
    logits agree to bf16 rounding (cosine, worst element), not bit for bit."""
    from pie_amd import driver as drvmod

    rng = np.random.default_rng(99)
    prompt = rng.integers(0, 2048, 19)
    outs = []
    for tune in (True, False):
        with drvmod.Driver(toml_config(tune_linears=tune)) as d:
            d.generate(prompt, 1, replicate=3)
            outs.append(oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16)).astype(np.float64).ravel())
            # the table the measurement left (what a deployment logs to know which kernels — and
            # so which rounding — this process runs): per linear and row count, -1 = cost model
            tab = d.export_tensor("info.tuned", np.int8).reshape(4, 129)
            assert np.all((tab >= -1) & (tab <= 3))
            if not tune:
                assert np.all(tab == -1)
            else:
                # llama-type q|k|v rows 2..4 always take the GEMV with the RoPE epilogue: not measured
                assert np.all(tab[0, 2:5] == -1) and np.all(tab[:, 5:17] == -1)
    a, b = outs
    assert a.shape == b.shape and cosine(a, b) > 0.9995
    assert np.max(np.abs(a - b)) <= 0.05 * np.max(np.abs(b)) + 1e-3
