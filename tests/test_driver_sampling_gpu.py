"""End-to-end GPU parity of the response half of the boundary: every sampler kind, BRLE logit
masks and speculative-draft verification through the driver, against the oracle's restatement
of the reference's host sampler applied to the driver's own logits."""
import numpy as np
import pytest

from driver_util import full_cfg, toml_config

pytestmark = pytest.mark.gpu

K = dict(multinomial=0, top_k=1, top_p=2, min_p=3, top_k_top_p=4, dist=6, raw=7, logprob=8,
         logprobs=9, entropy=10)
TOL = 3e-5


def prefill_args(prompt, ps, first_page=0):
    n = len(prompt)
    npg = (n + ps - 1) // ps
    return dict(token_ids=prompt, position_ids=np.arange(n), kv_page_indices=np.arange(npg) + first_page,
                kv_page_indptr=[0, npg], kv_last_page_lens=[n - (npg - 1) * ps], qo_indptr=[0, n])


def test_every_sampler_kind_on_one_position(gpu, oracle):
    from pie_amd import driver as drvmod

    cfg = full_cfg(vocab=4096)
    V = cfg["vocab"]
    rng = np.random.default_rng(71)
    prompt = rng.integers(0, V, 23)
    labels = [int(x) for x in rng.integers(0, V, 5)]
    samplers = [
        dict(kind=K["top_p"], temperature=0.0, p=1.0),                  # greedy
        dict(kind=K["raw"]),
        dict(kind=K["dist"], temperature=0.7, num_tokens=6),
        dict(kind=K["logprob"], token_id=labels[0]),
        dict(kind=K["logprobs"], token_ids=labels),
        dict(kind=K["entropy"]),
        dict(kind=K["top_k"], temperature=1.3, k=40, seed=11),
        dict(kind=K["min_p"], temperature=1.0, p=0.1, seed=12),
        dict(kind=K["multinomial"], temperature=2.0, seed=13),
        dict(kind=K["top_k_top_p"], temperature=1.5, k=100, p=0.9, seed=14),
    ]
    n = len(samplers)
    with drvmod.Driver(toml_config(vocab=V)) as d:
        args = prefill_args(prompt, cfg["page_size"])
        res = d.forward(drvmod.ForwardFrame(**args, sampling_indices=[len(prompt) - 1] * n,
                                            sampling_indptr=[0, n], samplers=samplers,
                                            sampler_indptr=[0, n]))
        assert res.num_requests == 1
        bits = d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[0]
        lg = oracle.bf16_to_f32(bits)
        raw = res.logits_of(0)
        assert len(raw) == 1 and np.array_equal(raw[0], lg)          # native f32 bytes of the row
        (ids, probs), = res.dists_of(0)
        wi, wp = oracle.distribution(lg, 0.7, 6)
        assert list(ids) == list(wi) and np.allclose(probs, wp, rtol=2e-6)
        lp = res.logprobs_of(0)
        assert len(lp) == 2 and len(lp[0]) == 1 and len(lp[1]) == 5
        assert np.allclose(lp[0], oracle.logprobs_at(lg, labels[:1]), atol=2e-5)
        assert np.allclose(lp[1], oracle.logprobs_at(lg, labels), atol=2e-5)
        ent, = res.entropies_of(0)
        assert abs(ent - oracle.entropy(lg)) < 2e-5 * max(1.0, oracle.entropy(lg))
        toks = res.tokens_of(0)
        assert len(toks) == 5 and toks[0] == int(np.argmax(lg))
        want = [("top_k", dict(temperature=1.3, top_k=40), 11), ("min_p", dict(temperature=1.0, min_p=0.1), 12),
                ("multinomial", dict(temperature=2.0), 13),
                ("top_k_top_p", dict(temperature=1.5, top_k=100, top_p=0.9), 14)]
        for got, (kind, kw, seed) in zip(toks[1:], want):
            tok, margin = oracle.sample_token(lg, kind, seed=seed, **kw)
            assert margin <= TOL or got == tok, (kind, got, tok, margin)
        # the same seeds give the same tokens again; the CSR shapes follow the response builder
        res2 = d.forward(drvmod.ForwardFrame(**args, sampling_indices=[len(prompt) - 1] * n,
                                             sampling_indptr=[0, n], samplers=samplers,
                                             sampler_indptr=[0, n]))
        assert res2.tokens == res.tokens
        assert res.dists_req_indptr == [0, 1] and res.dists_kv_indptr == [0, 6]
        assert res.logits_req_indptr == [0, 1] and res.logits_byte_indptr == [0, 4 * V]
        assert res.logprobs_req_indptr == [0, 2] and res.logprobs_val_indptr == [0, 1, 6]
        assert res.entropies_indptr == [0, 1] and res.tokens_indptr == [0, 5]


def test_embedding_slots_are_accepted_and_yield_nothing(gpu):
    """Wire sampler kind 5 (Embedding) has no field in the forward response; the reference's
    executor emits nothing for such a slot (driver/portable/src/executor/executor.cpp:1367-1392,
    default arm) and answers the others.  Same here: the request succeeds, the slots around the
    Embedding slot give what they give without it."""
    from pie_amd import driver as drvmod

    cfg = full_cfg(vocab=4096)
    V = cfg["vocab"]
    rng = np.random.default_rng(72)
    prompt = rng.integers(0, V, 17)
    greedy = dict(kind=K["top_p"], temperature=0.0, p=1.0)
    with drvmod.Driver(toml_config(vocab=V)) as d:
        args = prefill_args(prompt, cfg["page_size"])
        last = len(prompt) - 1
        plain = d.forward(drvmod.ForwardFrame(**args, sampling_indices=[last, last], sampling_indptr=[0, 2],
                                              samplers=[greedy, dict(kind=K["entropy"])], sampler_indptr=[0, 2]))
        res = d.forward(drvmod.ForwardFrame(**args, sampling_indices=[last, last, last], sampling_indptr=[0, 3],
                                            samplers=[greedy, dict(kind=5), dict(kind=K["entropy"])],
                                            sampler_indptr=[0, 3]))
        assert res.num_requests == 1 and plain.num_requests == 1
        assert res.tokens_of(0) == plain.tokens_of(0) and len(res.tokens_of(0)) == 1
        assert res.entropies_of(0) == plain.entropies_of(0) and len(res.entropies_of(0)) == 1
        assert not res.dists_of(0) and not res.logits_of(0) and not res.logprobs_of(0)
        only = d.forward(drvmod.ForwardFrame(**args, sampling_indices=[last], sampling_indptr=[0, 1],
                                             samplers=[dict(kind=5)], sampler_indptr=[0, 1]))
        assert only.num_requests == 1 and only.tokens_of(0) == []


def test_sampled_decode_batch_under_graphs_and_logit_masks(gpu, oracle):
    """Four contexts decode with different samplers (one constrained by a BRLE logit mask, one
    greedy); the decode body replays from its HIP graph, the samplers run after it."""
    from pie_amd import driver as drvmod

    cfg = full_cfg(vocab=4096)
    V, ps = cfg["vocab"], cfg["page_size"]
    rng = np.random.default_rng(72)
    prompt = rng.integers(0, V, 19)
    with drvmod.Driver(toml_config(vocab=V)) as d:
        ppc = 4
        for c in range(4):
            d.forward(drvmod.ForwardFrame(**prefill_args(prompt, ps, first_page=c * ppc)))
        allowed_lo, allowed_n = 1000, 24
        for step in range(3):
            pos = len(prompt) + step
            npg = (pos + 1 + ps - 1) // ps
            samplers = [dict(kind=K["top_p"], temperature=0.9, p=0.95, seed=100 + step),
                        dict(kind=K["top_k"], temperature=1.1, k=50, seed=200 + step),
                        dict(kind=K["top_p"], temperature=0.0, p=1.0),
                        dict(kind=K["min_p"], temperature=1.0, p=0.05, seed=300 + step)]
            fr = drvmod.ForwardFrame(
                [5 + step] * 4, [pos] * 4, np.concatenate([np.arange(npg) + c * ppc for c in range(4)]),
                np.arange(5) * npg, [pos + 1 - (npg - 1) * ps] * 4, np.arange(5),
                sampling_indices=[0] * 4, sampling_indptr=np.arange(5), samplers=samplers,
                sampler_indptr=np.arange(5), logit_masks=[[allowed_lo, allowed_n]],
                logit_mask_indptr=[0, 0, 1, 1, 1])      # request 1 only
            res = d.forward(fr)
            assert res.num_requests == 4 and res.tokens_indptr == [0, 1, 2, 3, 4]
            lg = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:4])
            masked = oracle.apply_brle_logit_mask(lg[1], [allowed_lo, allowed_n])
            checks = [("top_p", dict(temperature=0.9, top_p=0.95), 100 + step, lg[0]),
                      ("top_k", dict(temperature=1.1, top_k=50), 200 + step, masked),
                      ("top_p", dict(temperature=0.0), 1, lg[2]),
                      ("min_p", dict(temperature=1.0, min_p=0.05), 300 + step, lg[3])]
            for r, (kind, kw, seed, row) in enumerate(checks):
                tok, margin = oracle.sample_token(row, kind, seed=seed, **kw)
                assert margin <= TOL or res.tokens[r] == tok, (step, r, res.tokens[r], tok, margin)
            assert allowed_lo <= res.tokens[1] < allowed_lo + allowed_n


def test_speculative_drafts_are_verified(gpu, oracle):
    """Greedy verification of two drafts (the walk of resolve_request_output,
    driver/portable/src/executor/executor.cpp:204-248): the accepted prefix plus one token."""
    from pie_amd import driver as drvmod

    cfg = full_cfg()
    V, ps = cfg["vocab"], cfg["page_size"]
    rng = np.random.default_rng(73)
    prompt = rng.integers(0, V, 13)
    n = len(prompt)

    def run(drafts):
        with drvmod.Driver(toml_config()) as d:
            t0 = d.forward(drvmod.ForwardFrame(**prefill_args(prompt, ps))).tokens[0]
            truth = [t0]
            if drafts is None:        # plain greedy decode, one token per step
                for s in range(3):
                    pos = n + s
                    npg = (pos + 1 + ps - 1) // ps
                    truth.append(d.forward(drvmod.ForwardFrame(
                        [truth[-1]], [pos], np.arange(npg), [0, npg], [pos + 1 - (npg - 1) * ps], [0, 1])).tokens[0])
                return truth
            d1, d2 = drafts
            toks = [t0, d1, d2]                     # rows at positions n, n+1, n+2
            npg = (n + 3 + ps - 1) // ps
            res = d.forward(drvmod.ForwardFrame(
                toks, [n, n + 1, n + 2], np.arange(npg), [0, npg], [n + 3 - (npg - 1) * ps], [0, 3],
                sampling_indices=[0], sampling_indptr=[0, 1],
                samplers=[dict(kind=K["top_p"], temperature=0.0, p=1.0)], sampler_indptr=[0, 1],
                spec_token_ids=[d1, d2], spec_position_ids=[n + 1, n + 2], spec_indptr=[0, 2]))
            assert res.num_requests == 1
            return res.tokens_of(0)

    truth = run(None)                               # t0, t1, t2, t3
    t1, t2, t3 = truth[1:]
    assert run((t1, t2)) == [t1, t2, t3]            # both accepted + bonus
    wrong = (t2 + 1) % V
    assert run((t1, wrong)) == [t1, t2]             # second rejected: the model's token replaces it
    assert run(((t1 + 1) % V, t2)) == [t1]          # first rejected
