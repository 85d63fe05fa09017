"""Pins for the oracle's MoE functions (CPU only): routing against numpy float64 softmax and a
stable argsort, constructed ties, closed forms; the combine against a float64 weighted sum; the
MoE decoder forward against an independent dense fp64 transformer."""
import numpy as np
import pytest

from test_oracle_model import DenseRef, make_tensors


def test_topk_softmax_matches_float64_softmax_and_stable_argsort(oracle):
    rng = np.random.default_rng(400)
    for E, K in [(128, 8), (8, 2), (384, 6), (5, 5)]:
        logits = oracle.f32_to_bf16(rng.standard_normal((33, E)).astype(np.float32) * 2)
        idx, w = oracle.topk_softmax(logits, K)
        lf = oracle.bf16_to_f32(logits).astype(np.float64)
        p = np.exp(lf - lf.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        ref_idx = np.argsort(-p, axis=1, kind="stable")[:, :K]
        assert np.array_equal(idx, ref_idx)          # bf16 logits: distinct values or exact ties
        ref_w = np.take_along_axis(p, ref_idx, 1)
        ref_w /= ref_w.sum(axis=1, keepdims=True)
        assert np.allclose(w, ref_w, rtol=2e-6, atol=1e-9)
        assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)
        # norm_topk = false (driver/portable/src/graph_common.cpp:279-283): the same experts, their
        # softmax probabilities undivided
        idx_raw, w_raw = oracle.topk_softmax(logits, K, renorm=False)
        assert np.array_equal(idx_raw, ref_idx)
        assert np.allclose(w_raw, np.take_along_axis(p, ref_idx, 1), rtol=2e-6, atol=1e-9)
        if K < E:
            assert np.all(w_raw.sum(axis=1) < 1.0)


def test_topk_softmax_ties_go_to_the_lowest_index_and_closed_form(oracle):
    # all logits equal: the first K experts, weight 1/K each
    idx, w = oracle.topk_softmax(oracle.f32_to_bf16(np.full((2, 16), 0.75, np.float32)), 4)
    assert np.array_equal(idx, np.tile(np.arange(4), (2, 1))) and np.allclose(w, 0.25)
    # two tied maxima at 5 and 9, then a tie at 1 and 2
    lg = np.zeros((1, 12), np.float32)
    lg[0, [5, 9]] = 3.0
    lg[0, [1, 2]] = 1.0
    idx, w = oracle.topk_softmax(oracle.f32_to_bf16(lg), 3)
    assert idx.tolist() == [[5, 9, 1]]
    e3, e1 = np.exp(3.0), np.exp(1.0)
    assert np.allclose(w[0], np.array([e3, e3, e1]) / (2 * e3 + e1), rtol=1e-6)
    # logits 0,1,2,3 top-2: weights sigmoid(1), 1 - sigmoid(1)
    idx, w = oracle.topk_softmax(oracle.f32_to_bf16(np.arange(4, dtype=np.float32)[None]), 2)
    assert idx.tolist() == [[3, 2]]
    assert np.allclose(w[0], [1 / (1 + np.exp(-1.0)), 1 / (1 + np.exp(1.0))], rtol=1e-6)


def test_moe_combine_matches_float64_weighted_sum(oracle):
    rng = np.random.default_rng(401)
    N, K, H = 5, 8, 64
    yr = oracle.f32_to_bf16(rng.standard_normal((N * K, H)).astype(np.float32))
    w = rng.dirichlet(np.ones(K), N).astype(np.float32)
    res = oracle.f32_to_bf16(rng.standard_normal((N, H)).astype(np.float32))
    ref = (w.astype(np.float64)[:, :, None] * oracle.bf16_to_f32(yr).astype(np.float64).reshape(N, K, H)).sum(1)
    for base in (None, res):
        got = oracle.bf16_to_f32(oracle.moe_combine(yr, w, base)).astype(np.float64)
        want = ref + (oracle.bf16_to_f32(base).astype(np.float64) if base is not None else 0.0)
        want_b = oracle.bf16_to_f32(oracle.f32_to_bf16(want.astype(np.float32))).astype(np.float64)
        # one bf16 rounding of an fp32 sum: equal to the rounded float64 sum except at rounding
        # boundaries, never more than one bf16 step away
        assert (got == want_b).mean() > 0.99
        assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30)
    # one-hot weights select a route exactly
    w1 = np.zeros((N, K), np.float32)
    w1[np.arange(N), rng.integers(0, K, N)] = 1.0
    sel = oracle.moe_combine(yr, w1)
    assert np.array_equal(sel, yr.reshape(N, K, H)[np.arange(N), w1.argmax(1)])


@pytest.mark.parametrize("quant", ["bf16", "int8", "int4b8"])
def test_oracle_moe_forward_matches_dense_fp64(oracle, quant):
    from oracle.model import OracleModel

    cfg = dict(hidden=128, layers=2, q_heads=4, kv_heads=2, head_dim=32, intermediate=0, vocab=200,
               rms_eps=1e-5, rope_interleaved=0, qk_norm=True, quant=quant, group_size=64,
               page_size=4, total_pages=16, num_experts=6, top_k=2, expert_intermediate=64)
    rng = np.random.default_rng(402)
    t = make_tensors(oracle, rng, cfg)
    om = OracleModel(cfg, t)
    ref = DenseRef(oracle, cfg, t)
    prompt = rng.integers(0, cfg["vocab"], 9)
    toks, logits, _ = om.forward(prompt, np.arange(9), [3, 7, 1], [0, 3], [1], [0, 9],
                                 sampling_indices=np.arange(9), sampling_indptr=[0, 9],
                                 want_logits=True)
    good = 0
    for i, tk in enumerate(prompt):
        ref.min_gap = 1.0
        rl = ref.step(int(tk), i)
        if ref.min_gap < 0.004:
            continue   # a routing near-tie: the bf16 path may legitimately pick another expert
        lo = oracle.bf16_to_f32(logits[i]).astype(np.float64)
        assert lo @ rl / (np.linalg.norm(lo) * np.linalg.norm(rl)) >= 0.9995, i
        good += 1
    assert good >= 5


@pytest.mark.parametrize("quant", ["bf16", "fp8", "int4b8"])
def test_truth_mode_moe_forward_equals_dense_fp64(oracle, quant):
    """The double-precision forward over MoE layers (router softmax, top-k with the lowest index
    on ties, renormalised weights, unrounded expert sums) is the numpy fp64 transformer to
    summation-order accuracy — no routing near-tie can separate two fp64 evaluations here."""
    from oracle.model import OracleModel

    cfg = dict(hidden=128, layers=2, q_heads=4, kv_heads=2, head_dim=32, intermediate=0, vocab=200,
               rms_eps=1e-5, rope_interleaved=0, qk_norm=True, quant=quant, group_size=64,
               page_size=4, total_pages=16, num_experts=6, top_k=3, expert_intermediate=64)
    rng = np.random.default_rng(404)
    t = make_tensors(oracle, rng, cfg)
    om, ref = OracleModel(cfg, t), DenseRef(oracle, cfg, t)
    prompt = rng.integers(0, cfg["vocab"], 9)
    args = dict(token_ids=prompt, position_ids=np.arange(9), kv_page_indices=[3, 7, 1], kv_page_indptr=[0, 3],
                kv_last_page_lens=[1], qo_indptr=[0, 9], sampling_indices=np.arange(9), sampling_indptr=[0, 9])
    toks, logits, _ = om.forward_hp("f64", **args)
    _, lp, _ = om.forward_hp("P", **args)
    for i, tk in enumerate(prompt):
        ref.min_gap = 1.0
        rl = ref.step(int(tk), i)
        assert ref.min_gap > 1e-9
        assert np.max(np.abs(logits[i] - rl)) <= 1e-9 * np.max(np.abs(rl)), i
        assert int(toks[i]) == int(np.argmax(rl))
        if ref.min_gap > 1e-4:   # F32 / F16 noise cannot flip a router decision this wide
            assert lp[i] @ rl / (np.linalg.norm(lp[i]) * np.linalg.norm(rl)) >= 0.99999, i


def test_router_gap_reports_the_selection_margin(oracle):
    """router_gap() = (last chosen - first rejected router logit) / the token's largest logit
    magnitude, minimum over layers and tokens.  Router rows c_e * u with c = +-powers of two make
    every logit an exact multiple c_e * (u . x): whatever x is (either sign of u . x), the margin
    between the 2nd and 3rd is exactly 1/4 of the largest; identical rows give 0; a dense model
    reports no margin at all."""
    from oracle.model import OracleModel

    cfg = dict(hidden=128, layers=2, q_heads=4, kv_heads=2, head_dim=32, intermediate=0, vocab=200,
               rms_eps=1e-5, rope_interleaved=0, qk_norm=True, quant="bf16", group_size=64,
               page_size=4, total_pages=16, num_experts=6, top_k=2, expert_intermediate=64)
    rng = np.random.default_rng(403)
    t = make_tensors(oracle, rng, cfg)
    u = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal(128).astype(np.float32)))
    c = np.array([4, 2, 1, -1, -2, -4], np.float32)
    for l in range(2):
        t[f"layers.{l}.router"] = oracle.f32_to_bf16(c[:, None] * u[None, :])
    om = OracleModel(cfg, t)
    prompt = rng.integers(0, cfg["vocab"], 5)
    om.forward(prompt, np.arange(5), [3, 7], [0, 2], [1], [0, 5])
    assert om.router_gap() == 0.25
    for l in range(2):
        t[f"layers.{l}.router"] = oracle.f32_to_bf16(np.tile(u, (6, 1)))
    om = OracleModel(cfg, t)
    om.forward(prompt, np.arange(5), [3, 7], [0, 2], [1], [0, 5])
    assert om.router_gap() == 0.0
    toks = om.generate(prompt, 3)
    assert len(om.last_router_gaps) == 3 and toks.shape == (1, 3)

    dense = dict(cfg, num_experts=0, top_k=0, expert_intermediate=0, intermediate=64)
    od = OracleModel(dense, make_tensors(oracle, rng, dense))
    od.forward(prompt, np.arange(5), [3, 7], [0, 2], [1], [0, 5])
    assert od.router_gap() > 1e30
