"""CPU pins for the oracle's sampler suite (oracle/src/sampler.c): the published PCG32 sequence,
scipy closed forms, limits that reduce to argmax, hand-worked prefixes, sample frequencies."""
import numpy as np
import pytest
import scipy.special
import scipy.stats


def test_pcg32_matches_the_published_demo_sequence(oracle):
    # pcg32_srandom_r(&rng, 42u, 54u) of the PCG reference implementation (the first sequence pcg32-demo prints)
    want = [0xa15c02b7, 0x7b47f409, 0xba1d3330, 0x83d2f293, 0xbfa4784b, 0xcbed606e]
    assert [int(x) for x in oracle.pcg32_sequence(42, 54, 6)] == want


def test_first_uniform_is_the_top_24_bits_of_the_default_stream(oracle):
    for seed in (1, 7, 123456789, 2**32 - 1):
        first = int(oracle.pcg32_sequence(seed, 0xda3e39cb94b95bdb, 1)[0])
        u = oracle.pcg32_first_uniform(seed)
        assert u == (first >> 8) / 2.0**24 and 0.0 <= u < 1.0


def test_softmax_matches_scipy(oracle):
    rng = np.random.default_rng(1)
    lg = (rng.standard_normal(5000) * 4).astype(np.float32)
    for t in (0.3, 1.0, 2.5):
        p = oracle.softmax_temperature(lg, t)
        ref = scipy.special.softmax(lg.astype(np.float64) / t)
        assert np.allclose(p, ref, rtol=2e-6, atol=1e-12)
        assert abs(float(p.astype(np.float64).sum()) - 1.0) < 1e-5


def test_limits_that_reduce_to_argmax(oracle):
    rng = np.random.default_rng(2)
    lg = rng.standard_normal(3000).astype(np.float32)
    best = int(np.argmax(lg))
    for kind in ("multinomial", "top_k", "top_p", "min_p", "top_k_top_p"):
        assert oracle.sample_token(lg, kind, temperature=0.0, u=0.9)[0] == best
    for u in (0.0, 0.3, 0.999):
        assert oracle.sample_token(lg, "top_k", 1.0, top_k=1, u=u)[0] == best
        assert oracle.sample_token(lg, "top_p", 1.0, top_p=1e-9, u=u)[0] == best
        assert oracle.sample_token(lg, "min_p", 1.0, min_p=1.0, u=u)[0] == best
        assert oracle.sample_token(lg, "top_k_top_p", 1.0, top_k=5, top_p=0.0, u=u)[0] == best
    # first index wins an exact tie of the maximum
    tie = lg.copy()
    tie[[17, 900]] = 50.0
    assert oracle.sample_token(tie, "top_p", 0.0)[0] == 17


def logits_for(probs):
    return np.log(np.asarray(probs, np.float64)).astype(np.float32)


def test_hand_worked_prefixes(oracle):
    # probabilities 0.4 0.3 0.2 0.1 at ids 2 0 3 1
    lg = logits_for([0.3, 0.1, 0.4, 0.2])
    # top-p 0.65: prefix {0.4, 0.3} (0.7 >= 0.65), renormalised boundary at 4/7
    assert oracle.sample_token(lg, "top_p", 1.0, top_p=0.65, u=0.50)[0] == 2
    assert oracle.sample_token(lg, "top_p", 1.0, top_p=0.65, u=0.60)[0] == 0
    assert oracle.sample_token(lg, "top_p", 1.0, top_p=0.65, u=0.999)[0] == 0
    # top-p 0.75 takes a third entry
    assert oracle.sample_token(lg, "top_p", 1.0, top_p=0.75, u=0.999)[0] == 3
    # top-k 3 drops id 1 whatever u
    assert oracle.sample_token(lg, "top_k", 1.0, top_k=3, u=0.9999)[0] == 3
    assert oracle.sample_token(lg, "top_k", 1.0, top_k=0, u=0.9999)[0] == 1      # 0 = no cap
    # min-p 0.6: threshold 0.24 keeps {0.4, 0.3}
    assert oracle.sample_token(lg, "min_p", 1.0, min_p=0.6, u=0.999)[0] == 0
    # top-k 3 then top-p 0.95 over the *unrenormalised* prefix sums 0.4, 0.7, 0.9 -> all three
    assert oracle.sample_token(lg, "top_k_top_p", 1.0, top_k=3, top_p=0.95, u=0.999)[0] == 3
    # multinomial walks in index order: cumulative 0.3 0.4 0.8 1.0
    assert [oracle.sample_token(lg, "multinomial", 1.0, u=u)[0] for u in (0.1, 0.35, 0.5, 0.9)] == [0, 1, 2, 3]
    # equal probabilities: ascending id
    eq = logits_for([0.25, 0.25, 0.25, 0.25])
    assert [oracle.sample_token(eq, "top_k", 1.0, top_k=2, u=u)[0] for u in (0.2, 0.7)] == [0, 1]


def test_margin_reports_the_distance_to_the_decision(oracle):
    lg = logits_for([0.3, 0.1, 0.4, 0.2])
    tok, mg = oracle.sample_token(lg, "multinomial", 1.0, u=0.35)
    assert tok == 1 and abs(mg - 0.05) < 1e-6
    tok, mg = oracle.sample_token(lg, "top_p", 1.0, top_p=0.65, u=0.1)
    assert tok == 2 and abs(mg - 0.05) < 1e-6      # 0.7 - 0.65 decides the prefix


@pytest.mark.parametrize("kind,kw", [("multinomial", {}), ("top_k", {"top_k": 6}),
                                     ("top_p", {"top_p": 0.8}), ("min_p", {"min_p": 0.2})])
def test_sample_frequencies_follow_the_kept_distribution(oracle, kind, kw):
    rng = np.random.default_rng(5)
    V, T = 12, 0.9
    lg = rng.standard_normal(V).astype(np.float32) * 1.5
    p = scipy.special.softmax(lg.astype(np.float64) / T)
    order = np.argsort(-p, kind="stable")
    keep = np.ones(V, bool)
    if kind == "top_k":
        keep[:] = False
        keep[order[:6]] = True
    elif kind == "top_p":
        cut = int(np.searchsorted(np.cumsum(p[order]), 0.8)) + 1
        keep[:] = False
        keep[order[:cut]] = True
    elif kind == "min_p":
        keep = p >= 0.2 * p.max()
    q = np.where(keep, p, 0.0)
    q /= q.sum()
    n = 20000
    counts = np.zeros(V)
    for s in range(1, n + 1):
        counts[oracle.sample_token(lg, kind, T, seed=s, **kw)[0]] += 1
    assert np.all(counts[~keep] == 0)
    chi2 = float((((counts - n * q) ** 2)[keep] / (n * q[keep])).sum())
    assert chi2 < scipy.stats.chi2.ppf(0.9999, int(keep.sum()) - 1)


def test_distribution_is_the_sorted_head_of_the_softmax(oracle):
    rng = np.random.default_rng(6)
    lg = rng.standard_normal(400).astype(np.float32) * 2
    p = scipy.special.softmax(lg.astype(np.float64) / 0.7)
    order = np.argsort(-p, kind="stable")
    ids, vals = oracle.distribution(lg, 0.7, 10)
    assert list(ids) == list(order[:10]) and np.allclose(vals, p[order[:10]], rtol=3e-6)
    ids, vals = oracle.distribution(lg, 0.7, 0)       # 0 = the whole vocabulary
    assert list(ids) == list(order) and abs(float(vals.sum()) - 1.0) < 1e-5


def test_logprobs_and_entropy_match_scipy(oracle):
    rng = np.random.default_rng(7)
    lg = rng.standard_normal(6000).astype(np.float32) * 3
    ls = scipy.special.log_softmax(lg.astype(np.float64))
    labels = [0, 5999, 17, 17, 4242]
    assert np.allclose(oracle.logprobs_at(lg, labels), ls[labels], rtol=0, atol=2e-6)
    assert abs(oracle.entropy(lg) - float(-(np.exp(ls) * ls).sum())) < 1e-5
    assert abs(oracle.entropy(np.zeros(4096, np.float32)) - np.log(4096)) < 1e-5
    with pytest.raises(ValueError):
        oracle.logprobs_at(lg, [6000])


def test_brle_logit_mask(oracle):
    lg = np.arange(10, dtype=np.float32)
    assert np.array_equal(oracle.apply_brle_logit_mask(lg, []), lg)          # empty = no constraint
    # runs alternate false/true starting with false; past the last run everything is masked
    out = oracle.apply_brle_logit_mask(lg, [2, 3, 1, 2])
    allowed = np.array([0, 0, 1, 1, 1, 0, 1, 1, 0, 0], bool)
    assert np.array_equal(np.isneginf(out), ~allowed) and np.array_equal(out[allowed], lg[allowed])
    # a leading zero-length false run (the shape the runtime emits for "first n allowed")
    out = oracle.apply_brle_logit_mask(lg, [0, 4])
    assert np.array_equal(np.isneginf(out), np.arange(10) >= 4)
    # runs longer than the vocabulary are clipped
    out = oracle.apply_brle_logit_mask(lg, [1, 100])
    assert np.array_equal(np.isneginf(out), np.arange(10) < 1)
    # a masked vocabulary still samples inside the allowed set
    tok, _ = oracle.sample_token(oracle.apply_brle_logit_mask(lg, [7, 2]), "top_p", 1.0, top_p=0.99, u=0.5)
    assert tok in (7, 8)
