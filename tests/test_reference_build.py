"""The oracle's sampler and BRLE restatements against the reference's OWN code: oracle/build_ref.py
compiles driver/portable/src/sampler.cpp and driver/cuda/src/brle.cpp from the reference tree (with
an extern "C" shim of ours in front) into oracle/_ref/.  Skipped where neither that library nor the
reference tree exists.

What "equal" means for tokens: the reference orders candidates with std::sort / std::partial_sort,
which leave the order of equal probabilities unspecified, and bf16 logits make exactly equal
probabilities common; the oracle orders them by ascending token id.  A draw that lands inside a
group of bit-equal probabilities may therefore name another member of the group — and nothing
else may differ."""
import subprocess

import numpy as np
import pytest


@pytest.fixture(scope="module")
def ref(oracle):
    from oracle import ref as r

    if r.lib() is None:
        pytest.skip("no reference tree and no prebuilt oracle/_ref library")
    return r


def _rows(oracle, rng, S, V, bf16=True):
    lg = (rng.standard_normal((S, V)) * rng.choice([0.7, 2.0, 5.0, 8.0], size=(S, 1))).astype(np.float32)
    return oracle.bf16_to_f32(oracle.f32_to_bf16(lg)) if bf16 else lg


def test_reference_brle_unit_test_passes(ref):
    from oracle import build_ref

    if not build_ref.BRLE_TEST.exists():
        pytest.skip("reference test binary not built")
    proc = subprocess.run([str(build_ref.BRLE_TEST)], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0, proc.stdout + proc.stderr


@pytest.mark.parametrize("V,bf16", [(1000, True), (32000, True), (32000, False), (128256, True)])
def test_sample_token_equals_the_reference_except_inside_groups_of_equal_probability(oracle, ref, V, bf16):
    rng = np.random.default_rng(4100 + V + bf16)
    S = 160 if V <= 32000 else 40
    rows = _rows(oracle, rng, S, V, bf16)
    kinds = ["multinomial", "top_k", "top_p", "min_p", "top_k_top_p"]
    same = tie = 0
    for s in range(S):
        kind = kinds[s % 5]
        T = float(rng.choice([0.0, 0.6, 1.0, 1.7]))
        k = int(rng.choice([0, 1, 5, 50, 300]))
        p = float(rng.choice([0.3, 0.8, 0.95, 1.0]))
        mp = float(rng.choice([0.0, 0.05, 0.3]))
        seed = int(rng.integers(1, 2 ** 32))
        want = ref.sample_token(rows[s], kind, T, k, p, mp, seed)
        got, _ = oracle.sample_token(rows[s], kind, T, k, p, mp, seed=seed)   # u from the oracle's PCG32
        if got == want:
            same += 1
            continue
        pr = oracle.softmax_temperature(rows[s], T)
        assert kind != "multinomial", "the unsorted walk has no tie order to differ in"
        assert pr[got] == pr[want], (s, kind, T, k, p, mp, got, want, pr[got], pr[want])
        tie += 1
    print(f"V {V} bf16 {bf16}: {same} equal tokens, {tie} other members of a group of equal probabilities, "
          f"of {S} draws")
    if not bf16:
        assert tie <= S // 20       # float32 logits rarely collide


@pytest.mark.parametrize("scale", [8.0, 3.0, 1.0])
def test_where_the_batch_shortcut_of_the_reference_departs_from_its_full_rule(oracle, ref, scale):
    """For batches whose slots share one temperature the reference downloads the 256 most probable
    tokens per slot and finishes on the host (executor.cpp:586-629, sample_token_from_topk); this
    driver applies the full-vocabulary rule (sample_token) to every batch.  Both are the
    reference's own code here: they give the same token whenever the full rule keeps at most 256
    candidates (peaked rows: practically always), and differ only where the shortcut truncated —
    counted and printed per logit scale."""
    rng = np.random.default_rng(4150 + int(scale * 10))
    V, S = 32000, 150
    lg = oracle.bf16_to_f32(oracle.f32_to_bf16((rng.standard_normal((S, V)) * scale).astype(np.float32)))
    kinds = ["top_k", "top_p", "min_p", "top_k_top_p"]
    same = truncated = tie = 0
    for s in range(S):
        kind = kinds[s % 4]
        T = float(rng.choice([0.6, 1.0]))
        k = int(rng.choice([0, 5, 50, 200]))
        p = float(rng.choice([0.8, 0.95]))
        mp = float(rng.choice([0.02, 0.1]))
        seed = int(rng.integers(1, 2 ** 32))
        full = ref.sample_token(lg[s], kind, T, k, p, mp, seed)
        ids, vals = ref.distribution(lg[s], T, 256)            # the reference's softmax + top-256, descending
        short = ref.sample_token_from_topk(ids, vals, kind, T, k, p, mp, seed)
        # how many candidates the full rule keeps (float running sums, as apply_top_p / apply_min_p)
        pr = np.sort(oracle.softmax_temperature(lg[s], T))[::-1]
        pr = pr[pr > 0]
        keep = len(pr)
        if kind in ("top_k", "top_k_top_p") and 0 < k < keep:
            keep = k
        if kind in ("top_p", "top_k_top_p") and p < 1.0:
            cum = np.cumsum(pr[:keep], dtype=np.float32)
            hit = np.nonzero(cum >= np.float32(p))[0]
            keep = int(hit[0]) + 1 if len(hit) else keep
        if kind == "min_p":
            cut = int(np.sum(pr[:keep] >= np.float32(mp) * pr[0]))
            keep = cut if cut > 0 else keep
        if full == short:
            same += 1
        elif keep > 256:
            truncated += 1
        else:
            # (the two paths sort with partial_sort / sort over different ranges: equal probabilities
            # may come out in another order)
            prob = oracle.softmax_temperature(lg[s], T)
            assert prob[full] == prob[short], (s, kind, T, k, p, mp, keep, full, short)
            tie += 1
    print(f"logit scale {scale}: shortcut = full rule on {same} of {S} draws, {truncated} differ because the full "
          f"rule keeps more than 256 candidates, {tie} inside a group of equal probabilities")
    if scale >= 8.0:
        assert truncated <= S // 10


def test_temperature_zero_is_first_index_argmax(oracle, ref):
    rng = np.random.default_rng(4200)
    row = _rows(oracle, rng, 1, 5000)[0]
    row[[17, 900, 4000]] = row.max() + 1.0       # three tied maxima: the lowest index wins
    for kind in ("multinomial", "top_k", "top_p", "min_p", "top_k_top_p"):
        assert ref.sample_token(row, kind, 0.0, 5, 0.5, 0.1, 7) == 17
        assert oracle.sample_token(row, kind, 0.0, 5, 0.5, 0.1, seed=7)[0] == 17


@pytest.mark.parametrize("T", [0.5, 1.0, 2.5])
def test_distribution_logprobs_entropy_and_logit_mask_are_bit_equal(oracle, ref, T):
    rng = np.random.default_rng(4300 + int(T * 10))
    V = 20000
    row = _rows(oracle, rng, 1, V)[0]
    # full distribution (k = 0) = the softmax itself: values bit-equal, ids equal where unique
    ids_r, vals_r = ref.distribution(row, T, 0)
    ids_o, vals_o = oracle.distribution(row, T, 0)
    assert np.array_equal(vals_r, vals_o)
    uniq = np.concatenate([[True], vals_r[1:] != vals_r[:-1]]) & np.concatenate([vals_r[1:] != vals_r[:-1], [True]])
    assert np.array_equal(ids_r[uniq], ids_o[uniq])
    assert np.array_equal(np.sort(ids_r), np.arange(V))
    pr = oracle.softmax_temperature(row, T)
    assert np.array_equal(pr[ids_r], vals_r)          # softmax_with_temperature, bit for bit
    ids_r, vals_r = ref.distribution(row, T, 25)
    ids_o, vals_o = oracle.distribution(row, T, 25)
    assert np.array_equal(vals_r, vals_o)
    labels = rng.integers(0, V, 9)
    assert np.array_equal(ref.logprobs_at(row, labels), oracle.logprobs_at(row, labels))
    assert np.array_equal(ref.logprobs_at(row, labels[:1]), oracle.logprobs_at(row, labels[:1]))
    assert ref.entropy(row) == oracle.entropy(row)
    with pytest.raises(ValueError):
        ref.logprobs_at(row, [V])
    for runs in ([], [0, V], [5, 10, 100, 7], [0, 3, V * 2], [V + 5], [10, 0, 10, 5], [1] * 301):
        a, b = ref.apply_brle_logit_mask(row, runs), oracle.apply_brle_logit_mask(row, runs)
        assert np.array_equal(a, b), runs


def _random_runs(rng, limit):
    """BRLE runs (false, true, false, ...) whose total stays within `limit` keys."""
    runs, left = [], limit
    for _ in range(int(rng.integers(0, 7))):
        n = int(rng.integers(0, max(left, 0) + 1))
        runs.append(n)
        left -= n
    return runs


@pytest.mark.parametrize("page_size", [16, 4])
def test_attention_mask_decode_matches_the_oracle_visibility(oracle, ref, page_size):
    """brle::decode (the CUDA driver's packed qo x kv bitmap per request) against orc_brle_allow
    (the portable driver's mask builder, which also applies the causal limit): for runs that stay
    within a token's causal extent the two must agree bit for bit; a true run reaching past the
    token's own position is cut by the causal limit in the oracle (and in the kernels), as
    driver/portable/src/plan.cpp:54-94 does, while the bitmap keeps it."""
    rng = np.random.default_rng(4400 + page_size)
    for trial in range(40):
        R = int(rng.integers(1, 5))
        qo, kp, kl, masks, mi, toks = [0], [0], [], [], [0], []
        for r in range(R):
            kv_len = int(rng.integers(1, 70))
            qo_len = int(rng.integers(1, min(kv_len, 9) + 1))
            npg = (kv_len + page_size - 1) // page_size
            qo.append(qo[-1] + qo_len)
            kp.append(kp[-1] + npg)
            kl.append(kv_len - (npg - 1) * page_size)
            for q in range(qo_len):
                pos = kv_len - qo_len + q
                runs = _random_runs(rng, pos + 1) or [0, pos + 1]
                masks += runs
                mi.append(len(masks))
                toks.append((r, q, pos, kv_len, runs))
        packed, indptr, pure = ref.brle_decode(masks, mi, qo, kp, kl, page_size)
        for r, q, pos, kv_len, runs in toks:
            bits = np.unpackbits(packed[indptr[r]:indptr[r + 1]], bitorder="little")
            row = bits[q * kv_len:(q + 1) * kv_len]
            assert np.array_equal(row, oracle.brle_allow(runs, pos, kv_len)), (trial, r, q, runs)
        causal = all(runs == [0, pos + 1] for _, _, pos, _, runs in toks)
        assert pure == causal == ref.brle_is_pure_causal(masks, mi, qo, kp, kl, page_size)
    # a true run past the token's position: the bitmap keeps it, the causal limit cuts it
    packed, indptr, _ = ref.brle_decode([0, 8], [0, 2], [0, 1], [0, 1], [8], 16)
    assert np.unpackbits(packed, bitorder="little")[:8].tolist() == [1] * 8
    assert oracle.brle_allow([0, 8], 4, 8).tolist() == [1, 1, 1, 1, 1, 0, 0, 0]
    with pytest.raises(ValueError):
        ref.brle_decode([0, 1], [0, 5], [0, 1], [0, 1], [1], 16)      # indptr past the run array
