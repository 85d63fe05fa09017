"""GPU parity: device samplers through the C ABI vs the CPU oracle's restatement of the
reference's host sampler suite (driver/portable/src/sampler.cpp).

Tokens must equal the oracle's whenever the oracle's decision margin (distance of the deciding
comparison from its flipping point, in probability mass) exceeds TOL; the reference accumulates
its running sums sequentially in float, the kernel in double per 64 entries, and expf differs
in the last bit, so draws inside the margin may legitimately fall on the neighbouring token.
"""
import numpy as np
import pytest

from gpu_util import dev

pytestmark = pytest.mark.gpu

TOL = 3e-5   # probability mass; sequential float sums over <= 128k entries stay well inside


def make_logits(oracle, rng, S, V, scales):
    lg = rng.standard_normal((S, V)).astype(np.float32) * np.asarray(scales, np.float32)[:, None]
    bits = oracle.f32_to_bf16(lg)
    return bits, oracle.bf16_to_f32(bits)


def random_slots(rng, S):
    kinds = rng.choice(["multinomial", "top_k", "top_p", "min_p", "top_k_top_p"], size=S)
    temp = rng.choice([0.0, 0.6, 1.0, 1.7], size=S, p=[0.1, 0.3, 0.4, 0.2]).astype(np.float32)
    top_k = rng.choice([0, 1, 5, 50, 300], size=S).astype(np.uint32)
    top_p = rng.choice([0.3, 0.8, 0.95, 1.0], size=S).astype(np.float32)
    min_p = rng.choice([0.0, 0.05, 0.3], size=S).astype(np.float32)
    seeds = rng.integers(1, 2**32, size=S)
    return list(kinds), temp, top_k, top_p, min_p, seeds


@pytest.mark.parametrize("V", [1000, 32000, 128256])
def test_token_samplers_match_oracle(gpu, oracle, V):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(900 + V)
    S = 48 if V < 100000 else 24
    # flat rows (token mass near TOL) cannot be told apart from rounding; keep them a minority
    scales = rng.choice([0.7, 2.0, 5.0] if V <= 1000 else [3.0, 5.0, 8.0], size=S)
    bits, lg = make_logits(oracle, rng, S, V, scales)
    kinds, temp, top_k, top_p, min_p, seeds = random_slots(rng, S)
    u = np.array([oracle.pcg32_first_uniform(int(s)) for s in seeds], np.float32)
    f32 = ops.sample_gather_logits(dev(bits, gpu, torch.bfloat16))
    assert np.array_equal(f32.cpu().numpy(), lg)
    tokens, _, _, _ = ops.sample(f32, kinds, temp, top_k, top_p, min_p, u)
    torch.cuda.synchronize()
    got = tokens.cpu().numpy().view(np.uint32)
    near = 0
    for s in range(S):
        want, margin = oracle.sample_token(lg[s], kinds[s], float(temp[s]), int(top_k[s]),
                                           float(top_p[s]), float(min_p[s]), u=float(u[s]))
        if margin > TOL:
            assert got[s] == want, (s, kinds[s], temp[s], top_k[s], top_p[s], min_p[s], margin)
        else:
            near += 1
    assert near <= S // 4, near


@pytest.mark.parametrize("V", [32000, 128256])
def test_few_slots_take_the_many_block_front_end(gpu, oracle, V):
    """Calls of at most sixteen slots over a wide vocabulary run the row-wide passes over many
    blocks per slot before the one block per slot: the same slots sampled eight and one at a time
    give the tokens the oracle gives, and the tokens of a 24-slot call (one block per slot alone)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(905 + V)
    S = 24
    scales = rng.choice([3.0, 5.0, 8.0], size=S)
    bits, lg = make_logits(oracle, rng, S, V, scales)
    kinds, temp, top_k, top_p, min_p, seeds = random_slots(rng, S)
    u = np.array([oracle.pcg32_first_uniform(int(s)) for s in seeds], np.float32)
    f32 = ops.sample_gather_logits(dev(bits, gpu, torch.bfloat16))
    whole = ops.sample(f32, kinds, temp, top_k, top_p, min_p, u)[0].cpu().numpy().view(np.uint32)
    chunks = [(i, i + 8) for i in range(0, S, 8)] + [(i, i + 1) for i in range(5)]
    for lo, hi in chunks:
        sl = slice(lo, hi)
        got = ops.sample(f32[sl].contiguous(), kinds[sl], temp[sl], top_k[sl], top_p[sl], min_p[sl], u[sl])[0]
        got = got.cpu().numpy().view(np.uint32)
        assert np.array_equal(got, whole[sl]), (lo, hi)
        for s in range(lo, hi):
            want, margin = oracle.sample_token(lg[s], kinds[s], float(temp[s]), int(top_k[s]),
                                               float(top_p[s]), float(min_p[s]), u=float(u[s]))
            if margin > TOL:
                assert got[s - lo] == want, (s, kinds[s], temp[s], top_k[s], top_p[s], min_p[s], margin)


def test_sorted_order_and_rows_argument(gpu, oracle):
    """Rows picked out of a larger logits matrix; top_k = 1 / tiny top_p / min_p = 1 / T = 0 all
    reduce to the first-index argmax, also with an exact tie of the maximum."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(910)
    V = 5000
    bits, lg = make_logits(oracle, rng, 9, V, [3.0] * 9)
    lg[4, [77, 4000]] = 30.0
    bits = oracle.f32_to_bf16(lg)
    rows = np.array([4, 0, 8, 4, 2], np.int32)
    f32 = ops.sample_gather_logits(dev(bits, gpu, torch.bfloat16), rows=dev(rows, gpu))
    assert np.array_equal(f32.cpu().numpy(), lg[rows])
    kinds = ["top_k", "top_p", "min_p", "multinomial", "top_k_top_p"]
    temp = [1.0, 1.0, 1.0, 0.0, 1.0]
    tokens, _, _, _ = ops.sample(f32, kinds, temp, [1, 0, 0, 0, 7], [1.0, 1e-9, 1.0, 1.0, 0.0],
                                 [0.0, 0.0, 1.0, 0.0, 0.0], [0.99, 0.5, 0.7, 0.3, 0.9])
    got = tokens.cpu().numpy()
    assert list(got) == [int(np.argmax(lg[r])) for r in rows] and got[0] == 77 and got[3] == 77


def test_brle_logit_masks(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(911)
    V = 3000
    bits, lg = make_logits(oracle, rng, 5, V, [2.0] * 5)
    runs = [[], [0, 10], [100, 50, 7, 1, 2000, 3], [5, 5000], [V, 0]]
    f32 = ops.sample_gather_logits(dev(bits, gpu, torch.bfloat16), mask_runs=runs)
    got = f32.cpu().numpy()
    for s in range(5):
        assert np.array_equal(got[s], oracle.apply_brle_logit_mask(lg[s], runs[s])), s
    # sampling under a mask stays inside it and equals the oracle on the masked row
    kinds = ["top_p"] * 5
    u = [0.1, 0.5, 0.9, 0.3, 0.7]
    tokens, _, _, _ = ops.sample(f32, kinds, [1.0] * 5, [0] * 5, [0.9] * 5, [0.0] * 5, u)
    tok = tokens.cpu().numpy()
    for s in range(4):
        want, margin = oracle.sample_token(got[s], "top_p", 1.0, top_p=0.9, u=u[s])
        assert margin <= TOL or tok[s] == want
        assert np.isfinite(got[s, tok[s]])
    assert tok[4] == 0            # everything masked: no positive probability, token 0


@pytest.mark.parametrize("V", [4096, 128256])
def test_special_samplers_match_oracle(gpu, oracle, V):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(920 + V)
    S = 6
    bits, lg = make_logits(oracle, rng, S, V, [1.0, 3.0, 6.0, 2.0, 4.0, 0.5])
    kinds = ["dist", "dist", "logprob", "logprobs", "entropy", "raw_logits"]
    temp = [0.8, 1.0, 1.0, 1.0, 1.0, 1.0]
    ks = [20, 0]
    labels = [None, None, [int(rng.integers(V))], [int(x) for x in rng.integers(0, V, 7)], None, None]
    counts = [ks[0], V, 1, 7, 1, 0]
    f32 = ops.sample_gather_logits(dev(bits, gpu, torch.bfloat16))
    _, values, ids, indptr = ops.sample(f32, kinds, temp, [ks[0], ks[1], 0, 0, 0, 0], [1.0] * S,
                                        [0.0] * S, [0.0] * S, out_counts=counts, labels=labels)
    torch.cuda.synchronize()
    values, ids = values.cpu().numpy(), ids.cpu().numpy().view(np.uint32)
    for s in (0, 1):
        v, i = values[indptr[s]:indptr[s + 1]], ids[indptr[s]:indptr[s + 1]]
        wi, wv = oracle.distribution(lg[s], temp[s], ks[s])
        assert len(v) == len(wv) and np.allclose(v, wv, rtol=2e-6, atol=1e-30)
        assert np.all(v[:-1] >= v[1:]) and len(set(i.tolist())) == len(i)
        p = oracle.softmax_temperature(lg[s], temp[s])
        assert np.allclose(p[i], v, rtol=2e-6, atol=1e-30)       # each id carries its own probability
        same = wi == i                                          # order may differ only inside ties
        assert np.all(same | np.isclose(p[wi], p[i], rtol=4e-7, atol=1e-30))
    for s in (2, 3):
        got = values[indptr[s]:indptr[s + 1]]
        assert np.allclose(got, oracle.logprobs_at(lg[s], labels[s]), rtol=0, atol=2e-5)
    assert abs(values[indptr[4]] - oracle.entropy(lg[4])) < 2e-5 * max(1.0, oracle.entropy(lg[4]))
    with pytest.raises(ops.KernelError):
        ops.sample(f32[:1], ["logprob"], [1.0], [0], [1.0], [0.0], [0.0], out_counts=[1], labels=[[V]])


@pytest.mark.parametrize("slots", [1, 3])
def test_multinomial_draw_exactly_on_a_part_boundary(gpu, oracle, slots):
    """The many-block front end picks the part from the parts' sums and walks inside it.  Rows
    whose probabilities are exact binary fractions (64 equal logits, everything else masked to
    -inf) make every cumulative sum exact, so a uniform placed exactly on the cumulative mass at
    the end of a part must yield the first allowed token of the following part (rule: first
    index whose running sum exceeds u) — never a masked token, never the greedy fallback."""
    import torch
    from pie_amd import ops

    V, parts = 32768, 32
    seg = V // parts
    allowed = np.sort(np.concatenate([np.arange(parts) * seg + 5, np.arange(parts) * seg + seg - 3]))
    lg = np.full((slots, V), -np.inf, np.float32)
    lg[:, allowed] = 1.5
    f32 = dev(lg, gpu)
    cases = [(j, 2 * j / 64.0) for j in (1, 7, 31)] + [(None, 0.0), (None, 63.0 / 64.0), (None, 13.0 / 64.0)]
    for j, u in cases:
        uu = np.full(slots, u, np.float32)
        tok = ops.sample(f32, ["multinomial"] * slots, np.ones(slots, np.float32), np.zeros(slots, np.uint32),
                         np.ones(slots, np.float32), np.zeros(slots, np.float32), uu)[0]
        got = tok.cpu().numpy().view(np.uint32)
        want = allowed[int(np.floor(u * 64.0 + 1e-9))]      # cumulative (m + 1)/64 first exceeds u
        if j is not None:
            assert want == j * seg + 5                       # the first allowed token of part j
        assert np.all(got == want), (u, got, want)
        ref, _ = oracle.sample_token(lg[0], "multinomial", 1.0, 0, 1.0, 0.0, u=float(u))
        assert ref == want


@pytest.mark.parametrize("V", [32000, 128256])
def test_tokens_against_the_reference_build(gpu, oracle, V):
    """The device samplers against the reference's own sample_token, compiled from its sources
    (oracle/_ref): every draw must name the reference's token, another member of its group of
    bit-equal probabilities (the reference's sort leaves their order open), or — for draws
    whose deciding comparison lies within TOL of flipping — a neighbouring token; the three
    counts are printed."""
    import torch
    from oracle import ref
    from pie_amd import ops

    if ref.lib() is None:
        pytest.skip("no prebuilt oracle/_ref library on this machine")
    rng = np.random.default_rng(930 + V)
    S = 192 if V < 100000 else 64
    bits, lg = make_logits(oracle, rng, S, V, rng.choice([2.0, 3.0, 5.0, 8.0], size=S))
    kinds, temp, top_k, top_p, min_p, seeds = random_slots(rng, S)
    u = np.array([oracle.pcg32_first_uniform(int(s)) for s in seeds], np.float32)
    f32 = ops.sample_gather_logits(dev(bits, gpu, torch.bfloat16))
    got = np.concatenate([ops.sample(f32[i:i + 64], kinds[i:i + 64], temp[i:i + 64], top_k[i:i + 64],
                                     top_p[i:i + 64], min_p[i:i + 64], u[i:i + 64])[0].cpu().numpy().view(np.uint32)
                          for i in range(0, S, 64)])
    same = tie = near = 0
    for s in range(S):
        want = ref.sample_token(lg[s], kinds[s], float(temp[s]), int(top_k[s]), float(top_p[s]),
                                float(min_p[s]), int(seeds[s]))
        if got[s] == want:
            same += 1
            continue
        pr = oracle.softmax_temperature(lg[s], float(temp[s]))
        if pr[got[s]] == pr[want]:
            tie += 1
            continue
        _, margin = oracle.sample_token(lg[s], kinds[s], float(temp[s]), int(top_k[s]), float(top_p[s]),
                                        float(min_p[s]), u=float(u[s]))
        assert margin <= TOL, (s, kinds[s], temp[s], top_k[s], top_p[s], min_p[s], got[s], want, margin)
        near += 1
    print(f"V {V}: {same} draws equal to the reference's token, {tie} on another member of a group of equal "
          f"probabilities, {near} on a neighbour inside the decision margin, of {S}")
    assert near <= S // 16
