"""Planner parity on the CPU: the oracle planner is pinned by the reference's wire-layout
known answers and brute force; the driver's C++ planner (host-only entry point of
libpie_driver_hip.so, no GPU call) must agree with it bit-exactly, including its error
behaviour."""
import numpy as np
import pytest

from oracle import planner as op


def brute_slot(pages, ps, pos):
    """Independent statement: lay the request's pages out as one long row of slots."""
    flat = [int(p) * ps + s for p in pages for s in range(ps)]
    return flat[pos]


def test_oracle_known_answer_causal_decode():
    # runtime/src/inference/request.rs:810-830: decode at position 47, page_size 16,
    # pages [100,101,102], last_page_len 16.
    p = op.plan_forward([999], [47], [100, 101, 102], [0, 3], [16], [0, 1], [0], [0, 1], 16, 4096)
    assert p["seq_len"] == [48] and p["row_kv_len"] == [48] and p["max_kv_len"] == 48
    assert p["kv_slots"] == [102 * 16 + 15] and p["row_page_begin"] == [0]
    assert p["sample_rows"] == [0] and p["pure_decode"]


def test_oracle_physical_idx_brute_force():
    rng = np.random.default_rng(70)
    for ps in (4, 16, 32):
        pages = rng.permutation(50)[:7]
        for pos in range(7 * ps):
            assert op.physical_idx(pages, 0, ps, pos) == brute_slot(pages, ps, pos)
        # with an offset into a longer concatenated list
        cat = np.concatenate([rng.permutation(50)[:3], pages])
        assert op.physical_idx(cat, 3, ps, 2 * ps + 1) == brute_slot(pages, ps, 2 * ps + 1)


def test_oracle_prefill_rows_and_sampling():
    # two requests: a 5-token chunk appended to 6 cached tokens, and a 3-token fresh prefill
    p = op.plan_forward([1, 2, 3, 4, 5, 6, 7, 8], [6, 7, 8, 9, 10, 0, 1, 2],
                        [9, 4, 7, 2], [0, 3, 4], [3, 3], [0, 5, 8], [4, 1, 2], [0, 1, 3], 4, 16)
    assert p["seq_len"] == [11, 3] and not p["pure_decode"]
    assert p["row_kv_len"] == [7, 8, 9, 10, 11, 1, 2, 3]
    assert p["row_page_begin"] == [0] * 5 + [3] * 3
    assert p["kv_slots"] == [brute_slot([9, 4, 7], 4, q) for q in (6, 7, 8, 9, 10)] + [8, 9, 10]
    assert p["sample_rows"] == [4, 6, 7] and p["sample_indptr"] == [0, 1, 3]


@pytest.mark.parametrize("bad,msg", [
    (dict(position_ids=[47, 1]), "size mismatch"),
    (dict(kv_page_indptr=[0, 3, 3]), "kv_page_indptr length"),
    (dict(kv_last_page_lens=[16, 1]), "kv_last_page_lens length"),
    (dict(sampling_indptr=[0]), "sampling_indptr length"),
    (dict(kv_page_indices=[100, 101, 5000]), "out of bounds"),
    (dict(position_ids=[48]), "exceeds seq_len"),
    (dict(sampling_indices=[1]), "sampling_index"),
    (dict(kv_page_indptr=[0, 0], kv_last_page_lens=[0]), "empty KV state"),
    (dict(qo_indptr=[0, 0], token_ids=[], position_ids=[]), "zero tokens"),
])
def test_planner_errors_oracle_and_driver(bad, msg):
    from pie_amd import driver as drv

    base = dict(token_ids=[999], position_ids=[47], kv_page_indices=[100, 101, 102],
                kv_page_indptr=[0, 3], kv_last_page_lens=[16], qo_indptr=[0, 1],
                sampling_indices=[0], sampling_indptr=[0, 1])
    base.update(bad)
    with pytest.raises(op.PlanError, match=msg):
        op.plan_forward(page_size=16, total_pages=4096, **base)
    if msg == "sampling_indptr length":
        fr = drv.ForwardFrame(**base, samplers=[dict()], sampler_indptr=[0, 1])
    else:
        fr = drv.ForwardFrame(**base)
    with pytest.raises(ValueError, match=msg):
        drv.plan(fr, 16, 4096)


def random_batch(rng, ps, total_pages, R):
    tok, pos, pages, indptr, last, qo, sidx, sptr = [], [], [], [0], [], [0], [], [0]
    for _ in range(R):
        seq = int(rng.integers(1, 6 * ps))
        n_new = int(rng.integers(1, min(seq, 9) + 1))
        npg = (seq + ps - 1) // ps
        pages += rng.integers(0, total_pages, npg).tolist()
        indptr.append(len(pages))
        last.append(seq - (npg - 1) * ps)
        tok += rng.integers(0, 1000, n_new).tolist()
        pos += list(range(seq - n_new, seq))
        qo.append(len(tok))
        k = int(rng.integers(0, 3))
        sidx += sorted(rng.integers(0, n_new, k).tolist())
        sptr.append(len(sidx))
    return dict(token_ids=tok, position_ids=pos, kv_page_indices=pages, kv_page_indptr=indptr,
                kv_last_page_lens=last, qo_indptr=qo, sampling_indices=sidx, sampling_indptr=sptr)


@pytest.mark.parametrize("seed", range(6))
def test_driver_planner_matches_oracle_bit_exact(seed):
    from pie_amd import driver as drv

    rng = np.random.default_rng(80 + seed)
    ps = [16, 32, 16, 64, 16, 32][seed]
    b = random_batch(rng, ps, 500, int(rng.integers(1, 12)))
    want = op.plan_forward(page_size=ps, total_pages=500, **b)
    nslots = len(b["sampling_indices"])
    fr = drv.ForwardFrame(**b, samplers=[dict(temperature=0.0)] * nslots,
                          sampler_indptr=b["sampling_indptr"])
    got = drv.plan(fr, ps, 500)
    for k in ("positions", "kv_slots", "row_page_begin", "row_kv_len", "seq_len", "sample_rows",
              "sample_indptr"):
        assert np.array_equal(np.asarray(got[k], np.int64), np.asarray(want[k], np.int64)), k
    assert got["max_kv_len"] == want["max_kv_len"] and got["pure_decode"] == want["pure_decode"]
    assert got["all_greedy"] and not got["has_user_masks"]


def test_driver_planner_mask_and_sampler_flags():
    from pie_amd import driver as drv

    base = dict(token_ids=[5, 6], position_ids=[47, 9], kv_page_indices=[1, 2, 3, 4],
                kv_page_indptr=[0, 3, 4], kv_last_page_lens=[16, 10], qo_indptr=[0, 1, 2])
    # synthesised causal masks [0, pos+1] keep the fast path (driver/portable/src/plan.cpp:139-173)
    p = drv.plan(drv.ForwardFrame(**base, masks=[[0, 48], [0, 10]]), 16, 64)
    assert p["pure_decode"] and not p["has_user_masks"]
    p = drv.plan(drv.ForwardFrame(**base, masks=[[0, 4, 12, 32], [0, 10]]), 16, 64)
    assert p["has_user_masks"] and not p["pure_decode"]
    # temperature > 1e-5 or a non-token sampler kind leaves the all-greedy path
    samp = dict(sampling_indices=[0, 0], sampling_indptr=[0, 1, 2], sampler_indptr=[0, 1, 2])
    p = drv.plan(drv.ForwardFrame(**base, **samp, samplers=[dict(temperature=0.7), dict()]), 16, 64)
    assert not p["all_greedy"]
    p = drv.plan(drv.ForwardFrame(**base, **samp, samplers=[dict(kind=7), dict()]), 16, 64)
    assert not p["all_greedy"]
    p = drv.plan(drv.ForwardFrame(**base, **samp, samplers=[dict(kind=1, k=1), dict()]), 16, 64)
    assert p["all_greedy"]
