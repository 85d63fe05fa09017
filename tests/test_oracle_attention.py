"""Pins for the oracle's paged attention / KV write (CPU only): dense fp64 softmax attention
over rows gathered by an independent numpy path, and invariants of the page table."""
import numpy as np
import pytest

from paged_cases import gather_rows, make_paged_batch


def dense_attention(orc, q_bits, k_bits, v_bits, hq, scale, lim=None):
    """fp64 softmax attention of one query [hq, d] over dense rows [n, hk, d]."""
    q = orc.bf16_to_f32(q_bits).astype(np.float64)
    k = orc.bf16_to_f32(k_bits).astype(np.float64)
    v = orc.bf16_to_f32(v_bits).astype(np.float64)
    n, hk, d = k.shape
    if lim is not None:
        k, v, n = k[:lim], v[:lim], lim
    out = np.zeros((hq, d))
    lse = np.full((hq,), -np.inf)
    if n == 0:
        return out, lse
    for h in range(hq):
        s = (k[:, h // (hq // hk), :] @ q[h]) * scale
        m = s.max()
        p = np.exp(s - m)
        out[h] = (p[:, None] * v[:, h // (hq // hk), :]).sum(0) / p.sum()
        lse[h] = np.log(p.sum()) + m
    return out, lse


@pytest.mark.parametrize("hq,hk,d,ps", [(8, 2, 64, 16), (4, 4, 128, 16), (8, 1, 32, 4)])
def test_decode_matches_dense_fp64(oracle, hq, hk, d, ps):
    rng = np.random.default_rng(20)
    ctx = [1, ps - 1, ps, ps + 1, 5 * ps + 3, 0, 37]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    scale = 1.0 / np.sqrt(d)
    for mode, tol in ((2, 1e-6), (0, 2e-5)):
        o, o16, lse = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"],
                                               b["page_indptr"], b["last_lens"], hq, hk, d, ps,
                                               mode=mode)
        for r in range(len(ctx)):
            k, v = gather_rows(b, r, ps)
            assert k.shape[0] == ctx[r]
            ref, ref_lse = dense_attention(oracle, q[r], k, v, hq, scale)
            assert np.allclose(o[r], ref, rtol=0, atol=tol * 10), (mode, r)
            if ctx[r]:
                assert np.allclose(lse[r], ref_lse, rtol=0, atol=tol * 10)
            else:
                assert np.all(o[r] == 0) and np.all(np.isneginf(lse[r]))
        assert np.array_equal(o16, oracle.f32_to_bf16(o))


def test_explicit_scale_and_default(oracle):
    rng = np.random.default_rng(21)
    b = make_paged_batch(rng, [20], 1, 32, 4, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((1, 2, 32)).astype(np.float32))
    a = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"], b["page_indptr"],
                                 b["last_lens"], 2, 1, 32, 4, sm_scale=-1.0, mode=2)[0]
    c = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"], b["page_indptr"],
                                 b["last_lens"], 2, 1, 32, 4, sm_scale=1 / np.sqrt(32), mode=2)[0]
    e = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"], b["page_indptr"],
                                 b["last_lens"], 2, 1, 32, 4, sm_scale=0.5, mode=2)[0]
    assert np.allclose(a, c, atol=1e-7) and not np.allclose(a, e, atol=1e-3)
    k, v = gather_rows(b, 0, 4)
    assert np.allclose(e[0], dense_attention(oracle, q[0], k, v, 2, 0.5)[0], atol=1e-5)


def test_page_permutation_invariance_and_forked_prefix(oracle):
    rng = np.random.default_rng(22)
    hq, hk, d, ps = 4, 2, 64, 16
    ctx = [100, 70, 64, 90]
    b = make_paged_batch(rng, ctx, hk, d, ps, shared_prefix_tokens=48, shared_fraction=0.75,
                         f32_to_bf16=oracle.f32_to_bf16)
    assert len(b["sharers"]) == 3
    # the sharers really list the same physical pages for the prefix
    p0 = b["page_indices"][b["page_indptr"][0]:][:3]
    p1 = b["page_indices"][b["page_indptr"][1]:][:3]
    assert np.array_equal(p0, p1)
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    o = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"], b["page_indptr"],
                                 b["last_lens"], hq, hk, d, ps, mode=0)[0]
    # private copies of the prefix + a different physical placement: identical results
    perm = rng.permutation(b["num_pages"] + 3 * 3).astype(np.uint32)
    k2 = np.zeros((len(perm), ps, hk, d), np.uint16)
    v2 = np.zeros_like(k2)
    idx2, nxt = [], 0
    for r in range(len(ctx)):
        lo, hi = int(b["page_indptr"][r]), int(b["page_indptr"][r + 1])
        new = perm[nxt:nxt + hi - lo]
        nxt += hi - lo
        k2[new] = b["k_pages"][b["page_indices"][lo:hi]]
        v2[new] = b["v_pages"][b["page_indices"][lo:hi]]
        idx2.append(new)
    o2 = oracle.attn_decode_paged(q, k2, v2, np.concatenate(idx2), b["page_indptr"], b["last_lens"],
                                  hq, hk, d, ps, mode=0)[0]
    assert np.array_equal(o, o2)


def test_prefill_causal_limit_brute_force(oracle):
    rng = np.random.default_rng(23)
    hq, hk, d, ps = 2, 1, 32, 4
    # request 0: 5 new tokens on top of 6 cached (kv_len 11); request 1: pure prefill of 3
    ctx = [11, 3]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    qo = np.array([0, 5, 8], np.uint32)
    q = oracle.f32_to_bf16(rng.standard_normal((8, hq, d)).astype(np.float32))
    o, _, lse = oracle.attn_paged(q, b["k_pages"], b["v_pages"], qo, b["page_indices"],
                                  b["page_indptr"], b["last_lens"], hq, hk, d, ps, mode=2)
    for r, (lo, hi) in enumerate([(0, 5), (5, 8)]):
        k, v = gather_rows(b, r, ps)
        for i in range(hi - lo):
            lim = ctx[r] - (hi - lo) + i + 1  # attention_naive_paged.cu:194-198
            ref, ref_lse = dense_attention(oracle, q[lo + i], k, v, hq, 1 / np.sqrt(d), lim=lim)
            assert np.allclose(o[lo + i], ref, atol=1e-5)
            assert np.allclose(lse[lo + i], ref_lse, atol=1e-5)


def test_kv_write_slots(oracle):
    rng = np.random.default_rng(24)
    hk, d, ps = 2, 8, 4
    ctx = [6, 9, 1]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    qo = np.array([0, 2, 7, 8], np.uint32)  # 2, 5 and 1 new tokens
    T = 8
    kc = rng.integers(1, 2 ** 16, size=(T, hk, d)).astype(np.uint16)
    vc = rng.integers(1, 2 ** 16, size=(T, hk, d)).astype(np.uint16)
    kp = np.zeros_like(b["k_pages"])
    vp = np.zeros_like(b["v_pages"])
    oracle.kv_write(kc, vc, kp, vp, qo, b["page_indices"], b["page_indptr"], b["last_lens"], hk, d, ps)
    written = 0
    for r, n_new in enumerate([2, 5, 1]):
        pages = b["page_indices"][b["page_indptr"][r]:b["page_indptr"][r + 1]]
        for i in range(n_new):
            pos = ctx[r] - n_new + i  # the new tokens are the last n_new positions
            assert np.array_equal(kp[pages[pos // ps], pos % ps], kc[qo[r] + i])
            assert np.array_equal(vp[pages[pos // ps], pos % ps], vc[qo[r] + i])
            written += 1
    assert np.count_nonzero(kp.reshape(-1, hk * d).any(axis=1)) == written


def test_brle_visibility_follows_the_mask_builder(oracle):
    """build_attn_mask_f16 (driver/portable/src/plan.cpp:54-94) on hand-worked rows."""
    b = lambda runs, pos, n_kv, w=0: list(oracle.brle_allow(runs, pos, n_kv, w))
    assert b([], 3, 6) == [1, 1, 1, 1, 0, 0]                       # plain causal
    assert b([], 3, 6, 2) == [0, 0, 1, 1, 0, 0]                    # sliding window of 2
    assert b([0, 4], 3, 6) == [1, 1, 1, 1, 0, 0]                   # the synthesised causal shape
    assert b([1, 2, 1, 5], 5, 8) == [0, 1, 1, 0, 1, 1, 0, 0]       # holes; nothing past pos
    assert b([0, 2], 5, 8) == [1, 1, 0, 0, 0, 0, 0, 0]             # past the last run: hidden
    assert b([0, 100], 2, 8) == [1, 1, 1, 0, 0, 0, 0, 0]           # a mask cannot unmask the future
    assert b([2, 3], 9, 4) == [0, 0, 1, 1]                         # clipped to the context
    assert b([0, 6], 5, 8, 3) == [0, 0, 0, 1, 1, 1, 0, 0]          # window clips a true run


def test_masked_rows_equal_dense_attention_over_the_allowed_keys(oracle):
    from paged_cases import make_paged_batch

    rng = np.random.default_rng(77)
    hq, hk, d, ps = 4, 2, 64, 16
    ctx = [37, 20]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    # rows: three queries of request 0 (positions 30, 33, 36) and one of request 1
    row_begin = [int(b["page_indptr"][0])] * 3 + [int(b["page_indptr"][1])]
    row_len = [31, 34, 37, 20]
    q = oracle.f32_to_bf16(rng.standard_normal((4, hq, d)).astype(np.float32))
    allow = [oracle.brle_allow([3, 10, 5, 40], 30, 31), None,
             oracle.brle_allow([0, 1, 35, 1], 36, 37), np.zeros(20, np.uint8)]
    o32, _, lse = oracle.attn_rows_masked(q, b["k_pages"], b["v_pages"], b["page_indices"], row_begin,
                                          row_len, hq, hk, d, ps, allow)
    kf, vf = oracle.bf16_to_f32(b["k_pages"]).astype(np.float64), oracle.bf16_to_f32(b["v_pages"]).astype(np.float64)
    qf = oracle.bf16_to_f32(q).astype(np.float64)
    for r in range(4):
        pages = b["page_indices"][row_begin[r]:]
        keys = np.array([pages[j // ps] * ps + j % ps for j in range(row_len[r])])
        vis = np.ones(row_len[r], bool) if allow[r] is None else allow[r][:row_len[r]].astype(bool)
        for h in range(hq):
            K = kf.reshape(-1, hk, d)[keys[vis], h // (hq // hk)]
            Vv = vf.reshape(-1, hk, d)[keys[vis], h // (hq // hk)]
            if not vis.any():
                assert np.all(o32[r, h] == 0) and np.isneginf(lse[r, h])
                continue
            s = K @ qf[r, h] / np.sqrt(d)
            p = np.exp(s - s.max())
            assert np.allclose(o32[r, h], (p / p.sum()) @ Vv, rtol=1e-5, atol=1e-6)
            assert abs(lse[r, h] - (np.log(p.sum()) + s.max())) < 1e-4
