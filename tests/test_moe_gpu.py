"""GPU parity for the MoE row: routing (softmax, top-k, renormalisation and the expert-sorted
layout), the combine, and the whole expert block at the Qwen3-30B-A3B expert shape against the
oracle's per-route evaluation."""
import numpy as np
import pytest

from gpu_util import bits, dev, ulp_diff
from test_linear_fused_gpu import close_to_oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,E,K", [(1, 128, 8), (64, 128, 8), (7, 8, 2), (300, 384, 6), (5, 5, 5),
                                   (2100, 64, 4)])
def test_route_matches_oracle_and_layout_is_a_counting_sort(gpu, oracle, T, E, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(500 + T + E)
    logits = oracle.f32_to_bf16(rng.standard_normal((T, E)).astype(np.float32) * 2)
    if T > 6:
        logits[3, :] = logits[3, 0]            # a fully tied row: the first K experts win
        logits[5, 1:4] = logits[5].max()       # tied maxima: lowest indices first
    idx, w, offs, rtok, rpos = (t.cpu().numpy() for t in ops.moe_route(dev(logits, gpu, torch.bfloat16), K))
    oidx, ow = oracle.topk_softmax(logits, K)
    assert np.array_equal(idx, oidx)           # integer outputs: bit-exact
    assert np.allclose(w, ow, rtol=2e-6, atol=1e-9)
    # norm_topk = false: the same routes, the probabilities undivided
    idx_r, w_r = (t.cpu().numpy() for t in ops.moe_route(dev(logits, gpu, torch.bfloat16), K, renormalize=False)[:2])
    _, ow_r = oracle.topk_softmax(logits, K, renorm=False)
    assert np.array_equal(idx_r, oidx) and np.allclose(w_r, ow_r, rtol=2e-6, atol=1e-9)
    # layout: offsets are the exclusive scan of the per-expert route counts
    counts = np.bincount(idx.reshape(-1), minlength=E)
    assert np.array_equal(offs, np.concatenate([[0], np.cumsum(counts)]))
    flat = idx.reshape(-1)
    assert np.array_equal(np.sort(rpos), np.arange(T * K))      # a permutation
    assert np.all(rpos >= offs[flat]) and np.all(rpos < offs[flat + 1])
    assert np.array_equal(rtok[rpos], np.arange(T * K) // K)


@pytest.mark.parametrize("add", [False, True])
def test_combine_is_bit_exact(gpu, oracle, add):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(510)
    T, K, H = 37, 8, 2048
    yr = oracle.f32_to_bf16(rng.standard_normal((T * K, H)).astype(np.float32))
    w = rng.dirichlet(np.ones(K), T).astype(np.float32)
    pos = rng.permutation(T * K).astype(np.int32)
    sorted_y = np.empty_like(yr)
    sorted_y[pos] = yr
    base = oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    out = dev(base, gpu, torch.bfloat16).clone() if add else None
    got = bits(ops.moe_combine(dev(sorted_y, gpu, torch.bfloat16), dev(pos, gpu), dev(w, gpu), out))
    ref = oracle.moe_combine(yr, w, base if add else None)
    assert np.array_equal(got, ref)


def test_expert_block_at_c5_expert_shape(gpu, oracle):
    """norm'd activations -> router -> route -> grouped gate/up (+SwiGLU) -> grouped down ->
    combine, fp8 e4m3 experts with bf16 row scales: H 2048, expert FFN 768 (32 of the 128
    experts, top-4, to keep the CPU side small)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(520)
    T, H, Ie, E, K = 48, 2048, 768, 32, 4
    x = oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    router = oracle.f32_to_bf16(rng.standard_normal((E, H)).astype(np.float32) * (1.0 / np.sqrt(H)))

    def fp8_stack(n, k):
        w = oracle.f32_to_bf16(rng.standard_normal((E * n, k), dtype=np.float32) * 0.02)
        q, s = oracle.quant_fp8_per_channel(w)
        sb = oracle.f32_to_bf16(s)
        return q, sb
    gu_q, gu_s = fp8_stack(2 * Ie, H)      # canonical: per expert gate rows then up rows
    dn_q, dn_s = fp8_stack(H, Ie)

    # ---- oracle: per-route evaluation ----
    logits = oracle.gemm_bf16(x, router, mode=0)[1]
    oidx, ow = oracle.topk_softmax(logits, K)
    yr = np.empty((T * K, H), np.uint16)
    for r in range(T * K):
        t, e = r // K, oidx.reshape(-1)[r]
        g = oracle.gemm_fp8(x[t:t + 1], gu_q[e * 2 * Ie:(e + 1) * 2 * Ie],
                            oracle.bf16_to_f32(gu_s[e * 2 * Ie:(e + 1) * 2 * Ie]), mode=0)[1]
        a = oracle.swiglu(g)
        yr[r] = oracle.gemm_fp8(a, dn_q[e * H:(e + 1) * H], oracle.bf16_to_f32(dn_s[e * H:(e + 1) * H]),
                                mode=0)[1][0]
    ref = oracle.moe_combine(yr, ow, x)

    # ---- GPU ----
    xg = dev(x, gpu, torch.bfloat16)
    lg = ops.gemm_skinny(xg, ops.WeightView("bf16", dev(router, gpu, torch.bfloat16), None, 0, E, H))
    assert (ulp_diff(bits(lg), logits) <= 1).mean() > 0.99
    idx, w, offs, rtok, rpos = ops.moe_route(lg, K)
    perm = np.empty(2 * Ie, np.int64)
    perm[0::2], perm[1::2] = np.arange(Ie), np.arange(Ie) + Ie
    gu_qi = gu_q.reshape(E, 2 * Ie, H)[:, perm]
    gu_si = gu_s.reshape(E, 2 * Ie)[:, perm]
    h = ops.moe_grouped_gemm(xg, rtok, offs, "fp8", dev(gu_qi, gpu), dev(gu_si, gpu, torch.bfloat16),
                             2 * Ie, H, rows_hint=16, swiglu=True)
    y = ops.moe_grouped_gemm(h, None, offs, "fp8", dev(dn_q.reshape(E, H, Ie), gpu),
                             dev(dn_s.reshape(E, H), gpu, torch.bfloat16), H, Ie, rows_hint=16)
    out = bits(ops.moe_combine(y, rpos, w, xg.clone()))
    same_routes = np.array_equal(idx.cpu().numpy(), oidx)
    assert same_routes, "router near-tie flipped an expert; pick another seed"
    assert close_to_oracle(oracle, out, ref, rel=2.0 ** -6)
    assert (ulp_diff(out, ref) <= 1).mean() > 0.97
