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


@pytest.mark.parametrize("T,H,E,K", [(64, 2048, 128, 8), (1, 2048, 128, 8), (5, 512, 6, 2), (200, 4096, 64, 6),
                                     (17, 7168, 384, 8)])
def test_norm_route_in_one_launch(gpu, oracle, T, H, E, K):
    """pie_hip_moe_norm_route: the stored normalised rows are pie_hip_rmsnorm's bit for bit, the
    router logits are the oracle's bf16 products up to the order of the fp32 sum, and given the
    logits it stored the routing is the oracle's exactly, laid out as a counting sort."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(530 + T + E)
    x = dev(oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32) * 3.0), gpu, torch.bfloat16)
    nw = dev(oracle.f32_to_bf16((1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32)), gpu, torch.bfloat16)
    router = oracle.f32_to_bf16(rng.standard_normal((E, H)).astype(np.float32) * (1.0 / np.sqrt(H)))
    for renorm in (True, False):
        xn, lg, idx, w, offs, rtok, rpos = ops.moe_norm_route(x, nw, 1e-6, dev(router, gpu, torch.bfloat16), K,
                                                              renormalize=renorm)
        assert np.array_equal(bits(xn), bits(ops.rmsnorm_bf16(x, nw, 1e-6)))
        want = oracle.gemm_bf16(bits(xn), router, mode=0)[1]
        assert (ulp_diff(bits(lg), want) <= 1).all() and (bits(lg) == want).mean() > 0.97
        oidx, ow = oracle.topk_softmax(bits(lg), K, renorm=renorm)
        idx, w, offs, rtok, rpos = (t.cpu().numpy() for t in (idx, w, offs, rtok, rpos))
        assert np.array_equal(idx, oidx)
        assert np.allclose(w, ow, rtol=2e-6, atol=1e-9)
        counts = np.bincount(idx.reshape(-1), minlength=E)
        assert np.array_equal(offs, np.concatenate([[0], np.cumsum(counts)]))
        flat = idx.reshape(-1)
        assert np.array_equal(np.sort(rpos), np.arange(T * K))
        assert np.all(rpos >= offs[flat]) and np.all(rpos < offs[flat + 1])
        assert np.array_equal(rtok[rpos], np.arange(T * K) // K)
        # the same routing as the two-launch form gives on the same logits
        ref = ops.moe_route(lg, K, renormalize=renorm)
        assert np.array_equal(ref[0].cpu().numpy(), idx) and np.array_equal(ref[1].cpu().numpy(), w)


@pytest.mark.parametrize("T,K,H", [(64, 8, 2048), (3, 2, 512), (130, 6, 8192)])
def test_combine_with_the_next_norm_equals_the_two_launches(gpu, oracle, T, K, H):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(540 + T)
    y = dev(oracle.f32_to_bf16(rng.standard_normal((T * K, H)).astype(np.float32)), gpu, torch.bfloat16)
    w = dev(rng.dirichlet(np.ones(K), T).astype(np.float32), gpu)
    pos = dev(rng.permutation(T * K).astype(np.int32), gpu)
    base = dev(oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32)), gpu, torch.bfloat16)
    nw = dev(oracle.f32_to_bf16((1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32)), gpu, torch.bfloat16)
    a = base.clone()
    ops.moe_combine(y, pos, w, a)
    an = ops.rmsnorm_bf16(a, nw, 1e-6)
    b = base.clone()
    bn = ops.moe_combine_norm(y, pos, w, b, nw, 1e-6)
    assert np.array_equal(bits(a), bits(b)) and np.array_equal(bits(an), bits(bn))


def _expert_block(gpu, oracle, seed, T, E, K, tiled, H=2048, Ie=768):
    """norm'd activations -> router -> route -> grouped gate/up (+SwiGLU) -> grouped down ->
    combine, fp8 e4m3 experts with bf16 row scales, against the oracle's per-route evaluation.
    `tiled`: the launches a driver with tile-major weights makes (gate|up in the block-shared
    grouped form, down in the wave-private grouped form over K = Ie), with the driver's
    rows-per-expert hint; otherwise the row-major entry."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(seed)
    x = oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    router = oracle.f32_to_bf16(rng.standard_normal((E, H)).astype(np.float32) * (1.0 / np.sqrt(H)))

    def fp8_stack(n, k):
        qs, ss = [], []
        for _ in range(E):      # expert by expert: the float copy of a whole stack is gigabytes
            w = oracle.f32_to_bf16(rng.standard_normal((n, k), dtype=np.float32) * 0.02)
            q, s = oracle.quant_fp8_per_channel(w)
            qs.append(q)
            ss.append(oracle.f32_to_bf16(s))
        return np.concatenate(qs), np.concatenate(ss)
    gu_q, gu_s = fp8_stack(2 * Ie, H)      # canonical: per expert gate rows then up rows
    dn_q, dn_s = fp8_stack(H, Ie)

    # ---- oracle: per-route evaluation ----
    logits = oracle.gemm_bf16(x, router, mode=0)[1]
    oidx, ow = oracle.topk_softmax(logits, K)
    yr = np.empty((T * K, H), np.uint16)
    act_ref = np.empty((T * K, Ie), np.uint16)
    for r in range(T * K):
        t, e = r // K, oidx.reshape(-1)[r]
        g = oracle.gemm_fp8(x[t:t + 1], gu_q[e * 2 * Ie:(e + 1) * 2 * Ie],
                            oracle.bf16_to_f32(gu_s[e * 2 * Ie:(e + 1) * 2 * Ie]), mode=0)[1]
        a = oracle.swiglu(g)
        act_ref[r] = a[0]
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
    gu_qi = dev(np.ascontiguousarray(gu_q.reshape(E, 2 * Ie, H)[:, perm]), gpu)
    gu_si = dev(np.ascontiguousarray(gu_s.reshape(E, 2 * Ie)[:, perm]), gpu, torch.bfloat16)
    dn_qg = dev(dn_q.reshape(E, H, Ie), gpu)
    dn_sg = dev(dn_s.reshape(E, H), gpu, torch.bfloat16)
    # the executor's hint (Executor::moe_block): twice the mean routes per expert, at most T
    hint = max(1, min(T, 2 * ((T * K + E - 1) // E))) if tiled else 16
    if tiled:
        # experts stacked along the rows: the tile-major copy keeps expert e at the same stride
        gu_qi = ops.repack_mfma_tiles(ops.WeightView("fp8", gu_qi.reshape(E * 2 * Ie, H), None, 0,
                                                     E * 2 * Ie, H)).data.reshape(E, 2 * Ie, -1)
        dn_qg = ops.repack_mfma_tiles(ops.WeightView("fp8", dn_qg.reshape(E * H, Ie), None, 0,
                                                     E * H, Ie)).data.reshape(E, H, -1)
    h = ops.moe_grouped_gemm(xg, rtok, offs, "fp8", gu_qi, gu_si, 2 * Ie, H, rows_hint=hint, swiglu=True,
                             tiled=tiled)
    y = ops.moe_grouped_gemm(h, None, offs, "fp8", dn_qg, dn_sg, H, Ie, rows_hint=hint, tiled=tiled)
    out = bits(ops.moe_combine(y, rpos, w, xg.clone()))
    same_routes = np.array_equal(idx.cpu().numpy(), oidx)
    assert same_routes, "router near-tie flipped an expert; pick another seed"
    # every stage against the oracle: the SwiGLU'd gate|up rows (route-sorted on the GPU) ...
    pos = rpos.cpu().numpy()
    hb = bits(h)[pos]
    assert close_to_oracle(oracle, hb, act_ref, rel=2.0 ** -6)
    assert (ulp_diff(hb, act_ref) <= 1).mean() > 0.97
    # ... the down projection of each route ...
    yb = bits(y)[pos]
    assert close_to_oracle(oracle, yb, yr, rel=2.0 ** -6)
    assert (ulp_diff(yb, yr) <= 1).mean() > 0.95
    # ... and the combined block
    assert close_to_oracle(oracle, out, ref, rel=2.0 ** -6)
    assert (ulp_diff(out, ref) <= 1).mean() > 0.97
    return dict(xg=xg, rtok=rtok, offs=offs, gu=(gu_qi, gu_si), dn=(dn_qg, dn_sg), hint=hint,
                gu_q=gu_q, gu_s=gu_s, dn_q=dn_q, dn_s=dn_s, oidx=oidx, rpos=pos)


def test_expert_block_at_c5_expert_shape(gpu, oracle):
    """H 2048, expert FFN 768, 32 of the 128 experts, top-4, through the row-major entry."""
    _expert_block(gpu, oracle, 520, T=48, E=32, K=4, tiled=False)


def test_expert_block_at_c5_full_routing_through_the_tile_major_kernels(gpu, oracle):
    """The Qwen3-30B-A3B decode batch as the driver runs it: 64 tokens, 128 experts, top-8,
    H 2048, expert FFN 768, fp8 e4m3 with bf16 row scales, tile-major weights — gate|up through
    the block-shared grouped kernel, down through the wave-private grouped kernel over K = 768
    (six 128-blocks) — every stage against the oracle, then exactness of single weights."""
    import torch
    from pie_amd import ops

    T, E, K, H, Ie = 64, 128, 8, 2048, 768
    st = _expert_block(gpu, oracle, 521, T=T, E=E, K=K, tiled=True)
    # one-hot activation rows reproduce single dequantised weights bit for bit (operand layouts
    # of both grouped kernels): route r of expert e reads a row that is 1 at column c_r
    rng = np.random.default_rng(522)
    offs = st["offs"].cpu().numpy()
    routes = int(offs[-1])
    expert_of = np.repeat(np.arange(E), np.diff(offs))
    # down: K = Ie
    cols = rng.integers(0, Ie, routes)
    a = np.zeros((routes, Ie), np.float32)
    a[np.arange(routes), cols] = 1.0
    y = bits(ops.moe_grouped_gemm(dev(oracle.f32_to_bf16(a), gpu, torch.bfloat16), None, st["offs"], "fp8",
                                  st["dn"][0], st["dn"][1], H, Ie, rows_hint=st["hint"], tiled=True))
    dn_q = st["dn_q"].reshape(E, H, Ie)
    dn_s = oracle.bf16_to_f32(st["dn_s"].reshape(E, H))
    want = oracle.f32_to_bf16(oracle.fp8_decode(dn_q[expert_of, :, cols]) * dn_s[expert_of])
    # (compared as values: a weight code of -0 gives -0 here and +0 from an accumulator that starts at +0)
    assert np.array_equal(oracle.bf16_to_f32(y), oracle.bf16_to_f32(want))
    # gate|up without SwiGLU: K = H, rows gathered by route
    cols = rng.integers(0, H, T)
    a = np.zeros((T, H), np.float32)
    a[np.arange(T), cols] = 1.0
    g = bits(ops.moe_grouped_gemm(dev(oracle.f32_to_bf16(a), gpu, torch.bfloat16), st["rtok"], st["offs"],
                                  "fp8", st["gu"][0], st["gu"][1], 2 * Ie, H, rows_hint=st["hint"],
                                  tiled=True))
    perm = np.empty(2 * Ie, np.int64)
    perm[0::2], perm[1::2] = np.arange(Ie), np.arange(Ie) + Ie
    gu_q = st["gu_q"].reshape(E, 2 * Ie, H)[:, perm]
    gu_s = oracle.bf16_to_f32(st["gu_s"].reshape(E, 2 * Ie)[:, perm])
    tok = st["rtok"].cpu().numpy()
    want = oracle.f32_to_bf16(oracle.fp8_decode(gu_q[expert_of, :, cols[tok]]) * gu_s[expert_of])
    assert np.array_equal(oracle.bf16_to_f32(g), oracle.bf16_to_f32(want))
