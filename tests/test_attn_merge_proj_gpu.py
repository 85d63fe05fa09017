"""The attention output projection with the decode attention's split merge in its prologue
(`pie_hip_attn_rows_paged_partials` + `pie_hip_linear_attn_merge`) against the two launches it
replaces (`pie_hip_attn_rows_paged`, whose parity with the oracle `tests/test_attn_decode_gpu.py`
and `tests/test_kv_quant_gpu.py` hold, then `pie_hip_linear_fused`): bit-identical outputs."""
import numpy as np
import pytest

from gpu_util import bits, dev
from paged_cases import make_paged_batch

pytestmark = pytest.mark.gpu


def _weight(kind, N, K, gpu, rng):
    import torch
    from pie_amd import ops

    if kind == "int4b8":
        data = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, (N, K // 8), dtype=np.int64).astype(np.int32)).to(gpu)
        scale = (torch.rand((N, K // 128), device=gpu) * 0.006 + 0.002).bfloat16()
        return ops.WeightView(kind, data, scale, 128, N, K)
    if kind == "bf16":
        return ops.WeightView(kind, (torch.randn((N, K), device=gpu) * 0.02).bfloat16(), None, 0, N, K)
    codes = torch.from_numpy(rng.integers(0, 256, (N, K), dtype=np.int64).astype(np.uint8)).to(gpu)
    if kind == "fp8":
        codes = torch.where((codes & 0x7F) == 0x7F, torch.zeros_like(codes), codes)
    else:
        codes = codes.view(torch.int8)
    return ops.WeightView(kind, codes, (torch.rand(N, device=gpu) * 0.01 + 0.002).bfloat16(), 0, N, K)


@pytest.mark.parametrize("kind", ["int4b8", "int8", "fp8", "bf16"])
@pytest.mark.parametrize("ctx,hq,hk,d,N", [
    ([600], 32, 8, 128, 4096),        # the 8B decode step: five of eight split slots in use
    ([1], 32, 8, 128, 4096),          # one key: a single split of the plan's many
    ([1024], 32, 8, 128, 512),        # every slot in use
    ([300, 17], 32, 8, 128, 4096),    # two rows, four slots, rows of different extents
    ([260, 0], 16, 2, 64, 1024),      # a row without keys: zeros into the projection
    ([1000], 32, 4, 128, 4096),       # 30B-A3B heads (eight query heads per kv head)
])
def test_projection_with_merge_equals_attention_then_projection(gpu, oracle, kind, ctx, hq, hk, d, N):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(700 + len(ctx) + hq + d + sum(ctx))
    ps = 16
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = dev(oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32)), gpu, torch.bfloat16)
    kp, vp = dev(b["k_pages"], gpu, torch.bfloat16), dev(b["v_pages"], gpu, torch.bfloat16)
    pages = dev(b["page_indices"].view(np.int32), gpu)
    begin, lens = dev(b["page_indptr"][:-1].astype(np.int32), gpu), dev(np.asarray(ctx, np.int32), gpu)
    # the bound a driver's graph bucket would pass: the next multiple of 512
    max_kv = (max(ctx) + 511) // 512 * 512
    ups, ns = ops.attn_decode_plan(len(ctx), hk, max_kv)
    assert ns >= 2, "the case must split"
    w = _weight(kind, N, hq * d, gpu, rng)
    resid = (torch.randn((len(ctx), N), device=gpu)).bfloat16()

    o = ops.attention_rows_paged(q, kp, vp, pages, begin, lens, max_kv)
    for beta in (0, 1):
        ref = ops.linear_fused(o.reshape(len(ctx), hq * d), w, y=resid.clone() if beta else None, beta=beta)
        part = ops.attention_rows_paged_partials(q, kp, vp, pages, begin, lens, max_kv)
        got = ops.linear_attn_merge(part, ns, ups, lens, hq, d, w, y=resid.clone() if beta else None, beta=beta)
        assert np.array_equal(bits(got), bits(ref))


def test_projection_with_merge_over_one_byte_pools(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(720)
    ctx, hq, hk, d, ps, fmt = [700], 32, 8, 128, 16, "fp8_per_token_head"
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    P = b["num_pages"]
    pools = {}
    for name in ("k_pages", "v_pages"):
        codes, scales, _ = oracle.kv_quant_rows(b[name].reshape(P * ps * hk, d), fmt)
        pools[name] = (dev(codes.reshape(P, ps, hk, d), gpu),
                       dev(np.ascontiguousarray(scales.reshape(P, ps, hk).transpose(0, 2, 1)), gpu))
    q = dev(oracle.f32_to_bf16(rng.standard_normal((1, hq, d)).astype(np.float32)), gpu, torch.bfloat16)
    pages = dev(b["page_indices"].view(np.int32), gpu)
    begin, lens = dev(b["page_indptr"][:-1].astype(np.int32), gpu), dev(np.asarray(ctx, np.int32), gpu)
    max_kv = 1024
    ups, ns = ops.attn_decode_plan(1, hk, max_kv)
    w = _weight("int4b8", 4096, hq * d, gpu, rng)
    o, _ = ops.attention_rows_paged_kvq(fmt, q, pools["k_pages"][0], pools["v_pages"][0], pools["k_pages"][1],
                                        pools["v_pages"][1], pages, begin, lens)
    ref = ops.linear_fused(o.reshape(1, hq * d), w)
    part = ops.attention_rows_paged_partials(q, pools["k_pages"][0], pools["v_pages"][0], pages, begin, lens, max_kv,
                                             fmt=fmt, k_scales=pools["k_pages"][1], v_scales=pools["v_pages"][1])
    got = ops.linear_attn_merge(part, ns, ups, lens, hq, d, w)
    assert np.array_equal(bits(got), bits(ref))


def test_shapes_the_merge_prologue_does_not_take_are_refused(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(730)
    hq, d = 32, 128
    w = _weight("int4b8", 256, hq * d, gpu, rng)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=gpu)
    lens3 = torch.full((3,), 100, dtype=torch.int32, device=gpu)
    with pytest.raises(ops.KernelError):          # three rows
        ops.linear_attn_merge(ws, 2, 8, lens3, hq, d, w)
    with pytest.raises(ops.KernelError):          # two rows with more than four splits
        ops.linear_attn_merge(ws, 8, 8, lens3[:2], hq, d, w)
    with pytest.raises(ops.KernelError):          # more than eight splits
        ops.linear_attn_merge(ws, 16, 8, lens3[:1], hq, d, w)
    with pytest.raises(ops.KernelError):          # a single split: nothing to merge
        ops.linear_attn_merge(ws, 1, 8, lens3[:1], hq, d, w)
