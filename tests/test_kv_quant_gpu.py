"""GPU parity for the one-byte KV-cache formats: the quantising KV write is bit-exact against the
oracle (codes and scales), and paged attention over such pools matches the oracle's attention
over the dequantised values (float(code) * scale)."""
import numpy as np
import pytest

from gpu_util import dev
from paged_cases import make_paged_batch

pytestmark = pytest.mark.gpu

FORMATS = ["fp8_e4m3", "int8_per_token_head", "fp8_per_token_head", "fp8_e5m2"]


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("hk,d", [(8, 128), (2, 64), (3, 96)])
def test_kv_write_quant_bit_exact(gpu, oracle, fmt, hk, d):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(40 + hk + d)
    N, pages, ps = 37, 9, 16
    k = oracle.f32_to_bf16((rng.standard_normal((N, hk, d)) * rng.uniform(0.05, 20, (N, hk, 1))).astype(np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal((N, hk, d)).astype(np.float32))
    k[3] = 0                                                   # an all-zero token
    slots = rng.permutation(pages * ps)[:N].astype(np.int64)
    slots[5] = -1                                              # a token without a slot
    kp = torch.full((pages, ps, hk, d), 0x55, dtype=torch.uint8, device=gpu)
    vp = torch.full((pages, ps, hk, d), 0x55, dtype=torch.uint8, device=gpu)
    scaled = fmt not in ("fp8_e4m3", "fp8_e5m2")
    # scale pools are [pages, kv heads, page_size]
    ks = torch.full((pages, hk, ps), -7.0, dtype=torch.float32, device=gpu) if scaled else None
    vs = torch.full((pages, hk, ps), -7.0, dtype=torch.float32, device=gpu) if scaled else None
    ops.kv_write_quant(fmt, dev(k, gpu, torch.bfloat16), dev(v, gpu, torch.bfloat16), dev(slots, gpu),
                       kp, vp, ks, vs)
    torch.cuda.synchronize()
    for src, pool, sc in ((k, kp, ks), (v, vp, vs)):
        codes, scales, _ = oracle.kv_quant_rows(src.reshape(N * hk, d), fmt)
        want = np.full((pages * ps, hk, d), 0x55, np.uint8)
        want_s = np.full((pages * ps, hk), -7.0, np.float32)
        for t in range(N):
            if slots[t] >= 0:
                want[slots[t]] = codes.reshape(N, hk, d)[t]
                if scaled:
                    want_s[slots[t]] = scales.reshape(N, hk)[t]
        assert np.array_equal(pool.cpu().numpy().reshape(pages * ps, hk, d), want)
        if scaled:
            got_s = sc.cpu().numpy().transpose(0, 2, 1).reshape(pages * ps, hk)   # -> [slot, head]
            assert np.array_equal(got_s, want_s)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("hq,hk,d,ps", [(32, 8, 128, 16), (8, 8, 128, 32), (16, 2, 64, 16), (4, 4, 64, 16)])
def test_attention_over_quantised_pool_matches_oracle(gpu, oracle, fmt, hq, hk, d, ps):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(50 + hq + d + ps)
    ctx = [1, 15, 16, 17, 33, 100, 257, 0, 1500, 5]
    b = make_paged_batch(rng, ctx, hk, d, ps, shared_prefix_tokens=2 * ps, shared_fraction=0.3,
                         f32_to_bf16=oracle.f32_to_bf16)
    P = b["num_pages"]
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    pools = {}
    for name in ("k_pages", "v_pages"):
        codes, scales, deq = oracle.kv_quant_rows(b[name].reshape(P * ps * hk, d), fmt)
        pools[name] = (codes.reshape(P, ps, hk, d),
                       None if scales is None else np.ascontiguousarray(scales.reshape(P, ps, hk).transpose(0, 2, 1)),
                       deq.reshape(P, ps, hk, d))
    begin, lens = b["page_indptr"][:-1].astype(np.int32), np.asarray(ctx, np.int32)
    sc = lambda s: None if s is None else dev(s, gpu)
    o, lse = ops.attention_rows_paged_kvq(
        fmt, dev(q, gpu, torch.bfloat16), dev(pools["k_pages"][0], gpu), dev(pools["v_pages"][0], gpu),
        sc(pools["k_pages"][1]), sc(pools["v_pages"][1]), dev(b["page_indices"].view(np.int32), gpu),
        dev(begin, gpu), dev(lens, gpu), lse=True)
    torch.cuda.synchronize()
    truth, _, lse64 = oracle.attn_rows_f32kv(q, pools["k_pages"][2], pools["v_pages"][2], b["page_indices"],
                                             begin, lens, hq, hk, d, ps, mode=2)
    got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
    # one bf16 rounding of the output + fp32 softmax / accumulation error, as for bf16 pools
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x tol"
    lse_g = lse.cpu().numpy()
    fin = np.isfinite(lse64)
    assert np.array_equal(np.isneginf(lse_g), np.isneginf(lse64))
    assert np.allclose(lse_g[fin], lse64[fin], rtol=0, atol=2e-4)


@pytest.mark.parametrize("fmt,hq,hk,d,ps,rows,longest", [
    ("fp8_per_token_head", 32, 8, 128, 16, 70, 800), ("int8_per_token_head", 32, 8, 128, 16, 40, 1600),
    ("fp8_e5m2", 16, 4, 64, 32, 140, 800), ("int8_per_token_head", 32, 4, 128, 16, 70, 1600),
    ("int8_per_token_head", 4, 2, 128, 16, 100, 2500), ("int8_per_token_head", 2, 1, 64, 16, 200, 2100),
    ("int8_per_token_head", 8, 2, 64, 48, 150, 2000)])   # (the oracle's fp8 quantiser is slow: int8 for the larger pools)
def test_large_ragged_batch_over_quantised_pools_takes_the_chunked_launch(gpu, oracle, fmt, hq, hk, d, ps, rows,
                                                                          longest):
    """Batches whose split grid would queue blocks run as equal chunks of the batch's keys, one wave
    per kv head, pieces of a row merged from consecutive slots: empty rows, rows of one key, rows that
    end inside a unit, rows cut by several chunks and chunks that cover many short rows."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(70 + hq + d + rows)
    ctx = rng.integers(0, longest + 1, size=rows)
    ctx[0], ctx[1], ctx[2], ctx[3], ctx[-1] = longest, 0, 1, 17, 16
    ctx[5:15] = rng.integers(1, 20, size=10)                  # a run of short rows inside one chunk
    ctx = [int(c) for c in ctx]
    assert ops.attn_decode_is_chunked(fmt, rows, hk, max(ctx))
    assert not ops.attn_decode_is_chunked("bf16", rows, hk, max(ctx))
    b = make_paged_batch(rng, ctx, hk, d, ps, shared_prefix_tokens=2 * ps, shared_fraction=0.2,
                         f32_to_bf16=oracle.f32_to_bf16)
    P = b["num_pages"]
    q = oracle.f32_to_bf16(rng.standard_normal((rows, hq, d)).astype(np.float32))
    pools = {}
    for name in ("k_pages", "v_pages"):
        codes, scales, deq = oracle.kv_quant_rows(b[name].reshape(P * ps * hk, d), fmt)
        pools[name] = (codes.reshape(P, ps, hk, d),
                       None if scales is None else np.ascontiguousarray(scales.reshape(P, ps, hk).transpose(0, 2, 1)),
                       deq.reshape(P, ps, hk, d))
    begin, lens = b["page_indptr"][:-1].astype(np.int32), np.asarray(ctx, np.int32)
    sc = lambda s: None if s is None else dev(s, gpu)
    args = (fmt, dev(q, gpu, torch.bfloat16), dev(pools["k_pages"][0], gpu), dev(pools["v_pages"][0], gpu),
            sc(pools["k_pages"][1]), sc(pools["v_pages"][1]), dev(b["page_indices"].view(np.int32), gpu),
            dev(begin, gpu), dev(lens, gpu))
    o, lse = ops.attention_rows_paged_kvq(*args, lse=True)
    o2, _ = ops.attention_rows_paged_kvq(*args, lse=True)      # a second launch over the same workspace shape
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.uint16), o2.view(torch.uint16))
    truth, _, lse64 = oracle.attn_rows_f32kv(q, pools["k_pages"][2], pools["v_pages"][2], b["page_indices"],
                                             begin, lens, hq, hk, d, ps, mode=2)
    got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x tol"
    assert not np.any(got[1]), "a row without keys is all zeros"
    lse_g = lse.cpu().numpy()
    fin = np.isfinite(lse64)
    assert np.array_equal(np.isneginf(lse_g), np.isneginf(lse64))
    assert np.allclose(lse_g[fin], lse64[fin], rtol=0, atol=2e-4)


@pytest.mark.parametrize("fmt,hq,hk,d,rows,ctx_lo,ctx_hi", [
    ("fp8_per_token_head", 32, 8, 128, 16, 580, 640), ("int8_per_token_head", 32, 4, 128, 64, 900, 1000),
    ("fp8_e5m2", 16, 8, 64, 24, 300, 330), ("int8_per_token_head", 32, 8, 128, 40, 480, 512)])
def test_rows_declared_equally_long_over_quantised_pools(gpu, oracle, fmt, hq, hk, d, rows, ctx_lo, ctx_hi):
    """The equal-length hint over one-byte pools: one block of eight waves per (row, kv head) for 16, 24
    and 64 x 4 rows, one four-wave block per pair for 40 rows — no split, nothing merged — against the
    oracle over the dequantised pools and against the launch without the hint."""
    import torch
    from pie_amd import ops

    ps = 16
    rng = np.random.default_rng(33 + rows + d)
    ctx = [int(c) for c in rng.integers(ctx_lo, ctx_hi + 1, size=rows)]
    ctx[1] = 0
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    P = b["num_pages"]
    q = oracle.f32_to_bf16(rng.standard_normal((rows, hq, d)).astype(np.float32))
    pools = {}
    for name in ("k_pages", "v_pages"):
        codes, scales, deq = oracle.kv_quant_rows(b[name].reshape(P * ps * hk, d), fmt)
        pools[name] = (codes.reshape(P, ps, hk, d),
                       None if scales is None else np.ascontiguousarray(scales.reshape(P, ps, hk).transpose(0, 2, 1)),
                       deq.reshape(P, ps, hk, d))
    begin, lens = b["page_indptr"][:-1].astype(np.int32), np.asarray(ctx, np.int32)
    sc = lambda s: None if s is None else dev(s, gpu)
    args = (fmt, dev(q, gpu, torch.bfloat16), dev(pools["k_pages"][0], gpu), dev(pools["v_pages"][0], gpu),
            sc(pools["k_pages"][1]), sc(pools["v_pages"][1]), dev(b["page_indices"].view(np.int32), gpu),
            dev(begin, gpu), dev(lens, gpu))
    o, lse = ops.attention_rows_paged_kvq(*args, lse=True, uniform=True)
    o_plain, _ = ops.attention_rows_paged_kvq(*args, lse=True)
    torch.cuda.synchronize()
    truth, _, lse64 = oracle.attn_rows_f32kv(q, pools["k_pages"][2], pools["v_pages"][2], b["page_indices"],
                                             begin, lens, hq, hk, d, ps, mode=2)
    got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    assert np.all(np.abs(got - truth) <= tol)
    assert not np.any(got[1]), "a row without keys is all zeros"
    lse_g = lse.cpu().numpy()
    fin = np.isfinite(lse64)
    assert np.array_equal(np.isneginf(lse_g), np.isneginf(lse64))
    assert np.allclose(lse_g[fin], lse64[fin], rtol=0, atol=2e-4)
    plain = oracle.bf16_to_f32(o_plain.view(torch.uint16).cpu().numpy()).astype(np.float64)
    assert np.all(np.abs(got - plain) <= 2.0 ** -7 * np.maximum(np.abs(got), np.abs(plain)) + 1e-4)


def test_chunk_that_covers_more_rows_than_its_item_table_holds(gpu, oracle):
    """240 rows of a few keys next to 16 long ones: the chunks inside the run of short rows cover 40
    of them, more than one table of items, so a block builds its table twice."""
    import torch
    from pie_amd import ops

    fmt, hq, hk, d, ps = "int8_per_token_head", 8, 8, 64, 16
    rng = np.random.default_rng(91)
    ctx = [10000] * 8 + [int(c) for c in rng.integers(1, 17, size=240)] + [10000] * 8
    rows = len(ctx)
    assert ops.attn_decode_is_chunked(fmt, rows, hk, max(ctx))
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    P = b["num_pages"]
    q = oracle.f32_to_bf16(rng.standard_normal((rows, hq, d)).astype(np.float32))
    pools = {}
    for name in ("k_pages", "v_pages"):
        codes, scales, deq = oracle.kv_quant_rows(b[name].reshape(P * ps * hk, d), fmt)
        pools[name] = (codes.reshape(P, ps, hk, d), np.ascontiguousarray(scales.reshape(P, ps, hk).transpose(0, 2, 1)),
                       deq.reshape(P, ps, hk, d))
    begin, lens = b["page_indptr"][:-1].astype(np.int32), np.asarray(ctx, np.int32)
    o, _ = ops.attention_rows_paged_kvq(
        fmt, dev(q, gpu, torch.bfloat16), dev(pools["k_pages"][0], gpu), dev(pools["v_pages"][0], gpu),
        dev(pools["k_pages"][1], gpu), dev(pools["v_pages"][1], gpu), dev(b["page_indices"].view(np.int32), gpu),
        dev(begin, gpu), dev(lens, gpu), lse=True)
    torch.cuda.synchronize()
    truth, _, _ = oracle.attn_rows_f32kv(q, pools["k_pages"][2], pools["v_pages"][2], b["page_indices"],
                                         begin, lens, hq, hk, d, ps, mode=2)
    got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x tol"


def test_quantised_pool_argument_checks(gpu):
    import torch
    from pie_amd import ops

    q = torch.zeros((1, 8, 128), dtype=torch.bfloat16, device=gpu)
    pool = torch.zeros((2, 16, 2, 128), dtype=torch.uint8, device=gpu)
    idx = torch.zeros(1, dtype=torch.int32, device=gpu)
    one = torch.ones(1, dtype=torch.int32, device=gpu)
    with pytest.raises(ops.KernelError):   # per-token-head formats need their scales
        ops.attention_rows_paged_kvq("int8_per_token_head", q, pool, pool, None, None, idx, idx, one)
    sc = torch.ones((2, 16, 2), dtype=torch.float32, device=gpu)
    with pytest.raises(ops.KernelError):   # plain fp8 takes none
        ops.attention_rows_paged_kvq("fp8_e4m3", q, pool, pool, sc, sc, idx, idx, one)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("hq,hk,d,interleaved,qk_norm", [(8, 2, 128, True, False), (4, 4, 64, False, True),
                                                        (4, 1, 256, False, False), (6, 3, 96, True, True)])
def test_rope_and_quantising_write_in_one_launch_equal_the_two_kernels(gpu, oracle, fmt, hq, hk, d,
                                                                       interleaved, qk_norm):
    """RoPE + quantising KV write fused: q, codes and scales are the bytes of the rope kernel
    (into staged bf16 rows) followed by the quantising write (both pinned against the oracle)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(60 + hq + d)
    N, pages, ps = 21, 6, 16
    packed = dev(oracle.f32_to_bf16((rng.standard_normal((N, (hq + 2 * hk) * d)) * 3).astype(np.float32)), gpu,
                 torch.bfloat16)
    pos = rng.integers(0, 3000, N).astype(np.int32)
    tab = ops.rope_table(dev(pos, gpu), dev(oracle.rope_inv_freq(d, 500000.0), gpu), d)
    slots = rng.permutation(pages * ps)[:N].astype(np.int64)
    slots[2] = -1
    sg = dev(slots, gpu)
    qn = dev(oracle.f32_to_bf16(rng.uniform(0.5, 1.5, d).astype(np.float32)), gpu, torch.bfloat16) if qk_norm else None
    kn = dev(oracle.f32_to_bf16(rng.uniform(0.5, 1.5, d).astype(np.float32)), gpu, torch.bfloat16) if qk_norm else None
    scaled = fmt not in ("fp8_e4m3", "fp8_e5m2")

    def pools():
        kp = torch.full((pages, ps, hk, d), 0x55, dtype=torch.uint8, device=gpu)
        vp = torch.full((pages, ps, hk, d), 0x55, dtype=torch.uint8, device=gpu)
        ks = torch.full((pages, hk, ps), -7.0, dtype=torch.float32, device=gpu) if scaled else None
        vs = torch.full((pages, hk, ps), -7.0, dtype=torch.float32, device=gpu) if scaled else None
        return kp, vp, ks, vs

    a = pools()
    q1 = ops.qkv_rope_kvwrite_quant(fmt, packed, a[0], a[1], a[2], a[3], tab, sg, hq, hk, d, interleaved, qn, kn,
                                    eps=1e-6)
    # two kernels: rotated K / V as bf16 rows (row t in slot t), then the quantising write
    k_rows = torch.zeros((N, hk, d), dtype=torch.bfloat16, device=gpu)
    v_rows = torch.zeros((N, hk, d), dtype=torch.bfloat16, device=gpu)
    iota = dev(np.arange(N, dtype=np.int64), gpu)
    q2 = ops.qkv_rope_kvwrite(packed, k_rows, v_rows, tab, iota, hq, hk, d, interleaved, qn, kn, eps=1e-6)
    b = pools()
    ops.kv_write_quant(fmt, k_rows, v_rows, sg, b[0], b[1], b[2], b[3])
    torch.cuda.synchronize()
    assert torch.equal(q1.view(torch.int16), q2.view(torch.int16))
    for x, y in zip(a, b):
        if x is not None:
            assert torch.equal(x, y)
    assert not torch.all(a[0] == 0x55)


@pytest.mark.parametrize("hk,d", [(8, 128), (2, 64), (4, 256), (3, 48)])
def test_fp4_block_write_is_bit_exact_and_pages_expand_to_the_oracles_values(gpu, oracle, hk, d):
    """The 4-bit block format: codes (two per byte), block scales and the bf16 expansion of the
    written pages against the oracle's quantiser, bit for bit; pages the list does not name stay
    untouched."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(90 + hk + d)
    N, pages, ps = 41, 9, 16
    nb = d // 16
    k = oracle.f32_to_bf16((rng.standard_normal((N, hk, d)) * rng.uniform(0.05, 20, (N, hk, 1))).astype(np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal((N, hk, d)).astype(np.float32))
    k[3] = 0                                                   # an all-zero token
    v[7, :, 16:32] = 0                                         # an all-zero block
    slots = rng.permutation(pages * ps)[:N].astype(np.int64)
    slots[5] = -1                                              # a token without a slot
    kp = torch.full((pages, ps, hk, d // 2), 0x55, dtype=torch.uint8, device=gpu)
    vp = torch.full((pages, ps, hk, d // 2), 0x55, dtype=torch.uint8, device=gpu)
    ks = torch.full((pages, hk, ps, nb), -7.0, dtype=torch.float32, device=gpu)
    vs = torch.full((pages, hk, ps, nb), -7.0, dtype=torch.float32, device=gpu)
    for name in ("fp4_e2m1", "nvfp4"):
        ops.kv_write_quant(name, dev(k, gpu, torch.bfloat16), dev(v, gpu, torch.bfloat16), dev(slots, gpu),
                           kp, vp, ks, vs)
    torch.cuda.synchronize()
    deq = {}
    for tag, src, pool, sc in (("k", k, kp, ks), ("v", v, vp, vs)):
        codes, scales, dq = oracle.kv_quant_rows(src.reshape(N * hk, d), "nvfp4")
        want = np.full((pages * ps, hk, d // 2), 0x55, np.uint8)
        want_s = np.full((pages * ps, hk, nb), -7.0, np.float32)
        want_d = np.zeros((pages * ps, hk, d), np.float32)
        for t in range(N):
            if slots[t] >= 0:
                want[slots[t]] = codes.reshape(N, hk, d // 2)[t]
                want_s[slots[t]] = scales.reshape(N, hk, nb)[t]
                want_d[slots[t]] = dq.reshape(N, hk, d)[t]
        assert np.array_equal(pool.cpu().numpy().reshape(pages * ps, hk, d // 2), want)
        got_s = sc.cpu().numpy().transpose(0, 2, 1, 3).reshape(pages * ps, hk, nb)   # -> [slot, head, block]
        assert np.array_equal(got_s, want_s)
        deq[tag] = want_d
    # expansion of the pages that hold tokens (one of them named twice); the others keep their fill
    written = np.unique(slots[slots >= 0] // ps)
    ids = np.concatenate([written[:-1], written[:1]]).astype(np.int32)
    ko = torch.full((pages, ps, hk, d), 3.0, dtype=torch.bfloat16, device=gpu)
    vo = torch.full((pages, ps, hk, d), 3.0, dtype=torch.bfloat16, device=gpu)
    ops.kv_dequant_pages("nvfp4", kp, vp, ks, vs, ko, vo, dev(ids, gpu))
    torch.cuda.synchronize()
    mask = np.zeros(pages * ps, bool)
    mask[slots[slots >= 0]] = True
    for tag, out in (("k", ko), ("v", vo)):
        got = oracle.bf16_to_f32(out.view(torch.uint16).cpu().numpy()).reshape(pages * ps, hk, d)
        named = np.isin(np.arange(pages * ps) // ps, ids)
        assert np.array_equal(got[mask & named], deq[tag][mask & named])
        assert np.all(got[~named] == 3.0)


@pytest.mark.parametrize("fmt", FORMATS)
def test_page_expansion_of_one_byte_pools_is_code_times_scale_rounded_to_bf16(gpu, oracle, fmt):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(17)
    pages, ps, hk, d = 6, 16, 4, 128
    src = oracle.f32_to_bf16((rng.standard_normal((pages * ps * hk, d)) * 3).astype(np.float32))
    codes, scales, dq = oracle.kv_quant_rows(src, fmt)
    kp = dev(codes.reshape(pages, ps, hk, d), gpu)
    sc = None if scales is None else dev(np.ascontiguousarray(scales.reshape(pages, ps, hk).transpose(0, 2, 1)), gpu)
    ko = torch.zeros((pages, ps, hk, d), dtype=torch.bfloat16, device=gpu)
    vo = torch.zeros_like(ko)
    ids = dev(np.array([4, 0, 5, 2], np.int32), gpu)
    ops.kv_dequant_pages(fmt, kp, kp, sc, sc, ko, vo, ids)
    torch.cuda.synchronize()
    want = oracle.f32_to_bf16(dq).reshape(pages, ps, hk, d)
    got = ko.view(torch.uint16).cpu().numpy()
    for pg in (4, 0, 5, 2):
        assert np.array_equal(got[pg], want[pg])
    assert np.all(got[1] == 0) and np.all(got[3] == 0)
    assert np.array_equal(vo.view(torch.uint16).cpu().numpy(), got)
