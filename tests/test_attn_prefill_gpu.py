"""GPU parity: matrix-core prefill attention (tiles of query rows over paged KV) against the CPU
oracle's per-row attention and against the per-row kernel."""
import numpy as np
import pytest

from paged_cases import make_paged_batch

pytestmark = pytest.mark.gpu


def build_rows(b, ctx, chunks, tile_rows):
    """chunks[r] = (first position, count) of request r's query tokens -> row arrays + tiles."""
    row_begin, row_len, tiles = [], [], []
    for r, (p0, n) in enumerate(chunks):
        base = len(row_begin)
        for i in range(n):
            row_begin.append(int(b["page_indptr"][r]))
            row_len.append(min(ctx[r], p0 + i + 1))
        for t0 in range(0, n, tile_rows):
            tiles.append((base + t0, min(tile_rows, n - t0)))
    return (np.array(row_begin, np.int32), np.array(row_len, np.int32),
            np.array([t[0] for t in tiles], np.int32), np.array([t[1] for t in tiles], np.int32))


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("hq,hk,d,ps", [(8, 2, 128, 16), (8, 1, 128, 32), (4, 2, 64, 16), (4, 4, 64, 16),
                                        (32, 8, 128, 16), (8, 2, 128, 48)])
def test_tiles_match_oracle_and_row_kernel(gpu, oracle, hq, hk, d, ps, half):
    import torch

    from pie_amd import ops

    rng = np.random.default_rng(60 + hq + d)
    ctx = [200, 75, 33, 1]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    tr = ops.attn_prefill_tile_rows(hq, hk)
    assert tr == 128 // (hq // hk)
    if half:
        tr //= 2
    # a later chunk of a long prompt, a whole short prompt, a prompt shorter than a tile, one token
    chunks = [(120, 80), (0, 75), (0, 33), (0, 1)]
    row_begin, row_len, tile_start, tile_n = build_rows(b, ctx, chunks, tr)
    rows = len(row_begin)
    q = oracle.f32_to_bf16(rng.standard_normal((rows, hq, d)).astype(np.float32))
    dev = lambda a, dt=None: (lambda t: t.view(dt) if dt is not None else t)(
        torch.from_numpy(np.ascontiguousarray(a)).to(gpu))
    args = (dev(q, torch.bfloat16), dev(b["k_pages"], torch.bfloat16), dev(b["v_pages"], torch.bfloat16),
            dev(b["page_indices"].view(np.int32)), dev(row_begin), dev(row_len))
    o = ops.attention_prefill_tiles(*args, dev(tile_start), dev(tile_n), rows_per_tile=tr)
    torch.cuda.synchronize()
    got_bits = o.view(torch.uint16).cpu().numpy()
    got = oracle.bf16_to_f32(got_bits).astype(np.float64)
    truth, _, _ = oracle.attn_rows_masked(q, b["k_pages"], b["v_pages"], b["page_indices"], row_begin,
                                          row_len, hq, hk, d, ps, [None] * rows)
    # one bf16 rounding of the output + fp32 softmax / accumulation error: the decode kernels' bar
    # (the weights reach the second product as hi + lo bf16 pairs, 16 significant bits)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x tol at {np.unravel_index(np.argmax(err / tol), err.shape)}"
    row = ops.attention_rows_paged(*args, int(row_len.max())).view(torch.uint16).cpu().numpy()
    # against the per-row kernel (fp32 weights): the same bar, and mostly the same bf16 value
    # (ulp distances grow without bound for outputs near zero, so they are only counted)
    rowf = oracle.bf16_to_f32(row).astype(np.float64)
    assert np.all(np.abs(got - rowf) <= 2.0 ** -7 * np.maximum(np.abs(rowf), np.abs(got)) + 2e-4)
    ulp = np.abs(got_bits.astype(np.int32) - row.astype(np.int32))
    assert (ulp <= 1).mean() > 0.97


@pytest.mark.parametrize("fmt", ["fp8_e4m3", "int8_per_token_head", "fp8_per_token_head", "fp8_e5m2"])
@pytest.mark.parametrize("hq,hk,d,ps", [(8, 2, 128, 16), (4, 4, 64, 16), (32, 8, 128, 32)])
def test_tiles_over_one_byte_pools_match_the_oracle(gpu, oracle, fmt, hq, hk, d, ps):
    """The tile kernel over quantised pools against the oracle's attention over the dequantised
    values float(code) * scale (codes and scales written by the library's quantising write,
    itself bit-exact against the oracle's quantiser), to the bar of the bf16 pools; the per-row
    kernel over the same pools is compared as well."""
    import torch

    from pie_amd import ops

    rng = np.random.default_rng(70 + hq + d)
    ctx = [200, 75, 33, 1]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    tr = ops.attn_prefill_tile_rows(hq, hk)
    chunks = [(120, 80), (0, 75), (0, 33), (0, 1)]
    row_begin, row_len, tile_start, tile_n = build_rows(b, ctx, chunks, tr)
    rows = len(row_begin)
    q = oracle.f32_to_bf16(rng.standard_normal((rows, hq, d)).astype(np.float32))
    dev = lambda a, dt=None: (lambda t: t.view(dt) if dt is not None else t)(
        torch.from_numpy(np.ascontiguousarray(a)).to(gpu))
    # quantise the bf16 pools slot by slot with the library's own write kernel
    pages = b["k_pages"].shape[0]
    kp = torch.zeros((pages, ps, hk, d), dtype=torch.uint8, device=gpu)
    vp = torch.zeros_like(kp)
    scaled = fmt not in ("fp8_e4m3", "fp8_e5m2")
    ks = torch.ones((pages, hk, ps), dtype=torch.float32, device=gpu) if scaled else None
    vs = torch.ones((pages, hk, ps), dtype=torch.float32, device=gpu) if scaled else None
    slots = dev(np.arange(pages * ps, dtype=np.int64))
    ops.kv_write_quant(fmt, dev(b["k_pages"], torch.bfloat16).reshape(pages * ps, hk, d),
                       dev(b["v_pages"], torch.bfloat16).reshape(pages * ps, hk, d), slots, kp, vp, ks, vs)
    qd, pi, rb, rl = dev(q, torch.bfloat16), dev(b["page_indices"].view(np.int32)), dev(row_begin), dev(row_len)
    o = ops.attention_prefill_tiles_kvq(fmt, qd, kp, vp, ks, vs, pi, rb, rl, dev(tile_start), dev(tile_n),
                                        rows_per_tile=tr)
    ref = ops.attention_rows_paged_kvq(fmt, qd, kp, vp, ks, vs, pi, rb, rl)[0]
    torch.cuda.synchronize()
    got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
    # the oracle: its own quantiser on the same bf16 rows (the codes the GPU wrote, bit for bit),
    # attention in double over float(code) * scale
    deq = {}
    for name in ("k_pages", "v_pages"):
        codes, scales, dq = oracle.kv_quant_rows(b[name].reshape(pages * ps * hk, d), fmt)
        deq[name] = dq.reshape(pages, ps, hk, d)
        pool = (kp if name == "k_pages" else vp).cpu().numpy()
        assert np.array_equal(pool.reshape(-1, d), codes)
    truth, _, _ = oracle.attn_rows_f32kv(q, deq["k_pages"], deq["v_pages"], b["page_indices"], row_begin, row_len,
                                         hq, hk, d, ps, mode=2)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x tol"
    want = oracle.bf16_to_f32(ref.view(torch.uint16).cpu().numpy()).astype(np.float64)
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.maximum(np.abs(want), np.abs(got)) + 2e-4)
