"""GPU parity: paged-KV decode attention through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

from paged_cases import make_paged_batch

pytestmark = pytest.mark.gpu


def run_gpu(gpu, q, b, hq, hk, d, ps, max_kv_len, sm_scale=-1.0, want_lse=True):
    import torch

    from pie_amd import ops

    def dev(a, dt=None):
        t = torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
        return t.view(dt) if dt is not None else t

    R = q.shape[0]
    lse = torch.empty((R, hq), dtype=torch.float32, device=gpu) if want_lse else None
    o = ops.attention_paged_decode(
        dev(q, torch.bfloat16), dev(b["k_pages"], torch.bfloat16), dev(b["v_pages"], torch.bfloat16),
        dev(b["page_indices"].view(np.int32)), dev(b["page_indptr"].view(np.int32)),
        dev(b["last_lens"].view(np.int32)), max_kv_len, sm_scale=sm_scale, lse=lse)
    torch.cuda.synchronize()
    return o.view(torch.uint16).cpu().numpy(), (lse.cpu().numpy() if want_lse else None)


def check(oracle, o_bits, lse, q, b, hq, hk, d, ps, sm_scale=-1.0):
    truth, _, lse64 = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"],
                                               b["page_indptr"], b["last_lens"], hq, hk, d, ps,
                                               sm_scale=sm_scale, mode=2)
    got = oracle.bf16_to_f32(o_bits).astype(np.float64)
    # one bf16 rounding of the output + fp32 softmax/accumulation error (V ~ N(0,1))
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x tol at {np.argmax(err / tol)}"
    if lse is not None:
        fin = np.isfinite(lse64)
        assert np.array_equal(np.isneginf(lse), np.isneginf(lse64))
        assert np.allclose(lse[fin], lse64[fin], rtol=0, atol=1e-4)
    # and within 1 bf16 ulp of the reference-order fp32 evaluation almost everywhere
    _, o0, _ = oracle.attn_decode_paged(q, b["k_pages"], b["v_pages"], b["page_indices"],
                                        b["page_indptr"], b["last_lens"], hq, hk, d, ps,
                                        sm_scale=sm_scale, mode=0)
    dd = np.abs(o_bits.astype(np.int32) - o0.astype(np.int32))
    assert (dd <= 1).mean() > 0.99


@pytest.mark.parametrize("hq,hk,d,ps", [
    (32, 8, 128, 16), (8, 8, 128, 16), (16, 8, 128, 32), (32, 4, 128, 16),
    (32, 8, 64, 16), (8, 4, 64, 32), (4, 4, 64, 16), (16, 2, 64, 16),
])
def test_decode_matches_oracle_ragged(gpu, oracle, hq, hk, d, ps):
    rng = np.random.default_rng(hq * 1000 + hk * 100 + d + ps)
    ctx = [1, 15, 16, 17, 31, 33, 64, 100, 257, 0, 1000, 5]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    o, lse = run_gpu(gpu, q, b, hq, hk, d, ps, max(ctx))
    check(oracle, o, lse, q, b, hq, hk, d, ps)


@pytest.mark.parametrize("max_kv_len", [64, 1024, 4096, 8192, 100000])
def test_split_plans_agree(gpu, oracle, max_kv_len):
    """Different max_kv_len bounds pick different split grids; the result must not depend on it
    beyond fp32 merge rounding."""
    rng = np.random.default_rng(31)
    hq, hk, d, ps = 32, 8, 128, 16
    ctx = [64, 1, 40, 17]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    o, lse = run_gpu(gpu, q, b, hq, hk, d, ps, max_kv_len)
    check(oracle, o, lse, q, b, hq, hk, d, ps)


def test_single_request_long_context_and_scale(gpu, oracle):
    rng = np.random.default_rng(32)
    hq, hk, d, ps = 32, 8, 128, 16
    ctx = [2048 + 7]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((1, hq, d)).astype(np.float32))
    for scale in (-1.0, 0.05, 0.25):
        o, lse = run_gpu(gpu, q, b, hq, hk, d, ps, ctx[0], sm_scale=scale)
        check(oracle, o, lse, q, b, hq, hk, d, ps, sm_scale=scale)


def test_forked_prefix_equals_private_copies(gpu, oracle):
    rng = np.random.default_rng(33)
    hq, hk, d, ps = 32, 8, 128, 16
    ctx = [1024 + 300, 1024 + 5, 1024, 700, 1500, 1024 + 64, 90, 2000]
    b = make_paged_batch(rng, ctx, hk, d, ps, shared_prefix_tokens=1024, shared_fraction=0.5,
                         f32_to_bf16=oracle.f32_to_bf16)
    assert len(b["sharers"]) == 4
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    o, lse = run_gpu(gpu, q, b, hq, hk, d, ps, max(ctx))
    check(oracle, o, lse, q, b, hq, hk, d, ps)
    # private copies at other physical pages: bit-identical output
    total = int(b["page_indptr"][-1])
    perm = rng.permutation(total + 5).astype(np.uint32)[:total]
    b2 = dict(b)
    b2["k_pages"] = np.zeros((total + 5, ps, hk, d), np.uint16)
    b2["v_pages"] = np.zeros_like(b2["k_pages"])
    b2["k_pages"][perm] = b["k_pages"][b["page_indices"]]
    b2["v_pages"][perm] = b["v_pages"][b["page_indices"]]
    b2["page_indices"] = perm
    o2, _ = run_gpu(gpu, q, b2, hq, hk, d, ps, max(ctx))
    assert np.array_equal(o, o2)


def test_garbage_in_unused_slots_is_ignored(gpu, oracle):
    """Slots past kv_len in the last page may hold NaN/Inf bit patterns."""
    rng = np.random.default_rng(34)
    hq, hk, d, ps = 8, 2, 128, 16
    ctx = [21, 3]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((2, hq, d)).astype(np.float32))
    o_clean, _ = run_gpu(gpu, q, b, hq, hk, d, ps, 32)
    for r, c in enumerate(ctx):
        last_page = b["page_indices"][b["page_indptr"][r + 1] - 1]
        b["k_pages"][last_page, c % ps:] = 0x7FC0  # NaN
        b["v_pages"][last_page, c % ps:] = 0x7F80  # +Inf
    o, lse = run_gpu(gpu, q, b, hq, hk, d, ps, 32)
    assert np.array_equal(o, o_clean)
    assert np.all(np.isfinite(lse))


def test_baseline_shape_batch64(gpu, oracle):
    """BASELINE attention config: 32q/8kv d128 page 16, batch 64, ctx U[512,8192], 25% of the
    sequences share a forked 1024-token prefix.  Oracle on a sample of requests (fp64), plus
    the forked-prefix and LSE invariants on all."""
    rng = np.random.default_rng(35)
    hq, hk, d, ps = 32, 8, 128, 16
    ctx = rng.integers(512, 8193, size=64)
    ctx[:16] = np.maximum(ctx[:16], 1024)
    b = make_paged_batch(rng, ctx, hk, d, ps, shared_prefix_tokens=1024, shared_fraction=0.25,
                         f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((64, hq, d)).astype(np.float32))
    o, lse = run_gpu(gpu, q, b, hq, hk, d, ps, int(ctx.max()))
    check(oracle, o, lse, q, b, hq, hk, d, ps)


def test_back_to_back_calls_share_workspace(gpu, oracle):
    """Calls queued in a row over one workspace, with different inputs and different split
    grids, must each give their own result (no partial of an earlier call is picked up)."""
    import torch

    from pie_amd import ops

    hq, hk, d, ps = 32, 8, 128, 16
    cases = []
    for seed, ctx in [(41, [700, 33, 1500, 0, 260]), (42, [2048]), (43, [90, 900, 64, 1024, 17, 300])]:
        rng = np.random.default_rng(seed)
        b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
        q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
        ref, _ = run_gpu(gpu, q, b, hq, hk, d, ps, max(ctx), want_lse=False)
        check(oracle, ref, None, q, b, hq, hk, d, ps)
        dev = lambda a, dt=None: (lambda t: t.view(dt) if dt is not None else t)(
            torch.from_numpy(np.ascontiguousarray(a)).to(gpu))
        cases.append((ref, max(ctx), dev(q, torch.bfloat16), dev(b["k_pages"], torch.bfloat16),
                      dev(b["v_pages"], torch.bfloat16), dev(b["page_indices"].view(np.int32)),
                      dev(b["page_indptr"].view(np.int32)), dev(b["last_lens"].view(np.int32))))
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=gpu)
    outs = []
    for it in range(30):   # queued back to back, no host synchronisation in between
        ref, mx, q, k, v, pi, pp, ll = cases[it % 3]
        outs.append((it, ops.attention_paged_decode(q, k, v, pi, pp, ll, mx, workspace=ws)))
    torch.cuda.synchronize()
    for it, o in outs:
        assert np.array_equal(o.view(torch.uint16).cpu().numpy(), cases[it % 3][0]), it


@pytest.mark.parametrize("hq,hk,d", [(8, 2, 128), (4, 4, 64)])
def test_rows_with_custom_masks_match_oracle(gpu, oracle, hq, hk, d):
    """Per-row extents with BRLE masks and a sliding window: visible keys only, rows with no
    visible key give zeros, unmasked rows equal the unmasked entry point."""
    import torch

    from pie_amd import ops

    rng = np.random.default_rng(55 + d)
    ps = 16
    ctx = [300, 77, 1100]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    # rows: (request, position)
    rows = [(0, 299), (0, 150), (1, 76), (1, 10), (2, 1099), (2, 600), (2, 0), (0, 40)]
    runs = [[], [10, 50, 20, 1000], [0, 1, 70, 6], [11, 5], [500, 1, 300, 299], [0, 601], [1, 4], [0, 3, 30, 8]]
    row_begin = np.array([b["page_indptr"][r] for r, _ in rows], np.int32)
    row_len = np.array([p + 1 for _, p in rows], np.int32)
    q = oracle.f32_to_bf16(rng.standard_normal((len(rows), hq, d)).astype(np.float32))
    dev = lambda a, dt=None: (lambda t: t.view(dt) if dt is not None else t)(
        torch.from_numpy(np.ascontiguousarray(a)).to(gpu))
    args = (dev(q, torch.bfloat16), dev(b["k_pages"], torch.bfloat16), dev(b["v_pages"], torch.bfloat16),
            dev(b["page_indices"].view(np.int32)), dev(row_begin), dev(row_len), int(row_len.max()))
    for window in (0, 64):
        lse = torch.empty((len(rows), hq), dtype=torch.float32, device=gpu)
        o = ops.attention_rows_paged(*args, mask_runs=runs, window=window, lse=lse)
        torch.cuda.synchronize()
        got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
        allow = [oracle.brle_allow(runs[i], rows[i][1], int(row_len[i]), window) for i in range(len(rows))]
        truth, _, lse64 = oracle.attn_rows_masked(q, b["k_pages"], b["v_pages"], b["page_indices"],
                                                  row_begin, row_len, hq, hk, d, ps, allow)
        tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4
        assert np.all(np.abs(got - truth) <= tol)
        fin = np.isfinite(lse64)
        lg = lse.cpu().numpy()
        assert np.array_equal(np.isneginf(lg), ~fin) and np.allclose(lg[fin], lse64[fin], atol=1e-4)
        assert not allow[3].any() and np.all(got[3] == 0)          # runs end before any visible key
    # no masks, no window: the unmasked entry point's result (that one runs the matrix-core
    # kernel, the masked one the dot-product kernel: same values to a bf16 step)
    plain = ops.attention_rows_paged(*args).view(torch.uint16).cpu().numpy().astype(np.int32)
    masked = ops.attention_rows_paged(*args, mask_runs=[[]] * len(rows)).view(torch.uint16).cpu().numpy().astype(np.int32)
    same_sign = (plain >> 15) == (masked >> 15)
    assert (np.abs(plain - masked)[same_sign] <= 1).mean() > 0.99
    pf, mf = oracle.bf16_to_f32(plain.astype(np.uint16)), oracle.bf16_to_f32(masked.astype(np.uint16))
    assert np.all(np.abs(pf - mf) <= 2.0 ** -7 * np.maximum(np.abs(pf), np.abs(mf)) + 2e-4)


@pytest.mark.parametrize("ctx_kind", ["equal", "ragged"])
@pytest.mark.parametrize("rows,hq,hk,d", [(64, 32, 8, 128), (32, 16, 8, 64), (64, 32, 4, 128), (16, 32, 8, 128), (24, 16, 8, 128)])
def test_rows_declared_equally_long_take_one_round_and_match_the_oracle(gpu, oracle, rows, hq, hk, d, ctx_kind):
    """pie_hip_attn_rows_paged_kvq_uniform: a batch of about equal contexts plans one round of blocks
    (64 rows x 8 kv heads: one block per row and head, no merge; 16 or 24 rows: one block of eight waves
    per row and head); the hint only changes the plan, so a
    ragged batch given it by mistake, empty row included, still comes out right."""
    import torch

    from pie_amd import ops

    ps = 16
    rng = np.random.default_rng(rows + hq + d)
    ctx = [int(c) for c in (rng.integers(600, 641, size=rows) if ctx_kind == "equal"
                            else rng.integers(0, 1300, size=rows))]
    if ctx_kind == "ragged":
        ctx[0], ctx[1] = 1290, 0
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((rows, hq, d)).astype(np.float32))

    def dev(a, dt=None):
        t = torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
        return t.view(dt) if dt is not None else t

    begin, lens = b["page_indptr"][:-1].astype(np.int32), np.asarray(ctx, np.int32)
    args = ("bf16", dev(q, torch.bfloat16), dev(b["k_pages"], torch.bfloat16), dev(b["v_pages"], torch.bfloat16),
            None, None, dev(b["page_indices"].view(np.int32)), dev(begin), dev(lens))
    o, lse = ops.attention_rows_paged_kvq(*args, lse=True, uniform=True)
    o_plain, _ = ops.attention_rows_paged_kvq(*args, lse=True)
    torch.cuda.synchronize()
    check(oracle, o.view(torch.uint16).cpu().numpy(), lse.cpu().numpy(), q, b, hq, hk, d, ps)
    # the two plans differ by the rounding of the split merge only
    a0 = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy())
    a1 = oracle.bf16_to_f32(o_plain.view(torch.uint16).cpu().numpy())
    assert np.all(np.abs(a0 - a1) <= 2.0 ** -7 * np.maximum(np.abs(a0), np.abs(a1)) + 1e-4)
