"""GPU test of the attention entry point that allocates nothing
(`pie_hip_attn_rows_paged_static`): through the C ABI, against `pie_hip_attn_rows_paged` on the
same inputs, bit for bit (same kernels, the split partials in the library's built-in scratch
array instead of a caller workspace), and against the CPU oracle; two calls in a row, the second
with a smaller batch, so stale partials of the first call must not leak into the second."""
import numpy as np
import pytest

from paged_cases import make_paged_batch

pytestmark = pytest.mark.gpu


def _case(gpu, oracle, seed, ctx, hq, hk, d, ps):
    import torch

    rng = np.random.default_rng(seed)
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    dev = lambda a, dt=None: (lambda t: t.view(dt) if dt is not None else t)(
        torch.from_numpy(np.ascontiguousarray(a)).to(gpu))
    row_begin = b["page_indptr"][:-1].astype(np.int32)
    row_len = np.asarray(ctx, np.int32)
    args = (dev(q, torch.bfloat16), dev(b["k_pages"], torch.bfloat16), dev(b["v_pages"], torch.bfloat16),
            dev(b["page_indices"].view(np.int32)), dev(row_begin), dev(row_len), int(max(ctx)))
    return q, b, row_begin, row_len, args


def test_static_scratch_entry_point_matches_workspace_entry_point(gpu, oracle):
    import torch

    from pie_amd import ops

    hq, hk, d, ps = 32, 8, 128, 16
    big = _case(gpu, oracle, 71, [1500, 33, 2048, 0, 700, 4100, 260, 16], hq, hk, d, ps)
    small = _case(gpu, oracle, 72, [300, 90], hq, hk, d, ps)
    # both need split partials (more than one split), the first more than the second
    need = [ops.attn_decode_workspace_bytes(len(c[3]), hq, hk, d, c[4][6]) for c in (big, small)]
    assert need[0] > need[1] > 0 and need[0] <= ops.ATTN_STATIC_SCRATCH_BYTES
    outs = []
    for q, b, row_begin, row_len, args in (big, small):
        o = torch.empty_like(args[0])
        lse = torch.empty((len(row_len), hq), dtype=torch.float32, device=gpu)
        ops.attention_rows_paged_static(*args, o=o, lse=lse)     # queued back to back
        outs.append((o, lse))
    torch.cuda.synchronize()
    for (q, b, row_begin, row_len, args), (o, lse) in zip((big, small), outs):
        lse_ref = torch.empty_like(lse)
        ref = ops.attention_rows_paged(*args, lse=lse_ref)
        torch.cuda.synchronize()
        assert torch.equal(o.view(torch.uint16), ref.view(torch.uint16))
        assert torch.equal(lse.view(torch.int32), lse_ref.view(torch.int32))
        allow = [np.ones(int(n), np.uint8) for n in row_len]
        truth, _, lse64 = oracle.attn_rows_masked(q, b["k_pages"], b["v_pages"], b["page_indices"],
                                                  row_begin, row_len, hq, hk, d, ps, allow)
        got = oracle.bf16_to_f32(o.view(torch.uint16).cpu().numpy()).astype(np.float64)
        tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 1e-4   # one bf16 rounding + fp32 softmax
        assert np.all(np.abs(got - truth) <= tol)
        fin = np.isfinite(lse64)
        assert np.allclose(lse.cpu().numpy()[fin], lse64[fin], atol=1e-4)


def test_static_scratch_entry_point_refuses_oversized_batches(gpu):
    import torch

    from pie_amd import ops

    hq, hk, d, ps = 64, 8, 128, 16
    rows = 380   # two splits: 380 rows x 64 heads x 2 x 130 floats = 25 MB exceed the 16 MiB array
    assert ops.attn_decode_workspace_bytes(rows, hq, hk, d, 4096) > ops.ATTN_STATIC_SCRATCH_BYTES
    q = torch.zeros((rows, hq, d), dtype=torch.bfloat16, device=gpu)
    pool = torch.zeros((4, ps, hk, d), dtype=torch.bfloat16, device=gpu)
    idx = torch.zeros(256, dtype=torch.int32, device=gpu)
    rb = torch.zeros(rows, dtype=torch.int32, device=gpu)
    rl = torch.ones(rows, dtype=torch.int32, device=gpu)
    with pytest.raises(ops.KernelError, match="unsupported"):
        ops.attention_rows_paged_static(q, pool, pool, idx, rb, rl, 4096, o=torch.empty_like(q))
