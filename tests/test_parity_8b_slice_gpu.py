"""GPU parity at the real shape: slices of the Llama-3-8B-shaped W4A16 decoder (hidden 4096, FFN
14336, 32 q / 8 kv heads of 128, vocab 128256, group 128) with contexts of about 512 tokens.

Three evaluations of the same decode step start from the same KV state (the GPU's prefill,
copied into the oracle's pools): the driver on the GPU, the oracle with the bf16 rounding points
("mode C"), and the oracle in double precision ("f64", the value both approximate).  The bar is
relative to the truth: the GPU may deviate from it by no more than 1.5 times what the mode-C
oracle itself deviates (1 - cosine of the logits), so a difference between GPU and oracle that
grows with depth is accepted only as far as it is rounding noise shared by both.  Tokens must
agree with the truth wherever its top-2 gap exceeds the measured deviation.

The batches are forked contexts: every request reads a prefix of the same prefilled pages in
place (different prefix lengths, so ragged) and writes its own tail page, each with its own
token — no two rows of a batch are alike."""
import numpy as np
import pytest

from driver_util import cosine, full_cfg, oracle_model_from_driver, toml_config

pytestmark = pytest.mark.gpu

SHAPE = dict(arch="llama3", hidden=4096, q_heads=32, kv_heads=8, head_dim=128, intermediate=14336,
             vocab=128256, quant="int4b8", group_size=128, page_size=16)
PREFIX_PAGES = 32      # 512 tokens


def _forked_batch(drvmod, rng, vocab, R, step, tokens_prev=None):
    """Request r reads the first (PREFIX_PAGES - r % 4) shared pages and its own tail page
    PREFIX_PAGES + r; at `step` it appends one token at position prefix_len + step."""
    toks = rng.integers(0, vocab, R) if tokens_prev is None else tokens_prev
    pages, indptr, last, pos = [], [0], [], []
    for r in range(R):
        npre = PREFIX_PAGES - r % 4
        pages += list(range(npre)) + [PREFIX_PAGES + r]
        indptr.append(len(pages))
        last.append(step + 1)
        pos.append(npre * 16 + step)
    return dict(token_ids=toks, position_ids=pos, kv_page_indices=pages, kv_page_indptr=indptr,
                kv_last_page_lens=last, qo_indptr=np.arange(R + 1))


def _setup(oracle, drvmod, layers, rows, seed):
    # (a forked batch names the shared pages once per request: the executor takes up to
    # 4 * total_pages + max_forward_tokens page references per forward)
    kw = dict(SHAPE, layers=layers, total_pages=max(PREFIX_PAGES + rows + 1, 8 * rows), max_forward_tokens=512,
              max_forward_requests=max(rows, 1), seed=seed)
    cfg = full_cfg(**kw)
    d = drvmod.Driver(toml_config(**kw))
    om, _ = oracle_model_from_driver(d, cfg)
    rng = np.random.default_rng(seed)
    n = PREFIX_PAGES * 16
    prompt = rng.integers(0, cfg["vocab"], n)
    d.forward(drvmod.ForwardFrame(prompt, np.arange(n), np.arange(PREFIX_PAGES), [0, PREFIX_PAGES], [16], [0, n]))
    # the GPU's prefilled pages become everybody's starting state
    shape = om.k_pages[0].shape
    for l in range(layers):
        om.k_pages[l][:] = d.export_tensor(f"kv.k.{l}", np.uint16).reshape(shape)
        om.v_pages[l][:] = d.export_tensor(f"kv.v.{l}", np.uint16).reshape(shape)
    return d, om, cfg, rng


def _dev(a, t):
    """1 - cosine per row."""
    a, t = a.astype(np.float64), t.astype(np.float64)
    return 1.0 - np.sum(a * t, axis=1) / (np.linalg.norm(a, axis=1) * np.linalg.norm(t, axis=1))


@pytest.mark.parametrize("rows", [1, 16])
def test_four_layer_slice_is_as_close_to_the_truth_as_the_oracle(gpu, oracle, rows):
    from pie_amd import driver as drvmod

    d, om, cfg, rng = _setup(oracle, drvmod, 4, rows, 811 + rows)
    try:
        om.seed_hp_pools("f64")
        V = cfg["vocab"]
        toks = None
        worst_g = worst_c = 0.0
        for step in range(3 if rows == 1 else 2):
            args = _forked_batch(drvmod, rng, V, rows, step, toks)
            res = d.forward(drvmod.ForwardFrame(**args))
            lg = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:rows])
            _, lc, _ = om.forward(**args, want_logits=True)
            lc = oracle.bf16_to_f32(lc)
            ttok, lt, _ = om.forward_hp("f64", **args)
            dg, dc = _dev(lg, lt), _dev(lc, lt)
            # the bar: no further from the truth than 1.5 x the mode-C oracle's own distance
            # (per row, with the batch mean as the floor for rows where the oracle got lucky)
            assert np.all(dg <= 1.5 * np.maximum(dc, dc.mean())), (step, dg, dc)
            assert dg.mean() <= 1.5 * dc.mean()
            assert np.all(dg < 3e-4) and np.all(dc < 3e-4)     # four layers of bf16 noise, not more
            assert np.all(_dev(lg, lc) < 4e-4)
            worst_g, worst_c = max(worst_g, dg.max()), max(worst_c, dc.max())
            for r in range(rows):
                top2 = np.sort(lt[r])[-2:]
                if top2[1] - top2[0] > 2.0 * np.max(np.abs(lg[r] - lt[r])):
                    assert res.tokens[r] == int(ttok[r]), (step, r)
                assert res.tokens[r] == int(np.argmax(lg[r]))
            toks = np.asarray(ttok, np.uint32)   # everybody continues with the truth's tokens
        print(f"rows {rows}: worst 1-cos vs f64: gpu {worst_g:.2e}, oracle-C {worst_c:.2e}")
    finally:
        d.close()


def test_two_layer_slice_at_64_rows_matches_the_oracle(gpu, oracle):
    """A 64-row decode batch at the 8B width (four side-by-side skinny-GEMM passes, matrix-core
    decode attention over 64 forked ragged contexts) against the mode-C oracle, every row."""
    from pie_amd import driver as drvmod

    rows = 64
    d, om, cfg, rng = _setup(oracle, drvmod, 2, rows, 877)
    try:
        V = cfg["vocab"]
        args = _forked_batch(drvmod, rng, V, rows, 0)
        res = d.forward(drvmod.ForwardFrame(**args))
        lg = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:rows])
        otok, lc, _ = om.forward(**args, want_logits=True)
        lc = oracle.bf16_to_f32(lc)
        assert np.all(_dev(lg, lc) < 1e-4)
        assert np.max(np.abs(lg - lc)) <= 0.02 * np.max(np.abs(lc))
        for r in range(rows):
            top2 = np.sort(lc[r])[-2:]
            if top2[1] - top2[0] > 2.0 ** -6 * abs(top2[1]):
                assert res.tokens[r] == int(otok[r]), r
        # rows are not permuted: each row is far closer to its own oracle row than to any other
        cross = _dev(lg[:-1], lc[1:])
        assert np.all(cross > 100 * _dev(lg, lc).max())
    finally:
        d.close()


def test_full_depth_decode_is_as_close_to_the_truth_as_the_oracle(gpu, oracle):
    """All 32 layers of the 8B-shaped W4A16 decoder (the benchmark's headline model), batch 1:
    three decode steps from a 512-token context evaluated three ways from the same KV state.
    1 - cosine grows linearly with depth for any bf16 pipeline (about 1e-3 at 32 layers), so
    the bar is the three-way one: the GPU is no further from the double-precision logits than
    1.5 times the mode-C oracle's own distance; tokens agree with the truth wherever its top-2
    gap exceeds twice the GPU's largest logit deviation."""
    from pie_amd import driver as drvmod

    d, om, cfg, rng = _setup(oracle, drvmod, 32, 1, 907)
    try:
        om.seed_hp_pools("f64")
        V = cfg["vocab"]
        toks = None
        rep = []
        for step in range(3):
            args = _forked_batch(drvmod, rng, V, 1, step, toks)
            res = d.forward(drvmod.ForwardFrame(**args))
            lg = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:1])
            _, lc, _ = om.forward(**args, want_logits=True)
            lc = oracle.bf16_to_f32(lc)
            ttok, lt, _ = om.forward_hp("f64", **args)
            dg, dc = float(_dev(lg, lt)[0]), float(_dev(lc, lt)[0])
            rep.append((dg, dc, float(_dev(lg, lc)[0])))
            assert dg <= 1.5 * dc, (step, dg, dc)
            assert dg < 3e-3 and dc < 3e-3             # 32 layers of bf16 noise, not more
            assert rep[-1][2] < 3e-3
            top2 = np.sort(lt[0])[-2:]
            if top2[1] - top2[0] > 2.0 * np.max(np.abs(lg[0] - lt[0])):
                assert res.tokens[0] == int(ttok[0]), step
            assert res.tokens[0] == int(np.argmax(lg[0]))
            toks = np.asarray(ttok, np.uint32)
        print("32 layers, per step (gpu vs f64, oracle-C vs f64, gpu vs oracle-C) 1-cos:",
              [tuple(f"{v:.2e}" for v in r) for r in rep])
    finally:
        d.close()
