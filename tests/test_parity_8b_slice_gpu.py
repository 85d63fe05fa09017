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


def test_prefill_at_the_8b_width_matches_the_oracles_own_prefill(gpu, oracle):
    """The prefill path at the real width (tiled matrix-core GEMMs over hidden 4096 / FFN 14336,
    tile attention over 32 q / 8 kv heads of 128): a ragged 200-token prompt through two layers,
    against the mode-C oracle prefilling the same prompt itself — last-token logits, and the K / V
    pages both left behind (layer 0: projection + rotation of identical inputs; layer 1: one layer
    of rounding noise), then one decode step on top of each side's own pages."""
    from pie_amd import driver as drvmod

    layers, n = 2, 200
    kw = dict(SHAPE, layers=layers, total_pages=16, max_forward_tokens=256, max_forward_requests=1, seed=931)
    cfg = full_cfg(**kw)
    V = cfg["vocab"]
    rng = np.random.default_rng(931)
    prompt = rng.integers(0, V, n)
    npg = (n + 15) // 16
    frame = dict(token_ids=prompt, position_ids=np.arange(n), kv_page_indices=np.arange(npg),
                 kv_page_indptr=[0, npg], kv_last_page_lens=[n - (npg - 1) * 16], qo_indptr=[0, n])
    with drvmod.Driver(toml_config(**kw)) as d:
        om, _ = oracle_model_from_driver(d, cfg)
        res = d.forward(drvmod.ForwardFrame(**frame))
        lg = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:1])
        otok, lc, _ = om.forward(**frame, want_logits=True)
        lc = oracle.bf16_to_f32(lc)
        assert _dev(lg, lc)[0] < 1e-4
        assert np.max(np.abs(lg - lc)) <= 0.02 * np.max(np.abs(lc))
        top2 = np.sort(lc[0])[-2:]
        if top2[1] - top2[0] > 4.0 * np.sqrt(np.mean((lg - lc) ** 2)):
            assert res.tokens[0] == int(otok[0])
        shape = om.k_pages[0].shape
        used = n * shape[2] * shape[3]
        for l in range(layers):
            for name, pool in (("k", om.k_pages[l]), ("v", om.v_pages[l])):
                g = oracle.bf16_to_f32(d.export_tensor(f"kv.{name}.{l}", np.uint16).reshape(shape)).reshape(-1)[:used]
                o = oracle.bf16_to_f32(pool).reshape(-1)[:used]
                same = float(np.mean(g == o))
                dv = float(_dev(g[None], o[None])[0])
                print(f"layer {l} {name}: {same:.4f} of the stored values bit-equal, 1 - cos {dv:.2e}")
                # (layer 0: the norm's summation order and the tiled GEMM's weights-to-bf16-first
                # evaluation separate the two by at most a bf16 step; layer 1 sits behind a whole
                # layer of bf16 rounding points)
                assert same > (0.9 if l == 0 else 0.15), (l, name, same)
                assert dv < (1e-5 if l == 0 else 5e-5), (l, name)
        # one decode step on each side's own pages
        step = dict(token_ids=[int(otok[0])], position_ids=[n], kv_page_indices=np.arange(npg),
                    kv_page_indptr=[0, npg], kv_last_page_lens=[n + 1 - (npg - 1) * 16], qo_indptr=[0, 1])
        d.forward(drvmod.ForwardFrame(**step))
        lg = oracle.bf16_to_f32(d.export_tensor("debug.logits", np.uint16).reshape(-1, V)[:1])
        _, lc, _ = om.forward(**step, want_logits=True)
        assert _dev(lg, oracle.bf16_to_f32(lc))[0] < 1e-4
