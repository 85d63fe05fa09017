"""Pins for the oracle's KV-cache quantiser (driver/cuda/src/kernels/kv_paged.cu:155-297) and the
f32-pool attention it feeds: the reference test's own source pattern and bars
(driver/cuda/tests/test_kv_cache_quant.cu:34-40, :98-160, :230-262), independent numpy / torch
evaluations of the same rules, and hand-worked rounding cases."""
import numpy as np
import pytest
import torch

from paged_cases import make_paged_batch

FORMATS = ["fp8_e4m3", "int8_per_token_head", "fp8_per_token_head", "fp8_e5m2"]


def reference_source(value: bool):
    """source_value() of the reference test: 2 tokens x 2 heads x 17 dims."""
    t, h, d = np.meshgrid(np.arange(2), np.arange(2), np.arange(17), indexing="ij")
    sign = np.where((t + h + d + (1 if value else 0)) & 1, -1.0, 1.0)
    base = 0.03 * (d - 8) + 0.11 * (h + 1) + 0.17 * (t + 1)
    return (sign * base).astype(np.float32).reshape(4, 17)


def e4m3_qdq(x):
    """Saturating round-to-nearest-even e4m3fn through torch (independent of the oracle)."""
    t = torch.from_numpy(np.clip(x, -448.0, 448.0).astype(np.float32))
    return t.to(torch.float8_e4m3fn).to(torch.float32).numpy()


def e5m2_qdq(x):
    """Saturating round-to-nearest-even e5m2 through torch (independent of the oracle)."""
    t = torch.from_numpy(np.clip(x, -57344.0, 57344.0).astype(np.float32))
    return t.to(torch.float8_e5m2).to(torch.float32).numpy()


def independent_qdq(xf, fmt):
    """expected_qdq / expected_scale of the reference test, evaluated with numpy."""
    if fmt == "fp8_e4m3":
        return e4m3_qdq(xf), None
    if fmt == "fp8_e5m2":
        return e5m2_qdq(xf), None
    qmax = np.float32(127.0 if fmt.startswith("int8") else 448.0)
    amax = np.abs(xf).max(axis=1)
    scale = np.where(amax > 0, amax / qmax, np.float32(1.0)).astype(np.float32)
    if fmt.startswith("int8"):
        q = np.clip(np.rint(xf / scale[:, None]), -128, 127).astype(np.float32)
        return q * scale[:, None], scale
    return e4m3_qdq(xf / scale[:, None]) * scale[:, None], scale


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("value", [False, True])
def test_reference_pattern_within_reference_bars(oracle, fmt, value):
    x = oracle.f32_to_bf16(reference_source(value))
    xf = oracle.bf16_to_f32(x)
    codes, scales, deq = oracle.kv_quant_rows(x, fmt)
    want, want_scale = independent_qdq(xf, fmt)
    assert np.max(np.abs(deq - want)) <= 0.02          # the reference test's bar
    if want_scale is not None:
        assert np.max(np.abs(scales - want_scale)) <= 1e-5
        assert np.array_equal(scales, want_scale)      # same fp32 division
    else:
        assert scales is None


@pytest.mark.parametrize("fmt", FORMATS)
def test_codes_equal_an_independent_evaluation(oracle, fmt):
    """The kernel's exact arithmetic: x * (1 / scale) in fp32, then rint / the e4m3 cast."""
    rng = np.random.default_rng(11)
    x = oracle.f32_to_bf16((rng.standard_normal((64, 128)) * rng.uniform(0.01, 30, (64, 1))).astype(np.float32))
    xf = oracle.bf16_to_f32(x)
    codes, scales, deq = oracle.kv_quant_rows(x, fmt)
    if fmt == "fp8_e5m2":
        got = torch.from_numpy(codes.copy()).view(torch.float8_e5m2).to(torch.float32).numpy()
        assert scales is None and np.array_equal(got, e5m2_qdq(xf)) and np.array_equal(deq, got)
        return
    if fmt == "fp8_e4m3":
        scale = np.ones(64, np.float32)
    else:
        qmax = np.float32(127.0 if fmt.startswith("int8") else 448.0)
        scale = (np.abs(xf).max(axis=1) / qmax).astype(np.float32)
        assert np.array_equal(scales, scale)
    pre = xf * (np.float32(1.0) / scale)[:, None]
    if fmt.startswith("int8"):
        want = np.clip(np.rint(pre), -128, 127)
        assert np.array_equal(codes.view(np.int8).astype(np.float32), want)
        assert np.array_equal(deq, want.astype(np.float32) * scale[:, None])
        assert np.all(np.abs(codes.view(np.int8)).max(axis=1) == 127)     # the absmax element
    else:
        want = e4m3_qdq(pre)
        got = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
        assert np.array_equal(got, want)
        assert np.array_equal(deq, want * scale[:, None])
        if fmt == "fp8_per_token_head":
            assert np.all(np.abs(got).max(axis=1) == 448.0)


def test_hand_worked_rounding_and_zero_rows(oracle):
    # scale = 127 * 2^-7 / 127 = 2^-7 exactly; 2.5 and 3.5 steps round to even, -0.5 steps to -0
    row = np.array([127, 2.5, 3.5, -2.5, -0.5, 0.4375, 126.5, -127] + [0] * 8, np.float32) * 2.0 ** -7
    x = oracle.f32_to_bf16(np.stack([row, np.zeros(16, np.float32)]))
    assert np.array_equal(oracle.bf16_to_f32(x)[0], row)           # all exact in bf16
    codes, scales, deq = oracle.kv_quant_rows(x, "int8_per_token_head")
    assert scales[0] == 2.0 ** -7 and scales[1] == 1.0              # all-zero row: scale 1
    assert list(codes.view(np.int8)[0][:8]) == [127, 2, 4, -2, 0, 0, 126, -127]
    assert not codes[1].any() and not deq[1].any()
    codes, scales, _ = oracle.kv_quant_rows(x, "fp8_per_token_head")
    assert scales[0] == np.float32(127 * 2.0 ** -7) / np.float32(448.0) and scales[1] == 1.0
    assert codes[0][0] == 0x7E and codes[0][7] == 0xFE              # +-448
    # plain fp8: values beyond 448 saturate, NaN-free
    big = oracle.f32_to_bf16(np.array([[1000.0, -1000.0, 448.0, 0.0625, 0.0]], np.float32))
    codes, scales, deq = oracle.kv_quant_rows(big, "fp8_e4m3")
    assert scales is None and list(deq[0]) == [448.0, -448.0, 448.0, 0.0625, 0.0]


def test_attention_over_f32_pools_equals_dense_attention(oracle):
    """The f32-pool attention against numpy fp64 softmax attention over gathered rows, and
    against the bf16-pool oracle when the pools hold the same values."""
    rng = np.random.default_rng(5)
    hq, hk, d, ps = 8, 2, 64, 16
    ctx = [1, 17, 40, 0, 100]
    b = make_paged_batch(rng, ctx, hk, d, ps, f32_to_bf16=oracle.f32_to_bf16)
    q = oracle.f32_to_bf16(rng.standard_normal((len(ctx), hq, d)).astype(np.float32))
    kf, vf = oracle.bf16_to_f32(b["k_pages"]), oracle.bf16_to_f32(b["v_pages"])
    begin, lens = b["page_indptr"][:-1], np.asarray(ctx, np.int32)
    o32, _, lse = oracle.attn_rows_f32kv(q, kf, vf, b["page_indices"], begin, lens, hq, hk, d, ps)
    ref32, _, ref_lse = oracle.attn_rows_masked(q, b["k_pages"], b["v_pages"], b["page_indices"], begin,
                                                lens, hq, hk, d, ps, [None] * len(ctx), mode=2)
    assert np.array_equal(o32, ref32) and np.array_equal(lse, ref_lse)
    # a scaled pool: dense fp64 attention over the gathered dequantised rows
    kf2 = (kf * 0.37).astype(np.float32)
    o32, _, _ = oracle.attn_rows_f32kv(q, kf2, vf, b["page_indices"], begin, lens, hq, hk, d, ps)
    qf = oracle.bf16_to_f32(q).astype(np.float64)
    for r, n in enumerate(ctx):
        if n == 0:
            assert not o32[r].any()
            continue
        pages = b["page_indices"][int(begin[r]):int(begin[r]) + (n + ps - 1) // ps]
        K = kf2[pages].reshape(-1, hk, d)[:n].astype(np.float64)
        V = vf[pages].reshape(-1, hk, d)[:n].astype(np.float64)
        for h in range(hq):
            s = K[:, h // (hq // hk)] @ qf[r, h] / np.sqrt(d)
            p = np.exp(s - s.max())
            want = (p / p.sum()) @ V[:, h // (hq // hk)]
            assert np.allclose(o32[r, h], want, rtol=1e-6, atol=1e-6)


def test_e5m2_codes_against_torch(oracle):
    """Every e5m2 code decodes to torch's float8_e5m2 value; encoding is round-to-nearest-even
    with saturation at 57344 on ties, subnormals, the overflow edge and random values."""
    import ctypes as C

    codes = np.arange(256, dtype=np.uint8)
    dec = np.zeros(256, np.float32)
    oracle.lib().orc_fp8_e5m2_decode(C.c_void_p(codes.ctypes.data), C.c_void_p(dec.ctypes.data), C.c_size_t(256))
    want = torch.from_numpy(codes.copy()).view(torch.float8_e5m2).to(torch.float32).numpy()
    fin = np.isfinite(want)
    assert np.array_equal(dec[fin], want[fin]) and np.array_equal(np.isnan(dec), np.isnan(want))
    assert np.array_equal(np.isinf(dec), np.isinf(want))
    rng = np.random.default_rng(12)
    x = np.concatenate([rng.standard_normal(5000) * 10.0 ** rng.integers(-6, 5, 5000),
                        [0.0, 1.125, 1.375, -1.125, 2.0 ** -16, 2.0 ** -17, 3 * 2.0 ** -17, 57344.0, 61439.0, 1e9, -1e9,
                         2.0 ** -14, 1.5 * 2.0 ** -16]]).astype(np.float32)
    enc = np.zeros(x.size, np.uint8)
    oracle.lib().orc_fp8_e5m2_encode(C.c_void_p(x.ctypes.data), C.c_void_p(enc.ctypes.data), C.c_size_t(x.size))
    got = torch.from_numpy(enc).view(torch.float8_e5m2).to(torch.float32).numpy()
    assert np.array_equal(got, e5m2_qdq(x))
    assert got[-3] == -57344.0 and got[-4] == 57344.0   # saturated, never inf


# ---- 4-bit block format ("fp4_e2m1" / "nvfp4": e2m1 codes, one fp32 scale per 16 elements) ----
FP4_LEVELS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], np.float32)


def fp4_independent(xf):
    """write_kv_fp4_block_kernel restated with numpy: (codes [rows, d] unpacked, scales [rows, nb],
    bf16-rounded level * scale)."""
    rows, d = xf.shape
    nb = (d + 15) // 16
    codes = np.zeros((rows, d), np.uint8)
    scales = np.ones((rows, nb), np.float32)
    for b in range(nb):
        blk = xf[:, 16 * b:16 * b + 16]
        amax = np.abs(blk).max(axis=1)
        sc = np.where(amax > 0, amax / np.float32(6.0), np.float32(1.0)).astype(np.float32)
        scales[:, b] = sc
        y = (blk * (np.float32(1.0) / sc)[:, None]).astype(np.float32)
        err = np.abs(np.abs(y)[:, :, None] - FP4_LEVELS[None, None, :])
        mag = np.argmin(err, axis=2)          # first minimum: the smaller magnitude on a tie
        codes[:, 16 * b:16 * b + 16] = (mag | np.where(y < 0, 8, 0)).astype(np.uint8)
    lev = np.where(codes & 8, -FP4_LEVELS[codes & 7], FP4_LEVELS[codes & 7])
    sc_full = np.repeat(scales, 16, axis=1)[:, :d]
    return codes, scales, (lev * sc_full).astype(np.float32)


@pytest.mark.parametrize("name", ["fp4_e2m1", "nvfp4"])
@pytest.mark.parametrize("value", [False, True])
def test_fp4_reference_pattern_within_reference_bars(oracle, name, value):
    """The reference test's source pattern (17 dims: a full block and a one-element block) with
    its bars: 0.02 on the values, 1e-5 on the scales (test_kv_cache_quant.cu:128-139, :158-169)."""
    x = oracle.f32_to_bf16(reference_source(value))
    xf = oracle.bf16_to_f32(x)
    codes, scales, deq = oracle.kv_quant_rows(x, name)
    assert codes.shape == (4, 9) and scales.shape == (4, 2)
    want_codes, want_scales, want = fp4_independent(xf)
    # the reference test divides by the scale where the kernel multiplies by its reciprocal
    amax = np.stack([np.abs(xf[:, :16]).max(axis=1), np.abs(xf[:, 16:]).max(axis=1)], axis=1)
    assert np.max(np.abs(scales - amax / 6.0)) <= 1e-5
    assert np.max(np.abs(deq - want)) <= 0.02
    assert np.array_equal(scales, want_scales)


def test_fp4_codes_packing_and_dequant_equal_an_independent_evaluation(oracle):
    rng = np.random.default_rng(77)
    x = oracle.f32_to_bf16((rng.standard_normal((64, 128)) * rng.uniform(0.01, 30, (64, 1))).astype(np.float32))
    x[3] = 0                                           # an all-zero row: scale 1, codes 0
    x[5, 16:32] = 0                                    # an all-zero block inside a row
    xf = oracle.bf16_to_f32(x)
    codes, scales, deq = oracle.kv_quant_rows(x, "nvfp4")
    want_codes, want_scales, want = fp4_independent(xf)
    unpacked = np.stack([codes & 0xF, codes >> 4], axis=2).reshape(64, 128)   # even element in the low nibble
    assert np.array_equal(unpacked, want_codes)
    assert np.array_equal(scales, want_scales)
    assert np.all(scales[3] == 1.0) and np.all(codes[3] == 0) and scales[5, 1] == 1.0
    # dequantised values are bf16(level * scale)
    assert np.array_equal(deq, oracle.bf16_to_f32(oracle.f32_to_bf16(want)))
    # every block's largest magnitude maps to level 6 and comes back within one bf16 rounding
    top = np.abs(deq).reshape(64, 8, 16).max(axis=2)
    ref = np.abs(xf).reshape(64, 8, 16).max(axis=2)
    assert np.all(np.abs(top - ref) <= ref * 2.0 ** -8)


def test_fp4_hand_worked_levels_and_ties(oracle):
    """One block whose largest magnitude is 6 (scale exactly 1): every midpoint between two levels
    goes to the smaller magnitude, the sign bit follows x < 0, -0 keeps code 0."""
    vals = np.array([6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -0.75, -5.0, 5.5, 0.3, -0.0, 2.51, -6.0],
                    np.float32)
    x = oracle.f32_to_bf16(vals.reshape(1, 16))
    assert np.array_equal(oracle.bf16_to_f32(x).reshape(-1)[:8], vals[:8])   # all exact in bf16 except 0.3, 2.51
    codes, scales, deq = oracle.kv_quant_rows(x, "fp4_e2m1")
    assert scales.shape == (1, 1) and scales[0, 0] == 1.0
    got = np.stack([codes & 0xF, codes >> 4], axis=2).reshape(-1)
    want = [7, 0, 1, 2, 3, 4, 5, 6, 8 | 0, 8 | 1, 8 | 6, 7, 1, 0, 5, 8 | 7]
    assert list(got) == want
    assert list(deq.reshape(-1)[:8]) == [6.0, 0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0]
