"""Pins for the oracle's per-layer ops (CPU only): textbook closed forms in numpy fp64,
rotation identities, tie rules, literal cases."""
import numpy as np
import pytest


def bf(oracle, x):
    return oracle.f32_to_bf16(np.asarray(x, np.float32))


def test_embed_rows_and_out_of_vocab(oracle):
    tab = np.arange(5 * 8, dtype=np.uint16).reshape(5, 8)
    y = oracle.embed(np.array([3, 0, 4, 7, 2 ** 31], np.uint32), tab)
    assert np.array_equal(y[0], tab[3]) and np.array_equal(y[2], tab[4])
    assert np.array_equal(y[3], tab[0]) and np.array_equal(y[4], tab[0])  # embed.cu:16


def test_rmsnorm_closed_form(oracle):
    rng = np.random.default_rng(40)
    x = bf(oracle, rng.standard_normal((5, 96)) * 3)
    w = bf(oracle, rng.standard_normal(96))
    y = oracle.bf16_to_f32(oracle.rmsnorm(x, w, 1e-5))
    xf = oracle.bf16_to_f32(x).astype(np.float64)
    ref = xf / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-5) * oracle.bf16_to_f32(w)
    assert np.all(np.abs(y - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-7)
    # scale invariance of the direction: rmsnorm(4x) == rmsnorm(x) up to eps
    y4 = oracle.bf16_to_f32(oracle.rmsnorm(bf(oracle, oracle.bf16_to_f32(x) * 4), w, 0.0))
    y1 = oracle.bf16_to_f32(oracle.rmsnorm(x, w, 0.0))
    assert np.array_equal(y4, y1)
    # literal: x = [3, 4] -> rms = sqrt(12.5); w = 1
    lit = oracle.bf16_to_f32(oracle.rmsnorm(bf(oracle, [[3, 4]]), bf(oracle, [1, 1]), 0.0))
    assert np.allclose(lit, [[3 / np.sqrt(12.5), 4 / np.sqrt(12.5)]], rtol=2 ** -8)


def test_residual_rmsnorm_rounds_the_sum_first(oracle):
    rng = np.random.default_rng(41)
    x = bf(oracle, rng.standard_normal((3, 64)))
    r = bf(oracle, rng.standard_normal((3, 64)))
    w = bf(oracle, np.ones(64))
    y, h = oracle.rmsnorm(x, w, 1e-6, residual=r)
    hs = bf(oracle, oracle.bf16_to_f32(x) + oracle.bf16_to_f32(r))  # rmsnorm.cu:74-76
    assert np.array_equal(h, hs)
    assert np.array_equal(y, oracle.rmsnorm(hs, w, 1e-6))


def test_inv_freq_plain_and_llama3(oracle):
    d, theta = 128, 500000.0
    f = oracle.rope_inv_freq(d, theta)
    i = np.arange(d // 2)
    assert np.allclose(f, theta ** (-2.0 * i / d), rtol=1e-6)
    # llama3.1 published rule (transformers _compute_llama3_parameters): factor 8, low 1, high 4, 8192
    g = oracle.rope_inv_freq(d, theta, 8.0, 1.0, 4.0, 8192).astype(np.float64)
    base = theta ** (-2.0 * i / d)
    wl = 2 * np.pi / base
    exp = np.where(wl < 8192 / 4.0, base, np.where(wl > 8192 / 1.0, base / 8.0, 0))
    mid = (wl >= 8192 / 4.0) & (wl <= 8192 / 1.0)
    smooth = (8192 / wl - 1.0) / (4.0 - 1.0)
    exp = np.where(mid, (1 - smooth) * base / 8.0 + smooth * base, exp)
    assert mid.any() and (wl > 8192).any() and (wl < 2048).any()
    assert np.allclose(g, exp, rtol=1e-6)
    # factor <= 0 disables scaling (model.cpp:1423)
    assert np.array_equal(oracle.rope_inv_freq(d, theta, 0.0, 1.0, 4.0, 8192), f)


def test_rope_table_values(oracle):
    f = oracle.rope_inv_freq(8, 10000.0)
    tab = oracle.rope_table(np.array([0, 1, 7], np.int32), f, 8)
    assert np.array_equal(tab[0], [1, 1, 1, 1, 0, 0, 0, 0])
    assert np.allclose(tab[2, :4], np.cos(7 * f.astype(np.float64)), atol=1e-6)
    assert np.allclose(tab[2, 4:], np.sin(7 * f.astype(np.float64)), atol=1e-6)


@pytest.mark.parametrize("interleaved", [0, 1])
def test_rope_rotation_identities(oracle, interleaved):
    rng = np.random.default_rng(42)
    hq, hk, d, N = 2, 1, 16, 6
    f = oracle.rope_inv_freq(d, 10000.0)
    packed = bf(oracle, rng.standard_normal((N, (hq + 2 * hk) * d)))
    pos = np.array([0, 1, 5, 9, 100, 1000], np.int32)
    tab = oracle.rope_table(pos, f, d)
    slots = np.arange(N, dtype=np.int64)
    kp = np.zeros((N, 1, hk, d), np.uint16)
    vp = np.zeros_like(kp)
    q = oracle.qkv_rope_kvwrite(packed, kp, vp, tab, slots, hq, hk, d, interleaved)
    pf = oracle.bf16_to_f32(packed).reshape(N, hq + 2 * hk, d).astype(np.float64)
    qf = oracle.bf16_to_f32(q).astype(np.float64)
    kf = oracle.bf16_to_f32(kp).reshape(N, hk, d).astype(np.float64)
    # position 0 is the identity; v is copied verbatim
    assert np.array_equal(q[0], packed[0].reshape(hq + 2 * hk, d)[:hq])
    assert np.array_equal(vp.reshape(N, hk, d), packed.reshape(N, hq + 2 * hk, d)[:, hq + hk:])
    # a rotation preserves the norm of every head (up to bf16 rounding of the outputs)
    assert np.allclose(np.linalg.norm(qf, axis=2), np.linalg.norm(pf[:, :hq], axis=2), rtol=2e-2)
    # explicit rotation of the documented pairing
    half = d // 2
    for n in range(N):
        ang = pos[n] * f.astype(np.float64)
        for h in range(hq):
            x = pf[n, h]
            ia = 2 * np.arange(half) if interleaved else np.arange(half)
            ib = ia + 1 if interleaved else ia + half
            ref = np.zeros(d)
            ref[ia] = x[ia] * np.cos(ang) - x[ib] * np.sin(ang)
            ref[ib] = x[ib] * np.cos(ang) + x[ia] * np.sin(ang)
            assert np.all(np.abs(qf[n, h] - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-5)
    # relative-position property: <R(p)q, R(p')k> depends only on p - p' (pairs n=1,2 vs 2,3: diff 4)
    # checked in fp64 on the documented rotation rather than on rounded outputs
    assert kf.shape == (N, hk, d)


def test_qk_norm_then_rope(oracle):
    rng = np.random.default_rng(43)
    hq, hk, d, N = 2, 2, 32, 3
    f = oracle.rope_inv_freq(d, 1e6)
    packed = bf(oracle, rng.standard_normal((N, (hq + 2 * hk) * d)) * 2)
    qw, kw = bf(oracle, rng.uniform(0.5, 1.5, d)), bf(oracle, rng.uniform(0.5, 1.5, d))
    pos = np.array([3, 0, 17], np.int32)
    tab = oracle.rope_table(pos, f, d)
    kp = np.zeros((4, 2, hk, d), np.uint16)
    vp = np.zeros_like(kp)
    slots = np.array([5, 0, -1], np.int64)  # last token has no slot: K/V untouched
    q = oracle.qkv_rope_kvwrite(packed, kp, vp, tab, slots, hq, hk, d, 0, qw, kw, 1e-6)
    pf = oracle.bf16_to_f32(packed).reshape(N, hq + 2 * hk, d).astype(np.float64)
    half = d // 2
    for n in range(N):
        ang = pos[n] * f.astype(np.float64)
        for h in range(hq + hk):
            x = pf[n, h]
            w = oracle.bf16_to_f32(qw if h < hq else kw).astype(np.float64)
            xn = x / np.sqrt((x ** 2).mean() + 1e-6) * w
            ref = np.concatenate([xn[:half] * np.cos(ang) - xn[half:] * np.sin(ang),
                                  xn[half:] * np.cos(ang) + xn[:half] * np.sin(ang)])
            if h < hq:
                got = oracle.bf16_to_f32(q[n, h])
            elif slots[n] >= 0:
                got = oracle.bf16_to_f32(kp.reshape(-1, hk, d)[slots[n], h - hq])
            else:
                continue
            assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-5)
    used = {5, 0}
    flat = kp.reshape(-1, hk * d)
    assert all(flat[s].any() == (s in used) for s in range(flat.shape[0]))


def test_swiglu_closed_form(oracle):
    rng = np.random.default_rng(44)
    gu = bf(oracle, rng.standard_normal((4, 32)) * 4)
    y = oracle.bf16_to_f32(oracle.swiglu(gu))
    g = oracle.bf16_to_f32(gu)[:, :16].astype(np.float64)
    u = oracle.bf16_to_f32(gu)[:, 16:].astype(np.float64)
    ref = g / (1 + np.exp(-g)) * u
    assert np.all(np.abs(y - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-7)
    assert oracle.swiglu(bf(oracle, [[0.0, 5.0]]))[0, 0] == 0


def test_argmax_ties_and_nan(oracle):
    lg = bf(oracle, [[1, 7, 7, 3], [-1, -1, -1, -1], [np.nan, 2, 2, 1], [np.nan] * 4,
                     [-np.inf, -np.inf, 0, 0]])
    assert oracle.argmax_bf16(lg).tolist() == [1, 0, 1, 0, 2]
    rng = np.random.default_rng(45)
    big = bf(oracle, rng.standard_normal((3, 1000)))
    assert np.array_equal(oracle.argmax_bf16(big), np.argmax(oracle.bf16_to_f32(big), axis=1))


def test_gemm_bf16_against_fp64(oracle):
    rng = np.random.default_rng(46)
    a, w = bf(oracle, rng.standard_normal((3, 200))), bf(oracle, rng.standard_normal((7, 200)))
    truth = oracle.bf16_to_f32(a).astype(np.float64) @ oracle.bf16_to_f32(w).astype(np.float64).T
    y2, _ = oracle.gemm_bf16(a, w, mode=2)
    y0, y0b = oracle.gemm_bf16(a, w, mode=0)
    assert np.allclose(y2, truth, rtol=1e-6, atol=1e-6)
    assert np.allclose(y0, truth, rtol=0, atol=1e-4)
    assert np.array_equal(y0b, oracle.f32_to_bf16(y0))


def test_yarn_frequencies_hand_worked(oracle):
    """YaRN's frequency table (driver/cuda/src/kernels/rope.cu:495-507,552-589): with head_dim
    128, theta 10000, an original context of 4096, beta_fast 32 and beta_slow 1 the correction
    dims are 128 ln(4096 / (32 * 2 pi)) / (2 ln 10000) = 20.94 -> 20 and
    128 ln(4096 / (2 pi)) / (2 ln 10000) = 45.03 -> 46: pairs up to 20 keep their frequency,
    pairs from 46 on are divided by the factor, pair 33 sits exactly half way."""
    d, theta, factor = 128, 10000.0, 4.0
    f = oracle.rope_inv_freq_yarn(d, theta, factor, 32.0, 1.0, 4096).astype(np.float64)
    base = theta ** (-2.0 * np.arange(d // 2) / d)
    assert np.allclose(f[:21], base[:21], rtol=1e-6)
    assert np.allclose(f[46:], base[46:] / factor, rtol=1e-6)
    assert np.allclose(f[33], base[33] * (0.5 + 0.5 / factor), rtol=1e-6)
    assert np.all(np.diff(f / base) <= 1e-6)                       # the ratio only falls along the ramp (f32 table)
    assert np.all((f / base)[21:46] < 1.0) and np.all((f / base)[21:46] > 1.0 / factor)
    # factor 1: nothing changes; a ramp that would pass the last pair is clipped to it
    assert np.allclose(oracle.rope_inv_freq_yarn(d, theta, 1.0, 32.0, 1.0, 4096), base, rtol=1e-6)
    g = oracle.rope_inv_freq_yarn(64, 10000.0, 8.0, 32.0, 1e-6, 4096).astype(np.float64)
    b64 = 10000.0 ** (-2.0 * np.arange(32) / 64)
    assert np.allclose(g[31], b64[31] / 8.0, rtol=1e-6)


def test_scaled_rope_table_multiplies_cos_and_sin(oracle):
    import ctypes as C

    pos = np.array([0, 3, 1000], np.int32)
    inv = oracle.rope_inv_freq(64, 10000.0)
    plain = oracle.rope_table(pos, inv, 64)
    out = np.zeros_like(plain)
    oracle.lib().orc_rope_table_scaled(C.c_void_p(pos.ctypes.data), C.c_void_p(inv.ctypes.data),
                                       C.c_void_p(out.ctypes.data), C.c_int(3), C.c_int(64), C.c_float(1.25))
    assert np.array_equal(out, plain * np.float32(1.25))
    assert np.allclose(out[0, :32], 1.25) and np.allclose(out[0, 32:], 0.0)
