"""Pins for the oracle's quantised-format and weight-only linear functions (CPU only).

None of these retype the oracle's formula: they use literal known answers from
the format definition, round trips, numpy's fp64 matmul on independently
dequantised weights, and algebraic invariants.
"""
import numpy as np
import pytest


def rand_bf16(rng, shape, std=1.0):
    from oracle import f32_to_bf16

    return f32_to_bf16(rng.standard_normal(shape).astype(np.float32) * std)


def py_nibbles(word):
    """Independent statement of the format: nibble j (4 bits at 4*j) -> element j, minus 8."""
    return [((word >> (4 * j)) & 0xF) - 8 for j in range(8)]


def test_unpack_known_answers(oracle):
    # driver/cuda/src/kernels/dequant_wna16.cu:31-36: lane j reads bits [4j, 4j+4).
    packed = np.array([[0x76543210, 0xFEDCBA98, 0x00000000, 0xFFFFFFFF, 0x8000000F]], np.uint32)
    q = oracle.unpack_w4(packed, 1, 40)
    expect = [-8, -7, -6, -5, -4, -3, -2, -1, 0, 1, 2, 3, 4, 5, 6, 7] + [-8] * 8 + [7] * 8 + \
             [7, -8, -8, -8, -8, -8, -8, 0]
    assert q.tolist() == [expect]


def test_unpack_every_nibble_every_position(oracle):
    words = []
    for pos in range(8):
        for nib in range(16):
            words.append((nib << (4 * pos)) | (0x88888888 & ~(0xF << (4 * pos))))
    packed = np.array([words], np.uint32)
    q = oracle.unpack_w4(packed, 1, len(words) * 8)[0].reshape(-1, 8)
    for i, w in enumerate(words):
        assert q[i].tolist() == py_nibbles(w)
        pos, nib = divmod(i, 16)
        assert q[i][pos] == nib - 8 and all(q[i][j] == 0 for j in range(8) if j != pos)


def test_pack_unpack_round_trip(oracle):
    rng = np.random.default_rng(1)
    q = rng.integers(-8, 8, size=(7, 64), dtype=np.int8)
    packed = oracle.pack_w4(q)
    assert packed.shape == (7, 8)
    assert np.array_equal(oracle.unpack_w4(packed, 7, 64), q)
    # and against python ints
    for n in range(7):
        for w in range(8):
            assert py_nibbles(int(packed[n, w])) == q[n, 8 * w:8 * w + 8].tolist()


def test_dequant_matches_exact_product(oracle):
    rng = np.random.default_rng(2)
    N, K, G = 5, 256, 128
    q = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    packed = oracle.pack_w4(q)
    scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
    w = oracle.bf16_to_f32(oracle.dequant_w4a16(packed, scale, N, K, G))
    s = np.repeat(oracle.bf16_to_f32(scale), G, axis=1)
    exact = q.astype(np.float64) * s.astype(np.float64)
    # one bf16 rounding of an exactly representable-in-f32 product
    assert np.all(np.abs(w - exact) <= np.abs(exact) * 2.0 ** -8 + 1e-30)
    # q in {-8,...,7} times a bf16 scale has <= 11 significant bits; powers of two are exact
    pow2 = np.isin(np.abs(q), [0, 1, 2, 4, 8])
    assert np.array_equal(w[pow2], exact[pow2].astype(np.float32))


@pytest.mark.parametrize("M,N,K,G", [(1, 9, 256, 128), (3, 4, 512, 32), (2, 6, 384, 128)])
def test_gemm_w4a16_against_fp64_matmul(oracle, M, N, K, G):
    rng = np.random.default_rng(3)
    q = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    packed = oracle.pack_w4(q)
    scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
    act = rand_bf16(rng, (M, K))
    x = oracle.bf16_to_f32(act).astype(np.float64)
    wd = q.astype(np.float64) * np.repeat(oracle.bf16_to_f32(scale), G, axis=1).astype(np.float64)
    truth = x @ wd.T
    absum = np.abs(x) @ np.abs(wd).T
    y2, _, ab = oracle.gemm_w4a16(act, packed, scale, G, mode=2, want_abs=True)
    assert np.allclose(y2, truth, rtol=1e-6, atol=1e-6)
    assert np.allclose(ab, absum, rtol=1e-12)
    y0, y0b = oracle.gemm_w4a16(act, packed, scale, G, mode=0)
    assert np.all(np.abs(y0 - truth) <= 1e-6 * K ** 0.5 * absum + 1e-7)
    # bf16 output is the rounding of the f32 value
    assert np.array_equal(y0b, oracle.f32_to_bf16(y0))
    # dequant-then-GEMM uses bf16-rounded weights: error bounded by 2^-9 relative per weight
    y1, _ = oracle.gemm_w4a16(act, packed, scale, G, mode=1)
    wr = oracle.bf16_to_f32(oracle.dequant_w4a16(packed, scale, N, K, G)).astype(np.float64)
    assert np.allclose(y1, x @ wr.T, rtol=0, atol=1e-5 * absum.max())


def test_gemm_w4a16_one_hot_and_extremes(oracle):
    rng = np.random.default_rng(4)
    N, K, G = 8, 256, 128
    q = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    q[0, :] = -8
    q[1, :] = 7
    packed = oracle.pack_w4(q)
    scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
    wd = oracle.bf16_to_f32(oracle.dequant_w4a16(packed, scale, N, K, G))
    s = np.repeat(oracle.bf16_to_f32(scale), G, axis=1)
    for k in (0, 5, 127, 128, 255):
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        y, yb = oracle.gemm_w4a16(oracle.f32_to_bf16(x), packed, scale, G, mode=0)
        assert np.array_equal(y[0], (q[:, k].astype(np.float32) * s[:, k]))
        assert np.array_equal(oracle.bf16_to_f32(yb)[0], wd[:, k])
    ones = oracle.f32_to_bf16(np.ones((1, K), np.float32))
    y, _ = oracle.gemm_w4a16(ones, packed, scale, G, mode=2)
    sg = oracle.bf16_to_f32(scale).astype(np.float64)
    assert np.allclose(y[0, 0], -8 * G * sg[0].sum(), rtol=1e-6)
    assert np.allclose(y[0, 1], 7 * G * sg[1].sum(), rtol=1e-6)


def test_gemm_w4a16_linear_in_scale_and_beta(oracle):
    rng = np.random.default_rng(5)
    N, K, G = 6, 256, 64
    packed = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)
    scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
    scale2 = oracle.f32_to_bf16(oracle.bf16_to_f32(scale) * 2.0)  # exact doubling
    act = rand_bf16(rng, (2, K))
    y, _ = oracle.gemm_w4a16(act, packed, scale, G, mode=0)
    y2, _ = oracle.gemm_w4a16(act, packed, scale2, G, mode=0)
    assert np.array_equal(y2, 2 * y)
    yin = rand_bf16(rng, (2, N))
    yb, _ = oracle.gemm_w4a16(act, packed, scale, G, mode=0, y_in=yin)
    assert np.allclose(yb, y.astype(np.float64) + oracle.bf16_to_f32(yin), rtol=1e-7, atol=0)


def test_int8_quant_known_answers(oracle):
    # driver/portable/tests/test_kv_cache_quant.cpp:60-71: -0.5 at scale 1/127 -> -64 (half to even)
    w = oracle.f32_to_bf16(np.array([[1.0, -0.5, 0.25], [3.0, -1.5, 0.75], [0, 0, 0]], np.float32))
    q, s = oracle.quant_int8_per_channel(w)
    assert q.tolist() == [[127, -64, 32], [127, -64, 32], [0, 0, 0]]
    assert s[0] == np.float32(1.0) / np.float32(127.0)
    assert s[1] == np.float32(3.0) / np.float32(127.0)
    assert s[2] == 1.0  # degenerate row, quant_bf16_to_fp8.cu:311-313
    d = oracle.bf16_to_f32(oracle.dequant_int8_per_channel(q, s))
    assert np.allclose(d[0], [1.0, -64 / 127, 32 / 127], rtol=2 ** -8)


def test_int8_quant_properties(oracle):
    rng = np.random.default_rng(6)
    w = rand_bf16(rng, (16, 300), std=0.02)
    q, s = oracle.quant_int8_per_channel(w)
    wf = oracle.bf16_to_f32(w)
    assert np.all(np.abs(q).max(axis=1) == 127)
    assert np.allclose(s, np.abs(wf).max(axis=1) / 127.0, rtol=1e-6)
    # |w - q*s| <= s/2 (+ float slack)
    assert np.all(np.abs(wf - q * s[:, None]) <= 0.5 * s[:, None] * (1 + 1e-5))


@pytest.mark.parametrize("M,N,K", [(1, 10, 320), (4, 3, 64)])
def test_gemm_w8a16_against_fp64_matmul(oracle, M, N, K):
    rng = np.random.default_rng(7)
    w = rand_bf16(rng, (N, K), std=0.02)
    q, s = oracle.quant_int8_per_channel(w)
    act = rand_bf16(rng, (M, K))
    x = oracle.bf16_to_f32(act).astype(np.float64)
    truth = (x @ q.astype(np.float64).T) * s.astype(np.float64)[None, :]
    absum = (np.abs(x) @ np.abs(q.astype(np.float64)).T) * s[None, :]
    y2, _, ab = oracle.gemm_w8a16(act, q, s, mode=2, want_abs=True)
    assert np.allclose(y2, truth, rtol=1e-6, atol=1e-7)
    assert np.allclose(ab, absum, rtol=1e-12)
    y0, y0b = oracle.gemm_w8a16(act, q, s, mode=0)
    assert np.all(np.abs(y0 - truth) <= 1e-6 * K ** 0.5 * absum + 1e-7)
    assert np.array_equal(y0b, oracle.f32_to_bf16(y0))
    y1, _ = oracle.gemm_w8a16(act, q, s, mode=1)
    wd = oracle.bf16_to_f32(oracle.dequant_int8_per_channel(q, s)).astype(np.float64)
    assert np.allclose(y1, x @ wd.T, rtol=0, atol=1e-5 * absum.max())


def test_bf16_rounding_helpers(oracle):
    # ties to even at the bf16 boundary: 1 + 2^-8 is a tie between 1.0 and 1+2^-7 -> 1.0
    x = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -0.0, np.inf],
                 np.float32)
    b = oracle.f32_to_bf16(x)
    assert b.tolist() == [0x3F80, 0x3F82, 0x3F81, 0x8000, 0x7F80]
    assert np.isnan(oracle.bf16_to_f32(oracle.f32_to_bf16(np.array([np.nan], np.float32))))[0]


def test_fp8_e4m3_decode_table(oracle):
    b = np.arange(256, dtype=np.uint8)
    f = oracle.fp8_decode(b)
    # literal anchors of the OCP e4m3fn format
    assert f[0x00] == 0 and f[0x01] == 2.0 ** -9 and f[0x07] == 7 * 2.0 ** -9
    assert f[0x08] == 2.0 ** -6 and f[0x38] == 1.0 and f[0x3C] == 1.5 and f[0x40] == 2.0
    assert f[0x7E] == 448.0 and np.isnan(f[0x7F]) and np.isnan(f[0xFF]) and f[0xFE] == -448.0
    fin = np.delete(f[:128], 0x7F)
    assert np.all(np.diff(fin) > 0)  # codes are monotonic
    assert np.array_equal(f[128:255], -f[:127])
    # torch's float8_e4m3fn agrees on every finite code
    import torch
    t = torch.from_numpy(b.copy()).view(torch.float8_e4m3fn).float().numpy()
    ok = ~np.isnan(f)
    assert np.array_equal(t[ok], f[ok])


def test_fp8_quant_round_trip_and_rounding(oracle):
    import torch
    rng = np.random.default_rng(8)
    w = rand_bf16(rng, (6, 256), std=0.02)
    q, s = oracle.quant_fp8_per_channel(w)
    wf = oracle.bf16_to_f32(w)
    assert np.allclose(s, np.abs(wf).max(axis=1) / 448.0, rtol=1e-6)
    assert np.all(np.abs(oracle.fp8_decode(q)).max(axis=1) == 448.0)
    # the quantiser's rounding is round-to-nearest-even saturating: same bytes as torch's cast
    scaled = (wf * (np.float32(448.0) / np.abs(wf).max(axis=1, keepdims=True))).astype(np.float32)
    tq = torch.from_numpy(scaled).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, tq)
    # exactly representable values survive
    codes = np.delete(np.arange(255, dtype=np.uint8), [0x7F, 0x80])
    vals = oracle.fp8_decode(codes)
    row = oracle.f32_to_bf16(np.concatenate([vals, [448.0]]).astype(np.float32)[None, :] / 8)
    q2, s2 = oracle.quant_fp8_per_channel(row)
    assert s2[0] == np.float32(56.0) / np.float32(448.0)
    assert np.array_equal(oracle.fp8_decode(q2[0, :-1]), vals)


def test_gemm_fp8_against_fp64(oracle):
    rng = np.random.default_rng(9)
    w = rand_bf16(rng, (9, 128), std=0.02)
    q, s = oracle.quant_fp8_per_channel(w)
    act = rand_bf16(rng, (2, 128))
    x = oracle.bf16_to_f32(act).astype(np.float64)
    wd = oracle.fp8_decode(q).astype(np.float64)
    truth = (x @ wd.T) * s[None, :]
    y2, _ = oracle.gemm_fp8(act, q, s, mode=2)
    y0, y0b = oracle.gemm_fp8(act, q, s, mode=0)
    assert np.allclose(y2, truth, rtol=1e-6, atol=1e-8)
    assert np.allclose(y0, truth, rtol=0, atol=1e-5 * np.abs(truth).max())
    assert np.array_equal(y0b, oracle.f32_to_bf16(y0))
