"""GPU parity: W4A16 unpack / dequant / GEMV through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(arr, device, dtype=None):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(arr)).to(device)
    if dtype is not None:
        t = t.view(dtype)
    return t


def _bits(t):
    import torch

    return t.view(torch.uint16).cpu().numpy() if t.dtype == torch.bfloat16 else t.cpu().numpy()


def make_case(oracle, seed, M, N, K, G, act_std=1.0):
    rng = np.random.default_rng(seed)
    packed = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)
    scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
    act = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32) * act_std)
    return packed, scale, act


def gpu_gemv(gpu, packed, scale, act, G, y_in=None, **tune):
    import torch

    from pie_amd import ops

    w = ops.int4b8_view(_t(packed.view(np.int32), gpu), _t(scale, gpu, torch.bfloat16), G)
    a = _t(act, gpu, torch.bfloat16)
    y = None if y_in is None else _t(y_in, gpu, torch.bfloat16)
    out = ops.gemv_w4a16(a, w, y=y, beta=0 if y_in is None else 1, **tune)
    torch.cuda.synchronize()
    return _bits(out)


def check_against_oracle(oracle, y_bits, packed, scale, act, G, y_in=None):
    truth, _, absum = oracle.gemm_w4a16(act, packed, scale, G, mode=2, y_in=y_in, want_abs=True)
    got = oracle.bf16_to_f32(y_bits).astype(np.float64)
    truth = truth.astype(np.float64)
    if y_in is not None:
        absum = absum + np.abs(oracle.bf16_to_f32(y_in))
    # one bf16 rounding (half ulp = 2^-9 of the binade, <= 2^-8 relative) + fp32 accumulation
    # of the offset-binary (128+n) products (<= 3e-5 of the absolute sum, see kernel header)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 3e-5 * absum + 1e-30
    bad = np.abs(got - truth) > tol
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; worst " \
                          f"{np.max(np.abs(got - truth) / tol):.2f}x"
    # and within one bf16 ulp of the reference-order fp32 evaluation
    _, y0 = oracle.gemm_w4a16(act, packed, scale, G, mode=0, y_in=y_in)
    d = np.abs(y_bits.astype(np.int32) - y0.astype(np.int32))
    same_sign = (y_bits >> 15) == (y0 >> 15)
    near_zero = np.abs(truth) < 1e-3 * absum
    assert np.all((d <= 1) & same_sign | near_zero)
    assert (d == 0).mean() > 0.9


def test_unpack_and_dequant_bit_exact(gpu, oracle):
    import torch

    from pie_amd import ops

    rng = np.random.default_rng(10)
    for (N, K, G) in [(3, 64, 32), (17, 1024, 128), (64, 4096, 128)]:
        packed = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)
        scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
        pt = _t(packed.view(np.int32), gpu)
        q = ops.unpack_w4(pt).cpu().numpy()
        assert np.array_equal(q, oracle.unpack_w4(packed, N, K))
        w = ops.dequant_wna16_int4b8_to_bf16(pt, _t(scale, gpu, torch.bfloat16), G)
        assert np.array_equal(_bits(w), oracle.dequant_w4a16(packed, scale, N, K, G))
    # every nibble value in every position
    words = np.array([[(nib << (4 * pos)) for pos in range(8) for nib in range(16)]], np.uint32)
    q = ops.unpack_w4(_t(words.view(np.int32), gpu)).cpu().numpy()
    assert np.array_equal(q, oracle.unpack_w4(words, 1, words.shape[1] * 8))


@pytest.mark.parametrize("M,N,K,G", [
    (1, 64, 256, 128), (1, 100, 2048, 128), (1, 33, 2304, 128), (1, 7, 32, 32),
    (1, 512, 4096, 128), (1, 130, 14336, 128), (2, 48, 4096, 128), (3, 20, 1024, 64),
    (4, 36, 2048, 32), (5, 24, 512, 128), (8, 16, 4096, 128),
])
def test_gemv_matches_oracle(gpu, oracle, M, N, K, G):
    packed, scale, act = make_case(oracle, 100 + M + N + K, M, N, K, G)
    y = gpu_gemv(gpu, packed, scale, act, G)
    check_against_oracle(oracle, y, packed, scale, act, G)


@pytest.mark.parametrize("rpw,rpb", [(1, 1), (1, 8), (2, 2), (3, 1), (3, 4), (4, 1), (4, 4)])
def test_gemv_every_tiling(gpu, oracle, rpw, rpb):
    packed, scale, act = make_case(oracle, 7, 2, 77, 4096, 128)
    y = gpu_gemv(gpu, packed, scale, act, 128, rows_per_wave=rpw, waves_per_simd=rpb)
    check_against_oracle(oracle, y, packed, scale, act, 128)


def test_gemv_beta_residual(gpu, oracle):
    packed, scale, act = make_case(oracle, 8, 2, 96, 2048, 128)
    rng = np.random.default_rng(9)
    y_in = oracle.f32_to_bf16(rng.standard_normal((2, 96)).astype(np.float32))
    y = gpu_gemv(gpu, packed, scale, act, 128, y_in=y_in)
    check_against_oracle(oracle, y, packed, scale, act, 128, y_in=y_in)


def test_gemv_one_hot_recovers_dequantised_rows(gpu, oracle):
    N, K, G = 40, 2048, 128
    packed, scale, _ = make_case(oracle, 11, 1, N, K, G)
    wd = oracle.dequant_w4a16(packed, scale, N, K, G)
    for k in (0, 3, 4, 31, 32, 127, 128, 1000, 2047):
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        y = gpu_gemv(gpu, packed, scale, oracle.f32_to_bf16(x), G)
        assert np.array_equal(y[0], wd[:, k]), f"k={k}"


def test_gemv_extreme_weights(gpu, oracle):
    N, K, G = 16, 4096, 128
    _, scale, act = make_case(oracle, 12, 1, N, K, G)
    q = np.full((N, K), -8, np.int8)
    q[N // 2:] = 7
    packed = oracle.pack_w4(q)
    y = gpu_gemv(gpu, packed, scale, act, G)
    check_against_oracle(oracle, y, packed, scale, act, G)


@pytest.mark.parametrize("N,K", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_gemv_full_size(gpu, oracle, N, K):
    """BASELINE sweep shapes at M=1: oracle on every row, plus exact linearity in the scales."""
    G = 128
    packed, scale, act = make_case(oracle, N + K, 1, N, K, G)
    y = gpu_gemv(gpu, packed, scale, act, G)
    check_against_oracle(oracle, y, packed, scale, act, G)
    scale2 = oracle.f32_to_bf16(oracle.bf16_to_f32(scale) * 2.0)
    y2 = gpu_gemv(gpu, packed, scale2, act, G)
    assert np.array_equal(oracle.bf16_to_f32(y2), 2.0 * oracle.bf16_to_f32(y))


def test_gemv_rejects_bad_shapes(gpu, oracle):
    from pie_amd import ops

    packed, scale, act = make_case(oracle, 13, 1, 8, 64, 32)
    with pytest.raises(ops.KernelError):
        gpu_gemv(gpu, packed, scale[:, :1], act, 32)  # scale shape
    with pytest.raises(ops.KernelError):
        gpu_gemv(gpu, packed, scale, act[:, :32], 32)  # K mismatch
