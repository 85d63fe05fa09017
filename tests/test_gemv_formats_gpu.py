"""GPU parity: int8 / fp8 / bf16 weight-streaming GEMV through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

from gpu_util import bits, dev

pytestmark = pytest.mark.gpu


def check(oracle, got_bits, truth, absum, rel_acc):
    got = oracle.bf16_to_f32(got_bits).astype(np.float64)
    tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + rel_acc * absum + 1e-30
    err = np.abs(got - truth)
    assert np.all(err <= tol), f"worst {np.max(err / tol):.2f}x"


@pytest.mark.parametrize("M,N,K", [(1, 64, 2048), (1, 300, 8192), (2, 50, 2048), (4, 33, 512),
                                   (1, 16, 1040), (6, 40, 2048)])
@pytest.mark.parametrize("scale_dtype", ["f32", "bf16"])
def test_w8a16(gpu, oracle, M, N, K, scale_dtype):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(60 + N + K)
    w = oracle.f32_to_bf16(rng.standard_normal((N, K)).astype(np.float32) * 0.02)
    q, s = oracle.quant_int8_per_channel(w)
    if scale_dtype == "bf16":
        sb = oracle.f32_to_bf16(s)
        s = oracle.bf16_to_f32(sb)
        s_dev = dev(sb, gpu, torch.bfloat16)
    else:
        s_dev = dev(s, gpu)
    act = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    yin = oracle.f32_to_bf16(rng.standard_normal((M, N)).astype(np.float32))
    for y_in in (None, yin):
        y = ops.gemv_w8a16(dev(act, gpu, torch.bfloat16), dev(q, gpu), s_dev,
                           y=None if y_in is None else dev(y_in, gpu, torch.bfloat16),
                           beta=0 if y_in is None else 1)
        truth, _, ab = oracle.gemm_w8a16(act, q, s, mode=2, y_in=y_in, want_abs=True)
        # offset-binary bytes (0..255) accumulate 128*sum|x| of cancelling mass in fp32
        check(oracle, bits(y), truth.astype(np.float64), ab + (0 if y_in is None else 1), 2e-5)


def test_w8a16_full_size_llama1b_shapes(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(61)
    for (N, K) in [(2048 + 1024, 2048), (2048, 8192)]:
        q = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        s = rng.uniform(1e-4, 1e-3, N).astype(np.float32)
        act = oracle.f32_to_bf16(rng.standard_normal((1, K)).astype(np.float32))
        y = ops.gemv_w8a16(dev(act, gpu, torch.bfloat16), dev(q, gpu), dev(s, gpu))
        truth, _, ab = oracle.gemm_w8a16(act, q, s, mode=2, want_abs=True)
        check(oracle, bits(y), truth.astype(np.float64), ab, 2e-5)
        # exact linearity in the per-row scale
        y2 = ops.gemv_w8a16(dev(act, gpu, torch.bfloat16), dev(q, gpu), dev(s * 2, gpu))
        assert np.array_equal(oracle.bf16_to_f32(bits(y2)), 2 * oracle.bf16_to_f32(bits(y)))


@pytest.mark.parametrize("M,N,K", [(1, 768, 2048), (1, 2048, 768), (3, 40, 1024), (1, 128, 2048)])
def test_fp8(gpu, oracle, M, N, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(62 + N)
    w = oracle.f32_to_bf16(rng.standard_normal((N, K)).astype(np.float32) * 0.02)
    q, s = oracle.quant_fp8_per_channel(w)
    act = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    y = ops.gemv_fp8(dev(act, gpu, torch.bfloat16), dev(q, gpu), dev(s, gpu))
    truth, _, ab = oracle.gemm_fp8(act, q, s, mode=2, want_abs=True)
    check(oracle, bits(y), truth.astype(np.float64), ab, 2e-6)


def test_fp8_every_finite_code_decodes_exactly(gpu, oracle):
    """One-hot activations read single weights back: the in-register fp8 decode is bit-exact."""
    import torch
    from pie_amd import ops

    codes = np.array([c for c in range(256) if c not in (0x7F, 0xFF)], np.uint8)
    N, K = len(codes), 32
    q = np.zeros((N, K), np.uint8)
    q[:, 7] = codes
    act = np.zeros((1, K), np.float32)
    act[0, 7] = 1.0
    y = ops.gemv_fp8(dev(oracle.f32_to_bf16(act), gpu, torch.bfloat16), dev(q, gpu),
                     dev(np.ones(N, np.float32), gpu))
    assert np.array_equal(oracle.bf16_to_f32(bits(y))[0], oracle.fp8_decode(codes))


@pytest.mark.parametrize("M,N,K", [(1, 1000, 4096), (1, 128, 2048), (2, 77, 1536), (4, 64, 64),
                                   (1, 5, 8)])
def test_bf16(gpu, oracle, M, N, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(63 + N)
    w = oracle.f32_to_bf16(rng.standard_normal((N, K)).astype(np.float32) * 0.02)
    act = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    y = ops.gemv_bf16(dev(act, gpu, torch.bfloat16), dev(w, gpu, torch.bfloat16))
    truth, _, ab = oracle.gemm_bf16(act, w, mode=2, want_abs=True)
    check(oracle, bits(y), truth.astype(np.float64), ab, 2e-6)


def test_bf16_lm_head_shape_and_greedy_token(gpu, oracle):
    """lm_head [128256, 2048] at batch 1: the argmax of the GPU logits is the oracle's token
    (ties/near-ties resolved against the fp64 logits)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(64)
    V, H = 128256, 2048
    w = oracle.f32_to_bf16(rng.standard_normal((V, H)).astype(np.float32) * 0.02)
    act = oracle.f32_to_bf16(rng.standard_normal((1, H)).astype(np.float32))
    logits = ops.gemv_bf16(dev(act, gpu, torch.bfloat16), dev(w, gpu, torch.bfloat16))
    tok = int(ops.argmax_bf16(logits).cpu()[0])
    truth, _, ab = oracle.gemm_bf16(act, w, mode=2, want_abs=True)
    check(oracle, bits(logits), truth.astype(np.float64), ab, 2e-6)
    assert tok == int(oracle.argmax_bf16(bits(logits))[0])
    top2 = np.sort(truth[0])[-2:]
    if top2[1] - top2[0] > 2.0 ** -7 * abs(top2[1]):  # not a near-tie at bf16 resolution
        assert tok == int(np.argmax(truth[0]))


@pytest.mark.parametrize("M,V,H", [(1, 128256, 2048), (3, 32000, 4096), (4, 5000, 512), (2, 1024, 256)])
def test_lm_head_with_argmax_equals_gemv_then_argmax(gpu, oracle, M, V, H):
    """The fused form (GEMV that keeps per-lane (value, row) pairs + a small reduce) returns the
    bytes of the plain GEMV with the fused norm and the token of the row argmax over them — also
    with ties (the lowest index wins), a NaN (never wins) and an all -inf row (token 0)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(70 + M)
    w = oracle.f32_to_bf16(rng.standard_normal((V, H)).astype(np.float32) * 0.02)
    # repeated rows make exact ties among the largest logits likely somewhere
    w[V // 2] = w[7]
    w[V - 1] = w[7]
    act = oracle.f32_to_bf16(rng.standard_normal((M, H)).astype(np.float32))
    nw = oracle.f32_to_bf16(rng.uniform(0.5, 1.5, H).astype(np.float32))
    a, wg, nwg = dev(act, gpu, torch.bfloat16), dev(w, gpu, torch.bfloat16), dev(nw, gpu, torch.bfloat16)
    logits, toks = ops.lm_head_argmax(a, wg, norm_weight=nwg)
    plain = ops.linear_fused(a, ops.WeightView("bf16", wg, None, 0, V, H), norm_weight=nwg)
    assert np.array_equal(bits(logits), bits(plain))
    want = oracle.argmax_bf16(bits(plain))
    assert np.array_equal(toks.cpu().numpy().astype(np.int64), np.asarray(want).astype(np.int64))
    assert np.array_equal(toks.cpu().numpy(), ops.argmax_bf16(plain).cpu().numpy())
    # a row that favours the duplicated weight row: its three copies tie, index 7 wins
    act2 = np.tile(oracle.bf16_to_f32(w[7])[None, :], (M, 1)) * 8.0
    a2 = dev(oracle.f32_to_bf16(act2.astype(np.float32)), gpu, torch.bfloat16)
    lg2, tk2 = ops.lm_head_argmax(a2, wg)
    l2 = oracle.bf16_to_f32(bits(lg2))
    assert np.all(l2[:, 7] == l2[:, V // 2]) and np.all(l2[:, 7] == l2[:, V - 1])
    assert np.all(tk2.cpu().numpy() == np.argmax(l2, axis=1)) and np.all(np.argmax(l2, axis=1) == 7)
    # NaN activations: every logit NaN -> token 0 (nothing compares greater); inf weights: -inf rows
    a3 = a.clone()
    a3[0, :] = float("nan")
    _, tk3 = ops.lm_head_argmax(a3, wg)
    assert int(tk3[0]) == int(ops.argmax_bf16(ops.gemv_bf16(a3, wg))[0])
