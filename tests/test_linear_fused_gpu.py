"""GPU parity: the fused projection (RMSNorm in the staging, SwiGLU in the epilogue) against the
composition of the separately pinned oracle ops — the fusion must not change values."""
import numpy as np
import pytest

from gpu_util import bits, dev, ulp_diff

pytestmark = pytest.mark.gpu


def make_weight(oracle, rng, kind, N, K, G=128):
    import torch
    from pie_amd import ops

    w = oracle.f32_to_bf16(rng.standard_normal((N, K)).astype(np.float32) * 0.02)
    if kind == "int4b8":
        packed = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)
        scale = oracle.f32_to_bf16(rng.uniform(0.002, 0.008, size=(N, K // G)).astype(np.float32))
        return dict(kind=kind, data=packed, scale=scale, G=G), \
            lambda gpu: ops.WeightView("int4b8", dev(packed, gpu), dev(scale, gpu, torch.bfloat16), G, N, K)
    if kind == "int8":
        q, s = oracle.quant_int8_per_channel(w)
        return dict(kind=kind, data=q, scale=s), \
            lambda gpu: ops.WeightView("int8", dev(q, gpu), dev(s, gpu), 0, N, K)
    if kind == "fp8":
        q, s = oracle.quant_fp8_per_channel(w)
        sb = oracle.f32_to_bf16(s)
        return dict(kind=kind, data=q, scale=oracle.bf16_to_f32(sb)), \
            lambda gpu: ops.WeightView("fp8", dev(q, gpu), dev(sb, gpu, torch.bfloat16), 0, N, K)
    return dict(kind=kind, data=w), lambda gpu: ops.WeightView("bf16", dev(w, gpu, torch.bfloat16), None, 0, N, K)


def close_to_oracle(oracle, got_bits, ref_bits, rel=2.0 ** -7, floor=2e-3):
    """bf16 outputs of a long dot product: relative to the value, with a floor relative to the
    largest output for elements that are sums of cancelling terms."""
    g = oracle.bf16_to_f32(got_bits).astype(np.float64)
    r = oracle.bf16_to_f32(ref_bits).astype(np.float64)
    tol = rel * np.abs(r) + floor * np.abs(r).max()
    return bool(np.all(np.abs(g - r) <= tol))


def oracle_linear(oracle, wd, act, y_in=None):
    if wd["kind"] == "int4b8":
        return oracle.gemm_w4a16(act, wd["data"], wd["scale"], wd["G"], mode=0, y_in=y_in)[1]
    if wd["kind"] == "int8":
        return oracle.gemm_w8a16(act, wd["data"], wd["scale"], mode=0, y_in=y_in)[1]
    if wd["kind"] == "fp8":
        return oracle.gemm_fp8(act, wd["data"], wd["scale"], mode=0, y_in=y_in)[1]
    return oracle.gemm_bf16(act, wd["data"], mode=0, y_in=y_in)[1]


@pytest.mark.parametrize("kind", ["int4b8", "int8", "fp8", "bf16"])
@pytest.mark.parametrize("M,N,K", [(1, 256, 2048), (3, 96, 4096), (6, 64, 1024)])
def test_norm_fused_equals_norm_then_linear(gpu, oracle, kind, M, N, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(110 + M + N)
    wd, mk = make_weight(oracle, rng, kind, N, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32) * 3)
    nw = oracle.f32_to_bf16(rng.uniform(0.5, 1.5, K).astype(np.float32))
    w = mk(gpu)
    xg, nwg = dev(x, gpu, torch.bfloat16), dev(nw, gpu, torch.bfloat16)
    fused = bits(ops.linear_fused(xg, w, norm_weight=nwg, eps=1e-5))
    # same kernels, unfused: must be bit-identical (the staged activations are the same bf16 values
    # up to the block-vs-kernel reduction order of the sum of squares)
    xn = ops.rmsnorm_bf16(xg, nwg, 1e-5)
    unfused = bits(ops.linear_fused(xn, w))
    d = ulp_diff(fused, unfused)
    assert d.max() <= 1 and (d == 0).mean() > 0.97
    ref = oracle_linear(oracle, wd, oracle.rmsnorm(x, nw, 1e-5))
    assert close_to_oracle(oracle, fused, ref)
    assert (ulp_diff(fused, ref) <= 1).mean() > 0.98


@pytest.mark.parametrize("kind", ["int4b8", "int8", "fp8", "bf16"])
@pytest.mark.parametrize("M,N,K", [
    # rows of up to 4096 values: one activation vector per thread in the register prologue
    (2, 64, 4096), (4, 40, 4096),
    # longer rows: four vectors per thread (one or two activation rows), two with three or four
    (1, 64, 6144), (1, 48, 14336), (2, 48, 14336), (1, 40, 4224), (1, 32, 16384), (4, 40, 8192),
    # past the registers' reach: the two-pass prologue through LDS
    (3, 40, 14336), (1, 32, 18432),
])
def test_norm_fused_over_every_activation_prologue(gpu, oracle, kind, M, N, K):
    """The GEMV picks its activation prologue from the row length and the row count; every
    variant stages the same bf16 values (fused norm on and off) as the norm kernel followed by
    the plain projection."""
    import torch
    from pie_amd import ops

    if kind in ("int8", "fp8") and K > 15360:
        pytest.skip("one-byte weights stage their activations as f32: rows of up to 15 360 values (the driver sends longer ones to the matrix-core GEMM)")
    rng = np.random.default_rng(130 + M + K)
    wd, mk = make_weight(oracle, rng, kind, N, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32) * 2)
    nw = oracle.f32_to_bf16(rng.uniform(0.5, 1.5, K).astype(np.float32))
    w = mk(gpu)
    xg, nwg = dev(x, gpu, torch.bfloat16), dev(nw, gpu, torch.bfloat16)
    plain = bits(ops.linear_fused(xg, w))
    ref_plain = oracle_linear(oracle, wd, x)
    assert close_to_oracle(oracle, plain, ref_plain)
    assert (ulp_diff(plain, ref_plain) <= 1).mean() > 0.98
    fused = bits(ops.linear_fused(xg, w, norm_weight=nwg, eps=1e-5))
    unfused = bits(ops.linear_fused(ops.rmsnorm_bf16(xg, nwg, 1e-5), w))
    d = ulp_diff(fused, unfused)
    assert d.max() <= 1 and (d == 0).mean() > 0.97
    assert close_to_oracle(oracle, fused, oracle_linear(oracle, wd, oracle.rmsnorm(x, nw, 1e-5)))


@pytest.mark.parametrize("kind", ["int4b8", "int8", "fp8", "bf16"])
@pytest.mark.parametrize("M,I,K", [(1, 256, 2048), (2, 1024, 512), (4, 152, 1024), (5, 64, 4096)])
def test_swiglu_epilogue_equals_linear_then_swiglu(gpu, oracle, kind, M, I, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(120 + M + I)
    wd, mk = make_weight(oracle, rng, kind, 2 * I, K)   # canonical rows: gate then up
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    # interleave rows (gate_0, up_0, gate_1, ...) for the fused kernel
    perm = np.empty(2 * I, np.int64)
    perm[0::2], perm[1::2] = np.arange(I), np.arange(I) + I
    wi = dict(wd)
    wi["data"] = wd["data"][perm]
    if "scale" in wd:
        wi["scale"] = wd["scale"][perm]
    _, mk_i = None, None
    w_can = mk(gpu)
    w_int = ops.WeightView(w_can.kind, w_can.data[torch.from_numpy(perm).to(gpu)].contiguous(),
                           None if w_can.scale is None else w_can.scale[torch.from_numpy(perm).to(gpu)].contiguous(),
                           w_can.group_size, w_can.N, w_can.K)
    xg = dev(x, gpu, torch.bfloat16)
    fused = bits(ops.linear_fused(xg, w_int, swiglu=True))
    assert fused.shape == (M, I)
    unfused = bits(ops.swiglu_bf16(ops.linear_fused(xg, w_can)))
    assert np.array_equal(fused, unfused)   # same sums, same rounding points: bit-identical
    ref = oracle.swiglu(oracle_linear(oracle, wd, x))
    assert close_to_oracle(oracle, fused, ref, rel=2.0 ** -6)
    assert (ulp_diff(fused, ref) <= 1).mean() > 0.97


def test_norm_and_swiglu_together_with_residual_variant(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(130)
    K, I, M = 2048, 512, 2
    wd, mk = make_weight(oracle, rng, "int4b8", 2 * I, K)
    perm = np.empty(2 * I, np.int64)
    perm[0::2], perm[1::2] = np.arange(I), np.arange(I) + I
    w_can = mk(gpu)
    idx = torch.from_numpy(perm).to(gpu)
    w_int = ops.WeightView("int4b8", w_can.data[idx].contiguous(), w_can.scale[idx].contiguous(), 128, 2 * I, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32) * 2)
    nw = oracle.f32_to_bf16(rng.uniform(0.5, 1.5, K).astype(np.float32))
    xg, nwg = dev(x, gpu, torch.bfloat16), dev(nw, gpu, torch.bfloat16)
    both = bits(ops.linear_fused(xg, w_int, norm_weight=nwg, swiglu=True))
    steps = bits(ops.swiglu_bf16(ops.linear_fused(ops.rmsnorm_bf16(xg, nwg, 1e-5), w_can)))
    d = ulp_diff(both, steps)
    assert (d == 0).mean() > 0.9 and (d <= 2).mean() > 0.995
    # beta with swiglu is rejected, beta without is fine
    with pytest.raises(ops.KernelError):
        ops.linear_fused(xg, w_int, y=torch.zeros(M, I, device=gpu, dtype=torch.bfloat16), beta=1, swiglu=True)


@pytest.mark.parametrize("kind", ["int4b8", "int8", "fp8", "bf16"])
@pytest.mark.parametrize("M,hq,hk,d,K", [(1, 8, 2, 64, 512), (3, 4, 4, 128, 1024), (4, 32, 8, 128, 4096)])
def test_qkv_rope_epilogue_equals_projection_then_rope_kernel(gpu, oracle, kind, M, hq, hk, d, K):
    """The fused q|k|v projection with RoPE and the KV write in its epilogue must give exactly
    the bytes of the projection followed by the (separately pinned) rope + KV-write kernel:
    q, and the touched K / V slots (one token without a slot)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(140 + M + hq)
    N = (hq + 2 * hk) * d
    wd, mk = make_weight(oracle, rng, kind, N, K)
    w = mk(gpu)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    nw = oracle.f32_to_bf16(rng.uniform(0.5, 1.5, K).astype(np.float32))
    xg, nwg = dev(x, gpu, torch.bfloat16), dev(nw, gpu, torch.bfloat16)
    pos = rng.integers(0, 500, M).astype(np.int32)
    inv = oracle.rope_inv_freq(d, 10000.0)
    tab = ops.rope_table(dev(pos, gpu), dev(inv, gpu), d)
    slots = rng.permutation(40)[:M].astype(np.int64)
    if M > 1:
        slots[1] = -1
    sg = dev(slots, gpu)
    pools = [torch.full((40, hk, d), 0.5, device=gpu, dtype=torch.bfloat16) for _ in range(4)]
    q1 = ops.qkv_rope_fused(xg, w, tab, sg, pools[0], pools[1], hq, hk, d, norm_weight=nwg)
    packed = ops.linear_fused(xg, w, norm_weight=nwg)
    q2 = ops.qkv_rope_kvwrite(packed, pools[2], pools[3], tab, sg, hq, hk, d, True)
    assert np.array_equal(bits(q1), bits(q2))
    assert np.array_equal(bits(pools[0]), bits(pools[2]))
    assert np.array_equal(bits(pools[1]), bits(pools[3]))
    # half-split pairing (Llama / Qwen checkpoints): weights with re-ordered q / k rows and
    # pairing = 2 give the bytes of the original weights followed by the half-split rope kernel;
    # so does the rope kernel's own mode 2 over the re-ordered projection
    wp = ops.pair_qk_rows(w, hq, hk, d)
    hp = [torch.full((40, hk, d), 0.5, device=gpu, dtype=torch.bfloat16) for _ in range(6)]
    q3 = ops.qkv_rope_fused(xg, wp, tab, sg, hp[0], hp[1], hq, hk, d, norm_weight=nwg, pairing=2)
    q4 = ops.qkv_rope_kvwrite(packed, hp[2], hp[3], tab, sg, hq, hk, d, 0)
    q5 = ops.qkv_rope_kvwrite(ops.linear_fused(xg, wp, norm_weight=nwg), hp[4], hp[5], tab, sg, hq, hk, d, 2)
    assert np.array_equal(bits(q3), bits(q4)) and np.array_equal(bits(q5), bits(q4))
    assert np.array_equal(bits(hp[0]), bits(hp[2])) and np.array_equal(bits(hp[1]), bits(hp[3]))
    assert np.array_equal(bits(hp[4]), bits(hp[2])) and np.array_equal(bits(hp[5]), bits(hp[3]))
    assert not np.array_equal(bits(q3), bits(q1))
    # and against the oracle's projection + rope
    ref_packed = oracle_linear(oracle, wd, oracle.rmsnorm(x, nw, 1e-5))
    kp = np.full((40, hk, d), oracle.f32_to_bf16(np.float32(0.5)), np.uint16)
    vp = kp.copy()
    tab_np = tab.cpu().numpy()
    qo = oracle.qkv_rope_kvwrite(ref_packed, kp, vp, tab_np, slots, hq, hk, d, 1)
    assert (ulp_diff(bits(q1).reshape(M, -1), np.asarray(qo).reshape(M, -1)) <= 2).mean() > 0.97
