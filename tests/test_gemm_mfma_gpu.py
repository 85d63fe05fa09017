"""GPU parity: the tiled matrix-core GEMM (prefill / large M) against the CPU oracle in the
reference's large-M evaluation order (int4: dequantise to bf16, then bf16 GEMM with fp32 sums;
int8/fp8/bf16: exact bf16 weights, row scale on the fp32 sum)."""
import numpy as np
import pytest

from gpu_util import bits, dev, ulp_diff
from test_linear_fused_gpu import close_to_oracle, make_weight

pytestmark = pytest.mark.gpu

KINDS = ["int4b8", "int8", "fp8", "bf16"]


def oracle_gemm(oracle, wd, act, y_in=None):
    if wd["kind"] == "int4b8":
        return oracle.gemm_w4a16(act, wd["data"], wd["scale"], wd["G"], mode=1, y_in=y_in)[1]
    if wd["kind"] == "int8":
        return oracle.gemm_w8a16(act, wd["data"], wd["scale"], mode=0, y_in=y_in)[1]
    if wd["kind"] == "fp8":
        return oracle.gemm_fp8(act, wd["data"], wd["scale"], mode=0, y_in=y_in)[1]
    return oracle.gemm_bf16(act, wd["data"], mode=0, y_in=y_in)[1]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,N,K", [(128, 256, 256), (200, 200, 1024), (65, 384, 512), (300, 130, 64),
                                   (1, 128, 128)])
def test_gemm_matches_oracle(gpu, oracle, kind, M, N, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(600 + M + N)
    wd, mk = make_weight(oracle, rng, kind, N, K, G=64 if K % 128 else 128)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    got = bits(ops.gemm_mfma(dev(x, gpu, torch.bfloat16), mk(gpu)))
    ref = oracle_gemm(oracle, wd, x)
    assert got.shape == ref.shape
    assert close_to_oracle(oracle, got, ref)
    assert (ulp_diff(got, ref) <= 1).mean() > 0.98


@pytest.mark.parametrize("kind", KINDS)
def test_gemm_one_hot_rows_are_exact(gpu, oracle, kind):
    """One-hot activations read single dequantised weights: bit-exact, which pins the tile
    indexing, both operand layouts and the in-flight dequantisation."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(610)
    M, N, K = 150, 272, 320
    wd, mk = make_weight(oracle, rng, kind, N, K, G=64)
    ks = rng.integers(0, K, size=M)
    x = np.zeros((M, K), np.float32)
    x[np.arange(M), ks] = 1.0
    xb = oracle.f32_to_bf16(x)
    got = bits(ops.gemm_mfma(dev(xb, gpu, torch.bfloat16), mk(gpu)))
    assert np.array_equal(got, oracle_gemm(oracle, wd, xb))


@pytest.mark.parametrize("kind", ["int4b8", "fp8"])
def test_gemm_beta_and_swiglu(gpu, oracle, kind):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(611)
    M, I, K = 140, 192, 512
    wd, mk = make_weight(oracle, rng, kind, 2 * I, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    xg = dev(x, gpu, torch.bfloat16)
    w = mk(gpu)
    y0 = oracle.f32_to_bf16(rng.standard_normal((M, 2 * I)).astype(np.float32))
    got = bits(ops.gemm_mfma(xg, w, y=dev(y0, gpu, torch.bfloat16).clone(), beta=1))
    ref = oracle_gemm(oracle, wd, x, y_in=y0)
    assert close_to_oracle(oracle, got, ref) and (ulp_diff(got, ref) <= 1).mean() > 0.98
    perm = np.empty(2 * I, np.int64)
    perm[0::2], perm[1::2] = np.arange(I), np.arange(I) + I
    idx = torch.from_numpy(perm).to(gpu)
    wi = ops.WeightView(w.kind, w.data[idx].contiguous(), w.scale[idx].contiguous(), w.group_size,
                        w.N, w.K)
    fused = bits(ops.gemm_mfma(xg, wi, swiglu=True))
    unfused = bits(ops.swiglu_bf16(ops.gemm_mfma(xg, w)))
    assert fused.shape == (M, I) and np.array_equal(fused, unfused)


def test_gemm_rejects_unsupported_k(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(612)
    wd, mk = make_weight(oracle, rng, "bf16", 64, 96)
    with pytest.raises(ops.KernelError):
        ops.gemm_mfma(torch.zeros(8, 96, device=gpu, dtype=torch.bfloat16), mk(gpu))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,N,K", [(64, 256, 4096), (33, 130, 2048), (100, 384, 1024), (16, 512, 14336),
                                   (128, 4096, 512)])
def test_gemm_split_k_matches_oracle(gpu, oracle, kind, M, N, K):
    """Decode-batch form: K shares per output tile, fp32 partials summed by the second kernel
    (64-row block tiles up to M = 64, ragged last share when the steps do not divide)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(630 + M + N)
    wd, mk = make_weight(oracle, rng, kind, N, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    xg, w = dev(x, gpu, torch.bfloat16), mk(gpu)
    got = bits(ops.gemm_mfma(xg, w, split_k=True))
    ref = oracle_gemm(oracle, wd, x)
    assert close_to_oracle(oracle, got, ref)
    assert (ulp_diff(got, ref) <= 1).mean() > 0.98
    single = bits(ops.gemm_mfma(xg, w))
    assert (ulp_diff(got, single) <= 1).mean() > 0.98


@pytest.mark.parametrize("kind", ["int4b8", "fp8"])
def test_gemm_split_k_beta_swiglu_one_hot(gpu, oracle, kind):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(631)
    M, I, K = 48, 192, 2048
    assert ops.gemm_mfma_workspace_bytes(M, 2 * I, K) > 0
    wd, mk = make_weight(oracle, rng, kind, 2 * I, K)
    w = mk(gpu)
    ks = rng.integers(0, K, size=M)
    x = np.zeros((M, K), np.float32)
    x[np.arange(M), ks] = 1.0
    xb = oracle.f32_to_bf16(x)
    assert np.array_equal(bits(ops.gemm_mfma(dev(xb, gpu, torch.bfloat16), w, split_k=True)),
                          oracle_gemm(oracle, wd, xb))
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    xg = dev(x, gpu, torch.bfloat16)
    y0 = oracle.f32_to_bf16(rng.standard_normal((M, 2 * I)).astype(np.float32))
    got = bits(ops.gemm_mfma(xg, w, y=dev(y0, gpu, torch.bfloat16).clone(), beta=1, split_k=True))
    ref = oracle_gemm(oracle, wd, x, y_in=y0)
    assert close_to_oracle(oracle, got, ref) and (ulp_diff(got, ref) <= 1).mean() > 0.98
    perm = np.empty(2 * I, np.int64)
    perm[0::2], perm[1::2] = np.arange(I), np.arange(I) + I
    idx = torch.from_numpy(perm).to(gpu)
    wi = ops.WeightView(w.kind, w.data[idx].contiguous(), w.scale[idx].contiguous(), w.group_size,
                        w.N, w.K)
    fused = bits(ops.gemm_mfma(xg, wi, swiglu=True, split_k=True))
    unfused = bits(ops.swiglu_bf16(ops.gemm_mfma(xg, w, split_k=True)))
    assert np.array_equal(fused, unfused)
