"""GPU parity of the W4A16 GEMM sweep at its real shapes: K = 4096 with N in {4096, 14336} and
K = 14336 with N = 4096, M in {8, 32, 128, 2048}, symmetric int4 in [-8, 7] packed 8 per word,
group 128, bf16 scales ~ U(0.005, 0.02), activations ~ N(0, 1) — through the kernels a decode
batch or a prefill of those sizes really runs (the instantiations depend on N, K and M):
the skinny matrix-core GEMM over tile-major weights (M = 8, 32, 128), the tiled matrix-core GEMM
(M = 128, 2048) and its split-K form (M = 128).

The oracle runs on a seeded sample of output columns (and of activation rows at M = 2048) so the
CPU time stays bounded; the whole output is covered by the exact structural check: one-hot
activation rows must return single dequantised weights, bit for bit, in every column."""
import numpy as np
import pytest

from gpu_util import bits, dev, ulp_diff
from test_linear_fused_gpu import close_to_oracle

pytestmark = pytest.mark.gpu

G = 128
SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336)]   # (N, K)


def _case(oracle, rng, M, N, K):
    packed = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)
    scale = oracle.f32_to_bf16(rng.uniform(0.005, 0.02, size=(N, K // G)).astype(np.float32))
    act = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    return packed, scale, act


def _kernels(ops, M):
    """name -> (callable(act, row-major view, tile-major view), oracle evaluation mode)."""
    k = {}
    if M <= 128:
        k["skinny"] = (lambda a, w, wt: ops.gemm_skinny(a, wt), 0)
    if M >= 128:
        k["tiled"] = (lambda a, w, wt: ops.gemm_mfma(a, w), 1)
    if M == 128:
        k["tiled_split_k"] = (lambda a, w, wt: ops.gemm_mfma(a, w, split_k=True), 1)
    return k


# The fused gate|up projection of the 8B model, the widest matrix a decode batch multiplies: its
# tile count is what sends 17-32 and 33-64 rows to the eight-tiles-per-wave instantiations.
GATE_UP = [(28672, 4096, 16), (28672, 4096, 32), (28672, 4096, 64)]   # (N, K, M)


@pytest.mark.parametrize("M", [8, 32, 128, 2048])
@pytest.mark.parametrize("N,K", SHAPES)
def test_sweep_shapes_match_oracle_on_sampled_columns(gpu, oracle, N, K, M):
    _sampled_columns(gpu, oracle, N, K, M)


@pytest.mark.parametrize("N,K,M", GATE_UP)
def test_gate_up_shape_matches_oracle_on_sampled_columns(gpu, oracle, N, K, M):
    _sampled_columns(gpu, oracle, N, K, M)


def _sampled_columns(gpu, oracle, N, K, M):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(N + K + M)
    packed, scale, act = _case(oracle, rng, M, N, K)
    w = ops.int4b8_view(dev(packed, gpu), dev(scale, gpu, torch.bfloat16), G)
    wt = ops.repack_mfma_tiles(w)
    a = dev(act, gpu, torch.bfloat16)
    cols = np.sort(rng.choice(N, 192, replace=False))
    cols[:4] = [0, 1, N - 2, N - 1][:4]            # the edges of the output too
    cols = np.unique(cols)
    rows = np.arange(M) if M <= 128 else np.unique(np.concatenate([[0, 1, M - 1], rng.choice(M, 45, replace=False)]))
    sub_p, sub_s, sub_a = packed[cols], scale[cols], act[rows]
    truth, _, absum = oracle.gemm_w4a16(sub_a, sub_p, sub_s, G, mode=2, want_abs=True)
    truth = truth.astype(np.float64)
    for name, (fn, mode) in _kernels(ops, M).items():
        if name == "tiled_split_k" and ops.gemm_mfma_workspace_bytes(M, N, K) == 0:
            continue
        y = bits(fn(a, w, wt))
        assert y.shape == (M, N), name
        got_bits = y[np.ix_(rows, cols)]
        got = oracle.bf16_to_f32(got_bits).astype(np.float64)
        if mode == 0:
            # fused order: one bf16 rounding + fp32 accumulation of the offset-binary products
            tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 3e-5 * absum
        else:
            # dequantise-then-GEMM order: each weight rounded to bf16 first (2^-9 relative, random
            # sign: the sum moves by <= 2^-9 * sqrt(K) mean products, far below 4e-4 of the sum
            # of magnitudes), then as above
            tol = 2.0 ** -8 * np.maximum(np.abs(truth), np.abs(got)) + 4e-4 * absum
        bad = np.abs(got - truth) > tol
        assert not bad.any(), f"{name}: {bad.sum()} of {bad.size} outside tolerance, worst " \
                              f"{np.max(np.abs(got - truth) / tol):.2f}x"
        # and next to the oracle's evaluation in the same order: within a bf16 step almost everywhere
        _, ref = oracle.gemm_w4a16(sub_a, sub_p, sub_s, G, mode=mode)
        assert close_to_oracle(oracle, got_bits, ref), name
        assert (ulp_diff(got_bits, ref) <= 1).mean() > 0.98, name


@pytest.mark.parametrize("M", [8, 32, 128, 2048])
@pytest.mark.parametrize("N,K", SHAPES)
def test_sweep_shapes_one_hot_rows_are_exact_everywhere(gpu, oracle, N, K, M):
    """Row m of the activations is the unit vector e_k(m): y[m, n] must be bf16(q[n, k] * s[n, k/G])
    for every one of the N columns — tile indexing, operand layouts, bias removal and the K split
    of every instantiation, over the whole output."""
    _one_hot_rows(gpu, oracle, N, K, M)


@pytest.mark.parametrize("N,K,M", GATE_UP)
def test_gate_up_shape_one_hot_rows_are_exact_everywhere(gpu, oracle, N, K, M):
    _one_hot_rows(gpu, oracle, N, K, M)


def _one_hot_rows(gpu, oracle, N, K, M):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(N + 2 * K + M)
    packed, scale, _ = _case(oracle, rng, 1, N, K)
    ks = rng.integers(0, K, size=M)
    ks[:3] = [0, K - 1, K // 2]
    x = np.zeros((M, K), np.float32)
    x[np.arange(M), ks] = 1.0
    w = ops.int4b8_view(dev(packed, gpu), dev(scale, gpu, torch.bfloat16), G)
    wt = ops.repack_mfma_tiles(w)
    a = dev(oracle.f32_to_bf16(x), gpu, torch.bfloat16)
    nib = ((packed[:, ks // 8] >> (4 * (ks % 8)).astype(np.uint32)) & 0xF).astype(np.float32) - 8.0   # [N, M]
    want = oracle.f32_to_bf16((nib * oracle.bf16_to_f32(scale[:, ks // G])).T.copy())                   # [M, N]
    for name, (fn, _) in _kernels(ops, M).items():
        if name == "tiled_split_k" and ops.gemm_mfma_workspace_bytes(M, N, K) == 0:
            continue
        assert np.array_equal(bits(fn(a, w, wt)), want), name
