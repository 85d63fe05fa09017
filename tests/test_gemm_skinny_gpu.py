"""GPU parity: the matrix-core skinny GEMM (5 <= M <= a few dozen rows) and the MoE grouped GEMM
against the CPU oracle's fused-order quantised GEMM (fp32 sums differ only in order), plus exact
structural checks (one-hot activations recover the dequantised rows bit-exactly)."""
import numpy as np
import pytest

from gpu_util import bits, dev, ulp_diff
from test_linear_fused_gpu import close_to_oracle, make_weight, oracle_linear

pytestmark = pytest.mark.gpu

KINDS = ["int4b8", "int8", "fp8", "bf16"]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,N,K", [(5, 64, 512), (8, 200, 1024), (16, 256, 4096), (17, 96, 2048),
                                   (32, 1040, 1536), (45, 48, 512),
                                   # enough 16-row tiles for two and four tiles per block
                                   (8, 12304, 512), (20, 24592, 512)])
def test_skinny_matches_oracle(gpu, oracle, kind, M, N, K):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(300 + M + N)
    wd, mk = make_weight(oracle, rng, kind, N, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = mk(gpu)
    got = bits(ops.gemm_skinny(dev(x, gpu, torch.bfloat16), w))
    ref = oracle_linear(oracle, wd, x)
    assert got.shape == ref.shape
    assert close_to_oracle(oracle, got, ref)
    assert (ulp_diff(got, ref) <= 1).mean() > 0.98


@pytest.mark.parametrize("kind", KINDS)
def test_skinny_equals_gemv_path_rowwise(gpu, oracle, kind):
    """Same contract as the GEMV: every activation row gives the value the GEMV gives for it
    (sum order differs, so within one bf16 step on almost all elements)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(311)
    M, N, K = 24, 512, 2048
    wd, mk = make_weight(oracle, rng, kind, N, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = mk(gpu)
    xg = dev(x, gpu, torch.bfloat16)
    a = bits(ops.gemm_skinny(xg, w))
    b = bits(ops.linear_fused(xg, w))
    d = ulp_diff(a, b)
    assert (d <= 1).mean() > 0.99 and close_to_oracle(oracle, a, b)


@pytest.mark.parametrize("kind", KINDS)
def test_skinny_one_hot_rows_are_exact(gpu, oracle, kind):
    """act = one-hot rows: y[m, n] must be bf16(dequantised w[n, k_m]) exactly — pins the
    lane/k layout of both MFMA operands and the offset-binary bias removal."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(312)
    M, N, K = 16, 80, 1024
    wd, mk = make_weight(oracle, rng, kind, N, K)
    ks = rng.choice(K, size=M, replace=False)
    x = np.zeros((M, K), np.float32)
    x[np.arange(M), ks] = 1.0
    xb = oracle.f32_to_bf16(x)
    got = bits(ops.gemm_skinny(dev(xb, gpu, torch.bfloat16), mk(gpu)))
    ref = oracle_linear(oracle, wd, xb)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("kind", ["int4b8", "fp8"])
@pytest.mark.parametrize("tiled,M", [(False, 12), (True, 12), (True, 37)])
def test_skinny_beta_and_swiglu(gpu, oracle, kind, tiled, M):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(313)
    I, K = 192, 1024
    wd, mk = make_weight(oracle, rng, kind, 2 * I, K)
    x = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    xg = dev(x, gpu, torch.bfloat16)
    w = mk(gpu)
    lay = ops.repack_mfma_tiles if tiled else (lambda v: v)
    # residual accumulate
    y0 = oracle.f32_to_bf16(rng.standard_normal((M, 2 * I)).astype(np.float32))
    got = bits(ops.gemm_skinny(xg, lay(w), y=dev(y0, gpu, torch.bfloat16).clone(), beta=1))
    ref = oracle_linear(oracle, wd, x, y_in=y0)
    assert close_to_oracle(oracle, got, ref) and (ulp_diff(got, ref) <= 1).mean() > 0.98
    # swiglu epilogue over interleaved rows
    perm = np.empty(2 * I, np.int64)
    perm[0::2], perm[1::2] = np.arange(I), np.arange(I) + I
    idx = torch.from_numpy(perm).to(gpu)
    wi = ops.WeightView(w.kind, w.data[idx].contiguous(), w.scale[idx].contiguous(), w.group_size,
                        w.N, w.K)
    fused = bits(ops.gemm_skinny(xg, lay(wi), swiglu=True))
    assert fused.shape == (M, I)
    unfused = bits(ops.swiglu_bf16(ops.gemm_skinny(xg, lay(w))))
    assert np.array_equal(fused, unfused)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(xg, lay(wi), y=torch.zeros(M, I, device=gpu, dtype=torch.bfloat16), beta=1,
                        swiglu=True)


def test_skinny_rejects_unsupported_k(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(314)
    wd, mk = make_weight(oracle, rng, "int4b8", 32, 640)   # K not a multiple of 512
    x = torch.zeros(8, 640, device=gpu, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x, mk(gpu))


@pytest.mark.parametrize("kind", ["fp8", "int4b8", "bf16"])
@pytest.mark.parametrize("swiglu", [False, True])
def test_moe_grouped_gemm_matches_per_expert_oracle(gpu, oracle, kind, swiglu):
    """Routes sorted by expert, gathered activation rows, empty experts, an expert with more
    rows than one tile."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(320)
    E, N, K, T = 6, 96, 512, 20
    counts = np.array([3, 0, 21, 1, 0, 7])
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    R = int(offs[-1])
    rows = rng.integers(0, T, size=R).astype(np.int32)
    x = oracle.f32_to_bf16(rng.standard_normal((T, K)).astype(np.float32))
    experts = [make_weight(oracle, rng, kind, N, K) for _ in range(E)]
    views = [mk(gpu) for _, mk in experts]
    wstack = torch.stack([v.data for v in views]).contiguous()
    sstack = None if views[0].scale is None else torch.stack([v.scale for v in views]).contiguous()
    got = bits(ops.moe_grouped_gemm(dev(x, gpu, torch.bfloat16), dev(rows, gpu), dev(offs, gpu),
                                    kind, wstack, sstack, N, K, rows_hint=16,
                                    group_size=views[0].group_size, swiglu=swiglu))
    ref = np.zeros((R, N), np.uint16)
    for e in range(E):
        lo, hi = offs[e], offs[e + 1]
        if hi > lo:
            ref[lo:hi] = oracle_linear(oracle, experts[e][0], x[rows[lo:hi]])
    if swiglu:
        # kernel pairs adjacent rows (gate_i, up_i) = canonical rows (2i, 2i+1)
        canon = np.concatenate([ref[:, 0::2], ref[:, 1::2]], axis=1)
        ref = oracle.swiglu(canon)
    assert got.shape == ref.shape
    assert close_to_oracle(oracle, got, ref, rel=2.0 ** -6)
    assert (ulp_diff(got, ref) <= 1).mean() > 0.97


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("N,K", [(80, 1024), (100, 512), (12304, 512)])
def test_tile_major_repack_is_the_documented_permutation(gpu, oracle, kind, N, K):
    """dst[((t*nb + b)*64 + 16q + j)*16 ..] = the 16 bytes at byte 64b + 16q of row 16t + j; rows
    past N are zero; int4: codes 2i, 2i + 1 of every 32-bit word sit in nibbles i, i + 4, and the
    group scales become [tile][group][16]."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(330 + N)
    wd, mk = make_weight(oracle, rng, kind, N, K)
    w = mk(gpu)
    t = ops.repack_mfma_tiles(w)
    src = w.data.contiguous().view(torch.uint8).cpu().numpy().reshape(N, -1)
    row_bytes = src.shape[1]
    nb, tiles = row_bytes // 64, (N + 15) // 16
    padded = np.zeros((tiles * 16, row_bytes), np.uint8)
    padded[:N] = src
    want = padded.reshape(tiles, 16, nb, 4, 16).transpose(0, 2, 3, 1, 4)      # [t][b][q][j][16 bytes]
    if kind == "int4b8":
        words = np.ascontiguousarray(want).reshape(-1).view(np.uint32)
        paired = np.zeros_like(words)
        for i in range(4):
            paired |= ((words >> np.uint32(8 * i)) & np.uint32(0xF)) << np.uint32(4 * i)
            paired |= ((words >> np.uint32(8 * i + 4)) & np.uint32(0xF)) << np.uint32(4 * i + 16)
        want = paired.view(np.uint8)
    assert np.array_equal(t.data.view(torch.uint8).cpu().numpy().reshape(-1), want.reshape(-1))
    if kind == "int4b8":
        sc = w.scale.view(torch.uint16).cpu().numpy()
        ps = np.zeros((tiles * 16, sc.shape[1]), np.uint16)
        ps[:N] = sc
        want_s = ps.reshape(tiles, 16, -1).transpose(0, 2, 1)                 # [t][g][j]
        assert np.array_equal(t.scale.view(torch.uint16).cpu().numpy().reshape(-1), want_s.reshape(-1))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,N,K", [(5, 64, 512), (16, 256, 4096), (17, 100, 2048), (45, 48, 512),
                                   (8, 12304, 512), (20, 24592, 512),
                                   # long K: seven chunks per K slice; 1536: a K slice left empty
                                   (6, 64, 14336), (32, 1040, 1536), (1, 4096, 4096), (3, 8192, 1024),
                                   # fewer rows than a tile (a router), two passes over small matrices
                                   (21, 8, 512), (21, 768, 512), (21, 512, 512), (130, 72, 1024),
                                   # 32-row passes (more than 32 rows): whole, ragged, K split over waves
                                   (64, 1040, 1536), (48, 4096, 2048), (33, 256, 4096)])
def test_skinny_over_tile_major_weights_matches_oracle_and_row_major(gpu, oracle, kind, M, N, K):
    """Tile-major weights run the wave-private kernel (another split of K, so another sum order):
    same bar against the oracle as the row-major path, and within one bf16 step of that path on
    almost every element."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(340 + M + N)
    wd, mk = make_weight(oracle, rng, kind, N, K)
    w = mk(gpu)
    x = dev(oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32)), gpu, torch.bfloat16)
    a = bits(ops.gemm_skinny(x, w))
    b = bits(ops.gemm_skinny(x, ops.repack_mfma_tiles(w)))
    ref = oracle_linear(oracle, wd, bits(x))
    assert close_to_oracle(oracle, b, ref)
    assert (ulp_diff(b, ref) <= 1).mean() > 0.98
    assert (ulp_diff(a, b) <= 1).mean() > 0.98


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M", [16, 48])
def test_skinny_tile_major_one_hot_rows_are_exact(gpu, oracle, kind, M):
    """One-hot activations over tile-major weights: y[m, n] is bf16(dequantised w[n, k_m]) exactly,
    whatever K slice and chunk k_m falls in (48 rows: the 32-row passes, the second half empty)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(341)
    N, K = 96, 4096
    wd, mk = make_weight(oracle, rng, kind, N, K)
    ks = np.array([0, 1, 7, 8, 31, 127, 128, 255, 256, 511, 512, 1023, 2048, 3000, 4094, 4095])
    ks = np.concatenate([ks, (ks * 7 + 3) % K, (ks * 13 + 130) % K])[:M]
    x = np.zeros((M, K), dtype=np.float32)
    x[np.arange(M), ks] = 1.0
    xb = oracle.f32_to_bf16(x)
    got = bits(ops.gemm_skinny(dev(xb, gpu, torch.bfloat16), ops.repack_mfma_tiles(mk(gpu))))
    ref = oracle_linear(oracle, wd, xb)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("kind", ["fp8", "int4b8", "bf16"])
@pytest.mark.parametrize("swiglu", [False, True])
def test_moe_grouped_gemm_over_tile_major_experts(gpu, oracle, kind, swiglu):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(350)
    E, N, K, T = 6, 96, 1024, 20
    counts = np.array([3, 0, 21, 1, 0, 7])
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = rng.integers(0, T, size=int(offs[-1])).astype(np.int32)
    x = dev(oracle.f32_to_bf16(rng.standard_normal((T, K)).astype(np.float32)), gpu, torch.bfloat16)
    views = [make_weight(oracle, rng, kind, N, K)[1](gpu) for _ in range(E)]
    wstack = torch.stack([v.data for v in views]).contiguous()
    sstack = None if views[0].scale is None else torch.stack([v.scale for v in views]).contiguous()
    args = dict(rows_hint=16, group_size=views[0].group_size, swiglu=swiglu)
    a = bits(ops.moe_grouped_gemm(x, dev(rows, gpu), dev(offs, gpu), kind, wstack, sstack, N, K, **args))
    tiled = ops.repack_mfma_tiles(ops.WeightView(kind, wstack, sstack, views[0].group_size, E * N, K))
    ws = tiled.data.reshape(E, N, -1)
    ss = tiled.scale if kind != "int4b8" else tiled.scale.reshape(E, N, -1)
    ss = sstack if kind != "int4b8" else ss
    b = bits(ops.moe_grouped_gemm(x, dev(rows, gpu), dev(offs, gpu), kind, ws, ss, N, K, tiled=True, **args))
    # the row-major path is checked against the per-expert oracle above; the tile-major kernel
    # splits K differently, so its sums differ from it in order only
    assert a.shape == b.shape
    assert (ulp_diff(a, b) <= 1).mean() > 0.98 and close_to_oracle(oracle, b, a)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("M,hq,hk,d,K", [(5, 8, 2, 64, 512), (16, 4, 4, 128, 1024), (37, 32, 8, 128, 4096)])
def test_qkv_rope_epilogue_of_the_skinny_gemm_equals_projection_then_rope_kernel(gpu, oracle, kind, M, hq, hk,
                                                                                 d, K):
    """A decode batch's q|k|v projection with RoPE and the KV write in the skinny GEMM's epilogue:
    exactly the bytes of the same projection followed by the rope + KV-write kernel — q, and the
    touched K / V slots (one token without a slot)."""
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(360 + M + hq)
    N = (hq + 2 * hk) * d
    wd, mk = make_weight(oracle, rng, kind, N, K)
    wt = ops.repack_mfma_tiles(mk(gpu))
    x = dev(oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32)), gpu, torch.bfloat16)
    pos = rng.integers(0, 500, M).astype(np.int32)
    tab = ops.rope_table(dev(pos, gpu), dev(oracle.rope_inv_freq(d, 10000.0), gpu), d)
    slots = rng.permutation(64)[:M].astype(np.int64)
    slots[1] = -1
    sg = dev(slots, gpu)
    pools = [torch.full((64, hk, d), 0.5, device=gpu, dtype=torch.bfloat16) for _ in range(4)]
    q1 = ops.qkv_rope_skinny_tiled(x, wt, tab, sg, pools[0], pools[1], hq, hk, d)
    q2 = ops.qkv_rope_kvwrite(ops.gemm_skinny(x, wt), pools[2], pools[3], tab, sg, hq, hk, d, True)
    assert np.array_equal(bits(q1), bits(q2))
    assert np.array_equal(bits(pools[0]), bits(pools[2]))
    assert np.array_equal(bits(pools[1]), bits(pools[3]))
    assert not np.all(bits(pools[0]) == bits(torch.full((64, hk, d), 0.5, device=gpu, dtype=torch.bfloat16)))
    # half-split pairing over weights with re-ordered q / k rows (pairing = 2): the bytes of the
    # original weights followed by the half-split rope kernel
    wp = ops.repack_mfma_tiles(ops.pair_qk_rows(mk(gpu), hq, hk, d))
    hp = [torch.full((64, hk, d), 0.5, device=gpu, dtype=torch.bfloat16) for _ in range(4)]
    q3 = ops.qkv_rope_skinny_tiled(x, wp, tab, sg, hp[0], hp[1], hq, hk, d, pairing=2)
    q4 = ops.qkv_rope_kvwrite(ops.gemm_skinny(x, wt), hp[2], hp[3], tab, sg, hq, hk, d, 0)
    assert np.array_equal(bits(q3), bits(q4))
    assert np.array_equal(bits(hp[0]), bits(hp[2])) and np.array_equal(bits(hp[1]), bits(hp[3]))
