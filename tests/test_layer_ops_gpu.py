"""GPU parity for the per-layer kernels (embed, norms, RoPE + KV write, SwiGLU, argmax, page
copies) through the C ABI vs the CPU oracle.  Copies and index work are bit-exact; float ops
agree within one bf16 step (summation order and libm differ in the last fp32 bit)."""
import numpy as np
import pytest

from gpu_util import bits, dev, ulp_diff

pytestmark = pytest.mark.gpu


def bf(oracle, x):
    return oracle.f32_to_bf16(np.asarray(x, np.float32))


def test_embed_bit_exact(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(50)
    tab = rng.integers(0, 2 ** 16, size=(1000, 2048)).astype(np.uint16)
    tok = np.array([0, 999, 5, 5, 1000, 2 ** 31 - 1, 17], np.uint32)
    y = ops.embed_bf16(dev(tok, gpu), dev(tab, gpu, torch.bfloat16))
    assert np.array_equal(bits(y), oracle.embed(tok, tab))


@pytest.mark.parametrize("rows,H", [(1, 2048), (3, 4096), (2, 64), (2, 8192), (1, 14336)])
def test_rmsnorm(gpu, oracle, rows, H):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(51 + H)
    x = bf(oracle, rng.standard_normal((rows, H)) * 2)
    w = bf(oracle, rng.uniform(0.5, 1.5, H))
    y = bits(ops.rmsnorm_bf16(dev(x, gpu, torch.bfloat16), dev(w, gpu, torch.bfloat16), 1e-5))
    ref = oracle.rmsnorm(x, w, 1e-5)
    d = ulp_diff(y, ref)
    assert d.max() <= 1 and (d == 0).mean() > 0.98
    r = bf(oracle, rng.standard_normal((rows, H)))
    h = dev(x, gpu, torch.bfloat16)
    y2 = bits(ops.residual_add_rmsnorm_bf16(h, dev(r, gpu, torch.bfloat16),
                                            dev(w, gpu, torch.bfloat16), 1e-5))
    ref2, href = oracle.rmsnorm(x, w, 1e-5, residual=r)
    assert np.array_equal(bits(h), href)  # the rounded sum is bit-exact
    d = ulp_diff(y2, ref2)
    assert d.max() <= 1 and (d == 0).mean() > 0.98


def test_rope_table(gpu, oracle):
    from pie_amd import ops

    f = oracle.rope_inv_freq(128, 500000.0, 8.0, 1.0, 4.0, 8192)
    pos = np.array([0, 1, 2, 17, 2047, 8191, 100000], np.int32)
    tab = ops.rope_table(dev(pos, gpu), dev(f, gpu), 128).cpu().numpy()
    ref = oracle.rope_table(pos, f, 128)
    assert np.array_equal(tab[0], ref[0])
    assert np.allclose(tab, ref, rtol=0, atol=3e-7)


@pytest.mark.parametrize("hq,hk,d,interleaved,qknorm", [
    (32, 8, 128, 0, False), (32, 8, 64, 1, False), (32, 4, 128, 0, True), (4, 4, 64, 1, True)])
def test_qkv_rope_kvwrite(gpu, oracle, hq, hk, d, interleaved, qknorm):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(52 + hq + d)
    N, ps, pages = 9, 16, 5
    packed = bf(oracle, rng.standard_normal((N, (hq + 2 * hk) * d)))
    f = oracle.rope_inv_freq(d, 500000.0)
    pos = rng.integers(0, 4096, N).astype(np.int32)
    pos[0] = 0
    tab = oracle.rope_table(pos, f, d)
    slots = rng.permutation(pages * ps)[:N].astype(np.int64)
    slots[3] = -1
    qw = bf(oracle, rng.uniform(0.5, 1.5, d)) if qknorm else None
    kw = bf(oracle, rng.uniform(0.5, 1.5, d)) if qknorm else None
    kp0 = rng.integers(0, 2 ** 15, size=(pages, ps, hk, d)).astype(np.uint16)
    vp0 = rng.integers(0, 2 ** 15, size=(pages, ps, hk, d)).astype(np.uint16)
    kp_ref, vp_ref = kp0.copy(), vp0.copy()
    q_ref = oracle.qkv_rope_kvwrite(packed, kp_ref, vp_ref, tab, slots, hq, hk, d, interleaved,
                                    qw, kw, 1e-6)
    kp, vp = dev(kp0, gpu, torch.bfloat16), dev(vp0, gpu, torch.bfloat16)
    q = ops.qkv_rope_kvwrite(dev(packed, gpu, torch.bfloat16), kp, vp, dev(tab, gpu),
                             dev(slots, gpu), hq, hk, d, interleaved,
                             None if qw is None else dev(qw, gpu, torch.bfloat16),
                             None if kw is None else dev(kw, gpu, torch.bfloat16), 1e-6)
    assert np.array_equal(bits(vp), vp_ref)  # V is a copy: bit-exact, untouched slots intact
    if qknorm:
        assert ulp_diff(bits(q), q_ref).max() <= 1 and ulp_diff(bits(kp), kp_ref).max() <= 1
    else:
        # same table, same fp32 expression: bit-exact
        assert np.array_equal(bits(q), q_ref) and np.array_equal(bits(kp), kp_ref)
    untouched = np.ones(pages * ps, bool)
    untouched[slots[slots >= 0]] = False
    assert np.array_equal(bits(kp).reshape(pages * ps, -1)[untouched],
                          kp0.reshape(pages * ps, -1)[untouched])


def test_swiglu(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(53)
    gu = bf(oracle, rng.standard_normal((5, 2 * 1024)) * 3)
    y = bits(ops.swiglu_bf16(dev(gu, gpu, torch.bfloat16)))
    d = ulp_diff(y, oracle.swiglu(gu))
    assert d.max() <= 1 and (d == 0).mean() > 0.98


def test_argmax_ties_nan_and_vocab(gpu, oracle):
    import torch
    from pie_amd import ops

    rng = np.random.default_rng(54)
    V = 128256
    lg = bf(oracle, rng.standard_normal((6, V)))
    lg[1, 77] = lg[1, 90000] = 0x4120      # tie at 10.0 -> lowest index
    lg[2, :] = 0xBF80                       # all equal -> 0
    lg[3, 5] = 0x7FC0                       # NaN never wins
    lg[4, V - 1] = 0x4200                   # last element
    lg[5, :] = 0x7FC0                       # all NaN -> 0
    out = ops.argmax_bf16(dev(lg, gpu, torch.bfloat16)).cpu().numpy().astype(np.uint32)
    assert np.array_equal(out, oracle.argmax_bf16(lg))
    assert out[1] == 77 and out[2] == 0 and out[4] == V - 1 and out[5] == 0


def test_copy_kv_pages(gpu):
    import torch
    from pie_amd import ops

    pool = torch.randint(0, 2 ** 15, (12, 16, 8, 128), dtype=torch.int16, device=gpu)
    ref = pool.clone()
    srcs = torch.tensor([3, 0, 11], dtype=torch.int32, device=gpu)
    dsts = torch.tensor([5, 7, 1], dtype=torch.int32, device=gpu)
    ops.copy_kv_pages(pool, srcs, dsts)
    ref[dsts.long()] = ref[srcs.long()]
    assert torch.equal(pool, ref)
    with pytest.raises(ops.KernelError):
        ops.copy_kv_pages(pool, srcs, torch.tensor([5, 7, 12], dtype=torch.int32, device=gpu))
