"""GPU: the driver loaded from a Hugging Face snapshot holds exactly the tensors an independent
host computation gives (fusion, interleave, quantisation with the oracle's quantisers), and its
forward pass matches the oracle model built from the files (never from the driver's memory)."""
import numpy as np
import pytest

from driver_util import cosine
from snapshot_util import expected_tensors, write_snapshot

pytestmark = pytest.mark.gpu


def snapshot_toml(directory, quant, group=128, scale_dtype="bf16", key="hf_path"):
    return f"""
[model]
{key} = "{directory}"
quant = "{quant}"
group_size = {group}
scale_dtype = "{scale_dtype}"

[batching]
kv_page_size = 16
total_pages = 32
max_forward_tokens = 128
max_forward_requests = 8

[runtime]
verbose = true
"""


def driver_cfg(cfg, quant, group, scale_dtype="bf16"):
    return dict(cfg, quant=quant, group_size=group, scale_dtype=scale_dtype, page_size=16, total_pages=32,
                rms_eps=1e-6)


CASES = [
    (dict(arch="llama3", hidden=256, layers=2, q_heads=4, kv_heads=2, head_dim=64, intermediate=512,
          vocab=512), "bf16", "bf16"),
    (dict(arch="llama3", hidden=256, layers=2, q_heads=4, kv_heads=2, head_dim=64, intermediate=512,
          vocab=512, rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                       high_freq_factor=4.0, original_max_position_embeddings=64)),
     "int4b8", "f16"),
    (dict(arch="qwen3", hidden=256, layers=2, q_heads=4, kv_heads=1, head_dim=128, intermediate=512,
          vocab=512, tie=True), "int8", "f32"),
    (dict(arch="qwen3_moe", hidden=256, layers=2, q_heads=4, kv_heads=2, head_dim=64, intermediate=0,
          vocab=512, num_experts=4, top_k=2, expert_intermediate=256), "fp8", "bf16"),
]


@pytest.mark.parametrize("cfg,quant,dtype", CASES, ids=lambda v: v if isinstance(v, str) else v.get("arch", ""))
def test_loaded_tensors_and_forward(gpu, oracle, tmp_path, cfg, quant, dtype):
    from oracle.model import OracleModel, model_from_driver
    from pie_amd import driver as drvmod

    rng = np.random.default_rng(17)
    d = str(tmp_path / "snap")
    group = 64
    stored = write_snapshot(d, oracle, rng, cfg, dtype=dtype)
    want = expected_tensors(oracle, stored, cfg, quant, group)
    with drvmod.Driver(snapshot_toml(d, quant, group)) as drv:
        caps = drv.capabilities()
        assert caps["vocab_size"] == cfg["vocab"] and caps["arch_name"] == cfg["arch"]
        _, got = model_from_driver(drv, driver_cfg(cfg, quant, group))
        for name, a in want.items():
            g = got[name]
            assert np.array_equal(np.asarray(g).reshape(-1).view(np.uint8),
                                  np.ascontiguousarray(a).reshape(-1).view(np.uint8)), name
        # forward parity against the model built from the files
        ocfg = dict(hidden=cfg["hidden"], layers=cfg["layers"], q_heads=cfg["q_heads"],
                    kv_heads=cfg["kv_heads"], head_dim=cfg["head_dim"], intermediate=cfg["intermediate"],
                    vocab=cfg["vocab"], rms_eps=1e-6, rope_interleaved=0, qk_norm=cfg["arch"] != "llama3",
                    quant=quant, group_size=group, page_size=16, total_pages=32)
        if cfg["arch"] == "qwen3_moe":
            ocfg.update(num_experts=cfg["num_experts"], top_k=cfg["top_k"],
                        expert_intermediate=cfg["expert_intermediate"])
        want["inv_freq"] = got["inv_freq"]
        rs = cfg.get("rope_scaling")
        ref_freq = oracle.rope_inv_freq(cfg["head_dim"], 10000.0, *((rs["factor"], rs["low_freq_factor"],
                                        rs["high_freq_factor"], rs["original_max_position_embeddings"]) if rs else ()))
        assert np.allclose(got["inv_freq"], ref_freq, rtol=1e-6)
        om = OracleModel(ocfg, want)
        prompt = rng.integers(0, cfg["vocab"], 21)
        args = dict(token_ids=prompt, position_ids=np.arange(21), kv_page_indices=[3, 9], kv_page_indptr=[0, 2],
                    kv_last_page_lens=[5], qo_indptr=[0, 21])
        res = drv.forward(drvmod.ForwardFrame(**args))
        otok, olog, _ = om.forward(**args, want_logits=True)
        glog = drv.export_tensor("debug.logits", np.uint16).reshape(-1, cfg["vocab"])
        g, o = oracle.bf16_to_f32(glog[0]), oracle.bf16_to_f32(olog[0])
        assert cosine(g, o) >= 0.9999
        top2 = np.sort(o)[-2:]
        if top2[1] - top2[0] > 2.0 ** -6 * abs(top2[1]) + 1e-6:
            assert res.tokens[0] == otok[0]


def test_packed_int4_checkpoint_is_taken_as_stored(gpu, oracle, tmp_path):
    """compressed-tensors pack-quantized weights (weight_packed / weight_scale) go to the device
    unchanged (rows fused, gate/up interleaved), through the CUDA driver's `snapshot_dir` key."""
    from oracle.model import model_from_driver
    from pie_amd import driver as drvmod

    cfg = CASES[0][0]
    rng = np.random.default_rng(18)
    d = str(tmp_path / "packed")
    group = 32
    stored = write_snapshot(d, oracle, rng, cfg, dtype="bf16", packed_int4_group=group)
    want = expected_tensors(oracle, stored, cfg, "int4b8", group)
    with drvmod.Driver(snapshot_toml(d, "int4b8", group, key="snapshot_dir")) as drv:
        _, got = model_from_driver(drv, driver_cfg(cfg, "int4b8", group))
        for name, a in want.items():
            assert np.array_equal(np.asarray(got[name]).reshape(-1).view(np.uint8),
                                  np.ascontiguousarray(a).reshape(-1).view(np.uint8)), name
    with pytest.raises(Exception):
        drvmod.Driver(snapshot_toml(d, "int8", group))      # a packed checkpoint cannot be re-quantised
