"""CPU: the driver's Hugging Face snapshot reader (config.json mapping + safetensors headers),
through its host-only inspection hook, against files written with the safetensors package."""
import json
import os

import numpy as np
import pytest

from snapshot_util import write_snapshot

CFG = dict(arch="qwen3", hidden=64, layers=2, q_heads=4, kv_heads=2, head_dim=32, intermediate=96,
           vocab=128)


def test_reader_sees_every_tensor_of_every_file(oracle, tmp_path):
    from pie_amd import driver as drvmod

    rng = np.random.default_rng(5)
    d = str(tmp_path / "snap")
    stored = write_snapshot(d, oracle, rng, CFG, dtype="bf16", files=3)
    info = drvmod.snapshot_info(d)
    assert info["arch"] == "qwen3" and info["hidden"] == 64 and info["layers"] == 2
    assert (info["q_heads"], info["kv_heads"], info["head_dim"]) == (4, 2, 32)
    assert info["intermediate"] == 96 and info["vocab"] == 128 and not info["tie_embeddings"]
    assert abs(info["rms_eps"] - 1e-6) < 1e-12 and info["rope_theta"] == 10000.0
    assert set(info["tensors"]) == set(stored)
    for name, a in stored.items():
        e = info["tensors"][name]
        assert e["dtype"] == "BF16" and e["shape"] == list(a.shape) and e["bytes"] == a.size * 2
        want = oracle.f32_to_bf16(a).reshape(-1)[:4].view(np.uint8)
        assert e["first_bytes"] == [int(x) for x in want[:len(e["first_bytes"])]]


def test_dtypes_moe_fields_and_rope_scaling(oracle, tmp_path):
    from pie_amd import driver as drvmod

    rng = np.random.default_rng(6)
    cfg = dict(arch="qwen3_moe", hidden=64, layers=1, q_heads=2, kv_heads=1, head_dim=32, intermediate=0,
               vocab=64, num_experts=4, top_k=2, expert_intermediate=32, tie=True)
    d = str(tmp_path / "moe")
    write_snapshot(d, oracle, rng, cfg, dtype="f16", files=1)
    info = drvmod.snapshot_info(d)
    assert info["arch"] == "qwen3_moe" and (info["num_experts"], info["top_k"], info["expert_intermediate"]) == (4, 2, 32)
    assert info["tie_embeddings"] and "lm_head.weight" not in info["tensors"]
    assert info["tensors"]["model.layers.0.mlp.experts.3.down_proj.weight"] == \
        dict(dtype="F16", shape=[64, 32], bytes=64 * 32 * 2,
             first_bytes=info["tensors"]["model.layers.0.mlp.experts.3.down_proj.weight"]["first_bytes"])
    llama = dict(CFG, arch="llama3", rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                                       high_freq_factor=4.0,
                                                       original_max_position_embeddings=8192))
    d2 = str(tmp_path / "llama")
    write_snapshot(d2, oracle, rng, llama, dtype="f32", files=1)
    info = drvmod.snapshot_info(d2)
    assert info["arch"] == "llama3" and info["rope_factor"] == 8.0
    assert info["tensors"]["model.norm.weight"]["dtype"] == "F32"


def test_reader_errors(oracle, tmp_path):
    from pie_amd import driver as drvmod

    with pytest.raises(RuntimeError, match="cannot open"):
        drvmod.snapshot_info(str(tmp_path / "missing"))
    d = tmp_path / "bad"
    os.makedirs(d)
    (d / "config.json").write_text(json.dumps(dict(model_type="gpt2")))
    with pytest.raises(RuntimeError, match="unsupported model_type"):
        drvmod.snapshot_info(str(d))
    (d / "config.json").write_text(json.dumps(dict(model_type="llama", hidden_size=64)))
    with pytest.raises(RuntimeError, match="no .safetensors"):
        drvmod.snapshot_info(str(d))
    (d / "x.safetensors").write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{\"a\":1}")
    with pytest.raises(RuntimeError):
        drvmod.snapshot_info(str(d))


def _write_raw(path, header: dict, payload: bytes):
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(len(h).to_bytes(8, "little") + h + payload)


@pytest.mark.parametrize("entry,msg", [
    (dict(dtype="BF16", shape=[4, 4], data_offsets=[0, 16]), "holds 16 bytes"),      # too few bytes for the shape
    (dict(dtype="BF16", shape=[4, 4], data_offsets=[0, 64]), "out of range"),        # past the end of the file
    (dict(dtype="BF16", shape=[-4, -4], data_offsets=[0, 32]), "bad dimension"),
    (dict(dtype="BF16", shape=[2.5, 4], data_offsets=[0, 20]), "bad dimension"),
    (dict(dtype="BF16", shape=[2 ** 40, 2 ** 40], data_offsets=[0, 32]), "overflows"),
    (dict(dtype="Q4", shape=[4, 4], data_offsets=[0, 32]), "unknown dtype"),
    (dict(dtype=7, shape=[4, 4], data_offsets=[0, 32]), "malformed"),
    (dict(dtype="BF16", shape="4x4", data_offsets=[0, 32]), "malformed"),
    (dict(dtype="BF16", shape=[4, 4], data_offsets=[-1, 31]), "out of range"),
])
def test_corrupt_safetensors_headers_are_refused(tmp_path, entry, msg):
    """A header is never trusted: byte counts must equal shape x dtype size, dimensions are whole
    and non-negative, dtypes known, offsets inside the file."""
    from pie_amd import driver as drvmod

    d = tmp_path / "corrupt"
    os.makedirs(d)
    (d / "config.json").write_text(json.dumps(dict(model_type="llama", hidden_size=64, num_hidden_layers=1,
                                                   num_attention_heads=2, num_key_value_heads=1,
                                                   intermediate_size=64, vocab_size=64)))
    _write_raw(d / "model.safetensors", {"model.norm.weight": entry}, b"\0" * 32)
    with pytest.raises(RuntimeError, match=msg):
        drvmod.snapshot_info(str(d))


def test_well_formed_raw_header_is_accepted(tmp_path):
    from pie_amd import driver as drvmod

    d = tmp_path / "fine"
    os.makedirs(d)
    (d / "config.json").write_text(json.dumps(dict(model_type="llama", hidden_size=64, num_hidden_layers=1,
                                                   num_attention_heads=2, num_key_value_heads=1,
                                                   intermediate_size=64, vocab_size=64)))
    _write_raw(d / "model.safetensors",
               {"model.norm.weight": dict(dtype="BF16", shape=[4, 4], data_offsets=[0, 32])}, b"\1" * 32)
    info = drvmod.snapshot_info(str(d))
    assert info["tensors"]["model.norm.weight"]["bytes"] == 32
