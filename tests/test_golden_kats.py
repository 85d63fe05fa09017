"""The CPU oracle against the known answers collected in tests/golden/reference_kats.json
(constants of the reference's own tests and kernel sources; each entry cites its origin)."""
import json
from pathlib import Path

import numpy as np
import pytest

KATS = json.loads((Path(__file__).parent / "golden" / "reference_kats.json").read_text())


def test_decode_plan_known_answer():
    from oracle import planner as op

    k = KATS["decode_plan"]
    i = k["input"]
    p = op.plan_forward(i["token_ids"], i["position_ids"], i["kv_page_indices"], i["kv_page_indptr"],
                        i["kv_last_page_lens"], i["qo_indptr"], i["sampling_indices"], i["sampling_indptr"],
                        i["page_size"], i["total_pages"])
    for key, want in k["expect"].items():
        got = p[key]
        assert (list(got) if isinstance(want, list) else got) == want, key


def test_int4_unpack_known_answer(oracle):
    k = KATS["int4_unpack"]
    packed = np.array([k["packed_words"]], np.uint32)
    assert oracle.unpack_w4(packed, 1, 8 * len(k["packed_words"])).tolist() == [k["expect"]]


def test_int8_per_channel_quant_known_answer(oracle):
    k = KATS["int8_per_channel_quant"]
    q, s = oracle.quant_int8_per_channel(oracle.f32_to_bf16(np.array(k["rows"], np.float32)))
    assert q.tolist() == k["expect_codes"]
    for got, (num, den) in zip(s, k["expect_scale_num_den"]):
        assert got == np.float32(num) / np.float32(den)


def test_pcg32_known_answer(oracle):
    k = KATS["pcg32"]
    got = [int(x) for x in oracle.pcg32_sequence(k["seed"], k["stream"], len(k["expect_hex"]))]
    assert got == [int(h, 16) for h in k["expect_hex"]]


@pytest.mark.parametrize("case", KATS["brle_masks"]["cases"], ids=lambda c: f"runs{c['runs']}-pos{c['pos']}-w{c['window']}")
def test_brle_mask_known_answers(oracle, case):
    assert list(oracle.brle_allow(case["runs"], case["pos"], case["n_kv"], case["window"])) == case["expect"]
