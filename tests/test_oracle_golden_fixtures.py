"""The CPU oracle against the committed fixture of the reference's own known-answer vectors
(tests/golden/reference_vectors.json: data only, every entry naming the reference test it comes from)."""
import json
import os

import numpy as np
import pytest

FIX = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def test_block_bytes(oracle):
    assert oracle.BLOCK_BYTES[oracle.Q6K] == FIX["block_bytes"]["q6_k"]
    assert oracle.BLOCK_BYTES[oracle.Q8_0] == FIX["block_bytes"]["q8_0"]


@pytest.mark.parametrize("v", FIX["dequantize_q6_k"], ids=lambda v: v["source"][:40])
def test_dequantize_q6_k(oracle, v):
    y = oracle.dequantize_row(oracle.Q6K, np.array(v["bytes"], np.uint8))
    assert y[0] == v["expect_first"] and np.all(y[1:] == v["expect_rest"])


@pytest.mark.parametrize("v", FIX["dequantize_q8_0"], ids=lambda v: v["source"][:40])
def test_dequantize_q8_0(oracle, v):
    assert np.all(oracle.dequantize_row(oracle.Q8_0, np.array(v["bytes"], np.uint8)) == v["expect_all"])


@pytest.mark.parametrize("v", FIX["route_token"], ids=lambda v: v["source"][-60:])
def test_route_token(oracle, v):
    ids, w = oracle.route_token(np.array(v["logits"], np.float32), v["k"])
    assert list(ids) == v["ids"]
    if "weights_sum" in v:
        assert abs(float(w.sum()) - v["weights_sum"]) < 1e-5
    if v.get("weights_descending"):
        assert all(w[i] > w[i + 1] for i in range(len(w) - 1))
    if "weights_each" in v:
        assert np.allclose(w, v["weights_each"])


@pytest.mark.parametrize("v", FIX["route_batch"], ids=lambda v: v["source"][-30:])
def test_route_batch(oracle, v):
    ids, _ = oracle.route_batch(np.array(v["logits"], np.float32), v["k"])
    assert ids.tolist() == v["ids"]


@pytest.mark.parametrize("v", FIX["moe_align_block_size"], ids=lambda v: v["source"][-40:])
def test_moe_align_block_size(oracle, v):
    d = oracle.moe_align_block_size(v["topk_ids"], v["block_size"], v["num_experts"])
    assert d.sorted_token_ids.tolist() == v["sorted_token_ids"]
    assert d.expert_ids.tolist() == v["expert_ids"]
    assert d.num_tokens_post_pad == v["num_tokens_post_pad"]


@pytest.mark.parametrize("v", FIX["gemv"], ids=lambda v: v["source"][-50:])
def test_gemv(oracle, v):
    assert oracle.gemv(v["w"], v["rows"], v["cols"], v["x"]).tolist() == v["y"]


@pytest.mark.parametrize("v", FIX["argmax"], ids=lambda v: str(v["x"]))
def test_argmax(oracle, v):
    assert oracle.argmax(v["x"]) == v["index"]


@pytest.mark.parametrize("v", FIX["rms_norm"], ids=lambda v: str(v["x"]))
def test_rms_norm(oracle, v):
    out = oracle.rms_norm(v["x"], v["w"], v["eps"])
    assert np.abs(out - np.array(v["y"], np.float32)).max() <= v["atol"]


@pytest.mark.parametrize("v", FIX["scalars"], ids=lambda v: "%s(%s)" % (v["fn"], v["x"]))
def test_scalars(oracle, v):
    assert abs(getattr(oracle, v["fn"])(v["x"]) - v["y"]) <= v["atol"]


@pytest.mark.parametrize("v", FIX["geometry_capacities"], ids=lambda v: str(v["max_tokens"]))
def test_geometry_capacities(oracle, v):
    assert oracle.lib().xo_max_flat_pairs(v["max_tokens"], v["top_k"]) == v["max_flat_pairs"]
    assert oracle.sorted_capacity(v["num_experts"], v["top_k"], v["block_size"], v["max_tokens"]) == v["sorted_capacity"]
    assert oracle.expert_block_capacity(v["num_experts"], v["top_k"], v["block_size"], v["max_tokens"]) == v["expert_block_capacity"]
