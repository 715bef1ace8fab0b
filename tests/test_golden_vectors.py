"""The reference's own known answers for this path, kept as data in tests/golden/reference_known_answers.json
(written by tests/golden/make_known_answers.py), run against the oracle here and against the HIP path through
the C ABI in the GPU half of this file."""
import json
import math
import os

import numpy as np
import pytest

from oracle import binding as orc

GOLDEN = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")))


def logits_of(case):
    return np.array([math.nan if v == "nan" else v for v in case["logits"]], dtype=np.float32)


def check_codec(dequantize, case):
    out = dequantize(case["type"], np.array(case["bytes"], dtype=np.uint8))
    assert out.size == case.get("count", 1), case["cite"]
    for i, v in case["expect"].items():
        assert out[int(i)] == np.float32(v), (case["cite"], i)


def check_routing(route, case):
    ids, w = route(logits_of(case), case["tokens"], case["experts"], case["k"])
    if "ids" in case:
        assert ids.tolist() == case["ids"], case["cite"]
    for t, prefix in enumerate(case.get("ids_prefix", [])):
        assert ids[t, :len(prefix)].tolist() == prefix, case["cite"]
    if "weights" in case:
        assert np.all(np.abs(w - np.array(case["weights"])) < case["tol"]), case["cite"]
    if case.get("weights_softmax_of_selected_logits"):
        sel = [case["logits"][i] for i in case["ids"][0]]
        z = sum(math.exp(l) for l in sel)
        assert all(abs(float(g) - math.exp(l) / z) < case["tol"] for g, l in zip(w[0], sel)), case["cite"]
        assert abs(float(w[0].sum()) - 1.0) < case["tol"]
    if case.get("weights_finite_and_sum_to_one"):
        assert np.all(np.isfinite(w)) and np.all(np.abs(w.sum(axis=1) - 1.0) < case["tol"]), case["cite"]
    if "weight_at" in case:
        at = case["weight_at"]
        assert abs(float(w[at["token"], at["slot"]]) - at["value"]) < case["tol"], case["cite"]


@pytest.mark.parametrize("case", GOLDEN["codec"], ids=lambda c: f"type{c['type']}")
def test_oracle_dequantizes_the_reference_blocks(case):
    check_codec(orc.dequantize, case)


@pytest.mark.parametrize("case", GOLDEN["codec_refused"], ids=lambda c: f"{c['n_bytes']}B")
def test_oracle_refuses_partial_blocks(case):
    with pytest.raises(orc.OracleError):
        orc.dequantize(case["type"], np.zeros(case["n_bytes"], dtype=np.uint8))


@pytest.mark.parametrize("case", GOLDEN["router_qwen4exp"], ids=lambda c: c["cite"])
def test_oracle_routes_the_reference_logits(case):
    check_routing(orc.route_ggml, case)


@pytest.mark.parametrize("case", GOLDEN["router_refused"], ids=lambda c: f"k{c['k']}-{len(c['logits'])}")
def test_oracle_refuses_what_the_reference_refuses(case):
    with pytest.raises(orc.OracleError, match=case.get("message")):
        orc.route_ggml(logits_of(case), case["tokens"], case["experts"], case["k"])


@pytest.mark.parametrize("case", GOLDEN["renormalize_qwen4exp"], ids=lambda c: str(c["weights"]))
def test_oracle_clamps_a_vanishing_weight_sum(case):
    w = orc.renormalize_ggml(case["weights"])
    if "expect" in case:
        assert w.tolist() == case["expect"]
    else:
        assert abs(float(w[0]) - case["expect_first"]) < case["tol"]


# --- the same vectors through the C ABI of the HIP library ------------------------------------

@pytest.fixture(scope="module")
def handle():
    from mummu_amd import moe as M
    with M.SparseMoe(M.SparseMoeConfig(64, 32, 16, 2), max_tokens=8) as m:
        yield M, m


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLDEN["codec"], ids=lambda c: f"type{c['type']}")
def test_gpu_dequantizes_the_reference_blocks(handle, case):
    check_codec(handle[0].dequantize, case)


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLDEN["codec_refused"], ids=lambda c: f"{c['n_bytes']}B")
def test_gpu_refuses_partial_blocks(handle, case):
    M = handle[0]
    with pytest.raises(M.MoeError):
        M.dequantize(case["type"], np.zeros(case["n_bytes"], dtype=np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLDEN["router_qwen4exp"], ids=lambda c: c["cite"])
def test_gpu_routes_the_reference_logits(handle, case):
    M, m = handle
    check_routing(lambda lg, n, e, k: M.route(m, lg, n, e, k), case)


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLDEN["router_refused"], ids=lambda c: f"k{c['k']}-{len(c['logits'])}")
def test_gpu_refuses_what_the_reference_refuses(handle, case):
    M, m = handle
    with pytest.raises(M.MoeError, match=case.get("message")):
        M.route(m, logits_of(case), case["tokens"], case["experts"], case["k"])
