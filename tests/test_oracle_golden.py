"""The CPU oracle against the known answers the reference's own tests hold
(TestCustomModelsFromONNX.cxx:330-349,372-391,693-712,860-990,1023-1052)."""
import json
import os

import numpy as np
import pytest

from sofie_amd import onnx_wire
import replay
from oracle import oracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLD, "expected.json")) as f:
    EXPECTED = json.load(f)

# The reference compares with 1e-3 absolute (TestCustomModelsFromONNX.cxx:328).
TOL = 1e-3


@pytest.mark.parametrize("name", sorted(EXPECTED))
def test_oracle_matches_reference_known_answer(name):
    entry = EXPECTED[name]
    graph = onnx_wire.load(os.path.join(GOLD, "onnx", name + ".onnx"))
    feeds = replay.fixture_feeds(entry, graph)
    y = replay.run_graph(graph, feeds, oracle)
    want = np.array(entry["expected"], np.float32)
    assert y.size == want.size
    assert np.max(np.abs(y.reshape(-1) - want)) <= TOL
    if name.startswith("Conv") or name.startswith("Einsum"):
        # integer-valued data: the answer is exact
        assert np.array_equal(y.reshape(-1), want)


def test_linear_fixture_against_float64_closed_form():
    graph = onnx_wire.load(os.path.join(GOLD, "onnx", "Linear_16.onnx"))
    x = np.ones((16, 100), np.float32)
    y = replay.run_graph(graph, {graph["inputs"][0][0]: x}, oracle)
    env = {k: v.astype(np.float64) for k, v in graph["initializers"].items()}
    env[graph["inputs"][0][0]] = x.astype(np.float64)
    for node in graph["nodes"]:
        i = node["inputs"]
        if node["op_type"] == "Gemm":
            env[node["outputs"][0]] = env[i[0]] @ env[i[1]].T + env[i[2]]
        else:
            env[node["outputs"][0]] = np.maximum(env[i[0]], 0)
    truth = env[graph["outputs"][0][0]]
    assert np.max(np.abs(y - truth)) <= 1e-5 * np.max(np.abs(truth))
