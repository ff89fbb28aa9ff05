"""The JSON wire format of mugraphs against the reference's own checkpoint data
(tests/golden/gqa_spec_decode_checkpoint_excerpt.json: the computation graph and every
ninth accepted graph of demo/checkpoint_group_query_attn_spec_decode.json, verbatim):
loading rebuilds the same graphs, writing reproduces the file's objects."""
import ctypes
import json
import os

import pytest

from attention_superoptimizer_amd import _native as N
from attention_superoptimizer_amd import graph as G
from helpers import GOLDEN, load_gqa_fixture


@pytest.fixture(scope="module")
def excerpt():
    with open(os.path.join(GOLDEN, "gqa_spec_decode_checkpoint_excerpt.json")) as f:
        return json.load(f)


def _normalise(doc):
    """guids renamed by first appearance (a rebuilt graph draws fresh ones); the field the
    checkpoint's older schema lacks is dropped."""
    names = {}

    def walk(x, key=None):
        if isinstance(x, dict):
            return {k: walk(v, k) for k, v in x.items() if k != "reduction_dimx"}
        if isinstance(x, list):
            return [walk(v) for v in x]
        if key == "guid":
            return names.setdefault(x, len(names))
        return x

    return walk(doc)


def _plans(g):
    out = []
    for i in range(g.num_operators):
        if g.op_type(i) == 1999:
            p = g.lowered(i, True)
            out.append((list(p.grid_dim), p.forloop_range, p.reduction_dimx, p.smem_bytes,
                        p.num_operators, list(p.operator_types)[:p.num_operators],
                        list(p.parameters)[:p.num_parameters]))
    return out


def test_written_json_reproduces_the_checkpoint_objects(excerpt):
    G.set_smem_budget(1 << 20)
    for ops in [excerpt["computation_graph"]] + excerpt["generated_graphs"]:
        g = G.KNGraph.from_json(ops)
        try:
            back = json.loads(g.to_json())
        finally:
            g.close()
        assert _normalise(back) == _normalise(ops)


def test_loaded_graphs_lower_like_the_converted_fixture(excerpt):
    """the same graphs rebuilt from the trimmed fixture through the builder API"""
    G.set_smem_budget(1 << 20)
    fixture = load_gqa_fixture()
    for idx, ops in zip(excerpt["indices"], excerpt["generated_graphs"]):
        a = G.KNGraph.from_json(ops)
        try:
            b, _ = G.build_from_spec(fixture["generated_graphs"][idx])
            try:
                assert a.num_operators == b.num_operators
                assert _plans(a) == _plans(b) and len(_plans(a)) >= 1
            finally:
                b.close()
        finally:
            a.close()


def test_reduction_dimx_defaults_and_round_trips(excerpt):
    G.set_smem_budget(1 << 20)
    ops = excerpt["generated_graphs"][0]
    assert all("reduction_dimx" not in op.get("plan", {}) for op in ops)   # older schema
    g = G.KNGraph.from_json(ops)
    try:
        back = json.loads(g.to_json())
    finally:
        g.close()
    plans = [op["plan"] for op in back if op["op_type"] == "kn_customized_op"]
    assert plans and all(p["reduction_dimx"] == 64 for p in plans)
    g2 = G.KNGraph.from_json(back)           # and what we write loads again
    try:
        assert _normalise(json.loads(g2.to_json())) == _normalise(back)
    finally:
        g2.close()


def test_malformed_json_is_rejected():
    for text in ["", "[", '[{"op_type": "kn_input_op"}]', '{"a": 1}x', '[{"op_type":"kn_matmul_op","input_tensors":[{"guid":1},{"guid":2}],"output_tensors":[{"guid":3}]}]'.replace("kn_matmul_op", "kn_nonsense")]:
        with pytest.raises((ValueError, SystemError, OSError)):
            G.KNGraph.from_json(text)
