"""Every example plan of the reference (cpp_examples/*.cc and the thread-block matmul test,
tests/threadblock/matmul.cu:163-189), at the size the reference runs it, on the device in both
domains: fingerprints bit for bit against the oracle and against the un-fused graph (the
reference's own check, has_same_fingerprint of the two), fp16 against the oracle's fp16 golden
within |gpu - golden| <= 1e-3 + 1e-2 |golden|, on the default route and on the interpreter."""

import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16, uniform_fp
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu

EXAMPLES = ["dnn", "group_query_attn_inc_decode", "group_query_attn_spec_decode",
            "group_query_attn_prefill", "multi_head_attn_inc_decode", "multi_head_attn_spec_decode",
            "multi_head_attn_prefill", "multi_query_attn_inc_decode", "multi_query_attn_spec_decode",
            "multi_query_attn_prefill", "lora", "mlp", "moe", "tb_matmul_test"]
# fp16 inputs: N(0, std), small enough that exp stays finite and that an fp16 for-loop
# accumulator stays where one of its ulps is below the tolerance
STD = {"moe": 0.02, "tb_matmul_test": 0.03, "lora": 0.05, "mlp": 0.02}
# Inputs taken by magnitude.  moe sums exp(.) ~ 1 against 4096 weights: with weights of both
# signs the fp16 for-loop accumulator passes through values of a few units on its way to a
# result near zero, and two correct evaluations that order a tile product's fp32 additions
# differently end one ulp OF THE ACCUMULATOR apart, above the tolerance around that result.
NON_NEGATIVE = {"moe": (2,)}
OPT_FORCE_INTERPRETER = 1

_golden = {}


def _spec(name):
    from attention_superoptimizer_amd import workloads as W
    return W.REFERENCE_EXAMPLES[name]


def test_the_list_is_every_example_the_reference_has():
    from attention_superoptimizer_amd import workloads as W
    assert sorted(EXAMPLES) == sorted(W.REFERENCE_EXAMPLES)


@pytest.mark.parametrize("name", EXAMPLES)
def test_example_fingerprints_at_full_size(rt, name):
    spec, ref = _spec(name)
    for what, ins in (("idx % 25651 inputs, as the reference fills them", None),
                      ("random inputs", {i: uniform_fp(op["dims"], 100 + i)
                                         for i, op in enumerate(spec) if op["op"] == "input"})):
        print(name, what, flush=True)
        g, vals = rt.build_from_spec(spec)
        try:
            for i, op in enumerate(spec):
                if op["op"] == "input" and ins is not None:
                    vals[i][0].write_fingerprint(ins[i])
                else:
                    g.fingerprint(i)
            got = [[t.read_fingerprint() for t in v] for v in vals]
        finally:
            g.close()
        want = orc.eval_graph(spec, "fp", ins, threads=16)
        for i, op in enumerate(spec):
            for j, w in enumerate(want[i]):
                assert np.array_equal(got[i][j], w), (name, what, i, j, op["op"])
        # the un-fused graph on the device gives the same fingerprint
        g, vals = rt.build_from_spec(ref)
        try:
            for i, op in enumerate(ref):
                if op["op"] == "input" and ins is not None:
                    vals[i][0].write_fingerprint(ins[i])
                else:
                    g.fingerprint(i)
            assert np.array_equal(vals[-1][0].read_fingerprint(), got[-1][0]), (name, what)
        finally:
            g.close()


@pytest.mark.parametrize("route", ["default", "interpreter"])
@pytest.mark.parametrize("name", EXAMPLES)
def test_example_fp16_at_full_size(rt, abi, name, route):
    spec, _ = _spec(name)
    ins = {i: normal_f16(op["dims"], STD.get(name, 0.05), 60 + i)
           for i, op in enumerate(spec) if op["op"] == "input"}
    for i in NON_NEGATIVE.get(name, ()):
        ins[i] = np.abs(ins[i])
    if name not in _golden:
        _golden[name] = orc.eval_graph(spec, "f16", ins, threads=16)
    want = _golden[name]
    print(name, route, flush=True)
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 1 if route == "interpreter" else 0) == 0
    g, vals = rt.build_from_spec(spec)
    try:
        for i, op in enumerate(spec):
            if op["op"] == "input":
                vals[i][0].write_data(ins[i])
            else:
                g.execute(i)
        for i, op in enumerate(spec):
            if op["op"] == "input":
                continue
            for j, w in enumerate(want[i]):
                assert_f16_close(vals[i][j].read_data(), w, what=f"{name} ({route}) op {i} ({op['op']}) out {j}")
    finally:
        g.close()
        assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 0) == 0
