"""GPU parity of batched verification: the verdict and every output fingerprint of
generated candidate mugraphs against the CPU oracle, bit for bit; at full size the
verdicts against what the generator constructed (fused rewrites equal, mutants not)."""
import numpy as np
import pytest

from attention_superoptimizer_amd import candidates as C
from helpers import uniform_fp
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu


def _inputs(spec, seed):
    ins, j = {}, 0
    for i, op in enumerate(spec):
        if op["op"] == "input":
            ins[i] = uniform_fp(op["dims"], seed ^ (j << 40))
            j += 1
    return ins


def _outputs(spec, vals):
    used = {tuple(r) for op in spec for r in op.get("in", [])}
    return [vals[i][j] for i in range(len(spec)) for j in range(len(vals[i])) if (i, j) not in used]


def _verify_problem(rt, prob):
    """Builds the reference and all candidates, runs one batched verify; returns
    (verdicts, per-candidate lists of output arrays, reference outputs)."""
    ref_g, ref_vals = rt.build_from_spec(prob["reference"])
    graphs = []
    try:
        ref_g.fingerprint_seeded(prob["input_seed"])
        vals = []
        for c in prob["candidates"]:
            g, v = rt.build_from_spec(c["spec"])
            graphs.append(g)
            vals.append(v)
        verdicts, stats = rt.verify_batch(graphs, ref_g, prob["input_seed"])
        outs = [[t.read_fingerprint() for t in _outputs(c["spec"], v)]
                for c, v in zip(prob["candidates"], vals)]
        ref_out = [t.read_fingerprint() for t in _outputs(prob["reference"], ref_vals)]
        assert stats["kernel_ops"] == sum(len(c["spec"]) for c in prob["candidates"])
        return verdicts, outs, ref_out
    finally:
        for g in reversed(graphs):
            g.close()
        ref_g.close()


def test_verify_batch_matches_oracle(rt):
    """Reduced dims (<= 128): every candidate output and verdict equals the oracle's."""
    probs = C.generate(num_problems=8, per_problem=8, max_dim=128)
    for prob in probs:
        verdicts, outs, ref_out = _verify_problem(rt, prob)
        seed = prob["input_seed"]
        want_ref = _outputs(prob["reference"],
                            orc.eval_graph(prob["reference"], "fp", _inputs(prob["reference"], seed),
                                           threads=8))
        assert len(ref_out) == len(want_ref)
        for a, b in zip(ref_out, want_ref):
            assert np.array_equal(a, b), prob["family"]
        for c, verdict, got in zip(prob["candidates"], verdicts, outs):
            want = _outputs(c["spec"], orc.eval_graph(c["spec"], "fp", _inputs(c["spec"], seed),
                                                      threads=8))
            assert len(got) == len(want)
            for a, b in zip(got, want):
                assert np.array_equal(a, b), (prob["family"], c["expect_equal"])
            oracle_verdict = len(want) == len(want_ref) and all(
                a.shape == b.shape and np.array_equal(a, b) for a, b in zip(want_ref, want))
            assert verdict == oracle_verdict == c["expect_equal"]


def test_verify_batch_full_size_verdicts(rt):
    """Full dims ([64, 1024]): rewrites verify equal, mutants unequal."""
    probs = C.generate(num_problems=8, per_problem=16, seed=0xBEEF)
    for prob in probs:
        verdicts, _, _ = _verify_problem(rt, prob)
        assert verdicts == [c["expect_equal"] for c in prob["candidates"]], prob["family"]


def test_verify_batch_iota_inputs_and_output_count(rt):
    """input_seed 0 = the reference's `idx % 25651` inputs; a candidate with a different
    number of outputs is rejected without a compare."""
    prob = C.generate(num_problems=1, per_problem=4, max_dim=128)[0]
    ref_g, _ = rt.build_from_spec(prob["reference"])
    graphs = []
    try:
        ref_g.fingerprint_seeded(0)
        for c in prob["candidates"]:
            graphs.append(rt.build_from_spec(c["spec"])[0])
        two_outputs = prob["reference"] + [{"op": "exp", "in": [[0, 0]]}]
        graphs.append(rt.build_from_spec(two_outputs)[0])
        verdicts, stats = rt.verify_batch(graphs, ref_g, 0)
        assert verdicts == [c["expect_equal"] for c in prob["candidates"]] + [False]
        assert stats["compares"] == len(prob["candidates"])
    finally:
        for g in reversed(graphs):
            g.close()
        ref_g.close()


def test_checkpoint_graphs_loaded_from_json_verify_equal(rt):
    """The reference's own checkpoint objects (original schema) loaded through the JSON
    wire format: every graph its search accepted verifies equal to the computation graph
    with the reference's `idx % 25651` inputs."""
    import json
    import os
    from helpers import GOLDEN
    with open(os.path.join(GOLDEN, "gqa_spec_decode_checkpoint_excerpt.json")) as f:
        doc = json.load(f)
    ref_g = rt.KNGraph.from_json(doc["computation_graph"])
    graphs = []
    try:
        ref_g.fingerprint_seeded(0)
        for ops in doc["generated_graphs"]:
            graphs.append(rt.KNGraph.from_json(ops))
        verdicts, stats = rt.verify_batch(graphs, ref_g, 0)
        assert verdicts == [True] * len(graphs)
        assert stats["customized_ops"] >= len(graphs)
    finally:
        for g in reversed(graphs):
            g.close()
        ref_g.close()
