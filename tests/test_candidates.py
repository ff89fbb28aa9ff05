"""CPU checks of the candidate-mugraph generator: determinism, the search limits it claims
to respect, that every plan lowers through the host API and fits the device's LDS, and that
the oracle agrees with the constructed verdicts (rewrites equal, mutants unequal)."""
import ctypes

import numpy as np

from attention_superoptimizer_amd import _native as N
from attention_superoptimizer_amd import candidates as C
from attention_superoptimizer_amd import graph as G
from helpers import uniform_fp
from oracle import evaluate as orc


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


def test_generator_is_deterministic_and_within_search_limits():
    a = C.generate(num_problems=16, per_problem=16)
    b = C.generate(num_problems=16, per_problem=16)
    assert a == b
    assert C.generate(num_problems=2, per_problem=2, seed=1) != C.generate(num_problems=2, per_problem=2, seed=2)
    for prob in a:
        for c in prob["candidates"]:
            spec = c["spec"]
            assert 8 <= c["operators"] <= 12
            assert len(spec) <= 5                                   # MAX_NUM_KERNEL_GRAPH_OP
            cust = [op for op in spec if op["op"] == "customized"]
            assert 1 <= len(cust) <= 2                              # MAX_NUM_THREADBLOCK
            for op in cust:
                assert len(op["plan"]["input_map"]) <= 3           # MAX_NUM_THREADBLOCK_INPUT
                assert len(op["plan"]["input_map"]) + len(op["plan"]["ops"]) <= 8
            for op in spec:
                if op["op"] == "input":
                    assert all(d == 1 or 64 <= d <= 1024 and d & (d - 1) == 0 for d in op["dims"][-2:])


def test_all_4096_candidates_lower_and_fit_lds():
    G.set_smem_budget(1 << 20)
    probs = C.generate()
    assert sum(len(p["candidates"]) for p in probs) == 4096
    for prob in probs:
        for spec in [prob["reference"]] + [c["spec"] for c in prob["candidates"]]:
            g, _ = G.build_from_spec(spec)
            try:
                for i, op in enumerate(spec):
                    if op["op"] != "customized":
                        continue
                    pl = g.lowered(i, True)
                    lds = ctypes.c_int()
                    ie, oe = (ctypes.c_longlong * 4)(), (ctypes.c_longlong * 4)()
                    assert N.backend().mi355_plan_extents(ctypes.byref(pl), ie, oe, ctypes.byref(lds), None) == 0
                    assert lds.value <= 160 * 1024
            finally:
                g.close()


def test_oracle_agrees_with_constructed_verdicts():
    for prob in C.generate(num_problems=8, per_problem=8, max_dim=128):
        seed = prob["input_seed"]
        ref = _outputs(prob["reference"],
                       orc.eval_graph(prob["reference"], "fp", _inputs(prob["reference"], seed)))
        for c in prob["candidates"]:
            out = _outputs(c["spec"], orc.eval_graph(c["spec"], "fp", _inputs(c["spec"], seed)))
            eq = len(out) == len(ref) and all(
                a.shape == b.shape and np.array_equal(a, b) for a, b in zip(ref, out))
            assert eq == c["expect_equal"], (prob["family"], c["expect_equal"])
