"""Layout selection (reference src/search/search.cc:625-777): the enumeration and the
validity rules, checked on the host against an independent count, and the choice it makes
under a synthetic cost.  The measured variant runs in test_gpu_layout_search.py."""
import itertools
import json

from attention_superoptimizer_amd import graph as G
from attention_superoptimizer_amd import workloads as W

ROW, COL, ROW32, ROW64, COL32, COL64 = 200, 201, 203, 204, 206, 207
EXPLORED = [ROW, COL, ROW32, ROW64, COL32, COL64]
MATMUL_PAIRS = {(ROW, COL), (ROW32, COL32), (ROW64, COL64)}
ROW_FAMILY = {ROW, 202, ROW32, ROW64}
NAMES = {ROW: "SmemRowMajor", COL: "SmemColumnMajor",
         ROW32: "SmemRowMajorTensorOpMultiplicand_Crosswise32",
         ROW64: "SmemRowMajorTensorOpMultiplicand_Crosswise64",
         COL32: "SmemColumnMajorTensorOpMultiplicand_Crosswise32",
         COL64: "SmemColumnMajorTensorOpMultiplicand_Crosswise64"}


DROW, DCOL = 100, 101


def _split(layouts):
    """(device-tensor layouts, loader tile layouts) of a cost callback's list."""
    return tuple(l for l in layouts if l < 200), tuple(l for l in layouts if l >= 200)


def _matmul_graph():
    spec, _ = W.BASELINE_CONFIGS["C1_fused_matmul"]()
    return G.build_from_spec(spec)[0]


def _loader_layouts(graph, op_index):
    ops = json.loads(graph.to_json())
    tb = ops[op_index]["bgraph"]["operators"]
    return [o["output_tensors"][0]["layout"] for o in tb if o["op_type"] == "tb_input_op"]


def test_matmul_plan_enumeration_matches_an_independent_count():
    """A . B as one customized op: device tensors A, B, C take 2 layouts each; the loaders'
    tiles 6 each, of which the matmul admits 3 pairs; its result 6, of which the saver
    admits the 3 row-major ones.  2^3 * 3 * 3 = 72 complete assignments, and the operator
    is costed once per distinct set of layouts its time can depend on: those of A, B and C
    and the pair of loader layouts (an input operator's cost depends on none)."""
    g = _matmul_graph()
    try:
        seen = []

        def cost(op, layouts):
            seen.append((op, tuple(layouts)))
            return 1.0

        st = G.optimize_layout(g, cost)
        brute = 0
        for a, b, c in itertools.product(EXPLORED, repeat=3):
            if (a, b) in MATMUL_PAIRS and c in ROW_FAMILY:
                brute += 1
        assert st["assignments"] == 8 * brute == 72
        assert not st["truncated"]
        # inputs A and B once each, the customized op once per (A, B, C, admissible pair)
        want = [(0, ()), (1, ())] + [(2, d + p) for d in itertools.product((DROW, DCOL), repeat=3)
                                     for p in MATMUL_PAIRS]
        assert sorted(seen) == sorted(want)
        assert st["measurements"] == len(seen) == 26 and st["unrunnable"] == 0
    finally:
        g.close()


def test_the_cheapest_assignment_is_left_on_the_graph():
    g = _matmul_graph()
    try:
        want = (ROW64, COL64)

        def cost(op, layouts):
            if op != 2:
                return 0.0
            device, loaders = _split(layouts)
            # B column-major is worth one unit, the right pair of tile layouts two
            return 4.0 - (1.0 if device == (DROW, DCOL, DROW) else 0.0) - (2.0 if loaders == want else 0.0)

        st = G.optimize_layout(g, cost)
        assert st["best_ms"] == 1.0 and st["worst_ms"] == 4.0
        assert _loader_layouts(g, 2) == [NAMES[l] for l in want]
        # the device tensors carry the chosen layouts, and so do the copies the customized
        # operator, its loaders and its saver hold
        ops = json.loads(g.to_json())
        assert [o["output_tensors"][0]["layout"] for o in ops] == ["DmemRowMajor", "DmemColumnMajor", "DmemRowMajor"]
        assert [t["layout"] for t in ops[2]["input_tensors"]] == ["DmemRowMajor", "DmemColumnMajor"]
        held = [o["dtensor"]["layout"] for o in ops[2]["bgraph"]["operators"] if "dtensor" in o]
        assert held == ["DmemRowMajor", "DmemColumnMajor", "DmemRowMajor"]
        # the copies the consumers hold follow: the matmul's operands carry the same layouts
        tb = json.loads(g.to_json())[2]["bgraph"]["operators"]
        mm = [o for o in tb if o["op_type"] == "tb_matmul_op"][0]
        assert [t["layout"] for t in mm["input_tensors"]] == [NAMES[l] for l in want]
    finally:
        g.close()


def test_attention_plan_rules_prune_the_search():
    """matmul -> exp -> reduction -> div -> matmul: Q and K may form any of the three
    admissible pairs; the reduction only takes a plain row- or column-major S, P = S / sum
    inherits that, and the second matmul then needs P row-major and V plain column-major.
    Of the 6^3 loader assignments three survive."""
    spec, _ = W.BASELINE_CONFIGS["C2_gqa_decode"]()
    G.set_smem_budget(1 << 20)  # the plan's tiles need more than the reference's 96 KB
    g = G.build_from_spec(spec)[0]
    try:
        costed = set()

        def cost(op, layouts):
            if _split(layouts)[1]:
                costed.add(_split(layouts)[1])
            return 1.0

        st = G.optimize_layout(g, cost)
        assert costed == {(ROW, COL, COL), (ROW32, COL32, COL), (ROW64, COL64, COL)}
        # 2^4 device-tensor layouts x 3 loader assignments x the 3 row-major layouts of O
        assert st["assignments"] == 16 * 3 * 3 and not st["truncated"]
        assert _loader_layouts(g, 3) == [NAMES[ROW], NAMES[COL], NAMES[COL]]  # first of the ties
    finally:
        g.close()


def test_assignment_budget_truncates():
    g = _matmul_graph()
    try:
        st = G.optimize_layout(g, lambda op, loaders: 1.0, max_assignments=10)
        assert st["assignments"] == 10 and st["truncated"]
    finally:
        g.close()
