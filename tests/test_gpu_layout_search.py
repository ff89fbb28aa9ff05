"""Layout selection measured on the device (reference src/search/search.cc:699-777), and the
property it rests on: a declared LDS layout changes the time of a customized op, never its
result beyond the fp16 tolerance."""
import itertools
import json

import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu

OPT_FORCE_INTERPRETER, OPT_PLAN_SMEM_LAYOUT = 1, 3
KERNEL_INTERP = 2
LAYOUTS = ["SmemRowMajor", "SmemColumnMajor",
           "SmemRowMajorTensorOpMultiplicand_Crosswise16",
           "SmemRowMajorTensorOpMultiplicand_Crosswise32",
           "SmemRowMajorTensorOpMultiplicand_Crosswise64",
           "SmemColumnMajorTensorOpMultiplicand_Crosswise16",
           "SmemColumnMajorTensorOpMultiplicand_Crosswise32",
           "SmemColumnMajorTensorOpMultiplicand_Crosswise64",
           "SmemUnknownLayout"]


@pytest.fixture
def declared_layouts(abi):
    """fp16 interpreter, loader tiles laid out as the plan declares."""
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 1) == 0
    assert abi.mi355_set_option(OPT_PLAN_SMEM_LAYOUT, 1) == 0
    yield
    assert abi.mi355_set_option(OPT_PLAN_SMEM_LAYOUT, 0) == 0
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 0) == 0


def _matmul_spec(layouts):
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config1_fused_matmul()
    spec = json.loads(json.dumps(spec))
    spec[2]["plan"]["input_smem_layouts"] = list(layouts)
    return spec


def test_results_do_not_depend_on_declared_layouts(rt, abi, declared_layouts):
    """Every pair of declared layouts for the two loaders of A . B (the admissible ones,
    the ones the reference's search would prune, and 'unknown') gives the oracle's result."""
    import ctypes
    from attention_superoptimizer_amd import _native as N
    ins = {0: normal_f16([64, 1024], 0.1, 10), 1: normal_f16([1024, 1024], 0.1, 11)}
    want = orc.eval_graph(_matmul_spec(["SmemRowMajor"] * 2), "f16", ins, threads=8)[2][0]
    for la, lb in itertools.product(LAYOUTS, repeat=2):
        spec = _matmul_spec([la, lb])
        print("layouts", la, lb, flush=True)
        g, vals = rt.build_from_spec(spec)
        try:
            vals[0][0].write_data(ins[0])
            vals[1][0].write_data(ins[1])
            g.execute(2)
            info = N.Mi355LaunchInfo()
            N.backend().mi355_last_launch(ctypes.byref(info))
            assert info.kernel_id == KERNEL_INTERP
            assert_f16_close(vals[2][0].read_data(), want, what=f"A {la}, B {lb}")
        finally:
            g.close()


def test_optimize_layout_measured(rt, abi):
    """On the interpreter route the search measures the three admissible loader assignments
    under each of the 2^3 storage orders of A, B and C, leaves the fastest on the graph, and
    that one is no slower than the layout the lowering picks by itself (10 % margin for timing
    noise)."""
    from attention_superoptimizer_amd import graph as G
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 1) == 0
    try:
        g, vals = rt.build_from_spec(_matmul_spec(["SmemUnknownLayout"] * 2))
        try:
            vals[0][0].write_data(normal_f16([64, 1024], 0.1, 10))
            vals[1][0].write_data(normal_f16([1024, 1024], 0.1, 11))
            automatic_ms = g.profile(2)
            st = G.optimize_layout(g)
            print("layout search:", st, "automatic", automatic_ms, flush=True)
            assert st["assignments"] == 72 and st["measurements"] == 2 + 8 * 3 and not st["truncated"]
            assert st["unrunnable"] == 0
            assert st["best_ms"] <= st["first_ms"] <= st["worst_ms"]
            assert st["best_ms"] <= 1.10 * automatic_ms
            tb = json.loads(g.to_json())[2]["bgraph"]["operators"]
            la, lb = [o["output_tensors"][0]["layout"] for o in tb if o["op_type"] == "tb_input_op"]
            assert (la, lb) in {("SmemRowMajor", "SmemColumnMajor"),
                                ("SmemRowMajorTensorOpMultiplicand_Crosswise32",
                                 "SmemColumnMajorTensorOpMultiplicand_Crosswise32"),
                                ("SmemRowMajorTensorOpMultiplicand_Crosswise64",
                                 "SmemColumnMajorTensorOpMultiplicand_Crosswise64")}
            # the search switches the option back off
            g.execute(2)
        finally:
            g.close()
    finally:
        assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 0) == 0


def test_a_pruned_layout_is_slower(rt, abi, declared_layouts):
    """What the validity rules are for: A declared column-major is not k-contiguous, the tile
    matmul leaves the matrix cores, and the op takes several times longer.  (B may be staged
    either way: a row-major B tile is gathered with transposing LDS reads.)"""
    times = {}
    for la in ("SmemRowMajorTensorOpMultiplicand_Crosswise32", "SmemColumnMajor"):
        g, vals = rt.build_from_spec(
            _matmul_spec([la, "SmemColumnMajorTensorOpMultiplicand_Crosswise32"]))
        try:
            vals[0][0].write_data(normal_f16([64, 1024], 0.1, 10))
            vals[1][0].write_data(normal_f16([1024, 1024], 0.1, 11))
            times[la] = g.profile(2)
        finally:
            g.close()
    print("ms per launch:", times, flush=True)
    assert times["SmemColumnMajor"] > 2.0 * times["SmemRowMajorTensorOpMultiplicand_Crosswise32"]


def _device_layouts(g):
    return [o["output_tensors"][0]["layout"] for o in json.loads(g.to_json())]


def test_a_fused_operator_is_costed_per_storage_order(rt, abi):
    """With the fused routes on (the default), what the search can change for C1's customized
    op is the storage order of A, B and C: a fused GEMM kernel runs while A and C are row-major
    (one measurement per order of B, whatever the tiles' layouts: the kernel stages operands
    its own way), the interpreter otherwise (one per order and admissible pair of tile
    layouts).  The cheapest assignment keeps C row-major, is cheaper than the dearest, and
    the graph left behind computes the oracle's result from data written in the chosen orders."""
    from attention_superoptimizer_amd import graph as G
    spec = _matmul_spec(["SmemUnknownLayout"] * 2)
    ins = {0: normal_f16([64, 1024], 0.1, 10), 1: normal_f16([1024, 1024], 0.1, 11)}
    g, vals = rt.build_from_spec(spec)
    try:
        for i, a in ins.items():
            vals[i][0].write_data(a)
        fused_ms = g.profile(2)
        st = G.optimize_layout(g)
        print("layout search on the fused route:", st, "as declared", fused_ms, _device_layouts(g), flush=True)
        assert st["assignments"] == 72 and not st["truncated"] and st["unrunnable"] == 0
        assert st["measurements"] == 2 + 2 + 6 * 3
        assert st["best_ms"] < st["worst_ms"]
        assert st["best_ms"] <= 1.10 * fused_ms
        assert _device_layouts(g)[2] == "DmemRowMajor"
        for i, a in ins.items():
            vals[i][0].write_data(a)  # in the order the search chose
        g.execute(2)
        want = orc.eval_graph(spec, "f16", ins, threads=8)[2][0]
        assert_f16_close(vals[2][0].read_data(), want, what="C1 under the chosen layouts")
    finally:
        g.close()


def test_layout_search_chooses_the_storage_order_of_keys_and_values(rt, abi):
    """The decode-attention graph: Q row-major with K and V in one storage order runs on the
    fused attention kernel (two of the sixteen orders, at different speeds), every other order
    on the interpreter, tens of times slower.  The search leaves one of the two on the graph,
    and the graph computes the oracle's result from data written in the chosen orders."""
    from attention_superoptimizer_amd import graph as G
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config2_gqa_decode()
    G.set_smem_budget(1 << 20)
    ins = {i: normal_f16(op["dims"], 0.125, 40 + i) for i, op in enumerate(spec) if op["op"] == "input"}
    g, vals = rt.build_from_spec(spec)
    try:
        st = G.optimize_layout(g)
        lay = _device_layouts(g)
        print("layout search on decode attention:", st, lay, flush=True)
        assert st["assignments"] == 16 * 3 * 3 and not st["truncated"]
        # 2 fused orders, 14 on the interpreter with 3 admissible tile assignments each
        assert st["measurements"] == 3 + 2 + 14 * 3
        assert lay[0] == "DmemRowMajor" and lay[1] == lay[2] and lay[3] == "DmemRowMajor"
        assert st["worst_ms"] > 5.0 * st["best_ms"]
        for i, a in ins.items():
            vals[i][0].write_data(a)
        g.execute(3)
        want = orc.eval_graph(spec, "f16", ins, threads=8)[3][0]
        assert_f16_close(vals[3][0].read_data(), want, what="C2 under the chosen layouts")
    finally:
        g.close()


@pytest.mark.parametrize("forced", [0, 1], ids=["default-route", "interpreter"])
def test_a_column_major_result_is_stored_column_by_column(rt, abi, forced):
    """A search whose cost favours a column-major C leaves the saver's device tensor
    column-major; the customized op then runs on the interpreter (the fused kernels store rows)
    and writes C column by column: read back in that order, it is the oracle's result."""
    from attention_superoptimizer_amd import _native as N
    from attention_superoptimizer_amd import graph as G
    import ctypes
    spec = _matmul_spec(["SmemUnknownLayout"] * 2)
    ins = {0: normal_f16([64, 1024], 0.1, 20), 1: normal_f16([1024, 1024], 0.1, 21)}
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, forced) == 0
    g, vals = rt.build_from_spec(spec)
    try:
        def cost(op, layouts):
            return 1.0 if op == 2 and [l for l in layouts if l < 200] == [100, 101, 101] else 2.0

        G.optimize_layout(g, cost)
        assert _device_layouts(g) == ["DmemRowMajor", "DmemColumnMajor", "DmemColumnMajor"]
        assert vals[2][0].column_major and vals[1][0].column_major and not vals[0][0].column_major
        for i, a in ins.items():
            vals[i][0].write_data(a)
        g.execute(2)
        info = N.Mi355LaunchInfo()
        N.backend().mi355_last_launch(ctypes.byref(info))
        assert info.kernel_id == KERNEL_INTERP
        want = orc.eval_graph(spec, "f16", ins, threads=8)[2][0]
        assert_f16_close(vals[2][0].read_data(), want, what="column-major C")
    finally:
        g.close()
        assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 0) == 0
