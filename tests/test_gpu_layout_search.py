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
    """On the interpreter route the search measures three admissible loader assignments,
    leaves the fastest on the graph, and that one is no slower than the layout the lowering
    picks by itself (10 % margin for timing noise)."""
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
            assert st["assignments"] == 72 and st["measurements"] == 5 and not st["truncated"]
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


def test_a_fused_operator_is_measured_once(rt, abi):
    """With the fused routes on (the default), C1's customized op runs on a fused GEMM kernel
    that keeps its tiles in its own layout: the search measures the kernel that actually runs,
    once, and every one of the 72 assignments gets that time."""
    from attention_superoptimizer_amd import graph as G
    g, vals = rt.build_from_spec(_matmul_spec(["SmemUnknownLayout"] * 2))
    try:
        vals[0][0].write_data(normal_f16([64, 1024], 0.1, 10))
        vals[1][0].write_data(normal_f16([1024, 1024], 0.1, 11))
        fused_ms = g.profile(2)
        st = G.optimize_layout(g)
        print("layout search on the fused route:", st, "fused", fused_ms, flush=True)
        assert st["assignments"] == 72 and st["measurements"] == 3 and not st["truncated"]
        assert st["best_ms"] == st["worst_ms"]
        assert st["best_ms"] < 3.0 * fused_ms
    finally:
        g.close()
