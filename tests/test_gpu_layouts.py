"""GPU parity of the fp16 path on BOTH storage orders of its operands.

A DmemColumnMajor tensor holds each [rows, cols] matrix column by column (reference
include/mirage/threadblock/cuda/input_loader.h:221-247; every attention plan of the reference
declares K and V that way, every GEMM plan its weights).  The logical values and therefore the
golden do not depend on the layout, so every case runs with its B-side operands row-major and
column-major and both results must meet the oracle's fp16 golden:

    |gpu - golden| <= 1e-3 + 1e-2 |golden|

Fingerprint buffers are row-major whatever the declaration (input_loader.h:457-467); the last
test checks that a layout change leaves fingerprints alone."""
import ctypes

import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16, uniform_fp
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu

ROW, COL = "DmemRowMajor", "DmemColumnMajor"
KERNEL_INTERP, KERNEL_ATTENTION, KERNEL_GEMM, KERNEL_COMBINE = 2, 3, 4, 5


def _with_layouts(spec, layouts):
    """A copy of `spec` whose input operators take the layouts of `layouts` (op index -> name)."""
    out = []
    for i, op in enumerate(spec):
        op = dict(op)
        if op["op"] == "input" and i in layouts:
            op["layout"] = layouts[i]
        out.append(op)
    return out


def _run_f16(rt, spec, ins):
    from attention_superoptimizer_amd import _native as N
    g, vals = rt.build_from_spec(spec)
    kernels = []
    try:
        for i, op in enumerate(spec):
            if op["op"] == "input":
                vals[i][0].write_data(ins[i])
            else:
                g.execute(i)
                if op["op"] == "customized":
                    info = N.Mi355LaunchInfo()
                    N.backend().mi355_last_launch(ctypes.byref(info))
                    kernels.append(info.kernel_id)
        return [[t.read_data() for t in v] for v in vals], kernels
    finally:
        g.close()


def _b_side_inputs(spec):
    """Input operators that are declared column-major in the catalogue (K, V, weights)."""
    return [i for i, op in enumerate(spec) if op["op"] == "input" and op.get("layout") == COL]


def _both_layouts(rt, abi, spec, ins, what, routes=("fused", "interpreter"), want=None):
    """Runs `spec` with its B-side operands row- and column-major on each route and checks every
    customized operator's outputs against the oracle; returns the kernels of the fused route."""
    if want is None:
        want = orc.eval_graph(spec, "f16", ins, threads=8)
    b_side = _b_side_inputs(spec)
    assert b_side, what
    fused_kernels = {}
    for layout in (COL, ROW):
        sp = _with_layouts(spec, {i: layout for i in b_side})
        for route in routes:
            assert abi.mi355_set_option(1, 1 if route == "interpreter" else 0) == 0
            try:
                got, kernels = _run_f16(rt, sp, ins)
            finally:
                assert abi.mi355_set_option(1, 0) == 0
            if route == "interpreter":
                assert all(k == KERNEL_INTERP for k in kernels), (what, layout, kernels)
            else:
                fused_kernels[layout] = kernels
            for i, op in enumerate(sp):
                if op["op"] == "customized":
                    for j, w in enumerate(want[i]):
                        assert_f16_close(got[i][j], w, what=f"{what}, B side {layout}, {route}, op {i} out {j}")
    return fused_kernels


def test_data_round_trips_through_a_column_major_buffer(rt, abi):
    """write_data / read_data move LOGICAL values; the device buffer of a column-major tensor holds
    the transposed matrices (checked through a raw copy of the buffer)."""
    from attention_superoptimizer_amd import graph as G
    g = G.KNGraph()
    try:
        t = g.new_input((3, 16, 40), layout=COL)
        r = g.new_input((3, 16, 40), layout=ROW)
        a = normal_f16([3, 16, 40], 1.0, 5)
        t.write_data(a)
        r.write_data(a)
        assert np.array_equal(t.read_data(), a) and np.array_equal(r.read_data(), a)
        raw = np.empty((3, 40, 16), np.float16)
        assert abi.mi355_memcpy_d2h(raw.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(t.device_ptr(False)),
                                    raw.nbytes) == 0
        assert np.array_equal(raw, a.swapaxes(1, 2))
    finally:
        g.close()


def test_config2_both_layouts(rt, abi):
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config2_gqa_decode()
    ins = {i: normal_f16(op["dims"], 0.125, 40 + i) for i, op in enumerate(spec) if op["op"] == "input"}
    kernels = _both_layouts(rt, abi, spec, ins, "C2")
    assert kernels[COL] == [KERNEL_ATTENTION] and kernels[ROW] == [KERNEL_ATTENTION]


def test_config3_heads_both_layouts(rt, abi):
    """Config C3 at its full sequence length and head size on 4 of its 32 heads, 64-key tiles; the
    interpreter route runs too (the tiles fit its LDS)."""
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config3_mha_prefill(heads=4, q_split=16, F=32)
    ins = {i: normal_f16(op["dims"], 128 ** -0.5, 50 + i) for i, op in enumerate(spec) if op["op"] == "input"}
    # (values of one sign: the un-normalised numerator then grows steadily over the 32 iterations,
    # so one fp16 ulp of its accumulator stays inside the tolerance; the cancelling case is
    # test_gpu_oracle_slices.py's, with the accumulator's path in the bound)
    ins[2] = np.abs(ins[2])
    kernels = _both_layouts(rt, abi, spec, ins, "C3, 4 heads")
    for layout in (COL, ROW):
        assert kernels[layout] == [KERNEL_ATTENTION, KERNEL_COMBINE], (layout, kernels)


@pytest.mark.parametrize("keys", [128, 256, 512])
def test_config3_wider_key_tiles_both_layouts(rt, abi, keys):
    """The same problem with its key range walked in tiles of 128 / 256 / 512 keys (strips of 64
    inside the throughput kernel, fp32 sums across the strips of an iteration): 8 heads, against
    the oracle's golden for that plan on 2 heads and
    against float64 softmax attention on all of them."""
    from attention_superoptimizer_amd import workloads as W
    heads = 8
    spec, _ = W.config3_mha_prefill(heads=heads, q_split=16, F=2048 // keys)
    ins = {i: normal_f16(op["dims"], 128 ** -0.5, 60 + i) for i, op in enumerate(spec) if op["op"] == "input"}
    ins[2] = np.abs(ins[2])  # (see test_config3_heads_both_layouts)
    # the oracle on the thread blocks of heads 0 and 5 (grid (heads, 1, 16): bx + heads * bz)
    blocks = [h + heads * bz for h in (0, 5) for bz in range(16)]
    gold1 = orc.customized(spec[3]["plan"], [ins[0], ins[1], ins[2]], f16=True, threads=8, blocks=blocks)
    s = np.einsum("hqd,hdk->hqk", ins[0].astype(np.float64), ins[1].astype(np.float64))
    e = np.exp(s)
    exact = np.einsum("hqk,hkd->hqd", e / e.sum(-1, keepdims=True), ins[2].astype(np.float64))
    for layout in (COL, ROW):
        sp = _with_layouts(spec, {1: layout, 2: layout})
        got, kernels = _run_f16(rt, sp, ins)
        assert kernels == [KERNEL_ATTENTION, KERNEL_COMBINE], (layout, kernels)
        for j in range(2):
            mask = orc.written(gold1[j])
            assert mask.any()
            assert_f16_close(got[3][j][mask], gold1[j].view(np.float16)[mask],
                             what=f"C3 {keys}-key tiles, {layout}, op1 out {j}")
        assert_f16_close(got[4][0], exact.astype(np.float16), what=f"C3 {keys}-key tiles, {layout}, vs float64")


@pytest.mark.parametrize("name", ["group_query_attn_inc_decode", "multi_head_attn_prefill", "lora", "mlp"])
def test_example_plans_both_layouts(rt, abi, name):
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.REFERENCE_EXAMPLES[name]
    std = {"lora": 0.05, "mlp": 0.02}.get(name, 0.125)
    ins = {i: normal_f16(op["dims"], std, 70 + i) for i, op in enumerate(spec) if op["op"] == "input"}
    if name == "mlp":
        ins[0] = np.abs(ins[0])  # (keeps the 8192-term sums away from cancellation)
        ins[1] = np.abs(ins[1])
    elif name not in ("lora",):
        ins[2] = np.abs(ins[2])  # (numerators that grow steadily, see test_config3_heads_both_layouts)
    _both_layouts(rt, abi, spec, ins, name)


def test_gemm_configs_both_layouts_on_both_fused_kernels(rt, abi):
    """C1 and C4 at full size, a reduced C5a: weights row- and column-major, on the kernel that cuts
    the for-loop into ranges and on the one-launch kernel (option 7 = 1 / 2)."""
    from attention_superoptimizer_amd import workloads as W
    cases = {
        "C1": (W.config1_fused_matmul()[0], {0: 0.1, 1: 0.1}),
        "C4": (W.config4_lora()[0], {0: 0.25, 1: 0.02, 2: 0.02, 3: 0.02}),
        "C5s": (W.config5_gated_mlp(m=8, d=1024, h=3584, grid1=56, F1=4, grid2=16, F2=14)[0],
                {0: 0.25, 1: 0.02, 2: 0.02, 3: 0.02}),
    }
    for what, (spec, stds) in cases.items():
        ins = {i: normal_f16(op["dims"], stds[i], 80 + i) for i, op in enumerate(spec) if op["op"] == "input"}
        want = orc.eval_graph(spec, "f16", ins, threads=8)
        for mode in (1, 2):
            assert abi.mi355_set_option(7, mode) == 0
            try:
                kernels = _both_layouts(rt, abi, spec, ins, f"{what}, gemm kernel {mode}", routes=("fused",),
                                        want=want)
            finally:
                assert abi.mi355_set_option(7, 0) == 0
            for layout in (COL, ROW):
                assert all(k == KERNEL_GEMM for k in kernels[layout]), (what, mode, layout, kernels)


def test_ragged_column_major_tiles_on_the_interpreter(rt, abi):
    """Tiles whose contiguous direction is not a multiple of 8 elements take the interpreter's
    scalar loads: a column-major A operand, a column-major B operand, both, [30, 44] . [44, 52]."""
    m, k, n = 30, 44, 52
    for la, lb in ((ROW, COL), (COL, ROW), (COL, COL)):
        spec = [
            {"op": "input", "dims": [2, m, k], "layout": la}, {"op": "input", "dims": [2, k, n], "layout": lb},
            {"op": "customized", "in": [[0, 0], [1, 0]], "plan": {
                "grid_dim": [2, 1, 1], "forloop_range": 2, "reduction_dimx": 64,
                "input_map": [[0, -1, -1], [0, -1, -1]], "forloop_dim": [2, 1], "output_map": [0, -1, -1],
                "ops": [["tb_matmul_op", [[0, 0], [1, 0]]]]}},
        ]
        ins = {0: normal_f16([2, m, k], 0.3, 1), 1: normal_f16([2, k, n], 0.3, 2)}
        want = orc.eval_graph(spec, "f16", ins)[2][0]
        got, kernels = _run_f16(rt, spec, ins)
        assert kernels == [KERNEL_INTERP]
        assert_f16_close(got[2][0], want, what=f"ragged tiles, A {la}, B {lb}")


def test_kernel_level_operators_read_column_major_inputs(rt, abi):
    """The un-fused graph of every attention example has column-major K and V feeding kernel-level
    matmuls (e.g. cpp_examples/group_query_attn_inc_decode.cc:16-27); element-wise operators and
    reductions get a row-major copy of a column-major input."""
    for la, lb in ((ROW, ROW), (ROW, COL), (COL, ROW), (COL, COL)):
        spec = [
            {"op": "input", "dims": [3, 70, 96], "layout": la}, {"op": "input", "dims": [3, 96, 130], "layout": lb},
            {"op": "matmul", "in": [[0, 0], [1, 0]]},
            {"op": "exp", "in": [[1, 0]]},
            {"op": "mul", "in": [[1, 0], [3, 0]]},
            {"op": "reduction", "in": [[1, 0]], "dim": 2, "size": 1},
            {"op": "reduction", "in": [[0, 0]], "dim": 1, "size": 35},
        ]
        ins = {0: normal_f16([3, 70, 96], 0.1, 3), 1: normal_f16([3, 96, 130], 0.1, 4)}
        want = orc.eval_graph(spec, "f16", ins)
        got, _ = _run_f16(rt, spec, ins)
        for i in range(2, len(spec)):
            assert_f16_close(got[i][0], want[i][0], what=f"A {la}, B {lb}, op {i} ({spec[i]['op']})")


def test_fingerprints_do_not_depend_on_the_layout(rt):
    """The fingerprint of a column-major tensor is row-major like any other: config C2 with K and V
    in either order gives the same output fingerprint, equal to the oracle's."""
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config2_gqa_decode()
    ins = {i: uniform_fp(op["dims"], 9 + i) for i, op in enumerate(spec) if op["op"] == "input"}
    want = orc.eval_graph(spec, "fp", ins, threads=8)[3][0]
    for layout in (COL, ROW):
        sp = _with_layouts(spec, {1: layout, 2: layout})
        g, vals = rt.build_from_spec(sp)
        try:
            for i in ins:
                vals[i][0].write_fingerprint(ins[i])
            g.fingerprint(3)
            assert np.array_equal(vals[3][0].read_fingerprint(), want), layout
        finally:
            g.close()
