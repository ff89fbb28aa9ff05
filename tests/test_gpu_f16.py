"""GPU parity of the fp16 execution path against the fp16 golden of the CPU oracle.

Tolerance (the bar this backend is held to): |gpu - golden| <= 1e-3 + 1e-2 * |golden|
element-wise.  The golden is fp32 arithmetic with one fp16 rounding per materialised
tile and fp16 for-loop accumulators (semantics of the reference's generated
programs, src/kernel/triton_code_gen.cc:223-333)."""
import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu


KERNEL_INTERP, KERNEL_ATTENTION, KERNEL_GEMM, KERNEL_COMBINE = 2, 3, 4, 5
_last_kernels = []


@pytest.fixture(params=["fused", "interpreter"])
def path(request, abi):
    """Every customized op is checked on both fp16 routes: the fused kernel its shape
    selects (if any) and the generic LDS interpreter."""
    assert abi.mi355_set_option(1, 1 if request.param == "interpreter" else 0) == 0
    yield request.param
    assert abi.mi355_set_option(1, 0) == 0


@pytest.fixture(params=["ranges", "pieces", "interpreter"])
def gemm_path(request, abi):
    """The skinny-GEMM plans on each route: the fused kernel that cuts the for-loop into ranges
    (plus the launch that adds them), the one-launch kernel that cuts the output tile into
    pieces, and the generic LDS interpreter."""
    assert abi.mi355_set_option(1, 1 if request.param == "interpreter" else 0) == 0
    assert abi.mi355_set_option(7, {"ranges": 1, "pieces": 2, "interpreter": 0}[request.param]) == 0
    yield "fused" if request.param != "interpreter" else "interpreter"
    assert abi.mi355_set_option(7, 0) == 0
    assert abi.mi355_set_option(1, 0) == 0


def _graph_f16(rt, spec, inputs):
    import ctypes
    from attention_superoptimizer_amd import _native as N
    g, vals = rt.build_from_spec(spec)
    del _last_kernels[:]
    try:
        for i, op in enumerate(spec):
            if op["op"] == "input":
                vals[i][0].write_data(inputs[i])
            else:
                g.execute(i)
                if op["op"] == "customized":
                    info = N.Mi355LaunchInfo()
                    N.backend().mi355_last_launch(ctypes.byref(info))
                    _last_kernels.append(info.kernel_id)
        return [[t.read_data() for t in v] for v in vals]
    finally:
        g.close()


def _inputs(spec, stds, seed=0):
    return {i: normal_f16(op["dims"], stds.get(i, 1.0) if isinstance(stds, dict) else stds, seed + i)
            for i, op in enumerate(spec) if op["op"] == "input"}


def _check(rt, spec, ins, what, threads=8):
    got = _graph_f16(rt, spec, ins)
    want = orc.eval_graph(spec, "f16", ins, threads=threads)
    for i in range(len(spec)):
        if spec[i]["op"] == "input":
            continue
        for j, w in enumerate(want[i]):
            assert_f16_close(got[i][j], w, what=f"{what} op {i} ({spec[i]['op']}) out {j}")
    return got


def test_kernel_level_ops(rt):
    spec = [
        {"op": "input", "dims": [3, 70, 96]}, {"op": "input", "dims": [3, 96, 130]},
        {"op": "input", "dims": [3, 70, 1]},
        {"op": "matmul", "in": [[0, 0], [1, 0]]},
        {"op": "exp", "in": [[3, 0]]},
        {"op": "reduction", "in": [[4, 0]], "dim": 2, "size": 1},
        {"op": "div", "in": [[4, 0], [5, 0]]},
        {"op": "add", "in": [[6, 0], [2, 0]]},
        {"op": "mul", "in": [[7, 0], [7, 0]]},
        {"op": "silu", "in": [[8, 0]]},
        {"op": "reduction", "in": [[9, 0]], "dim": 2, "size": 65},
        {"op": "reduction", "in": [[9, 0]], "dim": 1, "size": 1},
    ]
    _check(rt, spec, _inputs(spec, 0.1), "kernel ops")


def _expect(path, fused_kernel):
    return fused_kernel if path == "fused" else KERNEL_INTERP


def test_config1_fused_matmul(rt, gemm_path):
    path = gemm_path
    from attention_superoptimizer_amd import workloads as W
    spec, ref = W.config1_fused_matmul()
    ins = _inputs(spec, W.INPUT_STD["C1_fused_matmul"], 10)
    got = _check(rt, spec, ins, "C1")
    assert _last_kernels == [_expect(path, KERNEL_GEMM)]
    # textbook special case: the op is a plain GEMM
    exact = ins[0].astype(np.float64) @ ins[1].astype(np.float64)
    assert_f16_close(got[2][0], exact, rtol=1e-2, atol=4e-3, what="C1 vs float64 GEMM")


def test_config2_gqa_decode(rt, path):
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config2_gqa_decode()
    ins = _inputs(spec, W.INPUT_STD["C2_gqa_decode"], 20)
    got = _check(rt, spec, ins, "C2")[3][0]
    assert _last_kernels == [KERNEL_ATTENTION if path == "fused" else KERNEL_INTERP]
    # independent statement: per (head, kv block of 256, tile of 64) softmax-without-max
    Q, K, V = (ins[i].astype(np.float64) for i in range(3))
    out = np.zeros((2, 256, 1024))
    for h in range(2):
        for blk in range(16):
            acc = np.zeros((256, 64))
            for it in range(4):
                s = blk * 256 + it * 64
                e = np.exp(Q[h] @ K[h][:, s:s + 64])
                acc += (e / e.sum(axis=1, keepdims=True)) @ V[h][s:s + 64]
            out[h][:, blk * 64:(blk + 1) * 64] = acc
    assert_f16_close(got, out, rtol=1e-2, atol=2e-3, what="C2 vs float64 statement")


def test_config3_mha_prefill_small(rt, path):
    from attention_superoptimizer_amd import workloads as W
    spec, ref = W.config3_mha_prefill(heads=2, seq=512, hd=128, q_split=4, kv_split=2, F=4)
    ins = _inputs(spec, 128 ** -0.5, 30)
    got = _check(rt, spec, ins, "C3 small")[-1][0]
    assert _last_kernels == ([KERNEL_ATTENTION, KERNEL_COMBINE] if path == "fused"
                             else [KERNEL_INTERP, KERNEL_INTERP])
    # textbook special case: numerator / denominator = softmax(Q K^T) V
    Q, K, V = (ins[i].astype(np.float64) for i in range(3))
    s = Q @ K
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    att = (p / p.sum(axis=-1, keepdims=True)) @ V
    assert_f16_close(got, att, rtol=1e-2, atol=2e-3, what="C3 vs softmax attention")


def test_config3_single_kv_block(rt, path):
    """the benchmark's tiling shape: one block walks the whole key range (kv_split 1),
    so op2 folds a single partial result"""
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config3_mha_prefill(heads=2, seq=512, hd=128, q_split=4, kv_split=1, F=8)
    _check(rt, spec, _inputs(spec, 128 ** -0.5, 31), "C3 single kv block")
    assert _last_kernels == ([KERNEL_ATTENTION, KERNEL_COMBINE] if path == "fused"
                             else [KERNEL_INTERP, KERNEL_INTERP])


def test_config4_lora(rt, gemm_path):
    path = gemm_path
    from attention_superoptimizer_amd import workloads as W
    spec, ref = W.config4_lora()
    ins = _inputs(spec, W.INPUT_STD["C4_lora"], 40)
    got = _check(rt, spec, ins, "C4")[4][0]
    assert _last_kernels == [_expect(path, KERNEL_GEMM)]
    # independent statement: X.W + (X.A).B in float64
    X, Wm, A, B = (ins[i].astype(np.float64) for i in range(4))
    assert_f16_close(got, X @ Wm + (X @ A) @ B, rtol=1e-2, atol=4e-3, what="C4 vs float64")


def test_config5_gated_mlp_small(rt, gemm_path):
    path = gemm_path
    from attention_superoptimizer_amd import workloads as W
    spec, ref = W.config5_gated_mlp(m=8, d=1024, h=3584, grid1=56, F1=4, grid2=16, F2=14)
    ins = _inputs(spec, W.INPUT_STD["C5a_gated_mlp"], 50)
    got = _check(rt, spec, ins, "C5a small")[-1][0]
    assert _last_kernels == [_expect(path, KERNEL_GEMM)] * 2
    X, W1, W3, W2 = (ins[i].astype(np.float64) for i in range(4))
    gate = X @ W1
    exact = ((gate / (1 + np.exp(-gate))) * (X @ W3)) @ W2
    assert_f16_close(got, exact, rtol=2e-2, atol=4e-3, what="C5a vs float64")


def test_gemm_family_shapes(rt, gemm_path):
    """for-loop split over workgroups (few blocks) and unsplit (many blocks), 16/32/64-row
    tiles, exp prologue"""
    path = gemm_path
    from attention_superoptimizer_amd import workloads as W
    cases = {
        "unsplit": W.tiled_matmul(1024, 4096, 128, (16, 64, 1), 2, (0, -1, -1), (-1, 1, -1), (0, 1, -1)),
        "split": W.tiled_matmul(32, 512, 2048, (8, 1, 1), 16, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),
        "rows16": W.tiled_matmul(16, 256, 1024, (4, 1, 1), 4, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),
        "uneven": W.tiled_matmul(64, 128, 448, (2, 1, 1), 7, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),
    }
    for name, (spec, ref) in cases.items():
        ins = _inputs(spec, 0.1, 80)
        _check(rt, spec, ins, name)
        assert _last_kernels == [_expect(path, KERNEL_GEMM)], name
    spec = [
        {"op": "input", "dims": [16, 1024]}, {"op": "input", "dims": [1024, 256]},
        {"op": "customized", "in": [[0, 0], [1, 0]], "plan": {
            "grid_dim": [4, 1, 1], "forloop_range": 8, "input_map": [[-1, -1, -1], [1, -1, -1]],
            "forloop_dim": [1, 0], "output_map": [1, -1, -1],
            "ops": [["tb_exp_op", [[0, 0]]], ["tb_matmul_op", [[2, 0], [1, 0]]]]}},
    ]
    _check(rt, spec, _inputs(spec, 0.05, 81), "exp prologue")
    assert _last_kernels == [_expect(path, KERNEL_GEMM)]


def test_reference_examples_f16(rt, path):
    """The reference's example plans, fp16, small-valued inputs so exp stays finite."""
    from attention_superoptimizer_amd import workloads as W
    for name in ["group_query_attn_inc_decode", "group_query_attn_spec_decode",
                 "multi_head_attn_inc_decode", "multi_head_attn_prefill",
                 "multi_query_attn_inc_decode", "dnn", "lora", "mlp"]:
        spec, ref = W.REFERENCE_EXAMPLES[name]
        ins = _inputs(spec, 0.05, 60)
        _check(rt, spec, ins, name)
        # every attention plan takes the fused kernel, the 8-row decode tile included (padded
        # with zero rows)
        if path == "fused" and name in ("group_query_attn_inc_decode", "group_query_attn_spec_decode",
                                        "multi_head_attn_inc_decode", "multi_head_attn_prefill",
                                        "multi_query_attn_inc_decode", "dnn"):
            assert _last_kernels[0] == KERNEL_ATTENTION, (name, _last_kernels)


@pytest.mark.parametrize("rows,F,kv_blocks,lanes", [
    (8, 4, 16, 0),     # the reference's plan: one iteration per wavefront
    (8, 8, 4, 0),      # two iterations per wavefront, two tile pairs in flight
    (8, 16, 2, 0),     # four
    (16, 16, 2, 0),    # a full row group
    (8, 19, 1, 0),     # uneven: wavefronts with five and four iterations
    (8, 30, 1, 0),     # eight lanes, up to four iterations each
    (8, 16, 2, 4),     # four lanes with two tile pairs each, by request
    (8, 30, 1, 4),     # ... eight iterations per lane
    (8, 40, 1, 0),     # too long for the direct variant: register-transposed staging
    (16, 3, 2, 0),     # fewer iterations than lanes
])
def test_decode_row_groups_on_the_direct_staging_kernel(rt, abi, rows, F, kv_blocks, lanes):
    """8- and 16-row query tiles (incremental decode) against a for-loop of any length: the
    looped direct-staging kernel, both forms (two outputs + combine; single op with div),
    against the golden.  Also on the register-transposed variant (attention mode 3)."""
    from attention_superoptimizer_amd import workloads as W
    seq = 64 * F * kv_blocks
    spec, _ = W.gqa_inc_decode(groups=3, rows=rows, seq=seq, kv_blocks=kv_blocks, F=F)
    single, _ = W.config2_gqa_decode(groups=3, rows=rows, seq=seq, kv_blocks=kv_blocks, F=F)
    assert abi.mi355_set_option(6, lanes) == 0
    try:
        for what, sp in (("two-stage", spec), ("single op", single)):
            ins = _inputs(sp, 0.125, 200 + F)
            _check(rt, sp, ins, f"decode {what} rows {rows} F {F}")
            assert _last_kernels[0] == KERNEL_ATTENTION, (what, _last_kernels)
            info = N_launch_info()
        assert abi.mi355_set_option(2, 3) == 0
        try:
            ins = _inputs(spec, 0.125, 300 + F)
            _check(rt, spec, ins, f"decode rows {rows} F {F}, register-transposed variant")
            assert _last_kernels[0] == KERNEL_ATTENTION
        finally:
            assert abi.mi355_set_option(2, 0) == 0
    finally:
        assert abi.mi355_set_option(6, 0) == 0


@pytest.mark.parametrize("F, units_per_lane", [(8, 2), (16, 4), (32, 8)])
def test_decode_grid_large_enough_for_two_workgroups_per_cu(rt, abi, F, units_per_lane):
    """512 blocks (64 groups x 8 key blocks) of 8 query rows: the direct-staging kernel runs them
    as workgroups of four single-buffered lanes (73,728 B of LDS: two per compute unit), each
    lane streaming F / 4 tile pairs, against the golden."""
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.gqa_inc_decode(groups=64, rows=8, seq=64 * F * 8, kv_blocks=8, F=F)
    ins = _inputs(spec, 0.125, 700 + F)
    ins[2] = np.abs(ins[2])  # (sums that grow steadily: an accumulator ulp stays inside the tolerance)
    _check(rt, spec, ins, f"decode 512 blocks, F {F}", threads=16)
    assert _last_kernels[0] == KERNEL_ATTENTION, _last_kernels


@pytest.mark.parametrize("rows,nk,F,kv_blocks,groups", [
    (64, 32, 8, 2, 3),      # two iterations per 64-key strip, a wavefront per strip
    (64, 32, 16, 1, 3),     # ... eight strips
    (16, 32, 32, 1, 3),     # a lone row group: eight lanes, two strips each
    (64, 16, 16, 2, 3),     # four iterations per strip (16-deep matrix instruction)
    (16, 16, 32, 1, 3),
    (8, 16, 8, 2, 3),       # 8-row tile
    (64, 32, 8, 16, 8),     # two row groups per wavefront (enough blocks to fill the chip)
    (64, 16, 16, 16, 8),
    (16, 128, 4, 2, 3),     # two strips per iteration
    (64, 128, 4, 2, 3),
    (16, 256, 16, 1, 3),    # four strips per iteration, two iterations per lane
    (16, 256, 5, 1, 3),
    (32, 256, 2, 2, 3),
])
def test_attention_key_tiles_of_other_widths(rt, abi, rows, nk, F, kv_blocks, groups):
    """Key tiles of 16 / 32 / 128 / 256 on the direct-staging kernel's 64-key strips, against
    the golden: the two-output form always, the form with the division inside where the
    kernel takes it (tiles up to 64 keys)."""
    from attention_superoptimizer_amd import workloads as W
    seq = nk * F * kv_blocks
    two_stage, _ = W.gqa_inc_decode(groups=groups, rows=rows, seq=seq, kv_blocks=kv_blocks, F=F)
    single, _ = W.config2_gqa_decode(groups=groups, rows=rows, seq=seq, kv_blocks=kv_blocks, F=F)
    cases = [("two-stage", two_stage)] + ([("single op", single)] if nk <= 64 else [])
    for what, spec in cases:
        # (small values: the un-normalised numerators stay below 1, where an fp16 ulp of the
        # accumulator is inside the absolute tolerance)
        ins = _inputs(spec, 0.05, 400 + nk + F)
        _check(rt, spec, ins, f"{what}: rows {rows}, key tile {nk}, for-loop {F}")
        assert _last_kernels[0] == KERNEL_ATTENTION, (what, _last_kernels)


def N_launch_info():
    import ctypes
    from attention_superoptimizer_amd import _native as N
    info = N.Mi355LaunchInfo()
    N.backend().mi355_last_launch(ctypes.byref(info))
    return info


def test_gqa_fixture_graphs_f16(rt, path):
    """A sample of the 69 recorded GQA graphs in fp16 (K tiles of 256 keys, Q tiles of 16 rows)."""
    from helpers import load_gqa_fixture
    fx = load_gqa_fixture()
    for gi in (0, 17, 25, 29, 44, 68):
        spec = fx["generated_graphs"][gi]
        ins = _inputs(spec, 0.05, 70)
        _check(rt, spec, ins, f"fixture graph {gi}")


def test_value_columns_cut_into_pieces_run_as_one_block(rt, abi):
    """The recorded programs whose grid cuts the 64 value columns into 16 pieces of 4 (every
    piece's block repeats the same scores and stores its own copy of the row sums): the fused
    route runs each (batch, query tile) as one block with the whole value tile -- 32
    workgroups (2 x 4 query tiles x 4 row groups) instead of 128 blocks -- and matches the golden
    on both outputs, every copy of the row sums included."""
    from helpers import load_gqa_fixture
    fx = load_gqa_fixture()
    for gi in (60, 65):
        spec = fx["generated_graphs"][gi]
        plan = spec[3]["plan"]
        assert plan["grid_dim"] == [2, 16, 4] and spec[3]["out_dims"] == [[2, 256, 16], [2, 256, 64]]
        ins = _inputs(spec, 0.05, 170 + gi)
        # (values of one sign: the 4096-key sums then grow steadily, and an fp16 ulp of the
        # accumulator stays inside the relative tolerance of the final value)
        ins[2] = np.abs(ins[2])
        _check(rt, spec, ins, f"fixture graph {gi}", threads=16)
        assert _last_kernels[0] == KERNEL_ATTENTION, _last_kernels


@pytest.mark.parametrize("gi, what", [
    (1, "div of a [16,64] tile by its [16,1] row sums"),
    (7, "div of [256,4] column pieces by whole-tile row sums"),
    (13, "div, tiles cut along the last dim of both inputs, stored along rows"),
    (22, "partial denominators folded, div, then the partial numerators folded"),
    (23, "both folds first, then div"),
    (28, "div inside a for-loop of 16, the saver accumulates"),
    (60, "div of [256,4] column pieces by their own copy of the row sums"),
])
def test_recorded_second_operators_take_the_fused_fold(rt, abi, gi, what):
    """Every shape of second operator in the recorded programs -- the division before, after or
    without the folds, inside a for-loop, on 4-column pieces -- runs on the fused fold kernel
    and matches the golden."""
    from helpers import load_gqa_fixture
    spec = load_gqa_fixture()["generated_graphs"][gi]
    ins = _inputs(spec, 0.05, 270 + gi)
    ins[2] = np.abs(ins[2])  # (steadily growing sums in the first operator, see above)
    _check(rt, spec, ins, f"fixture graph {gi}: {what}", threads=16)
    assert _last_kernels == [KERNEL_ATTENTION, KERNEL_COMBINE], _last_kernels


def test_column_pieces_with_the_division_inside(rt, abi):
    """A single-op attention plan (division inside the block) whose grid cuts the value columns
    into 4 pieces of 16: merged into one block per query tile on the fused route, same result as
    the interpreter's block-by-block evaluation and the golden."""
    spec = [
        {"op": "input", "dims": [2, 64, 64]}, {"op": "input", "dims": [2, 64, 256]},
        {"op": "input", "dims": [2, 256, 64]},
        {"op": "customized", "in": [[0, 0], [1, 0], [2, 0]], "plan": {
            "grid_dim": [2, 4, 2], "forloop_range": 4,
            "input_map": [[0, -1, 1], [0, -1, -1], [0, 2, -1]], "forloop_dim": [-1, 2, 1],
            "output_map": [0, 2, 1],
            "ops": [["tb_matmul_op", [[0, 0], [1, 0]]], ["tb_exp_op", [[3, 0]]],
                    ["tb_reduction_2_op", [[4, 0]]], ["tb_div_op", [[4, 0], [5, 0]]],
                    ["tb_matmul_op", [[6, 0], [2, 0]]]]}},
    ]
    for force in (0, 1):
        assert abi.mi355_set_option(1, force) == 0
        try:
            _check(rt, spec, _inputs(spec, 0.1, 610), f"column pieces, division inside, forced={force}")
            assert _last_kernels == [KERNEL_INTERP if force else KERNEL_ATTENTION], _last_kernels
        finally:
            assert abi.mi355_set_option(1, 0) == 0


def test_streaming_kernels_are_deterministic(rt, abi):
    """The kernels whose wavefronts stream several tiles through ONE LDS buffer each (a strip is
    overwritten by direct-to-LDS transfers as soon as its operands have been read), and the other
    fused kernels: 40 launches
    of the same operator give the same bits.  (A transfer issued while operand reads of the
    buffer were still outstanding once made whole 16-column blocks differ from run to run.)"""
    from helpers import load_gqa_fixture
    from attention_superoptimizer_amd import workloads as W
    cases = [("recorded program 0, 256-key tiles as four strips, two iterations per lane",
              load_gqa_fixture()["generated_graphs"][0], 3, 0),
             ("direct-staging decode, four tile pairs per lane",
              W.gqa_inc_decode(groups=64, rows=8, seq=64 * 16 * 8, kv_blocks=8, F=16)[0], 3, 0),
             ("one-launch GEMM, five iterations per lane",
              W.tiled_matmul(64, 128, 10240, (2, 1, 1), 40, (-1, -1, -1), (1, -1, -1), (1, -1, -1))[0], 2, 2)]
    fx = load_gqa_fixture()["generated_graphs"]
    cases += [("recorded program 22 (32-key tiles, two iterations per strip)", fx[22], 3, 0),
              ("recorded program 41 (16-key tiles, four iterations per strip)", fx[41], 3, 0),
              ("recorded program 60 (value columns in pieces)", fx[60], 3, 0),
              ("C2, the headline plan", W.config2_gqa_decode()[0], 3, 0),
              ("the reference's dnn example (8-row tiles, 8 iterations)", W.REFERENCE_EXAMPLES["dnn"][0], 3, 0),
              ("C3 at reduced size, throughput kernel",
               W.config3_mha_prefill(heads=4, seq=1024, hd=128, q_split=8, kv_split=1, F=16)[0], 3, 0),
              ("LoRA, range-splitting kernel", W.config4_lora(m=16, d=1024, r=16, grid=16, F=4)[0], 4, 1),
              ("LoRA, one-launch kernel", W.config4_lora(m=16, d=1024, r=16, grid=16, F=4)[0], 4, 2)]
    for what, spec, op, gemm_mode in cases:
        assert abi.mi355_set_option(7, gemm_mode) == 0
        g, vals = rt.build_from_spec(spec)
        try:
            for i, o in enumerate(spec):
                if o["op"] == "input":
                    vals[i][0].write_data(normal_f16(o["dims"], 0.05, 800 + i))
            first = None
            for run in range(40):
                g.execute(op)
                outs = [t.read_data().view(np.uint16).copy() for t in vals[op]]
                if first is None:
                    first = outs
                else:
                    for a, b in zip(first, outs):
                        assert np.array_equal(a, b), f"{what}: launch {run} differs in {int((a != b).sum())} elements"
        finally:
            g.close()
            assert abi.mi355_set_option(7, 0) == 0


def test_profile_loops_leave_the_results_of_a_plain_run(rt, abi):
    """mi355_customized_profile captures what one call launches and repeats it (kernel by
    kernel; for 512 launches and more as chains of 256 kernel nodes, one graph launch each).
    Whatever the loop's length, the outputs afterwards are the bits a plain run leaves --
    checked twice per plan, with plain runs and cleared outputs between the loops, on a
    one-kernel plan, a two-kernel plan (range kernel + fold) and the generic interpreter."""
    import ctypes
    from attention_superoptimizer_amd import workloads as W
    cases = [("C2, direct-staging attention", W.config2_gqa_decode()[0], 3, 0, 0),
             ("LoRA, range kernel and its fold", W.config4_lora(m=16, d=1024, r=16, grid=16, F=4)[0], 4, 1, 0),
             ("C1 on the interpreter", W.config1_fused_matmul()[0], 2, 0, 1)]
    for what, spec, op, gemm_mode, interpreter in cases:
        assert abi.mi355_set_option(7, gemm_mode) == 0
        assert abi.mi355_set_option(1, interpreter) == 0
        g, vals = rt.build_from_spec(spec)
        try:
            for i, o in enumerate(spec):
                if o["op"] == "input":
                    vals[i][0].write_data(normal_f16(o["dims"], 0.05, 900 + i))
            g.execute(op)
            plain = [t.read_data().view(np.uint16).copy() for t in vals[op]]
            pl = g.lowered(op, fingerprint=False)
            i_p = (ctypes.c_void_p * 4)(*[vals[a][b].device_ptr(False) for a, b in spec[op]["in"]])
            o_p = (ctypes.c_void_p * 4)(*[t.device_ptr(False) for t in vals[op]])
            ms = ctypes.c_float()
            for warmup, iters in ((0, 3), (256, 1024), (5, 700), (0, 512)):
                for t in vals[op]:
                    t.write_data(np.full(t.dims, np.nan, np.float16))
                assert abi.mi355_customized_profile(ctypes.byref(pl), i_p, o_p, 0, warmup, iters,
                                                    ctypes.byref(ms)) == 0
                assert ms.value > 0
                for a, t in zip(plain, vals[op]):
                    b = t.read_data().view(np.uint16)
                    assert np.array_equal(a, b), f"{what}: after {warmup} + {iters} launches {int((a != b).sum())} elements differ"
                g.execute(op)  # plain work between the loops
                for a, t in zip(plain, vals[op]):
                    assert np.array_equal(a, t.read_data().view(np.uint16)), what
        finally:
            g.close()
            assert abi.mi355_set_option(7, 0) == 0
            assert abi.mi355_set_option(1, 0) == 0


def test_attention_throughput_variant(rt, abi):
    """the pipelined 32-rows-per-wavefront variant, forced on small problems: both forms,
    both head sizes"""
    from attention_superoptimizer_amd import workloads as W
    assert abi.mi355_set_option(2, 2) == 0
    try:
        spec, _ = W.config2_gqa_decode()
        _check(rt, spec, _inputs(spec, W.INPUT_STD["C2_gqa_decode"], 90), "C2 throughput variant")
        assert _last_kernels == [KERNEL_ATTENTION]
        spec, _ = W.config3_mha_prefill(heads=2, seq=512, hd=128, q_split=4, kv_split=2, F=4)
        _check(rt, spec, _inputs(spec, 128 ** -0.5, 91), "C3 small throughput variant")
        assert _last_kernels[0] == KERNEL_ATTENTION
        spec, _ = W.REFERENCE_EXAMPLES["multi_head_attn_prefill"]   # Q tile [64, 64], form B
        _check(rt, spec, _inputs(spec, 0.05, 92), "mha prefill throughput variant")
        assert _last_kernels[0] == KERNEL_ATTENTION
        # 256-row query tiles at head size 64 run as wavefronts of 64 rows (C2 above: the form
        # with the division inside; here the two-output form)
        spec, _ = W.gqa_inc_decode(groups=2, rows=256, seq=1024, kv_blocks=2, F=8)
        _check(rt, spec, _inputs(spec, 0.05, 93), "256-row tiles, two outputs, throughput variant")
        assert _last_kernels[0] == KERNEL_ATTENTION and N_launch_info is not None
    finally:
        assert abi.mi355_set_option(2, 0) == 0


def test_attention_latency_variants_agree(rt, abi):
    """The two latency variants of the fused attention kernel (tiles streamed straight into
    LDS and gathered with transposing reads / tiles transposed in registers while staged)
    make the same roundings in the same order: identical fp16 outputs, each within the
    tolerance of the golden.  C2 and the reference's decode examples with one iteration per
    wavefront, both forms (with and without the division)."""
    from attention_superoptimizer_amd import workloads as W
    cases = [(W.config2_gqa_decode()[0], W.INPUT_STD["C2_gqa_decode"], "C2"),
             (W.REFERENCE_EXAMPLES["dnn"][0], 0.05, "dnn"),                       # 8 iterations, 8 wavefronts
             (W.REFERENCE_EXAMPLES["multi_head_attn_inc_decode"][0], 0.05, "mha inc decode")]
    for spec, stds, what in cases:
        ins = _inputs(spec, stds, 95)
        outs = {}
        # (attention mode, direct-lanes knob): streamed with two row groups per wavefront where
        # the size allows, streamed with one, register-transposed
        for mode, lanes in ((0, 0), (0, 1), (3, 0)):
            assert abi.mi355_set_option(2, mode) == 0 and abi.mi355_set_option(6, lanes) == 0
            try:
                got = _check(rt, spec, ins, f"{what} mode {mode} lanes {lanes}")
                assert _last_kernels[0] == KERNEL_ATTENTION
                outs[mode, lanes] = [got[i] for i in range(len(spec)) if spec[i]["op"] == "customized"]
            finally:
                assert abi.mi355_set_option(2, 0) == 0 and abi.mi355_set_option(6, 0) == 0
        for other in ((0, 1), (3, 0)):
            for a, b in zip(outs[0, 0], outs[other]):
                for x, y in zip(a, b):
                    assert np.array_equal(x, y), (what, other)


def test_one_launch_gemm_shapes(rt, abi):
    """The one-launch kernel on the shapes its lanes and pieces must cover: 8 / 16 / 48 / 64
    activation rows, k tiles of 64 / 128 / 256, for-loops of 1, 3 (fewer iterations than lanes),
    16 and 40 (several per lane), a block count that is no multiple of 8, a 3-D grid, LoRA with
    a small k tile, two weights, silu * mul."""
    from attention_superoptimizer_amd import workloads as W
    assert abi.mi355_set_option(7, 2) == 0
    try:
        cases = {
            "rows8 k64 F3": W.tiled_matmul(8, 192, 192, (3, 1, 1), 3, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),
            "rows48 k128 F1": W.tiled_matmul(48, 320, 128, (5, 1, 1), 1, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),
            "rows64 k256 F40": W.tiled_matmul(64, 128, 10240, (2, 1, 1), 40, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),
            "grid 2x3": W.tiled_matmul(32, 192, 256, (2, 3, 1), 4, (0, -1, -1), (-1, 1, -1), (0, 1, -1)),
            "lora k64": W.config4_lora(m=16, d=256, r=16, grid=4, F=4),
            "gated mlp": W.config5_gated_mlp(m=8, d=512, h=640, grid1=10, F1=4, grid2=8, F2=5),
        }
        for name, (spec, _) in cases.items():
            ins = _inputs(spec, 0.1, 90)
            _check(rt, spec, ins, name)
            assert all(k == KERNEL_GEMM for k in _last_kernels), (name, _last_kernels)
    finally:
        assert abi.mi355_set_option(7, 0) == 0


def test_gemm_kernels_agree_to_the_last_bit(rt, abi):
    """Full-size C1, C4 and C5a on the two fused GEMM kernels: both round every iteration's
    product tile to fp16 and add the tiles in iteration order, so they agree bit for bit."""
    from attention_superoptimizer_amd import workloads as W
    for name in ("C1_fused_matmul", "C4_lora", "C5a_gated_mlp"):
        spec, _ = W.BASELINE_CONFIGS[name]()
        ins = _inputs(spec, W.INPUT_STD[name], 0xBEEF00)
        outs = {}
        for mode in (1, 2):
            assert abi.mi355_set_option(7, mode) == 0
            try:
                outs[mode] = _graph_f16(rt, spec, ins)
                assert all(k == KERNEL_GEMM for k in _last_kernels), (name, mode, _last_kernels)
                info = N_launch_info()
                print(name, "mode", mode, "workgroups", info.workgroups, "threads", info.threads,
                      "lds", info.lds_bytes, "split", info.row_split, flush=True)
            finally:
                assert abi.mi355_set_option(7, 0) == 0
        for i, op in enumerate(spec):
            if op["op"] == "customized":
                for a, b in zip(outs[1][i], outs[2][i]):
                    assert np.array_equal(a, b), (name, i)


def test_full_size_configs_routes_agree(rt, abi):
    """Full benchmark sizes, where the scalar golden is too slow to run: the fused kernel
    and the generic LDS interpreter (each checked against the golden at reduced size) must
    agree within the tolerance, and C3 must be softmax attention (float64 on the host, four
    of the 32 heads)."""
    from attention_superoptimizer_amd import workloads as W
    for name in ("C1_fused_matmul", "C3_mha_prefill", "C4_lora", "C5a_gated_mlp"):
        spec, _ = W.BASELINE_CONFIGS[name]()
        ins = _inputs(spec, W.INPUT_STD[name], 0xC0FFEE00)
        outs = {}
        for route, force in (("fused", 0), ("interpreter", 1)):
            assert abi.mi355_set_option(1, force) == 0
            try:
                outs[route] = _graph_f16(rt, spec, ins)[-1][0]
                kernels = list(_last_kernels)
            finally:
                assert abi.mi355_set_option(1, 0) == 0
            if route == "fused":
                assert all(k != KERNEL_INTERP for k in kernels), (name, kernels)
            else:
                assert all(k == KERNEL_INTERP for k in kernels), (name, kernels)
        assert_f16_close(outs["fused"], outs["interpreter"], what=f"{name} fused vs interpreter")
        if name == "C3_mha_prefill":
            Q, K, V = (ins[i][:4].astype(np.float64) for i in range(3))
            s = Q @ K
            p = np.exp(s - s.max(axis=-1, keepdims=True))
            att = (p / p.sum(axis=-1, keepdims=True)) @ V
            assert_f16_close(outs["fused"][:4], att, rtol=1e-2, atol=2e-3, what="C3 vs softmax attention")


# ---- kernel-level fp16 operators (the un-fused graphs every example of the reference times first) --
def _abi_matmul(rt, abi, batch, m, n, k, a_cm, b_cm, seed):
    """C = A . B through mi355_f16_matmul_layout on tensors of the arena; returns (A, B, C) as
    logical arrays."""
    from attention_superoptimizer_amd import graph as G
    g = G.KNGraph()
    try:
        lay = {0: "DmemRowMajor", 1: "DmemColumnMajor"}
        A = g.new_input((batch, m, k), layout=lay[a_cm])
        B = g.new_input((batch, k, n), layout=lay[b_cm])
        C = g.new_input((batch, m, n))
        a, b = normal_f16([batch, m, k], 0.1, seed), normal_f16([batch, k, n], 0.1, seed + 1)
        A.write_data(a)
        B.write_data(b)
        C.write_data(np.full((batch, m, n), np.nan, np.float16))
        import ctypes
        assert abi.mi355_f16_matmul_layout(ctypes.c_void_p(A.device_ptr(False)), ctypes.c_void_p(B.device_ptr(False)),
                                           ctypes.c_void_p(C.device_ptr(False)), batch, m, n, k, a_cm, b_cm) == 0
        assert abi.mi355_sync() == 0
        return a, b, C.read_data()
    finally:
        g.close()


@pytest.mark.parametrize("batch,m,n,k", [
    (3, 70, 130, 96),      # streaming kernel, 128 x 128 tiles, ragged edges
    (1, 33, 47, 50),       # k not a multiple of 8: the general-purpose kernel
    (2, 257, 300, 64),     # n not a multiple of 8: masked scalar stores at the edge
    (1, 16, 4096, 4096),   # the skinny product of the un-fused LoRA graph: k cut into ranges
    (1, 16, 16, 4096),     # its rank-16 factor: one tile, sixteen ranges
    (2, 256, 64, 4096),    # P . V of the un-fused decode graph: four tiles, long k
    (1, 3600, 3700, 256),  # 256 x 256 tiles with ragged edges on both sides
])
def test_kernel_level_matmul_shapes_and_layouts(rt, abi, batch, m, n, k):
    """mi355_f16_matmul_layout against fp32 numpy rounded once, every storage order of A and B."""
    for a_cm, b_cm in ((0, 1), (0, 0), (1, 1), (1, 0)):
        a, b, got = _abi_matmul(rt, abi, batch, m, n, k, a_cm, b_cm, 31)
        want = orc.f16_matmul(a, b)
        assert_f16_close(got, want, what=f"[{batch},{m},{k}] . [{batch},{k},{n}], A cm {a_cm}, B cm {b_cm}")


def test_kernel_level_matmul_4096_cubed_by_samples_and_checksums(rt, abi):
    """4096^3 (the size the streaming kernel is measured on): 4096 sampled elements against
    float64 dot products at the fp16 tolerance, and every row / column sum of C against
    A . (B . 1) and (1 . A) . B (a dropped or doubled k step, a misplaced tile or a wrong edge
    shows in a sum even where no sample falls)."""
    n = 4096
    a, b, got = _abi_matmul(rt, abi, 1, n, n, n, 0, 1, 77)
    a64, b64, c64 = a[0].astype(np.float64), b[0].astype(np.float64), got[0].astype(np.float64)
    rng = np.random.default_rng(5)
    ii, jj = rng.integers(0, n, 4096), rng.integers(0, n, 4096)
    want = np.einsum("sk,ks->s", a64[ii], b64[:, jj])
    assert_f16_close(got[0][ii, jj], want.astype(np.float16), what="4096^3 samples")
    # sums of 4096 outputs each rounded to fp16 (|c| ~ 0.64, ulp ~ 5e-4): allow 4096 * 3e-4
    assert np.abs(c64.sum(1) - a64 @ b64.sum(1)).max() < 1.3
    assert np.abs(c64.sum(0) - a64.sum(0) @ b64).max() < 1.3


OPT_F16_MATMUL_ROUTE = 8


@pytest.fixture
def vendor_route(abi):
    import ctypes
    try:
        ctypes.CDLL("librocblas.so.5")
    except OSError:
        try:
            ctypes.CDLL("/opt/rocm/lib/librocblas.so.5")
        except OSError:
            pytest.skip("rocBLAS is not installed: the vendor route of the fp16 matmul cannot run")
    assert abi.mi355_set_option(OPT_F16_MATMUL_ROUTE, 1) == 0
    yield
    assert abi.mi355_set_option(OPT_F16_MATMUL_ROUTE, 0) == 0


@pytest.mark.parametrize("batch,m,n,k", [
    (3, 70, 130, 96),
    (1, 33, 47, 50),
    (1, 16, 4096, 4096),
    (2, 256, 64, 4096),
    (1, 1024, 1024, 1024),
])
def test_kernel_level_matmul_on_the_vendor_library(rt, abi, vendor_route, batch, m, n, k):
    """The second route of mi355_f16_matmul_layout (the vendor's BLAS, opened at run time) in
    every storage order of A and B: the operand order, transposes and leading dimensions it
    hands to a column-major library are what a wrong storage order would break."""
    for a_cm, b_cm in ((0, 1), (0, 0), (1, 1), (1, 0)):
        a, b, got = _abi_matmul(rt, abi, batch, m, n, k, a_cm, b_cm, 41)
        want = orc.f16_matmul(a, b)
        assert_f16_close(got, want, what=f"vendor [{batch},{m},{k}] . [{batch},{k},{n}], A cm {a_cm}, B cm {b_cm}")


def test_the_vendor_route_runs_the_matmul_operators_of_a_graph(rt, abi, vendor_route):
    """KNMatmulOp::run reaches the same entry point: an un-fused attention graph (Q . K^T with K
    column-major, exp, row sums, division, P . V) on the vendor route against the oracle."""
    spec = [
        {"op": "input", "dims": [2, 256, 64]},
        {"op": "input", "dims": [2, 64, 512], "layout": "DmemColumnMajor"},
        {"op": "input", "dims": [2, 512, 64]},
        {"op": "matmul", "in": [[0, 0], [1, 0]]},
        {"op": "exp", "in": [[3, 0]]},
        {"op": "reduction", "in": [[4, 0]], "dim": 2, "size": 1},
        {"op": "div", "in": [[4, 0], [5, 0]]},
        {"op": "matmul", "in": [[6, 0], [2, 0]]},
    ]
    _check(rt, spec, _inputs(spec, {0: 0.1, 1: 0.1, 2: 1.0}), "vendor route, un-fused attention")


def test_kernel_level_elementwise_and_reductions_large_and_ragged(rt):
    """The vector paths (16 bytes per lane) and their scalar tails: large tensors, row lengths
    that are not multiples of 8, one value per row as the second operand, sums along rows and
    columns."""
    for dims in ([4, 1000, 1024], [3, 70, 130], [2, 513, 1001]):
        b, r, c = dims
        spec = [
            {"op": "input", "dims": dims}, {"op": "input", "dims": dims}, {"op": "input", "dims": [b, r, 1]},
            {"op": "exp", "in": [[0, 0]]},
            {"op": "silu", "in": [[1, 0]]},
            {"op": "add", "in": [[3, 0], [4, 0]]},
            {"op": "reduction", "in": [[3, 0]], "dim": 2, "size": 1},
            {"op": "div", "in": [[3, 0], [6, 0]]},
            {"op": "mul", "in": [[7, 0], [2, 0]]},
            {"op": "reduction", "in": [[5, 0]], "dim": 1, "size": 1},
            {"op": "reduction", "in": [[0, 0]], "dim": 0, "size": 1},
        ]
        _check(rt, spec, _inputs(spec, 0.5, seed=11), f"kernel ops {dims}")
