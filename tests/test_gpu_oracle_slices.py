"""GPU parity where the earlier tests had a gap: the thread-block operators the reference
never defines (add, mul, silu), an in-place operator on a loop-invariant tile, and the
benchmark configurations at FULL size against the CPU oracle.

Thread blocks of a customized op share nothing (customized_kernel.cu:307-603), so the
scalar oracle run on a subset of the blocks reproduces exactly those blocks' output tiles:
that is how C3 (2 of 32 heads, every block of both operators) is affordable at full size.
C5a is small enough for the oracle to run whole.

Bars: fingerprints bit-exact; fp16 |gpu - golden| <= 1e-3 + 1e-2 |golden|."""
import ctypes

import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16, uniform_fp
from oracle import evaluate as orc
from test_oracle import tb_add_mul_case, tb_add_mul_exact

pytestmark = pytest.mark.gpu

ROUTES_FP = {"auto": (0, 0), "vector-dot": (0, 1), "interpreter": (1, 0), "interpreter, vector-dot": (1, 1)}


def _launch_kernel_id():
    from attention_superoptimizer_amd import _native as N
    info = N.Mi355LaunchInfo()
    N.backend().mi355_last_launch(ctypes.byref(info))
    return info.kernel_id


def _run(rt, spec, ins, f16):
    """Every operator of `spec` on the GPU through the host API; returns (per-op outputs,
    kernel ids of the customized ops)."""
    g, vals = rt.build_from_spec(spec)
    kernels = []
    try:
        for i, op in enumerate(spec):
            if op["op"] == "input":
                (vals[i][0].write_data if f16 else vals[i][0].write_fingerprint)(ins[i])
            else:
                print(f"  gpu op {i} ({op['op']}) {'f16' if f16 else 'fp'}", flush=True)
                (g.execute if f16 else g.fingerprint)(i)
                if op["op"] == "customized":
                    kernels.append(_launch_kernel_id())
        outs = [[(t.read_data() if f16 else t.read_fingerprint()) for t in v] for v in vals]
        return outs, kernels
    finally:
        g.close()


class _Options:
    def __init__(self, abi, **opts):
        self.abi, self.opts = abi, opts

    def __enter__(self):
        for k, v in self.opts.items():
            assert self.abi.mi355_set_option(int(k[1:]), v) == 0

    def __exit__(self, *exc):
        for k in self.opts:
            assert self.abi.mi355_set_option(int(k[1:]), 0) == 0


# ---- thread-block add / mul ---------------------------------------------------------
def test_threadblock_add_mul_fingerprint(rt, abi):
    spec = tb_add_mul_case()
    for seed in (1, 2):
        ins = {0: uniform_fp([2, 8, 12], seed), 1: uniform_fp([2, 8, 12], seed + 10)}
        want = orc.eval_graph(spec, "fp", ins)[2][0]
        assert np.array_equal(want, tb_add_mul_exact(ins[0], ins[1]))
        for route, (forced, vector_only) in ROUTES_FP.items():
            with _Options(abi, o1=forced, o4=vector_only):
                got, kernels = _run(rt, spec, ins, False)
            assert np.array_equal(got[2][0], want), (seed, route)
    worst = np.full((2, 8, 12), 25650, np.uint16)
    got, _ = _run(rt, spec, {0: worst, 1: worst}, False)
    assert np.array_equal(got[2][0], tb_add_mul_exact(worst, worst))


def test_threadblock_add_mul_f16(rt, abi):
    spec = tb_add_mul_case()
    ins = {0: normal_f16([2, 8, 12], 0.3, 5), 1: normal_f16([2, 8, 12], 0.3, 6)}
    want = orc.eval_graph(spec, "f16", ins)[2][0]
    for forced in (0, 1):
        with _Options(abi, o1=forced):
            got, _ = _run(rt, spec, ins, True)
        assert_f16_close(got[2][0], want, what=f"tb add/mul, forced interpreter {forced}")


def test_threadblock_add_mul_wider_tiles(rt, abi):
    """The same operators on tiles wide enough for the interpreters' vector paths
    ([1,64,128] with [1,64,1] and [1,1,128]), fp and f16, against the oracle."""
    spec = [
        {"op": "input", "dims": [4, 64, 256]}, {"op": "input", "dims": [4, 64, 256]},
        {"op": "customized", "in": [[0, 0], [1, 0]], "plan": {
            "grid_dim": [4, 1, 1], "forloop_range": 2, "reduction_dimx": 64,
            "input_map": [[0, -1, -1], [0, -1, -1]], "forloop_dim": [2, 2],
            "output_map": [0, -1, -1],
            "ops": [["tb_reduction_2_op", [[0, 0]]], ["tb_reduction_1_op", [[1, 0]]],
                    ["tb_add_op", [[0, 0], [2, 0]]], ["tb_mul_op", [[4, 0], [3, 0]]],
                    ["tb_add_op", [[2, 0], [3, 0]]], ["tb_mul_op", [[5, 0], [1, 0]]],
                    ["tb_add_op", [[7, 0], [6, 0]]]]}},
    ]
    ins = {0: uniform_fp([4, 64, 256], 3), 1: uniform_fp([4, 64, 256], 4)}
    want = orc.eval_graph(spec, "fp", ins, threads=4)[2][0]
    got, _ = _run(rt, spec, ins, False)
    assert np.array_equal(got[2][0], want)
    ins = {0: normal_f16([4, 64, 256], 0.05, 7), 1: normal_f16([4, 64, 256], 0.05, 8)}
    want = orc.eval_graph(spec, "f16", ins, threads=4)[2][0]
    got, _ = _run(rt, spec, ins, True)
    assert_f16_close(got[2][0], want, what="tb add/mul wide tiles")


# ---- an in-place operator on a tile that does not move with the for-loop --------------
def _invariant_unary_case(unary, m=32, k=64, n=32, F=4, grid=1):
    """sum over i of f(A) . B_i: A has forloop_dim -1, so its tile origin never moves, yet the
    reference reloads it every iteration (customized_kernel.cu:323-328) and f, which writes in
    place (src/threadblock/element_unary.cc:46), must see the loaded values each time."""
    return [
        {"op": "input", "dims": [m, k]}, {"op": "input", "dims": [k, n * F * grid]},
        {"op": "customized", "in": [[0, 0], [1, 0]], "plan": {
            "grid_dim": [grid, 1, 1], "forloop_range": F, "reduction_dimx": 64,
            "input_map": [[-1, -1, -1], [1, -1, -1]], "forloop_dim": [-1, 1],
            "output_map": [1, -1, -1],
            "ops": [[f"tb_{unary}_op", [[0, 0]]], ["tb_matmul_op", [[2, 0], [1, 0]]]]}},
    ]


@pytest.mark.parametrize("unary", ["exp", "silu"])
@pytest.mark.parametrize("shape", [(32, 64, 32, 4, 1), (16, 128, 64, 3, 2), (8, 24, 20, 2, 1)])
def test_in_place_unary_on_loop_invariant_tile(rt, abi, unary, shape):
    spec = _invariant_unary_case(unary, *shape)
    ins = {0: uniform_fp(spec[0]["dims"], 21), 1: uniform_fp(spec[1]["dims"], 22)}
    want = orc.eval_graph(spec, "fp", ins)[2][0]
    # exact statement: f(A) . (sum of the B tiles of a block), f applied ONCE
    fA = orc.fp_unary(unary, ins[0]).astype(object)
    m, k, n, F, grid = shape
    Bs = ins[1].astype(object).reshape(k, grid, F, n).sum(axis=2)          # [k, grid, n]
    exact = np.concatenate([fA.dot(Bs[:, b, :]) for b in range(grid)], axis=1) % 25651
    assert np.array_equal(want, exact.astype(np.uint16))
    for route, (forced, vector_only) in ROUTES_FP.items():
        with _Options(abi, o1=forced, o4=vector_only):
            got, kernels = _run(rt, spec, ins, False)
        assert np.array_equal(got[2][0], want), (route, kernels)
    ins16 = {0: normal_f16(spec[0]["dims"], 0.5, 23), 1: normal_f16(spec[1]["dims"], 0.1, 24)}
    want16 = orc.eval_graph(spec, "f16", ins16)[2][0]
    for forced in (0, 1):
        with _Options(abi, o1=forced):
            got, kernels = _run(rt, spec, ins16, True)
        assert_f16_close(got[2][0], want16, what=f"{unary} on invariant tile, forced {forced}, {kernels}")


# ---- full-size configurations against the oracle -----------------------------------------
def _compare_written(got, want, f16, what, peak=None):
    m = orc.written(want)
    assert m.any(), what
    if f16:
        outside = assert_f16_close(got[m], want.view(np.float16)[m], what=what,
                                   peak=None if peak is None else peak[m], strict_outliers=2e-4)
        print(f"  {what}: {outside} of {int(m.sum())} elements outside the plain tolerance", flush=True)
    else:
        assert np.array_equal(got[m], want[m]), what
    return int(m.sum())


def _running_peak(tiles):
    """max over i of |t_0 + ... + t_i| for an iterable of float64 tiles."""
    acc = peak = None
    for t in tiles:
        acc = t if acc is None else acc + t
        peak = np.abs(acc) if peak is None else np.maximum(peak, np.abs(acc))
    return peak


@pytest.mark.parametrize("f16", [False, True], ids=["fp", "f16"])
def test_config3_full_size_heads_vs_oracle(rt, f16):
    """C3 at Q/K/V 32 x 2048 x 128: every thread block of 8 of the 32 heads of both customized
    operators (128 + 512 blocks) through the scalar oracle, compared with the GPU's tensors."""
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config3_mha_prefill()
    heads = (0, 5, 13, 16, 21, 27, 30, 31)
    if f16:
        ins = {i: normal_f16(spec[i]["dims"], 128 ** -0.5, 300 + i) for i in range(3)}
    else:
        ins = {i: uniform_fp(spec[i]["dims"], 300 + i) for i in range(3)}
    got, kernels = _run(rt, spec, ins, f16)
    if f16:
        assert kernels == [3, 5], kernels   # fused attention, fused combine
    p1, p2 = spec[3]["plan"], spec[4]["plan"]
    gx, gy, gz = p1["grid_dim"]
    blocks1 = [h + gx * (by + gy * bz) for h in heads for by in range(gy) for bz in range(gz)]
    print("  oracle op1,", len(blocks1), "blocks", flush=True)
    want1 = orc.customized(p1, [ins[0], ins[1], ins[2]], f16=f16, threads=16, blocks=blocks1)
    peaks = [None, None]
    if f16:
        # The un-normalised numerator sums 32 tiles of magnitude ~1 to values of magnitude
        # ~4-16 that often cancel: its accumulator's path (float64 replay) enters the bound.
        F, nk = p1["forloop_range"], 2048 // p1["forloop_range"]
        peaks = [np.zeros(want1[0].shape), np.zeros(want1[1].shape)]
        for h in heads:
            Q, K, V = (ins[i][h].astype(np.float64) for i in range(3))
            E = np.exp(Q @ K)
            peaks[0][h] = _running_peak(E[:, i * nk:(i + 1) * nk] @ V[i * nk:(i + 1) * nk] for i in range(F))
            peaks[1][h] = _running_peak(E[:, i * nk:(i + 1) * nk].sum(1, keepdims=True) for i in range(F))
    n = sum(_compare_written(got[3][j], w, f16, f"C3 op1 out {j}", peaks[j]) for j, w in enumerate(want1))
    assert n == len(heads) * (2048 * 128 + 2048 * 1 * p1["grid_dim"][1])
    gx, gy, _ = p2["grid_dim"]
    blocks2 = [h + gx * by for h in heads for by in range(gy)]
    print("  oracle op2,", len(blocks2), "blocks", flush=True)
    src = [w.view(np.float16) if f16 else w for w in want1]
    want2 = orc.customized(p2, src, f16=f16, threads=16, blocks=blocks2)
    assert _compare_written(got[4][0], want2[0], f16, "C3 op2") == len(heads) * 2048 * 128


@pytest.mark.parametrize("f16", [False, True], ids=["fp", "f16"])
def test_config5a_full_size_vs_oracle(rt, f16):
    """C5a at X[8,4096], W1/W3[4096,14336], W2[14336,4096]: the whole mugraph (224 + 64 thread
    blocks) through the scalar oracle."""
    from attention_superoptimizer_amd import workloads as W
    spec, _ = W.config5_gated_mlp()
    if f16:
        std = W.INPUT_STD["C5a_gated_mlp"]
        ins = {i: normal_f16(spec[i]["dims"], std[i], 500 + i) for i in range(4)}
    else:
        ins = {i: uniform_fp(spec[i]["dims"], 500 + i) for i in range(4)}
    got, kernels = _run(rt, spec, ins, f16)
    if f16:
        assert kernels == [4, 4], kernels   # fused skinny GEMM, both operators
    print("  oracle, whole graph", flush=True)
    want = orc.eval_graph(spec, "f16" if f16 else "fp", ins, threads=16)
    for i in (4, 5):
        for j, w in enumerate(want[i]):
            if f16:
                assert_f16_close(got[i][j], w, what=f"C5a op {i} out {j}")
            else:
                assert np.array_equal(got[i][j], w), (i, j)


def _c4_peak(ins, F=16):
    X, Wm, A, B = (ins[i].astype(np.float64) for i in range(4))
    kt = X.shape[1] // F
    return _running_peak(X[:, i * kt:(i + 1) * kt] @ Wm[i * kt:(i + 1) * kt] +
                         (X[:, i * kt:(i + 1) * kt] @ A[i * kt:(i + 1) * kt]) @ B for i in range(F))


def _c5a_peaks(ins, gate, up, F1=16, F2=56):
    X, W1, W3, W2 = (ins[i].astype(np.float64) for i in range(4))
    kt = X.shape[1] // F1
    pg = _running_peak(X[:, i * kt:(i + 1) * kt] @ W1[i * kt:(i + 1) * kt] for i in range(F1))
    pu = _running_peak(X[:, i * kt:(i + 1) * kt] @ W3[i * kt:(i + 1) * kt] for i in range(F1))
    g, u = gate.astype(np.float64), up.astype(np.float64)
    H = (g / (1 + np.exp(-g))) * u
    kt = H.shape[1] // F2
    po = _running_peak(H[:, i * kt:(i + 1) * kt] @ W2[i * kt:(i + 1) * kt] for i in range(F2))
    return pg, pu, po


@pytest.mark.parametrize("route", ["fused", "interpreter"])
def test_unit_normal_activations_c4_c5a(rt, abi, route):
    """C4 and C5a with X ~ N(0, 1) (weights N(0, 0.02)): outputs of magnitude up to ~10 whose
    16 / 56 fp16 partial sums often cancel.  Both fp16 routes must stay within the bound that
    counts the accumulator's own ulp, with at most 0.2 % of the elements outside the plain
    tolerance -- and the fused kernels, which keep the iteration order of the additions, no
    worse than the interpreter."""
    from attention_superoptimizer_amd import workloads as W
    with _Options(abi, o1=1 if route == "interpreter" else 0):
        spec, _ = W.config4_lora()
        ins = {i: normal_f16(spec[i]["dims"], (1.0, 0.02, 0.02, 0.02)[i], 900 + i) for i in range(4)}
        got, _ = _run(rt, spec, ins, True)
        want = orc.eval_graph(spec, "f16", ins, threads=16)
        n = assert_f16_close(got[4][0], want[4][0], what="C4, X ~ N(0,1)", peak=_c4_peak(ins),
                             strict_outliers=2e-3)
        print(f"  C4 {route}: {n} of {want[4][0].size} outside the plain tolerance", flush=True)
        spec, _ = W.config5_gated_mlp()
        ins = {i: normal_f16(spec[i]["dims"], (1.0, 0.02, 0.02, 0.02)[i], 900 + i) for i in range(4)}
        got, _ = _run(rt, spec, ins, True)
        want = orc.eval_graph(spec, "f16", ins, threads=16)
        pg, pu, po = _c5a_peaks(ins, want[4][0], want[4][1])
        assert_f16_close(got[4][0], want[4][0], what="C5a gate", peak=pg, strict_outliers=2e-3)
        assert_f16_close(got[4][1], want[4][1], what="C5a up", peak=pu, strict_outliers=2e-3)
        n = assert_f16_close(got[5][0], want[5][0], what="C5a, X ~ N(0,1)", peak=po, strict_outliers=2e-3)
        print(f"  C5a {route}: {n} of {want[5][0].size} outside the plain tolerance", flush=True)
