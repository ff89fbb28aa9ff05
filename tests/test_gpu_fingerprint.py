"""GPU parity of the fingerprint path: HIP kernels (through the C ABI and the
host API above it) against the CPU oracle, bit for bit."""
import ctypes

import numpy as np
import pytest

from helpers import FP_PQ, load_gqa_fixture, uniform_fp
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu


def _graph_fp(rt, spec, inputs=None):
    """Builds spec through the host API, fingerprints every op, returns per-op outputs."""
    g, vals = rt.build_from_spec(spec)
    try:
        for i, op in enumerate(spec):
            if op["op"] == "input" and inputs is not None and i in inputs:
                vals[i][0].write_fingerprint(inputs[i])
            else:
                g.fingerprint(i)
        return [[t.read_fingerprint() for t in v] for v in vals]
    finally:
        g.close()


@pytest.mark.parametrize("shape", [(1, 16, 64, 48), (3, 70, 33, 129), (2, 256, 64, 4096),
                                   (1, 5, 7, 3), (1, 130, 200, 72), (3, 64, 128, 64),
                                   (1, 192, 320, 448)])
def test_kernel_matmul_matches_oracle(rt, shape):
    b, m, n, k = shape
    A = uniform_fp((b, m, k), 11)
    B = uniform_fp((b, k, n), 12)
    spec = [{"op": "input", "dims": [b, m, k]}, {"op": "input", "dims": [b, k, n]},
            {"op": "matmul", "in": [[0, 0], [1, 0]]}]
    got = _graph_fp(rt, spec, {0: A, 1: B})[2][0]
    want = orc.fp_matmul(A, B)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape", [(1, 33, 65, 4100), (1, 64, 64, 65536 + 128), (2, 128, 192, 1024)])
def test_kernel_matmul_extreme_values(rt, shape):
    """All operands 25650: the largest products, k long enough to need folding (ragged
    shapes take the general kernel, multiples of 64 the aligned one)."""
    b, m, n, k = shape
    A = np.full((b, m, k), FP_PQ - 1, np.uint16)
    B = np.full((b, k, n), FP_PQ - 1, np.uint16)
    spec = [{"op": "input", "dims": [b, m, k]}, {"op": "input", "dims": [b, k, n]},
            {"op": "matmul", "in": [[0, 0], [1, 0]]}]
    got = _graph_fp(rt, spec, {0: A, 1: B})[2][0]
    assert np.all(got == (k * (FP_PQ - 1) ** 2) % FP_PQ)


def test_kernel_elementwise_and_reduction(rt):
    X = uniform_fp((2, 64, 96), 3)
    Y = uniform_fp((2, 64, 1), 4)
    Z = uniform_fp((2, 1, 96), 5)
    spec = [
        {"op": "input", "dims": [2, 64, 96]}, {"op": "input", "dims": [2, 64, 1]},
        {"op": "input", "dims": [2, 1, 96]},
        {"op": "exp", "in": [[0, 0]]},
        {"op": "div", "in": [[3, 0], [1, 0]]},
        {"op": "add", "in": [[4, 0], [2, 0]]},
        {"op": "mul", "in": [[5, 0], [0, 0]]},
        {"op": "silu", "in": [[6, 0]]},
        {"op": "reduction", "in": [[7, 0]], "dim": 2, "size": 1},
        {"op": "reduction", "in": [[7, 0]], "dim": 2, "size": 32},
        {"op": "reduction", "in": [[7, 0]], "dim": 1, "size": 1},
        {"op": "reduction", "in": [[7, 0]], "dim": 0, "size": 1},
        {"op": "div", "in": [[1, 0], [2, 0]]},
    ]
    ins = {0: X, 1: Y, 2: Z}
    got = _graph_fp(rt, spec, ins)
    want = orc.eval_graph(spec, "fp", ins)
    for i in range(3, len(spec)):
        assert np.array_equal(got[i][0], want[i][0]), spec[i]


def test_iota_inputs_and_compare(rt):
    spec = [{"op": "input", "dims": [3, 100, 91]}, {"op": "input", "dims": [3, 100, 91]}]
    g, vals = rt.build_from_spec(spec)
    try:
        g.fingerprint_all()
        a = vals[0][0].read_fingerprint()
        assert np.array_equal(a.ravel(), np.arange(a.size) % FP_PQ)
        assert vals[0][0].has_same_fingerprint(vals[1][0])
        b = a.copy()
        b[2, 99, 90] ^= 1
        vals[1][0].write_fingerprint(b)
        assert not vals[0][0].has_same_fingerprint(vals[1][0])
    finally:
        g.close()


def test_uniform_fill_matches_host_generator(rt, abi):
    spec = [{"op": "input", "dims": [5, 77, 13]}]
    g, vals = rt.build_from_spec(spec)
    try:
        t = vals[0][0]
        assert abi.mi355_fp_fill_uniform(ctypes.c_void_p(t.device_ptr(True)), t.num_elements, 1234) == 0
        assert np.array_equal(t.read_fingerprint(), uniform_fp(t.dims, 1234))
    finally:
        g.close()


def _fused_matmul_routes(rt, abi, spec, ins, op_index=2):
    """Fingerprints the customized op of `spec` four ways: fused kernel and interpreter, each on
    the matrix cores where the shapes allow and with the vector-dot path only.  Returns
    {route: (kernel id, LDS bytes, output)}."""
    import ctypes as ct
    from attention_superoptimizer_amd import _native as N
    got = {}
    routes = {"auto": (0, 0), "vector-dot": (0, 1), "interpreter": (1, 0), "interpreter, vector-dot": (1, 1)}
    for route, (forced, vector_only) in routes.items():
        assert abi.mi355_set_option(1, forced) == 0 and abi.mi355_set_option(4, vector_only) == 0
        try:
            g, vals = rt.build_from_spec(spec)
            try:
                for i, a in ins.items():
                    vals[i][0].write_fingerprint(a)
                g.fingerprint(op_index)
                info = N.Mi355LaunchInfo()
                N.backend().mi355_last_launch(ct.byref(info))
                got[route] = (info.kernel_id, info.lds_bytes, vals[op_index][0].read_fingerprint())
            finally:
                g.close()
        finally:
            assert abi.mi355_set_option(1, 0) == 0 and abi.mi355_set_option(4, 0) == 0
    return got


@pytest.mark.parametrize("m,n,k,grid,F,amap,bmap,omap", [
    (128, 256, 256, (4, 2, 1), 4, (-1, 0, -1), (1, -1, -1), (1, 0, -1)),     # 64x64 tiles, k chunk 64
    # matrix-core route: k tiles of 16 / 48 / 80 (chunks of several iterations share a matrix
    # instruction, the last one partly empty), tiles of 16 / 48 rows or columns, one / two /
    # many 32 x 32 pieces per tile, for-loops split over workgroups
    (16, 16, 16 * 7, (1, 1, 1), 7, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),
    (48, 32, 48 * 5, (1, 1, 1), 5, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),
    (32, 64, 80 * 3, (1, 1, 1), 3, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),
    (96, 240, 32 * 9, (3, 2, 1), 9, (-1, 0, -1), (1, -1, -1), (1, 0, -1)),    # 48 x 80 tiles
    (256, 128, 2048, (2, 1, 1), 128, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),  # 256 x 64 tiles, k 16
    (64, 64, 16 * 1001, (1, 1, 1), 1001, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),
    # 2048 blocks of 16 x 32 outputs: a workgroup takes 4 x 2 neighbouring blocks as one tile
    (1024, 1024, 256, (32, 64, 1), 4, (-1, 0, -1), (1, -1, -1), (1, 0, -1)),
    # 128 x 16 tiles, 512 blocks: two neighbours along x share their A strips
    (512, 2048, 128, (128, 4, 1), 8, (-1, 0, -1), (1, -1, -1), (1, 0, -1)),
    (256, 256, 512, (2, 2, 1), 4, (-1, 0, -1), (1, -1, -1), (1, 0, -1)),     # 128x128 tiles, 4 register tiles
    (64, 64, 512, (1, 1, 1), 8, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),   # one block: for-loop split 8 ways
    (16, 40, 96, (1, 1, 1), 4, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),    # 16x40 tile, k tile 24 -> chunk 8
    (64, 1024, 1024, (16, 1, 1), 16, (-1, -1, -1), (1, -1, -1), (1, -1, -1)),  # config C1
    (96, 192, 320, (2, 3, 1), 2, (-1, 0, -1), (1, -1, -1), (1, 0, -1)),      # 32x96 tiles, k tile 160 -> chunk 32
    # 40,000 iterations of an 8-deep k tile: 625 steps per workgroup after the 64-way split, so
    # the running sums are folded mid-way
    (16, 32, 320000, (1, 1, 1), 40000, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1)),
])
def test_fused_matmul_fingerprint_equals_interpreter_and_oracle(rt, abi, m, n, k, grid, F, amap, bmap, omap):
    """A load-load-matmul-accumulate plan runs on the fused fingerprint matmul kernel; forced
    through the interpreter it must give the same uint16 tensor, and both the oracle's."""
    from attention_superoptimizer_amd import workloads as W
    spec = W.tiled_matmul(m, n, k, grid, F, amap, bmap, omap)[0]
    ins = {0: uniform_fp(spec[0]["dims"], 31), 1: uniform_fp(spec[1]["dims"], 32)}
    ins[0].flat[:7] = 25650  # worst-case operands in one corner
    ins[1].flat[:7] = 25650
    want = orc.eval_graph(spec, "fp", ins, threads=8)[2][0]
    got = _fused_matmul_routes(rt, abi, spec, ins)
    for route, (kernel_id, _, out) in got.items():
        assert kernel_id == (1 if route.startswith("interpreter") else 6), route
        assert np.array_equal(out, want), route


def test_fused_matmul_fingerprint_takes_tiles_the_interpreter_cannot_hold(rt, abi):
    """A [128,256] and B [256,128] tiles need 197 KB of LDS in the interpreter; the fused
    kernels keep no tile there (the matrix-core one reads residue planes, the vector-dot one
    streams k chunks of 64 through LDS) and match the oracle."""
    from attention_superoptimizer_amd import workloads as W
    spec = W.tiled_matmul(512, 512, 1024, (4, 4, 1), 4, (-1, 0, -1), (1, -1, -1), (1, 0, -1))[0]
    ins = {0: uniform_fp(spec[0]["dims"], 41), 1: uniform_fp(spec[1]["dims"], 42)}
    want = orc.eval_graph(spec, "fp", ins, threads=8)[2][0]
    for vector_only, lds in ((0, 32768), (1, 2 * 2 * 16 * (128 + 4 + 128) * 4)):
        assert abi.mi355_set_option(4, vector_only) == 0
        try:
            g, vals = rt.build_from_spec(spec)
            try:
                vals[0][0].write_fingerprint(ins[0])
                vals[1][0].write_fingerprint(ins[1])
                g.fingerprint(2)
                info = N_launch_info()
                assert info.kernel_id == 6 and info.lds_bytes == lds
                assert np.array_equal(vals[2][0].read_fingerprint(), want)
            finally:
                g.close()
        finally:
            assert abi.mi355_set_option(4, 0) == 0


def N_launch_info():
    import ctypes as ct
    from attention_superoptimizer_amd import _native as N
    info = N.Mi355LaunchInfo()
    N.backend().mi355_last_launch(ct.byref(info))
    return info


def test_fused_matmul_fingerprint_batched_operands_and_mismatched_maps(rt, abi):
    """Matrix-core route over 3-D operands (grid z walks the batch dim), and over plans whose
    maps do not describe A.B (the for-loop walks A's rows; both loaders take the same block
    column): every route must give what the plan says, i.e. the oracle's answer."""
    from attention_superoptimizer_amd import workloads as W
    cases = []
    b, m, n, k = 3, 64, 96, 128
    cases.append(([W._inp([b, m, k]), W._inp([b, k, n]),
                   {"op": "customized", "in": [[0, 0], [1, 0]],
                    "plan": W._plan((2, 3, b), 4, [(1, -1, 0), (-1, 2, 0)], (2, 1), (1, 2, 0),
                                    [("tb_matmul_op", [(0, 0), (1, 0)])])}], 51))
    # for-loop over A's rows and B's rows: sum over i of A[32 i : 32 i + 32, :64] . B[64 i : 64 i + 64, :]
    cases.append(([W._inp([128, 64]), W._inp([256, 48]),
                   {"op": "customized", "in": [[0, 0], [1, 0]],
                    "plan": W._plan((1, 1, 1), 4, [(-1, -1, -1), (-1, -1, -1)], (0, 0), (-1, -1, -1),
                                    [("tb_matmul_op", [(0, 0), (1, 0)])])}], 52))
    for spec, seed in cases:
        ins = {0: uniform_fp(spec[0]["dims"], seed), 1: uniform_fp(spec[1]["dims"], seed + 100)}
        want = orc.eval_graph(spec, "fp", ins, threads=8)[2][0]
        got = _fused_matmul_routes(rt, abi, spec, ins)
        for route, (kernel_id, lds, out) in got.items():
            assert np.array_equal(out, want), (route, spec[2]["plan"])
        assert got["auto"][0] == 6 and got["auto"][1] == 32768


@pytest.mark.parametrize("pro", [("exp", None), (None, "silu"), ("silu", "exp")])
def test_fused_matmul_fingerprint_with_operand_prologues(rt, abi, pro):
    """exp / silu of a loaded tile before the matmul (the second op of the MLP plans): on the
    matrix-core route the operator is applied once per element while the operand tensor is
    split into planes; the other routes run the plan in the interpreter.  All equal the oracle."""
    from attention_superoptimizer_amd import workloads as W
    m, n, k, F = 64, 256, 512, 4
    ops, a_ref, b_ref, nxt = [], (0, 0), (1, 0), 2
    for which, name in enumerate(pro):
        if name is not None:
            ops.append((f"tb_{name}_op", [(which, 0)]))
            if which == 0:
                a_ref = (nxt, 0)
            else:
                b_ref = (nxt, 0)
            nxt += 1
    ops.append(("tb_matmul_op", [a_ref, b_ref]))
    spec = [W._inp([m, k]), W._inp([k, n]),
            {"op": "customized", "in": [[0, 0], [1, 0]],
             "plan": W._plan((4, 1, 1), F, [(-1, -1, -1), (1, -1, -1)], (1, 0), (1, -1, -1), ops)}]
    ins = {0: uniform_fp(spec[0]["dims"], 71), 1: uniform_fp(spec[1]["dims"], 72)}
    ins[0].flat[:5] = [0, 1, 112, 113, 25650]
    want = orc.eval_graph(spec, "fp", ins, threads=8)[2][0]
    got = _fused_matmul_routes(rt, abi, spec, ins)
    for route, (kernel_id, lds, out) in got.items():
        assert kernel_id == (6 if route == "auto" else 1), route
        assert np.array_equal(out, want), route


@pytest.mark.parametrize("m,n,k,grid,F,epi,pro,fused", [
    (64, 256, 512, (4, 1, 1), 8, "exp", None, True),      # k tile 64: one step per iteration
    (64, 256, 512, (4, 1, 1), 4, "silu", "exp", True),    # k tile 128, exp(A) before, silu after
    (32, 32, 1024, (1, 1, 1), 16, "exp", None, True),     # one 32 x 32 piece: wavefronts share iterations
    (64, 32, 64 * 37, (1, 1, 1), 37, "exp", None, True),  # two pieces, 37 iterations: uneven shares, split for-loop
    (64, 256, 512, (4, 1, 1), 16, "exp", None, True),     # k tile 32: a step of two chunks per iteration
    (64, 256, 256, (4, 1, 1), 16, "exp", None, True),     # k tile 16: a step of one chunk
    (32, 32, 1024, (1, 1, 1), 32, "exp", None, True),     # k tile 32, one piece shared by four wavefronts
    (64, 32, 48 * 21, (1, 1, 1), 21, "silu", None, True), # k tile 48, two pieces, uneven shares
    (64, 256, 80 * 4, (4, 1, 1), 4, "exp", None, False),  # k tile 80: not whole steps, interpreter
])
def test_fused_matmul_fingerprint_with_operator_on_the_products(rt, abi, m, n, k, grid, F, epi, pro, fused):
    """exp / silu of every iteration's product before the saver adds it up (sum over
    iterations of f(A_it . B_it)): on the matrix-core route each iteration's residue sums are
    recombined, the operator applied and the result added to a running sum."""
    from attention_superoptimizer_amd import workloads as W
    ops, a_ref, nxt = [], (0, 0), 2
    if pro is not None:
        ops.append((f"tb_{pro}_op", [(0, 0)]))
        a_ref, nxt = (nxt, 0), nxt + 1
    ops.append(("tb_matmul_op", [a_ref, (1, 0)]))
    ops.append((f"tb_{epi}_op", [(nxt, 0)]))
    b_imap = (1, -1, -1) if grid[0] > 1 else (-1, -1, -1)
    omap = (1, -1, -1) if grid[0] > 1 else (-1, -1, -1)
    spec = [W._inp([m, k]), W._inp([k, n]),
            {"op": "customized", "in": [[0, 0], [1, 0]],
             "plan": W._plan(grid, F, [(-1, -1, -1), b_imap], (1, 0), omap, ops)}]
    ins = {0: uniform_fp(spec[0]["dims"], 81), 1: uniform_fp(spec[1]["dims"], 82)}
    want = orc.eval_graph(spec, "fp", ins, threads=8)[2][0]
    got = _fused_matmul_routes(rt, abi, spec, ins)
    for route, (kernel_id, lds, out) in got.items():
        assert kernel_id == (6 if route == "auto" and fused else 1), route
        assert np.array_equal(out, want), route


def test_many_fills_and_many_compares_in_one_launch(rt, abi):
    """mi355_fp_fill_many over 40 tensors of ragged sizes = the single-tensor fill of each;
    mi355_fp_equal_enqueue_many over 40 pairs = the verdict of each pair (every third pair is
    made to differ in one element, at the very end or the very start)."""
    sizes = [1 + 37 * i + (i % 5) * 4096 for i in range(40)]
    spec = [{"op": "input", "dims": [n]} for n in sizes] * 2
    g, vals = rt.build_from_spec(spec)
    try:
        left, right = [v[0] for v in vals[:40]], [v[0] for v in vals[40:]]
        for side in (left, right):
            ptrs = (ctypes.c_void_p * 40)(*[t.device_ptr(True) for t in side])
            ns = (ctypes.c_size_t * 40)(*sizes)
            seeds = (ctypes.c_uint64 * 40)(*[9000 + i for i in range(40)])
            assert abi.mi355_fp_fill_many(ptrs, ns, seeds, 40, 0) == 0
        for i, t in enumerate(left):
            assert np.array_equal(t.read_fingerprint(), uniform_fp(t.dims, 9000 + i)), i
        # tensors of equal length and seed (the same input of several candidates) are computed
        # once and stored to each: every one of them must still hold the sequence
        same = list(range(0, 40, 5))  # sizes 1, 186, 371, ... with i % 5 == 0
        rep = [left[i] for i in same] + [right[i] for i in same]
        ptrs = (ctypes.c_void_p * 16)(*[t.device_ptr(True) for t in rep])
        ns = (ctypes.c_size_t * 16)(*([sizes[i] for i in same] * 2))
        seeds = (ctypes.c_uint64 * 16)(*([77 + (i % 10) for i in same] * 2))
        assert abi.mi355_fp_fill_many(ptrs, ns, seeds, 16, 0) == 0
        for j, t in enumerate(rep):
            i = same[j % 8]
            assert np.array_equal(t.read_fingerprint(), uniform_fp(t.dims, 77 + (i % 10))), j
        for side in (left, right):  # back to the values the compares below expect
            ptrs = (ctypes.c_void_p * 40)(*[t.device_ptr(True) for t in side])
            ns = (ctypes.c_size_t * 40)(*sizes)
            seeds = (ctypes.c_uint64 * 40)(*[9000 + i for i in range(40)])
            assert abi.mi355_fp_fill_many(ptrs, ns, seeds, 40, 0) == 0
        differ = [i % 3 == 1 for i in range(40)]
        for i, t in enumerate(right):
            if differ[i]:
                a = t.read_fingerprint()
                a[-1 if i % 2 else 0] ^= 1
                t.write_fingerprint(a)
        assert abi.mi355_fp_equal_reset(100, 40) == 0
        pa = (ctypes.c_void_p * 40)(*[t.device_ptr(True) for t in left])
        pb = (ctypes.c_void_p * 40)(*[t.device_ptr(True) for t in right])
        ns = (ctypes.c_size_t * 40)(*sizes)
        slots = (ctypes.c_int * 40)(*[100 + i for i in range(40)])
        assert abi.mi355_fp_equal_enqueue_many(pa, pb, ns, slots, 40) == 0
        eq = (ctypes.c_ubyte * 40)()
        assert abi.mi355_fp_equal_collect(100, 40, eq) == 0
        assert [bool(e) for e in eq] == [not d for d in differ]
    finally:
        g.close()


def _matmul_many(abi, rt, shapes, fill):
    """Runs mi355_fp_matmul_many over (batch, m, n, k) shapes; returns inputs and outputs."""
    spec = []
    for b, m, n, k in shapes:
        spec += [{"op": "input", "dims": [b, m, k]}, {"op": "input", "dims": [b, k, n]},
                 {"op": "input", "dims": [b, m, n]}]
    g, vals = rt.build_from_spec(spec)
    try:
        cnt = len(shapes)
        ins = []
        for i, (b, m, n, k) in enumerate(shapes):
            A, B = fill(i, (b, m, k)), fill(100 + i, (b, k, n))
            vals[3 * i][0].write_fingerprint(A)
            vals[3 * i + 1][0].write_fingerprint(B)
            vals[3 * i + 2][0].write_fingerprint(np.full((b, m, n), 7, np.uint16))
            ins.append((A, B))
        pa = (ctypes.c_void_p * cnt)(*[vals[3 * i][0].device_ptr(True) for i in range(cnt)])
        pb = (ctypes.c_void_p * cnt)(*[vals[3 * i + 1][0].device_ptr(True) for i in range(cnt)])
        pc = (ctypes.c_void_p * cnt)(*[vals[3 * i + 2][0].device_ptr(True) for i in range(cnt)])
        arr = lambda j: (ctypes.c_int * cnt)(*[s[j] for s in shapes])
        assert abi.mi355_fp_matmul_many(pa, pb, pc, arr(0), arr(1), arr(2), arr(3), cnt) == 0
        return ins, [vals[3 * i + 2][0].read_fingerprint() for i in range(cnt)]
    finally:
        g.close()


def test_many_matmuls_on_the_matrix_cores_match_oracle(rt, abi):
    """mi355_fp_matmul_many (signed-byte residue planes, int8 matrix instructions) over ragged,
    batched, tiny and large shapes = the oracle's `(r + a*b) % 25651` chains, bit for bit; more
    matmuls than one group takes; both workgroup shapes (64x64 tiles, and 32x32 tiles whose
    wavefronts share k)."""
    shapes = [(1, 16, 64, 48), (3, 70, 33, 129), (2, 256, 64, 4096), (1, 5, 7, 3), (1, 130, 200, 72),
              (3, 64, 128, 64), (1, 192, 320, 448), (1, 1024, 1024, 256), (1, 1, 1, 1),
              (4, 512, 512, 64), (1, 64, 1024, 1024), (1, 33, 65, 4100)]
    shapes = shapes + [(1, 16 + 16 * (i % 5), 32 + 8 * i, 64 + 24 * i) for i in range(28)]
    ins, got = _matmul_many(abi, rt, shapes, lambda i, d: uniform_fp(d, 60 + i))
    for (A, B), C, s in zip(ins, got, shapes):
        assert np.array_equal(C, orc.fp_matmul(A, B)), s


def test_large_matmuls_on_128_tiles_match_oracle(rt, abi):
    """Matmuls with 256 or more output tiles of 128 x 128, or of 128 x 64 when there are fewer
    of the wide ones, take the kernel that stages operand strips through LDS (shapes of both
    kinds below): ragged edges in rows, columns and k, a batch, one k step and an odd number of
    them, both tile orders, together with small matmuls in the same call; with the option that
    keeps 64 x 64 tiles the same calls give the same bits."""
    shapes = [(1, 2008, 1544, 200), (3, 1024, 1024, 72), (1, 48, 80, 64), (1, 2048, 2048, 64),
              (2, 1100, 1500, 330), (1, 16, 16, 16),
              # 512 tiles or more: the order in which workgroups take tiles follows the XCDs; tile
              # rows that are no multiple of 8, tile counts that are no multiple of 8, a batch
              (1, 2700, 3200, 64), (3, 1700, 1800, 100)]
    fill = lambda i, d: uniform_fp(d, 900 + i)
    ins, got = _matmul_many(abi, rt, shapes, fill)
    for (A, B), C, s in zip(ins, got, shapes):
        assert np.array_equal(C, orc.fp_matmul(A, B)), s
    assert abi.mi355_set_option(4, 2) == 0
    try:
        _, again = _matmul_many(abi, rt, shapes, fill)
    finally:
        assert abi.mi355_set_option(4, 0) == 0
    for C, D, s in zip(got, again, shapes):
        assert np.array_equal(C, D), s
    x = (114 * 25425 + 112 * 227) % FP_PQ       # = -113 (mod 227), 112 (mod 113)
    _, ext = _matmul_many(abi, rt, [(1, 1536, 2048, 8192)], lambda i, d: np.full(d, x, np.uint16))
    assert np.all(ext[0] == (8192 * x * x) % FP_PQ)


@pytest.mark.parametrize("n,k", [(2048, 640), (2048, 600), (1024, 640), (1024, 1000)],
                         ids=["128x128 tiles", "128x128 tiles, ragged k", "128x64 tiles", "128x64 tiles, ragged k"])
def test_128_row_tiles_take_every_operand_of_the_last_k_step(rt, abi, n, k):
    """The kernels on 128-row tiles prefetch B^T with loads that complete behind the compiler's
    back.  An operand read before it landed would be the one of an earlier step, or of the call
    before: so the same device buffers are multiplied three times in a row -- as filled, then
    with only the last 64 of k changed in B, then with only those changed in A -- and every
    product must equal the oracle's on slices of rows and columns from every corner, and the
    64 x 64-tile kernel's (ordinary loads) everywhere."""
    m = 2048
    A = uniform_fp((1, m, k), 3100 + k)
    B = uniform_fp((1, k, n), 3200 + k)
    A2, B2 = A.copy(), B.copy()
    B2[:, k - 64:, :] = uniform_fp((1, 64, n), 3300 + k)
    A2[:, :, k - 64:] = uniform_fp((1, m, 64), 3400 + k)
    spec = [{"op": "input", "dims": [1, m, k]}, {"op": "input", "dims": [1, k, n]},
            {"op": "input", "dims": [1, m, n]}]
    rows = np.r_[0:8, 1016:1032, m - 8:m]
    cols = np.r_[0:8, n // 2 - 8:n // 2 + 8, n - 8:n]
    g, vals = rt.build_from_spec(spec)
    try:
        a, b, c = (vals[i][0] for i in range(3))
        products = []
        for step, (x, y) in enumerate([(A, B), (A, B2), (A2, B2)]):
            a.write_fingerprint(x)
            b.write_fingerprint(y)
            got = {}
            for route in (0, 2):
                c.write_fingerprint(np.full((1, m, n), 7, np.uint16))
                assert abi.mi355_set_option(4, route) == 0
                try:
                    assert abi.mi355_fp_matmul(ctypes.c_void_p(a.device_ptr(True)), ctypes.c_void_p(b.device_ptr(True)),
                                               ctypes.c_void_p(c.device_ptr(True)), 1, m, n, k) == 0
                finally:
                    assert abi.mi355_set_option(4, 0) == 0
                got[route] = c.read_fingerprint()
            assert np.array_equal(got[0][0, rows, :], orc.fp_matmul(x[:, rows, :], y)[0]), step
            assert np.array_equal(got[0][0][:, cols], orc.fp_matmul(x, y[:, :, cols])[0]), step
            assert np.array_equal(got[0], got[2]), step
            products.append(got[0])
        # (the changes are seen: they alter the products)
        assert not np.array_equal(products[0], products[1]) and not np.array_equal(products[1], products[2])
    finally:
        g.close()


def test_the_self_check_of_the_128_row_tile_kernels_passes(rt, abi):
    """What mi355_init ran once on this device; on demand it gives the same verdict and leaves
    the routes as they were."""
    passed = ctypes.c_int(-1)
    assert abi.mi355_fp_big_tiles_check(ctypes.byref(passed)) == 0
    assert passed.value == 1


def test_full_size_matmul_checksum_of_checksums(rt, abi):
    """4096 x 4096 x 4096, uniform inputs: too large for the oracle as a whole, so the check is
    linear algebra in the ring: (1^T A) B = 1^T (A B) and A (B 1) = (A B) 1.  The two vector
    products are the oracle's; the sums are exact integer arithmetic."""
    n = 4096
    ins, got = _matmul_many(abi, rt, [(1, n, n, n)], lambda i, d: uniform_fp(d, 4000 + i))
    (A, B), C = ins[0], got[0]
    A2, B2, C2 = (x.reshape(n, n).astype(np.int64) for x in (A, B, C))
    assert C2.max() < FP_PQ
    col_of_a = (A2.sum(axis=0) % FP_PQ).astype(np.uint16).reshape(1, 1, n)
    row_of_b = (B2.sum(axis=1) % FP_PQ).astype(np.uint16).reshape(1, n, 1)
    want_cols = orc.fp_matmul(col_of_a, B.reshape(1, n, n)).reshape(n).astype(np.int64)
    want_rows = orc.fp_matmul(A.reshape(1, n, n), row_of_b).reshape(n).astype(np.int64)
    assert np.array_equal(C2.sum(axis=0) % FP_PQ, want_cols)
    assert np.array_equal(C2.sum(axis=1) % FP_PQ, want_rows)


def test_matrix_core_matmul_extreme_values_and_long_k(rt, abi):
    """Operands whose residues are the largest in magnitude the planes hold (-113 mod 227,
    112 mod 113), k long enough that a wavefront's int32 sums must be folded on the way."""
    x = (114 * 25425 + 112 * 227) % FP_PQ       # = -113 (mod 227), 112 (mod 113)
    y = (113 * 25425 + 112 * 227) % FP_PQ       # = +113 (mod 227)
    assert x % 227 == 114 and y % 227 == 113 and x % 113 == 112
    shapes = [(1, 16, 16, 800000), (1, 48, 32, 70000), (2, 128, 192, 1024)]
    for a, b in ((x, x), (x, y), (FP_PQ - 1, FP_PQ - 1)):
        fill = lambda i, d: np.full(d, a if i < 100 else b, np.uint16)
        _, got = _matmul_many(abi, rt, shapes, fill)
        for C, (_, m, n, k) in zip(got, shapes):
            assert np.all(C == (k * a * b) % FP_PQ), (a, b, k)


def test_many_binary_operators_in_one_launch(rt, abi):
    """mi355_fp_binary_many over 30 add / mul / div operators of unlike shapes, with operands
    broadcast along any axis, = the oracle's element-wise result of each."""
    shapes = [((3, 70, 33), (3, 70, 33)), ((2, 64, 96), (2, 64, 1)), ((2, 64, 96), (2, 1, 96)),
              ((1, 1, 257), (4, 5, 257)), ((1000,), (1000,)), ((16, 1), (16, 4096)),
              ((2, 3, 5, 7), (2, 1, 5, 1)), ((1, 512, 512), (1, 512, 512)), ((7, 1), (1, 9)),
              ((1,), (1,))]
    names, codes = ["add", "mul", "div"], [1008, 1009, 1010]
    cases = [(shapes[i % len(shapes)], i % 3) for i in range(30)]
    spec = []
    for (sa, sb), _ in cases:
        so = list(np.broadcast_shapes(sa, sb))
        spec += [{"op": "input", "dims": list(sa)}, {"op": "input", "dims": list(sb)},
                 {"op": "input", "dims": so}]
    g, vals = rt.build_from_spec(spec)
    try:
        n = len(cases)
        want = []
        for i, ((sa, sb), which) in enumerate(cases):
            A, B = uniform_fp(sa, 500 + i), uniform_fp(sb, 700 + i)
            vals[3 * i][0].write_fingerprint(A)
            vals[3 * i + 1][0].write_fingerprint(B)
            want.append(orc.fp_binary(names[which], A, B))
        pad = lambda d: list(d) + [1] * (4 - len(d))
        ops = (ctypes.c_int * n)(*[codes[w] for _, w in cases])
        in1 = (ctypes.c_void_p * n)(*[vals[3 * i][0].device_ptr(True) for i in range(n)])
        in2 = (ctypes.c_void_p * n)(*[vals[3 * i + 1][0].device_ptr(True) for i in range(n)])
        out = (ctypes.c_void_p * n)(*[vals[3 * i + 2][0].device_ptr(True) for i in range(n)])
        d1 = (ctypes.c_int * (4 * n))(*sum([pad(sa) for (sa, _), _ in cases], []))
        d2 = (ctypes.c_int * (4 * n))(*sum([pad(sb) for (_, sb), _ in cases], []))
        do = (ctypes.c_int * (4 * n))(*sum([pad(np.broadcast_shapes(sa, sb)) for (sa, sb), _ in cases], []))
        nd = (ctypes.c_int * n)(*[len(sa) for (sa, _), _ in cases])
        assert abi.mi355_fp_binary_many(ops, in1, d1, in2, d2, out, do, nd, n) == 0
        for i in range(n):
            assert np.array_equal(vals[3 * i + 2][0].read_fingerprint(), want[i]), cases[i]
        # more operators than one launch takes, or a shape that does not broadcast: refused
        assert abi.mi355_fp_binary_many(ops, in1, d1, in2, d2, out, do, nd, 33) != 0
        d2[1] = 5
        assert abi.mi355_fp_binary_many(ops, in1, d1, in2, d2, out, do, nd, n) != 0
    finally:
        g.close()


def test_batched_customized_fingerprints_of_generated_candidates(rt, abi):
    """Many small, unlike customized ops (the generator's candidates, dims <= 256) through
    mi355_customized_fp_batch in one call = one mi355_customized_fp each, bit for bit."""
    from attention_superoptimizer_amd import _native as N
    from attention_superoptimizer_amd import candidates as C
    problems = C.generate(num_problems=4, per_problem=12, seed=77, max_dim=256)
    built, plans, ins, outs, want = [], [], [], [], []
    try:
        for prob in problems:
            for cand in prob["candidates"]:
                spec = cand["spec"]
                # candidates whose customized op consumes only graph inputs
                idx = [i for i, op in enumerate(spec) if op["op"] == "customized"
                       and all(spec[a]["op"] == "input" for a, _ in op["in"])]
                if not idx:
                    continue
                g, vals = rt.build_from_spec(spec)
                built.append((g, vals, idx[0]))
                for i, op in enumerate(spec):
                    if op["op"] == "input":
                        vals[i][0].write_fingerprint(uniform_fp(op["dims"], 4000 + i))
                g.fingerprint(idx[0])
                want.append([t.read_fingerprint() for t in vals[idx[0]]])
                for t in vals[idx[0]]:
                    t.write_fingerprint(np.zeros(t.dims, np.uint16))
                plans.append(g.lowered(idx[0], True))
                row_in = [vals[a][b].device_ptr(True) for a, b in spec[idx[0]]["in"]]
                row_out = [t.device_ptr(True) for t in vals[idx[0]]]
                ins += row_in + [0] * (4 - len(row_in))
                outs += row_out + [0] * (4 - len(row_out))
        n = len(plans)
        assert n >= 24
        arr = (N.Mi355Plan * n)(*plans)
        assert abi.mi355_sync() == 0
        print("batch of", n, "customized ops", flush=True)
        assert abi.mi355_customized_fp_batch(arr, n, (ctypes.c_void_p * len(ins))(*ins),
                                             (ctypes.c_void_p * len(outs))(*outs)) == 0, N.last_error()
        assert abi.mi355_sync() == 0
        for k, (g, vals, i) in enumerate(built):
            for a, b in zip([t.read_fingerprint() for t in vals[i]], want[k]):
                assert np.array_equal(a, b), k
    finally:
        for g, _, _ in reversed(built):
            g.close()


def _check_examples(rt, names, random_inputs):
    from attention_superoptimizer_amd import workloads as W
    for name in names:
        spec, ref = W.REFERENCE_EXAMPLES[name]
        if name == "moe":
            spec, ref = W.moe_example(8, 1024)
        if name == "tb_matmul_test":
            spec, ref = W.tiled_matmul(512, 512, 256, (8, 8, 1), 4, (0, -1, -1), (-1, 1, -1), (0, 1, -1))
        ins = None
        if random_inputs:
            ins = {i: uniform_fp(op["dims"], 100 + i) for i, op in enumerate(spec) if op["op"] == "input"}
        got = _graph_fp(rt, spec, ins)
        want = orc.eval_graph(spec, "fp", ins, threads=8)
        for i, op in enumerate(spec):
            for j, w in enumerate(want[i]):
                assert np.array_equal(got[i][j], w), (name, i, j, op["op"])
        got_ref = _graph_fp(rt, ref, ins)
        assert np.array_equal(got_ref[-1][0], got[-1][0]), f"{name}: mugraph != un-fused graph on the GPU"


def test_reference_examples_iota_inputs(rt):
    """The reference's own integration checks (cpp_examples/*.cc: has_same_fingerprint of
    the hand-written mugraph and the un-fused graph), inputs idx % 25651 as there."""
    _check_examples(rt, ["group_query_attn_inc_decode", "group_query_attn_spec_decode",
                         "multi_head_attn_inc_decode", "multi_head_attn_prefill",
                         "multi_query_attn_inc_decode", "multi_query_attn_spec_decode",
                         "lora", "mlp", "moe", "tb_matmul_test", "dnn"], False)


def test_reference_examples_random_inputs(rt):
    _check_examples(rt, ["group_query_attn_inc_decode", "group_query_attn_prefill",
                         "multi_head_attn_spec_decode", "lora", "mlp", "moe", "tb_matmul_test"], True)


def test_gqa_fixture_graphs(rt):
    """Every one of the 69 graphs the reference's search verified must fingerprint-equal
    the computation graph, on the GPU, and match the oracle bit for bit."""
    fx = load_gqa_fixture()
    ref_spec = fx["computation_graph"]
    want = orc.eval_graph(ref_spec, "fp")[-1][0]
    got_ref = _graph_fp(rt, ref_spec)[-1][0]
    assert np.array_equal(got_ref, want)
    for gi, spec in enumerate(fx["generated_graphs"]):
        got = _graph_fp(rt, spec)[-1][0]
        assert np.array_equal(got, want), f"fixture graph {gi}"


def test_baseline_configs_fingerprint(rt):
    from attention_superoptimizer_amd import workloads as W
    cases = {
        "C1": W.config1_fused_matmul(),
        "C2": W.config2_gqa_decode(),
        "C3s": W.config3_mha_prefill(heads=2, seq=512, hd=128, q_split=4, kv_split=2, F=4),
        "C4": W.config4_lora(),
        "C5s": W.config5_gated_mlp(m=8, d=1024, h=3584, grid1=56, F1=4, grid2=16, F2=14),
    }
    for name, (spec, ref) in cases.items():
        ins = {i: uniform_fp(op["dims"], 7 + i) for i, op in enumerate(spec) if op["op"] == "input"}
        got = _graph_fp(rt, spec, ins)
        want = orc.eval_graph(spec, "fp", ins, threads=8)
        for i in range(len(spec)):
            for j, w in enumerate(want[i]):
                assert np.array_equal(got[i][j], w), (name, i, j)
        if ref is not None:
            got_ref = _graph_fp(rt, ref, ins)
            assert np.array_equal(got_ref[-1][0], got[-1][0]), name


def test_customized_fp_batch_matches_single_launches(rt, abi):
    """mi355_customized_fp_batch over several independent plans = one mi355_customized_fp
    each, bit for bit."""
    from attention_superoptimizer_amd import _native as N
    from attention_superoptimizer_amd import workloads as W
    specs = [W.tiled_matmul(128, 256, 256, (4, 2, 1), 4, (-1, 0, -1), (1, -1, -1), (1, 0, -1))[0],
             W.tiled_matmul(64, 64, 512, (1, 1, 1), 8, (-1, -1, -1), (-1, -1, -1), (-1, -1, -1))[0],
             W.config1_fused_matmul()[0], W.config2_gqa_decode()[0]]
    built, plans, ins, outs, want = [], (N.Mi355Plan * len(specs))(), [], [], []
    try:
        for k, spec in enumerate(specs):
            g, vals = rt.build_from_spec(spec)
            built.append(g)
            idx = len(spec) - 1
            for i, op in enumerate(spec):
                if op["op"] == "input":
                    vals[i][0].write_fingerprint(uniform_fp(op["dims"], 500 + 10 * k + i))
            g.fingerprint(idx)
            want.append([t.read_fingerprint() for t in vals[idx]])
            for t in vals[idx]:
                t.write_fingerprint(np.zeros(t.dims, np.uint16))
            plans[k] = g.lowered(idx, True)
            row_in = [vals[a][b].device_ptr(True) for a, b in spec[idx]["in"]]
            row_out = [t.device_ptr(True) for t in vals[idx]]
            ins += row_in + [0] * (4 - len(row_in))
            outs += row_out + [0] * (4 - len(row_out))
            built[-1]._vals = vals
        i_p = (ctypes.c_void_p * len(ins))(*ins)
        o_p = (ctypes.c_void_p * len(outs))(*outs)
        assert abi.mi355_customized_fp_batch(plans, len(specs), i_p, o_p) == 0, N.last_error()
        assert abi.mi355_sync() == 0
        for k, spec in enumerate(specs):
            got = [t.read_fingerprint() for t in built[k]._vals[len(spec) - 1]]
            for a, b in zip(got, want[k]):
                assert np.array_equal(a, b), k
    finally:
        for g in reversed(built):
            g.close()


def test_full_size_configs_equal_their_unfused_graphs(rt):
    """At the benchmark's full sizes the oracle is too slow to be the checker; the
    size-independent property is the one the reference's search relies on: a mugraph and the
    un-fused kernel graph it rewrites have the same fingerprint.  The un-fused side runs
    on the kernel-level fingerprint operators, code the customized-op interpreter shares
    nothing with.  Both input conventions: uniform values and the reference's idx % 25651."""
    from attention_superoptimizer_amd import workloads as W
    for name in ("C1_fused_matmul", "C3_mha_prefill", "C4_lora", "C5a_gated_mlp"):
        spec, ref = W.BASELINE_CONFIGS[name]()
        assert ref is not None
        for seed in (0, 0xC0FFEE):
            g, _ = rt.build_from_spec(spec)
            r, _ = rt.build_from_spec(ref)
            try:
                r.fingerprint_seeded(seed)
                verdicts, _ = rt.verify_batch([g], r, seed)
                assert verdicts == [True], (name, seed)
            finally:
                r.close()
                g.close()
