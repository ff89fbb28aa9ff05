"""Pins the CPU oracle before anything is checked against it (no GPU needed).

The reference holds no numeric golden outputs for this path; what it does hold is
(a) 69 mugraphs its own search verified fingerprint-equal to a computation graph
(demo/checkpoint_group_query_attn_spec_decode.json, trimmed into tests/golden/) and
(b) 13 hand-written plans asserted fingerprint-equal to their un-fused graphs
(cpp_examples/*.cc).  Those, closed forms, the ring homomorphism and an independent
numpy statement of the semantics pin the C restatement."""
import numpy as np
import pytest

from helpers import FP_PQ, load_gqa_fixture, normal_f16, uniform_fp
from oracle import evaluate as orc
from oracle import lowering, np_semantics as nps
from attention_superoptimizer_amd import workloads as W


# ---- tables and constants: closed forms --------------------------------------
def test_constants_crt():
    assert 227 * 113 == FP_PQ
    assert 227 % 113 == 1 and 227 % 227 == 0           # FP_P_MUL_Q_MOD_1
    assert 25425 % 227 == 1 and 25425 % 113 == 0       # FP_Q_MUL_P_MOD_1


def test_tables_closed_forms():
    e, p, q = orc.tables()
    assert list(e[:8]) == [1, 3, 9, 27, 81, 16, 48, 144]
    assert all(int(e[i]) == pow(3, i, 227) for i in range(113))
    assert pow(3, 113, 227) == 1 and all(pow(3, d, 227) != 1 for d in range(1, 113))
    assert p[0] == 1 and p[1] == 1 and q[0] == 1 and q[1] == 1
    assert all(int(p[i]) == pow(i, 225, 227) for i in range(1, 227))  # Fermat inverse
    assert all(int(q[i]) == pow(i, 111, 113) for i in range(1, 113))
    assert all((i * int(p[i])) % 227 == 1 for i in range(1, 227))


def test_input_is_iota():
    a = orc.fp_input([3, 5, 9000])
    assert np.array_equal(a.ravel(), np.arange(a.size) % FP_PQ)


# ---- ring homomorphism: result == exact integer arithmetic mod 25651 ----------
def test_matmul_is_exact_mod_pq():
    rng = np.random.default_rng(1)
    A = rng.integers(0, FP_PQ, size=(2, 7, 300)).astype(np.uint16)
    B = rng.integers(0, FP_PQ, size=(2, 300, 5)).astype(np.uint16)
    exact = np.array([[[sum(int(A[b, i, k]) * int(B[b, k, j]) for k in range(300)) % FP_PQ
                        for j in range(5)] for i in range(7)] for b in range(2)])
    assert np.array_equal(orc.fp_matmul(A, B), exact)
    # worst case: every product is 25650^2 and k is long
    A = np.full((1, 2, 5000), FP_PQ - 1, np.uint16)
    B = np.full((1, 5000, 3), FP_PQ - 1, np.uint16)
    assert np.all(orc.fp_matmul(A, B) == (5000 * (FP_PQ - 1) ** 2) % FP_PQ)


def test_signed_byte_residue_planes_reproduce_the_matmul():
    """The arithmetic the matrix-core fingerprint kernels rely on, restated in numpy: operands
    split into signed bytes (mod 227 recentred to [-113, 113], mod 113 as it is), exact int32
    dot products per field, and ONE recombination `(u * 25425 + v * 227) mod 25651` of the
    unreduced sums u (made non-negative by adding 83715 * 25651) and v equal the oracle's
    `(r + a*b) % 25651` chain; so does exp taken from the mod-113 sum alone."""
    rng = np.random.default_rng(7)
    A = rng.integers(0, FP_PQ, size=(1, 9, 4096)).astype(np.uint16)
    B = rng.integers(0, FP_PQ, size=(1, 4096, 6)).astype(np.uint16)
    A[0, 0, :] = (114 * 25425 + 112 * 227) % FP_PQ   # -113 mod 227, 112 mod 113: extreme bytes
    B[0, :, 0] = (113 * 25425 + 112 * 227) % FP_PQ

    def planes(X):
        p = X.astype(np.int64) % 227
        p = np.where(p > 113, p - 227, p)
        q = X.astype(np.int64) % 113
        assert p.min() >= -113 and p.max() <= 113 and q.max() <= 112
        return p, q

    (ap, aq), (bp, bq) = planes(A), planes(B)
    u, v = ap @ bp, aq @ bq
    assert np.abs(u).max() < 2 ** 31 - 2 ** 17 and v.min() >= 0 and v.max() < 2 ** 31
    offset = 83715 * FP_PQ
    assert offset == 2147373465 and offset < 2 ** 31
    a = (u + offset) % FP_PQ
    b = v % FP_PQ
    assert (a * 25425 + b * 227).max() < 2 ** 32
    z = (a * 25425 + b * 227) % FP_PQ
    want = orc.fp_matmul(A, B)
    assert np.array_equal(z, want)
    exp_tbl = np.asarray(orc.tables()[0], np.int64)
    lifted = (exp_tbl[:113] * 25425) % FP_PQ
    assert np.array_equal(lifted[v % 113], orc.fp_unary("exp", want))


def test_add_mul_broadcast_exhaustive_small():
    """every broadcast pattern of <=3 dims of size <=3 against numpy broadcasting"""
    rng = np.random.default_rng(2)
    for nd in (1, 2, 3):
        for full in np.ndindex(*([3] * nd)):
            shape = [s + 1 for s in full]
            for mask1 in np.ndindex(*([2] * nd)):
                for mask2 in np.ndindex(*([2] * nd)):
                    s1 = [d if m else 1 for d, m in zip(shape, mask1)]
                    s2 = [d if m else 1 for d, m in zip(shape, mask2)]
                    x = rng.integers(0, FP_PQ, size=s1).astype(np.uint16)
                    y = rng.integers(0, FP_PQ, size=s2).astype(np.uint16)
                    xi, yi = x.astype(np.int64), y.astype(np.int64)
                    assert np.array_equal(orc.fp_binary("add", x, y), (xi + yi) % FP_PQ)
                    assert np.array_equal(orc.fp_binary("mul", x, y), (xi * yi) % FP_PQ)


def test_reduction_three_statements_agree():
    """reduction_kernel.cu's stride rule == reshape/sum (the Triton generator's
    statement) == the thread-block flat rule, for every dim and group size"""
    x = uniform_fp((4, 6, 24), 3)
    xi = x.astype(np.int64)
    for dim in range(3):
        for size in (1, 2, x.shape[dim]):
            want = orc.strided_reduce(xi, dim, size) % FP_PQ
            assert np.array_equal(orc.fp_reduce(x, dim, size), want)
    # group size 2 along the last dim: out[..., j] = in[..., j] + in[..., j+2] + ...
    got = orc.fp_reduce(x, 2, 2)
    assert np.array_equal(got[..., 0], xi[..., 0::2].sum(-1) % FP_PQ)


# ---- exp / div: identities of the reference's conventions ---------------------
def test_exp_is_homomorphism_lifted_by_crt():
    x = np.arange(FP_PQ, dtype=np.uint16)
    e = orc.fp_unary("exp", x).astype(np.int64)
    assert np.all(e % 113 == 0)                                  # lifted to 0 mod 113
    assert np.array_equal(e % 227, np.array([pow(3, int(v) % 113, 227) for v in x]))
    a, b = uniform_fp((1000,), 5), uniform_fp((1000,), 6)
    s = ((a.astype(np.int64) + b) % FP_PQ).astype(np.uint16)
    prod = orc.fp_binary("mul", orc.fp_unary("exp", a), orc.fp_unary("exp", b)).astype(np.int64)
    # exp(a)*exp(b) and exp(a+b) agree mod 227 whenever a+b did not wrap mod 25651
    nowrap = (a.astype(np.int64) + b) < FP_PQ
    assert np.array_equal(prod[nowrap] % 227, orc.fp_unary("exp", s).astype(np.int64)[nowrap] % 227)


def test_div_inverts_mul_and_zero_convention():
    x, y = uniform_fp((4000,), 7), uniform_fp((4000,), 8)
    inv = (y % 227 != 0) & (y % 113 != 0)
    back = orc.fp_binary("div", orc.fp_binary("mul", x, y), y)
    assert np.array_equal(back[inv], x[inv])
    # residues that are 0 map to inverse 1: dividing by 0 returns x
    z = np.zeros_like(x)
    assert np.array_equal(orc.fp_binary("div", x, z), x)
    assert np.array_equal(orc.fp_binary("div", x, np.ones_like(x)), x)


# ---- silu (an extension of this backend; the reference has no such operator) -------
def _silu_closed_form(x: int) -> int:
    """silu(x) = x / (1 + exp(-x)) residue by residue, in Python integers.  exp lifts to 0
    mod 113, so the denominator is 1 mod 113 and the mod-113 residue of x passes through;
    mod 227 the denominator is 1 + 3^((-x) mod 113), never 0 (see the test below)."""
    neg = (FP_PQ - x) % FP_PQ
    den = (1 + pow(3, neg % 113, 227)) % 227
    inv = pow(den, 225, 227)
    sp, sq = (x % 227) * inv % 227, x % 113
    return (sp * 25425 + sq * 227) % FP_PQ


def test_silu_closed_form_and_invariants():
    x = np.arange(FP_PQ, dtype=np.uint16)
    s = orc.fp_unary("silu", x)
    assert np.array_equal(s, np.array([_silu_closed_form(int(v)) for v in x]))
    assert s[0] == 0
    # the same value through the PUBLIC primitives: div(x, add(1, exp(neg x)))
    neg = ((FP_PQ - x.astype(np.int64)) % FP_PQ).astype(np.uint16)
    den = orc.fp_binary("add", np.ones_like(x), orc.fp_unary("exp", neg))
    assert np.array_equal(s, orc.fp_binary("div", x, den))
    # the denominator is invertible for EVERY x: it is 1 mod 113, and 1 + 3^k = 0 mod 227 would
    # put -1 into the subgroup generated by 3, whose order 113 is odd.  So silu(x) * (1 +
    # exp(-x)) == x with no exception, and the zero-divisor convention of div never applies.
    assert np.all(den % 113 == 1) and np.all(den % 227 != 0)
    assert np.array_equal(orc.fp_binary("mul", s, den), x)
    assert np.array_equal(s.astype(np.int64) % 113, x.astype(np.int64) % 113)
    # mistakes this catches: exp(x) for exp(-x), a dropped "1 +", mul for div
    wrong_sign = orc.fp_binary("div", x, orc.fp_binary("add", np.ones_like(x), orc.fp_unary("exp", x)))
    no_one = orc.fp_binary("div", x, orc.fp_unary("exp", neg))
    assert not np.array_equal(s, wrong_sign) and not np.array_equal(s, no_one)


# ---- thread-block add / mul (extensions: the reference's lowering asserts on them) ----
def tb_add_mul_case():
    """A customized op built from thread-block add and mul with every broadcast a 3-D tile
    admits ([1,r,c] with [1,r,1], with [1,1,c], [1,r,1] with [1,1,c], small operand first),
    over two blocks and a two-iteration for-loop.  119 program ints."""
    spec = [
        {"op": "input", "dims": [2, 8, 12]}, {"op": "input", "dims": [2, 8, 12]},
        {"op": "customized", "in": [[0, 0], [1, 0]], "plan": {
            "grid_dim": [2, 1, 1], "forloop_range": 2, "reduction_dimx": 4,
            "input_map": [[0, -1, -1], [0, -1, -1]], "forloop_dim": [2, 2],
            "output_map": [0, -1, -1],
            "ops": [["tb_reduction_2_op", [[0, 0]]],            # 2: [1,8,1]
                    ["tb_reduction_1_op", [[1, 0]]],            # 3: [1,1,6]
                    ["tb_add_op", [[0, 0], [2, 0]]],            # 4: [1,8,6] + [1,8,1]
                    ["tb_mul_op", [[4, 0], [3, 0]]],            # 5: [1,8,6] * [1,1,6]
                    ["tb_add_op", [[2, 0], [3, 0]]],            # 6: [1,8,1] + [1,1,6]
                    ["tb_mul_op", [[5, 0], [6, 0]]],            # 7
                    ["tb_mul_op", [[3, 0], [2, 0]]],            # 8: [1,1,6] * [1,8,1]
                    ["tb_add_op", [[7, 0], [8, 0]]]]}},         # 9
    ]
    return spec


def tb_add_mul_exact(A, B):
    """The same computation in Python integers of unbounded size, one modulus at the end."""
    A, B = A.astype(object), B.astype(object)
    out = np.zeros((2, 8, 6), object)
    for b in range(2):
        for it in range(2):
            a, bb = A[b][:, it * 6:(it + 1) * 6], B[b][:, it * 6:(it + 1) * 6]
            r2 = a.sum(axis=1).reshape(8, 1)
            r1 = bb.sum(axis=0).reshape(1, 6)
            out[b] = out[b] + ((a + r2) * r1) * (r2 + r1) + r1 * r2
    return (out % FP_PQ).astype(np.uint16)


def test_threadblock_add_mul_exact_integers():
    spec = tb_add_mul_case()
    for seed in (1, 2):
        A, B = uniform_fp([2, 8, 12], seed), uniform_fp([2, 8, 12], seed + 10)
        got = orc.eval_graph(spec, "fp", {0: A, 1: B})[2]
        assert len(got) == 1 and got[0].shape == (2, 8, 6)
        assert np.array_equal(got[0], tb_add_mul_exact(A, B))
    # worst-case operands: every intermediate product is as large as the ring allows
    A = np.full((2, 8, 12), FP_PQ - 1, np.uint16)
    assert np.array_equal(orc.eval_graph(spec, "fp", {0: A, 1: A})[2][0], tb_add_mul_exact(A, A))
    # an operand swap or add-for-mul changes the answer (the check can fail)
    bad = tb_add_mul_case()
    bad[2]["plan"]["ops"][3][0] = "tb_add_op"
    A, B = uniform_fp([2, 8, 12], 1), uniform_fp([2, 8, 12], 11)
    assert not np.array_equal(orc.eval_graph(bad, "fp", {0: A, 1: B})[2][0], tb_add_mul_exact(A, B))


def test_block_subset_reproduces_those_blocks():
    """customized(blocks=...) runs the listed thread blocks only: their tiles equal the
    whole-grid run, everything else is left untouched"""
    spec, _ = W.config2_gqa_decode()
    ins = [uniform_fp(spec[i]["dims"], 60 + i) for i in range(3)]
    full = orc.customized(spec[3]["plan"], ins, threads=8)[0]
    part = orc.customized(spec[3]["plan"], ins, threads=2, blocks=[1, 6, 31])[0]
    m = orc.written(part)
    assert m.sum() == 3 * 256 * 64 and np.array_equal(part[m], full[m])
    assert m[1, :, 0:64].all() and m[0, :, 3 * 64:4 * 64].all() and m[1, :, 15 * 64:].all()


# ---- the interpreter ------------------------------------------------------------
def test_degenerate_plan_equals_kernel_ops():
    """grid (1,1,1), for-loop 1: a customized op is its kernel-level ops"""
    spec = [
        {"op": "input", "dims": [1, 16, 32]}, {"op": "input", "dims": [1, 32, 24]},
        {"op": "customized", "in": [[0, 0], [1, 0]], "plan": {
            "grid_dim": [1, 1, 1], "forloop_range": 1, "reduction_dimx": 8,
            "input_map": [[-1, -1, -1], [-1, -1, -1]], "forloop_dim": [-1, -1],
            "output_map": [-1, -1, -1],
            "ops": [["tb_matmul_op", [[0, 0], [1, 0]]], ["tb_exp_op", [[2, 0]]],
                    ["tb_reduction_2_op", [[3, 0]]], ["tb_div_op", [[3, 0], [4, 0]]],
                    ["tb_reduction_2_to_dimx_op", [[5, 0]]]]}},
    ]
    ins = {0: uniform_fp([1, 16, 32], 1), 1: uniform_fp([1, 32, 24], 2)}
    got = orc.eval_graph(spec, "fp", ins)[2]
    m = orc.fp_matmul(ins[0], ins[1])
    e = orc.fp_unary("exp", m)
    d = orc.fp_binary("div", e, orc.fp_reduce(e, 2, 1))
    assert len(got) == 1 and np.array_equal(got[0], orc.fp_reduce(d, 2, 8))


@pytest.mark.parametrize("name", sorted(W.REFERENCE_EXAMPLES))
def test_reference_example_equivalences(name):
    """cpp_examples/*.cc end with assert(ref.has_same_fingerprint(mugraph)), inputs idx % 25651"""
    spec, ref = W.REFERENCE_EXAMPLES[name]
    if name == "moe":
        spec, ref = W.moe_example(8, 1024)
    if name == "tb_matmul_test":
        spec, ref = W.tiled_matmul(256, 256, 256, (4, 4, 1), 4, (0, -1, -1), (-1, 1, -1), (0, 1, -1))
    a = orc.eval_graph(spec, "fp", threads=8)[-1][0]
    b = orc.eval_graph(ref, "fp")[-1][0]
    assert a.shape == b.shape and np.array_equal(a, b)


def test_gqa_fixture_all_69_graphs():
    fx = load_gqa_fixture()
    assert fx["num_valid_kernel_graphs"] == 69 == len(fx["generated_graphs"])
    want = orc.eval_graph(fx["computation_graph"], "fp")[-1][0]
    for gi, spec in enumerate(fx["generated_graphs"]):
        vals = orc.eval_graph(spec, "fp", threads=8)
        assert np.array_equal(vals[-1][0], want), f"fixture graph {gi}"
        for i, op in enumerate(spec):
            assert [list(v.shape) for v in vals[i]] == op["out_dims"]
            if op["op"] == "customized":   # shared-memory accounting matches the recorded bgraph
                tg = lowering.build_tb_graph(op["plan"], [list(vals[a][b].shape) for a, b in op["in"]])
                assert tg.smem_offset == op["smem_offset"]


def test_c_interpreter_agrees_with_numpy_semantics():
    """mechanism (flat program, strides, offsets) vs meaning (array slices), fp and f16"""
    cases = [W.config1_fused_matmul()[0], W.config2_gqa_decode()[0],
             W.REFERENCE_EXAMPLES["lora"][0], W.REFERENCE_EXAMPLES["mlp"][0],
             W.REFERENCE_EXAMPLES["group_query_attn_spec_decode"][0],
             W.config5_gated_mlp(m=8, d=256, h=512, grid1=8, F1=4, grid2=4, F2=4)[0]]
    for spec in cases:
        ins = {i: uniform_fp(op["dims"], 40 + i) for i, op in enumerate(spec) if op["op"] == "input"}
        vals = orc.eval_graph(spec, "fp", ins, threads=8)
        for i, op in enumerate(spec):
            if op["op"] == "customized":
                got = nps.customized(op["plan"], [vals[a][b] for a, b in op["in"]])
                for x, y in zip(got, vals[i]):
                    assert np.array_equal(x, y)
    spec = W.config2_gqa_decode()[0]
    ins = {i: normal_f16(op["dims"], 0.125, i) for i, op in enumerate(spec) if op["op"] == "input"}
    a = orc.eval_graph(spec, "f16", ins, threads=8)[3][0]
    b = nps.customized(spec[3]["plan"], [ins[0], ins[1], ins[2]], f16=True)[0]
    # same semantics, different fp32 summation order inside matmuls: a few fp16 ulps
    assert np.allclose(a.astype(np.float32), b.astype(np.float32), rtol=4e-3, atol=2e-4)


def test_partition_invariance():
    """a linear plan gives the same result under different grid / for-loop factorisations"""
    outs = []
    for grid, F in [((16, 1, 1), 16), ((4, 1, 1), 64), ((64, 1, 1), 2), ((1, 1, 1), 1)]:
        spec, _ = W.tiled_matmul(64, 1024, 256, grid, F, (-1, -1, -1), (1, -1, -1), (1, -1, -1))
        outs.append(orc.eval_graph(spec, "fp", threads=8)[-1][0])
    assert all(np.array_equal(outs[0], o) for o in outs[1:])


# ---- fp16 golden: textbook special cases ----------------------------------------
def test_f16_conversions_bit_exact():
    bits = np.arange(65536, dtype=np.uint16)
    f = np.zeros(65536, np.float32)
    orc.lib().orc_f16_to_f32(orc._p(bits), orc._p(f), bits.size)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32), ref.view(np.uint32))
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * s
                        for s in (1e-8, 1e-5, 1e-3, 1.0, 100.0, 7e4)])
    h = np.zeros(x.size, np.uint16)
    orc.lib().orc_f32_to_f16(orc._p(x), orc._p(h), x.size)
    with np.errstate(over="ignore"):
        assert np.array_equal(h, x.astype(np.float16).view(np.uint16))


def test_f16_golden_gemm_and_attention():
    spec, _ = W.config1_fused_matmul()
    ins = {0: normal_f16([64, 1024], 0.1, 1), 1: normal_f16([1024, 1024], 0.1, 2)}
    got = orc.eval_graph(spec, "f16", ins, threads=8)[2][0].astype(np.float64)
    exact = ins[0].astype(np.float64) @ ins[1].astype(np.float64)
    assert np.max(np.abs(got - exact)) < 4e-3      # 16 fp16-rounded partial sums of size ~0.3
    spec, ref = W.config3_mha_prefill(heads=1, seq=256, hd=128, q_split=2, kv_split=2, F=2)
    ins = {i: normal_f16(spec[i]["dims"], 128 ** -0.5, 10 + i) for i in range(3)}
    got = orc.eval_graph(spec, "f16", ins, threads=8)[-1][0].astype(np.float64)
    Q, K, V = (ins[i].astype(np.float64) for i in range(3))
    s = Q @ K
    p = np.exp(s - s.max(-1, keepdims=True))
    att = (p / p.sum(-1, keepdims=True)) @ V
    assert np.max(np.abs(got - att)) < 2e-3
