"""Host-side logic of the product without a GPU: graph construction through the
mirage:: API (host-only runtime), lowering against the oracle's restatement, the
soft-failure contract, the LIFO arena, and the C ABI's symbols."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from helpers import load_gqa_fixture
from oracle import lowering
from attention_superoptimizer_amd import _native as N
from attention_superoptimizer_amd import graph as G
from attention_superoptimizer_amd import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(autouse=True)
def _budget():
    G.set_smem_budget(1 << 20)
    yield
    G.set_smem_budget(96 * 1024)


def _compare_lowering(spec):
    g, vals = G.build_from_spec(spec)
    try:
        for i, op in enumerate(spec):
            if op["op"] != "customized":
                continue
            p = g.lowered(i, True)
            ins = [vals[a][b] for a, b in op["in"]]
            tg = lowering.build_tb_graph(op["plan"], [list(t.dims) for t in ins],
                                         [t.layout for t in ins], 1 << 20)
            types, params = lowering.lower(tg)
            assert list(p.operator_types[:p.num_operators]) == types
            assert list(p.parameters[:p.num_parameters]) == params
            assert p.smem_bytes == tg.smem_offset
            assert [list(t.dims) for t in vals[i]] == lowering.output_dims(tg)
            assert list(p.grid_dim) == op["plan"]["grid_dim"]
            assert p.forloop_range == op["plan"]["forloop_range"]
    finally:
        g.close()


@pytest.mark.parametrize("name", sorted(W.REFERENCE_EXAMPLES))
def test_lowering_matches_oracle_examples(name):
    _compare_lowering(W.REFERENCE_EXAMPLES[name][0])


@pytest.mark.parametrize("name", sorted(W.BASELINE_CONFIGS))
def test_lowering_matches_oracle_configs(name):
    _compare_lowering(W.BASELINE_CONFIGS[name]()[0])


def test_lowering_matches_fixture_graphs():
    fx = load_gqa_fixture()
    for spec in fx["generated_graphs"]:
        g, vals = G.build_from_spec(spec)
        try:
            for i, op in enumerate(spec):
                assert [list(t.dims) for t in vals[i]] == op["out_dims"]
                if op["op"] == "customized":   # the reference recorded its own smem_offset
                    assert g.lowered(i, True).smem_bytes == op["smem_offset"]
        finally:
            g.close()
    _compare_lowering(fx["generated_graphs"][0])


def test_program_sizes_quoted_for_the_reference_plans():
    """GQA single-op plan = 3*19+6+2+5+9+6+17 = 102 ints; LoRA = 4*19+6+7+7+6+17 = 119"""
    g, _ = G.build_from_spec(W.config2_gqa_decode()[0])
    assert g.lowered(3).num_parameters == 102
    g.close()
    g, _ = G.build_from_spec(W.REFERENCE_EXAMPLES["lora"][0])
    assert g.lowered(4).num_parameters == 119
    g.close()


def test_shape_inference_and_soft_failures():
    g = G.KNGraph()
    try:
        A = g.new_input((2, 8, 16))
        B = g.new_input((2, 16, 4))
        C = g.matmul(A, B)
        assert C.dims == (2, 8, 4) and C.layout == 100          # outputs are row-major
        assert g.reduction(C, 2).dims == (2, 8, 1)
        assert g.reduction(C, 1, 4).dims == (2, 4, 4)
        S = g.new_input((2, 8, 1))
        assert g.div(C, S).dims == (2, 8, 4)
        n = g.num_operators
        with pytest.raises(G.InfeasibleOperator):
            g.matmul(A, C)                                       # inner dims differ
        with pytest.raises(G.InfeasibleOperator):
            g.matmul(A, g.new_input((3, 16, 4)))                 # batch dims differ
        with pytest.raises(G.InfeasibleOperator):
            g.add(C, g.new_input((2, 8, 3)))                     # not broadcastable
        with pytest.raises(G.InfeasibleOperator):
            g.reduction(C, 3)                                    # dim out of range
        with pytest.raises(G.InfeasibleOperator):
            g.reduction(C, 2, 3)                                 # 4 % 3 != 0
        assert g.num_operators == n + 2                          # only the two inputs were added
    finally:
        g.close()


def test_arena_is_lifo_and_bounded():
    rt = N.runtime()
    base = rt.mirage_arena_offset()
    g = G.KNGraph()
    A = g.new_input((4, 100, 33))
    nbytes = (4 * 100 * 33 * 2 + 15) // 16 * 16
    assert rt.mirage_arena_offset() == base + 2 * nbytes         # data + fingerprint buffers
    assert A.device_ptr(True) - A.device_ptr(False) == nbytes
    g.exp(A)
    assert rt.mirage_arena_offset() == base + 4 * nbytes
    g.pop_operator()
    assert rt.mirage_arena_offset() == base + 2 * nbytes
    with pytest.raises(G.InfeasibleOperator):                    # larger than the whole arena
        g.new_input((1 << 15, 1 << 15, 1 << 5))
    g.close()
    assert rt.mirage_arena_offset() == base


def test_smem_budget_is_enforced_by_default():
    """the reference's 96 KB cap: config C2 does not fit it, the spec-decode example does"""
    G.set_smem_budget(96 * 1024)
    g, _ = G.build_from_spec(W.REFERENCE_EXAMPLES["group_query_attn_spec_decode"][0])
    g.close()
    code = ("import os; os.environ['MIRAGE_HOST_ONLY']='1'\n"
            "from attention_superoptimizer_amd import graph as G, workloads as W\n"
            "G.build_from_spec(W.config2_gqa_decode()[0])\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert r.returncode != 0 and "infeasible" in r.stderr


def test_device_work_fails_loudly_without_a_gpu():
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    code = ("import os; os.environ['MIRAGE_HOST_ONLY']='1'\n"
            "from attention_superoptimizer_amd import graph as G\n"
            "g=G.KNGraph(); A=g.new_input((4,4)); g.fingerprint(0)\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert r.returncode != 0 and "host-only" in r.stderr
    # the two-call verification hands work to threads: it must refuse before starting any
    code = ("import os; os.environ['MIRAGE_HOST_ONLY']='1'\n"
            "from attention_superoptimizer_amd import graph as G\n"
            "g=G.KNGraph(); A=g.new_input((4,4)); r=G.KNGraph(); r.new_input((4,4))\n"
            "G.verify_batch_begin([g], r, 1)\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert r.returncode != 0 and "host-only" in r.stderr
    code = ("import os; os.environ.pop('MIRAGE_HOST_ONLY', None)\n"
            "from attention_superoptimizer_amd import graph as G\n"
            "g=G.KNGraph(); g.new_input((4,4))\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True,
                       env={k: v for k, v in os.environ.items() if k != "MIRAGE_HOST_ONLY"})
    assert r.returncode != 0 and "cannot initialise the MI355X backend" in r.stderr


def test_abi_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mi355_abi.h")).read()
    declared = set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = N.backend()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared but not exported"
    assert declared == set(N.ABI), (declared ^ set(N.ABI))
    # no compute without a device: entry points refuse instead of crashing
    if not os.path.exists("/dev/kfd"):
        assert lib.mi355_is_initialised() == 0
        assert lib.mi355_sync() == -5
        assert b"mi355_init" in lib.mi355_last_error()


def test_plan_extents_and_validation():
    ab = N.backend()
    g, vals = G.build_from_spec(W.config1_fused_matmul()[0])
    p = g.lowered(2, True)
    ie, oe = (ctypes.c_longlong * 4)(), (ctypes.c_longlong * 4)()
    l1, l2 = ctypes.c_int(), ctypes.c_int()
    assert ab.mi355_plan_extents(ctypes.byref(p), ie, oe, ctypes.byref(l1), ctypes.byref(l2)) == 0
    assert list(ie[:2]) == [64 * 1024, 1024 * 1024] and oe[0] == 64 * 1024
    assert 0 < l1.value <= 160 * 1024 and 0 < l2.value <= 160 * 1024
    p.parameters[13] = 512                       # claim the A matrix has 512 columns
    assert ab.mi355_plan_extents(ctypes.byref(p), ie, oe, None, None) == -3
    assert b"walks outside" in ab.mi355_last_error()
    p = g.lowered(2, True)
    p.num_parameters -= 1
    assert ab.mi355_plan_extents(ctypes.byref(p), ie, oe, None, None) == -3
    p = g.lowered(2, True)
    p.operator_types[2] = 2050
    assert ab.mi355_plan_extents(ctypes.byref(p), ie, oe, None, None) == -4
    g.close()


def test_verify_ring_never_hands_out_what_a_live_batch_owns():
    """Compare-slot ranges and mark pairs of verification batches in flight (verify.cc): a new
    batch never overlaps a live one; ranges and marks come back when a batch ends; the 33rd
    batch in flight, or a range no free stretch can hold, is refused."""
    import ctypes
    from attention_superoptimizer_amd import _native as N
    rt = N.runtime()
    ring = ctypes.c_void_p(rt.mirage_verify_ring_create())
    try:
        first, ticket = ctypes.c_int(), ctypes.c_int()
        live = {}

        def acquire(n):
            rc = rt.mirage_verify_ring_acquire(ring, n, ctypes.byref(first), ctypes.byref(ticket))
            if rc != 0:
                return None
            for f, c in live.values():
                assert n == 0 or c == 0 or first.value >= f + c or f >= first.value + n, "overlap"
            assert ticket.value not in live and 0 <= ticket.value < 32
            assert 0 <= first.value and first.value + n <= 65536
            live[ticket.value] = (first.value, n)
            return ticket.value

        def release(t):
            rt.mirage_verify_ring_release(ring, t)
            del live[t]

        # three batches of 30,000 slots: the third does not fit until the first has ended
        a, b = acquire(30000), acquire(30000)
        assert a is not None and b is not None
        assert acquire(30000) is None
        release(a)
        c = acquire(30000)
        assert c is not None and live[c][0] == 0          # wrapped into the freed stretch, not onto b
        assert acquire(10000) is None                     # 5,536 free slots at the end only
        d = acquire(5000)
        assert d is not None and live[d][0] == 60000
        for t in list(live):
            release(t)
        # 32 batches in flight use every mark pair; the 33rd is refused until one ends
        ts = [acquire(16) for _ in range(32)]
        assert None not in ts and len(set(ts)) == 32
        assert acquire(16) is None
        release(ts[7])
        assert acquire(16) == ts[7]
        # long run of begin / end with a few in flight: wraps the ring many times
        for t in list(live):
            release(t)
        import random
        rnd = random.Random(5)
        order = []
        for _ in range(2000):
            if len(order) < 4 or (len(order) < 20 and rnd.random() < 0.5):
                t = acquire(rnd.choice([0, 1, 64, 4096, 9000]))
                if t is not None:
                    order.append(t)
                    continue
            release(order.pop(0))
        assert acquire(65537) is None
    finally:
        rt.mirage_verify_ring_destroy(ring)
