"""GPU parity of batched verification: the verdict and every output fingerprint of
generated candidate mugraphs against the CPU oracle, bit for bit; at full size the
verdicts against what the generator constructed (fused rewrites equal, mutants not)."""
import numpy as np
import pytest

from attention_superoptimizer_amd import candidates as C
from helpers import uniform_fp
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu


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


def _verify_problem(rt, prob):
    """Builds the reference and all candidates, runs one batched verify; returns
    (verdicts, per-candidate lists of output arrays, reference outputs)."""
    ref_g, ref_vals = rt.build_from_spec(prob["reference"])
    graphs = []
    try:
        ref_g.fingerprint_seeded(prob["input_seed"])
        vals = []
        for c in prob["candidates"]:
            g, v = rt.build_from_spec(c["spec"])
            graphs.append(g)
            vals.append(v)
        verdicts, stats = rt.verify_batch(graphs, ref_g, prob["input_seed"])
        outs = [[t.read_fingerprint() for t in _outputs(c["spec"], v)]
                for c, v in zip(prob["candidates"], vals)]
        ref_out = [t.read_fingerprint() for t in _outputs(prob["reference"], ref_vals)]
        assert stats["kernel_ops"] == sum(len(c["spec"]) for c in prob["candidates"])
        return verdicts, outs, ref_out
    finally:
        for g in reversed(graphs):
            g.close()
        ref_g.close()


def test_verify_batch_matches_oracle(rt):
    """Reduced dims (<= 128): every candidate output and verdict equals the oracle's."""
    probs = C.generate(num_problems=8, per_problem=8, max_dim=128)
    for prob in probs:
        verdicts, outs, ref_out = _verify_problem(rt, prob)
        seed = prob["input_seed"]
        want_ref = _outputs(prob["reference"],
                            orc.eval_graph(prob["reference"], "fp", _inputs(prob["reference"], seed),
                                           threads=8))
        assert len(ref_out) == len(want_ref)
        for a, b in zip(ref_out, want_ref):
            assert np.array_equal(a, b), prob["family"]
        for c, verdict, got in zip(prob["candidates"], verdicts, outs):
            want = _outputs(c["spec"], orc.eval_graph(c["spec"], "fp", _inputs(c["spec"], seed),
                                                      threads=8))
            assert len(got) == len(want)
            for a, b in zip(got, want):
                assert np.array_equal(a, b), (prob["family"], c["expect_equal"])
            oracle_verdict = len(want) == len(want_ref) and all(
                a.shape == b.shape and np.array_equal(a, b) for a, b in zip(want_ref, want))
            assert verdict == oracle_verdict == c["expect_equal"]


def test_inputs_read_through_one_tensor_keep_every_graph_right(rt):
    """A batch reads inputs number j of equal element count through the first graph's tensor,
    and a launch splits an operand that several fused matmul plans share into residue planes
    once.  Graphs of one batch whose inputs have the same counts but other shapes, other
    operand roles and other prologues (so: the same bytes seen as [64,128] and as [128,64],
    with and without exp in front) must still each give the oracle's outputs."""
    from attention_superoptimizer_amd import workloads as W

    def matmul_graph(m, k, n, tiles, exp_on_a):
        mt, nt, kt = tiles
        ops = []
        a_ref = (0, 0)
        if exp_on_a:
            ops.append(("tb_exp_op", [(0, 0)]))
            a_ref = (2, 0)
        ops.append(("tb_matmul_op", [a_ref, (1, 0)]))
        gx, gy = n // nt, m // mt
        return [W._inp([m, k]), W._inp([k, n]),
                {"op": "customized", "in": [[0, 0], [1, 0]],
                 "plan": W._plan((gx, gy, 1), k // kt,
                                 [(-1, 0, -1) if gy > 1 else (-1, -1, -1), (1, -1, -1) if gx > 1 else (-1, -1, -1)],
                                 (1, 0), (1 if gx > 1 else -1, 0 if gy > 1 else -1, -1), ops)}]

    # inputs 0 and 1 hold 8192 elements in every graph: [64,128].[128,64] and [128,64].[64,128]
    specs = [matmul_graph(64, 128, 64, (32, 32, 64), False),
             matmul_graph(128, 64, 128, (32, 64, 32), False),
             matmul_graph(64, 128, 64, (16, 32, 32), True),
             matmul_graph(64, 128, 64, (64, 64, 128), False),
             matmul_graph(128, 64, 128, (64, 32, 64), True),
             matmul_graph(64, 128, 64, (32, 32, 64), True),
             matmul_graph(128, 64, 128, (128, 128, 64), False),
             matmul_graph(64, 128, 64, (16, 64, 16), False)]
    seed = 0x5A5A0001
    ref_g, _ = rt.build_from_spec(specs[0])
    built = [rt.build_from_spec(sp) for sp in specs]
    try:
        ref_g.fingerprint_seeded(seed)
        verdicts, _ = rt.verify_batch([g for g, _ in built], ref_g, seed)
        want_ref = _outputs(specs[0], orc.eval_graph(specs[0], "fp", _inputs(specs[0], seed), threads=8))[0]
        for k, (sp, (_, vals)) in enumerate(zip(specs, built)):
            want = _outputs(sp, orc.eval_graph(sp, "fp", _inputs(sp, seed), threads=8))
            got = [t.read_fingerprint() for t in _outputs(sp, vals)]
            assert len(got) == len(want) == 1
            assert np.array_equal(got[0], want[0]), k
            assert verdicts[k] == (want[0].shape == want_ref.shape and np.array_equal(want[0], want_ref)), k
        # the same product under other tiles is equal; other shapes and exp in front are not
        assert verdicts == [True, False, False, True, False, False, False, True]
    finally:
        for g, _ in reversed(built):
            g.close()
        ref_g.close()


def test_verify_batch_full_size_verdicts(rt):
    """Full dims ([64, 1024]): rewrites verify equal, mutants unequal."""
    probs = C.generate(num_problems=8, per_problem=16, seed=0xBEEF)
    for prob in probs:
        verdicts, _, _ = _verify_problem(rt, prob)
        assert verdicts == [c["expect_equal"] for c in prob["candidates"]], prob["family"]


def test_the_whole_benchmark_batch_verifies_as_constructed(rt):
    """The batch the fingerprint benchmark times -- 64 problems of 64 candidates at full dims,
    4096 candidate mugraphs -- through the same batched verify: every verdict is the one the
    generator constructed (a fused rewrite equals its reference, a mutant does not), and for
    every eighth candidate each output fingerprint and the verdict equal the oracle's."""
    probs = C.generate(num_problems=64, per_problem=64)
    assert sum(len(p["candidates"]) for p in probs) == 4096
    checked = 0
    for n, prob in enumerate(probs):
        verdicts, outs, ref_out = _verify_problem(rt, prob)
        assert verdicts == [c["expect_equal"] for c in prob["candidates"]], (n, prob["family"])
        seed = prob["input_seed"]
        want_ref = _outputs(prob["reference"],
                            orc.eval_graph(prob["reference"], "fp", _inputs(prob["reference"], seed), threads=8))
        assert len(ref_out) == len(want_ref) and all(np.array_equal(a, b) for a, b in zip(ref_out, want_ref))
        for k in range(n % 8, len(prob["candidates"]), 8):
            c = prob["candidates"][k]
            want = _outputs(c["spec"], orc.eval_graph(c["spec"], "fp", _inputs(c["spec"], seed), threads=8))
            assert len(outs[k]) == len(want)
            for a, b in zip(outs[k], want):
                assert np.array_equal(a, b), (n, k, prob["family"])
            oracle_verdict = len(want) == len(want_ref) and all(
                a.shape == b.shape and np.array_equal(a, b) for a, b in zip(want_ref, want))
            assert verdicts[k] == oracle_verdict, (n, k, prob["family"])
            checked += 1
        if n % 8 == 7:
            print("problems verified:", n + 1, "candidates checked against the oracle:", checked, flush=True)
    assert checked == 512


def test_verify_batches_in_flight_match_one_at_a_time(rt):
    """Four submissions in flight (verify_batch_begin x 4, then verify_batch_end x 4, the
    reference graphs fingerprinted as part of their batches): same verdicts and the same
    candidate outputs as one blocking verify_batch per problem; repeated so that marks and
    compare-slot ranges are reused."""
    probs = C.generate(num_problems=8, per_problem=12, seed=0xF11E, max_dim=256)
    want = {}
    for k, prob in enumerate(probs):
        verdicts, outs, ref_out = _verify_problem(rt, prob)
        assert verdicts == [c["expect_equal"] for c in prob["candidates"]]
        want[k] = (verdicts, outs, ref_out)
    for queues in (4, 2, 1, 2, 4):  # queues a submission is dealt over; groups of queues rotate
        rt.set_verify_queues_per_batch(queues)
        for first in range(0, len(probs), 4):
            built = []
            try:
                for prob in probs[first:first + 4]:
                    ref_g, ref_vals = rt.build_from_spec(prob["reference"])
                    cands = [rt.build_from_spec(c["spec"]) for c in prob["candidates"]]
                    built.append((prob, ref_g, ref_vals, cands))
                tickets = [rt.verify_batch_begin([g for g, _ in cands], ref_g, prob["input_seed"])
                           for prob, ref_g, _, cands in built]
                for k, (ticket, (prob, ref_g, ref_vals, cands)) in enumerate(zip(tickets, built)):
                    verdicts, stats = rt.verify_batch_end(ticket)
                    w_verdicts, w_outs, w_ref = want[first + k]
                    assert verdicts == w_verdicts
                    assert stats["compares"] == len(cands)
                    ref_out = [t.read_fingerprint() for t in _outputs(prob["reference"], ref_vals)]
                    assert all(np.array_equal(a, b) for a, b in zip(ref_out, w_ref))
                    for c, (_, vals), w in zip(prob["candidates"], cands, w_outs):
                        got = [t.read_fingerprint() for t in _outputs(c["spec"], vals)]
                        assert all(np.array_equal(a, b) for a, b in zip(got, w))
            finally:
                for prob, ref_g, _, cands in reversed(built):
                    for g, _ in reversed(cands):
                        g.close()
                    ref_g.close()
    rt.set_verify_queues_per_batch(4)


def test_sixteen_batches_in_flight_on_one_queue_each(rt):
    """The benchmark's shape: sixteen submissions begun before the first is ended, each on one
    queue, ended newest first and then oldest first: verdicts as constructed and the same
    candidate outputs as a blocking verify_batch of the same problem."""
    probs = C.generate(num_problems=16, per_problem=8, seed=0x16F1, max_dim=256)
    want = [_verify_problem(rt, prob) for prob in probs]
    rt.set_verify_queues_per_batch(1)
    try:
        for order in (list(reversed(range(16))), list(range(16))):
            built = []
            try:
                for prob in probs:
                    ref_g, ref_vals = rt.build_from_spec(prob["reference"])
                    cands = [rt.build_from_spec(c["spec"]) for c in prob["candidates"]]
                    built.append((prob, ref_g, ref_vals, cands))
                tickets = [rt.verify_batch_begin([g for g, _ in cands], ref_g, prob["input_seed"])
                           for prob, ref_g, _, cands in built]
                for k in order:
                    prob, ref_g, ref_vals, cands = built[k]
                    verdicts, stats = rt.verify_batch_end(tickets[k])
                    assert verdicts == [c["expect_equal"] for c in prob["candidates"]], (k, prob["family"])
                    assert verdicts == want[k][0] and stats["compares"] == len(cands)
                    for c, (_, vals), w in zip(prob["candidates"], cands, want[k][1]):
                        got = [t.read_fingerprint() for t in _outputs(c["spec"], vals)]
                        assert all(np.array_equal(a, b) for a, b in zip(got, w)), (k, prob["family"])
            finally:
                for prob, ref_g, _, cands in reversed(built):
                    for g, _ in reversed(cands):
                        g.close()
                    ref_g.close()
    finally:
        rt.set_verify_queues_per_batch(4)


def test_marks_order_queues_and_report_only_their_work(rt, abi):
    """A compare enqueued on queue 1 behind a mark that queue 0 recorded after filling its
    operand sees the filled values; waiting for the mark queue 1 recorded is enough to read
    the slot."""
    import ctypes
    n = 1 << 20
    spec = [{"op": "input", "dims": [n]}, {"op": "input", "dims": [n]}]
    g, vals = rt.build_from_spec(spec)
    try:
        a, b = vals[0][0], vals[1][0]
        a.write_fingerprint(np.zeros(n, np.uint16))
        b.write_fingerprint(np.ones(n, np.uint16))
        assert abi.mi355_sync() == 0
        assert abi.mi355_queue_current() == 0
        for rep in range(3):
            slot = 60000 + rep
            assert abi.mi355_fp_equal_reset(slot, 1) == 0
            seed = 31 + rep
            for t in (a, b):  # queue 0: both tensors get the same sequence
                assert abi.mi355_fp_fill_uniform(ctypes.c_void_p(t.device_ptr(True)), n, seed) == 0
            assert abi.mi355_mark_record(10) == 0
            assert abi.mi355_queue_select(1) == 0
            try:
                assert abi.mi355_mark_wait_queue(10, 0) == 0
                assert abi.mi355_fp_equal_enqueue(ctypes.c_void_p(a.device_ptr(True)),
                                                  ctypes.c_void_p(b.device_ptr(True)), n, slot) == 0
                assert abi.mi355_mark_record(11) == 0
            finally:
                assert abi.mi355_queue_select(0) == 0
            assert abi.mi355_mark_wait_host(11) == 0
            eq = (ctypes.c_ubyte * 1)()
            assert abi.mi355_fp_equal_read(slot, 1, eq) == 0
            assert eq[0] == 1
            assert abi.mi355_mark_wait_host(10) == 0
        assert abi.mi355_mark_record(64) != 0 and abi.mi355_mark_wait_queue(0, 4) != 0
    finally:
        assert abi.mi355_sync() == 0
        g.close()


def test_verify_batch_iota_inputs_and_output_count(rt):
    """input_seed 0 = the reference's `idx % 25651` inputs; a candidate with a different
    number of outputs is rejected without a compare."""
    prob = C.generate(num_problems=1, per_problem=4, max_dim=128)[0]
    ref_g, _ = rt.build_from_spec(prob["reference"])
    graphs = []
    try:
        ref_g.fingerprint_seeded(0)
        for c in prob["candidates"]:
            graphs.append(rt.build_from_spec(c["spec"])[0])
        two_outputs = prob["reference"] + [{"op": "exp", "in": [[0, 0]]}]
        graphs.append(rt.build_from_spec(two_outputs)[0])
        verdicts, stats = rt.verify_batch(graphs, ref_g, 0)
        assert verdicts == [c["expect_equal"] for c in prob["candidates"]] + [False]
        assert stats["compares"] == len(prob["candidates"])
    finally:
        for g in reversed(graphs):
            g.close()
        ref_g.close()


def test_checkpoint_graphs_loaded_from_json_verify_equal(rt):
    """The reference's own checkpoint objects (original schema) loaded through the JSON
    wire format: every graph its search accepted verifies equal to the computation graph
    with the reference's `idx % 25651` inputs."""
    import json
    import os
    from helpers import GOLDEN
    with open(os.path.join(GOLDEN, "gqa_spec_decode_checkpoint_excerpt.json")) as f:
        doc = json.load(f)
    ref_g = rt.KNGraph.from_json(doc["computation_graph"])
    graphs = []
    try:
        ref_g.fingerprint_seeded(0)
        for ops in doc["generated_graphs"]:
            graphs.append(rt.KNGraph.from_json(ops))
        verdicts, stats = rt.verify_batch(graphs, ref_g, 0)
        assert verdicts == [True] * len(graphs)
        assert stats["customized_ops"] >= len(graphs)
    finally:
        for g in reversed(graphs):
            g.close()
        ref_g.close()
