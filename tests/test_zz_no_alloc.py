"""mi355_customized_fp_static -- the entry point that allocates nothing -- against
mi355_customized_fp, through the C ABI, bit for bit: two calls in a row, the second with a
smaller input (the static scratch keeps the first call's contents), then a plan without a
split for-loop, a third call on the first plan again, a plan that gets fewer ranges than
mi355_customized_fp gives it because theirs would not fit the array, and the refusal of a plan
of which not even two ranges fit."""
import ctypes

import numpy as np
import pytest

from helpers import uniform_fp
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu


def _both(rt, abi, spec, seed):
    """Runs the last (customized) operator of `spec` through both entry points; returns
    (outputs of mi355_customized_fp, outputs of mi355_customized_fp_static, oracle outputs,
    launch info of the static call)."""
    from attention_superoptimizer_amd import _native as N
    g, vals = rt.build_from_spec(spec)
    try:
        idx = len(spec) - 1
        ins = {}
        for i, op in enumerate(spec):
            if op["op"] == "input":
                ins[i] = uniform_fp(op["dims"], seed + i)
                vals[i][0].write_fingerprint(ins[i])
        plan = g.lowered(idx, True)
        i_p = (ctypes.c_void_p * 4)(*[vals[a][b].device_ptr(True) for a, b in spec[idx]["in"]])
        o_p = (ctypes.c_void_p * 4)(*[t.device_ptr(True) for t in vals[idx]])
        outs = []
        info = N.Mi355LaunchInfo()
        for fn in (abi.mi355_customized_fp, abi.mi355_customized_fp_static):
            for t in vals[idx]:
                t.write_fingerprint(np.full(t.dims, 7, np.uint16))
            rc = fn(ctypes.byref(plan), i_p, o_p)
            assert rc == 0, N.last_error()
            abi.mi355_last_launch(ctypes.byref(info))
            assert abi.mi355_sync() == 0
            outs.append([t.read_fingerprint() for t in vals[idx]])
        want = orc.eval_graph(spec, "fp", ins, threads=8)[idx]
        return outs[0], outs[1], want, info
    finally:
        g.close()


def test_static_scratch_entry_point_matches_the_allocating_one(rt, abi):
    from attention_superoptimizer_amd import workloads as W
    calls = [
        ("C1: 16 blocks x 16 ranges, 2 MiB of partial sums", W.config1_fused_matmul()[0], 16),
        ("smaller: 4 blocks x 8 ranges", W.tiled_matmul(32, 256, 512, (4, 1, 1), 8, (-1, -1, -1),
                                                        (1, -1, -1), (1, -1, -1))[0], 8),
        ("C2: attention plan, 32 blocks x 4 ranges, 4 MiB", W.config2_gqa_decode()[0], 4),
        ("no split: 256 blocks", W.tiled_matmul(256, 1024, 128, (16, 16, 1), 2, (0, -1, -1),
                                                (-1, 1, -1), (0, 1, -1))[0], 1),
        ("C1 again", W.config1_fused_matmul()[0], 16),
    ]
    for k, (what, spec, ranges) in enumerate(calls):
        print("  ", what, flush=True)
        a, b, want, info = _both(rt, abi, spec, 100 * k)
        assert info.kernel_id == 1 and info.row_split == ranges, (what, info.row_split)
        for x, y, w in zip(a, b, want):
            assert np.array_equal(y, w), what + ": static entry point vs oracle"
            assert np.array_equal(x, y), what + ": static entry point vs mi355_customized_fp"


def test_static_scratch_entry_point_takes_fewer_ranges_when_four_do_not_fit(rt, abi):
    """64 blocks -> mi355_customized_fp cuts the for-loop into 4 ranges: 4 x 256 x 8192 outputs
    x 2 bytes = 16 MiB of partial sums.  The static array holds 8 MiB: two ranges, same bits."""
    from attention_superoptimizer_amd import workloads as W
    spec = W.tiled_matmul(256, 8192, 64, (64, 1, 1), 4, (-1, -1, -1), (1, -1, -1), (1, -1, -1))[0]
    g, vals = rt.build_from_spec(spec)
    try:
        for i in (0, 1):
            vals[i][0].write_fingerprint(uniform_fp(spec[i]["dims"], 500 + i))
        plan = g.lowered(2, True)
        i_p = (ctypes.c_void_p * 4)(*[vals[a][b].device_ptr(True) for a, b in spec[2]["in"]])
        o_p = (ctypes.c_void_p * 4)(*[t.device_ptr(True) for t in vals[2]])
        assert abi.mi355_customized_fp(ctypes.byref(plan), i_p, o_p) == 0
        want = vals[2][0].read_fingerprint()
        vals[2][0].write_fingerprint(np.full(want.shape, 7, np.uint16))
        assert abi.mi355_customized_fp_static(ctypes.byref(plan), i_p, o_p) == 0
        assert abi.mi355_sync() == 0
        assert np.array_equal(vals[2][0].read_fingerprint(), want)
    finally:
        g.close()


def test_static_scratch_entry_point_refuses_what_does_not_fit(rt, abi):
    from attention_superoptimizer_amd import _native as N
    from attention_superoptimizer_amd import workloads as W
    # 128 blocks -> 2 ranges x 256 x 16384 outputs x 2 bytes = 16 MiB of partial sums
    spec = W.tiled_matmul(256, 16384, 64, (128, 1, 1), 4, (-1, -1, -1), (1, -1, -1), (1, -1, -1))[0]
    g, vals = rt.build_from_spec(spec)
    try:
        plan = g.lowered(2, True)
        i_p = (ctypes.c_void_p * 4)(*[vals[a][b].device_ptr(True) for a, b in spec[2]["in"]])
        o_p = (ctypes.c_void_p * 4)(*[t.device_ptr(True) for t in vals[2]])
        assert abi.mi355_customized_fp_static(ctypes.byref(plan), i_p, o_p) == -4   # MI355_ERR_UNSUPPORTED
        assert "static" in N.last_error() and "16777216" in N.last_error()
        assert abi.mi355_customized_fp_static(None, i_p, o_p) == -3
    finally:
        g.close()
