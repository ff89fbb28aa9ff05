"""The programs Graph::generate_hip_program writes, run on the device.  Each example graph is
generated in two forms (codegen.py): as the backend itself would run it -- a customized
operator of a fused family is an instantiation of that family's kernel -- and with every
customized operator as the specialised interpreter.  Either form gives the output of the
backend's matching route bit for bit (it is the same code, with the recognition and the
dispatch done at generation time), and the oracle's within the fp16 tolerance; the generated
decode-attention program is as fast as the backend's own launch."""
import ctypes
import os
import time

import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu

OPT_FORCE_INTERPRETER = 1

# standard deviations of the normal inputs, by graph and input position
STD = {"C1_fused_matmul": 0.1, "C2_gqa_decode": 0.125, "C3_mha_prefill": 128 ** -0.5,
       "C4_lora": {0: 0.25, 1: 0.02, 2: 0.02, 3: 0.02},
       "C5a_gated_mlp": {0: 0.25, 1: 0.02, 2: 0.02, 3: 0.02}, "mlp": 0.05}
# |V| for the prefill attention graph: with V of both signs the fp16 for-loop accumulators pass
# through values far above the final one, and two correct evaluations that order a tile product's
# fp32 additions differently end one accumulator ulp apart, above the plain tolerance
NON_NEGATIVE = {"C3_mha_prefill": (2,)}

_oracle_cache = {}


def _library(name):
    from attention_superoptimizer_amd import codegen as CG
    if not os.path.exists(CG.library_path(name)):  # nothing built: generate and compile now
        CG.compile_library(CG.generate(name), CG.library_path(name))
    lib = ctypes.CDLL(CG.library_path(name))
    lib.graphdef_launch.restype = ctypes.c_int
    lib.graphdef_launch.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
    lib.graphdef_tensor_elements.restype = ctypes.c_longlong
    return lib


def _inputs(name, spec):
    std = STD[name]
    ins = {i: normal_f16(op["dims"], std.get(i, 1.0) if isinstance(std, dict) else std, 70 + i)
           for i, op in enumerate(spec) if op["op"] == "input"}
    for i in NON_NEGATIVE.get(name, ()):
        ins[i] = np.abs(ins[i])
    return ins


@pytest.mark.parametrize("interpreter", [False, True], ids=["fused", "interpreter"])
@pytest.mark.parametrize("name", ["C1_fused_matmul", "C2_gqa_decode", "C3_mha_prefill", "C4_lora",
                                  "C5a_gated_mlp", "mlp"])
def test_generated_program_matches_the_backend(rt, abi, name, interpreter):
    from attention_superoptimizer_amd import codegen as CG
    spec = CG.example_spec(name)
    lib = _library(name + (CG.INTERPRETER_SUFFIX if interpreter else ""))
    ins = _inputs(name, spec)
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 1 if interpreter else 0) == 0
    g, vals = rt.build_from_spec(spec)
    try:
        for i, a in ins.items():
            vals[i][0].write_data(a)
        customized = [i for i, op in enumerate(spec) if op["op"] == "customized"]
        for i in range(len(spec)):
            if spec[i]["op"] != "input":
                g.execute(i)
        backend = {i: [t.read_data() for t in vals[i]] for i in customized}
        # the program sees the same device tensors, in creation order
        tensors = [t for v in vals for t in v]
        assert lib.graphdef_num_tensors() == len(tensors)
        for k, t in enumerate(tensors):
            assert lib.graphdef_tensor_elements(k) == int(np.prod(t.dims))
        for i in customized:
            for t in vals[i]:
                t.write_data(np.zeros(t.dims, np.float16))
        assert abi.mi355_sync() == 0
        ptrs = (ctypes.c_void_p * len(tensors))(*[t.device_ptr(False) for t in tensors])
        print("launching generated program", name, "interpreter" if interpreter else "fused", flush=True)
        assert lib.graphdef_launch(ptrs, None) == 0
        assert lib.graphdef_sync() == 0
        if name not in _oracle_cache:
            _oracle_cache[name] = orc.eval_graph(spec, "f16", ins, threads=8)
        want = _oracle_cache[name]
        for i in customized:
            for j, t in enumerate(vals[i]):
                got = t.read_data()
                assert np.array_equal(got.view(np.uint16), backend[i][j].view(np.uint16)), \
                    f"{name}: op {i} output {j} differs from the backend's own launch"
                assert_f16_close(got, want[i][j], what=f"{name} op {i} out {j} vs oracle")
    finally:
        g.close()
        assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 0) == 0


def test_generated_decode_attention_runs_at_the_backends_speed(rt, abi):
    """Host wall clock per launch over 1024 back-to-back launches, after as many untimed ones:
    the generated program of the decode-attention graph against the backend's own launch of
    the same customized operator.  They launch the same kernel; the bound of 2x leaves room for
    the difference between the two launch loops."""
    from attention_superoptimizer_amd import _native as N
    from attention_superoptimizer_amd import codegen as CG
    name, launches = "C2_gqa_decode", 1024
    spec = CG.example_spec(name)
    lib = _library(name)
    ins = _inputs(name, spec)
    g, vals = rt.build_from_spec(spec)
    try:
        for i, a in ins.items():
            vals[i][0].write_data(a)
        tensors = [t for v in vals for t in v]
        ptrs = (ctypes.c_void_p * len(tensors))(*[t.device_ptr(False) for t in tensors])
        op = next(i for i, o in enumerate(spec) if o["op"] == "customized")
        plan = g.lowered(op, fingerprint=False)
        i_p = (ctypes.c_void_p * 4)(*[vals[a][b].device_ptr(False) for a, b in spec[op]["in"]])
        o_p = (ctypes.c_void_p * 4)(*[t.device_ptr(False) for t in vals[op]])
        ms = ctypes.c_float()

        def generated():
            for _ in range(launches):
                assert lib.graphdef_launch(ptrs, None) == 0
            assert lib.graphdef_sync() == 0

        def backend():
            assert abi.mi355_customized_profile(ctypes.byref(plan), i_p, o_p, 0, 0, launches,
                                                ctypes.byref(ms)) == 0, N.last_error()
            assert abi.mi355_sync() == 0

        us = {}
        for what, run in (("backend", backend), ("generated", generated)):
            run()  # untimed
            t0 = time.perf_counter()
            run()
            us[what] = (time.perf_counter() - t0) * 1e6 / launches
        print("decode attention, us per launch:", us, flush=True)
        assert us["generated"] <= 2.0 * us["backend"], us
    finally:
        g.close()
