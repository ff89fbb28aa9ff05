"""The programs Graph::generate_hip_program writes, run on the device: the specialised
kernel of every customized op gives the fp16 interpreter's output bit for bit (it is the same
arithmetic with the dispatch removed), and the oracle's within the fp16 tolerance."""
import ctypes
import os

import numpy as np
import pytest

from helpers import assert_f16_close, normal_f16
from oracle import evaluate as orc

pytestmark = pytest.mark.gpu

OPT_FORCE_INTERPRETER = 1


def _library(name):
    from attention_superoptimizer_amd import codegen as CG
    if not os.path.exists(CG.library_path(name)):  # nothing built: generate and compile now
        CG.compile_library(CG.generate(name), CG.library_path(name))
    lib = ctypes.CDLL(CG.library_path(name))
    lib.graphdef_launch.restype = ctypes.c_int
    lib.graphdef_launch.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
    lib.graphdef_tensor_elements.restype = ctypes.c_longlong
    return lib


@pytest.mark.parametrize("name,std", [("C1_fused_matmul", 0.1), ("C2_gqa_decode", 0.125),
                                      ("C4_lora", {0: 0.25, 1: 0.02, 2: 0.02, 3: 0.02}),
                                      ("mlp", 0.05)])
def test_generated_program_matches_the_interpreter(rt, abi, name, std):
    from attention_superoptimizer_amd import codegen as CG
    spec = CG.example_spec(name)
    lib = _library(name)
    ins = {i: normal_f16(op["dims"], std.get(i, 1.0) if isinstance(std, dict) else std, 70 + i)
           for i, op in enumerate(spec) if op["op"] == "input"}
    assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 1) == 0
    g, vals = rt.build_from_spec(spec)
    try:
        for i, a in ins.items():
            vals[i][0].write_data(a)
        customized = [i for i, op in enumerate(spec) if op["op"] == "customized"]
        for i in range(len(spec)):
            if spec[i]["op"] != "input":
                g.execute(i)
        interp = {i: [t.read_data() for t in vals[i]] for i in customized}
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
        print("launching generated program", name, flush=True)
        assert lib.graphdef_launch(ptrs, None) == 0
        assert lib.graphdef_sync() == 0
        want = orc.eval_graph(spec, "f16", ins, threads=8)
        for i in customized:
            for j, t in enumerate(vals[i]):
                got = t.read_data()
                assert np.array_equal(got.view(np.uint16), interp[i][j].view(np.uint16)), \
                    f"{name}: op {i} output {j} differs from the interpreter"
                assert_f16_close(got, want[i][j], what=f"{name} op {i} out {j} vs oracle")
    finally:
        g.close()
        assert abi.mi355_set_option(OPT_FORCE_INTERPRETER, 0) == 0
