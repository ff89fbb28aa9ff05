"""Graph::generate_hip_program on the host (this backend's counterpart of the reference's
generate_triton_program, src/kernel/triton_code_gen.cc:354-450): what the emitted program
contains, that emission is deterministic, and that hipcc accepts it for gfx950.  The programs
run in test_gpu_generated_hip.py."""
import os
import re
import subprocess

import pytest

from attention_superoptimizer_amd import codegen as CG
from attention_superoptimizer_amd import graph as G
from attention_superoptimizer_amd import workloads as W


def _emit(spec, path):
    G.set_smem_budget(1 << 20)
    g, _ = G.build_from_spec(spec)
    try:
        g.generate_hip_program(str(path))
    finally:
        g.close()
    return open(path).read()


def test_program_structure_of_the_decode_attention_graph(tmp_path):
    spec, _ = W.config2_gqa_decode()
    text = _emit(spec, tmp_path / "c2.hip")
    # one kernel for the one customized op, specialised: literal grid, for-loop and tiles
    assert text.count("__global__") == 1
    assert "void graphdef_kernel_0(_Float16 const *__restrict__ in0" in text
    assert "graphdef_kernel_0<<<dim3(2, 16, 1), kThreads," in text
    assert "for (int it = 0; it < 4; it++)" in text
    assert text.count("tb_matmul<256, 64, 64,") == 2          # S = Q.K and O = P.V
    assert "__expf(x)" in text and "a / b" in text             # exp, div
    assert "sum of 64 elements, stride 1" in text              # row sums
    assert "if (it == 0) {" in text                            # Q is loop invariant: loaded once
    # 3 loaders + matmul + exp + reduction + div + matmul + saver, a barrier after each
    assert len(re.findall(r"// op \d+:", text)) == 9
    assert text.count("__syncthreads();") == 9
    # launcher: inputs are device tensors 0..2, the output tensor 3; 4 tensors in all
    assert "void const *in[] = {dtensors[0], dtensors[1], dtensors[2]};" in text
    assert "void *out[] = {dtensors[3]};" in text
    assert "graphdef_num_tensors(void) { return 4; }" in text
    assert "kTensorElements[] = {32768, 524288, 524288, 524288}" in text
    assert "int main()" in text and "#ifndef GRAPHDEF_NO_MAIN" in text


def test_only_customized_operators_are_emitted(tmp_path):
    """The gated MLP runs as two customized ops; an un-fused graph has none and yields a
    program with an empty launcher (the reference skips non-customized operators too)."""
    spec, ref = W.config5_gated_mlp()
    text = _emit(spec, tmp_path / "c5.hip")
    assert text.count("__global__") == 2
    assert "graphdef_kernel_1_launch(in, out, stream)" in text
    assert "x / (1.0f + __expf(-x))" in text                  # SiLU
    text = _emit(ref, tmp_path / "ref.hip")
    assert text.count("__global__") == 0 and "graphdef_launch" in text


def test_emission_is_deterministic(tmp_path):
    spec, _ = W.config4_lora()
    assert _emit(spec, tmp_path / "a.hip") == _emit(spec, tmp_path / "b.hip")


def test_hipcc_compiles_the_program_for_gfx950(tmp_path):
    if not os.path.exists(CG.HIPCC):
        pytest.skip("no hipcc")
    spec, _ = W.config1_fused_matmul()
    _emit(spec, tmp_path / "c1.hip")
    CG.compile_library(str(tmp_path / "c1.hip"), str(tmp_path / "libc1.so"))
    syms = subprocess.check_output(["nm", "-D", "--defined-only", str(tmp_path / "libc1.so")]).decode()
    for name in ("graphdef_launch", "graphdef_kernel_0_launch", "graphdef_num_tensors",
                 "graphdef_tensor_elements", "graphdef_sync"):
        assert f" T {name}" in syms
