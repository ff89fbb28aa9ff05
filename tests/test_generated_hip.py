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


def _emit(spec, path, interpreter=False):
    """`interpreter`: with the force-interpreter option on, every customized operator is printed
    as the specialised interpreter; otherwise one of a fused family is printed as that family's
    kernel (what the backend itself would launch)."""
    from attention_superoptimizer_amd import _native as N
    G.set_smem_budget(1 << 20)
    assert N.backend().mi355_set_option(1, 1 if interpreter else 0) == 0
    g, _ = G.build_from_spec(spec)
    try:
        g.generate_hip_program(str(path))
    finally:
        g.close()
        assert N.backend().mi355_set_option(1, 0) == 0
    return open(path).read()


def test_fused_families_are_emitted_as_their_kernels(tmp_path):
    """An operator the backend runs on a fused kernel is emitted as that launch: the kernel
    template of include/mi355_kernels/ with literal arguments, grid, LDS size and parameter
    block -- no interpreter kernel in the file."""
    spec, _ = W.config2_gqa_decode()
    text = _emit(spec, tmp_path / "c2.hip")
    assert text.count("__global__") == 0
    assert '#include "mi355_kernels/attention.h"' in text
    assert ("mi355::attn_direct_kernel<64, 64, 64, true, 4, 2, 1, 1, 1, 1, false, true>"
            "<<<dim3(16, 16, 1), 256, 81920, stream>>>(P);") in text
    # K [2, 64, 4096] and V [2, 4096, 64] are column-major: leading dimensions 64 and 4096
    assert "P.k = mi355::TileAddr{in[1], {262144, 16384, 0, 4096}, 64};" in text
    assert "P.v = mi355::TileAddr{in[2], {262144, 256, 0, 64}, 4096};" in text
    assert "hipFuncAttributeMaxDynamicSharedMemorySize, 81920" in text
    assert "void const *in[] = {dtensors[0], dtensors[1], dtensors[2]};" in text
    # C3: throughput attention kernel, then the fold-and-divide kernel
    spec, _ = W.config3_mha_prefill()
    text = _emit(spec, tmp_path / "c3.hip")
    assert text.count("__global__") == 0
    assert "mi355::attn_stream_kernel<128, 64, 128, false, 4, 2, true, 1><<<dim3(32, 1, 16), 256, 65536, stream>>>(P);" in text
    assert '#include "mi355_kernels/combine.h"' in text and "mi355::combine_fused_kernel<8, 0, 4><<<dim3(32, 64, 1), 256, 0, stream>>>(P);" in text
    # C4: the range kernel and its fold share a workspace the program allocates once
    spec, _ = W.config4_lora()
    text = _emit(spec, tmp_path / "c4.hip")
    assert "mi355::gemm_fused_kernel<1, 1, 0, true, 256, true><<<" in text
    assert "mi355::gemm_combine_kernel<1><<<dim3(64, 1, 1), 256, 0, stream>>>(P);" in text
    assert "static void *scratch = nullptr;" in text and "P.scratch = static_cast<_Float16 *>(scratch);" in text
    # C1: the one-launch kernel
    spec, _ = W.config1_fused_matmul()
    text = _emit(spec, tmp_path / "c1.hip")
    assert "mi355::gemm_lanes_kernel<64, 1, 0, false, true><<<dim3(256, 1, 1), 1024," in text


def test_program_structure_of_the_decode_attention_graph(tmp_path):
    spec, _ = W.config2_gqa_decode()
    text = _emit(spec, tmp_path / "c2.hip", interpreter=True)
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
    text = _emit(spec, tmp_path / "c5.hip", interpreter=True)
    assert text.count("__global__") == 2
    assert "graphdef_kernel_1_launch(in, out, stream)" in text
    assert "x / (1.0f + __expf(-x))" in text                  # SiLU
    text = _emit(ref, tmp_path / "ref.hip")
    assert text.count("__global__") == 0 and "graphdef_launch" in text


def test_emission_is_deterministic(tmp_path):
    spec, _ = W.config4_lora()
    assert _emit(spec, tmp_path / "a.hip") == _emit(spec, tmp_path / "b.hip")
    assert _emit(spec, tmp_path / "c.hip", True) == _emit(spec, tmp_path / "d.hip", True)


def test_hipcc_compiles_the_program_for_gfx950(tmp_path):
    if not os.path.exists(CG.HIPCC):
        pytest.skip("no hipcc")
    spec, _ = W.config1_fused_matmul()
    for interpreter in (False, True):
        _emit(spec, tmp_path / "c1.hip", interpreter)
        CG.compile_library(str(tmp_path / "c1.hip"), str(tmp_path / "libc1.so"))
        syms = subprocess.check_output(["nm", "-D", "--defined-only", str(tmp_path / "libc1.so")]).decode()
        for name in ("graphdef_launch", "graphdef_kernel_0_launch", "graphdef_num_tensors",
                     "graphdef_tensor_elements", "graphdef_sync"):
            assert f" T {name}" in syms
        # a kernel's host-side handle is a weak global symbol named after the kernel, and the
        # backend library instantiates the same templates: each library binds its own
        dyn = subprocess.check_output(["readelf", "-d", str(tmp_path / "libc1.so")]).decode()
        assert "SYMBOLIC" in dyn
