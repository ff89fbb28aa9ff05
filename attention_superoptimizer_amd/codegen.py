"""Generated HIP programs: drives Graph::generate_hip_program (this backend's counterpart of
the reference's generate_triton_program, src/kernel/triton_code_gen.cc:354-450) and compiles
what it writes.

`python -m attention_superoptimizer_amd.codegen` generates and compiles the programs of
EXAMPLES into attention_superoptimizer_amd/generated/ (host code only: hipcc cross-compiles
for gfx950 without a GPU); the build recipe runs it, the GPU tests load the libraries.
"""
from __future__ import annotations

import os
import subprocess
import sys
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
GENERATED = os.path.join(HERE, "generated")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -ffp-contract=on: with the default (fast) the compiler may pair the terms of a short,
# fully unrolled multiply-add chain into two-element dot products, which round differently
# from the fp16 interpreter's chain; "on" keeps every fused multiply-add as written
# -I include: a customized operator of one of the fused families (attention, skinny GEMM,
# fold-and-divide) is emitted as an instantiation of that family's kernel from
# include/mi355_kernels/*.h
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=on",
         "-I", os.path.join(os.path.dirname(HERE), "include"),
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-mllvm", "-amdgpu-mfma-vgpr-form",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]

# graphs whose programs the build generates and the GPU tests run; each in two forms: as the
# backend itself would run it (fused-family kernels where one applies) and, under the name
# with INTERPRETER_SUFFIX, every customized operator as the specialised interpreter
EXAMPLES = ["C1_fused_matmul", "C2_gqa_decode", "C3_mha_prefill", "C4_lora", "C5a_gated_mlp", "mlp"]
INTERPRETER_SUFFIX = "_interp"
OPT_FORCE_INTERPRETER = 1


def example_spec(name: str) -> List[dict]:
    from . import workloads as W
    if name.endswith(INTERPRETER_SUFFIX):
        name = name[:-len(INTERPRETER_SUFFIX)]
    if name in W.BASELINE_CONFIGS:
        return W.BASELINE_CONFIGS[name]()[0]
    return W.REFERENCE_EXAMPLES[name][0]


def source_path(name: str) -> str:
    return os.path.join(GENERATED, name + ".hip")


def library_path(name: str) -> str:
    return os.path.join(GENERATED, "lib" + name + ".so")


def program_path(name: str) -> str:
    return os.path.join(GENERATED, name)


def generate(name: str) -> str:
    """Builds the example graph through the host API and writes its HIP program."""
    from . import _native as N
    from . import graph as G
    G.set_smem_budget(1 << 20)
    os.makedirs(GENERATED, exist_ok=True)
    forced = 1 if name.endswith(INTERPRETER_SUFFIX) else 0
    if N.backend().mi355_set_option(OPT_FORCE_INTERPRETER, forced) != 0:
        raise RuntimeError("mi355_set_option failed")
    g, _ = G.build_from_spec(example_spec(name))
    try:
        g.generate_hip_program(source_path(name))
    finally:
        g.close()
        N.backend().mi355_set_option(OPT_FORCE_INTERPRETER, 0)
    return source_path(name)


def compile_library(src: str, out: str) -> None:
    """The program without its main(), as a shared library exporting graphdef_launch."""
    # -Bsymbolic: the program's kernels are instantiations of templates the backend library
    # instantiates too, and a kernel's host-side handle is a weak global symbol of that name;
    # loaded into one process, each library must launch through its own handles
    subprocess.check_call([HIPCC] + FLAGS + ["-DGRAPHDEF_NO_MAIN", "-shared", "-fPIC", "-fvisibility=hidden",
                                             "-Wl,-Bsymbolic", src, "-o", out])


def compile_program(src: str, out: str) -> None:
    subprocess.check_call([HIPCC] + FLAGS + [src, "-o", out])


def build_examples() -> None:
    for name in EXAMPLES + [e + INTERPRETER_SUFFIX for e in EXAMPLES]:
        src = generate(name)
        compile_library(src, library_path(name))
        compile_program(src, program_path(name))
        print("generated and compiled", src, flush=True)


if __name__ == "__main__":
    build_examples()
    sys.exit(0)
