"""The boundary as a maintainer of the reference meets it: the CMake build (in place of the
reference's CMakeLists.txt / cmake/cuda.cmake), the `operator json()` call sites of the
reference compiled against include/mirage, and the checkpoint object."""
import ctypes
import json
import os
import re
import shutil
import subprocess
import sys

import pytest

from helpers import GOLDEN

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "attention_superoptimizer_amd")


def _abi_symbols():
    text = open(os.path.join(ROOT, "include", "mi355_abi.h")).read()
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_by_the_in_tree_library():
    syms = subprocess.check_output(["nm", "-D", "--defined-only", os.path.join(PKG, "libmi355_backend.so")]).decode()
    have = set(re.findall(r" T (mi355_[a-z0-9_]+)", syms))
    missing = [s for s in _abi_symbols() if s not in have]
    assert not missing, missing
    # kernel handles are weak global symbols named after the kernel: the library binds its own
    # (a generated program in the same process instantiates some of the same templates)
    assert "SYMBOLIC" in subprocess.check_output(
        ["readelf", "-d", os.path.join(PKG, "libmi355_backend.so")]).decode()


def test_options_take_their_documented_values_only():
    """mi355_set_option needs no device: every option of the header accepts its documented
    values and refuses the next one; the vendor's BLAS is not a link dependency (it is opened
    when the option that asks for it is used)."""
    lib = ctypes.CDLL(os.path.join(PKG, "libmi355_backend.so"))
    text = open(os.path.join(ROOT, "include", "mi355_abi.h")).read()
    opts = dict((name, int(v)) for name, v in re.findall(r"#define (MI355_OPT_[A-Z0-9_]+) (\d+)", text))
    assert sorted(opts.values()) == list(range(1, len(opts) + 1))
    assert lib.mi355_set_option(opts["MI355_OPT_F16_MATMUL_ROUTE"], 1) == 0
    assert lib.mi355_set_option(opts["MI355_OPT_F16_MATMUL_ROUTE"], 0) == 0
    assert lib.mi355_set_option(opts["MI355_OPT_F16_MATMUL_ROUTE"], 2) != 0
    assert lib.mi355_set_option(opts["MI355_OPT_GEMM_MODE"], 3) != 0
    assert lib.mi355_set_option(len(opts) + 1, 0) != 0
    needed = subprocess.check_output(["readelf", "-d", os.path.join(PKG, "libmi355_backend.so")]).decode()
    assert "rocblas" not in needed


@pytest.mark.skipif(shutil.which("cmake") is None, reason="cmake not installed")
def test_cmake_configures_and_builds_for_gfx950(tmp_path):
    """project(... LANGUAGES CXX HIP), CMAKE_HIP_ARCHITECTURES gfx950, targets mi355_backend,
    mirage_runtime and mirage_profile; no CUDA, cutlass, z3 or cuDNN anywhere."""
    text = open(os.path.join(ROOT, "CMakeLists.txt")).read()
    assert re.search(r"project\(MIRAGE LANGUAGES CXX HIP\)", text)
    assert "CMAKE_HIP_ARCHITECTURES gfx950" in text
    code = "\n".join(line for line in text.splitlines() if not line.lstrip().startswith("#"))
    for gone in ("CUDA", "cutlass", "Z3", "cudnn", "cublas"):
        assert gone.lower() not in code.lower(), gone
    build = tmp_path / "build"
    gen = ["-G", "Ninja"] if shutil.which("ninja") else []
    subprocess.check_call(["cmake", "-S", ROOT, "-B", str(build)] + gen, stdout=subprocess.DEVNULL)
    subprocess.check_call(["cmake", "--build", str(build), "-j8"], stdout=subprocess.DEVNULL,
                          stderr=subprocess.DEVNULL)
    backend, runtime = build / "libmi355_backend.so", build / "libmirage_runtime.so"
    assert backend.exists() and runtime.exists() and (build / "mirage_profile").exists()
    syms = subprocess.check_output(["nm", "-D", "--defined-only", str(backend)]).decode()
    have = set(re.findall(r" T (mi355_[a-z0-9_]+)", syms))
    assert not [s for s in _abi_symbols() if s not in have]
    assert "SYMBOLIC" in subprocess.check_output(["readelf", "-d", str(backend)]).decode()
    # the code object is gfx950 and nothing else
    notes = subprocess.check_output(["strings", "-n", "8", str(backend)]).decode()
    assert "gfx950" in notes and "gfx90a" not in notes and "gfx942" not in notes
    # the CMake-built pair loads and lowers a plan (host-only: no device here)
    probe = (
        "import ctypes,sys\n"
        f"b=ctypes.CDLL(r'{backend}',mode=ctypes.RTLD_GLOBAL); r=ctypes.CDLL(r'{runtime}',mode=ctypes.RTLD_GLOBAL)\n"
        "r.mirage_graph_create.restype=ctypes.c_void_p\n"
        "g=r.mirage_graph_create(); assert g\n"
        "assert b.mi355_is_initialised()==0\n"
        "print('ok')\n")
    env = dict(os.environ, MIRAGE_HOST_ONLY="1")
    out = subprocess.check_output([sys.executable, "-c", probe], env=env).decode()
    assert out.strip() == "ok"


def test_reference_json_call_sites_compile_and_run(tmp_path):
    """json(*op) on KNOperator* / TBOperator*, json(bgraph), json(g), `ifs >> j`, `cout << j`."""
    exe = tmp_path / "operator_json"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
                           "-I", "/opt/rocm/include", "-o", str(exe),
                           os.path.join(ROOT, "tests", "cpp", "operator_json.cc"),
                           "-L" + PKG, "-lmirage_runtime", "-lmi355_backend", "-Wl,-rpath," + PKG])
    env = dict(os.environ, MIRAGE_HOST_ONLY="1", MIRAGE_SMEM_BUDGET=str(1 << 20))
    r = subprocess.run([str(exe)], env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    ops = json.loads(r.stdout)
    assert [o["op_type"] for o in ops] == ["kn_input_op", "kn_input_op", "kn_customized_op", "kn_exp_op"]
    tb = ops[2]["bgraph"]["operators"]
    assert [o["op_type"] for o in tb] == ["tb_input_op", "tb_input_op", "tb_matmul_op", "tb_exp_op",
                                         "tb_reduction_1_op", "tb_output_op"]
    assert tb[0]["forloop_dim"] == 1 and tb[5]["output_map"] == {"x": 1, "y": -1, "z": -1}


def test_checkpoint_object_loads_and_passes_through():
    """The reference's own checkpoint object (search.h:46-68), all top-level fields."""
    from attention_superoptimizer_amd import graph as G
    path = os.path.join(GOLDEN, "gqa_spec_decode_checkpoint_excerpt.json")
    want = json.load(open(path))
    G.set_smem_budget(1 << 20)
    cp = G.Checkpoint.load(path)
    try:
        assert cp.num_graphs == len(want["generated_graphs"]) == 8
        assert cp.counters == (want["num_total_kernel_graphs"], want["num_total_random_tests"],
                               want["num_valid_kernel_graphs"]) == (90747825, 704019, 69)
        assert cp.best_run_time == want["best_profile_result"]["run_time"]
        back = json.loads(cp.to_json())
        for key in ("computation_graph", "best_graph", "config", "callstack", "generated_graphs"):
            assert back[key] == want[key], key
        assert json.loads(cp.graph_json(-1)) == want["computation_graph"]
        for i in range(cp.num_graphs):
            g = cp.graph(i)
            try:
                assert g.num_operators == len(want["generated_graphs"][i])
            finally:
                g.close()
    finally:
        cp.close()
    with pytest.raises(ValueError):
        G.Checkpoint.load(os.path.join(GOLDEN, "no_such_file.json"))


def test_single_graph_file_round_trips_as_a_checkpoint(tmp_path):
    """A single-graph file (what cpp_examples/profile.cc takes) loads as a one-graph checkpoint
    whose best profile was never set; what it writes is valid JSON with a finite run time (the
    reference's "infinity" is 1000 ms, src/profile_result.cc:7-9) and loads again.  A run time
    spelled null (how a writer spells a non-finite float) reads back as that same sentinel."""
    from attention_superoptimizer_amd import graph as G
    want = json.load(open(os.path.join(GOLDEN, "gqa_spec_decode_checkpoint_excerpt.json")))
    G.set_smem_budget(1 << 20)
    single = tmp_path / "single.json"
    single.write_text(json.dumps(want["generated_graphs"][0]))
    cp = G.Checkpoint.load(str(single))
    try:
        assert cp.num_graphs == 1 and cp.best_run_time == 1000.0
        text = cp.to_json()
        back = json.loads(text)  # Python's parser rejects inf / nan spelled any way but null
        assert back["best_profile_result"]["run_time"] == 1000.0
        assert back["generated_graphs"] == [want["generated_graphs"][0]]
    finally:
        cp.close()
    again = tmp_path / "again.json"
    again.write_text(text)
    cp2 = G.Checkpoint.load(str(again))
    try:
        assert cp2.num_graphs == 1 and cp2.best_run_time == 1000.0
    finally:
        cp2.close()
    back["best_profile_result"]["run_time"] = None
    nulled = tmp_path / "nulled.json"
    nulled.write_text(json.dumps(back))
    cp3 = G.Checkpoint.load(str(nulled))
    try:
        assert cp3.best_run_time == 1000.0
        assert json.loads(cp3.to_json())["best_profile_result"]["run_time"] == 1000.0
    finally:
        cp3.close()


def test_build_refuses_register_spills_in_kernels_with_asynchronous_register_loads():
    """build.py reads the compiler's resource report for the kernels whose inline-assembly
    loads write registers behind the compiler's back and fails the build when one of them
    spills (a spill between such a load and its wait would save stale data)."""
    from attention_superoptimizer_amd import build as B

    def report(name, scratch, spilled):
        head = "csrc/backend/x.hip:1:1: remark: "
        tail = " [-Rpass-analysis=kernel-resource-usage]\n"
        return (head + f"Function Name: _ZN5mi355{len(name)}{name}E" + tail +
                head + "    VGPRs: 235" + tail +
                head + f"    ScratchSize [bytes/lane]: {scratch}" + tail +
                head + "    Occupancy [waves/SIMD]: 2" + tail +
                head + f"    VGPRs Spill: {spilled}" + tail)

    text = report("fp_mfma_matmul_kernel", 64, 3) + report("fp_mfma_matmul_big_kernel", 0, 0)
    usage = B.resource_usage(text)
    assert len(usage) == 2
    assert B.spilling(usage, "fp_mfma_matmul_big_kernel") == []
    assert B.spilling(usage, "fp_mfma_matmul_kernel")[0]["VGPRs Spill"] == "3"
    assert B.spilling(B.resource_usage(report("fp_mfma_matmul_big_kernel", 528, 0)),
                      "fp_mfma_matmul_big_kernel")[0]["ScratchSize [bytes/lane]"] == "528"
    with pytest.raises(RuntimeError):
        B.spilling(usage, "no_such_kernel")
    for names in B.NO_SPILL_KERNELS.values():
        assert names
