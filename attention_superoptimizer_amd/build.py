"""Build recipe: compiles the gfx950 backend and the host runtime in-tree with hipcc.

  libmi355_backend.so   HIP kernels + the C ABI of include/mi355_abi.h
  libmirage_runtime.so  the mirage:: host API (C++) + its C facade for ctypes
  mirage_profile        the reference's cpp_examples/profile.cc over that API
  generated/            HIP programs written by Graph::generate_hip_program for the example
                        graphs of codegen.py, compiled as libraries and executables

Run as `python -m attention_superoptimizer_amd.build`.
"""
from __future__ import annotations

import os
import subprocess
from concurrent.futures import ThreadPoolExecutor
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
BACKEND_LIB = os.path.join(HERE, "libmi355_backend.so")
RUNTIME_LIB = os.path.join(HERE, "libmirage_runtime.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: packed FP32 forms have produced silent wrong results on these boxes
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
                # MFMA results stay in VGPRs: with accumulators in AGPRs every use of a product by
                # vector code costs a v_accvgpr_read (the fingerprint matmul kernels' step: 144 ->
                # 96 vector instructions, their verification family 271 K -> 340 K candidates/s)
                "-mllvm", "-amdgpu-mfma-vgpr-form"]


# source file -> kernels that must build without register spills (see build_backend)
NO_SPILL_KERNELS = {"fp_mfma.hip": ["fp_mfma_matmul_big_kernel"]}
# fewest wavefronts per SIMD those kernels are written for (two workgroups per compute unit):
# fewer means the register allocation is no longer the one the hand-placed loads and waits
# were checked against
MIN_OCCUPANCY = {"fp_mfma_matmul_big_kernel": 2}


def resource_usage(remarks):
    """Per kernel (mangled name) the figures of hipcc's -Rpass-analysis=kernel-resource-usage."""
    usage, name = {}, None
    for line in remarks.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif name and "remark:" in line and ":" in line.split("remark:")[1]:
            key, _, value = line.split("remark:")[1].partition(":")
            usage.setdefault(name, {})[key.strip()] = value.split("[")[0].strip()
    return usage


def spilling(usage, kernel):
    """Resource figures of the kernels named `kernel` that use scratch memory or spill vector
    registers; raises if the compiler reported nothing for that name."""
    hits = [u for n, u in usage.items() if kernel in n]
    if not hits:
        raise RuntimeError(f"no resource usage reported for {kernel}")
    least = MIN_OCCUPANCY.get(kernel, 0)
    return [u for u in hits if u.get("ScratchSize [bytes/lane]") != "0" or u.get("VGPRs Spill") != "0" or
            int(u.get("Occupancy [waves/SIMD]", least)) < least]


def _sources(sub, exts):
    d = os.path.join(CSRC, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(exts))


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_backend():
    srcs = _sources("backend", (".hip", ".cc"))
    objs = [os.path.splitext(s)[0] + ".o" for s in srcs]

    def compile_one(pair):
        s, o = pair
        lang = ["-x", "hip"] if s.endswith(".hip") else []
        cmd = [HIPCC] + DEVICE_FLAGS + ["-I", INCLUDE, "-I", os.path.join(CSRC, "backend"), "-c"] + lang + [s, "-o", o]
        must_not_spill = NO_SPILL_KERNELS.get(os.path.basename(s))
        if not must_not_spill:
            _run(cmd)
            return
        # kernels whose inline-assembly loads land in registers behind the compiler's back: a
        # spill between such a load and its wait would save stale data, so the build fails on one
        cmd.append("-Rpass-analysis=kernel-resource-usage")
        print(" ".join(cmd), flush=True)
        done = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
        if done.returncode != 0:
            sys.stderr.write(done.stderr)
            raise subprocess.CalledProcessError(done.returncode, cmd)
        usage = resource_usage(done.stderr)
        for kernel in must_not_spill:
            bad = spilling(usage, kernel)
            if bad:
                raise RuntimeError(f"{s}: {kernel} spills registers or lost occupancy: {bad}")

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    # -Bsymbolic: kernel handles are weak global symbols named after the kernel; a generated
    # program loaded into the same process instantiates some of the same templates, and each
    # library must launch through its own handles
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", BACKEND_LIB] + objs + ["-ldl"])


def build_runtime():
    srcs = _sources("host", (".cc",))
    if not srcs:
        return
    _run(["g++", "-O2", "-fPIC", "-std=c++17", "-shared", "-D__HIP_PLATFORM_AMD__",
          "-I", INCLUDE, "-I", "/opt/rocm/include", "-o", RUNTIME_LIB] + srcs +
         ["-L" + HERE, "-lmi355_backend", "-Wl,-rpath,$ORIGIN", "-pthread"])


def build_tools():
    """mirage_profile: loads a graph / checkpoint JSON, fingerprints and times it (the
    reference's cpp_examples/profile.cc)."""
    _run(["g++", "-O2", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I", INCLUDE, "-I", "/opt/rocm/include",
          "-o", os.path.join(HERE, "mirage_profile"), os.path.join(CSRC, "examples", "profile.cc"),
          "-L" + HERE, "-lmirage_runtime", "-lmi355_backend", "-Wl,-rpath,$ORIGIN"])


def build_generated():
    """Generated HIP programs of the example graphs (codegen.py), in a process of their own:
    building the graphs loads the runtime just built, in host-only mode."""
    env = dict(os.environ, MIRAGE_HOST_ONLY="1")
    _run_env([sys.executable, "-m", "attention_superoptimizer_amd.codegen"], env)


def _run_env(cmd, env):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd, env=env, cwd=ROOT)


def main():
    build_backend()
    if os.path.isdir(os.path.join(CSRC, "host")):
        build_runtime()
        build_tools()
        build_generated()
    return 0


if __name__ == "__main__":
    sys.exit(main())
