"""Graph-level driver of the CPU oracle (ctypes over mugraph_oracle.c).

TEST INFRASTRUCTURE ONLY.  Evaluates a whole kernel graph — kernel-level ops
and customized ops — either over the fingerprint ring Z_25651 (uint16) or as
the fp16 golden (fp32 arithmetic, one fp16 rounding per stored element).

Graph spec = list of kernel ops, each a dict:
  {"op": "input", "dims": [...], "layout": "DmemRowMajor"}
  {"op": "matmul" | "exp" | "silu" | "add" | "mul" | "div", "in": [[op, ts], ...]}
  {"op": "reduction", "in": [[op, ts]], "dim": d, "size": s}
  {"op": "customized", "in": [[op, ts], ...], "plan": {...}}      (plan: see lowering.py)
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import lowering

FP_PQ = 25651
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmugraph_oracle.so")
_lib = None

KN_BINARY = {"add": 1008, "mul": 1009, "div": 1010}


def build(force: bool = False) -> str:
    """Compile the C restatement with gcc (scalar, -O2, no vectorisation pragmas)."""
    src = os.path.join(_HERE, "mugraph_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-fPIC", "-shared", "-o", _LIB_PATH, src,
                               "-lpthread", "-lm"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        L.orc_build_tables.argtypes = [vp, vp, vp]
        L.orc_fp_input.argtypes = [vp, sz]
        L.orc_fp_matmul.argtypes = [vp, vp, vp, ci, ci, ci, ci]
        L.orc_fp_exp.argtypes = [vp, vp, sz]
        L.orc_fp_silu.argtypes = [vp, vp, sz]
        L.orc_fp_binary.argtypes = [ci, vp, vp, vp, vp, vp, vp, ci]
        L.orc_fp_reduce.argtypes = [vp, vp, sz, ci, ci, ci]
        L.orc_fp_equal.argtypes = [vp, vp, sz]
        L.orc_fp_equal.restype = ci
        L.orc_f16_matmul.argtypes = [vp, vp, vp, ci, ci, ci, ci]
        L.orc_f16_to_f32.argtypes = [vp, vp, sz]
        L.orc_f32_to_f16.argtypes = [vp, vp, sz]
        L.orc_customized.argtypes = [ci, ci, vp, vp, vp, ci, ci, vp, ci, vp, ci, ci, ci]
        L.orc_customized.restype = ci
        L.orc_customized_blocks.argtypes = [ci, ci, vp, vp, vp, ci, ci, vp, ci, vp, ci, ci, ci, vp, ci]
        L.orc_customized_blocks.restype = ci
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def tables():
    e = np.zeros(113, np.uint16)
    p = np.zeros(227, np.uint16)
    q = np.zeros(113, np.uint16)
    lib().orc_build_tables(_p(e), _p(p), _p(q))
    return e, p, q


def fp_input(dims: Sequence[int]) -> np.ndarray:
    a = np.zeros(int(np.prod(dims)), np.uint16)
    lib().orc_fp_input(_p(a), a.size)
    return a.reshape(dims)


def fp_matmul(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    m, k, n = A.shape[-2], A.shape[-1], B.shape[-1]
    batch = int(np.prod(A.shape[:-2])) if A.ndim > 2 else 1
    C = np.zeros(A.shape[:-1] + (n,), np.uint16)
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    lib().orc_fp_matmul(_p(A), _p(B), _p(C), batch, m, n, k)
    return C


def fp_unary(name: str, A: np.ndarray) -> np.ndarray:
    A = np.ascontiguousarray(A)
    out = np.zeros_like(A)
    getattr(lib(), "orc_fp_" + name)(_p(A), _p(out), A.size)
    return out


def fp_binary(name: str, A: np.ndarray, B: np.ndarray) -> np.ndarray:
    nd = A.ndim
    od = tuple(max(a, b) for a, b in zip(A.shape, B.shape))
    out = np.zeros(od, np.uint16)
    d1 = np.array(A.shape, np.int32)
    d2 = np.array(B.shape, np.int32)
    d3 = np.array(od, np.int32)
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    lib().orc_fp_binary(KN_BINARY[name], _p(A), _p(d1), _p(B), _p(d2), _p(out), _p(d3), nd)
    return out


def fp_reduce(A: np.ndarray, dim: int, size: int = 1) -> np.ndarray:
    """src/kernel/cuda/reduction_kernel.cu:110-133 (host half) + kernel."""
    od = list(A.shape)
    od[dim] = size
    out = np.zeros(od, np.uint16)
    out_stride = int(np.prod(od[dim:]))
    in_stride = int(np.prod(A.shape[dim:]))
    factor = A.shape[dim] // size
    A = np.ascontiguousarray(A)
    lib().orc_fp_reduce(_p(A), _p(out), out.size, factor, in_stride, out_stride)
    return out


UNTOUCHED = 0xFFFF  # not a fingerprint (>= 25651); as fp16 bits, a NaN no golden here produces


def customized(plan: dict, inputs: List[np.ndarray], f16: bool = False, threads: int = 1,
               smem_limit: int = 1 << 30, input_layouts=None, blocks=None) -> List[np.ndarray]:
    """One customized op: build + lower the thread-block graph, run the C interpreter.

    `blocks`: linear thread-block indices bx + grid.x * (by + grid.y * bz) to run instead of
    the whole grid; output elements no listed block writes hold UNTOUCHED (see written())."""
    g = lowering.build_tb_graph(plan, [list(a.shape) for a in inputs], input_layouts, smem_limit)
    types, params = lowering.lower(g)
    fill = 0 if blocks is None else UNTOUCHED
    outs = [np.full(d, fill, np.uint16) for d in lowering.output_dims(g)]
    ins = [np.ascontiguousarray(a.view(np.uint16) if a.dtype == np.float16 else a) for a in inputs]
    run_program(types, params, g.grid_dim, g.forloop_range, g.smem_offset, ins, outs, f16, threads,
                blocks)
    return outs


def written(out: np.ndarray) -> np.ndarray:
    """Mask of the elements a block-subset run of customized() produced."""
    return out.view(np.uint16) != UNTOUCHED


def run_program(types, params, grid, forloop_range, smem_bytes, ins, outs, f16=False, threads=1,
                blocks=None):
    t_arr = np.array(types, np.int32)
    p_arr = np.array(params, np.int32)
    g_arr = np.array(grid, np.int32)
    in_ptrs = (ctypes.c_void_p * 4)(*[a.ctypes.data for a in ins])
    out_ptrs = (ctypes.c_void_p * 4)(*[a.ctypes.data for a in outs])
    b_arr = None if blocks is None else np.ascontiguousarray(blocks, dtype=np.int32)
    rc = lib().orc_customized_blocks(len(types), len(params), _p(t_arr), _p(p_arr), _p(g_arr),
                                     int(forloop_range), int(smem_bytes), in_ptrs, len(ins),
                                     out_ptrs, len(outs), 1 if f16 else 0, int(threads),
                                     None if b_arr is None else _p(b_arr),
                                     0 if b_arr is None else int(b_arr.size))
    assert rc == 0


# ---- fp16 golden, kernel-level ops (fp32 math, one rounding per element) ----
def f16_matmul(A, B):
    return np.matmul(A.astype(np.float32), B.astype(np.float32)).astype(np.float16)


def f16_unary(name, A):
    x = A.astype(np.float32)
    with np.errstate(over="ignore"):
        y = np.exp(x) if name == "exp" else x / (1.0 + np.exp(-x))
    return y.astype(np.float16)


def f16_binary(name, A, B):
    x, y = A.astype(np.float32), B.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        z = {"add": np.add, "mul": np.multiply, "div": np.divide}[name](x, y)
    return z.astype(np.float16)


def strided_reduce(x: np.ndarray, dim: int, size: int) -> np.ndarray:
    """out[..., j, ...] = sum_k in[..., j + k*size, ...] — the `inner_range` rule of
    reduction_kernel.cu:86-107 / reduction.h:147-156 written with a reshape."""
    shp = list(x.shape)
    f = shp[dim] // size
    return x.reshape(shp[:dim] + [f, size] + shp[dim + 1:]).sum(axis=dim)


def f16_reduce(A, dim, size=1):
    return strided_reduce(A.astype(np.float32), dim, size).astype(np.float16)


def eval_graph(graph: List[dict], mode: str = "fp", inputs: Optional[Dict[int, np.ndarray]] = None,
               threads: int = 1) -> List[List[np.ndarray]]:
    """Evaluate every op; returns per-op lists of output arrays.

    mode "fp": uint16 ring arithmetic; inputs default to idx % 25651
    (src/kernel/cuda/input_kernel.cu:56-61).  mode "f16": fp16 golden; inputs
    (float16 arrays keyed by op index) are required.
    """
    f16 = mode == "f16"
    vals: List[List[np.ndarray]] = []

    def get(ref):
        return vals[ref[0]][ref[1]]

    for i, op in enumerate(graph):
        k = op["op"]
        if k == "input":
            if inputs is not None and i in inputs:
                a = np.asarray(inputs[i]).reshape(op["dims"])
            else:
                assert not f16, "fp16 golden needs explicit inputs"
                a = fp_input(op["dims"])
            vals.append([a])
        elif k == "matmul":
            A, B = (get(r) for r in op["in"])
            vals.append([f16_matmul(A, B) if f16 else fp_matmul(A, B)])
        elif k in ("exp", "silu"):
            A = get(op["in"][0])
            vals.append([f16_unary(k, A) if f16 else fp_unary(k, A)])
        elif k in ("add", "mul", "div"):
            A, B = (get(r) for r in op["in"])
            vals.append([f16_binary(k, A, B) if f16 else fp_binary(k, A, B)])
        elif k == "reduction":
            A = get(op["in"][0])
            sz = op.get("size", 1)
            vals.append([f16_reduce(A, op["dim"], sz) if f16 else fp_reduce(A, op["dim"], sz)])
        elif k == "customized":
            ins = [get(r) for r in op["in"]]
            outs = customized(op["plan"], ins, f16=f16, threads=threads)
            if f16:
                outs = [o.view(np.float16) for o in outs]
            vals.append(outs)
        else:
            raise ValueError(k)
    return vals
