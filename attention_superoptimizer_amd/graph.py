"""Python mirror of the mirage:: host API (the reference's PyGraph,
python/mirage/_cython/core.pyx:180-236), bound over the C facade with ctypes.

    g = KNGraph()
    Q = g.new_input((2, 256, 64)); K = g.new_input((2, 64, 4096)); ...
    out, = g.customized([Q, K, V], plan)      # plan: dict, see workloads.py
    g.fingerprint_all(); g.operators ...
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import _native as N

DT_FLOAT16 = 921
DMEM_LAYOUT = {"DmemRowMajor": 100, "DmemColumnMajor": 101}
SMEM_LAYOUT = {
    "SmemRowMajor": 200, "SmemColumnMajor": 201,
    "SmemRowMajorTensorOpMultiplicand_Crosswise16": 202,
    "SmemRowMajorTensorOpMultiplicand_Crosswise32": 203,
    "SmemRowMajorTensorOpMultiplicand_Crosswise64": 204,
    "SmemColumnMajorTensorOpMultiplicand_Crosswise16": 205,
    "SmemColumnMajorTensorOpMultiplicand_Crosswise32": 206,
    "SmemColumnMajorTensorOpMultiplicand_Crosswise64": 207,
    "SmemUnknownLayout": 299,
}
KN_OP = {"exp": 1007, "add": 1008, "mul": 1009, "div": 1010, "silu": 1011}
TB_OP = {
    "tb_matmul_op": 2003, "tb_exp_op": 2007, "tb_add_op": 2008, "tb_mul_op": 2009,
    "tb_div_op": 2010, "tb_silu_op": 2012,
    "tb_reduction_0_op": 2101, "tb_reduction_1_op": 2102, "tb_reduction_2_op": 2103,
    "tb_reduction_0_to_dimx_op": 2104, "tb_reduction_1_to_dimx_op": 2105,
    "tb_reduction_2_to_dimx_op": 2106,
    "tb_concat_0_op": 2200, "tb_concat_1_op": 2201, "tb_concat_2_op": 2202,
}


class InfeasibleOperator(RuntimeError):
    """create_* returned nullptr: shapes disagree or a budget is exhausted."""


def set_smem_budget(nbytes: int) -> None:
    """threadblock::Graph::set_smem_budget."""
    N.runtime().mirage_set_smem_budget(int(nbytes))


def device_ready() -> bool:
    return bool(N.runtime().mirage_device_ready())


class DTensor:
    """Handle of a mirage::kernel::DTensor owned by an operator of a KNGraph."""

    def __init__(self, handle: int):
        self._h = ctypes.c_void_p(handle)
        nd, dt, lay = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        dims = (ctypes.c_int * 4)()
        guid = ctypes.c_longlong()
        N.runtime().mirage_tensor_info(self._h, nd, dims, dt, lay, guid)
        self.dims = tuple(dims[i] for i in range(nd.value))
        self.data_type, self.guid = dt.value, guid.value

    @property
    def layout(self) -> int:
        """The tensor's DmemLayout now (a layout search may have changed it)."""
        nd, dt, lay = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        dims = (ctypes.c_int * 4)()
        guid = ctypes.c_longlong()
        N.runtime().mirage_tensor_info(self._h, nd, dims, dt, lay, guid)
        return lay.value

    @property
    def num_elements(self) -> int:
        return int(np.prod(self.dims))

    def device_ptr(self, fingerprint: bool) -> int:
        return N.runtime().mirage_tensor_ptr(self._h, 1 if fingerprint else 0)

    def write_fingerprint(self, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a, dtype=np.uint16)
        assert a.size == self.num_elements
        rc = N.runtime().mirage_tensor_write(self._h, 1, a.ctypes.data_as(ctypes.c_void_p), a.nbytes)
        assert rc == 0, N.last_error()

    def read_fingerprint(self) -> np.ndarray:
        a = np.empty(self.dims, np.uint16)
        rc = N.runtime().mirage_tensor_read(self._h, 1, a.ctypes.data_as(ctypes.c_void_p), a.nbytes)
        assert rc == 0, N.last_error()
        return a

    @property
    def column_major(self) -> bool:
        return self.layout == DMEM_LAYOUT["DmemColumnMajor"] and len(self.dims) >= 2

    def write_data(self, a: np.ndarray) -> None:
        """Uploads the LOGICAL values `a` (shape = dims).  The fp16 buffer of a DmemColumnMajor
        tensor holds each [rows, cols] matrix column by column, as the reference's fp16 loader
        reads it (include/mirage/threadblock/cuda/input_loader.h:221-247); the fingerprint
        buffer is row-major whatever the layout (input_loader.h:457-467)."""
        a = np.asarray(a, dtype=np.float16)
        assert a.size == self.num_elements
        a = a.reshape(self.dims)
        if self.column_major:
            a = a.swapaxes(-1, -2)
        a = np.ascontiguousarray(a)
        rc = N.runtime().mirage_tensor_write(self._h, 0, a.ctypes.data_as(ctypes.c_void_p), a.nbytes)
        assert rc == 0, N.last_error()

    def read_data(self) -> np.ndarray:
        """The logical values (shape = dims), whatever the buffer's layout."""
        dims = list(self.dims)
        if self.column_major:
            dims[-1], dims[-2] = dims[-2], dims[-1]
        a = np.empty(dims, np.float16)
        rc = N.runtime().mirage_tensor_read(self._h, 0, a.ctypes.data_as(ctypes.c_void_p), a.nbytes)
        assert rc == 0, N.last_error()
        return np.ascontiguousarray(a.swapaxes(-1, -2)) if self.column_major else a

    def has_same_fingerprint(self, other: "DTensor") -> bool:
        return bool(N.runtime().mirage_tensor_same_fingerprint(self._h, other._h))


def _c_plan(plan: dict) -> N.MirageCPlan:
    p = N.MirageCPlan()
    n_in = len(plan["input_map"])
    assert n_in <= 4 and len(plan["ops"]) <= 16
    for i in range(3):
        p.grid_dim[i] = plan["grid_dim"][i]
        p.block_dim[i] = plan.get("block_dim", [128, 1, 1])[i]
        p.output_map[i] = plan["output_map"][i]
    p.forloop_range = plan["forloop_range"]
    p.reduction_dimx = plan.get("reduction_dimx", 64)
    p.num_inputs = n_in
    lay = plan.get("input_smem_layouts") or ["SmemRowMajor"] * n_in
    for i in range(n_in):
        for j in range(3):
            p.input_map[i][j] = plan["input_map"][i][j]
        p.forloop_dim[i] = plan["forloop_dim"][i]
        p.input_smem_layout[i] = SMEM_LAYOUT[lay[i]] if isinstance(lay[i], str) else int(lay[i])
    p.num_ops = len(plan["ops"])
    for i, (name, operands) in enumerate(plan["ops"]):
        p.op_type[i] = TB_OP[name] if isinstance(name, str) else int(name)
        assert len(operands) <= 2
        p.op_num_operands[i] = len(operands)
        for j, (a, b) in enumerate(operands):
            p.op_operands[i][j][0] = a
            p.op_operands[i][j][1] = b
    return p


class KNGraph:
    """mirage::kernel::Graph."""

    def __init__(self, _handle=None):
        self._rt = N.runtime()
        self._g = ctypes.c_void_p(_handle if _handle is not None else self._rt.mirage_graph_create())

    @classmethod
    def from_json(cls, text) -> "KNGraph":
        """from_json(json, Graph) of the reference (src/kernel/graph.cc:39-159): rebuilds a
        kernel graph from its JSON wire format (a str, or an already decoded list)."""
        import json as _json
        if not isinstance(text, str):
            text = _json.dumps(text)
        h = N.runtime().mirage_graph_from_json(text.encode())
        if not h:
            raise ValueError("malformed mugraph JSON")
        return cls(_handle=h)

    def generate_hip_program(self, path: str) -> None:
        """Graph::generate_hip_program: writes a self-contained HIP program (one specialised
        gfx950 kernel per customized operator, a launcher, a timing main) -- this backend's
        counterpart of the reference's generate_triton_program
        (src/kernel/triton_code_gen.cc:354-450)."""
        assert self._rt.mirage_graph_generate_hip_program(self._g, path.encode()) == 0

    def to_json(self) -> str:
        """to_json(json, Graph) (src/kernel/graph.cc:33-37), one line, sorted keys."""
        n = self._rt.mirage_graph_to_json(self._g, None, 0)
        buf = ctypes.create_string_buffer(n + 1)
        self._rt.mirage_graph_to_json(self._g, buf, n + 1)
        return buf.value.decode()

    def close(self):
        if self._g is not None:
            self._rt.mirage_graph_destroy(self._g)
            self._g = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        # graphs share one LIFO arena: destruction order is the caller's business
        pass

    def _wrap(self, handle, what) -> DTensor:
        if not handle:
            raise InfeasibleOperator(what)
        return DTensor(handle)

    @property
    def num_operators(self) -> int:
        return self._rt.mirage_graph_num_operators(self._g)

    def new_input(self, dims: Sequence[int], dtype: int = DT_FLOAT16,
                  layout: str = "DmemRowMajor") -> DTensor:
        d = (ctypes.c_int * len(dims))(*dims)
        return self._wrap(self._rt.mirage_graph_new_input(self._g, d, len(dims), dtype,
                                                          DMEM_LAYOUT[layout]), "new_input")

    def matmul(self, A: DTensor, B: DTensor) -> DTensor:
        return self._wrap(self._rt.mirage_graph_matmul(self._g, A._h, B._h), "matmul")

    def _unary(self, name, A):
        return self._wrap(self._rt.mirage_graph_unary(self._g, KN_OP[name], A._h), name)

    def _binary(self, name, A, B):
        return self._wrap(self._rt.mirage_graph_binary(self._g, KN_OP[name], A._h, B._h), name)

    def exp(self, A): return self._unary("exp", A)
    def silu(self, A): return self._unary("silu", A)
    def add(self, A, B): return self._binary("add", A, B)
    def mul(self, A, B): return self._binary("mul", A, B)
    def div(self, A, B): return self._binary("div", A, B)

    def reduction(self, A: DTensor, dim: int, size: int = 1) -> DTensor:
        return self._wrap(self._rt.mirage_graph_reduction(self._g, A._h, dim, size), "reduction")

    def customized(self, inputs: List[DTensor], plan: dict) -> List[DTensor]:
        cp = _c_plan(plan)
        ins = (ctypes.c_void_p * len(inputs))(*[t._h for t in inputs])
        outs = (ctypes.c_void_p * 4)()
        n = self._rt.mirage_graph_customized(self._g, ins, len(inputs), ctypes.byref(cp), outs, 4)
        if n < 0:
            raise InfeasibleOperator("customized")
        return [DTensor(outs[i]) for i in range(n)]

    def pop_operator(self) -> None:
        assert self._rt.mirage_graph_pop_operator(self._g) == 0

    # ---- per-operator device work ------------------------------------------------
    def op_type(self, idx: int) -> int:
        return self._rt.mirage_op_type(self._g, idx)

    def outputs(self, idx: int) -> List[DTensor]:
        n = self._rt.mirage_op_num_outputs(self._g, idx)
        return [DTensor(self._rt.mirage_op_output(self._g, idx, j)) for j in range(n)]

    def fingerprint(self, idx: int) -> None:
        assert self._rt.mirage_op_fingerprint(self._g, idx) == 0

    def fingerprint_all(self, skip_inputs: bool = False) -> None:
        """op->fingerprint() for every operator, as the reference's verify loop does
        (src/search/search.cc:601-603)."""
        for i in range(self.num_operators):
            if skip_inputs and self.op_type(i) == 1001:
                continue
            self.fingerprint(i)

    def fingerprint_seeded(self, input_seed: int) -> dict:
        """fingerprint() of every operator; input number j holds uniform values drawn
        from (input_seed, j) when input_seed != 0, `idx % 25651` otherwise."""
        st = N.MirageVerifyStats()
        assert self._rt.mirage_graph_fingerprint(self._g, input_seed, ctypes.byref(st)) == 0
        return _stats(st)

    def execute(self, idx: int) -> None:
        assert self._rt.mirage_op_execute(self._g, idx) == 0

    def execute_all(self) -> None:
        for i in range(self.num_operators):
            self.execute(i)

    def profile(self, idx: int) -> float:
        """Mean milliseconds per launch (reference profile() protocol)."""
        return float(self._rt.mirage_op_profile(self._g, idx))

    def profile_all(self):
        """What the reference's cpp_examples/profile.cc does with a graph (:25-34):
        fingerprint() of every operator, then profile() of every operator.  Returns
        (sum of the mean milliseconds per launch, per-operator list)."""
        n = self.num_operators
        per_op = (ctypes.c_float * n)()
        total = float(self._rt.mirage_graph_profile(self._g, per_op, n))
        return total, [float(per_op[i]) for i in range(n)]

    def lowered(self, idx: int, fingerprint: bool = True) -> N.Mi355Plan:
        p = N.Mi355Plan()
        rc = self._rt.mirage_op_lowered(self._g, idx, 1 if fingerprint else 0, ctypes.byref(p), None)
        assert rc == 0
        return p


class Checkpoint:
    """A search checkpoint (reference include/mirage/search/search.h:46-68) or a single graph
    file, loaded by the host runtime: the computation graph, the generated graphs in wire
    format, best_profile_result, config / callstack (uninterpreted) and the counters."""

    def __init__(self, handle):
        self._rt = N.runtime()
        self._h = ctypes.c_void_p(handle)
        counters = (ctypes.c_longlong * 3)()
        self.best_run_time = float(self._rt.mirage_checkpoint_summary(self._h, counters))
        self.counters = tuple(int(c) for c in counters)
        self.num_graphs = int(self._rt.mirage_checkpoint_num_graphs(self._h))

    @classmethod
    def load(cls, path: str) -> "Checkpoint":
        h = N.runtime().mirage_checkpoint_load(os.fsencode(path))
        if not h:
            raise ValueError(f"cannot load a checkpoint or graph from {path}")
        return cls(h)

    def graph_json(self, index: int) -> str:
        """-2: the whole checkpoint, -1: the computation graph, i >= 0: generated graph i."""
        n = self._rt.mirage_checkpoint_json(self._h, index, None, 0)
        if n < 0:
            raise IndexError(index)
        buf = ctypes.create_string_buffer(n + 1)
        self._rt.mirage_checkpoint_json(self._h, index, buf, n + 1)
        return buf.value.decode()

    def to_json(self) -> str:
        return self.graph_json(-2)

    def graph(self, index: int) -> "KNGraph":
        return KNGraph.from_json(self.graph_json(index))

    def close(self):
        if self._h is not None:
            self._rt.mirage_checkpoint_destroy(self._h)
            self._h = None


def _stats(st) -> dict:
    return {"kernel_ops": st.kernel_ops, "customized_ops": st.customized_ops,
            "compares": st.compares, "fp_bytes": st.fp_bytes, "matmul_macs": st.matmul_macs,
            "enqueue_seconds": st.enqueue_seconds, "wait_seconds": st.wait_seconds}


def optimize_layout(graph: "KNGraph", cost=None, max_assignments: int = 0) -> dict:
    """KernelGraphGenerator::optimize_layout (reference src/search/search.cc:699-777):
    enumerates the layouts of every kernel-level output tensor and of every tile inside
    the customized operators, costs each complete assignment and leaves `graph` under the
    cheapest one.  `cost(op_index, layouts) -> ms` replaces the measurement by
    KNOperator::profile (which needs the device); `layouts` are the ones the operator's cost
    may depend on: DmemLayout values of the device tensors it reads, then of those it writes,
    then SmemLayout values of its loaders' tiles (none for an input operator).  Device tensors
    whose layout changed hold their old contents in the old order: write their data again."""
    st = N.MirageLayoutStats()
    if cost is None:
        cb = N.LAYOUT_COST_FN()
    else:
        cb = N.LAYOUT_COST_FN(lambda user, op, lay, n: float(cost(op, [lay[i] for i in range(n)])))
    rc = N.runtime().mirage_optimize_layout(graph._g, max_assignments, cb, None, ctypes.byref(st))
    assert rc == 0
    return {"assignments": st.assignments, "measurements": st.measurements,
            "unrunnable": st.unrunnable, "truncated": bool(st.truncated), "first_ms": st.first_ms, "best_ms": st.best_ms,
            "worst_ms": st.worst_ms}


def verify_batch(candidates: Sequence["KNGraph"], reference: "KNGraph", input_seed: int = 0):
    """Batched KernelGraphGenerator::verify (reference src/search/search.cc:569-623):
    fingerprints every candidate and compares its outputs with the (already
    fingerprinted) outputs of `reference` on the device, one synchronisation for the
    whole batch.  Returns (list of bool, stats)."""
    n = len(candidates)
    arr = (ctypes.c_void_p * n)(*[c._g for c in candidates])
    eq = (ctypes.c_ubyte * n)()
    st = N.MirageVerifyStats()
    rc = N.runtime().mirage_verify_batch(arr, n, reference._g, input_seed, eq, ctypes.byref(st))
    assert rc == 0
    return [bool(eq[i]) for i in range(n)], _stats(st)


def verify_batch_begin(candidates: Sequence["KNGraph"], reference: "KNGraph", input_seed: int = 0,
                       fingerprint_reference: bool = True):
    """First half of verify_batch: lowers and enqueues everything from the runtime's worker
    threads and returns a ticket at once, so that the caller can build and submit the next
    batch while the device works on this one.  With `fingerprint_reference` the reference
    graph is fingerprinted as part of the batch.  The graphs must stay open until
    verify_batch_end(ticket) has returned."""
    n = len(candidates)
    arr = (ctypes.c_void_p * n)(*[c._g for c in candidates])
    handle = N.runtime().mirage_verify_batch_begin(arr, n, reference._g, input_seed,
                                                   1 if fingerprint_reference else 0)
    assert handle
    return (handle, n)


def set_verify_queues_per_batch(queues: int) -> None:
    """How many backend queues a verification batch is dealt over (default: all four).  With
    several batches in flight, fewer queues per batch put more candidates into every launch."""
    N.runtime().mirage_verify_set_queues_per_batch(queues)


def verify_batch_end(ticket):
    """Second half: waits for this batch's compares only.  Returns (list of bool, stats)."""
    handle, n = ticket
    eq = (ctypes.c_ubyte * n)()
    st = N.MirageVerifyStats()
    rc = N.runtime().mirage_verify_batch_end(handle, n, eq, ctypes.byref(st))
    assert rc == 0
    return [bool(eq[i]) for i in range(n)], _stats(st)


def build_from_spec(spec: List[dict], graph: Optional[KNGraph] = None):
    """Builds a graph spec (see workloads.py) through the host API.
    Returns (graph, per-operator lists of output tensors)."""
    g = graph or KNGraph()
    vals: List[List[DTensor]] = []

    def get(ref):
        return vals[ref[0]][ref[1]]

    for op in spec:
        k = op["op"]
        if k == "input":
            vals.append([g.new_input(op["dims"], DT_FLOAT16, op.get("layout", "DmemRowMajor"))])
        elif k == "matmul":
            vals.append([g.matmul(get(op["in"][0]), get(op["in"][1]))])
        elif k in ("exp", "silu"):
            vals.append([g._unary(k, get(op["in"][0]))])
        elif k in ("add", "mul", "div"):
            vals.append([g._binary(k, get(op["in"][0]), get(op["in"][1]))])
        elif k == "reduction":
            vals.append([g.reduction(get(op["in"][0]), op["dim"], op.get("size", 1))])
        elif k == "customized":
            vals.append(g.customized([get(r) for r in op["in"]], op["plan"]))
        else:
            raise ValueError(k)
    return g, vals
