"""Host-side half of the CPU oracle: thread-block graph construction and lowering.

TEST INFRASTRUCTURE ONLY (see the header of mugraph_oracle.c).  This module
restates, in Python, how the reference turns an ExecutionPlan into a
thread-block graph (shape inference, shared-memory bump allocation, output
discovery) and how it serialises that graph into the flat-int program the
device interpreter walks.  The shipped host library does the same work in
C++; tests compare the two programs int for int.

A plan is a plain dict using the reference's JSON field names
(include/mirage/threadblock/graph.h:28-53):
  grid_dim [x,y,z], block_dim [x,y,z], forloop_range, reduction_dimx,
  input_map [[x,y,z]...], forloop_dim [...], output_map [x,y,z],
  ops [[ "tb_matmul_op", [[op_idx, ts_idx], ...] ], ...]
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

# include/mirage/type.h:79-103
TB_INPUT_OP = 2001
TB_OUTPUT_OP = 2002
TB_MATMUL_OP = 2003
TB_EXP_OP = 2007
TB_ADD_OP = 2008
TB_MUL_OP = 2009
TB_DIV_OP = 2010
TB_SILU_OP = 2012  # extension: absent from the reference
TB_REDUCTION_0_OP = 2101
TB_REDUCTION_0_TO_DIMX_OP = 2104
TB_CONCAT_0_OP = 2200

TB_OP_BY_NAME = {
    "tb_input_op": TB_INPUT_OP,
    "tb_output_op": TB_OUTPUT_OP,
    "tb_matmul_op": TB_MATMUL_OP,
    "tb_exp_op": TB_EXP_OP,
    "tb_add_op": TB_ADD_OP,
    "tb_mul_op": TB_MUL_OP,
    "tb_div_op": TB_DIV_OP,
    "tb_silu_op": TB_SILU_OP,
    "tb_reduction_0_op": 2101,
    "tb_reduction_1_op": 2102,
    "tb_reduction_2_op": 2103,
    "tb_reduction_0_to_dimx_op": 2104,
    "tb_reduction_1_to_dimx_op": 2105,
    "tb_reduction_2_to_dimx_op": 2106,
    "tb_concat_0_op": 2200,
    "tb_concat_1_op": 2201,
    "tb_concat_2_op": 2202,
}

# include/mirage/layout.h:22-45
DMEM_LAYOUT = {"DmemRowMajor": 100, "DmemColumnMajor": 101, "DmemUnknownLayout": 199}
SMEM_LAYOUT = {
    "SmemRowMajor": 200,
    "SmemColumnMajor": 201,
    "SmemRowMajorTensorOpMultiplicand_Crosswise16": 202,
    "SmemRowMajorTensorOpMultiplicand_Crosswise32": 203,
    "SmemRowMajorTensorOpMultiplicand_Crosswise64": 204,
    "SmemColumnMajorTensorOpMultiplicand_Crosswise16": 205,
    "SmemColumnMajorTensorOpMultiplicand_Crosswise32": 206,
    "SmemColumnMajorTensorOpMultiplicand_Crosswise64": 207,
    "SmemUnknownLayout": 299,
}

MAX_SMEM_SIZE = 96 * 1024  # include/mirage/type.h:35


@dataclass
class STensor:
    dims: List[int]
    smem_offset: int
    layout: int = 200
    owner: int = -1  # index of the producing operator in TBGraph.operators

    @property
    def numel(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n

    @property
    def size(self) -> int:  # fp16 / uint16 storage: 2 bytes (smem_tensor.h:108-134)
        return self.numel * 2


@dataclass
class TBOp:
    op_type: int
    inputs: List[STensor] = field(default_factory=list)
    outputs: List[STensor] = field(default_factory=list)
    # input loader
    dtensor_dims: Optional[List[int]] = None
    dtensor_layout: int = 100
    input_map: Optional[Sequence[int]] = None
    forloop_dim: int = -1
    # output saver
    output_map: Optional[Sequence[int]] = None
    out_dtensor_dims: Optional[List[int]] = None


class PlanError(ValueError):
    """The plan is infeasible (the reference would return nullptr / assert)."""


class TBGraph:
    def __init__(self, grid_dim, block_dim, forloop_range, reduction_dimx,
                 smem_limit: int = MAX_SMEM_SIZE):
        self.grid_dim = list(grid_dim)
        self.block_dim = list(block_dim)
        self.forloop_range = int(forloop_range)
        self.reduction_dimx = int(reduction_dimx)
        assert self.reduction_dimx > 0
        self.operators: List[TBOp] = []
        self.smem_offset = 0
        self.smem_limit = smem_limit

    # src/threadblock/graph.cc:43-52
    def _allocate(self, numel: int) -> int:
        ret = self.smem_offset
        self.smem_offset += (numel * 2 + 15) & ~15
        if self.smem_offset > self.smem_limit:
            raise PlanError("shared-memory budget exceeded")
        return ret

    def _push(self, op: TBOp) -> TBOp:
        for t in op.outputs:
            t.owner = len(self.operators)
        self.operators.append(op)
        return op

    # src/threadblock/input_loader.cc:33-140
    def new_input(self, dtensor_dims, dlayout, input_map, forloop_dim, slayout=200) -> STensor:
        dims = list(dtensor_dims)
        for g in range(3):
            if self.grid_dim[g] > 1 and input_map[g] >= 0:
                d = input_map[g]
                if dims[d] <= 0 or dims[d] % self.grid_dim[g] != 0:
                    raise PlanError("grid does not divide input dim")
                dims[d] //= self.grid_dim[g]
        if forloop_dim >= 0:
            if dims[forloop_dim] <= 0 or dims[forloop_dim] % self.forloop_range != 0:
                raise PlanError("forloop_range does not divide input dim")
            dims[forloop_dim] //= self.forloop_range
        for i in range(len(dims) - 2):
            if dims[i] != 1:
                raise PlanError("input tile has a leading dim != 1")
        n = 1
        for d in dims:
            n *= d
        st = STensor(dims, self._allocate(n), slayout)
        self._push(TBOp(TB_INPUT_OP, [], [st], dtensor_dims=list(dtensor_dims),
                        dtensor_layout=dlayout, input_map=list(input_map),
                        forloop_dim=forloop_dim))
        return st

    # src/threadblock/matmul.cc:30-82
    def matmul(self, A: STensor, B: STensor) -> STensor:
        nd = len(A.dims)
        if len(B.dims) != nd or A.dims[-1] != B.dims[-2]:
            raise PlanError("matmul shape mismatch")
        for i in range(nd - 2):
            if A.dims[i] != 1 or B.dims[i] != 1:
                raise PlanError("thread-block matmul cannot be batched")
        dims = list(A.dims)
        dims[-1] = B.dims[-1]
        n = 1
        for d in dims:
            n *= d
        st = STensor(dims, self._allocate(n), 200)
        self._push(TBOp(TB_MATMUL_OP, [A, B], [st]))
        return st

    # src/threadblock/element_unary.cc:36-49 (in place)
    def unary(self, A: STensor, op_type: int) -> STensor:
        st = STensor(list(A.dims), A.smem_offset, A.layout)
        self._push(TBOp(op_type, [A], [st]))
        return st

    # src/threadblock/element_binary.cc:47-93
    def binary(self, A: STensor, B: STensor, op_type: int) -> STensor:
        if len(A.dims) != len(B.dims):
            raise PlanError("binary rank mismatch")
        for a, b in zip(A.dims, B.dims):
            if a != b and a > 1 and b > 1:
                raise PlanError("binary shapes not broadcastable")
        dims = [max(a, b) for a, b in zip(A.dims, B.dims)]
        n = 1
        for d in dims:
            n *= d
        st = STensor(dims, self._allocate(n), A.layout)
        self._push(TBOp(op_type, [A, B], [st]))
        return st

    # src/threadblock/reduction.cc:30-94
    def reduction(self, A: STensor, dim: int, to_dimx: bool) -> STensor:
        if dim >= len(A.dims):
            raise PlanError("reduction dim out of range")
        if not to_dimx and dim < len(A.dims) - 2:
            raise PlanError("plain reduction only on the last two dims")
        dims = list(A.dims)
        size = self.reduction_dimx if to_dimx else 1
        dims[dim] = size
        n = 1
        for d in dims:
            n *= d
        st = STensor(dims, self._allocate(n), A.layout)
        op_type = (TB_REDUCTION_0_TO_DIMX_OP if to_dimx else TB_REDUCTION_0_OP) + dim
        self._push(TBOp(op_type, [A], [st]))
        return st

    # src/threadblock/concat.cc:30-70
    def concat(self, A: STensor, B: STensor, dim: int) -> STensor:
        if len(A.dims) != len(B.dims) or dim >= len(A.dims):
            raise PlanError("concat rank mismatch")
        for i, (a, b) in enumerate(zip(A.dims, B.dims)):
            if i != dim and a != b:
                raise PlanError("concat shape mismatch")
        dims = list(A.dims)
        dims[dim] = A.dims[dim] + B.dims[dim]
        n = 1
        for d in dims:
            n *= d
        st = STensor(dims, self._allocate(n), A.layout)
        self._push(TBOp(TB_CONCAT_0_OP + dim, [A, B], [st]))
        return st

    # src/threadblock/output.cc:39-79
    def new_output(self, S: STensor, output_map) -> List[int]:
        acc = STensor(list(S.dims), self._allocate(S.numel), S.layout)
        ddims = list(S.dims)
        for g in range(3):
            if self.grid_dim[g] > 1 and output_map[g] >= 0:
                ddims[output_map[g]] *= self.grid_dim[g]
        self._push(TBOp(TB_OUTPUT_OP, [S], [acc], output_map=list(output_map),
                        out_dtensor_dims=ddims))
        return ddims


def build_tb_graph(plan: dict, input_dims: Sequence[Sequence[int]],
                   input_layouts: Optional[Sequence[int]] = None,
                   smem_limit: int = MAX_SMEM_SIZE) -> TBGraph:
    """src/kernel/customized.cc:65-186: plan -> thread-block graph."""
    g = TBGraph(plan["grid_dim"], plan.get("block_dim", [128, 1, 1]),
                plan["forloop_range"], plan.get("reduction_dimx", 64), smem_limit)
    n_in = len(plan["input_map"])
    assert len(input_dims) == n_in and len(plan["forloop_dim"]) == n_in
    slay = plan.get("input_smem_layouts") or ["SmemRowMajor"] * n_in
    for i in range(n_in):
        dl = input_layouts[i] if input_layouts else 100
        g.new_input(input_dims[i], dl, plan["input_map"][i], plan["forloop_dim"][i],
                    SMEM_LAYOUT.get(slay[i], 200) if isinstance(slay[i], str) else slay[i])
    for name, idxs in plan["ops"]:
        t = TB_OP_BY_NAME[name] if isinstance(name, str) else int(name)
        ins = [g.operators[a].outputs[b] for a, b in idxs]
        if t == TB_MATMUL_OP:
            g.matmul(ins[0], ins[1])
        elif t in (TB_EXP_OP, TB_SILU_OP):
            g.unary(ins[0], t)
        elif t in (TB_ADD_OP, TB_MUL_OP, TB_DIV_OP):
            g.binary(ins[0], ins[1], t)
        elif 2101 <= t <= 2103:
            g.reduction(ins[0], t - 2101, False)
        elif 2104 <= t <= 2106:
            g.reduction(ins[0], t - 2104, True)
        elif 2200 <= t <= 2202:
            g.concat(ins[0], ins[1], t - 2200)
        else:
            raise PlanError(f"unsupported thread-block operator {name}")
    # customized.cc:147-185: every output tensor of a non-input operator that no
    # later operator consumes becomes a graph output, in operator order
    n_ops = len(g.operators)
    for i in range(n_ops):
        op = g.operators[i]
        if op.op_type == TB_INPUT_OP:
            continue
        for t in op.outputs:
            used = any(u is t for j in range(i + 1, n_ops) for u in g.operators[j].inputs)
            if not used:
                g.new_output(t, plan["output_map"])
    return g


def output_dims(g: TBGraph) -> List[List[int]]:
    return [op.out_dtensor_dims for op in g.operators if op.op_type == TB_OUTPUT_OP]


def lower(g: TBGraph) -> Tuple[List[int], List[int]]:
    """src/threadblock/graph.cc:68-432 -> (operator_types, parameters)."""
    types: List[int] = []
    P: List[int] = []
    F = g.forloop_range
    for op in g.operators:
        types.append(op.op_type)
        t = op.op_type
        if t == TB_INPUT_OP:
            st = op.outputs[0]
            dt = op.dtensor_dims
            nd = len(st.dims)
            R, C = nd - 2, nd - 1
            im, fd = op.input_map, op.forloop_dim
            P += [(st.dims[R] if im[gq] == R else 0) * (F if fd == R else 1) for gq in range(3)]
            P += [(st.dims[C] if im[gq] == C else 0) * (F if fd == C else 1) for gq in range(3)]
            P += [st.dims[R] if fd == R else 0, st.dims[C] if fd == C else 0]
            gb = [0, 0, 0]
            gf = 0
            if nd > 2:
                strides = [0] * nd
                strides[nd - 3] = dt[R] * dt[C]
                for j in range(nd - 4, -1, -1):
                    strides[j] = strides[j + 1] * dt[j + 1]
                for gq in range(3):
                    if 0 <= im[gq] < nd - 2:
                        gb[gq] = strides[im[gq]]
                if 0 <= fd < nd - 2:
                    gf = st.dims[fd] * strides[fd]
            P += gb + [gf]
            P += [dt[R], dt[C], st.dims[R], st.dims[C], op.dtensor_layout, st.layout,
                  st.smem_offset]
        elif t == TB_OUTPUT_OP:
            s_in, acc = op.inputs[0], op.outputs[0]
            dt = op.out_dtensor_dims
            nd = len(s_in.dims)
            R, C = nd - 2, nd - 1
            om = op.output_map
            P += [s_in.dims[R] if om[gq] == R else 0 for gq in range(3)]
            P += [s_in.dims[C] if om[gq] == C else 0 for gq in range(3)]
            gb = [0, 0, 0]
            if nd > 2:
                strides = [0] * nd
                strides[nd - 3] = dt[R] * dt[C]
                for j in range(nd - 4, -1, -1):
                    strides[j] = strides[j + 1] * dt[j + 1]
                for gq in range(3):
                    if 0 <= om[gq] < nd - 2:
                        gb[gq] = strides[om[gq]]
            P += gb
            P += [dt[R], dt[C], s_in.dims[R], s_in.dims[C], 100, s_in.layout,
                  s_in.smem_offset, acc.smem_offset]
        elif t == TB_MATMUL_OP:
            A, B = op.inputs
            Cc = op.outputs[0]
            P += [A.dims[-2], B.dims[-1], A.dims[-1], A.smem_offset, B.smem_offset,
                  Cc.smem_offset]
        elif t in (TB_EXP_OP, TB_SILU_OP):
            P += [op.inputs[0].smem_offset, op.inputs[0].numel]
        elif t in (TB_ADD_OP, TB_MUL_OP, TB_DIV_OP):
            def shape3(s: STensor) -> List[int]:
                d = s.dims
                for i in range(len(d) - 3):
                    assert d[i] == 1
                return [d[-3] if len(d) > 2 else 1, d[-2] if len(d) > 1 else 1, d[-1]]
            P += shape3(op.inputs[0]) + shape3(op.inputs[1])
            P += [op.inputs[0].smem_offset, op.inputs[1].smem_offset, op.outputs[0].smem_offset]
        elif 2101 <= t <= 2106:
            i_t, o_t = op.inputs[0], op.outputs[0]
            rd = (t - 2104) if t >= 2104 else (t - 2101)
            deg = i_t.numel // o_t.numel
            inner = 1
            for i in range(rd, len(o_t.dims)):
                inner *= o_t.dims[i]
            P += [o_t.numel, deg, inner, i_t.smem_offset, o_t.smem_offset]
        elif 2200 <= t <= 2202:
            A, B = op.inputs
            o_t = op.outputs[0]
            cd = t - 2200
            inner = 1
            for i in range(cd + 1, len(o_t.dims)):
                inner *= o_t.dims[i]
            P += [o_t.numel, A.dims[cd], B.dims[cd], inner, A.smem_offset, B.smem_offset,
                  o_t.smem_offset]
        else:
            raise PlanError("unsupported thread-block operator in lowering")
    # kernel_params.h:26-29 limits; graph.cc:421-430 ordering invariants
    n_in = sum(1 for x in types if x == TB_INPUT_OP)
    n_out = sum(1 for x in types if x == TB_OUTPUT_OP)
    if len(types) > 16 or len(P) > 120 or n_in > 4 or n_out > 4:
        raise PlanError("program exceeds NewKernelParams limits")
    assert all(x == TB_INPUT_OP for x in types[:n_in])
    assert all(x == TB_OUTPUT_OP for x in types[len(types) - n_out:])
    return types, P
