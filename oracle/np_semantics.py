"""Second, independent statement of mugraph semantics in numpy.

TEST INFRASTRUCTURE ONLY.  Where mugraph_oracle.c + lowering.py follow the
reference's *mechanism* (flat-int program, strides, shared-memory offsets),
this module states the *meaning* of a customized op directly on array slices:
block (bx,by,bz) owns the bx-th / by-th / bz-th part of every input along the
dims its input_map names, for-loop iteration i owns the i-th part of that along
forloop_dim, ops act on whole tiles, outputs accumulate over iterations and
land in the block's part of the output along output_map.  Integer arithmetic is
done exactly (float64 BLAS on integers < 2^53, then one modulus), so agreement
with the C transcription also checks that its per-step `%` is a ring
homomorphism.  Plans in which one tensor dim is split by two grid dims, or a
leading (batch) dim is split by both a grid dim and the for-loop, are rejected:
the reference's stride rule for them does not describe a partition.
"""
from __future__ import annotations

from typing import List

import numpy as np

FP_P, FP_Q, FP_PQ = 227, 113, 25651


def _tables():
    e = [1]
    for _ in range(112):
        e.append(e[-1] * 3 % FP_P)
    divp = [1] + [pow(i, FP_P - 2, FP_P) for i in range(1, FP_P)]
    divq = [1] + [pow(i, FP_Q - 2, FP_Q) for i in range(1, FP_Q)]
    return np.array(e, np.int64), np.array(divp, np.int64), np.array(divq, np.int64)


_EXP, _DIVP, _DIVQ = _tables()


class Ring:
    """Z_25651 with the reference's exp / div conventions."""

    @staticmethod
    def matmul(a, b):
        return np.rint(np.matmul(a.astype(np.float64), b.astype(np.float64))).astype(np.int64) % FP_PQ

    @staticmethod
    def exp(a):
        return (_EXP[a % FP_Q] * 25425) % FP_PQ

    @staticmethod
    def div(a, b):
        return ((a % FP_P) * _DIVP[b % FP_P] * 25425 + (a % FP_Q) * _DIVQ[b % FP_Q] * 227) % FP_PQ

    @staticmethod
    def add(a, b):
        return (a + b) % FP_PQ

    @staticmethod
    def mul(a, b):
        return (a * b) % FP_PQ

    @classmethod
    def silu(cls, a):
        return cls.div(a, (1 + cls.exp((FP_PQ - a) % FP_PQ)) % FP_PQ)

    @staticmethod
    def sum(a, axis):
        return a.sum(axis=axis) % FP_PQ

    @staticmethod
    def store(a):
        return a

    zero_accum = None
    dtype = np.int64


class Half:
    """fp16 golden: fp32 math, one fp16 rounding per materialised tensor."""

    @staticmethod
    def _r(x):
        return x.astype(np.float16).astype(np.float32)

    @classmethod
    def matmul(cls, a, b):
        return cls._r(np.matmul(a, b))

    @classmethod
    def exp(cls, a):
        with np.errstate(over="ignore"):
            return cls._r(np.exp(a))

    @classmethod
    def silu(cls, a):
        with np.errstate(over="ignore"):
            return cls._r(a / (1.0 + np.exp(-a)))

    @classmethod
    def div(cls, a, b):
        with np.errstate(divide="ignore", invalid="ignore"):
            return cls._r(a / b)

    @classmethod
    def add(cls, a, b):
        return cls._r(a + b)

    @classmethod
    def mul(cls, a, b):
        return cls._r(a * b)

    @classmethod
    def sum(cls, a, axis):
        return cls._r(a.sum(axis=axis, dtype=np.float32))

    dtype = np.float32


def _part(x, dim, nparts, idx):
    n = x.shape[dim] // nparts
    sl = [slice(None)] * x.ndim
    sl[dim] = slice(idx * n, (idx + 1) * n)
    return x[tuple(sl)]


def customized(plan: dict, inputs: List[np.ndarray], f16: bool = False) -> List[np.ndarray]:
    A = Half if f16 else Ring
    grid = plan["grid_dim"]
    F = plan["forloop_range"]
    dimx = plan.get("reduction_dimx", 64)
    n_in = len(inputs)
    xs = [np.asarray(a).astype(A.dtype) for a in inputs]
    outs = None
    for i in range(n_in):
        im, fd, nd = plan["input_map"][i], plan["forloop_dim"][i], xs[i].ndim
        used = [im[g] for g in range(3) if grid[g] > 1 and im[g] >= 0]
        if len(set(used)) != len(used):
            raise NotImplementedError("one dim split by two grid dims")
        if 0 <= fd < nd - 2 and fd in used:
            raise NotImplementedError("batch dim split by grid and for-loop")
    for bz in range(grid[2]):
        for by in range(grid[1]):
            for bx in range(grid[0]):
                b = (bx, by, bz)
                accs = None
                for it in range(F):
                    vals = []  # vals[op_idx] = [tensor]
                    for i in range(n_in):
                        t = xs[i]
                        im, fd = plan["input_map"][i], plan["forloop_dim"][i]
                        for g in range(3):
                            if grid[g] > 1 and im[g] >= 0:
                                t = _part(t, im[g], grid[g], b[g])
                        if fd >= 0:
                            t = _part(t, fd, F, it)
                        vals.append([t])
                    consumed = set()
                    for name, idxs in plan["ops"]:
                        ins = [vals[a][c] for a, c in idxs]
                        for a, c in idxs:
                            consumed.add((a, c))
                        if name == "tb_matmul_op":
                            r = A.matmul(ins[0], ins[1])
                        elif name in ("tb_exp_op", "tb_silu_op"):
                            r = getattr(A, name[3:-3])(ins[0])
                        elif name in ("tb_add_op", "tb_mul_op", "tb_div_op"):
                            r = getattr(A, name[3:-3])(ins[0], ins[1])
                        elif name.startswith("tb_reduction_"):
                            d = int(name[len("tb_reduction_")])
                            size = dimx if name.endswith("to_dimx_op") else 1
                            x = ins[0]
                            shp = list(x.shape)
                            f = shp[d] // size
                            r = A.sum(x.reshape(shp[:d] + [f, size] + shp[d + 1:]), axis=d)
                        elif name.startswith("tb_concat_"):
                            d = int(name[len("tb_concat_")])
                            r = np.concatenate(ins, axis=d)
                        else:
                            raise ValueError(name)
                        vals.append([r])
                    produced = [(j, 0) for j in range(n_in, len(vals))]
                    finals = [vals[j][c] for j, c in produced if (j, c) not in consumed]
                    if accs is None:
                        accs = [A.add(np.zeros_like(x), x) if f16 else x for x in finals]
                    else:
                        accs = [A.add(a, x) for a, x in zip(accs, finals)]
                if outs is None:
                    outs = []
                    for a in accs:
                        shp = list(a.shape)
                        for g in range(3):
                            if grid[g] > 1 and plan["output_map"][g] >= 0:
                                shp[plan["output_map"][g]] *= grid[g]
                        outs.append(np.zeros(shp, A.dtype))
                for o, a in zip(outs, accs):
                    sl = [slice(None)] * o.ndim
                    for g in range(3):
                        om = plan["output_map"][g]
                        if grid[g] > 1 and om >= 0:
                            n = a.shape[om]
                            cur = sl[om]
                            base = 0 if cur == slice(None) else cur.start
                            # two grid dims on one output dim would overlap: reject
                            if cur != slice(None):
                                raise NotImplementedError("one output dim split by two grid dims")
                            sl[om] = slice(base + b[g] * n, base + (b[g] + 1) * n)
                    o[tuple(sl)] = a
    if f16:
        return [o.astype(np.float16) for o in outs]
    return [o.astype(np.uint16) for o in outs]
