"""Seeded generator of candidate mugraphs for batched fingerprint verification.

A *problem* is an un-fused reference kernel graph over tensors whose dims are
powers of two in [64, 1024]; its *candidates* are mugraphs a superoptimizer search
would submit for it: the same computation re-expressed with customized operators
under different grids, tilings and for-loop ranges (fingerprint-equal to the
reference by construction), plus *mutants* that are well-formed but compute
something else (fingerprint-unequal).  Limits follow the reference's search
(include/mirage/search/config.h:18-22): at most 5 kernel-level operators with at
most 2 customized ones, at most 3 loaders and 7 thread-block operators per
customized op.  Every candidate has 8-12 operators, counting kernel-level
operators (inputs included) and thread-block operators (loaders included, output
savers not counted, as the reference counts them).

Graph specs use the format of workloads.py.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

from .workloads import COL, ROW, _inp, _plan  # noqa: F401

MASK = (1 << 64) - 1
# tile elements (uint16) one thread block may hold; keeps every plan well inside LDS
TILE_BUDGET = 64 * 1024


class Rng:
    """splitmix64 stream: the same candidates on every platform."""

    def __init__(self, seed: int):
        self.s = seed & MASK

    def next(self) -> int:
        self.s = (self.s + 0x9E3779B97F4A7C15) & MASK
        x = self.s
        x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & MASK
        x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & MASK
        return x ^ (x >> 31)

    def below(self, n: int) -> int:
        return self.next() % n

    def pick(self, seq):
        return seq[self.below(len(seq))]

    def pow2(self, lo: int, hi: int) -> int:
        opts = []
        v = lo
        while v <= hi:
            opts.append(v)
            v *= 2
        return self.pick(opts)


def _divisor_tiles(n: int, lo: int, hi: int) -> List[int]:
    """Power-of-two tile sizes t with lo <= t <= min(hi, n) dividing n."""
    out, t = [], lo
    while t <= min(hi, n):
        if n % t == 0:
            out.append(t)
        t *= 2
    return out or [n]


def _matmul_op(rng: Rng, a_ref, b_ref, m: int, n: int, k: int) -> dict:
    """A[m,k] . B[k,n] as one customized op: rows over grid.y, columns over grid.x,
    k over the for-loop (plan shape of the reference's tests/threadblock/matmul.cu:163-189)."""
    while True:
        mt = rng.pick(_divisor_tiles(m, 16, 128))
        nt = rng.pick(_divisor_tiles(n, 32, 128))
        kt = rng.pick(_divisor_tiles(k, 32, 256))
        if mt * kt + kt * nt + 2 * mt * nt <= TILE_BUDGET:
            break
    gx, gy = n // nt, m // mt
    a_imap = (-1, 0, -1) if gy > 1 else (-1, -1, -1)
    b_imap = (1, -1, -1) if gx > 1 else (-1, -1, -1)
    omap = (1 if gx > 1 else -1, 0 if gy > 1 else -1, -1)
    return {"op": "customized", "in": [a_ref, b_ref],
            "plan": _plan((gx, gy, 1), k // kt, [a_imap, b_imap], (1, 0), omap,
                          [("tb_matmul_op", [(0, 0), (1, 0)])])}


# ---------------------------------------------------------------------------
# problem families: each returns (reference graph, function(rng, mutant) -> candidate)
# ---------------------------------------------------------------------------
def _family_matmul_add(rng: Rng):
    """Y = A.B + C; candidates fuse the matmul (8 operators)."""
    m, n, k = rng.pow2(64, 1024), rng.pow2(64, 1024), rng.pow2(64, 1024)
    ins = [_inp([m, k]), _inp([k, n], COL), _inp([m, n])]
    ref = ins + [{"op": "matmul", "in": [[0, 0], [1, 0]]},
                 {"op": "add", "in": [[3, 0], [2, 0]]}]

    def cand(r: Rng, mutant: bool):
        g = ins + [_matmul_op(r, [0, 0], [1, 0], m, n, k)]
        # mutant: the product is exponentiated before the bias is added
        if mutant:
            g[3]["plan"]["ops"].append(["tb_exp_op", [[2, 0]]])
        g.append({"op": "add", "in": [[3, 0], [2, 0]]})
        return g

    return ref, cand


def _family_mlp(rng: Rng):
    """Y = exp(X.W1).W2 (reference cpp_examples/mlp.cc:8-30); candidates run the first
    matmul at kernel level (9 operators) or as a customized op (12 operators) and fuse
    exp into the second."""
    m = rng.pow2(64, 128)
    k, h, n = rng.pow2(64, 1024), rng.pow2(64, 1024), rng.pow2(64, 1024)
    ins = [_inp([m, k]), _inp([k, h], COL), _inp([h, n], COL)]
    ref = ins + [{"op": "matmul", "in": [[0, 0], [1, 0]]},
                 {"op": "exp", "in": [[3, 0]]},
                 {"op": "matmul", "in": [[4, 0], [2, 0]]}]

    def cand(r: Rng, mutant: bool):
        g = list(ins)
        if r.below(2) == 0:
            g.append({"op": "matmul", "in": [[0, 0], [1, 0]]})
        else:
            g.append(_matmul_op(r, [0, 0], [1, 0], m, h, k))
        while True:
            hc = r.pick(_divisor_tiles(h, 32, 256))
            nt = r.pick(_divisor_tiles(n, 32, 128))
            if 2 * m * hc + hc * nt + 2 * m * nt <= TILE_BUDGET:
                break
        gx = n // nt
        ops = [("tb_exp_op", [(0, 0)]), ("tb_matmul_op", [(2, 0), (1, 0)])]
        if mutant:  # exp dropped
            ops = [("tb_matmul_op", [(0, 0), (1, 0)])]
        g.append({"op": "customized", "in": [[3, 0], [2, 0]],
                  "plan": _plan((gx, 1, 1), h // hc,
                                [(-1, -1, -1), (1, -1, -1) if gx > 1 else (-1, -1, -1)], (1, 0),
                                (1 if gx > 1 else -1, -1, -1), ops)})
        return g

    return ref, cand


def _family_attention(rng: Rng):
    """O = softmax-without-shift(Q.K).V on [b, m, 64] x [b, 64, s] x [b, s, 64] as ONE
    customized op whose block sees the whole key range (12 operators); the reference
    graph is the one every attention example compares against
    (cpp_examples/group_query_attn_inc_decode.cc:16-27)."""
    b, m, s = rng.pick([1, 2, 4, 8]), rng.pow2(64, 256), rng.pow2(64, 256)
    q, k, v = [b, m, 64], [b, 64, s], [b, s, 64]
    ins = [_inp(q), _inp(k, COL), _inp(v, COL)]
    ref = ins + [{"op": "matmul", "in": [[0, 0], [1, 0]]},
                 {"op": "exp", "in": [[3, 0]]},
                 {"op": "reduction", "in": [[4, 0]], "dim": 2, "size": 1},
                 {"op": "div", "in": [[4, 0], [5, 0]]},
                 {"op": "matmul", "in": [[6, 0], [2, 0]]}]

    def cand(r: Rng, mutant: bool):
        while True:
            mq = r.pick(_divisor_tiles(m, 16, 64))
            if mq * 64 * 2 + 2 * 64 * s + 2 * mq * s + mq <= TILE_BUDGET:
                break
        qs = m // mq
        gx = b
        q_imap = (0 if gx > 1 else -1, -1, 1 if qs > 1 else -1)
        kv_imap = (0 if gx > 1 else -1, -1, -1)
        omap = (0 if gx > 1 else -1, -1, 1 if qs > 1 else -1)
        ops = [("tb_matmul_op", [(0, 0), (1, 0)]),
               ("tb_exp_op", [(3, 0)]),
               ("tb_reduction_2_op", [(4, 0)]),
               ("tb_div_op", [(4, 0), (5, 0)]),
               ("tb_matmul_op", [(6, 0), (2, 0)])]
        if mutant:  # the row sums are taken before the exponential
            ops[1:4] = [("tb_reduction_2_op", [(3, 0)]),
                        ("tb_exp_op", [(3, 0)]),
                        ("tb_div_op", [(5, 0), (4, 0)])]
        return ins + [{"op": "customized", "in": [[0, 0], [1, 0], [2, 0]],
                       "plan": _plan((gx, 1, qs), 1, [q_imap, kv_imap, kv_imap], (-1, -1, -1),
                                     omap, ops)}]

    return ref, cand


def _family_row_softmax(rng: Rng):
    """Y = exp(X.W) / rowsum(exp(X.W)); the normalisation is one customized op over row
    blocks, the matmul runs at kernel level (8 operators) or fused (11 operators)."""
    m, k, n = rng.pow2(64, 1024), rng.pow2(64, 1024), rng.pow2(64, 512)
    ins = [_inp([m, k]), _inp([k, n], COL)]
    ref = ins + [{"op": "matmul", "in": [[0, 0], [1, 0]]},
                 {"op": "exp", "in": [[2, 0]]},
                 {"op": "reduction", "in": [[3, 0]], "dim": 1, "size": 1},
                 {"op": "div", "in": [[3, 0], [4, 0]]}]

    def cand(r: Rng, mutant: bool):
        g = list(ins)
        if r.below(2) == 0:
            g.append({"op": "matmul", "in": [[0, 0], [1, 0]]})
        else:
            g.append(_matmul_op(r, [0, 0], [1, 0], m, n, k))
        while True:
            mt = r.pick(_divisor_tiles(m, 16, 64))
            if 3 * mt * n + mt <= TILE_BUDGET:
                break
        gx = m // mt
        ops = [("tb_exp_op", [(0, 0)]),
               ("tb_reduction_1_op", [(1, 0)]),
               ("tb_div_op", [(1, 0), (2, 0)])]
        if mutant:  # rows are summed before the exponential
            ops = [("tb_reduction_1_op", [(0, 0)]),
                   ("tb_exp_op", [(0, 0)]),
                   ("tb_div_op", [(2, 0), (1, 0)])]
        imap = (0, -1, -1) if gx > 1 else (-1, -1, -1)
        g.append({"op": "customized", "in": [[2, 0]],
                  "plan": _plan((gx, 1, 1), 1, [imap], (-1,), imap, ops)})
        return g

    return ref, cand


FAMILIES = {
    "matmul_add": _family_matmul_add,
    "mlp": _family_mlp,
    "attention": _family_attention,
    "row_softmax": _family_row_softmax,
}


def count_operators(spec: List[dict]) -> int:
    n = 0
    for op in spec:
        n += 1
        if op["op"] == "customized":
            n += len(op["plan"]["input_map"]) + len(op["plan"]["ops"])
    return n


def generate(num_problems: int = 64, per_problem: int = 64, seed: int = 0x5EED,
             mutant_every: int = 4, max_dim: int = 1024) -> List[Dict]:
    """`num_problems` problems of `per_problem` candidates each.  Candidate j of a
    problem is a mutant when j % mutant_every == mutant_every - 1.  `max_dim` shrinks
    every tensor dim for CPU-sized tests (dims stay powers of two >= 64)."""
    names = sorted(FAMILIES)
    problems = []
    for p in range(num_problems):
        rng = Rng(seed * 1000003 + p)
        if max_dim < 1024:
            real = rng.pow2
            rng.pow2 = lambda lo, hi, real=real: real(lo, max(lo, min(hi, max_dim)))
        family = names[p % len(names)]
        ref, cand = FAMILIES[family](rng)
        cands = []
        for j in range(per_problem):
            mutant = (j % mutant_every) == mutant_every - 1
            spec = cand(rng, mutant)
            cands.append({"spec": spec, "expect_equal": not mutant,
                          "operators": count_operators(spec)})
        problems.append({"family": family, "reference": ref, "candidates": cands,
                         "input_seed": (0xF1A9 << 16) + p + 1})
    return problems
