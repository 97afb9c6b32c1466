"""Seeded generator of random routines in the loop IR: sequences of maps, row / column / total
reductions, matrix-vector and outer-product accumulations, inlined scalar reductions, strided reads
and small matrix products over one shared family of nodes, so that consecutive statements depend on
each other the way lowered tensor code does (read-after-write, write-after-read, in-place updates,
accumulation onto earlier results). Only continuous operations are used: a difference in the last
bit of an intermediate cannot flip a branch."""
from __future__ import annotations

import numpy as np

from ocannl_amd import llir as L
from ocannl_amd import workloads as W


class Gen:
    def __init__(self, seed: int, precs=("single",), recompute: bool = False):
        self.rng = np.random.default_rng(seed)
        self.seed = seed
        L.reset_symbols(0)
        rng = self.rng
        self.R = int(rng.choice([3, 17, 64, 200, 512]))
        self.C = int(rng.choice([5, 64, 130, 256, 1024, 2048]))
        if self.R * self.C > 300000:
            self.R = 64
        if recompute and self.C > 256:     # (inlined reductions are drawn for rows of at most 256)
            self.C = 130
        self._id = 0
        pick = lambda: str(rng.choice(precs))
        self.mats = [self.node(f"m{k}", pick(), (self.R, self.C)) for k in range(4)]
        self.rows = [self.node(f"r{k}", pick(), (self.R,)) for k in range(3)]
        self.cols = [self.node(f"c{k}", pick(), (self.C,)) for k in range(2)]
        self.wide = self.node("wide", pick(), (self.R, 2 * self.C))
        self.tr = self.node("tr", pick(), (self.C, self.R))
        self.sq = self.node("sq", pick(), (self.C, self.C)) if self.C <= 256 else None
        self.scal = self.node("s", "single", (1,))
        # the extended family: a stack of matrices sliced by a static index, integer matrices, a
        # routine-local vector (a stack array in the serial C code), partial ranges and fixed positions
        self.S = 3
        self.stack = self.node("stack", pick(), (self.S, self.R, self.C))
        self.slot = L.StaticSymbol(L.fresh_symbol(), self.S)
        self.ints = [self.node(f"k{k}", "int32", (self.R, self.C)) for k in range(2)]
        self.irow = self.node("krow", "int32", (self.R,))
        self.tmp = self.node("tmp", "single", (min(self.C, 2048),))
        self.tmp.mode = "local"
        self.used_static = False
        self.extended = False
        # `recompute`: statements that spell out again, symbol for symbol, an inlined reduction that an
        # earlier statement stored -- what the reference's inlining of a tensor into every reader at
        # the assigned position leaves in a routine -- with whatever the draw puts in between
        self.recompute = recompute
        self.inlined = []      # builders of the stored expressions so far: (node stored to, f(i, j) -> scalar)
        self.nodes = self.mats + self.rows + self.cols + [self.wide, self.tr, self.scal] + ([self.sq] if self.sq else [])

    def wide_acc(self, nodes):
        """Destinations for accumulations over a loop: the checker rounds a bf16 accumulator after
        every step (cc_backend.ml:155-323) where lanes sharing the loop round once, so sums of many
        terms go to fp32 / fp64 nodes (one is made so if the draw left none)."""
        ok = [n for n in nodes if n.prec != "bfloat16"]
        if not ok:
            nodes[0].prec = "single"
            ok = [nodes[0]]
        return ok

    def node(self, name, prec, dims):
        self._id += 1
        return L.Node(self._id, name, prec, dims)

    def init(self):
        rng = np.random.default_rng(self.seed + 1000)
        out = {n.id: W.as_prec(rng.uniform(-1, 1, n.dims).astype(np.float32), n.prec) for n in self.nodes + [self.stack]}
        for n in self.ints + [self.irow]:
            out[n.id] = rng.integers(-50, 50, n.dims).astype(np.int32)
        return out

    # ---- expressions ---------------------------------------------------------------------------
    def leaf(self, i, j):
        """A read that makes sense at point (i, j); either index may be None."""
        rng = self.rng
        opts = [L.Get(self.scal, (L.Fixed(0),)), L.Const(float(rng.choice([0.5, -0.25, 1.0, 2.0])))]
        if i is not None:
            opts += [L.Get(n, (L.It(i),)) for n in self.rows]
        if j is not None:
            opts += [L.Get(n, (L.It(j),)) for n in self.cols]
        if i is not None and j is not None:
            opts += [L.Get(n, (L.It(i), L.It(j))) for n in self.mats] * 3
            opts += [L.Get(self.tr, (L.It(j), L.It(i))),
                     L.Get(self.wide, (L.It(i), L.Affine(((2, j),), int(rng.integers(0, 2)))))]
        return opts[int(rng.integers(len(opts)))]

    def expr(self, i, j, depth=None):
        rng = self.rng
        depth = int(rng.integers(1, 4)) if depth is None else depth
        if depth == 0:
            return self.leaf(i, j)
        k = int(rng.integers(0, 10))
        sub = lambda: self.expr(i, j, depth - 1)
        if k < 4:
            return L.Binop(str(rng.choice(["add", "sub", "mul", "max", "min"])), sub(), sub())
        if k < 7:
            return L.Unop(str(rng.choice(["relu", "neg", "tanh", "sat01"])), sub())
        if k == 7:
            return L.Ternop("fma", sub(), sub(), sub())
        if k == 8:
            return L.Unop("exp", L.Unop("tanh", sub()))
        return L.Binop("mul", L.Const(0.5), sub())

    def term(self, accum, count, i, j):
        """What a reduction over `count` positions accumulates: sums are means, so that values stay of
        order one through chains of statements and rounding differences are not blown up."""
        e = self.expr(i, j, 1)
        return L.Binop("mul", L.Const(1.0 / count), e) if accum == "add" else e

    # ---- statements ----------------------------------------------------------------------------
    def nest(self, syms_exts, body):
        for s, e in reversed(syms_exts):
            body = [L.For(s, 0, e - 1, body)]
        return body

    def reduce_init(self, node, accum):
        rng = self.rng
        k = int(rng.integers(0, 3))
        if k == 0:
            return []                                                   # accumulate onto what is there
        if accum == "add" and k == 1:
            return [L.ZeroOut(node)]
        v = 0.0 if accum == "add" else float("-inf") if accum == "max" else float("inf")
        return L.loop_over_dims(node.dims, lambda idcs: [L.Set(node, idcs, L.Const(v))])

    def extended_stmt(self):
        rng, R, C = self.rng, self.R, self.C
        i, j = L.fresh_symbol(), L.fresh_symbol()
        kind = int(rng.integers(0, 8))
        pick = lambda xs: xs[int(rng.integers(len(xs)))]
        st = L.It(self.slot.sym)
        if kind == 0:                                                    # read a slice chosen at run time
            self.used_static = True
            d = pick(self.mats)
            return self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), L.Binop(
                "add", L.Binop("mul", L.Const(0.5), L.Get(self.stack, (st, L.It(i), L.It(j)))), self.expr(i, j, 1)))])
        if kind == 1:                                                    # write one
            self.used_static = True
            return self.nest([(i, R), (j, C)], [L.Set(self.stack, (st, L.It(i), L.It(j)), self.expr(i, j, 2))])
        if kind == 2:                                                    # part of the rows / columns only
            d = pick(self.mats)
            r0, r1 = sorted(int(x) for x in rng.integers(0, R, 2)); c0, c1 = sorted(int(x) for x in rng.integers(0, C, 2))
            return [L.For(i, r0, r1, [L.For(j, c0, c1, [L.Set(d, (L.It(i), L.It(j)), self.expr(i, j, 2))])])]
        if kind == 3:                                                    # fixed positions
            d = pick(self.mats)
            col, row = int(rng.integers(0, C)), int(rng.integers(0, R))
            if rng.random() < 0.5:
                return self.nest([(i, R)], [L.Set(pick(self.wide_acc(self.rows)), (L.It(i),), L.Get(d, (L.It(i), L.Fixed(col))))])
            return self.nest([(j, C)], [L.Set(d, (L.Fixed(row), L.It(j)), self.expr(None, j, 1))])
        if kind == 4:                                                    # integer map
            d, a = pick(self.ints), pick(self.ints)
            op = str(rng.choice(["add", "sub", "max", "min"]))
            return self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), L.Binop(
                op, L.Get(a, (L.It(i), L.It(j))), L.Binop("mod", L.Get(self.irow, (L.It(i),)), L.Const(7.0))))])
        if kind == 5:                                                    # integer row sums / maxima: exact
            acc = str(rng.choice(["add", "max"]))
            init = [L.ZeroOut(self.irow)] if acc == "add" and rng.random() < 0.5 else []
            lhs = (L.It(i),)
            return init + self.nest([(i, R), (j, C)], [L.Set(self.irow, lhs, L.Binop(
                acc, L.Get(self.irow, lhs), L.Get(pick(self.ints), (L.It(i), L.It(j)))))])
        if kind == 6 and C <= 2048:                                      # through a routine-local vector
            a, d = pick(self.mats), pick(self.mats)
            row = int(rng.integers(0, R))
            i2, j2 = L.fresh_symbol(), L.fresh_symbol()
            return (self.nest([(j, C)], [L.Set(self.tmp, (L.It(j),), L.Unop("tanh", L.Get(a, (L.Fixed(row), L.It(j)))))]) +
                    self.nest([(i2, R), (j2, C)], [L.Set(d, (L.It(i2), L.It(j2)), L.Binop(
                        "add", L.Get(self.tmp, (L.It(j2),)), L.Binop("mul", L.Const(0.5), L.Get(d, (L.It(i2), L.It(j2))))))]))
        # integers into floats and back
        d, a = pick(self.mats), pick(self.ints)
        return self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), L.Binop(
            "mul", L.Const(0.01), L.Binop("add", L.Get(a, (L.It(i), L.It(j))), self.expr(i, j, 1))))])

    def stmt(self):
        rng, R, C = self.rng, self.R, self.C
        if self.extended and rng.random() < 0.5:
            return self.extended_stmt()
        i, j = L.fresh_symbol(), L.fresh_symbol()
        kind = int(rng.integers(0, 11))
        pick = lambda xs: xs[int(rng.integers(len(xs)))]
        if self.recompute and self.inlined and rng.random() < 0.35:      # an earlier stored expression again
            _, build = pick(self.inlined)
            d = pick(self.mats)
            form = int(rng.integers(0, 3))
            if form == 0:
                value = L.Binop("add", L.Binop("mul", L.Const(0.5), build(i, j)), L.Binop("mul", L.Const(0.25), L.Get(pick(self.mats), (L.It(i), L.It(j)))))
            elif form == 1:
                value = L.Binop("relu_gate", L.Binop("sub", build(i, j), L.Const(0.1)), L.Get(pick(self.mats), (L.It(i), L.It(j))))
            else:                                                        # over part of the rows only
                hi = max(0, R // 2 - 1)
                return [L.For(i, 0, hi, [L.For(j, 0, C - 1, [L.Set(d, (L.It(i), L.It(j)), L.Binop("mul", L.Const(0.5), build(i, j)))])])]
            return self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), value)])
        if self.recompute and C <= 256 and rng.random() < 0.3:
            kind = 9
        if kind <= 2:                                                    # map over a matrix
            d = pick(self.mats)
            order = [(i, R), (j, C)] if rng.random() < 0.8 else [(j, C), (i, R)]
            return self.nest(order, [L.Set(d, (L.It(i), L.It(j)), self.expr(i, j))])
        if kind == 3:                                                    # map over a row or column vector
            if rng.random() < 0.5:
                d = pick(self.rows)
                return self.nest([(i, R)], [L.Set(d, (L.It(i),), self.expr(i, None))])
            d = pick(self.cols)
            return self.nest([(j, C)], [L.Set(d, (L.It(j),), self.expr(None, j))])
        if kind in (4, 5):                                               # row reduction
            d = pick(self.wide_acc(self.rows))
            acc = str(rng.choice(["add", "add", "max", "min"]))
            lhs = (L.It(i),)
            return self.reduce_init(d, acc) + self.nest([(i, R), (j, C)], [L.Set(d, lhs, L.Binop(acc, L.Get(d, lhs), self.term(acc, C, i, j)))])
        if kind == 6:                                                    # column reduction
            d = pick(self.wide_acc(self.cols))
            acc = str(rng.choice(["add", "max"]))
            lhs = (L.It(j),)
            order = [(j, C), (i, R)] if rng.random() < 0.5 else [(i, R), (j, C)]
            return self.reduce_init(d, acc) + self.nest(order, [L.Set(d, lhs, L.Binop(acc, L.Get(d, lhs), self.term(acc, R, i, j)))])
        if kind == 7:                                                    # total (few enough terms that the
            lhs = (L.Fixed(0),)                                          # order of summation stays in the noise)
            if R * C <= 4096:
                return self.nest([(i, R), (j, C)], [L.Set(self.scal, lhs, L.Binop(
                    "add", L.Get(self.scal, lhs), L.Binop("mul", L.Const(1.0 / (R * C)), self.expr(i, j, 1))))])
            return self.nest([(i, R)], [L.Set(self.scal, lhs, L.Binop(
                "add", L.Get(self.scal, lhs), L.Binop("mul", L.Const(1.0 / R), self.expr(i, None, 1))))])
        if kind == 8:                                                    # matrix-vector / outer product
            m, r, c = pick(self.mats), pick(self.rows), pick(self.cols)
            if rng.random() < 0.5:
                r = pick(self.wide_acc(self.rows))
                return self.nest([(i, R), (j, C)], [L.Set(r, (L.It(i),), L.Ternop(
                    "fma", L.Get(m, (L.It(i), L.It(j))), L.Get(c, (L.It(j),)), L.Get(r, (L.It(i),))))])
            return self.nest([(i, R), (j, C)], [L.Set(m, (L.It(i), L.It(j)), L.Ternop(
                "fma", L.Get(r, (L.It(i),)), L.Get(c, (L.It(j),)), L.Get(m, (L.It(i), L.It(j)))))])
        if kind == 9 and C <= 256:                                       # inlined scalar reduction
            d, a = pick(self.mats), pick(self.mats)
            sids = [int(rng.integers(100, 10000))]
            c = pick(self.cols)
            if self.recompute and d is a and rng.random() < 0.8:         # (in place, nothing can be read back)
                d = pick([m for m in self.mats if m is not a])
            t = self.node(f"t{self._id}", "single", (1,))
            t.mode = "virtual"

            def build(i, j, a=a, c=c, t=t, sids=sids):
                k = L.fresh_symbol()
                sc = L.Scope(t, sids.pop() if sids else int(rng.integers(100, 10000)))
                scope = L.LocalScope(sc, [L.SetLocal(sc, L.Const(0.0)), L.For(k, 0, C - 1, [L.SetLocal(sc, L.Binop(
                    "add", L.GetLocal(sc), L.Binop("mul", L.Get(a, (L.It(i), L.It(k))), L.Get(c, (L.It(k),)))))])])
                # (an average of bounded values: applied in place, along a row, it cannot grow)
                return L.Binop("mul", L.Const(0.5), L.Binop("add", L.Get(a, (L.It(i), L.It(j))), L.Binop("mul", L.Const(1.0 / C), scope)))

            self.inlined.append((d, build))
            if self.recompute and rng.random() < 0.3:                    # the value through a relu, as a layer stores it
                return self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), L.Unop("relu", L.Binop("sub", build(i, j), L.Const(0.1))))])
            first = self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), build(i, j))])
            if self.recompute and rng.random() < 0.4:                    # read again right away, into another matrix
                i2, j2 = L.fresh_symbol(), L.fresh_symbol()
                d2 = pick([m for m in self.mats if m is not d and m is not a] or self.mats)
                first += self.nest([(i2, R), (j2, C)], [L.Set(d2, (L.It(i2), L.It(j2)), L.Binop("sub", build(i2, j2), L.Get(d, (L.It(i2), L.It(j2)))))])
            return first
        if self.sq is not None:                                          # matrix product m[i, j] = sum_k a[i, k] sq[k, j]
            d, a = self.wide_acc(self.mats)[0], self.mats[1]
            k = L.fresh_symbol()
            lhs = (L.It(i), L.It(j))
            # (from zero, or on top of what the tensor holds, scaled down so that values stay of order one)
            start = [L.ZeroOut(d)] if rng.random() < 0.5 else self.nest([(i, R), (j, C)], [L.Set(d, lhs, L.Binop("mul", L.Const(0.01), L.Get(d, lhs)))])
            i, j = L.fresh_symbol(), L.fresh_symbol()
            lhs = (L.It(i), L.It(j))
            return start + self.nest([(i, R), (j, C), (k, C)], [L.Set(d, lhs, L.Ternop(
                "fma", L.Get(a, (L.It(i), L.It(k))), L.Get(self.sq, (L.It(k), L.It(j))), L.Get(d, lhs)))])
        d = pick(self.mats)
        return self.nest([(i, R), (j, C)], [L.Set(d, (L.It(i), L.It(j)), self.expr(i, j))])

    def routine(self, n_stmts=None):
        n = int(self.rng.integers(4, 12)) if n_stmts is None else n_stmts
        body = []
        for k in range(n):
            body.append(L.Comment(f"statement {k}"))
            body += self.stmt()
        return L.Routine(f"fuzz_{self.seed}", body, static_indices=[self.slot] if self.used_static else [])
