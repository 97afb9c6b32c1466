"""Workload generator: builds the loop IR that OCANNL's unchanged frontend would hand to a backend.

The OCaml frontend (``Tensor`` / ``Operation`` / ``Train`` / ``nn_blocks``) is outside the
backend boundary and cannot run where this build is tested, so the tests and the benchmark need a
stand-in that emits routines of the same *shape*: accumulating assignments with projections, lowered
to loop nests, differentiated by accumulation into gradient nodes, with single-use intermediates
inlined.  This module restates just enough of it:

* lowering of one accumulating assignment to a loop nest -- ``Assignments.to_low_level``'s
  ``loop_accum`` (arrayjit/lib/assignments.ml:311-488): one loop per product-space axis of
  dimension > 1, ``Fixed_idx 0`` for dimension-1 axes, plain ``:=`` when the projection is
  injective and surjective, else ``Zero_out``/neutral fill + ``lhs := accum(lhs, rhs)``;
  ``a*b + c`` becomes ``fma`` (arrayjit/lib/low_level.ml:1631-1634);
* the operations and their gradient rules used by the five benchmark configurations
  (tensor/operation.ml:55-508): ``g1 =+ g * v2; g2 =+ v1 * g`` for products, relu / tanh / exp /
  log / sqrt / division / where / max-reduction rules as written there;
* ``Train.grad_update`` / ``sgd_one`` (lib/train.ml:61-90) and the Adam recipe of
  docs/migration_guide.md:639-652;
* inlining of nodes that are computed once and read once per cell (the effect of
  ``virtualize_max_visits = 1``, arrayjit/lib/low_level.ml:535-571,1165-1316), producing the
  ``Local_scope`` reductions seen in test/einsum/inline_permuted_view-c_fwd.ll.expected; an opt-in
  mode (``inline="visits"``) also treats reads at the position being assigned as free, as the
  reference's visit count does (low_level.ml:496-552);
* memory modes: parameters, inputs and outputs in context; other nodes ``local`` when at most
  ``stack_threshold_in_bytes`` = 16384 bytes, else in context (arrayjit/lib/tnode.ml:152-171).

Axes are named: every tensor carries a tuple of axis labels and operations align operands by
label, which is what OCANNL's projections inference arrives at for these graphs.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple

from . import llir as L

STACK_THRESHOLD = 16384


@dataclass(eq=False)
class T:
    """A tensor: value node, optional gradient node, and how to backpropagate through it."""

    value: L.Node
    axes: Tuple[str, ...]
    grad: Optional[L.Node] = None
    children: Tuple["T", ...] = ()
    fwd: List[L.Stmt] = field(default_factory=list)       # this op's own forward statements
    bwd: Optional[Callable[[], List[L.Stmt]]] = None       # this op's gradient statements
    label: str = ""

    @property
    def dims(self) -> Tuple[int, ...]:
        return self.value.dims

    def ext(self) -> Dict[str, int]:
        return dict(zip(self.axes, self.value.dims))


class Graph:
    """A session: node ids, default precisions (``Tensor.default_value_prec`` /
    ``default_grad_prec``, tensor/tensor.ml:164-165)."""

    def __init__(self, value_prec: str = "single", grad_prec: str = "single", first_id: int = 1,
                 reduce_order: str = "last"):
        self.value_prec = value_prec
        self.grad_prec = grad_prec
        self._next = first_id
        self._scope = 0
        self.reduce_order = reduce_order   # "last": reduced axes innermost; "first": outermost
        self.forced_ctx: set = set()

    # ---- nodes ---------------------------------------------------------------------------
    def node(self, ident: str, dims: Sequence[int], prec: Optional[str] = None, mode: Optional[str] = None) -> L.Node:
        prec = prec or self.value_prec
        dims = tuple(int(d) for d in dims)
        n = L.Node(self._next, f"{ident}_{self._next}" if mode != "named" else ident, prec, dims, "ctx")
        self._next += 1
        if mode in ("ctx", "local"):
            n.mode = mode
        else:
            n.mode = "ctx" if n.size_in_bytes > STACK_THRESHOLD else "local"
        return n

    def scope(self, node: L.Node) -> L.Scope:
        self._scope += 1
        return L.Scope(node, self._scope)

    # ---- leaves --------------------------------------------------------------------------
    def param(self, ident: str, axes: Sequence[str], dims: Sequence[int], prec: Optional[str] = None) -> T:
        v = self.node(ident, dims, prec, "ctx")
        g = self.node(ident + "_grad", dims, self.grad_prec)
        v._is_param = True
        g._is_grad = True
        g._is_param_grad = True
        return T(v, tuple(axes), g, label=ident)

    def input(self, ident: str, axes: Sequence[str], dims: Sequence[int], prec: Optional[str] = None) -> T:
        v = self.node(ident, dims, prec, "ctx")
        v._is_param = True
        return T(v, tuple(axes), None, label=ident)

    def constant(self, value: float, prec: Optional[str] = None) -> "ConstT":
        return ConstT(float(value), prec or self.value_prec)

    # ---- lowering of one accumulating assignment -------------------------------------------
    def lower(self, lhs: L.Node, lhs_axes: Sequence[str], space: Sequence[Tuple[str, int]],
              rhs: Callable[[Dict[str, L.AxisIndex]], L.Scalar], accum: str = "add",
              init_neutral: bool = True) -> List[L.Stmt]:
        """``lhs[lhs_axes] accum= rhs`` over the product space (assignments.ml:311-488)."""
        space = list(space)
        reduced = [(l, e) for l, e in space if l not in lhs_axes and e > 1]
        kept = [(l, e) for l, e in space if l in lhs_axes]
        idx: Dict[str, L.AxisIndex] = {l: L.Fixed(0) for l, e in space if e == 1}
        if self.reduce_order == "first":
            space = reduced + kept
        else:
            space = kept + reduced
        loops: List[Tuple[int, int]] = []
        for label, e in space:
            if e == 1:
                idx[label] = L.Fixed(0)
            else:
                s = L.fresh_symbol()
                idx[label] = L.It(s)
                loops.append((s, e))
        for label in lhs_axes:
            idx.setdefault(label, L.Fixed(0))
        lhs_idcs = tuple(idx[a] for a in lhs_axes)
        rhs2 = rhs(idx)
        injective = not reduced
        out: List[L.Stmt] = []
        if init_neutral and injective:
            stmt = L.Set(lhs, lhs_idcs, rhs2)       # can_skip_accumulation
        else:
            self_get = L.Get(lhs, lhs_idcs)
            if accum == "add" and isinstance(rhs2, L.Binop) and rhs2.op == "mul":
                val = L.Ternop("fma", rhs2.a, rhs2.b, self_get)
            elif accum == "sub":
                val = L.Binop("sub", self_get, rhs2)
            else:
                val = L.Binop(accum, self_get, rhs2)
            stmt = L.Set(lhs, lhs_idcs, val)
            if init_neutral:
                if accum == "add":
                    out.append(L.ZeroOut(lhs))
                    if not getattr(lhs, "_touched", False):
                        lhs.zero_initialized_by_code = True
                else:   # Fetch (Constant neutral) (assignments.ml:770-775)
                    neutral = {"max": float("-inf"), "min": float("inf"), "mul": 1.0}[accum]
                    out.extend(L.loop_over_dims(lhs.dims, lambda ix: [L.Set(lhs, ix, L.Const(neutral))]))
        lhs._touched = True
        body: List[L.Stmt] = [stmt]
        for s, e in reversed(loops):
            body = [L.For(s, 0, e - 1, body)]
        return out + body

    # ---- operations ------------------------------------------------------------------------
    def _result(self, ident: str, axes: Sequence[str], ext: Dict[str, int], prec: Optional[str], diff: bool):
        dims = [ext[a] for a in axes]
        v = self.node(ident, dims, prec)
        g = self.node(ident + "_grad", dims, self.grad_prec) if diff else None
        if g is not None:
            g._is_grad = True
        return v, g

    @staticmethod
    def _get(t, idx):
        if isinstance(t, ConstT):
            return L.Const(t.value)
        if getattr(t, "_getter", None) is not None:
            return t._getter(idx)
        return L.Get(t.value, tuple(idx[a] for a in t.axes))

    def _space(self, out_axes, operands) -> List[Tuple[str, int]]:
        ext: Dict[str, int] = {}
        order: List[str] = list(out_axes)
        for t in operands:
            if isinstance(t, ConstT):
                continue
            for a, d in zip(t.axes, t.dims):
                if a in ext and ext[a] != d and 1 not in (ext[a], d):
                    raise ValueError(f"axis {a}: {ext[a]} vs {d}")
                ext[a] = max(ext.get(a, 1), d)
                if a not in order:
                    order.append(a)
        return [(a, ext.get(a, 1)) for a in order]

    def nary(self, ident: str, operands: Sequence, out_axes: Sequence[str],
             value_fn: Callable[..., L.Scalar], grad_fns: Sequence[Optional[Callable[..., L.Scalar]]],
             accum: str = "add", prec: Optional[str] = None) -> T:
        """Generic operation: ``v[out] accum= value_fn(v1[..], v2[..], ...)`` over the union of the
        operands' axes; ``grad_fns[i](g, v, v1, v2, ...)`` is what is accumulated (``=+``) into
        operand i's gradient over the same product space."""
        operands = list(operands)
        out_axes = tuple(out_axes)
        space = self._space(out_axes, operands)
        ext = dict(space)
        diff = any((not isinstance(t, ConstT)) and t.grad is not None for t in operands)
        v, g = self._result(ident, out_axes, ext, prec, diff)
        res = T(v, out_axes, g, tuple(t for t in operands if not isinstance(t, ConstT)), label=ident)
        res.fwd = self.lower(v, out_axes, space, lambda idx: value_fn(*[self._get(t, idx) for t in operands]),
                             accum=accum, init_neutral=True)

        def bwd() -> List[L.Stmt]:
            out: List[L.Stmt] = []
            for i, t in enumerate(operands):
                if isinstance(t, ConstT) or t.grad is None or grad_fns[i] is None:
                    continue
                fn = grad_fns[i]

                def rhs(idx, fn=fn):
                    gget = L.Get(g, tuple(idx[a] for a in out_axes))
                    vget = L.Get(v, tuple(idx[a] for a in out_axes))
                    return fn(gget, vget, *[self._get(o, idx) for o in operands])

                out += self.lower(t.grad, t.axes, space, rhs, accum="add", init_neutral=False)
            return out

        res.bwd = bwd if diff else None
        return res

    # tensor/operation.ml:55-99
    def add(self, a, b, out_axes=None, ident="add"):
        out_axes = out_axes or self._union_axes(a, b)
        return self.nary(ident, [a, b], out_axes, lambda x, y: L.Binop("add", x, y),
                         [lambda g, v, x, y: g, lambda g, v, x, y: g])

    def sub(self, a, b, out_axes=None, ident="sub"):
        out_axes = out_axes or self._union_axes(a, b)
        return self.nary(ident, [a, b], out_axes, lambda x, y: L.Binop("sub", x, y),
                         [lambda g, v, x, y: g, lambda g, v, x, y: L.Unop("neg", g)])

    def mul(self, a, b, out_axes=None, ident="mul"):
        """Pointwise product, or with ``out_axes`` dropping shared axes: an einsum contraction."""
        out_axes = out_axes or self._union_axes(a, b)
        return self.nary(ident, [a, b], out_axes, lambda x, y: L.Binop("mul", x, y),
                         [lambda g, v, x, y: L.Binop("mul", g, y), lambda g, v, x, y: L.Binop("mul", x, g)])

    einsum = mul

    def div(self, a, b, out_axes=None, ident="div", prec=None):
        out_axes = out_axes or self._union_axes(a, b)
        return self.nary(ident, [a, b], out_axes, lambda x, y: L.Binop("div", x, y), prec=prec, grad_fns=
                         [lambda g, v, x, y: L.Binop("div", g, y),
                          lambda g, v, x, y: L.Binop("mul", g, L.Binop(
                              "div", L.Binop("mul", L.Const(-1.0), x), L.Binop("mul", y, y)))])


    def unary(self, op: str, a: T, ident: Optional[str] = None, prec=None):
        rules = {   # tensor/operation.ml:163-296
            "relu": lambda g, v, x: L.Binop("relu_gate", x, g),
            "exp": lambda g, v, x: L.Binop("mul", g, v),
            "log": lambda g, v, x: L.Binop("div", g, x),
            "sqrt": lambda g, v, x: L.Binop("div", g, L.Binop("mul", L.Const(2.0), v)),
            "tanh": lambda g, v, x: L.Binop("mul", g, L.Binop("sub", L.Const(1.0), L.Binop("mul", v, v))),
            "neg": lambda g, v, x: L.Unop("neg", g),
            "recip": lambda g, v, x: L.Binop("mul", g, L.Binop("mul", L.Const(-1.0), L.Binop("mul", v, v))),
            "id": lambda g, v, x: g,
        }
        return self.nary(ident or op, [a], a.axes, lambda x: L.Unop(op, x) if op != "id" else x, [rules[op]], prec=prec)

    def reduce(self, a: T, out_axes: Sequence[str], accum: str = "add", ident: Optional[str] = None, prec=None):
        """``einsum1`` / ``einmax1`` (tensor/operation.ml:504-508,583-593)."""
        if accum == "add":
            gfn = lambda g, v, x: g
        elif accum == "max":
            gfn = lambda g, v, x: L.Ternop("where", L.Binop("eq", v, x), g, L.Const(0.0))
        else:
            raise ValueError(accum)
        return self.nary(ident or ("sum" if accum == "add" else accum), [a], out_axes, lambda x: x, [gfn],
                         accum=accum, prec=prec)

    def where(self, cond: T, a, b, ident="where"):
        """tensor/operation.ml:455-464: no gradient to the predicate."""
        out_axes = self._union_axes(cond, a, b)
        return self.nary(ident, [cond, a, b], out_axes, lambda c, x, y: L.Ternop("where", c, x, y),
                         [None, lambda g, v, c, x, y: L.Ternop("where", c, g, L.Const(0.0)),
                          lambda g, v, c, x, y: L.Ternop("where", c, L.Const(0.0), g)])

    def _union_axes(self, *ts):
        """Result axes of a broadcasting pointwise operation: those of the operand of highest rank
        in its own order (so that the result shares its layout), then any the others add."""
        out: List[str] = []
        ranked = sorted((t for t in ts if not isinstance(t, ConstT)), key=lambda t: -len(t.axes))
        for t in ranked:
            for a in t.axes:
                if a not in out:
                    out.append(a)
        return tuple(out)

    # ---- assembling forward / backward code (tensor/tensor.ml:415-495) ----------------------
    @staticmethod
    def topo(root: T) -> List[T]:
        seen, order = set(), []

        def visit(t: T):
            if id(t) in seen:
                return
            seen.add(id(t))
            for c in t.children:
                visit(c)
            order.append(t)

        visit(root)
        return order

    def forward(self, root: T) -> List[L.Stmt]:
        out: List[L.Stmt] = [L.Comment(f"{root.label} fwd")]
        for t in self.topo(root):
            out += t.fwd
        return out

    def grad_update(self, loss: T) -> List[L.Stmt]:
        """``Train.grad_update`` (lib/train.ml:61-75): forward; zero grads; loss.grad =: 1;
        backprop in reverse order of computation."""
        loss.value.mode = "ctx"
        self.forced_ctx.add(loss.value.id)
        order = self.topo(loss)
        out: List[L.Stmt] = [L.Comment(f"{loss.label} forward and gradient update")]
        out += self.forward(loss)
        out.append(L.Comment(f"{loss.label} zero grads and backprop"))
        seen = set()
        for t in order:
            if t.grad is not None and t.grad.id not in seen:
                seen.add(t.grad.id)
                out.append(L.ZeroOut(t.grad))
                if not getattr(t.grad, "_touched", False):
                    t.grad.zero_initialized_by_code = True
                t.grad._touched = True
        out += L.loop_over_dims(loss.grad.dims, lambda ix: [L.Set(loss.grad, ix, L.Const(1.0))])
        for t in reversed(order):
            if t.bwd is not None:
                out += t.bwd()
        return out

    def backprop_from(self, root: T, comment: str = "backprop") -> List[L.Stmt]:
        """Backprop with the root gradient supplied by the caller (a context node that is not
        zeroed): zero every other gradient, then the gradient assignments in reverse order."""
        root.grad.mode = "ctx"
        self.forced_ctx.add(root.grad.id)
        order = self.topo(root)
        out: List[L.Stmt] = [L.Comment(comment)]
        seen = set()
        for t in order:
            if t.grad is not None and t.grad is not root.grad and t.grad.id not in seen:
                seen.add(t.grad.id)
                out.append(L.ZeroOut(t.grad))
                if not getattr(t.grad, "_touched", False):
                    t.grad.zero_initialized_by_code = True
                t.grad._touched = True
        for t in reversed(order):
            if t.bwd is not None:
                out += t.bwd()
        return out

    # ---- optimisers -----------------------------------------------------------------------
    def sgd_update(self, params: Sequence[T], learning_rate: T, momentum: float = 0.0,
                   weight_decay: float = 0.0, nesterov: bool = False, lr_idx=None) -> List[L.Stmt]:
        """``Train.sgd_one`` per parameter (lib/train.ml:76-90); ``learning_rate`` is a 1-element
        tensor (or indexed by a static symbol through ``lr_idx``)."""
        out: List[L.Stmt] = [L.Comment("sgd_update")]
        for p in params:
            axes = [f"_p{i}" for i in range(len(p.dims))]
            space = list(zip(axes, p.dims))
            out.append(L.Comment(f"{p.label} param sgd step"))
            delta = self.node(f"sgd_delta_{p.label}", p.dims, p.value.prec)
            out += self.lower(delta, axes, space, lambda idx: L.Binop(
                "add", L.Get(p.grad, tuple(idx[a] for a in axes)),
                L.Binop("mul", L.Const(weight_decay), L.Get(p.value, tuple(idx[a] for a in axes)))))
            if momentum > 0.0:
                mom = self.node(f"sgd_momentum_{p.label}", p.dims, p.value.prec, "ctx")
                p.sgd_momentum = mom
                out += self.lower(mom, axes, space, lambda idx: L.Binop(
                    "add", L.Binop("mul", L.Const(momentum), L.Get(mom, tuple(idx[a] for a in axes))),
                    L.Get(delta, tuple(idx[a] for a in axes))))
                if nesterov:
                    out += self.lower(delta, axes, space, lambda idx: L.Binop(
                        "mul", L.Const(momentum), L.Get(mom, tuple(idx[a] for a in axes))),
                        accum="add", init_neutral=False)
                else:
                    out += self.lower(delta, axes, space, lambda idx: L.Get(mom, tuple(idx[a] for a in axes)))
            lr_ix = lr_idx if lr_idx is not None else tuple(L.Fixed(0) for _ in learning_rate.dims)
            out += self.lower(p.value, axes, space, lambda idx: L.Binop(
                "mul", L.Get(learning_rate.value, lr_ix), L.Get(delta, tuple(idx[a] for a in axes))),
                accum="sub", init_neutral=False)
        return out

    def adam_update(self, params: Sequence[T], lr: float = 1e-3, beta1: float = 0.9, beta2: float = 0.999,
                    eps: float = 1e-8) -> List[L.Stmt]:
        """Adam as written in docs/migration_guide.md:639-652 (no bias correction):
        m = b1*m + (1-b1)*g; v = b2*v + (1-b2)*g*g; p -= lr * m / (sqrt(v) + eps)."""
        out: List[L.Stmt] = [L.Comment("adam_update")]
        for p in params:
            axes = [f"_p{i}" for i in range(len(p.dims))]
            space = list(zip(axes, p.dims))
            m = self.node(f"adam_m_{p.label}", p.dims, p.value.prec, "ctx")
            v = self.node(f"adam_v_{p.label}", p.dims, p.value.prec, "ctx")
            p.adam_m, p.adam_v = m, v
            ix = lambda idx: tuple(idx[a] for a in axes)
            out.append(L.Comment(f"{p.label} param adam step"))
            out += self.lower(m, axes, space, lambda idx: L.Binop(
                "add", L.Binop("mul", L.Const(beta1), L.Get(m, ix(idx))),
                L.Binop("mul", L.Const(1.0 - beta1), L.Get(p.grad, ix(idx)))))
            out += self.lower(v, axes, space, lambda idx: L.Binop(
                "add", L.Binop("mul", L.Const(beta2), L.Get(v, ix(idx))),
                L.Binop("mul", L.Const(1.0 - beta2), L.Binop("mul", L.Get(p.grad, ix(idx)), L.Get(p.grad, ix(idx))))))
            out += self.lower(p.value, axes, space, lambda idx: L.Binop(
                "div", L.Binop("mul", L.Const(lr), L.Get(m, ix(idx))),
                L.Binop("add", L.Unop("sqrt", L.Get(v, ix(idx))), L.Const(eps))),
                accum="sub", init_neutral=False)
        return out


@dataclass
class ConstT:
    value: float
    prec: str = "single"


# ------------------------------------------------------------------------------------------------
# inlining of single-visit nodes
# ------------------------------------------------------------------------------------------------

def _subst_idx(ix: L.AxisIndex, m: Dict[int, L.AxisIndex]) -> L.AxisIndex:
    if isinstance(ix, L.It) and ix.sym in m:
        return m[ix.sym]
    if isinstance(ix, L.Affine):
        terms, off = [], ix.offset
        for c, s in ix.terms:
            r = m.get(s)
            if r is None:
                terms.append((c, s))
            elif isinstance(r, L.It):
                terms.append((c, r.sym))
            elif isinstance(r, L.Fixed):
                off += c * r.i
            else:
                raise ValueError("affine-in-affine substitution")
        return L.Affine(tuple(terms), off)
    return ix


def _subst_scalar(s: L.Scalar, m: Dict[int, L.AxisIndex], self_get=None) -> L.Scalar:
    def ix(idcs):
        return tuple(_subst_idx(i, m) for i in idcs)

    if isinstance(s, L.Get):
        if self_get is not None and s.node is self_get[0]:
            return L.GetLocal(self_get[1])
        return L.Get(s.node, ix(s.idcs))
    if isinstance(s, L.GetMerge):
        return L.GetMerge(s.node, ix(s.idcs))
    if isinstance(s, L.GetDynamic):
        return L.GetDynamic(s.node, ix(s.idcs), s.dyn_axis, _subst_scalar(s.dyn_value, m, self_get), s.dyn_prec)
    if isinstance(s, L.EmbedIndex):
        return L.EmbedIndex(_subst_idx(s.idx, m))
    if isinstance(s, L.Unop):
        return L.Unop(s.op, _subst_scalar(s.arg, m, self_get), s.arg_prec)
    if isinstance(s, L.Binop):
        return L.Binop(s.op, _subst_scalar(s.a, m, self_get), _subst_scalar(s.b, m, self_get))
    if isinstance(s, L.Ternop):
        return L.Ternop(s.op, _subst_scalar(s.a, m, self_get), _subst_scalar(s.b, m, self_get),
                        _subst_scalar(s.c, m, self_get), s.a_prec)
    if isinstance(s, L.LocalScope):
        return L.LocalScope(s.scope, _subst_stmts(s.body, m))
    return s


def _subst_stmts(body: Sequence[L.Stmt], m: Dict[int, L.AxisIndex]) -> List[L.Stmt]:
    out = []
    for c in body:
        if isinstance(c, L.For):
            s2 = L.fresh_symbol()
            m2 = dict(m)
            m2[c.sym] = L.It(s2)
            out.append(L.For(s2, c.from_, c.to, _subst_stmts(c.body, m2)))
        elif isinstance(c, L.SetLocal):
            out.append(L.SetLocal(c.scope, _subst_scalar(c.value, m)))
        elif isinstance(c, L.Set):
            out.append(L.Set(c.node, tuple(_subst_idx(i, m) for i in c.idcs), _subst_scalar(c.value, m)))
        else:
            out.append(c)
    return out


def _count_gets(body: Sequence[L.Stmt], node: L.Node) -> int:
    n = 0

    def sc(s):
        nonlocal n
        if isinstance(s, (L.Get, L.GetMerge, L.GetDynamic)) and s.node is node:
            n += 1
        if isinstance(s, L.GetDynamic):
            sc(s.dyn_value)
        elif isinstance(s, L.Unop):
            sc(s.arg)
        elif isinstance(s, L.Binop):
            sc(s.a); sc(s.b)
        elif isinstance(s, L.Ternop):
            sc(s.a); sc(s.b); sc(s.c)
        elif isinstance(s, L.LocalScope):
            st(s.body)

    def st(b):
        for c in b:
            if isinstance(c, L.For):
                st(c.body)
            elif isinstance(c, (L.Set, L.SetLocal)):
                sc(c.value)
            elif isinstance(c, L.SetFromVec):
                sc(c.arg)

    st(body)
    return n


def _perfect_nest(stmt: L.Stmt):
    """Returns ([(sym, from, to)...], inner statements)."""
    loops = []
    cur = stmt
    while isinstance(cur, L.For):
        loops.append((cur.sym, cur.from_, cur.to))
        inner = [c for c in cur.body if not isinstance(c, L.Comment)]
        if len(inner) == 1 and isinstance(inner[0], L.For):
            cur = inner[0]
        else:
            return loops, inner
    return loops, [cur]


def inline_single_use(g: Graph, body: List[L.Stmt], keep: Sequence[L.Node] = (), visits: bool = False) -> List[L.Stmt]:
    """Inline every local/intermediate node that is defined by one statement group and read
    exactly once, by a statement whose loops all index that read (one visit per cell).

    ``visits=True`` follows the reference's visit count more closely (arrayjit/lib/low_level.ml:496-552
    with ``virtualize_max_visits`` = 1): a read at the very position being assigned is not a visit, so a
    tensor computed once per cell by a pointwise statement is inlined into ANY number of such readers
    (and recomputed there), plus at most one reader that visits every cell once; and a gradient that is
    zeroed and then accumulated into by a single pointwise statement counts as computed once (the
    gradients of parameters stay in memory: the optimiser's routine reads them)."""
    keep_ids = {n.id for n in keep} | set(g.forced_ctx)
    body = list(body)
    changed = True
    while changed:
        changed = False
        writes: Dict[int, List[int]] = {}
        for i, c in enumerate(body):
            if isinstance(c, L.ZeroOut):
                writes.setdefault(c.node.id, []).append(i)
            elif isinstance(c, (L.For, L.Set)):
                loops, inner = _perfect_nest(c)
                for x in inner:
                    for w in _written_nodes([x]):
                        writes.setdefault(w.id, []).append(i)
        for nid, idxs in writes.items():
            node = _node_at(body, idxs[0], nid)
            if node is None or nid in keep_ids or getattr(node, "_is_param", False):
                continue
            if getattr(node, "_is_grad", False) and (not visits or getattr(node, "_is_param_grad", False)):
                continue
            idxs = sorted(set(idxs))
            # definition group: [Set nest] or [ZeroOut/neutral-fill, accumulate nest], contiguous
            # (visits: the zero fill may stand anywhere ahead, as zero_grads puts it)
            if len(idxs) == 1:
                def_i, fill_i = idxs[0], None
            elif len(idxs) == 2 and (idxs[1] == idxs[0] + 1 or (visits and isinstance(body[idxs[0]], L.ZeroOut))):
                fill_i, def_i = idxs
            else:
                continue
            loops, inner = _perfect_nest(body[def_i])
            if len(inner) != 1 or not isinstance(inner[0], L.Set) or inner[0].node is not node:
                continue
            dset = inner[0]
            if _count_gets(body[:def_i], node) or _count_gets([body[def_i]], node) > (0 if fill_i is None else 1):
                continue
            if fill_i is not None and not _is_neutral_fill(body[fill_i], node):
                continue
            uses = [i for i in range(def_i + 1, len(body)) if _count_gets([body[i]], node)]
            if not uses or (not visits and _count_gets(body[def_i + 1:], node) != 1):
                continue
            use_i = uses[-1]
            if not _inputs_unchanged(body, def_i, use_i, dset):
                continue
            # the definition's lhs axes must be distinct plain iterators (or Fixed 0)
            par = {}
            ok = True
            for p, ixp in enumerate(dset.idcs):
                if isinstance(ixp, L.It) and ixp.sym not in par:
                    par[ixp.sym] = p
                elif isinstance(ixp, L.Fixed) and ixp.i == 0 and node.dims[p] == 1:
                    pass
                else:
                    ok = False
            red = [(s, f, t) for (s, f, t) in loops if s not in par]
            if not ok or (fill_i is None and red):
                continue
            if len(uses) == 1 and _count_gets([body[use_i]], node) == 1:
                new_uses = {use_i: _inline_into(g, body[use_i], node, dset, par, red, fill_i is not None)}
            else:
                # several reads: only a pointwise definition, every read but one at the position being assigned
                if red:
                    continue
                # (the one reader that visits every cell once is given up when the definition itself holds an
                # inlined reduction: nested into a second reduction it would be recomputed per addend)
                budget = {"visits": 0 if _has_local_scope(dset.value) else 1}
                new_uses = {u: _inline_into(g, body[u], node, dset, par, red, fill_i is not None, budget) for u in uses}
            if any(v is None for v in new_uses.values()):
                continue
            for u, v in new_uses.items():
                body[u] = v
            for i in sorted([x for x in (def_i, fill_i) if x is not None], reverse=True):
                del body[i]
            node.mode = "virtual"
            changed = True
            break
    return body


def _has_local_scope(s: L.Scalar) -> bool:
    if isinstance(s, L.LocalScope):
        return True
    if isinstance(s, L.Unop):
        return _has_local_scope(s.arg)
    if isinstance(s, L.Binop):
        return _has_local_scope(s.a) or _has_local_scope(s.b)
    if isinstance(s, L.Ternop):
        return _has_local_scope(s.a) or _has_local_scope(s.b) or _has_local_scope(s.c)
    return False


def _written_nodes(stmts) -> List[L.Node]:
    out = []
    for c in stmts:
        if isinstance(c, L.For):
            out += _written_nodes(c.body)
        elif isinstance(c, (L.Set, L.SetFromVec, L.ZeroOut)):
            out.append(c.node)
    return out


def _node_at(body, i, nid):
    for n in _written_nodes([body[i]]):
        if n.id == nid:
            return n
    return None


def _is_neutral_fill(stmt, node) -> bool:
    if isinstance(stmt, L.ZeroOut):
        return stmt.node is node
    loops, inner = _perfect_nest(stmt)
    return len(inner) == 1 and isinstance(inner[0], L.Set) and inner[0].node is node and isinstance(inner[0].value, L.Const)


def _read_nodes(s: L.Scalar, acc: set):
    if isinstance(s, (L.Get, L.GetDynamic, L.GetMerge)):
        acc.add(s.node.id)
    if isinstance(s, L.GetDynamic):
        _read_nodes(s.dyn_value, acc)
    elif isinstance(s, L.Unop):
        _read_nodes(s.arg, acc)
    elif isinstance(s, L.Binop):
        _read_nodes(s.a, acc); _read_nodes(s.b, acc)
    elif isinstance(s, L.Ternop):
        _read_nodes(s.a, acc); _read_nodes(s.b, acc); _read_nodes(s.c, acc)
    elif isinstance(s, L.LocalScope):
        for c in s.body:
            if isinstance(c, (L.Set, L.SetLocal)):
                _read_nodes(c.value, acc)
            elif isinstance(c, L.For):
                for x in _flatten(c.body):
                    if isinstance(x, (L.Set, L.SetLocal)):
                        _read_nodes(x.value, acc)


def _flatten(body):
    for c in body:
        if isinstance(c, L.For):
            yield from _flatten(c.body)
        else:
            yield c


def _inputs_unchanged(body, def_i, use_i, dset) -> bool:
    reads: set = set()
    _read_nodes(dset.value, reads)
    reads.discard(dset.node.id)
    for i in range(def_i + 1, use_i + 1):
        for w in _written_nodes([body[i]]):
            if w.id in reads:
                return False
    return True


def _inline_into(g: Graph, use_stmt, node, dset, par, red, is_reduction, budget=None):
    """Rewrite the single ``Get node`` inside ``use_stmt``; None if the read is not one-visit.
    With ``budget`` (a dict holding the visits still allowed, shared over all statements that read the
    node): rewrite every read; a read at the position the statement assigns is free, any other has to
    be one-visit and takes one from the budget."""
    found = {"n": 0}

    def enclosing_ok(get: L.Get, loop_syms: List[int]) -> bool:
        used = set()
        for ixp in get.idcs:
            used.update(L.index_symbols(ixp))
            if not isinstance(ixp, (L.It, L.Fixed)):
                return False
        return all(s in used for s in loop_syms)

    def build(get: L.Get) -> L.Scalar:
        m = {s: get.idcs[p] for s, p in par.items()}
        if not is_reduction:
            return _subst_scalar(dset.value, m)
        sc = g.scope(node)
        m2 = dict(m)
        loops = []
        for (s, f, t) in red:
            s2 = L.fresh_symbol()
            m2[s] = L.It(s2)
            loops.append((s2, f, t))
        upd = _subst_scalar(dset.value, m2, self_get=(node, sc))
        inner: List[L.Stmt] = [L.SetLocal(sc, upd)]
        for (s2, f, t) in reversed(loops):
            inner = [L.For(s2, f, t, inner)]
        neutral = 0.0
        if isinstance(dset.value, L.Binop) and dset.value.op in ("max", "min"):
            neutral = float("-inf") if dset.value.op == "max" else float("inf")
        return L.LocalScope(sc, [L.SetLocal(sc, L.Const(neutral))] + inner)

    def wrap(get: L.Get, lhs):
        v = build(get)
        # a value of another precision than the statement it lands in is still rounded to its own first
        if budget is not None and lhs is not None and lhs.node.prec != node.prec and not isinstance(v, L.LocalScope):
            sc = g.scope(node)
            return L.LocalScope(sc, [L.SetLocal(sc, v)])
        return v

    def sc_rw(s, loop_syms, lhs=None):
        if isinstance(s, L.Get) and s.node is node:
            positional = budget is not None and lhs is not None and tuple(s.idcs) == tuple(lhs.idcs)
            if not positional:
                if not enclosing_ok(s, loop_syms):
                    raise _NoInline()
                if budget is not None:
                    if budget["visits"] <= 0:
                        raise _NoInline()
                    budget["visits"] -= 1
            found["n"] += 1
            return wrap(s, lhs)
        if isinstance(s, L.Unop):
            return L.Unop(s.op, sc_rw(s.arg, loop_syms, lhs), s.arg_prec)
        if isinstance(s, L.Binop):
            return L.Binop(s.op, sc_rw(s.a, loop_syms, lhs), sc_rw(s.b, loop_syms, lhs))
        if isinstance(s, L.Ternop):
            return L.Ternop(s.op, sc_rw(s.a, loop_syms, lhs), sc_rw(s.b, loop_syms, lhs), sc_rw(s.c, loop_syms, lhs), s.a_prec)
        if isinstance(s, L.LocalScope):
            if _count_gets(s.body, node):
                raise _NoInline()
            return s
        return s

    def st_rw(c, loop_syms):
        if isinstance(c, L.For):
            return L.For(c.sym, c.from_, c.to, [st_rw(x, loop_syms + [c.sym]) for x in c.body])
        if isinstance(c, L.Set):
            return L.Set(c.node, c.idcs, sc_rw(c.value, loop_syms, c))
        if isinstance(c, L.SetLocal):
            return L.SetLocal(c.scope, sc_rw(c.value, loop_syms))
        if isinstance(c, L.SetFromVec) and _count_gets([c], node):
            raise _NoInline()
        return c

    try:
        new = st_rw(use_stmt, [])
    except _NoInline:
        return None
    if budget is not None:
        return new if found["n"] >= 1 else None
    return new if found["n"] == 1 else None


class _NoInline(Exception):
    pass


def make_routine(g: Graph, name: str, body: List[L.Stmt], statics: Sequence[L.StaticSymbol] = (),
                 inline: bool = True, outputs: Sequence[L.Node] = ()) -> L.Routine:
    """``Train.to_routine`` (lib/train.ml:119-137): outputs are materialised; then the
    optimiser's inlining."""
    for n in outputs:
        n.mode = "ctx"
    if inline:
        body = inline_single_use(g, body, keep=outputs, visits=inline == "visits")
    return L.Routine(name, body, list(statics))


# ------------------------------------------------------------------------------------------------
# further operations used by the language-model configurations
# ------------------------------------------------------------------------------------------------

def rename(t: T, mapping: Dict[str, str]) -> T:
    """The same tensor under other axis labels (e.g. keys indexed by ``t`` instead of ``s``)."""
    return T(t.value, tuple(mapping.get(a, a) for a in t.axes), t.grad, (t,), label=t.label)


def gather_rows(g: Graph, table: T, ids: T, table_axis: str, ident: str = "embed") -> T:
    """Embedding lookup in the form the optimiser's one-hot rewrite produces
    (arrayjit/lib/low_level.ml:2193-2215): ``where(in_range(id), table[.., @dyn id, ..], 0)`` with
    the guard evaluated in double; the table gradient keeps the one-hot contraction
    ``g_table[e, v] += g[.., e] * (v == id[..])``."""
    out_axes = tuple(ids.axes) + tuple(a for a in table.axes if a != table_axis)
    ext = dict(zip(ids.axes, ids.dims))
    ext.update(dict(zip(table.axes, table.dims)))
    classes = ext[table_axis]
    v, gr = g._result(ident, out_axes, ext, None, table.grad is not None)
    res = T(v, out_axes, gr, (table, ids), label=ident)
    dyn_axis = table.axes.index(table_axis)

    def value(idx):
        iv = L.Get(ids.value, tuple(idx[a] for a in ids.axes))
        lower = L.Binop("lt", L.Const(-1.0), iv)
        upper = L.Binop("lt", iv, L.Const(float(classes)))
        integral = L.Binop("eq", iv, L.Unop("trunc", iv, "double"))
        guard = L.Binop("and", L.Binop("and", lower, upper), integral)
        tix = tuple(L.Fixed(0) if a == table_axis else idx[a] for a in table.axes)
        gather = L.GetDynamic(table.value, tix, dyn_axis, iv, ids.value.prec)
        return L.Ternop("where", guard, gather, L.Const(0.0), "double")

    space = [(a, ext[a]) for a in out_axes]
    res.fwd = g.lower(v, out_axes, space, value)

    def bwd():
        if table.grad is None:
            return []
        sp = space + [(table_axis, classes)]

        def rhs(idx):
            onehot = L.Binop("eq", L.EmbedIndex(idx[table_axis]), L.Get(ids.value, tuple(idx[a] for a in ids.axes)))
            return L.Binop("mul", L.Get(gr, tuple(idx[a] for a in out_axes)), onehot)

        return g.lower(table.grad, table.axes, sp, rhs, accum="add", init_neutral=False)

    res.bwd = bwd
    return res


def softmax(g: Graph, x: T, axis: str, ident: str = "softmax") -> T:
    """``Nn_blocks.softmax`` (lib/nn_blocks.ml:137-143): max over the axis, exp of the shifted
    values, division by their sum."""
    rest = tuple(a for a in x.axes if a != axis)
    max_vals = g.reduce(x, rest, accum="max", ident=ident + "_max")
    exp_vals = g.unary("exp", g.sub(x, max_vals, x.axes, ident=ident + "_shift"), ident=ident + "_exp")
    denom = g.reduce(exp_vals, rest, ident=ident + "_sum")
    return g.div(exp_vals, denom, x.axes, ident=ident)


def layer_norm(g: Graph, x: T, axis: str, label: str, epsilon: float = 1e-5):
    """``Nn_blocks.layer_norm`` exactly as written (lib/nn_blocks.ml:251-258): note that ``mean``
    there is the SUM over the axis and ``centered = (x - mean) / dim``."""
    rest = tuple(a for a in x.axes if a != axis)
    d = dict(zip(x.axes, x.dims))[axis]
    gamma = g.param(f"gamma_{label}", (axis,), (d,))
    beta = g.param(f"beta_{label}", (axis,), (d,))
    mean = g.reduce(x, rest, ident=f"mean_{label}")
    centered = g.div(g.sub(x, mean, x.axes), ConstT(float(d)), x.axes, ident=f"centered_{label}")
    variance = g.reduce(g.mul(centered, centered, x.axes), rest, ident=f"variance_{label}")
    std_dev = g.unary("sqrt", g.add(variance, ConstT(epsilon), rest), ident=f"std_{label}")
    normalized = g.div(centered, std_dev, x.axes, ident=f"normalized_{label}")
    out = g.add(g.mul(gamma, normalized, x.axes), beta, x.axes, ident=f"ln_{label}")
    return out, [gamma, beta]
