"""Low-level loop IR ("LLIR") exchanged across the backend boundary.

This is the data model of what OCANNL hands to a device backend: the record
``Low_level.optimized`` (arrayjit/lib/low_level.mli:160-166), i.e. the statement
type ``Low_level.t`` / ``scalar_t`` (low_level.mli:22-68), index expressions
``Indexing.axis_index`` (arrayjit/lib/indexing.ml:104-120), static index symbols
(indexing.ml:32-36), precisions ``Ops.prec`` (arrayjit/lib/ops.ml:35-48) and the
few ``Tnode.t`` / ``traced_array`` fields a backend reads (id, identifier,
precision, dims, memory mode, ``zero_initialized_by_code``, ``read_only``).

Three renderings exist:

* :func:`to_wire` -- the S-expression wire format parsed by the C++ library
  (``ocannl_hip_compile``).  The OCaml stub emits the same text.
* :func:`to_ll` -- the human ``.ll`` text of ``Low_level.to_doc``
  (low_level.ml:2544-2648); used to pin builders against ``*.ll.expected``.
* the C text produced by the CPU checker under ``oracle/``.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple, Union

# --------------------------------------------------------------------------------------
# Precisions (ops.ml:35-48, 209-222, 359-374)
# --------------------------------------------------------------------------------------

PRECS = (
    "void", "byte", "uint16", "int32", "uint32", "int64", "uint64", "uint4x32",
    "half", "bfloat16", "fp8", "single", "double",
)

PREC_BYTES = {
    "void": 0, "byte": 1, "uint16": 2, "int32": 4, "uint32": 4, "int64": 8, "uint64": 8,
    "uint4x32": 16, "half": 2, "bfloat16": 2, "fp8": 1, "single": 4, "double": 8,
}

FLOAT_PRECS = ("half", "bfloat16", "fp8", "single", "double")
INT_LIKE_PRECS = ("byte", "uint16", "int32", "uint32", "int64", "uint64", "fp8")

INDEX_PREC = "uint32"  # Ops.index_prec () without large_models (ops.ml:64)

_PROMOTE_ORDER = (
    "uint4x32", "double", "single", "bfloat16", "half", "fp8", "uint64", "int64", "uint32",
    "int32", "uint16", "byte",
)


def promote_prec(p1: str, p2: str) -> str:
    """``Ops.promote_prec`` (ops.ml:243-269): first match in dominance order wins."""
    for p in _PROMOTE_ORDER:
        if p1 == p:
            return p1
        if p2 == p:
            return p2
    return "void"


# --------------------------------------------------------------------------------------
# Operations (ops.ml:376-445)
# --------------------------------------------------------------------------------------

BINOPS = (
    "arg1", "arg2", "add", "sub", "mul", "div", "pow", "relu_gate", "sat01_gate", "max", "min",
    "mod", "lt", "eq", "ne", "or", "and", "threefry4x32_crypto", "threefry4x32_light",
)
UNOPS = (
    "id", "relu", "sat01", "exp", "log", "exp2", "log2", "sin", "cos", "sqrt", "recip",
    "recip_sqrt", "neg", "trunc", "tanh", "not", "uint4x32_to_prec_uniform1",
)
TERNOPS = ("where", "fma", "mul3")
VEC_UNOPS = ("uint4x32_to_prec_uniform",)

# ``.ll`` infix spellings (ops.ml:531-551) for the "nice infix" operators (ops.ml:527-529).
_LL_INFIX = {
    "add": "+", "sub": "-", "mul": "*", "div": "/", "pow": "**", "lt": "<", "eq": "=",
    "ne": "<>", "or": "||", "and": "&&", "mod": "%", "threefry4x32_crypto": "^^^^",
    "threefry4x32_light": "^^",
}
# uncurried fallback spellings (ops.ml:555-575)
_LL_PREFIX = {"arg1": "fst", "arg2": "snd", "relu_gate": "relu_gate",
              "sat01_gate": "sat01_gate", "max": "max", "min": "min"}


# --------------------------------------------------------------------------------------
# Tensor nodes, symbols, indices
# --------------------------------------------------------------------------------------

@dataclass(eq=False)
class Node:
    """The backend-visible part of a ``Tnode.t`` (tnode.ml:33-64) plus its traced flags.

    ``mode``: ``"ctx"`` -- materialised in the context: a kernel pointer parameter
    (c_syntax.ml:1028-1042 "Ctx"/"Global"); ``"local"`` -- lives only inside the routine
    (a C stack array in the ``cc`` backend, c_syntax.ml:1179-1196); ``"virtual"`` -- fully
    inlined, never stored.
    """

    id: int
    ident: str
    prec: str
    dims: Tuple[int, ...]
    mode: str = "ctx"
    zero_initialized_by_code: bool = False
    read_only: bool = False

    def __post_init__(self):
        assert self.prec in PRECS, self.prec
        assert self.mode in ("ctx", "local", "virtual"), self.mode
        self.dims = tuple(int(d) for d in self.dims)

    @property
    def num_elems(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n

    @property
    def size_in_bytes(self) -> int:
        return self.num_elems * PREC_BYTES[self.prec]

    def __repr__(self):
        return f"Node({self.id}:{self.ident}<{self.prec}>{list(self.dims)} {self.mode})"


_symbol_counter = [0]


def fresh_symbol() -> int:
    """``Indexing.get_symbol`` (indexing.ml:10-15)."""
    _symbol_counter[0] += 1
    return _symbol_counter[0]


def reset_symbols(start: int = 0) -> None:
    _symbol_counter[0] = start


@dataclass(frozen=True)
class StaticSymbol:
    """``Indexing.static_symbol`` (indexing.ml:32-36)."""

    sym: int
    range: Optional[int] = None


@dataclass(frozen=True)
class Fixed:
    i: int


@dataclass(frozen=True)
class It:
    sym: int


@dataclass(frozen=True)
class Affine:
    """Σ coeff·sym + offset (indexing.ml:107-116)."""

    terms: Tuple[Tuple[int, int], ...]
    offset: int = 0


@dataclass(frozen=True)
class SubAxis:
    """``Indexing.Sub_axis`` (indexing.ml:116): the axis belongs to an adjacent multi-axis index --
    the vectorised initialisers (assignments.ml:684-763) walk a whole tensor through an ``Affine``
    index on its last axis and mark the others ``Sub_axis``. It prints as nothing (indexing.ml:473)
    and adds nothing to the offset (indexing.ml:429, c_syntax.ml:367-379): position 0 of its axis."""


AxisIndex = Union[Fixed, It, Affine, SubAxis]


def sym_ident(s: int) -> str:
    return f"i{s}"


def axis_index_str(idx: AxisIndex) -> str:
    """``Doc_helpers.pp_axis_index`` (indexing.ml:454-476)."""
    if isinstance(idx, It):
        return sym_ident(idx.sym)
    if isinstance(idx, Fixed):
        return str(idx.i)
    if isinstance(idx, SubAxis):
        return ""
    terms = [sym_ident(s) if c == 1 else f"{c}*{sym_ident(s)}" for c, s in idx.terms]
    if idx.offset > 0:
        terms.append(str(idx.offset))
    elif idx.offset < 0:
        terms.append("-" + str(-idx.offset))
    if not terms:
        return "0"
    return "+".join(terms)


def index_symbols(idx: AxisIndex) -> Tuple[int, ...]:
    if isinstance(idx, It):
        return (idx.sym,)
    if isinstance(idx, Affine):
        return tuple(s for _, s in idx.terms)
    return ()


# --------------------------------------------------------------------------------------
# Scalars
# --------------------------------------------------------------------------------------

@dataclass(frozen=True)
class Scope:
    """``Low_level.scope_id`` (low_level.mli:8-16): a scalar local typed by its node."""

    node: Node
    scope_id: int

    @property
    def name(self) -> str:
        return f"v{self.scope_id}_{self.node.ident}"


@dataclass(eq=False)
class Get:
    node: Node
    idcs: Tuple[AxisIndex, ...]


@dataclass(eq=False)
class GetDynamic:
    """Guarded gather: axis ``dyn_axis`` of the offset is the integer value of ``dyn_value``
    (low_level.mli:43-52)."""

    node: Node
    idcs: Tuple[AxisIndex, ...]
    dyn_axis: int
    dyn_value: "Scalar"
    dyn_prec: str = ""

    def __post_init__(self):
        if not self.dyn_prec:
            self.dyn_prec = scalar_precision(self.dyn_value)


@dataclass(eq=False)
class GetMerge:
    node: Node
    idcs: Tuple[AxisIndex, ...]


@dataclass(eq=False)
class GetLocal:
    scope: Scope


@dataclass(eq=False)
class LocalScope:
    scope: Scope
    body: List["Stmt"]


@dataclass(eq=False)
class Const:
    value: float


@dataclass(eq=False)
class ConstBits:
    value: int


@dataclass(eq=False)
class EmbedIndex:
    idx: AxisIndex


@dataclass(eq=False)
class Unop:
    op: str
    arg: "Scalar"
    arg_prec: str = ""

    def __post_init__(self):
        assert self.op in UNOPS, self.op
        if not self.arg_prec:
            self.arg_prec = scalar_precision(self.arg)


@dataclass(eq=False)
class Binop:
    op: str
    a: "Scalar"
    b: "Scalar"

    def __post_init__(self):
        assert self.op in BINOPS, self.op


@dataclass(eq=False)
class Ternop:
    op: str
    a: "Scalar"
    b: "Scalar"
    c: "Scalar"
    a_prec: str = ""

    def __post_init__(self):
        assert self.op in TERNOPS, self.op
        if not self.a_prec:
            self.a_prec = scalar_precision(self.a)


Scalar = Union[Get, GetDynamic, GetMerge, GetLocal, LocalScope, Const, ConstBits, EmbedIndex,
               Unop, Binop, Ternop]


def scalar_precision(s: Scalar) -> str:
    """``Low_level.scalar_precision`` (low_level.ml:76-90)."""
    if isinstance(s, (Get, GetDynamic, GetMerge)):
        return s.node.prec
    if isinstance(s, (GetLocal, LocalScope)):
        return s.scope.node.prec
    if isinstance(s, Const):
        return "single"
    if isinstance(s, ConstBits):
        return "int64"
    if isinstance(s, EmbedIndex):
        return INDEX_PREC
    if isinstance(s, Ternop):
        return s.a_prec
    if isinstance(s, Binop):
        return scalar_precision(s.a)
    if isinstance(s, Unop):
        return s.arg_prec
    raise TypeError(s)


# --------------------------------------------------------------------------------------
# Statements
# --------------------------------------------------------------------------------------

@dataclass(eq=False)
class Comment:
    text: str


@dataclass(eq=False)
class For:
    sym: int
    from_: int
    to: int  # inclusive (c_syntax.ml:450-456)
    body: List["Stmt"]


@dataclass(eq=False)
class ZeroOut:
    node: Node


@dataclass(eq=False)
class Set:
    node: Node
    idcs: Tuple[AxisIndex, ...]
    value: Scalar


@dataclass(eq=False)
class SetFromVec:
    node: Node
    idcs: Tuple[AxisIndex, ...]
    length: int
    op: str
    arg: Scalar
    arg_prec: str = ""

    def __post_init__(self):
        assert self.op in VEC_UNOPS
        if not self.arg_prec:
            self.arg_prec = scalar_precision(self.arg)


@dataclass(eq=False)
class SetLocal:
    scope: Scope
    value: Scalar


@dataclass(eq=False)
class DeclareLocal:
    scope: Scope
    needs_init: bool = False


Stmt = Union[Comment, For, ZeroOut, Set, SetFromVec, SetLocal, DeclareLocal]


@dataclass(eq=False)
class Routine:
    """One compiled unit: ``Low_level.optimized`` + the name and static indices given to
    ``Lowered_backend.compile`` (backend_impl.ml:347)."""

    name: str
    body: List[Stmt]
    static_indices: List[StaticSymbol] = field(default_factory=list)
    merge_node: Optional[Node] = None

    def nodes(self) -> List[Node]:
        """All nodes mentioned by the code, in first-occurrence order."""
        seen, out = set(), []

        def visit(n: Node):
            if n.id not in seen:
                seen.add(n.id)
                out.append(n)

        def sc(s: Scalar):
            if isinstance(s, (Get, GetMerge)):
                visit(s.node)
            elif isinstance(s, GetDynamic):
                visit(s.node)
                sc(s.dyn_value)
            elif isinstance(s, GetLocal):
                visit(s.scope.node)
            elif isinstance(s, LocalScope):
                visit(s.scope.node)
                st(s.body)
            elif isinstance(s, Unop):
                sc(s.arg)
            elif isinstance(s, Binop):
                sc(s.a)
                sc(s.b)
            elif isinstance(s, Ternop):
                sc(s.a)
                sc(s.b)
                sc(s.c)

        def st(body: Sequence[Stmt]):
            for c in body:
                if isinstance(c, For):
                    st(c.body)
                elif isinstance(c, ZeroOut):
                    visit(c.node)
                elif isinstance(c, Set):
                    visit(c.node)
                    sc(c.value)
                elif isinstance(c, SetFromVec):
                    visit(c.node)
                    sc(c.arg)
                elif isinstance(c, SetLocal):
                    visit(c.scope.node)
                    sc(c.value)
                elif isinstance(c, DeclareLocal):
                    visit(c.scope.node)

        st(self.body)
        if self.merge_node is not None:
            visit(self.merge_node)
        return out

    def param_nodes(self) -> List[Node]:
        return [n for n in self.nodes() if n.mode == "ctx"]


def loop_over_dims(dims: Sequence[int], body) -> List[Stmt]:
    """``Low_level.loop_over_dims`` (low_level.ml:2657-2680): a fresh loop per axis of
    dimension > 1, ``Fixed 0`` otherwise; ``body(idcs) -> [Stmt]``."""

    def rec(rev_idcs, rest):
        if not rest:
            return body(tuple(reversed(rev_idcs)))
        d, *tail = rest
        if d == 1:
            return rec([Fixed(0)] + rev_idcs, tail)
        s = fresh_symbol()
        return [For(s, 0, d - 1, rec([It(s)] + rev_idcs, tail))]

    return rec([], list(dims))


def loop_over_padding_region(dims: Sequence[int], padding: Sequence[Tuple[int, int]], body) -> List[Stmt]:
    """``Low_level.loop_over_padding_region`` (low_level.ml:2705-2802): loops that visit exactly the
    margin of a padded node, never its data region. ``padding[axis] = (left, right)``. Per padded
    axis: the left strip over all remaining axes, the middle range recursing into the later axes,
    the right strip over all remaining axes; the left strip and the middle share one symbol, the
    right strip takes a fresh one. ``body(idcs) -> [Stmt]``."""
    dims = list(dims)

    def build(any_padding: bool, axis: int, rev_idcs) -> List[Stmt]:
        if axis >= len(dims):
            return body(tuple(reversed(rev_idcs))) if any_padding else []
        dim, (left, right) = dims[axis], padding[axis]
        index = fresh_symbol()
        if left <= 0 and right <= 0:
            return [For(index, 0, dim - 1, build(any_padding, axis + 1, [It(index)] + rev_idcs))]

        def strip(sym):
            return loop_over_dims(dims[axis + 1:], lambda rest: body(tuple(reversed(rev_idcs)) + (It(sym),) + tuple(rest)))

        out: List[Stmt] = []
        if left > 0:
            out.append(For(index, 0, left - 1, strip(index)))
        if left <= dim - right - 1:
            out.append(For(index, left, dim - right - 1, build(any_padding, axis + 1, [It(index)] + rev_idcs)))
        if right > 0:
            right_index = fresh_symbol()
            out.append(For(right_index, dim - right, dim - 1, strip(right_index)))
        return out

    return build(False, 0, [])


# --------------------------------------------------------------------------------------
# ``.ll`` text (low_level.ml:2544-2648)
# --------------------------------------------------------------------------------------

def fmt_g16(c: float) -> str:
    """OCaml ``Printf.sprintf "%.16g"``."""
    return "%.16g" % c


def _ll_printers(with_prec: bool = False):
    """(scalar printer, statement printer) of the ``.ll`` text form."""
    def ident(n: Node) -> str:
        return n.ident + (f"<{n.prec}>" if with_prec else "")

    def local(s: Scope) -> str:
        return f"v{s.scope_id}_" + ident(s.node)

    def idcs(ix) -> str:
        return ", ".join(axis_index_str(i) for i in ix)

    def sc(s: Scalar) -> str:
        if isinstance(s, LocalScope):
            return local(s.scope) + " { " + " ".join(st(c) for c in s.body) + " }"
        if isinstance(s, GetLocal):
            return local(s.scope)
        if isinstance(s, GetMerge):
            return f"{ident(s.node)}.merge[{idcs(s.idcs)}]"
        if isinstance(s, Get):
            return f"{ident(s.node)}[{idcs(s.idcs)}]"
        if isinstance(s, GetDynamic):
            return f"{ident(s.node)}[{idcs(s.idcs)}]@dyn[{s.dyn_axis}]=({sc(s.dyn_value)})"
        if isinstance(s, Const):
            return fmt_g16(s.value)
        if isinstance(s, ConstBits):
            return "0x%X" % s.value
        if isinstance(s, EmbedIndex):
            return axis_index_str(s.idx)
        if isinstance(s, Ternop):
            return f"{s.op}({sc(s.a)}, {sc(s.b)}, {sc(s.c)})"
        if isinstance(s, Binop):
            if s.op == "arg1":
                return sc(s.a)
            if s.op == "arg2":
                return sc(s.b)
            if s.op in _LL_INFIX:
                return f"({sc(s.a)} {_LL_INFIX[s.op]} {sc(s.b)})"
            return f"{_LL_PREFIX[s.op]}({sc(s.a)}, {sc(s.b)})"
        if isinstance(s, Unop):
            if s.op == "id":
                return sc(s.arg)
            return f"{s.op}({sc(s.arg)})"
        raise TypeError(s)

    def st(c: Stmt) -> str:
        if isinstance(c, Comment):
            return f"/* {c.text} */"
        if isinstance(c, For):
            return (f"for {sym_ident(c.sym)} = {c.from_} to {c.to} {{ "
                    + " ".join(st(x) for x in c.body) + " }")
        if isinstance(c, ZeroOut):
            return f"zero_out {ident(c.node)};"
        if isinstance(c, Set):
            return f"{ident(c.node)}[{idcs(c.idcs)}] := {sc(c.value)};"
        if isinstance(c, SetFromVec):
            return (f"{ident(c.node)}[{idcs(c.idcs)}]<{c.length}> := "
                    f"{c.op}({sc(c.arg)}, <{c.length}>);")
        if isinstance(c, SetLocal):
            return f"{local(c.scope)} := {sc(c.value)};"
        if isinstance(c, DeclareLocal):
            return f"declare {local(c.scope)};"
        raise TypeError(c)

    return sc, st


def ll_statement(c: "Stmt", with_prec: bool = False) -> str:
    """One statement in the ``.ll`` text form: what the reference attaches to a ``Set`` as its
    ``debug`` string (the text that in-routine logging prints after ``# ``)."""
    return _ll_printers(with_prec)[1](c)


def to_ll(r: Routine, with_prec: bool = False) -> str:
    _, st = _ll_printers(with_prec)

    def static(s: StaticSymbol) -> str:
        if s.range is None:
            return sym_ident(s.sym)
        return f"{sym_ident(s.sym)} : [0..{s.range - 1}]"

    head = f"{r.name} ({', '.join(static(s) for s in r.static_indices)}): "
    return head + " ".join(st(c) for c in r.body)


# --------------------------------------------------------------------------------------
# Wire format
# --------------------------------------------------------------------------------------

def _q(s: str) -> str:
    return '"' + s.replace("\\", "\\\\").replace('"', '\\"') + '"'


def _wire_idx(i: AxisIndex) -> str:
    if isinstance(i, Fixed):
        return f"(fixed {i.i})"
    if isinstance(i, It):
        return f"(it {i.sym})"
    if isinstance(i, SubAxis):
        return "(sub)"
    terms = " ".join(f"({c} {s})" for c, s in i.terms)
    return f"(affine ({terms}) {i.offset})"


def _wire_idcs(ix) -> str:
    return "(" + " ".join(_wire_idx(i) for i in ix) + ")"


def _wire_scalar(s: Scalar) -> str:
    if isinstance(s, Get):
        return f"(get {s.node.id} {_wire_idcs(s.idcs)})"
    if isinstance(s, GetMerge):
        return f"(get_merge {s.node.id} {_wire_idcs(s.idcs)})"
    if isinstance(s, GetDynamic):
        return (f"(get_dyn {s.node.id} {_wire_idcs(s.idcs)} {s.dyn_axis} {s.dyn_prec} "
                f"{_wire_scalar(s.dyn_value)})")
    if isinstance(s, GetLocal):
        return f"(get_local {s.scope.node.id} {s.scope.scope_id})"
    if isinstance(s, LocalScope):
        return (f"(local_scope {s.scope.node.id} {s.scope.scope_id} "
                f"{_wire_stmts(s.body)})")
    if isinstance(s, Const):
        return f"(const {float(s.value).hex()})"
    if isinstance(s, ConstBits):
        return f"(bits {int(s.value)})"
    if isinstance(s, EmbedIndex):
        return f"(index {_wire_idx(s.idx)})"
    if isinstance(s, Unop):
        return f"(unop {s.op} {s.arg_prec} {_wire_scalar(s.arg)})"
    if isinstance(s, Binop):
        return f"(binop {s.op} {_wire_scalar(s.a)} {_wire_scalar(s.b)})"
    if isinstance(s, Ternop):
        return (f"(ternop {s.op} {s.a_prec} {_wire_scalar(s.a)} {_wire_scalar(s.b)} "
                f"{_wire_scalar(s.c)})")
    raise TypeError(s)


_WIRE_DEBUG = [False]   # to_wire(..., debug=True): every Set carries its `.ll` text


def _wire_stmt(c: Stmt) -> str:
    if isinstance(c, Comment):
        return f"(comment {_q(c.text)})"
    if isinstance(c, For):
        return f"(for {c.sym} {c.from_} {c.to} {_wire_stmts(c.body)})"
    if isinstance(c, ZeroOut):
        return f"(zero_out {c.node.id})"
    if isinstance(c, Set):
        if _WIRE_DEBUG[0]:
            return f"(set {c.node.id} {_wire_idcs(c.idcs)} {_wire_scalar(c.value)} {_q(ll_statement(c))})"
        return f"(set {c.node.id} {_wire_idcs(c.idcs)} {_wire_scalar(c.value)})"
    if isinstance(c, SetFromVec):
        return (f"(set_vec {c.node.id} {_wire_idcs(c.idcs)} {c.length} {c.op} {c.arg_prec} "
                f"{_wire_scalar(c.arg)})")
    if isinstance(c, SetLocal):
        return f"(set_local {c.scope.node.id} {c.scope.scope_id} {_wire_scalar(c.value)})"
    if isinstance(c, DeclareLocal):
        return (f"(declare_local {c.scope.node.id} {c.scope.scope_id} "
                f"{1 if c.needs_init else 0})")
    raise TypeError(c)


def _wire_stmts(body: Sequence[Stmt]) -> str:
    return "(" + "\n".join(_wire_stmt(c) for c in body) + ")"


def to_wire(r: Routine, debug: bool = False) -> str:
    """Serialise a routine (``debug``: every ``set`` carries, as a last string, the statement's
    ``.ll`` text -- the ``debug`` field of ``Low_level.Set`` that in-routine logging prints).  Grammar (S-expressions; atoms are integers, identifiers,
    C99 hex floats, or double-quoted strings)::

        (routine NAME
          (static (SYM RANGE|-1) ...)
          (merge NODE_ID|-1)
          (nodes (ID IDENT PREC MODE ZERO_INIT READ_ONLY (DIM ...)) ...)
          (body STMT ...))
    """
    _WIRE_DEBUG[0] = debug
    try:
        body_text = _wire_stmts(r.body)[1:-1]
    finally:
        _WIRE_DEBUG[0] = False
    statics = " ".join(f"({s.sym} {-1 if s.range is None else s.range})"
                       for s in r.static_indices)
    nodes = "\n".join(
        f"({n.id} {_q(n.ident)} {n.prec} {n.mode} {int(n.zero_initialized_by_code)} "
        f"{int(n.read_only)} ({' '.join(str(d) for d in n.dims)}))"
        for n in r.nodes())
    merge = -1 if r.merge_node is None else r.merge_node.id
    return (f"(routine {_q(r.name)}\n(static {statics})\n(merge {merge})\n(nodes\n{nodes})\n"
            f"(body\n{body_text}))\n")
