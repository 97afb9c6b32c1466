"""TEST INFRASTRUCTURE -- CPU checker, not part of the shipped product path.

Restatement of OCANNL's ``cc`` backend code printer: given a routine in the loop IR, produce
the C translation unit the reference would hand to ``cc -O3 -march=native -shared -fPIC``.

Follows, function by function:

* ``C_syntax.compile_proc``      arrayjit/lib/c_syntax.ml:1021-1210  -> :func:`emit_proc`
* ``C_syntax.pp_ll``             c_syntax.ml:441-704                 -> :meth:`_Emitter.stmt`
* ``C_syntax.pp_scalar``         c_syntax.ml:706-855                 -> :meth:`_Emitter.scalar`
* ``C_syntax.pp_array_offset``   c_syntax.ml:367-379                 -> :func:`array_offset`
* ``Pure_C_config``              c_syntax.ml:96-321 (uint32_t loop indices, uint64_t under the
  ``large_models`` setting; no prefixes)
* ``CC_syntax_config`` overrides arrayjit/lib/cc_backend.ml:155-323 (bf16/half/fp8 computed in
  float with a conversion around every single operation)
* op spelling tables             arrayjit/lib/ops.ml:579-863
* ``reads_scope_before_set``     arrayjit/lib/low_level.ml:1998-2037

Pinned by: token-for-token equality with the reference-held generated C
(test/operations/top_down_prec.c.expected, zero_out_local_decl.c.expected,
test_where_precision.c.expected, arrayjit/test/test_zero_out_codegen.expected,
arrayjit/test/test_local_scope_init.expected) in tests/test_oracle_emit.py.

Layout differs from the reference's PPrint output only in white space (line breaking).

Debug-log emission (``debug_log_from_routines``, c_syntax.ml:441-704 log branches, ``debug_float``
c_syntax.ml:857-1018, the parameter header c_syntax.ml:1112-1150, ``Pure_C_config.pp_log_statement``
c_syntax.ml:299-321) is restated too (``emit_proc(..., debug_log=True)``): pinned by token equality
with test/operations/test_log_stmt_format.c.expected (tests/test_oracle_emit.py).
"""
from __future__ import annotations

import os
import sys
from typing import Dict, List, Sequence, Tuple

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from ocannl_amd import llir as L  # noqa: E402

# ---------------------------------------------------------------------------------------
# ops.ml tables
# ---------------------------------------------------------------------------------------

C_TYP = {  # Ops.c_typ_of_prec, ops.ml:324-337
    "byte": "unsigned char", "uint16": "unsigned short", "int32": "int", "uint32": "uint32_t",
    "int64": "long long", "uint64": "uint64_t", "uint4x32": "uint4x32_t", "half": "HALF_T",
    "bfloat16": "unsigned short", "fp8": "unsigned char", "single": "float", "double": "double",
    "void": "void",
}

# ``Utils.settings.large_models``: a startup-fixed global of the reference, read when the source is
# generated (c_syntax.ml:17-24). It widens loop indices and integer arguments to 64 bits
# (c_syntax.ml:111-112) and ``Ops.index_prec ()`` to uint64 (ops.ml:64).
LARGE_MODELS = False


def index_prec() -> str:
    return "uint64" if LARGE_MODELS else L.INDEX_PREC


_INTISH = ("byte", "uint16", "int32", "uint32", "int64", "uint64", "fp8")
_DBL_OR_INTISH = ("double",) + _INTISH


def c_vec_typ(length: int, prec: str) -> str:
    """Ops.c_vec_typ_of_prec, ops.ml:339-351."""
    table = {
        ("single", 4): "float4_t", ("double", 2): "double2_t", ("int32", 4): "int32x4_t",
        ("uint32", 4): "uint32x4_t", ("int64", 2): "int64x2_t", ("uint64", 2): "uint64x2_t",
        ("byte", 16): "int8x16_t", ("fp8", 16): "int8x16_t", ("uint16", 8): "uint16x8_t",
        ("bfloat16", 8): "uint16x8_t", ("half", 8): "half8_t",
    }
    if (prec, length) in table:
        return table[(prec, length)]
    if length == 1:
        return C_TYP[prec]
    raise ValueError("c_vec_typ: invalid combination")


def binop_c_syntax(prec: str, op: str) -> Tuple[str, str, str]:
    """Ops.binop_c_syntax, ops.ml:579-630."""
    if op in ("add", "sub", "mul", "div"):
        return ("(", {"add": " +", "sub": " -", "mul": " *", "div": " /"}[op], ")")
    if op == "pow":
        if prec == "double":
            return ("pow(", ",", ")")
        if prec in _INTISH:
            raise ValueError("ToPowOf not supported for integer precisions")
        return ("powf(", ",", ")")
    if op == "relu_gate":
        return ("(", " > 0 ?", " : 0)") if prec in _INTISH else ("(", " > 0.0 ?", " : 0.0)")
    if op == "sat01_gate":
        if prec in _INTISH:
            return ("(abs(", " ) > 0 ? 0 : (", "))")
        if prec == "single":
            return ("(fabsf(floorf(", ")) > 0.0 ? 0.0 : (", "))")
        return ("(fabs(floor(", ")) > 0.0 ? 0.0 : (", "))")
    if op == "max":
        return ("fmax(", ",", ")") if prec in _DBL_OR_INTISH else ("fmaxf(", ",", ")")
    if op == "min":
        return ("fmin(", ",", ")") if prec in _DBL_OR_INTISH else ("fminf(", ",", ")")
    simple = {"mod": " %", "lt": " <", "eq": " ==", "ne": " !=", "or": " ||", "and": " &&"}
    if op in simple:
        return ("(", simple[op], ")")
    if op == "threefry4x32_crypto":
        return ("arrayjit_threefry4x32_crypto(", ",", ")")
    if op == "threefry4x32_light":
        return ("arrayjit_threefry4x32_light(", ",", ")")
    raise ValueError(f"binop_c_syntax: {op} is not an operator")


def unop_c_syntax(prec: str, op: str) -> Tuple[str, str]:
    """Ops.unop_c_syntax, ops.ml:688-782."""
    wide = prec in _DBL_OR_INTISH
    fmax = "fmax" if wide else "fmaxf"
    fmin = "fmin" if wide else "fminf"
    if op == "id":
        return ("", "")
    if op == "relu":
        return ("fmax(0, ", ")") if prec in _INTISH else (fmax + "(0.0, ", ")")
    if op == "sat01":
        if prec in _INTISH:
            return ("fmax(0, fmin(1, ", "))")
        return (fmax + "(0.0, " + fmin + "(1.0, ", "))")
    libm = {"exp": "exp", "log": "log", "exp2": "exp2", "log2": "log2", "sin": "sin",
            "cos": "cos", "sqrt": "sqrt"}
    if op in libm:
        return ((libm[op] if wide else libm[op] + "f") + "(", ")")
    if op == "recip":
        if prec in _INTISH:
            raise ValueError("Recip not supported for integer precisions")
        return ("(1.0 / (", "))")
    if op == "recip_sqrt":
        if prec in _INTISH:
            raise ValueError("Recip_sqrt not supported for integer precisions")
        return ("(1.0 / sqrt(", "))") if prec == "double" else ("(1.0 / sqrtf(", "))")
    if op == "neg":
        return ("(-(", "))")
    if op == "trunc":
        return ("trunc(", ")") if prec == "double" else ("truncf(", ")")
    if op == "tanh":
        if prec in _INTISH:
            raise ValueError("Tanh_approx not supported for integer precisions")
        return ("tanhf(", ")")
    if op == "not":
        return ("(", " == 0.0 ? 1.0 : 0.0)")
    if op == "uint4x32_to_prec_uniform1":
        if prec == "uint4x32":
            raise ValueError("Uint4x32_to_prec_uniform1 not supported for Uint4x32")
        return ("uint4x32_to_" + prec + "_uniform(", ")")
    raise ValueError(op)


def vec_unop_c_syntax(prec: str, op: str) -> Tuple[str, str]:
    """Ops.vec_unop_c_syntax, ops.ml:784-788."""
    if prec == "uint4x32":
        raise ValueError("Uint4x32_to_prec_uniform not supported for Uint4x32")
    return ("uint4x32_to_" + prec + "_uniform_vec(", ")")


def ternop_c_syntax(prec: str, op: str) -> Tuple[str, str, str, str]:
    """Ops.ternop_c_syntax, ops.ml:793-806."""
    if op == "where":
        if prec in _INTISH:
            return ("((", ") != 0 ? (", ") : (", "))")
        return ("((", ") != 0.0 ? (", ") : (", "))")
    if op == "fma":
        return ("fma(", ",", ",", ")") if prec in _DBL_OR_INTISH else ("fmaf(", ",", ",", ")")
    if op == "mul3":
        return ("((", ") * (", ") * (", "))")
    raise ValueError(op)


_PLAIN_INTS = ("byte", "uint16", "int32", "uint32", "int64", "uint64")


def convert_precision(from_: str, to: str) -> Tuple[str, str]:
    """Ops.c_convert_precision, ops.ml:808-876."""
    if from_ == to:
        return ("", "")
    f, t = from_, to
    if (f, t) == ("bfloat16", "single"):
        return ("bfloat16_to_single(", ")")
    if (f, t) == ("single", "bfloat16"):
        return ("single_to_bfloat16(", ")")
    if (f, t) == ("bfloat16", "double"):
        return ("(double)bfloat16_to_single(", ")")
    if (f, t) == ("double", "bfloat16"):
        return ("single_to_bfloat16((float)", ")")
    if (f, t) == ("fp8", "single"):
        return ("fp8_to_single(", ")")
    if (f, t) == ("single", "fp8"):
        return ("single_to_fp8(", ")")
    if (f, t) == ("fp8", "double"):
        return ("(double)fp8_to_single(", ")")
    if (f, t) == ("double", "fp8"):
        return ("single_to_fp8((float)", ")")
    if (f, t) == ("bfloat16", "half"):
        return ("FLOAT_TO_HALF(bfloat16_to_single(", "))")
    if (f, t) == ("half", "bfloat16"):
        return ("single_to_bfloat16(HALF_TO_FLOAT(", "))")
    if f == "bfloat16" and t in _PLAIN_INTS:
        return ("(" + C_TYP[t] + ")bfloat16_to_single(", ")")
    if f in _PLAIN_INTS and t == "bfloat16":
        return ("single_to_bfloat16((float)", ")")
    if (f, t) == ("fp8", "half"):
        return ("FLOAT_TO_HALF(fp8_to_single(", "))")
    if (f, t) == ("half", "fp8"):
        return ("single_to_fp8(HALF_TO_FLOAT(", "))")
    if f == "fp8" and t in _PLAIN_INTS:
        return ("(" + C_TYP[t] + ")fp8_to_single(", ")")
    if f in _PLAIN_INTS and t == "fp8":
        return ("single_to_fp8((float)", ")")
    if (f, t) == ("bfloat16", "fp8"):
        return ("single_to_fp8(bfloat16_to_single(", "))")
    if (f, t) == ("fp8", "bfloat16"):
        return ("single_to_bfloat16(fp8_to_single(", "))")
    if (f, t) == ("half", "single"):
        return ("HALF_TO_FLOAT(", ")")
    if (f, t) == ("single", "half"):
        return ("FLOAT_TO_HALF(", ")")
    if (f, t) == ("half", "double"):
        return ("(double)HALF_TO_FLOAT(", ")")
    if (f, t) == ("double", "half"):
        return ("FLOAT_TO_HALF((float)", ")")
    if f == "half" and t in _PLAIN_INTS:
        return ("(" + C_TYP[t] + ")HALF_TO_FLOAT(", ")")
    if f in _PLAIN_INTS and t == "half":
        return ("FLOAT_TO_HALF((float)", ")")
    if f == "uint4x32":
        return ("uint4x32_to_" + t + "(", ")")
    if t == "uint4x32":
        return (f + "_to_uint4x32(", ")")
    return ("(" + C_TYP[t] + ")(", ")")


# cc_backend.ml:169-323: reduced precisions compute in float around each operation.
_VIA_FLOAT = {
    "bfloat16": ("bfloat16_to_single(", "single_to_bfloat16("),
    "half": ("HALF_TO_FP(", "FP_TO_HALF("),
    "fp8": ("fp8_to_single(", "single_to_fp8("),
}


def cc_ternop(prec: str, op: str, v1: str, v2: str, v3: str) -> str:
    if prec in _VIA_FLOAT:
        to_f, from_f = _VIA_FLOAT[prec]
        p, i1, i2, s = ternop_c_syntax("single", op)
        return f"{from_f}{p}{to_f}{v1}){i1} {to_f}{v2}){i2} {to_f}{v3}){s})"
    p, i1, i2, s = ternop_c_syntax(prec, op)
    return f"{p}{v1}{i1} {v2}{i2} {v3}{s}"


def cc_binop(prec: str, op: str, v1: str, v2: str) -> str:
    if op in ("threefry4x32_crypto", "threefry4x32_light"):
        if prec != "uint4x32":
            raise ValueError(f"{op} on non-uint4x32 precision")
        return f"arrayjit_{op}({v1}, {v2})"
    if prec in _VIA_FLOAT:
        to_f, from_f = _VIA_FLOAT[prec]
        p, i, s = binop_c_syntax("single", op)
        return f"{from_f}{p}{to_f}{v1}){i} {to_f}{v2}){s})"
    p, i, s = binop_c_syntax(prec, op)
    return f"{p}{v1}{i} {v2}{s}"


def cc_unop(prec: str, op: str, v: str) -> str:
    if prec in _VIA_FLOAT:
        to_f, from_f = _VIA_FLOAT[prec]
        p, s = unop_c_syntax("single", op)
        return f"{from_f}{p}{to_f}{v}){s})"
    p, s = unop_c_syntax(prec, op)
    return f"{p}{v}{s}"


# ---------------------------------------------------------------------------------------
# printer
# ---------------------------------------------------------------------------------------

def array_offset(idcs: Sequence[L.AxisIndex], dims: Sequence[int]) -> str:
    """Row-major Horner form ``((i0) * d1 + i1) * d2 + i2`` (c_syntax.ml:367-379)."""
    if len(idcs) == 0:
        return "0"
    doc = L.axis_index_str(idcs[0])
    for i in range(1, len(idcs)):
        ix = L.axis_index_str(idcs[i])
        if doc == "":                       # only Sub_axis so far: nothing to scale yet
            doc = ix
        elif ix == "":                      # Sub_axis: the axis is spanned, no position of its own
            doc = f"({doc}) * {dims[i]}"
        else:
            doc = f"({doc}) * {dims[i]} + {ix}"
    return doc


def const_str(c: float) -> str:
    if c == float("inf"):
        return "INFINITY"
    if c == float("-inf"):
        return "(-INFINITY)"
    if c != c:
        return "NAN"
    return L.fmt_g16(c)


def reads_scope_before_set(target: L.Scope, body: Sequence[L.Stmt]) -> bool:
    """low_level.ml:1998-2037."""

    def same(s: L.Scope) -> bool:
        return s.scope_id == target.scope_id and s.node.id == target.node.id

    def sc_reads(s) -> bool:
        if isinstance(s, L.GetLocal):
            return same(s.scope)
        if isinstance(s, L.LocalScope):
            return any(st_reads(c) for c in s.body)
        if isinstance(s, L.Ternop):
            return sc_reads(s.a) or sc_reads(s.b) or sc_reads(s.c)
        if isinstance(s, L.Binop):
            return sc_reads(s.a) or sc_reads(s.b)
        if isinstance(s, L.Unop):
            return sc_reads(s.arg)
        if isinstance(s, L.GetDynamic):
            return sc_reads(s.dyn_value)
        return False

    def st_reads(c) -> bool:
        if isinstance(c, L.For):
            return any(st_reads(x) for x in c.body)
        if isinstance(c, L.Set):
            return sc_reads(c.value)
        if isinstance(c, L.SetFromVec):
            return sc_reads(c.arg)
        if isinstance(c, L.SetLocal):
            return sc_reads(c.value)
        return False

    def scan_seq(stmts) -> str:
        for c in stmts:
            r = scan(c)
            if r != "neither":
                return r
        return "neither"

    def scan(c) -> str:
        if isinstance(c, L.Set):
            return "read" if sc_reads(c.value) else "neither"
        if isinstance(c, L.SetFromVec):
            return "read" if sc_reads(c.arg) else "neither"
        if isinstance(c, L.SetLocal):
            if sc_reads(c.value):
                return "read"
            return "written" if same(c.scope) else "neither"
        if isinstance(c, L.For):
            r = scan_seq(c.body)
            if r == "written":
                return "written" if c.from_ <= c.to else "neither"
            return r
        return "neither"

    return scan_seq(body) != "written"


class _Emitter:
    def __init__(self, routine: L.Routine, debug_log: bool = False, full_printf: bool = True):
        self.r = routine
        self.zero_out_seen = set()
        # debug_log_from_routines (utils.ml:591): every statement logs what it computes.
        # full_printf: `%g` values; otherwise (the `prefer_backend_uniformity` setting,
        # cc_backend.ml:164-165) `%de-3` of the value times 1000 (c_syntax.ml:117-123).
        self.debug_log = debug_log
        self.float_log_style = "%g" if full_printf else "%de-3"
        self.full_printf = full_printf

    # -- logging (Pure_C_config, c_syntax.ml:117-123,293-321)
    def styled_log_arg(self, doc: str) -> str:
        return doc if self.full_printf else f"(int)({doc} * 1000.0)"

    def log_statement(self, base_message: str, args: Sequence[str]) -> str:
        lit = base_message.replace("\n", "\\n")
        tail = "".join(", " + a for a in args)
        return f'if (log_file_name && log_file) fprintf(log_file, "{lit}"{tail});'

    def debug_float(self, prec: str, s: L.Scalar, guard: str = None):
        """c_syntax.ml:857-1018: the expression as the log shows it, with `{=value}` after every read,
        and the printf arguments behind it: ("acc", offset expression) | ("val", C expression)."""
        st = self.float_log_style

        def guarded(access: str) -> str:
            return access if guard is None else f"({guard} ? {access} : 0)"

        if isinstance(s, L.LocalScope):
            return self.debug_float(prec, L.GetLocal(s.scope), guard)
        if isinstance(s, L.GetLocal):
            p, q = convert_precision(s.scope.node.prec, prec)
            v = f"{p}{self.scope_name(s.scope)}{q}"
            return v + "{=" + st + "}", [("val", v)]
        if isinstance(s, L.GetMerge):
            p, q = convert_precision(s.node.prec, prec)
            off = array_offset(s.idcs, s.node.dims)
            return f"{p}merge_buffer[%u]{q}" + "{=" + st + "}", [("acc", off), ("val", guarded(f"{p}merge_buffer[{off}]{q}"))]
        if isinstance(s, L.Get):
            p, q = convert_precision(s.node.prec, prec)
            off = array_offset(s.idcs, s.node.dims)
            return f"{p}{s.node.ident}[%u]{q}" + "{=" + st + "}", [("acc", off), ("val", guarded(f"{p}{s.node.ident}[{off}]{q}"))]
        if isinstance(s, L.GetDynamic):
            p, q = convert_precision(s.dyn_prec, prec)
            _, idx_e = self.scalar(s.dyn_prec, s.dyn_value, "")
            return f"{s.node.ident}@dyn_idx" + "{=" + st + "}", [("val", f"{p}{idx_e}{q}")]
        if isinstance(s, L.Const):
            p, q = convert_precision("double", prec)
            return f"{p}{const_str(s.value)}{q}", []
        if isinstance(s, L.ConstBits):
            p, q = convert_precision("int64", prec)
            return f"{p}{int(s.value)}LL{q}", []
        if isinstance(s, L.EmbedIndex):
            ix = L.axis_index_str(s.idx)
            return (ix if ix else "0"), []
        if isinstance(s, L.Binop) and s.op == "arg1":
            return self.debug_float(prec, s.a, guard)
        if isinstance(s, L.Binop) and s.op == "arg2":
            return self.debug_float(prec, s.b, guard)
        if isinstance(s, L.Ternop):
            if s.op == "where":
                _, cond_c = self.scalar(s.a_prec, s.a, "")
                compose = lambda c: c if guard is None else f"({guard} && {c})"   # noqa: E731
                d1, a1 = self.debug_float(s.a_prec, s.a, guard)
                d2, a2 = self.debug_float(prec, s.b, compose(cond_c))
                d3, a3 = self.debug_float(prec, s.c, compose(f"(!({cond_c}))"))
            else:
                d1, a1 = self.debug_float(prec, s.a, guard)
                d2, a2 = self.debug_float(prec, s.b, guard)
                d3, a3 = self.debug_float(prec, s.c, guard)
            return cc_ternop(prec, s.op, d1, d2, d3), a1 + a2 + a3
        if isinstance(s, L.Binop):
            d1, a1 = self.debug_float(prec, s.a, guard)
            d2, a2 = self.debug_float(prec, s.b, guard)
            return cc_binop(prec, s.op, d1, d2), a1 + a2
        if isinstance(s, L.Unop):
            arg_prec = s.arg_prec if s.op == "uint4x32_to_prec_uniform1" else prec
            d, a = self.debug_float(arg_prec, s.arg, guard)
            return cc_unop(prec, s.op, d), a
        raise TypeError(s)

    def _log_args(self, args) -> List[str]:
        return [a if kind == "acc" else self.styled_log_arg(a) for kind, a in args]

    # -- c_syntax.ml:424-432
    def zero_out_loop_redundant(self, n: L.Node) -> bool:
        return n.zero_initialized_by_code and n.mode == "local"

    def scope_name(self, s: L.Scope) -> str:
        return f"v{s.scope_id}_{s.node.ident}"

    def init_zero(self, prec: str) -> str:
        p, s = convert_precision("int32", prec)
        return f" = {p}0{s}"

    def stmts(self, body: Sequence[L.Stmt], ind: str, in_loop: bool, log_set_locals: bool = True) -> List[str]:
        out: List[str] = []
        for c in body:
            out.extend(self.stmt(c, ind, in_loop, log_set_locals))
        return out

    def stmt(self, c: L.Stmt, ind: str, in_loop: bool, log_set_locals: bool = True) -> List[str]:
        if isinstance(c, L.Comment):
            if self.debug_log:
                return [ind + self.log_statement("COMMENT: " + c.text + "\n", [])]
            return [f"{ind}/* {c.text} */"]
        if isinstance(c, L.For):
            s = L.sym_ident(c.sym)
            head = f"{ind}for ({C_TYP[index_prec()]} {s} = {c.from_}; {s} <= {c.to}; ++{s}) {{"
            body = self.stmts(c.body, ind + "  ", True, log_set_locals)
            if self.debug_log:
                body = [ind + "  " + self.log_statement(f"index {s} = %d\n", [s])] + body
            return [head] + body + [ind + "}"]
        if isinstance(c, L.ZeroOut):
            first = c.node.id not in self.zero_out_seen
            self.zero_out_seen.add(c.node.id)
            if first and not in_loop and self.zero_out_loop_redundant(c.node):
                return []
            node = c.node

            def zero(idcs):
                st = L.Set(node, idcs, L.Const(0.0))
                st.debug = node.ident + " := 0"          # c_syntax.ml:479
                return [st]
            loops = L.loop_over_dims(node.dims, zero)
            return self.stmts(loops, ind, in_loop, log_set_locals)
        if isinstance(c, L.Set):
            defs, val = self.scalar(c.node.prec, c.value, ind + "  ")
            off = array_offset(c.idcs, c.node.dims)
            if self.debug_log:                           # c_syntax.ml:493-535
                st = self.float_log_style
                dbg, args = self.debug_float(c.node.prec, c.value)
                text = getattr(c, "debug", None) or L.ll_statement(c)
                lhs = f"{c.node.ident}[{off}]"
                lines = [f"{C_TYP[c.node.prec]} new_set_v = {val};",
                         self.log_statement("# " + text + "\n", []),
                         self.log_statement(f"{c.node.ident}[%u]{{={st}}} = {st} = {dbg}\n",
                                            [off, self.styled_log_arg(lhs), self.styled_log_arg("new_set_v")]
                                            + self._log_args(args)),
                         "fflush(log_file);",
                         f"{lhs} = new_set_v;"]
                return self._with_defs(defs, lines, ind, always_block=True)
            asg = f"{c.node.ident}[{off}] = {val};"
            return self._with_defs(defs, [asg], ind)
        if isinstance(c, L.SetFromVec):
            prec = c.node.prec
            defs, arg = self.scalar(c.arg_prec, c.arg, ind + "  ")
            p, s = vec_unop_c_syntax(prec, c.op)
            lines = [f"{c_vec_typ(c.length, prec)} vec_result = {p}{arg}{s};"]
            for i in range(c.length):
                last = c.idcs[-1]
                if isinstance(last, L.Fixed):
                    el = tuple(c.idcs[:-1]) + (L.Fixed(last.i + i),)
                    off = array_offset(el, c.node.dims)
                else:
                    off = array_offset(c.idcs, c.node.dims) + f" + {i}"
                v = "vec_result" if c.length == 1 else f"vec_result.v[{i}]"
                lines.append(f"{c.node.ident}[{off}] = {v};")
            if self.debug_log:                           # c_syntax.ml:590-640
                st = self.float_log_style
                text = getattr(c, "debug", None) or L.ll_statement(c)
                logs = [self.log_statement("# " + text + "\n", [])]
                for i in range(c.length):
                    last = c.idcs[-1]
                    if isinstance(last, L.Fixed):
                        off = array_offset(tuple(c.idcs[:-1]) + (L.Fixed(last.i + i),), c.node.dims)
                    else:
                        off = array_offset(c.idcs, c.node.dims) + f" + {i}"
                    logs.append(self.log_statement(
                        f"{c.node.ident}[%u]{{={st}}} = vec_result.v[{i}] = {st}\n",
                        [off, self.styled_log_arg(f"{c.node.ident}[{off}]"), self.styled_log_arg(f"vec_result.v[{i}]")]))
                logs.append("fflush(log_file);")
                return self._with_defs(defs, lines[:1] + logs + lines[1:], ind, always_block=True)
            if not defs:
                # c_syntax.ml:640: no enclosing block in this case
                return [ind + ln for ln in lines]
            return self._with_defs(defs, lines, ind)
        if isinstance(c, L.SetLocal):
            defs, val = self.scalar(c.scope.node.prec, c.value, ind + "  ")
            if self.debug_log and log_set_locals:        # c_syntax.ml:649-684
                st = self.float_log_style
                name = self.scope_name(c.scope)
                dbg, args = self.debug_float(c.scope.node.prec, c.value)
                lines = [f"{C_TYP[c.scope.node.prec]} new_set_local_v = {val};",
                         self.log_statement(f"# local {name} := {val}\n", []),
                         self.log_statement(f"{name}{{={st}}} = {st} = {dbg}\n",
                                            [self.styled_log_arg(name), self.styled_log_arg("new_set_local_v")]
                                            + self._log_args(args)),
                         "fflush(log_file);",
                         f"{name} = new_set_local_v;"]
                return self._with_defs(defs, lines, ind, always_block=True)
            return self._with_defs(defs, [f"{self.scope_name(c.scope)} = {val};"], ind)
        if isinstance(c, L.DeclareLocal):
            prec = c.scope.node.prec
            init = self.init_zero(prec) if c.needs_init else ""
            return [f"{ind}{C_TYP[prec]} {self.scope_name(c.scope)}{init};"]
        raise TypeError(c)

    def _with_defs(self, defs, lines: List[str], ind: str, always_block: bool = False) -> List[str]:
        if not defs and always_block:
            return [ind + "{"] + [ind + "  " + ln for ln in lines] + [ind + "}"]
        if not defs:
            return [ind + ln for ln in lines]
        # c_syntax.ml:406-409: dedup by scope id, sorted by scope id
        uniq: Dict[int, List[str]] = {}
        for sid, d in defs:
            uniq.setdefault(sid, d)
        out = [ind + "{"]
        for sid in sorted(uniq):
            out.extend(uniq[sid])
        out.extend(ind + "  " + ln for ln in lines)
        out.append(ind + "}")
        return out

    def scalar(self, prec: str, s: L.Scalar, ind: str):
        """Returns (local definitions [(scope_id, lines)], expression)."""
        if isinstance(s, L.LocalScope):
            sp = s.scope.node.prec
            init = self.init_zero(sp) if reads_scope_before_set(s.scope, s.body) else ""
            lines = [f"{ind}{C_TYP[sp]} {self.scope_name(s.scope)}{init};"]
            lines += self.stmts(s.body, ind, True, log_set_locals=False)   # c_syntax.ml:725
            p, q = convert_precision(sp, prec)
            return [(s.scope.scope_id, lines)], f"{p}{self.scope_name(s.scope)}{q}"
        if isinstance(s, L.GetLocal):
            p, q = convert_precision(s.scope.node.prec, prec)
            return [], f"{p}{self.scope_name(s.scope)}{q}"
        if isinstance(s, L.GetMerge):
            p, q = convert_precision(s.node.prec, prec)
            return [], f"{p}merge_buffer[{array_offset(s.idcs, s.node.dims)}]{q}"
        if isinstance(s, L.Get):
            p, q = convert_precision(s.node.prec, prec)
            return [], f"{p}{s.node.ident}[{array_offset(s.idcs, s.node.dims)}]{q}"
        if isinstance(s, L.GetDynamic):
            p, q = convert_precision(s.node.prec, prec)
            ddefs, dexpr = self.scalar(s.dyn_prec, s.dyn_value, ind)
            dyn = f"(({C_TYP[index_prec()]})({dexpr}))"
            dims = s.node.dims
            parts = [dyn if i == s.dyn_axis else L.axis_index_str(ix)
                     for i, ix in enumerate(s.idcs)]
            doc = parts[0] if parts else "0"
            for i in range(1, len(parts)):
                doc = f"({doc}) * {dims[i]} + {parts[i]}"
            return ddefs, f"{p}{s.node.ident}[{doc}]{q}"
        if isinstance(s, L.Const):
            p, q = convert_precision("double", prec)
            cs = const_str(s.value)
            if p == "" and s.value < 0.0 and s.value != float("-inf"):
                return [], f"({cs}){q}"
            return [], f"{p}{cs}{q}"
        if isinstance(s, L.ConstBits):
            p, q = convert_precision("int64", prec)
            return [], f"{p}{int(s.value)}LL{q}"
        if isinstance(s, L.EmbedIndex):
            p, q = convert_precision(index_prec(), prec)
            return [], f"{p}{L.axis_index_str(s.idx)}{q}"
        if isinstance(s, L.Binop) and s.op == "arg1":
            return self.scalar(prec, s.a, ind)
        if isinstance(s, L.Binop) and s.op == "arg2":
            return self.scalar(prec, s.b, ind)
        if isinstance(s, L.Ternop):
            if s.op == "where":  # heterogeneous: the condition keeps its own precision
                d1, e1 = self.scalar(s.a_prec, s.a, ind)
            else:
                d1, e1 = self.scalar(prec, s.a, ind)
            d2, e2 = self.scalar(prec, s.b, ind)
            d3, e3 = self.scalar(prec, s.c, ind)
            return d1 + d2 + d3, cc_ternop(prec, s.op, e1, e2, e3)
        if isinstance(s, L.Binop):
            d1, e1 = self.scalar(prec, s.a, ind)
            d2, e2 = self.scalar(prec, s.b, ind)
            return d1 + d2, cc_binop(prec, s.op, e1, e2)
        if isinstance(s, L.Unop):
            arg_prec = s.arg_prec if s.op == "uint4x32_to_prec_uniform1" else prec
            d, e = self.scalar(arg_prec, s.arg, ind)
            return d, cc_unop(prec, s.op, e)
        raise TypeError(s)


def kernel_params(r: L.Routine, debug_log: bool = False) -> List[Tuple[str, object]]:
    """Parameter declarations sorted by declaration string (c_syntax.ml:1080-1084).

    Returns [(decl, source)] with source a Node (pointer), a StaticSymbol (int), the
    string "merge" or, with logging, "log" (the log file's name, c_syntax.ml:1067-1073)."""
    params: List[Tuple[str, object]] = []
    if debug_log:
        params.append(("const char* log_file_name", "log"))
    if r.merge_node is not None:
        params.append((f"const {C_TYP[r.merge_node.prec]} *merge_buffer", "merge"))
    for s in r.static_indices:
        params.append((f"const {C_TYP[index_prec()]} {L.sym_ident(s.sym)}", s))
    for n in r.nodes():
        if n.mode == "ctx":
            params.append((f"{C_TYP[n.prec]} *{n.ident}", n))
    params.sort(key=lambda p: p[0].encode())
    return params


def emit_proc(r: L.Routine, debug_log: bool = False, full_printf: bool = True) -> str:
    """The routine's C function (without builtins), c_syntax.ml:1021-1210.  ``debug_log``: with the
    statements that log every computed value to the file named by the extra first parameter."""
    em = _Emitter(r, debug_log, full_printf)
    params = kernel_params(r, debug_log)
    out = [f" void {r.name}("]
    out.append(",\n".join("    " + d for d, _ in params) + ") {")
    if debug_log:
        # c_syntax.ml:1098-1150: open the file, then the initial state of every parameter
        out += ["  FILE* log_file = NULL;", "  if (log_file_name) {", '    log_file = fopen(log_file_name, "w");', "  }",
                "  /* Debug initial parameter state. */"]
        for decl, src in params:
            if src == "log":
                continue
            if src == "merge":
                out.append("  " + em.log_statement(f"{decl} &[{r.merge_node.num_elems}] = %p\n", ["(void*)merge_buffer"]))
            elif isinstance(src, L.Node):
                out.append("  " + em.log_statement(f"{decl} &[{src.num_elems}] = %p\n", [f"(void*){src.ident}"]))
            else:
                out.append("  " + em.log_statement(f"{decl} = %d\n", [L.sym_ident(src.sym)]))
    else:
        out.append("")
    out.append("  /* Local declarations and initialization. */")
    for n in r.nodes():
        if n.mode == "local":
            init = " = {0}" if n.zero_initialized_by_code else ""
            out.append(f"  {C_TYP[n.prec]} {n.ident}[{n.num_elems}]{init};")
    out.append("")
    out.append("  /* Main logic. */")
    out.extend(em.stmts(r.body, "  ", False))
    if debug_log:
        out.append("  if (log_file) { fclose(log_file); log_file = NULL; }")   # c_syntax.ml:1200-1206
    out.append("}")
    return "\n".join(out)


_BUILTINS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "builtins_cc.h")


def emit_translation_unit(routines: Sequence[L.Routine], debug_log: bool = False, full_printf: bool = True) -> str:
    """Builtins + all procedures, as ``Cc_backend.compile_batch`` lays them out
    (cc_backend.ml:345-376); the whole builtins header is prepended instead of the
    reference's per-key filtering (c_syntax.ml:330-362), which only removes dead code."""
    with open(_BUILTINS) as f:
        text = f.read()
    return text + "\n" + "\n".join(emit_proc(r, debug_log, full_printf) for r in routines) + "\n"
