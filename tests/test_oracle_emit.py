"""Pins oracle/cc_emit.py: (1) text equality, modulo white space, with generated C the
reference's tests hold; (2) bit equality of the compiled result with the reference's own
generated C compiled unchanged (oracle/_ref, built from the reference tree when present)."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, ROOT
from ocannl_amd import llir as L
from oracle import cc_emit, cc_oracle


def _norm(text: str) -> str:
    lines = [ln.strip() for ln in text.strip().splitlines()]
    out, locs, in_locals = [], [], False
    for ln in lines:
        if ln.startswith("/* Local declarations"):
            in_locals = True
            out.append(ln)
        elif ln.startswith("/* Main logic."):
            in_locals = False
            out.extend(sorted(locs))
            out.append(ln)
        elif in_locals:
            locs.append(ln)
        else:
            out.append(ln)
    return re.sub(r"\s+", "", "".join(out))


def _golden(name: str) -> str:
    with open(os.path.join(GOLDEN, name)) as f:
        return f.read()


def _top_down_prec():
    # test/operations/top_down_prec.ml: d = (a + b) *. c with b half, d bfloat16; the sum
    # n6 is virtual and inlined (top_down_prec-unoptimized.ll.expected shows it before inlining)
    a = L.Node(1, "a", "half", (1,))
    b = L.Node(2, "b", "half", (1,))
    c = L.Node(3, "c", "bfloat16", (1,))
    d = L.Node(4, "d", "bfloat16", (1,))
    z = (L.Fixed(0),)
    body = [L.Comment("d fwd"),
            L.Set(d, z, L.Binop("mul", L.Binop("add", L.Get(a, z), L.Get(b, z)), L.Get(c, z))),
            L.Comment("end")]
    return L.Routine("d_fwd", body), (a, b, c, d)


def _where_precision():
    a = L.Node(1, "a_then_val", "half", (1,))
    w = L.Node(2, "where", "single", (1,))
    cnd = L.Node(3, "cond_condition", "byte", (1,))
    b = L.Node(4, "b_else_val", "bfloat16", (1,))
    z = (L.Fixed(0),)
    body = [L.Comment("where fwd"),
            L.Set(w, z, L.Ternop("where", L.Get(cnd, z), L.Get(a, z), L.Get(b, z))),
            L.Comment("end")]
    return L.Routine("where_fwd", body), (a, w, cnd, b)


def _zero_out_local_decl():
    L.reset_symbols(6)
    sparse = L.Node(1, "sparse", "single", (4, 3), mode="local", zero_initialized_by_code=True)
    out = L.Node(2, "out", "single", (4,))
    i7 = L.fresh_symbol()
    L.reset_symbols(9)
    i10 = L.fresh_symbol()
    body = [L.Comment("out fwd"),
            L.ZeroOut(sparse),
            L.For(i7, 0, 3, [L.Set(sparse, (L.It(i7), L.Fixed(0)), L.EmbedIndex(L.It(i7)))]),
            L.For(i10, 0, 3, [L.Set(out, (L.It(i10),), L.Binop(
                "mul", L.Get(sparse, (L.It(i10), L.Fixed(2))),
                L.Get(sparse, (L.It(i10), L.Fixed(2)))))]),
            L.Comment("end")]
    return L.Routine("out_fwd", body), (sparse, out)


def test_text_top_down_prec():
    r, _ = _top_down_prec()
    assert _norm(cc_emit.emit_proc(r)) == _norm(_golden("top_down_prec.proc.c.expected"))


def test_text_where_precision():
    r, _ = _where_precision()
    assert _norm(cc_emit.emit_proc(r)) == _norm(_golden("test_where_precision.proc.c.expected"))


def test_text_zero_out_local_decl():
    r, _ = _zero_out_local_decl()
    assert _norm(cc_emit.emit_proc(r)) == _norm(_golden("zero_out_local_decl.proc.c.expected"))


def test_text_zero_out_codegen():
    # arrayjit/test/test_zero_out_codegen.ml: Zero_out; Set; Zero_out on one local, and a
    # first-touch Zero_out inside a loop on another: only the very first is elided.
    L.reset_symbols(0)
    a = L.Node(1, "acc_a", "single", (2,), mode="local", zero_initialized_by_code=True)
    b = L.Node(2, "acc_b", "single", (2,), mode="local", zero_initialized_by_code=True)
    i1 = L.fresh_symbol()
    body = [L.ZeroOut(a), L.Set(a, (L.Fixed(0),), L.Const(7.0)), L.ZeroOut(a),
            L.For(i1, 0, 3, [L.ZeroOut(b)])]
    r = L.Routine("zero_out_codegen", body)
    assert _norm(cc_emit.emit_proc(r)) == _norm(_golden("test_zero_out_codegen.proc.c.expected"))


def _log_stmt_format():
    # test/operations/test_log_stmt_format.ml: c = a + b on one-element tensors, compiled with
    # debug_log_from_routines (and `%de-3` values: the prefer_backend_uniformity log style)
    a = L.Node(1, "a", "single", (1,)); b = L.Node(2, "b", "single", (1,)); c = L.Node(3, "c", "single", (1,))
    z = (L.Fixed(0),)
    body = [L.Comment("c fwd"), L.Set(c, z, L.Binop("add", L.Get(a, z), L.Get(b, z))), L.Comment("end")]
    return L.Routine("c_fwd", body), (a, b, c)


def test_text_log_stmt_format():
    # the log statements of c_syntax.ml:493-535 (Set), :539-546 (comments), :1112-1150 (parameter
    # header), :1200-1206 (closing the file), as the reference's own golden holds them
    r, _ = _log_stmt_format()
    assert _norm(cc_emit.emit_proc(r, debug_log=True, full_printf=False)) == _norm(_golden("test_log_stmt_format.proc.c.expected"))
    # without the option nothing of it is emitted
    assert "fprintf" not in cc_emit.emit_proc(r)


def test_logging_checker_writes_the_lines_the_format_promises(tmp_path):
    # the compiled checker, run with a log file: header lines, comments, `# statement`, value line
    r, (a, b, c) = _log_stmt_format()
    lib = cc_oracle.CompiledOracle([r], debug_log=True, full_printf=False)
    bufs = {a.id: np.array([1.0], np.float32), b.id: np.array([1.0], np.float32), c.id: np.zeros(1, np.float32)}
    log = tmp_path / "c_fwd.log"
    lib.run("c_fwd", bufs, log_file=str(log))
    assert bufs[c.id][0] == 2.0
    lines = log.read_text().splitlines()
    assert [re.sub(r"= 0x[0-9a-f]+|= \(nil\)", "= 0xNNNN", ln) for ln in lines[:3]] == [
        "float *a &[1] = 0xNNNN", "float *b &[1] = 0xNNNN", "float *c &[1] = 0xNNNN"]
    assert lines[3:] == ["COMMENT: c fwd", "# c[0] := (a[0] + b[0]);",
                         "c[0]{=0e-3} = 2000e-3 = (a[0]{=1000e-3} + b[0]{=1000e-3})", "COMMENT: end"]
    # ... and with full printf support, `%g` values (cc_backend.ml:164-165)
    lib = cc_oracle.CompiledOracle([r], debug_log=True)
    lib.run("c_fwd", bufs, log_file=str(log))
    assert log.read_text().splitlines()[5] == "c[0]{=2} = 2 = (a[0]{=1} + b[0]{=1})"


def _sections(text):
    parts = re.split(r"^=== .* ===\n", text, flags=re.M)
    return [p for p in parts[1:]]


def test_text_local_scope_init():
    # arrayjit/test/test_local_scope_init.ml: a Local_scope / Declare_local gets "= (float)(0)"
    # exactly when the scope is read before it is definitely written.
    secs = _sections(_golden("test_local_scope_init.expected"))
    em = cc_emit._Emitter(L.Routine("x", []))
    z = (L.Fixed(0),)

    def node(i, name, dims=(1,)):
        return L.Node(i, name, "single", dims)

    # 1: write-before-read
    src, out = node(1, "src"), node(2, "out")
    sc = L.Scope(src, 10)
    st = L.Set(out, z, L.LocalScope(sc, [L.SetLocal(sc, L.Get(src, z))]))
    assert _norm("\n".join(em.stmt(st, "", False))) == _norm(secs[0])
    # 2: read-before-write accumulator
    src2, out2 = node(3, "src2", (4,)), node(4, "out2")
    sc = L.Scope(src2, 20)
    st = L.Set(out2, z, L.LocalScope(sc, [L.For(2, 0, 3, [L.SetLocal(sc, L.Binop(
        "add", L.GetLocal(sc), L.Get(src2, (L.It(2),))))])]))
    assert _norm("\n".join(em.stmt(st, "", False))) == _norm(secs[1])
    # 3: empty body -> needs init
    srcn, outn = node(5, "src_noop"), node(6, "out_noop")
    sc = L.Scope(srcn, 60)
    st = L.Set(outn, z, L.LocalScope(sc, []))
    assert _norm("\n".join(em.stmt(st, "", False))) == _norm(secs[2])
    # 4: a write inside a zero-trip loop does not count as a definite write
    sel, outel = node(7, "src_el"), node(8, "out_el")
    sc = L.Scope(sel, 50)
    st = L.Set(outel, z, L.LocalScope(sc, [
        L.For(3, 5, 0, [L.SetLocal(sc, L.Const(0.0))]),
        L.SetLocal(sc, L.Binop("add", L.GetLocal(sc), L.Const(1.0)))]))
    assert _norm("\n".join(em.stmt(st, "", False))) == _norm(secs[3])
    # 5/6: hoisted Declare_local
    s3, o3, o4 = node(9, "src3"), node(10, "out3"), node(11, "out4")
    sc = L.Scope(s3, 30)
    sts = [L.DeclareLocal(sc, False), L.SetLocal(sc, L.Get(s3, z)),
           L.Set(o3, z, L.GetLocal(sc)), L.Set(o4, z, L.GetLocal(sc))]
    assert _norm("\n".join(em.stmts(sts, "", False))) == _norm(secs[4])
    s4, o5, o6 = node(12, "src4", (4,)), node(13, "out5"), node(14, "out6")
    sc = L.Scope(s4, 40)
    sts = [L.DeclareLocal(sc, True),
           L.For(4, 0, 3, [L.SetLocal(sc, L.Binop("add", L.GetLocal(sc),
                                                   L.Get(s4, (L.It(4),))))]),
           L.Set(o5, z, L.GetLocal(sc)), L.Set(o6, z, L.GetLocal(sc))]
    assert _norm("\n".join(em.stmts(sts, "", False))) == _norm(secs[5])


# ---- against the reference's own generated C, compiled unchanged -------------------------

@pytest.fixture(scope="module")
def ref_dir(reference_root):
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "ref"], check=True,
                   capture_output=True)
    d = os.path.join(ROOT, "oracle", "_ref")
    if not os.path.exists(os.path.join(d, "top_down_prec.so")):
        pytest.skip("oracle/_ref not built")
    return d


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def test_ref_top_down_prec_bits(ref_dir):
    r, (a, b, c, d) = _top_down_prec()
    ref = ctypes.CDLL(os.path.join(ref_dir, "top_down_prec.so"))
    mine = cc_oracle.CompiledOracle([r])
    rng = np.random.default_rng(3)
    for _ in range(500):
        av = rng.standard_normal(1).astype(np.float16) * np.float16(rng.choice([1e-3, 1, 100]))
        bv = rng.standard_normal(1).astype(np.float16)
        cv = (rng.standard_normal(1).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        d1 = np.zeros(1, np.uint16)
        d2 = np.zeros(1, np.uint16)
        # x86 gcc 11 has no _Float16: HALF_T is uint16_t in both builds
        ref.d_fwd(_ptr(av.view(np.uint16)), _ptr(bv.view(np.uint16)), _ptr(cv), _ptr(d1))
        mine.run("d_fwd", {1: av.view(np.uint16), 2: bv.view(np.uint16), 3: cv, 4: d2})
        assert d1[0] == d2[0]


def test_ref_where_precision_bits(ref_dir):
    r, (a, w, cnd, b) = _where_precision()
    ref = ctypes.CDLL(os.path.join(ref_dir, "test_where_precision.so"))
    mine = cc_oracle.CompiledOracle([r])
    rng = np.random.default_rng(4)
    for k in range(100):
        av = rng.standard_normal(1).astype(np.float16).view(np.uint16)
        bv = (rng.standard_normal(1).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        cv = np.array([k % 3], np.uint8)
        w1, w2 = np.zeros(1, np.float32), np.zeros(1, np.float32)
        # parameter order = sorted declarations: a_then_val, where, cond_condition, b_else_val
        ref.where_fwd(_ptr(av), _ptr(w1), _ptr(cv), _ptr(bv))
        mine.run("where_fwd", {1: av, 2: w2, 3: cv, 4: bv})
        assert w1.view(np.uint32)[0] == w2.view(np.uint32)[0]


def test_ref_zero_out_local_decl_bits(ref_dir):
    r, (sparse, out) = _zero_out_local_decl()
    ref = ctypes.CDLL(os.path.join(ref_dir, "zero_out_local_decl.so"))
    mine = cc_oracle.CompiledOracle([r])
    o1, o2 = np.full(4, 7, np.float32), np.full(4, 9, np.float32)
    ref.out_fwd(_ptr(o1))
    mine.run("out_fwd", {2: o2})
    assert (o1 == o2).all() and (o1 == 0).all()


def test_param_order_is_by_declaration_string():
    r, _ = _where_precision()
    decls = [d for d, _ in cc_emit.kernel_params(r)]
    assert decls == ["HALF_T *a_then_val", "float *where", "unsigned char *cond_condition",
                     "unsigned short *b_else_val"]


def test_large_models_widens_loop_indices_and_integer_arguments():
    # c_syntax.ml:111-112: `loop_index_type` and `arg_int_prefix` turn uint64_t under large_models;
    # the results of a routine do not depend on the setting
    import numpy as np
    from oracle import cc_oracle
    L.reset_symbols(0)
    a = L.Node(1, "a", "single", (5, 7)); b = L.Node(2, "b", "single", (7,))
    st = L.StaticSymbol(L.fresh_symbol(), 5)
    j = L.fresh_symbol()
    r = L.Routine("row_of", [L.For(j, 0, 6, [L.Set(b, (L.It(j),), L.Binop(
        "add", L.Get(a, (L.It(st.sym), L.It(j))), L.EmbedIndex(L.It(j))))])], static_indices=[st])
    av = np.arange(35, dtype=np.float32).reshape(5, 7)
    outs = []
    for large in (False, True):
        cc_emit.LARGE_MODELS = large
        try:
            lib = cc_oracle.CompiledOracle([r])
            typ = "uint64_t" if large else "uint32_t"
            assert f"for ({typ} " in lib.source and f"const {typ} {L.sym_ident(st.sym)}" in lib.source
            bufs = {a.id: av.copy(), b.id: np.zeros(7, np.float32)}
            lib.run(r.name, bufs, {st.sym: 3})
            outs.append(bufs[b.id])
        finally:
            cc_emit.LARGE_MODELS = False
    assert np.array_equal(outs[0], av[3] + np.arange(7)) and np.array_equal(outs[0], outs[1])
