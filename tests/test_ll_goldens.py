"""The IR text form (`Low_level.to_doc`, arrayjit/lib/low_level.ml:2544-2648) printed by
ocannl_amd/llir.py:to_ll, token-equal to the `.ll` files the reference's tests hold
(test/einsum/*.ll.expected, test/operations/*-unoptimized.ll.expected) -- and the same routines run
through the CPU checker (and, on a GPU, through the HIP library) against their closed forms."""
import os
import re

import numpy as np
import pytest

from conftest import GOLDEN
from ocannl_amd import llir as L
from parity import OracleRun


def _tokens(text):
    return re.sub(r"\s+", "", text)


def _golden(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return f.read()


def _for(sym, to, body):
    return L.For(sym, 0, to, body)


def inline_permuted_view():
    """test/einsum/inline_permuted_view.ml: c = a * b with a 3x5 and b 5x4 ranges; the product is
    inlined into the permuted copy as a Local_scope reduction."""
    a = L.Node(1, "r3x5_a", "single", (3, 5)); b = L.Node(2, "r5x4_b", "single", (5, 4))
    n2 = L.Node(3, "n2", "single", (3, 4), mode="virtual"); c = L.Node(4, "c", "single", (4, 3))
    sc = L.Scope(n2, 1)
    it = L.It
    body = [
        L.Comment("c fwd"),
        _for(10, 2, [_for(11, 4, [L.Set(a, (it(10), it(11)), L.EmbedIndex(L.Affine(((5, 10), (1, 11)), 0)))])]),
        _for(12, 4, [_for(13, 3, [L.Set(b, (it(12), it(13)), L.EmbedIndex(L.Affine(((4, 12), (1, 13)), 0)))])]),
        _for(17, 3, [_for(18, 2, [L.Set(c, (it(17), it(18)), L.LocalScope(sc, [
            L.SetLocal(sc, L.Const(0.0)),
            _for(19, 4, [L.SetLocal(sc, L.Ternop("fma", L.Get(a, (it(18), it(19))), L.Get(b, (it(19), it(17))), L.GetLocal(sc)))]),
        ]))])]),
        L.Comment("end"),
    ]
    want = (np.arange(15, dtype=np.float32).reshape(3, 5) @ np.arange(20, dtype=np.float32).reshape(5, 4)).T
    return L.Routine("c_fwd", body), {"c": c}, {"c": want}


def cse_routine():
    """test/einsum/test_cse.ml: d = c * c with c = a * b inlined ONCE (common subexpression): the
    scope is defined at its first use and read by name at the second."""
    a = L.Node(1, "r3x4_a", "single", (3, 4)); b = L.Node(2, "r4_b", "single", (4,))
    cn = L.Node(3, "c", "single", (3,), mode="virtual"); d = L.Node(4, "cse_d", "single", (3,))
    sc = L.Scope(cn, 1)
    it = L.It
    body = [
        L.Comment("cse_d fwd"),
        _for(7, 2, [_for(8, 3, [L.Set(a, (it(7), it(8)), L.EmbedIndex(L.Affine(((4, 7), (1, 8)), 0)))])]),
        _for(9, 3, [L.Set(b, (it(9),), L.EmbedIndex(it(9)))]),
        _for(12, 2, [L.Set(d, (it(12),), L.Binop("mul", L.GetLocal(sc), L.LocalScope(sc, [
            L.SetLocal(sc, L.Const(0.0)),
            _for(13, 3, [L.SetLocal(sc, L.Ternop("fma", L.Get(a, (it(12), it(13))), L.Get(b, (it(13),)), L.GetLocal(sc)))]),
        ])))]),
        L.Comment("end"),
    ]
    cv = np.arange(12, dtype=np.float32).reshape(3, 4) @ np.arange(4, dtype=np.float32)
    return L.Routine("cse_d_fwd", body), {"cse_d": d}, {"cse_d": cv * cv}


def n3_fwd():
    """test/operations/threefry4x32_demo.ml before optimisation: seed 42, counters 0..4, the light
    threefry, then eight half-precision uniforms per counter."""
    seed = L.Node(1, "random_seed", "uint4x32", (5,)); n1 = L.Node(2, "n1", "uint4x32", (5,))
    tf = L.Node(3, "threefry4x32_light", "uint4x32", (5,)); n3 = L.Node(4, "n3", "half", (40,))
    it = L.It
    body = [
        L.Comment("n3 fwd"),
        _for(5, 4, [L.Set(seed, (it(5),), L.ConstBits(42))]),
        _for(6, 4, [L.Set(n1, (it(6),), L.EmbedIndex(it(6)))]),
        _for(7, 4, [L.Set(tf, (it(7),), L.Binop("threefry4x32_light", L.Get(seed, (it(7),)), L.Get(n1, (it(7),))))]),
        _for(8, 4, [L.SetFromVec(n3, (L.Affine(((8, 8),), 0),), 8, "uint4x32_to_prec_uniform", L.Get(tf, (it(8),)))]),
        L.Comment("end"),
    ]
    return L.Routine("n3_fwd", body), {"n3": n3}, None


def top_down_prec():
    a = L.Node(1, "a", "half", (1,)); b = L.Node(2, "b", "half", (1,)); n6 = L.Node(6, "n6", "half", (1,))
    c = L.Node(3, "c", "bfloat16", (1,)); d = L.Node(4, "d", "bfloat16", (1,))
    z = (L.Fixed(0),)
    body = [L.Comment("d fwd"), L.Set(n6, z, L.Binop("add", L.Get(a, z), L.Get(b, z))),
            L.Set(d, z, L.Binop("mul", L.Get(n6, z), L.Get(c, z))), L.Comment("end")]
    return L.Routine("d_fwd", body)


def where_precision():
    a = L.Node(1, "a_then_val", "half", ()); w = L.Node(2, "where", "single", ())
    cnd = L.Node(3, "cond_condition", "byte", ()); b = L.Node(4, "b_else_val", "bfloat16", ())
    body = [L.Comment("where fwd"), L.Set(w, (), L.Ternop("where", L.Get(cnd, ()), L.Get(a, ()), L.Get(b, ()))),
            L.Comment("end")]
    return L.Routine("where_fwd", body)


def zero_out_local_decl():
    n0 = L.Node(1, "n0", "single", (4,)); sparse = L.Node(2, "sparse", "single", (4, 3))
    n2 = L.Node(3, "n2", "single", (4,)); n3 = L.Node(4, "n3", "single", (4,)); out = L.Node(5, "out", "single", (4,))
    it = L.It
    body = [
        L.Comment("out fwd"),
        _for(6, 3, [L.Set(n0, (it(6),), L.EmbedIndex(it(6)))]),
        L.ZeroOut(sparse),
        _for(7, 3, [L.Set(sparse, (it(7), L.Fixed(0)), L.Get(n0, (it(7),)))]),
        _for(8, 3, [L.Set(n2, (it(8),), L.Get(sparse, (it(8), L.Fixed(2))))]),
        _for(9, 3, [L.Set(n3, (it(9),), L.Get(sparse, (it(9), L.Fixed(2))))]),
        _for(10, 3, [L.Set(out, (it(10),), L.Binop("mul", L.Get(n3, (it(10),)), L.Get(n2, (it(10),))))]),
        L.Comment("end"),
    ]
    return L.Routine("out_fwd", body), {"out": out, "sparse": sparse}, \
        {"out": np.zeros(4, np.float32), "sparse": np.array([[i, 0, 0] for i in range(4)], np.float32)}


def test_ll_text_inline_permuted_view():
    assert _tokens(L.to_ll(inline_permuted_view()[0])) == _tokens(_golden("inline_permuted_view-c_fwd.ll.expected"))


def test_ll_text_cse():
    assert _tokens(L.to_ll(cse_routine()[0])) == _tokens(_golden("test_cse-cse_d_fwd.ll.expected"))


def test_ll_text_n3_with_prec():
    assert _tokens(L.to_ll(n3_fwd()[0], with_prec=True)) == _tokens(_golden("n3_fwd_with_prec-unoptimized.ll.expected"))


def test_ll_text_top_down_prec():
    assert _tokens(L.to_ll(top_down_prec(), with_prec=True)) == _tokens(_golden("top_down_prec-unoptimized.ll.expected"))


def test_ll_text_where_precision():
    assert _tokens(L.to_ll(where_precision(), with_prec=True)) == _tokens(_golden("test_where_precision-unoptimized.ll.expected"))


def test_ll_text_zero_out_local_decl():
    assert _tokens(L.to_ll(zero_out_local_decl()[0], with_prec=True)) == _tokens(_golden("zero_out_local_decl-unoptimized.ll.expected"))


N3_EXPECTED = [  # test/operations/threefry4x32_demo.ml:31-73 (tolerance 0.01)
    0.443, 0.464, 0.673, 0.732, 0.333, 0.561, 0.852, 0.507, 0.378, 0.502, 0.656, 0.966, 0.356, 0.803, 0.334, 0.995]


def _check(run_get, which):
    r, nodes, want = which()
    get = run_get(r, nodes)
    if want is None:   # n3: the reference's own expected uniforms
        got = get("n3").astype(np.float64)
        assert np.max(np.abs(got[:16] - np.array(N3_EXPECTED))) < 0.01 and np.all((got >= 0) & (got < 1))
        return got
    for k, w in want.items():
        assert np.array_equal(get(k), w), k
    return None


def _oracle(r, nodes):
    o = OracleRun(r, {})
    o.step()
    return lambda k: o.get(nodes[k])


@pytest.mark.parametrize("which", [inline_permuted_view, cse_routine, n3_fwd, zero_out_local_decl])
def test_golden_routines_on_the_checker(which):
    _check(_oracle, which)


@pytest.mark.gpu
@pytest.mark.parametrize("which", [inline_permuted_view, cse_routine, n3_fwd, zero_out_local_decl])
def test_golden_routines_on_the_gpu(which):
    from ocannl_amd.backend import HipRun

    def hip(r, nodes):
        h = HipRun(r, {})
        h.step()
        vals = {k: h.get(n) for k, n in nodes.items()}
        h.close()
        return lambda k: vals[k]

    got = _check(hip, which)
    if got is not None:   # PRNG output: bit-identical with the checker
        want = _check(_oracle, which)
        assert np.array_equal(got, want)
