"""Whole-routine known answers that the reference's own tests hold, run through the harness
(ocannl_amd/frontend.py) and then BOTH the CPU checker and -- on a GPU -- the HIP library:
  * micrograd: g, a.grad, b.grad of test/operations/micrograd_demo_logging.ml as logged in
    micrograd_demo_logging-sync_cc-0-0.log.expected (forward code + reverse-mode derivatives);
  * the einsum tables of test/einsum/einsum_trivia.ml:378-481 (pointwise, batched matrix product,
    outer batch product, sums over batch axes; operand layout batch @ output @ input);
  * test/operations/hello_world_op.ml:479-548 (matrix-vector product plus bias);
  * test/operations/zero2hero_1of7_exec.ml: the polynomial 3x^2 - 4x + 5 with every node's value and
    gradient at x = 5 and its two sweeps (:22-101, the second through a static index), the
    four-parameter product-sum with an SGD step between two gradient passes (:103-136), the
    two-input neuron (:169-178), as zero2hero_1of7_exec.expected prints them;
  * test/operations/test_where_simple.ml (the `where` ternary and its two gradient statements,
    tensor/operation.ml:457-467), test_fma_logic.ml (pointwise and compose-accumulate `fma`),
    rope_test.ml Tests 1 and 2 (de-interleave / interleave through `2*i` and `2*i + 1` affine indices,
    tensor/operation.ml:342-372, and the rotation of lib/nn_blocks.ml:195-207), written in the loop IR
    directly;
  * test/einsum/test_padding_reset.ml (one padded input read by a max over 3 x 3 windows, whose margin has
    to hold -infinity, then by a sum over 3 x 3 windows, whose margin has to hold 0: the margin-only
    reset loops of low_level.ml:2705-2802 run between the two), test_max_pool2d.ml (stride 2, window 2
    over 0..15) and test_tropical_kernel.ml (max over the window of input + kernel);
  * test/einsum/test_accumulation_semantics.ml: a sum over the output axis, a diagonal (`i => ii`) and a
    fixed-index projection (`i => i0`) whose untouched cells hold the zeros of the Zero_out in front of
    them, a transpose.
The expected numbers are in tests/golden/kat.json exactly as the reference prints them."""
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN
from ocannl_amd import llir as L
from ocannl_amd.frontend import ConstT, Graph, make_routine
from parity import OracleRun


@pytest.fixture(scope="module")
def kat():
    with open(os.path.join(GOLDEN, "kat.json")) as f:
        return json.load(f)


def micrograd():
    """test/operations/micrograd_demo_logging.ml:42-51 (integer powers unrolled to products, as
    low_level.ml:1154-1163 does before code generation)."""
    L.reset_symbols(0)
    g = Graph("single", "single")
    one = ("x",)
    a = g.param("a", one, (1,)); b = g.param("b", one, (1,))
    c = g.add(a, b, one, "c0")
    d = g.add(g.mul(a, b, one), g.mul(b, g.mul(b, b, one), one), one, "d0")
    c = g.add(g.add(c, c, one), ConstT(1.0), one, "c1")
    c = g.add(g.add(g.add(c, ConstT(1.0), one), c, one), g.unary("neg", a), one, "c2")
    d = g.add(g.add(d, g.mul(d, ConstT(2.0), one), one), g.unary("relu", g.add(b, a, one)), one, "d1")
    d = g.add(g.add(d, g.mul(ConstT(3.0), d, one), one), g.unary("relu", g.sub(b, a, one)), one, "d2")
    e = g.sub(c, d, one, "e")
    f = g.mul(e, e, one, "f")
    gg = g.div(f, ConstT(2.0), one, "g0")
    gg = g.add(gg, g.div(ConstT(10.0), f, one), one, "g")
    body = g.grad_update(gg)
    a.grad.mode = b.grad.mode = "ctx"   # Train.set_materialized diff.grad
    r = make_routine(g, "micrograd_update", body, outputs=[gg.value, a.grad, b.grad])
    init = {a.value.id: np.array([-4.0], np.float32), b.value.id: np.array([2.0], np.float32)}
    return r, init, {"g": gg.value, "a_grad": a.grad, "b_grad": b.grad}


def einsum_trivia():
    """a: batch 2, output 4, input 3; b: batch 2, output 5, input 4; values 0, 1, 2, ... in
    row-major batch @ output @ input order (TDSL.range_of_shape)."""
    L.reset_symbols(0)
    g = Graph("single", "single")
    A = lambda ax: ax   # noqa: E731
    a = g.input("a", ("b", "h", "i"), (2, 4, 3))
    b = g.input("b", ("b", "o", "h"), (2, 5, 4))
    a2 = g.mul(a, a, ("b", "h", "i"), ident="a2")
    c = g.einsum(b, a, ("b", "o", "i"), ident="c")                 # b|h->o; b|i->h => b|i->o
    from ocannl_amd.frontend import rename
    a_outer = rename(a, {"b": "a"})                                 # a|i->h; b|h->o => ab|i->o
    d = g.einsum(a_outer, b, ("a", "b", "o", "i"), ident="d")
    e = g.einsum(a, b, ("o", "i"), ident="e")                       # b|i->h; b|h->o => i->o
    f = g.einsum(a_outer, b, ("o", "i"), ident="f")                 # a|i->h; b|h->o => i->o
    outs = {"a2": a2, "c": c, "d": d, "e": e, "f": f}
    body = []
    for t in outs.values():
        body += t.fwd
    r = make_routine(g, "einsum_trivia_fwd", body, outputs=[t.value for t in outs.values()])
    init = {a.value.id: np.arange(24, dtype=np.float32).reshape(2, 4, 3),
            b.value.id: np.arange(40, dtype=np.float32).reshape(2, 5, 4)}
    return r, init, {k: t.value for k, t in outs.items()}


def hello_world(n_out, n_in, hey_value, vec, bias):
    L.reset_symbols(0)
    g = Graph("single", "single")
    hey = g.param("hey", ("o", "i"), (n_out, n_in))
    x = g.input("x", ("i",), (n_in,)); bb = g.input("bias", ("o",), (n_out,))
    y = g.add(g.einsum(hey, x, ("o",), ident="hx"), bb, ("o",), "y")
    r = make_routine(g, "hello_world_fwd", g.forward(y), outputs=[y.value])
    init = {hey.value.id: np.full((n_out, n_in), hey_value, np.float32), x.value.id: np.asarray(vec, np.float32),
            bb.value.id: np.asarray(bias, np.float32)}
    return r, init, {"y": y.value}


def zero2hero_poly(sweep=None):
    """f = 3 x^2 - 4 x + 5 (zero2hero_1of7_exec.ml:26,62): every intermediate a tensor of its own, as
    `Train.every_non_literal_materialized` leaves them.  `sweep` (a list of values): x is element
    `step` of a vector -- `x_flat @| step_sym`, the slice by a static symbol of :66-72, whose backward
    statement adds x's gradient into that element of the vector's gradient."""
    L.reset_symbols(0)
    g = Graph("single", "single")
    one = ("o",)
    statics = []
    if sweep is None:
        x = g.param("x", one, (1,))
        init_x = {x.value.id: np.array([5.0], np.float32)}
        extra = {}
    else:
        from ocannl_amd.frontend import T
        flat = g.param("x_flat", ("s", "o"), (len(sweep), 1))
        step = L.StaticSymbol(L.fresh_symbol(), len(sweep))
        statics = [step]
        xv = g.node("x", (1,), mode="ctx"); xg = g.node("x_grad", (1,), mode="ctx")
        x = T(xv, one, xg, (flat,), label="x")
        x.fwd = [L.Set(xv, (L.Fixed(0),), L.Get(flat.value, (L.It(step.sym), L.Fixed(0))))]
        at = (L.It(step.sym), L.Fixed(0))
        x.bwd = lambda: [L.Set(flat.grad, at, L.Binop("add", L.Get(flat.grad, at), L.Get(xg, (L.Fixed(0),))))]
        init_x = {flat.value.id: np.asarray(sweep, np.float32).reshape(-1, 1)}
        extra = {"step": step}
    pw = g.mul(x, x, one, "pow")
    t3 = g.mul(ConstT(3.0), pw, one, "three_x2")
    t4 = g.mul(ConstT(4.0), x, one, "four_x")
    mi = g.sub(t3, t4, one, "minus")
    f = g.add(mi, ConstT(5.0), one, "f")
    body = g.grad_update(f)
    nodes = {"pow": pw.value, "three_x2": t3.value, "four_x": t4.value, "minus": mi.value, "f": f.value, "x": x.value,
             "grad_f": f.grad, "grad_minus": mi.grad, "grad_three_x2": t3.grad, "grad_four_x": t4.grad, "grad_pow": pw.grad,
             "grad_x": x.grad}
    for n in nodes.values():
        n.mode = "ctx"
    r = make_routine(g, "zero2hero_poly", body, statics=statics, outputs=list(nodes.values()))
    return r, init_x, nodes, extra


def zero2hero_simple_gradients():
    """l = (a * b + c) * f with a gradient routine and a separate SGD routine (learning rate 0.1,
    zero2hero_1of7_exec.ml:103-136)."""
    L.reset_symbols(0)
    g = Graph("single", "single")
    one = ("o",)
    a = g.param("a", one, (1,)); b = g.param("b", one, (1,)); c = g.param("c", one, (1,)); f = g.param("f", one, (1,))
    e = g.mul(a, b, one, "e")
    d = g.add(e, c, one, "d")
    l = g.mul(d, f, one, "l")
    grad_body = g.grad_update(l)
    lr = g.input("learning_rate", one, (1,))
    nodes = {"a": a.value, "b": b.value, "c": c.value, "f": f.value, "e": e.value, "d": d.value, "l": l.value,
             "grad_a": a.grad, "grad_b": b.grad, "grad_c": c.grad, "grad_f": f.grad, "grad_e": e.grad, "grad_d": d.grad,
             "grad_l": l.grad}
    for n in nodes.values():
        n.mode = "ctx"
    sgd_body = g.sgd_update([a, b, c, f], lr)
    grad = make_routine(g, "simple_grad", grad_body, outputs=list(nodes.values()))
    sgd = make_routine(g, "simple_sgd", sgd_body, outputs=[a.value, b.value, c.value, f.value])
    init = {a.value.id: np.array([2.0], np.float32), b.value.id: np.array([-3.0], np.float32),
            c.value.id: np.array([10.0], np.float32), f.value.id: np.array([-2.0], np.float32),
            lr.value.id: np.array([0.1], np.float32)}
    return grad, sgd, init, nodes


def zero2hero_neuron():
    """v = w . x + b with w = [-3, 1], x = [2, 0], b = 6.7 (zero2hero_1of7_exec.ml:169-178)."""
    L.reset_symbols(0)
    g = Graph("single", "single")
    w = g.param("w", ("o", "i"), (1, 2)); x = g.param("x", ("i",), (2,)); b = g.param("b", ("o",), (1,))
    m = g.einsum(w, x, ("o",), ident="mul")
    v = g.add(m, b, ("o",), "v")
    body = g.grad_update(v)
    nodes = {"v": v.value, "mul": m.value, "grad_w": w.grad, "grad_x": x.grad, "grad_b": b.grad}
    for n in nodes.values():
        n.mode = "ctx"
    r = make_routine(g, "neuron_2d", body, outputs=list(nodes.values()))
    init = {w.value.id: np.array([[-3.0, 1.0]], np.float32), x.value.id: np.array([2.0, 0.0], np.float32),
            b.value.id: np.array([6.7], np.float32)}
    return r, init, nodes


def where_simple(cond_value):
    """result =:+ where cond x y; x.grad =+ where cond g 0; y.grad =+ where cond 0 g
    (tensor/operation.ml:462-466) around Train.grad_update."""
    L.reset_symbols(0)
    mk = lambda i, name: L.Node(i, name, "single", (1,))
    cond, x, y, res, xg, yg, rg = (mk(i + 1, n) for i, n in enumerate(("cond", "x", "y", "result", "x_grad", "y_grad", "result_grad")))
    at = (L.Fixed(0),)
    G = lambda n: L.Get(n, at)
    body = [L.ZeroOut(res), L.Set(res, at, L.Binop("add", G(res), L.Ternop("where", G(cond), G(x), G(y)))),
            L.ZeroOut(xg), L.ZeroOut(yg), L.Set(rg, at, L.Const(1.0)),
            L.Set(xg, at, L.Binop("add", G(xg), L.Ternop("where", G(cond), G(rg), L.Const(0.0)))),
            L.Set(yg, at, L.Binop("add", G(yg), L.Ternop("where", G(cond), L.Const(0.0), G(rg))))]
    init = {1: np.array([cond_value], np.float32), 2: np.array([2.0], np.float32), 3: np.array([3.0], np.float32)}
    return L.Routine("where_simple", body), init, {"x": x, "y": y, "result": res, "x_grad": xg, "y_grad": yg}


def fma_logic():
    """out[i] = fma(a[i], x[i], b[i]) and out2 =:+ fma(p[o, k], q[k], r[o]) with p 1 x 1 (test_fma_logic.ml:36-57)."""
    L.reset_symbols(0)
    a, x, b, out = (L.Node(i + 1, n, "single", (4,)) for i, n in enumerate(("a", "x", "b", "out")))
    p = L.Node(5, "p", "single", (1, 1)); q = L.Node(6, "q", "single", (1,)); r = L.Node(7, "r", "single", (1,))
    out2 = L.Node(8, "out2", "single", (1,))
    i, o, kk = L.fresh_symbol(), L.fresh_symbol(), L.fresh_symbol()
    body = [L.For(i, 0, 3, [L.Set(out, (L.It(i),), L.Ternop("fma", L.Get(a, (L.It(i),)), L.Get(x, (L.It(i),)), L.Get(b, (L.It(i),))))]),
            L.ZeroOut(out2),
            L.For(o, 0, 0, [L.For(kk, 0, 0, [L.Set(out2, (L.It(o),), L.Binop("add", L.Get(out2, (L.It(o),)), L.Ternop(
                "fma", L.Get(p, (L.It(o), L.It(kk))), L.Get(q, (L.It(kk),)), L.Get(r, (L.It(o),)))))])])]
    f32 = lambda *v: np.array(v, np.float32)
    init = {1: f32(1, 2, 3, 4), 2: f32(10, 20, 30, 40), 3: f32(0.5, 0.5, 0.5, 0.5), 5: f32(3).reshape(1, 1), 6: f32(2), 7: f32(10)}
    return L.Routine("fma_logic", body), init, {"pointwise": out, "compose_accumulate": out2}


def rope():
    """rope_test.ml Test 1 (interleave (deinterleave_even x) (deinterleave_odd x) of 1..6) and Test 2
    (d_k 4, three positions, x[pos, i] = 4 pos + i + 1, frequencies 10000^(-2k/4)): every `=:+` is a
    Zero_out and an accumulation, the halves are addressed through affine indices."""
    L.reset_symbols(0)
    ids = iter(range(1, 40))
    N = lambda name, dims: L.Node(next(ids), name, "single", dims)
    body = []

    def split(src, lead, half):      # deinterleave_even / _odd of the last axis
        outs = []
        for off, name in ((0, "even"), (1, "odd")):
            t = N(f"{src.ident}_{name}", lead + (half,))
            syms = [L.fresh_symbol() for _ in lead] + [L.fresh_symbol()]
            lhs = tuple(L.It(s) for s in syms)
            rhs = tuple(L.It(s) for s in syms[:-1]) + (L.Affine(((2, syms[-1]),), off),)
            nest = [L.Set(t, lhs, L.Binop("add", L.Get(t, lhs), L.Get(src, rhs)))]
            for s, d in reversed(list(zip(syms, lead + (half,)))):
                nest = [L.For(s, 0, d - 1, nest)]
            body.extend([L.ZeroOut(t)] + nest)
            outs.append(t)
        return outs

    def join(even, odd, lead, half, name):
        t = N(name, lead + (2 * half,))
        body.append(L.ZeroOut(t))
        for off, src in ((0, even), (1, odd)):
            syms = [L.fresh_symbol() for _ in lead] + [L.fresh_symbol()]
            rhs = tuple(L.It(s) for s in syms)
            lhs = tuple(L.It(s) for s in syms[:-1]) + (L.Affine(((2, syms[-1]),), off),)
            nest = [L.Set(t, lhs, L.Binop("add", L.Get(t, lhs), L.Get(src, rhs)))]
            for s, d in reversed(list(zip(syms, lead + (half,)))):
                nest = [L.For(s, 0, d - 1, nest)]
            body.extend(nest)
        return t

    x6 = N("x_deint", (6,))
    e6, o6 = split(x6, (), 3)
    round_trip = join(e6, o6, (), 3, "roundtrip")
    seq, dk = 3, 4
    x = N("x", (seq, dk)); freqs = N("rope_freqs", (dk // 2,)); pos = N("pos_idx", (seq,))
    xe, xo = split(x, (seq,), dk // 2)
    cos_a, sin_a, oe, oo = (N(n, (seq, dk // 2)) for n in ("cos_a", "sin_a", "out_even", "out_odd"))
    p, kf = L.fresh_symbol(), L.fresh_symbol()
    at = (L.It(p), L.It(kf))
    angle = lambda: L.Binop("mul", L.Get(pos, (L.It(p),)), L.Get(freqs, (L.It(kf),)))
    G = lambda n: L.Get(n, at)
    body.append(L.For(p, 0, seq - 1, [L.For(kf, 0, dk // 2 - 1, [
        L.Set(cos_a, at, L.Unop("cos", angle())), L.Set(sin_a, at, L.Unop("sin", angle())),
        L.Set(oe, at, L.Binop("sub", L.Binop("mul", G(xe), G(cos_a)), L.Binop("mul", G(xo), G(sin_a)))),
        L.Set(oo, at, L.Binop("add", L.Binop("mul", G(xe), G(sin_a)), L.Binop("mul", G(xo), G(cos_a))))])]))
    rotated = join(oe, oo, (seq,), dk // 2, "rotated")
    init = {x6.id: np.arange(1, 7, dtype=np.float32),
            x.id: (np.arange(seq * dk, dtype=np.float32) + 1).reshape(seq, dk),
            freqs.id: np.array([10000.0 ** (-2.0 * k / dk) for k in range(dk // 2)], np.float32),
            pos.id: np.arange(seq, dtype=np.float32)}
    return L.Routine("rope_kat", body), init, {"roundtrip": round_trip, "rotated": rotated}


def check_small_ops(run_cls, kat):
    for key, cond in (("true", 1.0), ("false", 0.0)):
        r, init, nodes = where_simple(cond)
        run = run_cls(r, init)
        run.step()
        for name, want in kat["where_simple"][key].items():
            assert float(run.get(nodes[name])[0]) == want, (key, name)
        run.close()
    r, init, nodes = fma_logic()
    run = run_cls(r, init)
    run.step()
    for name, want in kat["fma_logic"].items():
        if not name.startswith("_"):
            assert list(run.get(nodes[name])) == want, name
    run.close()
    r, init, nodes = rope()
    run = run_cls(r, init)
    run.step()
    assert list(run.get(nodes["roundtrip"])) == kat["rope"]["roundtrip"]
    rot = run.get(nodes["rotated"])
    assert [f"{v:.2f}" for v in rot[0]] == kat["rope"]["position0"]
    assert [f"{v:.4f}" for v in rot[1]] == kat["rope"]["position1"]
    run.close()


def windows():
    """The three window routines.  The padded input is uploaded with junk in its margin: only the reset
    loops make the stated answers come out."""
    L.reset_symbols(0)
    f32 = "single"
    xin = L.Node(1, "input", f32, (6, 6))          # 4 x 4 with a margin of one on every side
    pooled = L.Node(2, "pooled", f32, (4, 4)); conv = L.Node(3, "conv_out", f32, (4, 4))
    r = L.Node(4, "r4x4x1", f32, (4, 4, 1)); mp = L.Node(5, "max_pool2d", f32, (2, 2, 1))
    kern = L.Node(6, "k", f32, (2, 2)); trop = L.Node(7, "tropical", f32, (2, 2, 1))
    padding = ((1, 1), (1, 1))
    body = []

    def window_nest(out, out_idx, ext, stmt):
        nest = [stmt]
        for sym, e in reversed(ext):
            nest = [L.For(sym, 0, e - 1, nest)]
        return nest

    # max over 3 x 3 windows of the padded input, margin = -infinity
    body += L.loop_over_padding_region(xin.dims, padding, lambda ix: [L.Set(xin, ix, L.Const(float("-inf")))])
    body += L.loop_over_dims(pooled.dims, lambda ix: [L.Set(pooled, ix, L.Const(float("-inf")))])
    oh, ow, wh, ww = (L.fresh_symbol() for _ in range(4))
    at = (L.It(oh), L.It(ow)); win = (L.Affine(((1, oh), (1, wh)), 0), L.Affine(((1, ow), (1, ww)), 0))
    body += window_nest(pooled, at, [(oh, 4), (ow, 4), (wh, 3), (ww, 3)],
                        L.Set(pooled, at, L.Binop("max", L.Get(pooled, at), L.Get(xin, win))))
    # sum over 3 x 3 windows of the SAME input times 1, margin = 0
    body += L.loop_over_padding_region(xin.dims, padding, lambda ix: [L.Set(xin, ix, L.Const(0.0))])
    body.append(L.ZeroOut(conv))
    oh, ow, kh, kw = (L.fresh_symbol() for _ in range(4))
    at = (L.It(oh), L.It(ow)); win = (L.Affine(((1, oh), (1, kh)), 0), L.Affine(((1, ow), (1, kw)), 0))
    body += window_nest(conv, at, [(oh, 4), (ow, 4), (kh, 3), (kw, 3)],
                        L.Set(conv, at, L.Ternop("fma", L.Get(xin, win), L.Const(1.0), L.Get(conv, at))))
    # max-pool stride 2 window 2, and the tropical kernel: max over the window of input + k
    for out, with_kernel in ((mp, False), (trop, True)):
        body += L.loop_over_dims(out.dims, lambda ix: [L.Set(out, ix, L.Const(float("-inf")))])
        oh, ow, c, wh, ww = (L.fresh_symbol() for _ in range(5))
        at = (L.It(oh), L.It(ow), L.It(c))
        src = L.Get(r, (L.Affine(((2, oh), (1, wh)), 0), L.Affine(((2, ow), (1, ww)), 0), L.It(c)))
        val = L.Binop("add", src, L.Get(kern, (L.It(wh), L.It(ww)))) if with_kernel else src
        body += window_nest(out, at, [(oh, 2), (ow, 2), (c, 1), (wh, 2), (ww, 2)], L.Set(out, at, L.Binop("max", L.Get(out, at), val)))
    padded = np.full((6, 6), 777.0, np.float32)
    padded[1:5, 1:5] = np.arange(16, dtype=np.float32).reshape(4, 4) - 16.0
    init = {1: padded, 4: np.arange(16, dtype=np.float32).reshape(4, 4, 1), 6: np.arange(4, dtype=np.float32).reshape(2, 2)}
    return L.Routine("windows_kat", body), init, {"pooled": pooled, "conv": conv, "max_pool": mp, "tropical": trop}


def check_windows(run_cls, kat):
    k = kat["windows"]
    r, init, nodes = windows()
    run = run_cls(r, init)
    for _ in range(2):                      # the reference runs the pair twice: the resets hold across runs
        run.step()
        pooled, conv = run.get(nodes["pooled"]), run.get(nodes["conv"])
        w = k["padding_reset"]
        assert (float(pooled[0, 0]), float(pooled[1, 1]), float(conv[0, 0]), float(conv[1, 1])) == \
            (w["pooled_0_0"], w["pooled_1_1"], w["conv_0_0"], w["conv_1_1"])
        assert np.isfinite(conv).all() and np.isfinite(pooled).all()
    assert list(run.get(nodes["max_pool"]).ravel()) == k["max_pool_4x4_stride2_window2"]
    assert list(run.get(nodes["tropical"]).ravel()) == k["tropical_4x4_kernel_0123"]
    run.close()


def accumulation_semantics():
    """The four assignments of test_accumulation_semantics.ml:20-101 as `=:+` lowers them: Zero_out,
    then the accumulating Set over the product space.  Results are uploaded full of junk."""
    L.reset_symbols(0)
    f32 = "single"
    r3 = L.Node(1, "r2x4x3", f32, (2, 4, 3)); red = L.Node(2, "result", f32, (2, 3))
    v5 = L.Node(3, "v5", f32, (5,)); diag = L.Node(4, "diagonal", f32, (5, 5))
    v4 = L.Node(5, "v4", f32, (4,)); sparse = L.Node(6, "sparse", f32, (4, 3))
    m = L.Node(7, "r3x4", f32, (3, 4)); tr = L.Node(8, "transposed", f32, (4, 3))
    b, i, o, d, p, q, t = (L.fresh_symbol() for _ in range(7))
    acc = lambda node, lhs, rhs: L.Set(node, lhs, L.Binop("add", L.Get(node, lhs), rhs))
    body = [L.ZeroOut(red), L.For(b, 0, 1, [L.For(i, 0, 2, [L.For(o, 0, 3, [
                acc(red, (L.It(b), L.It(i)), L.Get(r3, (L.It(b), L.It(o), L.It(i))))])])]),
            L.ZeroOut(diag), L.For(d, 0, 4, [acc(diag, (L.It(d), L.It(d)), L.Get(v5, (L.It(d),)))]),
            L.ZeroOut(sparse), L.For(p, 0, 3, [acc(sparse, (L.It(p), L.Fixed(0)), L.Get(v4, (L.It(p),)))]),
            L.For(q, 0, 3, [L.For(t, 0, 2, [L.Set(tr, (L.It(q), L.It(t)), L.Get(m, (L.It(t), L.It(q))))])])]
    junk = lambda n: np.full(n.dims, 55.0, np.float32)
    init = {1: np.arange(24, dtype=np.float32).reshape(2, 4, 3), 3: np.arange(5, dtype=np.float32),
            5: np.arange(4, dtype=np.float32), 7: np.arange(12, dtype=np.float32).reshape(3, 4),
            2: junk(red), 4: junk(diag), 6: junk(sparse), 8: junk(tr)}
    return L.Routine("accumulation_semantics", body), init, {"reduction": red, "diagonal": diag, "sparse": sparse, "transposed": tr}


def check_accumulation(run_cls, kat):
    r, init, nodes = accumulation_semantics()
    run = run_cls(r, init)
    for _ in range(2):
        run.step()
        for name, node in nodes.items():
            assert np.array_equal(run.get(node), np.asarray(kat["accumulation_semantics"][name], np.float32)), name
    run.close()


def sig3(x):
    """The reference's table format: three significant digits, cut off rather than rounded (its
    tables print 2198 as 2.19e+3 and 1694 as 1.69e+3)."""
    def cut(v):
        if v == 0.0:
            return 0.0
        unit = 10.0 ** (int(np.floor(np.log10(abs(v)))) - 2)
        return float(np.floor(abs(v) / unit + 1e-9) * unit) * (1.0 if v > 0 else -1.0)
    return np.vectorize(cut)(np.asarray(x, np.float64))


def check_micrograd(get, kat):
    k = kat["micrograd"]
    for name, key in (("g", "g_milli"), ("a_grad", "a_grad_milli"), ("b_grad", "b_grad_milli")):
        v = float(get(name)[0])
        assert int(v * 1000.0) == k[key], (name, v, k[key])   # the log prints integer thousandths


def check_einsum(get, kat):
    k = kat["einsum_trivia"]
    for name in ("a2", "c", "d", "e", "f"):
        assert np.array_equal(sig3(get(name)), np.asarray(k[name], np.float64)), name


def check_hello(run_factory, kat):
    k = kat["hello_world"]
    get = run_factory(*hello_world(3, 2, 7.0, [2, 3], [4, 5, 6]))
    assert list(get("y")) == k["matmul_2x3"]
    get = run_factory(*hello_world(20, 20, 0.5, np.arange(20), np.arange(20)))
    y = get("y")
    assert [float(y[0]), float(y[1]), float(y[-2]), float(y[-1])] == k["big_matrix_first2_last2"]
    assert np.array_equal(y, 95.0 + np.arange(20, dtype=np.float32))


def check_zero2hero(run_cls, kat):
    """`run_cls(routine, init)` gives an object with step(static=None), get(node), and from_host-like
    `set(node, array)`; the same driver for the checker and the HIP library."""
    k = kat["zero2hero"]
    # the polynomial at x = 5: every value and gradient of the printed tree
    r, init, nodes, _ = zero2hero_poly()
    run = run_cls(r, init)
    run.step()
    for name, want in k["poly_at_5"].items():
        assert float(run.get(nodes[name])[0]) == want, name
    # :38-52 sweeps x over -5 .. 4 by assigning it between runs
    ys = []
    for v in np.arange(10, dtype=np.float32) - 5.0:
        run.set(nodes["x"], np.array([v], np.float32))
        run.step()
        ys.append(float(run.get(nodes["f"])[0]))
    w = k["poly_sweep_int"]
    assert (len(ys), min(ys), max(ys), ys[0]) == (w["count"], w["min"], w["max"], w["first"])
    run.close()
    # :60-101 sweeps through a static index over x_flat = i / 10 - 5 and reads f and x's gradient
    xs = [i / 10.0 - 5.0 for i in range(100)]
    r, init, nodes, extra = zero2hero_poly(xs)
    run = run_cls(r, init)
    ys, dys = [], []
    for i in range(100):
        run.step({extra["step"].sym: i})
        ys.append(float(run.get(nodes["f"])[0])); dys.append(float(run.get(nodes["grad_x"])[0]))
    w = k["poly_sweep_tenths"]
    r2 = lambda v: float(f"{v:.2f}")     # print_summary prints %.2f
    assert (len(ys), r2(min(ys)), r2(max(ys)), r2(ys[0])) == (w["count"], w["ys_min"], w["ys_max"], w["ys_first"])
    assert (r2(min(dys)), r2(max(dys)), r2(dys[0])) == (w["dys_min"], w["dys_max"], w["dys_first"])
    run.close()
    # the product-sum: gradients, an SGD step, gradients again
    grad, sgd, init, nodes = zero2hero_simple_gradients()
    run = run_cls([grad, sgd], init)
    run.step(index=0)
    for name, want in k["simple_gradients"]["first"].items():
        assert float(run.get(nodes[name])[0]) == want, name
    run.step(index=1)
    for name, want in k["simple_gradients"]["after_sgd"].items():
        assert abs(float(run.get(nodes[name])[0]) - want) < 1e-6, name
    run.step(index=0)
    for name, want in k["simple_gradients"]["second"].items():
        got = float(run.get(nodes[name])[0])
        assert float(f"{got:.3g}") == want, (name, got)     # the tree prints three significant digits
    run.close()
    # the two-input neuron
    r, init, nodes = zero2hero_neuron()
    run = run_cls(r, init)
    run.step()
    w = k["neuron_2d"]
    assert abs(float(run.get(nodes["v"])[0]) - w["v"]) < 1e-6 and float(run.get(nodes["mul"])[0]) == w["mul"]
    assert list(run.get(nodes["grad_w"]).ravel()) == w["grad_w"] and list(run.get(nodes["grad_x"])) == w["grad_x"]
    assert float(run.get(nodes["grad_b"])[0]) == w["grad_b"]
    run.close()


class _CheckerSession:
    """One or several routines over shared host buffers, through the CPU checker."""

    def __init__(self, routines, init):
        from oracle import cc_oracle
        from parity import oracle_buffers
        self.routines = routines if isinstance(routines, list) else [routines]
        self.lib = cc_oracle.CompiledOracle(self.routines)
        self.bufs = {}
        for r in self.routines:
            for k, v in oracle_buffers(r, init).items():
                self.bufs.setdefault(k, v)

    def step(self, static=None, index=0):
        r = self.routines[index]
        self.lib.run(r.name, {n.id: self.bufs[n.id] for n in r.param_nodes()}, static or {})

    def get(self, node):
        return self.bufs[node.id]

    def set(self, node, values):
        self.bufs[node.id][...] = values

    def close(self):
        pass


def _hip_session(options):
    from ocannl_amd import backend as B

    class Session:
        """The same through the HIP library: one compiled batch, one context, one linked routine each."""

        def __init__(self, routines, init):
            self.routines = routines if isinstance(routines, list) else [routines]
            self.code = B.compile_batch(self.routines, options)
            self.ctx = B.Context()
            for r in self.routines:
                self.ctx.allocate(r.param_nodes())
                for n in r.param_nodes():
                    if n.id in init:
                        self.ctx.set_values(n, init[n.id])
            self.rts = [self.ctx.link(self.code, i) for i in range(len(self.routines))]

        def step(self, static=None, index=0):
            for sym, v in (static or {}).items():
                self.rts[index].set_static(sym, v)
            self.rts[index].run()

        def get(self, node):
            return self.ctx.get_values(node)

        def set(self, node, values):
            self.ctx.set_values(node, values)

        def close(self):
            B.await_(self.ctx.dev)
            self.rts = []
            self.ctx.free()

    return Session


def oracle_factory(r, init, nodes):
    o = OracleRun(r, init)
    o.step()
    return lambda name: o.get(nodes[name])


def test_micrograd_known_answers_checker(kat):
    check_micrograd(oracle_factory(*micrograd()), kat)


def test_einsum_tables_checker(kat):
    check_einsum(oracle_factory(*einsum_trivia()), kat)


def test_hello_world_checker(kat):
    check_hello(oracle_factory, kat)


def test_zero2hero_known_answers_checker(kat):
    check_zero2hero(_CheckerSession, kat)


def test_where_fma_rope_known_answers_checker(kat):
    check_small_ops(_CheckerSession, kat)


def test_window_known_answers_checker(kat):
    check_windows(_CheckerSession, kat)


def test_accumulation_semantics_checker(kat):
    check_accumulation(_CheckerSession, kat)


def hip_factory(options):
    from ocannl_amd.backend import HipRun

    def make(r, init, nodes):
        h = HipRun(r, init, options)
        h.step()
        vals = {k: h.get(n) for k, n in nodes.items()}
        h.close()
        return lambda name: vals[name]
    return make


@pytest.mark.gpu
@pytest.mark.parametrize("options", [None, "mfma=0;coop=0", "serial=0;parallel=0"])
def test_known_answers_on_the_gpu(kat, options):
    make = hip_factory(options)
    check_micrograd(make(*micrograd()), kat)
    check_einsum(make(*einsum_trivia()), kat)
    check_hello(make, kat)
    check_zero2hero(_hip_session(options), kat)
    check_small_ops(_hip_session(options), kat)
    check_windows(_hip_session(options), kat)
    check_accumulation(_hip_session(options), kat)
