"""Whole-routine known answers that the reference's own tests hold, run through the harness
(ocannl_amd/frontend.py) and then BOTH the CPU checker and -- on a GPU -- the HIP library:
  * micrograd: g, a.grad, b.grad of test/operations/micrograd_demo_logging.ml as logged in
    micrograd_demo_logging-sync_cc-0-0.log.expected (forward code + reverse-mode derivatives);
  * the einsum tables of test/einsum/einsum_trivia.ml:378-481 (pointwise, batched matrix product,
    outer batch product, sums over batch axes; operand layout batch @ output @ input);
  * test/operations/hello_world_op.ml:479-548 (matrix-vector product plus bias).
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
