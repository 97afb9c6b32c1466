"""A value that an earlier statement stored is read back instead of being computed again (the routine
form the visit rule of low_level.ml:496-552 produces spells an inlined reduction out at every reader) --
and only where that is the same number: same extents, nothing written in between, no precision lost in
the store.  Every case runs against the checker; the compile-only half of each case (was it rewritten
or not) needs no GPU."""
import re

import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L
from parity import HipRun, OracleRun, rel_err

K = 48


def _rowsum(tmp, a, i):
    """``v { v := 0; for k { v := fma(a[i, k], a[i, k], v) } }`` typed by ``tmp``."""
    sc = L.Scope(tmp, L.fresh_symbol())
    k = L.fresh_symbol()
    return L.LocalScope(sc, [
        L.SetLocal(sc, L.Const(0.0)),
        L.For(k, 0, K - 1, [L.SetLocal(sc, L.Ternop("fma", L.Get(a, (L.It(i), L.It(k))), L.Get(a, (L.It(i), L.It(k))), L.GetLocal(sc)))])])


def _wrapped(tmp, value):
    """``v { v := value }``: how the lowering keeps a value rounded to the precision of ``tmp`` first."""
    sc = L.Scope(tmp, L.fresh_symbol())
    return L.LocalScope(sc, [L.SetLocal(sc, value)])


def _case(kind):
    L.reset_symbols(0)
    rows_a = 64
    rows_t = 32 if kind == "short" else rows_a
    t_prec = "bfloat16" if kind == "narrow" else "single"
    a = L.Node(1, "a", "single", (rows_a, K))
    t = L.Node(2, "t", t_prec, (rows_t,))
    u = L.Node(3, "u", "single", (rows_a,))
    d = L.Node(4, "d", "single", (rows_a,))
    tmp = L.Node(5, "s", "single", (1,), mode="virtual")
    tmp16 = L.Node(6, "h", "bfloat16", (1,), mode="virtual")
    i, j = L.fresh_symbol(), L.fresh_symbol()
    shifted = lambda x: L.Binop("sub", x, L.Const(40.0))
    if kind == "relu":
        body = [L.For(i, 0, rows_t - 1, [L.Set(t, (L.It(i),), L.Unop("relu", shifted(_rowsum(tmp, a, i))))])]
        body.append(L.For(j, 0, rows_a - 1, [L.Set(u, (L.It(j),), L.Binop("relu_gate", shifted(_rowsum(tmp, a, j)), L.Get(d, (L.It(j),))))]))
    elif kind in ("narrow", "widened"):
        # the sum rounded to fp32 and stored as bf16 loses bits; rounded to bf16 and stored as fp32 it does not
        w = tmp if kind == "narrow" else tmp16
        body = [L.For(i, 0, rows_t - 1, [L.Set(t, (L.It(i),), _wrapped(w, _rowsum(tmp, a, i)))])]
        body.append(L.For(j, 0, rows_a - 1, [L.Set(u, (L.It(j),), L.Binop("mul", _wrapped(w, _rowsum(tmp, a, j)), L.Get(d, (L.It(j),))))]))
    else:
        body = [L.For(i, 0, rows_t - 1, [L.Set(t, (L.It(i),), _rowsum(tmp, a, i))])]
        if kind == "overwritten":
            body.append(L.Set(a, (L.Fixed(3), L.Fixed(5)), L.Const(7.0)))
        body.append(L.For(j, 0, rows_a - 1, [L.Set(u, (L.It(j),), L.Binop("add", L.Binop("mul", _rowsum(tmp, a, j), L.Get(d, (L.It(j),))), L.Const(1.0)))]))
    r = L.Routine(f"reuse_{kind}", body)
    rng = np.random.default_rng(11)
    init = {1: rng.standard_normal((rows_a, K)).astype(np.float32), 4: rng.standard_normal(rows_a).astype(np.float32)}
    return r, init, t, u


CASES = [("same", True), ("relu", True), ("widened", True), ("short", False), ("overwritten", False), ("narrow", False)]


def _reduction_loops(code):
    return len(re.findall(rf"for \(uint32_t i\d+ = [^;]*; i\d+ <= {K - 1};", code.source()))


@pytest.mark.parametrize("kind,rewritten", CASES)
def test_which_recomputations_become_reads(kind, rewritten):
    r, _, _, _ = _case(kind)
    assert _reduction_loops(B.compile(r, "reuse=0")) == 2
    assert _reduction_loops(B.compile(r)) == (1 if rewritten else 2), kind


@pytest.mark.gpu
@pytest.mark.parametrize("kind,rewritten", CASES)
def test_reused_values_against_the_checker(kind, rewritten):
    r, init, t, u = _case(kind)
    hip, ora = HipRun(r, init), OracleRun(r, init)
    hip.step(); ora.step()
    assert rel_err(hip.get(u), ora.get(u), "single") <= 1e-4, kind
    hip.close()
