"""GPU parity of the planner's kernel-fusing rewrites at sizes where they switch on: row groups
(register-cached and fenced), split column reductions, lane-cooperative scalar reductions, bf16
operand copies kept by the producing kernels, the single-workgroup kernel for tiny routines."""
import re

import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L
from ocannl_amd import workloads as W
from parity import HipRun, OracleRun, rel_err
from test_gpu_models import _err, _widened_init

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("prec,tol,vocab", [("single", 1e-4, 2048), ("bfloat16", 2e-2, 2048), ("bfloat16", 2e-2, 1088)])
def test_transformer_with_row_groups_and_operand_copies(prec, tol, vocab):
    # seq 128: soft-max rows of 128 (2 per lane of a wave: kept in registers); vocab 2048: a workgroup per
    # row (8 per lane, kept in registers, sums exchanged through LDS); vocab 1088: 17 per lane of a wave,
    # through memory with fences; bf16 values with fp32 gradients: mirrored bf16 copies
    kw = dict(batch=4, seq=128, d_model=128, heads=2, d_ff=256, layers=1, vocab=vocab, grad_prec="single", lr=0.05)
    w = W.transformer(prec=prec, **kw)
    wr = W.transformer(prec="single", **kw)
    hip = HipRun(w.routine, w.init)
    src = hip.code.source()
    assert "row0_" in src and "it_" in src
    assert ("red_[" in src) if vocab == 2048 else ("__builtin_amdgcn_fence" in src)
    if prec == "bfloat16":
        assert re.search(r"bf\d+_\w+\[[^\]]*\] = single_to_bfloat16\(", src)
    n_default = len(hip.code.kernels())
    n_plain = len(B.compile(w.routine, "rows=0;bf16_copies=0").kernels())
    assert n_default < n_plain
    ora = OracleRun(wr.routine, _widened_init(w, wr))
    for _ in range(2):
        hip.step(); ora.step()
        lh = float(W.to_float(hip.get(w.nodes["loss"]), w.nodes["loss"].prec)[0]); lo = float(ora.get(wr.nodes["loss"])[0])
        assert abs(lh - lo) <= tol * max(abs(lo), 1.0), (lh, lo)
    for name in ("w_embed", "w_q_l0", "w_ffn2_l0", "w_out", "gamma_ln1_l0", "beta_ln2_l0", "pos_encoding"):
        assert _err(W.to_float(hip.get(w.nodes[name]), prec), ora.get(wr.nodes[name]), prec) <= tol, name
    hip.close()


def test_row_groups_equal_separate_kernels_bit_for_bit():
    # fusing phases into row groups changes where values live, not what is computed
    kw = dict(batch=4, seq=128, d_model=128, heads=2, d_ff=256, layers=1, vocab=512, prec="single", grad_prec="single")
    w = W.transformer(**kw)
    a, b = HipRun(w.routine, w.init), HipRun(w.routine, w.init, "rows=0")
    assert len(a.code.kernels()) < len(b.code.kernels())
    a.step(); b.step()
    for name in ("loss", "w_q_l0", "w_out", "gamma_ln1_l0"):
        assert np.array_equal(a.get(w.nodes[name]), b.get(w.nodes[name])), name
    a.close(); b.close()


@pytest.mark.parametrize("accumulate", [False, True])
def test_split_column_reduction(accumulate):
    # out[j] (+)= sum_i x[i, j] * y[i, j]: small output, reduction over the slow axis
    rows, cols = 4096, 256
    L.reset_symbols(0)
    x = L.Node(1, "x", "single", (rows, cols)); y = L.Node(2, "y", "single", (rows, cols))
    out = L.Node(3, "out", "single", (cols,))
    j, i = L.fresh_symbol(), L.fresh_symbol()
    body = [] if accumulate else [L.ZeroOut(out)]
    body.append(L.For(j, 0, cols - 1, [L.For(i, 0, rows - 1, [
        L.Set(out, (L.It(j),), L.Ternop("fma", L.Get(x, (L.It(i), L.It(j))), L.Get(y, (L.It(i), L.It(j))),
                                         L.Get(out, (L.It(j),))))])]))
    r = L.Routine("colsum", body)
    rng = np.random.default_rng(3)
    init = {1: rng.standard_normal((rows, cols)).astype(np.float32), 2: rng.standard_normal((rows, cols)).astype(np.float32),
            3: rng.standard_normal(cols).astype(np.float32)}
    hip, ora = HipRun(r, init), OracleRun(r, init)
    src = hip.code.source()
    assert re.search(r"part\d+_out", src), "the reduction was not split"
    assert len(hip.code.kernels()) == 2
    hip.step(); ora.step()
    assert rel_err(hip.get(out), ora.get(out), "single") <= 1e-4
    # the unsplit, sequential version is bit-identical to the checker
    seq = HipRun(r, init, "coop=0")
    seq.step()
    assert np.array_equal(seq.get(out), ora.get(out))
    hip.close(); seq.close()


def test_split_reduction_over_several_loops_one_of_them_not_from_zero():
    # out[p, q] += sum_{a = 1..6, b < 12, c < 64} x[a, b, c, p, q]: the two outer loops become whole
    # slices, the third is divided, and all three are the digits of ONE slice axis of the partial
    # tensor (6 x 12 x 2 = 144 slices, the first loop shifted to start at zero), which the second half
    # walks with one loop shared by a group of lanes
    A, Bq, C, P, Q = 7, 12, 64, 8, 64
    L.reset_symbols(0)
    x = L.Node(1, "x", "single", (A, Bq, C, P, Q)); out = L.Node(2, "out", "single", (P, Q))
    p_, q_, a_, b_, c_ = (L.fresh_symbol() for _ in range(5))
    body = [L.For(p_, 0, P - 1, [L.For(q_, 0, Q - 1, [L.For(a_, 1, A - 1, [L.For(b_, 0, Bq - 1, [L.For(c_, 0, C - 1, [
        L.Set(out, (L.It(p_), L.It(q_)), L.Binop("add", L.Get(out, (L.It(p_), L.It(q_))),
                                                 L.Get(x, (L.It(a_), L.It(b_), L.It(c_), L.It(p_), L.It(q_)))))])])])])])]
    r = L.Routine("sum3", body)
    rng = np.random.default_rng(11)
    init = {1: rng.standard_normal((A, Bq, C, P, Q)).astype(np.float32), 2: rng.standard_normal((P, Q)).astype(np.float32)}
    hip, ora = HipRun(r, init), OracleRun(r, init)
    src = hip.code.source()
    m = re.search(r"float \* __restrict__ (part\d+_out)", src)
    assert m and len(hip.code.kernels()) == 2, "the reduction was not split"
    assert re.search(re.escape(m.group(1)) + r"\[\(\(24\*i\d+\+2\*i\d+\+i\d+\+-24\) \* 8", src), "slices not on one axis"
    assert re.search(r"for \(uint32_t i\d+ = 0 \+ lane_; i\d+ <= 143; i\d+ \+= 16\)", src), "second half: sixteen lanes over the slices"
    hip.step(); ora.step()
    assert rel_err(hip.get(out), ora.get(out), "single") <= 1e-4
    want = init[2].astype(np.float64) + init[1][1:].astype(np.float64).sum(axis=(0, 1, 2))
    assert np.max(np.abs(hip.get(out) - want)) <= 1e-4 * np.max(np.abs(want))
    hip.close()


def test_scalar_reduction_shared_by_lanes():
    # loss = (sum_i -log p[i]) / n written as an inlined scalar reduction inside one statement
    n = 8192
    L.reset_symbols(0)
    p = L.Node(1, "p", "single", (n,)); loss = L.Node(2, "loss", "single", (1,))
    acc = L.Node(3, "acc", "single", (1,), mode="virtual")
    i = L.fresh_symbol()
    sc = L.Scope(acc, 1)
    scope = L.LocalScope(sc, [
        L.SetLocal(sc, L.Const(0.0)),
        L.For(i, 0, n - 1, [L.SetLocal(sc, L.Binop("add", L.GetLocal(sc), L.Unop("neg", L.Unop("log", L.Get(p, (L.It(i),))))))])])
    r = L.Routine("nll", [L.Set(loss, (L.Fixed(0),), L.Binop("div", scope, L.Const(float(n))))])
    init = {1: np.random.default_rng(5).uniform(0.05, 1.0, n).astype(np.float32)}
    hip, ora = HipRun(r, init), OracleRun(r, init)
    assert "ocn_xshfl" in hip.code.source()
    hip.step(); ora.step()
    assert rel_err(hip.get(loss), ora.get(loss), "single") <= 1e-4
    hip.close()


def test_tiny_routine_is_one_workgroup_with_identical_results():
    w = W.moons_mlp()
    sym = w.statics["batch_n"].sym
    one, many = HipRun(w.routine, w.init, "coop=0"), HipRun(w.routine, w.init, "coop=0;serial=0")
    assert len(one.code.kernels()) == 1 and len(many.code.kernels()) > 10
    ora = OracleRun(w.routine, w.init)
    for step in range(10):
        st = {sym: step}
        one.step(st); many.step(st); ora.step(st)
    for name in ("w1", "w2", "w3", "b1"):
        assert np.array_equal(one.get(w.nodes[name]), many.get(w.nodes[name])), name
        assert rel_err(one.get(w.nodes[name]), ora.get(w.nodes[name]), "single") <= 1e-5, name
    one.close(); many.close()


def test_integer_row_sums_stay_exact():
    # lanes share a row only through floating-point accumulators: a uint32 sum (wrapping, values far
    # beyond 2^24) must come out bit-exact, so integer rows are walked sequentially
    rows, cols = 96, 2048
    L.reset_symbols(0)
    x = L.Node(1, "x", "uint32", (rows, cols)); s = L.Node(2, "s", "uint32", (rows,))
    i, j = L.fresh_symbol(), L.fresh_symbol()
    r = L.Routine("usum", [L.For(i, 0, rows - 1, [L.For(j, 0, cols - 1, [
        L.Set(s, (L.It(i),), L.Binop("add", L.Get(s, (L.It(i),)), L.Get(x, (L.It(i), L.It(j)))))])])])
    xv = np.random.default_rng(3).integers(0, 1 << 32, size=(rows, cols), dtype=np.uint64).astype(np.uint32)
    hip, ora = HipRun(r, {x.id: xv}), OracleRun(r, {x.id: xv})
    hip.step(); ora.step()
    want = xv.sum(axis=1, dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(ora.get(s), want)
    assert np.array_equal(hip.get(s), want)
    hip.close()


def test_bf16_operand_copy_follows_every_kind_of_writer():
    # an fp32 tensor G feeds bf16 contractions three times: after generated stores (its bf16 copy is
    # written by those stores), after a matrix-core contraction has accumulated into it (the copy no
    # longer stands for it: a fresh conversion pass), and after a zero fill (the copy is zeroed too)
    M, N, K = 128, 128, 128
    L.reset_symbols(0)
    ids = iter(range(1, 50))
    node = lambda name, prec, dims: L.Node(next(ids), name, prec, dims)
    X = node("x", "single", (M, K)); G = node("g", "single", (M, K)); Wb = node("w", "bfloat16", (N, K))
    Ab = node("a", "bfloat16", (M, N)); outs = [node(f"out{k}", "single", (M, N)) for k in range(3)]
    def nest(exts, body):
        syms = [L.fresh_symbol() for _ in exts]
        b = body(*[L.It(s) for s in syms])
        for s, e in reversed(list(zip(syms, exts))):
            b = [L.For(s, 0, e - 1, b)]
        return b
    fma = lambda p, q, c: L.Ternop("fma", p, q, c)
    read_g = lambda o: nest((M, N, K), lambda m, n, k: [L.Set(o, (m, n), fma(L.Get(G, (m, k)), L.Get(Wb, (n, k)), L.Get(o, (m, n))))])
    body = nest((M, K), lambda m, k: [L.Set(G, (m, k), L.Binop("mul", L.Const(0.5), L.Get(X, (m, k))))])
    body += [L.ZeroOut(outs[0])] + read_g(outs[0])
    body += nest((M, K, N), lambda m, k, n: [L.Set(G, (m, k), fma(L.Get(Ab, (m, n)), L.Get(Wb, (n, k)), L.Get(G, (m, k))))])
    body += [L.ZeroOut(outs[1])] + read_g(outs[1])
    body += [L.ZeroOut(G), L.ZeroOut(outs[2])] + read_g(outs[2])
    r = L.Routine("mirror_chain", body)
    rng = np.random.default_rng(4)
    init = {X.id: rng.standard_normal(X.dims).astype(np.float32), Wb.id: W.as_prec(rng.standard_normal(Wb.dims).astype(np.float32), "bfloat16"),
            Ab.id: W.as_prec(rng.standard_normal(Ab.dims).astype(np.float32) / 16, "bfloat16")}
    hip = HipRun(r, init, "min_mfma_flops=1")
    # four contractions in three launches: the second and third reads of G take conversion passes of
    # their own, so the second may wait for the third and share its launch; the first may not (its
    # operand is the copy kept by G's stores, which the contraction into G invalidates)
    ks = hip.code.kernels()
    assert sum(k["kind"] == "mfma" for k in ks) == 3 and sum(k["batch"] for k in ks if k["kind"] == "mfma") == 4
    hip.step()
    bf = lambda a: W.to_float(W.as_prec(np.asarray(a, np.float32), "bfloat16"), "bfloat16").astype(np.float64)
    w64, a64 = W.to_float(init[Wb.id], "bfloat16").astype(np.float64), W.to_float(init[Ab.id], "bfloat16").astype(np.float64)
    g1 = (0.5 * init[X.id]).astype(np.float32)
    g2 = (g1.astype(np.float64) + a64 @ w64).astype(np.float32)
    for got, want in ((hip.get(outs[0]), bf(g1) @ w64.T), (hip.get(outs[1]), bf(g2) @ w64.T)):
        assert np.max(np.abs(got - want)) <= 2e-2 * np.max(np.abs(want))
    assert not hip.get(outs[2]).any() and not hip.get(G).any()
    hip.close()


def test_independent_small_statements_run_side_by_side():
    # p_k = p_k - lr (g_k + 0 p_k) for seven parameters of different shapes, as two statements each (the
    # shape of an SGD step): the seven deltas do not touch one another, neither do the seven updates, and
    # every update reads its delta -- two launches instead of fourteen
    # (one launch when each delta / update pair has been fused into a row group first)
    L.reset_symbols(0)
    shapes = [(512,), (512,), (64, 48), (2048,), (7,), (300, 10), (33, 5, 3)]
    ids = iter(range(1, 100))
    lr = L.Node(next(ids), "lr", "single", (1,))
    params, grads, deltas, body = [], [], [], []
    for k, dims in enumerate(shapes):
        p, g, d = (L.Node(next(ids), f"{n}{k}", "single", dims) for n in ("p", "g", "delta"))
        params.append(p); grads.append(g); deltas.append(d)
    def nest(dims, stmt):
        syms = [L.fresh_symbol() for _ in dims]
        b = [stmt(tuple(L.It(s) for s in syms))]
        for s, e in reversed(list(zip(syms, dims))):
            b = [L.For(s, 0, e - 1, b)]
        return b
    for p, g, d in zip(params, grads, deltas):
        body += nest(p.dims, lambda ix: L.Set(d, ix, L.Binop("add", L.Get(g, ix), L.Binop("mul", L.Const(0.0), L.Get(p, ix)))))
        body += nest(p.dims, lambda ix: L.Set(p, ix, L.Binop("sub", L.Get(p, ix), L.Binop("mul", L.Get(lr, (L.Fixed(0),)), L.Get(d, ix)))))
    r = L.Routine("small_updates", body)
    rng = np.random.default_rng(8)
    init = {n.id: rng.standard_normal(n.dims).astype(np.float32) for n in params + grads}
    init[lr.id] = np.array([0.1], np.float32)
    ora = OracleRun(r, init)
    ora.step(); ora.step()
    for opts, launches in (("serial=0;rows=0", 2), ("serial=0;rows=0;parallel=0", 14), ("serial=0", 1)):
        hip = HipRun(r, init, opts)
        assert len(hip.code.kernels()) == launches, hip.code.kernels()
        hip.step(); hip.step()
        for n in params + deltas:     # (the host compiler may fuse the multiply into the subtraction: last bit)
            assert rel_err(hip.get(n), ora.get(n), "single") <= 1e-6, (opts, n.ident)
        hip.close()
