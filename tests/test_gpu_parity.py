"""GPU parity tests: the HIP library (through the C ABI) against the CPU checker on identical
seeded inputs.  Tolerances follow the stated bar: fp32 within 1e-4 relative, bf16 within 2e-2,
loss curves over 100 steps within 1e-3."""
import numpy as np
import pytest

from ocannl_amd import llir as L
from ocannl_amd import workloads as W
from parity import HipRun, OracleRun, rel_err

pytestmark = pytest.mark.gpu


def _small_contraction():
    L.reset_symbols(0)
    a = L.Node(1, "a", "single", (3, 5)); b = L.Node(2, "b", "single", (5, 4)); c = L.Node(3, "c", "single", (4, 3))
    d = L.Node(4, "d", "single", (4, 3))
    i, j, k = L.fresh_symbol(), L.fresh_symbol(), L.fresh_symbol()
    sc = L.Scope(L.Node(9, "n2", "single", (1,), mode="virtual"), 1)
    body = [
        L.Comment("c fwd"),
        L.For(i, 0, 3, [L.For(j, 0, 2, [L.Set(c, (L.It(i), L.It(j)), L.Unop("relu", L.LocalScope(sc, [
            L.SetLocal(sc, L.Const(0.0)),
            L.For(k, 0, 4, [L.SetLocal(sc, L.Ternop("fma", L.Get(a, (L.It(j), L.It(k))), L.Get(b, (L.It(k), L.It(i))),
                                                    L.GetLocal(sc)))])])))])]),
        L.ZeroOut(d),
        L.For(i, 0, 3, [L.For(j, 0, 2, [L.For(k, 0, 4, [L.Set(d, (L.It(i), L.It(j)), L.Ternop(
            "fma", L.Get(a, (L.It(j), L.It(k))), L.Get(b, (L.It(k), L.It(i))), L.Get(d, (L.It(i), L.It(j)))))])])]),
    ]
    return L.Routine("c_fwd", body), (a, b, c, d)


def test_small_contraction_bit_exact():
    # the generated kernels keep the reference's sequential summation order: fp32 bit equality
    r, (a, b, c, d) = _small_contraction()
    rng = np.random.default_rng(0)
    init = {1: rng.standard_normal((3, 5)).astype(np.float32), 2: rng.standard_normal((5, 4)).astype(np.float32)}
    hip, ora = HipRun(r, init), OracleRun(r, init)
    hip.step(); ora.step()
    for n in (c, d):
        assert np.array_equal(hip.get(n).view(np.uint32), ora.get(n).view(np.uint32))
    hip.close()


@pytest.mark.parametrize("inline", [True, False])
def test_moons_mlp_loss_curve(inline):
    w = W.moons_mlp(inline=inline)
    sym = w.statics["batch_n"].sym
    hip, ora = HipRun(w.routine, w.init), OracleRun(w.routine, w.init)
    lh, lo = [], []
    for step in range(100):
        st = {sym: step % w.statics["batch_n"].range}
        hip.step(st); ora.step(st)
        lh.append(float(hip.get(w.nodes["loss"])[0])); lo.append(float(ora.get(w.nodes["loss"])[0]))
    lh, lo = np.array(lh), np.array(lo)
    assert np.max(np.abs(lh - lo)) <= 1e-3, (lh[:5], lo[:5])
    for name in ("w1", "b1", "w2", "b2", "w3"):
        assert rel_err(hip.get(w.nodes[name]), ora.get(w.nodes[name]), "single") <= 1e-3, name
    hip.close()


def test_static_index_range_is_checked():
    from ocannl_amd import backend as B
    w = W.moons_mlp()
    hip = HipRun(w.routine, w.init)
    with pytest.raises(B.User_error):
        hip.step({w.statics["batch_n"].sym: w.statics["batch_n"].range})
    with pytest.raises(B.User_error):
        hip.step({w.statics["batch_n"].sym: -1})
    hip.close()


@pytest.mark.parametrize("prec,out_prec,tol", [("single", "single", 1e-4), ("bfloat16", "single", 2e-2),
                                                ("bfloat16", "bfloat16", 2e-2)])
@pytest.mark.parametrize("order", ["last", "first"])
def test_dense_contraction_mfma_small(prec, out_prec, tol, order):
    w = W.dense_contraction(b=256, i=192, o=128, prec=prec, out_prec=out_prec, reduce_order=order)
    rng = np.random.default_rng(5)
    # gradients accumulate into existing contents
    w.init[w.nodes["dx"].id] = W.as_prec(rng.standard_normal((256, 192)).astype(np.float32), out_prec)
    w.init[w.nodes["dw"].id] = W.as_prec(rng.standard_normal((128, 192)).astype(np.float32), out_prec)
    hip = HipRun(w.routine, w.init, options="min_mfma_flops=1")
    kinds = [k["kind"] for k in hip.code.kernels()]
    assert kinds.count("mfma") == 3, hip.code.kernels()
    ora = OracleRun(w.routine, w.init)
    hip.step(); ora.step()
    for name in ("y", "dx", "dw"):
        got, want = hip.get(w.nodes[name]), ora.get(w.nodes[name])
        if out_prec == "bfloat16":
            # the checker rounds the running sum to bf16 after every step; compare both to fp64
            x = W.to_float(w.init[w.nodes["x"].id], prec); wt = W.to_float(w.init[w.nodes["w"].id], prec)
            dy = W.to_float(w.init[w.nodes["dy"].id], prec)
            exact = {"y": x @ wt.T, "dx": W.to_float(w.init[w.nodes["dx"].id], out_prec) + dy @ wt,
                     "dw": W.to_float(w.init[w.nodes["dw"].id], out_prec) + dy.T @ x}[name]
            scale = np.max(np.abs(exact))
            assert np.max(np.abs(W.to_float(got, out_prec) - exact)) / scale <= tol, name
            assert np.max(np.abs(W.to_float(want, out_prec) - exact)) / scale <= 5 * tol, name
        else:
            assert rel_err(got, want, out_prec) <= tol, name
    hip.close()


@pytest.mark.parametrize("prec,tol", [("bfloat16", 2e-2), ("single", 1e-4)])
def test_dense_contraction_full_size_sampled_rows(prec, tol):
    """Benchmark configuration 3 at full size (b=8192, i=o=4096): too large for the serial checker, so a
    random sample of output rows is recomputed in float64 on the host from the same inputs."""
    b, i, o = 8192, 4096, 4096
    w = W.dense_contraction(b=b, i=i, o=o, prec=prec, out_prec="single")
    hip = HipRun(w.routine, w.init)
    assert [k["kind"] for k in hip.code.kernels()] == ["mfma"] * 3
    hip.step()
    x = W.to_float(w.init[w.nodes["x"].id], prec); wt = W.to_float(w.init[w.nodes["w"].id], prec)
    dy = W.to_float(w.init[w.nodes["dy"].id], prec)
    rng = np.random.default_rng(11)
    rows = np.sort(rng.choice(b, 48, replace=False)); orows = np.sort(rng.choice(o, 48, replace=False))
    y = hip.get(w.nodes["y"]).astype(np.float64)
    want = x[rows] @ wt.T
    assert np.max(np.abs(y[rows] - want)) / np.max(np.abs(want)) <= tol
    dx = hip.get(w.nodes["dx"]).astype(np.float64)
    want = dy[rows] @ wt
    assert np.max(np.abs(dx[rows] - want)) / np.max(np.abs(want)) <= tol
    dw = hip.get(w.nodes["dw"]).astype(np.float64)
    want = dy[:, orows].T @ x
    assert np.max(np.abs(dw[orows] - want)) / np.max(np.abs(want)) <= tol
    # linearity in the accumulating gradients: a second run adds the same amount again
    hip.step()
    dx2 = hip.get(w.nodes["dx"]).astype(np.float64)
    assert np.max(np.abs(dx2[rows] - 2 * dx[rows])) / np.max(np.abs(dx[rows])) <= 1e-5
    hip.close()


@pytest.mark.parametrize("prec,tol", [("single", 1e-4), ("bfloat16", 2e-2)])
def test_split_k_weight_gradient_shape(prec, tol):
    """Small output, long reduction (the dW shape): K is split over workgroups and the partials are
    summed in a fixed order; two runs must agree bit for bit."""
    w = W.dense_contraction(b=4096, i=128, o=128, prec=prec, out_prec="single", which=("dw",), reduce_order="first")
    rng = np.random.default_rng(3)
    w.init[w.nodes["dw"].id] = rng.standard_normal((128, 128)).astype(np.float32)
    hip = HipRun(w.routine, w.init, "min_mfma_flops=1")
    assert [k["kind"] for k in hip.code.kernels()] == ["mfma"]
    hip.step()
    got = hip.get(w.nodes["dw"]).astype(np.float64)
    x = W.to_float(w.init[w.nodes["x"].id], prec); dy = W.to_float(w.init[w.nodes["dy"].id], prec)
    want = w.init[w.nodes["dw"].id].astype(np.float64) + dy.T @ x
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) <= tol
    hip2 = HipRun(w.routine, w.init, "min_mfma_flops=1")
    hip2.step()
    assert np.array_equal(hip2.get(w.nodes["dw"]).view(np.uint32), hip.get(w.nodes["dw"]).view(np.uint32))
    hip.close(); hip2.close()


def test_single_to_bfloat16_bit_exact_on_all_float_classes():
    # the device rounds fp32 -> bf16 in hardware; the checker restates the host's integer rounding
    # (builtins.c:620-627): both must agree on every bit pattern, NaN payloads included
    rng = np.random.default_rng(7)
    n = 1 << 22
    bits = rng.integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32)
    special = np.array([0x00000000, 0x80000000, 0x00000001, 0x007FFFFF, 0x00800000, 0x7F7FFFFF, 0xFF7FFFFF,
                        0x7F800000, 0xFF800000, 0x7FC00000, 0x7FFFFFFF, 0xFFFFFFFF, 0x7F800001, 0x3F808000,
                        0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7F8000, 0x00008000, 0x00018000], np.uint32)
    bits[:special.size] = special
    # every pattern whose low half sits on a rounding boundary, over a sweep of high halves
    hi = (np.arange(1 << 16, dtype=np.uint32) << 16)
    bits[special.size:special.size + (1 << 16)] = hi | 0x8000
    bits[special.size + (1 << 16):special.size + (2 << 16)] = hi | 0x7FFF
    L.reset_symbols(0)
    x = L.Node(1, "x", "single", (n,)); y = L.Node(2, "y", "bfloat16", (n,))
    i = L.fresh_symbol()
    r = L.Routine("to_bf16", [L.For(i, 0, n - 1, [L.Set(y, (L.It(i),), L.Get(x, (L.It(i),)))])])
    init = {1: bits.view(np.float32)}
    hip, ora = HipRun(r, init), OracleRun(r, init)
    hip.step(); ora.step()
    got, want = hip.get(y).view(np.uint16), ora.get(y).view(np.uint16)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(bits[k]), hex(got[k]), hex(want[k])) for k in bad[:8]]
    hip.close()


def test_routine_scope_scalar_locals():
    # arrayjit/test/test_local_scope_init.expected, cases 5 and 6: a Declare_local hoisted to routine
    # scope is written by one statement and read by later ones (kernels of their own here)
    L.reset_symbols(10)
    z = (L.Fixed(0),)
    s3 = L.Node(9, "src3", "single", (1,)); o3 = L.Node(10, "out3", "single", (1,)); o4 = L.Node(11, "out4", "single", (1,))
    s4 = L.Node(12, "src4", "single", (4,)); o5 = L.Node(13, "out5", "single", (1,)); o6 = L.Node(14, "out6", "single", (1,))
    a, b = L.Scope(s3, 30), L.Scope(s4, 40)
    body = [L.DeclareLocal(a, False), L.SetLocal(a, L.Get(s3, z)),
            L.Set(o3, z, L.GetLocal(a)), L.Set(o4, z, L.Binop("mul", L.GetLocal(a), L.Const(2.0))),
            L.DeclareLocal(b, True),
            L.For(4, 0, 3, [L.SetLocal(b, L.Binop("add", L.GetLocal(b), L.Get(s4, (L.It(4),))))]),
            L.Set(o5, z, L.GetLocal(b)), L.Set(o6, z, L.Binop("add", L.GetLocal(b), L.GetLocal(a)))]
    r = L.Routine("hoisted_locals", body)
    init = {9: np.array([1.5], np.float32), 12: np.array([1, 2, 3, 4.25], np.float32)}
    for opts in (None, "serial=0"):
        hip, ora = HipRun(r, init, opts), OracleRun(r, init)
        hip.step(); ora.step()
        for n in (o3, o4, o5, o6):
            assert np.array_equal(hip.get(n), ora.get(n)), n.ident
        assert hip.get(o5)[0] == 10.25 and hip.get(o6)[0] == 11.75
        hip.close()
