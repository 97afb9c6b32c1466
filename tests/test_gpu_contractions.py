"""The MFMA contraction kernels against an fp64 recomputation, over every operand layout /
precision / epilogue combination and over ragged, batched and split-K shapes.  The kernels take
their inputs exactly (bf16 operands are exact in fp64; fp32 operands of a bf16 contraction are
rounded to bf16 first, as the kernel does), so the only error is fp32 accumulation order."""
import numpy as np
import pytest

from ocannl_amd import llir as L
from ocannl_amd import workloads as W
from parity import HipRun

pytestmark = pytest.mark.gpu


def _routine(M, N, K, a_prec, b_prec, c_prec, a_kc, b_kc, accumulate, batch=0):
    """C[(z,) m, n] (+)= sum_k A * B with A stored [m][k] (a_kc) or [k][m], B stored [n][k] (b_kc) or [k][n]."""
    L.reset_symbols(0)
    bd = (batch,) if batch else ()
    A = L.Node(1, "a", a_prec, bd + ((M, K) if a_kc else (K, M)))
    B = L.Node(2, "b", b_prec, bd + ((N, K) if b_kc else (K, N)))
    C = L.Node(3, "c", c_prec, bd + (M, N))
    z, m, n, k = (L.fresh_symbol() for _ in range(4))
    zi = (L.It(z),) if batch else ()
    ai = zi + ((L.It(m), L.It(k)) if a_kc else (L.It(k), L.It(m)))
    bi = zi + ((L.It(n), L.It(k)) if b_kc else (L.It(k), L.It(n)))
    ci = zi + (L.It(m), L.It(n))
    nest = L.For(m, 0, M - 1, [L.For(n, 0, N - 1, [L.For(k, 0, K - 1, [
        L.Set(C, ci, L.Ternop("fma", L.Get(A, ai), L.Get(B, bi), L.Get(C, ci)))])])])
    if batch:
        nest = L.For(z, 0, batch - 1, [nest])
    body = ([] if accumulate else [L.ZeroOut(C)]) + [nest]
    return L.Routine("contract", body), A, B, C


def _check(M, N, K, a_prec, b_prec, c_prec, a_kc, b_kc, accumulate, batch=0, seed=0, copies=True):
    r, A, B, C = _routine(M, N, K, a_prec, b_prec, c_prec, a_kc, b_kc, accumulate, batch)
    rng = np.random.default_rng(seed)
    av = rng.standard_normal(A.dims).astype(np.float32); bv = rng.standard_normal(B.dims).astype(np.float32)
    cv = rng.standard_normal(C.dims).astype(np.float32)
    init = {1: W.as_prec(av, a_prec), 2: W.as_prec(bv, b_prec), 3: W.as_prec(cv, c_prec)}
    hip = HipRun(r, init, "min_mfma_flops=1" + ("" if copies else ";bf16_copies=0"))
    ks = hip.code.kernels()
    mixed = copies and (a_prec == "single") != (b_prec == "single")
    # (a contraction with one fp32 operand gets a pass that rounds that operand to bf16 first)
    assert [k["kind"] for k in ks] == (["generated", "mfma"] if mixed else ["mfma"]), ks
    hip.step()
    got = W.to_float(hip.get(C), c_prec).astype(np.float64)
    bf16_compute = not (a_prec == "single" and b_prec == "single")
    a64 = W.to_float(W.as_prec(av, "bfloat16" if bf16_compute else a_prec), "bfloat16" if bf16_compute else a_prec).astype(np.float64)
    b64 = W.to_float(W.as_prec(bv, "bfloat16" if bf16_compute else b_prec), "bfloat16" if bf16_compute else b_prec).astype(np.float64)
    if not a_kc: a64 = np.swapaxes(a64, -1, -2)
    if not b_kc: b64 = np.swapaxes(b64, -1, -2)
    want = a64 @ np.swapaxes(b64, -1, -2)
    if accumulate:
        want = want + W.to_float(init[3], c_prec).astype(np.float64)
    scale = np.max(np.abs(want))
    err = np.max(np.abs(got - want)) / scale
    tol = 2.0 ** -8 if c_prec == "bfloat16" else 2e-6 * max(1.0, np.sqrt(K) / 8)
    assert err <= tol, (err, tol, ks[-1]["name"])
    hip.close()
    return ks[-1]["name"]


@pytest.mark.parametrize("a_kc", [True, False])
@pytest.mark.parametrize("b_kc", [True, False])
@pytest.mark.parametrize("precs", [("bfloat16", "bfloat16", "single"), ("bfloat16", "bfloat16", "bfloat16"),
                                   ("single", "bfloat16", "single"), ("bfloat16", "single", "single"),
                                   ("single", "single", "single")])
@pytest.mark.parametrize("accumulate", [False, True])
def test_layouts_precisions_epilogues_on_a_ragged_shape(a_kc, b_kc, precs, accumulate):
    # 136 x 72 x 200: no extent is a multiple of the tile or of the K stage; contiguous extents are
    # multiples of 8 as the planner requires
    name = _check(136, 72, 200, precs[0], precs[1], precs[2], a_kc, b_kc, accumulate)
    assert ("gemm_f32" in name) == (precs[0] == "single" and precs[1] == "single")


@pytest.mark.parametrize("a_kc", [True, False])
@pytest.mark.parametrize("b_kc", [True, False])
@pytest.mark.parametrize("which", ["a", "b"])
def test_fp32_operand_rounded_inside_the_kernel(a_kc, b_kc, which):
    # without the bf16 scratch copy the kernel itself rounds the fp32 operand on the way into LDS
    precs = ("single", "bfloat16") if which == "a" else ("bfloat16", "single")
    name = _check(264, 136, 328, precs[0], precs[1], "single", a_kc, b_kc, True, seed=6, copies=False)
    assert "float" in name
    _check(1024, 1024, 512, precs[0], precs[1], "bfloat16", a_kc, b_kc, False, seed=7, copies=False)


@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 256, 64), (264, 520, 72), (1000, 24, 1032), (512, 384, 1024),
                                   (2048, 1024, 512)])
@pytest.mark.parametrize("layout", [(True, True), (True, False), (False, False)])
def test_shapes_full_and_ragged_tiles(shape, layout):
    M, N, K = shape
    _check(M, N, K, "bfloat16", "bfloat16", "single", layout[0], layout[1], True, seed=1)


@pytest.mark.parametrize("layout", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("c_prec", ["single", "bfloat16"])
def test_split_k(layout, c_prec):
    # small output, long K: split over workgroups, partial tiles summed in index order
    _check(128, 256, 8192, "bfloat16", "bfloat16", c_prec, layout[0], layout[1], True, seed=2)
    _check(72, 136, 4096, "single", "bfloat16", c_prec, layout[0], layout[1], False, seed=3)


@pytest.mark.parametrize("layout", [(True, True), (True, False), (False, True)])
def test_batched(layout):
    _check(136, 64, 72, "bfloat16", "bfloat16", "single", layout[0], layout[1], False, batch=12, seed=4)
    _check(256, 256, 64, "single", "bfloat16", "single", layout[0], layout[1], True, batch=16, seed=5)


def test_split_k_is_deterministic():
    r, A, B, C = _routine(128, 128, 8192, "bfloat16", "bfloat16", "single", False, False, False)
    rng = np.random.default_rng(9)
    init = {1: W.as_prec(rng.standard_normal(A.dims).astype(np.float32), "bfloat16"),
            2: W.as_prec(rng.standard_normal(B.dims).astype(np.float32), "bfloat16")}
    outs = []
    for _ in range(3):
        hip = HipRun(r, init, "min_mfma_flops=1")
        hip.step(); hip.step()
        outs.append(hip.get(C).copy())
        hip.close()
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


@pytest.mark.parametrize("prec", ["single", "bfloat16"])
def test_operands_sliced_by_static_and_fixed_indices(prec):
    # c[s2, m, n] = sum_k a[s1, m, k] * b[3, k, n]: one operand slice is chosen at run time by a
    # static index (a kernel-launch argument folded into the operand's base address), one by a fixed
    # position, and the result goes to a run-time slice too
    S, M, N, K = 4, 192, 160, 256
    L.reset_symbols(0)
    A = L.Node(1, "a", prec, (S, M, K)); B = L.Node(2, "b", prec, (5, K, N)); C = L.Node(3, "c", "single", (S, M, N))
    s1, s2 = L.StaticSymbol(L.fresh_symbol(), S), L.StaticSymbol(L.fresh_symbol(), S)
    m, n, k = (L.fresh_symbol() for _ in range(3))
    ci = (L.It(s2.sym), L.It(m), L.It(n))
    nest = L.For(m, 0, M - 1, [L.For(n, 0, N - 1, [L.For(k, 0, K - 1, [L.Set(C, ci, L.Ternop(
        "fma", L.Get(A, (L.It(s1.sym), L.It(m), L.It(k))), L.Get(B, (L.Fixed(3), L.It(k), L.It(n))), L.Get(C, ci)))])])])
    r = L.Routine("sliced", [nest], static_indices=[s1, s2])
    rng = np.random.default_rng(2)
    av, bv = (rng.standard_normal(x.dims).astype(np.float32) for x in (A, B))
    init = {1: W.as_prec(av, prec), 2: W.as_prec(bv, prec)}
    hip = HipRun(r, init, "min_mfma_flops=1")
    assert [k["kind"] for k in hip.code.kernels()] == ["mfma"]
    a64, b64 = W.to_float(init[1], prec).astype(np.float64), W.to_float(init[2], prec).astype(np.float64)
    want = np.zeros(C.dims)
    for va, vc in ((0, 1), (3, 1), (2, 0)):          # accumulates: slice 1 of c receives two products
        hip.step({s1.sym: va, s2.sym: vc})
        want[vc] += a64[va] @ b64[3]
    got = hip.get(C).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
    assert not got[2:].any()
    with pytest.raises(hip.B.User_error):
        hip.step({s1.sym: S, s2.sym: 0})             # out of range: refused before anything is enqueued
    hip.close()


def _product_nest(A, B, C, M, N, K, a_kc, b_kc):
    m, n, k = (L.fresh_symbol() for _ in range(3))
    ai = (L.It(m), L.It(k)) if a_kc else (L.It(k), L.It(m))
    bi = (L.It(n), L.It(k)) if b_kc else (L.It(k), L.It(n))
    ci = (L.It(m), L.It(n))
    return L.For(m, 0, M - 1, [L.For(n, 0, N - 1, [L.For(k, 0, K - 1, [
        L.Set(C, ci, L.Ternop("fma", L.Get(A, ai), L.Get(B, bi), L.Get(C, ci)))])])])


def _f64(x, prec, kc):
    v = W.to_float(x, prec).astype(np.float64)
    return v if kc else v.T


@pytest.mark.parametrize("shape", [(256, 384, 512), (136, 72, 200), (128, 128, 4096), (512, 256, 256)])
@pytest.mark.parametrize("layout", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("precs", [("bfloat16", "single", True), ("bfloat16", "bfloat16", False), ("single", "single", False)])
@pytest.mark.parametrize("members", [2, 3, 4])
def test_independent_products_of_one_shape_share_a_launch(shape, layout, precs, members):
    # y_g (+)= x w_g for two to four weights, with a pointwise statement on an unrelated tensor in
    # between.  (Two or four members whose tile count allows it each keep to XCDs of their own: the
    # workgroup -> member / tile mapping differs from the plain one.)
    M, N, K = shape
    a_kc, b_kc = layout
    prec, c_prec, accumulate = precs
    G = members
    L.reset_symbols(0)
    X = L.Node(1, "x", prec, (M, K) if a_kc else (K, M))
    Ws = [L.Node(2 + g, f"w{g}", prec, (N, K) if b_kc else (K, N)) for g in range(G)]
    Ys = [L.Node(6 + g, f"y{g}", c_prec, (M, N)) for g in range(G)]
    U = L.Node(10, "u", "single", (64,))
    i = L.fresh_symbol()
    bump = L.For(i, 0, 63, [L.Set(U, (L.It(i),), L.Binop("add", L.Get(U, (L.It(i),)), L.Const(1.0)))])
    body = []
    for g in range(G):
        if not accumulate:
            body.append(L.ZeroOut(Ys[g]))
        body.append(_product_nest(X, Ws[g], Ys[g], M, N, K, a_kc, b_kc))
        if g == 0:
            body.append(bump)
    r = L.Routine("group", body)
    rng = np.random.default_rng(12)
    init = {x.id: W.as_prec(rng.standard_normal(x.dims).astype(np.float32), x.prec) for x in [X] + Ws + Ys}
    init[U.id] = np.zeros(64, np.float32)
    x64 = _f64(init[X.id], prec, a_kc)
    outs = {}
    for opts, launches in (("min_mfma_flops=1", 1), ("min_mfma_flops=1;groups=0", G)):
        hip = HipRun(r, init, opts)
        ks = hip.code.kernels()
        assert sorted(k["kind"] for k in ks) == ["generated"] + ["mfma"] * launches, ks
        hip.step()
        outs[launches] = [W.to_float(hip.get(y), c_prec).astype(np.float64) for y in Ys]
        assert np.array_equal(hip.get(U), np.ones(64, np.float32))
        hip.close()
    tol = 2.0 ** -8 if c_prec == "bfloat16" else 2e-6 * max(1.0, np.sqrt(K) / 8)
    for g in range(G):
        want = x64 @ _f64(init[Ws[g].id], prec, b_kc).T
        if accumulate:
            want = want + W.to_float(init[Ys[g].id], c_prec).astype(np.float64)
        for got in outs.values():
            assert np.max(np.abs(got[g] - want)) <= tol * np.max(np.abs(want)), (g, layout, precs)
    # grouped and separate launches sum in the same order: identical bits
    for g in range(G):
        assert np.array_equal(outs[1][g], outs[G][g])


def test_a_product_that_reads_another_products_result_is_not_grouped_with_it():
    M = N = K = 256
    L.reset_symbols(0)
    X = L.Node(1, "x", "bfloat16", (M, K)); W0 = L.Node(2, "w0", "bfloat16", (N, K)); W1 = L.Node(3, "w1", "bfloat16", (N, K))
    Y = L.Node(4, "y", "bfloat16", (M, N)); Z = L.Node(5, "z", "bfloat16", (M, N))
    body = [L.ZeroOut(Y), _product_nest(X, W0, Y, M, N, K, True, True), L.ZeroOut(Z), _product_nest(Y, W1, Z, M, N, K, True, True)]
    r = L.Routine("dependent", body)
    rng = np.random.default_rng(13)
    init = {x.id: W.as_prec(rng.standard_normal(x.dims).astype(np.float32) / 16, "bfloat16") for x in (X, W0, W1)}
    hip = HipRun(r, init, "min_mfma_flops=1")
    assert [k["kind"] for k in hip.code.kernels()] == ["mfma", "mfma"]
    hip.step()
    y = W.to_float(hip.get(Y), "bfloat16").astype(np.float64)
    want = y @ W.to_float(init[3], "bfloat16").astype(np.float64).T
    got = W.to_float(hip.get(Z), "bfloat16").astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2.0 ** -7 * np.max(np.abs(want))
    hip.close()


@pytest.mark.parametrize("shape", [(256, 256, 512), (136, 72, 200), (128, 128, 8192)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_producer_epilogue_writes_the_bf16_copy_its_consumer_reads(shape, accumulate):
    # g (fp32) (+)= a b, then out = g w with bf16 w: the second contraction wants g in bf16, and the
    # first one's epilogue (or its split-K reduction pass) writes that copy -- no conversion pass.
    M, N, K = shape
    L.reset_symbols(0)
    A = L.Node(1, "a", "bfloat16", (M, K)); B = L.Node(2, "b", "bfloat16", (N, K)); G = L.Node(3, "g", "single", (M, N))
    Wt = L.Node(4, "w", "bfloat16", (64, N)); Out = L.Node(5, "out", "single", (M, 64))
    body = ([] if accumulate else [L.ZeroOut(G)]) + [_product_nest(A, B, G, M, N, K, True, True),
                                                     L.ZeroOut(Out), _product_nest(G, Wt, Out, M, 64, N, True, True)]
    r = L.Routine("producer_copy", body)
    rng = np.random.default_rng(21)
    init = {x.id: W.as_prec(rng.standard_normal(x.dims).astype(np.float32) / 4, x.prec) for x in (A, B, G, Wt)}
    hip = HipRun(r, init, "min_mfma_flops=1")
    assert [k["kind"] for k in hip.code.kernels()] == ["mfma", "mfma"], hip.code.kernels()
    hip.step()
    g = hip.get(G).astype(np.float64)
    want_g = _f64(init[1], "bfloat16", True) @ _f64(init[2], "bfloat16", True).T + (init[3].astype(np.float64) if accumulate else 0.0)
    assert np.max(np.abs(g - want_g)) <= 2e-6 * max(1.0, np.sqrt(K) / 8) * np.max(np.abs(want_g))
    g_bf = W.to_float(W.as_prec(hip.get(G), "bfloat16"), "bfloat16").astype(np.float64)   # the copy: g as stored, rounded
    want = g_bf @ _f64(init[4], "bfloat16", True).T
    got = hip.get(Out).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2e-6 * max(1.0, np.sqrt(N) / 8) * np.max(np.abs(want))
    hip.close()


@pytest.mark.parametrize("shape", [(256, 384, 512), (136, 72, 200), (128, 128, 4096)])
@pytest.mark.parametrize("layout", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_chain_of_products_into_one_result_is_one_launch(shape, layout, accumulate):
    # c (+)= a0 b0; c =+ a1 b1; c =+ a2 b2 (the gradient of a tensor that feeds three projections),
    # with a pointwise statement on an unrelated tensor in between: one launch runs K over the three
    # operand pairs and touches c once; full, ragged and split-K shapes
    M, N, K = shape
    a_kc, b_kc = layout
    L.reset_symbols(0)
    As = [L.Node(1 + p, f"a{p}", "bfloat16", (M, K) if a_kc else (K, M)) for p in range(3)]
    Bs = [L.Node(4 + p, f"b{p}", "bfloat16", (N, K) if b_kc else (K, N)) for p in range(3)]
    C = L.Node(7, "c", "single", (M, N)); U = L.Node(8, "u", "single", (64,))
    i = L.fresh_symbol()
    bump = L.For(i, 0, 63, [L.Set(U, (L.It(i),), L.Binop("add", L.Get(U, (L.It(i),)), L.Const(1.0)))])
    body = ([] if accumulate else [L.ZeroOut(C)]) + [_product_nest(As[0], Bs[0], C, M, N, K, a_kc, b_kc), bump] + \
        [_product_nest(As[p], Bs[p], C, M, N, K, a_kc, b_kc) for p in (1, 2)]
    r = L.Routine("chain", body)
    rng = np.random.default_rng(11)
    init = {x.id: W.as_prec(rng.standard_normal(x.dims).astype(np.float32), "bfloat16") for x in As + Bs}
    init[C.id] = rng.standard_normal(C.dims).astype(np.float32)
    init[U.id] = np.zeros(64, np.float32)
    want = sum(_f64(init[As[p].id], "bfloat16", a_kc) @ _f64(init[Bs[p].id], "bfloat16", b_kc).T for p in range(3))
    if accumulate:
        want = want + init[C.id].astype(np.float64)
    for opts, launches in (("min_mfma_flops=1", 1), ("min_mfma_flops=1;chains=0", 3)):
        hip = HipRun(r, init, opts)
        ks = hip.code.kernels()
        assert sorted(k["kind"] for k in ks) == ["generated"] + ["mfma"] * launches, ks
        if launches == 1:
            mf = [k for k in ks if k["kind"] == "mfma"][0]
            assert mf["k"] == 3 * K and mf["flops"] == 6.0 * M * N * K and mf["name"].endswith("2, true>")
        hip.step()
        got = hip.get(C).astype(np.float64)
        assert np.max(np.abs(got - want)) <= 2e-6 * max(1.0, np.sqrt(3 * K) / 8) * np.max(np.abs(want)), launches
        assert np.array_equal(hip.get(U), np.ones(64, np.float32))
        hip.close()


def test_operand_rewritten_between_two_products_is_not_read_from_a_stale_copy():
    from test_capi_cpu import _stale_copy_routine
    r, n = _stale_copy_routine()
    rng = np.random.default_rng(21)
    xv = rng.uniform(-1, 1, n["x"].dims).astype(np.float32)
    wv = W.to_bf16_bits(rng.uniform(-1, 1, n["w"].dims).astype(np.float32))
    init = {n["x"].id: xv, n["w"].id: wv, n["u"].id: rng.uniform(-1, 1, n["u"].dims).astype(np.float32)}
    hip = HipRun(r, init, "min_mfma_flops=0")
    hip.step()
    wf = W.from_bf16_bits(wv).astype(np.float64)
    xb = W.from_bf16_bits(W.to_bf16_bits(xv)).astype(np.float64)
    c1, c2 = hip.get(n["c1"]).astype(np.float64), hip.get(n["c2"]).astype(np.float64)
    assert np.allclose(c1, xb @ wf.T, rtol=1e-4, atol=1e-4)
    assert np.allclose(c2, 2.0 * (xb @ wf.T), rtol=1e-4, atol=1e-4)       # (doubling commutes with rounding)
    assert np.allclose(hip.get(n["y1"]), init[n["u"].id].sum(1), rtol=1e-4, atol=1e-4)
    hip.close()


@pytest.mark.parametrize("copies", [True, False])
def test_mixed_precision_product_against_the_reference_semantics(copies):
    # The serial C code widens the bf16 operand and multiplies in fp32 with the fp32 operand exact
    # (arrayjit/lib/cc_backend.ml:171-186); the matrix-core kernel rounds the fp32 operand to bf16
    # first (in a copy pass, or on the way into LDS).  This measures that deviation against the checker
    # itself, not against a model of the kernel: it has to stay inside the 2e-2 bar for bf16 work.
    from parity import OracleRun
    r, A, B, C = _routine(192, 128, 256, "single", "bfloat16", "single", True, True, False)
    rng = np.random.default_rng(31)
    init = {1: rng.standard_normal(A.dims).astype(np.float32),
            2: W.as_prec(rng.standard_normal(B.dims).astype(np.float32), "bfloat16")}
    ora = OracleRun(r, init)
    hip = HipRun(r, init, "min_mfma_flops=1" + ("" if copies else ";bf16_copies=0"))
    assert any(k["kind"] == "mfma" for k in hip.code.kernels())
    ora.step(); hip.step()
    want, got = ora.get(C).astype(np.float64), hip.get(C).astype(np.float64)
    err = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    print(f"fp32 x bf16 product: relative Frobenius error against the serial fp32-operand semantics {err:.2e}")
    assert 1e-4 < err <= 2e-2      # a real deviation (one bf16 rounding of an operand), well inside the bar
    hip.close()


@pytest.mark.parametrize("shape", [(256, 384, 128), (136, 72, 200), (1024, 2048, 512)])
def test_bias_and_relu_consumers_folded_into_the_epilogue(shape):
    # an mlp layer as the optimiser hands it over: y[b, o] := (the inlined product w x) + bias[o];
    # z := relu(y).  By default the contraction's epilogue stores y and z itself (`epilogues=0`: the
    # product goes to scratch and two pointwise statements follow).  Same roundings in the same order:
    # bit for bit the same y and z, on full tiles (16-byte stores) and ragged ones.
    from ocannl_amd.frontend import Graph, make_routine
    from ocannl_amd import backend as B
    Bn, O, I = shape
    L.reset_symbols(0)
    g = Graph("bfloat16", "single")
    x = g.input("x", ("b", "i"), (Bn, I)); w = g.param("w", ("o", "i"), (O, I)); bias = g.param("bias", ("o",), (O,))
    y = g.add(g.einsum(w, x, ("b", "o"), ident="wx"), bias, ("b", "o"), ident="y")
    z = g.unary("relu", y, ident="z")
    r = make_routine(g, "mlp_layer", g.forward(z), outputs=[y.value, z.value])
    rng = np.random.default_rng(Bn)
    init = {x.value.id: W.as_prec(rng.standard_normal((Bn, I)).astype(np.float32), "bfloat16"),
            w.value.id: W.as_prec((rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32), "bfloat16"),
            bias.value.id: W.as_prec(rng.standard_normal(O).astype(np.float32), "bfloat16")}
    folded, apart = HipRun(r, init, "min_mfma_flops=1"), HipRun(r, init, "min_mfma_flops=1;epilogues=0;fused=0")
    kf, ka = folded.code.kernels(), apart.code.kernels()
    assert [k["kind"] for k in kf] == ["mfma"] and len(ka) > 1, (kf, ka)
    folded.step(); apart.step()
    yf, zf = folded.get(y.value), folded.get(z.value)
    assert np.array_equal(yf, apart.get(y.value)) and np.array_equal(zf, apart.get(z.value))
    # (with a contracted extent of at most 128 the third form exists too: the product as the prologue of
    # the row-wise kernel that adds the bias and applies relu)
    third = HipRun(r, init, "min_mfma_flops=1;epilogues=0")
    if [k["kind"] for k in third.code.kernels()] == ["generated"]:
        third.step()
        assert np.array_equal(yf, third.get(y.value)) and np.array_equal(zf, third.get(z.value))
    third.close()
    # and against the mathematics: relu(w x + bias) in float64 from the same bf16 inputs
    want = W.to_float(init[x.value.id], "bfloat16") @ W.to_float(init[w.value.id], "bfloat16").T + W.to_float(init[bias.value.id], "bfloat16")
    assert np.max(np.abs(W.to_float(yf, "bfloat16") - want)) <= 2.0 ** -7 * np.max(np.abs(want))
    assert np.array_equal(W.to_float(zf, "bfloat16"), np.maximum(W.to_float(yf, "bfloat16"), 0.0))
    assert np.any(W.to_float(zf, "bfloat16") > 0) and np.any(W.to_float(yf, "bfloat16") < 0)
    folded.close(); apart.close()


@pytest.mark.parametrize("shape", [(256, 384, 128), (136, 72, 200), (1024, 2048, 512)])
def test_relu_of_the_biased_product_in_one_statement_is_folded_too(shape):
    # the same layer as the reference's visit rule hands it over when z is the only reader of y:
    # z := relu(the inlined product + bias[o]) in ONE statement (low_level.ml:496-552).  The epilogue then
    # stores relu of the biased, rounded result as C and nothing else: bit for bit what the statement
    # computes from the product kept in scratch, and what the two-statement form stores as z.
    from ocannl_amd.frontend import Graph, make_routine
    Bn, O, I = shape
    def build(inline):
        L.reset_symbols(0)
        g = Graph("bfloat16", "single")
        x = g.input("x", ("b", "i"), (Bn, I)); w = g.param("w", ("o", "i"), (O, I)); bias = g.param("bias", ("o",), (O,))
        y = g.add(g.einsum(w, x, ("b", "o"), ident="wx"), bias, ("b", "o"), ident="y")
        z = g.unary("relu", y, ident="z")
        outs = [z.value] if inline else [y.value, z.value]
        r = make_routine(g, "mlp_layer", g.forward(z), outputs=outs, **({"inline": "visits"} if inline else {}))
        return r, x, w, bias, y, z
    r, x, w, bias, y, z = build(True)
    assert all(n.id != y.value.id or n.mode == "virtual" for n in r.nodes()), "the harness did not inline y: the test would not reach the fold"
    rng = np.random.default_rng(Bn)
    init = {x.value.id: W.as_prec(rng.standard_normal((Bn, I)).astype(np.float32), "bfloat16"),
            w.value.id: W.as_prec((rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32), "bfloat16"),
            bias.value.id: W.as_prec(rng.standard_normal(O).astype(np.float32), "bfloat16")}
    folded, apart = HipRun(r, init, "min_mfma_flops=1"), HipRun(r, init, "min_mfma_flops=1;epilogues=0;fused=0")
    kf, ka = folded.code.kernels(), apart.code.kernels()
    assert [k["kind"] for k in kf] == ["mfma"] and len(ka) > 1, (kf, ka)
    folded.step(); apart.step()
    zf = folded.get(z.value)
    assert np.array_equal(zf, apart.get(z.value))
    from parity import OracleRun
    ora = OracleRun(r, init); ora.step()
    # (the checker adds the products one by one in bf16, the matrix cores in fp32: the bar is the relative
    # Frobenius error, as for the other bf16 contractions)
    want, got = W.to_float(ora.get(z.value), "bfloat16").astype(np.float64), W.to_float(zf, "bfloat16").astype(np.float64)
    assert np.linalg.norm(got - want) <= 2e-2 * np.linalg.norm(want)
    r2, x2, w2, bias2, y2, z2 = build(False)
    two = HipRun(r2, {x2.value.id: init[x.value.id], w2.value.id: init[w.value.id], bias2.value.id: init[bias.value.id]}, "min_mfma_flops=1")
    two.step()
    assert np.array_equal(zf, two.get(z2.value))
    assert np.any(W.to_float(zf, "bfloat16") > 0) and np.any(W.to_float(zf, "bfloat16") == 0)
    folded.close(); apart.close(); two.close()
