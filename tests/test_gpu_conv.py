"""Convolution-style loop nests: axes indexed by sums of loop symbols (`stride * o + k`,
lib/nn_blocks.ml:418-428; projections of tensor/shape.ml with `Affine` indices, indexing.ml:104-120).
Forward, both gradients, a strided max-pool and the patch (stride = window) case where the sum is a
one-to-one map and may be spread over threads."""
import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L
from parity import HipRun, OracleRun

pytestmark = pytest.mark.gpu


def _conv(stride, ksz, prec="single", b=3, oh=6, ow=5, ic=4, oc=8):
    L.reset_symbols(0)
    ih, iw = stride * (oh - 1) + ksz, stride * (ow - 1) + ksz
    x = L.Node(1, "x", prec, (b, ih, iw, ic)); w = L.Node(2, "w", prec, (oc, ksz, ksz, ic))
    y = L.Node(3, "y", prec, (b, oh, ow, oc)); dy = L.Node(4, "y_grad", prec, (b, oh, ow, oc))
    dx = L.Node(5, "x_grad", prec, (b, ih, iw, ic)); dw = L.Node(6, "w_grad", prec, (oc, ksz, ksz, ic))
    pool = L.Node(7, "pool", prec, (b, oh, ow, ic))

    def nest(stmt_of):
        s = [L.fresh_symbol() for _ in range(7)]
        bb, o1, o2, c, k1, k2, i = s
        xi = (L.It(bb), L.Affine(((stride, o1), (1, k1)), 0), L.Affine(((stride, o2), (1, k2)), 0), L.It(i))
        yi = (L.It(bb), L.It(o1), L.It(o2), L.It(c))
        wi = (L.It(c), L.It(k1), L.It(k2), L.It(i))
        body = [stmt_of(xi, yi, wi)]
        for sym, ext in reversed(list(zip(s, (b, oh, ow, oc, ksz, ksz, ic)))):
            body = [L.For(sym, 0, ext - 1, body)]
        return body

    fma = lambda p, q, acc: L.Ternop("fma", p, q, acc)
    body = [L.ZeroOut(y)]
    body += nest(lambda xi, yi, wi: L.Set(y, yi, fma(L.Get(x, xi), L.Get(w, wi), L.Get(y, yi))))
    body += [L.ZeroOut(dx)]
    body += nest(lambda xi, yi, wi: L.Set(dx, xi, fma(L.Get(dy, yi), L.Get(w, wi), L.Get(dx, xi))))
    body += [L.ZeroOut(dw)]
    body += nest(lambda xi, yi, wi: L.Set(dw, wi, fma(L.Get(dy, yi), L.Get(x, xi), L.Get(dw, wi))))
    # max-pool over the same windows, per input channel
    s = [L.fresh_symbol() for _ in range(6)]
    bb, o1, o2, i, k1, k2 = s
    pi = (L.It(bb), L.It(o1), L.It(o2), L.It(i))
    xi = (L.It(bb), L.Affine(((stride, o1), (1, k1)), 0), L.Affine(((stride, o2), (1, k2)), 0), L.It(i))
    pb = [L.Set(pool, pi, L.Binop("max", L.Get(pool, pi), L.Get(x, xi)))]
    for sym, ext in reversed(list(zip(s, (b, oh, ow, ic, ksz, ksz)))):
        pb = [L.For(sym, 0, ext - 1, pb)]
    body += L.loop_over_dims(pool.dims, lambda idcs: [L.Set(pool, idcs, L.Const(float("-inf")))])
    body += pb
    return L.Routine(f"conv_s{stride}_k{ksz}", body), dict(x=x, w=w, y=y, dy=dy, dx=dx, dw=dw, pool=pool)


@pytest.mark.parametrize("stride,ksz", [(1, 3), (2, 3), (2, 2), (3, 2)])
def test_convolution_forward_and_gradients(stride, ksz):
    r, n = _conv(stride, ksz)
    rng = np.random.default_rng(stride * 10 + ksz)
    init = {n[k].id: rng.uniform(-1, 1, n[k].dims).astype(np.float32) for k in ("x", "w", "dy")}
    hip, ora = HipRun(r, init, "mfma=0;coop=0;serial=0"), OracleRun(r, init)
    hip.step(); ora.step()
    for k in ("y", "dx", "dw", "pool"):
        got, want = hip.get(n[k]), ora.get(n[k])
        # same order of accumulation per element as the sequential code: only fused multiply-add
        # contraction by either compiler may differ
        assert np.allclose(got, want, rtol=2e-6, atol=2e-6), k
    assert np.array_equal(hip.get(n["pool"]), ora.get(n["pool"]))
    hip.close()
    # default options (lanes sharing reductions): within the floating-point bar
    hip = HipRun(r, init)
    hip.step()
    for k in ("y", "dx", "dw", "pool"):
        assert np.allclose(hip.get(n[k]), ora.get(n[k]), rtol=1e-4, atol=1e-5), k
    hip.close()


def test_overlapping_windows_are_not_spread_over_threads():
    # stride 1, window 3: positions o + k meet for different (o, k), so the input gradient may only
    # be parallel over axes that are not such sums; stride = window is one-to-one and stays parallel
    for (stride, ksz, expect_spatial) in ((1, 3, False), (2, 2, True)):
        r, n = _conv(stride, ksz)
        src = B.compile(r, "mfma=0;coop=0;serial=0;rows=0").source()
        k = src[src.find("x_grad["):]
        head = src[:src.find("x_grad[" )]
        kernel = head[head.rfind("extern \"C\""):] + k[:k.find("\n}\n")]
        threads = int(__import__("re").search(r"pt_ >= (\d+)ull", kernel).group(1))
        b, ih, iw, ic = n["dx"].dims
        if expect_spatial:
            assert threads > b * ic
        else:
            assert threads == b * ic


def _padded_same_conv(b=2, h=7, w=6, ic=3, oc=5, ksz=3, neutral=0.0):
    L.reset_symbols(0)
    pad = ksz // 2
    padding = ((0, 0), (pad, pad), (pad, pad), (0, 0))
    xp = L.Node(1, "x_padded", "single", (b, h + 2 * pad, w + 2 * pad, ic))
    wt = L.Node(2, "w", "single", (oc, ksz, ksz, ic))
    y = L.Node(3, "y", "single", (b, h, w, oc))
    mp = L.Node(4, "maxpool", "single", (b, h, w, ic))
    body = [L.Comment("reset padding margins of x_padded")]
    body += L.loop_over_padding_region(xp.dims, padding, lambda idcs: [L.Set(xp, idcs, L.Const(neutral))])
    s = [L.fresh_symbol() for _ in range(7)]
    bb, o1, o2, c, k1, k2, i = s
    xi = (L.It(bb), L.Affine(((1, o1), (1, k1)), 0), L.Affine(((1, o2), (1, k2)), 0), L.It(i))
    yi = (L.It(bb), L.It(o1), L.It(o2), L.It(c))
    nest = [L.Set(y, yi, L.Ternop("fma", L.Get(xp, xi), L.Get(wt, (L.It(c), L.It(k1), L.It(k2), L.It(i))), L.Get(y, yi)))]
    for sym, ext in reversed(list(zip(s, (b, h, w, oc, ksz, ksz, ic)))):
        nest = [L.For(sym, 0, ext - 1, nest)]
    body += [L.ZeroOut(y)] + nest
    s = [L.fresh_symbol() for _ in range(6)]
    bb, o1, o2, i, k1, k2 = s
    pi = (L.It(bb), L.It(o1), L.It(o2), L.It(i))
    xi = (L.It(bb), L.Affine(((1, o1), (1, k1)), 0), L.Affine(((1, o2), (1, k2)), 0), L.It(i))
    pb = [L.Set(mp, pi, L.Binop("max", L.Get(mp, pi), L.Get(xp, xi)))]
    for sym, ext in reversed(list(zip(s, (b, h, w, ic, ksz, ksz)))):
        pb = [L.For(sym, 0, ext - 1, pb)]
    body += L.loop_over_dims(mp.dims, lambda idcs: [L.Set(mp, idcs, L.Const(float("-inf")))]) + pb
    return L.Routine("same_conv", body), xp, wt, y, mp, pad


@pytest.mark.parametrize("neutral", [0.0, float("-inf")])
@pytest.mark.parametrize("options", ["mfma=0;coop=0;serial=0", None])
def test_padded_node_margins_are_reset_before_a_same_convolution(neutral, options):
    # the margin of a padded node is reset to the operation's neutral value by loops that visit
    # only the margin (assignments.ml:281-298); accesses carry the left padding as an offset (:202-218)
    r, xp, wt, y, mp, pad = _padded_same_conv(neutral=neutral)
    rng = np.random.default_rng(5)
    xv = rng.uniform(-1, 1, xp.dims).astype(np.float32)      # margins start as garbage
    init = {xp.id: xv, wt.id: rng.uniform(-1, 1, wt.dims).astype(np.float32)}
    hip, ora = HipRun(r, init, options), OracleRun(r, init)
    hip.step(); ora.step()
    got = hip.get(xp)
    assert np.array_equal(got, ora.get(xp))
    assert np.array_equal(got[:, pad:-pad, pad:-pad, :], xv[:, pad:-pad, pad:-pad, :])      # data untouched
    margin = np.ones(xp.dims, bool); margin[:, pad:-pad, pad:-pad, :] = False
    assert np.all(got[margin] == np.float32(neutral))
    assert np.array_equal(hip.get(mp), ora.get(mp))
    if neutral == 0.0:
        assert np.allclose(hip.get(y), ora.get(y), rtol=1e-5, atol=1e-5)
    hip.close()


def test_input_gradient_at_matrix_core_size_with_overlapping_windows():
    # x_grad[b, o1+k1, o2+k2, i] += y_grad * w at a size the matrix-core kernels would take (M, N >= 16,
    # min_mfma_flops=0): the overlapping windows keep it a generated kernel, and the result is the
    # checker's; the one-to-one case (stride = window) may go to the matrix cores and has to agree too
    from test_capi_cpu import _conv_input_gradient
    for stride, ksz in ((1, 3), (3, 3)):
        r, n = _conv_input_gradient(stride, ksz, b=2, oh=8, ow=8, ic=32, oc=32)
        rng = np.random.default_rng(stride)
        init = {n[k].id: rng.uniform(-1, 1, n[k].dims).astype(np.float32) for k in ("w", "dy")}
        ora = OracleRun(r, init)
        ora.step()
        for opts in ("min_mfma_flops=0", "min_mfma_flops=0;mfma=0;coop=0"):
            hip = HipRun(r, init, opts)
            hip.step()
            assert np.allclose(hip.get(n["dx"]), ora.get(n["dx"]), rtol=1e-4, atol=1e-4), (stride, opts)
            hip.close()
