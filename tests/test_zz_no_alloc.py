"""The entry point that allocates nothing: ocannl_hip_routine_run_static_scratch runs a linked routine
with its scratch memory (routine-local tensors, tensors the planner materialises, the split-K
workspace) in the library's static device array.  Its results have to be those of
ocannl_hip_routine_run, bit for bit, on two calls in a row of which the second is the smaller one
(the array then still holds the first call's contents); a routine that needs more than the array is
refused."""
import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L
from ocannl_amd import workloads as W

pytestmark = pytest.mark.gpu


def _split_k_product(M, N, K, seed):
    """C = A B^T with a long K and a small output (the split-K path: partial tiles in the workspace),
    then a row sum of C into a routine-local vector that feeds the output `s`."""
    L.reset_symbols(0)
    A = L.Node(1, "a", "bfloat16", (M, K)); Bn = L.Node(2, "b", "bfloat16", (N, K))
    C = L.Node(3, "c", "single", (M, N))
    t = L.Node(4, "t", "single", (M,), mode="local")
    s = L.Node(5, "s", "single", (M,))
    m, n, k, i, j, q = (L.fresh_symbol() for _ in range(6))
    body = [
        L.ZeroOut(C),
        L.For(m, 0, M - 1, [L.For(n, 0, N - 1, [L.For(k, 0, K - 1, [L.Set(C, (L.It(m), L.It(n)), L.Ternop(
            "fma", L.Get(A, (L.It(m), L.It(k))), L.Get(Bn, (L.It(n), L.It(k))), L.Get(C, (L.It(m), L.It(n)))))])])]),
        L.ZeroOut(t),
        L.For(i, 0, M - 1, [L.For(j, 0, N - 1, [L.Set(t, (L.It(i),), L.Binop(
            "add", L.Get(t, (L.It(i),)), L.Get(C, (L.It(i), L.It(j)))))])]),
        L.For(q, 0, M - 1, [L.Set(s, (L.It(q),), L.Binop("mul", L.Const(0.5), L.Get(t, (L.It(q),))))]),
    ]
    rng = np.random.default_rng(seed)
    init = {1: W.as_prec(rng.standard_normal(A.dims).astype(np.float32), "bfloat16"),
            2: W.as_prec(rng.standard_normal(Bn.dims).astype(np.float32), "bfloat16")}
    return L.Routine(f"splitk_{M}x{N}x{K}", body), init, (C, s)


def _both_ways(routine, init, outs, options="min_mfma_flops=1"):
    res = []
    for static in (False, True):
        h = B.HipRun(routine, init, options)
        h.step(static_scratch=static)
        res.append([h.get(n).copy() for n in outs])
        h.close()
    return res


def test_static_scratch_run_equals_the_allocating_run_twice_in_a_row():
    big = _split_k_product(128, 256, 8192, seed=1)        # 4 splits x 128 x 256 floats of workspace
    small = _split_k_product(128, 128, 4096, seed=2)      # smaller: runs over the first call's leftovers
    for r, init, outs in (big, small):
        code = B.compile(r, "min_mfma_flops=1")
        assert any(k["kind"] == "mfma" for k in code.kernels())
        ref, got = _both_ways(r, init, outs)
        for a, b in zip(ref, got):
            assert np.array_equal(a, b)
        assert np.any(ref[0] != 0)
    # a training step with routine-local gradients, zero fills and a static index, several steps
    w = W.moons_mlp()
    sym = w.statics["batch_n"].sym
    for opts in (None, "serial=0"):
        runs = [B.HipRun(w.routine, w.init, opts) for _ in range(2)]
        dev = runs[1].ctx.dev
        for step in range(4):
            runs[0].step({sym: step})
            B.await_(dev)
            # the successful path allocates nothing: pool bytes, scratch bytes, live events and
            # routines of the device read the same before and after
            used, info = B.get_used_memory(dev), B.get_debug_info(dev)
            runs[1].step({sym: step}, static_scratch=True)
            B.await_(dev)
            assert B.get_used_memory(dev) == used and B.get_debug_info(dev) == info
        for name in ("loss", "w1", "w2", "w3", "b1"):
            assert np.array_equal(runs[0].get(w.nodes[name]), runs[1].get(w.nodes[name])), name
        for h in runs:
            h.close()


def test_static_scratch_refuses_a_routine_beyond_the_array():
    # a routine-local tensor of 48 MiB: more than the 32 MiB array
    L.reset_symbols(0)
    n = 12 << 20
    x = L.Node(1, "x", "single", (n,)); t = L.Node(2, "t", "single", (n,), mode="local"); y = L.Node(3, "y", "single", (n,))
    i, j = L.fresh_symbol(), L.fresh_symbol()
    r = L.Routine("too_big", [
        L.For(i, 0, n - 1, [L.Set(t, (L.It(i),), L.Binop("mul", L.Const(2.0), L.Get(x, (L.It(i),))))]),
        L.For(j, 0, n - 1, [L.Set(y, (L.It(j),), L.Binop("add", L.Get(t, (L.It(j),)), L.Const(1.0)))])])
    h = B.HipRun(r, {1: np.ones(n, np.float32)}, "rows=0;parallel=0")
    dev = h.ctx.dev
    used = B.get_used_memory(dev)
    with pytest.raises(B.User_error, match="static scratch"):
        h.step(static_scratch=True)
    assert B.get_used_memory(dev) == used
    h.step()                                    # the allocating entry point still runs it
    assert np.all(h.get(y) == 3.0)
    h.close()
