"""Random routines (tests/fuzz_llir.py) through the HIP library and through the CPU checker on the
same inputs: a search for structural mistakes of the planner (a dependence missed when phases are
fused, a stale cached value, a wrong thread mapping), which show as errors of order one. With lanes
not sharing reductions the two sides run the same operations in the same order and differ by fused
multiply-add contraction and the last bits of libm, amplified through a dozen in-place statements;
with the default options summation order changes as well, and an fp32 operand of a contraction
with a bf16 partner is rounded to bf16 for the matrix cores (the bf16 bar applies downstream)."""
import numpy as np
import pytest

from fuzz_llir import Gen
from ocannl_amd import workloads as W
from parity import HipRun, OracleRun

pytestmark = pytest.mark.gpu


def _compare(hip, ora, gen, tol, label):
    for n in hip.routine.param_nodes():
        got = W.to_float(hip.get(n), n.prec)
        want = W.to_float(ora.get(n), n.prec)
        finite = np.abs(want[np.isfinite(want)])
        scale = max(1.0, float(finite.max())) if finite.size else 1.0
        t = max(tol, 2e-2) if n.prec == "bfloat16" else tol
        with np.errstate(invalid="ignore"):
            same = (got == want) | (np.isnan(got) & np.isnan(want))    # equal infinities, NaN on both sides
            diff = np.where(same, 0.0, np.abs(got - want))
        bad = ~(diff <= t * scale)                                     # a NaN on one side only is a mismatch
        assert not bad.any(), (label, gen.seed, n, int(bad.sum()), float(np.nanmax(diff)), scale)


@pytest.mark.parametrize("seed", range(int(__import__("os").environ.get("FUZZ_SEEDS", 24))))
def test_random_single_precision_routines(seed):
    gen = Gen(seed)
    r = gen.routine()
    init = gen.init()
    ora = OracleRun(r, init)
    ora.step(); ora.step()
    for options, tol in (("mfma=0;coop=0", 5e-4), ("serial=0", 5e-4), (None, 5e-4)):
        hip = HipRun(r, init, options)
        hip.step(); hip.step()
        _compare(hip, ora, gen, tol, options)
        hip.close()


@pytest.mark.parametrize("seed", range(1000, 1000 + int(__import__("os").environ.get("FUZZ_SEEDS", 24)) // 2))
def test_random_mixed_precision_routines(seed):
    # bf16 / fp32 / fp64 nodes mixed: every operation is computed in the precision of its destination
    # with bf16 rounded after each one (cc_backend.ml:155-323); sums over a loop go to non-bf16 nodes
    gen = Gen(seed, precs=("single", "single", "bfloat16", "double"))
    r = gen.routine()
    init = gen.init()
    ora = OracleRun(r, init)
    ora.step()
    for options, tol in (("mfma=0;coop=0", 5e-4), (None, 2e-2)):
        hip = HipRun(r, init, options)
        hip.step()
        _compare(hip, ora, gen, tol, options)
        hip.close()


@pytest.mark.parametrize("seed", range(2000, 2000 + int(__import__("os").environ.get("FUZZ_SEEDS", 24))))
def test_random_routines_with_slices_integers_and_locals(seed):
    # adds: slices of a stacked node chosen by a static index (a kernel argument set before each run),
    # loops over part of a range, fixed positions, int32 maps and exact int32 row reductions, values
    # passed through a routine-local vector
    gen = Gen(seed)
    gen.extended = True
    r = gen.routine()
    init = gen.init()
    ora = OracleRun(r, init)
    slots = [{gen.slot.sym: v} if gen.used_static else {} for v in (2, 0)]
    for st in slots:
        ora.step(st)
    for options, tol in (("mfma=0;coop=0", 5e-4), ("serial=0", 5e-4), (None, 5e-4)):
        hip = HipRun(r, init, options)
        for st in slots:
            hip.step(st)
        _compare(hip, ora, gen, tol, options)
        for n in hip.routine.param_nodes():
            if n.prec == "int32":
                assert np.array_equal(hip.get(n), ora.get(n)), (options, seed, n)
        hip.close()


def _random_contraction(seed):
    """c[batch.., m.., n..] (+)= sum_k a[perm(batch, m, k)] * b[perm(batch, n, k)] with one or two
    symbols per class, every tensor's axes in a random order, the loops in a random order."""
    from ocannl_amd import llir as L
    rng = np.random.default_rng(seed)
    L.reset_symbols(0)
    def syms(kind, choices, lo, hi):
        n = int(rng.integers(lo, hi + 1))
        return [(kind, L.fresh_symbol(), int(rng.choice(choices))) for _ in range(n)]
    batch = syms("b", [2, 3, 4], 0, 2)
    ms = syms("m", [8, 24, 50, 128, 200], 1, 2)
    ns = syms("n", [8, 16, 40, 128, 136], 1, 2)
    ks = syms("k", [8, 32, 72, 256], 1, 2)
    ext = lambda xs: int(np.prod([e for _, _, e in xs])) if xs else 1
    # big enough for the matrix cores, small enough for the serial checker
    while 2 * ext(batch) * ext(ms) * ext(ns) * ext(ks) < (1 << 23):
        ks[0] = ("k", ks[0][1], ks[0][2] * 2)
    while ext(batch) * ext(ms) * ext(ns) * ext(ks) > 3e8:
        big = max((batch + ms + ns + ks), key=lambda t: t[2])
        lst = {"b": batch, "m": ms, "n": ns, "k": ks}[big[0]]
        lst[lst.index(big)] = (big[0], big[1], max(2, big[2] // 2))
    structured = bool(rng.random() < 0.75)

    def tensor(ident, name, prec, *classes):
        if structured:
            # the reference's layout rule: batch axes, then output axes, then input axes
            # (tensor/shape.ml:1689-1690), either of the last two groups first (a transposed view in
            # a backprop contraction)
            groups = [list(g) for g in classes]       # (one order per class, shared by all three tensors)
            tail = groups[1:]
            if rng.random() < 0.5:
                tail.reverse()
            order = groups[0] + [t for g in tail for t in g]
        else:
            order = [t for g in classes for t in g]
            rng.shuffle(order)
        return L.Node(ident, name, prec, tuple(e for _, _, e in order)), tuple(L.It(s) for _, s, _ in order), order
    pa, pb = (str(rng.choice(["single", "bfloat16"])) for _ in range(2))
    pc = str(rng.choice(["single", "bfloat16"])) if (pa, pb) == ("bfloat16", "bfloat16") else "single"
    a, ai, ao = tensor(1, "a", pa, batch, ms, ks)
    b, bi, bo = tensor(2, "b", pb, batch, ns, ks)
    c, ci, co = tensor(3, "c", pc, batch, ms, ns)
    loops = batch + ms + ns + ks
    if rng.random() < 0.6:                       # reductions innermost, as projections usually give
        outer = batch + ms + ns
        rng.shuffle(outer)
        loops = outer + ks
    else:
        rng.shuffle(loops)
    body = [L.Set(c, ci, L.Ternop("fma", L.Get(a, ai), L.Get(b, bi), L.Get(c, ci)))]
    for _, s, e in reversed(loops):
        body = [L.For(s, 0, e - 1, body)]
    accumulate = bool(rng.random() < 0.4)
    r = L.Routine(f"contract_{seed}", ([] if accumulate else [L.ZeroOut(c)]) + body)
    letters = {s: chr(ord("a") + k) for k, (_, s, _) in enumerate(batch + ms + ns + ks)}
    spec = ",".join("".join(letters[s] for _, s, _ in o) for o in (ao, bo)) + "->" + "".join(letters[s] for _, s, _ in co)
    return r, (a, b, c), spec, accumulate, structured


@pytest.mark.parametrize("seed", range(3000, 3000 + int(__import__("os").environ.get("FUZZ_SEEDS", 24))))
def test_random_contractions_against_float64(seed):
    # the planner has to sort the symbols into batch / row / column / reduction classes, merge what is
    # contiguous, and hand strides to the matrix-core kernels; numpy's einsum in float64 is the judge
    from ocannl_amd import backend as B
    r, (a, b, c), spec, accumulate, structured = _random_contraction(seed)
    rng = np.random.default_rng(seed + 7)
    val = {n.id: W.as_prec(rng.uniform(-1, 1, n.dims).astype(np.float32), n.prec) for n in (a, b, c)}
    hip = HipRun(r, val)
    kinds = [k["kind"] for k in hip.code.kernels()]
    hip.step()
    f64 = lambda n: W.to_float(val[n.id], n.prec)
    want = np.einsum(spec, f64(a), f64(b)) + (f64(c) if accumulate else 0.0)
    got = W.to_float(hip.get(c), c.prec)
    scale = max(1.0, float(np.abs(want).max()))
    tol = 2e-2 if "bfloat16" in (a.prec, b.prec, c.prec) else 1e-4
    err = float(np.abs(got - want).max())
    if err > tol * scale and c.prec == "bfloat16" and "mfma" not in kinds:
        # a bf16 accumulator rounded after every step (the reference's rule, kept by a generated kernel
        # that walks the reduction in one thread) drifts from the exact sum: the serial checker judges
        ora = OracleRun(r, val)
        ora.step()
        err = float(np.abs(got - W.to_float(ora.get(c), c.prec)).max())
    assert err <= tol * scale, (seed, spec, a, b, c, kinds, err, scale)
    hip.close()
