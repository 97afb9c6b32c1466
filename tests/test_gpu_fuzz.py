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
