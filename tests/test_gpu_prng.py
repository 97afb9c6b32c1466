"""Parameter initialisation kernels (threefry4x32 + uniform conversion): integer work, so the bar
is bit equality with the CPU checker, plus the reference's own known answers."""
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN
from ocannl_amd import llir as L
from parity import HipRun, OracleRun

pytestmark = pytest.mark.gpu


def _uniform_vec_routine(n, prec, length):
    # test/operations/n3_fwd_with_prec-unoptimized.ll.expected after inlining: one Set_from_vec per
    # counter, key = Constant_bits 42, counter = the loop index
    L.reset_symbols(0)
    out = L.Node(1, "n3", prec, (n * length,))
    u4 = L.Node(2, "bits", "uint4x32", (1,), mode="virtual")
    i = L.fresh_symbol()
    bits = L.Binop("threefry4x32_light", L.ConstBits(42), L.EmbedIndex(L.It(i)))
    body = [L.For(i, 0, n - 1, [L.SetFromVec(out, (L.Affine(((length, i),), 0),), length,
                                              "uint4x32_to_prec_uniform", bits, "uint4x32")])]
    del u4
    return L.Routine("n3_fwd", body), out


def test_uniform_vec_single_known_answers():
    with open(os.path.join(GOLDEN, "kat.json")) as f:
        kat = json.load(f)
    r, out = _uniform_vec_routine(10, "single", 4)
    hip, ora = HipRun(r, {}), OracleRun(r, {})
    hip.step(); ora.step()
    got = hip.get(out)
    assert np.array_equal(got.view(np.uint32), ora.get(out).view(np.uint32))
    want = kat["threefry_light_key42_single_uniform_first5"]
    assert [float("%.4g" % v) for v in got[:5]] == want
    assert ((got >= 0) & (got < 1)).all()
    hip.close()


def test_uniform_vec_of_a_tensor_id_known_answer():
    # test/operations/test_vec_simple.ml: the key is the tensor's own id (a Constant_bits,
    # arrayjit/lib/assignments.ml:793-796; 1 in that program), the counter the constant 42; the four
    # single-precision numbers of test_vec_simple.expected:4-7
    with open(os.path.join(GOLDEN, "kat.json")) as f:
        want = json.load(f)["threefry_light_selfid1_key42_single_uniform_vec4"]
    L.reset_symbols(0)
    out = L.Node(1, "uniform_floats", "single", (4,))
    bits = L.Binop("threefry4x32_light", L.ConstBits(1), L.ConstBits(42))
    r = L.Routine("vec_simple", [L.SetFromVec(out, (L.Fixed(0),), 4, "uint4x32_to_prec_uniform", bits, "uint4x32")])
    hip, ora = HipRun(r, {}), OracleRun(r, {})
    hip.step(); ora.step()
    got = hip.get(out)
    assert np.array_equal(got.view(np.uint32), ora.get(out).view(np.uint32))
    assert [float("%.4g" % v) for v in got] == want
    hip.close()


@pytest.mark.parametrize("prec,length", [("half", 8), ("bfloat16", 8), ("double", 2), ("uint32", 4), ("byte", 16)])
def test_uniform_vec_other_precisions_bit_exact(prec, length):
    r, out = _uniform_vec_routine(64, prec, length)
    hip, ora = HipRun(r, {}), OracleRun(r, {})
    hip.step(); ora.step()
    g, w = hip.get(out), ora.get(out)
    assert np.array_equal(g.view(np.uint8), w.view(np.uint8))
    if prec == "half":
        with open(os.path.join(GOLDEN, "kat.json")) as f:
            want = json.load(f)["threefry_light_key42_half_uniform_vec_40"]
        assert np.max(np.abs(g[:40].astype(np.float64) - np.array(want))) < 0.01
    hip.close()


@pytest.mark.parametrize("variant", ["threefry4x32_light", "threefry4x32_crypto"])
def test_param_init_uniform1(variant):
    # tensor/operation.ml:720-737: p = 0.5 * (uniform1(threefry(threefry(self_id, seed), offset)) - 0.5)
    L.reset_symbols(0)
    w = L.Node(1, "w", "single", (37, 53))
    i, j = L.fresh_symbol(), L.fresh_symbol()
    key = L.Binop(variant, L.ConstBits(7), L.ConstBits(42))
    bits = L.Binop(variant, key, L.EmbedIndex(L.Affine(((53, i), (1, j)), 0)))
    u = L.Unop("uint4x32_to_prec_uniform1", bits, "uint4x32")
    val = L.Binop("mul", L.Const(0.5), L.Binop("sub", u, L.Const(0.5)))
    r = L.Routine("init_w", [L.For(i, 0, 36, [L.For(j, 0, 52, [L.Set(w, (L.It(i), L.It(j)), val)])])])
    hip, ora = HipRun(r, {}), OracleRun(r, {})
    hip.step(); ora.step()
    g, o = hip.get(w), ora.get(w)
    assert np.array_equal(g.view(np.uint32), o.view(np.uint32))
    assert g.min() >= -0.25 and g.max() < 0.25 and abs(float(g.mean())) < 0.02
    hip.close()


@pytest.mark.parametrize("prec,length", [("single", 4), ("bfloat16", 8)])
def test_vectorised_init_of_a_matrix_through_sub_axis_indices(prec, length):
    # a 2-D parameter filled by the vectorised initialiser (assignments.ml:684-763): one loop over the
    # counters, the last axis indexed `length * i` across row boundaries, the row axis `Sub_axis`
    # (indexing.ml:116: spanned by the adjacent index, nothing of its own in the offset)
    rows, cols = 12, 10
    n = rows * cols // length
    L.reset_symbols(0)
    out = L.Node(1, "w", prec, (rows, cols))
    i = L.fresh_symbol()
    bits = L.Binop("threefry4x32_light", L.ConstBits(7), L.EmbedIndex(L.It(i)))
    r = L.Routine("init_w", [L.For(i, 0, n - 1, [L.SetFromVec(
        out, (L.SubAxis(), L.Affine(((length, i),), 0)), length, "uint4x32_to_prec_uniform", bits, "uint4x32")])])
    hip, ora = HipRun(r, {}), OracleRun(r, {})
    assert f"w[{length}*i{i} + 1]" in ora.lib.source                 # flat offset: no row term
    hip.step(); ora.step()
    got, want = hip.get(out), ora.get(out)
    assert np.array_equal(got, want)
    # the same numbers as a flat vector of the same length gets
    r1, flat = _uniform_vec_routine(n, prec, length)
    r1.body[0].body[0].arg.a.value = 7
    flat_run = OracleRun(r1, {})
    flat_run.step()
    assert np.array_equal(want.reshape(-1), flat_run.get(flat))
    hip.close()
