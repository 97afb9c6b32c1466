"""64-bit offsets in generated kernels: the reference's ``large_models`` setting widens loop indices
and integer arguments (c_syntax.ml:111-112, ops.ml:64). The HIP path switches by itself when a node
has more than 2^31 - 1 elements, and on request (``large_models=1``)."""
import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L
from ocannl_amd import workloads as W
from oracle import cc_emit, cc_oracle
from parity import HipRun

pytestmark = pytest.mark.gpu


def test_wide_offsets_change_no_result():
    # the same routine with 32-bit and with 64-bit offsets: every fused form of the planner is crossed
    kw = dict(batch=4, seq=128, d_model=128, heads=2, d_ff=256, layers=1, vocab=2048, prec="bfloat16", grad_prec="single")
    w = W.transformer(**kw)
    a, b = HipRun(w.routine, w.init), HipRun(w.routine, w.init, "large_models=1")
    assert "uint64_t i" in b.code.source() and "uint64_t i" not in a.code.source()
    for _ in range(2):
        a.step(); b.step()
    for name in ("loss", "w_embed", "w_q_l0", "w_ffn2_l0", "w_out", "gamma_ln1_l0", "pos_encoding"):
        assert np.array_equal(a.get(w.nodes[name]), b.get(w.nodes[name])), name
    a.close(); b.close()


def test_static_index_and_gather_with_wide_offsets():
    w = W.char_mlp()
    a, b = HipRun(w.routine, w.init), HipRun(w.routine, w.init, "large_models=1")
    for _ in range(3):
        a.step(); b.step()
    for n in w.outputs or [w.nodes["loss"]]:
        assert np.array_equal(a.get(n), b.get(n)), n
    a.close(); b.close()


def test_node_beyond_32_bit_offsets():
    # byte nodes of 2^32 + 2^16 elements: a pointwise map and a row sum whose offsets pass 2^32.
    # The checker runs with the reference's large_models setting; numpy pins both independently.
    rows, cols = (1 << 16) + 1, 1 << 16
    L.reset_symbols(0)
    x = L.Node(1, "x", "byte", (rows, cols)); y = L.Node(2, "y", "byte", (rows, cols))
    s = L.Node(3, "s", "uint32", (rows,))
    i, j, i2, j2 = (L.fresh_symbol() for _ in range(4))
    r = L.Routine("wide", [
        L.For(i, 0, rows - 1, [L.For(j, 0, cols - 1, [
            L.Set(y, (L.It(i), L.It(j)), L.Binop("add", L.Get(x, (L.It(i), L.It(j))), L.Const(3.0)))])]),
        L.For(i2, 0, rows - 1, [L.For(j2, 0, cols - 1, [
            L.Set(s, (L.It(i2),), L.Binop("add", L.Get(s, (L.It(i2),)), L.Get(y, (L.It(i2), L.It(j2)))))])]),
    ])
    code = B.compile(r)
    assert "uint64_t i" in code.source()
    rng = np.random.default_rng(0)
    xv = rng.integers(0, 256, size=(rows, cols), dtype=np.uint8)
    ctx = B.Context()
    ctx.allocate([x, y, s])
    ctx.set_values(x, xv)
    rt = ctx.link(code)
    rt.run()
    got_s = ctx.get_values(s)
    got_y = ctx.get_values(y)
    want_y = xv + np.uint8(3)
    assert np.array_equal(got_y[-2:], want_y[-2:]) and np.array_equal(got_y, want_y)
    want_s = want_y.sum(axis=1, dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(got_s, want_s)
    del got_y
    cc_emit.LARGE_MODELS = True
    try:
        bufs = {x.id: xv, y.id: cc_oracle.host_array(y), s.id: cc_oracle.host_array(s)}
        lib = cc_oracle.CompiledOracle([r])
        assert "for (uint64_t i" in lib.source
        lib.run(r.name, bufs, {})
    finally:
        cc_emit.LARGE_MODELS = False
    assert np.array_equal(bufs[y.id], want_y) and np.array_equal(bufs[s.id], got_s)
    ctx.free()
