"""Routines that read the merge buffer: the gradient-merging step of the reference's data-parallel
update (lib/parallel.ml:164-383) as it looks on one device with two contexts. A transfer
``device_to_device ~into_merge_buffer`` (cuda_backend.ml:289-314) fills the stream's merge buffer,
then a routine whose code reads ``g.merge`` runs against it; the buffer is bound when the routine is
scheduled (cuda_backend.ml:1009-1011), so it may be regrown between runs."""
import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L
from ocannl_amd import workloads as W
from oracle import cc_oracle

pytestmark = pytest.mark.gpu


def _merge_routine(prec, dims, name="merge_grad"):
    L.reset_symbols(0)
    p = L.Node(1, "p", "single", dims)
    g = L.Node(2, "g_grad", prec, dims)
    lr = L.Node(3, "lr", "single", (1,))
    body = [L.Comment("g =+ g.merge")]
    body += L.loop_over_dims(dims, lambda idcs: [L.Set(g, idcs, L.Binop("add", L.Get(g, idcs), L.GetMerge(g, idcs)))])
    body += [L.Comment("p =- lr * g")]
    body += L.loop_over_dims(dims, lambda idcs: [L.Set(p, idcs, L.Binop(
        "sub", L.Get(p, idcs), L.Binop("mul", L.Get(lr, (L.Fixed(0),)), L.Get(g, idcs))))])
    return L.Routine(name, body, merge_node=g), p, g, lr


def _values(node, seed):
    rng = np.random.default_rng(seed)
    return W.as_prec(rng.uniform(-1, 1, node.dims).astype(np.float32), node.prec)


@pytest.mark.parametrize("prec", ["single", "bfloat16", "double"])
def test_merge_routine_matches_the_checker(prec):
    dims = (37, 64)
    r, p, g, lr = _merge_routine(prec, dims)
    code = B.compile(r)
    assert "merge_buffer[" in code.source()
    assert ("merge_buffer", g.id) in [(k, i) for k, i, _ in code.kparams()]
    mine, other = B.Context(), B.Context()
    for ctx, seed in ((mine, 1), (other, 2)):
        ctx.allocate([p, g, lr])
        ctx.set_values(p, _values(p, seed)); ctx.set_values(g, _values(g, seed + 10))
        ctx.set_values(lr, np.array([0.1], np.float32))
    rt = mine.link(code)
    # nothing transferred yet (pool 0 absent): scheduling the routine is a user error
    try:
        B.free_pool(mine.dev, pool_id=0)
    except B.Invalid_argument:
        pass
    with pytest.raises(B.User_error):
        rt.run()
    pool, off = other.ctx_buffers[g.id]
    B.device_to_device(dst=mine.dev, dst_pool_id=-1, dst_offset=0, src=other.dev, src_pool_id=pool, src_offset=off,
                       size_in_bytes=g.size_in_bytes)
    rt.run()
    bufs = {p.id: _values(p, 1), g.id: _values(g, 11), lr.id: np.array([0.1], np.float32)}
    cc_oracle.CompiledOracle([r]).run(r.name, bufs, {}, merge=_values(g, 12))
    assert np.array_equal(mine.get_values(g), bufs[g.id])
    # p - lr * g may or may not be contracted into one fused multiply-add by either compiler
    assert np.allclose(mine.get_values(p), bufs[p.id], rtol=1e-6, atol=1e-7)
    # the other context is untouched
    assert np.array_equal(other.get_values(g), _values(g, 12))
    mine.free(); other.free()


def test_merge_buffer_regrown_between_runs():
    small, big = (8, 16), (64, 512)
    rs, ps, gs, lrs = _merge_routine("single", small, "merge_small")
    rb, pb, gb, lrb = _merge_routine("single", big, "merge_big")
    a, b = B.Context(), B.Context()
    a.allocate([ps, gs, lrs]); b.allocate([gs])
    b.set_values(gs, _values(gs, 5))
    rt_s = a.link(B.compile(rs))
    a2, b2 = B.Context(), B.Context()
    a2.allocate([pb, gb, lrb]); b2.allocate([gb])
    b2.set_values(gb, _values(gb, 6))
    rt_b = a2.link(B.compile(rb))
    for rt, src_ctx, g in ((rt_s, b, gs), (rt_b, b2, gb), (rt_s, b, gs)):
        pool, off = src_ctx.ctx_buffers[g.id]
        B.device_to_device(dst=a.dev, dst_pool_id=-1, dst_offset=0, src=a.dev, src_pool_id=pool, src_offset=off,
                           size_in_bytes=g.size_in_bytes)
        rt.run()
    assert np.array_equal(a.get_values(gs), _values(gs, 5) + _values(gs, 5))
    assert np.array_equal(a2.get_values(gb), _values(gb, 6))
    for c in (a, b, a2, b2):
        c.free()
