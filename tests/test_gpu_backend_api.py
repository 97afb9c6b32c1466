"""GPU tests of the device half of the boundary: pools, copies, events, bookkeeping."""
import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    B.initialize()
    assert B.num_devices() >= 1
    return B.get_device(0)


def test_device_properties(dev):
    assert B.get_name(dev) == "hip:0"
    props = B.static_properties()
    assert "gfx950" in props and "multiprocessor_count 256" in props
    assert "pools" in B.get_debug_info(dev)
    with pytest.raises(B.Invalid_argument):
        B.get_device(99)


def test_pool_offsets_do_not_clobber(dev):
    # twin of test/operations/test_cuda_pool_offset.real.ml: p = a + b and q = a *. b, both outputs
    # bump-packed in ONE pool at distinct offsets, must hold independent values.
    L.reset_symbols(0)
    a = L.Node(1, "a", "single", (2,)); b = L.Node(2, "b", "single", (2,))
    p = L.Node(3, "p", "single", (2,)); q = L.Node(4, "q", "single", (2,))
    i, j = L.fresh_symbol(), L.fresh_symbol()
    r = L.Routine("combo", [
        L.For(i, 0, 1, [L.Set(p, (L.It(i),), L.Binop("add", L.Get(a, (L.It(i),)), L.Get(b, (L.It(i),))))]),
        L.For(j, 0, 1, [L.Set(q, (L.It(j),), L.Binop("mul", L.Get(a, (L.It(j),)), L.Get(b, (L.It(j),))))])])
    used0 = B.get_used_memory(dev)
    B.alloc_pool(dev, pool_id=901, size_in_bytes=32, alignment=8)
    B.memset_zero(dev, pool_id=901, offset=0, size_in_bytes=32)
    locs = {1: (901, 0), 2: (901, 8), 3: (901, 16), 4: (901, 24)}
    assert locs[3][0] == locs[4][0] and locs[3][1] != locs[4][1]
    B.from_host(dev, pool_id=901, offset=0, src=np.array([1.0, 2.0], np.float32))
    B.from_host(dev, pool_id=901, offset=8, src=np.array([3.0, 4.0], np.float32))
    assert B.get_used_memory(dev) == used0 + 32
    rt = B.link(dev, B.compile(r), locs)
    rt.run()
    B.await_(dev)
    pv, qv = np.zeros(2, np.float32), np.zeros(2, np.float32)
    B.to_host(dev, pool_id=901, offset=16, dst=pv)
    B.to_host(dev, pool_id=901, offset=24, dst=qv)
    B.await_(dev)
    assert pv.tolist() == [4.0, 6.0] and qv.tolist() == [3.0, 8.0]
    del rt
    B.free_pool(dev, pool_id=901)
    assert B.get_used_memory(dev) == used0
    with pytest.raises(B.Invalid_argument):
        B.free_pool(dev, pool_id=901)


def test_events_and_device_to_device(dev):
    B.alloc_pool(dev, pool_id=902, size_in_bytes=1 << 20, alignment=256)
    B.alloc_pool(dev, pool_id=903, size_in_bytes=1 << 20, alignment=256)
    src = np.arange(1 << 18, dtype=np.float32)
    B.from_host(dev, pool_id=902, offset=0, src=src)
    B.device_to_device(dst=dev, dst_pool_id=903, dst_offset=0, src=dev, src_pool_id=902, src_offset=0,
                       size_in_bytes=src.nbytes)
    ev = B.all_work(dev)
    B.will_wait_for(dev, ev)
    B.sync(ev)
    assert B.is_done(ev)
    B.await_(dev)
    assert B.is_idle(dev)
    out = np.zeros_like(src)
    B.to_host(dev, pool_id=903, offset=0, dst=out)
    B.await_(dev)
    assert np.array_equal(out, src)
    # into the merge buffer (pool 0 grows on demand, cuda_backend.ml:130-134)
    B.device_to_device(dst=dev, dst_pool_id=-1, dst_offset=0, src=dev, src_pool_id=902, src_offset=0,
                       size_in_bytes=4096)
    out = np.zeros(1024, np.float32)
    B.to_host(dev, pool_id=0, offset=0, dst=out)
    B.await_(dev)
    assert np.array_equal(out, src[:1024])
    with pytest.raises(B.Invalid_argument):
        B.to_host(dev, pool_id=903, offset=(1 << 20) - 4, dst=np.zeros(4, np.float32))
    for p in (902, 903, 0):
        B.free_pool(dev, pool_id=p)


def test_link_reports_missing_node(dev):
    a = L.Node(1, "a", "single", (2,)); b = L.Node(2, "b", "single", (2,))
    r = L.Routine("cp", [L.For(1, 0, 1, [L.Set(a, (L.It(1),), L.Get(b, (L.It(1),)))])])
    B.alloc_pool(dev, pool_id=904, size_in_bytes=64, alignment=8)
    with pytest.raises(B.User_error):
        B.link(dev, B.compile(r), {1: (904, 0)})
    B.free_pool(dev, pool_id=904)


def test_link_rejects_misaligned_contraction_operand(dev):
    # the matrix-core kernels read 16-byte chunks: an operand packed at a 4-byte aligned offset
    # (what element-size alignment alone would allow) is a user error, reported at link time
    from ocannl_amd import workloads as W
    w = W.dense_contraction(b=256, i=128, o=128, prec="single", out_prec="single")
    code = B.compile(w.routine)
    assert any(k["kind"] == "mfma" for k in code.kernels())
    nodes = w.routine.param_nodes()
    total, locs = 0, {}
    for n in nodes:
        locs[n.id] = (905, total)
        total += (n.size_in_bytes + 255) // 256 * 256
    B.alloc_pool(dev, pool_id=905, size_in_bytes=total + 256, alignment=256)
    rt = B.link(dev, code, locs)          # aligned: fine
    del rt
    bad = dict(locs)
    first = nodes[0].id
    bad[first] = (905, locs[first][1] + 4)
    with pytest.raises(B.User_error, match="16-byte"):
        B.link(dev, code, bad)
    B.free_pool(dev, pool_id=905)
