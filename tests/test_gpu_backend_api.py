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


def test_contraction_operands_at_element_aligned_offsets_against_the_checker(dev):
    # The shared layer packs nodes at offsets aligned to the element size only
    # (arrayjit/lib/backends.ml:22-51) and the reference's backends link whatever it hands them
    # (cuda_backend.ml:983-1051).  The matrix-core kernels read 16-byte chunks, so a context whose
    # operands sit at 4-byte aligned offsets is linked in the routine's other form (generated
    # kernels): same results, no error.
    from ocannl_amd import workloads as W
    from parity import OracleRun, rel_err
    w = W.dense_contraction(b=256, i=128, o=128, prec="single", out_prec="single")
    code = B.compile(w.routine)
    assert any(k["kind"] == "mfma" for k in code.kernels())
    nodes = w.routine.param_nodes()
    ora = OracleRun(w.routine, w.init)
    ora.step()
    for shift in (0, 4):
        total, locs = shift, {}
        for n in nodes:                      # tightly packed: every node right behind the previous one
            locs[n.id] = (905, total)
            total += n.size_in_bytes
        B.alloc_pool(dev, pool_id=905, size_in_bytes=total, alignment=256)
        B.memset_zero(dev, pool_id=905, offset=0, size_in_bytes=total)
        for n in nodes:
            if n.id in w.init:
                B.from_host(dev, pool_id=905, offset=locs[n.id][1], src=np.ascontiguousarray(w.init[n.id]))
        rt = B.link(dev, code, locs)
        rt.run()
        B.await_(dev)
        for out in w.outputs:
            got = np.zeros(out.dims, np.float32)
            B.to_host(dev, pool_id=905, offset=locs[out.id][1], dst=got)
            B.await_(dev)
            assert rel_err(got, ora.get(out).reshape(out.dims), "single") <= 1e-4, (shift, out.ident)
        del rt
        B.free_pool(dev, pool_id=905)


@pytest.mark.parametrize("how", ["graphs", "static_scratch"])
def test_zero_fill_as_a_kernel_stays_inside_its_node(dev, how):
    # A Zero_out of a context node whose size is not a multiple of 16 bytes, in a tightly packed pool
    # (node offsets aligned to the element size, as arrayjit/lib/backends.ml:22-51 packs them): the
    # fill kernel that replaces hipMemsetAsync under graph capture and in the entry point that may not
    # allocate must leave the neighbouring node alone.
    L.reset_symbols(0)
    g = L.Node(1, "g", "single", (10,)); x = L.Node(2, "x", "single", (10,)); keep = L.Node(3, "keep", "single", (6,))
    one = L.Node(4, "one", "single", (1,))
    i = L.fresh_symbol()
    # (the fill of g survives planning: the statement after it does not touch g everywhere; `one` makes
    # a second launch so that the routine is worth a graph)
    r = L.Routine("fills", [L.ZeroOut(g), L.ZeroOut(one),
                            L.For(i, 0, 4, [L.Set(g, (L.It(i),), L.Binop("add", L.Get(g, (L.It(i),)), L.Get(x, (L.It(i),))))]),
                            L.Set(one, (L.Fixed(0),), L.Binop("add", L.Get(one, (L.Fixed(0),)), L.Const(1.0)))])
    code = B.compile(r, "serial=0;parallel=0;graphs=1" if how == "graphs" else "serial=0;parallel=0")
    assert any(k["kind"] == "fill" for k in code.kernels()), code.kernels()
    # pool: 4 bytes of lead-in, g (40 bytes) at offset 4, keep right behind it, then one and x
    locs = {1: (906, 4), 3: (906, 44), 4: (906, 68), 2: (906, 72)}
    B.alloc_pool(dev, pool_id=906, size_in_bytes=112, alignment=4)
    sentinel = np.full(28, 7.0, np.float32)
    B.from_host(dev, pool_id=906, offset=0, src=sentinel)
    B.from_host(dev, pool_id=906, offset=72, src=np.arange(10, dtype=np.float32))
    rt = B.link(dev, code, locs)
    for _ in range(3):                       # (the first run is direct, later ones replay the graph)
        if how == "graphs":
            rt.run()
        else:
            rt.run_static_scratch()
        B.await_(dev)
    got = np.zeros(28, np.float32)
    B.to_host(dev, pool_id=906, offset=0, dst=got)
    B.await_(dev)
    assert got[0] == 7.0                                         # lead-in
    assert got[1:11].tolist() == [0, 1, 2, 3, 4, 0, 0, 0, 0, 0]  # g
    assert got[11:17].tolist() == [7.0] * 6                      # keep
    assert got[17] == 1.0                                        # one
    del rt
    B.free_pool(dev, pool_id=906)


def test_compile_batch_links_and_runs_each_routine(dev):
    # Lowered_backend.compile_batch + link per routine (arrayjit/lib/backend_impl.ml:349-355;
    # cuda_backend.ml:930-974): two routines that share nodes, one code object, one context
    from ocannl_amd import workloads as W
    from parity import OracleRun
    w1 = W.dense_contraction(b=128, i=64, o=96, prec="single", which=("fwd",))
    r1 = w1.routine
    x = w1.nodes["x"]
    L.reset_symbols(100)
    i, j = L.fresh_symbol(), L.fresh_symbol()
    out = L.Node(900, "rowsum", "single", (x.dims[0],))
    r2 = L.Routine("second_routine", [L.ZeroOut(out), L.For(i, 0, x.dims[0] - 1, [L.For(j, 0, x.dims[1] - 1, [L.Set(
        out, (L.It(i),), L.Binop("add", L.Get(out, (L.It(i),)), L.Get(x, (L.It(i), L.It(j)))))])])])
    code = B.compile_batch([r1, r2], "min_mfma_flops=0")
    ctx = B.Context(dev)
    for n in r1.param_nodes():
        if n.id in w1.init:
            ctx.set_values(n, w1.init[n.id])
    rt0, rt1 = ctx.link(code, 0), ctx.link(code, 1)
    rt1.run(); rt0.run()
    o1, o2 = OracleRun(r1, w1.init), OracleRun(r2, {x.id: w1.init[x.id]})
    o1.step(); o2.step()
    y = w1.nodes["y"]
    assert np.allclose(ctx.get_values(y), o1.get(y), rtol=1e-4, atol=1e-5)
    assert np.allclose(ctx.get_values(out), o2.get(out), rtol=1e-5, atol=1e-5)
    del rt0, rt1
    ctx.free()


def test_routine_outlives_its_code_handle(dev):
    # the launch closure keeps what it needs alive (context_lifetime, cuda_backend.ml:1046-1051):
    # freeing the code handle first, as a finaliser may, leaves the linked routine usable
    L.reset_symbols(0)
    a = L.Node(1, "a", "single", (64,)); b = L.Node(2, "b", "single", (64,))
    st = L.StaticSymbol(L.fresh_symbol(), 4)
    i = L.fresh_symbol()
    r = L.Routine("scaled", [L.For(i, 0, 63, [L.Set(b, (L.It(i),), L.Binop(
        "mul", L.Get(a, (L.It(i),)), L.EmbedIndex(L.It(st.sym))))])], static_indices=[st])
    code = B.compile(r)
    ctx = B.Context(dev)
    ctx.set_values(a, np.arange(64, dtype=np.float32))
    rt = ctx.link(code)
    B.load_library().ocannl_hip_code_free(code._h)
    code._h = None
    garbage = [B.compile(r) for _ in range(4)]   # churn the allocator where the code object lived
    rt.set_static(st.sym, 3)
    rt.run()
    assert np.array_equal(ctx.get_values(b), 3.0 * np.arange(64, dtype=np.float32))
    with pytest.raises(B.User_error):
        rt.set_static(st.sym, 4)
        rt.run()
    del rt, garbage
    ctx.free()


def test_failed_link_releases_what_it_allocated(dev):
    from ocannl_amd import workloads as W
    w = W.moons_mlp()                      # has routine-local nodes: link allocates an arena
    code = B.compile(w.routine)
    before = B.get_used_memory(dev)
    info = B.get_debug_info(dev)
    with pytest.raises(B.User_error):
        B.link(dev, code, {})              # every context node missing
    assert B.get_used_memory(dev) == before and B.get_debug_info(dev) == info


def test_static_indices_travel_as_64_bit_under_large_models(dev):
    # c_syntax.ml:111-112: with large_models static indices are uint64_t arguments
    L.reset_symbols(0)
    a = L.Node(1, "a", "single", (5, 7)); b = L.Node(2, "b", "single", (7,))
    st = L.StaticSymbol(L.fresh_symbol(), 5)
    j = L.fresh_symbol()
    r = L.Routine("row_of", [L.For(j, 0, 6, [L.Set(b, (L.It(j),), L.Binop(
        "add", L.Get(a, (L.It(st.sym), L.It(j))), L.EmbedIndex(L.It(j))))])], static_indices=[st])
    av = np.arange(35, dtype=np.float32).reshape(5, 7)
    for opts, typ in ((None, "const uint32_t "), ("large_models=1", "const uint64_t ")):
        code = B.compile(r, opts)
        assert typ + L.sym_ident(st.sym) in code.source()
        ctx = B.Context(dev)
        ctx.set_values(a, av)
        rt = ctx.link(code)
        rt.set_static(st.sym, 3)
        rt.run()
        assert np.array_equal(ctx.get_values(b), av[3] + np.arange(7))
        del rt
        ctx.free()
