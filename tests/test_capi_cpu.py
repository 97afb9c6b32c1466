"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, and
the compile half (parse -> plan -> HIP source -> hiprtc for gfx950) works without a GPU."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from ocannl_amd import backend as B
from ocannl_amd import llir as L
from ocannl_amd import workloads as W


def test_library_exports_every_declared_symbol():
    with open(os.path.join(ROOT, "include", "ocannl_hip.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(ocannl_hip_[a-z_0-9]+)\s*\(", header))
    assert declared == set(B.EXPORTS)
    lib = ctypes.CDLL(B.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name


def test_compile_needs_no_gpu_and_reports_kernels():
    w = W.moons_mlp()
    code = B.compile(w.routine, "serial=0;parallel=0")
    ks = code.kernels()
    assert len(ks) > 10 and all(k["kind"] in ("generated", "fill") for k in ks)
    # independent small phases share launches
    assert len(B.compile(w.routine, "serial=0").kernels()) < len(ks)
    # by default a routine of tiny phases becomes ONE single-workgroup kernel
    assert len(B.compile(w.routine).kernels()) == 1
    src = code.source()
    assert "extern \"C\" __global__" in src and "arrayjit_threefry4x32_light" in src
    kinds = {k for k, _, _ in code.kparams()}
    assert kinds == {"ptr", "static_idx"}
    ids = {i for k, i, _ in code.kparams() if k == "ptr"}
    assert ids == {n.id for n in w.routine.param_nodes()}


def test_big_contraction_is_planned_as_mfma_with_the_right_shape():
    w = W.dense_contraction(b=512, i=256, o=384, prec="bfloat16", out_prec="single")
    ks = [k for k in B.compile(w.routine).kernels() if k["kind"] == "mfma"]
    assert [(k["m"], k["n"], k["k"]) for k in ks] == [(512, 384, 256), (512, 256, 384), (384, 256, 512)]
    assert all(k["flops"] == 2.0 * 512 * 256 * 384 for k in ks)
    # the Zero_out in front of the forward contraction is folded into it (beta = 0)
    assert not any(k["kind"] == "fill" for k in B.compile(w.routine).kernels())


def test_small_contraction_stays_generic_and_sequential_order():
    w = W.dense_contraction(b=8, i=8, o=8, prec="single")
    code = B.compile(w.routine)
    assert all(k["kind"] == "generated" for k in code.kernels())
    assert "fmaf(" in code.source()


def test_malformed_ir_is_invalid_argument():
    lib = B.load_library()
    h = ctypes.c_void_p()
    for text in (b"(routine", b"(routine \"x\" (nodes (1 \"a\" single ctx 0 0 (2))) (body (zero_out 7)))",
                 b"(routine \"x\" (nodes (1 \"a\" nosuch ctx 0 0 (2))) (body))",
                 b"(routine \"x\" (nodes (1 \"a\" single ctx 0 0 (2 2))) (body (set 1 ((fixed 0)) (const 0x0p+0))))"):
        rc = lib.ocannl_hip_compile(text, len(text), ctypes.byref(h))
        assert rc == -2, text
        assert lib.ocannl_hip_last_error()


def test_threefry_on_wrong_precision_is_user_error():
    # arrayjit/lib/cc_backend.ml:231-246: threefry on a non-uint4x32 destination is rejected
    a = L.Node(1, "a", "single", (4,))
    b = L.Node(2, "b", "single", (4,))
    r = L.Routine("bad", [L.For(1, 0, 3, [L.Set(a, (L.It(1),), L.Binop(
        "threefry4x32_light", L.Get(b, (L.It(1),)), L.Get(b, (L.It(1),))))])])
    with pytest.raises(B.User_error):
        B.compile(r)


def test_plan_pool_segments_matches_reference_rule():
    # arrayjit/lib/backends.ml:22-51: bump packing with alignment, new pool when the cap is hit
    assign, sizes = B.plan_pool_segments([(8, 8), (8, 8), (100, 64), (40, 8)], cap=128)
    assert assign == [(0, 0), (0, 8), (1, 0), (2, 0)] or assign == [(0, 0), (0, 8), (1, 0), (1, 104)]
    assign, sizes = B.plan_pool_segments([(8, 256), (8, 256)])
    assert assign == [(0, 0), (0, 256)] and sizes == [264]
    with pytest.raises(B.User_error):
        B.plan_pool_segments([(200, 8)], cap=128)


def test_planner_rewrites_show_in_the_generated_source():
    # compile-only checks (no GPU): the kernel-fusing rewrites fire on shapes that call for them and
    # each can be switched off
    import re
    from ocannl_amd import llir as L
    kw = dict(batch=4, seq=128, d_model=128, heads=2, d_ff=256, layers=1, vocab=2048, prec="bfloat16", grad_prec="single")
    w = W.transformer(**kw)
    full = B.compile(w.routine)
    src = full.source()
    assert "row0_" in src                                   # row groups
    assert re.search(r"bf\d+_\w+\[[^\]]*\] = single_to_bfloat16\(", src)   # bf16 operand copies kept by producers
    fills = lambda code: sum(k["kind"] == "fill" for k in code.kernels())
    assert fills(full) <= 1                                 # zero fills folded into their consumers
    plain = B.compile(w.routine, "rows=0;bf16_copies=0")
    assert "row0_" not in plain.source() and len(plain.kernels()) > len(full.kernels())
    assert all(k["name"].startswith("gemm_bf16_kernel") for k in full.kernels() if k["kind"] == "mfma")
    # a column sum over many rows is split into partial sums + a combine
    L.reset_symbols(0)
    x = L.Node(1, "x", "single", (4096, 256)); out = L.Node(2, "out", "single", (256,))
    j, i = L.fresh_symbol(), L.fresh_symbol()
    r = L.Routine("colsum", [L.For(j, 0, 255, [L.For(i, 0, 4095, [
        L.Set(out, (L.It(j),), L.Binop("add", L.Get(out, (L.It(j),)), L.Get(x, (L.It(i), L.It(j)))))])])])
    assert len(B.compile(r).kernels()) == 2 and len(B.compile(r, "coop=0").kernels()) == 1


def test_padding_region_loops_visit_exactly_the_margin():
    # low_level.ml:2705-2802 by brute force: run the loops in Python and count visits per cell
    import itertools
    import numpy as np
    for dims, padding in (((4, 5), ((1, 2), (0, 0))), ((3, 6, 5), ((0, 0), (2, 1), (1, 1))), ((5,), ((0, 3),)),
                          ((2, 4, 4, 3), ((0, 0), (1, 1), (1, 1), (0, 0))), ((3, 3), ((0, 0), (0, 0)))):
        L.reset_symbols(0)
        visits = np.zeros(dims, int)
        stmts = L.loop_over_padding_region(dims, padding, lambda idcs: [L.Set(L.Node(1, "t", "single", dims), idcs, L.Const(0.0))])

        def run(body, env):
            for st in body:
                if isinstance(st, L.For):
                    for v in range(st.from_, st.to + 1):
                        run(st.body, {**env, st.sym: v})
                else:
                    visits[tuple(env[ix.sym] if isinstance(ix, L.It) else ix.i for ix in st.idcs)] += 1
        run(stmts, {})
        want = np.ones(dims, int)
        want[tuple(slice(l, d - r) for d, (l, r) in zip(dims, padding))] = 0
        assert np.array_equal(visits, want), (dims, padding)
