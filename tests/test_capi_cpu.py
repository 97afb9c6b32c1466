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
    assert all(k["name"].startswith(("gemm_bf16_kernel", "gemm_bf16_dtl_kernel")) for k in full.kernels() if k["kind"] == "mfma")
    # a gradient that several statements of one row group accumulate into is stored once, by the last of
    # them (the earlier values live in the group's registers); apart, every statement stores it
    stores = lambda text, name: len(re.findall(name + r"_\d+\[[^\]]*\] = ", text))
    assert stores(src, "counts_grad") == 1 and stores(plain.source(), "counts_grad") == 2
    assert stores(src, "centered_ln1_l0_grad") == 1 and stores(plain.source(), "centered_ln1_l0_grad") == 3
    # a column sum over many rows is split into partial sums + a combine
    L.reset_symbols(0)
    x = L.Node(1, "x", "single", (4096, 256)); out = L.Node(2, "out", "single", (256,))
    j, i = L.fresh_symbol(), L.fresh_symbol()
    r = L.Routine("colsum", [L.For(j, 0, 255, [L.For(i, 0, 4095, [
        L.Set(out, (L.It(j),), L.Binop("add", L.Get(out, (L.It(j),)), L.Get(x, (L.It(i), L.It(j)))))])])])
    assert len(B.compile(r).kernels()) == 2 and len(B.compile(r, "coop=0").kernels()) == 1
    # the combine walks the 512 slices of an output with 32 lanes that take slices next to one another
    # (16 each), not with one thread
    combine = B.compile(r).source().split("colsum_k1(")[1]
    assert "gtid_ % 32u" in combine and "ocn_xshfl(part_, 16)" in combine and "+= 32)" in combine


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


def _conv_input_gradient(stride, ksz, b=8, oh=32, ow=32, ic=64, oc=64):
    """x_grad[b, stride*o1+k1, stride*o2+k2, i] += y_grad[b, o1, o2, c] * w[c, k1, k2, i]
    (the input gradient of lib/nn_blocks.ml:418-428's convolution)."""
    L.reset_symbols(0)
    ih, iw = stride * (oh - 1) + ksz, stride * (ow - 1) + ksz
    w = L.Node(2, "w", "single", (oc, ksz, ksz, ic)); dy = L.Node(4, "y_grad", "single", (b, oh, ow, oc))
    dx = L.Node(5, "x_grad", "single", (b, ih, iw, ic))
    s = [L.fresh_symbol() for _ in range(7)]
    bb, o1, o2, c, k1, k2, i = s
    xi = (L.It(bb), L.Affine(((stride, o1), (1, k1)), 0), L.Affine(((stride, o2), (1, k2)), 0), L.It(i))
    yi = (L.It(bb), L.It(o1), L.It(o2), L.It(c))
    wi = (L.It(c), L.It(k1), L.It(k2), L.It(i))
    body = [L.Set(dx, xi, L.Ternop("fma", L.Get(dy, yi), L.Get(w, wi), L.Get(dx, xi)))]
    for sym, ext in reversed(list(zip(s, (b, oh, ow, oc, ksz, ksz, ic)))):
        body = [L.For(sym, 0, ext - 1, body)]
    return L.Routine(f"conv_dx_s{stride}_k{ksz}", [L.ZeroOut(dx)] + body), dict(w=w, dy=dy, dx=dx)


def test_overlapping_window_accumulation_is_not_a_matrix_core_contraction():
    # stride 1, window 3: different (o, k) meet on one element of x_grad, which the contraction kernels'
    # plain read-add-write epilogue would lose; such a nest stays a generated kernel.  With
    # stride = window the map is one-to-one and the matrix cores may take it.
    r, _ = _conv_input_gradient(1, 3)
    assert all(k["kind"] != "mfma" for k in B.compile(r, "min_mfma_flops=0").kernels())
    r, _ = _conv_input_gradient(3, 3)
    assert any(k["kind"] == "mfma" for k in B.compile(r, "min_mfma_flops=0").kernels())


def _stale_copy_routine(n=256):
    """zero_out y1; zero_out y2; c1 = x * w; x := 2 x; y1 += ..; y2 += ..; c2 = x * w with x fp32 and w
    bf16: the second product must not reuse the bf16 copy of x made for the first."""
    L.reset_symbols(0)
    x = L.Node(1, "x", "single", (n, n)); w = L.Node(2, "w", "bfloat16", (n, n))
    c1 = L.Node(3, "c1", "single", (n, n)); c2 = L.Node(4, "c2", "single", (n, n))
    y1 = L.Node(5, "y1", "single", (n,)); y2 = L.Node(6, "y2", "single", (n,))
    u = L.Node(7, "u", "single", (n, n))

    def matmul(c):
        i, j, k = L.fresh_symbol(), L.fresh_symbol(), L.fresh_symbol()
        return [L.ZeroOut(c), L.For(i, 0, n - 1, [L.For(j, 0, n - 1, [L.For(k, 0, n - 1, [L.Set(
            c, (L.It(i), L.It(j)), L.Ternop("fma", L.Get(x, (L.It(i), L.It(k))), L.Get(w, (L.It(j), L.It(k))),
                                            L.Get(c, (L.It(i), L.It(j)))))])])])]

    def rowsum(y):
        i, k = L.fresh_symbol(), L.fresh_symbol()
        return [L.For(i, 0, n - 1, [L.For(k, 0, n - 1, [L.Set(y, (L.It(i),), L.Binop(
            "add", L.Get(y, (L.It(i),)), L.Get(u, (L.It(i), L.It(k)))))])])]

    i, j = L.fresh_symbol(), L.fresh_symbol()
    scale = [L.For(i, 0, n - 1, [L.For(j, 0, n - 1, [L.Set(x, (L.It(i), L.It(j)), L.Binop(
        "mul", L.Const(2.0), L.Get(x, (L.It(i), L.It(j)))))])])]
    body = [L.ZeroOut(y1), L.ZeroOut(y2)] + matmul(c1) + scale + rowsum(y1) + rowsum(y2) + matmul(c2)
    return L.Routine("stale_copy", body), dict(x=x, w=w, c1=c1, c2=c2, y1=y1, y2=y2, u=u)


def test_bf16_copy_of_an_operand_rewritten_between_two_products_is_refreshed():
    # zero fills grouped ahead of their sums (as zero_grads-then-backprop orders them) are folded away
    # after the copy was planned; the second product still has to see the rewritten operand
    r, _ = _stale_copy_routine()
    code = B.compile(r, "min_mfma_flops=0")
    src = code.source()
    # two distinct bf16 copies of x: one converted before x is rewritten, one kept by the kernel that rewrites it
    copies = set(re.findall(r"\b(bf\d+_x)\[[^\]]*\] = ", src))
    assert len(copies) >= 2, src


def test_compile_batch_holds_every_routine():
    # Lowered_backend.compile_batch (arrayjit/lib/backend_impl.ml:349-353): several routines, one code
    w1 = W.dense_contraction(b=64, i=64, o=64, prec="single", which=("fwd",))
    r1 = w1.routine
    a = r1.param_nodes()[0]
    L.reset_symbols(100)
    i = L.fresh_symbol()
    out = L.Node(900, "rowsum", "single", (a.dims[0],))
    j = L.fresh_symbol()
    r2 = L.Routine("second_routine", [L.ZeroOut(out), L.For(i, 0, a.dims[0] - 1, [L.For(j, 0, a.dims[1] - 1, [L.Set(
        out, (L.It(i),), L.Binop("add", L.Get(out, (L.It(i),)), L.Get(a, (L.It(i), L.It(j)))))])])])
    code = B.compile_batch([r1, r2])
    lib = B.load_library()
    n = ctypes.c_int()
    assert lib.ocannl_hip_code_num_routines(code._h, ctypes.byref(n)) == 0 and n.value == 2
    buf = ctypes.create_string_buffer(64)
    assert lib.ocannl_hip_code_routine_name(code._h, 1, buf, 64) == 0 and buf.value.decode() == "second_routine"
    assert code.index_of("second_routine") == 1
    assert {i for k, i, _ in code.kparams(1) if k == "ptr"} == {a.id, out.id}
    assert len(code.kernels(0)) >= 1 and len(code.kernels(1)) >= 1
    assert "second_routine_k0" in code.source()
    assert lib.ocannl_hip_code_routine_name(code._h, 2, buf, 64) == -2


def test_debug_log_source_follows_the_reference_line_format():
    # c_syntax.ml:493-535: `# <statement>` then `lhs[%u]{=old} = new = <expression with {=value} after
    # every read>`; comments as `COMMENT: text`; cuda_backend.ml:874-893: `<log id>: ` prefix, `$` for \n
    a = L.Node(1, "a", "single", (4,)); b = L.Node(2, "b", "bfloat16", (4,)); c = L.Node(3, "c", "single", (4,))
    L.reset_symbols(0)
    i = L.fresh_symbol()
    r = L.Routine("logged", [L.Comment("c fwd"), L.For(i, 0, 3, [L.Set(c, (L.It(i),), L.Ternop(
        "fma", L.Get(a, (L.It(i),)), L.Get(b, (L.It(i),)), L.Const(0.5)))]), L.Comment("end")])
    code = B.compile(r, "debug_log=1")
    src = code.source()
    assert 'printf("%d: COMMENT: c fwd$", log_id);' in src and 'printf("%d: COMMENT: end$", log_id);' in src
    assert 'printf("%d: # c[i1] := fma(a[i1], b[i1], 0.5);$", log_id);' in src
    assert ('printf("%d: c[%u]{=%g} = %g = fmaf(a[%u]{=%g}, bfloat16_to_single(b[%u]){=%g}, (float)(0.5))$", log_id, '
            '(unsigned)(i1), (double)(c[i1]), (double)(new_set_v), (unsigned)(i1), (double)(a[i1]), (unsigned)(i1), '
            '(double)(bfloat16_to_single(b[i1])));') in src
    # one thread walks the loop in order; the kernel takes the log id; without the option nothing is printed
    assert "for (uint32_t i1 = 0; i1 <= 3; ++i1)" in src and "const int log_id" in src
    assert "printf" not in B.compile(r).source().split("extern \"C\"", 1)[1]


def test_weight_gradients_go_to_the_side_queue_and_fused_prologues_show_up():
    kw = dict(batch=32, seq=256, d_model=512, heads=8, d_ff=1024, layers=2, vocab=512, prec="bfloat16", grad_prec="single")
    w = W.transformer(**kw)
    ks = B.compile(w.routine, "side_queue=1").kernels()
    side = [k for k in ks if k["queue"] == 1]
    assert side and all(k["kind"] == "mfma" for k in side)
    assert all(k["queue"] == 0 for k in B.compile(w.routine).kernels())   # (off unless asked for)
    # Q K^T ahead of the soft-max chain runs inside the row-wise kernel (one launch less per block)
    fused, apart = B.compile(w.routine), B.compile(w.routine, "fused=0")
    assert "ocn_rowtile_contract<256, 64, 16, unsigned short, 264>" in fused.source().split("extern \"C\"", 1)[1]
    n = lambda c: sum(k["kind"] == "mfma" for k in c.kernels())
    assert n(B.compile(w.routine, "proj=0")) == n(apart) - 2
    # ... and attention weights times V runs in there as well
    assert "ocn_rowtile_project<256, 64, 16, 4, 264>" in fused.source().split("extern \"C\"", 1)[1]
    assert n(fused) == n(apart) - 4


def test_memory_operands_of_conditionals_are_loaded_ahead_of_the_statement():
    # `g[i] = relu_gate(a[i], b[i])` and `w[i] = where(a[i], b[i], c[i])`: written as C conditionals the
    # loads of b and c would wait for the condition (two dependent trips to memory); reads through plain
    # loop iterators are in range whatever the condition says and are issued first.  A read through an
    # affine index (a convolution window that the condition may be guarding) stays where it is.
    L.reset_symbols(0)
    n = 4096
    a, b, c = (L.Node(k + 1, s, "single", (n,)) for k, s in enumerate("abc"))
    g, w, v = L.Node(4, "g", "single", (n,)), L.Node(5, "w", "single", (n,)), L.Node(6, "v", "single", (n // 2,))
    i, j, k = L.fresh_symbol(), L.fresh_symbol(), L.fresh_symbol()
    body = [L.For(i, 0, n - 1, [L.Set(g, (L.It(i),), L.Binop("relu_gate", L.Get(a, (L.It(i),)), L.Get(b, (L.It(i),))))]),
            L.For(j, 0, n - 1, [L.Set(w, (L.It(j),), L.Ternop("where", L.Get(a, (L.It(j),)), L.Get(b, (L.It(j),)), L.Get(c, (L.It(j),))))]),
            L.For(k, 0, n // 2 - 1, [L.Set(v, (L.It(k),), L.Binop("relu_gate", L.Get(a, (L.It(k),)),
                                                                   L.Get(b, (L.Affine([(2, k)], 1),))))])]
    src = B.compile(L.Routine("conditionals", body), "parallel=0;rows=0").source().split("extern \"C\"", 1)[1]
    assert re.search(r"const float (w\d+_) = b\[i\d+\];\s*g\[i\d+\] = \(a\[i\d+\] > 0\.0 \? \1 : 0\.0\);", src), src
    assert len(re.findall(r"const float w\d+_ = [bc]\[", src)) == 3, src
    assert re.search(r"v\[[^\]]*\] = \(a\[[^\]]*\] > 0\.0 \? b\[[^\]]*\] : 0\.0\);", src), src


def _scores_then_row_chain(rewrite_operand: bool):
    # x[s, t] = sum_d a[s, d] * b[t, d] feeding a row-wise chain over the rows s (max, exp of the shifted
    # value); optionally the chain also stores into the operand a itself
    S, T, D = 512, 128, 128
    L.reset_symbols(0)
    a = L.Node(1, "a", "bfloat16", (S, D)); b = L.Node(2, "b", "bfloat16", (T, D))
    x = L.Node(3, "x", "bfloat16", (S, T), mode="local"); m = L.Node(4, "m", "bfloat16", (S,), mode="local")
    y = L.Node(5, "y", "bfloat16", (S, T))
    s, t, d = L.fresh_symbol(), L.fresh_symbol(), L.fresh_symbol()
    body = [L.ZeroOut(x), L.For(s, 0, S - 1, [L.For(t, 0, T - 1, [L.For(d, 0, D - 1, [L.Set(x, (L.It(s), L.It(t)), L.Ternop(
        "fma", L.Get(a, (L.It(s), L.It(d))), L.Get(b, (L.It(t), L.It(d))), L.Get(x, (L.It(s), L.It(t)))))])])])]
    s2, t2 = L.fresh_symbol(), L.fresh_symbol()
    body.append(L.For(s2, 0, S - 1, [L.Set(m, (L.It(s2),), L.Const(float("-inf")))]))
    s3 = L.fresh_symbol()
    body.append(L.For(s3, 0, S - 1, [L.For(t2, 0, T - 1, [L.Set(m, (L.It(s3),), L.Binop(
        "max", L.Get(m, (L.It(s3),)), L.Get(x, (L.It(s3), L.It(t2)))))])]))
    s4, t4 = L.fresh_symbol(), L.fresh_symbol()
    body.append(L.For(s4, 0, S - 1, [L.For(t4, 0, T - 1, [L.Set(y, (L.It(s4), L.It(t4)), L.Unop(
        "exp", L.Binop("sub", L.Get(x, (L.It(s4), L.It(t4))), L.Get(m, (L.It(s4),)))))])]))
    if rewrite_operand:
        s5, t5 = L.fresh_symbol(), L.fresh_symbol()
        body.append(L.For(s5, 0, S - 1, [L.For(t5, 0, T - 1, [L.Set(a, (L.It(s5), L.It(t5)), L.Get(y, (L.It(s5), L.It(t5))))])]))
    return L.Routine("scores_chain", body)


def test_a_row_group_that_rewrites_an_operand_keeps_the_contraction_apart():
    # The contraction ahead of a row-wise chain becomes that kernel's prologue (each workgroup computes
    # its own 32 rows of x) -- unless the chain itself stores into an operand of the contraction: one
    # workgroup's stores would then race with another workgroup's prologue loads, which a kernel
    # boundary used to order.
    fused = B.compile(_scores_then_row_chain(False))
    body = fused.source().split('extern "C"', 1)[1]
    assert "ocn_rowtile_contract<" in body and not any(k["kind"] == "mfma" for k in fused.kernels())
    apart = B.compile(_scores_then_row_chain(True))
    body = apart.source().split('extern "C"', 1)[1]
    assert "ocn_rowtile_contract<" not in body
    assert sum(k["kind"] == "mfma" for k in apart.kernels()) == 1


def test_a_recomputed_contraction_reads_the_stored_relu_output_instead():
    # With the reference's visit rule the sum `product + bias` behind a relu is virtual
    # (test/einsum/moons_demo_variant.expected:39-44), so the relu's backward statement
    # `g1 =+ relu_gate(v1, g)` holds the whole product again; the planner reads the stored relu output
    # there (v1 > 0 exactly when relu(v1) > 0) instead of a 128-long loop per element.
    import re
    kw = dict(batch=4, seq=64, d_model=128, heads=2, d_ff=256, layers=1, vocab=256, prec="bfloat16", grad_prec="single")
    w = W.transformer(inline="visits", **kw)
    loops = lambda code: len(re.findall(r"for \(uint32_t i\d+ = 0; i\d+ <= 127; \+\+i\d+\) \{\s*v\d+_ffn1", code.source()))
    assert loops(B.compile(w.routine, "reuse=0")) >= 1
    assert loops(B.compile(w.routine)) == 0
