"""The serialised form of ``Low_level.optimized``, constructor by constructor (CPU only).

Every constructor of ``Low_level.t`` / ``scalar_t`` (arrayjit/lib/low_level.mli:22-68) and of
``Indexing.axis_index`` (indexing.ml:104-120) is written here as the OCaml serialiser prints it
(``ocaml/hip_wire.ml``), fed to the library's reader through the C ABI, and recognised by what the
generated kernel source then contains.  The same routine built with ``ocannl_amd.llir`` has to
serialise to the same text: the Python writer is the executable twin of the OCaml one."""
import ctypes

import pytest

from ocannl_amd import backend as B
from ocannl_amd import llir as L

NODES = """(nodes
(1 "a" single ctx 0 1 (4 6))
(2 "b" bfloat16 ctx 0 1 (4 6))
(3 "c" single ctx 0 0 (4 6))
(4 "v" single virtual 0 0 (1))
(5 "key" uint4x32 ctx 0 1 (1))
(6 "r" single ctx 0 0 (8))
(7 "tbl" single ctx 0 1 (27 10))
(8 "ix" single ctx 0 1 (4))
(9 "g" single ctx 0 0 (4 10))
(10 "t" single local 1 0 (4)))"""


def compile_wire(body: str, static: str = "", merge: int = -1, options: str = "mfma=0;coop=0;serial=0;rows=0;parallel=0"):
    text = f'(routine "wire_case"\n(static {static})\n(merge {merge})\n{NODES}\n(body\n{body}))\n'.encode()
    lib = B.load_library()
    h = ctypes.c_void_p()
    rc = lib.ocannl_hip_compile_opts(text, len(text), options.encode(), ctypes.byref(h))
    if rc != 0:
        raise AssertionError(lib.ocannl_hip_last_error().decode())
    need = ctypes.c_size_t()
    assert lib.ocannl_hip_code_source(h, None, 0, ctypes.byref(need)) == 0
    buf = ctypes.create_string_buffer(need.value)
    assert lib.ocannl_hip_code_source(h, buf, need.value, None) == 0
    lib.ocannl_hip_code_free(h)
    return buf.value.decode().split('extern "C"', 1)[1]


def loop2(inner: str) -> str:
    return f"(for 1 0 3 ((for 2 0 5 ({inner}))))"


IJ = "((it 1) (it 2))"

CASES = {
    # --- Low_level.t ---
    "Comment": ('(comment "c fwd")\n' + loop2(f"(set 3 {IJ} (const 0x1.0000000000000p+0))"), "(float)(1)"),
    "For_loop+Set": (loop2(f"(set 3 {IJ} (get 1 {IJ}))"), "c[(i1) * 6 + i2] = a[(i1) * 6 + i2]"),
    "Zero_out": ("(zero_out 10)\n(for 1 0 3 ((set 10 ((it 1)) (binop add (get 10 ((it 1))) (get 8 ((it 1)))))))"
                 "\n(for 1 0 3 ((set 8 ((it 1)) (get 10 ((it 1))))))", "t["),
    "Set_from_vec": ("(set_vec 6 ((affine ((4 1)) 0)) 4 uint4x32_to_prec_uniform uint4x32 (get 5 ((fixed 0))))".join(
        ["(for 1 0 1 (", "))"]), "uint4x32_to_single_uniform_vec("),
    # hoisted common subexpressions: Declare_local / Set_local statements, Get_local readers
    "Declare_local+Set_local+Get_local": (loop2(
        f"(declare_local 4 7 0)\n(set_local 4 7 (binop mul (get 1 {IJ}) (get 1 {IJ})))\n"
        f"(set 3 {IJ} (binop add (get_local 4 7) (get_local 4 7)))"), "v7_v"),
    # --- scalar_t ---
    # an inlined reduction: the scope declares its own local
    "Local_scope": (loop2(
        f"(set 3 {IJ} (local_scope 4 8 ((set_local 4 8 (const 0x0.0p+0))\n"
        "(for 3 0 5 ((set_local 4 8 (binop add (get_local 4 8) (get 1 ((it 1) (it 3))))))))))"), "v8_v"),
    "Get_dynamic": ("(for 1 0 3 ((for 2 0 9 ((set 9 ((it 1) (it 2)) (get_dyn 7 ((fixed 0) (it 2)) 0 single (get 8 ((it 1)))))))))",
                    "tbl[(((uint32_t)(ix[i1]))) * 10 + i2]"),
    "Get_merge_buffer": (loop2(f"(set 3 {IJ} (binop add (get 3 {IJ}) (get_merge 1 {IJ})))"), "merge_buffer["),
    "Ternop+arg_prec": (loop2(f"(set 3 {IJ} (ternop fma single (get 1 {IJ}) (get 2 {IJ}) (get 3 {IJ})))"),
                        "fmaf(a[(i1) * 6 + i2], bfloat16_to_single(b[(i1) * 6 + i2]), c[(i1) * 6 + i2])"),
    "Where": (loop2(f"(set 3 {IJ} (ternop where bfloat16 (get 2 {IJ}) (get 1 {IJ}) (const -0x1.0000000000000p+1)))"), "?"),
    "Binop": (loop2(f"(set 3 {IJ} (binop relu_gate (get 1 {IJ}) (get 2 {IJ})))"), "> 0.0 ?"),
    "Unop+arg_prec": (loop2(f"(set 3 {IJ} (unop exp single (get 1 {IJ})))"), "expf(a[(i1) * 6 + i2])"),
    "Constant": (loop2(f"(set 3 {IJ} (const 0x1.999999999999ap-4))"), "(float)(0.1)"),
    "Constant special": (loop2(f"(set 3 {IJ} (const -inf))"), "INFINITY"),
    "Constant_bits": ("(set 5 ((fixed 0)) (bits 42))", "42"),
    "Embed_index": (loop2(f"(set 3 {IJ} (index (it 2)))"), "(float)(i2)"),
    # --- Indexing.axis_index ---
    "Fixed_idx": (loop2(f"(set 3 {IJ} (get 1 ((fixed 3) (it 2))))"), "a[(3) * 6 + i2]"),
    "Affine": ("(for 1 0 1 ((for 2 0 1 ((set 3 ((it 1) (it 2)) (get 1 ((affine ((2 1) (1 2)) 0) (affine ((3 2)) 1))))))))",
               "a[(2*i1+i2) * 6 + 3*i2+1]"),
    "Sub_axis": ("(for 1 0 1 ((set_vec 6 ((affine ((4 1)) 0)) 4 uint4x32_to_prec_uniform uint4x32 (get 5 ((sub))))))",
                 "key[0]"),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_reader_takes_every_constructor(name):
    body, expected = CASES[name]
    merge = 1 if name == "Get_merge_buffer" else -1
    src = compile_wire(body, merge=merge)
    assert expected in src, src


def test_static_symbols_and_their_ranges():
    # Indexing.static_symbol with and without a range; the symbol is a kernel parameter read at launch
    src = compile_wire("(for 2 0 5 ((set 3 ((it 9) (it 2)) (get 1 ((it 9) (it 2))))))", static="(9 4) (11 -1)")
    assert "i9" in src


def test_staged_compilation_and_unknown_heads_are_refused():
    # Staged_compilation cannot cross the boundary (the OCaml side raises before serialising); anything
    # the reader does not know is Invalid_argument, never a crash
    lib = B.load_library()
    for bad in ("(staged x)", "(set 3 ((it 1)) (frob 1))", "(set 3 ((concat 1 2) (fixed 0)) (const 0x0.0p+0))"):
        text = f'(routine "bad"\n(static )\n(merge -1)\n{NODES}\n(body\n{bad}))\n'.encode()
        h = ctypes.c_void_p()
        assert lib.ocannl_hip_compile(text, len(text), ctypes.byref(h)) == -2


def test_python_writer_prints_what_the_ocaml_writer_prints():
    # the same statements built with the host model serialise to the text written above
    L.reset_symbols(1)
    a = L.Node(1, "a", "single", (4, 6)); b = L.Node(2, "b", "bfloat16", (4, 6)); c = L.Node(3, "c", "single", (4, 6))
    i, j = 1, 2
    st = L.For(i, 0, 3, [L.For(j, 0, 5, [L.Set(c, (L.It(i), L.It(j)), L.Ternop(
        "fma", L.Get(a, (L.It(i), L.It(j))), L.Get(b, (L.It(i), L.It(j))), L.Get(c, (L.It(i), L.It(j)))))])])
    text = L.to_wire(L.Routine("wire_case", [st]))
    assert loop2(f"(set 3 {IJ} (ternop fma single (get 1 {IJ}) (get 2 {IJ}) (get 3 {IJ})))") in text
    # (the OCaml writer lists nodes by id, this one by first appearance: the reader takes any order)
    assert text.startswith('(routine "wire_case"\n(static )\n(merge -1)\n(nodes\n')
    assert '(1 "a" single ctx 0 0 (4 6))' in text and '(2 "b" bfloat16 ctx 0 0 (4 6))' in text
    # hexadecimal floats: 13 hex digits, as Python's float.hex and ocaml/hip_wire.ml's hex_float print them
    st2 = L.For(i, 0, 3, [L.For(j, 0, 5, [L.Set(c, (L.It(i), L.It(j)), L.Const(0.1))])])
    assert "(const 0x1.999999999999ap-4)" in L.to_wire(L.Routine("wire_case", [st2]))
    st3 = L.For(i, 0, 3, [L.For(j, 0, 5, [L.Set(c, (L.It(i), L.It(j)), L.Const(float("-inf")))])])
    assert "(const -inf)" in L.to_wire(L.Routine("wire_case", [st3]))
