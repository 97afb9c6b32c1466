"""Pins oracle/builtins_cc.h against the reference-held known answers and closed forms."""
import ctypes
import json
import os
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, ROOT


@pytest.fixture(scope="module")
def lib():
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "builtins"], check=True,
                   capture_output=True)
    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "_build", "libbuiltins_cc.so"))
    lib.ocn_x_u4_to_single.restype = ctypes.c_float
    lib.ocn_x_u4_to_double.restype = ctypes.c_double
    lib.ocn_x_bf16_to_single.restype = ctypes.c_float
    lib.ocn_x_bf16_to_single.argtypes = [ctypes.c_uint16]
    lib.ocn_x_single_to_bf16.restype = ctypes.c_uint16
    lib.ocn_x_single_to_bf16.argtypes = [ctypes.c_float]
    lib.ocn_x_fp8_to_single.restype = ctypes.c_float
    lib.ocn_x_fp8_to_single.argtypes = [ctypes.c_uint8]
    lib.ocn_x_single_to_fp8.restype = ctypes.c_uint8
    lib.ocn_x_single_to_fp8.argtypes = [ctypes.c_float]
    lib.ocn_x_half_bits_to_single.restype = ctypes.c_float
    lib.ocn_x_half_bits_to_single.argtypes = [ctypes.c_uint16]
    lib.ocn_x_single_to_half_bits.restype = ctypes.c_uint16
    lib.ocn_x_single_to_half_bits.argtypes = [ctypes.c_float]
    lib.ocn_x_u4_to_bf16.restype = ctypes.c_uint16
    lib.ocn_x_int64_to_uint4x32.argtypes = [ctypes.c_int64, ctypes.c_void_p]
    lib.ocn_x_uint32_to_uint4x32.argtypes = [ctypes.c_uint32, ctypes.c_void_p]
    return lib


@pytest.fixture(scope="module")
def kat():
    with open(os.path.join(GOLDEN, "kat.json")) as f:
        return json.load(f)


def _u4(vals):
    return (ctypes.c_uint32 * 4)(*vals)


def _light(lib, key42, n):
    """uint4x32 bits for counter n as in test/operations/test_threefry4x32.ml: key =
    Constant_bits 42 (int64 -> uint4x32), counter = range value (uint32 -> uint4x32)."""
    key = _u4([0] * 4)
    lib.ocn_x_int64_to_uint4x32(key42, key)
    ctr = _u4([0] * 4)
    lib.ocn_x_uint32_to_uint4x32(n, ctr)
    out = _u4([0] * 4)
    lib.ocn_x_threefry_light(key, ctr, out)
    return out


def test_key_and_counter_spreading(lib):
    key = _u4([9] * 4)
    lib.ocn_x_int64_to_uint4x32(42, key)
    assert list(key) == [42, 0, 0, 0]
    lib.ocn_x_int64_to_uint4x32(-1, key)
    assert list(key) == [0xFFFFFFFF, 0xFFFFFFFF, 0, 0]
    ctr = _u4([0] * 4)
    n = 0x12345678
    lib.ocn_x_uint32_to_uint4x32(n, ctr)
    rot16 = ((n << 16) | (n >> 16)) & 0xFFFFFFFF
    assert list(ctr) == [n, n ^ 0x9E3779B9, n ^ 0x6C078965, n ^ rot16]


def test_threefry_light_single_uniform_kat(lib, kat):
    # test/operations/test_threefry4x32.ml:37-46 -- the vectorised converter fills 4 floats per
    # counter: counter 0 -> values [0..3], counter 1 -> value [4].
    got = []
    for n in range(2):
        out = (ctypes.c_float * 4)()
        lib.ocn_x_u4_to_single_vec(_light(lib, 42, n), out)
        got += list(out)
    want = kat["threefry_light_key42_single_uniform_first5"]
    for g, w in zip(got[:5], want):
        assert float("%.4g" % g) == w, (got[:5], want)
    assert all(0.0 <= g < 1.0 for g in got)


def test_threefry_of_a_tensor_id_single_uniform_kat(lib, kat):
    # test/operations/test_vec_simple.ml: threefry4x32 (embed_self_id ()) 42L, the light variant by
    # default (arrayjit/lib/utils.ml:40), through the vectorised converter in single precision.  The
    # id is a Constant_bits (arrayjit/lib/assignments.ml:793-796; the tensor's id in that program is 1),
    # spread as an int64 like the 42: the four numbers of test_vec_simple.expected:4-7.
    key, ctr, out = _u4([0] * 4), _u4([0] * 4), _u4([0] * 4)
    lib.ocn_x_int64_to_uint4x32(1, key)
    lib.ocn_x_int64_to_uint4x32(42, ctr)
    lib.ocn_x_threefry_light(key, ctr, out)
    f4 = (ctypes.c_float * 4)()
    lib.ocn_x_u4_to_single_vec(out, f4)
    assert [float("%.4g" % v) for v in f4] == kat["threefry_light_selfid1_key42_single_uniform_vec4"]
    # a neighbouring id or the 32-bit spreading gives other numbers: the answer pins both
    lib.ocn_x_int64_to_uint4x32(2, key)
    lib.ocn_x_threefry_light(key, ctr, out); lib.ocn_x_u4_to_single_vec(out, f4)
    assert [float("%.4g" % v) for v in f4] != kat["threefry_light_selfid1_key42_single_uniform_vec4"]
    lib.ocn_x_uint32_to_uint4x32(1, key)
    lib.ocn_x_threefry_light(key, ctr, out); lib.ocn_x_u4_to_single_vec(out, f4)
    assert [float("%.4g" % v) for v in f4] != kat["threefry_light_selfid1_key42_single_uniform_vec4"]


def test_threefry_light_half_uniform_vec_kat(lib, kat):
    # test/operations/threefry4x32_demo.ml:31-73: 5 counters x 8 half values, tolerance 0.01
    got = []
    for n in range(5):
        out = (ctypes.c_float * 8)()
        lib.ocn_x_u4_to_half_vec_as_float(_light(lib, 42, n), out)
        got += list(out)
    want = kat["threefry_light_key42_half_uniform_vec_40"]
    assert len(got) == len(want) == 40
    assert max(abs(g - w) for g, w in zip(got, want)) < 0.01


def test_threefry_structure_invariants(lib):
    # A wrong rotation, a dropped key word or a missing counter increment changes these.
    z = _u4([0] * 4)
    out = _u4([0] * 4)
    lib.ocn_x_threefry_light(z, z, out)
    # zero key / zero counter: state stays 0 through the mixes; the final injection adds
    # ks[1..4] = (0,0,0,C240) and 1 to word 3.
    assert list(out) == [0, 0, 0, 0x1BD11BDA + 1]
    # independent python model of the documented algorithm (builtins.c:156-323)
    def rotl(x, n):
        return ((x << n) | (x >> (32 - n))) & 0xFFFFFFFF

    def pair(x, r):
        x = list(x)
        for a, b in ((r[0], r[1]), (r[2], r[3])):
            x[0] = (x[0] + x[1]) & 0xFFFFFFFF; x[1] = rotl(x[1], a) ^ x[0]
            x[2] = (x[2] + x[3]) & 0xFFFFFFFF; x[3] = rotl(x[3], b) ^ x[2]
            x[1], x[3] = x[3], x[1]
        return x

    def model(key, ctr, groups):
        ks = list(key) + [key[0] ^ key[1] ^ key[2] ^ key[3] ^ 0x1BD11BDA]
        x = [(c + k) & 0xFFFFFFFF for c, k in zip(ctr, key)]
        r0, r1 = (13, 15, 26, 6), (17, 29, 16, 24)
        if groups == 0:
            x = pair(pair(x, r0), r1)
            x = [(x[i] + ks[(1 + i) % 5]) & 0xFFFFFFFF for i in range(4)]
            x[3] = (x[3] + 1) & 0xFFFFFFFF
            return x
        for g in range(1, groups + 1):
            x = pair(pair(pair(pair(x, r0), r1), r0), r1)
            x = [(x[i] + ks[(g + i) % 5]) & 0xFFFFFFFF for i in range(4)]
            x[3] = (x[3] + g) & 0xFFFFFFFF
        return x

    rng = np.random.default_rng(0)
    for _ in range(50):
        key = [int(v) for v in rng.integers(0, 2**32, 4, dtype=np.uint64)]
        ctr = [int(v) for v in rng.integers(0, 2**32, 4, dtype=np.uint64)]
        lib.ocn_x_threefry_light(_u4(key), _u4(ctr), out)
        assert list(out) == model(key, ctr, 0)
        lib.ocn_x_threefry_crypto(_u4(key), _u4(ctr), out)
        assert list(out) == model(key, ctr, 5)


def test_uniform_closed_forms(lib):
    x = _u4([0xFFFFFFFF, 0xFFFFFFFF, 1, 2])
    assert lib.ocn_x_u4_to_single(x) == np.float32(1.0) - np.float32(2.0 ** -24)
    assert lib.ocn_x_u4_to_double(x) == (2.0 ** 64 - 1) * 2.0 ** -64 or lib.ocn_x_u4_to_double(x) == 1.0
    x = _u4([0x80000000, 0, 0, 0])
    assert lib.ocn_x_u4_to_single(x) == 0.5
    assert lib.ocn_x_u4_to_double(x) == 2.0 ** -33
    # bf16 uniform = RNE of the 24-bit single uniform
    assert lib.ocn_x_u4_to_bf16(x) == 0x3F00
    x = _u4([0x00FFFF00, 0, 0, 0])  # (x>>8)*2^-24 = 65535*2^-24 -> rounds to 2^-8 in bf16
    assert lib.ocn_x_u4_to_bf16(x) == 0x3B80


def test_bf16_known_answers(lib, kat):
    for x, bits, back in kat["bf16"]:
        x, back = float(x), float(back)
        b = lib.ocn_x_single_to_bf16(x)
        assert b == int(bits, 16)
        got = lib.ocn_x_bf16_to_single(b)
        assert got == back or abs(got - back) < 5e-7


def test_bf16_exhaustive_against_bit_model(lib):
    # widening is an exact shift for all 2^16 patterns; narrowing a widened value is identity
    # except that the add-0x7FFF trick has no NaN special case (still returns the same bits).
    for b in range(0, 1 << 16, 1):
        f = lib.ocn_x_bf16_to_single(b)
        w = np.array([b << 16], dtype=np.uint32).view(np.float32)[0]
        if w != w:
            assert f != f
            continue
        assert f == w
        assert lib.ocn_x_single_to_bf16(f) == b
    # round-to-nearest-even on ties and near-ties
    def f32(u):
        return float(np.array([u], dtype=np.uint32).view(np.float32)[0])
    assert lib.ocn_x_single_to_bf16(f32(0x3F808000)) == 0x3F80  # tie -> even (down)
    assert lib.ocn_x_single_to_bf16(f32(0x3F818000)) == 0x3F82  # tie -> even (up)
    assert lib.ocn_x_single_to_bf16(f32(0x3F808001)) == 0x3F81
    assert lib.ocn_x_single_to_bf16(f32(0x3F807FFF)) == 0x3F80
    rng = np.random.default_rng(1)
    xs = rng.standard_normal(2000).astype(np.float32)
    for x in xs:
        u = int(np.array([x], dtype=np.float32).view(np.uint32)[0])
        want = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF
        assert lib.ocn_x_single_to_bf16(float(x)) == want


def test_fp8_known_answers_and_exhaustive(lib, kat):
    for x, bits, back in kat["fp8"]:
        b = lib.ocn_x_single_to_fp8(float(x))
        assert b == int(bits, 16), (x, hex(b))
        assert lib.ocn_x_fp8_to_single(b) == float(back)
    # E5M2 decode against the format definition for all 256 codes
    for v in range(256):
        s, e, m = v >> 7, (v >> 2) & 31, v & 3
        got = lib.ocn_x_fp8_to_single(v)
        if v == 0:
            assert got == 0.0
        elif e == 31:
            assert (got != got) if m else (got == (-np.inf if s else np.inf))
        else:
            mag = (m / 4.0) * 2.0 ** -14 if e == 0 else (1 + m / 4.0) * 2.0 ** (e - 15)
            assert got == (-mag if s else mag)


def test_half_roundtrip_exhaustive(lib):
    bits = np.arange(1 << 16, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    for b in range(0, 1 << 16, 1):
        got = lib.ocn_x_half_bits_to_single(b)
        w = float(want[b])
        if w != w:
            assert got != got
        else:
            assert got == w
            assert lib.ocn_x_single_to_half_bits(w) == b or (w == 0.0)


# ---- the restatement against the reference's own C, in bulk -------------------------------------------

@pytest.fixture(scope="module")
def ref_lib(reference_root):
    """The reference's builtins.c (its plain-C part) compiled unchanged by `make -C oracle ref`."""
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "ref"], check=True, capture_output=True)
    return ctypes.CDLL(os.path.join(ROOT, "oracle", "_ref", "builtins_ref.so"))


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


@pytest.mark.parametrize("crypto", [0, 1], ids=["light", "crypto"])
def test_threefry_bit_identical_to_reference_c(lib, ref_lib, crypto):
    # builtins.c:195-323, both variants: 20 000 random (key, counter) pairs plus structured ones
    # (zero key, zero counter, all ones, single bits) that a wrong rotation or key-schedule index shows
    rng = np.random.default_rng(7 + crypto)
    n = 20000
    keys = rng.integers(0, 2**32, (n, 4), dtype=np.uint64).astype(np.uint32)
    ctrs = rng.integers(0, 2**32, (n, 4), dtype=np.uint64).astype(np.uint32)
    keys[:64] = 0; ctrs[64:128] = 0; keys[128:160] = 0xFFFFFFFF; ctrs[160:192] = 0xFFFFFFFF
    for b in range(128):
        keys[200 + b] = 0; keys[200 + b, b // 32] = 1 << (b % 32)
        ctrs[400 + b] = 0; ctrs[400 + b, b // 32] = 1 << (b % 32)
    keys, ctrs = np.ascontiguousarray(keys), np.ascontiguousarray(ctrs)
    mine, theirs = np.zeros((n, 4), np.uint32), np.ones((n, 4), np.uint32)
    lib.ocn_x_batch_threefry(crypto, _p(keys), _p(ctrs), _p(mine), n)
    ref_lib.ocn_x_batch_threefry(crypto, _p(keys), _p(ctrs), _p(theirs), n)
    assert np.array_equal(mine, theirs)
    # and the two variants are different functions of their input
    other = np.zeros((n, 4), np.uint32)
    lib.ocn_x_batch_threefry(1 - crypto, _p(keys), _p(ctrs), _p(other), n)
    assert not np.array_equal(mine, other)


def test_uniform_converters_bit_identical_to_reference_c(lib, ref_lib):
    # builtins.c:345-528: every uint4x32 -> uniform converter, vector and scalar forms
    rng = np.random.default_rng(11)
    n = 20000
    xs = rng.integers(0, 2**32, (n, 4), dtype=np.uint64).astype(np.uint32)
    xs[:8] = 0; xs[8:16] = 0xFFFFFFFF; xs[16:24] = 0x00FFFFFF; xs[24:32] = 0x80000000
    xs = np.ascontiguousarray(xs)

    def run(l):
        f4, d2 = np.zeros((n, 4), np.float32), np.zeros((n, 2), np.float64)
        b8, h8 = np.zeros((n, 8), np.uint16), np.zeros((n, 8), np.float32)
        f1, d1, b1 = np.zeros(n, np.float32), np.zeros(n, np.float64), np.zeros(n, np.uint16)
        l.ocn_x_batch_uniform(_p(xs), _p(f4), _p(d2), _p(b8), _p(h8), _p(f1), _p(d1), _p(b1), n)
        return f4, d2, b8, h8, f1, d1, b1

    for name, a, b in zip(("single_vec", "double_vec", "bf16_vec", "half_vec", "single", "double", "bf16"), run(lib), run(ref_lib)):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), name


def test_conversions_and_spreading_bit_identical_to_reference_c(lib, ref_lib):
    # builtins.c:531-606 (X -> uint4x32) and :611-743 (bf16, fp8): random bit patterns of every float
    # class (normals, subnormals, infinities, NaNs, both zeros) plus values near the fp8 range edges
    rng = np.random.default_rng(13)
    n = 40000
    bits = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    bits[:6] = [0, 0x80000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x00000001]
    xs = bits.view(np.float32).copy()
    xs[100:2100] = rng.uniform(-70000, 70000, 2000).astype(np.float32)
    xs[2100:4100] = (rng.standard_normal(2000) * 1e-5).astype(np.float32)

    def conv(l):
        bf, f8 = np.zeros(n, np.uint16), np.zeros(n, np.uint8)
        bfb, f8b = np.zeros(n, np.float32), np.zeros(n, np.float32)
        l.ocn_x_batch_convert(_p(xs), _p(bf), _p(f8), _p(bfb), _p(f8b), n)
        return bf, f8, bfb.view(np.uint32), f8b.view(np.uint32)

    for name, a, b in zip(("single_to_bf16", "single_to_fp8", "bf16_to_single", "fp8_to_single"), conv(lib), conv(ref_lib)):
        assert np.array_equal(a, b), name

    def spread(l):
        a, b, c = (np.zeros((n, 4), np.uint32) for _ in range(3))
        l.ocn_x_batch_spread(_p(bits), _p(a), _p(b), _p(c), n)
        return a, b, c

    for name, a, b in zip(("uint32", "int64", "single"), spread(lib), spread(ref_lib)):
        assert np.array_equal(a, b), name + "_to_uint4x32"
