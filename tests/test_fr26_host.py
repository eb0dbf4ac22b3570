"""CPU checks of the 26-bit-limb lazy Fr arithmetic used by the streaming kernels (host build of
grape_amd/csrc/fr26.hpp) against Python integers: canonical products, Montgomery in/out, integer
embedding, sums of products with signed (difference) operands, weighted sums of 64 terms."""
import ctypes
import os
import random
import subprocess
import numpy as np
import pytest
import bigref as br

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "native", "fr26_host.cpp")
BN = br.CURVE == "bn254"
LIB = os.path.join(HERE, "native", "libfr26_host_bn254.so" if BN else "libfr26_host.so")
R = br.R_MOD


@pytest.fixture(scope="module")
def lib():
    deps = [SRC] + [os.path.join(HERE, "..", "grape_amd", "csrc", f) for f in ("fr26.hpp", "field.hpp", "divstep.hpp")]
    if not os.path.exists(LIB) or any(os.path.getmtime(d) > os.path.getmtime(LIB) for d in deps):
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-unknown-pragmas"]
                              + (["-DGRAPE_CURVE_BN254"] if BN else []) + ["-o", LIB, SRC])
    return ctypes.CDLL(LIB)


def _p(vals):
    return np.ascontiguousarray(br.fr_pack(vals).view(np.uint32).reshape(len(vals), 8))


def _u32(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))


def _val(a):
    return br.fr_unpack(np.ascontiguousarray(a).view(np.uint64).reshape(1, 4))[0]


EDGE = [0, 1, 2, R - 1, R - 2, (1 << 254) % R, (1 << 255) % R, (1 << 26) - 1, 1 << 26, (1 << 234) - 1, R >> 1, 2**64 - 1]


def test_mulc_and_montgomery(lib):
    rng = random.Random(1)
    vals = EDGE + [rng.randrange(R) for _ in range(60)]
    out = np.zeros(8, dtype=np.uint32)
    for a in vals:
        pa = _p([a])[0]
        for b in vals[:16] + vals[-5:]:
            lib.t26_mulc(_u32(pa), _u32(_p([b])[0]), _u32(out))
            assert _val(out) == a * b % R
        # from_mont gives the plain integer, to_mont of the plain limbs gives the packed form back
        lib.t26_from_mont(_u32(pa), _u32(out))
        plain = np.ascontiguousarray(br.ints_to_limbs([a], 4).view(np.uint32).reshape(8))
        assert np.array_equal(out, plain)
        lib.t26_to_mont(_u32(plain), _u32(out))
        assert np.array_equal(out, pa)


def test_inverse_by_divsteps(lib):
    """1/a through batched divsteps on 30-bit limbs against pow(a, -1, r) and against the a^(r-2) ladder it
    replaces at the top level of a batched inversion; 1/0 = 0 as in the reference"""
    rng = random.Random(7)
    vals = EDGE + [rng.randrange(R) for _ in range(300)] + [rng.randrange(1 << k) for k in (1, 5, 30, 31, 60, 61, 90, 200)]
    out, out2 = np.zeros(8, dtype=np.uint32), np.zeros(8, dtype=np.uint32)
    for a in vals:
        lib.t26_inverse_by(_u32(_p([a])[0]), _u32(out))
        lib.t26_inverse_ladder(_u32(_p([a])[0]), _u32(out2))
        want = pow(a, -1, R) if a % R else 0
        assert _val(out) == want, hex(a)
        assert _val(out2) == want, hex(a)


def test_integer_embedding(lib):
    out = np.zeros(8, dtype=np.uint32)
    for x in (0, 1, -1, 2, -2, 32767, -32768, 2**31 - 1, -2**31, 123456, -654321, 1 << 26, -(1 << 26)):
        lib.t26_from_i32(ctypes.c_int32(x), _u32(out))
        assert _val(out) == x % R
    for x in (0, 1, 2**32 - 1, 65536, 1 << 26):
        lib.t26_from_u32(ctypes.c_uint32(x), _u32(out))
        assert _val(out) == x


def test_lazy_signed_sum(lib):
    rng = random.Random(2)
    out = np.zeros(8, dtype=np.uint32)
    for n in (1, 2, 7, 16):
        for trial in range(20):
            pick = lambda: rng.choice(EDGE) if rng.random() < 0.3 else rng.randrange(R)
            a0, a1, b0, b1 = ([pick() for _ in range(n)] for _ in range(4))
            lib.t26_lazy_sum(_u32(_p(a0)), _u32(_p(a1)), _u32(_p(b0)), _u32(_p(b1)), n, _u32(out))
            want = sum((x1 - x0) * (y1 - y0) + x0 * y1 for x0, x1, y0, y1 in zip(a0, a1, b0, b1)) % R
            assert _val(out) == want


def test_weighted_sum_64(lib):
    rng = random.Random(3)
    out = np.zeros(8, dtype=np.uint32)
    for n in (1, 3, 64):
        for trial in range(10):
            w = [R - 1 if trial == 0 else rng.randrange(R) for _ in range(n)]
            t = [R - 1 if trial == 0 else rng.randrange(R) for _ in range(n)]
            lib.t26_weighted_sum(_u32(_p(w)), _u32(_p(t)), n, _u32(out))
            assert _val(out) == sum(x * y for x, y in zip(w, t)) % R


def test_split_weighted_sum_and_wide_canon(lib):
    rng = random.Random(4)
    out = np.zeros(8, dtype=np.uint32)
    for n, S in ((1, 2), (5, 4), (128, 2), (256, 4), (64, 1), (200, 4)):
        for trial in range(6):
            w = [R - 1 if trial == 0 else rng.randrange(R) for _ in range(n)]
            t = [R - 1 if trial == 0 else rng.randrange(R) for _ in range(n)]
            lib.t26_weighted_sum_split(_u32(_p(w)), _u32(_p(t)), n, S, _u32(out))
            assert _val(out) == sum(x * y for x, y in zip(w, t)) % R
    for k in (0, 1, 2, 15, 30):
        for a in EDGE + [rng.randrange(R) for _ in range(10)]:
            for b in (0, 1, R - 1, rng.randrange(R)):
                lib.t26_canon_wide(_u32(_p([a % R])[0]), _u32(_p([b])[0]), k, _u32(out))
                assert _val(out) == (k * (a % R) + b) % R


def test_single_product_fold_and_canon4(lib):
    """lo + v*(hi - lo) with one limb product and lo added into the upper accumulator columns: every
    pairing of the edge values (differences of either sign, v = 0, 1, r-1) and random triples; the
    nine-word canonicalisation on multiples k*a + b up to just below 4r"""
    rng = random.Random(5)
    out = np.zeros(8, dtype=np.uint32)
    vals = EDGE + [rng.randrange(R) for _ in range(12)]
    for v in [0, 1, R - 1, R >> 1] + [rng.randrange(R) for _ in range(6)]:
        pv = _p([v])[0]
        for lo in vals:
            plo = _p([lo])[0]
            for hi in vals:
                lib.t26_fold1(_u32(pv), _u32(plo), _u32(_p([hi])[0]), _u32(out))
                assert _val(out) == (lo + v * (hi - lo)) % R, (v, lo, hi)
    for k in (0, 1, 2, 3):
        for a in EDGE + [rng.randrange(R) for _ in range(10)]:
            for b in (0, 1, R - 1, R - 2, rng.randrange(R)):
                if k * (a % R) + b >= 4 * R:
                    continue
                lib.t26_canon4(_u32(_p([a % R])[0]), _u32(_p([b])[0]), k, _u32(out))
                assert _val(out) == (k * (a % R) + b) % R


def test_table_fold(lib):
    """the fold through ten precomputed multiples of the challenge: row j of the table is the integer
    v * 2^(26 j + 52) mod r in 26-bit limbs, and lo + v*(hi - lo) comes out canonical for every pairing
    of the edge values (differences of either sign, an absent hi) and v = 0, 1, r-1, r/2"""
    rng = random.Random(6)
    out = np.zeros(8, dtype=np.uint32)
    tab = np.zeros(100, dtype=np.int32)
    vals = EDGE + [rng.randrange(R) for _ in range(12)]
    for v in [0, 1, R - 1, R >> 1, R - 2] + [rng.randrange(R) for _ in range(6)]:
        lib.t26_fold_table(_u32(_p([v])[0]), tab.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
        for j in range(10):
            row = sum(int(tab[10 * j + k]) << (26 * k) for k in range(10))
            assert all(0 <= int(tab[10 * j + k]) < (1 << 26) for k in range(10))
            assert row == (v << (26 * j + 52)) % R, (v, j)
        for lo in vals:
            plo = _p([lo])[0]
            for hi in vals:
                lib.t26_foldt(tab.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), _u32(plo), _u32(_p([hi])[0]), _u32(out))
                assert _val(out) == (lo + v * (hi - lo)) % R, (v, lo, hi)
