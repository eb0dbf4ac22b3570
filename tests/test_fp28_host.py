"""CPU checks of the 28-bit-limb lazy Fp arithmetic used by the commitment kernels (host build of
grape_amd/csrc/fp28.hpp): products, squares, conversions and lazily reduced expressions against
Python integers; sums of points through the 28-bit mixed addition against textbook affine
arithmetic, including the exceptional cases (doubling, cancellation, identity)."""
import ctypes
import os
import random
import subprocess
import numpy as np
import pytest
import bigref as br

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "native", "fp28_host.cpp")
BN = br.CURVE == "bn254"
LIB = os.path.join(HERE, "native", "libfp28_host_bn254.so" if BN else "libfp28_host.so")
P = br.P_MOD
FW = 2 * br.FP_LIMBS          # 32-bit words of an Fp element in memory
PB = P.bit_length()


@pytest.fixture(scope="module")
def lib():
    deps = [SRC] + [os.path.join(HERE, "..", "grape_amd", "csrc", f) for f in ("fp28.hpp", "curve.hpp", "field.hpp")]
    if not os.path.exists(LIB) or any(os.path.getmtime(d) > os.path.getmtime(LIB) for d in deps):
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-unknown-pragmas"]
                              + (["-DGRAPE_CURVE_BN254"] if BN else []) + ["-o", LIB, SRC])
    return ctypes.CDLL(LIB)


def _p32(vals):
    """canonical values -> (n, FW) uint32 Montgomery (memory form) limbs"""
    return np.ascontiguousarray(br.fp_pack(vals).view(np.uint32).reshape(len(vals), FW))


def _u32(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))


def _val(a):
    return br.fp_unpack(np.ascontiguousarray(a).view(np.uint64).reshape(1, br.FP_LIMBS))[0]


EDGE = [0, 1, 2, P - 1, P - 2, 1 << (PB - 1), (1 << PB) % P, (1 << 28) - 1, 1 << 28, (1 << (PB - 17)) - 1, P >> 1]


def test_mul_sqr_roundtrip(lib):
    rng = random.Random(1)
    vals = EDGE + [rng.randrange(P) for _ in range(60)]
    out = np.zeros(FW, dtype=np.uint32)
    for a in vals:
        pa = _p32([a])[0]
        lib.t28_roundtrip(_u32(pa), _u32(out))
        assert _val(out) == a
        lib.t28_roundtrip_lazy(_u32(pa), _u32(out))
        assert _val(out) == a
        lib.t28_sqr(_u32(pa), _u32(out))
        assert _val(out) == a * a % P
        for b in vals[:14] + vals[-4:]:
            pb = _p32([b])[0]
            lib.t28_mul(_u32(pa), _u32(pb), _u32(out))
            assert _val(out) == a * b % P


def test_lazy_expression(lib):
    rng = random.Random(2)
    out = np.zeros(FW, dtype=np.uint32)
    for _ in range(200):
        a, b, c, d = (rng.choice(EDGE) if rng.random() < 0.3 else rng.randrange(P) for _ in range(4))
        pa, pb, pc, pd = (_p32([x])[0] for x in (a, b, c, d))
        lib.t28_lazy(_u32(pa), _u32(pb), _u32(pc), _u32(pd), _u32(out))
        assert _val(out) == (a - b - 2 * c) * d % P


def test_zero_detection(lib):
    plain = lambda v: np.ascontiguousarray(br.ints_to_limbs([v], br.FP_LIMBS).view(np.uint32).reshape(FW))
    for k in (0, 1, 2):
        assert lib.t28_is_zero(_u32(plain(0)), k) == 1
        assert lib.t28_is_zero(_u32(plain(1)), k) == 0
        assert lib.t28_is_zero(_u32(plain(P - 1)), k) == 0


def _points(ks):
    return [br.g1_mul(k, br.G1) for k in ks]


def _sum28(lib, pts, negs):
    arr = np.ascontiguousarray(br.g1_pack(pts).view(np.uint32).reshape(len(pts), 2 * FW))
    neg = np.array(negs, dtype=np.int32)
    xyzz = np.zeros(4 * FW, dtype=np.uint32)
    slow = lib.t28_sum(_u32(arr), neg.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), len(pts), _u32(xyzz))
    aff = np.zeros(2 * FW, dtype=np.uint32)
    lib.t28_xyzz_to_affine(_u32(xyzz), _u32(aff))
    return br.g1_unpack(aff.view(np.uint64).reshape(1, br.G1_WORDS))[0], slow


def test_point_sums_vs_textbook(lib):
    rng = random.Random(3)
    ks = [rng.randrange(1, br.R_MOD) for _ in range(40)]
    pts = _points(ks)
    negs = [rng.random() < 0.5 for _ in pts]
    got, slow = _sum28(lib, pts, negs)
    want = None
    for p, n in zip(pts, negs):
        want = br.g1_add(want, br.g1_neg(p) if n else p)
    assert got == want and slow == 0


def test_exceptional_cases_take_the_exact_path(lib):
    a, b = br.g1_mul(5, br.G1), br.g1_mul(7, br.G1)
    # doubling: a + a ; cancellation: a - a ; identity operands ; then keep adding
    got, slow = _sum28(lib, [a, a, b], [False, False, False])
    assert got == br.g1_add(br.g1_add(a, a), b) and slow == 1
    got, slow = _sum28(lib, [a, a, b], [False, True, False])
    assert got == b and slow == 1
    got, slow = _sum28(lib, [None, a, None, b], [False] * 4)
    assert got == br.g1_add(a, b) and slow == 0
    got, slow = _sum28(lib, [a, a], [True, False])
    assert got is None and slow == 1
    got, slow = _sum28(lib, [], [])
    assert got is None
    # a long chain of the same point: 1,2,3,...: only the first addition doubles
    got, slow = _sum28(lib, [a] * 9, [False] * 9)
    assert got == br.g1_mul(45, br.G1) and slow == 1


def test_inverse(lib):
    rng = random.Random(4)
    out = np.zeros(FW, dtype=np.uint32)
    for a in [1, 2, P - 1, 1 << (PB - 1)] + [rng.randrange(1, P) for _ in range(10)]:
        lib.t28_inverse(_u32(_p32([a])[0]), _u32(out))
        assert _val(out) == pow(a, -1, P)


def test_inverse_by_divsteps(lib):
    rng = random.Random(6)
    out = np.zeros(FW, dtype=np.uint32)
    vals = [1, 2, 3, P - 1, P - 2, 1 << (PB - 1), (1 << PB) % P, (P + 1) // 2, 0xffffffff, 1 << 64]
    vals += [rng.randrange(1, P) for _ in range(300)]
    for a in vals:
        lib.t28_inverse_by(_u32(_p32([a])[0]), _u32(out))
        assert _val(out) == pow(a, -1, P), hex(a)


def _sum_tree(lib, pts, negs):
    arr = np.ascontiguousarray(br.g1_pack(pts).view(np.uint32).reshape(len(pts), 2 * FW))
    neg = np.array(negs, dtype=np.int32)
    aff = np.zeros(2 * FW, dtype=np.uint32)
    slow = lib.t28_sum_tree(_u32(arr), neg.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), len(pts), _u32(aff))
    return br.g1_unpack(aff.view(np.uint64).reshape(1, br.G1_WORDS))[0], slow


def test_accumulator_plus_accumulator(lib):
    rng = random.Random(5)
    pts = _points([rng.randrange(1, br.R_MOD) for _ in range(21)])
    negs = [rng.random() < 0.5 for _ in pts]
    got, slow = _sum_tree(lib, pts, negs)
    want = None
    for p, n in zip(pts, negs):
        want = br.g1_add(want, br.g1_neg(p) if n else p)
    assert got == want and slow == 0
    a, b = br.g1_mul(5, br.G1), br.g1_mul(7, br.G1)
    # the two halves hold the same point / opposite points / one of them is the identity
    assert _sum_tree(lib, [a, a], [False, False]) == (br.g1_add(a, a), 1)
    assert _sum_tree(lib, [a, a], [False, True]) == (None, 1)
    assert _sum_tree(lib, [a], [False]) == (a, 0)
    assert _sum_tree(lib, [a, b, b, a], [False, False, True, True])[0] is None


def test_doubling_chain_horner(lib):
    """sum_j 2^(d j) P_j by Horner with the 28-bit doubling (from the top point down): against the
    textbook group law for several chain lengths, with identities among the points and after them"""
    rng = random.Random(6)
    for n, d in ((1, 3), (2, 1), (3, 16), (5, 7), (4, 17)):
        ks = [rng.randrange(1, br.R_MOD) for _ in range(n)]
        pts = _points(ks)
        if n >= 3:
            pts[1] = None
        arr = br.g1_pack(pts).view(np.uint32).reshape(-1)
        aff = np.zeros(2 * FW, dtype=np.uint32)
        lib.t28_horner(_u32(np.ascontiguousarray(arr)), n, d, _u32(aff))
        got = br.g1_unpack(aff.view(np.uint64).reshape(1, br.G1_WORDS))[0]
        want = None
        for p in pts:                      # first point is the most significant
            want = br.g1_mul(1 << d, want) if want is not None else None
            want = br.g1_add(want, p)
        assert got == want, (n, d)


def _affine_batch(lib, pts, dbl, base):
    arr = np.ascontiguousarray(br.g1_pack(pts).view(np.uint32).reshape(len(pts), 2 * FW))
    b = np.ascontiguousarray(br.g1_pack([base]).view(np.uint32).reshape(2 * FW))
    flags = np.array(dbl, dtype=np.int32)
    out = np.zeros((len(pts), 2 * FW), dtype=np.uint32)
    rc = lib.t28_affine_batch(_u32(arr), flags.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), len(pts), _u32(b), _u32(out))
    return rc, br.g1_unpack(out.view(np.uint64).reshape(len(pts), br.G1_WORDS))


def test_affine_additions_sharing_one_inversion(lib):
    """The table generator's level step - multiples k*B + h*B for a run of k, the doubling h*B + h*B
    among them - as affine additions behind one shared inversion, against the textbook group law;
    coordinates come out canonical (checked inside the host twin: codes 2 and 3); a run that holds
    a pair without a finite affine sum (equal points not flagged as a doubling, opposite points) is
    reported instead of computed"""
    rng = random.Random(8)
    B = br.g1_mul(rng.randrange(1, br.R_MOD), br.G1)
    h = 64
    base = br.g1_mul(h, B)
    ks = list(range(1, 41)) + [h]
    pts = [br.g1_mul(k, B) for k in ks]
    rc, got = _affine_batch(lib, pts, [k == h for k in ks], base)
    assert rc == 0
    assert got == [br.g1_mul(k + h, B) for k in ks]
    # one element, and the doubling alone
    rc, got = _affine_batch(lib, pts[:1], [False], base)
    assert rc == 0 and got == [br.g1_mul(1 + h, B)]
    rc, got = _affine_batch(lib, [base], [True], base)
    assert rc == 0 and got == [br.g1_mul(2 * h, B)]
    # random pairs of unrelated points
    qs = _points([rng.randrange(1, br.R_MOD) for _ in range(12)])
    rc, got = _affine_batch(lib, qs, [False] * len(qs), base)
    assert rc == 0 and got == [br.g1_add(q, base) for q in qs]
    # no finite affine sum: the same point without the doubling flag, and the opposite point
    assert _affine_batch(lib, pts[:3] + [base], [False] * 4, base)[0] == 1
    assert _affine_batch(lib, [br.g1_neg(base)] + pts[:3], [False] * 4, base)[0] == 1
