"""ctypes binding of the CPU oracle (oracle/libgrape_oracle.so) for the test-suite and the
benchmark's cpu_baseline leg.  The oracle is test infrastructure, never a product path."""
import ctypes
import os
import subprocess
import numpy as np

from bigref import FP_LIMBS as FPL, G1_WORDS as G1W

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_LIB = None

u64p = ctypes.POINTER(ctypes.c_uint64)
u32p = ctypes.POINTER(ctypes.c_uint32)
i32p = ctypes.POINTER(ctypes.c_int32)
i64p = ctypes.POINTER(ctypes.c_int64)


def lib():
    global _LIB
    if _LIB is None:
        import bigref
        name = "libgrape_oracle_bn254.so" if bigref.CURVE == "bn254" else "libgrape_oracle.so"
        path = os.path.join(_ORACLE_DIR, name)
        if not os.path.exists(path):
            subprocess.check_call(["make", "-C", _ORACLE_DIR, "-s"])
        _LIB = ctypes.CDLL(path)
        _LIB.orc_num_threads.restype = ctypes.c_int
        _LIB.orc_log2.restype = ctypes.c_uint32
        _LIB.orc_log2.argtypes = [ctypes.c_uint32]
        _LIB.orc_g1_on_curve.restype = ctypes.c_int
        _LIB.orc_prove_matmul.restype = ctypes.c_int
        _LIB.orc_tlookup_prove.restype = ctypes.c_int
    return _LIB


def P(a, ty=u64p):
    """pointer to a C-contiguous numpy array (or None)."""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ty)


def c64(x):
    return ctypes.c_uint64(int(x))


def c32(x):
    return ctypes.c_uint32(int(x))


def ci32(x):
    return ctypes.c_int32(int(x))


def _bin(name, a, b, width=4):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    b = np.ascontiguousarray(b, dtype=np.uint64)
    r = np.zeros(width, dtype=np.uint64)
    getattr(lib(), name)(P(r), P(a), P(b))
    return r


def _un(name, a, width=4):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    r = np.zeros(width, dtype=np.uint64)
    getattr(lib(), name)(P(r), P(a))
    return r


def fr_add(a, b): return _bin("orc_fr_add", a, b)
def fr_sub(a, b): return _bin("orc_fr_sub", a, b)
def fr_mul(a, b): return _bin("orc_fr_mul", a, b)
def fr_neg(a): return _un("orc_fr_neg", a)
def fr_inv(a): return _un("orc_fr_inv", a)
def fp_add(a, b): return _bin("orc_fp_add", a, b, FPL)
def fp_sub(a, b): return _bin("orc_fp_sub", a, b, FPL)
def fp_mul(a, b): return _bin("orc_fp_mul", a, b, FPL)
def fp_neg(a): return _un("orc_fp_neg", a, FPL)
def fp_inv(a): return _un("orc_fp_inv", a, FPL)


def vec2(name, a, b):
    a = np.ascontiguousarray(a, dtype=np.uint64).reshape(-1, 4)
    b = np.ascontiguousarray(b, dtype=np.uint64).reshape(-1, 4)
    r = np.zeros_like(a)
    getattr(lib(), name)(P(r), P(a), P(b), c64(a.shape[0]))
    return r


def vec1(name, a):
    a = np.ascontiguousarray(a, dtype=np.uint64).reshape(-1, 4)
    r = np.zeros_like(a)
    getattr(lib(), name)(P(r), P(a), c64(a.shape[0]))
    return r


def vec_bcast(name, a, x):
    a = np.ascontiguousarray(a, dtype=np.uint64).reshape(-1, 4)
    x = np.ascontiguousarray(x, dtype=np.uint64).reshape(4)
    r = np.zeros_like(a)
    getattr(lib(), name)(P(r), P(a), P(x), c64(a.shape[0]))
    return r


def from_i32(x):
    x = np.ascontiguousarray(x, dtype=np.int32).reshape(-1)
    r = np.zeros((x.shape[0], 4), dtype=np.uint64)
    lib().orc_fr_vec_from_i32(P(r), P(x, i32p), c64(x.shape[0]))
    return r


def from_u32(x):
    x = np.ascontiguousarray(x, dtype=np.uint32).reshape(-1)
    r = np.zeros((x.shape[0], 4), dtype=np.uint64)
    lib().orc_fr_vec_from_u32(P(r), P(x, u32p), c64(x.shape[0]))
    return r


def fr_sum(a):
    a = np.ascontiguousarray(a, dtype=np.uint64).reshape(-1, 4)
    r = np.zeros(4, dtype=np.uint64)
    lib().orc_fr_sum(P(r), P(a), c64(a.shape[0]))
    return r


def partial_eval(t, N, x, c, idx, gap):
    """returns the whole (mutated) buffer; the result occupies the first N/c elements."""
    t = np.array(t, dtype=np.uint64).reshape(-1, 4)
    x = np.ascontiguousarray(x, dtype=np.uint64).reshape(-1, 4)
    lib().orc_fr_partial_eval(P(t), c64(N), P(x), c32(c), c32(idx), c32(gap))
    return t


def mle_eval(t, u):
    t = np.array(t, dtype=np.uint64).reshape(-1, 4)
    u = np.ascontiguousarray(u, dtype=np.uint64).reshape(-1, 4)
    r = np.zeros(4, dtype=np.uint64)
    lib().orc_fr_mle_eval(P(r), P(t), c64(t.shape[0]), P(u), c32(u.shape[0]))
    return r


def g1_generator():
    r = np.zeros(G1W, dtype=np.uint64)
    lib().orc_g1_generator(P(r))
    return r


def g1_make_generators(k_plain):
    k = np.ascontiguousarray(k_plain, dtype=np.uint64).reshape(-1, 4)
    r = np.zeros((k.shape[0], G1W), dtype=np.uint64)
    lib().orc_g1_make_generators(P(r), P(k), c64(k.shape[0]))
    return r


def g1_table(gens, W):
    gens = np.ascontiguousarray(gens, dtype=np.uint64).reshape(-1, G1W)
    n = gens.shape[0]
    r = np.zeros((W * n, G1W), dtype=np.uint64)
    lib().orc_g1_table(P(r), P(gens), c64(n), c32(W))
    return r


def commit_i32(scalars, table, rowlen, npoints):
    s = np.ascontiguousarray(scalars, dtype=np.int32).reshape(-1)
    table = np.ascontiguousarray(table, dtype=np.uint64)
    rows = s.shape[0] // rowlen
    r = np.zeros((rows, G1W), dtype=np.uint64)
    lib().orc_commit_i32(P(r), P(s, i32p), P(table), c64(s.shape[0]), c32(rowlen), c64(npoints))
    return r


def commit_fr(scalars_mont, table, rowlen, npoints):
    s = np.ascontiguousarray(scalars_mont, dtype=np.uint64).reshape(-1, 4)
    table = np.ascontiguousarray(table, dtype=np.uint64)
    rows = s.shape[0] // rowlen
    r = np.zeros((rows, G1W), dtype=np.uint64)
    lib().orc_commit_fr(P(r), P(s), P(table), c64(s.shape[0]), c32(rowlen), c64(npoints))
    return r


def msm_naive_i64(scalars, gens):
    s = np.ascontiguousarray(scalars, dtype=np.int64).reshape(-1)
    gens = np.ascontiguousarray(gens, dtype=np.uint64).reshape(-1, G1W)
    r = np.zeros(G1W, dtype=np.uint64)
    lib().orc_msm_naive_i64(P(r), P(s, i64p), P(gens), c64(s.shape[0]))
    return r


def prove_matmul(A, B, L, N, M, K, u, v, claim):
    """returns (status, transcript[rounds,4,4], final_claim, A_claim, B_claim)."""
    A = np.array(A, dtype=np.uint64).reshape(-1, 4)
    B = np.array(B, dtype=np.uint64).reshape(-1, 4)
    u = np.ascontiguousarray(u, dtype=np.uint64).reshape(-1, 4)
    v = np.ascontiguousarray(v, dtype=np.uint64).reshape(-1, 4)
    claim = np.array(claim, dtype=np.uint64).reshape(4)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    ac = np.zeros(4, dtype=np.uint64)
    bc = np.zeros(4, dtype=np.uint64)
    st = lib().orc_prove_matmul(P(A), P(B), c32(L), c32(N), c32(M), c32(K), P(u), c32(u.shape[0]),
                                P(v), c32(v.shape[0]), P(claim), P(tr), ctypes.byref(nr), P(ac), P(bc))
    return st, tr[: nr.value].copy(), claim, ac, bc


def prove_elemul(A, B, L, M, N, u, v, claim):
    """returns (status, transcript[rounds,4,4], final_claim, A_claim, B_claim)."""
    A = np.array(A, dtype=np.uint64).reshape(-1, 4)
    B = np.array(B, dtype=np.uint64).reshape(-1, 4)
    u = np.ascontiguousarray(u, dtype=np.uint64).reshape(-1, 4)
    v = np.ascontiguousarray(v, dtype=np.uint64).reshape(-1, 4)
    claim = np.array(claim, dtype=np.uint64).reshape(4)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    ac = np.zeros(4, dtype=np.uint64)
    bc = np.zeros(4, dtype=np.uint64)
    st = lib().orc_prove_elemul(P(A), P(B), c32(L), c32(M), c32(N), P(u), c32(u.shape[0]), P(v), c32(v.shape[0]),
                                P(claim), P(tr), ctypes.byref(nr), P(ac), P(bc))
    return st, tr[: nr.value].copy(), claim, ac, bc


def combine_claims(X, claims, u_rows, v):
    """returns (status, transcript[nv,4,4], X(v))."""
    X = np.array(X, dtype=np.uint64).reshape(-1, 4)
    claims = np.ascontiguousarray(claims, dtype=np.uint64).reshape(-1, 4)
    v = np.ascontiguousarray(v, dtype=np.uint64).reshape(-1, 4)
    u = np.ascontiguousarray(u_rows, dtype=np.uint64).reshape(claims.shape[0], v.shape[0], 4)
    tr = np.zeros((max(v.shape[0], 1), 4, 4), dtype=np.uint64)
    ret = np.zeros(4, dtype=np.uint64)
    st = lib().orc_combine_claims(P(X), c32(X.shape[0]), P(claims), c32(claims.shape[0]), P(u), P(v), c32(v.shape[0]), P(tr), P(ret))
    return st, tr[: v.shape[0]].copy(), ret


def histogram(vals_mont, low, length):
    v = np.ascontiguousarray(vals_mont, dtype=np.uint64).reshape(-1, 4)
    h = np.zeros(length, dtype=np.uint32)
    lib().orc_histogram(P(h, u32p), P(v), c64(v.shape[0]), ci32(low), c32(length))
    return h


def tlookup_prep(vals_mont, low, length):
    v = np.ascontiguousarray(vals_mont, dtype=np.uint64).reshape(-1, 4)
    m = np.zeros((length, 4), dtype=np.uint64)
    lib().orc_tlookup_prep(P(m), P(v), c64(v.shape[0]), ci32(low), c32(length))
    return m


def tlookup_init(low, length, beta, map_mont=None, r=None):
    T = np.zeros((length, 4), dtype=np.uint64)
    B = np.zeros((length, 4), dtype=np.uint64)
    beta = np.ascontiguousarray(beta, dtype=np.uint64).reshape(4)
    if map_mont is not None:
        map_mont = np.ascontiguousarray(map_mont, dtype=np.uint64).reshape(-1, 4)
        r = np.ascontiguousarray(r, dtype=np.uint64).reshape(4)
    lib().orc_tlookup_init(P(T), P(B), ci32(low), c32(length), P(beta), P(map_mont), P(r))
    return T, B


def tlookup_prove(S, T, B, m, alpha, beta, u, v):
    """returns (status, transcript[rounds,4,4], S_claim)."""
    S = np.array(S, dtype=np.uint64).reshape(-1, 4)
    T = np.ascontiguousarray(T, dtype=np.uint64).reshape(-1, 4)
    B = np.ascontiguousarray(B, dtype=np.uint64).reshape(-1, 4)
    m = np.ascontiguousarray(m, dtype=np.uint64).reshape(-1, 4)
    alpha = np.ascontiguousarray(alpha, dtype=np.uint64).reshape(4)
    beta = np.ascontiguousarray(beta, dtype=np.uint64).reshape(4)
    u = np.ascontiguousarray(u, dtype=np.uint64).reshape(-1, 4)
    v = np.ascontiguousarray(v, dtype=np.uint64).reshape(-1, 4)
    assert u.shape == v.shape
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    sc = np.zeros(4, dtype=np.uint64)
    st = lib().orc_tlookup_prove(P(S), c64(S.shape[0]), P(T), P(B), P(m), c32(T.shape[0]), P(alpha),
                                 P(beta), P(u), P(v), c32(u.shape[0]), P(tr), ctypes.byref(nr), P(sc))
    return st, tr[: nr.value].copy(), sc
