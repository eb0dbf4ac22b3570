"""ctypes binding of the C entry points over the C++ host classes (grape_amd/host/host_capi.h)."""
import ctypes
import os
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
from ._capi import CURVE, FP_WORDS
LIB_PATH = os.path.join(_HERE, "host", "libgrape_host_bn254.so" if CURVE == "bn254" else "libgrape_host.so")
G1W = FP_WORDS              # u64 words of an affine point (2 coordinates of FP_WORDS / 2)
_lib = None

NAMES = ["grape_host_last_error", "grape_host_seed", "grape_host_last_prove_seconds", "grape_host_last_commit_seconds", "grape_host_set_indexed_commit", "grape_host_set_input_format", "grape_host_set_int_folds", "grape_host_prove_matmul", "grape_host_prove_elemul",
         "grape_host_combine_claims", "grape_host_mle_eval", "grape_host_hyrax_commit_i32", "grape_host_hyrax_commit_fr",
         "grape_host_hyrax_open_verify", "grape_host_hyrax_open", "grape_host_tlookup_range_prove", "grape_host_tlookup_mapping_prove", "grape_host_tlookup_mapping_prove_ex",
         "grape_host_fr_op", "grape_host_g1_mul_generator", "grape_host_bin_io", "grape_host_findsize", "grape_host_load_data",
         "grape_host_generate_data", "grape_host_single_commit", "grape_host_layer_witness_new", "grape_host_layer_witness_generate",
         "grape_host_layer_witness_names", "grape_host_layer_witness_tensor", "grape_host_layer_witness_save",
         "grape_host_layer_witness_free", "grape_host_witness_tables", "grape_host_to_float16"]


class HostError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HostError("%s not found: build it with `python grape_amd/host/build.py`" % LIB_PATH)
        from . import _capi
        _capi.load()                       # the kernel library first (dependency)
        lib = ctypes.CDLL(LIB_PATH)
        for n in NAMES:
            getattr(lib, n)
        lib.grape_host_last_error.restype = ctypes.c_char_p
        lib.grape_host_seed.argtypes = [ctypes.c_uint64]
        lib.grape_host_last_prove_seconds.restype = ctypes.c_double
        lib.grape_host_last_commit_seconds.restype = ctypes.c_double
        lib.grape_host_findsize.restype = ctypes.c_ulong
        lib.grape_host_to_float16.restype = ctypes.c_double
        lib.grape_host_to_float16.argtypes = [ctypes.c_double]
        lib.grape_host_findsize.argtypes = [ctypes.c_char_p]
        lib.grape_host_bin_io.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        lib.grape_host_load_data.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_uint32)]
        lib.grape_host_generate_data.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint32]
        _lib = lib
    return _lib


def set_indexed_commit(on):
    load().grape_host_set_indexed_commit(1 if on else 0)


def set_input_format(fmt):
    """0: tensor arguments are field elements (default); 1: int32 values that each call embeds itself"""
    if load().grape_host_set_input_format({"fr": 0, "i32": 1}[fmt]) != 0:
        raise HostError("unknown input format")


def set_int_folds(on):
    """with int32 inputs: openings and evaluations fold the integers directly (default) or embed them first"""
    load().grape_host_set_int_folds(1 if on else 0)


def last_commit_seconds():
    return load().grape_host_last_commit_seconds()


def last_prove_seconds():
    return load().grape_host_last_prove_seconds()


def _check(rc):
    if rc != 0:
        raise HostError(load().grape_host_last_error().decode())


def _hp(a):
    """pointer to a host numpy array (or None)"""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def _dp(t):
    return ctypes.c_void_p(t.data_ptr())


def _fr(a, n=None):
    a = np.ascontiguousarray(a, dtype=np.uint64).reshape(-1, 4)
    if n is not None:
        assert a.shape[0] == n
    return a


def prove_matmul(dA, dB, L, N, M, K, u, v, claim):
    lib = load()
    u, v = _fr(u), _fr(v)
    claim = np.array(claim, dtype=np.uint64).reshape(4)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    ac, bc = np.zeros(4, dtype=np.uint64), np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_prove_matmul(_dp(dA), _dp(dB), L, N, M, K, _hp(u), u.shape[0], _hp(v), v.shape[0], _hp(claim),
                                       _hp(tr), ctypes.byref(nr), _hp(ac), _hp(bc)))
    return tr[: nr.value].copy(), claim, ac, bc


def prove_elemul(dA, dB, L, M, N, u, v, claim):
    lib = load()
    u, v = _fr(u), _fr(v)
    claim = np.array(claim, dtype=np.uint64).reshape(4)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    ac, bc = np.zeros(4, dtype=np.uint64), np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_prove_elemul(_dp(dA), _dp(dB), L, M, N, _hp(u), u.shape[0], _hp(v), v.shape[0], _hp(claim),
                                       _hp(tr), ctypes.byref(nr), _hp(ac), _hp(bc)))
    return tr[: nr.value].copy(), claim, ac, bc


def combine_claims(dX, size, claims, us, v):
    lib = load()
    claims, v = _fr(claims), _fr(v)
    us = np.ascontiguousarray(us, dtype=np.uint64).reshape(claims.shape[0], v.shape[0], 4)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    res = np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_combine_claims(_dp(dX), size, _hp(claims), claims.shape[0], _hp(us), _hp(v), v.shape[0],
                                         _hp(tr), ctypes.byref(nr), _hp(res)))
    return tr[: nr.value].copy(), res


def mle_eval(dT, size, u):
    lib = load()
    u = _fr(u)
    out = np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_mle_eval(_dp(dT), size, _hp(u), u.shape[0], _hp(out)))
    return out


def hyrax_commit_i32(d_scalars, size, N, d_table, npoints, com_scale=16, layer_num=1):
    lib = load()
    rows = size // (N * com_scale)
    out = np.zeros((rows, G1W), dtype=np.uint64)
    _check(lib.grape_host_hyrax_commit_i32(_dp(d_scalars), size, N, _dp(d_table), npoints, com_scale, layer_num, _hp(out)))
    return out


def hyrax_commit_fr(d_scalars, size, N, d_table, npoints, com_scale=16, layer_num=1):
    lib = load()
    rows = size // (N * com_scale)
    out = np.zeros((rows, G1W), dtype=np.uint64)
    _check(lib.grape_host_hyrax_commit_fr(_dp(d_scalars), size, N, _dp(d_table), npoints, com_scale, layer_num, _hp(out)))
    return out


def hyrax_open_verify(d_tensor, size, N, d_table, npoints, eval_point, c, com_scale=16, layer_num=1):
    lib = load()
    pt = _fr(eval_point)
    c = _fr(c, 1)
    res = np.zeros(4, dtype=np.uint64)
    ok = ctypes.c_int(0)
    _check(lib.grape_host_hyrax_open_verify(_dp(d_tensor), size, N, _dp(d_table), npoints, com_scale, layer_num, _hp(pt),
                                            pt.shape[0], _hp(c), _hp(res), ctypes.byref(ok)))
    return res, bool(ok.value)


def hyrax_open(d_tensor, size, N, d_table, npoints, eval_point, c, com_scale=16, layer_num=1):
    """Hyrax::open of a copy of the tensor; returns the opened evaluation"""
    lib = load()
    pt = _fr(eval_point)
    c = _fr(c, 1)
    res = np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_hyrax_open(_dp(d_tensor), size, N, _dp(d_table), npoints, com_scale, layer_num, _hp(pt), pt.shape[0],
                                     _hp(c), _hp(res)))
    return res


def tlookup_range_prove(dS, D, low, length, alpha, u, v, d_table, npoints, com_scale, msm_size, want_commitments=False,
                        want_m=True):
    lib = load()
    alpha, u, v = _fr(alpha, 1), _fr(u), _fr(v)
    size = 1 << max(0, (length - 1).bit_length())
    m = np.zeros((size, 4), dtype=np.uint64) if want_m else None
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    sc = np.zeros(4, dtype=np.uint64)
    Dp = 1 << max(0, (D - 1).bit_length())
    comA = np.zeros((Dp // (msm_size * com_scale), G1W), dtype=np.uint64) if want_commitments else None
    logn = (size - 1).bit_length()
    mN = 1 << (logn // 2)
    comm = np.zeros((size // (mN * com_scale), G1W), dtype=np.uint64) if want_commitments else None
    ct = ctypes.c_double(0)
    _check(lib.grape_host_tlookup_range_prove(_dp(dS), D, low, length, _hp(alpha), _hp(u), _hp(v), u.shape[0], _dp(d_table),
                                              npoints, com_scale, msm_size, _hp(m), _hp(tr), ctypes.byref(nr), _hp(sc),
                                              _hp(comA), _hp(comm), ctypes.byref(ct)))
    return {"m": m, "transcript": tr[: nr.value].copy(), "S_claim": sc, "com_A": comA, "com_m": comm, "commit_s": ct.value}


def tlookup_mapping_prove(dS_in, dS_out, D, low, length, table, alpha, r, u, v, d_table, npoints, com_scale, msm_size):
    lib = load()
    alpha, r, u, v = _fr(alpha, 1), _fr(r, 1), _fr(u), _fr(v)
    table = np.ascontiguousarray(table, dtype=np.int32)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    sc = np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_tlookup_mapping_prove(_dp(dS_in), _dp(dS_out), D, low, length, _hp(table), _hp(alpha), _hp(r),
                                                _hp(u), _hp(v), u.shape[0], _dp(d_table), npoints, com_scale, msm_size,
                                                _hp(tr), ctypes.byref(nr), _hp(sc)))
    return tr[: nr.value].copy(), sc


def tlookup_mapping_prove_ex(dS_in, dS_out, D, low, length, table, alpha, r, u, v, d_table, npoints, com_scale, msm_size,
                             hot_min_count=0):
    """returns (transcript, S(v), com_A, entries with a table row, elements committed as full-width scalars,
    whether the rows were found in place from an earlier proof of the same lookup object)"""
    lib = load()
    alpha, r, u, v = _fr(alpha, 1), _fr(r, 1), _fr(u), _fr(v)
    table = np.ascontiguousarray(table, dtype=np.int32)
    tr = np.zeros((64, 4, 4), dtype=np.uint64)
    nr = ctypes.c_uint32(0)
    sc = np.zeros(4, dtype=np.uint64)
    Dp = 1 << max(0, (D - 1).bit_length())
    com_a = np.zeros((Dp // (msm_size * com_scale), G1W), dtype=np.uint64)
    stats = (ctypes.c_uint64 * 3)()
    _check(lib.grape_host_tlookup_mapping_prove_ex(_dp(dS_in), _dp(dS_out), D, low, length, _hp(table), _hp(alpha), _hp(r),
                                                   _hp(u), _hp(v), u.shape[0], _dp(d_table), npoints, com_scale, msm_size,
                                                   _hp(tr), ctypes.byref(nr), _hp(sc), hot_min_count, _hp(com_a), stats))
    return tr[: nr.value].copy(), sc, com_a, int(stats[0]), int(stats[1]), bool(stats[2])


def fr_op(op, a, b=None):
    lib = load()
    a = _fr(a, 1)
    b = _fr(b, 1) if b is not None else None
    out = np.zeros(4, dtype=np.uint64)
    _check(lib.grape_host_fr_op(op, _hp(a), _hp(b), _hp(out)))
    return out


def g1_mul_generator(k_mont):
    lib = load()
    k = _fr(k_mont, 1)
    out = np.zeros(G1W, dtype=np.uint64)
    _check(lib.grape_host_g1_mul_generator(_hp(k), _hp(out)))
    return out


# ------------------------------------------------------------------ file helpers (ioutils.hpp)
def savebin(filename, ptr, size, is_gpu=True):
    _check(load().grape_host_bin_io(0, os.fsencode(filename), ctypes.c_void_p(ptr), size, 1 if is_gpu else 0))


def loadbin(filename, ptr, size, is_gpu=True):
    _check(load().grape_host_bin_io(1, os.fsencode(filename), ctypes.c_void_p(ptr), size, 1 if is_gpu else 0))


def findsize(filename):
    return load().grape_host_findsize(os.fsencode(filename))


def load_data(filename):
    """int32 file -> (device pointer, element count); release the pointer with grape_free"""
    p, n = ctypes.c_void_p(0), ctypes.c_uint32(0)
    _check(load().grape_host_load_data(os.fsencode(filename), ctypes.byref(p), ctypes.byref(n)))
    return p.value, n.value


def generate_data(size):
    p = ctypes.c_void_p(0)
    _check(load().grape_host_generate_data(ctypes.byref(p), size))
    return p.value


def single_commit(d_scalars, N, d_table, npoints):
    out = np.zeros(G1W, dtype=np.uint64)
    _check(load().grape_host_single_commit(_dp(d_scalars), N, _dp(d_table), npoints, _hp(out)))
    return out


# ------------------------------------------------------------------ witness generator
WEIGHT_ORDER = ("Q", "K", "V", "O", "gate", "up", "down", "NormFirst", "NormSecond")


def witness_tables():
    """(exp table, SiLU table) as numpy int32 arrays, from the C++ generator"""
    e = np.zeros(1 << 20, dtype=np.int32)
    s = np.zeros(1 << 19, dtype=np.int32)
    _check(load().grape_host_witness_tables(_hp(e), _hp(s)))
    return e, s


def to_float16(x):
    return load().grape_host_to_float16(float(x))


class LayerWitness:
    """handle on the C++ LayerWitness; tensors come back as torch int32 views of device memory that
    stay valid while this object lives"""

    def __init__(self, seq_len, dim, hidden):
        self._h = ctypes.c_void_p()
        self.shape = (seq_len, dim, hidden)
        _check(load().grape_host_layer_witness_new(ctypes.byref(self._h), ctypes.c_uint32(seq_len), ctypes.c_uint32(dim), ctypes.c_uint32(hidden)))

    def generate(self, x, weights, exp_table, silu_table, eps=1e-5):
        """x, weights[name], tables: contiguous CUDA int32 tensors"""
        self._keep = (x, dict(weights), exp_table, silu_table)
        ptrs = (ctypes.c_void_p * 9)(*[weights[k].data_ptr() for k in WEIGHT_ORDER])
        _check(load().grape_host_layer_witness_generate(self._h, _dp(x), ptrs, _dp(exp_table), _dp(silu_table), ctypes.c_double(eps)))

    def names(self):
        buf = ctypes.create_string_buffer(1 << 14)
        _check(load().grape_host_layer_witness_names(self._h, buf, ctypes.c_size_t(len(buf))))
        return [n for n in buf.value.decode().split("\n") if n]

    def tensor(self, name):
        """host copy (numpy int32, flat)"""
        p = ctypes.c_void_p()
        n = ctypes.c_size_t(0)
        _check(load().grape_host_layer_witness_tensor(self._h, name.encode(), ctypes.byref(p), ctypes.byref(n)))
        out = np.zeros(n.value, dtype=np.int32)
        from . import _capi
        _capi.check(_capi.load().grape_memcpy_d2h(_hp(out), p, n.value * 4, None))
        return out

    def device_ptr(self, name):
        p = ctypes.c_void_p()
        n = ctypes.c_size_t(0)
        _check(load().grape_host_layer_witness_tensor(self._h, name.encode(), ctypes.byref(p), ctypes.byref(n)))
        return p.value, n.value

    def save(self, data_dir, group):
        _check(load().grape_host_layer_witness_save(self._h, data_dir.encode(), ctypes.c_uint32(group)))

    def close(self):
        if self._h:
            _check(load().grape_host_layer_witness_free(self._h))
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
