"""Thin Python helpers over the C ABI for tests and benchmarks.

Device memory comes from torch (plumbing only): an Fr tensor of n elements is a CUDA int32
tensor of shape (n, 8) whose bytes are the fr_t array; affine G1 points are (n, 24) for
BLS12-381 and (n, 16) for BN254.  Host-side values travel as numpy uint64 arrays of shape
(n, 4) / (n, 12 or 8).
Every helper enqueues on torch's current stream.
"""
import ctypes
import numpy as np
import torch

from . import _capi

_initialised = False


def init(device=0):
    global _initialised
    lib = _capi.load()
    if not _initialised:
        torch.cuda.set_device(device)
        _capi.check(lib.grape_init(device))
        _initialised = True
    return lib


def _s():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def sync():
    _capi.check(init().grape_stream_sync(_s()))


# ------------------------------------------------------------------ host <-> device
def to_dev(a):
    """numpy array (any integer dtype) -> device tensor viewing the same bytes as int32."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint64:
        t = torch.from_numpy(a.view(np.int64)).cuda().view(torch.int32)
        return t.reshape(a.shape[0], -1) if a.ndim == 2 else t
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def fr_to_host(t):
    """device (n,8) int32 -> numpy uint64 (n,4)."""
    return t.detach().cpu().contiguous().numpy().view(np.uint64).reshape(-1, 4)


def g1_to_host(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint64).reshape(-1, _capi.FP_WORDS)


def fr_empty(n):
    return torch.empty((max(int(n), 0), 8), dtype=torch.int32, device="cuda")


def g1_empty(n):
    return torch.empty((int(n), 2 * _capi.FP_WORDS), dtype=torch.int32, device="cuda")


# ------------------------------------------------------------------ Fr tensors
def _ew(name, a, b, out=None):
    lib = init()
    out = fr_empty(a.shape[0]) if out is None else out
    _capi.check(getattr(lib, name)(_p(out), _p(a), _p(b), a.shape[0], _s()))
    return out


def fr_add(a, b, out=None): return _ew("grape_fr_add", a, b, out)
def fr_sub(a, b, out=None): return _ew("grape_fr_sub", a, b, out)
def fr_mul(a, b, out=None): return _ew("grape_fr_mul", a, b, out)
def fr_bcast_add(a, x, out=None): return _ew("grape_fr_bcast_add", a, x, out)
def fr_bcast_mul(a, x, out=None): return _ew("grape_fr_bcast_mul", a, x, out)


def fr_from_i32(x):
    lib = init()
    out = fr_empty(x.numel())
    _capi.check(lib.grape_fr_from_i32(_p(out), _p(x), x.numel(), _s()))
    return out


def fr_from_u32(x):
    lib = init()
    out = fr_empty(x.numel())
    _capi.check(lib.grape_fr_from_u32(_p(out), _p(x), x.numel(), _s()))
    return out


def fr_to_mont(a):
    lib = init()
    out = fr_empty(a.shape[0])
    _capi.check(lib.grape_fr_to_mont(_p(out), _p(a), a.shape[0], _s()))
    return out


def fr_from_mont(a):
    lib = init()
    out = fr_empty(a.shape[0])
    _capi.check(lib.grape_fr_from_mont(_p(out), _p(a), a.shape[0], _s()))
    return out


def fr_batch_inverse(a, out=None):
    lib = init()
    out = fr_empty(a.shape[0]) if out is None else out
    _capi.check(lib.grape_fr_batch_inverse(_p(out), _p(a), a.shape[0], _s()))
    return out


def fr_shift_inverse(a, beta, out=None):
    lib = init()
    out = fr_empty(a.shape[0]) if out is None else out
    _capi.check(lib.grape_fr_shift_inverse(_p(out), _p(a), _p(beta), a.shape[0], _s()))
    return out


def fr_sum(a, n=None):
    lib = init()
    out = fr_empty(1)
    n = a.shape[0] if n is None else n
    _capi.check(lib.grape_fr_sum(_p(out), _p(a), n, _s()))
    return out


def fr_sum_by_dim(a, rows, dim):
    lib = init()
    out = fr_empty(rows * dim)
    _capi.check(lib.grape_fr_sum_by_dim(_p(out), _p(a), rows, dim, _s()))
    return out


def fr_pad(a, N, pad_N, pad_size, pad_val):
    lib = init()
    out = fr_empty(pad_size)
    _capi.check(lib.grape_fr_pad(_p(out), _p(a), N, pad_N, pad_size, _p(pad_val), _s()))
    return out


def i32_pad(a, N, pad_N, pad_size):
    lib = init()
    out = torch.empty(pad_size, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_i32_pad(_p(out), _p(a), N, pad_N, pad_size, _s()))
    return out


def fr_fold(t, N, x, c, idx, gap):
    """in place; the result is t[: N // c]."""
    lib = init()
    _capi.check(lib.grape_fr_fold(_p(t), N, _p(x), c, idx, gap, _s()))
    return t


# ------------------------------------------------------------------ sumcheck / tlookup
def fr_fold_i32(ints, N, x, c, idx, gap):
    """fold of the integer tensor `ints` (as its embedding into Fr); returns the [N/(c*gap)][gap] result"""
    lib = init()
    out = fr_empty(max(1, lib.grape_fr_fold_i32_elems(N, c, gap)))
    _capi.check(lib.grape_fr_fold_i32(_p(out), _p(ints), N, _p(x), c, idx, gap, _s()))
    return out[: N // (c * gap) * gap]


def sumcheck_round2_claim(A, B, in_size, out_size, v, claim):
    """claim (device, one element) is replaced by the next round's claim; returns the three sums"""
    lib = init()
    sums = fr_empty(3)
    _capi.check(lib.grape_sumcheck_round2_claim(_p(A), _p(B), in_size, out_size, _p(v), _p(claim), _p(sums), _s()))
    return sums


def sumcheck_round2(A, B, in_size, out_size, v):
    lib = init()
    sums = fr_empty(3)
    _capi.check(lib.grape_sumcheck_round2(_p(A), _p(B), in_size, out_size, _p(v), _p(sums), _s()))
    return sums


def sumcheck_round2_tail(A, B, in_size, rounds, v, v_end_index):
    """rounds from in_size (<= 512) down, challenges v[v_end_index - 1], v[v_end_index - 2], ...;
    returns the sums as a (3 * rounds, 8) tensor"""
    lib = init()
    sums = fr_empty(3 * max(rounds, 1))
    v_end = v.data_ptr() + 32 * v_end_index
    _capi.check(lib.grape_sumcheck_round2_tail(_p(A), _p(B), in_size, rounds, ctypes.c_void_p(v_end), _p(sums), _s()))
    return sums


def sumcheck_round2_coeffs(A, B, a, b, c, in_size, out_size, v, want_sums=True):
    lib = init()
    sums = fr_empty(3) if want_sums else None
    _capi.check(lib.grape_sumcheck_round2_coeffs(_p(A), _p(B), _p(a), _p(b), _p(c), in_size, out_size, _p(v), _p(sums), _s()))
    return sums


def sumcheck_round1(X, a, b, in_size, out_size, v):
    lib = init()
    _capi.check(lib.grape_sumcheck_round1(_p(X), _p(a), _p(b), in_size, out_size, _p(v), _s()))


def tlookup_hist(vals, low, length, hist=None):
    lib = init()
    if hist is None:
        hist = torch.zeros(length, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_tlookup_hist(_p(hist), _p(vals), vals.shape[0], low, length, _s()))
    return hist


def tlookup_index(vals, low, length):
    lib = init()
    out = torch.empty(vals.shape[0], dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_tlookup_index(_p(out), _p(vals), vals.shape[0], low, length, _s()))
    return out


def tlookup_hist_index(idx1, length, hist=None):
    lib = init()
    if hist is None:
        hist = torch.zeros(length, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_tlookup_hist_index(_p(hist), _p(idx1), idx1.shape[0], length, _s()))
    return hist


def tlookup_index_inverse(key, low, B, cmp=None, cmp_table=None, write_A=True):
    """returns (idx1, A, mismatches); write_A=False: indices and the count only (A is None)"""
    lib = init()
    n = key.shape[0]
    idx1 = torch.empty(n, dtype=torch.int32, device="cuda")
    A = fr_empty(n) if write_A else None
    mm = ctypes.c_size_t(0)
    _capi.check(lib.grape_tlookup_index_inverse(_p(idx1), _p(A), _p(key), n, low, B.shape[0], _p(B),
                                                _p(cmp) if cmp is not None else None, _p(cmp_table) if cmp_table is not None else None,
                                                ctypes.byref(mm), _s()))
    return idx1, A, mm.value


def fr_axpy(x, r, y, out=None):
    lib = init()
    out = fr_empty(x.shape[0]) if out is None else out
    _capi.check(lib.grape_fr_axpy(_p(out), _p(x), _p(r), _p(y), x.shape[0], _s()))
    return out


def tlookup_hot_select(hist, min_count, max_hot):
    """returns (slot1, hot_list[:n_hot], n_hot, cold_elements)"""
    lib = init()
    length = hist.shape[0]
    slot1 = torch.empty(length, dtype=torch.int32, device="cuda")
    hot = torch.empty(length, dtype=torch.int32, device="cuda")
    info = (ctypes.c_uint64 * 2)()
    _capi.check(lib.grape_tlookup_hot_select(_p(hist), length, min_count, max_hot, _p(slot1), _p(hot), info, _s()))
    return slot1, hot[:int(info[0])], int(info[0]), int(info[1])


def tlookup_hot_index(idx1, slot1):
    lib = init()
    out = torch.empty_like(idx1)
    _capi.check(lib.grape_tlookup_hot_index(_p(out), _p(idx1), idx1.shape[0], _p(slot1), slot1.shape[0], _s()))
    return out


def fr_mask_cold(X, hot1):
    lib = init()
    out = fr_empty(X.shape[0])
    _capi.check(lib.grape_fr_mask_cold(_p(out), _p(X), _p(hot1), X.shape[0], _s()))
    return out


def fr_gather(src, index_list):
    lib = init()
    out = fr_empty(index_list.shape[0])
    _capi.check(lib.grape_fr_gather(_p(out), _p(src), _p(index_list), index_list.shape[0], _s()))
    return out


def commit_fr_sparse(scalars, skip, rowlen, table, N, c, nw, K):
    lib = init()
    size = scalars.shape[0]
    out = g1_empty(size // rowlen)
    _capi.check(lib.grape_commit_fr_sparse(_p(out), _p(scalars), _p(skip), size, rowlen, _p(table), N, c, nw, K, _s()))
    return out


def g1_affine_add(a, b):
    lib = init()
    out = g1_empty(a.shape[0])
    _capi.check(lib.grape_g1_affine_add(_p(out), _p(a), _p(b), a.shape[0], _s()))
    return out


def tlookup_inverse_by_table(S, idx1, T, B, A=None):
    """returns (A, mismatches)"""
    lib = init()
    A = fr_empty(S.shape[0]) if A is None else A
    mm = ctypes.c_size_t(0)
    _capi.check(lib.grape_tlookup_inverse_by_table(_p(A), _p(S), _p(idx1), _p(T), _p(B), S.shape[0], T.shape[0], ctypes.byref(mm), _s()))
    return A, mm.value


def tlookup_init(low, length, beta, map_t=None, r=None):
    lib = init()
    T, B = fr_empty(length), fr_empty(length)
    _capi.check(lib.grape_tlookup_init(_p(T), _p(B), low, length, _p(beta), _p(map_t), _p(r), _s()))
    return T, B


def tlookup_poly(A, S, beta, n_out):
    lib = init()
    o = [fr_empty(n_out) for _ in range(3)]
    _capi.check(lib.grape_tlookup_poly(_p(A), _p(S), _p(beta), _p(o[0]), _p(o[1]), _p(o[2]), n_out, _s()))
    return o


def tlookup_poly_sum(A, n_out):
    lib = init()
    o = [fr_empty(n_out) for _ in range(2)]
    _capi.check(lib.grape_tlookup_poly_sum(_p(A), _p(o[0]), _p(o[1]), n_out, _s()))
    return o


def tlookup_round_sums(A, S, beta, eq, n_out):
    lib = init()
    sums = fr_empty(8)
    _capi.check(lib.grape_tlookup_round_sums(_p(A), _p(S), _p(beta), _p(eq), n_out, _p(sums), _s()))
    return sums


def tlookup_table_round(B, T, m, beta, eq, n_out, v):
    """one launch: 5 weighted sums over (B, T + beta), 3 sums over (m, B), then B, T, m folded in place by v"""
    lib = init()
    sums = fr_empty(8)
    _capi.check(lib.grape_tlookup_table_round(_p(B), _p(T), _p(m), _p(beta), _p(eq), n_out, _p(v), _p(sums), _s()))
    return sums


def tlookup_mb_sums(m, B, n_out):
    lib = init()
    sums = fr_empty(3)
    _capi.check(lib.grape_tlookup_mb_sums(_p(m), _p(B), n_out, _p(sums), _s()))
    return sums


def eq_table(u, nu=None):
    lib = init()
    nu = u.shape[0] if nu is None else nu
    e = fr_empty(1 << nu)
    _capi.check(lib.grape_eq_table(_p(e), _p(u) if nu else None, nu, _s()))
    return e


def eq_table_halve(e, n_out):
    lib = init()
    _capi.check(lib.grape_eq_table_halve(_p(e), n_out, _s()))


def eq_pyramid(u, nu=None):
    """all levels of eq(u[0..j-1], .) in one tensor; level j = out[2^j - 1 : 2^(j+1) - 1]"""
    lib = init()
    nu = u.shape[0] if nu is None else nu
    pyr = fr_empty(lib.grape_eq_pyramid_elems(nu))
    _capi.check(lib.grape_eq_pyramid(_p(pyr), _p(u) if nu else None, nu, _s()))
    return pyr


def wround2(A, S, beta, e, in_size, n_out, v, plain_sums=False, rowlen=1, rowpad=1, inverse_pair=False, no_middle=False):
    """inverse_pair: the caller states A * (S + beta) = 1 at every index and weights that sum to one;
    no_middle: the middle coefficient is left out (sums[1] = 0) for a caller that takes it from the round's claim"""
    lib = init()
    sums = fr_empty(5 if plain_sums else 3)
    mode = 3 if no_middle else (2 if inverse_pair else (1 if plain_sums else 0))
    _capi.check(lib.grape_wround2(_p(A), _p(S), _p(beta), _p(e), in_size, n_out, rowlen, rowpad, _p(v), mode,
                                  _p(sums), _s()))
    return sums


def wround2_split(A, S, beta, e, in_size, n_out, v, plain_sums=False, rowlen=1, rowpad=1, inverse_pair=False, no_middle=False,
                  table=True):
    """wround2 through its two halves: the table of the challenge's multiples (table=True and n_out >= 2^16), the
    pass over the operands into a work buffer of the caller, the finishing of the sums"""
    lib = init()
    sums = fr_empty(5 if plain_sums else 3)
    mode = 3 if no_middle else (2 if inverse_pair else (1 if plain_sums else 0))
    partial = torch.empty(lib.grape_wround2_partial_bytes(n_out) // 4, dtype=torch.int32, device="cuda")
    tab = None
    if table and n_out >= (1 << 16):
        tab = torch.empty(100, dtype=torch.int32, device="cuda")
        _capi.check(lib.grape_fold_tables(_p(tab), _p(v), 1, _s()))
    _capi.check(lib.grape_wround2_queue(_p(A), _p(S), _p(beta), _p(e), in_size, n_out, rowlen, rowpad, _p(v), mode,
                                        _p(tab), _p(partial), _s()))
    _capi.check(lib.grape_wround2_finish(_p(sums), _p(partial), n_out, mode, _s()))
    return sums


def wround2_first_indexed(S, idx1, B, beta, e, n_out, v):
    """first round of a lookup whose logUp tensor A = B[idx1 - 1] was never written out; returns (sums, folded A)"""
    lib = init()
    sums = fr_empty(5)
    A = fr_empty(n_out)
    partial = torch.empty(lib.grape_wround2_partial_bytes(n_out) // 4, dtype=torch.int32, device="cuda")
    tab = torch.empty(100, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_fold_tables(_p(tab), _p(v), 1, _s()))
    _capi.check(lib.grape_wround2_queue_indexed(_p(A), _p(S), _p(idx1), _p(B), B.shape[0], _p(beta), _p(e), n_out, _p(v), _p(tab),
                                                _p(partial), _s()))
    _capi.check(lib.grape_wround2_finish(_p(sums), _p(partial), n_out, 2, _s()))
    return sums, A


def sumcheck_round2_seg(A, B, in_size, out_size, seglen, e, v):
    lib = init()
    sums = fr_empty(3)
    _capi.check(lib.grape_sumcheck_round2_seg(_p(A), _p(B), in_size, out_size, seglen, _p(e), _p(v), _p(sums), _s()))
    return sums


def wsum1_multi(X, tables, in_size, n_out):
    lib = init()
    sums = fr_empty(2 * len(tables))
    arr = (ctypes.c_void_p * len(tables))(*[t.data_ptr() for t in tables])
    _capi.check(lib.grape_wsum1_multi(_p(X), arr, len(tables), in_size, n_out, _p(sums), _s()))
    return sums


def fr_fold_msb_multi(tensors, n_out, v):
    lib = init()
    arr = (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])
    _capi.check(lib.grape_fr_fold_msb_multi(arr, len(tensors), n_out, _p(v), _s()))


# ------------------------------------------------------------------ G1
def g1_generator():
    lib = init()
    out = np.zeros(_capi.FP_WORDS, dtype=np.uint64)
    _capi.check(lib.grape_g1_generator(out.ctypes.data_as(ctypes.c_void_p)))
    return out


def g1_make_generators(k_plain):
    """k_plain: numpy uint64 (n,4) canonical scalars -> device affine points (n,24)."""
    lib = init()
    k = to_dev(np.ascontiguousarray(k_plain, dtype=np.uint64).reshape(-1, 4))
    base = to_dev(g1_generator().reshape(1, _capi.FP_WORDS))
    out = g1_empty(k.shape[0])
    _capi.check(lib.grape_g1_scalar_mul_base(_p(out), _p(k), _p(base), k.shape[0], _s()))
    return out


def g1_table_gen(gens, W):
    lib = init()
    n = gens.shape[0]
    out = g1_empty(W * n)
    _capi.check(lib.grape_g1_table_gen(_p(out), _p(gens), n, W, _s()))
    return out


# 32-bit words of a wide-table entry: 2 x 14 limbs padded to 32 (one cache line) on BLS12-381,
# 2 x 10 limbs stored dense on BN254
WIDE_ENTRY_WORDS = 20 if _capi.CURVE == "bn254" else 32


def g1_wide_table_gen(gens, c, nw, K):
    lib = init()
    n = gens.shape[0]
    nbytes = lib.grape_g1_wide_table_bytes(n, nw, K)
    words = WIDE_ENTRY_WORDS
    out = torch.empty((nbytes // (4 * words), words), dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_g1_wide_table_gen(_p(out), _p(gens), n, c, nw, K, _s()))
    return out


def wide_table_entries_to_host(table, idx):
    """decode entries of a wide table into affine points (x, y) as Python integers
    (None for the identity); for tests."""
    if _capi.CURVE == "bn254":
        P, L = 21888242871839275222246405745257275088696311157297823662689037894645226208583, 10
    else:
        P, L = 0x1a0111ea397fe69a4b1ba7b6434bacd764774b84f38512bf6730d2a0f6b0f6241eabfffeb153ffffb9feffffffffaaab, 14
    rinv = pow(1 << (28 * L), -1, P)
    rows = table[idx].cpu().numpy()
    out = []
    for r in rows:
        x = sum(int(r[i]) << (28 * i) for i in range(L))
        y = sum(int(r[L + i]) << (28 * i) for i in range(L))
        out.append(None if (x == 0 and y == 0) else (x * rinv % P, y * rinv % P))
    return out


def commit_i32(scalars, rowlen, table, N, c, nw, K, out=None):
    lib = init()
    size = scalars.numel()
    out = g1_empty(size // rowlen) if out is None else out
    _capi.check(lib.grape_commit_i32(_p(out), _p(scalars), size, rowlen, _p(table), N, c, nw, K, _s()))
    return out


def stream_create():
    """a stream of the library's own (default priority, its own scratch memory); returns the handle"""
    h = ctypes.c_void_p()
    _capi.check(init().grape_stream_create(ctypes.byref(h)))
    return h


def stream_destroy(h):
    _capi.check(init().grape_stream_destroy(h))


def stream_sync(h):
    _capi.check(init().grape_stream_sync(h))


def commit_i32_nowait(scalars, rowlen, table, N, c, nw, K, out, flag, stream):
    """queues the commitment on `stream` (a handle from stream_create) and returns; `flag` is a device
    int32 the caller has cleared, set when a scalar does not fit the table's digits"""
    lib = init()
    _capi.check(lib.grape_commit_i32_nowait(_p(out), _p(scalars), scalars.numel(), rowlen, _p(table), N, c, nw, K, _p(flag), stream))
    return out


def commit_fr(scalars, rowlen, table, N, c, nw, K, out=None):
    lib = init()
    size = scalars.shape[0]
    out = g1_empty(size // rowlen) if out is None else out
    _capi.check(lib.grape_commit_fr(_p(out), _p(scalars), size, rowlen, _p(table), N, c, nw, K, _s()))
    return out


def g1_strided_table_gen(gens, c, J, nsets):
    lib = init()
    N = gens.shape[0]
    nbytes = lib.grape_g1_wide_table_bytes(N, nsets, 1 << (c - 1))
    table = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_g1_strided_table_gen(_p(table), _p(gens), N, c, J, nsets, _s()))
    return table


def commit_fr_strided(scalars, rowlen, table, N, c, J, nsets, out=None):
    lib = init()
    size = scalars.shape[0]
    out = g1_empty(size // rowlen) if out is None else out
    _capi.check(lib.grape_commit_fr_strided(_p(out), _p(scalars), size, rowlen, _p(table), N, c, J, nsets, _s()))
    return out


def commit_i32_ref_table(scalars, rowlen, table, npoints):
    lib = init()
    size = scalars.numel()
    out = g1_empty(size // rowlen)
    _capi.check(lib.grape_commit_i32_ref_table(_p(out), _p(scalars), size, rowlen, _p(table), npoints, _s()))
    return out


def commit_fr_ref_table(scalars, rowlen, table, npoints):
    lib = init()
    size = scalars.shape[0]
    out = g1_empty(size // rowlen)
    _capi.check(lib.grape_commit_fr_ref_table(_p(out), _p(scalars), size, rowlen, _p(table), npoints, _s()))
    return out


def g1_affine_to_jacobian(a):
    lib = init()
    out = torch.empty((a.shape[0], 3 * _capi.FP_WORDS), dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_g1_affine_to_jacobian(_p(out), _p(a), a.shape[0], _s()))
    return out


def g1_jacobian_to_affine(a):
    lib = init()
    out = g1_empty(a.shape[0])
    _capi.check(lib.grape_g1_jacobian_to_affine(_p(out), _p(a), a.shape[0], _s()))
    return out


# ------------------------------------------------------------------ witness generation
def _i32(*shape):
    return torch.empty(shape, dtype=torch.int32, device="cuda")


def wit_matmul_rescale(a, b, scale, want_r=True, transpose_out=False):
    """a: (L, N, K) or (N, K) int32, b: (L, M, K) or (M, K) -> quotient, remainder of a . b^T"""
    lib = init()
    batched = a.dim() == 3
    L = a.shape[0] if batched else 1
    N, K = a.shape[-2], a.shape[-1]
    M = b.shape[-2]
    assert b.shape[-1] == K and (not batched or b.shape[0] == L)
    shape = ((L,) if batched else ()) + ((M, N) if transpose_out else (N, M))
    q = _i32(*shape)
    r = _i32(*shape) if want_r else None
    _capi.check(lib.grape_wit_matmul_rescale(_p(q), _p(r), _p(a), _p(b), L, N, M, K, int(scale), 1 if transpose_out else 0, _s()))
    return q, r


def wit_set_matmul_method(method):
    """0 = choose, 1 = multiply-add kernels only, 2 = matrix cores (error when not applicable)"""
    _capi.check(init().grape_wit_set_matmul_method(int(method)))


def wit_elemul_rescale(a, b, scale):
    lib = init()
    q, r = torch.empty_like(a), torch.empty_like(a)
    _capi.check(lib.grape_wit_elemul_rescale(_p(q), _p(r), _p(a), _p(b), a.numel(), int(scale), _s()))
    return q, r


def wit_table_lookup(x, low, table):
    lib = init()
    out = torch.empty_like(x)
    _capi.check(lib.grape_wit_table_lookup(_p(out), _p(x), x.numel(), int(low), table.numel(), _p(table), _s()))
    return out


def wit_add(a, b):
    lib = init()
    out = torch.empty_like(a)
    _capi.check(lib.grape_wit_add_i32(_p(out), _p(a), _p(b), a.numel(), _s()))
    return out


def wit_softmax(scores, table, bit_shift=20, index_bits=20, scale=1 << 16):
    """scores (rows, cols) int32 -> dict of the tensors the reference saves for its table softmax"""
    lib = init()
    rows, cols = scores.shape
    out = {"max": _i32(rows, 1), "exp_input": _i32(rows, cols), "exp_output": _i32(rows, cols), "exp_sum": _i32(rows, 1),
           "softmax_output": _i32(rows, cols), "softmax_lookup_query": _i32(rows, cols)}
    _capi.check(lib.grape_wit_softmax(_p(out["max"]), _p(out["exp_input"]), _p(out["exp_output"]), _p(out["exp_sum"]),
                                      _p(out["softmax_output"]), _p(out["softmax_lookup_query"]), _p(scores), rows, cols,
                                      _p(table), bit_shift, index_bits, int(scale), _s()))
    return out


def wit_row_sumsq(x):
    lib = init()
    rows, cols = x.shape
    out = torch.empty(rows, dtype=torch.int64, device="cuda")
    _capi.check(lib.grape_wit_row_sumsq(_p(out), _p(x), rows, cols, _s()))
    return out


def wit_rmsnorm_apply(x, rms, w, scale=1 << 16):
    lib = init()
    rows, cols = x.shape
    outs = [_i32(rows, cols) for _ in range(4)]
    _capi.check(lib.grape_wit_rmsnorm_apply(_p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(x), _p(rms), _p(w), rows, cols,
                                            int(scale), _s()))
    return outs


def wit_status():
    """status bits set since the last call (synchronises and clears them)"""
    lib = init()
    f = ctypes.c_uint32(0)
    _capi.check(lib.grape_wit_status(ctypes.byref(f), _s()))
    return f.value


# ------------------------------------------------------------------ measurement
def bench_copy(nbytes, iters=10):
    lib = init()
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    src.zero_()
    ms = ctypes.c_float(0)
    _capi.check(lib.grape_bench_copy(_p(dst), _p(src), nbytes, iters, ctypes.byref(ms), _s()))
    return ms.value


def bench_copy_fr(n, iters=10):
    lib = init()
    src, dst = fr_empty(n), fr_empty(n)
    src.zero_()
    ms = ctypes.c_float(0)
    _capi.check(lib.grape_bench_copy_fr(_p(dst), _p(src), n, iters, ctypes.byref(ms), _s()))
    return ms.value


def bench_mad(blocks=4096, inner=256, iters=5):
    lib = init()
    r = ctypes.c_double(0)
    _capi.check(lib.grape_bench_mad_u64_u32(blocks, inner, iters, ctypes.byref(r), _s()))
    return r.value


def profile_enable(on=True):
    _capi.check(init().grape_profile_enable(1 if on else 0))


def profile_last():
    """kernel durations (ms) of the most recent profiled call, in launch order."""
    lib = init()
    buf = (ctypes.c_float * 8)()
    n = ctypes.c_int(0)
    _capi.check(lib.grape_profile_last(buf, 8, ctypes.byref(n)))
    return [buf[i] for i in range(n.value)]
