"""Empty inputs: every entry point that takes an element count accepts zero, launches nothing and
leaves its outputs alone (the reference's kernels are launched with (n + 255) / 256 blocks, i.e.
none; here a zero-sized launch would be an error, so each entry point returns early)."""
import numpy as np
import pytest

import bigref as br
from gpuutil import rand_fr

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops as o
    o.init(0)
    return o


def test_field_entry_points_accept_zero_elements(ops):
    import torch
    e = ops.fr_empty(0)
    x = ops.to_dev(rand_fr(1, 1))
    assert ops.fr_add(e, e).shape[0] == 0
    assert ops.fr_sub(e, e).shape[0] == 0
    assert ops.fr_mul(e, e).shape[0] == 0
    assert ops.fr_bcast_add(e, x).shape[0] == 0
    assert ops.fr_bcast_mul(e, x).shape[0] == 0
    assert ops.fr_from_i32(torch.empty(0, dtype=torch.int32, device="cuda")).shape[0] == 0
    assert ops.fr_to_mont(e).shape[0] == 0
    assert ops.fr_from_mont(e).shape[0] == 0
    assert ops.fr_batch_inverse(e).shape[0] == 0
    assert ops.fr_shift_inverse(e, x).shape[0] == 0
    assert not np.any(ops.fr_to_host(ops.fr_sum(e, 0)))


def test_protocol_entry_points_accept_zero_elements(ops):
    import torch
    e = ops.fr_empty(0)
    x = ops.to_dev(rand_fr(1, 2))
    hist = ops.tlookup_hist(e, -8, 16)
    assert hist.cpu().numpy().sum() == 0
    assert ops.tlookup_index(e, -8, 16).shape[0] == 0
    ops.fr_fold_msb_multi([ops.fr_empty(0)], 0, x)
    assert ops.fr_pad(e, 3, 4, 0, x).shape[0] == 0
    assert ops.i32_pad(torch.empty(0, dtype=torch.int32, device="cuda"), 3, 4, 0).shape[0] == 0
    ops.fr_fold(e, 0, x, 1, 0, 1)
    assert ops.fr_sum_by_dim(e, 0, 4).shape[0] == 0
    # a protocol round over no indices has no meaning: refused, not silently "proved"
    from grape_amd import GrapeError
    for call in (lambda: ops.sumcheck_round2(e, e, 0, 0, x), lambda: ops.tlookup_round_sums(e, e, x, e, 0),
                 lambda: ops.tlookup_mb_sums(e, e, 0)):
        with pytest.raises(GrapeError):
            call()


def test_commitment_of_no_rows(ops):
    import torch
    k = [3, 5, 7, 11]
    dev = ops.g1_make_generators(k)
    wide = ops.g1_wide_table_gen(dev, 8, 5, 128)
    out = ops.commit_i32(torch.empty(0, dtype=torch.int32, device="cuda"), 4, wide, 4, 8, 5, 128)
    assert out.shape[0] == 0
    wide_fr = ops.g1_wide_table_gen(dev, 8, 32, 128)
    assert ops.commit_fr(ops.fr_empty(0), 4, wide_fr, 4, 8, 32, 128).shape[0] == 0
    tab = ops.g1_table_gen(dev, 256)
    assert ops.commit_i32_ref_table(torch.empty(0, dtype=torch.int32, device="cuda"), 4, tab, 4).shape[0] == 0
    assert ops.commit_fr_ref_table(ops.fr_empty(0), 4, tab, 4).shape[0] == 0
    assert ops.g1_affine_to_jacobian(ops.g1_empty(0)).shape[0] == 0


def test_witness_entry_points_accept_zero_rows(ops):
    import torch
    z = torch.empty((0, 8), dtype=torch.int32, device="cuda")
    w = torch.ones((4, 8), dtype=torch.int32, device="cuda")
    q, r = ops.wit_matmul_rescale(z, w, 1 << 16)
    assert q.shape[0] == 0 and r.shape[0] == 0
    q, r = ops.wit_elemul_rescale(z, z, 1 << 16)
    assert q.numel() == 0
    assert ops.wit_add(z, z).numel() == 0
    table = torch.arange(16, dtype=torch.int32, device="cuda")
    assert ops.wit_table_lookup(z, 0, table).numel() == 0
    assert ops.wit_row_sumsq(z).numel() == 0
    big = torch.zeros(1 << 20, dtype=torch.int32, device="cuda")
    assert ops.wit_softmax(z, big)["softmax_output"].numel() == 0
    assert ops.wit_rmsnorm_apply(z, torch.empty(0, dtype=torch.int32, device="cuda"), torch.ones(8, dtype=torch.int32, device="cuda"))[0].numel() == 0
    assert ops.wit_status() == 0


def test_freed_blocks_are_handed_out_again_and_released(ops):
    """grape_free keeps blocks, grape_malloc hands a kept block to a request of exactly its
    size, grape_alloc_cache_release gives them back"""
    import ctypes
    from grape_amd import _capi
    lib = _capi.load()
    lib.grape_alloc_cache_release(None)
    n = 64 << 20
    p, q, r = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    _capi.check(lib.grape_malloc(ctypes.byref(p), n))
    first = p.value
    _capi.check(lib.grape_free(p))
    _capi.check(lib.grape_malloc(ctypes.byref(q), n + 16))       # another size: a fresh block
    _capi.check(lib.grape_malloc(ctypes.byref(r), n))            # the same size: the kept block
    assert r.value == first and q.value != first
    _capi.check(lib.grape_free(q))
    _capi.check(lib.grape_free(r))
    released = ctypes.c_size_t(0)
    _capi.check(lib.grape_alloc_cache_release(ctypes.byref(released)))
    assert released.value == 2 * n + 16
    _capi.check(lib.grape_alloc_cache_release(ctypes.byref(released)))
    assert released.value == 0


def test_memset_zero_of_any_size_and_alignment(ops):
    """grape_memset_zero clears exactly the bytes asked for, also when size or address is no
    multiple of four (a fill kernel in every case: nothing a captured stream could not replay)"""
    import ctypes
    import torch
    from grape_amd import _capi
    lib = _capi.load()
    buf = torch.full((4096,), 0x5a, dtype=torch.uint8, device="cuda")
    for off, n in ((0, 1024), (1, 7), (3, 1001), (16, 0), (2000, 2096)):
        buf.fill_(0x5a)
        _capi.check(lib.grape_memset_zero(ctypes.c_void_p(buf.data_ptr() + off), n, None))
        torch.cuda.synchronize()
        h = buf.cpu().numpy()
        assert not h[off:off + n].any() and (h[:off] == 0x5a).all() and (h[off + n:] == 0x5a).all(), (off, n)


def test_host_to_device_copies_of_every_size_class(ops):
    """grape_memcpy_h2d carries payloads of at most 1 KiB as a kernel argument and copies longer or
    unaligned ones: 4 bytes to 1 KiB, just above it, odd lengths and odd destinations all arrive,
    neighbours stay untouched, and the host buffer may be overwritten as soon as the call returns"""
    import ctypes
    import torch
    from grape_amd import _capi
    lib = ops.init()
    rng = np.random.default_rng(11)
    for nbytes, off in ((4, 0), (32, 0), (32, 64), (1020, 4), (1024, 0), (1028, 0), (4096, 0), (30, 0), (32, 2), (1, 5)):
        dst = torch.full((8192,), 0xA5, dtype=torch.uint8, device="cuda")
        src = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
        keep = src.copy()
        _capi.check(lib.grape_memcpy_h2d(ctypes.c_void_p(dst.data_ptr() + off), src.ctypes.data_as(ctypes.c_void_p), nbytes, None))
        src[:] = 0                                   # the call has taken what it needs
        torch.cuda.synchronize()
        got = dst.cpu().numpy()
        assert np.array_equal(got[off:off + nbytes], keep), (nbytes, off)
        assert (got[:off] == 0xA5).all() and (got[off + nbytes:] == 0xA5).all(), (nbytes, off)
    # stream order: a value written, used and overwritten on the same stream
    a = ops.to_dev(rand_fr(4, 3))
    one = rand_fr(1, 4)
    two = rand_fr(1, 5)
    slot = torch.zeros(8, dtype=torch.int32, device="cuda")
    outs = []
    for val in (one, two):
        buf = np.ascontiguousarray(val).view(np.uint32).copy()
        _capi.check(lib.grape_memcpy_h2d(ctypes.c_void_p(slot.data_ptr()), buf.ctypes.data_as(ctypes.c_void_p), 32, None))
        outs.append(slot.clone())
    torch.cuda.synchronize()
    assert np.array_equal(outs[0].cpu().numpy().view(np.uint32), np.ascontiguousarray(one).view(np.uint32).reshape(-1))
    assert np.array_equal(outs[1].cpu().numpy().view(np.uint32), np.ascontiguousarray(two).view(np.uint32).reshape(-1))
