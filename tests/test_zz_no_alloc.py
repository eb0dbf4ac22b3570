"""grape_sumcheck_round2_noalloc (partial sums in a fixed array inside the code object, no
allocation inside the call) against grape_sumcheck_round2 through the C ABI: two calls in a row,
the second with a smaller input, sums and folded tensors bit-exact; the device's free memory does
not change across a call; the largest size it accepts (a grid that reaches the last rows of the
array); the size limit is refused."""
import ctypes
import numpy as np
import pytest

from gpuutil import rand_fr

pytestmark = pytest.mark.gpu


def _round(lib, fn, A, B, in_size, out_size, v, torch, same_free_memory=False, on_device=False):
    a, b = A.clone(), B.clone()
    sums = torch.zeros((3, 8), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    rc = fn(ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()), in_size, out_size, ctypes.c_void_p(v.data_ptr()),
            ctypes.c_void_p(sums.data_ptr()), None)
    assert rc == 0, lib.grape_last_error()
    assert lib.grape_stream_sync(None) == 0
    if same_free_memory:
        # nothing was allocated on the device by the call (the driver's own figure, not torch's pool)
        assert torch.cuda.mem_get_info()[0] == free_before
    if on_device:
        return a[:out_size], b[:out_size], sums
    return a[:out_size].cpu().numpy(), b[:out_size].cpu().numpy(), sums.cpu().numpy()


def test_noalloc_round_equals_pooled_round_twice_in_a_row():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops, _capi
    ops.init(0)
    lib = _capi.load()
    # first call: 2^21 - 12345 live elements (ragged: the upper half is partly past the live extent,
    # 2^20 output indices = 1024 workgroups of partial sums, the grid's cap at this size); second call: a
    # much smaller, ragged input that leaves most of the array holding the first call's partial sums
    for seed, in_size in ((1, (1 << 21) - 12345), (2, 1000 + 77)):
        out_size = 1
        while 2 * out_size < in_size:
            out_size *= 2
        A, B, v = ops.to_dev(rand_fr(in_size, 10 * seed)), ops.to_dev(rand_fr(in_size, 10 * seed + 1)), ops.to_dev(rand_fr(1, 10 * seed + 2))
        want = _round(lib, lib.grape_sumcheck_round2, A, B, in_size, out_size, v, torch)
        got = _round(lib, lib.grape_sumcheck_round2_noalloc, A, B, in_size, out_size, v, torch, same_free_memory=True)
        for g, w, what in zip(got, want, ("folded A", "folded B", "sums")):
            assert np.array_equal(g, w), (what, in_size)
        # and the first call again after the small one would have to be unaffected by its leftovers
    A, B, v = ops.to_dev(rand_fr(4096, 31)), ops.to_dev(rand_fr(4096, 32)), ops.to_dev(rand_fr(1, 33))
    want = _round(lib, lib.grape_sumcheck_round2, A, B, 4096, 2048, v, torch)
    got = _round(lib, lib.grape_sumcheck_round2_noalloc, A, B, 4096, 2048, v, torch)
    assert all(np.array_equal(g, w) for g, w in zip(got, want))
    # the largest round the entry point accepts: 2^26 output indices = 4096 workgroups, the last row of the array
    # (operands made on the device: an arithmetic progression times a random element, full-width values)
    n, h = 1 << 27, 1 << 26
    seeds = rand_fr(3, 41)
    A = ops.fr_from_i32(torch.arange(n, dtype=torch.int32, device="cuda") + 1)
    ops.fr_bcast_mul(A, ops.to_dev(seeds[0:1]), out=A)
    B = ops.fr_from_i32(torch.arange(n, dtype=torch.int32, device="cuda") * 3 + 7)
    ops.fr_bcast_mul(B, ops.to_dev(seeds[1:2]), out=B)
    v = ops.to_dev(seeds[2:3])
    want = _round(lib, lib.grape_sumcheck_round2, A, B, n - 5, h, v, torch, on_device=True)
    got = _round(lib, lib.grape_sumcheck_round2_noalloc, A, B, n - 5, h, v, torch, same_free_memory=True, on_device=True)
    assert all(torch.equal(g, w) for g, w in zip(got, want))
    del A, B, want, got
    torch.cuda.empty_cache()
    A, B, v = ops.to_dev(rand_fr(4096, 31)), ops.to_dev(rand_fr(4096, 32)), ops.to_dev(rand_fr(1, 33))
    # beyond the limit of the static array: refused before anything is launched
    sums = torch.zeros((3, 8), dtype=torch.int32, device="cuda")
    rc = lib.grape_sumcheck_round2_noalloc(ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(B.data_ptr()), (1 << 27) + 2, (1 << 26) + 1,
                                           ctypes.c_void_p(v.data_ptr()), ctypes.c_void_p(sums.data_ptr()), None)
    assert rc != 0 and b"limit" in lib.grape_last_error()
