"""grape_sumcheck_round2_noalloc (partial sums in a fixed array inside the code object, no
allocation inside the call) against grape_sumcheck_round2 through the C ABI: two calls in a row,
the second with a smaller input, sums and folded tensors bit-exact; the size limit is refused."""
import ctypes
import numpy as np
import pytest

from gpuutil import rand_fr

pytestmark = pytest.mark.gpu


def _round(lib, fn, A, B, in_size, out_size, v, torch):
    a, b = A.clone(), B.clone()
    sums = torch.zeros((3, 8), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    rc = fn(ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()), in_size, out_size, ctypes.c_void_p(v.data_ptr()),
            ctypes.c_void_p(sums.data_ptr()), None)
    assert rc == 0, lib.grape_last_error()
    assert lib.grape_stream_sync(None) == 0
    return a[:out_size].cpu().numpy(), b[:out_size].cpu().numpy(), sums.cpu().numpy()


def test_noalloc_round_equals_pooled_round_twice_in_a_row():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops, _capi
    ops.init(0)
    lib = _capi.load()
    # first call: 2^21 + 12345 live elements (ragged: the upper half is partly past the live extent,
    # 2^20 output indices = 4096 workgroups of partial sums); second call: a much smaller, ragged
    # input that leaves most of the array holding the first call's partial sums
    for seed, in_size in ((1, (1 << 21) - 12345), (2, 1000 + 77)):
        out_size = 1
        while 2 * out_size < in_size:
            out_size *= 2
        A, B, v = ops.to_dev(rand_fr(in_size, 10 * seed)), ops.to_dev(rand_fr(in_size, 10 * seed + 1)), ops.to_dev(rand_fr(1, 10 * seed + 2))
        want = _round(lib, lib.grape_sumcheck_round2, A, B, in_size, out_size, v, torch)
        got = _round(lib, lib.grape_sumcheck_round2_noalloc, A, B, in_size, out_size, v, torch)
        for g, w, what in zip(got, want, ("folded A", "folded B", "sums")):
            assert np.array_equal(g, w), (what, in_size)
        # and the first call again after the small one would have to be unaffected by its leftovers
    A, B, v = ops.to_dev(rand_fr(4096, 31)), ops.to_dev(rand_fr(4096, 32)), ops.to_dev(rand_fr(1, 33))
    want = _round(lib, lib.grape_sumcheck_round2, A, B, 4096, 2048, v, torch)
    got = _round(lib, lib.grape_sumcheck_round2_noalloc, A, B, 4096, 2048, v, torch)
    assert all(np.array_equal(g, w) for g, w in zip(got, want))
    # beyond the limit of the static array: refused before anything is launched
    sums = torch.zeros((3, 8), dtype=torch.int32, device="cuda")
    rc = lib.grape_sumcheck_round2_noalloc(ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(B.data_ptr()), (1 << 27) + 2, (1 << 26) + 1,
                                           ctypes.c_void_p(v.data_ptr()), ctypes.c_void_p(sums.data_ptr()), None)
    assert rc != 0 and b"limit" in lib.grape_last_error()
