"""Sizes past the 32-bit boundaries: element counts above 2^31, byte offsets above 2^36 and more
than 2^32 committed scalars - where an index kept in 32 bits would wrap.  Checked through closed
forms and by recomputing single rows, not against the oracle (it would take hours)."""
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


def test_field_tensor_of_more_than_2_pow_31_elements(ops):
    import torch
    n = (1 << 31) + 77
    x_host = rand_fr(1, 5)
    x = ops.to_dev(x_host)
    t = ops.fr_empty(n)
    t.zero_()
    ops.fr_bcast_add(t, x, out=t)                      # every element = x
    xv = br.fr_unpack(x_host)[0]
    assert br.fr_unpack(ops.fr_to_host(ops.fr_sum(t)))[0] == xv * n % br.R_MOD
    # the last elements really were written
    assert br.fr_unpack(ops.fr_to_host(t[n - 3:].contiguous())) == [xv] * 3
    ops.fr_mul(t, t, out=t)                            # every element = x^2
    assert br.fr_unpack(ops.fr_to_host(ops.fr_sum(t)))[0] == xv * xv % br.R_MOD * n % br.R_MOD
    # fold of the first 2^31 elements over its leading dimension: a constant tensor stays constant
    # under (1-u)*lo + u*hi, so every output equals x^2
    u = ops.to_dev(rand_fr(4, 6))
    ops.fr_fold(t, 1 << 31, u, 16, 0, 1 << 27)
    got = br.fr_unpack(ops.fr_to_host(t[(1 << 27) - 2:(1 << 27)].contiguous()))
    assert got == [xv * xv % br.R_MOD] * 2
    del t
    torch.cuda.empty_cache()


def test_commitment_in_several_slabs_and_the_32_bit_size_bound(ops):
    """more rows than one launch takes (the partial sums of 32768 row segments fill the 512 MiB
    work buffer): rows on both sides of the slab boundary against the oracle and against the same
    rows committed alone; more than 2^28 scalars in one call are refused before anything is launched"""
    import ctypes
    import torch
    import orc
    from grape_amd import _capi, GrapeError
    rowlen, rows = 8, 40000
    k = rand_fr(rowlen, 11)
    dev = ops.g1_make_generators(k)
    host = orc.g1_make_generators(k)
    wide = ops.g1_wide_table_gen(dev, 16, 1, 32768)
    W = np.random.default_rng(12).integers(-32768, 32768, (rows, rowlen)).astype(np.int32)
    dW = torch.from_numpy(W).cuda()
    out = ops.commit_i32(dW.view(-1), rowlen, wide, rowlen, 16, 1, 32768)
    assert out.shape[0] == rows
    got = ops.g1_to_host(out)
    pick = [0, 32766, 32767, 32768, 32769, rows - 1]
    want = orc.commit_i32(np.ascontiguousarray(W[pick]), orc.g1_table(host, 256), rowlen, rowlen)
    assert np.array_equal(got[pick], want)
    for r in pick:
        one = ops.commit_i32(dW[r].contiguous(), rowlen, wide, rowlen, 16, 1, 32768)
        assert torch.equal(one[0], out[r]), r
    # full-width scalars through the same slabs
    wide_fr = ops.g1_wide_table_gen(dev, 8, 32, 128)
    s = rand_fr(rows * rowlen, 13)
    out_fr = ops.g1_to_host(ops.commit_fr(ops.to_dev(s), rowlen, wide_fr, rowlen, 8, 32, 128))
    sub = np.ascontiguousarray(s.reshape(rows, rowlen, 4)[[32767, 32768, rows - 1]].reshape(-1, 4))
    assert np.array_equal(out_fr[[32767, 32768, rows - 1]], orc.commit_fr(sub, orc.g1_table(host, 256), rowlen, rowlen))
    # more than 2^28 scalars in one call: refused (nothing is read - the pointers are those of the small tensors)
    lib = _capi.load()
    for size in ((1 << 28) + rowlen, (1 << 32), (1 << 32) + 8 * rowlen):
        rc = lib.grape_commit_i32(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(dW.data_ptr()), size, rowlen,
                                  ctypes.c_void_p(wide.data_ptr()), rowlen, 16, 1, 32768, None)
        assert rc != 0 and b"2^28" in lib.grape_last_error()
        with pytest.raises(GrapeError):
            _capi.check(lib.grape_commit_fr(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(dW.data_ptr()), size, rowlen,
                                            ctypes.c_void_p(wide_fr.data_ptr()), rowlen, 8, 32, 128, None))


def test_commitment_of_2_pow_28_scalars_in_two_full_slabs(ops):
    """65536 rows of 4096 int16-range scalars (1 GiB of int32, two launches of 32768 rows): rows at
    the slab boundary and at both ends equal the same rows committed alone, and one of them the
    big-integer sum"""
    import torch
    rowlen, rows = 4096, 65536
    k = rand_fr(rowlen, 21)
    dev = ops.g1_make_generators(k)
    wide = ops.g1_wide_table_gen(dev, 16, 1, 32768)
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    W = torch.randint(-32768, 32768, (rows, rowlen), dtype=torch.int32, device="cuda", generator=g)
    out = ops.commit_i32(W.view(-1), rowlen, wide, rowlen, 16, 1, 32768)
    assert out.shape[0] == rows
    for r in (0, 32767, 32768, rows - 1):
        one = ops.commit_i32(W[r].contiguous(), rowlen, wide, rowlen, 16, 1, 32768)
        assert torch.equal(one[0], out[r]), r
    r = 32768
    want = br.g1_msm([int(v) for v in W[r].cpu().numpy()], br.g1_unpack(ops.g1_to_host(dev)))
    assert br.g1_unpack(ops.g1_to_host(out[r:r + 1].contiguous()))[0] == want
    del W, out, wide
    torch.cuda.empty_cache()
