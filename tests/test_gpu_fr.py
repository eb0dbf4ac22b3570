"""GPU parity of the Fr tensor kernels against the CPU oracle, bit-exact, through the C ABI."""
import numpy as np
import pytest
import bigref as br
import orc
from gpuutil import rand_fr, assert_same

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops as o
    o.init(0)
    return o


def test_config1_mul_and_sum(ops):
    # BASELINE config 1: 2^16 random elements times 2^16 random elements, then the full sum
    n = 1 << 16
    a, b = rand_fr(n, 1), rand_fr(n, 2)
    da, db = ops.to_dev(a), ops.to_dev(b)
    prod = ops.fr_mul(da, db)
    assert_same(ops.fr_to_host(prod), orc.vec2("orc_fr_vec_mul", a, b), "mul")
    want_sum = orc.fr_sum(orc.vec2("orc_fr_vec_mul", a, b))
    assert_same(ops.fr_to_host(ops.fr_sum(prod))[0], want_sum, "sum")
    # the input of sum is left intact
    assert_same(ops.fr_to_host(prod), orc.vec2("orc_fr_vec_mul", a, b), "mul after sum")


@pytest.mark.parametrize("n", [1, 63, 64, 65, 255, 257, 1000, 70001])
def test_elementwise_ragged(ops, n):
    a, b = rand_fr(n, 10 + n), rand_fr(n, 20 + n)
    # edge values in front: 0, 1 (Montgomery one), r-1
    edge = br.fr_pack([0, 1, br.R_MOD - 1])
    a[: min(3, n)] = edge[: min(3, n)]
    da, db = ops.to_dev(a), ops.to_dev(b)
    assert_same(ops.fr_to_host(ops.fr_add(da, db)), orc.vec2("orc_fr_vec_add", a, b), "add")
    assert_same(ops.fr_to_host(ops.fr_sub(da, db)), orc.vec2("orc_fr_vec_sub", a, b), "sub")
    assert_same(ops.fr_to_host(ops.fr_mul(da, db)), orc.vec2("orc_fr_vec_mul", a, b), "mul")
    x = ops.to_dev(b[:1].copy())
    assert_same(ops.fr_to_host(ops.fr_bcast_mul(da, x)), orc.vec_bcast("orc_fr_vec_bcast_mul", a, b[0]), "bmul")
    assert_same(ops.fr_to_host(ops.fr_bcast_add(da, x)), orc.vec_bcast("orc_fr_vec_bcast_add", a, b[0]), "badd")
    assert_same(ops.fr_to_host(ops.fr_sum(da))[0], orc.fr_sum(a), "sum")
    # in place
    ops.fr_mul(da, db, out=da)
    assert_same(ops.fr_to_host(da), orc.vec2("orc_fr_vec_mul", a, b), "mul in place")


def test_sum_large_and_empty(ops):
    n = (1 << 20) + 12345
    a = rand_fr(n, 3)
    assert_same(ops.fr_to_host(ops.fr_sum(ops.to_dev(a)))[0], orc.fr_sum(a), "sum large")
    assert_same(ops.fr_to_host(ops.fr_sum(ops.fr_empty(0), 0))[0], np.zeros(4, dtype=np.uint64), "sum empty")
    # closed form: sum of n copies of x is n*x
    x = rand_fr(1, 4)
    rep = np.repeat(x, 5000, axis=0)
    got = br.fr_unpack(ops.fr_to_host(ops.fr_sum(ops.to_dev(rep))))[0]
    assert got == br.fr_unpack(x)[0] * 5000 % br.R_MOD


def test_int_embedding_and_montgomery(ops):
    import torch
    xs = np.array([0, 1, -1, 2, -2, 32767, -32768, 2**31 - 1, -2**31, 123456, -654321] * 50, dtype=np.int32)
    got = ops.fr_to_host(ops.fr_from_i32(torch.from_numpy(xs).cuda()))
    assert_same(got, orc.from_i32(xs), "from_i32")
    assert br.fr_unpack(got[:11]) == [int(x) % br.R_MOD for x in xs[:11]]
    us = np.array([0, 1, 2**32 - 1, 65536, 77] * 30, dtype=np.uint32)
    got = ops.fr_to_host(ops.fr_from_u32(ops.to_dev(us)))
    assert_same(got, orc.from_u32(us), "from_u32")
    a = rand_fr(1000, 5)
    da = ops.to_dev(a)
    plain = ops.fr_from_mont(da)
    assert_same(ops.fr_to_host(plain), orc.vec1("orc_fr_vec_from_mont", a), "from_mont")
    assert_same(ops.fr_to_host(ops.fr_to_mont(plain)), a, "to_mont round trip")


@pytest.mark.parametrize("n", [1, 7, 8, 9, 4096, 4097, 50000, 300000])
def test_batch_inverse(ops, n):
    a = rand_fr(n, 30 + n)
    a[0] = 0                                   # 1/0 = 0
    if n > 100:
        a[57] = 0
        a[n - 1] = 0
    got = ops.fr_to_host(ops.fr_batch_inverse(ops.to_dev(a)))
    if n <= 5000:
        assert_same(got, orc.vec1("orc_fr_vec_inv", a), "inverse")
    else:
        # x * x^-1 = 1 for every non-zero x, 0 stays 0 (size-independent property) + a sample vs oracle
        prod = orc.vec2("orc_fr_vec_mul", got, a)
        one = br.fr_pack([1])[0]
        nz = a.any(axis=1)
        assert np.array_equal(prod[nz], np.broadcast_to(one, (int(nz.sum()), 4)))
        assert not got[~nz].any()
        idx = np.arange(0, n, max(1, n // 997))
        assert_same(got[idx], orc.vec1("orc_fr_vec_inv", a[idx]), "inverse sample")
    beta = rand_fr(1, 99)
    got = ops.fr_to_host(ops.fr_shift_inverse(ops.to_dev(a), ops.to_dev(beta)))
    idx = np.arange(0, n, max(1, n // 997))
    want = orc.vec1("orc_fr_vec_inv", orc.vec_bcast("orc_fr_vec_bcast_add", a[idx], beta[0]))
    assert_same(got[idx], want, "shift inverse")


def test_pad_and_sum_by_dim(ops):
    import torch
    rows, N, padN = 5, 11, 16
    a = rand_fr(rows * N, 6)
    pv = rand_fr(1, 7)
    got = ops.fr_to_host(ops.fr_pad(ops.to_dev(a), N, padN, rows * padN, ops.to_dev(pv)))
    want = np.zeros((rows * padN, 4), dtype=np.uint64)
    orc.lib().orc_fr_pad(orc.P(want), orc.P(a), orc.c32(N), orc.c32(padN), orc.c64(rows * padN), orc.P(pv))
    assert_same(got, want, "pad")
    xi = np.arange(rows * N, dtype=np.int32) - 20
    goti = ops.i32_pad(torch.from_numpy(xi).cuda(), N, padN, rows * padN).cpu().numpy()
    wanti = np.zeros(rows * padN, dtype=np.int32)
    orc.lib().orc_i32_pad(orc.P(wanti, orc.i32p), orc.P(xi, orc.i32p), orc.c32(N), orc.c32(padN), orc.c64(rows * padN))
    assert np.array_equal(goti, wanti)
    rows, dim = 37, 130
    a = rand_fr(rows * dim, 8)
    got = ops.fr_to_host(ops.fr_sum_by_dim(ops.to_dev(a), rows, dim))
    want = np.zeros_like(a)
    orc.lib().orc_fr_sum_by_dim(orc.P(want), orc.P(a), orc.c64(rows), orc.c64(dim))
    assert_same(got, want, "sum_by_dim")


FOLD_CASES = [
    # (outer, c, gap)
    (1, 8, 1), (1, 11, 3), (3, 5, 4), (2, 16, 2), (4, 2, 8), (1, 1, 5), (5, 7, 1),
    (1, 2048, 64), (1, 4096, 1), (1, 1000, 37), (3, 300, 20), (2, 64, 4096), (1, 172, 256),
    (1, 1 << 18, 1), (1, 100000, 3), (1, 2, 1 << 17), (7, 1 << 13, 2),
]


@pytest.mark.parametrize("outer,c,gap", FOLD_CASES)
def test_fold_vs_oracle(ops, outer, c, gap):
    n = outer * c * gap
    t = rand_fr(n, 40 + c + gap)
    L = br.log2ceil(c)
    pre = 3
    x = rand_fr(pre + L + 2, 50 + c)
    dt = ops.to_dev(t)
    ops.fr_fold(dt, n, ops.to_dev(x), c, pre, gap)
    got = ops.fr_to_host(dt)[: outer * gap]
    want = orc.partial_eval(t, n, x, c, pre, gap)[: outer * gap]
    assert_same(got, want, "fold")


@pytest.mark.parametrize("outer,c,gap", [
    (1, 16, 1 << 19),        # one thread per output: 2^19 outputs of 16 terms
    (1, 16, 1 << 18),        # two waves share an output
    (1, 16, 1 << 17),        # four waves share an output, partial sums meet in LDS
    (1, 13, 1 << 17),        # ragged last term under a lane predicate
    (300, 4096, 1),          # many outer slabs, contiguous axis, several passes through scratch
    (1, 1 << 21, 1),         # a full evaluation: pass, pass, LDS finish
])
def test_fold_large_shapes_vs_oracle(ops, outer, c, gap):
    """shapes large enough to take every pass variant of the fold (the small cases above all
    run as four waves per output or in the LDS finish kernel)"""
    n = outer * c * gap
    t = rand_fr(n, 90 + (c % 97) + (gap % 89))
    x = rand_fr(br.log2ceil(c) + 1, 91 + (c % 97))
    dt = ops.to_dev(t)
    ops.fr_fold(dt, n, ops.to_dev(x), c, 1, gap)
    got = ops.fr_to_host(dt)[: outer * gap]
    want = orc.partial_eval(t, n, x, c, 1, gap)[: outer * gap]
    assert_same(got, want, "fold")


@pytest.mark.parametrize("outer,c,gap", [
    (1, 16, 1 << 19), (1, 16, 1 << 17), (1, 13, 1 << 17), (300, 4096, 1), (1, 1 << 21, 1),    # every pass variant
    (1, 2048, 4096),          # an opening's fold over the rows of a 2048 x 4096 tensor
    (3, 8, 5), (1, 1, 77), (2, 37, 16), (1, 1024, 2),                                          # finish kernel alone, nothing to bind
])
def test_fold_of_an_integer_tensor(ops, outer, c, gap):
    """grape_fr_fold_i32 against the fold of the embedded tensor (grape_fr_from_i32 + grape_fr_fold, itself pinned
    against the oracle above), bit for bit; integers over the whole int32 range, both signs"""
    import torch
    n = outer * c * gap
    rng = np.random.default_rng(101 + c + gap)
    ints = rng.integers(-(1 << 31), 1 << 31, size=n, dtype=np.int64).astype(np.int32)
    ints[:4] = [-(1 << 31), (1 << 31) - 1, 0, -1]
    di = torch.from_numpy(ints).cuda()
    x = ops.to_dev(rand_fr(br.log2ceil(c) + 3, 102 + c))
    want = ops.fr_from_i32(di)
    ops.fr_fold(want, n, x, c, 2, gap)
    got = ops.fr_fold_i32(di, n, x, c, 2, gap)
    assert_same(ops.fr_to_host(got), ops.fr_to_host(want)[: outer * gap], "fold of integers")
    assert np.array_equal(di.cpu().numpy(), ints)            # the input is left alone
    if n <= 1 << 16:
        assert_same(ops.fr_to_host(got), orc.partial_eval(ops.fr_to_host(ops.fr_from_i32(di)), n, ops.fr_to_host(x), c, 2, gap)[: outer * gap],
                    "fold of integers against the oracle")


def test_fold_full_eval_config3_shape_slice(ops):
    # the two folds of BASELINE config 3 at reduced token/feature counts but the real K = 4096
    # stride: A [N=64][K=4096] over N with id = log2(M), B [M=128][K=4096] over M with id = 0
    K, N, M = 4096, 64, 128
    x = rand_fr(7 + 6, 60)
    A = rand_fr(N * K, 61)
    dA = ops.to_dev(A)
    ops.fr_fold(dA, N * K, ops.to_dev(x), N, 7, K)
    assert_same(ops.fr_to_host(dA)[:K], orc.partial_eval(A, N * K, x, N, 7, K)[:K], "fold A")
    B = rand_fr(M * K, 62)
    dB = ops.to_dev(B)
    ops.fr_fold(dB, M * K, ops.to_dev(x), M, 0, K)
    assert_same(ops.fr_to_host(dB)[:K], orc.partial_eval(B, M * K, x, M, 0, K)[:K], "fold B")


def test_fold_linearity_large(ops):
    # size-independent property at a large size: fold(a + b) = fold(a) + fold(b), and the fold
    # of a constant tensor over a power-of-two axis is that constant
    n, c, gap = 1 << 22, 1 << 10, 1 << 12
    a, b = rand_fr(n, 70), rand_fr(n, 71)
    x = rand_fr(10, 72)
    dx = ops.to_dev(x)
    da, db = ops.to_dev(a), ops.to_dev(b)
    dab = ops.fr_add(da, db)
    ops.fr_fold(da, n, dx, c, 0, gap)
    ops.fr_fold(db, n, dx, c, 0, gap)
    ops.fr_fold(dab, n, dx, c, 0, gap)
    lhs = ops.fr_to_host(dab)[:gap]
    rhs = ops.fr_to_host(ops.fr_add(da[:gap].contiguous(), db[:gap].contiguous()))
    assert_same(lhs, rhs, "fold linearity")
    const = np.repeat(rand_fr(1, 73), n, axis=0)
    dc = ops.to_dev(const)
    ops.fr_fold(dc, n, dx, c, 0, gap)
    assert_same(ops.fr_to_host(dc)[:gap], const[:gap], "fold of a constant")
