"""GPU parity of the G1 / Hyrax commitment kernels against the CPU oracle (affine, bit-exact)."""
import numpy as np
import pytest
import bigref as br
import orc
from gpuutil import rand_fr, gaussian_i16, assert_same

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops as o
    o.init(0)
    return o


def _scalars(n, seed):
    """canonical (non-Montgomery) scalars < r for generator derivation."""
    return rand_fr(n, seed)


@pytest.fixture(scope="module")
def gens64(ops):
    k = _scalars(64, 100)
    host = orc.g1_make_generators(k)
    dev = ops.g1_make_generators(k)
    return k, host, dev


def test_generator_constant(ops):
    assert_same(ops.g1_generator(), orc.g1_generator(), "generator")


def test_make_generators(ops, gens64):
    k, host, dev = gens64
    assert_same(ops.g1_to_host(dev), host, "k*G")
    # special scalars: 0 -> infinity (0,0), 1 -> G, r-1 -> -G
    ks = br.ints_to_limbs([0, 1, br.R_MOD - 1, 2], 4)
    got = br.g1_unpack(ops.g1_to_host(ops.g1_make_generators(ks)))
    assert got == [None, br.G1, br.g1_neg(br.G1), br.g1_add(br.G1, br.G1)]


def test_reference_table(ops, gens64):
    k, host, dev = gens64
    n, W = 16, 256
    got = ops.g1_to_host(ops.g1_table_gen(dev[:n].contiguous(), W))
    assert_same(got, orc.g1_table(host[:n], W), "table")
    assert not got[:n].any()                  # w = 0 row is infinity


def test_reference_table_edge_shapes(ops, gens64):
    """the reference-format table for one generator and for few, with one multiple (the identity row only),
    two, an odd count, one more than the first chain of the generator and the reference's 256"""
    k, host, dev = gens64
    for n, W in ((1, 1), (1, 2), (3, 3), (5, 17), (2, 18), (64, 33), (7, 256)):
        got = ops.g1_to_host(ops.g1_table_gen(dev[:n].contiguous(), W))
        assert_same(got, orc.g1_table(host[:n], W), "table n=%d W=%d" % (n, W))


def test_wide_table_entries(ops, gens64):
    k, host, dev = gens64
    n, c, nw, K = 8, 8, 3, 128
    table = ops.g1_wide_table_gen(dev[:n].contiguous(), c, nw, K)
    assert table.numel() * 4 == nw * K * n * 4 * ops.WIDE_ENTRY_WORDS
    pts = br.g1_unpack(host[:n])
    cases = [(0, 1, 0), (0, 128, 7), (1, 1, 3), (1, 77, 2), (2, 128, 5), (2, 2, 0), (0, 65, 1), (1, 64, 6)]
    idx = [(w * K + (kk - 1)) * n + i for (w, kk, i) in cases]
    got = ops.wide_table_entries_to_host(table, idx)
    for (w, kk, i), pt in zip(cases, got):
        assert pt == br.g1_mul(kk << (c * w), pts[i])


def _table_case(ops, pts, c, nw, K, ks):
    import torch
    n = len(pts)
    dev = torch.from_numpy(br.g1_pack(pts)).cuda()
    table = ops.g1_wide_table_gen(dev, c, nw, K)
    cases = [(w, kk, i) for w in range(nw) for kk in ks for i in range(n)]
    idx = [(w * K + (kk - 1)) * n + i for (w, kk, i) in cases]
    got = ops.wide_table_entries_to_host(table, idx)
    for (w, kk, i), pt in zip(cases, got):
        assert pt == br.g1_mul(kk << (c * w), pts[i]), (c, nw, K, w, kk, i)


def test_wide_table_levels(ops, gens64):
    """entries above the first 16 multiples come from the level step (E[h + k] = E[k] + E[h], affine
    additions behind shared inversions): every level's first and last entry, the doubling
    E[2h] and entries inside runs, for power-of-two and ragged K, against Python integers"""
    k, host, dev = gens64
    pts = br.g1_unpack(host[:5])
    _table_case(ops, pts, 9, 2, 256, [1, 2, 15, 16, 17, 18, 31, 32, 33, 63, 64, 65, 66, 100, 127, 128, 129, 191, 192, 193, 255, 256])
    _table_case(ops, pts, 9, 2, 200, [64, 65, 128, 129, 130, 192, 193, 199, 200])
    _table_case(ops, pts[:2], 12, 1, 2048, [64, 65, 1024, 1025, 1088, 1089, 1537, 2047, 2048])
    _table_case(ops, pts[:3], 6, 3, 32, [1, 16, 17, 31, 32])
    _table_case(ops, pts[:3], 4, 3, 8, [1, 7, 8])              # below the first chain's length: no level at all


def test_wide_table_with_degenerate_bases(ops, gens64):
    """a generator set that holds the identity (and, where the curve has one, a point of order three):
    their multiples repeat or vanish, no affine sum exists for some of them, and the level step
    hands such levels to the general addition - all entries still equal the multiples"""
    k, host, dev = gens64
    pts = br.g1_unpack(host[:3])
    pts.insert(1, None)
    if br.CURVE != "bn254":
        assert br.g1_on_curve((0, 2)) and br.g1_mul(3, (0, 2)) is None
        pts.append((0, 2))
    _table_case(ops, pts, 8, 2, 256, [1, 2, 3, 16, 17, 18, 19, 32, 33, 64, 65, 66, 128, 129, 130, 131, 255, 256])


def test_commit_i32_small_vs_oracle_and_bigint(ops, gens64):
    import torch
    k, host, dev = gens64
    n, rows = 64, 6
    rng = np.random.default_rng(5)
    S = rng.integers(-2**31, 2**31, size=(rows, n)).astype(np.int32)
    S[0] = 0
    S[1] = 0
    S[1, 3] = -1
    S[2, :8] = [-2**31, 2**31 - 1, 65535, -65536, 32768, -32768, 32767, -32767]
    table_ref = orc.g1_table(host, 256)
    want = orc.commit_i32(S, table_ref, n, n)
    dS = torch.from_numpy(S).cuda()
    # general int32: radix 2^8 signed digits, 5 windows
    wide = ops.g1_wide_table_gen(dev, 8, 5, 128)
    assert_same(ops.g1_to_host(ops.commit_i32(dS, n, wide, n, 8, 5, 128)), want, "commit i32 c=8")
    # radix 2^16, 3 windows
    wide16 = ops.g1_wide_table_gen(dev[:16].contiguous(), 16, 3, 32768)
    S16 = S[:, :16].copy()
    want16 = orc.commit_i32(S16, orc.g1_table(host[:16], 256), 16, 16)
    assert_same(ops.g1_to_host(ops.commit_i32(torch.from_numpy(S16).cuda(), 16, wide16, 16, 16, 3, 32768)), want16, "commit i32 c=16")
    # reference-format table path
    dtab = ops.g1_table_gen(dev, 256)
    assert_same(ops.g1_to_host(ops.commit_i32_ref_table(dS, n, dtab, n)), want, "commit i32 ref table")
    got = br.g1_unpack(want)
    assert got[0] is None and got[1] == br.g1_neg(br.g1_unpack(host[3:4])[0])


def test_commitments_queued_on_three_streams(ops, gens64):
    """grape_commit_i32_nowait on three streams of the library in turn (each stream with its own scratch,
    output and digit-range flag): nine commitments of different matrices against the oracle, and a
    flag that is raised by the one commitment whose scalars do not fit"""
    import torch
    k, host, dev = gens64
    n, rows = 32, 300
    wide = ops.g1_wide_table_gen(dev[:n].contiguous(), 16, 1, 32768)
    tab = orc.g1_table(host[:n], 256)
    mats = [gaussian_i16((rows, n), 60 + i) for i in range(9)]
    dmats = [torch.from_numpy(m).cuda() for m in mats]
    streams = [ops.stream_create() for _ in range(3)]
    outs = [ops.g1_empty(rows) for _ in range(9)]
    flags = torch.zeros(9, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    try:
        for i in range(9):
            ops.commit_i32_nowait(dmats[i], n, wide, n, 16, 1, 32768, outs[i], flags[i:i + 1], streams[i % 3])
        for h in streams:
            ops.stream_sync(h)
        assert flags.tolist() == [0] * 9
        for i in range(9):
            assert_same(ops.g1_to_host(outs[i]), orc.commit_i32(mats[i], tab, n, n), "queued commitment %d" % i)
        bad = mats[4].copy()
        bad[7, 5] = 40000
        dbad = torch.from_numpy(bad).cuda()
        flags.zero_()
        torch.cuda.synchronize()
        for i in range(3):
            ops.commit_i32_nowait(dbad if i == 1 else dmats[i], n, wide, n, 16, 1, 32768, outs[i], flags[i:i + 1], streams[i])
        for h in streams:
            ops.stream_sync(h)
        assert flags.tolist()[:3] == [0, 1, 0]
    finally:
        for h in streams:
            ops.stream_destroy(h)


@pytest.mark.parametrize("rows,n", [(515, 64), (600, 256), (1100, 128), (2051, 64), (4096, 256)])
def test_waiting_and_queued_commitments_agree(ops, rows, n):
    """with 512 to 4096 rows a call that waits for its result (grape_commit_i32) and a queued one
    (grape_commit_i32_nowait) take different row reductions - four waves per eight rows with partial sums handed
    on through LDS, one wave per eight to two rows - over 64 to 256 partial sums per row: the same affine points
    bit for bit, and the oracle's"""
    import torch
    k = _scalars(n, 300 + n)
    host = orc.g1_make_generators(k)
    dev = ops.g1_make_generators(k)
    wide = ops.g1_wide_table_gen(dev, 8, 1, 128)
    rng = np.random.default_rng(rows * 7 + n)
    m = rng.integers(-100, 101, size=(rows, n), dtype=np.int32)
    m[3] = 0                                   # a row that sums to the identity
    m[5, 1:] = 0                               # a row of one term
    d = torch.from_numpy(m).cuda()
    waited = ops.g1_to_host(ops.commit_i32(d, n, wide, n, 8, 1, 128))
    h = ops.stream_create()
    out = ops.g1_empty(rows)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    try:
        ops.commit_i32_nowait(d, n, wide, n, 8, 1, 128, out, flag, h)
        ops.stream_sync(h)
    finally:
        ops.stream_destroy(h)
    assert flag.tolist() == [0]
    assert_same(ops.g1_to_host(out), waited, "queued against waiting")
    assert_same(waited, orc.commit_i32(m, orc.g1_table(host, 256), n, n), "against the oracle")


def test_commit_int16_fast_path(ops, gens64):
    import torch
    k, host, dev = gens64
    n, rows = 32, 40
    W = gaussian_i16((rows, n), 6)
    W[0, :4] = [-32768, 32767, 0, 1]
    wide = ops.g1_wide_table_gen(dev[:n].contiguous(), 16, 1, 32768)
    got = ops.g1_to_host(ops.commit_i32(torch.from_numpy(W).cuda(), n, wide, n, 16, 1, 32768))
    want = orc.commit_i32(W, orc.g1_table(host[:n], 256), n, n)
    assert_same(got, want, "int16 fast path")
    # a value outside int16 range is rejected, not silently mis-committed
    W[3, 3] = 40000
    from grape_amd import GrapeError
    with pytest.raises(GrapeError):
        ops.commit_i32(torch.from_numpy(W).cuda(), n, wide, n, 16, 1, 32768)


def test_commit_fr_config1_shape(ops):
    # BASELINE config 1: the 2^16 products committed as a 256 x 256 matrix with 256 generators
    k = _scalars(256, 101)
    host = orc.g1_make_generators(k)
    dev = ops.g1_make_generators(k)
    a, b = rand_fr(1 << 16, 1), rand_fr(1 << 16, 2)
    prod = orc.vec2("orc_fr_vec_mul", a, b)
    rows_checked = 6                              # the oracle takes ~1 s per row
    want = orc.commit_fr(prod[: rows_checked * 256], orc.g1_table(host, 256), 256, 256)
    wide = ops.g1_wide_table_gen(dev, 8, 32, 128)
    dprod = ops.fr_mul(ops.to_dev(a), ops.to_dev(b))
    got = ops.g1_to_host(ops.commit_fr(dprod, 256, wide, 256, 8, 32, 128))
    assert got.shape[0] == 256
    assert_same(got[:rows_checked], want, "commit fr")
    # every output is on the curve
    for pt in br.g1_unpack(got[::37]):
        assert br.g1_on_curve(pt)
    # the tensor is still in Montgomery form afterwards
    assert_same(ops.fr_to_host(dprod), prod, "scalars untouched")
    # reference-format table path on a few rows
    dtab = ops.g1_table_gen(dev, 256)
    got2 = ops.g1_to_host(ops.commit_fr_ref_table(dprod[: 3 * 256].contiguous(), 256, dtab, 256))
    assert_same(got2, want[:3], "commit fr ref table")


def test_commit_fr_edge_scalars_and_int_path_agreement(ops, gens64):
    import torch
    k, host, dev = gens64
    n = 16
    vals = [0, 1, br.R_MOD - 1, 255, 256, 128, 127, 129, (1 << 254), br.R_MOD - 128, 0x80808080, 2**64 - 1,
            2**128, 0x7f7f7f7f7f7f7f7f, 3, 5]
    s = br.fr_pack(vals)
    wide = ops.g1_wide_table_gen(dev[:n].contiguous(), 8, 32, 128)
    got = br.g1_unpack(ops.g1_to_host(ops.commit_fr(ops.to_dev(s), n, wide, n, 8, 32, 128)))[0]
    assert got == br.g1_msm(vals, br.g1_unpack(host[:n]))
    small = np.array([[5, -7, 300, -70000, 0, 0, 1, -1, 9, 8, 7, 6, 5, 4, 3, 2]], dtype=np.int32)
    a = ops.g1_to_host(ops.commit_fr(ops.fr_from_i32(torch.from_numpy(small).cuda()), n, wide, n, 8, 32, 128))
    wide5 = ops.g1_wide_table_gen(dev[:n].contiguous(), 8, 5, 128)
    b = ops.g1_to_host(ops.commit_i32(torch.from_numpy(small).cuda(), n, wide5, n, 8, 5, 128))
    assert_same(a, b, "int path == Fr path")


def test_commit_fr_half_range_recoding(ops, gens64):
    """windows that cover only 255 bits (nw * c = 255): a scalar above (r-1)/2 is committed as
    -(r - k), so the top window never carries out; scalars at and around r/2, at the ends of the
    field and with long carry chains against the big-integer sum"""
    k, host, dev = gens64
    n = 16
    r = br.R_MOD
    top = 1 << (r.bit_length() - 1)
    vals = [(r - 1) // 2, (r + 1) // 2, (r - 1) // 2 - 1, (r + 1) // 2 + 1, r - 1, r - 2, 1, 0,
            top - 1, top, (1 << 240) - 1, r - (1 << 240), 0x7fff7fff7fff7fff7fff, (1 << 254) % r, r // 3, 2 * r // 3]
    s = br.fr_pack(vals)
    want = br.g1_msm(vals, br.g1_unpack(host[:n]))
    for c, nw in ((15, 17), (5, 51), (16, 16)):
        wide = ops.g1_wide_table_gen(dev[:n].contiguous(), c, nw, 1 << (c - 1))
        got = br.g1_unpack(ops.g1_to_host(ops.commit_fr(ops.to_dev(s), n, wide, n, c, nw, 1 << (c - 1))))[0]
        assert got == want, (c, nw)
        # each scalar alone, so that no cancellation can hide a wrong digit
        rows = np.zeros((n, n, 4), dtype=np.uint64)
        for i in range(n):
            rows[i, i] = s[i]
        got = br.g1_unpack(ops.g1_to_host(ops.commit_fr(ops.to_dev(rows.reshape(n * n, 4)), n, wide, n, c, nw, 1 << (c - 1))))
        pts = br.g1_unpack(host[:n])
        for i in range(n):
            assert got[i] == br.g1_msm([vals[i]], [pts[i]]), (c, nw, i)
        del wide
    from grape_amd import GrapeError
    wide = ops.g1_wide_table_gen(dev[:n].contiguous(), 15, 16, 1 << 14)
    with pytest.raises(GrapeError):
        ops.commit_fr(ops.to_dev(s), n, wide, n, 15, 16, 1 << 14)       # 240 bits of windows: refused


@pytest.mark.parametrize("c,J", [(16, 4), (17, 8), (15, 2), (12, 22), (14, 1), (5, 7), (18, 15), (16, 16), (13, 3)])
def test_commit_fr_strided_table(ops, gens64, c, J):
    """full-width scalars through the strided table (every J-th window set, J residue sums combined by
    doublings, carry-free signed digits): edge scalars one by one and together against the big-integer
    sum, random rows against the per-window path and the oracle"""
    k, host, dev = gens64
    n = 16
    r = br.R_MOD
    nw = (255 + c - 1) // c
    nsets = (nw + J - 1) // J
    top = 1 << (r.bit_length() - 1)
    vals = [(r - 1) // 2, (r + 1) // 2, (r - 1) // 2 - 1, (r + 1) // 2 + 1, r - 1, r - 2, 1, 0,
            top - 1, top, (1 << 240) - 1, r - (1 << 240), 0x7fff7fff7fff7fff7fff, (1 << (c - 1)), (1 << (c - 1)) + 1, 2 * r // 3]
    s = br.fr_pack(vals)
    pts = br.g1_unpack(host[:n])
    table = ops.g1_strided_table_gen(dev[:n].contiguous(), c, J, nsets)
    got = br.g1_unpack(ops.g1_to_host(ops.commit_fr_strided(ops.to_dev(s), n, table, n, c, J, nsets)))[0]
    assert got == br.g1_msm(vals, pts)
    rows = np.zeros((n, n, 4), dtype=np.uint64)
    for i in range(n):
        rows[i, i] = s[i]
    got = br.g1_unpack(ops.g1_to_host(ops.commit_fr_strided(ops.to_dev(rows.reshape(n * n, 4)), n, table, n, c, J, nsets)))
    for i in range(n):
        assert got[i] == br.g1_msm([vals[i]], [pts[i]]), (c, J, i)
    del table
    # 24 random rows of 64 against the oracle's byte-window commitment (and 3 ragged rows of 40)
    table = ops.g1_strided_table_gen(dev, c, J, nsets)
    x = rand_fr(24 * 64, 300 + c)
    got = ops.g1_to_host(ops.commit_fr_strided(ops.to_dev(x), 64, table, 64, c, J, nsets))
    assert_same(got, orc.commit_fr(x, orc.g1_table(host, 256), 64, 64), "strided vs oracle")
    y = rand_fr(3 * 40, 400 + c)
    got = ops.g1_to_host(ops.commit_fr_strided(ops.to_dev(y), 40, table, 64, c, J, nsets))
    assert_same(got, orc.commit_fr(y, orc.g1_table(host, 256), 40, 64), "strided, short rows")


def test_commit_fr_strided_many_rows_and_long_rows(ops):
    """more (row, residue) units than one launch takes, and one long row cut into column segments:
    equal to the per-window path on the same scalars"""
    k = _scalars(2048, 811)
    dev = ops.g1_make_generators(k)
    # 20000 rows of 8 with J = 4: 80000 units, three launches
    small = dev[:8].contiguous()
    t1, w1 = ops.g1_strided_table_gen(small, 16, 4, 4), ops.g1_wide_table_gen(small, 8, 32, 128)
    x = ops.to_dev(rand_fr(20000 * 8, 812))
    a = ops.commit_fr_strided(x, 8, t1, 8, 16, 4, 4)
    b = ops.commit_fr(x, 8, w1, 8, 8, 32, 128)
    import torch
    assert torch.equal(a, b)
    # 3 rows of 2048 columns: 32 segments per (row, residue)
    t2, w2 = ops.g1_strided_table_gen(dev, 12, 22, 1), ops.g1_wide_table_gen(dev, 8, 32, 128)
    y = ops.to_dev(rand_fr(3 * 2048, 813))
    assert torch.equal(ops.commit_fr_strided(y, 2048, t2, 2048, 12, 22, 1), ops.commit_fr(y, 2048, w2, 2048, 8, 32, 128))
    from grape_amd import GrapeError
    with pytest.raises(GrapeError):
        ops.commit_fr_strided(y, 2048, t2, 2048, 12, 21, 1)        # 21 residues x 1 set < 22 windows


def test_commit_linearity_medium(ops):
    # size-independent property on a larger shape: com(a + b) = com(a) + com(b)
    import torch
    n, rows = 512, 64
    k = _scalars(n, 102)
    dev = ops.g1_make_generators(k)
    wide = ops.g1_wide_table_gen(dev, 16, 1, 32768)
    a = gaussian_i16((rows, n), 7, sigma=512)
    b = gaussian_i16((rows, n), 8, sigma=512)
    ca = br.g1_unpack(ops.g1_to_host(ops.commit_i32(torch.from_numpy(a).cuda(), n, wide, n, 16, 1, 32768)))
    cb = br.g1_unpack(ops.g1_to_host(ops.commit_i32(torch.from_numpy(b).cuda(), n, wide, n, 16, 1, 32768)))
    cab = br.g1_unpack(ops.g1_to_host(ops.commit_i32(torch.from_numpy(a + b).cuda(), n, wide, n, 16, 1, 32768)))
    for x, y, z in zip(ca, cb, cab):
        assert z == br.g1_add(x, y)
    # rows shorter than the generator set (table stride N > rowlen)
    c2 = ops.g1_to_host(ops.commit_i32(torch.from_numpy(a[:, :128].copy()).cuda(), 128, wide, n, 16, 1, 32768))
    host = orc.g1_make_generators(k[:128])
    assert_same(c2[:4], orc.commit_i32(a[:4, :128].copy(), orc.g1_table(host, 256), 128, 128), "stride")


def test_jacobian_conversions(ops, gens64):
    k, host, dev = gens64
    jac = ops.g1_affine_to_jacobian(dev)
    back = ops.g1_jacobian_to_affine(jac)
    assert_same(ops.g1_to_host(back), host, "affine -> jacobian -> affine")
    hj = jac.cpu().numpy().view(np.uint64).reshape(-1, 3 * br.FP_LIMBS)
    want = np.zeros((64, br.G1_WORDS), dtype=np.uint64)
    orc.lib().orc_g1_jac_to_affine(orc.P(want), orc.P(np.ascontiguousarray(hj)), orc.c64(64))
    assert_same(want, host, "oracle jacobian -> affine")


def test_reference_table_path_in_every_launch_shape(ops):
    """commitments through the reference-format table agree with the wide-table path when a row
    spans several column segments, when rows are many enough for several slabs, on ragged row
    lengths, on edge scalars, and with repeated generators (the exceptional additions)"""
    import torch
    k = _scalars(512, 303)
    k[5] = k[4]                                  # two equal generators: entry = accumulator can occur
    dev = ops.g1_make_generators(k)
    dtab = ops.g1_table_gen(dev, 256)
    wide = ops.g1_wide_table_gen(dev, 8, 32, 128)
    # one long row (segments), a few rows of ragged length, many short rows (slabs)
    for rows, rowlen in ((1, 512), (3, 200), (1100, 8)):
        s = rand_fr(rows * rowlen, rows + rowlen)
        s[0] = 0
        s[1] = br.fr_pack([br.R_MOD - 1])[0]
        s[2] = br.fr_pack([1])[0]
        if rowlen > 5:
            s[4] = s[5] = br.fr_pack([7])[0]     # 7*G + 7*G on the two equal generators
        d = ops.to_dev(s)
        got = ops.g1_to_host(ops.commit_fr_ref_table(d, rowlen, dtab, 512))
        want = ops.g1_to_host(ops.commit_fr(d, rowlen, wide, 512, 8, 32, 128))
        assert_same(got, want, "fr ref table %dx%d" % (rows, rowlen))
    wide_i = ops.g1_wide_table_gen(dev, 8, 5, 128)
    for rows, rowlen in ((1, 512), (2, 300), (9000, 4)):
        rng = np.random.default_rng(rows)
        v = rng.integers(-2**31, 2**31, size=(rows, rowlen), dtype=np.int64).astype(np.int32)
        v[0, :4] = [-2**31, 2**31 - 1, 0, -1]
        d = torch.from_numpy(v).cuda()
        got = ops.g1_to_host(ops.commit_i32_ref_table(d, rowlen, dtab, 512))
        want = ops.g1_to_host(ops.commit_i32(d, rowlen, wide_i, 512, 8, 5, 128))
        assert_same(got, want, "i32 ref table %dx%d" % (rows, rowlen))


@pytest.mark.parametrize("rowlen,rows,live", [(16, 5, 0.3), (200, 7, 0.02), (200, 7, 0.9), (64, 3, 0.0), (1000, 4, 0.07),
                                              (48, 4097, 0.3), (100, 5000, 0.02), (70, 4096, 0.9)])
def test_commit_fr_sparse_against_dense_commitment_of_masked_tensor(ops, rowlen, rows, live):
    """the commitment of the flagged-in elements only (queued per row, dense batches of 64 - of 32 with
    two rows per wave when the rows are many, an odd number of them included - a last partial batch,
    rows with none) equals the dense commitment of the tensor with the others zeroed, and the
    oracle's on a few rows"""
    import torch
    k = _scalars(rowlen, 131)
    dev = ops.g1_make_generators(k)
    rng = np.random.default_rng(rowlen + rows)
    s = rand_fr(rows * rowlen, 132)
    skip = (rng.random(rows * rowlen) >= live).astype(np.int32) * rng.integers(1, 9, size=rows * rowlen).astype(np.int32)
    if live > 0:
        skip[rowlen: 2 * rowlen] = 1                                   # one row with nothing live
    c, nw, K = 11, 24, 1024
    wide = ops.g1_wide_table_gen(dev, c, nw, K)
    got = ops.g1_to_host(ops.commit_fr_sparse(ops.to_dev(s), torch.from_numpy(skip).cuda(), rowlen, wide, rowlen, c, nw, K))
    masked = s.copy()
    masked[skip != 0] = 0
    want = ops.g1_to_host(ops.commit_fr(ops.to_dev(masked), rowlen, wide, rowlen, c, nw, K))
    assert_same(got, want, "sparse == dense of the masked tensor")
    if live > 0:
        assert not got[1].any()                                        # the empty row commits to infinity
    if rowlen <= 200:
        tab = orc.g1_table(orc.g1_make_generators(k), 256)
        assert_same(got[:1], orc.commit_fr(masked[:rowlen], tab, rowlen, rowlen), "oracle, first row")
