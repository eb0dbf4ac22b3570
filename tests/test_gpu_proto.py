"""GPU parity of the sumcheck-round and tlookup kernels against the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import bigref as br
import orc
from gpuutil import rand_fr, assert_same

pytestmark = pytest.mark.gpu
R = br.R_MOD


@pytest.fixture(scope="module")
def ops():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops as o
    o.init(0)
    return o


def _oracle_round2(A, B, in_size, out_size, v):
    A, B = A.copy(), B.copy()
    a = np.zeros((out_size, 4), dtype=np.uint64)
    b = np.zeros_like(a)
    c = np.zeros_like(a)
    orc.lib().orc_sumcheck_round2(orc.P(A), orc.P(B), orc.P(a), orc.P(b), orc.P(c), orc.c32(in_size), orc.c32(out_size), orc.P(v))
    return A, B, a, b, c


@pytest.mark.parametrize("in_size,out_size", [(2, 1), (8, 4), (6, 4), (5, 4), (4096, 2048), (3000, 2048), (1 << 17, 1 << 16), (100000, 65536),
                                              # long rounds: several indices per thread, upper halves that end inside a workgroup's range
                                              (1 << 22, 1 << 21), (3000001, 1 << 21), ((1 << 22) - 700, (1 << 21) - 300)])
def test_sumcheck_round2(ops, in_size, out_size):
    A, B = rand_fr(in_size, 1 + in_size), rand_fr(in_size, 2 + in_size)
    v = rand_fr(1, 3)
    wA, wB, wa, wb, wc = _oracle_round2(A, B, in_size, out_size, v)
    dA, dB = ops.to_dev(A), ops.to_dev(B)
    sums = ops.fr_to_host(ops.sumcheck_round2(dA, dB, in_size, out_size, ops.to_dev(v)))
    assert_same(ops.fr_to_host(dA)[:out_size], wA[:out_size], "folded A")
    assert_same(ops.fr_to_host(dB)[:out_size], wB[:out_size], "folded B")
    assert_same(sums[0], orc.fr_sum(wc), "sum c")
    assert_same(sums[1], orc.fr_sum(wb), "sum b")
    assert_same(sums[2], orc.fr_sum(wa), "sum a")
    # coefficient-array variant
    dA, dB = ops.to_dev(A), ops.to_dev(B)
    da, db, dc = ops.fr_empty(out_size), ops.fr_empty(out_size), ops.fr_empty(out_size)
    sums2 = ops.fr_to_host(ops.sumcheck_round2_coeffs(dA, dB, da, db, dc, in_size, out_size, ops.to_dev(v)))
    assert_same(ops.fr_to_host(da), wa, "a")
    assert_same(ops.fr_to_host(db), wb, "b")
    assert_same(ops.fr_to_host(dc), wc, "c")
    assert_same(sums2, sums, "sums")


@pytest.mark.parametrize("in_size", [512, 300, 257, 64, 3, 2, 1])
def test_sumcheck_tail_rounds_match_single_rounds(ops, in_size):
    """all remaining rounds in one launch give what the same rounds give one launch at a time"""
    rounds = br.log2ceil(in_size)
    A, B = rand_fr(in_size, 301 + in_size), rand_fr(in_size, 302 + in_size)
    v = rand_fr(rounds + 2, 303)
    dv = ops.to_dev(v)
    dA, dB = ops.to_dev(A), ops.to_dev(B)
    want = []
    n_in, n_out = in_size, (1 << (rounds - 1)) if rounds else 0
    for i in range(rounds):
        vi = dv[rounds + 1 - i - 1: rounds + 1 - i].contiguous()           # v[rounds], v[rounds-1], ...
        want.append(ops.fr_to_host(ops.sumcheck_round2(dA, dB, n_in, n_out, vi)))
        n_in, n_out = n_out, n_out // 2
    tA, tB = ops.to_dev(A), ops.to_dev(B)
    got = ops.fr_to_host(ops.sumcheck_round2_tail(tA, tB, in_size, rounds, dv, rounds + 1))
    if rounds:
        assert_same(got[: 3 * rounds], np.concatenate(want), "sums of every round")
        assert_same(ops.fr_to_host(tA)[:1], ops.fr_to_host(dA)[:1], "A bound at every challenge")
        assert_same(ops.fr_to_host(tB)[:1], ops.fr_to_host(dB)[:1], "B bound at every challenge")


def test_sumcheck_round1(ops):
    in_size, out_size = 1000, 512
    X = rand_fr(in_size, 11)
    v = rand_fr(1, 12)
    dX = ops.to_dev(X)
    da, db = ops.fr_empty(out_size), ops.fr_empty(out_size)
    ops.sumcheck_round1(dX, da, db, in_size, out_size, ops.to_dev(v))
    Xi = br.fr_unpack(X)
    vi = br.fr_unpack(v)[0]
    hi = [Xi[g + out_size] if g + out_size < in_size else 0 for g in range(out_size)]
    assert br.fr_unpack(ops.fr_to_host(db)) == Xi[:out_size]
    assert br.fr_unpack(ops.fr_to_host(da)) == [(h - l) % R for h, l in zip(hi, Xi)]
    assert br.fr_unpack(ops.fr_to_host(dX)[:out_size]) == [(l + vi * (h - l)) % R for h, l in zip(hi, Xi)]


def test_full_phase2_chain_matches_oracle_transcript(ops):
    # run 12 fused rounds on K = 4096 (BASELINE config 3's phase 2) and compare every round's
    # sums with the oracle's prove_matmul transcript for L = N = M = 1
    K = 4096
    A, B = rand_fr(K, 21), rand_fr(K, 22)
    v = rand_fr(12, 23)
    u = rand_fr(1, 24)[:0]
    prod = orc.vec2("orc_fr_vec_mul", A, B)
    claim = orc.fr_sum(prod)
    st, tr, final_claim, ac, bc = orc.prove_matmul(A, B, 1, 1, 1, K, u, v, claim)
    assert st == 0 and tr.shape[0] == 12
    dA, dB, dv = ops.to_dev(A), ops.to_dev(B), ops.to_dev(v)
    in_size, out_size = K, K // 2
    for i in range(12):
        vi = dv[12 - 1 - i: 12 - i].contiguous()
        sums = ops.fr_to_host(ops.sumcheck_round2(dA, dB, in_size, out_size, vi))
        assert_same(sums, tr[i][:3], "round %d" % i)
        in_size, out_size = out_size, out_size // 2
    assert_same(ops.fr_to_host(dA)[0], ac, "A(v)")
    assert_same(ops.fr_to_host(dB)[0], bc, "B(v)")


def test_histogram(ops):
    import torch
    low, length = -32768, 65536
    rng = np.random.default_rng(31)
    s = rng.integers(low, low + length, size=200000).astype(np.int32)
    vals = ops.fr_from_i32(torch.from_numpy(s).cuda())
    h = ops.tlookup_hist(vals, low, length).cpu().numpy().view(np.uint32)
    assert np.array_equal(h, np.bincount(s.astype(np.int64) - low, minlength=length).astype(np.uint32))
    assert_same(h[:, None], orc.histogram(orc.from_i32(s), low, length)[:, None], "hist vs oracle")
    # heavy collisions: everything in one bin
    same = ops.fr_from_i32(torch.full((100000,), 5, dtype=torch.int32, device="cuda"))
    h2 = ops.tlookup_hist(same, 0, 16).cpu().numpy()
    assert h2[5] == 100000 and h2.sum() == 100000
    # out-of-range values are ignored
    oob = ops.fr_from_i32(torch.tensor([100, -1, 3], dtype=torch.int32, device="cuda"))
    h3 = ops.tlookup_hist(oob, 0, 16).cpu().numpy()
    assert h3.sum() == 1 and h3[3] == 1


def test_histogram_long_witness(ops):
    """witnesses of 2^20 values and more take the LDS-counting path: ragged length, a table that
    is not a multiple of the bins held in LDS, a clipped (heavily repeated) value, values outside
    the table, and accumulation into a histogram that is not zero"""
    import torch
    low, length = -40000, 100003
    n = (1 << 20) + 4099
    rng = np.random.default_rng(32)
    s = np.rint(rng.normal(0.0, 30000.0, size=n)).astype(np.int64)
    s = np.clip(s, low - 50, low + length + 49)              # piles at both ends, 50 steps outside
    s[::7] = 12345
    s32 = s.astype(np.int32)
    vals = ops.fr_from_i32(torch.from_numpy(s32).cuda())
    inside = (s >= low) & (s < low + length)
    want = np.bincount(s[inside] - low, minlength=length).astype(np.uint32)
    h = ops.tlookup_hist(vals, low, length).cpu().numpy().view(np.uint32)
    assert np.array_equal(h, want)
    assert int(h.sum()) == int(inside.sum()) < n
    pre = torch.full((length,), 3, dtype=torch.int32, device="cuda")
    h2 = ops.tlookup_hist(vals, low, length, hist=pre).cpu().numpy().view(np.uint32)
    assert np.array_equal(h2, want + 3)
    # a large table of which the witness touches little: most (chunk of the witness, range of bins)
    # pairs are empty and are skipped; stray values put single elements into otherwise empty pairs
    low2, length2 = -(1 << 19), 1 << 20
    n2 = (1 << 21) + 5
    t = np.rint(rng.normal(0.0, 181.0, size=n2)).astype(np.int64)
    t[3] = low2
    t[n2 // 2] = low2 + length2 - 1
    t[n2 - 2] = 300000
    t[n2 - 1] = low2 + length2                                  # just outside
    want2 = np.bincount(t[:-1] - low2, minlength=length2).astype(np.uint32)
    h4 = ops.tlookup_hist(ops.fr_from_i32(torch.from_numpy(t.astype(np.int32)).cuda()), low2, length2).cpu().numpy().view(np.uint32)
    assert np.array_equal(h4, want2) and int(h4.sum()) == n2 - 1
    # small table, everything in one bin
    same = ops.fr_from_i32(torch.full(((1 << 20) + 1,), 5, dtype=torch.int32, device="cuda"))
    h3 = ops.tlookup_hist(same, 0, 16).cpu().numpy()
    assert h3[5] == (1 << 20) + 1 and h3.sum() == (1 << 20) + 1


@pytest.mark.parametrize("n", [5000, (1 << 20) + 77])
def test_index_histogram_and_inverse_by_table(ops, n):
    """indices made once serve the multiplicities and A = 1/(S+beta) = B[index]; elements that are
    outside the table or differ from their entry are reported, not written"""
    import torch
    low, length = -300, 1000
    rng = np.random.default_rng(33 + n)
    s = rng.integers(low, low + length, size=n).astype(np.int32)
    s[::11] = low + 5
    vals = ops.fr_from_i32(torch.from_numpy(s).cuda())
    idx1 = ops.tlookup_index(vals, low, length)
    assert np.array_equal(idx1.cpu().numpy(), s - low + 1)
    h = ops.tlookup_hist_index(idx1, length).cpu().numpy().view(np.uint32)
    assert np.array_equal(h, np.bincount(s.astype(np.int64) - low, minlength=length).astype(np.uint32))
    beta = ops.to_dev(br.fr_pack([length]))
    T, B = ops.tlookup_init(low, length, beta)
    A, mism = ops.tlookup_inverse_by_table(vals, idx1, T, B)
    assert mism == 0
    assert_same(ops.fr_to_host(A), ops.fr_to_host(ops.fr_shift_inverse(vals, beta)), "A from the table = batched inversion")
    # one value outside the table, one inside whose tensor element was altered afterwards
    s2 = s.copy()
    s2[7] = low + length + 3
    vals2 = ops.fr_from_i32(torch.from_numpy(s2).cuda())
    idx2 = ops.tlookup_index(vals2, low, length)
    assert idx2[7].item() == 0
    vals2[100] = ops.fr_from_i32(torch.tensor([int(s2[100]) + 1], dtype=torch.int32, device="cuda"))[0]
    A2, mism2 = ops.tlookup_inverse_by_table(vals2, idx2, T, B)
    assert mism2 == 2
    h2 = ops.tlookup_hist_index(idx2, length).cpu().numpy()
    assert h2.sum() == n - 1


def test_table_init(ops):
    low, length = -32768, 65536
    beta = br.fr_pack([length])
    T, B = ops.tlookup_init(low, length, ops.to_dev(beta))
    wT, wB = orc.tlookup_init(low, length, beta[0])
    assert_same(ops.fr_to_host(T), wT, "T")
    assert_same(ops.fr_to_host(B), wB, "B")
    mp = rand_fr(1024, 41)
    r = rand_fr(1, 42)
    T, B = ops.tlookup_init(-512, 1024, ops.to_dev(br.fr_pack([1024])), ops.to_dev(mp), ops.to_dev(r))
    wT, wB = orc.tlookup_init(-512, 1024, br.fr_pack([1024])[0], mp, r[0])
    assert_same(ops.fr_to_host(T), wT, "T mapped")
    assert_same(ops.fr_to_host(B), wB, "B mapped")


def test_tlookup_poly_kernels_and_fused_round(ops):
    n_out = 3000
    A, S = rand_fr(2 * n_out, 51), rand_fr(2 * n_out, 52)
    beta = rand_fr(1, 53)
    Ai, Si, bi = br.fr_unpack(A), br.fr_unpack(S), br.fr_unpack(beta)[0]
    o = [br.fr_unpack(ops.fr_to_host(t)) for t in ops.tlookup_poly(ops.to_dev(A), ops.to_dev(S), ops.to_dev(beta), n_out)]
    c00 = Ai[:n_out]
    c01 = [(Ai[t + n_out] - Ai[t]) % R for t in range(n_out)]
    c10 = [(Si[t] + bi) % R for t in range(n_out)]
    c11 = [(Si[t + n_out] - Si[t]) % R for t in range(n_out)]
    assert o[0] == [a * b % R for a, b in zip(c00, c10)]
    assert o[1] == [(a * b + c * d) % R for a, b, c, d in zip(c01, c10, c00, c11)]
    assert o[2] == [a * b % R for a, b in zip(c01, c11)]
    p = [br.fr_unpack(ops.fr_to_host(t)) for t in ops.tlookup_poly_sum(ops.to_dev(A), n_out)]
    assert p[0] == c00 and p[1] == c01
    # beta = NULL means zero
    o2 = [br.fr_unpack(ops.fr_to_host(t)) for t in ops.tlookup_poly(ops.to_dev(A), ops.to_dev(S), None, n_out)]
    assert o2[0] == [a * b % R for a, b in zip(c00, Si[:n_out])]


def test_fused_round_sums_equal_reference_steps(ops):
    # the fused kernel must give what the reference's poly kernel + three multilinear
    # evaluations + poly-sum kernel + two sums give (oracle restatement of those steps)
    logh = 12
    n_out = 1 << logh
    A, S = rand_fr(2 * n_out, 61), rand_fr(2 * n_out, 62)
    beta = rand_fr(1, 63)
    u = rand_fr(logh, 64)
    eq = ops.eq_table(ops.to_dev(u))
    sums = ops.fr_to_host(ops.tlookup_round_sums(ops.to_dev(A), ops.to_dev(S), ops.to_dev(beta), eq, n_out))
    o = [ops.fr_to_host(t) for t in ops.tlookup_poly(ops.to_dev(A), ops.to_dev(S), ops.to_dev(beta), n_out)]
    for k in range(3):
        assert_same(sums[k], orc.mle_eval(o[k], u), "weighted coefficient %d" % k)
    p = [ops.fr_to_host(t) for t in ops.tlookup_poly_sum(ops.to_dev(A), n_out)]
    assert_same(sums[3], orc.fr_sum(p[0]), "sum A0")
    assert_same(sums[4], orc.fr_sum(p[1]), "sum A1")
    m, B = rand_fr(2 * n_out, 65), rand_fr(2 * n_out, 66)
    mb = ops.fr_to_host(ops.tlookup_mb_sums(ops.to_dev(m), ops.to_dev(B), n_out))
    o = [ops.fr_to_host(t) for t in ops.tlookup_poly(ops.to_dev(m), ops.to_dev(B), None, n_out)]
    for k in range(3):
        assert_same(mb[k], orc.fr_sum(o[k]), "m*B coefficient %d" % k)


@pytest.mark.parametrize("n_out", [1, 3, 256, 5000, 1 << 16, (1 << 19) + 77])
def test_table_side_round_in_one_launch_equals_its_steps(ops, n_out):
    """grape_tlookup_table_round (sums over (B, T), sums over (m, B) and the fold of the three tensors, finished by the
    last workgroup of the launch) against the separate entry points; two rounds in a row on one stream, so that the
    second one finds the arrival counter as the first one left it"""
    logh = max(1, (n_out - 1).bit_length())
    beta, v = rand_fr(1, 163), rand_fr(2, 164)
    eq = ops.eq_table(ops.to_dev(rand_fr(logh, 165)))
    for rnd in range(2):
        B, T, m = rand_fr(2 * n_out, 160 + 10 * rnd), rand_fr(2 * n_out, 161 + 10 * rnd), rand_fr(2 * n_out, 162 + 10 * rnd)
        dB, dT, dm = ops.to_dev(B), ops.to_dev(T), ops.to_dev(m)
        want5 = ops.fr_to_host(ops.tlookup_round_sums(dB, dT, ops.to_dev(beta), eq, n_out))[:5]
        want3 = ops.fr_to_host(ops.tlookup_mb_sums(dm, dB, n_out))
        fB, fT, fm = ops.to_dev(B), ops.to_dev(T), ops.to_dev(m)
        dv = ops.to_dev(v[rnd:rnd + 1])
        ops.fr_fold_msb_multi([fB, fT, fm], n_out, dv)
        got = ops.fr_to_host(ops.tlookup_table_round(dB, dT, dm, ops.to_dev(beta), eq, n_out, dv))
        assert_same(got[:5], want5, "sums over (B, T)")
        assert_same(got[5:8], want3, "sums over (m, B)")
        for name, a, b in (("B", dB, fB), ("T", dT, fT), ("m", dm, fm)):
            assert_same(ops.fr_to_host(a)[:n_out], ops.fr_to_host(b)[:n_out], "folded " + name)


def test_eq_table_and_halving(ops):
    u = rand_fr(10, 71)
    ui = br.fr_unpack(u)
    e = ops.eq_table(ops.to_dev(u))
    got = br.fr_unpack(ops.fr_to_host(e))
    for i in (0, 1, 2, 513, 1023, 77):
        assert got[i] == br.eq_weight(i, ui)
    assert sum(got) % R == 1
    ops.eq_table_halve(e, 512)
    got2 = br.fr_unpack(ops.fr_to_host(e)[:512])
    for i in (0, 1, 511, 77):
        assert got2[i] == br.eq_weight(i, ui[:9])
    e0 = ops.eq_table(ops.to_dev(u), 0)
    assert br.fr_unpack(ops.fr_to_host(e0)) == [1]


def test_fold_msb_multi(ops):
    n_out = 5000
    ts = [rand_fr(2 * n_out, 80 + j) for j in range(5)]
    v = rand_fr(1, 90)
    dts = [ops.to_dev(t) for t in ts]
    ops.fr_fold_msb_multi(dts, n_out, ops.to_dev(v))
    for t, dt in zip(ts, dts):
        want = orc.partial_eval(t, 2 * n_out, v, 2, 0, n_out)[:n_out]
        assert_same(ops.fr_to_host(dt)[:n_out], want, "msb fold")


def test_eq_pyramid_levels(ops):
    """every level j of the pyramid is eq(u[0..j-1], .): against the product definition, the level's
    sum (1) and the older doubling table"""
    u = rand_fr(13, 171)
    ui = br.fr_unpack(u)
    pyr = ops.fr_to_host(ops.eq_pyramid(ops.to_dev(u)))
    assert pyr.shape[0] == (2 << 13) - 1
    for j in (0, 1, 2, 5, 9, 10, 11, 13):          # 9/10 straddle the one-workgroup head and the per-level launches
        lvl = br.fr_unpack(pyr[(1 << j) - 1:(2 << j) - 1])
        assert sum(lvl) % R == 1
        for i in {0, 1 % (1 << j), (1 << j) - 1, (1 << j) // 3, 77 % (1 << j)}:
            assert lvl[i] == br.eq_weight(i, ui[:j]), (j, i)
    assert_same(pyr[(1 << 13) - 1:], ops.fr_to_host(ops.eq_table(ops.to_dev(u))), "top level = eq table")
    assert br.fr_unpack(ops.fr_to_host(ops.eq_pyramid(ops.to_dev(u), 0))) == [1]


@pytest.mark.parametrize("in_size,n_out,beta,plain", [(2, 1, True, True), (8192, 4096, True, True), (8192, 4096, False, False),
                                                      (6001, 4096, False, False), (1 << 18, 1 << 17, True, True), (70000, 65536, True, False)])
def test_weighted_round_with_fused_fold(ops, in_size, n_out, beta, plain):
    """grape_wround2 against the unfused steps: coefficient arrays of the reference's kernel evaluated at
    the remaining variables (oracle), plain sums, and the MSB fold of both tensors (ragged upper halves
    read as zero)"""
    logh = br.log2ceil(n_out)
    A, S = rand_fr(in_size, 181 + in_size), rand_fr(in_size, 182 + in_size)
    bt, v, u = rand_fr(1, 183), rand_fr(1, 184), rand_fr(max(logh, 1), 185)
    Ap, Sp = np.zeros((2 * n_out, 4), dtype=np.uint64), np.zeros((2 * n_out, 4), dtype=np.uint64)
    Ap[:in_size], Sp[:in_size] = A, S
    dA, dS = ops.to_dev(A), ops.to_dev(S)
    e = ops.eq_pyramid(ops.to_dev(u), logh)[n_out - 1:2 * n_out - 1].contiguous()
    sums = ops.fr_to_host(ops.wround2(dA, dS, ops.to_dev(bt) if beta else None, e, in_size, n_out, ops.to_dev(v), plain_sums=plain))
    o = [ops.fr_to_host(t) for t in ops.tlookup_poly(ops.to_dev(Ap), ops.to_dev(Sp), ops.to_dev(bt) if beta else None, n_out)]
    for k in range(3):
        assert_same(sums[k], orc.mle_eval(o[k], u[:logh]), "weighted coefficient %d" % k)
    if plain:
        assert_same(sums[3], orc.fr_sum(Ap[:n_out]), "sum A0")
        assert_same(sums[4], orc.fr_sub(orc.fr_sum(Ap[n_out:]), orc.fr_sum(Ap[:n_out])), "sum A1 - A0")
    assert_same(ops.fr_to_host(dA)[:n_out], orc.partial_eval(Ap, 2 * n_out, v, 2, 0, n_out)[:n_out], "folded A")
    assert_same(ops.fr_to_host(dS)[:n_out], orc.partial_eval(Sp, 2 * n_out, v, 2, 0, n_out)[:n_out], "folded S")


@pytest.mark.parametrize("in_size,n_out", [(1 << 17, 1 << 16), ((1 << 18) - 1000, 1 << 17), (1 << 22, 1 << 21)])
def test_weighted_round_without_its_middle_coefficient(ops, in_size, n_out):
    """the long logUp rounds after the first: the variant that leaves the middle coefficient to the caller gives the other
    four sums and the folds of the general round (whose sums the tests above pin against the oracle), and writes zero
    in the middle slot; both fold through the table of the challenge's multiples at this size"""
    logh = br.log2ceil(n_out)
    A, S = rand_fr(in_size, 291 + n_out), rand_fr(in_size, 292 + n_out)
    bt, v, u = rand_fr(1, 293), rand_fr(1, 294), rand_fr(logh, 295)
    e = ops.eq_pyramid(ops.to_dev(u), logh)[n_out - 1:2 * n_out - 1].contiguous()
    dA1, dS1, dA2, dS2 = ops.to_dev(A), ops.to_dev(S), ops.to_dev(A), ops.to_dev(S)
    general = ops.fr_to_host(ops.wround2(dA1, dS1, ops.to_dev(bt), e, in_size, n_out, ops.to_dev(v), plain_sums=True))
    short = ops.fr_to_host(ops.wround2(dA2, dS2, ops.to_dev(bt), e, in_size, n_out, ops.to_dev(v), plain_sums=True, no_middle=True))
    assert_same(short[[0, 2, 3, 4]], general[[0, 2, 3, 4]], "the four sums")
    assert br.fr_unpack(short[1:2]) == [0]
    assert_same(ops.fr_to_host(dA2)[:n_out], ops.fr_to_host(dA1)[:n_out], "folded A")
    assert_same(ops.fr_to_host(dS2)[:n_out], ops.fr_to_host(dS1)[:n_out], "folded S")
    # the folds through the table against the oracle's fold
    assert_same(ops.fr_to_host(dA2)[:1000], orc.partial_eval(np.concatenate([A, np.zeros((2 * n_out - in_size, 4), dtype=np.uint64)]),
                                                               2 * n_out, v, 2, 0, n_out)[:1000], "folded A against the oracle")


@pytest.mark.parametrize("in_size,n_out,mode", [(1 << 17, 1 << 16, "no_middle"), ((1 << 18) - 1000, 1 << 17, "plain"), (1 << 19, 1 << 18, "three"),
                                                 (6000, 4096, "plain"), (1 << 18, 1 << 17, "no_table")])
def test_weighted_round_in_two_halves(ops, in_size, n_out, mode):
    """grape_fold_tables + grape_wround2_queue + grape_wround2_finish (work buffer and table of the caller's, finishing
    apart from the pass) against grape_wround2 on the same operands: sums and folds bit for bit"""
    logh = br.log2ceil(n_out)
    A, S = rand_fr(in_size, 301 + n_out), rand_fr(in_size, 302 + n_out)
    bt, v, u = rand_fr(1, 303), rand_fr(1, 304), rand_fr(logh, 305)
    e = ops.eq_pyramid(ops.to_dev(u), logh)[n_out - 1:2 * n_out - 1].contiguous()
    kw = dict(plain_sums=mode != "three", no_middle=mode == "no_middle")
    dA1, dS1, dA2, dS2 = ops.to_dev(A), ops.to_dev(S), ops.to_dev(A), ops.to_dev(S)
    whole = ops.fr_to_host(ops.wround2(dA1, dS1, ops.to_dev(bt), e, in_size, n_out, ops.to_dev(v), **kw))
    halves = ops.fr_to_host(ops.wround2_split(dA2, dS2, ops.to_dev(bt), e, in_size, n_out, ops.to_dev(v), table=mode != "no_table", **kw))
    assert_same(halves, whole, "sums")
    assert_same(ops.fr_to_host(dA2)[:n_out], ops.fr_to_host(dA1)[:n_out], "folded A")
    assert_same(ops.fr_to_host(dS2)[:n_out], ops.fr_to_host(dS1)[:n_out], "folded S")


@pytest.mark.parametrize("n_out", [1 << 16, 1 << 18])
def test_first_round_gathers_the_logup_tensor_from_its_table(ops, n_out):
    """a witness whose pass left only the table indices (A unwritten): the first round reads A[i] = B[index_i] itself and
    gives the sums, the folded A and the folded S of the round over the written-out tensor"""
    import torch
    low, length = -20000, 1 << 16
    n = 2 * n_out
    s = np.random.default_rng(311 + n_out).integers(low, low + length, size=n).astype(np.int32)
    vals = ops.fr_from_i32(torch.from_numpy(s).cuda())
    beta = ops.to_dev(br.fr_pack([length]))
    T, B = ops.tlookup_init(low, length, beta)
    idx_a, A, mism = ops.tlookup_index_inverse(vals, low, B)
    idx_b, none, mism_b = ops.tlookup_index_inverse(vals, low, B, write_A=False)
    assert mism == 0 and mism_b == 0 and none is None and torch.equal(idx_a, idx_b)
    logh = br.log2ceil(n_out)
    v, u = rand_fr(1, 312), rand_fr(logh, 313)
    e = ops.eq_pyramid(ops.to_dev(u), logh)[n_out - 1:2 * n_out - 1].contiguous()
    S1, S2 = vals.clone(), vals.clone()
    whole = ops.fr_to_host(ops.wround2(A, S1, beta, e, n, n_out, ops.to_dev(v), plain_sums=True, inverse_pair=True))
    sums, A2 = ops.wround2_first_indexed(S2, idx_b, B, beta, e, n_out, ops.to_dev(v))
    assert_same(ops.fr_to_host(sums), whole, "five sums")
    assert_same(ops.fr_to_host(A2), ops.fr_to_host(A)[:n_out], "folded A")
    assert_same(ops.fr_to_host(S2)[:n_out], ops.fr_to_host(S1)[:n_out], "folded S")
    # an element outside the table is counted by the index-only pass too
    s[5] = low + length + 9
    _, _, mism_c = ops.tlookup_index_inverse(ops.fr_from_i32(torch.from_numpy(s).cuda()), low, B, write_A=False)
    assert mism_c == 1


def test_fold_tables_of_several_challenges(ops):
    """one launch makes the tables of up to 64 challenges: table k equals the table made for challenge k alone"""
    import torch
    from grape_amd import _capi
    lib = ops.init()
    v = ops.to_dev(rand_fr(24, 306))
    many = torch.zeros(24 * 100, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_fold_tables(ops._p(many), ops._p(v), 24, None))
    for k in (0, 7, 23):
        one = torch.zeros(100, dtype=torch.int32, device="cuda")
        _capi.check(lib.grape_fold_tables(ops._p(one), ops._p(v[k:k + 1].contiguous()), 1, None))
        assert torch.equal(many[100 * k:100 * k + 100], one)
    with pytest.raises(_capi.GrapeError):
        _capi.check(lib.grape_fold_tables(ops._p(many), ops._p(v), 65, None))


@pytest.mark.parametrize("n_out,beta", [(1, True), (4096, True), (1 << 17, True), ((1 << 18), False)])
def test_weighted_round_of_an_inverse_pair(ops, n_out, beta):
    """the first round of a logUp proof, where A = 1/(S + beta): the variant that takes only the top
    coefficient (and writes 1 and its negative for the other two) gives the five sums and the folds
    of the general round, which in turn match the oracle's coefficients"""
    in_size = 2 * n_out
    logh = br.log2ceil(n_out)
    S = rand_fr(in_size, 281 + n_out)
    bt, v, u = rand_fr(1, 283), rand_fr(1, 284), rand_fr(max(logh, 1), 285)
    zero = np.zeros((1, 4), dtype=np.uint64)
    dbt = ops.to_dev(bt) if beta else None
    A = ops.fr_to_host(ops.fr_shift_inverse(ops.to_dev(S), ops.to_dev(bt if beta else zero)))
    e = ops.eq_pyramid(ops.to_dev(u), logh)[n_out - 1:2 * n_out - 1].contiguous()
    dA1, dS1, dA2, dS2 = ops.to_dev(A), ops.to_dev(S), ops.to_dev(A), ops.to_dev(S)
    general = ops.fr_to_host(ops.wround2(dA1, dS1, dbt, e, in_size, n_out, ops.to_dev(v), plain_sums=True))
    short = ops.fr_to_host(ops.wround2(dA2, dS2, dbt, e, in_size, n_out, ops.to_dev(v), plain_sums=True, inverse_pair=True))
    assert_same(short, general, "five sums")
    assert br.fr_unpack(short[:1]) == [1]
    assert_same(ops.fr_to_host(dA2)[:n_out], ops.fr_to_host(dA1)[:n_out], "folded A")
    assert_same(ops.fr_to_host(dS2)[:n_out], ops.fr_to_host(dS1)[:n_out], "folded S")
    if n_out <= 4096:
        o = [ops.fr_to_host(t) for t in ops.tlookup_poly(ops.to_dev(A), ops.to_dev(S), dbt, n_out)]
        for k in range(3):
            assert_same(short[k], orc.mle_eval(o[k], u[:logh]), "weighted coefficient %d" % k)


def test_weighted_round_on_padded_rows(ops):
    """rows of 11 elements whose weights live on rows padded to 16: row f, column j takes e[16 f + j]"""
    rows, rl, rp = 64, 11, 16
    n_out = rows * rl
    A, S = rand_fr(2 * n_out, 191), rand_fr(2 * n_out, 192)
    v, u = rand_fr(1, 193), rand_fr(10, 194)
    e = ops.eq_pyramid(ops.to_dev(u))[(1 << 10) - 1:].contiguous()        # 64 x 16 weights
    dA, dS = ops.to_dev(A), ops.to_dev(S)
    sums = br.fr_unpack(ops.fr_to_host(ops.wround2(dA, dS, None, e, 2 * n_out, n_out, ops.to_dev(v), rowlen=rl, rowpad=rp)))
    Ai, Si, ui = br.fr_unpack(A), br.fr_unpack(S), br.fr_unpack(u)
    want = [0, 0, 0]
    for f in range(rows):
        for j in range(rl):
            g = f * rl + j
            w = br.eq_weight(f * rp + j, ui)
            a0, a1, s0, s1 = Ai[g], Ai[g + n_out] - Ai[g], Si[g], Si[g + n_out] - Si[g]
            want[0] += w * a0 * s0
            want[1] += w * (a0 * s1 + a1 * s0)
            want[2] += w * a1 * s1
    assert sums == [x % R for x in want]


@pytest.mark.parametrize("nseg,seglen,ragged", [(1, 8, 0), (4, 96, 0), (32, 128, 0), (2, 20000, 0), (8, 300, 1000),
                                                (70000, 2, 3)])      # more segments than one launch's grid holds
def test_segment_weighted_round(ops, nseg, seglen, ragged):
    """grape_sumcheck_round2_seg: the three sums of every segment of seglen indices times that segment's
    weight, and the folds - against the plain round kernel run per segment"""
    out = nseg * seglen
    in_size = 2 * out - ragged
    A, B = rand_fr(in_size, 201 + nseg), rand_fr(in_size, 202 + nseg)
    v, w = rand_fr(1, 203), rand_fr(nseg, 204)
    dA, dB = ops.to_dev(A), ops.to_dev(B)
    got = ops.fr_to_host(ops.sumcheck_round2_seg(dA, dB, in_size, out, seglen, ops.to_dev(w), ops.to_dev(v)))
    wA, wB, wa, wb, wc = _oracle_round2(A, B, in_size, out, v)
    want = [np.zeros(4, dtype=np.uint64)] * 3
    for s_ in range(nseg):
        sl = slice(s_ * seglen, (s_ + 1) * seglen)
        for k, arr in enumerate((wc, wb, wa)):
            want[k] = orc.fr_add(want[k], orc.fr_mul(w[s_], orc.fr_sum(arr[sl])))
    for k in range(3):
        assert_same(got[k], want[k], "coefficient %d" % k)
    assert_same(ops.fr_to_host(dA)[:out], wA[:out], "folded A")
    assert_same(ops.fr_to_host(dB)[:out], wB[:out], "folded B")


def test_weighted_sums_of_one_tensor_against_several_tables(ops):
    n_out, logh, num = 1 << 13, 13, 5
    for in_size in (2 * n_out, 2 * n_out - 1000):
        X = rand_fr(in_size, 211)
        Xp = np.zeros((2 * n_out, 4), dtype=np.uint64)
        Xp[:in_size] = X
        us = [rand_fr(logh, 212 + j) for j in range(num)]
        tabs = [ops.eq_pyramid(ops.to_dev(uj))[n_out - 1:].contiguous() for uj in us]
        dX = ops.to_dev(X)
        got = ops.fr_to_host(ops.wsum1_multi(dX, tabs, in_size, n_out))
        assert_same(ops.fr_to_host(dX), X, "tensor untouched")
        d = orc.vec2("orc_fr_vec_sub", Xp[n_out:], Xp[:n_out])
        for j in range(num):
            assert_same(got[2 * j], orc.mle_eval(Xp[:n_out], us[j]), "claim %d, X0" % j)
            assert_same(got[2 * j + 1], orc.mle_eval(d, us[j]), "claim %d, X1 - X0" % j)


@pytest.mark.parametrize("in_size", [1 << 18, (1 << 18) - 3000, 5000, (1 << 22) - 12345])
def test_sumcheck_rounds_chained_through_their_claim(ops, in_size):
    """grape_sumcheck_round2_claim over four rounds in a row against grape_sumcheck_round2: the same
    three sums and folded tensors in every round (the middle coefficient comes from the claim), and the
    claim it leaves is the round polynomial's value at the challenge; sizes on both sides of the
    table-fold threshold, ragged included"""
    A, B = rand_fr(in_size, 401), rand_fr(in_size, 402)
    v = rand_fr(4, 403)
    dA, dB = ops.to_dev(A), ops.to_dev(B)
    cA, cB = ops.to_dev(A), ops.to_dev(B)
    Ai, Bi = br.fr_unpack(A), br.fr_unpack(B)
    claim = sum(x * y for x, y in zip(Ai, Bi)) % R
    d_claim = ops.to_dev(br.fr_pack([claim]))
    n_in = in_size
    n_out = 1 << (br.log2ceil(in_size) - 1)
    for k in range(4):
        dv = ops.to_dev(v[k:k + 1])
        want = ops.fr_to_host(ops.sumcheck_round2(dA, dB, n_in, n_out, dv))
        got = ops.fr_to_host(ops.sumcheck_round2_claim(cA, cB, n_in, n_out, dv, d_claim))
        assert_same(got, want, "sums of round %d" % k)
        assert_same(ops.fr_to_host(cA)[:n_out], ops.fr_to_host(dA)[:n_out], "folded A, round %d" % k)
        assert_same(ops.fr_to_host(cB)[:n_out], ops.fr_to_host(dB)[:n_out], "folded B, round %d" % k)
        c0, c1, c2 = br.fr_unpack(want)
        vk = br.fr_unpack(v[k:k + 1])[0]
        assert (2 * c0 + c1 + c2) % R == claim
        claim = (c0 + c1 * vk + c2 * vk * vk) % R
        assert br.fr_unpack(ops.fr_to_host(d_claim)) == [claim]
        n_in, n_out = n_out, n_out // 2
