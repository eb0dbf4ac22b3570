"""Pins the oracle's G1 arithmetic, generator table and both commitment paths against textbook
affine chord-and-tangent arithmetic on Python integers and a naive sum_i s_i*G_i."""
import random
import numpy as np
import bigref as br
import orc


def _gens(n, seed):
    rng = random.Random(seed)
    ks = [rng.randrange(1, br.R_MOD) for _ in range(n)]
    return ks, orc.g1_make_generators(br.ints_to_limbs(ks, 4))


def test_generator_and_order():
    g = br.g1_unpack(orc.g1_generator())[0]
    assert g == br.G1 and br.g1_on_curve(g)
    assert br.g1_mul(br.R_MOD, br.G1) is None            # the group has order r
    out = np.zeros(br.G1_WORDS, dtype=np.uint64)
    orc.lib().orc_g1_scalar_mul(orc.P(out), orc.P(orc.g1_generator()), orc.P(br.ints_to_limbs([br.R_MOD], 4)))
    assert br.g1_unpack(out)[0] is None


def test_scalar_mul_vs_textbook():
    ks, gens = _gens(6, 11)
    ks += [1, 2, br.R_MOD - 1]
    gens = np.concatenate([gens, orc.g1_make_generators(br.ints_to_limbs([1, 2, br.R_MOD - 1], 4))])
    for k, pt in zip(ks, br.g1_unpack(gens)):
        assert pt == br.g1_mul(k, br.G1)
        assert br.g1_on_curve(pt)
        assert orc.lib().orc_g1_on_curve(orc.P(br.g1_pack([pt])[0])) == 1


def test_add_special_cases():
    a = br.g1_mul(5, br.G1)
    b = br.g1_mul(7, br.G1)
    cases = [(a, b), (a, a), (a, br.g1_neg(a)), (None, a), (a, None), (None, None)]
    for x, y in cases:
        out = np.zeros(br.G1_WORDS, dtype=np.uint64)
        orc.lib().orc_g1_add_affine(orc.P(out), orc.P(br.g1_pack([x])[0]), orc.P(br.g1_pack([y])[0]))
        assert br.g1_unpack(out)[0] == br.g1_add(x, y)


def test_table_matches_multiples():
    ks, gens = _gens(3, 12)
    W = 20
    table = br.g1_unpack(orc.g1_table(gens, W))
    pts = br.g1_unpack(gens)
    for w in range(W):
        for i in range(3):
            assert table[w * 3 + i] == br.g1_mul(w, pts[i])   # entry 0 is infinity = (0,0)


def test_commit_i32_vs_naive():
    n, rows = 8, 5
    ks, gens = _gens(n, 13)
    pts = br.g1_unpack(gens)
    table = orc.g1_table(gens, 256)
    rng = random.Random(14)
    S = [[rng.randrange(-2**31, 2**31) for _ in range(n)] for _ in range(rows)]
    S[0] = [0] * n                                   # all-zero row -> infinity
    S[1] = [0] * n
    S[1][3] = -1                                     # single -1 -> -G_3
    S[2][0], S[2][1] = 255, -256                     # window boundaries
    S[3] = [-2**31, 2**31 - 1, 65535, -65536, 1, -1, 32768, -32768]
    got = br.g1_unpack(orc.commit_i32(np.array(S, dtype=np.int32), table, n, n))
    want = [br.g1_msm(row, pts) for row in S]
    assert got == want
    assert got[0] is None and got[1] == br.g1_neg(pts[3])
    for r in range(rows):
        naive = br.g1_unpack(orc.msm_naive_i64(np.array(S[r], dtype=np.int64), gens))[0]
        assert naive == want[r]


def test_commit_fr_vs_naive_and_int_path():
    n, rows = 4, 3
    ks, gens = _gens(n, 15)
    pts = br.g1_unpack(gens)
    table = orc.g1_table(gens, 256)
    rng = random.Random(16)
    S = [[rng.randrange(br.R_MOD) for _ in range(n)] for _ in range(rows)]
    S[1] = [0, 1, br.R_MOD - 1, 255]
    flat = [s for row in S for s in row]
    got = br.g1_unpack(orc.commit_fr(br.fr_pack(flat), table, n, n))
    assert got == [br.g1_msm(row, pts) for row in S]
    # the same small integers through both paths give the same points
    small = np.array([[5, -7, 300, -70000], [0, 0, 1, -1]], dtype=np.int32)
    a = orc.commit_i32(small, table, n, n)
    b = orc.commit_fr(orc.from_i32(small.reshape(-1)), table, n, n)
    assert np.array_equal(a, b)


def test_commit_linearity_and_table_stride():
    # npoints (table stride) larger than the row length, as Hyrax uses it
    n, npoints = 4, 6
    ks, gens = _gens(npoints, 17)
    table = orc.g1_table(gens, 256)
    a = np.array([[3, -4, 1000, 77]], dtype=np.int32)
    b = np.array([[-9, 14, 2, -77]], dtype=np.int32)
    ca = br.g1_unpack(orc.commit_i32(a, table, n, npoints))[0]
    cb = br.g1_unpack(orc.commit_i32(b, table, n, npoints))[0]
    cab = br.g1_unpack(orc.commit_i32(a + b, table, n, npoints))[0]
    assert cab == br.g1_add(ca, cb)
