"""Pins the oracle's tlookup / logUp restatement: multiplicities against numpy.bincount, the
logUp identity sum_j 1/(S_j+beta) = sum_i m_i/(T_i+beta), every round polynomial recomputed by
brute force from its definition on Python integers, and the returned value against the
multilinear extension of the witness at v."""
import random
import numpy as np
import pytest
import bigref as br
import orc

R = br.R_MOD


def _poly_at(coeffs, t):
    return sum(c * pow(t, i, R) for i, c in enumerate(coeffs)) % R


def _inv(x):
    return pow(x % R, -1, R)


def test_histogram_vs_bincount_and_pad_fixup():
    rng = np.random.default_rng(1)
    low, length = -8, 16
    s = rng.integers(low, low + length, size=100).astype(np.int32)
    h = orc.histogram(orc.from_i32(s), low, length)
    assert np.array_equal(h, np.bincount(s - low, minlength=length).astype(np.uint32))
    # a witness of 100 values is padded with zeros to 128: 28 extra hits on the bin of value 0
    m = br.fr_unpack(orc.tlookup_prep(orc.from_i32(s), low, length))
    want = np.bincount(s - low, minlength=length)
    want[-low] += 28
    assert m == [int(x) for x in want]


def test_table_init():
    low, length = -4, 8
    beta = length
    T, B = orc.tlookup_init(low, length, br.fr_pack([beta])[0])
    assert br.fr_unpack(T) == [(low + i) % R for i in range(length)]
    assert br.fr_unpack(B) == [_inv(low + i + beta) for i in range(length)]
    rng = random.Random(2)
    mp = [rng.randrange(-100, 100) % R for _ in range(length)]
    r = rng.randrange(R)
    T2, B2 = orc.tlookup_init(low, length, br.fr_pack([beta])[0], br.fr_pack(mp), br.fr_pack([r])[0])
    assert br.fr_unpack(T2) == [(low + i + r * mp[i]) % R for i in range(length)]
    assert br.fr_unpack(B2) == [_inv(low + i + r * mp[i] + beta) for i in range(length)]


@pytest.mark.parametrize("logD,logN,low", [(4, 2, -2), (5, 3, -4), (3, 3, 0), (6, 2, -1)])
def test_tlookup_prove_transcript(logD, logN, low):
    rng = random.Random(logD * 10 + logN)
    D, N = 1 << logD, 1 << logN
    S = [rng.randrange(low, low + N) for _ in range(D)]
    beta = N                                     # beta is the table size, not a random challenge
    alpha = rng.randrange(R)
    u = [rng.randrange(R) for _ in range(logD)]
    v = [rng.randrange(R) for _ in range(logD)]
    Sp = orc.from_i32(np.array(S, dtype=np.int32))
    T, B = orc.tlookup_init(low, N, br.fr_pack([beta])[0])
    m = orc.tlookup_prep(Sp, low, N)
    st, tr, s_claim = orc.tlookup_prove(Sp, T, B, m, br.fr_pack([alpha])[0], br.fr_pack([beta])[0],
                                        br.fr_pack(u), br.fr_pack(v))
    assert st == 0
    assert tr.shape[0] == logD

    # brute-force model
    Sv = [s % R for s in S]
    Av = [_inv(s + beta) for s in Sv]
    Tv = [(low + i) % R for i in range(N)]
    Bv = [_inv(t + beta) for t in Tv]
    mv = [int(x) for x in np.bincount(np.array(S) - low, minlength=N)]
    assert sum(Av) % R == sum(a * b for a, b in zip(mv, Bv)) % R          # logUp identity
    a, a2 = alpha, alpha * alpha % R
    C = (a2 - sum(x * y for x, y in zip(Bv, mv))) % R
    claim = (alpha + a2) % R
    rho = N * _inv(D) % R
    half_inv = _inv(2)
    uu = list(u)
    fold = lambda X, h, vt: [(X[g] + vt * (X[g + h] - X[g])) % R for g in range(h)]
    at_t = lambda X, h, g, t: (X[g] + t * (X[g + h] - X[g])) % R
    rnd = 0
    for i in range(logD - logN):                 # phase 1
        h = len(Av) // 2
        ut, vt = uu[-1], v[logD - 1 - i]
        ulow = uu[:-1]
        def p(t):
            s1 = sum(br.eq_weight(g, ulow) * at_t(Av, h, g, t) * (at_t(Sv, h, g, t) + beta) for g in range(h))
            s2 = sum(at_t(Av, h, g, t) for g in range(h))
            return (a * br.eq1(ut, t) * s1 + s2 + C * half_inv) % R
        coeffs = br.fr_unpack(tr[rnd])
        for t in (0, 1, 2, 3):
            assert _poly_at(coeffs, t) == p(t)
        assert (_poly_at(coeffs, 0) + _poly_at(coeffs, 1)) % R == claim
        claim = _poly_at(coeffs, vt)
        Av, Sv = fold(Av, h, vt), fold(Sv, h, vt)
        a = a * br.eq1(ut, vt) % R
        C = C * half_inv % R
        uu.pop()
        rnd += 1
    for i in range(logN):                        # phase 2
        h = len(Av) // 2
        ut, vt = uu[-1], v[logN - 1 - i]
        ulow = uu[:-1]
        def p(t):
            s1 = sum(br.eq_weight(g, ulow) * at_t(Av, h, g, t) * (at_t(Sv, h, g, t) + beta) for g in range(h))
            s2 = sum(br.eq_weight(g, ulow) * at_t(Bv, h, g, t) * (at_t(Tv, h, g, t) + beta) for g in range(h))
            s3 = sum(at_t(Av, h, g, t) for g in range(h))
            s4 = sum(at_t(mv, h, g, t) * at_t(Bv, h, g, t) for g in range(h))
            return (br.eq1(ut, t) * (a * s1 + rho * a2 * s2) + s3 - rho * s4) % R
        coeffs = br.fr_unpack(tr[rnd])
        for t in (0, 1, 2, 3):
            assert _poly_at(coeffs, t) == p(t)
        assert (_poly_at(coeffs, 0) + _poly_at(coeffs, 1)) % R == claim
        claim = _poly_at(coeffs, vt)
        Av, Sv, Bv, Tv, mv = (fold(X, h, vt) for X in (Av, Sv, Bv, Tv, mv))
        a = a * br.eq1(ut, vt) % R
        a2 = a2 * br.eq1(ut, vt) % R
        uu.pop()
        rnd += 1
    assert br.fr_unpack(s_claim)[0] == Sv[0] == br.mle_eval([s % R for s in S], v)


def test_tlookup_rejects_out_of_range_witness():
    # a value outside the table breaks the logUp identity: the first round check must fail
    rng = random.Random(7)
    logD, N, low = 4, 4, 0
    S = [rng.randrange(0, 4) for _ in range(16)]
    S[3] = 9
    beta = N
    Sp = orc.from_i32(np.array(S, dtype=np.int32))
    T, B = orc.tlookup_init(low, N, br.fr_pack([beta])[0])
    m = orc.tlookup_prep(Sp, low, N)
    u = [rng.randrange(R) for _ in range(logD)]
    v = [rng.randrange(R) for _ in range(logD)]
    st, _, _ = orc.tlookup_prove(Sp, T, B, m, br.fr_pack([5])[0], br.fr_pack([beta])[0], br.fr_pack(u), br.fr_pack(v))
    assert st != 0
