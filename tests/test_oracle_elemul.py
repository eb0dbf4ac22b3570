"""Pins the oracle's element-wise product sumcheck (prove_eleMul) and claim merging
(combine_claims) by brute force over Python integers: every round polynomial is recomputed from
its definition at t = 0..3, the claim chain is followed, and the returned evaluations are the
multilinear extensions at the bound point.  Shapes include a non-power-of-two last axis, which
the reference treats as zero-padded to the next power of two."""
import random
import pytest
import bigref as br
import orc

R = br.R_MOD


def _poly_at(coeffs, t):
    return sum(c * pow(t, i, R) for i, c in enumerate(coeffs)) % R


@pytest.mark.parametrize("L,M,N", [(1, 4, 8), (2, 2, 4), (1, 1, 16), (1, 4, 6), (2, 1, 5), (1, 2, 1)])
def test_prove_elemul_transcript(L, M, N):
    rng = random.Random(1000 + L * 100 + M * 10 + N)
    first, size = L * M, L * M * N
    Np = 1 << br.log2ceil(N)
    k = br.log2ceil(first) + br.log2ceil(N)
    assert k == br.log2ceil(size)
    A = [rng.randrange(R) for _ in range(size)]
    B = [rng.randrange(R) for _ in range(size)]
    u = [rng.randrange(R) for _ in range(k)]
    v = [rng.randrange(R) for _ in range(k)]
    pad = lambda X: [X[f * N + n] if n < N else 0 for f in range(first) for n in range(Np)]
    a1, b1 = pad(A), pad(B)
    claim0 = sum(br.eq_weight(i, u) * a1[i] * b1[i] for i in range(len(a1))) % R
    st, tr, final_claim, ac, bc = orc.prove_elemul(br.fr_pack(A), br.fr_pack(B), L, M, N, br.fr_pack(u), br.fr_pack(v),
                                                  br.fr_pack([claim0])[0])
    assert st == 0 and tr.shape[0] == k
    claim, eq_acc = claim0, 1
    for i in range(k):
        half = len(a1) // 2
        ut, vt, u_low = u[k - 1 - i], v[k - 1 - i], u[:k - 1 - i]

        def at(t):
            tot = 0
            for lo in range(half):
                a = (a1[lo] + t * (a1[lo + half] - a1[lo])) % R
                b = (b1[lo] + t * (b1[lo + half] - b1[lo])) % R
                tot += br.eq_weight(lo, u_low) * a * b
            return tot % R * eq_acc % R * br.eq1(ut, t) % R
        coeffs = br.fr_unpack(tr[i])
        for t in (0, 1, 2, 3):
            assert _poly_at(coeffs, t) == at(t), (i, t)
        assert (_poly_at(coeffs, 0) + _poly_at(coeffs, 1)) % R == claim
        claim = _poly_at(coeffs, vt)
        eq_acc = eq_acc * br.eq1(ut, vt) % R
        a1 = [(a1[lo] + vt * (a1[lo + half] - a1[lo])) % R for lo in range(half)]
        b1 = [(b1[lo] + vt * (b1[lo + half] - b1[lo])) % R for lo in range(half)]
    assert br.fr_unpack(final_claim)[0] == claim
    assert br.fr_unpack(ac)[0] == a1[0] == br.mle_eval(pad(A), v)
    assert br.fr_unpack(bc)[0] == b1[0] == br.mle_eval(pad(B), v)
    assert a1[0] * b1[0] % R * eq_acc % R == claim


def test_prove_elemul_detects_wrong_claim_and_bad_shape():
    rng = random.Random(5)
    A = [rng.randrange(R) for _ in range(8)]
    B = [rng.randrange(R) for _ in range(8)]
    u = [rng.randrange(R) for _ in range(3)]
    v = [rng.randrange(R) for _ in range(3)]
    st, _, _, _, _ = orc.prove_elemul(br.fr_pack(A), br.fr_pack(B), 1, 2, 4, br.fr_pack(u), br.fr_pack(v), br.fr_pack([12345])[0])
    assert st == 1
    st, tr, _, _, _ = orc.prove_elemul(br.fr_pack(A + A[:4]), br.fr_pack(B + B[:4]), 1, 3, 4, br.fr_pack(u + u[:1]), br.fr_pack(v + v[:1]),
                                       br.fr_pack([0])[0])
    assert st == 4 and tr.shape[0] == 0      # L*M must be a power of two (src/prove.cu:122-124)


@pytest.mark.parametrize("nv,num", [(4, 3), (3, 1), (1, 2), (5, 4)])
def test_combine_claims_transcript(nv, num):
    rng = random.Random(2000 + nv * 10 + num)
    size = 1 << nv
    X = [rng.randrange(R) for _ in range(size)]
    us = [[rng.randrange(R) for _ in range(nv)] for _ in range(num)]
    v = [rng.randrange(R) for _ in range(nv)]
    claims = [br.mle_eval(X, uj) for uj in us]
    st, tr, ret = orc.combine_claims(br.fr_pack(X), br.fr_pack(claims), [br.fr_pack(uj) for uj in us], br.fr_pack(v))
    assert st == 0 and tr.shape[0] == nv
    claim = sum(claims) % R
    eq_acc = [1] * num
    x1 = list(X)
    for i in range(nv):
        half = len(x1) // 2
        left = nv - 1 - i
        vt = v[left]

        def at(t):
            xt = [(x1[lo] + t * (x1[lo + half] - x1[lo])) % R for lo in range(half)]
            return sum(eq_acc[j] * br.eq1(us[j][left], t) * br.mle_eval(xt, us[j][:left]) for j in range(num)) % R
        coeffs = br.fr_unpack(tr[i])
        assert coeffs[3] == 0
        for t in (0, 1, 2):
            assert _poly_at(coeffs, t) == at(t), (i, t)
        assert (_poly_at(coeffs, 0) + _poly_at(coeffs, 1)) % R == claim
        claim = _poly_at(coeffs, vt)
        for j in range(num):
            eq_acc[j] = eq_acc[j] * br.eq1(us[j][left], vt) % R
        x1 = [(x1[lo] + vt * (x1[lo + half] - x1[lo])) % R for lo in range(half)]
    assert br.fr_unpack(ret)[0] == x1[0] == br.mle_eval(X, v)
    assert sum(eq_acc) % R * x1[0] % R == claim


def test_combine_claims_detects_wrong_claim():
    rng = random.Random(7)
    X = [rng.randrange(R) for _ in range(8)]
    us = [[rng.randrange(R) for _ in range(3)] for _ in range(2)]
    v = [rng.randrange(R) for _ in range(3)]
    claims = [br.mle_eval(X, us[0]), (br.mle_eval(X, us[1]) + 1) % R]
    st, _, _ = orc.combine_claims(br.fr_pack(X), br.fr_pack(claims), [br.fr_pack(uj) for uj in us], br.fr_pack(v))
    assert st == 1
