"""Pins the oracle's matmul sumcheck (prove_matmul) by brute force: every round polynomial is
recomputed from its definition at t = 0, 1, 2 (and 3 for the cubic phase-1 rounds) over plain
Python integers, the first claim is Y(u) for an exact integer matrix product, and the final
evaluations are the multilinear extensions of A and B at the bound point."""
import random
import numpy as np
import pytest
import bigref as br
import orc

R = br.R_MOD


def _poly_at(coeffs, t):
    return sum(c * pow(t, i, R) for i, c in enumerate(coeffs)) % R


def _setup(L, N, M, K, seed):
    rng = random.Random(seed)
    A = np.array([rng.randrange(-2**15, 2**15) for _ in range(L * N * K)], dtype=np.int64).reshape(L, N, K)
    B = np.array([rng.randrange(-2**15, 2**15) for _ in range(L * M * K)], dtype=np.int64).reshape(L, M, K)
    Y = np.einsum("lnk,lmk->lnm", A.astype(object), B.astype(object))      # exact integers
    lM, lN, lL, lK = br.log2ceil(M), br.log2ceil(N), br.log2ceil(L), br.log2ceil(K)
    u = [rng.randrange(R) for _ in range(lM + lN + lL)]
    v = [rng.randrange(R) for _ in range(lK + lL)]
    return A, B, Y, u, v, (lM, lN, lL, lK)


@pytest.mark.parametrize("L,N,M,K", [(1, 4, 8, 16), (2, 4, 4, 8), (4, 2, 4, 4), (1, 3, 5, 6), (1, 8, 4, 1)])
def test_prove_matmul_transcript(L, N, M, K):
    A, B, Y, u, v, (lM, lN, lL, lK) = _setup(L, N, M, K, L * 100 + N * 10 + K)
    # claim = Y(u) with Y indexed [l][n][m], m fastest; zero-extend each axis to a power of two
    Mp, Np, Lp = 1 << lM, 1 << lN, 1 << lL
    Ypad = [0] * (Lp * Np * Mp)
    for l in range(L):
        for n in range(N):
            for m in range(M):
                Ypad[(l * Np + n) * Mp + m] = int(Y[l, n, m]) % R
    claim0 = br.mle_eval(Ypad, u)
    Af = [int(x) % R for x in A.reshape(-1)]
    Bf = [int(x) % R for x in B.reshape(-1)]
    st, tr, final_claim, ac, bc = orc.prove_matmul(br.fr_pack(Af), br.fr_pack(Bf), L, N, M, K,
                                                  br.fr_pack(u), br.fr_pack(v), br.fr_pack([claim0])[0])
    assert st == 0
    assert tr.shape[0] == lL + lK

    # brute-force model: Abar[l][k], Bbar[l][k] after binding n and m
    u_m, u_n, u_l = u[:lM], u[lM:lM + lN], u[lM + lN:]
    v_k, v_l = v[:lK], v[lK:]
    Kp = 1 << lK
    Abar = [[sum(int(A[l, n, k]) * br.eq_weight(n, u_n) for n in range(N)) % R if k < K else 0
             for k in range(Kp)] for l in range(L)] + [[0] * Kp for _ in range(Lp - L)]
    Bbar = [[sum(int(B[l, m, k]) * br.eq_weight(m, u_m) for m in range(M)) % R if k < K else 0
             for k in range(Kp)] for l in range(L)] + [[0] * Kp for _ in range(Lp - L)]
    claim = claim0
    eq_acc = 1
    rnd = 0
    # phase 1: top layer bit first, challenges taken from the back of v_l / u_l
    for i in range(lL):
        half = len(Abar) // 2
        ut, vt = u_l[lL - 1 - i], v_l[lL - 1 - i]
        u_low = u_l[:lL - 1 - i]
        def at(t):
            tot = 0
            for lo in range(half):
                w = br.eq_weight(lo, u_low)
                for k in range(Kp):
                    a = (Abar[lo][k] + t * (Abar[lo + half][k] - Abar[lo][k])) % R
                    b = (Bbar[lo][k] + t * (Bbar[lo + half][k] - Bbar[lo][k])) % R
                    tot += w * a * b
            return tot % R * eq_acc % R * br.eq1(ut, t) % R
        coeffs = br.fr_unpack(tr[rnd])
        for t in (0, 1, 2, 3):
            assert _poly_at(coeffs, t) == at(t)
        assert (_poly_at(coeffs, 0) + _poly_at(coeffs, 1)) % R == claim
        claim = _poly_at(coeffs, vt)
        eq_acc = eq_acc * br.eq1(ut, vt) % R
        Abar = [[(Abar[lo][k] + vt * (Abar[lo + half][k] - Abar[lo][k])) % R for k in range(Kp)] for lo in range(half)]
        Bbar = [[(Bbar[lo][k] + vt * (Bbar[lo + half][k] - Bbar[lo][k])) % R for k in range(Kp)] for lo in range(half)]
        rnd += 1
    a1, b1 = Abar[0], Bbar[0]
    for i in range(lK):
        half = len(a1) // 2
        vt = v_k[lK - 1 - i]
        def at2(t):
            return sum(((a1[k] + t * (a1[k + half] - a1[k])) % R) * ((b1[k] + t * (b1[k + half] - b1[k])) % R)
                       for k in range(half)) % R * eq_acc % R
        coeffs = br.fr_unpack(tr[rnd])
        assert coeffs[3] == 0
        for t in (0, 1, 2):
            assert _poly_at(coeffs, t) == at2(t)
        assert (_poly_at(coeffs, 0) + _poly_at(coeffs, 1)) % R == claim
        claim = _poly_at(coeffs, vt)
        a1 = [(a1[k] + vt * (a1[k + half] - a1[k])) % R for k in range(half)]
        b1 = [(b1[k] + vt * (b1[k + half] - b1[k])) % R for k in range(half)]
        rnd += 1
    assert br.fr_unpack(final_claim)[0] == claim
    assert br.fr_unpack(ac)[0] == a1[0] and br.fr_unpack(bc)[0] == b1[0]
    assert a1[0] * b1[0] % R * eq_acc % R == claim
    # final evaluations are the MLEs of A and B at (v_k | u_n | v_l) and (v_k | u_m | v_l)
    Apad = [0] * (Lp * Np * Kp)
    for l in range(L):
        for n in range(N):
            for k in range(K):
                Apad[(l * Np + n) * Kp + k] = int(A[l, n, k]) % R
    assert br.mle_eval(Apad, v_k + u_n + v_l) == a1[0]


def test_prove_matmul_detects_wrong_claim():
    A, B, Y, u, v, _ = _setup(1, 2, 2, 4, 9)
    Af = [int(x) % R for x in A.reshape(-1)]
    Bf = [int(x) % R for x in B.reshape(-1)]
    st, *_ = orc.prove_matmul(br.fr_pack(Af), br.fr_pack(Bf), 1, 2, 2, 4, br.fr_pack(u), br.fr_pack(v),
                              br.fr_pack([12345])[0])
    assert st == 2
