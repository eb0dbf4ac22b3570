"""Pins the oracle's fold (FrTensor::partial_eval) and multilinear evaluation against the
definition T(u) = sum_i t[i] * prod_j (u_j if bit_j(i) else 1-u_j), including extents that are
not powers of two (the missing partner of an odd tail counts as zero)."""
import random
import pytest
import bigref as br
import orc


def _rand(rng, n):
    return [rng.randrange(br.R_MOD) for _ in range(n)]


@pytest.mark.parametrize("outer,c,gap", [(1, 8, 1), (1, 11, 3), (3, 5, 4), (2, 16, 2), (4, 2, 8),
                                         (1, 1, 5), (5, 7, 1), (2, 13, 1), (1, 2, 16)])
def test_partial_eval_vs_definition(outer, c, gap):
    rng = random.Random(outer * 1000 + c * 10 + gap)
    n = outer * c * gap
    t = _rand(rng, n)
    L = br.log2ceil(c)
    pre = 2
    x = _rand(rng, pre + L + 1)          # challenges live at x[id : id+L]
    out = orc.partial_eval(br.fr_pack(t), n, br.fr_pack(x), c, pre, gap)
    want = br.fold_axis(t, outer, c, gap, x[pre:pre + L])
    assert br.fr_unpack(out[: outer * gap]) == want


@pytest.mark.parametrize("n", [1, 2, 3, 8, 11, 64, 100])
def test_mle_eval_vs_definition(n):
    rng = random.Random(n)
    t = _rand(rng, n)
    u = _rand(rng, br.log2ceil(n))
    if n == 1 << br.log2ceil(n):
        got = br.fr_unpack(orc.mle_eval(br.fr_pack(t), br.fr_pack(u)))[0]
    else:
        # operator()(u) reads a short tensor as rows of 11008; a general odd length goes
        # through the fold itself (c = n, gap = 1)
        got = br.fr_unpack(orc.partial_eval(br.fr_pack(t), n, br.fr_pack(u), n, 0, 1)[:1])[0]
    assert got == br.mle_eval(t, u)


def test_mle_eval_boolean_points_and_linearity():
    rng = random.Random(5)
    n = 16
    t = _rand(rng, n)
    for i in (0, 1, 6, 15):
        u = [(i >> j) & 1 for j in range(4)]
        assert br.fr_unpack(orc.mle_eval(br.fr_pack(t), br.fr_pack(u)))[0] == t[i]
    s = _rand(rng, n)
    u = _rand(rng, 4)
    a = br.fr_unpack(orc.mle_eval(br.fr_pack(t), br.fr_pack(u)))[0]
    b = br.fr_unpack(orc.mle_eval(br.fr_pack(s), br.fr_pack(u)))[0]
    ab = br.fr_unpack(orc.mle_eval(br.fr_pack([(x + y) % br.R_MOD for x, y in zip(t, s)]), br.fr_pack(u)))[0]
    assert ab == (a + b) % br.R_MOD


def test_mle_eval_11008_columns():
    # a tensor of k*11008 elements evaluated at a point of log2(k)+14 variables is read as
    # [k][11008] with each row zero-extended to 16384
    rng = random.Random(6)
    k = 2
    t = [rng.randrange(-2**15, 2**15) % br.R_MOD for _ in range(k * 11008)]
    u = _rand(rng, 15)
    got = br.fr_unpack(orc.mle_eval(br.fr_pack(t), br.fr_pack(u)))[0]
    padded = []
    for r in range(k):
        padded += t[r * 11008:(r + 1) * 11008] + [0] * (16384 - 11008)
    # brute force with vectorised weights to stay fast
    w_lo = [1]
    for uj in u[:14]:
        w_lo = [w * (1 - uj) % br.R_MOD for w in w_lo] + [w * uj % br.R_MOD for w in w_lo]
    rows = [sum(a * b for a, b in zip(padded[r * 16384:(r + 1) * 16384], w_lo)) % br.R_MOD for r in range(k)]
    want = (rows[0] * (1 - u[14]) + rows[1] * u[14]) % br.R_MOD
    assert got == want
