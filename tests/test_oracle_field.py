"""Pins the oracle's Fr / Fp arithmetic against closed forms on Python integers.

Results of every operation are canonical residues, so a correct implementation is unique:
the Montgomery product of packed a, b must be the packing of a*b mod m, and so on.  Edge
vectors exercise carries in every limb, the modulus boundary and zero.
"""
import random
import numpy as np
import bigref as br
import orc


def _edge_values(mod):
    vals = [0, 1, 2, mod - 1, mod - 2, (1 << 32) - 1, 1 << 32, (1 << 64) - 1, 1 << 64,
            (1 << 128) - 1, mod >> 1, (mod >> 1) + 1, (1 << 255) % mod, ((1 << 256) - 1) % mod]
    vals += [((1 << (64 * k)) - 1) % mod for k in range(1, 7)]
    return vals


def test_fr_constants_closed_form():
    # the oracle's "one" is 2^256 mod r: packing 1 must give it, and mul by packed 1 is identity
    one = br.fr_pack([1])[0]
    x = br.fr_pack([0x1234567890abcdef1234567890abcdef])[0]
    assert np.array_equal(orc.fr_mul(x, one), x)
    assert br.limbs_to_ints(one)[0] == (1 << 256) % br.R_MOD


def test_fr_ops_vs_bigint():
    rng = random.Random(1)
    vals = _edge_values(br.R_MOD) + [rng.randrange(br.R_MOD) for _ in range(40)]
    for a in vals:
        for b in vals[:20] + vals[-6:]:
            pa, pb = br.fr_pack([a])[0], br.fr_pack([b])[0]
            assert br.fr_unpack(orc.fr_add(pa, pb))[0] == (a + b) % br.R_MOD
            assert br.fr_unpack(orc.fr_sub(pa, pb))[0] == (a - b) % br.R_MOD
            assert br.fr_unpack(orc.fr_mul(pa, pb))[0] == (a * b) % br.R_MOD
            # outputs are canonical limbs, not just congruent
            assert br.limbs_to_ints(orc.fr_mul(pa, pb))[0] < br.R_MOD
        pa = br.fr_pack([a])[0]
        assert br.fr_unpack(orc.fr_neg(pa))[0] == (-a) % br.R_MOD
        inv = br.fr_unpack(orc.fr_inv(pa))[0]
        assert inv == (pow(a, -1, br.R_MOD) if a else 0)   # 1/0 = 0 convention


def test_fp_ops_vs_bigint():
    rng = random.Random(2)
    vals = _edge_values(br.P_MOD) + [rng.randrange(br.P_MOD) for _ in range(30)]
    for a in vals:
        for b in vals[:16] + vals[-6:]:
            pa, pb = br.fp_pack([a])[0], br.fp_pack([b])[0]
            assert br.fp_unpack(orc.fp_add(pa, pb))[0] == (a + b) % br.P_MOD
            assert br.fp_unpack(orc.fp_sub(pa, pb))[0] == (a - b) % br.P_MOD
            assert br.fp_unpack(orc.fp_mul(pa, pb))[0] == (a * b) % br.P_MOD
        pa = br.fp_pack([a])[0]
        assert br.fp_unpack(orc.fp_neg(pa))[0] == (-a) % br.P_MOD
        inv = br.fp_unpack(orc.fp_inv(pa))[0]
        assert inv == (pow(a, -1, br.P_MOD) if a else 0)


def test_montgomery_in_out():
    rng = random.Random(3)
    vals = [0, 1, br.R_MOD - 1] + [rng.randrange(br.R_MOD) for _ in range(20)]
    plain = br.ints_to_limbs(vals, 4)
    mont = orc.vec1("orc_fr_vec_to_mont", plain)
    assert br.limbs_to_ints(mont) == [v * br.FR_R % br.R_MOD for v in vals]
    back = orc.vec1("orc_fr_vec_from_mont", mont)
    assert br.limbs_to_ints(back) == vals


def test_int_embedding():
    xs = np.array([0, 1, -1, 2, -2, 32767, -32768, 2**31 - 1, -2**31, 123456, -654321], dtype=np.int32)
    got = br.fr_unpack(orc.from_i32(xs))
    assert got == [int(x) % br.R_MOD for x in xs]          # negatives are r - |x|
    us = np.array([0, 1, 2**32 - 1, 65536], dtype=np.uint32)
    assert br.fr_unpack(orc.from_u32(us)) == [int(x) for x in us]


def test_vector_ops_and_sum():
    rng = random.Random(4)
    n = 1000
    a = [rng.randrange(br.R_MOD) for _ in range(n)]
    b = [rng.randrange(br.R_MOD) for _ in range(n)]
    pa, pb = br.fr_pack(a), br.fr_pack(b)
    assert br.fr_unpack(orc.vec2("orc_fr_vec_mul", pa, pb)) == [x * y % br.R_MOD for x, y in zip(a, b)]
    assert br.fr_unpack(orc.vec2("orc_fr_vec_add", pa, pb)) == [(x + y) % br.R_MOD for x, y in zip(a, b)]
    assert br.fr_unpack(orc.vec2("orc_fr_vec_sub", pa, pb)) == [(x - y) % br.R_MOD for x, y in zip(a, b)]
    assert br.fr_unpack(orc.vec_bcast("orc_fr_vec_bcast_mul", pa, pb[7])) == [x * b[7] % br.R_MOD for x in a]
    assert br.fr_unpack(orc.vec_bcast("orc_fr_vec_bcast_add", pa, pb[7])) == [(x + b[7]) % br.R_MOD for x in a]
    assert br.fr_unpack(orc.fr_sum(pa))[0] == sum(a) % br.R_MOD
    a[5] = 0
    pa = br.fr_pack(a)
    assert br.fr_unpack(orc.vec1("orc_fr_vec_inv", pa)) == [pow(x, -1, br.R_MOD) if x else 0 for x in a]


def test_log2_is_ceil():
    L = orc.lib().orc_log2
    assert [L(n) for n in (0, 1, 2, 3, 4, 5, 8, 9, 11008, 16384, 16385)] == [0, 0, 1, 2, 2, 3, 3, 4, 14, 14, 15]
