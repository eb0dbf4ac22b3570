"""Pins of the witness-generator oracle (oracle/witness_oracle.py) by checks that do not retype its
formulas: Python big integers and exact rationals, brute force over all float16 values, and the
relations the prover later proves about the tensors."""
from fractions import Fraction
import numpy as np
import pytest
from oracle import witness_oracle as wo
import witutil


def test_rescale_is_round_half_up_with_centred_remainder():
    rng = np.random.default_rng(1)
    ys = np.concatenate([rng.integers(-(1 << 52), 1 << 52, 4000), np.array([0, 1, -1, 32767, 32768, -32768, -32769, 98304, -98304])])
    for s in (1 << 16, 1 << 20, 1 << 22, 1000):
        q, r = wo.rescale(ys % (s << 30) - (s << 29), s)
        for y, qi, ri in zip((ys % (s << 30) - (s << 29)).tolist(), q.tolist(), r.tolist()):
            assert qi * s + ri == y                       # exact decomposition
            assert -(s // 2) <= ri < s - s // 2           # remainder range the lookup proves
            # nearest integer to y/s, ties towards +infinity
            f = Fraction(y, s)
            assert abs(f - qi) <= Fraction(1, 2) and (f - qi != Fraction(1, 2))


def test_matmul_is_exact_on_large_entries():
    rng = np.random.default_rng(2)
    a = rng.integers(-(1 << 24), 1 << 24, (5, 37))
    w = rng.integers(-(1 << 24), 1 << 24, (4, 37))
    got = wo.matmul_t(a, w)
    want = [[sum(int(a[i, k]) * int(w[j, k]) for k in range(37)) for j in range(4)] for i in range(5)]
    assert got.tolist() == want


def test_float16_rounding_against_brute_force():
    """nearest float16 (ties to even mantissa) by exact rational search over every finite float16"""
    bits = np.arange(0x7c00, dtype=np.uint16)            # all non-negative finite values
    vals = bits.view(np.float16).astype(np.float64)
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.uniform(0, 400, 300), rng.uniform(0, 2, 300), rng.uniform(0, 0.01, 100),
                         (vals[1000:1400] + vals[1001:1401]) / 2])          # exact ties
    got = wo.to_float16(xs)
    for x, g in zip(xs.tolist(), got.tolist()):
        i = int(np.searchsorted(vals, x))
        cands = [j for j in (i - 1, i, i + 1) if 0 <= j < len(vals)]
        best = min(cands, key=lambda j: (abs(Fraction(vals[j]) - Fraction(x)), j & 1))
        assert g == vals[best], (x, g, vals[best])


def test_rms_int_matches_exact_arithmetic():
    rng = np.random.default_rng(4)
    x = np.rint(rng.normal(0, 65536.0, (16, 64))).astype(np.int64)
    x[3] = 0                                              # all-zero row: rms = float16(1/sqrt(eps))
    x[4] = 1 << 20
    got = wo.rms_int(x).reshape(-1)
    for row, g in zip(x.tolist(), got.tolist()):
        ms = sum(v * v for v in row) / (64 * 4294967296.0) + 1e-5
        true = 1.0 / ms ** 0.5
        h = g / 65536.0
        # the float16 value behind rms_int is within half a float16 step (2^-11 relative) of the true value
        assert abs(h - true) <= true * 2.0 ** -11 * 1.001 + 2.0 ** -17
    assert got[3] == int(np.rint(float(np.float16(1.0 / np.sqrt(1e-5))) * 65536))


def test_softmax_is_nearest_integer_and_query_range():
    rng = np.random.default_rng(5)
    table = wo.exp_table()
    scores = np.rint(rng.normal(0, 65536.0, (12, 50))).astype(np.int32)
    s = wo.softmax(scores, table)
    assert s["exp_input"].max() == 0 and np.all(s["exp_input"].max(axis=-1) == 0)
    assert np.array_equal(s["exp_output"], table[s["exp_input"].astype(np.int64) + (1 << 20) - 1])
    assert np.array_equal(s["exp_sum"].reshape(-1), s["exp_output"].astype(np.int64).sum(axis=-1))
    for e_row, o_row, q_row, tot in zip(s["exp_output"].tolist(), s["softmax_output"].tolist(),
                                        s["softmax_lookup_query"].tolist(), s["exp_sum"].reshape(-1).tolist()):
        for e, o, q in zip(e_row, o_row, q_row):
            f = Fraction(e * 65536, tot)
            assert abs(f - o) <= Fraction(1, 2)
            assert 0 <= q < 2 * tot                      # what the range lookup proves
            assert q == 2 * 65536 * e - tot * (2 * o - 1)
    # rows of probabilities sum to 1 at scale 2^16 up to rounding
    assert np.all(np.abs(s["softmax_output"].astype(np.int64).sum(axis=-1) - 65536) <= 50)


def test_tables_have_the_documented_anchors():
    e, s = wo.exp_table(), wo.silu_table()
    assert e.shape == (1 << 20,) and s.shape == (1 << 19,)
    assert e[-1] == 65536 and e[0] == 0 and np.all(np.diff(e.astype(np.int64)) >= 0)
    assert s[1 << 18] == 0 and s[(1 << 18) + 4096] == int(np.rint(65536 / (1 + np.exp(-1.0))))
    assert abs(int(s[-1]) - (64 * 65536 - 16)) <= 16 and abs(int(s[0])) <= 1


def test_lookup_rejects_out_of_range_like_the_reference():
    t = wo.silu_table()
    with pytest.raises(ValueError):
        wo.lut(np.array([1 << 18]), t, 1 << 18, 19)
    with pytest.raises(ValueError):
        wo.lut(np.array([-(1 << 18) - 1]), t, 1 << 18, 19)


def test_layer_satisfies_the_proved_relations():
    T, D, F = 8, 64, 176
    x, weights = witutil.layer_inputs(T, D, F, seed=6)
    tables = {"exp": wo.exp_table(), "silu": wo.silu_table()}
    w = wo.layer(x, weights, tables)
    i64 = lambda a: np.asarray(a, dtype=np.int64)
    S = 1 << 16

    def prod(a, b):            # a[n][k] b[m][k], Python integers
        return np.array([[sum(int(p) * int(q) for p, q in zip(ra, rb)) for rb in b.tolist()] for ra in a.tolist()], dtype=np.int64)

    checks = [("xq", w["Q/normOutFirst"], w["W/Q"], S), ("xk", w["Q/normOutFirst"], w["W/K"], S),
              ("scores", w["Q/xq"], w["Q/xk"], 1 << 22), ("qkv", w["Q/softmax_output"], w["Q/xv"], S),
              ("atten_out", w["Q/qkv"], w["W/O"], S), ("up_out", w["Q/normOutSecond"], w["W/up"], S),
              ("gate_out", w["Q/normOutSecond"], w["W/gate"], 1 << 20), ("down_out", w["Q/upSilu"], w["W/down"], S)]
    for name, a, b, s in checks:
        assert np.array_equal(i64(w["Q/" + name]) * s + i64(w["R/" + name]), prod(a, b)), name
        assert w["R/" + name].min() >= -(s // 2) and w["R/" + name].max() < s // 2, name
    assert np.array_equal(i64(w["Q/xv"]).T * S + i64(w["R/xv"]).T, prod(w["Q/normOutFirst"], w["W/V"]))
    for tag, src in (("First", w["Q/input"]), ("Second", w["Q/skip"])):
        assert np.array_equal(i64(w["Q/rmsw" + tag]) * S + i64(w["R/rmsw" + tag]), i64(w["Q/rms" + tag]) * i64(w["W/Norm" + tag]).reshape(1, -1))
        assert np.array_equal(i64(w["Q/normOut" + tag]) * S + i64(w["R/normOut" + tag]), i64(w["Q/rmsw" + tag]) * i64(src))
    assert np.array_equal(i64(w["Q/upSilu"]) * S + i64(w["R/upSilu"]), i64(w["Q/silu_out"]) * i64(w["Q/up_out"]))
    assert np.array_equal(w["Q/silu_out"], tables["silu"][i64(w["Q/gate_out"]) + (1 << 18)])
    assert np.array_equal(i64(w["Q/skip"]), i64(w["Q/input"]) + i64(w["Q/atten_out"]))
    assert np.array_equal(i64(w["Q/output"]), i64(w["Q/skip"]) + i64(w["Q/down_out"]))
    assert np.array_equal(w["Q/ffn_input"], w["Q/normOutSecond"])
    # the normalised activations have unit RMS at scale 2^16 (norm weights are 1 +- 3 %)
    rms = np.sqrt((i64(w["Q/normOutFirst"]).astype(np.float64) ** 2).mean(axis=-1)) / 65536
    assert np.all(np.abs(rms - 1.0) < 3e-2)
    assert set(w) == set(witutil.TENSOR_NAMES)
