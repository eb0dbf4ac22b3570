"""TEST INFRASTRUCTURE - CPU oracle of the quantised-layer witness generator.

A numpy restatement of the fixed-point rules of the reference's witness generator
(zzllama/llama/model.py): every tensor a decoder layer hands to the prover, as exact integers.
It exists to check the HIP kernels and the C++ host class; nothing in the shipped libraries may
import or run it.  Only the test-suite, the smoke check and the benchmark's cpu_baseline leg do.

Rules restated (file:line of zzllama/llama/model.py):
  * scales SCALE = 2^16, swiglu_scale = 2^20, qk_scale = 2^22                       (:22-24)
  * rescaling of an exact product y by S: q = floor((y + S/2) / S), r = y - q*S      (:489-491)
    (round half up; r in [-S/2, S/2))
  * products are exact integers (the reference multiplies in float64 below 2^53)      (:485-487)
  * softmax through the exp table: index = x - rowmax + 2^20 - 1, e = table[index],
    sum over the row, out = floor((e*SCALE + sum/2) / sum) (sum/2 floored),
    lookup query 2*SCALE*e - sum*(2*out - 1)                                          (:76-116)
  * SiLU through its table: index = x + 2^18, 19-bit range                            (:118-149)
  * RMSNorm: rms = float16(1/sqrt(mean((x/SCALE)^2) + eps)), rms_int = round(rms*SCALE),
    rms_w = rescale(rms_int * w), out = rescale(rms_w.q * x)                          (:216-257)
  * attention with one head, no rotary embedding, no mask, K/V straight from this call (:473-590)
  * feed-forward: gate rescaled by 2^20 into the SiLU table, up by 2^16, product and
    down projection rescaled by 2^16                                                  (:634-703)
  * block: h = x + attention(norm1(x)), out = h + ffn(norm2(h))                       (:760-775)
  * tensor names are the reference's file names under data/{W,Q,R}/                   (:46-63)

Where this restatement is not bit-faithful to the reference: the reference takes the mean of
squares in float32 with torch's reduction order and rsqrt in float32 before the float16 cast;
here the sum of squares is an exact integer and the rest is IEEE double arithmetic (one divide,
one add, one sqrt, one divide), then round-to-nearest-even to float16.  The float16 result can
differ from torch's only when 1/sqrt lies within float32 rounding noise of a float16 tie.  rms is
an advice value of the prover (every proved relation takes rms_int as given), so either choice
yields a valid witness; the rule above is the one the product implements, bit for bit.

How each function is pinned (tests/test_witness_oracle.py): rescale against Python big-integer
floor division and its two invariants; softmax against exact rational arithmetic (the output is
the nearest integer to e*SCALE/sum, ties up, iff the lookup query lies in [0, 2*sum)); the float16
rounding against a brute-force nearest-neighbour search over all float16 values with exact
rationals; matmul against Python integers; the layer against its own proved relations
(q*S + r = product for every rescaling, remainders inside the lookup ranges, table rows hit).
"""
import numpy as np

SCALE = 1 << 16          # model.py:22
SWIGLU_SCALE = 1 << 20   # model.py:23
QK_SCALE = 1 << 22       # model.py:24
EXP_BIT_SHIFT, EXP_INDEX_BITS = 20, 20      # model.py:565 (my_softmax(q_scores, lut, 20, 20))
SILU_BIT_SHIFT, SILU_INDEX_BITS = 18, 19    # model.py:666 (my_silu(x, lut, 18, 19))
NORM_EPS = 1e-5                             # model.py:162


def rescale(y, s):
    """exact int64 products -> (quotient, remainder) int32: model.py:489-491, :654-658"""
    y = np.asarray(y, dtype=np.int64)
    q = (y + s // 2) // s                  # numpy's // floors, like torch's on integers
    r = y - q * s
    assert np.all(np.abs(q) < (1 << 31)), "quotient leaves int32"
    return q.astype(np.int32), r.astype(np.int32)


def matmul_t(a, w):
    """a[n][k] . w[m][k] summed over k, exact (int64): model.py:485-487"""
    return np.matmul(np.asarray(a, dtype=np.int64), np.asarray(w, dtype=np.int64).T)


def exp_table():
    """The table the softmax indexes (the reference loads data/table/exp-table.bin, which is not in
    its tree): entry i stands for x = i - (2^20 - 1) <= 0 at the scores' scale 2^16 and holds
    round(exp(x / 2^16) * 2^16), so table[2^20 - 1] = SCALE."""
    x = np.arange(1 << EXP_INDEX_BITS, dtype=np.float64) - ((1 << EXP_BIT_SHIFT) - 1)
    return np.rint(np.exp(x / SCALE) * SCALE).astype(np.int32)


def silu_table():
    """The SiLU table (data/table/swiglu-table.bin in the reference, not in its tree): entry i stands
    for x = i - 2^18 at scale 2^12 (gate products are rescaled by 2^20, model.py:657) and holds
    round(x * sigmoid(x) * 2^16)."""
    x = (np.arange(1 << SILU_INDEX_BITS, dtype=np.float64) - (1 << SILU_BIT_SHIFT)) / float(1 << 12)
    return np.rint(x / (1.0 + np.exp(-x)) * SCALE).astype(np.int32)


def lut(x, table, offset, index_bits):
    """table[x + offset] with the reference's range assertions: model.py:84-95, :132-142"""
    idx = np.asarray(x, dtype=np.int64) + offset
    if np.any(idx < 0) or np.any(idx > (1 << index_bits) - 1):
        raise ValueError("table index out of range")
    return table[idx]


def softmax(q_scores, table):
    """model.py:76-116; returns the tensors it saves, all int32 as save_int writes them"""
    x = np.asarray(q_scores, dtype=np.int32)
    x_max = x.max(axis=-1, keepdims=True)
    shifted = x - x_max
    e = lut(shifted, table, (1 << EXP_BIT_SHIFT) - 1, EXP_INDEX_BITS).astype(np.int64)
    s = e.sum(axis=-1, keepdims=True)
    if np.any(s <= 0):
        raise ValueError("softmax row sums to zero")
    out = (e * SCALE + s // 2) // s
    query = e * 2 * SCALE - s * (2 * out - 1)
    return {"max": x_max.astype(np.int32), "exp_input": shifted.astype(np.int32), "exp_output": e.astype(np.int32),
            "exp_sum": s.astype(np.int32), "softmax_output": out.astype(np.int32),
            "softmax_lookup_query": query.astype(np.int32)}


def to_float16(x):
    """IEEE round-to-nearest-even of doubles to float16, returned as doubles"""
    return np.asarray(x, dtype=np.float64).astype(np.float16).astype(np.float64)


def rms_int(x, eps=NORM_EPS):
    """per row: round(float16(1 / sqrt(sum(x^2) / (D * 2^32) + eps)) * 2^16): model.py:193, :211-214"""
    x = np.asarray(x, dtype=np.int64)
    ss = np.array([sum(int(v) * int(v) for v in row) for row in x.reshape(-1, x.shape[-1])], dtype=object)
    assert all(v < (1 << 64) for v in ss), "sum of squares leaves 64 bits"
    s = np.array([float(v) for v in ss], dtype=np.float64)           # int -> double, correctly rounded
    t = s / (float(x.shape[-1]) * 4294967296.0) + eps
    h = to_float16(1.0 / np.sqrt(t))
    return np.rint(h * SCALE).astype(np.int64).astype(np.int32).reshape(x.shape[:-1] + (1,))


def rmsnorm(x, w, eps=NORM_EPS):
    """model.py:216-257 (w already round(weight * SCALE)); returns the six saved tensors"""
    x = np.asarray(x, dtype=np.int64)
    r_int = rms_int(x, eps)
    rms_w = r_int.astype(np.int64) * np.asarray(w, dtype=np.int64).reshape(1, -1)
    q_rms_w, r_rms_w = rescale(rms_w, SCALE)
    q_out, r_out = rescale(q_rms_w.astype(np.int64) * x, SCALE)
    return {"rms": r_int, "q_rmsw": q_rms_w, "r_rmsw": r_rms_w, "q_out": q_out, "r_out": r_out}


def attention(x, WQ, WK, WV, WO, table):
    """model.py:473-590 with one head; names are the reference's file names"""
    out = {}
    out["Q/xq"], out["R/xq"] = rescale(matmul_t(x, WQ), SCALE)
    out["Q/xk"], out["R/xk"] = rescale(matmul_t(x, WK), SCALE)
    q_xv, r_xv = rescale(matmul_t(x, WV), SCALE)
    out["Q/xv"], out["R/xv"] = np.ascontiguousarray(q_xv.T), np.ascontiguousarray(r_xv.T)     # saved transposed, :500-501
    out["Q/scores"], out["R/scores"] = rescale(matmul_t(out["Q/xq"], out["Q/xk"]), QK_SCALE)
    for k, v in softmax(out["Q/scores"], table).items():
        out["Q/" + k] = v
    out["Q/qkv"], out["R/qkv"] = rescale(matmul_t(out["Q/softmax_output"], q_xv.T), SCALE)
    out["Q/atten_out"], out["R/atten_out"] = rescale(matmul_t(out["Q/qkv"], WO), SCALE)
    return out


def feed_forward(x, w1, w2, w3, table):
    """model.py:634-703 (w1 = gate, w2 = down, w3 = up)"""
    out = {"Q/ffn_input": np.asarray(x, dtype=np.int32)}
    out["Q/up_out"], out["R/up_out"] = rescale(matmul_t(x, w3), SCALE)
    out["Q/gate_out"], out["R/gate_out"] = rescale(matmul_t(x, w1), SWIGLU_SCALE)
    out["Q/silu_out"] = lut(out["Q/gate_out"], table, 1 << SILU_BIT_SHIFT, SILU_INDEX_BITS).astype(np.int32)
    prod = out["Q/silu_out"].astype(np.int64) * out["Q/up_out"].astype(np.int64)
    out["Q/upSilu"], out["R/upSilu"] = rescale(prod, SCALE)
    out["Q/down_out"], out["R/down_out"] = rescale(matmul_t(out["Q/upSilu"], w2), SCALE)
    return out


def layer(x, weights, tables, eps=NORM_EPS):
    """One transformer block, model.py:760-775.  weights: dict with int32 arrays Q, K, V, O (dim x
    dim), gate, up (hidden x dim), down (dim x hidden), NormFirst, NormSecond (dim); tables: dict
    with 'exp' and 'silu'.  Returns {name: int32 array} named as the files the reference writes."""
    x = np.asarray(x, dtype=np.int32)
    out = {"Q/input": x}
    for k in ("Q", "K", "V", "O", "gate", "up", "down", "NormFirst", "NormSecond"):
        out["W/" + k] = np.asarray(weights[k], dtype=np.int32)
    n1 = rmsnorm(x, weights["NormFirst"], eps)
    out["Q/rmsFirst"], out["Q/rmswFirst"], out["R/rmswFirst"] = n1["rms"], n1["q_rmsw"], n1["r_rmsw"]
    out["Q/normOutFirst"], out["R/normOutFirst"] = n1["q_out"], n1["r_out"]
    out.update(attention(n1["q_out"], weights["Q"], weights["K"], weights["V"], weights["O"], tables["exp"]))
    h = (x.astype(np.int64) + out["Q/atten_out"]).astype(np.int32)
    out["Q/skip"] = h
    n2 = rmsnorm(h, weights["NormSecond"], eps)
    out["Q/rmsSecond"], out["Q/rmswSecond"], out["R/rmswSecond"] = n2["rms"], n2["q_rmsw"], n2["r_rmsw"]
    out["Q/normOutSecond"], out["R/normOutSecond"] = n2["q_out"], n2["r_out"]
    out.update(feed_forward(n2["q_out"], weights["gate"], weights["down"], weights["up"], tables["silu"]))
    out["Q/output"] = (h.astype(np.int64) + out["Q/down_out"]).astype(np.int32)
    return out
