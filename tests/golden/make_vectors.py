#!/usr/bin/env python3
"""Writes tests/golden/vectors.json (BLS12-381) or, under GRAPE_CURVE=bn254,
tests/golden/vectors_bn254.json: small known-answer vectors for the proving hot path.

The reference ships no vectors for this path, so these are computed here from the definitions
with Python integers only (tests/bigref.py: `%` arithmetic, textbook affine chord-and-tangent
group law, brute-force multilinear extensions).  Neither the C oracle nor the HIP library is
involved.  Values are canonical integers (not Montgomery residues) as hex strings; points are
affine [x, y] or null for the point at infinity.  The seeded draws freeze the generator of the
test inputs (numpy PCG64 through tests/gpuutil.rand_fr).

    python tests/golden/make_vectors.py        # rewrites vectors.json (deterministic)
"""
import json
import os
import random
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import bigref as br          # noqa: E402
from gpuutil import rand_fr  # noqa: E402

R = br.R_MOD


def hx(v):
    return hex(v)


def pt(p):
    return None if p is None else [hex(p[0]), hex(p[1])]


def main():
    rng = random.Random(20240917)
    out = {"modulus_r": hx(R), "modulus_p": hx(br.P_MOD)}

    # ---- Fr arithmetic
    edge = [0, 1, 2, R - 1, R - 2, (1 << 255) % R, (1 << 256) % R, (1 << 64) - 1, R >> 1]
    vals = edge + [rng.randrange(R) for _ in range(8)]
    fr = []
    for i, a in enumerate(vals):
        b = vals[(i * 7 + 3) % len(vals)]
        fr.append({"a": hx(a), "b": hx(b), "add": hx((a + b) % R), "sub": hx((a - b) % R), "mul": hx(a * b % R),
                   "inv_a": hx(pow(a, -1, R) if a else 0)})          # 1/0 = 0 (include/field/mont_t.cuh:1113-1119)
    out["fr"] = fr
    out["from_i32"] = [{"x": x, "fr": hx(x % R)} for x in (0, 1, -1, 32767, -32768, 2**31 - 1, -2**31)]

    # ---- the seeded test-input generator
    out["seeded_fr"] = {"seed": 7, "values": [hx(v) for v in br.fr_unpack(rand_fr(4, 7))]}

    # ---- G1
    G = br.G1
    ks = [1, 2, 3, 255, 256, 65535, R - 1, rng.randrange(R)]
    out["g1_multiples"] = [{"k": hx(k), "point": pt(br.g1_mul(k, G))} for k in ks]
    gen_scalars = br.fr_unpack(rand_fr(4, 11))
    gens = [br.g1_mul(s, G) for s in gen_scalars]
    out["generators"] = {"seed": 11, "scalars": [hx(s) for s in gen_scalars], "points": [pt(p) for p in gens]}
    out["g1_add"] = [{"a": pt(gens[0]), "b": pt(gens[1]), "sum": pt(br.g1_add(gens[0], gens[1]))},
                     {"a": pt(gens[2]), "b": pt(gens[2]), "sum": pt(br.g1_add(gens[2], gens[2]))},
                     {"a": pt(gens[3]), "b": pt(br.g1_neg(gens[3])), "sum": None},
                     {"a": None, "b": pt(gens[1]), "sum": pt(gens[1])}]

    # ---- Hyrax row commitments over the 4 generators above (rows of 4)
    ints = [[3, -1, 0, 32767], [-32768, 255, 256, -257], [0, 0, 0, 0]]
    out["commit_i32"] = {"rows": ints, "commitments": [pt(br.g1_msm([x % R for x in row], gens)) for row in ints]}
    frs = [[rng.randrange(R) for _ in range(4)] for _ in range(2)]
    out["commit_fr"] = {"rows": [[hx(x) for x in row] for row in frs],
                        "commitments": [pt(br.g1_msm(row, gens)) for row in frs]}

    # ---- fold (partial multilinear evaluation) and full evaluation
    folds = []
    for outer, c, gap in ((1, 4, 3), (2, 3, 2), (1, 11, 1), (3, 5, 4)):
        t = [rng.randrange(R) for _ in range(outer * c * gap)]
        x = [rng.randrange(R) for _ in range(br.log2ceil(c))]
        folds.append({"outer": outer, "c": c, "gap": gap, "t": [hx(v) for v in t], "x": [hx(v) for v in x],
                      "out": [hx(v) for v in br.fold_axis(t, outer, c, gap, x)]})
    out["fold"] = folds
    t = [rng.randrange(R) for _ in range(13)]
    u = [rng.randrange(R) for _ in range(4)]
    out["mle_eval"] = {"t": [hx(v) for v in t], "u": [hx(v) for v in u], "value": hx(br.mle_eval(t, u))}

    # ---- one sumcheck round of two tensors (src/prove.cu:29-46 and :101-105)
    rounds = []
    for in_size, out_size in ((8, 4), (7, 4), (5, 4)):
        A = [rng.randrange(R) for _ in range(in_size)]
        B = [rng.randrange(R) for _ in range(in_size)]
        v = rng.randrange(R)
        hiA = [A[g + out_size] if g + out_size < in_size else 0 for g in range(out_size)]
        hiB = [B[g + out_size] if g + out_size < in_size else 0 for g in range(out_size)]
        Aa = [(h - l) % R for h, l in zip(hiA, A)]
        Ba = [(h - l) % R for h, l in zip(hiB, B)]
        rounds.append({"in_size": in_size, "out_size": out_size, "A": [hx(x) for x in A], "B": [hx(x) for x in B], "v": hx(v),
                       "sums": [hx(sum(A[g] * B[g] for g in range(out_size)) % R),
                                hx(sum(Aa[g] * B[g] + A[g] * Ba[g] for g in range(out_size)) % R),
                                hx(sum(Aa[g] * Ba[g] for g in range(out_size)) % R)],
                       "A_folded": [hx((A[g] + v * Aa[g]) % R) for g in range(out_size)],
                       "B_folded": [hx((B[g] + v * Ba[g]) % R) for g in range(out_size)]})
    out["sumcheck_round2"] = rounds

    # ---- logUp table and multiplicities (src/tlookup.cu:5-30, :250-263)
    low, length, beta = -4, 8, 8
    S = [-4, 3, 3, 0, -1, 3, 2, -4, 0, 3, 7, -9]            # the last two are outside the range
    m = [sum(1 for s in S if s == low + t) for t in range(length)]
    out["tlookup"] = {"low": low, "len": length, "beta": hx(beta), "witness": S, "m": m,
                      "T": [hx((low + t) % R) for t in range(length)],
                      "B": [hx(pow((low + t + beta) % R, -1, R)) for t in range(length)]}

    with open(os.path.join(HERE, "vectors_bn254.json" if br.CURVE == "bn254" else "vectors.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")


if __name__ == "__main__":
    main()
