"""Known-answer vectors (tests/golden/vectors.json, written by tests/golden/make_vectors.py from
Python-integer definitions) against the CPU oracle (CPU tests) and against the HIP library
through its C ABI (gpu tests).  Bit-exact."""
import json
import os
import numpy as np
import pytest
import bigref as br
import orc
from gpuutil import rand_fr

HERE = os.path.dirname(os.path.abspath(__file__))
VECTORS = "vectors_bn254.json" if br.CURVE == "bn254" else "vectors.json"
with open(os.path.join(HERE, "golden", VECTORS)) as f:
    V = json.load(f)
R = br.R_MOD


def ints(xs):
    return [int(x, 16) for x in xs]


def points(ps):
    return [None if p is None else (int(p[0], 16), int(p[1], 16)) for p in ps]


@pytest.fixture(scope="module")
def ops():
    from grape_amd import ops as o
    o.init(0)
    return o


# ------------------------------------------------------------------ CPU: fixtures and oracle
def test_fixture_is_reproducible(tmp_path):
    """the committed file is what the generator writes today (frozen seeds, frozen PRNG)"""
    import subprocess, sys, shutil
    work = tmp_path / "golden"
    work.mkdir()
    shutil.copy(os.path.join(HERE, "golden", "make_vectors.py"), work / "make_vectors.py")
    for name in ("bigref.py", "gpuutil.py"):
        shutil.copy(os.path.join(HERE, name), tmp_path / name)
    subprocess.check_call([sys.executable, str(work / "make_vectors.py")])
    with open(work / VECTORS) as f:
        assert json.load(f) == V


def test_constants_and_seeded_draws():
    assert int(V["modulus_r"], 16) == R and int(V["modulus_p"], 16) == br.P_MOD
    assert br.fr_unpack(rand_fr(4, V["seeded_fr"]["seed"])) == ints(V["seeded_fr"]["values"])


def test_oracle_field_vectors():
    a = ints([c["a"] for c in V["fr"]]); b = ints([c["b"] for c in V["fr"]])
    pa, pb = br.fr_pack(a), br.fr_pack(b)
    for name, fn in (("add", orc.fr_add), ("sub", orc.fr_sub), ("mul", orc.fr_mul)):
        got = [br.fr_unpack(fn(pa[i], pb[i]))[0] for i in range(len(a))]
        assert got == ints([c[name] for c in V["fr"]]), name
    assert [br.fr_unpack(orc.fr_inv(pa[i]))[0] for i in range(len(a))] == ints([c["inv_a"] for c in V["fr"]])
    xs = np.array([c["x"] for c in V["from_i32"]], dtype=np.int64).astype(np.int32)
    assert br.fr_unpack(orc.from_i32(xs)) == ints([c["fr"] for c in V["from_i32"]])


def test_oracle_curve_and_commit_vectors():
    ks = ints([c["k"] for c in V["g1_multiples"]])
    got = br.g1_unpack(orc.g1_make_generators(br.ints_to_limbs(ks, 4)))
    assert got == points([c["point"] for c in V["g1_multiples"]])
    gens = orc.g1_make_generators(br.ints_to_limbs(ints(V["generators"]["scalars"]), 4))
    assert br.g1_unpack(gens) == points(V["generators"]["points"])
    table = orc.g1_table(gens, 256)
    rows = np.array(V["commit_i32"]["rows"], dtype=np.int32)
    assert br.g1_unpack(orc.commit_i32(rows, table, 4, 4)) == points(V["commit_i32"]["commitments"])
    frs = br.fr_pack([int(x, 16) for row in V["commit_fr"]["rows"] for x in row])
    assert br.g1_unpack(orc.commit_fr(frs, table, 4, 4)) == points(V["commit_fr"]["commitments"])


def test_oracle_fold_and_sumcheck_vectors():
    for c in V["fold"]:
        t = br.fr_pack(ints(c["t"]))
        n = c["outer"] * c["c"] * c["gap"]
        out = orc.partial_eval(t, n, br.fr_pack(ints(c["x"])), c["c"], 0, c["gap"])[: n // c["c"]]
        assert br.fr_unpack(out) == ints(c["out"]), (c["outer"], c["c"], c["gap"])
    m = V["mle_eval"]
    # a full evaluation is the fold of the whole tensor as one axis (the reference's operator()
    # reads a tensor shorter than 2^len(u) as rows of 11008, src/fr-tensor.cu:346-369)
    full = orc.partial_eval(br.fr_pack(ints(m["t"])), len(m["t"]), br.fr_pack(ints(m["u"])), len(m["t"]), 0, 1)
    assert br.fr_unpack(full[:1])[0] == int(m["value"], 16)
    t = V["tlookup"]
    T, B = orc.tlookup_init(t["low"], t["len"], br.fr_pack([int(t["beta"], 16)])[0])
    assert br.fr_unpack(T) == ints(t["T"]) and br.fr_unpack(B) == ints(t["B"])
    S = br.fr_pack([s % R for s in t["witness"]])
    assert list(orc.histogram(S, t["low"], t["len"])) == t["m"]


# ------------------------------------------------------------------ GPU: the library through its C ABI
@pytest.mark.gpu
def test_gpu_field_vectors(ops):
    import torch
    a = ints([c["a"] for c in V["fr"]]); b = ints([c["b"] for c in V["fr"]])
    da, db = ops.to_dev(br.fr_pack(a)), ops.to_dev(br.fr_pack(b))
    for name, fn in (("add", ops.fr_add), ("sub", ops.fr_sub), ("mul", ops.fr_mul)):
        assert br.fr_unpack(ops.fr_to_host(fn(da, db))) == ints([c[name] for c in V["fr"]]), name
    assert br.fr_unpack(ops.fr_to_host(ops.fr_batch_inverse(da))) == ints([c["inv_a"] for c in V["fr"]])
    xs = torch.tensor([c["x"] for c in V["from_i32"]], dtype=torch.int64).to(torch.int32).cuda()
    assert br.fr_unpack(ops.fr_to_host(ops.fr_from_i32(xs))) == ints([c["fr"] for c in V["from_i32"]])


@pytest.mark.gpu
def test_gpu_curve_and_commit_vectors(ops):
    import torch
    ks = ints([c["k"] for c in V["g1_multiples"]])
    got = br.g1_unpack(ops.g1_to_host(ops.g1_make_generators(br.ints_to_limbs(ks, 4))))
    assert got == points([c["point"] for c in V["g1_multiples"]])
    gens = ops.g1_make_generators(br.ints_to_limbs(ints(V["generators"]["scalars"]), 4))
    assert br.g1_unpack(ops.g1_to_host(gens)) == points(V["generators"]["points"])
    rows = torch.tensor(V["commit_i32"]["rows"], dtype=torch.int32).cuda().view(-1)
    frs = ops.to_dev(br.fr_pack([int(x, 16) for row in V["commit_fr"]["rows"] for x in row]))
    want_i, want_f = points(V["commit_i32"]["commitments"]), points(V["commit_fr"]["commitments"])
    # the reference's table format and algorithm
    table = ops.g1_table_gen(gens, 256)
    assert br.g1_unpack(ops.g1_to_host(ops.commit_i32_ref_table(rows, 4, table, 4))) == want_i
    assert br.g1_unpack(ops.g1_to_host(ops.commit_fr_ref_table(frs, 4, table, 4))) == want_f
    # wide fixed-base tables: one 16-bit digit for the small scalars, 13-bit windows for Fr
    wide16 = ops.g1_wide_table_gen(gens, 16, 1, 32768)
    assert br.g1_unpack(ops.g1_to_host(ops.commit_i32(rows, 4, wide16, 4, 16, 1, 32768))) == want_i
    wide13 = ops.g1_wide_table_gen(gens, 13, 20, 4096)
    assert br.g1_unpack(ops.g1_to_host(ops.commit_fr(frs, 4, wide13, 4, 13, 20, 4096))) == want_f


@pytest.mark.gpu
def test_gpu_fold_sumcheck_tlookup_vectors(ops):
    for c in V["fold"]:
        n = c["outer"] * c["c"] * c["gap"]
        t = ops.to_dev(br.fr_pack(ints(c["t"])))
        ops.fr_fold(t, n, ops.to_dev(br.fr_pack(ints(c["x"]))), c["c"], 0, c["gap"])
        assert br.fr_unpack(ops.fr_to_host(t)[: n // c["c"]]) == ints(c["out"]), (c["outer"], c["c"], c["gap"])
    m = V["mle_eval"]
    t = ops.to_dev(br.fr_pack(ints(m["t"])))
    ops.fr_fold(t, len(m["t"]), ops.to_dev(br.fr_pack(ints(m["u"]))), len(m["t"]), 0, 1)
    assert br.fr_unpack(ops.fr_to_host(t)[:1])[0] == int(m["value"], 16)
    for c in V["sumcheck_round2"]:
        dA, dB = ops.to_dev(br.fr_pack(ints(c["A"]))), ops.to_dev(br.fr_pack(ints(c["B"])))
        sums = ops.sumcheck_round2(dA, dB, c["in_size"], c["out_size"], ops.to_dev(br.fr_pack([int(c["v"], 16)])))
        assert br.fr_unpack(ops.fr_to_host(sums)) == ints(c["sums"])
        assert br.fr_unpack(ops.fr_to_host(dA)[: c["out_size"]]) == ints(c["A_folded"])
        assert br.fr_unpack(ops.fr_to_host(dB)[: c["out_size"]]) == ints(c["B_folded"])
    t = V["tlookup"]
    T, B = ops.tlookup_init(t["low"], t["len"], ops.to_dev(br.fr_pack([int(t["beta"], 16)])))
    assert br.fr_unpack(ops.fr_to_host(T)) == ints(t["T"]) and br.fr_unpack(ops.fr_to_host(B)) == ints(t["B"])
    S = ops.to_dev(br.fr_pack([s % R for s in t["witness"]]))
    assert list(ops.tlookup_hist(S, t["low"], t["len"]).cpu().numpy()) == t["m"]
