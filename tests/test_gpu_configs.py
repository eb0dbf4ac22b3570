"""The benchmark configurations at their full size, bit-exact against the CPU oracle.

configs[1]: Hyrax commitment of a 4096 x 4096 int16-range matrix, every row (src/Hyrax.cu:312-333).
configs[2]: prove_matmul of 2048 x 4096 by 4096 x 4096: transcript, A(v), B(v) (src/prove.cu:175-210).
configs[3]: tLookupRange::prove of 2^24 values in a 2^16-entry range through the lookup object's
            default path (indexed commitment of A through the scaled table): multiplicities, 24 round
            polynomials, S(v), commitments of A (sampled rows) and of m (src/tlookup.cu:288-343).
configs[4]: the layer's shapes the other three do not cover - the per-head product (32 x 2048 x 2048
            x 128, phase 1 over the head bits), a range lookup and a mapping lookup on rows of 11008
            padded to 16384 with 4096 generators (test/llm.cu:73-611); the whole layer in the
            reference's proof order at 2048 tokens runs in test_gpu_host.py.

The oracle takes seconds to a minute per case on the host cores; the GPU side is milliseconds.
These run under the default curve only (the benchmark configurations name BLS12-381)."""
import os
import numpy as np
import pytest

import bigref as br
import orc
from gpuutil import rand_fr, gaussian_i16, assert_same

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(br.CURVE != "bls12_381", reason="full-size configurations run on the default curve")]

NGEN = 4096


@pytest.fixture(scope="module")
def ops():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from grape_amd import ops as o
    o.init(0)
    return o


@pytest.fixture(scope="module")
def host():
    from grape_amd import _host
    _host.load()
    return _host


@pytest.fixture(scope="module")
def gens4096(ops):
    """4096 seeded generators on both sides and the oracle's own byte-window table (k * G_i, k < 256)"""
    k = rand_fr(NGEN, 20240002)
    hg = orc.g1_make_generators(k)
    dg = ops.g1_make_generators(k)
    assert np.array_equal(ops.g1_to_host(dg), hg)
    return hg, dg, orc.g1_table(hg, 256)


def test_configs1_commit_4096x4096_every_row(ops, gens4096):
    import torch
    hg, dg, htab = gens4096
    W = gaussian_i16((4096, 4096), 20240001)
    assert W.min() >= -32768 and W.max() <= 32767 and abs(float(W.std()) - 1024.0) < 8.0
    wide = ops.g1_wide_table_gen(dg, 16, 1, 32768)
    got = ops.g1_to_host(ops.commit_i32(torch.from_numpy(W).cuda().view(-1), 4096, wide, NGEN, 16, 1, 32768))
    del wide
    torch.cuda.empty_cache()
    want = orc.commit_i32(W, htab, 4096, NGEN)
    assert_same(got, want, "4096 row commitments")
    # one row against the big-integer sum as well
    assert br.g1_unpack(got[1234:1235])[0] == br.g1_msm([int(x) for x in W[1234]], br.g1_unpack(hg))


def test_configs2_prove_matmul_2048x4096x4096(ops, host):
    import torch
    N, M, K = 2048, 4096, 4096
    A, B = gaussian_i16((N, K), 31), gaussian_i16((M, K), 32)
    u, v = rand_fr(23, 33), rand_fr(12, 34)
    Af, Bf = orc.from_i32(A), orc.from_i32(B)
    # claim Y(u) = sum_k A(u_n, k) B(u_m, k), from the oracle's own folds
    a2 = orc.partial_eval(Af, N * K, u, N, 12, K)[:K]
    b2 = orc.partial_eval(Bf, M * K, u, M, 0, K)[:K]
    claim0 = orc.fr_sum(orc.vec2("orc_fr_vec_mul", a2, b2))
    st, wtr, wclaim, wac, wbc = orc.prove_matmul(Af, Bf, 1, N, M, K, u, v, claim0)
    assert st == 0 and wtr.shape[0] == 12
    del Af, Bf
    dA = ops.fr_from_i32(torch.from_numpy(A).cuda().view(-1))
    dB = ops.fr_from_i32(torch.from_numpy(B).cuda().view(-1))
    tr, claim, ac, bc = host.prove_matmul(dA, dB, 1, N, M, K, u, v, claim0)
    assert_same(tr, wtr, "12 round polynomials")
    assert_same(claim, wclaim, "final claim")
    assert_same(ac, wac, "A(v)")
    assert_same(bc, wbc, "B(v)")


def test_configs3_tlookup_range_2p24_in_2p16_indexed(ops, host, gens4096):
    import torch
    hg, dg, htab = gens4096
    logD, logN, low = 24, 16, -32768
    D, N = 1 << logD, 1 << logN
    S = np.random.default_rng(41).integers(low, low + N, size=D).astype(np.int32)
    alpha, u, v = rand_fr(1, 43), rand_fr(logD, 44), rand_fr(logD, 45)
    beta = br.fr_pack([N])[0]
    host.set_indexed_commit(True)
    table = ops.g1_table_gen(dg, 256)
    dS = ops.fr_from_i32(torch.from_numpy(S).cuda())
    res = host.tlookup_range_prove(dS, D, low, N, alpha, u, v, table, NGEN, 1, 4096, want_commitments=True)
    del dS
    # the same proof from the witness as integers (the prover's pass over it embeds it; the first round gathers A)
    host.set_input_format("i32")
    try:
        res_i = host.tlookup_range_prove(torch.from_numpy(S).cuda(), D, low, N, alpha, u, v, table, NGEN, 1, 4096, want_commitments=True)
    finally:
        host.set_input_format("fr")
    for key in ("m", "transcript", "S_claim", "com_A", "com_m"):
        assert_same(res_i[key], res[key], "integer witness: " + key)
    del table
    torch.cuda.empty_cache()
    assert br.fr_unpack(res["m"]) == [int(x) for x in np.bincount(S.astype(np.int64) - low, minlength=N)]
    Sp = orc.from_i32(S)
    T, B = orc.tlookup_init(low, N, beta)
    m = orc.tlookup_prep(Sp, low, N)
    assert_same(res["m"], m, "multiplicities")
    # commitments made inside prove: A = 1/(S+beta) on sampled rows of 4096, m on all of its rows of 256
    rows = [0, 1, 2047, 4094, 4095]
    for r in rows:
        Srow = Sp[r * 4096:(r + 1) * 4096]
        Ainv = orc.vec1("orc_fr_vec_inv", orc.vec_bcast("orc_fr_vec_bcast_add", Srow, beta))
        assert_same(res["com_A"][r:r + 1], orc.commit_fr(Ainv, htab, 4096, NGEN), "com(A) row %d" % r)
    assert res["com_A"].shape[0] == D // 4096 and res["com_m"].shape[0] == N // 256
    assert_same(res["com_m"], orc.commit_fr(m, htab, 256, NGEN), "com(m)")
    st, wtr, wsc = orc.tlookup_prove(Sp, T, B, m, alpha[0], beta, u, v)
    assert st == 0 and wtr.shape[0] == 24
    assert_same(res["transcript"], wtr, "24 round polynomials")
    assert_same(res["S_claim"], wsc, "S(v)")


def test_configs4_per_head_matmul_32x2048x2048x128(ops, host):
    """QK^T of the layer: 32 heads, phase 1 binds the 5 head bits before phase 2 binds the 7 bits of k"""
    import torch
    L, N, M, K = 32, 2048, 2048, 128
    A, B = gaussian_i16((L, N, K), 61), gaussian_i16((L, M, K), 62)
    u, v = rand_fr(11 + 11 + 5, 63), rand_fr(7 + 5, 64)
    Af, Bf = orc.from_i32(A), orc.from_i32(B)
    a2 = orc.partial_eval(Af, L * N * K, u, N, 11, K)[:L * K]           # [L][K]
    b2 = orc.partial_eval(Bf, L * M * K, u, M, 0, K)[:L * K]
    prod = orc.vec2("orc_fr_vec_mul", a2, b2).reshape(L, K, 4)
    per_head = np.stack([orc.fr_sum(prod[l]) for l in range(L)])
    claim0 = orc.mle_eval(per_head, u[22:27])
    st, wtr, wclaim, wac, wbc = orc.prove_matmul(Af, Bf, L, N, M, K, u, v, claim0)
    assert st == 0 and wtr.shape[0] == 12
    del Af, Bf
    dA = ops.fr_from_i32(torch.from_numpy(A).cuda().view(-1))
    dB = ops.fr_from_i32(torch.from_numpy(B).cuda().view(-1))
    tr, claim, ac, bc = host.prove_matmul(dA, dB, L, N, M, K, u, v, claim0)
    assert_same(tr, wtr, "5 + 7 round polynomials")
    assert_same(claim, wclaim, "final claim")
    assert_same(ac, wac, "A(v)")
    assert_same(bc, wbc, "B(v)")


def test_configs4_lookups_on_padded_ffn_rows(ops, host, gens4096):
    """64 tokens x 11008 FFN columns (padded to 64 x 16384 = 2^20 inside prove), 4096 generators, rows of
    4096: the rescaling range lookup (2^16 range) and the SiLU mapping lookup (the layer's 2^19-entry
    table, low = -2^18, test/llm.cu:63)"""
    import torch
    hg, dg, htab = gens4096
    table = ops.g1_table_gen(dg, 256)
    tokens, F = 64, 11008
    D, Dp = tokens * F, tokens * 16384
    logDp = 20
    rng = np.random.default_rng(71)
    # ---- range lookup
    low, N = -32768, 1 << 16
    S = rng.integers(low, low + N, size=D).astype(np.int32)
    alpha, u, v = rand_fr(1, 72), rand_fr(logDp, 73), rand_fr(logDp, 74)
    beta = br.fr_pack([N])[0]
    Sp = orc.from_i32(S)
    m = orc.tlookup_prep(Sp, low, N)
    Spad = np.zeros((Dp, 4), dtype=np.uint64)
    orc.lib().orc_fr_pad(orc.P(Spad), orc.P(Sp), orc.c32(F), orc.c32(16384), orc.c64(Dp), orc.P(np.zeros(4, dtype=np.uint64)))
    T, B = orc.tlookup_init(low, N, beta)
    st, wtr, wsc = orc.tlookup_prove(Spad, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    host.set_indexed_commit(True)
    res = host.tlookup_range_prove(ops.fr_from_i32(torch.from_numpy(S).cuda()), D, low, N, alpha, u, v, table, NGEN, 1, 4096,
                                   want_commitments=True)
    assert_same(res["m"], m, "multiplicities with the padding fix-up")
    assert_same(res["transcript"], wtr, "range lookup transcript")
    assert_same(res["S_claim"], wsc, "S(v)")
    for r in (0, 2, 3, Dp // 4096 - 1):          # rows 0..2 of a token hold data (row 2 partly), row 3 padding only
        Ainv = orc.vec1("orc_fr_vec_inv", orc.vec_bcast("orc_fr_vec_bcast_add", Spad[r * 4096:(r + 1) * 4096], beta))
        assert_same(res["com_A"][r:r + 1], orc.commit_fr(Ainv, htab, 4096, NGEN), "com(A) row %d" % r)
    # ---- mapping lookup through the layer's SiLU table
    _, silu = host.witness_tables()
    lowm, Nm = -(1 << 18), 1 << 19
    S_in = np.clip(np.rint(rng.normal(0.0, 40000.0, size=D)), lowm, lowm + Nm - 1).astype(np.int32)
    S_out = silu[S_in - lowm]
    alpha, r, u, v = rand_fr(1, 75), rand_fr(1, 76), rand_fr(logDp, 77), rand_fr(logDp, 78)
    beta = br.fr_pack([Nm])[0]
    T, B = orc.tlookup_init(lowm, Nm, beta, orc.from_i32(silu), r[0])
    m = orc.tlookup_prep(orc.from_i32(S_in), lowm, Nm)
    Sc = orc.vec2("orc_fr_vec_add", orc.vec_bcast("orc_fr_vec_bcast_mul", orc.from_i32(S_out), r[0]), orc.from_i32(S_in))
    pad_val = orc.fr_mul(orc.from_i32(silu[-lowm: -lowm + 1])[0], r[0])
    Spad = np.zeros((Dp, 4), dtype=np.uint64)
    orc.lib().orc_fr_pad(orc.P(Spad), orc.P(Sc), orc.c32(F), orc.c32(16384), orc.c64(Dp), orc.P(pad_val))
    st, wtr, wsc = orc.tlookup_prove(Spad, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    tr, sc = host.tlookup_mapping_prove(ops.fr_from_i32(torch.from_numpy(S_in).cuda()), ops.fr_from_i32(torch.from_numpy(S_out).cuda()),
                                        D, lowm, Nm, silu, alpha, r, u, v, table, NGEN, 1, 4096)
    assert_same(tr, wtr, "mapping lookup transcript")
    assert_same(sc, wsc, "S(v)")


def test_configs4_softmax_mapping_lookup_through_occupied_entries(ops, host, gens4096):
    """the layer's exponential lookup at its table size (2^20 entries, low = -2^19) and row length (4096
    generators) on 2^24 scores distributed like the layer's (Gaussian, sigma 181, plus 0.5 % spread over
    the whole table): the default path commits A through a per-proof table of the entries that reach
    the break-even count and the rest as full-width scalars.  Transcript and S(v) against the oracle,
    com(A) on sampled rows against the oracle's full-width commitment of 1/(S + beta), the split
    against numpy; the same witness through the plain path (no table) gives the same commitment."""
    import torch
    hg, dg, htab = gens4096
    table = ops.g1_table_gen(dg, 256)
    exp_map, _ = host.witness_tables()
    low, N = -(1 << 19), 1 << 20
    logD = 24
    D = 1 << logD
    rng = np.random.default_rng(91)
    S_in = np.clip(np.rint(rng.normal(0.0, 181.0, size=D)), low, low + N - 1).astype(np.int32)
    spread = rng.random(D) < 0.005
    S_in[spread] = rng.integers(low, low + N, size=int(spread.sum()))
    S_out = np.ascontiguousarray(exp_map[S_in - low])
    alpha, r, u, v = rand_fr(1, 92), rand_fr(1, 93), rand_fr(logD, 94), rand_fr(logD, 95)
    beta = br.fr_pack([N])[0]
    host.set_indexed_commit(True)
    dSi = ops.fr_from_i32(torch.from_numpy(S_in).cuda())
    dSo = ops.fr_from_i32(torch.from_numpy(S_out).cuda())
    tr, sc, com_a, n_hot, n_cold, reused = host.tlookup_mapping_prove_ex(dSi, dSo, D, low, N, exp_map, alpha, r, u, v, table, NGEN, 1, 4096)
    assert not reused
    counts = np.bincount(S_in.astype(np.int64) - low, minlength=N)
    thr = int(1.8 * 4096) + 1
    assert n_hot == int((counts >= thr).sum()) and n_hot > 100
    assert n_cold == int(counts[counts < thr].sum()) and 0 < n_cold < D // 5
    # the plain path on the same witness
    host.set_indexed_commit(False)
    tr2, sc2, com_a2, h2, c2, _ = host.tlookup_mapping_prove_ex(dSi, dSo, D, low, N, exp_map, alpha, r, u, v, table, NGEN, 1, 4096)
    host.set_indexed_commit(True)
    assert h2 == 0 and c2 == 0
    assert_same(com_a, com_a2, "com(A): occupied-entry table == full-width commitment")
    assert_same(tr, tr2, "transcripts")
    del dSi, dSo
    # the same proof from the two tensors as integers (one pass indexes, checks and combines them)
    host.set_input_format("i32")
    try:
        tr3, sc3, com_a3, h3, c3, _ = host.tlookup_mapping_prove_ex(torch.from_numpy(S_in).cuda(), torch.from_numpy(S_out).cuda(), D, low, N,
                                                                    exp_map, alpha, r, u, v, table, NGEN, 1, 4096)
    finally:
        host.set_input_format("fr")
    assert_same(tr3, tr, "integer witness: transcript")
    assert_same(sc3, sc, "integer witness: S(v)")
    assert_same(com_a3, com_a, "integer witness: com(A)")
    assert (h3, c3) == (n_hot, n_cold)
    del table
    torch.cuda.empty_cache()
    T, B = orc.tlookup_init(low, N, beta, orc.from_i32(exp_map), r[0])
    m = orc.tlookup_prep(orc.from_i32(S_in), low, N)
    S = orc.vec2("orc_fr_vec_add", orc.vec_bcast("orc_fr_vec_bcast_mul", orc.from_i32(S_out), r[0]), orc.from_i32(S_in))
    for rr in (0, 517, D // 4096 - 1):
        Ainv = orc.vec1("orc_fr_vec_inv", orc.vec_bcast("orc_fr_vec_bcast_add", S[rr * 4096:(rr + 1) * 4096], beta))
        assert_same(com_a[rr:rr + 1], orc.commit_fr(Ainv, htab, 4096, NGEN), "com(A) row %d" % rr)
    st, wtr, wsc = orc.tlookup_prove(S, T, B, m, alpha[0], beta, u, v)
    assert st == 0 and wtr.shape[0] == logD
    assert_same(tr, wtr, "transcript")
    assert_same(sc, wsc, "S(v)")
