"""GPU parity of the C++ host classes (FrTensor, Hyrax, prove_matmul, tLookupRange, ...) against
the CPU oracle: transcripts, claims, multiplicities and commitments, bit-exact."""
import random
import numpy as np
import pytest
import bigref as br
import orc
from gpuutil import rand_fr, gaussian_i16, assert_same

pytestmark = pytest.mark.gpu
R = br.R_MOD


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
def gens(ops):
    k = rand_fr(256, 500)
    h = orc.g1_make_generators(k)
    d = ops.g1_make_generators(k)
    return h, d


class _witness_as:
    """hands integer witnesses to the host calls as field tensors ("fr") or as the integers themselves ("i32": the
    provers then index and embed them in one pass)"""
    def __init__(self, host, ops, fmt):
        self.host, self.ops, self.fmt = host, ops, fmt

    def __enter__(self):
        self.host.set_input_format(self.fmt)
        return self

    def __exit__(self, *exc):
        self.host.set_input_format("fr")

    def dev(self, ints):
        import torch
        d = torch.from_numpy(np.ascontiguousarray(ints, dtype=np.int32)).cuda()
        return d if self.fmt == "i32" else self.ops.fr_from_i32(d)


def _int_tensor(shape, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(-2**15, 2**15, size=shape).astype(np.int32)


@pytest.mark.parametrize("L,N,M,K", [(1, 4, 8, 16), (2, 4, 4, 8), (4, 2, 4, 4), (1, 3, 5, 6), (1, 8, 4, 1),
                                     (1, 64, 128, 512), (2, 16, 32, 256), (1, 172, 64, 96),
                                     (1, 2, 2, 1 << 18)])        # long rounds: middle coefficient from the running claim
def test_prove_matmul_vs_oracle(ops, host, L, N, M, K):
    import torch
    A = _int_tensor(L * N * K, 1 + N)
    B = _int_tensor(L * M * K, 2 + M)
    lM, lN, lL, lK = br.log2ceil(M), br.log2ceil(N), br.log2ceil(L), br.log2ceil(K)
    u = rand_fr(br.log2ceil(L * N * M), 3)
    v = rand_fr(br.log2ceil(L * K), 4)
    assert u.shape[0] == lM + lN + lL or (N & (N - 1)) or (M & (M - 1))
    # claim = Y(u): exact integer matmul, embedded, evaluated by the oracle's own fold
    Y = np.einsum("lnk,lmk->lnm", A.reshape(L, N, K).astype(np.int64), B.reshape(L, M, K).astype(np.int64))
    Mp, Np, Lp = 1 << lM, 1 << lN, 1 << lL
    Ypad = np.zeros((Lp, Np, Mp), dtype=np.int64)
    Ypad[:L, :N, :M] = Y
    yf = br.fr_pack([int(x) % R for x in Ypad.reshape(-1)]) if Ypad.size <= 4096 else None
    if yf is None:
        # larger case: embed through two int32 halves (|Y| < 2^42)
        lo = (Ypad.reshape(-1) & 0xffff).astype(np.int32)
        hi = (Ypad.reshape(-1) >> 16).astype(np.int32)
        sh = br.fr_pack([1 << 16])[0]
        yf = orc.vec2("orc_fr_vec_add", orc.vec_bcast("orc_fr_vec_bcast_mul", orc.from_i32(hi), sh), orc.from_i32(lo))
    if u.shape[0] != lM + lN + lL:
        # Log2(L*N*M) differs from the sum of the logs: the point has no defined reading (the reference's folds would
        # read past its end), so the prover refuses the shape with the reference's message for mismatched operands
        dA = ops.fr_from_i32(torch.from_numpy(A).cuda())
        dB = ops.fr_from_i32(torch.from_numpy(B).cuda())
        for point in (u, rand_fr(lM + lN + lL, 3)):
            with pytest.raises(host.HostError, match="Incompatible dimensions"):
                host.prove_matmul(dA, dB, L, N, M, K, point, v, br.fr_pack([1])[0])
        return
    claim0 = orc.mle_eval(yf, u)
    Af, Bf = orc.from_i32(A), orc.from_i32(B)
    st, wtr, wclaim, wac, wbc = orc.prove_matmul(Af, Bf, L, N, M, K, u, v, claim0)
    assert st == 0
    dA = ops.fr_from_i32(torch.from_numpy(A).cuda())
    dB = ops.fr_from_i32(torch.from_numpy(B).cuda())
    tr, claim, ac, bc = host.prove_matmul(dA, dB, L, N, M, K, u, v, claim0)
    assert_same(tr, wtr, "transcript")
    assert_same(claim, wclaim, "final claim")
    assert_same(ac, wac, "A(v)")
    assert_same(bc, wbc, "B(v)")
    # the same proof from the operands as integers (the folds over the rows read them directly)
    with _witness_as(host, ops, "i32") as w:
        tr2, claim2, ac2, bc2 = host.prove_matmul(w.dev(A), w.dev(B), L, N, M, K, u, v, claim0)
    assert_same(tr2, wtr, "integer operands: transcript")
    assert_same(claim2, wclaim, "integer operands: final claim")
    assert_same(ac2, wac, "integer operands: A(v)")
    assert_same(bc2, wbc, "integer operands: B(v)")


@pytest.mark.parametrize("K", [4, 1 << 17])      # the long case starts with a round that takes its middle coefficient from the claim
def test_prove_matmul_rejects_wrong_claim(ops, host, K):
    import torch
    A, B = _int_tensor(2 * K, 5), _int_tensor(2 * K, 6)
    dA = ops.fr_from_i32(torch.from_numpy(A).cuda())
    dB = ops.fr_from_i32(torch.from_numpy(B).cuda())
    with pytest.raises(host.HostError, match="matmul_phase2"):
        host.prove_matmul(dA, dB, 1, 2, 2, K, rand_fr(2, 7), rand_fr(br.log2ceil(K), 8), br.fr_pack([12345])[0])


def test_mle_eval_operator(ops, host):
    t = rand_fr(4096, 11)
    u = rand_fr(12, 12)
    assert_same(host.mle_eval(ops.to_dev(t), 4096, u), orc.mle_eval(t, u), "T(u)")
    # rows of 11008 read as zero-extended to 16384
    t = orc.from_i32(_int_tensor(2 * 11008, 13))
    u = rand_fr(15, 14)
    assert_same(host.mle_eval(ops.to_dev(t), 2 * 11008, u), orc.mle_eval(t, u), "T(u), 11008 columns")


_RANGE_SHAPES = [(4, 2, -2), (5, 3, -4), (3, 3, 0), (12, 6, -32), (14, 8, -128), (16, 16, -32768)]


# every shape with the witness as a field tensor; four of them again with the witness handed over as integers
@pytest.mark.parametrize("logD,logN,low,indexed,fmt",
                         [s + (i, "fr") for s in _RANGE_SHAPES for i in (True, False)] +
                         [s + (i, "i32") for s in _RANGE_SHAPES if s[0] not in (5, 14) for i in (True, False)])
def test_tlookup_range_prove_vs_oracle(ops, host, gens, logD, logN, low, indexed, fmt):
    import torch
    host.set_indexed_commit(indexed)
    hg, dg = gens
    D, N = 1 << logD, 1 << logN
    rng = np.random.default_rng(logD * 7 + logN)
    S = rng.integers(low, low + N, size=D).astype(np.int32)
    alpha, u, v = rand_fr(1, 21), rand_fr(logD, 22), rand_fr(logD, 23)
    beta = br.fr_pack([N])[0]
    Sp = orc.from_i32(S)
    T, B = orc.tlookup_init(low, N, beta)
    m = orc.tlookup_prep(Sp, low, N)
    st, wtr, wsc = orc.tlookup_prove(Sp, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    table = ops.g1_table_gen(dg, 256)               # 256 generators: com(m) uses rows of 2^(logN/2)
    msm = min(D, 16)
    with _witness_as(host, ops, fmt) as w:
        res = host.tlookup_range_prove(w.dev(S), D, low, N, alpha, u, v, table, 256, 1, msm, want_commitments=True)
    assert_same(res["m"], m, "multiplicities")
    assert_same(res["transcript"], wtr, "transcript")
    assert_same(res["S_claim"], wsc, "S(v)")
    assert br.fr_unpack(res["m"]) == [int(x) for x in np.bincount(S.astype(np.int64) - low, minlength=N)]
    host.set_indexed_commit(True)
    # the commitments of A = 1/(S+beta) and of m made inside prove (through the scaled table
    # B[t] * G_i and the indexed commitment when `indexed`): every row up to 64 rows, else the two
    # ends, the middle and a seeded sample
    Ainv = orc.vec1("orc_fr_vec_inv", orc.vec_bcast("orc_fr_vec_bcast_add", Sp, beta))
    tab = orc.g1_table(hg, 256)
    nrows = D // msm
    assert res["com_A"].shape[0] == nrows
    rows = list(range(nrows)) if nrows <= 64 else sorted({0, 1, nrows // 2, nrows - 2, nrows - 1} | set(rng.integers(0, nrows, 24).tolist()))
    for r in rows:
        assert_same(res["com_A"][r:r + 1], orc.commit_fr(Ainv[r * msm:(r + 1) * msm], tab, msm, 256), "com(A) row %d" % r)
    mN = 1 << (logN // 2)
    assert_same(res["com_m"], orc.commit_fr(m, tab, mN, 256), "com(m)")


@pytest.mark.parametrize("fmt", ["fr", "i32"])
def test_tlookup_range_rejects_out_of_range(ops, host, gens, fmt):
    hg, dg = gens
    S = np.array([0, 1, 2, 3, 9, 1, 2, 3, 0, 0, 1, 1, 2, 2, 3, 3], dtype=np.int32)
    table = ops.g1_table_gen(dg[:16].contiguous(), 256)
    with _witness_as(host, ops, fmt) as w:
        with pytest.raises(host.HostError, match="tLookup_phase"):
            host.tlookup_range_prove(w.dev(S), 16, 0, 4, rand_fr(1, 31), rand_fr(4, 32), rand_fr(4, 33), table, 16, 1, 16)


@pytest.mark.parametrize("fmt", ["fr", "i32"])
def test_tlookup_pads_11008_rows(ops, host, gens, fmt):
    # a witness of 2 x 11008 values is padded to 2 x 16384 with zeros, which are counted in m
    import torch
    hg, dg = gens
    D, low, N = 2 * 11008, -8, 16
    rng = np.random.default_rng(41)
    S = rng.integers(low, low + N, size=D).astype(np.int32)
    alpha, u, v = rand_fr(1, 42), rand_fr(15, 43), rand_fr(15, 44)
    beta = br.fr_pack([N])[0]
    Sp = orc.from_i32(S)
    m = orc.tlookup_prep(Sp, low, N)
    Spad = np.zeros((32768, 4), dtype=np.uint64)
    orc.lib().orc_fr_pad(orc.P(Spad), orc.P(Sp), orc.c32(11008), orc.c32(16384), orc.c64(32768), orc.P(np.zeros(4, dtype=np.uint64)))
    T, B = orc.tlookup_init(low, N, beta)
    st, wtr, wsc = orc.tlookup_prove(Spad, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    table = ops.g1_table_gen(dg[:16].contiguous(), 256)
    with _witness_as(host, ops, fmt) as w:
        res = host.tlookup_range_prove(w.dev(S), D, low, N, alpha, u, v, table, 16, 1, 16)
    assert_same(res["m"], m, "multiplicities with pad fix-up")
    assert_same(res["transcript"], wtr, "transcript")
    assert_same(res["S_claim"], wsc, "S(v)")


@pytest.mark.parametrize("fmt", ["fr", "i32"])
def test_tlookup_mapping_prove_vs_oracle(ops, host, gens, fmt):
    import torch
    hg, dg = gens
    logD, logN, low = 10, 6, -32
    D, N = 1 << logD, 1 << logN
    rng = np.random.default_rng(51)
    fmap = rng.integers(-1000, 1000, size=N).astype(np.int32)      # a seeded synthetic table x -> f(x)
    S_in = rng.integers(low, low + N, size=D).astype(np.int32)
    S_out = fmap[S_in - low]
    alpha, r, u, v = rand_fr(1, 52), rand_fr(1, 53), rand_fr(logD, 54), rand_fr(logD, 55)
    beta = br.fr_pack([N])[0]
    T, B = orc.tlookup_init(low, N, beta, orc.from_i32(fmap), r[0])
    m = orc.tlookup_prep(orc.from_i32(S_in), low, N)
    S = orc.vec2("orc_fr_vec_add", orc.vec_bcast("orc_fr_vec_bcast_mul", orc.from_i32(S_out), r[0]), orc.from_i32(S_in))
    st, wtr, wsc = orc.tlookup_prove(S, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    table = ops.g1_table_gen(dg[:16].contiguous(), 256)
    with _witness_as(host, ops, fmt) as w:
        dSi, dSo = w.dev(S_in), w.dev(S_out)
        tr, sc = host.tlookup_mapping_prove(dSi, dSo, D, low, N, fmap, alpha, r, u, v, table, 16, 1, 16)
        assert_same(tr, wtr, "transcript")
        assert_same(sc, wsc, "S(v)")
        # a wrong output value is caught
        S_out2 = S_out.copy()
        S_out2[5] += 1
        with pytest.raises(host.HostError, match="tLookup_phase"):
            host.tlookup_mapping_prove(dSi, w.dev(S_out2), D, low, N, fmap, alpha, r, u, v, table, 16, 1, 16)


@pytest.mark.parametrize("fmt", ["fr", "i32"])
def test_tlookup_mapping_pads_11008_rows(ops, host, gens, fmt):
    # mapping lookup of 2 x 11008 pairs: padded to 2 x 16384 with the pair (0, f(0)), counted in m
    import torch
    hg, dg = gens
    D, low, N = 2 * 11008, -16, 32
    rng = np.random.default_rng(56)
    fmap = rng.integers(-1000, 1000, size=N).astype(np.int32)
    S_in = rng.integers(low, low + N, size=D).astype(np.int32)
    S_out = fmap[S_in - low]
    alpha, r, u, v = rand_fr(1, 57), rand_fr(1, 58), rand_fr(15, 59), rand_fr(15, 60)
    beta = br.fr_pack([N])[0]
    T, B = orc.tlookup_init(low, N, beta, orc.from_i32(fmap), r[0])
    m = orc.tlookup_prep(orc.from_i32(S_in), low, N)             # includes the pad fix-up of the zero bin
    S = orc.vec2("orc_fr_vec_add", orc.vec_bcast("orc_fr_vec_bcast_mul", orc.from_i32(S_out), r[0]), orc.from_i32(S_in))
    pad_val = orc.fr_mul(orc.from_i32(fmap[-low: -low + 1])[0], r[0])
    Spad = np.zeros((32768, 4), dtype=np.uint64)
    orc.lib().orc_fr_pad(orc.P(Spad), orc.P(S), orc.c32(11008), orc.c32(16384), orc.c64(32768), orc.P(pad_val))
    st, wtr, wsc = orc.tlookup_prove(Spad, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    table = ops.g1_table_gen(dg[:16].contiguous(), 256)
    with _witness_as(host, ops, fmt) as w:
        tr, sc = host.tlookup_mapping_prove(w.dev(S_in), w.dev(S_out), D, low, N, fmap, alpha, r, u, v, table, 16, 1, 16)
    assert_same(tr, wtr, "transcript")
    assert_same(sc, wsc, "S(v)")


def test_hyrax_class_commits(ops, host, gens):
    import torch
    hg, dg = gens
    npoints = 256
    table = ops.g1_table_gen(dg, 256)
    htab = orc.g1_table(hg, 256)
    # com_scale = 16 (the reference's value): rows of N*16
    W = gaussian_i16((8, 256), 61)
    got = host.hyrax_commit_i32(torch.from_numpy(W).cuda(), W.size, 16, table, npoints, com_scale=16)
    assert_same(got, orc.commit_i32(W, htab, 256, npoints), "Hyrax::commit(int*) int16 path")
    # values outside int16 fall back to the general int32 tables
    W2 = _int_tensor((4, 256), 62) * 40000
    got = host.hyrax_commit_i32(torch.from_numpy(W2).cuda(), W2.size, 16, table, npoints, com_scale=16)
    assert_same(got, orc.commit_i32(W2, htab, 256, npoints), "Hyrax::commit(int*) int32 path")
    # com_scale = 1, shorter rows than the generator set
    W3 = gaussian_i16((16, 64), 63)
    got = host.hyrax_commit_i32(torch.from_numpy(W3).cuda(), W3.size, 64, table, npoints, com_scale=1)
    assert_same(got, orc.commit_i32(W3, htab, 64, npoints), "com_scale = 1")
    s = rand_fr(2 * 64, 64)
    got = host.hyrax_commit_fr(ops.to_dev(s), 128, 4, table, npoints, com_scale=16)
    assert_same(got, orc.commit_fr(s, htab, 64, npoints), "Hyrax::commit(FrTensor&)")
    with pytest.raises(host.HostError, match="power of 2"):
        host.hyrax_commit_i32(torch.from_numpy(W).cuda(), W.size, 12, table, npoints, com_scale=16)
    with pytest.raises(host.HostError, match="Size too small"):
        host.hyrax_commit_i32(torch.from_numpy(W).cuda(), 128, 16, table, npoints, com_scale=16)


def test_single_commit(ops, host, gens):
    hg, dg = gens
    table = ops.g1_table_gen(dg, 256)
    s = rand_fr(64, 65)
    got = host.single_commit(ops.to_dev(s), 64, table, 256)
    assert_same(got, orc.commit_fr(s, orc.g1_table(hg, 256), 64, 256)[0], "single_commit")


def test_hyrax_open_and_verify(ops, host, gens):
    hg, dg = gens
    npoints = 64
    table = ops.g1_table_gen(dg[:64].contiguous(), 256)
    size, N = 64 * 8, 4                   # 8 rows of 4*16 = 64
    t = rand_fr(size, 71)
    pt = rand_fr(9, 72)
    c = rand_fr(1, 73)
    res, ok = host.hyrax_open_verify(ops.to_dev(t), size, N, table, npoints, pt, c, com_scale=16)
    assert ok
    assert_same(res, orc.mle_eval(t, pt), "opened value = T(point)")


@pytest.mark.parametrize("rows,N", [(8, 4), (2048, 256)])
def test_opening_and_evaluation_of_integer_tensors(ops, host, gens, rows, N):
    """Hyrax::open(const int*, ...) and FrTensor::eval_ints (the fold reads the integers) against get_data + open /
    operator() on the embedded tensor, and against the oracle's evaluation of that tensor"""
    import torch
    hg, dg = gens
    npoints = max(64, N)
    if npoints > dg.shape[0]:
        dg = ops.g1_make_generators(rand_fr(npoints, 74))
    table = ops.g1_table_gen(dg[:npoints].contiguous(), 256)
    size = rows * N
    ints = np.random.default_rng(75 + rows).integers(-(1 << 31), 1 << 31, size=size, dtype=np.int64).astype(np.int32)
    di = torch.from_numpy(ints).cuda()
    pt, c = rand_fr(br.log2ceil(size), 76), rand_fr(1, 77)
    want = orc.mle_eval(ops.fr_to_host(ops.fr_from_i32(di)), pt) if size <= 4096 else None
    host.set_input_format("i32")
    try:
        results = {}
        for folds in (True, False):
            host.set_int_folds(folds)
            results[folds] = (host.hyrax_open(di, size, N, table, npoints, pt, c, com_scale=1), host.mle_eval(di, size, pt))
    finally:
        host.set_int_folds(True)
        host.set_input_format("fr")
    assert_same(results[True][0], results[False][0], "opened value, integers folded directly")
    assert_same(results[True][1], results[False][1], "evaluation, integers folded directly")
    assert_same(results[True][0], results[True][1], "opening = evaluation")
    assert np.array_equal(di.cpu().numpy(), ints)
    if want is not None:
        assert_same(results[True][0], want, "against the oracle")


@pytest.mark.parametrize("L,M,N", [(1, 4, 8), (2, 2, 4), (1, 4, 6), (2, 1, 5), (1, 32, 64), (1, 2, 1)])
def test_prove_elemul_vs_oracle(ops, host, L, M, N):
    rng = random.Random(81 + L + M + N)
    n = L * M * N
    Np = 1 << br.log2ceil(N)
    k = br.log2ceil(n)
    A = [rng.randrange(R) for _ in range(n)]
    B = [rng.randrange(R) for _ in range(n)]
    u = [rng.randrange(R) for _ in range(k)]
    v = [rng.randrange(R) for _ in range(k)]
    pad = lambda X: [X[f * N + j] if j < N else 0 for f in range(L * M) for j in range(Np)]
    claim0 = sum(br.eq_weight(i, u) * a * b for i, (a, b) in enumerate(zip(pad(A), pad(B)))) % R
    pA, pB, pu, pv, pc = br.fr_pack(A), br.fr_pack(B), br.fr_pack(u), br.fr_pack(v), br.fr_pack([claim0])[0]
    st, wtr, wclaim, wac, wbc = orc.prove_elemul(pA, pB, L, M, N, pu, pv, pc)
    assert st == 0
    tr, claim, ac, bc = host.prove_elemul(ops.to_dev(pA), ops.to_dev(pB), L, M, N, pu, pv, pc)
    assert_same(tr, wtr, "round polynomials")
    assert_same(claim, wclaim, "final claim")
    assert_same(ac, wac, "A(v)")
    assert_same(bc, wbc, "B(v)")
    with pytest.raises(host.HostError, match="claim != p\\(0\\) \\+ p\\(1\\)"):
        host.prove_elemul(ops.to_dev(pA), ops.to_dev(pB), L, M, N, pu, pv, br.fr_pack([claim0 + 1])[0])


@pytest.mark.parametrize("nv,num", [(4, 3), (3, 1), (1, 2), (10, 4), (5, 17)])      # 17 claims: two launches of the multi-table kernel per round
def test_combine_claims_vs_oracle(ops, host, nv, num):
    X = rand_fr(1 << nv, 90 + nv)
    us = [rand_fr(nv, 91 + nv + j) for j in range(num)]
    vv = rand_fr(nv, 99 + nv)
    claims = np.stack([orc.partial_eval(X, 1 << nv, uj, 1 << nv, 0, 1)[0] for uj in us])
    st, wtr, wret = orc.combine_claims(X, claims, us, vv)
    assert st == 0
    tr, res = host.combine_claims(ops.to_dev(X), 1 << nv, claims, np.stack(us), vv)
    assert_same(tr, wtr, "round polynomials")
    assert_same(res, wret, "X(v)")


def test_file_helpers_and_on_disk_formats(ops, host, gens, tmp_path):
    """the reference's on-disk artefacts through savebin / loadbin / load_data: an int32 weight
    dump (data/W/*.bin), the generator table points.bin (256 x npoints affine points, entry
    w*npoints + i = w*G_i) and an Fr tensor dump; a table read back from disk commits to the same
    points as the oracle"""
    import torch
    from grape_amd import _capi
    hg, dg = gens
    npoints = 256
    table = ops.g1_table_gen(dg, 256)
    ops.sync()
    f_pts = str(tmp_path / "points.bin")
    host.savebin(f_pts, table.data_ptr(), table.numel() * 4)
    assert host.findsize(f_pts) == 256 * npoints * 8 * br.G1_WORDS
    assert np.array_equal(np.fromfile(f_pts, dtype=np.uint64).reshape(-1, br.G1_WORDS), orc.g1_table(hg, 256))
    table2 = torch.zeros_like(table)
    host.loadbin(f_pts, table2.data_ptr(), table2.numel() * 4)
    assert torch.equal(table, table2)
    # int32 weights: written by numpy as the reference's Python side does, read by load_data
    W = gaussian_i16((8, 256), 71)
    f_w = str(tmp_path / "w.bin")
    W.astype("<i4").tofile(f_w)
    ptr, n = host.load_data(f_w)
    assert n == W.size
    dW = torch.empty(W.size, dtype=torch.int32, device="cuda")
    lib = _capi.load()
    _capi.check(lib.grape_memcpy_d2d(dW.data_ptr(), ptr, W.size * 4, None))
    _capi.check(lib.grape_stream_sync(None))
    _capi.check(lib.grape_free(ptr))
    assert np.array_equal(dW.cpu().numpy().reshape(W.shape), W)
    got = host.hyrax_commit_i32(dW, W.size, 16, table2, npoints, com_scale=16)
    assert_same(got, orc.commit_i32(W, orc.g1_table(hg, 256), 256, npoints), "commit from on-disk table and weights")
    # Fr tensor dump: 32-byte Montgomery elements
    s = rand_fr(100, 72)
    ds = ops.to_dev(s)
    f_fr = str(tmp_path / "fr.bin")
    host.savebin(f_fr, ds.data_ptr(), 100 * 32)
    assert np.array_equal(np.fromfile(f_fr, dtype=np.uint64).reshape(-1, 4), s)
    # generate_data: deterministic, full int32 range
    p1, p2 = host.generate_data(4096), host.generate_data(4096)
    a, b = torch.empty(4096, dtype=torch.int32, device="cuda"), torch.empty(4096, dtype=torch.int32, device="cuda")
    _capi.check(lib.grape_memcpy_d2d(a.data_ptr(), p1, 4096 * 4, None))
    _capi.check(lib.grape_memcpy_d2d(b.data_ptr(), p2, 4096 * 4, None))
    _capi.check(lib.grape_stream_sync(None))
    _capi.check(lib.grape_free(p1)); _capi.check(lib.grape_free(p2))
    assert torch.equal(a, b) and a.min().item() < -2**30 and a.max().item() > 2**30


def test_cpp_driver_runs(ops, tmp_path):
    """the reference-style C++ driver (generators, table file, int and Fr commitments, opening and
    verification, matmul sumcheck, range lookup incl. a rejected witness) end to end"""
    import subprocess
    import driver_build
    exe = driver_build.build()
    res = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, timeout=280)
    assert res.returncode == 0, res.stderr
    assert "driver_flow OK" in res.stdout


@pytest.mark.parametrize("tokens", ["2048"])
def test_cpp_layer_driver_runs(ops, tmp_path, tokens):
    """one transformer block (2048 tokens, d_model 4096, FFN 11008) proved in the order of the
    reference's layer driver (test/llm.cu:73-611) by a C++ program against the host classes, on the
    witness of the library's own generator: 37 chained steps (openings, range and mapping lookups,
    matmul / element-product sumchecks, combine_claims), every one of the reference's assertions
    kept; runs in a child process because it holds tens of GB of tables"""
    import subprocess
    import torch
    import driver_build
    exe = driver_build.build(None, "layer_flow")
    torch.cuda.empty_cache()
    res = subprocess.run([exe, tokens, str(tmp_path)], capture_output=True, text=True, timeout=280)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    assert "layer_flow OK: 37 steps" in res.stdout


def test_cpp_commit_driver_runs(ops, tmp_path):
    """the reference's artefact pipeline (test/ppgen.cu, the witness files of zzllama/llama/model.py,
    test/commit.cu:37-183) by a C++ program against the host classes, at 1/16 of the model's widths:
    points.bin / cpu_points.bin written and read back, 32 witness files committed from disk into
    com{W,Q,R}, and the stored commitments verify openings of the stored tensors (a changed
    commitment does not)"""
    import subprocess
    import driver_build
    exe = driver_build.build(None, "commit_flow")
    res = subprocess.run([exe, str(tmp_path / "artefacts"), "64"], capture_output=True, text=True, timeout=280)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    assert "commit_flow OK" in res.stdout
    assert (tmp_path / "artefacts" / "comW" / "down-0.bin").stat().st_size > 0


def test_cpp_reference_programs_run(ops, tmp_path):
    """the reference's six single-protocol programs (test/matmul.cu, eleWiseMul.cu, combine_value.cu,
    tlookupTest.cu, tlookupMapTest.cu, HyraxTest.cu) as functions of a C++ program that keep their call
    sequences and read points.bin / cpu_points.bin / table/*.bin / {W,Q,R}/*.bin with loadbin and
    load_data; each result is also checked against a direct evaluation, and the two lookups refuse
    a witness that is off the table"""
    import subprocess
    import driver_build
    exe = driver_build.build(None, "programs_flow")
    res = subprocess.run([exe, str(tmp_path / "artefacts")], capture_output=True, text=True, timeout=280)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    assert "programs_flow OK" in res.stdout


def test_tlookup_mapping_keeps_its_rows_between_proofs(ops, host, gens):
    """a mapping lookup object proves several witnesses (the reference keeps one object for all layers):
    the rows B[t]*G_i built for the first are used again while they cover the witness, and are
    rebuilt when the occupied entries have moved; com(A) and the transcript always equal those of
    the plain full-width path"""
    import torch
    hg, dg = gens
    logN, low, msm = 12, -2048, 64
    N, D = 1 << logN, 1 << 13
    rng = np.random.default_rng(771)
    fmap = rng.integers(-1000, 1000, size=N).astype(np.int32)
    table = ops.g1_table_gen(dg[:msm].contiguous(), 256)
    alpha, r, u, v = rand_fr(1, 772), rand_fr(1, 773), rand_fr(13, 774), rand_fr(13, 775)

    def witness(centre, seed):
        g = np.random.default_rng(seed)
        s = np.clip(np.rint(g.normal(centre, 6.0, size=D)), low, low + N - 1).astype(np.int32)
        spread = g.random(D) < 0.05
        s[spread] = g.integers(low, low + N, size=int(spread.sum()))
        return s

    def prove(s_in, indexed=True):
        host.set_indexed_commit(indexed)
        dSi = ops.fr_from_i32(torch.from_numpy(s_in).cuda())
        dSo = ops.fr_from_i32(torch.from_numpy(fmap[s_in - low]).cuda())
        out = host.tlookup_mapping_prove_ex(dSi, dSo, D, low, N, fmap, alpha, r, u, v, table, msm, 1, msm)
        host.set_indexed_commit(True)
        return out

    w1, w2, w3 = witness(0.0, 1), witness(0.0, 2), witness(700.0, 3)
    tr1, sc1, com1, hot1, cold1, reused1 = prove(w1)
    assert not reused1 and hot1 > 0 and cold1 > 0
    tr1b, sc1b, com1b, hot1b, cold1b, reused1b = prove(w1)
    assert reused1b and hot1b == hot1 and cold1b == cold1
    assert_same(com1b, com1, "same witness, rows in place")
    assert_same(tr1b, tr1, "transcript")
    # another witness on the same entries: the rows serve it, its own elements outside them are counted
    tr2, sc2, com2, hot2, cold2, reused2 = prove(w2)
    assert reused2 and hot2 == hot1
    slot = np.bincount(w1.astype(np.int64) - low, minlength=N) >= int(1.8 * msm) + 1
    assert cold2 == int((~slot[w2.astype(np.int64) - low]).sum())
    tr2p, sc2p, com2p, h, c, _ = prove(w2, indexed=False)
    assert h == 0 and c == 0
    assert_same(com2, com2p, "com(A) through kept rows == full-width commitment")
    assert_same(tr2, tr2p, "transcript")
    # the occupied entries have moved: the kept rows cover almost nothing and are replaced
    tr3, sc3, com3, hot3, cold3, reused3 = prove(w3)
    assert not reused3 and hot3 > 0
    tr3p, sc3p, com3p, _, _, _ = prove(w3, indexed=False)
    assert_same(com3, com3p, "com(A) after the rows were rebuilt")
    assert_same(tr3, tr3p, "transcript")
    assert prove(w3)[5]


@pytest.mark.parametrize("hot_min_count,pad", [(0, False), (1, False), (40, False), (300, False), (40, True)])
def test_tlookup_mapping_commits_A_through_occupied_entries(ops, host, gens, hot_min_count, pad):
    """com(A) of a mapping lookup through a per-proof table of the entries that occur often: the
    witness sits on a few entries of a 4096-entry table (activations do), the rest of it is spread.
    Whatever the split between table rows and full-width scalars (none with the break-even count of
    this tiny shape, every occupied entry with 1, a mix with 40 or 300), the commitment is the
    oracle's commitment of A = 1/(S + beta), and the transcript does not change."""
    import torch
    hg, dg = gens
    logN, low = 12, -2048
    N = 1 << logN
    D = 2 * 11008 if pad else 1 << 13
    rng = np.random.default_rng(71 + hot_min_count)
    fmap = rng.integers(-1000, 1000, size=N).astype(np.int32)
    S_in = np.clip(np.rint(rng.normal(0.0, 6.0, size=D)), low, low + N - 1).astype(np.int32)
    spread = rng.random(D) < 0.1
    S_in[spread] = rng.integers(low, low + N, size=int(spread.sum()))
    S_out = fmap[S_in - low]
    logDp = 15 if pad else 13
    alpha, r, u, v = rand_fr(1, 72), rand_fr(1, 73), rand_fr(logDp, 74), rand_fr(logDp, 75)
    beta = br.fr_pack([N])[0]
    T, B = orc.tlookup_init(low, N, beta, orc.from_i32(fmap), r[0])
    m = orc.tlookup_prep(orc.from_i32(S_in), low, N)
    S = orc.vec2("orc_fr_vec_add", orc.vec_bcast("orc_fr_vec_bcast_mul", orc.from_i32(S_out), r[0]), orc.from_i32(S_in))
    if pad:
        pad_val = orc.fr_mul(orc.from_i32(fmap[-low: -low + 1])[0], r[0])
        Spad = np.zeros((32768, 4), dtype=np.uint64)
        orc.lib().orc_fr_pad(orc.P(Spad), orc.P(S), orc.c32(11008), orc.c32(16384), orc.c64(32768), orc.P(pad_val))
        S = Spad
    st, wtr, wsc = orc.tlookup_prove(S, T, B, m, alpha[0], beta, u, v)
    assert st == 0
    msm = 64
    table = ops.g1_table_gen(dg[:msm].contiguous(), 256)
    dSi = ops.fr_from_i32(torch.from_numpy(S_in).cuda())
    dSo = ops.fr_from_i32(torch.from_numpy(S_out).cuda())
    tr, sc, com_a, n_hot, n_cold, _ = host.tlookup_mapping_prove_ex(dSi, dSo, D, low, N, fmap, alpha, r, u, v, table, msm, 1, msm,
                                                                 hot_min_count=hot_min_count)
    assert_same(tr, wtr, "transcript")
    assert_same(sc, wsc, "S(v)")
    counts = np.bincount(S_in.astype(np.int64) - low, minlength=N)
    if pad:
        counts[-low] += 32768 - D
    thr = hot_min_count if hot_min_count else int(1.8 * msm) + 1
    assert n_hot == int((counts >= thr).sum())
    assert n_cold == int(counts[counts < thr].sum())
    if hot_min_count == 1:
        assert n_cold == 0
    if hot_min_count in (40, 300):
        assert n_hot > 0 and n_cold > 0
    Ainv = orc.vec1("orc_fr_vec_inv", orc.vec_bcast("orc_fr_vec_bcast_add", S, beta))
    tab = orc.g1_table(hg[:msm], 256)
    nrows = S.shape[0] // msm
    assert com_a.shape[0] == nrows
    rows = sorted({0, 1, nrows // 2, nrows - 2, nrows - 1} | set(rng.integers(0, nrows, 16).tolist()))
    for rr in rows:
        assert_same(com_a[rr:rr + 1], orc.commit_fr(Ainv[rr * msm:(rr + 1) * msm], tab, msm, msm), "com(A) row %d" % rr)


def test_occupied_entry_selection_kernels(ops):
    """the device steps of the occupancy commitment against numpy: slots in table order for entries at
    or above the count, the cap on the number of slots, the cold element count, the remapped
    indices, the masked tensor, the gathered scalars; and the affine sum of two commitments
    (equal, opposite and infinite operands included) against the oracle's group law"""
    import torch
    rng = np.random.default_rng(81)
    N, n = 5000, 100000
    idx1 = rng.integers(0, N + 1, size=n).astype(np.int32)          # 0 = outside the table
    idx1[: n // 2] = rng.integers(1, 40, size=n // 2)
    hist = np.bincount(idx1[idx1 > 0].astype(np.int64) - 1, minlength=N).astype(np.int32)
    for min_count, max_hot in [(1, N), (50, N), (50, 7), (10 ** 6, N)]:
        slot1, hot, n_hot, n_cold = ops.tlookup_hot_select(torch.from_numpy(hist).cuda(), min_count, max_hot)
        want_hot = np.nonzero(hist >= min_count)[0][:max_hot]
        assert n_hot == len(want_hot) and np.array_equal(hot.cpu().numpy(), want_hot)
        want_slot = np.zeros(N, dtype=np.int32)
        want_slot[want_hot] = np.arange(1, len(want_hot) + 1)
        assert np.array_equal(slot1.cpu().numpy(), want_slot)
        assert n_cold == int(hist.sum()) - int(hist[want_hot].sum())
        d_idx = torch.from_numpy(idx1).cuda()
        h1 = ops.tlookup_hot_index(d_idx, slot1).cpu().numpy()
        assert np.array_equal(h1, np.where(idx1 > 0, want_slot[np.maximum(idx1, 1) - 1], 0))
    X = rand_fr(3000, 82)
    h = rng.integers(0, 3, size=3000).astype(np.int32)
    got = ops.fr_to_host(ops.fr_mask_cold(ops.to_dev(X), torch.from_numpy(h).cuda()))
    want = X.copy()
    want[h != 0] = 0
    assert_same(got, want, "masked")
    lst = rng.integers(0, 3000, size=777).astype(np.int32)
    assert_same(ops.fr_to_host(ops.fr_gather(ops.to_dev(X), torch.from_numpy(lst).cuda())), X[lst], "gathered")
    # affine sums
    k = rand_fr(40, 83)
    hp = orc.g1_make_generators(k)
    a, b = hp[:20].copy(), hp[20:].copy()
    b[0] = a[0]                                   # doubling
    half = a.shape[1] // 2
    b[1, :half] = a[1, :half]
    b[1, half:] = orc.fp_neg(a[1, half:])         # opposite -> infinity
    a[2] = 0                                      # infinity + Q
    b[3] = 0                                      # P + infinity
    a[4] = 0
    b[4] = 0
    got = ops.g1_to_host(ops.g1_affine_add(ops.to_dev(a), ops.to_dev(b)))
    want = np.zeros_like(a)
    for i in range(a.shape[0]):
        orc.lib().orc_g1_add_affine(orc.P(want[i]), orc.P(a[i]), orc.P(b[i]))
    assert not want[1].any() and not want[4].any() and np.array_equal(want[2], b[2]) and np.array_equal(want[3], a[3])
    assert_same(got, want, "affine sums")


def test_index_and_inverse_in_one_pass_and_axpy(ops):
    """grape_tlookup_index_inverse against the two calls it replaces (index, then A = B[index] with
    the entry check), for a range witness and for a mapping witness with wrong outputs and keys
    outside the table; grape_fr_axpy against the oracle's scalar product and sum"""
    import torch
    rng = np.random.default_rng(101)
    low, N, n = -50, 128, 5000
    beta, r = br.fr_pack([N])[0], rand_fr(1, 102)
    fmap = rng.integers(-999, 999, size=N).astype(np.int32)
    keys = rng.integers(low, low + N, size=n).astype(np.int32)
    # range: every key inside
    T, B = orc.tlookup_init(low, N, beta)
    dK = ops.fr_from_i32(torch.from_numpy(keys).cuda())
    idx1, A, mm = ops.tlookup_index_inverse(dK, low, ops.to_dev(B))
    assert mm == 0
    assert np.array_equal(idx1.cpu().numpy(), keys - low + 1)
    assert_same(ops.fr_to_host(A), B[keys - low], "A = B[index]")
    # mapping: 7 wrong outputs and 5 keys outside the table are counted and left alone
    outs = fmap[keys - low].copy()
    wrong = rng.choice(n, 7, replace=False)
    outs[wrong] += 1
    keys2 = keys.copy()
    outside = np.setdiff1d(rng.choice(n, 20, replace=False), wrong)[:5]
    keys2[outside] = low + N + 3
    dK2 = ops.fr_from_i32(torch.from_numpy(keys2).cuda())
    dO = ops.fr_from_i32(torch.from_numpy(outs).cuda())
    Tm, Bm = orc.tlookup_init(low, N, beta, orc.from_i32(fmap), r[0])
    idx1, A, mm = ops.tlookup_index_inverse(dK2, low, ops.to_dev(Bm), cmp=dO, cmp_table=ops.fr_from_i32(torch.from_numpy(fmap).cuda()))
    assert mm == 12
    want_idx = keys2 - low + 1
    want_idx[outside] = 0
    assert np.array_equal(idx1.cpu().numpy(), want_idx)
    good = np.ones(n, dtype=bool)
    good[wrong] = False
    good[outside] = False
    assert_same(ops.fr_to_host(A)[good], Bm[(keys2 - low)[good]], "A where the element matches its entry")
    # x + r*y
    x, y = rand_fr(777, 103), rand_fr(777, 104)
    want = orc.vec2("orc_fr_vec_add", x, orc.vec_bcast("orc_fr_vec_bcast_mul", y, r[0]))
    assert_same(ops.fr_to_host(ops.fr_axpy(ops.to_dev(x), ops.to_dev(r), ops.to_dev(y))), want, "x + r*y")
