"""GPU parity tests of the witness-generation kernels against the numpy oracle
(oracle/witness_oracle.py), bit-exact, through the C ABI."""
import numpy as np
import pytest
import torch
from oracle import witness_oracle as wo
import witutil

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from grape_amd import ops as o
    o.init(0)
    o.wit_status()                          # start from a clean status word
    return o


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).cuda()


def host(t):
    return t.cpu().numpy()


SHAPES = [
    (1, 8, 64, 64, 1 << 16, False), (1, 8, 176, 64, 1 << 20, False), (1, 8, 64, 176, 1 << 16, False),
    (1, 8, 8, 64, 1 << 22, False), (1, 8, 64, 8, 1 << 16, True), (1, 130, 257, 100, 1 << 16, False),
    (3, 129, 40, 36, 1 << 16, True), (1, 5, 7, 13, 1 << 16, False), (2, 3, 9, 6, 1000, True),
    (1, 256, 384, 512, 1 << 16, False), (1, 1, 1, 4, 1 << 16, False), (1, 300, 128, 68, 12345, False)]


# method 1: every shape; method 2 (the matrix-core path) takes one batch with K a multiple of 4
@pytest.mark.parametrize("L,N,M,K,scale,tr,method",
                         [s + (1,) for s in SHAPES] + [s + (2,) for s in SHAPES if s[0] == 1 and s[3] % 4 == 0])
def test_matmul_rescale_matches_the_oracle(ops, L, N, M, K, scale, tr, method):
    """method 1: 64-bit multiply-add kernels; method 2: int8 matrix-core products of byte planes"""
    rng = np.random.default_rng(L * 1000 + N + M + K)
    a = rng.integers(-(1 << 20), 1 << 20, (L, N, K)).astype(np.int32)
    b = rng.integers(-(1 << 17), 1 << 17, (L, M, K)).astype(np.int32)
    ops.wit_set_matmul_method(method)
    try:
        q, r = ops.wit_matmul_rescale(dev(a), dev(b), scale, transpose_out=tr)
        q2, r2 = ops.wit_matmul_rescale(dev(a), dev(b), scale, want_r=False, transpose_out=tr)
    finally:
        ops.wit_set_matmul_method(0)
    for l in range(L):
        wq, wr = wo.rescale(wo.matmul_t(a[l], b[l]), scale)
        if tr:
            wq, wr = wq.T, wr.T
        assert np.array_equal(host(q)[l], wq) and np.array_equal(host(r)[l], wr)
    assert r2 is None and torch.equal(q2, q)
    assert ops.wit_status() == 0


@pytest.mark.parametrize("amax,bmax", [(50, 50), (1 << 13, 60), (60, 1 << 13), ((1 << 22) - 1, (1 << 14) - 1), ((1 << 14) - 1, (1 << 22) - 1),
                                       ((1 << 22) - 1, (1 << 22) - 1)])
def test_matrix_core_path_over_every_plane_count(ops, amax, bmax):
    """operands at the edges of the 1-, 2- and 3-plane ranges, including the extreme values themselves"""
    rng = np.random.default_rng(amax % 1000 + bmax % 777)
    N, M, K = 70, 130, 200
    a = rng.integers(-amax, amax + 1, (N, K)).astype(np.int32)
    b = rng.integers(-bmax, bmax + 1, (M, K)).astype(np.int32)
    a[0, :4] = (amax, -amax, amax, -amax)
    b[0, :4] = (bmax, -bmax, -bmax, bmax)
    a[1, :] = amax
    b[1, :] = -bmax
    ops.wit_set_matmul_method(2)
    try:
        q, r = ops.wit_matmul_rescale(dev(a), dev(b), 1 << 31)
    finally:
        ops.wit_set_matmul_method(0)
    wq, wr = wo.rescale(wo.matmul_t(a, b), 1 << 31)
    assert np.array_equal(host(q), wq) and np.array_equal(host(r), wr)
    assert ops.wit_status() == 0


@pytest.mark.parametrize("amax,bmax,K,tr", [(60, 60, 132, False), ((1 << 22) - 1, (1 << 14) - 1, 132, False), ((1 << 14) - 1, (1 << 22) - 1, 68, True),
                                            ((1 << 22) - 1, (1 << 22) - 1, 132, False), ((1 << 20), (1 << 15) - 1, 64, True)])
def test_matrix_core_path_with_a_tile_per_cu(ops, amax, bmax, K, tr):
    """a product of 17 x 16 tiles of 128 x 128 (ragged on both sides) takes the large-tile kernel: one, two and
    three K steps, every plane count, both output orders"""
    rng = np.random.default_rng(amax % 1000 + bmax % 777 + K)
    N, M = 2061, 1925
    a = rng.integers(-amax, amax + 1, (N, K)).astype(np.int32)
    b = rng.integers(-bmax, bmax + 1, (M, K)).astype(np.int32)
    a[N - 1, :] = amax
    b[M - 1, :] = -bmax
    ops.wit_set_matmul_method(2)
    try:
        q, r = ops.wit_matmul_rescale(dev(a), dev(b), 1 << 31, transpose_out=tr)
    finally:
        ops.wit_set_matmul_method(0)
    wq, wr = wo.rescale(wo.matmul_t(a, b), 1 << 31)
    if tr:
        wq, wr = wq.T, wr.T
    assert np.array_equal(host(q), wq) and np.array_equal(host(r), wr)
    assert ops.wit_status() == 0


def test_matrix_core_path_refuses_what_it_cannot_do(ops):
    from grape_amd import _capi
    a = np.full((8, 64), 1 << 22, dtype=np.int32)      # four byte planes
    b = np.ones((8, 64), dtype=np.int32)
    ops.wit_set_matmul_method(2)
    try:
        with pytest.raises(_capi.GrapeError):
            ops.wit_matmul_rescale(dev(a), dev(b), 1 << 16)
    finally:
        ops.wit_set_matmul_method(0)
    q, r = ops.wit_matmul_rescale(dev(a), dev(b), 1 << 16)      # the chooser falls back to the multiply-add kernel
    assert np.array_equal(host(q).astype(np.int64) * 65536 + host(r), wo.matmul_t(a, b))
    ops.wit_status()


def test_matmul_extreme_entries_stay_exact(ops):
    """products of the largest int32 activations with 25-bit weights accumulate exactly in 64 bits"""
    K = 64
    a = np.full((4, K), -(1 << 31), dtype=np.int64)
    a[1] = (1 << 31) - 1
    a[2, ::2] = (1 << 31) - 1
    b = np.full((3, K), (1 << 24) - 1, dtype=np.int64)
    b[1] = -(1 << 24)
    S = 1 << 31
    q, r = ops.wit_matmul_rescale(dev(a), dev(b), S)
    y = [[sum(x * z for x, z in zip(ra, rb)) for rb in b.tolist()] for ra in a.tolist()]
    assert host(q).tolist() == [[(v + S // 2) // S for v in row] for row in y]
    assert [[qq * S + rr for qq, rr in zip(qr, rr_)] for qr, rr_ in zip(host(q).tolist(), host(r).tolist())] == y
    assert ops.wit_status() == 0
    # a quotient that does not fit int32 is reported, not hidden
    ops.wit_matmul_rescale(dev(a), dev(b), 1 << 16)
    assert ops.wit_status() & 1
    assert ops.wit_status() == 0


def test_elementwise_kernels(ops):
    rng = np.random.default_rng(7)
    a = rng.integers(-(1 << 20), 1 << 20, 100003).astype(np.int32)
    b = rng.integers(-(1 << 22), 1 << 22, 100003).astype(np.int32)
    for s in (1 << 16, 1 << 20, 7777):
        q, r = ops.wit_elemul_rescale(dev(a), dev(b), s)
        wq, wr = wo.rescale(a.astype(np.int64) * b.astype(np.int64), s)
        assert np.array_equal(host(q), wq) and np.array_equal(host(r), wr)
    assert np.array_equal(host(ops.wit_add(dev(a), dev(b))), a + b)
    table = wo.silu_table()
    x = rng.integers(-(1 << 18), 1 << 18, 50000).astype(np.int32)
    x[:2] = (-(1 << 18), (1 << 18) - 1)
    got = ops.wit_table_lookup(dev(x), -(1 << 18), dev(table))
    assert np.array_equal(host(got), wo.lut(x, table, 1 << 18, 19))
    assert ops.wit_status() == 0
    x[5] = 1 << 18                                   # one past the table: the reference asserts here
    ops.wit_table_lookup(dev(x), -(1 << 18), dev(table))
    assert ops.wit_status() == 2


@pytest.mark.parametrize("rows,cols,sigma", [(12, 50, 65536.0), (3, 1, 1000.0), (5, 257, 40000.0), (2, 2048, 65536.0), (64, 300, 5.0)])
def test_softmax_matches_the_oracle(ops, rows, cols, sigma):
    rng = np.random.default_rng(rows * cols)
    scores = np.rint(rng.normal(0, sigma, (rows, cols))).astype(np.int32)
    table = wo.exp_table()
    got = ops.wit_softmax(dev(scores), dev(table))
    want = wo.softmax(scores, table)
    for k in want:
        assert np.array_equal(host(got[k]), want[k]), k
    assert ops.wit_status() == 0


def test_softmax_reports_an_index_outside_the_table(ops):
    scores = np.zeros((2, 8), dtype=np.int32)
    scores[1, 3] = -(1 << 20)                         # shifted index -1
    ops.wit_softmax(dev(scores), dev(wo.exp_table()))
    assert ops.wit_status() == 2


def test_row_sumsq_and_rmsnorm_apply(ops):
    rng = np.random.default_rng(9)
    for rows, cols in ((16, 64), (5, 4096), (3, 1000), (1, 1)):
        x = np.rint(rng.normal(0, 65536.0, (rows, cols))).astype(np.int32)
        if rows > 1:
            x[1] = 0
        got = host(ops.wit_row_sumsq(dev(x))).view(np.uint64)
        want = [sum(int(v) * int(v) for v in row) for row in x.tolist()]
        assert got.tolist() == want
        w = (65536 + np.rint(rng.normal(0, 2000.0, cols))).astype(np.int32)
        n = wo.rmsnorm(x, w)
        outs = ops.wit_rmsnorm_apply(dev(x), dev(n["rms"].reshape(-1)), dev(w))
        for t, k in zip(outs, ("q_rmsw", "r_rmsw", "q_out", "r_out")):
            assert np.array_equal(host(t), n[k]), k
    # large entries: 64 values of 2^31-1 squared stay below 2^64 (2^68 would not)
    big = np.full((2, 3), (1 << 31) - 1, dtype=np.int32)
    assert host(ops.wit_row_sumsq(dev(big))).view(np.uint64).tolist() == [3 * ((1 << 31) - 1) ** 2] * 2
    assert ops.wit_status() == 0
    ops.wit_row_sumsq(dev(np.full((1, 8), -(1 << 31), dtype=np.int64)))
    assert ops.wit_status() == 8


def test_full_size_matmul_properties(ops):
    """2048 x 4096 by 11008 x 4096 (the gate projection's shape): q*S + r equals the exact product on
    sampled entries, remainders lie in [-S/2, S/2), and the result is linear in the activations"""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    x = (torch.randn(2048, 4096, generator=g, device="cuda") * 65536).round().to(torch.int32)
    w = (torch.randn(11008, 4096, generator=g, device="cuda") * 1024).round().clamp_(-32768, 32767).to(torch.int32)
    S = 1 << 20
    q, r = ops.wit_matmul_rescale(x, w, S)
    assert int(r.min()) >= -(S // 2) and int(r.max()) < S // 2
    rng = np.random.default_rng(1)
    xs, ws = x.cpu().numpy().astype(np.int64), w.cpu().numpy().astype(np.int64)
    qh, rh = q.cpu().numpy().astype(np.int64), r.cpu().numpy().astype(np.int64)
    for n, m in zip(rng.integers(0, 2048, 200).tolist(), rng.integers(0, 11008, 200).tolist()):
        assert qh[n, m] * S + rh[n, m] == int(np.dot(xs[n], ws[m]))
    # whole rows against float64 products (exact below 2^53, as the reference relies on)
    rows = [0, 1, 777, 2047]
    y = torch.matmul(x[rows].double(), w.double().t()).to(torch.int64)
    assert torch.equal(q[rows].to(torch.int64) * S + r[rows].to(torch.int64), y)
    assert ops.wit_status() == 0


# ------------------------------------------------------------------ the C++ LayerWitness class
def _run_layer(T, D, F, seed):
    from grape_amd import _host as host
    x, weights = witutil.layer_inputs(T, D, F, seed)
    e, s = wo.exp_table(), wo.silu_table()
    lw = host.LayerWitness(T, D, F)
    lw.generate(dev(x), {k: dev(v) for k, v in weights.items()}, dev(e), dev(s))
    want = wo.layer(x, weights, {"exp": e, "silu": s})
    return lw, want


@pytest.mark.parametrize("T,D,F,seed", [(8, 64, 176, 6), (5, 36, 50, 7), (64, 256, 688, 8)])
def test_layer_witness_matches_the_oracle_tensor_by_tensor(ops, T, D, F, seed):
    lw, want = _run_layer(T, D, F, seed)
    assert sorted(lw.names()) == sorted(witutil.TENSOR_NAMES)
    for name in witutil.TENSOR_NAMES:
        got = lw.tensor(name)
        assert got.size == want[name].size, name
        assert np.array_equal(got, want[name].reshape(-1)), name
    lw.close()


def test_layer_witness_files_follow_the_reference_layout(ops, tmp_path):
    """save() appends raw int32 to <dir>/<W|Q|R>/<name>-<group>.bin, one layer after the other"""
    for d in ("W", "Q", "R"):
        (tmp_path / d).mkdir()
    lw, want = _run_layer(8, 64, 176, 6)
    lw.save(str(tmp_path), 3)
    lw.save(str(tmp_path), 3)                       # a second layer of the same group is appended
    for name in witutil.TENSOR_NAMES:
        data = np.fromfile(tmp_path / (name + "-3.bin"), dtype=np.int32)
        flat = want[name].reshape(-1)
        assert data.size == 2 * flat.size and np.array_equal(data[:flat.size], flat) and np.array_equal(data[flat.size:], flat), name
    lw.close()


def test_layer_witness_raises_where_the_reference_asserts(ops):
    from grape_amd import _host as host
    x, weights = witutil.layer_inputs(8, 64, 176, 9)
    weights["gate"] = weights["gate"] * 4096          # gate pre-activations far beyond the SiLU table
    lw = host.LayerWitness(8, 64, 176)
    with pytest.raises(host.HostError, match="table index"):
        lw.generate(dev(x), {k: dev(v) for k, v in weights.items()}, dev(wo.exp_table()), dev(wo.silu_table()))
    lw.close()
