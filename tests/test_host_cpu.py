"""CPU checks of the C++ host library: it loads, exports its C entry points, and its host-side
scalar / group arithmetic (used for round polynomials and openings) agrees with Python integers."""
import random
import numpy as np
import bigref as br


def test_host_library_loads_and_exports():
    from grape_amd import _host
    lib = _host.load()
    for n in _host.NAMES:
        assert hasattr(lib, n)


def test_host_fr_arithmetic_vs_bigint():
    from grape_amd import _host
    rng = random.Random(1)
    vals = [0, 1, br.R_MOD - 1, 2**64, 2**255 % br.R_MOD] + [rng.randrange(br.R_MOD) for _ in range(20)]
    for a in vals:
        for b in vals[:8]:
            pa, pb = br.fr_pack([a]), br.fr_pack([b])
            assert br.fr_unpack(_host.fr_op(0, pa, pb))[0] == (a + b) % br.R_MOD
            assert br.fr_unpack(_host.fr_op(1, pa, pb))[0] == (a - b) % br.R_MOD
            assert br.fr_unpack(_host.fr_op(2, pa, pb))[0] == (a * b) % br.R_MOD
        inv = br.fr_unpack(_host.fr_op(3, br.fr_pack([a])))[0]
        assert inv == (pow(a, -1, br.R_MOD) if a else 0)


def test_host_g1_scalar_mul_vs_textbook():
    from grape_amd import _host
    for k in (0, 1, 2, 12345678901234567890, br.R_MOD - 1):
        got = br.g1_unpack(_host.g1_mul_generator(br.fr_pack([k])))[0]
        assert got == br.g1_mul(k, br.G1)


def test_file_helpers_on_host_memory(tmp_path):
    """savebin / loadbin / findsize with host buffers (src/ioutils.cu:3-103): raw bytes, a short
    file leaves the destination untouched, a missing file is size 0"""
    from grape_amd import _host
    a = np.arange(1000, dtype=np.int32) * 7 - 3
    f = str(tmp_path / "t.bin")
    _host.savebin(f, a.ctypes.data, a.nbytes, is_gpu=False)
    assert _host.findsize(f) == a.nbytes
    assert np.array_equal(np.fromfile(f, dtype=np.int32), a)
    b = np.zeros_like(a)
    _host.loadbin(f, b.ctypes.data, b.nbytes, is_gpu=False)
    assert np.array_equal(a, b)
    c = np.full(2000, -1, dtype=np.int32)
    _host.loadbin(f, c.ctypes.data, c.nbytes, is_gpu=False)      # asks for more than the file holds
    assert (c == -1).all()
    assert _host.findsize(str(tmp_path / "absent.bin")) == 0


def test_cpp_driver_compiles_against_the_host_headers():
    """a driver in the reference's style builds with g++ against the host classes alone (no HIP
    headers, no kernels); the GPU suite runs it"""
    import os
    import driver_build
    assert os.path.exists(driver_build.build(None, "layer_flow"))
    assert os.path.exists(driver_build.build(None, "commit_flow"))
    assert os.path.exists(driver_build.build(None, "programs_flow"))
    exe = driver_build.build()
    assert os.path.exists(exe)


def test_witness_tables_and_float16_match_the_oracle():
    """the C++ table generators and float16 rounding against the numpy oracle (no GPU involved)"""
    import numpy as np
    from oracle import witness_oracle as wo
    from grape_amd import _host as host
    e, s = host.witness_tables()
    assert np.array_equal(e, wo.exp_table()) and np.array_equal(s, wo.silu_table())
    rng = np.random.default_rng(11)
    xs = np.concatenate([rng.uniform(0, 400, 2000), rng.uniform(0, 1e-3, 500), rng.uniform(0, 1e-7, 200),
                         np.array([0.0, 1.0, 65504.0, 2.0 ** -14, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 1.00048828125, 1.00146484375])])
    want = wo.to_float16(xs)
    for x, w in zip(xs.tolist(), want.tolist()):
        assert host.to_float16(x) == w, x
        assert host.to_float16(-x) == -w
