"""Shared helpers of the GPU parity tests: seeded inputs and oracle/HIP comparison."""
import numpy as np
import bigref as br


def rand_fr(n, seed):
    """n uniformly random Fr elements (rejection sampling of 255-bit draws), Montgomery limbs."""
    rng = np.random.default_rng(seed)
    out = np.zeros((n, 4), dtype=np.uint64)
    mod = np.array(br.ints_to_limbs([br.R_MOD], 4)[0])
    todo = np.arange(n)
    while todo.size:
        draw = rng.integers(0, 1 << 64, size=(todo.size, 4), dtype=np.uint64)
        draw[:, 3] &= np.uint64((1 << 63) - 1)
        # lexicographic compare from the top limb
        lt = np.zeros(todo.size, dtype=bool)
        decided = np.zeros(todo.size, dtype=bool)
        for j in (3, 2, 1, 0):
            lt |= (~decided) & (draw[:, j] < mod[j])
            decided |= draw[:, j] != mod[j]
        out[todo[lt]] = draw[lt]
        todo = todo[~lt]
    return out   # a uniformly random residue read as Montgomery form is a uniformly random element


def gaussian_i16(shape, seed, sigma=1024.0):
    rng = np.random.default_rng(seed)
    x = np.rint(rng.normal(0.0, sigma, size=shape))
    return np.clip(x, -32768, 32767).astype(np.int32)


def assert_same(got, want, what=""):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if not np.array_equal(got, want):
        bad = np.nonzero((got != want).reshape(got.shape[0], -1).any(axis=1))[0]
        raise AssertionError("%s: %d of %d entries differ, first at %d" % (what, bad.size, got.shape[0], bad[0]))
