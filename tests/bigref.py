"""Independent Python big-integer reference used to pin the CPU oracle.

Nothing here shares code with the oracle or the HIP library: field operations are plain
``%`` arithmetic on Python integers, the group law is the textbook affine chord-and-tangent
rule, multilinear extensions are evaluated by brute force from their definition.  The tests
compare the oracle (64-bit limbs, Montgomery form) with these closed forms.
"""
import os
import numpy as np

# The curve is chosen by the environment variable GRAPE_CURVE: "bls12_381" (default, the curve of
# the benchmark configurations) or "bn254" (the reference's active curve).
CURVE = os.environ.get("GRAPE_CURVE", "bls12_381")
if CURVE == "bn254":
    R_MOD = 21888242871839275222246405745257275088548364400416034343698204186575808495617
    P_MOD = 21888242871839275222246405745257275088696311157297823662689037894645226208583
    FP_LIMBS = 4      # 64-bit limbs of a base-field element
    CURVE_B = 3
    G1_X, G1_Y = 1, 2
elif CURVE == "bls12_381":
    R_MOD = 0x73eda753299d7d483339d80809a1d80553bda402fffe5bfeffffffff00000001
    P_MOD = 0x1a0111ea397fe69a4b1ba7b6434bacd764774b84f38512bf6730d2a0f6b0f6241eabfffeb153ffffb9feffffffffaaab
    FP_LIMBS = 6
    CURVE_B = 4
    G1_X = 0x17f1d3a73197d7942695638c4fa9ac0fc3688c4f9774b905a14e3a3f171bac586c55e83ff97a1aeffb3af00adb22c6bb
    G1_Y = 0x08b3f481e3aaa0f1a09e30ed741d8ae4fcf5e095d5d00af600db18cb2c04b3edd03cc744a2888ae40caa232946c5e7e1
else:
    raise ValueError("GRAPE_CURVE must be bls12_381 or bn254, not %r" % CURVE)
FR_R = 1 << 256                  # Montgomery radix of Fr
FP_R = 1 << (64 * FP_LIMBS)      # Montgomery radix of Fp
G1_WORDS = 2 * FP_LIMBS          # 64-bit words of an affine point
G1 = (G1_X, G1_Y)


# ---------------------------------------------------------------- limb packing
def ints_to_limbs(vals, nlimbs64):
    """list of Python ints -> (n, nlimbs64) uint64, little-endian limbs."""
    out = np.zeros((len(vals), nlimbs64), dtype=np.uint64)
    mask = (1 << 64) - 1
    for i, v in enumerate(vals):
        for j in range(nlimbs64):
            out[i, j] = (v >> (64 * j)) & mask
    return out


def limbs_to_ints(arr):
    arr = np.asarray(arr, dtype=np.uint64)
    arr = arr.reshape(-1, arr.shape[-1])
    return [sum(int(arr[i, j]) << (64 * j) for j in range(arr.shape[1])) for i in range(arr.shape[0])]


def fr_pack(vals):
    """canonical integers mod r -> Montgomery limbs (n,4)."""
    return ints_to_limbs([(v % R_MOD) * FR_R % R_MOD for v in vals], 4)


def fr_unpack(arr):
    rinv = pow(FR_R, -1, R_MOD)
    return [x * rinv % R_MOD for x in limbs_to_ints(np.asarray(arr).reshape(-1, 4))]


def fp_pack(vals):
    return ints_to_limbs([(v % P_MOD) * FP_R % P_MOD for v in vals], FP_LIMBS)


def fp_unpack(arr):
    rinv = pow(FP_R, -1, P_MOD)
    return [x * rinv % P_MOD for x in limbs_to_ints(np.asarray(arr).reshape(-1, FP_LIMBS))]


def g1_pack(points):
    """list of affine points (x,y) or None (infinity) -> (n, G1_WORDS) uint64 Montgomery."""
    flat = []
    for pt in points:
        if pt is None:
            flat += [0, 0]
        else:
            flat += [pt[0], pt[1]]
    return fp_pack(flat).reshape(len(points), G1_WORDS)


def g1_unpack(arr):
    arr = np.asarray(arr, dtype=np.uint64).reshape(-1, G1_WORDS)
    coords = fp_unpack(arr.reshape(-1, FP_LIMBS))
    out = []
    for i in range(arr.shape[0]):
        x, y = coords[2 * i], coords[2 * i + 1]
        out.append(None if (x == 0 and y == 0) else (x, y))
    return out


# ---------------------------------------------------------------- textbook G1
def g1_on_curve(pt):
    if pt is None:
        return True
    x, y = pt
    return (y * y - x * x * x - CURVE_B) % P_MOD == 0


def g1_neg(pt):
    if pt is None:
        return None
    return (pt[0], (-pt[1]) % P_MOD)


def g1_add(a, b):
    if a is None:
        return b
    if b is None:
        return a
    x1, y1 = a
    x2, y2 = b
    if x1 == x2:
        if (y1 + y2) % P_MOD == 0:
            return None
        lam = 3 * x1 * x1 * pow(2 * y1, -1, P_MOD) % P_MOD
    else:
        lam = (y2 - y1) * pow(x2 - x1, -1, P_MOD) % P_MOD
    x3 = (lam * lam - x1 - x2) % P_MOD
    y3 = (lam * (x1 - x3) - y1) % P_MOD
    return (x3, y3)


def g1_mul(k, pt):
    if k < 0:
        return g1_mul(-k, g1_neg(pt))
    acc = None
    add = pt
    while k:
        if k & 1:
            acc = g1_add(acc, add)
        add = g1_add(add, add)
        k >>= 1
    return acc


def g1_msm(scalars, points):
    acc = None
    for s, pt in zip(scalars, points):
        acc = g1_add(acc, g1_mul(s, pt))
    return acc


# ---------------------------------------------------------------- multilinear extensions
def log2ceil(n):
    """ceil(log2 n) with log2ceil(0) = log2ceil(1) = 0."""
    return 0 if n <= 1 else (n - 1).bit_length()


def eq_weight(i, u):
    """prod_j (u_j if bit_j(i) else 1-u_j), LSB-first."""
    w = 1
    for j, uj in enumerate(u):
        w = w * (uj if (i >> j) & 1 else (1 - uj)) % R_MOD
    return w


def mle_eval(t, u):
    """T(u) = sum_i t[i] * eq(i, u), zero-extended to 2^len(u)."""
    assert len(t) <= (1 << len(u))
    return sum(ti * eq_weight(i, u) for i, ti in enumerate(t)) % R_MOD


def fold_axis(t, outer, c, gap, x):
    """Fold the middle axis of a [outer][c][gap] array with challenges x (LSB-first, zero padded)."""
    L = log2ceil(c)
    assert len(x) == L
    out = []
    for o in range(outer):
        for g in range(gap):
            out.append(sum(t[(o * c + i) * gap + g] * eq_weight(i, x) for i in range(c)) % R_MOD)
    return out  # [outer][gap]


def eq1(u, t):
    """(1-u)(1-t) + u t."""
    return ((1 - u) * (1 - t) + u * t) % R_MOD
