// G1 group law (short Weierstrass, a = 0: BLS12-381 y^2 = x^3 + 4, BN254 y^2 = x^3 + 3) on
// Montgomery-form coordinates; the formulas never use b, so one body serves both curves.
//
// Point encodings follow the reference: affine infinity is (0,0) (include/curve/affine_t.cuh:28-39),
// a Jacobian point is at infinity when Z = 0 (include/curve/jacobian_t.cuh), an extended-Jacobian
// ("XYZZ": x = X/ZZ, y = Y/ZZZ, ZZ^3 = ZZZ^2) accumulator when ZZ = 0 (include/curve/xyzz_t.cuh).
// The mixed addition handles doubling (P = Q) and cancellation (P = -Q) exactly as
// xyzz_t.cuh:363-441 does, so any summation order gives the same group element.
// Formulas are the standard ones from the Explicit-Formulas Database (madd-2008-s, mdbl-2008-s-1,
// add-2008-s, dbl-2008-s-1 for XYZZ; dbl-2009-l for Jacobian).
#pragma once
#include "field.hpp"

namespace grape {

// Fp products used by the group law.  A translation unit may route them through out-of-line
// device functions (GRAPE_FP_MUL_OUTLINE) to keep kernels small: one shared multiplier body
// instead of a copy per call site.  The default is the inline multiplier.
#if defined(GRAPE_FP_MUL_OUTLINE) && defined(__HIP_DEVICE_COMPILE__)
__device__ __noinline__ Fp fp_mul_outline(Fp a, Fp b);
__device__ __noinline__ Fp fp_sqr_outline(Fp a);
__device__ __forceinline__ Fp fmul(const Fp& a, const Fp& b) { return fp_mul_outline(a, b); }
__device__ __forceinline__ Fp fsqr(const Fp& a) { return fp_sqr_outline(a); }
#else
GRAPE_HD Fp fmul(const Fp& a, const Fp& b) { return mul(a, b); }
GRAPE_HD Fp fsqr(const Fp& a) { return sqr(a); }
#endif

// a^(p-2) with the hooked multiplier (4-bit fixed windows, rolled loops).
GRAPE_HD Fp fp_inverse(const Fp& a) {
    Fp tbl[16];
    tbl[0] = Fp::one();
    tbl[1] = a;
    for (int i = 2; i < 16; i++) tbl[i] = fmul(tbl[i - 1], a);
    Fp acc = Fp::one();
    bool started = false;
    for (int limb = FpParams::N - 1; limb >= 0; limb--) {
        uint32_t e = 0;
        for (int k = 0; k < FpParams::N; k++) e = (k == limb) ? FpParams::pm2(k) : e;
        for (int nib = 7; nib >= 0; nib--) {
            if (started) {
                acc = fsqr(acc);
                acc = fsqr(acc);
                acc = fsqr(acc);
                acc = fsqr(acc);
            }
            uint32_t w = (e >> (4 * nib)) & 15u;
            if (w) {
                acc = fmul(acc, tbl[w]);
                started = true;
            }
        }
    }
    return acc;
}

// Affine coordinates of the standard generator in memory (Montgomery) form: the usual BLS12-381
// G1 generator resp. BN254's (1, 2) - what the reference's host group type calls one().
GRAPE_HD uint32_t g1_gen_x(int i) {
#if defined(GRAPE_CURVE_BN254)
    constexpr uint32_t t[8] = {0xc58f0d9du, 0xd35d438du, 0xf5c70b3du, 0x0a78eb28u,
                               0x7879462cu, 0x666ea36fu, 0x9a07df2fu, 0x0e0a77c1u};
#else
    constexpr uint32_t t[12] = {0xfd530c16u, 0x5cb38790u, 0x9976fff5u, 0x7817fc67u, 0x143ba1c1u, 0x154f95c7u,
                                0xf3d0e747u, 0xf0ae6acdu, 0x21dbf440u, 0xedce6eccu, 0x9e0bfb75u, 0x12017741u};
#endif
    return t[i];
}
GRAPE_HD uint32_t g1_gen_y(int i) {
#if defined(GRAPE_CURVE_BN254)
    constexpr uint32_t t[8] = {0x8b1e1b3au, 0xa6ba871bu, 0xeb8e167bu, 0x14f1d651u,
                               0xf0f28c58u, 0xccdd46deu, 0x340fbe5eu, 0x1c14ef83u};
#else
    constexpr uint32_t t[12] = {0x0ce72271u, 0xbaac93d5u, 0x7918fd8eu, 0x8c22631au, 0x570725ceu, 0xdd595f13u,
                                0x50405194u, 0x51ac5829u, 0xad0059c0u, 0x0e1c8c3fu, 0x5008a26au, 0x0bbc3efcu};
#endif
    return t[i];
}

struct alignas(16) G1Affine {
    Fp x, y;
    GRAPE_HD bool is_inf() const { return x.is_zero() & y.is_zero(); }
    static GRAPE_HD G1Affine inf() {
        G1Affine r;
        r.x = Fp::zero();
        r.y = Fp::zero();
        return r;
    }
};

struct alignas(16) G1Jac {
    Fp x, y, z;
    GRAPE_HD bool is_inf() const { return z.is_zero(); }
    static GRAPE_HD G1Jac inf() {
        G1Jac r;
        r.x = Fp::zero();
        r.y = Fp::zero();
        r.z = Fp::zero();
        return r;
    }
};

struct alignas(16) G1Xyzz {
    Fp x, y, zz, zzz;
    GRAPE_HD bool is_inf() const { return zz.is_zero(); }
    static GRAPE_HD G1Xyzz inf() {
        G1Xyzz r;
        r.x = Fp::zero();
        r.y = Fp::zero();
        r.zz = Fp::zero();
        r.zzz = Fp::zero();
        return r;
    }
    static GRAPE_HD G1Xyzz from_affine(const G1Affine& p) {
        G1Xyzz r;
        if (p.is_inf()) return inf();
        r.x = p.x;
        r.y = p.y;
        r.zz = Fp::one();
        r.zzz = Fp::one();
        return r;
    }
};

// acc += (negate ? -p : p), p affine. 8M + 2S on the common path.
GRAPE_HD void xyzz_add_affine(G1Xyzz& acc, const G1Affine& p, bool negate) {
    if (p.is_inf()) return;
    const Fp py = cneg(p.y, negate);
    if (acc.is_inf()) {
        acc.x = p.x;
        acc.y = py;
        acc.zz = Fp::one();
        acc.zzz = Fp::one();
        return;
    }
    Fp P = sub(fmul(p.x, acc.zz), acc.x);   // U2 - X1
    Fp R = sub(fmul(py, acc.zzz), acc.y);   // S2 - Y1
    if (!P.is_zero()) {
        Fp PP = fsqr(P);
        Fp PPP = fmul(P, PP);
        Fp Q = fmul(acc.x, PP);
        Fp X3 = sub(sub(sub(fsqr(R), PPP), Q), Q);
        Fp Y3 = sub(fmul(R, sub(Q, X3)), fmul(acc.y, PPP));
        acc.zz = fmul(acc.zz, PP);
        acc.zzz = fmul(acc.zzz, PPP);
        acc.x = X3;
        acc.y = Y3;
    } else if (R.is_zero()) {
        // same point: double the affine operand
        Fp U = dbl(py);
        Fp V = fsqr(U);
        Fp W = fmul(U, V);
        Fp S = fmul(p.x, V);
        Fp M = fsqr(p.x);
        M = add(add(M, M), M);
        Fp X3 = sub(sub(fsqr(M), S), S);
        Fp Y3 = sub(fmul(M, sub(S, X3)), fmul(W, py));
        acc.x = X3;
        acc.y = Y3;
        acc.zz = V;
        acc.zzz = W;
    } else {
        acc = G1Xyzz::inf();
    }
}

// acc = 2 * acc (dbl-2008-s-1, a = 0).
GRAPE_HD void xyzz_dbl(G1Xyzz& acc) {
    if (acc.is_inf()) return;
    Fp U = dbl(acc.y);
    if (U.is_zero()) {  // order-2 point cannot occur on a prime-order subgroup; keep total anyway
        acc = G1Xyzz::inf();
        return;
    }
    Fp V = fsqr(U);
    Fp W = fmul(U, V);
    Fp S = fmul(acc.x, V);
    Fp M = fsqr(acc.x);
    M = add(add(M, M), M);
    Fp X3 = sub(sub(fsqr(M), S), S);
    Fp Y3 = sub(fmul(M, sub(S, X3)), fmul(W, acc.y));
    acc.x = X3;
    acc.y = Y3;
    acc.zz = fmul(V, acc.zz);
    acc.zzz = fmul(W, acc.zzz);
}

// acc += q, both XYZZ. 12M + 2S on the common path.
GRAPE_HD void xyzz_add(G1Xyzz& acc, const G1Xyzz& q) {
    if (q.is_inf()) return;
    if (acc.is_inf()) {
        acc = q;
        return;
    }
    Fp U1 = fmul(acc.x, q.zz);
    Fp S1 = fmul(acc.y, q.zzz);
    Fp P = sub(fmul(q.x, acc.zz), U1);
    Fp R = sub(fmul(q.y, acc.zzz), S1);
    if (!P.is_zero()) {
        Fp PP = fsqr(P);
        Fp PPP = fmul(P, PP);
        Fp Q = fmul(U1, PP);
        Fp X3 = sub(sub(sub(fsqr(R), PPP), Q), Q);
        Fp Y3 = sub(fmul(R, sub(Q, X3)), fmul(S1, PPP));
        acc.zz = fmul(fmul(acc.zz, q.zz), PP);
        acc.zzz = fmul(fmul(acc.zzz, q.zzz), PPP);
        acc.x = X3;
        acc.y = Y3;
    } else if (R.is_zero()) {
        xyzz_dbl(acc);
    } else {
        acc = G1Xyzz::inf();
    }
}

// XYZZ -> Jacobian without inversion: the triple (X*ZZ, Y*ZZZ, ZZ) is a Jacobian representative
// with Z = ZZ, since x = X*ZZ/ZZ^2 and y = Y*ZZZ/ZZ^3 = Y/ZZZ (ZZZ^2 = ZZ^3).
GRAPE_HD G1Jac xyzz_to_jac(const G1Xyzz& p) {
    if (p.is_inf()) return G1Jac::inf();
    G1Jac r;
    r.x = fmul(p.x, p.zz);
    r.y = fmul(p.y, p.zzz);
    r.z = p.zz;
    return r;
}

GRAPE_HD G1Xyzz jac_to_xyzz(const G1Jac& p) {
    if (p.is_inf()) return G1Xyzz::inf();
    G1Xyzz r;
    r.x = p.x;
    r.y = p.y;
    r.zz = fsqr(p.z);
    r.zzz = fmul(r.zz, p.z);
    return r;
}

// Affine image given the inverse of ZZZ: 1/Z = ZZ/ZZZ, x = X/Z^2, y = Y/ZZZ.
GRAPE_HD G1Affine xyzz_to_affine_with_inv(const G1Xyzz& p, const Fp& zzz_inv) {
    if (p.is_inf()) return G1Affine::inf();
    Fp zinv = fmul(zzz_inv, p.zz);
    G1Affine r;
    r.x = fmul(p.x, fsqr(zinv));
    r.y = fmul(p.y, zzz_inv);
    return r;
}

GRAPE_HD G1Affine xyzz_to_affine(const G1Xyzz& p) {
    if (p.is_inf()) return G1Affine::inf();
    return xyzz_to_affine_with_inv(p, fp_inverse(p.zzz));
}

// Jacobian -> affine: x = X/Z^2, y = Y/Z^3; infinity maps to (0,0)
// (include/curve/jacobian_t.cuh:33-41).
GRAPE_HD G1Affine jac_to_affine(const G1Jac& p) {
    if (p.is_inf()) return G1Affine::inf();
    Fp zi = fp_inverse(p.z);
    Fp zi2 = fsqr(zi);
    G1Affine r;
    r.x = fmul(p.x, zi2);
    r.y = fmul(p.y, fmul(zi2, zi));
    return r;
}

}  // namespace grape
