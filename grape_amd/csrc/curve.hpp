// BLS12-381 G1 (y^2 = x^3 + 4 over Fp) group law on Montgomery-form coordinates.
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
    Fp P = sub(mul(p.x, acc.zz), acc.x);   // U2 - X1
    Fp R = sub(mul(py, acc.zzz), acc.y);   // S2 - Y1
    if (!P.is_zero()) {
        Fp PP = sqr(P);
        Fp PPP = mul(P, PP);
        Fp Q = mul(acc.x, PP);
        Fp X3 = sub(sub(sub(sqr(R), PPP), Q), Q);
        Fp Y3 = sub(mul(R, sub(Q, X3)), mul(acc.y, PPP));
        acc.zz = mul(acc.zz, PP);
        acc.zzz = mul(acc.zzz, PPP);
        acc.x = X3;
        acc.y = Y3;
    } else if (R.is_zero()) {
        // same point: double the affine operand
        Fp U = dbl(py);
        Fp V = sqr(U);
        Fp W = mul(U, V);
        Fp S = mul(p.x, V);
        Fp M = sqr(p.x);
        M = add(add(M, M), M);
        Fp X3 = sub(sub(sqr(M), S), S);
        Fp Y3 = sub(mul(M, sub(S, X3)), mul(W, py));
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
    Fp V = sqr(U);
    Fp W = mul(U, V);
    Fp S = mul(acc.x, V);
    Fp M = sqr(acc.x);
    M = add(add(M, M), M);
    Fp X3 = sub(sub(sqr(M), S), S);
    Fp Y3 = sub(mul(M, sub(S, X3)), mul(W, acc.y));
    acc.x = X3;
    acc.y = Y3;
    acc.zz = mul(V, acc.zz);
    acc.zzz = mul(W, acc.zzz);
}

// acc += q, both XYZZ. 12M + 2S on the common path.
GRAPE_HD void xyzz_add(G1Xyzz& acc, const G1Xyzz& q) {
    if (q.is_inf()) return;
    if (acc.is_inf()) {
        acc = q;
        return;
    }
    Fp U1 = mul(acc.x, q.zz);
    Fp S1 = mul(acc.y, q.zzz);
    Fp P = sub(mul(q.x, acc.zz), U1);
    Fp R = sub(mul(q.y, acc.zzz), S1);
    if (!P.is_zero()) {
        Fp PP = sqr(P);
        Fp PPP = mul(P, PP);
        Fp Q = mul(U1, PP);
        Fp X3 = sub(sub(sub(sqr(R), PPP), Q), Q);
        Fp Y3 = sub(mul(R, sub(Q, X3)), mul(S1, PPP));
        acc.zz = mul(mul(acc.zz, q.zz), PP);
        acc.zzz = mul(mul(acc.zzz, q.zzz), PPP);
        acc.x = X3;
        acc.y = Y3;
    } else if (R.is_zero()) {
        xyzz_dbl(acc);
    } else {
        acc = G1Xyzz::inf();
    }
}

// XYZZ -> Jacobian without inversion: (X*ZZ, Y*ZZZ, Z) with Z := ZZZ/ZZ is not available
// division-free, but (X*ZZ^2... ) is not needed: the triple (X*ZZ, Y*ZZZ, ZZ) satisfies
// x = X*ZZ/ZZ^2, y = Y*ZZZ/ZZ^3 because ZZZ^2 = ZZ^3.
GRAPE_HD G1Jac xyzz_to_jac(const G1Xyzz& p) {
    if (p.is_inf()) return G1Jac::inf();
    G1Jac r;
    r.x = mul(p.x, p.zz);
    r.y = mul(p.y, p.zzz);
    r.z = p.zz;
    return r;
}

GRAPE_HD G1Xyzz jac_to_xyzz(const G1Jac& p) {
    if (p.is_inf()) return G1Xyzz::inf();
    G1Xyzz r;
    r.x = p.x;
    r.y = p.y;
    r.zz = sqr(p.z);
    r.zzz = mul(r.zz, p.z);
    return r;
}

// Affine image given the inverse of ZZZ: 1/Z = ZZ/ZZZ, x = X/Z^2, y = Y/ZZZ.
GRAPE_HD G1Affine xyzz_to_affine_with_inv(const G1Xyzz& p, const Fp& zzz_inv) {
    if (p.is_inf()) return G1Affine::inf();
    Fp zinv = mul(zzz_inv, p.zz);
    G1Affine r;
    r.x = mul(p.x, sqr(zinv));
    r.y = mul(p.y, zzz_inv);
    return r;
}

GRAPE_HD G1Affine xyzz_to_affine(const G1Xyzz& p) {
    if (p.is_inf()) return G1Affine::inf();
    return xyzz_to_affine_with_inv(p, inverse(p.zzz));
}

// Jacobian -> affine: x = X/Z^2, y = Y/Z^3; infinity maps to (0,0)
// (include/curve/jacobian_t.cuh:33-41).
GRAPE_HD G1Affine jac_to_affine(const G1Jac& p) {
    if (p.is_inf()) return G1Affine::inf();
    Fp zi = inverse(p.z);
    Fp zi2 = sqr(zi);
    G1Affine r;
    r.x = mul(p.x, zi2);
    r.y = mul(p.y, mul(zi2, zi));
    return r;
}

}  // namespace grape
