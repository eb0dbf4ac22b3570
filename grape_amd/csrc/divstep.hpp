// Modular inversion by divsteps (Bernstein-Yang "safegcd"), batched 30 steps at a time on signed
// 30-bit limbs: the pieces shared by the base field's 28-bit form (fp28.hpp) and the memory form
// of either field (inverse_by below).  A 255-bit modulus takes at most 741 divsteps (25 batches of
// a few hundred instructions), a 381-bit one 1110 - an order of magnitude fewer sequential
// instructions than the a^(m-2) ladder, which matters wherever one inversion is a latency chain
// (the row epilogue of a commitment, the top level of a batched inversion).  The reference inverts
// with the same family of algorithm (include/field/mont_t.cuh:1058-1120, ct_inverse_mod_x).
#pragma once
#include "field.hpp"

namespace grape {
namespace divstep {

constexpr int32_t M30 = (1 << 30) - 1;

struct Mat { int32_t u, v, q, r; };

// 30 divsteps on the low words; returns the transition matrix scaled by 2^30:
//   u*f + v*g = 2^30 * f',   q*f + r*g = 2^30 * g'
GRAPE_HD int32_t divsteps30(int32_t delta, uint32_t f, uint32_t g, Mat& t) {
    int32_t u = 1, v = 0, q = 0, r = 1;
    for (int i = 0; i < 30; i++) {
        const bool swap = (delta > 0) & ((g & 1u) != 0);
        // (f, g) <- (g, -f), rows of the matrix alike, delta <- -delta
        const uint32_t nf = swap ? g : f;
        const uint32_t ng = swap ? (0u - f) : g;
        const int32_t nu = swap ? q : u, nv = swap ? r : v;
        const int32_t nq = swap ? -u : q, nr = swap ? -v : r;
        delta = swap ? -delta : delta;
        f = nf; g = ng; u = nu; v = nv; q = nq; r = nr;
        // make g even
        const bool odd = (g & 1u) != 0;
        g += odd ? f : 0u;
        q += odd ? u : 0;
        r += odd ? v : 0;
        delta += 1;
        g >>= 1;
        u <<= 1;
        v <<= 1;
    }
    t.u = u; t.v = v; t.q = q; t.r = r;
    return delta;
}

// (f, g) <- t * (f, g) / 2^30, exact
template <int L>
GRAPE_HD void update_fg(int32_t* f, int32_t* g, const Mat& t) {
    int64_t cf = (int64_t)t.u * f[0] + (int64_t)t.v * g[0];
    int64_t cg = (int64_t)t.q * f[0] + (int64_t)t.r * g[0];
    cf >>= 30;   // the low 30 bits are zero by construction
    cg >>= 30;
#pragma unroll
    for (int i = 1; i < L; i++) {
        cf += (int64_t)t.u * f[i] + (int64_t)t.v * g[i];
        cg += (int64_t)t.q * f[i] + (int64_t)t.r * g[i];
        f[i - 1] = (int32_t)cf & M30;
        g[i - 1] = (int32_t)cg & M30;
        cf >>= 30;
        cg >>= 30;
    }
    f[L - 1] = (int32_t)cf;
    g[L - 1] = (int32_t)cg;
}

// (d, e) <- t * (d, e) / 2^30 mod m, keeping both in (-2m, m).  M::limb(i): the modulus in 30-bit
// limbs; M::INV30: m^-1 mod 2^30.
template <int L, class M>
GRAPE_HD void update_de(int32_t* d, int32_t* e, const Mat& t) {
    const int32_t sd = d[L - 1] >> 31, se = e[L - 1] >> 31;   // all-ones when negative
    // a negative d (e) is replaced by d + m (e + m): that adds u*m (v*m) to the first row
    int32_t md = (t.u & sd) + (t.v & se);
    int32_t me = (t.q & sd) + (t.r & se);
    int64_t cd = (int64_t)t.u * d[0] + (int64_t)t.v * e[0];
    int64_t ce = (int64_t)t.q * d[0] + (int64_t)t.r * e[0];
    // choose the multiple of m that clears the low 30 bits
    md -= (int32_t)((M::INV30 * (uint32_t)cd + (uint32_t)md) & (uint32_t)M30);
    me -= (int32_t)((M::INV30 * (uint32_t)ce + (uint32_t)me) & (uint32_t)M30);
    cd += (int64_t)M::limb(0) * md;
    ce += (int64_t)M::limb(0) * me;
    cd >>= 30;
    ce >>= 30;
#pragma unroll
    for (int i = 1; i < L; i++) {
        cd += (int64_t)t.u * d[i] + (int64_t)t.v * e[i] + (int64_t)M::limb(i) * md;
        ce += (int64_t)t.q * d[i] + (int64_t)t.r * e[i] + (int64_t)M::limb(i) * me;
        d[i - 1] = (int32_t)cd & M30;
        e[i - 1] = (int32_t)ce & M30;
        cd >>= 30;
        ce >>= 30;
    }
    d[L - 1] = (int32_t)cd;
    e[L - 1] = (int32_t)ce;
}

// floor((49 b + 57) / 17) divsteps always suffice for b-bit inputs (Bernstein-Yang, b >= 46), taken 30 at a time
constexpr int batches_for_bits(int bits) { return ((49 * bits + 57) / 17 + 29) / 30; }

// the modulus of Mont<P> in 30-bit limbs, read off its 32-bit words
template <class P>
struct ModOf {
    static constexpr int L = (32 * P::N + 29) / 30;
    static constexpr uint32_t INV30 = (0u - P::M0) & (uint32_t)M30;     // P::M0 = -m^-1 mod 2^32
    static GRAPE_HD int32_t limb(int k) {
        const int bit = 30 * k, i0 = bit >> 5, sh = bit & 31;
        uint64_t w = (uint64_t)P::mod(i0) >> sh;
        if (i0 + 1 < P::N) w |= (uint64_t)P::mod(i0 + 1) << (32 - sh);
        return (int32_t)(w & (uint64_t)M30);
    }
};

// 1/a for a value in memory form (Montgomery, canonical in [0, m)); 0 for a = 0, which is the
// reference's convention.
template <class P>
GRAPE_HD Mont<P> inverse_by(const Mont<P>& a) {
    using M = ModOf<P>;
    constexpr int L = M::L, N = P::N;
    int32_t f[L], g[L], d[L], e[L];
#pragma unroll
    for (int k = 0; k < L; k++) {
        const int bit = 30 * k, i0 = bit >> 5, sh = bit & 31;
        uint64_t w = (uint64_t)a.v[i0] >> sh;
        if (i0 + 1 < N) w |= (uint64_t)a.v[i0 + 1] << (32 - sh);
        g[k] = (int32_t)(w & (uint64_t)M30);
        f[k] = M::limb(k);
        d[k] = 0;
        e[k] = 0;
    }
    e[0] = 1;
    int32_t delta = 1;
    for (int batch = 0; batch < batches_for_bits(32 * N); batch++) {
        uint32_t gz = 0;
#pragma unroll
        for (int k = 0; k < L; k++) gz |= (uint32_t)g[k];
        if (gz == 0) break;
        Mat m;
        delta = divsteps30(delta, (uint32_t)f[0] | ((uint32_t)f[1] << 30), (uint32_t)g[0] | ((uint32_t)g[1] << 30), m);
        update_de<L, M>(d, e, m);
        update_fg<L>(f, g, m);
    }
    // now g = 0, f = +-1 (f = m and d = 0 when a was 0) and d * a = f (mod m): the inverse is d * f.
    // d in (-2m, m): add m when negative, negate when f = -1, add m again when negative -> [0, m)
    const int32_t fneg = f[L - 1] >> 31;
    int32_t x[L];
    int32_t neg = d[L - 1] >> 31;
#pragma unroll
    for (int k = 0; k < L; k++) {
        const int32_t t = d[k] + (M::limb(k) & neg);
        x[k] = (t ^ fneg) - fneg;
    }
#pragma unroll
    for (int k = 0; k < L - 1; k++) {
        x[k + 1] += x[k] >> 30;
        x[k] &= M30;
    }
    neg = x[L - 1] >> 31;
#pragma unroll
    for (int k = 0; k < L; k++) x[k] += M::limb(k) & neg;
#pragma unroll
    for (int k = 0; k < L - 1; k++) {
        x[k + 1] += x[k] >> 30;
        x[k] &= M30;
    }
    // 30-bit limbs -> 32-bit words: the plain inverse of a value that carried the factor R, i.e. a^-1 R^-1
    Mont<P> r;
#pragma unroll
    for (int i = 0; i < N; i++) {
        const int bit = 32 * i, k0 = bit / 30, sh = bit % 30;
        uint64_t w = (uint64_t)(uint32_t)x[k0] >> sh;
        if (k0 + 1 < L) w |= (uint64_t)(uint32_t)x[k0 + 1] << (30 - sh);
        if (k0 + 2 < L && 60 - sh < 32) w |= (uint64_t)(uint32_t)x[k0 + 2] << (60 - sh);
        r.v[i] = (uint32_t)w;
    }
    // times R^3 (one Montgomery product takes a factor R off): a^-1 R, the memory form of 1/a
    Mont<P> rr;
#pragma unroll
    for (int i = 0; i < N; i++) rr.v[i] = P::rr(i);
    return mul(r, mul(rr, rr));
}

}  // namespace divstep
}  // namespace grape
