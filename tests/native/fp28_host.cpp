// Host build of the 28-bit-limb Fp arithmetic (grape_amd/csrc/fp28.hpp) behind a few C entry
// points, so that the CPU test-suite can check it against Python integers and the oracle.
#include <cstring>
#include <vector>
#include "../../grape_amd/csrc/fp28.hpp"
using namespace grape;
static constexpr int FW = FpParams::N;     // 32-bit words of an Fp element in memory
static constexpr size_t FB = 4 * FW;       // bytes

extern "C" {
// canonical memory form (FW x u32) in, canonical out, through the 28-bit domain
void t28_mul(const uint32_t* a, const uint32_t* b, uint32_t* out) {
    Fp x, y;
    memcpy(&x, a, FB);
    memcpy(&y, b, FB);
    Fp r = fp28::to_canonical(fp28::mul(fp28::from_canonical(x), fp28::from_canonical(y)));
    memcpy(out, &r, FB);
}
void t28_sqr(const uint32_t* a, uint32_t* out) {
    Fp x;
    memcpy(&x, a, FB);
    Fp r = fp28::to_canonical(fp28::sqr(fp28::from_canonical(x)));
    memcpy(out, &r, FB);
}
void t28_roundtrip_lazy(const uint32_t* a, uint32_t* out) {
    Fp x;
    memcpy(&x, a, FB);
    Fp r = fp28::to_canonical(fp28::from_canonical_lazy(x));
    memcpy(out, &r, FB);
}
void t28_roundtrip(const uint32_t* a, uint32_t* out) {
    Fp x;
    memcpy(&x, a, FB);
    Fp r = fp28::to_canonical(fp28::from_canonical(x));
    memcpy(out, &r, FB);
}
// (a - b - 2c) * d with lazy subtraction, the pattern of the mixed addition
void t28_lazy(const uint32_t* a, const uint32_t* b, const uint32_t* c, const uint32_t* d, uint32_t* out) {
    Fp xa, xb, xc, xd;
    memcpy(&xa, a, FB); memcpy(&xb, b, FB); memcpy(&xc, c, FB); memcpy(&xd, d, FB);
    Fp28 A = fp28::from_canonical(xa), B = fp28::from_canonical(xb), C = fp28::from_canonical(xc), D = fp28::from_canonical(xd);
    Fp28 t;
    for (int i = 0; i < fp28::N; i++) t.v[i] = A.v[i] - B.v[i] - 2 * C.v[i];
    Fp r = fp28::to_canonical(fp28::mul(fp28::normalize(t), D));
    memcpy(out, &r, FB);
}
int t28_is_zero(const uint32_t* a, int times_p) {
    // a canonical; checks is_zero_mod_p on (a + times_p * p) normalised
    Fp x;
    memcpy(&x, a, FB);
    Fp28 v = fp28::pack(x);
    for (int i = 0; i < fp28::N; i++) v.v[i] += times_p * fp28::P(i);
    return fp28::is_zero_mod_p(fp28::normalize(v)) ? 1 : 0;
}
// sum_i (+-) points[i] through the 28-bit mixed addition; affine points canonical 2 FW x u32;
// returns the number of exceptional steps that had to take the exact path
int t28_sum(const uint32_t* points, const int* negate, int n, uint32_t* out_xyzz) {
    Xyzz28 acc = xyzz28_inf();
    int slow = 0;
    for (int i = 0; i < n; i++) {
        G1Affine p;
        memcpy(&p, points + 2 * FW * i, 2 * FB);
        if (p.is_inf()) continue;
        Affine28 q;
        q.x = fp28::from_canonical(p.x);
        q.y = fp28::from_canonical(p.y);
        if (!xyzz28_madd(acc, q, negate[i] != 0)) {
            G1Xyzz c = xyzz28_to_canonical(acc);
            xyzz_add_affine(c, p, negate[i] != 0);
            acc = xyzz28_from_canonical(c);
            slow++;
        }
    }
    G1Xyzz r = xyzz28_to_canonical(acc);
    memcpy(out_xyzz, &r, 4 * FB);
    return slow;
}
// tree-style sum: partial sums of two halves combined with the accumulator+accumulator addition,
// affine result through the 28-bit inversion
int t28_sum_tree(const uint32_t* points, const int* negate, int n, uint32_t* out_affine) {
    Xyzz28 part[2] = {xyzz28_inf(), xyzz28_inf()};
    int slow = 0;
    for (int i = 0; i < n; i++) {
        G1Affine p;
        memcpy(&p, points + 2 * FW * i, 2 * FB);
        if (p.is_inf()) continue;
        Affine28 q;
        q.x = fp28::from_canonical(p.x);
        q.y = fp28::from_canonical(p.y);
        Xyzz28& acc = part[i & 1];
        if (!xyzz28_madd(acc, q, negate[i] != 0)) {
            G1Xyzz c = xyzz28_to_canonical(acc);
            xyzz_add_affine(c, p, negate[i] != 0);
            acc = xyzz28_from_canonical(c);
            slow++;
        }
    }
    if (!xyzz28_add(part[0], part[1])) {
        G1Xyzz c = xyzz28_to_canonical(part[0]);
        xyzz_add(c, xyzz28_to_canonical(part[1]));
        part[0] = xyzz28_from_canonical(c);
        slow++;
    }
    G1Affine r = xyzz28_to_affine(part[0]);
    memcpy(out_affine, &r, 2 * FB);
    return slow;
}
void t28_inverse(const uint32_t* a, uint32_t* out) {
    Fp x;
    memcpy(&x, a, FB);
    Fp r = fp28::to_canonical(fp28::inverse(fp28::from_canonical(x)));
    memcpy(out, &r, FB);
}
void t28_inverse_by(const uint32_t* a, uint32_t* out) {
    Fp x;
    memcpy(&x, a, FB);
    Fp r = fp28::to_canonical(fp28::inverse_by(fp28::from_canonical(x)));
    memcpy(out, &r, FB);
}
void t28_xyzz_to_affine(const uint32_t* xyzz, uint32_t* out) {
    G1Xyzz a;
    memcpy(&a, xyzz, 4 * FB);
    G1Affine r = xyzz_to_affine(a);
    memcpy(out, &r, 2 * FB);
}
// Horner pattern of the strided-table commitment: acc = points[0]; then for each further point
// `dbl` doublings of the accumulator and one accumulator+accumulator addition; affine result
void t28_horner(const uint32_t* points, int n, int dbl, uint32_t* out_affine) {
    Xyzz28 acc = xyzz28_inf();
    for (int i = 0; i < n; i++) {
        for (int d = 0; d < dbl && i > 0; d++) xyzz28_dbl(acc);
        G1Affine p;
        memcpy(&p, points + 2 * FW * i, 2 * FB);
        Xyzz28 q = xyzz28_inf();
        if (!p.is_inf()) {
            Affine28 a;
            a.x = fp28::from_canonical(p.x);
            a.y = fp28::from_canonical(p.y);
            xyzz28_madd(q, a, false);
        }
        if (!xyzz28_add(acc, q)) {
            G1Xyzz c = xyzz28_to_canonical(acc);
            xyzz_add(c, xyzz28_to_canonical(q));
            acc = xyzz28_from_canonical(c);
        }
    }
    G1Affine r = xyzz28_to_affine(acc);
    memcpy(out_affine, &r, 2 * FB);
}
// The table generator's step: out[k] = pts[k] + base for k < n (pts[k] == base is the doubling), as
// affine additions that share ONE inversion - forward pass of prefix products of the slope
// denominators, one inversion, backward pass.  Canonical affine points in and out (2 FW x u32).
// Returns 1 when the product of the denominators is congruent to zero (no finite affine addition
// for some k; nothing is written then).
int t28_affine_batch(const uint32_t* pts, const int* dbl, int n, const uint32_t* base, uint32_t* out) {
    auto load = [](const uint32_t* src) {
        G1Affine p;
        memcpy(&p, src, 2 * FB);
        Affine28 q;
        q.x = fp28::from_canonical(p.x);
        q.y = fp28::from_canonical(p.y);
        return q;
    };
    const Affine28 f = load(base);
    std::vector<Fp28> pre(n);
    Fp28 acc = fp28::one();
    for (int k = 0; k < n; k++) {
        pre[k] = acc;
        acc = fp28::mul(acc, affine28_slope_den(load(pts + 2 * FW * k), f, dbl[k] != 0));
    }
    if (fp28::is_zero_mod_p(acc)) return 1;
    Fp28 inv = fp28::inverse_by(acc);
    for (int k = n - 1; k >= 0; k--) {
        const Affine28 e = load(pts + 2 * FW * k);
        const Fp28 dinv = fp28::mul(inv, pre[k]);
        inv = fp28::mul(inv, affine28_slope_den(e, f, dbl[k] != 0));
        const Affine28 r = affine28_add_given_inverse(e, f, dbl[k] != 0, dinv);
        // the entry format wants canonical coordinates: check that here, limb by limb
        for (int i = 0; i < fp28::N - 1; i++)
            if (r.x.v[i] < 0 || r.x.v[i] > (int32_t)fp28::MASK || r.y.v[i] < 0 || r.y.v[i] > (int32_t)fp28::MASK) return 2;
        Fp28 dx = fp28::normalize(fp28::sub(r.x, [] { Fp28 p; for (int i = 0; i < fp28::N; i++) p.v[i] = fp28::P(i); return p; }()));
        Fp28 dy = fp28::normalize(fp28::sub(r.y, [] { Fp28 p; for (int i = 0; i < fp28::N; i++) p.v[i] = fp28::P(i); return p; }()));
        if (dx.v[fp28::N - 1] >= 0 || dy.v[fp28::N - 1] >= 0 || r.x.v[fp28::N - 1] < 0 || r.y.v[fp28::N - 1] < 0) return 3;
        G1Affine o;
        o.x = fp28::to_canonical(r.x);
        o.y = fp28::to_canonical(r.y);
        memcpy(out + 2 * FW * k, &o, 2 * FB);
    }
    return 0;
}
}
