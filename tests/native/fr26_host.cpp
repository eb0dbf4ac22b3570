// Host build of the 26-bit-limb lazy Fr arithmetic (grape_amd/csrc/fr26.hpp) behind C entry
// points, for the CPU test-suite.
#include <cstring>
#include "../../grape_amd/csrc/fr26.hpp"
#include "../../grape_amd/csrc/divstep.hpp"
using namespace grape;

static Fr ld(const uint32_t* p) { Fr x; memcpy(&x, p, 32); return x; }
static void st(uint32_t* p, const Fr& x) { memcpy(p, &x, 32); }

extern "C" {
// 1/a by divsteps and by the a^(r-2) ladder, memory form in and out
void t26_inverse_by(const uint32_t* a, uint32_t* out) { st(out, divstep::inverse_by(ld(a))); }
void t26_inverse_ladder(const uint32_t* a, uint32_t* out) { st(out, inverse(ld(a))); }
void t26_mulc(const uint32_t* a, const uint32_t* b, uint32_t* out) { st(out, fr26::mulc(ld(a), ld(b))); }
void t26_from_mont(const uint32_t* a, uint32_t* out) { st(out, fr26::from_montc(ld(a))); }
void t26_to_mont(const uint32_t* a, uint32_t* out) { st(out, fr26::to_montc(ld(a))); }
void t26_from_i32(int32_t x, uint32_t* out) { st(out, fr26::from_i32c(x)); }
void t26_from_u32(uint32_t x, uint32_t* out) { st(out, fr26::from_u32c(x)); }
// sum_i (a1_i - a0_i) * (b1_i - b0_i) + a0_i * b1_i  over n terms (n <= 16), signed lazy operands
void t26_lazy_sum(const uint32_t* a0, const uint32_t* a1, const uint32_t* b0, const uint32_t* b1, int n, uint32_t* out) {
    fr26::Acc C;
    fr26::acc_zero(C);
    for (int i = 0; i < n; i++) {
        fr26::Limbs A0 = fr26::pack(ld(a0 + 8 * i)), A1 = fr26::pack(ld(a1 + 8 * i));
        fr26::Limbs B0 = fr26::pack(ld(b0 + 8 * i)), B1 = fr26::pack(ld(b1 + 8 * i));
        fr26::mac(C, fr26::sub(A1, A0), fr26::sub(B1, B0));
        fr26::mac(C, A0, B1);
    }
    st(out, fr26::finish_sum(C, 2));     // |V| < 32 r^2 -> (-0.91 r, 1.91 r) + 2r
}
// sum_h w_h * t_h over n <= 64 terms with the weights carrying the radix factor (fold pattern)
void t26_weighted_sum(const uint32_t* w, const uint32_t* t, int n, uint32_t* out) {
    fr26::Acc C;
    fr26::acc_zero(C);
    for (int i = 0; i < n; i++) fr26::mac(C, fr26::weight16(ld(w + 8 * i)), fr26::pack(ld(t + 8 * i)));
    st(out, fr26::unpack(fr26::canon(fr26::reduce(C, 0), 2)));   // 64/35.3 + 1 = 2.82 r
}
// the same over n <= 64*S terms, every S-th term into one of S accumulators whose reduced values
// are added limb-wise and canonicalised by quotient estimate (split fold pattern)
void t26_weighted_sum_split(const uint32_t* w, const uint32_t* t, int n, int S, uint32_t* out) {
    fr26::Limbs r;
    for (int k = 0; k < fr26::N; k++) r.v[k] = 0;
    for (int q = 0; q < S; q++) {
        fr26::Acc C;
        fr26::acc_zero(C);
        for (int i = q; i < n; i += S) fr26::mac(C, fr26::weight16(ld(w + 8 * i)), fr26::pack(ld(t + 8 * i)));
        r = fr26::add(r, fr26::reduce(C, 0));
    }
    st(out, fr26::unpack(fr26::canon_wide(fr26::normalize(r))));
}
// k * a + b for canonical a, b and 0 <= k < 31, through canon_wide
void t26_canon_wide(const uint32_t* a, const uint32_t* b, int k, uint32_t* out) {
    fr26::Limbs A = fr26::pack(ld(a)), B = fr26::pack(ld(b)), r;
    for (int i = 0; i < fr26::N; i++) r.v[i] = k * A.v[i] + B.v[i];
    st(out, fr26::unpack(fr26::canon_wide(fr26::normalize(r))));
}
// lo + v * (hi - lo) through the single-product fold (v, lo, hi canonical; hi may be absent = zero)
void t26_fold1(const uint32_t* v, const uint32_t* lo, const uint32_t* hi, uint32_t* out) {
    const fr26::Limbs l = fr26::pack(ld(lo));
    st(out, fr26::fold1(fr26::weight16(ld(v)), l, fr26::sub(fr26::pack(ld(hi)), l)));
}
// the ten constants of the table fold for a challenge v, and lo + v * (hi - lo) through them
void t26_fold_table(const uint32_t* v, int32_t* tab) { fr26::fold_table(tab, ld(v)); }
void t26_foldt(const int32_t* tab, const uint32_t* lo, const uint32_t* hi, uint32_t* out) {
    const fr26::Limbs l = fr26::pack(ld(lo));
    st(out, fr26::foldt(tab, l, fr26::sub(fr26::pack(ld(hi)), l)));
}
// k * a + b for canonical a, b and 0 <= k <= 3 with k*a + b < 4r, through canon4_unpack
void t26_canon4(const uint32_t* a, const uint32_t* b, int k, uint32_t* out) {
    fr26::Limbs A = fr26::pack(ld(a)), B = fr26::pack(ld(b)), r;
    for (int i = 0; i < fr26::N; i++) r.v[i] = k * A.v[i] + B.v[i];
    st(out, fr26::canon4_unpack(fr26::normalize(r)));
}
}
