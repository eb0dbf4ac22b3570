// Fr (BLS12-381 or BN254, both r = 1 mod 2^26) on 10 signed limbs of 26 bits with lazy accumulation - the working form of the
// streaming Fr kernels (fold, sumcheck rounds, logUp rounds, element-wise products).
//
// Tensors stay in memory in the reference's format (8 x 32-bit limbs, canonical Montgomery
// residue x*2^256 mod r, include/field/mont_t.cuh:33); a kernel re-limbs an element on load
// (two instructions per limb) and multiplies in 26-bit limbs, where a limb product is < 2^52 and
// a 64-bit column accumulator absorbs hundreds of them: a product costs 100 multiply-adds, a SUM
// of products costs one Montgomery reduction in total, and differences are limb-wise.
// On gfx950 a 32x32+64 multiply-add issues at full rate, so this turns the fold / round kernels
// from instruction-bound (about 600 instructions per saturated 32-bit product) into HBM-bound.
//
// Radix bookkeeping.  The working Montgomery radix is 2^260, the memory radix 2^256:
//   reduce(a*b) = a*b / 2^260.  With a = x*2^256 and b = y*2^256 (memory form) that is
//   (x*y*2^256) / 16, so one operand carries an extra factor 16 (limbs times 16, or the constant
//   X16 applied to a finished sum) and the result is again the memory form of x*y.
#pragma once
#include "field.hpp"

namespace grape {
namespace fr26 {

constexpr int N = 10;
constexpr int W = 26;
constexpr uint32_t MASK = (1u << W) - 1;

struct Limbs {
    int32_t v[N];
};
struct Acc {            // columns of a double-width sum of limb products
    int64_t c[2 * N];
};

// The bounds quoted below (r/2^260 = 1/35.3) are those of BLS12-381; BN254's r is smaller
// (r/2^260 = 1/84.6), so every bound holds there with more room.
#if defined(GRAPE_CURVE_BN254)
GRAPE_HD int32_t R(int i) {   // the modulus r; R(0) = 1 and -r^-1 mod 2^26 = -1
    constexpr int32_t t[10] = {0x0000001, 0x07d64fc, 0x309143e, 0x121e6e5, 0x12833e8,
                               0x0605617, 0x1045b68, 0x280a6e1, 0x272e131, 0x00c1913};
    return t[i];
}
GRAPE_HD int32_t X16(int i) {   // 16 * 2^260 mod r: reduce(t * X16) = 16 t
    constexpr int32_t t[10] = {0x3fffab6, 0x0c7e327, 0x1faef6e, 0x2b0c4ca, 0x15d7570,
                               0x278a8d2, 0x2f48b70, 0x38d5c9d, 0x064ef86, 0x0035e45};
    return t[i];
}
GRAPE_HD int32_t C516(int i) {   // 2^516 mod r: reduce(x * C516) = x * 2^256 (into memory form)
    constexpr int32_t t[10] = {0x216da70, 0x39916b8, 0x1e31bb8, 0x078d716, 0x13fe3ab,
                               0x2ee0215, 0x1833d53, 0x1296312, 0x317f4e4, 0x0085b42};
    return t[i];
}

#else
GRAPE_HD int32_t R(int i) {   // the modulus r; R(0) = 1 and -r^-1 mod 2^26 = -1
    constexpr int32_t t[10] = {0x0000001, 0x3ffffc0, 0x1bfefff, 0x00bfff9, 0x153bda4,
                               0x2687601, 0x39d8080, 0x1f520cc, 0x353299d, 0x01cfb69};
    return t[i];
}
GRAPE_HD int32_t X16(int i) {   // 16 * 2^260 mod r: reduce(t * X16) = 16 t
    constexpr int32_t t[10] = {0x3fffdcb, 0x0008d3f, 0x3635000, 0x1840e7b, 0x22e7505,
                               0x3738f0f, 0x163642b, 0x1fe9bc5, 0x175276a, 0x0091f6d};
    return t[i];
}
GRAPE_HD int32_t C516(int i) {   // 2^516 mod r: reduce(x * C516) = x * 2^256 (into memory form)
    constexpr int32_t t[10] = {0x329c6cf, 0x3a6440f, 0x263d999, 0x2d5e49d, 0x1631138,
                               0x2e8703b, 0x37715f1, 0x1cf20a7, 0x246cc02, 0x00027fd};
    return t[i];
}

#endif

// 8 x 32-bit canonical -> 10 x 26-bit, non-negative
GRAPE_HD Limbs pack(const Fr& x) {
    Limbs r;
#pragma unroll
    for (int k = 0; k < N; k++) {
        const int bit = W * k, q = bit >> 5, s = bit & 31;
        uint64_t two = (uint64_t)x.v[q] | ((q + 1 < 8) ? ((uint64_t)x.v[q + 1] << 32) : 0);
        r.v[k] = (int32_t)((uint32_t)(two >> s) & MASK);
    }
    return r;
}
// the same with every limb times 16 (the radix correction factor)
GRAPE_HD Limbs pack16(const Fr& x) {
    Limbs r = pack(x);
#pragma unroll
    for (int k = 0; k < N; k++) r.v[k] <<= 4;
    return r;
}
// normalised non-negative limbs below 2^256 -> 8 x 32-bit
GRAPE_HD Fr unpack(const Limbs& a) {
    Fr r;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const int k0 = (32 * q) / W;
        uint64_t acc = 0;
#pragma unroll
        for (int t = 0; t < 3; t++) {
            const int k = k0 + t;
            if (k < N) {
                const int sh = W * k - 32 * q;
                if (sh >= 0) {
                    if (sh < 32) acc |= (uint64_t)(uint32_t)a.v[k] << sh;
                } else {
                    acc |= (uint64_t)(uint32_t)a.v[k] >> (-sh);
                }
            }
        }
        r.v[q] = (uint32_t)acc;
    }
    return r;
}

GRAPE_HD Limbs sub(const Limbs& a, const Limbs& b) {
    Limbs r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = a.v[i] - b.v[i];
    return r;
}
GRAPE_HD Limbs add(const Limbs& a, const Limbs& b) {
    Limbs r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = a.v[i] + b.v[i];
    return r;
}
GRAPE_HD Limbs normalize(const Limbs& a) {
    Limbs r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < N - 1; i++) {
        int32_t t = a.v[i] + c;
        r.v[i] = t & (int32_t)MASK;
        c = t >> W;
    }
    r.v[N - 1] = a.v[N - 1] + c;
    return r;
}

GRAPE_HD void acc_zero(Acc& C) {
#pragma unroll
    for (int k = 0; k < 2 * N; k++) C.c[k] = 0;
}
// C += a * b (100 multiply-adds).  The caller keeps |column| < 2^63: each call adds at most
// 10 * max|a limb| * max|b limb| to a column.
GRAPE_HD void mac(Acc& C, const Limbs& a, const Limbs& b) {
#pragma unroll
    for (int i = 0; i < N; i++) {
#pragma unroll
        for (int j = 0; j < N; j++) C.c[i + j] += (int64_t)a.v[i] * (int64_t)b.v[j];
    }
}
// Montgomery reduction of a column sum V: returns (V + M*r)/2^260 + add_r*r with 0 <= M < 2^260,
// limbs 0..8 normalised, top limb signed.  For |V| < B*r^2 the value lies in
// (add_r - B/35.3)*r .. (add_r + 1 + B/35.3)*r   (r/2^260 = 2^-5.143 = 1/35.3).
GRAPE_HD Limbs reduce(Acc& C, int add_r) {
#pragma unroll
    for (int i = 0; i < N; i++) {
        const int32_t m = (int32_t)((0u - (uint32_t)C.c[i]) & MASK);   // -r^-1 = -1 mod 2^26
        C.c[i] += (int64_t)m;                                          // m * R(0), R(0) = 1
#pragma unroll
        for (int j = 1; j < N; j++) C.c[i + j] += (int64_t)m * (int64_t)R(j);
        C.c[i + 1] += C.c[i] >> W;
    }
    Limbs r;
    int64_t c = 0;
#pragma unroll
    for (int k = 0; k < N - 1; k++) {
        int64_t t = C.c[N + k] + (int64_t)add_r * (int64_t)R(k) + c;
        r.v[k] = (int32_t)((uint32_t)t & MASK);
        c = t >> W;
    }
    r.v[N - 1] = (int32_t)(C.c[2 * N - 1] + (int64_t)add_r * (int64_t)R(N - 1) + c);
    return r;
}
// subtract r up to `times` times while the value stays non-negative: [0, (times+1) r) -> [0, r)
GRAPE_HD Limbs canon(Limbs t, int times) {
    for (int rep = 0; rep < times; rep++) {
        Limbs d;
#pragma unroll
        for (int i = 0; i < N; i++) d.v[i] = t.v[i] - R(i);
        d = normalize(d);
        const bool ok = d.v[N - 1] >= 0;
#pragma unroll
        for (int i = 0; i < N; i++) t.v[i] = ok ? d.v[i] : t.v[i];
    }
    return t;
}
// non-negative value below 32 r with limbs 0..8 normalised -> [0, r).  The quotient estimate
// from the top limb (r = R(9) * 2^234 + ...) is the true quotient or one less.
GRAPE_HD Limbs canon_wide(const Limbs& t) {
    const int32_t q = t.v[N - 1] / (R(N - 1) + 1);
    Limbs d;
#pragma unroll
    for (int i = 0; i < N; i++) d.v[i] = t.v[i] - q * R(i);
    return canon(normalize(d), 1);
}

// limb-wise sum of at most 16 packed elements or differences of packed elements (|limb| < 2^30,
// value within (-add_r * r, (32 - add_r) * r)) -> canonical element of memory form
GRAPE_HD Fr limb_sum_to_fr(const Limbs& s, int add_r) {
    Limbs d;
#pragma unroll
    for (int i = 0; i < N; i++) d.v[i] = s.v[i] + add_r * R(i);
    return unpack(canon_wide(normalize(d)));
}

// canonical product of two memory-form elements (memory form out): 16ab < 16 r^2 -> (0, 1.46r)
GRAPE_HD Fr mulc(const Fr& a, const Fr& b) {
    Acc C;
    acc_zero(C);
    mac(C, pack16(a), pack(b));
    return unpack(canon(reduce(C, 0), 1));
}
// a finished column sum of memory-form products (value/2^260 within (-lo_r, hi_r) multiples of
// r, lo_r + hi_r + 1 <= 34) -> canonical memory form of the sum of products
GRAPE_HD Fr finish_sum(Acc& C, int lo_r) {
    Limbs t = reduce(C, lo_r);          // in (0, 34 r)
    Limbs x;
#pragma unroll
    for (int i = 0; i < N; i++) x.v[i] = X16(i);
    Acc D;
    acc_zero(D);
    mac(D, t, x);                        // < 34 r^2 -> (0, 1.97 r)
    return unpack(canon(reduce(D, 0), 1));
}
// leave / enter memory (Montgomery) form
GRAPE_HD Fr from_montc(const Fr& a) {    // x*2^256 -> x: reduce(16 * a) = a / 2^256
    Acc C;
    acc_zero(C);
    const Limbs p = pack16(a);
#pragma unroll
    for (int i = 0; i < N; i++) C.c[i] = p.v[i];
    return unpack(canon(reduce(C, 0), 1));
}
GRAPE_HD Fr to_montc(const Fr& a) {      // x -> x*2^256
    Acc C;
    acc_zero(C);
    Limbs k;
#pragma unroll
    for (int i = 0; i < N; i++) k.v[i] = C516(i);
    mac(C, pack(a), k);                  // < r^2 -> (0, 1.03 r)
    return unpack(canon(reduce(C, 0), 1));
}
// small integer -> memory form; negatives as r - |x|
GRAPE_HD Fr from_i32c(int32_t x) {
    const uint32_t ax = x < 0 ? 0u - (uint32_t)x : (uint32_t)x;
    Acc C;
    acc_zero(C);
    const int32_t l0 = (int32_t)(ax & MASK), l1 = (int32_t)(ax >> W);
#pragma unroll
    for (int j = 0; j < N; j++) {
        C.c[j] += (int64_t)l0 * (int64_t)C516(j);
        C.c[j + 1] += (int64_t)l1 * (int64_t)C516(j);
    }
    Limbs t = canon(reduce(C, 0), 1);
    // negate: r - t unless t = 0
    uint32_t nz = 0;
#pragma unroll
    for (int i = 0; i < N; i++) nz |= (uint32_t)t.v[i];
    if (x < 0 && nz != 0) {
        Limbs d;
#pragma unroll
        for (int i = 0; i < N; i++) d.v[i] = R(i) - t.v[i];
        t = normalize(d);
    }
    return unpack(t);
}
GRAPE_HD Fr from_u32c(uint32_t ax) {
    Acc C;
    acc_zero(C);
    const int32_t l0 = (int32_t)(ax & MASK), l1 = (int32_t)(ax >> W);
#pragma unroll
    for (int j = 0; j < N; j++) {
        C.c[j] += (int64_t)l0 * (int64_t)C516(j);
        C.c[j + 1] += (int64_t)l1 * (int64_t)C516(j);
    }
    return unpack(canon(reduce(C, 0), 1));
}

// 16 * w mod r as normalised limbs (below 2^26) for a canonical element w: four modular
// doublings.  Use this (not pack16) for an operand that enters many accumulated products.
GRAPE_HD Limbs weight16(const Fr& w) {
    Fr t = grape::add(w, w);
    t = grape::add(t, t);
    t = grape::add(t, t);
    t = grape::add(t, t);
    return pack(t);
}

// Working limbs of a value in [0, 4r) (limbs 0..8 normalised, top limb non-negative) -> canonical
// memory form: nine 32-bit words, then a conditional subtraction of 2r and one of r on borrow chains
// (one instruction per word; the same step on 26-bit limbs costs three times as much).
GRAPE_HD Fr canon4_unpack(const Limbs& t) {
    uint32_t w[9];
    const Fr lo = unpack(t);                       // bits 0..255
#pragma unroll
    for (int i = 0; i < 8; i++) w[i] = lo.v[i];
    w[8] = (uint32_t)t.v[N - 1] >> (256 - W * (N - 1));   // bits 256 and up
#pragma unroll
    for (int rep = 0; rep < 2; rep++) {
        // rep 0 subtracts 2r (its ninth word is the bit shifted out of the top word of r), rep 1 subtracts r
        uint32_t d[9];
        uint32_t borrow = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t m = rep == 0 ? ((FrParams::mod(i) << 1) | (i ? FrParams::mod(i - 1) >> 31 : 0u)) : FrParams::mod(i);
            d[i] = detail::sbb32(w[i], m, borrow);
        }
        d[8] = detail::sbb32(w[8], rep == 0 ? FrParams::mod(7) >> 31 : 0u, borrow);
        const bool below = borrow != 0;            // w < 2r resp. r: keep w
#pragma unroll
        for (int i = 0; i < 9; i++) w[i] = below ? w[i] : d[i];
    }
    Fr r;
#pragma unroll
    for (int i = 0; i < 8; i++) r.v[i] = w[i];
    return r;
}

// lo + v * (hi - lo) in canonical memory form with w1 = weight16(v) and d = hi - lo as signed
// limbs: ONE limb product.  lo enters the accumulator as lo * 2^260 (its limbs are the starting
// values of columns N..2N-1), so the reduction returns v*d + lo directly: |w1 * d| < r^2 and
// 0 <= lo < r put the result, with one r added, in (0.97 r, 3.03 r).
GRAPE_HD Fr fold1(const Limbs& w1, const Limbs& lo, const Limbs& d) {
    Acc F;
#pragma unroll
    for (int i = 0; i < N; i++) {
        F.c[i] = 0;
        F.c[N + i] = (int64_t)(uint32_t)lo.v[i];
    }
    mac(F, w1, d);
    return canon4_unpack(reduce(F, 1));
}


// ---- fold by a challenge that every lane shares: multiplication and reduction in one table
// lo + v * d needs a product by the SAME v for every element of a round, so the reduction can be
// folded into the multiplier: with W_j = v * 2^(26 j + 52) mod r (ten canonical constants per
// challenge, made once by fold_table), sum_j d_j W_j = v * d * 2^52 (mod r) is a 10 x 10 limb
// product whose value stays below 10 * 2^26 r, and TWO Montgomery steps (dividing by 2^52) bring it
// to within 2^-22 r of [0, r) - against ten steps for a general product.  118 multiply-adds per
// fold instead of 190, and a third of the carry handling.
constexpr int kFoldTableWords = N * N;
// tab[j * N + k] = limb k of v * 2^(26 j + 52) mod r for the memory-form challenge v_mem
GRAPE_HD void fold_table(int32_t* tab, const Fr& v_mem) {
    Fr p52 = Fr::zero(), p26 = Fr::zero();
    p52.v[1] = 1u << 20;                      // the integer 2^52
    p26.v[0] = 1u << 26;                      // the integer 2^26
    const Fr step = to_montc(p26);            // mulc(x, step) = x * 2^26
    Fr w = mulc(v_mem, p52);                  // v_mem * 2^52 / 2^256 = v * 2^52
    for (int j = 0; j < N; j++) {
        const Limbs l = pack(w);
#pragma unroll
        for (int k = 0; k < N; k++) tab[j * N + k] = l.v[k];
        w = mulc(w, step);
    }
}
// Two Montgomery steps and the carry chain that finish a table fold: c holds lo * 2^52 + sum_j d_j W_j
// in twelve columns; returns lo + v * d in canonical memory form (the value before the last step lies
// in (0.99 r, 3.01 r)).
GRAPE_HD Fr foldt_finish(int64_t* c) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int32_t m = (int32_t)((0u - (uint32_t)c[i]) & MASK);
        c[i] += (int64_t)m;
#pragma unroll
        for (int j = 1; j < N; j++) c[i + j] += (int64_t)m * (int64_t)R(j);
        c[i + 1] += c[i] >> W;
    }
    Limbs r;
    int64_t carry = 0;
#pragma unroll
    for (int k = 0; k < N - 1; k++) {
        const int64_t t = c[2 + k] + (int64_t)R(k) + carry;                 // + one r
        r.v[k] = (int32_t)((uint32_t)t & MASK);
        carry = t >> W;
    }
    r.v[N - 1] = (int32_t)(c[N + 1] + (int64_t)R(N - 1) + carry);
    return canon4_unpack(r);
}
// lo + v * d in canonical memory form for canonical lo (limbs from pack) and signed limbs d = hi - lo
// (|limb| < 2^26), through the table of v's multiples.
template <class TabPtr>
GRAPE_HD Fr foldt(TabPtr tab, const Limbs& lo, const Limbs& d) {
    int64_t c[N + 2];
    c[0] = c[1] = 0;
#pragma unroll
    for (int k = 0; k < N; k++) c[k + 2] = (int64_t)(uint32_t)lo.v[k];      // lo * 2^52
#pragma unroll
    for (int j = 0; j < N; j++) {
#pragma unroll
        for (int k = 0; k < N; k++) c[k] += (int64_t)d.v[j] * (int64_t)tab[j * N + k];
    }
    return foldt_finish(c);
}

}  // namespace fr26
}  // namespace grape
