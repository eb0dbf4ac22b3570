// Fp on signed limbs of 28 bits with lazy reduction - the working form of the commitment kernels
// (14 limbs, radix 2^392, for BLS12-381; 10 limbs, radix 2^280, for BN254).
//
// Why: on gfx950 a 32x32+64 multiply-add (v_mad_i64_i32 / v_mad_u64_u32) issues at the same rate
// as an addition, so the cost of a field product is its instruction count, and with saturated
// 32-bit limbs two thirds of the instructions are carry handling.  With 28-bit limbs every limb
// product is < 2^58, a whole column of an (a*b + m*p) row set fits a 64-bit accumulator, and a
// limb product is exactly ONE instruction; signed limbs make subtraction limb-wise, with no
// borrow chain and no bias.
//
// Representation: x = sum_i v[i] * 2^(28 i), v[i] signed 32-bit.  "Normalised" means
// 0 <= v[i] < 2^28 for i < N-1 (the top limb carries the sign and the overflow).  A value stands
// for its residue mod p; arithmetic is Montgomery with radix R' = 2^(28 N).  The canonical memory
// form elsewhere in the library is the reference's: 32-bit limbs, radix 2^384 resp. 2^256
// (include/field/mont_t.cuh, include/field/bls12-381.cuh:7-23, include/field/alt_bn128.cuh);
// conversion is exact both ways.
//
// Bounds (checked by the callers' comments): mul28(a, b) needs |a| < alpha*p, |b| < beta*p with
// alpha*beta <= 2^11 and limb magnitudes with 14 * 2^(la+lb) < 2^62, i.e. la + lb <= 58; its
// result is normalised and lies in (0, 3p).  The figures are those of BLS12-381, the tighter
// case: BN254 leaves R'/p = 2^26 of head-room instead of 2^11 and sums 10 limb products.
#pragma once
#include "curve.hpp"
#include "divstep.hpp"

namespace grape {

#if defined(GRAPE_CURVE_BN254)
struct Fp28 {
    int32_t v[10];
};

namespace fp28 {

constexpr int N = 10;
constexpr int W = 28;
constexpr uint32_t MASK = (1u << W) - 1;
constexpr uint32_t PINV = 0x4866389u;   // -p^-1 mod 2^28

GRAPE_HD int32_t P(int i) {
    constexpr int32_t t[10] = {0x87cfd47, 0x208c16d, 0x1ca8d3c, 0x6a91687, 0x85d9781,
                               0xb681815, 0x9b85045, 0xe131a02, 0x0644e72, 0x0000003};
    return t[i];
}
GRAPE_HD int32_t P2(int i) {   // 2p
    constexpr int32_t t[10] = {0x0f9fa8e, 0x41182db, 0x3951a78, 0xd522d0e, 0x0bb2f02,
                               0x6d0302b, 0x370a08b, 0xc263405, 0x0c89ce5, 0x0000006};
    return t[i];
}
GRAPE_HD int32_t ONE(int i) {   // 2^280 mod p
    constexpr int32_t t[10] = {0xa0e0d96, 0x6a56a28, 0x56d8f97, 0x1e6c92b, 0xee608fc,
                               0x10581c8, 0x89f6e5c, 0x8c59c9e, 0x7359fa8, 0x0000000};
    return t[i];
}
GRAPE_HD int32_t CMEM(int i) {   // 2^256 mod p: mul28(x*2^280, CMEM) = x*2^256
    constexpr int32_t t[10] = {0x58f0d9d, 0x5d438dc, 0x70b3dd3, 0xeb28f5c, 0x62c0a78,
                               0x6f78794, 0xf666ea3, 0x9a07df2, 0xe0a77c1, 0x0000000};
    return t[i];
}
// Montgomery (radix 2^256) form of 2^24, 32-bit limbs: mul(x*2^256, MCONV) = x*2^280 mod p
GRAPE_HD uint32_t MCONV(int i) {
    constexpr uint32_t t[8] = {0x8a0e0d96u, 0x976a56a2u, 0x92b56d8fu, 0x08fc1e6cu,
                               0x581c8ee6u, 0x9f6e5c10u, 0x8c59c9e8u, 0x07359fa8u};
    return t[i];
}
GRAPE_HD int32_t CIN(int i) {   // 2^304 mod p: mul28(pack(x*2^256), CIN) = x*2^280
    constexpr int32_t t[10] = {0x8b6fea0, 0xa73d9f9, 0x09603cf, 0xb860a8d, 0x8b33888,
                               0x9628387, 0xb8b8d5d, 0x9a84442, 0xe142fd5, 0x0000000};
    return t[i];
}

#else
struct Fp28 {
    int32_t v[14];
};

namespace fp28 {

constexpr int N = 14;
constexpr int W = 28;
constexpr uint32_t MASK = (1u << W) - 1;
constexpr uint32_t PINV = 0xffcfffdu;   // -p^-1 mod 2^28

GRAPE_HD int32_t P(int i) {
    constexpr int32_t t[14] = {0xfffaaab, 0xfefffff, 0x3ffffb9, 0xfffeb15, 0x6241eab, 0xa0f6b0f, 0xf6730d2,
                               0xf38512b, 0x4774b84, 0x4bacd76, 0xba7b643, 0xe69a4b1, 0x1ea397f, 0x001a011};
    return t[i];
}
GRAPE_HD int32_t P2(int i) {   // 2p
    constexpr int32_t t[14] = {0xfff5556, 0xfdfffff, 0x7ffff73, 0xfffd62a, 0xc483d57, 0x41ed61e, 0xece61a5,
                               0xe70a257, 0x8ee9709, 0x9759aec, 0x74f6c86, 0xcd34963, 0x3d472ff, 0x0034022};
    return t[i];
}
GRAPE_HD int32_t ONE(int i) {   // 2^392 mod p
    constexpr int32_t t[14] = {0x347fcb8, 0xd800000, 0x002b119, 0x0cde6d2, 0xc7212e0, 0x83a2090, 0x037669f,
                               0xda0f73e, 0x9b09b42, 0x1297bb0, 0x515d98f, 0x012ca7c, 0x659fcfa, 0x000577a};
    return t[i];
}
GRAPE_HD int32_t CMEM(int i) {   // 2^384 mod p: mul28(x*2^392, CMEM) = x*2^384
    constexpr int32_t t[14] = {0x002fffd, 0x0900000, 0xc000276, 0x000bc40, 0x8baebf4, 0x5753c75, 0x55f4898,
                               0x7052574, 0x7ce5853, 0x56ec6d7, 0x71a97a2, 0xe4935c0, 0xec3fa80, 0x0015f65};
    return t[i];
}
// Montgomery (radix 2^384) form of 2^8, 32-bit limbs: mul(x*2^384, MCONV) = x*2^392 mod p
GRAPE_HD uint32_t MCONV(int i) {
    constexpr uint32_t t[12] = {0x0347fcb8u, 0x19d80000u, 0x6d2002b1u, 0x12e00cdeu, 0xa2090c72u, 0x37669f83u,
                                0xda0f73e0u, 0x09b09b42u, 0x8f1297bbu, 0xa7c515d9u, 0xfcfa012cu, 0x0577a659u};
    return t[i];
}
GRAPE_HD int32_t CIN(int i) {   // 2^400 mod p: mul28(pack(x*2^384), CIN) = x*2^392
    constexpr int32_t t[14] = {0x80e6299, 0x3500034, 0xeb12856, 0xdeb2699, 0xc988670, 0x4ef6697, 0x70983e8,
                               0xa4e6fe9, 0x3e8a053, 0xecf271e, 0xc20d323, 0x6eb6385, 0x47f1286, 0x00156da};
    return t[i];
}

#endif

GRAPE_HD Fp28 one() {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = ONE(i);
    return r;
}
GRAPE_HD Fp28 zero() {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = 0;
    return r;
}

// limb-wise, no carries: the caller tracks magnitudes
GRAPE_HD Fp28 add(const Fp28& a, const Fp28& b) {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = a.v[i] + b.v[i];
    return r;
}
GRAPE_HD Fp28 sub(const Fp28& a, const Fp28& b) {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = a.v[i] - b.v[i];
    return r;
}
GRAPE_HD Fp28 neg(const Fp28& a) {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = -a.v[i];
    return r;
}
GRAPE_HD Fp28 cneg(const Fp28& a, bool flag) {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = flag ? -a.v[i] : a.v[i];
    return r;
}

// signed carry propagation: same value, limbs 0..N-2 in [0, 2^28)
GRAPE_HD Fp28 normalize(const Fp28& a) {
    Fp28 r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < N - 1; i++) {
        int32_t t = a.v[i] + c;
        r.v[i] = t & (int32_t)MASK;
        c = t >> W;   // arithmetic
    }
    r.v[N - 1] = a.v[N - 1] + c;
    return r;
}

// Montgomery product a*b/R' (mod p), result normalised in (0, 3p).
GRAPE_HD Fp28 mul(const Fp28& a, const Fp28& b) {
    int64_t C[2 * N];
#pragma unroll
    for (int k = 0; k < 2 * N; k++) C[k] = 0;
#pragma unroll
    for (int i = 0; i < N; i++) {
#pragma unroll
        for (int j = 0; j < N; j++) C[i + j] += (int64_t)a.v[j] * (int64_t)b.v[i];
        const int32_t m = (int32_t)(((uint32_t)C[i] * PINV) & MASK);
#pragma unroll
        for (int j = 0; j < N; j++) C[i + j] += (int64_t)m * (int64_t)P(j);
        C[i + 1] += C[i] >> W;   // C[i] is now a multiple of 2^28
    }
    // the quotient may be slightly negative: add p, then carry-propagate
    Fp28 r;
    int64_t c = 0;
#pragma unroll
    for (int k = 0; k < N - 1; k++) {
        int64_t t = C[N + k] + (int64_t)P(k) + c;
        r.v[k] = (int32_t)((uint32_t)t & MASK);
        c = t >> W;
    }
    r.v[N - 1] = (int32_t)(C[2 * N - 1] + (int64_t)P(N - 1) + c);
    return r;
}

// a*b - c*d with one Montgomery reduction: both products accumulate in the same columns.
// Needs 14*(2^(la+lb) + 2^(lc+ld)) + 14*2^56 < 2^63 for the limb bounds and |ab| + |cd| <= 2^11 p^2
// for the values; the result is normalised in (0, 3p) like a product.
GRAPE_HD Fp28 mul_sub(const Fp28& a, const Fp28& b, const Fp28& c, const Fp28& d) {
    int64_t C[2 * N];
#pragma unroll
    for (int k = 0; k < 2 * N; k++) C[k] = 0;
    int32_t nc[N];                        // limb-wise negation keeps every step a multiply-add
#pragma unroll
    for (int j = 0; j < N; j++) nc[j] = -c.v[j];
#pragma unroll
    for (int i = 0; i < N; i++) {
#pragma unroll
        for (int j = 0; j < N; j++) C[i + j] += (int64_t)a.v[j] * (int64_t)b.v[i];
#pragma unroll
        for (int j = 0; j < N; j++) C[i + j] += (int64_t)nc[j] * (int64_t)d.v[i];
        const int32_t m = (int32_t)(((uint32_t)C[i] * PINV) & MASK);
#pragma unroll
        for (int j = 0; j < N; j++) C[i + j] += (int64_t)m * (int64_t)P(j);
        C[i + 1] += C[i] >> W;
    }
    Fp28 r;
    int64_t cy = 0;
#pragma unroll
    for (int k = 0; k < N - 1; k++) {
        int64_t t = C[N + k] + (int64_t)P(k) + cy;
        r.v[k] = (int32_t)((uint32_t)t & MASK);
        cy = t >> W;
    }
    r.v[N - 1] = (int32_t)(C[2 * N - 1] + (int64_t)P(N - 1) + cy);
    return r;
}

// a^2/R': the off-diagonal limb products are taken once with a doubled operand.
GRAPE_HD Fp28 sqr(const Fp28& a) {
    int64_t C[2 * N];
#pragma unroll
    for (int k = 0; k < 2 * N; k++) C[k] = 0;
    int32_t a2[N];
#pragma unroll
    for (int i = 0; i < N; i++) a2[i] = a.v[i] * 2;
#pragma unroll
    for (int i = 0; i < N; i++) {
        C[2 * i] += (int64_t)a.v[i] * (int64_t)a.v[i];
#pragma unroll
        for (int j = i + 1; j < N; j++) C[i + j] += (int64_t)a2[i] * (int64_t)a.v[j];
    }
#pragma unroll
    for (int i = 0; i < N; i++) {
        const int32_t m = (int32_t)(((uint32_t)C[i] * PINV) & MASK);
#pragma unroll
        for (int j = 0; j < N; j++) C[i + j] += (int64_t)m * (int64_t)P(j);
        C[i + 1] += C[i] >> W;
    }
    Fp28 r;
    int64_t c = 0;
#pragma unroll
    for (int k = 0; k < N - 1; k++) {
        int64_t t = C[N + k] + (int64_t)P(k) + c;
        r.v[k] = (int32_t)((uint32_t)t & MASK);
        c = t >> W;
    }
    r.v[N - 1] = (int32_t)(C[2 * N - 1] + (int64_t)P(N - 1) + c);
    return r;
}

// Is a normalised value in [0, 3p) congruent to zero, i.e. one of 0, p, 2p?
GRAPE_HD bool is_zero_mod_p(const Fp28& a) {
    uint32_t z0 = 0, z1 = 0, z2 = 0;
#pragma unroll
    for (int i = 0; i < N; i++) {
        z0 |= (uint32_t)a.v[i];
        z1 |= (uint32_t)(a.v[i] ^ P(i));
        z2 |= (uint32_t)(a.v[i] ^ P2(i));
    }
    return (z0 == 0) | (z1 == 0) | (z2 == 0);
}

// ---- conversions with the canonical 32-bit-limb Montgomery form (radix 2^384 resp. 2^256) ----
constexpr int FW = FpParams::N;   // 32-bit words of the canonical form
// pure re-limbing of a non-negative integer of FW words
GRAPE_HD Fp28 pack(const Fp& x) {
    Fp28 r;
#pragma unroll
    for (int k = 0; k < N; k++) {
        const int bit = W * k, q = bit >> 5, s = bit & 31;
        uint64_t two = (uint64_t)x.v[q] | ((q + 1 < FW) ? ((uint64_t)x.v[q + 1] << 32) : 0);
        r.v[k] = (int32_t)((uint32_t)(two >> s) & MASK);
    }
    return r;
}
// inverse of pack for a normalised, non-negative value below 2^(32 FW)
GRAPE_HD Fp unpack(const Fp28& a) {
    Fp r;
#pragma unroll
    for (int q = 0; q < FW; q++) {
        // word q covers bits [32q, 32q+32): limbs k0 = floor(32q/28) .. up to two more
        const int k0 = (32 * q) / W;
        uint64_t acc = 0;
#pragma unroll
        for (int t = 0; t < 3; t++) {
            const int k = k0 + t;
            if (k < N) {
                const int sh = W * k - 32 * q;   // position of limb k relative to the word
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
// canonical memory form (32-bit limbs) -> working form (28-bit limbs), canonical and normalised
GRAPE_HD Fp28 from_canonical(const Fp& x) {
    Fp m;
#pragma unroll
    for (int i = 0; i < FW; i++) m.v[i] = MCONV(i);
    return pack(fmul(x, m));
}
// the same conversion with the 28-bit multiplier only (a third of the instructions): the result is
// normalised in (0, 3p) instead of canonical, which every consumer of a product accepts
GRAPE_HD Fp28 from_canonical_lazy(const Fp& x) {
    Fp28 c;
#pragma unroll
    for (int i = 0; i < N; i++) c.v[i] = CIN(i);
    return mul(pack(x), c);
}
// value in (-9p, 3p), any limb form -> canonical memory form, 32-bit limbs
GRAPE_HD Fp to_canonical(const Fp28& a) {
    Fp28 c;
#pragma unroll
    for (int i = 0; i < N; i++) c.v[i] = CMEM(i);
    Fp28 t = mul(normalize(a), c);   // in (0, 3p), now with the radix of the memory form
    // subtract p while the result stays non-negative (at most twice)
#pragma unroll
    for (int rep = 0; rep < 2; rep++) {
        Fp28 d;
#pragma unroll
        for (int i = 0; i < N; i++) d.v[i] = t.v[i] - P(i);
        d = normalize(d);
        const bool ok = d.v[N - 1] >= 0;
#pragma unroll
        for (int i = 0; i < N; i++) t.v[i] = ok ? d.v[i] : t.v[i];
    }
    return unpack(t);
}

// a^(p-2) in the 28-bit form (4-bit fixed windows, rolled loops); a in (-9p, 3p), a != 0 mod p.
// Result normalised in (0, 3p).
GRAPE_HD Fp28 inverse(const Fp28& a) {
    Fp28 tbl[16];
    tbl[0] = one();
    tbl[1] = mul(normalize(a), one());      // bring into (0, 3p)
    for (int i = 2; i < 16; i++) tbl[i] = mul(tbl[i - 1], tbl[1]);
    Fp28 acc = one();
    bool started = false;
    for (int limb = FW - 1; limb >= 0; limb--) {
        uint32_t e = 0;
        for (int k = 0; k < FW; k++) e = (k == limb) ? FpParams::pm2(k) : e;
        for (int nib = 7; nib >= 0; nib--) {
            if (started) {
                acc = sqr(acc);
                acc = sqr(acc);
                acc = sqr(acc);
                acc = sqr(acc);
            }
            uint32_t w = (e >> (4 * nib)) & 15u;
            if (w) {
                acc = mul(acc, tbl[w]);
                started = true;
            }
        }
    }
    return acc;
}

// ------------------------------------------------------------------------------------------------
// Modular inversion by divsteps (divstep.hpp) for the 28-bit form: about 800 divsteps for a 381-bit
// modulus, i.e. some 27 batches of a few hundred instructions each - one inversion sits on the
// critical path of every row epilogue.
// ------------------------------------------------------------------------------------------------
namespace by {

using divstep::M30;
using divstep::Mat;
using divstep::divsteps30;

#if defined(GRAPE_CURVE_BN254)
constexpr int L = 9;                        // 9 x 30 = 270 bits
constexpr uint32_t PINV30 = 0x1b799c77u;    // p^-1 mod 2^30
GRAPE_HD int32_t P30(int i) {
    constexpr int32_t t[9] = {0x187cfd47, 0x3082305b, 0x071ca8d3, 0x205aa45a, 0x01585d97,
                              0x0116da06, 0x1a029b85, 0x139cb84c, 0x00003064};
    return t[i];
}
#else
constexpr int L = 13;                       // 13 x 30 = 390 bits
constexpr uint32_t PINV30 = 0x00030003u;    // p^-1 mod 2^30
GRAPE_HD int32_t P30(int i) {
    constexpr int32_t t[13] = {0x3fffaaab, 0x27fbffff, 0x153ffffb, 0x2affffac, 0x30f6241e, 0x034a83da, 0x112bf673,
                               0x12e13ce1, 0x2cd76477, 0x1ed90d2e, 0x29a4b1ba, 0x3a8e5ff9, 0x001a0111};
    return t[i];
}
#endif
struct PMod {
    static constexpr uint32_t INV30 = PINV30;
    static GRAPE_HD int32_t limb(int i) { return P30(i); }
};
// 1110 divsteps at most for 384 bits, 741 for 256 bits
constexpr int kBatches = divstep::batches_for_bits(32 * FpParams::N);

GRAPE_HD void update_fg(int32_t* f, int32_t* g, const Mat& t) { divstep::update_fg<L>(f, g, t); }
GRAPE_HD void update_de(int32_t* d, int32_t* e, const Mat& t) { divstep::update_de<L, PMod>(d, e, t); }

}  // namespace by

// R'^3 mod p: turns the plain inverse of a Montgomery-form value back into Montgomery form
GRAPE_HD int32_t R3(int i) {
#if defined(GRAPE_CURVE_BN254)
    constexpr int32_t t[10] = {0xfdd47fe, 0xb246b8d, 0x1ffde25, 0xb55ed86, 0x14bbcde,
                               0xad156f8, 0x483330b, 0x59ae72c, 0x1df6aee, 0x0000000};
#else
    constexpr int32_t t[14] = {0x1f7b890, 0x294cc4d, 0x9f3af22, 0xb5ba56c, 0xcb5c0cc, 0xc0d975c, 0xc89a8c5,
                               0x6c968b4, 0x22672ea, 0x91de8c9, 0x35652a6, 0x84977c8, 0x424bbb9, 0x00141ab};
#endif
    return t[i];
}

// 1/a in Montgomery form (radix R') for a in (-9p, 3p), a != 0 mod p; result normalised in (0, 3p).
GRAPE_HD Fp28 inverse_by(const Fp28& a) {
    using namespace by;
    // canonical integer of a (still carrying the Montgomery factor) in [0, p)
    Fp28 t = mul(normalize(a), one());
#pragma unroll
    for (int rep = 0; rep < 2; rep++) {
        Fp28 dd;
#pragma unroll
        for (int i = 0; i < N; i++) dd.v[i] = t.v[i] - P(i);
        dd = normalize(dd);
        const bool ok = dd.v[N - 1] >= 0;
#pragma unroll
        for (int i = 0; i < N; i++) t.v[i] = ok ? dd.v[i] : t.v[i];
    }
    // re-limb N x 28 -> L x 30
    int32_t f[L], g[L], d[L], e[L];
#pragma unroll
    for (int k = 0; k < L; k++) {
        const int bit = 30 * k, i0 = bit / W, sh = bit % W;
        uint64_t w = (uint64_t)(uint32_t)t.v[i0] >> sh;
        if (i0 + 1 < N) w |= (uint64_t)(uint32_t)t.v[i0 + 1] << (W - sh);
        if (i0 + 2 < N && 2 * W - sh < 30) w |= (uint64_t)(uint32_t)t.v[i0 + 2] << (2 * W - sh);
        g[k] = (int32_t)(w & (uint64_t)M30);
        f[k] = P30(k);
        d[k] = 0;
        e[k] = 0;
    }
    e[0] = 1;
    int32_t delta = 1;
    for (int batch = 0; batch < kBatches; batch++) {
        uint32_t gz = 0;
#pragma unroll
        for (int k = 0; k < L; k++) gz |= (uint32_t)g[k];
        if (gz == 0) break;
        Mat m;
        delta = divsteps30(delta, (uint32_t)f[0] | ((uint32_t)f[1] << 30), (uint32_t)g[0] | ((uint32_t)g[1] << 30), m);
        update_de(d, e, m);
        update_fg(f, g, m);
    }
    // now g = 0, f = +-1 and d * a = f (mod p): the inverse is d * f; bring it into [0, p)
    const int32_t fneg = f[L - 1] >> 31;          // all-ones when f = -1
    int64_t c = 0;
    int32_t x[L];
#pragma unroll
    for (int k = 0; k < L; k++) x[k] = (d[k] ^ fneg) - fneg;   // limb-wise negation when f = -1
    // x in (-2p, 2p): add 2p, then normalise (limbs to [0, 2^30), top signed but now positive)
#pragma unroll
    for (int k = 0; k < L - 1; k++) {
        int64_t s = (int64_t)x[k] + 2 * (int64_t)P30(k) + c;
        x[k] = (int32_t)s & M30;
        c = s >> 30;
    }
    x[L - 1] = (int32_t)((int64_t)x[L - 1] + 2 * (int64_t)P30(L - 1) + c);
    // re-limb L x 30 -> N x 28 (value in (0, 4p), below 2^(32 FW))
    Fp28 r;
#pragma unroll
    for (int k = 0; k < N; k++) {
        const int bit = W * k, i0 = bit / 30, sh = bit % 30;
        uint64_t w = (uint64_t)(uint32_t)x[i0] >> sh;
        if (i0 + 1 < L) w |= (uint64_t)(uint32_t)x[i0 + 1] << (30 - sh);
        r.v[k] = (int32_t)(w & (uint64_t)MASK);
    }
    Fp28 r3;
#pragma unroll
    for (int i = 0; i < N; i++) r3.v[i] = R3(i);
    return mul(r, r3);   // 4 * 1 <= 2^11
}

}  // namespace fp28

// ------------------------------------------------------------------------------------------------
// XYZZ accumulator in the 28-bit form.  Invariants between additions:
//   x in (-9p, 3p) normalised (signed top limb); y in (-3p, 3p) with |limbs| < 2^28;
//   zz, zzz in (0, 3p) normalised, never congruent to zero; `inf` marks the identity.
// ------------------------------------------------------------------------------------------------
struct Xyzz28 {
    Fp28 x, y, zz, zzz;
    bool inf;
};
struct Affine28 {   // canonical coordinates (in [0,p), normalised)
    Fp28 x, y;
};

GRAPE_HD Xyzz28 xyzz28_inf() {
    Xyzz28 r;
    r.x = fp28::zero();
    r.y = fp28::zero();
    r.zz = fp28::zero();
    r.zzz = fp28::zero();
    r.inf = true;
    return r;
}

GRAPE_HD G1Xyzz xyzz28_to_canonical(const Xyzz28& a) {
    if (a.inf) return G1Xyzz::inf();
    G1Xyzz r;
    r.x = fp28::to_canonical(a.x);
    r.y = fp28::to_canonical(a.y);
    r.zz = fp28::to_canonical(a.zz);
    r.zzz = fp28::to_canonical(a.zzz);
    return r;
}
GRAPE_HD Xyzz28 xyzz28_from_canonical(const G1Xyzz& a) {
    Xyzz28 r;
    r.inf = a.is_inf();
    r.x = fp28::from_canonical(a.x);
    r.y = fp28::from_canonical(a.y);
    r.zz = fp28::from_canonical(a.zz);
    r.zzz = fp28::from_canonical(a.zzz);
    return r;
}

// acc += (negate ? -p : p) for a finite affine point p (the caller skips the identity).
// Returns false when the addition is one of the exceptional cases (p = +-acc): then acc is left
// untouched and the caller must take the exact slow path.
GRAPE_HD bool xyzz28_madd(Xyzz28& acc, const Affine28& p, bool negate) {
    using namespace fp28;
    if (acc.inf) {
        acc.x = p.x;
        acc.y = cneg(p.y, negate);
        acc.zz = one();
        acc.zzz = one();
        acc.inf = false;
        return true;
    }
    const Fp28 U2 = mul(p.x, acc.zz);                  // 1 * 3            -> (0,3p)
    const Fp28 S2 = mul(p.y, acc.zzz);                 // 1 * 3            -> (0,3p)
    const Fp28 Pd = sub(U2, acc.x);                    // (-3p,12p), |limb| < 2^29
    const Fp28 R = sub(cneg(S2, negate), acc.y);       // (-6p, 6p), |limb| < 2^29
    const Fp28 PP = sqr(Pd);                           // 144 <= 2^11, 29+29 <= 58
    const Fp28 ZZ3 = mul(acc.zz, PP);                  // 9
    if (is_zero_mod_p(ZZ3)) return false;              // PP = 0  <=>  P = 0: doubling or cancellation
    const Fp28 PPP = mul(Pd, PP);                      // 12 * 3 = 36
    const Fp28 Q = mul(acc.x, PP);                     // 9 * 3 = 27
    const Fp28 RR = sqr(R);                            // 36
    Fp28 X3;
#pragma unroll
    for (int i = 0; i < N; i++) X3.v[i] = RR.v[i] - PPP.v[i] - 2 * Q.v[i];   // (-9p, 3p), |limb| < 2^30
    X3 = normalize(X3);
    const Fp28 T = sub(Q, X3);                         // (-3p, 12p), |limb| < 2^29
    const Fp28 Y3 = mul_sub(R, T, acc.y, PPP);         // 6*12 + 3*3 = 81 <= 2^11; limbs 29+29, 28+28 -> (0, 3p)
    acc.zzz = mul(acc.zzz, PPP);                       // 9
    acc.zz = ZZ3;
    acc.x = X3;
    acc.y = Y3;
    return true;
}

// acc <- 2 * acc in the 28-bit form (curve with a = 0, 6M + 3S: U = 2Y, V = U^2, W = U V, S = X V,
// M = 3 X^2, X3 = M^2 - 2S, Y3 = M (S - X3) - W Y, ZZ3 = V ZZ, ZZZ3 = W ZZZ).  No exceptional case on
// a group of odd prime order; the identity stays the identity.
GRAPE_HD void xyzz28_dbl(Xyzz28& acc) {
    using namespace fp28;
    if (acc.inf) return;
    Fp28 U;
#pragma unroll
    for (int i = 0; i < N; i++) U.v[i] = 2 * acc.y.v[i];            // (-6p, 6p), |limb| < 2^29
    const Fp28 V = sqr(U);                                          // 36
    const Fp28 Wd = mul(U, V);                                      // 6 * 3
    const Fp28 S = mul(acc.x, V);                                   // 9 * 3
    const Fp28 X2 = sqr(acc.x);                                     // 81
    Fp28 M;
#pragma unroll
    for (int i = 0; i < N; i++) M.v[i] = 3 * X2.v[i];               // (0, 9p)
    M = normalize(M);
    const Fp28 MM = sqr(M);                                         // 81
    Fp28 X3;
#pragma unroll
    for (int i = 0; i < N; i++) X3.v[i] = MM.v[i] - 2 * S.v[i];     // (-6p, 3p)
    X3 = normalize(X3);
    const Fp28 T = sub(S, X3);                                      // (-3p, 9p), |limb| < 2^29
    const Fp28 Y3 = mul_sub(M, T, Wd, acc.y);                       // 81 + 9; limbs 28+29, 28+28
    acc.zz = mul(V, acc.zz);                                        // 9
    acc.zzz = mul(Wd, acc.zzz);                                     // 9
    acc.x = X3;
    acc.y = Y3;
}

// acc += q, both accumulators in the 28-bit form (12M + 2S).  Returns false, leaving acc
// untouched, in the exceptional cases q = +-acc; identities are handled here.
GRAPE_HD bool xyzz28_add(Xyzz28& acc, const Xyzz28& q) {
    using namespace fp28;
    if (q.inf) return true;
    if (acc.inf) {
        acc = q;
        return true;
    }
    const Fp28 U1 = mul(acc.x, q.zz);                  // 9 * 3 = 27
    const Fp28 U2 = mul(q.x, acc.zz);
    const Fp28 S1 = mul(acc.y, q.zzz);                 // 3 * 3
    const Fp28 S2 = mul(q.y, acc.zzz);
    const Fp28 Pd = sub(U2, U1);                       // (-3p, 3p)
    const Fp28 R = sub(S2, S1);                        // (-3p, 3p)
    const Fp28 PP = sqr(Pd);                           // 9
    const Fp28 ZZ3 = mul(mul(acc.zz, q.zz), PP);       // 9, 9
    if (is_zero_mod_p(ZZ3)) return false;
    const Fp28 PPP = mul(Pd, PP);                      // 9
    const Fp28 Q = mul(U1, PP);                        // 9
    const Fp28 RR = sqr(R);                            // 9
    Fp28 X3;
#pragma unroll
    for (int i = 0; i < N; i++) X3.v[i] = RR.v[i] - PPP.v[i] - 2 * Q.v[i];   // (-9p, 3p)
    X3 = normalize(X3);
    const Fp28 T = sub(Q, X3);                         // (-3p, 12p)
    const Fp28 Y3 = mul_sub(R, T, S1, PPP);            // 36 + 9
    acc.zzz = mul(mul(acc.zzz, q.zzz), PPP);
    acc.zz = ZZ3;
    acc.x = X3;
    acc.y = Y3;
    return true;
}

// affine image in canonical 32-bit form; the identity maps to (0,0)
GRAPE_HD G1Affine xyzz28_to_affine(const Xyzz28& a) {
    using namespace fp28;
    if (a.inf) return G1Affine::inf();
    const Fp28 zzz_inv = inverse_by(a.zzz);
    const Fp28 zinv = mul(zzz_inv, a.zz);             // 1/Z
    G1Affine r;
    r.x = to_canonical(mul(a.x, sqr(zinv)));
    r.y = to_canonical(mul(a.y, zzz_inv));
    return r;
}

// ------------------------------------------------------------------------------------------------
// Affine + affine with the inversion supplied by the caller (Montgomery's trick over many
// independent additions: table generation).  Inputs are finite points with canonical coordinates.
// ------------------------------------------------------------------------------------------------
// a normalised value in [0, 2^k p) -> the representative in [0, p)
template <int K>
GRAPE_HD Fp28 fp28_below_p(Fp28 t) {
#pragma unroll
    for (int s = K - 1; s >= 0; s--) {
        Fp28 d;
#pragma unroll
        for (int i = 0; i < fp28::N; i++) d.v[i] = t.v[i] - fp28::P(i) * (1 << s);
        d = fp28::normalize(d);
        const bool ok = d.v[fp28::N - 1] >= 0;
#pragma unroll
        for (int i = 0; i < fp28::N; i++) t.v[i] = ok ? d.v[i] : t.v[i];
    }
    return t;
}
// denominator of the slope of e + f (x_e - x_f), or of 2 f (2 y_f) when `dbl`; a value congruent
// to zero means that the sum is no finite affine addition (e = +-f, or a point of order two)
GRAPE_HD Fp28 affine28_slope_den(const Affine28& e, const Affine28& f, bool dbl) {
    Fp28 r;
#pragma unroll
    for (int i = 0; i < fp28::N; i++) r.v[i] = dbl ? 2 * f.y.v[i] : e.x.v[i] - f.x.v[i];
    return r;
}
// e + f (2 f when `dbl`; then e must equal f) given dinv = 1 / affine28_slope_den(e, f, dbl), a
// product output in (0, 3p): 3M + 1S (one more S for the doubling), coordinates canonical
GRAPE_HD Affine28 affine28_add_given_inverse(const Affine28& e, const Affine28& f, bool dbl, const Fp28& dinv) {
    using namespace fp28;
    Fp28 num;
    if (dbl) {
        const Fp28 xx = sqr(f.x);                       // (0, 3p)
#pragma unroll
        for (int i = 0; i < N; i++) num.v[i] = 3 * xx.v[i];
        num = normalize(num);                           // (0, 9p)
    } else {
        num = sub(e.y, f.y);                            // (-p, p)
    }
    const Fp28 lam = mul(num, dinv);                    // 9 * 3 = 27 <= 2^11
    const Fp28 ll = sqr(lam);                           // (0, 3p)
    Fp28 x3;
#pragma unroll
    for (int i = 0; i < N; i++) x3.v[i] = ll.v[i] - e.x.v[i] - f.x.v[i] + P2(i);   // (0, 5p)
    x3 = fp28_below_p<3>(normalize(x3));
    const Fp28 ly = mul(lam, sub(e.x, x3));             // 3 * 1
    Fp28 y3;
#pragma unroll
    for (int i = 0; i < N; i++) y3.v[i] = ly.v[i] - e.y.v[i] + P(i);               // (0, 4p)
    Affine28 r;
    r.x = x3;
    r.y = fp28_below_p<2>(normalize(y3));
    return r;
}

}  // namespace grape
