// Montgomery prime-field arithmetic on 32-bit limbs for BLS12-381 Fr (8 limbs, R = 2^256)
// and Fp (12 limbs, R = 2^384), written for gfx950: every limb product is a 32x32+64 -> 64
// multiply-add (v_mad_u64_u32) and carries ride in the upper half of the 64-bit result.
//
// Semantics follow the reference's mont_t (include/field/mont_t.cuh:30-1134) with the constants
// of include/field/bls12-381.cuh:7-45: values are stored as canonical Montgomery residues
// (x * R mod m, always < m), little-endian limbs; add/sub/mul/sqr/cneg/to/from return canonical
// results, and the reciprocal of zero is zero (mont_t.cuh:1113-1119).
//
// The same code compiles for the host (used by the host-side Fr / G1 value types), so the
// memory image of a host value and of a device element are identical.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define GRAPE_HD __host__ __device__ __forceinline__
#else
#define GRAPE_HD inline __attribute__((always_inline))
#endif

namespace grape {

// ---------------------------------------------------------------------------------------------
// Parameter packs. Limb accessors are functions with local constexpr tables so that, after
// unrolling, every modulus limb becomes a scalar literal on the device (no VGPRs, no loads).
// ---------------------------------------------------------------------------------------------
// The curve is chosen when the library is compiled: BLS12-381 (include/field/bls12-381.cuh) by
// default, BN254 (include/field/alt_bn128.cuh) with -DGRAPE_CURVE_BN254.
#if defined(GRAPE_CURVE_BN254)
struct FrParams {   // BN254 scalar field (include/field/alt_bn128.cuh: ALT_BN128_r, rRR, rone, m0)
    static constexpr int N = 8;
    static constexpr uint32_t M0 = 0xefffffffu;  // -r^-1 mod 2^32
    static GRAPE_HD uint32_t mod(int i) {
        constexpr uint32_t t[8] = {0xf0000001u, 0x43e1f593u, 0x79b97091u, 0x2833e848u,
                                   0x8181585du, 0xb85045b6u, 0xe131a029u, 0x30644e72u};
        return t[i];
    }
    static GRAPE_HD uint32_t one(int i) {  // 2^256 mod r
        constexpr uint32_t t[8] = {0x4ffffffbu, 0xac96341cu, 0x9f60cd29u, 0x36fc7695u,
                                   0x7879462eu, 0x666ea36fu, 0x9a07df2fu, 0x0e0a77c1u};
        return t[i];
    }
    static GRAPE_HD uint32_t rr(int i) {  // 2^512 mod r
        constexpr uint32_t t[8] = {0xae216da7u, 0x1bb8e645u, 0xe35c59e3u, 0x53fe3ab1u,
                                   0x53bb8085u, 0x8c49833du, 0x7f4e44a5u, 0x0216d0b1u};
        return t[i];
    }
    static GRAPE_HD uint32_t pm2(int i) {  // r - 2 (Fermat exponent)
        constexpr uint32_t t[8] = {0xefffffffu, 0x43e1f593u, 0x79b97091u, 0x2833e848u,
                                   0x8181585du, 0xb85045b6u, 0xe131a029u, 0x30644e72u};
        return t[i];
    }
};

struct FpParams {   // BN254 base field (include/field/alt_bn128.cuh: ALT_BN128_P, RR, one, M0)
    static constexpr int N = 8;
    static constexpr uint32_t M0 = 0xe4866389u;  // -p^-1 mod 2^32
    static GRAPE_HD uint32_t mod(int i) {
        constexpr uint32_t t[8] = {0xd87cfd47u, 0x3c208c16u, 0x6871ca8du, 0x97816a91u,
                                   0x8181585du, 0xb85045b6u, 0xe131a029u, 0x30644e72u};
        return t[i];
    }
    static GRAPE_HD uint32_t one(int i) {  // 2^256 mod p
        constexpr uint32_t t[8] = {0xc58f0d9du, 0xd35d438du, 0xf5c70b3du, 0x0a78eb28u,
                                   0x7879462cu, 0x666ea36fu, 0x9a07df2fu, 0x0e0a77c1u};
        return t[i];
    }
    static GRAPE_HD uint32_t rr(int i) {  // 2^512 mod p
        constexpr uint32_t t[8] = {0x538afa89u, 0xf32cfc5bu, 0xd44501fbu, 0xb5e71911u,
                                   0x0a417ff6u, 0x47ab1effu, 0xcab8351fu, 0x06d89f71u};
        return t[i];
    }
    static GRAPE_HD uint32_t pm2(int i) {  // p - 2
        constexpr uint32_t t[8] = {0xd87cfd45u, 0x3c208c16u, 0x6871ca8du, 0x97816a91u,
                                   0x8181585du, 0xb85045b6u, 0xe131a029u, 0x30644e72u};
        return t[i];
    }
};

#else
struct FrParams {
    static constexpr int N = 8;
    static constexpr uint32_t M0 = 0xffffffffu;  // -r^-1 mod 2^32
    static GRAPE_HD uint32_t mod(int i) {
        constexpr uint32_t t[8] = {0x00000001u, 0xffffffffu, 0xfffe5bfeu, 0x53bda402u,
                                   0x09a1d805u, 0x3339d808u, 0x299d7d48u, 0x73eda753u};
        return t[i];
    }
    static GRAPE_HD uint32_t one(int i) {  // 2^256 mod r
        constexpr uint32_t t[8] = {0xfffffffeu, 0x00000001u, 0x00034802u, 0x5884b7fau,
                                   0xecbc4ff5u, 0x998c4fefu, 0xacc5056fu, 0x1824b159u};
        return t[i];
    }
    static GRAPE_HD uint32_t rr(int i) {  // 2^512 mod r
        constexpr uint32_t t[8] = {0xf3f29c6du, 0xc999e990u, 0x87925c23u, 0x2b6cedcbu,
                                   0x7254398fu, 0x05d31496u, 0x9f59ff11u, 0x0748d9d9u};
        return t[i];
    }
    static GRAPE_HD uint32_t pm2(int i) {  // r - 2 (Fermat exponent)
        constexpr uint32_t t[8] = {0xffffffffu, 0xfffffffeu, 0xfffe5bfeu, 0x53bda402u,
                                   0x09a1d805u, 0x3339d808u, 0x299d7d48u, 0x73eda753u};
        return t[i];
    }
};

struct FpParams {
    static constexpr int N = 12;
    static constexpr uint32_t M0 = 0xfffcfffdu;  // -p^-1 mod 2^32
    static GRAPE_HD uint32_t mod(int i) {
        constexpr uint32_t t[12] = {0xffffaaabu, 0xb9feffffu, 0xb153ffffu, 0x1eabfffeu,
                                    0xf6b0f624u, 0x6730d2a0u, 0xf38512bfu, 0x64774b84u,
                                    0x434bacd7u, 0x4b1ba7b6u, 0x397fe69au, 0x1a0111eau};
        return t[i];
    }
    static GRAPE_HD uint32_t one(int i) {  // 2^384 mod p
        constexpr uint32_t t[12] = {0x0002fffdu, 0x76090000u, 0xc40c0002u, 0xebf4000bu,
                                    0x53c758bau, 0x5f489857u, 0x70525745u, 0x77ce5853u,
                                    0xa256ec6du, 0x5c071a97u, 0xfa80e493u, 0x15f65ec3u};
        return t[i];
    }
    static GRAPE_HD uint32_t rr(int i) {  // 2^768 mod p
        constexpr uint32_t t[12] = {0x1c341746u, 0xf4df1f34u, 0x09d104f1u, 0x0a76e6a6u,
                                    0x4c95b6d5u, 0x8de5476cu, 0x939d83c0u, 0x67eb88a9u,
                                    0xb519952du, 0x9a793e85u, 0x92cae3aau, 0x11988fe5u};
        return t[i];
    }
    static GRAPE_HD uint32_t pm2(int i) {  // p - 2
        constexpr uint32_t t[12] = {0xffffaaa9u, 0xb9feffffu, 0xb153ffffu, 0x1eabfffeu,
                                    0xf6b0f624u, 0x6730d2a0u, 0xf38512bfu, 0x64774b84u,
                                    0x434bacd7u, 0x4b1ba7b6u, 0x397fe69au, 0x1a0111eau};
        return t[i];
    }
};

#endif

// ---------------------------------------------------------------------------------------------
// Field element
// ---------------------------------------------------------------------------------------------
template <class P>
struct alignas(16) Mont {
    static constexpr int N = P::N;
    uint32_t v[N];

    static GRAPE_HD Mont zero() {
        Mont r;
#pragma unroll
        for (int i = 0; i < N; i++) r.v[i] = 0;
        return r;
    }
    static GRAPE_HD Mont one() {
        Mont r;
#pragma unroll
        for (int i = 0; i < N; i++) r.v[i] = P::one(i);
        return r;
    }
    static GRAPE_HD Mont rr() {
        Mont r;
#pragma unroll
        for (int i = 0; i < N; i++) r.v[i] = P::rr(i);
        return r;
    }
    // Plain (non-Montgomery) small integer; callers follow with to_mont().
    static GRAPE_HD Mont from_u32_raw(uint32_t x) {
        Mont r = zero();
        r.v[0] = x;
        return r;
    }

    GRAPE_HD bool is_zero() const {
        uint32_t acc = 0;
#pragma unroll
        for (int i = 0; i < N; i++) acc |= v[i];
        return acc == 0;
    }
    GRAPE_HD bool operator==(const Mont& o) const {
        uint32_t acc = 0;
#pragma unroll
        for (int i = 0; i < N; i++) acc |= v[i] ^ o.v[i];
        return acc == 0;
    }
    GRAPE_HD bool operator!=(const Mont& o) const { return !(*this == o); }
};

namespace detail {

// One word of a carry / borrow chain (carry and borrow are 0 or 1).  With clang the builtins become
// one add-with-carry / subtract-with-borrow instruction per word on the device (64-bit emulation of
// the chain costs three to four times as many instructions there); other compilers spell it out.
GRAPE_HD uint32_t adc32(uint32_t a, uint32_t b, uint32_t& carry) {
#if defined(__clang__)
    unsigned int out;
    const uint32_t r = __builtin_addc(a, b, carry, &out);
    carry = out;
    return r;
#else
    const uint64_t t = (uint64_t)a + b + carry;
    carry = (uint32_t)(t >> 32);
    return (uint32_t)t;
#endif
}
GRAPE_HD uint32_t sbb32(uint32_t a, uint32_t b, uint32_t& borrow) {
#if defined(__clang__)
    unsigned int out;
    const uint32_t r = __builtin_subc(a, b, borrow, &out);
    borrow = out;
    return r;
#else
    const uint64_t t = (uint64_t)a - b - borrow;
    borrow = (uint32_t)(t >> 32) & 1u;
    return (uint32_t)t;
#endif
}

// r = a - mod if a >= mod else a (a < 2*mod assumed, carry_in is the bit above limb N-1).
template <class P>
GRAPE_HD void final_sub(uint32_t* r, const uint32_t* a, uint32_t carry_in) {
    constexpr int N = P::N;
    uint32_t d[N];
    uint32_t borrow = 0;
#pragma unroll
    for (int i = 0; i < N; i++) d[i] = sbb32(a[i], P::mod(i), borrow);
    // a >= mod  <=>  no final borrow, or the overflow bit was set
    bool ge = (borrow == 0) | (carry_in != 0);
#pragma unroll
    for (int i = 0; i < N; i++) r[i] = ge ? d[i] : a[i];
}

}  // namespace detail

template <class P>
GRAPE_HD Mont<P> add(const Mont<P>& a, const Mont<P>& b) {
    constexpr int N = P::N;
    uint32_t s[N];
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < N; i++) s[i] = detail::adc32(a.v[i], b.v[i], c);
    Mont<P> r;
    detail::final_sub<P>(r.v, s, c);
    return r;
}

template <class P>
GRAPE_HD Mont<P> sub(const Mont<P>& a, const Mont<P>& b) {
    constexpr int N = P::N;
    uint32_t d[N];
    uint32_t borrow = 0;
#pragma unroll
    for (int i = 0; i < N; i++) d[i] = detail::sbb32(a.v[i], b.v[i], borrow);
    // add the modulus back when the subtraction wrapped
    const uint32_t mask = (uint32_t)0 - borrow;
    Mont<P> r;
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = detail::adc32(d[i], P::mod(i) & mask, c);
    return r;
}

// -a when flag, a otherwise; -0 = 0 (mont_t.cuh:303 cneg).
template <class P>
GRAPE_HD Mont<P> cneg(const Mont<P>& a, bool flag) {
    constexpr int N = P::N;
    uint32_t nz = 0;
#pragma unroll
    for (int i = 0; i < N; i++) nz |= a.v[i];
    bool doit = flag & (nz != 0);
    Mont<P> r;
    uint32_t borrow = 0;
#pragma unroll
    for (int i = 0; i < N; i++) {
        const uint32_t t = detail::sbb32(P::mod(i), a.v[i], borrow);
        r.v[i] = doit ? t : a.v[i];
    }
    return r;
}

template <class P>
GRAPE_HD Mont<P> neg(const Mont<P>& a) {
    return cneg(a, true);
}

template <class P>
GRAPE_HD Mont<P> dbl(const Mont<P>& a) {
    return add(a, a);
}

// Montgomery product a*b/R mod m. Coarsely-integrated operand scanning: for each limb of b,
// one multiply-accumulate row and one reduction row; the running value stays below 2m and,
// because both moduli leave spare top bits, always fits N+1 limbs.
template <class P>
GRAPE_HD Mont<P> mul(const Mont<P>& a, const Mont<P>& b) {
    constexpr int N = P::N;
    uint32_t t[N + 1];
#pragma unroll
    for (int i = 0; i <= N; i++) t[i] = 0;
#pragma unroll
    for (int i = 0; i < N; i++) {
        uint64_t c = 0;
        const uint32_t bi = b.v[i];
#pragma unroll
        for (int j = 0; j < N; j++) {
            uint64_t acc = (uint64_t)a.v[j] * bi + t[j] + c;
            t[j] = (uint32_t)acc;
            c = acc >> 32;
        }
        uint64_t top = (uint64_t)t[N] + c;  // < 2^33
        const uint32_t m = t[0] * P::M0;
        uint64_t acc = (uint64_t)m * P::mod(0) + t[0];
        c = acc >> 32;
#pragma unroll
        for (int j = 1; j < N; j++) {
            acc = (uint64_t)m * P::mod(j) + t[j] + c;
            t[j - 1] = (uint32_t)acc;
            c = acc >> 32;
        }
        top += c;
        t[N - 1] = (uint32_t)top;
        t[N] = (uint32_t)(top >> 32);
    }
    Mont<P> r;
    detail::final_sub<P>(r.v, t, t[N]);
    return r;
}

template <class P>
GRAPE_HD Mont<P> sqr(const Mont<P>& a) {
    return mul(a, a);
}

// Montgomery form in/out (mont_t.cuh:453 to(), :483 from()).
template <class P>
GRAPE_HD Mont<P> to_mont(const Mont<P>& a) {
    return mul(a, Mont<P>::rr());
}
template <class P>
GRAPE_HD Mont<P> from_mont(const Mont<P>& a) {
    Mont<P> o = Mont<P>::zero();
    o.v[0] = 1;
    return mul(a, o);
}

// a^(m-2): the inverse for a != 0 and 0 for a == 0, which is the reference's convention.
// Deliberately a rolled loop (4-bit fixed windows): code size matters more than the last
// few multiplies because callers amortise inversions over batches.
template <class P>
GRAPE_HD Mont<P> inverse(const Mont<P>& a) {
    constexpr int N = P::N;
    Mont<P> tbl[16];
    tbl[0] = Mont<P>::one();
    tbl[1] = a;
    for (int i = 2; i < 16; i++) tbl[i] = mul(tbl[i - 1], a);
    Mont<P> acc = Mont<P>::one();
    bool started = false;
    for (int limb = N - 1; limb >= 0; limb--) {
        uint32_t e = 0;
        // rolled selection of the exponent limb keeps the loop body small
        for (int k = 0; k < N; k++) e = (k == limb) ? P::pm2(k) : e;
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

using Fr = Mont<FrParams>;
using Fp = Mont<FpParams>;

// Embedding of a machine integer: |x| as a residue, negated for x < 0, then into Montgomery
// form (the reference's int_to_fr, src/fr-tensor.cu:30-39).
GRAPE_HD Fr fr_from_i32(int32_t x) {
    uint32_t ax = x < 0 ? (uint32_t)0 - (uint32_t)x : (uint32_t)x;
    Fr r = to_mont(Fr::from_u32_raw(ax));
    return cneg(r, x < 0);
}
GRAPE_HD Fr fr_from_u32(uint32_t x) { return to_mont(Fr::from_u32_raw(x)); }

}  // namespace grape
