// Host-side scalar and group value types with the subset of the libff interface the
// reference's protocol code uses (include/ec_operation.cuh:12-14: Fr = libff Fr, bn128 = libff
// G1): zero/one/random_element, construction from long, invert, + - * and comparisons, scalar
// times point.  The memory image of Fr is the device fr_t (canonical Montgomery limbs), so
// values cross the host/device boundary by plain copies as in src/fr-tensor.cu:214,352,437.
#pragma once
#include <cstdint>
#include <cstring>
#include <iosfwd>
#include <vector>
#include "../csrc/curve.hpp"

typedef grape::Fr fr_t;        // device element types, as named by include/field/bls12-381.cuh
typedef grape::Fp fp_t;
typedef grape::G1Affine affine_t;
typedef grape::G1Jac jacob_t;
typedef grape::G1Xyzz bucket_t;
typedef unsigned int uint;

class Fr {
public:
    fr_t v;

    Fr() : v(grape::Fr::zero()) {}
    Fr(long x);
    explicit Fr(const fr_t& raw) : v(raw) {}

    static Fr zero() { return Fr(); }
    static Fr one() { return Fr(grape::Fr::one()); }
    // Uniform element by rejection sampling of 255-bit draws.  The bits come from the operating
    // system's generator (getrandom), as libff's random_element draws from std::random_device
    // (src/ec_operation.cu:35,55), unless seed() has put the process into its reproducible mode
    // (a xoshiro256** stream behind a mutex) - for tests and benchmarks only: with a known seed the
    // blinding row of Hyrax::open, the lookups' alpha and r and the generator scalars are all
    // predictable.  seed_from_os() returns to the default.  Safe to call from several threads.
    static Fr random_element();
    static void seed(uint64_t s);
    static void seed_from_os();
    static bool seeded();

    bool is_zero() const { return v.is_zero(); }
    Fr& invert();                       // in place, 1/0 = 0; returns *this like libff
    Fr inverse() const { Fr t(*this); t.invert(); return t; }
    Fr squared() const { return Fr(grape::sqr(v)); }

    Fr operator+(const Fr& o) const { return Fr(grape::add(v, o.v)); }
    Fr operator-(const Fr& o) const { return Fr(grape::sub(v, o.v)); }
    Fr operator*(const Fr& o) const { return Fr(grape::mul(v, o.v)); }
    Fr operator-() const { return Fr(grape::neg(v)); }
    Fr& operator+=(const Fr& o) { v = grape::add(v, o.v); return *this; }
    Fr& operator-=(const Fr& o) { v = grape::sub(v, o.v); return *this; }
    Fr& operator*=(const Fr& o) { v = grape::mul(v, o.v); return *this; }
    bool operator==(const Fr& o) const { return v == o.v; }
    bool operator!=(const Fr& o) const { return v != o.v; }

    // canonical (non-Montgomery) limbs, little endian
    void to_plain(uint32_t out[8]) const;
};
static_assert(sizeof(Fr) == 32, "Fr must have the fr_t memory image");
std::ostream& operator<<(std::ostream& os, const Fr& x);

// G1 point in Jacobian coordinates; the memory image is the device jacob_t.
class G1 {
public:
    jacob_t p;

    G1() : p(grape::G1Jac::inf()) {}
    explicit G1(const jacob_t& raw) : p(raw) {}
    explicit G1(const affine_t& a);

    static G1 zero() { return G1(); }
    static G1 one();                     // the standard generator
    static G1 random_element();          // random scalar times the generator (see Fr::random_element)

    bool is_zero() const { return p.is_inf(); }
    affine_t to_affine() const;
    G1 operator+(const G1& o) const;
    G1 operator-(const G1& o) const;
    G1 operator-() const;
    G1 dbl() const;
    bool operator==(const G1& o) const;
    bool operator!=(const G1& o) const { return !(*this == o); }
};
static_assert(sizeof(G1) == 3 * 4 * grape::FpParams::N, "G1 must have the jacob_t memory image (144 bytes for BLS12-381, 96 for BN254)");
G1 operator*(const Fr& k, const G1& pt);

typedef G1 bn128;   // the reference's name for its host group type

// Multiples of ONE point that is multiplied again and again (Hyrax's G in every opening): the
// 6-bit-window multiples k * 2^(6w) * P, so that a scalar multiple is 43 additions and no doubling
// (0.1 ms where the double-and-add ladder of operator* takes 0.8 ms).  Same result as k * P.
class G1FixedBase {
public:
    explicit G1FixedBase(const G1& base);
    G1 mul(const Fr& k) const;

private:
    static constexpr int kBits = 6, kWindows = (255 + kBits - 1) / kBits, kPerWindow = (1 << kBits) - 1;
    std::vector<grape::G1Xyzz> table_;     // [w * kPerWindow + (k - 1)]
};
