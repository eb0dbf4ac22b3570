#include "fr.hpp"
#include "../csrc/divstep.hpp"
#include <atomic>
#include <errno.h>
#include <sys/random.h>
#include <iomanip>
#include <mutex>
#include <ostream>
#include <stdexcept>

namespace {
// Deterministic generator of the opt-in seeded mode (tests, benchmarks): xoshiro256**.
struct Xoshiro {
    uint64_t s[4];
    static uint64_t splitmix(uint64_t& x) {
        uint64_t z = (x += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    void seed(uint64_t x) { for (int i = 0; i < 4; i++) s[i] = splitmix(x); }
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t next() {
        uint64_t r = rotl(s[1] * 5, 7) * 9, t = s[1] << 17;
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]; s[2] ^= t; s[3] = rotl(s[3], 45);
        return r;
    }
};
// The random source of Fr::random_element.  By default every draw comes from the operating
// system's generator (getrandom(2), the source behind libff's std::random_device draws,
// src/ec_operation.cu:35,55): blinding rows, challenges and generator scalars are unpredictable and
// never repeat between processes.  Fr::seed(s) switches the whole process to a reproducible stream
// (one generator behind a mutex, so OpenMP callers stay safe, though their interleaving is not
// reproducible); Fr::seed_from_os() switches back.
std::mutex g_rng_mu;
std::atomic<bool> g_seeded{false};
Xoshiro g_xo;

// 64 random bits from the OS, buffered per thread
uint64_t os_random64() {
    thread_local uint64_t buf[64];
    thread_local size_t have = 0;
    if (have == 0) {
        size_t got = 0;
        unsigned char* p = reinterpret_cast<unsigned char*>(buf);
        while (got < sizeof buf) {
            ssize_t n = getrandom(p + got, sizeof buf - got, 0);
            if (n < 0) {
                if (errno == EINTR) continue;
                throw std::runtime_error("Fr::random_element: getrandom failed");
            }
            got += (size_t)n;
        }
        have = 64;
    }
    const uint64_t w = buf[--have];
    buf[have] = 0;                       // a word is handed out once and not kept
    return w;
}
// four words of one draw: one lock per element in the reproducible mode, none in the default mode
void next256(uint64_t w[4]) {
    if (g_seeded.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_rng_mu);
        if (g_seeded.load(std::memory_order_relaxed)) {
            for (int i = 0; i < 4; i++) w[i] = g_xo.next();
            return;
        }
    }
    for (int i = 0; i < 4; i++) w[i] = os_random64();
}
bool below_modulus(const uint32_t* a) {
    for (int i = 7; i >= 0; i--) {
        uint32_t m = grape::FrParams::mod(i);
        if (a[i] < m) return true;
        if (a[i] > m) return false;
    }
    return false;
}
}  // namespace

Fr::Fr(long x) {
    unsigned long ax = x < 0 ? 0ul - (unsigned long)x : (unsigned long)x;
    fr_t raw = grape::Fr::zero();
    raw.v[0] = (uint32_t)ax;
    raw.v[1] = (uint32_t)(ax >> 32);
    v = grape::to_mont(raw);
    if (x < 0) v = grape::neg(v);
}

void Fr::seed(uint64_t s) {
    std::lock_guard<std::mutex> lock(g_rng_mu);
    g_xo.seed(s);
    g_seeded.store(true, std::memory_order_release);
}
void Fr::seed_from_os() {
    std::lock_guard<std::mutex> lock(g_rng_mu);
    g_seeded.store(false, std::memory_order_release);
}
bool Fr::seeded() { return g_seeded.load(std::memory_order_acquire); }

Fr Fr::random_element() {
    for (;;) {
        fr_t raw;
        uint64_t w[4];
        next256(w);
        for (int i = 0; i < 4; i++) {
            raw.v[2 * i] = (uint32_t)w[i];
            raw.v[2 * i + 1] = (uint32_t)(w[i] >> 32);
        }
        raw.v[7] &= 0x7fffffffu;
        if (below_modulus(raw.v)) return Fr(raw);   // a uniform residue read as Montgomery form is uniform
    }
}

// by divsteps (a tenth of the a^(r-2) ladder's time on the host as on the device); 1/0 = 0
Fr& Fr::invert() {
    v = grape::divstep::inverse_by(v);
    return *this;
}

void Fr::to_plain(uint32_t out[8]) const {
    fr_t t = grape::from_mont(v);
    for (int i = 0; i < 8; i++) out[i] = t.v[i];
}

std::ostream& operator<<(std::ostream& os, const Fr& x) {
    uint32_t w[8];
    x.to_plain(w);
    std::ios_base::fmtflags f = os.flags();
    os << "0x";
    for (int i = 7; i >= 0; i--) os << std::hex << std::setw(8) << std::setfill('0') << w[i];
    os.flags(f);
    return os;
}

// ------------------------------------------------------------------ G1
G1::G1(const affine_t& a) {
    if (a.is_inf()) {
        p = grape::G1Jac::inf();
    } else {
        p.x = a.x;
        p.y = a.y;
        p.z = grape::Fp::one();
    }
}

G1 G1::one() {
    affine_t a;
    for (int i = 0; i < grape::FpParams::N; i++) {
        a.x.v[i] = grape::g1_gen_x(i);
        a.y.v[i] = grape::g1_gen_y(i);
    }
    return G1(a);
}

G1 G1::random_element() { return Fr::random_element() * G1::one(); }

affine_t G1::to_affine() const { return grape::jac_to_affine(p); }

G1 G1::operator+(const G1& o) const {
    grape::G1Xyzz a = grape::jac_to_xyzz(p);
    grape::xyzz_add(a, grape::jac_to_xyzz(o.p));
    return G1(grape::xyzz_to_jac(a));
}
G1 G1::operator-() const {
    G1 r(*this);
    r.p.y = grape::neg(r.p.y);
    return r;
}
G1 G1::operator-(const G1& o) const { return *this + (-o); }
G1 G1::dbl() const {
    grape::G1Xyzz a = grape::jac_to_xyzz(p);
    grape::xyzz_dbl(a);
    return G1(grape::xyzz_to_jac(a));
}
bool G1::operator==(const G1& o) const {
    if (is_zero() || o.is_zero()) return is_zero() && o.is_zero();
    // X1*Z2^2 == X2*Z1^2 and Y1*Z2^3 == Y2*Z1^3
    using namespace grape;
    Fp z1 = sqr(p.z), z2 = sqr(o.p.z);
    if (mul(p.x, z2) != mul(o.p.x, z1)) return false;
    return mul(p.y, mul(z2, o.p.z)) == mul(o.p.y, mul(z1, p.z));
}

G1 operator*(const Fr& k, const G1& pt) {
    uint32_t w[8];
    k.to_plain(w);
    grape::G1Xyzz base = grape::jac_to_xyzz(pt.p);
    grape::G1Xyzz acc = grape::G1Xyzz::inf();
    for (int i = 255; i >= 0; i--) {
        grape::xyzz_dbl(acc);
        if ((w[i >> 5] >> (i & 31)) & 1) grape::xyzz_add(acc, base);
    }
    return G1(grape::xyzz_to_jac(acc));
}

G1FixedBase::G1FixedBase(const G1& base) : table_((size_t)kWindows * kPerWindow) {
    grape::G1Xyzz b = grape::jac_to_xyzz(base.p);
    for (int w = 0; w < kWindows; w++) {
        grape::G1Xyzz acc = b;
        for (int k = 1; k <= kPerWindow; k++) {
            table_[(size_t)w * kPerWindow + (k - 1)] = acc;
            grape::xyzz_add(acc, b);                       // after the last entry: 2^kBits * b, the next window's base
        }
        b = acc;
    }
}

G1 G1FixedBase::mul(const Fr& k) const {
    uint32_t w[9];
    k.to_plain(w);
    w[8] = 0;
    grape::G1Xyzz acc = grape::G1Xyzz::inf();
    for (int i = 0; i < kWindows; i++) {
        const int bit = i * kBits;
        const uint64_t two = (uint64_t)w[bit >> 5] | ((uint64_t)w[(bit >> 5) + 1] << 32);
        const uint32_t d = (uint32_t)(two >> (bit & 31)) & (uint32_t)kPerWindow;
        if (d) grape::xyzz_add(acc, table_[(size_t)i * kPerWindow + (d - 1)]);
    }
    return G1(grape::xyzz_to_jac(acc));
}
