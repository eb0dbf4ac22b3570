// G1 kernels: generator derivation, fixed-base tables and the Hyrax row-commitment kernels.
//
// Commitment design (one GPU, 288 GB of HBM): all rows of a matrix are committed against the
// SAME generators, so the work per scalar is bought down with memory — a table of
// k * 2^(c*w) * G_i for every digit value k and window w turns each signed radix-2^c digit into
// exactly one mixed addition into a single per-lane accumulator (no per-window accumulators,
// no doubling chain at the end).  For int16-range weights c = 16 makes that one addition per
// matrix element.  Lanes own columns (coalesced scalar reads), accumulate in extended Jacobian
// (XYZZ) coordinates, and a second kernel folds the 64 lane partials of each row and maps the
// result to affine coordinates.
#define GRAPE_FP_MUL_OUTLINE 1
#include "common.hpp"
#include "commit_geometry.hpp"
#include "fp28.hpp"
#include "fr26.hpp"

namespace grape {

// The one shared body of the Fp multiplier / squarer (about a thousand instructions each, so
// every branch inside stays short-range).
__device__ __noinline__ Fp fp_mul_outline(Fp a, Fp b) { return mul(a, b); }
__device__ __noinline__ Fp fp_sqr_outline(Fp a) { return sqr(a); }

// Memory images in 32-bit words: an Fp element is FW words (12 for BLS12-381, 8 for BN254), an
// affine point 2 FW, a Jacobian point 3 FW, an XYZZ point 4 FW; L28 is the limb count of the
// 28-bit working form.
constexpr int FW = FpParams::N;
constexpr int L28 = fp28::N;

__device__ __forceinline__ Fp ld_fp(const uint32_t* p) {
    const uint4* q = reinterpret_cast<const uint4*>(p);
    Fp r;
#pragma unroll
    for (int i = 0; i < FW / 4; i++) {
        const uint4 a = q[i];
        r.v[4 * i] = a.x; r.v[4 * i + 1] = a.y; r.v[4 * i + 2] = a.z; r.v[4 * i + 3] = a.w;
    }
    return r;
}
__device__ __forceinline__ void st_fp(uint32_t* p, const Fp& a) {
    uint4* q = reinterpret_cast<uint4*>(p);
#pragma unroll
    for (int i = 0; i < FW / 4; i++) q[i] = make_uint4(a.v[4 * i], a.v[4 * i + 1], a.v[4 * i + 2], a.v[4 * i + 3]);
}
__device__ __forceinline__ G1Affine ld_affine(const uint32_t* base, size_t i) {
    G1Affine r;
    r.x = ld_fp(base + 2 * FW * i);
    r.y = ld_fp(base + 2 * FW * i + FW);
    return r;
}
__device__ __forceinline__ void st_affine(uint32_t* base, size_t i, const G1Affine& p) {
    st_fp(base + 2 * FW * i, p.x);
    st_fp(base + 2 * FW * i + FW, p.y);
}
__device__ __forceinline__ G1Xyzz ld_xyzz(const uint32_t* base, size_t i) {
    G1Xyzz r;
    r.x = ld_fp(base + 4 * FW * i);
    r.y = ld_fp(base + 4 * FW * i + FW);
    r.zz = ld_fp(base + 4 * FW * i + 2 * FW);
    r.zzz = ld_fp(base + 4 * FW * i + 3 * FW);
    return r;
}
__device__ __forceinline__ void st_xyzz(uint32_t* base, size_t i, const G1Xyzz& p) {
    st_fp(base + 4 * FW * i, p.x);
    st_fp(base + 4 * FW * i + FW, p.y);
    st_fp(base + 4 * FW * i + 2 * FW, p.zz);
    st_fp(base + 4 * FW * i + 3 * FW, p.zzz);
}
__device__ __forceinline__ Fr ld_fr8(const uint32_t* base, size_t i) {
    const uint4* p = reinterpret_cast<const uint4*>(base) + 2 * i;
    uint4 lo = p[0], hi = p[1];
    Fr r;
    r.v[0] = lo.x; r.v[1] = lo.y; r.v[2] = lo.z; r.v[3] = lo.w;
    r.v[4] = hi.x; r.v[5] = hi.y; r.v[6] = hi.z; r.v[7] = hi.w;
    return r;
}

// Wide-table entry: an affine point in the 28-bit working form, x[L28] then y[L28] as 32-bit
// words.  BLS12-381's 112 bytes are padded to 128, so that every gather is exactly one cache line;
// BN254's 80 bytes are stored dense (a multiple of 16 bytes: the loads stay aligned, half of the
// entries straddle two lines) - the table is 37.5 % smaller, which is what lets 15-bit windows fit
// the table budget there.
constexpr int kWideEntryWords = (2 * L28 <= 20) ? 2 * L28 : 32;
static_assert(kWideEntryWords % 4 == 0 && kWideEntryWords >= 2 * L28, "entry layout");
__device__ __forceinline__ Affine28 ld_entry28(const uint32_t* table, size_t e) {
    const uint4* q = reinterpret_cast<const uint4*>(table + (size_t)kWideEntryWords * e);
    uint4 w[L28 / 2];
#pragma unroll
    for (int i = 0; i < L28 / 2; i++) w[i] = q[i];
    const uint32_t* f = reinterpret_cast<const uint32_t*>(w);
    Affine28 r;
#pragma unroll
    for (int i = 0; i < L28; i++) {
        r.x.v[i] = (int32_t)f[i];
        r.y.v[i] = (int32_t)f[L28 + i];
    }
    return r;
}
__device__ __forceinline__ void st_entry28(uint32_t* table, size_t e, const G1Affine& a) {
    Fp28 x = fp28::from_canonical(a.x), y = fp28::from_canonical(a.y);
    uint32_t f[kWideEntryWords];
#pragma unroll
    for (int i = 0; i < L28; i++) {
        f[i] = (uint32_t)x.v[i];
        f[L28 + i] = (uint32_t)y.v[i];
    }
#pragma unroll
    for (int i = 2 * L28; i < kWideEntryWords; i++) f[i] = 0;
    uint4* q = reinterpret_cast<uint4*>(table + (size_t)kWideEntryWords * e);
#pragma unroll
    for (int i = 0; i < kWideEntryWords / 4; i++) q[i] = make_uint4(f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]);
}
__device__ __forceinline__ bool entry_is_inf(const Affine28& a) {
    uint32_t z = 0;
#pragma unroll
    for (int i = 0; i < L28; i++) z |= (uint32_t)a.x.v[i] | (uint32_t)a.y.v[i];
    return z == 0;
}
// Per-lane partial accumulator in memory: x, y, zz, zzz (L28 words each), the identity flag and
// padding = 64 words (256 bytes).
using geom::kPartialWords;
__device__ __forceinline__ void st_partial28(uint32_t* base, size_t i, const Xyzz28& a) {
    uint32_t f[64];
#pragma unroll
    for (int k = 0; k < L28; k++) {
        f[k] = (uint32_t)a.x.v[k];
        f[L28 + k] = (uint32_t)a.y.v[k];
        f[2 * L28 + k] = (uint32_t)a.zz.v[k];
        f[3 * L28 + k] = (uint32_t)a.zzz.v[k];
    }
    f[4 * L28] = a.inf ? 1u : 0u;
#pragma unroll
    for (int k = 4 * L28 + 1; k < 64; k++) f[k] = 0;
    uint4* q = reinterpret_cast<uint4*>(base + geom::partial_word(i));
#pragma unroll
    for (int k = 0; k < 16; k++) q[k] = make_uint4(f[4 * k], f[4 * k + 1], f[4 * k + 2], f[4 * k + 3]);
}
__device__ __forceinline__ Xyzz28 ld_partial28(const uint32_t* base, size_t i) {
    const uint4* q = reinterpret_cast<const uint4*>(base + geom::partial_word(i));
    uint4 w[L28 + 1];
#pragma unroll
    for (int k = 0; k < L28 + 1; k++) w[k] = q[k];
    const uint32_t* f = reinterpret_cast<const uint32_t*>(w);
    Xyzz28 a;
#pragma unroll
    for (int k = 0; k < L28; k++) {
        a.x.v[k] = (int32_t)f[k];
        a.y.v[k] = (int32_t)f[L28 + k];
        a.zz.v[k] = (int32_t)f[2 * L28 + k];
        a.zzz.v[k] = (int32_t)f[3 * L28 + k];
    }
    a.inf = f[4 * L28] != 0;
    return a;
}
__device__ __forceinline__ Xyzz28 shfl_down_xyzz28(const Xyzz28& a, int off) {
    Xyzz28 r;
#pragma unroll
    for (int k = 0; k < L28; k++) {
        r.x.v[k] = __shfl_down(a.x.v[k], off, 64);
        r.y.v[k] = __shfl_down(a.y.v[k], off, 64);
        r.zz.v[k] = __shfl_down(a.zz.v[k], off, 64);
        r.zzz.v[k] = __shfl_down(a.zzz.v[k], off, 64);
    }
    r.inf = __shfl_down((int)a.inf, off, 64) != 0;
    return r;
}
// acc += q for two 28-bit accumulators, exceptional cases through the canonical-form addition
__device__ __forceinline__ void padd28(Xyzz28& acc, const Xyzz28& q) {
    if (!xyzz28_add(acc, q)) {
        G1Xyzz c = xyzz28_to_canonical(acc);
        xyzz_add(c, xyzz28_to_canonical(q));
        acc = xyzz28_from_canonical(c);
    }
}

// acc += +-entry through the 28-bit mixed addition; the rare exceptional step (entry = +-acc)
// goes through the exact canonical-form addition.
__device__ __forceinline__ void madd28(Xyzz28& acc, const Affine28& e, bool negate) {
    if (entry_is_inf(e)) return;
    if (!xyzz28_madd(acc, e, negate)) {
        G1Xyzz c = xyzz28_to_canonical(acc);
        G1Affine a;
        a.x = fp28::to_canonical(e.x);
        a.y = fp28::to_canonical(e.y);
        xyzz_add_affine(c, a, negate);
        acc = xyzz28_from_canonical(c);
    }
}

// acc += k * G_col for a canonical (non-Montgomery) 255-bit scalar k: signed radix-2^c digits,
// one gather and one mixed addition per non-zero digit.
// One signed radix-2^c digit of a canonical scalar: window w, incoming carry -> magnitude, sign,
// outgoing carry.
__device__ __forceinline__ uint32_t fr_digit(const Fr& k, uint32_t w, uint32_t c, uint32_t& carry, bool& neg) {
    const uint32_t half = 1u << (c - 1), mask = (1u << c) - 1u;
    const uint32_t bit = w * c;
    // c <= 16 bits starting at `bit`, possibly straddling two limbs
    const uint32_t limb = bit >> 5, sh = bit & 31;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        lo = (q == (int)limb) ? k.v[q] : lo;
        hi = (q == (int)limb + 1) ? k.v[q] : hi;
    }
    const uint64_t both = ((uint64_t)hi << 32) | lo;
    const uint32_t d = ((uint32_t)(both >> sh) & mask) + carry;
    neg = d > half;                      // digit in (half, 2^c] -> d - 2^c, carry 1
    carry = neg ? 1u : 0u;
    return neg ? (mask + 1u - d) : d;
}

// acc += k * G_col through the wide table: one gather and one mixed addition per non-zero digit.
// While the addition of digit w runs, the table line of digit w+1 is already on its way (one
// word of it is touched right after the entry of digit w has been requested).
__device__ __forceinline__ void madd_scalar_fr(Xyzz28& acc, const Fr& k_in, const uint32_t* table, size_t N, uint32_t col,
                                               uint32_t c, uint32_t nw, uint32_t K, int* err_flag) {
    // The scalar is taken as +-|k| with |k| <= (r-1)/2 < 2^254 (r - k and the negated point when k is
    // in the upper half): the top window then never carries out, and nw = ceil(255/c) windows are
    // enough - one addition fewer per scalar at c = 15.
    Fr k = k_in;
    uint32_t borrow = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t half_i = (FrParams::mod(i) >> 1) | (i + 1 < 8 ? FrParams::mod(i + 1) << 31 : 0u);
        const uint64_t t = (uint64_t)half_i - (uint64_t)k.v[i] - (uint64_t)borrow;
        borrow = (uint32_t)(t >> 63);
    }
    const bool flip = borrow != 0;                        // k > (r-1)/2
    k = cneg(k, flip);
    uint32_t nwin = nw;
    while (nwin > 0 && (nwin - 1) * c >= 256) nwin--;     // windows that start inside the scalar
    uint32_t carry = 0;
    bool neg = false;
    uint32_t mag = nwin ? fr_digit(k, 0, c, carry, neg) : 0;
    uint32_t touch = 0;
    for (uint32_t w = 0; w < nwin; w++) {
        bool neg_n = false;
        const uint32_t mag_n = (w + 1 < nwin) ? fr_digit(k, w + 1, c, carry, neg_n) : 0;
        if (mag != 0) {
            if (mag > K) {
                *err_flag = 1;
            } else {
                const Affine28 e = ld_entry28(table, geom::table_entry(w, K, mag, N, col));
                // unconditional, so that the compiler counts the outstanding loads exactly
                const size_t nxt = (mag_n != 0 && mag_n <= K) ? geom::table_entry(w + 1, K, mag_n, N, col) : (size_t)col;
                touch = table[(size_t)kWideEntryWords * nxt];
                if (kWideEntryWords % 32 != 0) touch |= table[(size_t)kWideEntryWords * nxt + kWideEntryWords - 1];   // dense entries: both lines
                madd28(acc, e, neg != flip);
            }
        }
        mag = mag_n;
        neg = neg_n;
    }
    asm volatile("" ::"v"(touch));      // keeps the last touch alive until here
    if (carry) *err_flag = 1;   // cannot happen for canonical scalars when nw*c >= 255
}

__device__ __forceinline__ G1Xyzz shfl_down_xyzz(const G1Xyzz& a, int off) {
    G1Xyzz r;
#pragma unroll
    for (int i = 0; i < FW; i++) {
        r.x.v[i] = __shfl_down(a.x.v[i], off, 64);
        r.y.v[i] = __shfl_down(a.y.v[i], off, 64);
        r.zz.v[i] = __shfl_down(a.zz.v[i], off, 64);
        r.zzz.v[i] = __shfl_down(a.zzz.v[i], off, 64);
    }
    return r;
}

// The group operations are always inlined into the kernels; only the Fp multiplier and squarer
// are out-of-line.  An out-of-line device function large enough to need far branches is not
// safe: the compiler's far-branch expansion inside a non-kernel function borrows s[30:31] - the
// return address - so such a function never returns once the far path is taken (seen in the
// generated code of an out-of-line mixed addition: the "accumulator is at infinity for every
// active lane" path jumped through s[30:31] and the final s_setpc_b64 s[30:31] then looped
// forever).  Kernels have no return address to lose, and the multiplier body is far below the
// +-128 KiB range of a short branch.
__device__ __forceinline__ void madd(G1Xyzz& acc, const G1Affine& p, bool negate) { xyzz_add_affine(acc, p, negate); }
__device__ __forceinline__ void padd(G1Xyzz& acc, const G1Xyzz& q) { xyzz_add(acc, q); }
__device__ __forceinline__ void pdbl(G1Xyzz& acc) { xyzz_dbl(acc); }
// 1/a for a canonical, non-zero a: through the 28-bit form and its divstep inversion (about ten
// thousand instructions) instead of the a^(p-2) ladder on saturated limbs (about six hundred thousand)
__device__ __forceinline__ Fp fp_inverse_fast(const Fp& a) {
    return fp28::to_canonical(fp28::inverse_by(fp28::from_canonical_lazy(a)));
}
__device__ __forceinline__ G1Affine to_affine(const G1Xyzz& p) {
    if (p.is_inf()) return G1Affine::inf();
    return xyzz_to_affine_with_inv(p, fp_inverse_fast(p.zzz));
}

// k * P for a 256-bit canonical scalar held in 8 limbs
__device__ __forceinline__ G1Xyzz scalar_mul(const G1Affine& p, const uint32_t* k, int top_bit) {
    G1Xyzz acc = G1Xyzz::inf();
    for (int i = top_bit; i >= 0; i--) {
        pdbl(acc);
        if ((k[i >> 5] >> (i & 31)) & 1) madd(acc, p, false);
    }
    return acc;
}

__global__ void __launch_bounds__(64) scalar_mul_base_kernel(uint32_t* out, const uint32_t* k, const uint32_t* base, size_t n) {
    size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n) return;
    uint32_t kk[8];
#pragma unroll
    for (int j = 0; j < 8; j++) kk[j] = k[8 * i + j];
    G1Affine p = ld_affine(base, 0);
    st_affine(out, i, to_affine(scalar_mul(p, kk, 255)));
}

// bases[w*N + i] = 2^(c*w) * G_i, affine
__global__ void __launch_bounds__(64) window_bases_kernel(uint32_t* bases, const uint32_t* gens, size_t N, uint32_t c, uint32_t nw) {
    size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= N) return;
    G1Affine g = ld_affine(gens, i);
    st_affine(bases, i, g);
    G1Xyzz cur = G1Xyzz::from_affine(g);
    for (uint32_t w = 1; w < nw; w++) {
        for (uint32_t d = 0; d < c; d++) pdbl(cur);
        st_affine(bases, (size_t)w * N + i, to_affine(cur));
    }
}

// One thread per (window w, generator i, chunk j): XYZZ multiples k*B for k = j*CH+1 .. j*CH+CH
// (clipped to K) into tmp[((j - j0)*CH + t) * (nw*N) + w*N + i].
__global__ void __launch_bounds__(64) wide_chain_kernel(uint32_t* tmp, const uint32_t* bases, size_t N, uint32_t nw, uint32_t K,
                                                        uint32_t CH, uint32_t j0, uint32_t nj) {
    size_t tid = (size_t)blockIdx.x * 64 + threadIdx.x;
    size_t per_chunk = (size_t)nw * N;
    if (tid >= per_chunk * nj) return;
    uint32_t jj = (uint32_t)(tid / per_chunk);
    size_t wi = tid - (size_t)jj * per_chunk;       // w*N + i
    uint32_t j = j0 + jj;
    G1Affine B = ld_affine(bases, wi);
    uint32_t kstart[8] = {j * CH + 1, 0, 0, 0, 0, 0, 0, 0};
    G1Xyzz acc = scalar_mul(B, kstart, 31 - __clz((int)kstart[0]));
    for (uint32_t t = 0; t < CH; t++) {
        uint32_t k = j * CH + 1 + t;
        if (k > K) break;
        st_xyzz(tmp, ((size_t)jj * CH + t) * per_chunk + wi, acc);
        madd(acc, B, false);
    }
}

// Batched XYZZ -> affine (Montgomery's trick over 8 entries per thread, strided so that lanes
// stay adjacent).  Entry e of tmp goes to dst[map(e)] where, for the wide table,
// e = (jj*CH + t)*(nw*N) + w*N + i  ->  ((w*K) + (j0*CH + jj*CH + t))*N + i.
constexpr int kNormChunk = 8;
__global__ void __launch_bounds__(64) wide_normalize_kernel(uint32_t* table, const uint32_t* tmp, size_t N, uint32_t nw, uint32_t K,
                                                            uint32_t CH, uint32_t j0, size_t n_entries) {
    size_t t0 = (size_t)blockIdx.x * 64 + threadIdx.x;
    size_t nthreads = (n_entries + kNormChunk - 1) / kNormChunk;
    if (t0 >= nthreads) return;
    Fp pre[kNormChunk];
    Fp acc = Fp::one();
#pragma unroll
    for (int k = 0; k < kNormChunk; k++) {
        size_t e = t0 + (size_t)k * nthreads;
        pre[k] = acc;
        if (e < n_entries) {
            Fp zzz = ld_fp(tmp + 4 * FW * e + 3 * FW);
            if (!zzz.is_zero()) acc = fmul(acc, zzz);
        }
    }
    Fp inv = fp_inverse_fast(acc);
    const size_t per_chunk = (size_t)nw * N;
#pragma unroll
    for (int k = kNormChunk - 1; k >= 0; k--) {
        size_t e = t0 + (size_t)k * nthreads;
        if (e >= n_entries) continue;
        G1Xyzz p = ld_xyzz(tmp, e);
        size_t kk = e / per_chunk;                  // jj*CH + t
        size_t wi = e - kk * per_chunk;
        size_t w = wi / N, i = wi - w * N;
        size_t kidx = (size_t)j0 * CH + kk;         // k - 1
        if (kidx >= K) continue;
        G1Affine a = G1Affine::inf();
        if (!p.zzz.is_zero()) {
            Fp zi = fmul(inv, pre[k]);
            inv = fmul(inv, p.zzz);
            a = xyzz_to_affine_with_inv(p, zi);
        }
        st_entry28(table, (w * K + kidx) * N + i, a);
    }
}

// ------------------------------------------------------------------------------------------------
// Table generation by levels: once the multiples 1..have of every base are in the table, the next
// cnt <= have are E[have + k] = E[k] + E[have] (k = have is the doubling of E[have]) - additions
// of two AFFINE entries that are already final, all independent.  An affine addition is 3M + 1S
// once the inverse of its slope's denominator is known, and Montgomery's trick shares one
// inversion over a thread's run of consecutive k: a forward pass multiplies the denominators up,
// parking every prefix product in the destination entry it belongs to (free until the backward
// pass fills it), one divstep inversion, and a backward pass that peels the inverses off and
// writes the sums.  About 6 products and 0.5 KB of traffic per entry, where a chain of mixed
// XYZZ additions plus the normalisation of every entry costs 17 products and an inversion per 8.
// A run whose denominators multiply to zero (a base that is the identity or has small order: no
// generator of the prime-order group) raises *degenerate and leaves its entries to
// wide_extend_exact_kernel.
// ------------------------------------------------------------------------------------------------
constexpr uint32_t kExtendRun = 64;   // additions that share one inversion
constexpr uint32_t kFirstChain = 16;  // multiples of a base made by the chain of mixed additions before the levels start
constexpr int kFp28Quads = (L28 + 3) / 4;
__device__ __forceinline__ Fp28 ld_fp28(const uint32_t* p) {
    const uint4* q = reinterpret_cast<const uint4*>(p);
    uint4 w[kFp28Quads];
#pragma unroll
    for (int i = 0; i < kFp28Quads; i++) w[i] = q[i];
    const uint32_t* f = reinterpret_cast<const uint32_t*>(w);
    Fp28 r;
#pragma unroll
    for (int i = 0; i < L28; i++) r.v[i] = (int32_t)f[i];
    return r;
}
__device__ __forceinline__ void st_fp28(uint32_t* p, const Fp28& a) {
    uint32_t f[4 * kFp28Quads];
#pragma unroll
    for (int i = 0; i < 4 * kFp28Quads; i++) f[i] = i < L28 ? (uint32_t)a.v[i] : 0u;
    uint4* q = reinterpret_cast<uint4*>(p);
#pragma unroll
    for (int i = 0; i < kFp28Quads; i++) q[i] = make_uint4(f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]);
}
static_assert(4 * kFp28Quads <= kWideEntryWords, "a prefix product must fit the entry it is parked in");
__device__ __forceinline__ void st_entry28_raw(uint32_t* table, size_t e, const Affine28& a) {
    uint32_t f[kWideEntryWords];
#pragma unroll
    for (int i = 0; i < L28; i++) {
        f[i] = (uint32_t)a.x.v[i];
        f[L28 + i] = (uint32_t)a.y.v[i];
    }
#pragma unroll
    for (int i = 2 * L28; i < kWideEntryWords; i++) f[i] = 0;
    uint4* q = reinterpret_cast<uint4*>(table + (size_t)kWideEntryWords * e);
#pragma unroll
    for (int i = 0; i < kWideEntryWords / 4; i++) q[i] = make_uint4(f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]);
}

// One thread per (run of `run` consecutive k, window w, generator i); i is the fastest index, so a
// wave reads and writes adjacent entries.
__global__ void __launch_bounds__(kBlock) wide_extend_kernel(uint32_t* table, size_t N, uint32_t nw, uint32_t K, uint32_t have,
                                                             uint32_t cnt, uint32_t run, int* degenerate) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t per = (size_t)nw * N;
    const uint32_t nruns = (cnt + run - 1) / run;
    if (t >= per * nruns) return;
    const uint32_t r = (uint32_t)(t / per);
    const size_t wi = t - (size_t)r * per;
    const size_t w = wi / N, i = wi - w * N;
    const uint32_t k0 = r * run + 1;                              // first k of the run
    const uint32_t k1 = k0 + run < cnt + 1 ? k0 + run : cnt + 1;  // one past its last
    const size_t e0 = w * K * N + i;                              // entry of the multiple k: e0 + (k-1) N
    const Affine28 f = ld_entry28(table, e0 + (size_t)(have - 1) * N);
    bool bad = entry_is_inf(f);
    Fp28 acc = fp28::one();
    for (uint32_t k = k0; k < k1; k++) {
        const Affine28 e = ld_entry28(table, e0 + (size_t)(k - 1) * N);
        bad |= entry_is_inf(e);
        st_fp28(table + (size_t)kWideEntryWords * (e0 + (size_t)(have + k - 1) * N), acc);
        acc = fp28::mul(acc, affine28_slope_den(e, f, k == have));
    }
    bad |= fp28::is_zero_mod_p(acc);
    if (bad) {
        *degenerate = 1;
        return;
    }
    Fp28 inv = fp28::inverse_by(acc);
    for (uint32_t k = k1 - 1; k >= k0; k--) {
        const size_t dst = e0 + (size_t)(have + k - 1) * N;
        const Affine28 e = ld_entry28(table, e0 + (size_t)(k - 1) * N);
        const Fp28 dinv = fp28::mul(inv, ld_fp28(table + (size_t)kWideEntryWords * dst));
        inv = fp28::mul(inv, affine28_slope_den(e, f, k == have));
        st_entry28_raw(table, dst, affine28_add_given_inverse(e, f, k == have, dinv));
    }
}

// The same level through the general addition, one thread per entry, every exceptional case
// handled (identity, equal and opposite points): runs only when the level met a degenerate run.
__global__ void __launch_bounds__(64) wide_extend_exact_kernel(uint32_t* table, size_t N, uint32_t nw, uint32_t K, uint32_t have,
                                                               uint32_t cnt, const int* degenerate) {
    if (*degenerate == 0) return;
    const size_t per = (size_t)nw * N;
    for (size_t t = (size_t)blockIdx.x * 64 + threadIdx.x; t < per * cnt; t += (size_t)gridDim.x * 64) {
        const uint32_t k = (uint32_t)(t / per) + 1;
        const size_t wi = t - (size_t)(k - 1) * per;
        const size_t w = wi / N, i = wi - w * N;
        const size_t e0 = w * K * N + i;
        Xyzz28 acc = xyzz28_inf();
        madd28(acc, ld_entry28(table, e0 + (size_t)(k - 1) * N), false);
        madd28(acc, ld_entry28(table, e0 + (size_t)(have - 1) * N), false);
        st_entry28(table, e0 + (size_t)(have + k - 1) * N, xyzz28_to_affine(acc));
    }
}

// Reference-format table from a one-window wide table over the generators i0 .. i0+ns:
// out[w*N + i0 + i] = w * G_(i0+i) in the canonical memory form (w = 0: the identity), one product
// per coordinate to change the limb form and the Montgomery radix.
__global__ void __launch_bounds__(kBlock) ref_from_wide_kernel(uint32_t* out, const uint32_t* wide, size_t N, size_t i0, size_t ns, uint32_t W) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= ns * W) return;
    const size_t w = t / ns, i = t - w * ns;
    G1Affine a = G1Affine::inf();
    if (w > 0) {
        const Affine28 e = ld_entry28(wide, (w - 1) * ns + i);
        a.x = fp28::to_canonical(e.x);
        a.y = fp28::to_canonical(e.y);
    }
    st_affine(out, w * N + i0 + i, a);
}

// ------------------------------------------------------------------------------------------------
// commitment, wide table
// ------------------------------------------------------------------------------------------------
// Each wave owns one row segment of `seg` columns; lane l takes columns l, l+64, ...
// partial[(row*nseg + s)*64 + lane] receives the lane's XYZZ accumulator.
template <bool FR>
__global__ void __launch_bounds__(kBlock) commit_wide_kernel(uint32_t* partial, const void* scalars, uint32_t rowlen, size_t rows,
                                                             uint32_t seg, uint32_t nseg, const uint32_t* table, size_t N,
                                                             uint32_t c, uint32_t nw, uint32_t K, int* err_flag) {
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
    if (wave >= rows * nseg) return;
    const geom::WaveSpan span = geom::wave_span(wave, nseg, seg, rowlen);
    const size_t row = span.row;
    const uint32_t s = span.s, col_end = span.col_end;
    const uint32_t half = 1u << (c - 1), mask = (c == 32) ? 0xffffffffu : ((1u << c) - 1u);
    Xyzz28 acc = xyzz28_inf();
    // int path: the scalars of the next two columns are kept in flight (the next one addresses
    // the table line to touch, the one after is being loaded)
    int32_t sc1 = 0, sc2 = 0;
    if (!FR) {
        const uint32_t c0 = s * seg + lane;
        if (c0 + 64 < col_end) sc1 = ((const int32_t*)scalars)[geom::scalar_index(row, rowlen, c0 + 64)];
        if (c0 + 128 < col_end) sc2 = ((const int32_t*)scalars)[geom::scalar_index(row, rowlen, c0 + 128)];
    }
    int32_t sc0 = (!FR && s * seg + lane < col_end) ? ((const int32_t*)scalars)[geom::scalar_index(row, rowlen, s * seg + lane)] : 0;
    // destination of the look-ahead touches: one register for the whole loop, read only after it.  (Declared
    // inside the loop it is free again at the top of the next iteration, the compiler reuses it for an
    // address there and has to wait for every outstanding load first - 1.5 % of the kernel's time.)
    uint32_t touch = 0;
    for (uint32_t col = s * seg + lane; col < col_end; col += 64) {
        if (FR) {
            const Fr k = from_mont(ld_fr8((const uint32_t*)scalars, geom::scalar_index(row, rowlen, col)));
            madd_scalar_fr(acc, k, table, N, col, c, nw, K, err_flag);
        } else {
            int64_t v = sc0;
            const int64_t v_next = sc1;
            sc0 = sc1;
            sc1 = sc2;
            sc2 = (col + 192 < col_end) ? ((const int32_t*)scalars)[geom::scalar_index(row, rowlen, col + 192)] : 0;
            // The table line of the NEXT column's first digit is touched (one word) right after
            // this column's own entry is requested, so that it is in cache when its turn comes:
            // with two waves per SIMD an exposed HBM round trip per addition costs issue slots.
            // (the touch is unconditional - a column without a successor touches its own first
            // table line - because the compiler counts outstanding loads exactly only in
            // straight-line code; a conditional load after the entry's would make it wait for both)
            size_t next_entry = col;
            bool have_next = false;
            if (col + 64 < col_end) {
                int64_t vn = v_next;
                int64_t dn = vn & (int64_t)mask;
                vn >>= c;
                if (dn > (int64_t)half || (dn == (int64_t)half && vn < 0)) dn -= (int64_t)mask + 1;
                const uint32_t magn = (uint32_t)(dn < 0 ? -dn : dn);
                have_next = magn != 0 && magn <= K;
                if (have_next) next_entry = geom::table_entry(0, K, magn, N, col + 64);
            }
            const uint32_t* touch_ptr = table + (size_t)kWideEntryWords * next_entry;
            for (uint32_t w = 0; w < nw; w++) {
                int64_t d = v & (int64_t)mask;
                v >>= c;                            // arithmetic shift keeps the sign
                // digits above half go negative with a carry; exactly half goes negative only
                // when what remains is negative (so that -2^(c-1) recodes to one digit)
                if (d > (int64_t)half || (d == (int64_t)half && v < 0)) {
                    d -= (int64_t)mask + 1;
                    v += 1;
                }
                const bool neg = d < 0;
                const uint32_t mag = (uint32_t)(neg ? -d : d);
                if (mag != 0) {
                    if (mag > K) { *err_flag = 1; continue; }
                    const Affine28 e = ld_entry28(table, geom::table_entry(w, K, mag, N, col));
                    touch = *touch_ptr;
                    if (kWideEntryWords % 32 != 0) touch |= touch_ptr[kWideEntryWords - 1];   // dense entries: both lines
                    madd28(acc, e, neg);
                }
            }
            if (v != 0) *err_flag = 1;              // scalar does not fit nw windows
        }
    }
    asm volatile("" ::"v"(touch));                  // keeps the touches alive until here
    st_partial28(partial, wave * 64 + lane, acc);
}

// Scaled table: out[t*ncols + i] = s_t * G_i for a short list of scalars s_t (Montgomery Fr).
// Stage 1 leaves XYZZ points (canonical form) in tmp[(t - t0)*ncols + i]; stage 2 normalises
// 8 per thread and writes 128-byte working-form entries.
__global__ void __launch_bounds__(kBlock) scaled_chain_kernel(uint32_t* tmp, const uint32_t* scalars, size_t t0, size_t nt,
                                                              size_t ncols, const uint32_t* table, size_t N, uint32_t c,
                                                              uint32_t nw, uint32_t K, int* err_flag) {
    size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (tid >= nt * ncols) return;
    const size_t tt = tid / ncols;
    const uint32_t col = (uint32_t)(tid - tt * ncols);
    const Fr k = from_mont(ld_fr8(scalars, t0 + tt));
    Xyzz28 acc = xyzz28_inf();
    madd_scalar_fr(acc, k, table, N, col, c, nw, K, err_flag);
    st_xyzz(tmp, tid, xyzz28_to_canonical(acc));
}
__global__ void __launch_bounds__(64) scaled_normalize_kernel(uint32_t* out, const uint32_t* tmp, size_t e0, size_t n_entries) {
    size_t t0 = (size_t)blockIdx.x * 64 + threadIdx.x;
    size_t nthreads = (n_entries + kNormChunk - 1) / kNormChunk;
    if (t0 >= nthreads) return;
    Fp pre[kNormChunk];
    Fp acc = Fp::one();
#pragma unroll
    for (int k = 0; k < kNormChunk; k++) {
        size_t e = t0 + (size_t)k * nthreads;
        pre[k] = acc;
        if (e < n_entries) {
            Fp zzz = ld_fp(tmp + 4 * FW * e + 3 * FW);
            if (!zzz.is_zero()) acc = fmul(acc, zzz);
        }
    }
    Fp inv = fp_inverse_fast(acc);
#pragma unroll
    for (int k = kNormChunk - 1; k >= 0; k--) {
        size_t e = t0 + (size_t)k * nthreads;
        if (e >= n_entries) continue;
        G1Xyzz p = ld_xyzz(tmp, e);
        G1Affine a = G1Affine::inf();
        if (!p.zzz.is_zero()) {
            Fp zi = fmul(inv, pre[k]);
            inv = fmul(inv, p.zzz);
            a = xyzz_to_affine_with_inv(p, zi);
        }
        st_entry28(out, e0 + e, a);
    }
}

// ------------------------------------------------------------------------------------------------
// commitment, strided table (full-width scalars)
// ------------------------------------------------------------------------------------------------
// A per-window table spends its bytes on ceil(255/c) sets of 2^(c-1) multiples.  Keeping only every
// J-th set - entries k * 2^(c J q) * G_i for q < nsets = ceil(nw / J) - leaves room for wider windows
// within the same bytes: window w = q J + j is looked up in set q, and the J residues j get their own
// sums A_j, combined per row as sum_j 2^(c j) A_j by a Horner chain of (J - 1) c doublings.  With
// 4096 generators c = 16, J = 4 is 16 additions per scalar from 68 GB where the per-window table
// gives 19 from 82 GB; with 262144 generators c = 12, J = 22 (one set, 68 GB) is 22 additions where
// no per-window table above c = 8 fits.
//
// Digits are taken carry-free: with H = sum_w 2^(c w + c - 1), digit_w = ((k + H) >> c w mod 2^c) - 2^(c-1)
// lies in [-2^(c-1), 2^(c-1)) and sum_w digit_w 2^(c w) = k, so any window can be read on its own.
// One wave per (row, residue, column segment); lanes own columns.
__device__ __forceinline__ uint32_t window_bits(const Fr& k, uint32_t w, uint32_t c) {
    const uint32_t bit = w * c, limb = bit >> 5, sh = bit & 31;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        lo = (q == (int)limb) ? k.v[q] : lo;
        hi = (q == (int)limb + 1) ? k.v[q] : hi;
    }
    const uint64_t both = ((uint64_t)hi << 32) | lo;
    return (uint32_t)(both >> sh) & ((1u << c) - 1u);
}
// The bias H restricted to the bits a 256-bit word can hold: bit (c w + c - 1) for every window whose
// top bit lies below 256 (a window that reaches past bit 255 keeps its digit unsigned: see digit_of).
__device__ __forceinline__ Fr window_bias(uint32_t c, uint32_t nw) {
    Fr h = Fr::zero();
    for (uint32_t w = 0; w < nw; w++) {
        const uint32_t pos = w * c + c - 1;
#pragma unroll
        for (int i = 0; i < 8; i++) h.v[i] |= ((pos >> 5) == (uint32_t)i) ? (1u << (pos & 31)) : 0u;
    }
    return h;
}
// |k| + H for the half-range representative of a Montgomery-form scalar; flip = the scalar was negated.
// |k| <= (r-1)/2 < 0.91 * 2^254 and H < 1.01 * 2^255, so the sum stays below 2^256.
__device__ __forceinline__ Fr biased_half_range(const Fr& k_mont, const Fr& H, bool& flip) {
    Fr k = fr26::from_montc(k_mont);
    uint32_t borrow = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t half_i = (FrParams::mod(i) >> 1) | (i + 1 < 8 ? FrParams::mod(i + 1) << 31 : 0u);
        (void)detail::sbb32(half_i, k.v[i], borrow);
    }
    flip = borrow != 0;                                   // k > (r-1)/2
    k = cneg(k, flip);
    uint32_t carry = 0;
    Fr out;
#pragma unroll
    for (int i = 0; i < 8; i++) out.v[i] = detail::adc32(k.v[i], H.v[i], carry);
    return out;
}
// signed digit of window w of a biased scalar: in [-2^(c-1), 2^(c-1)) (unsigned, below 2^(256 - c w), for
// a top window whose bias bit does not exist)
__device__ __forceinline__ int32_t digit_of(const Fr& kb, uint32_t w, uint32_t c) {
    const int32_t bits = (int32_t)window_bits(kb, w, c);
    return (w * c + c - 1 < 256) ? bits - (int32_t)(1u << (c - 1)) : bits;
}

__global__ void __launch_bounds__(kBlock) commit_strided_kernel(uint32_t* partial, const uint32_t* scalars, uint32_t rowlen, size_t rows,
                                                                uint32_t seg, uint32_t nseg, const uint32_t* table, size_t N,
                                                                uint32_t c, uint32_t nw, uint32_t K, uint32_t J, uint32_t nsets) {
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
    if (wave >= rows * J * nseg) return;
    const geom::WaveSpan span = geom::wave_span(wave, nseg, seg, rowlen);   // "row" here is (row, residue)
    const size_t row = span.row / J;
    const uint32_t j = (uint32_t)(span.row - row * J);
    const Fr H = window_bias(c, nw);                      // wave-uniform
    Xyzz28 acc = xyzz28_inf();
    for (uint32_t col = span.s * seg + lane; col < span.col_end; col += 64) {
        bool flip;
        const Fr kb = biased_half_range(ld_fr8(scalars, geom::scalar_index(row, rowlen, col)), H, flip);
        // digit of set 0 now, the next set's one addition ahead (its table line is touched early)
        int32_t d = j < nw ? digit_of(kb, j, c) : 0;
        uint32_t touch = 0;
        for (uint32_t q = 0; q < nsets; q++) {
            const uint32_t wn = (q + 1) * J + j;
            const int32_t d_n = (q + 1 < nsets && wn < nw) ? digit_of(kb, wn, c) : 0;
            if (d != 0) {
                const bool neg = d < 0;
                const uint32_t mag = (uint32_t)(neg ? -d : d);
                const Affine28 e = ld_entry28(table, geom::table_entry(q, K, mag, N, col));
                const uint32_t mag_n = (uint32_t)(d_n < 0 ? -d_n : d_n);
                const size_t nxt = mag_n != 0 ? geom::table_entry(q + 1, K, mag_n, N, col) : (size_t)col;
                touch = table[(size_t)kWideEntryWords * nxt];
                if (kWideEntryWords % 32 != 0) touch |= table[(size_t)kWideEntryWords * nxt + kWideEntryWords - 1];
                madd28(acc, e, neg != flip);
            }
            d = d_n;
        }
        asm volatile("" ::"v"(touch));
    }
    st_partial28(partial, wave * 64 + lane, acc);
}

// total_row = sum_j 2^(c j) A[row * J + j] by Horner from the top residue down, then affine
__global__ void __launch_bounds__(64) strided_horner_kernel(uint32_t* out, const uint32_t* sums, size_t rows, uint32_t J, uint32_t c) {
    const size_t row = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (row >= rows) return;
    Xyzz28 total = ld_partial28(sums, row * J + (J - 1));
    for (int j = (int)J - 2; j >= 0; j--) {
        for (uint32_t d = 0; d < c; d++) xyzz28_dbl(total);
        padd28(total, ld_partial28(sums, row * J + j));
    }
    st_affine(out, row, xyzz28_to_affine(total));
}

// ------------------------------------------------------------------------------------------------
// commitment of the few elements of a tensor that a flag array lets through (full-width scalars)
// ------------------------------------------------------------------------------------------------
// G lanes per row, 64 / G rows per wave.  Every lane group sweeps its row's flags G columns at a
// time and queues the columns whose flag is zero in LDS; whenever some group has G queued (and once
// more at the end of the rows) every lane takes one queued column of its row, loads its scalar and
// adds scalar * G_col through the per-window table.  Lanes therefore work on dense batches however
// thinly the live elements are spread: sweeping the whole tensor with the dense kernel costs a
// recoding per element and an addition slot per WAVE that holds one live element - 80 ms for 2^27
// elements of which 0.7 % are live, against 3 ms here.  With many rows G = 32: a row of 4096 with
// 27 live elements fills 27 of 32 lanes of its batch instead of 27 of 64.
template <int G>
__global__ void __launch_bounds__(64) commit_sparse_fr_kernel(uint32_t* partial, const uint32_t* scalars, const int32_t* __restrict__ skip,
                                                              uint32_t rowlen, size_t rows, const uint32_t* table, size_t N,
                                                              uint32_t c, uint32_t nw, uint32_t K, int* err_flag) {
    constexpr int R = 64 / G;                            // rows per wave
    __shared__ uint32_t queue[R][2 * G];
    const int lane = threadIdx.x;
    const int grp = lane / G, sub = lane % G;
    const size_t row = (size_t)blockIdx.x * R + grp;
    const bool have_row = row < rows;
    const unsigned long long gmask = (G == 64 ? ~0ull : ((1ull << (G & 63)) - 1ull)) << (grp * G);
    Xyzz28 acc = xyzz28_inf();
    uint32_t qn = 0;                                     // queued columns of this lane's row (uniform within the group)
    for (uint32_t base = 0;; base += G) {
        const bool last = base >= rowlen;
        if (!last) {
            const uint32_t col = base + sub;
            const bool take = have_row && col < rowlen && skip[geom::scalar_index(row, rowlen, col)] == 0;
            const unsigned long long m = __ballot(take) & gmask;
            if (take) queue[grp][qn + __popcll(m & ((1ull << lane) - 1ull))] = col;
            qn += (uint32_t)__popcll(m);
            __syncthreads();
        }
        // wave-uniform trigger: some group's batch is full, or the rows have ended with something queued
        const bool go = last ? __any(qn > 0) : __any(qn >= (uint32_t)G);
        if (go) {
            const uint32_t n = qn < (uint32_t)G ? qn : (uint32_t)G;
            if ((uint32_t)sub < n) {
                const uint32_t col = queue[grp][sub];
                const Fr k = from_mont(ld_fr8(scalars, geom::scalar_index(row, rowlen, col)));
                madd_scalar_fr(acc, k, table, N, col, c, nw, K, err_flag);
            }
            __syncthreads();
            const uint32_t moved = (uint32_t)sub + G < qn ? queue[grp][sub + G] : 0u;
            __syncthreads();
            if ((uint32_t)sub + G < qn) queue[grp][sub] = moved;
            qn -= n;
            __syncthreads();
        }
        if (last) break;
    }
    if (have_row) st_partial28(partial, row * G + sub, acc);
}

// Row epilogue: 2^lg_lpr lanes per row, each sums its share of the partials serially, then a
// tree over those lanes; the leader maps the row sum to affine coordinates.  All in the 28-bit form.
template <bool AFFINE>
__global__ void __launch_bounds__(64) commit_reduce_kernel(uint32_t* out, const uint32_t* partial, size_t rows, uint32_t nparts,
                                                           uint32_t lg_lpr) {
    const int lane = threadIdx.x & 63;
    const int lpr = 1 << lg_lpr;                       // lanes per row: 8, 16, 32 or 64
    const int sub = lane & (lpr - 1);
    const size_t row = geom::reduce_row(blockIdx.x, lane, lg_lpr);
    Xyzz28 acc = xyzz28_inf();
    // one addition site serves both the serial part and the tree steps (code size)
    const uint32_t nserial = (nparts + lpr - 1) >> lg_lpr;
    for (uint32_t step = 0; step < nserial + lg_lpr; step++) {
        Xyzz28 q;
        bool doit;
        if (step < nserial) {
            const uint32_t j = sub + (step << lg_lpr);
            doit = row < rows && j < nparts;
            q = doit ? ld_partial28(partial, row * nparts + j) : xyzz28_inf();
        } else {
            const int off = (lpr >> 1) >> (step - nserial);
            q = shfl_down_xyzz28(acc, off);
            doit = sub + off < lpr;
        }
        if (doit) padd28(acc, q);
    }
    if (row < rows && sub == 0) {
        if (AFFINE) st_affine(out, row, xyzz28_to_affine(acc));
        else st_partial28(out, row, acc);        // left as an accumulator (256 bytes) for a later combination
    }
}

// Row epilogue for many rows: a workgroup of four waves takes eight rows, 32 lanes a row (thread t: row t & 7,
// share t >> 3).  Every lane sums its share of the row's partial sums, waves 2 and 3 hand theirs to waves 0 and 1
// through LDS, wave 1 hands its to wave 0, and wave 0 finishes with three shuffle steps: for 64 partial sums a
// chain of 6 additions instead of the 10 of eight lanes per row, with every lane of the early steps at work (a
// tree by shuffles alone would keep all four waves issuing with idle lanes).  Both barriers are reached by all
// four waves; waves 1 to 3 leave after the second.
using geom::kTreeRows;
constexpr int kTreeLdsWords = 4 * L28 + 1;
__device__ __forceinline__ void st_lds_xyzz28(uint32_t* lds, int slot, const Xyzz28& a) {
#pragma unroll
    for (int k = 0; k < L28; k++) {
        lds[(0 * L28 + k) * 192 + slot] = (uint32_t)a.x.v[k];
        lds[(1 * L28 + k) * 192 + slot] = (uint32_t)a.y.v[k];
        lds[(2 * L28 + k) * 192 + slot] = (uint32_t)a.zz.v[k];
        lds[(3 * L28 + k) * 192 + slot] = (uint32_t)a.zzz.v[k];
    }
    lds[4 * L28 * 192 + slot] = a.inf ? 1u : 0u;
}
__device__ __forceinline__ Xyzz28 ld_lds_xyzz28(const uint32_t* lds, int slot) {
    Xyzz28 a;
#pragma unroll
    for (int k = 0; k < L28; k++) {
        a.x.v[k] = (int32_t)lds[(0 * L28 + k) * 192 + slot];
        a.y.v[k] = (int32_t)lds[(1 * L28 + k) * 192 + slot];
        a.zz.v[k] = (int32_t)lds[(2 * L28 + k) * 192 + slot];
        a.zzz.v[k] = (int32_t)lds[(3 * L28 + k) * 192 + slot];
    }
    a.inf = lds[4 * L28 * 192 + slot] != 0;
    return a;
}
template <bool AFFINE>
__global__ void __launch_bounds__(geom::kTreeThreads, 2) commit_reduce_tree_kernel(uint32_t* out, const uint32_t* partial, size_t rows, uint32_t nparts) {
    __shared__ uint32_t lds[kTreeLdsWords * 192];      // slots 0..127: waves 2, 3; slots 128..191: wave 1
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const size_t row = geom::tree_row(blockIdx.x, t);
    const uint32_t sub = geom::tree_share(t);
    const bool have = row < rows;
    Xyzz28 acc = xyzz28_inf();
    const uint32_t nserial = (nparts + 31) >> 5;
    // one addition site serves every step (code size)
    for (uint32_t step = 0; step < nserial + 5; step++) {
        Xyzz28 q = xyzz28_inf();
        bool doit = false;
        if (step < nserial) {
            const uint32_t j = sub + (step << 5);
            doit = have && j < nparts;
            if (doit) q = ld_partial28(partial, row * nparts + j);
        } else if (step == nserial) {
            if (wave >= 2) st_lds_xyzz28(lds, t - 128, acc);
            __syncthreads();
            if (wave < 2) {
                q = ld_lds_xyzz28(lds, t);
                doit = true;
            }
        } else if (step == nserial + 1) {
            if (wave == 1) st_lds_xyzz28(lds, 128 + lane, acc);
            __syncthreads();
            if (wave != 0) return;
            q = ld_lds_xyzz28(lds, 128 + lane);
            doit = true;
        } else {
            const int off = 32 >> (step - nserial - 2);      // 32, 16, 8: the partner holds the same row
            q = shfl_down_xyzz28(acc, off);
            doit = lane + off < 64;
        }
        if (doit) padd28(acc, q);
    }
    if (t < kTreeRows && have) {
        if (AFFINE) st_affine(out, row, xyzz28_to_affine(acc));
        else st_partial28(out, row, acc);
    }
}

// ------------------------------------------------------------------------------------------------
// commitment through the reference-format table (entry k * npoints + i = k * G_i, k < 256, canonical
// affine points): the reference's algorithm (byte windows, 8 doublings between windows,
// src/Hyrax.cu:46-167) re-ordered so that it fills the chip whatever the number of rows - one wave
// per (row, window, column segment) sums its table entries in the 28-bit form, the row-reduction
// kernel folds the lanes and segments of every (row, window), and a last kernel runs the Horner
// chain over a row's windows.  A table entry is converted on the fly (one 28-bit product per
// coordinate); no wide table has to be built, which is what single rows (Hyrax::open's blinding
// row, single_commit) and rows too long for a wide table need.
// ------------------------------------------------------------------------------------------------
template <bool FR>
__global__ void __launch_bounds__(kBlock, 2) commit_ref28_kernel(uint32_t* partial, const void* scalars, uint32_t rowlen, size_t rows,
                                                                 uint32_t seg, uint32_t nseg, const uint32_t* table, size_t npoints) {
    constexpr uint32_t nwin = FR ? 32 : 4;
    const size_t unit = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 6;      // one wave per unit
    const uint32_t lane = threadIdx.x & 63;
    if (unit >= rows * nwin * nseg) return;
    const uint32_t sg = (uint32_t)(unit % nseg);
    const size_t rw = unit / nseg;
    const uint32_t w = (uint32_t)(rw % nwin);
    const size_t row = rw / nwin;
    const uint32_t col_end = (sg + 1) * seg < rowlen ? (sg + 1) * seg : rowlen;
    Xyzz28 acc = xyzz28_inf();
    for (uint32_t col = sg * seg + lane; col < col_end; col += 64) {
        uint32_t idx;
        bool neg = false;
        if (FR) {
            const Fr k = fr26::from_montc(ld_fr8((const uint32_t*)scalars, row * rowlen + col));
            uint32_t limb = 0;
#pragma unroll
            for (int q = 0; q < 8; q++) limb = (q == (int)(w >> 2)) ? k.v[q] : limb;
            idx = (limb >> (8 * (w & 3))) & 255u;
        } else {
            const int32_t sv = ((const int32_t*)scalars)[row * rowlen + col];
            neg = sv < 0;
            const uint32_t a = neg ? (uint32_t)0 - (uint32_t)sv : (uint32_t)sv;
            idx = (a >> (8 * w)) & 255u;
        }
        if (idx) {
            const G1Affine a = ld_affine(table, (size_t)idx * npoints + col);
            if (!a.is_inf()) {
                Affine28 e;
                e.x = fp28::from_canonical_lazy(a.x);      // in (0, 3p): fine for every product it enters
                e.y = fp28::from_canonical_lazy(a.y);
                if (!xyzz28_madd(acc, e, neg)) {           // entry = +-accumulator: exact canonical-form addition
                    G1Xyzz c = xyzz28_to_canonical(acc);
                    xyzz_add_affine(c, a, neg);
                    acc = xyzz28_from_canonical(c);
                }
            }
        }
    }
    st_partial28(partial, unit * 64 + lane, acc);
}

// total = sum_w 2^(8 w) * sums[row * nwin + w]: one thread per row
__global__ void __launch_bounds__(64) commit_ref_horner_kernel(uint32_t* out, const uint32_t* sums, size_t rows, uint32_t nwin) {
    const size_t row = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (row >= rows) return;
    G1Xyzz total = G1Xyzz::inf();
    for (int w = (int)nwin - 1; w >= 0; w--) {
        for (int d = 0; d < 8; d++) pdbl(total);
        madd(total, ld_affine(sums, row * nwin + w), false);
    }
    st_affine(out, row, to_affine(total));
}

__global__ void __launch_bounds__(64) affine_to_jac_kernel(uint32_t* out, const uint32_t* in, size_t n) {
    size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n) return;
    G1Affine a = ld_affine(in, i);
    bool inf = a.is_inf();
    st_fp(out + 3 * FW * i, a.x);
    st_fp(out + 3 * FW * i + FW, a.y);
    st_fp(out + 3 * FW * i + 2 * FW, inf ? Fp::zero() : Fp::one());
}
__global__ void __launch_bounds__(64) jac_to_affine_kernel(uint32_t* out, const uint32_t* in, size_t n) {
    size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n) return;
    G1Jac p;
    p.x = ld_fp(in + 3 * FW * i);
    p.y = ld_fp(in + 3 * FW * i + FW);
    p.z = ld_fp(in + 3 * FW * i + 2 * FW);
    G1Affine a = G1Affine::inf();
    if (!p.is_inf()) {
        const Fp zi = fp_inverse_fast(p.z), zi2 = fsqr(zi);
        a.x = fmul(p.x, zi2);
        a.y = fmul(p.y, fmul(zi2, zi));
    }
    st_affine(out, i, a);
}

// out[i] = a[i] + b[i] for affine points (either may be the point at infinity, or both equal or opposite)
__global__ void __launch_bounds__(64) affine_add_kernel(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n) {
    size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n) return;
    G1Xyzz acc = G1Xyzz::inf();
    madd(acc, ld_affine(a, i), false);
    madd(acc, ld_affine(b, i), false);
    st_affine(out, i, to_affine(acc));
}

}  // namespace grape

using namespace grape;

#define CHECK_PTR16(p) GRAPE_REQUIRE((p) != nullptr && (reinterpret_cast<uintptr_t>(p) & 15) == 0, #p " must be a 16-byte aligned device pointer")

using geom::reduce_lanes_log2;
// Largest commitment one call accepts: 2^28 scalars (1 GiB of int32, 8 GiB of field elements), the
// largest size the GPU tests run; the host classes split longer tensors by rows.
constexpr size_t kMaxCommitScalars = (size_t)1 << 28;

// Row reduction of `rows` rows of `nparts` partial sums each.  With few rows the chain of additions of
// the reducing lanes is what takes the time (one row of 4096 partial sums on 64 lanes: 64 + 6 additions
// one after the other, 1 ms), so those go through two levels: every 256 partial sums of a row become
// one (4 + 6 additions, one wave per group), then the groups of a row are folded (`tmp`: one
// accumulator of 256 bytes per group).
constexpr uint32_t kReduceGroup = 256;
static size_t reduce_tmp_bytes(size_t rows, uint32_t nparts) { return rows * (size_t)(nparts / kReduceGroup + 1) * (4 * kPartialWords); }
template <bool AFFINE>
static void launch_reduce(uint32_t* out, const uint32_t* partial, size_t rows, uint32_t nparts, uint32_t lg_lpr, uint32_t* tmp, hipStream_t s,
                          bool alone = false) {
    if (tmp && lg_lpr == 6 && nparts >= 4 * kReduceGroup && nparts % kReduceGroup == 0) {
        const uint32_t groups = nparts / kReduceGroup;
        commit_reduce_kernel<false><<<(unsigned)(rows * groups), 64, 0, s>>>(tmp, partial, rows * groups, kReduceGroup, 6);
        uint32_t lg2 = 0;
        while ((1u << lg2) < groups && lg2 < 6) lg2++;
        const size_t per_wave = (size_t)64 >> lg2;
        commit_reduce_kernel<AFFINE><<<(unsigned)((rows + per_wave - 1) / per_wave), 64, 0, s>>>(out, tmp, rows, groups, lg2);
        return;
    }
    // `alone`: the caller waits for this result with nothing queued behind it - the four-wave kernel's shorter
    // chain is the gain (0.29 against 0.35 ms for 4096 rows of 64).  Beside other kernels it is the loss: its
    // waves hold half as many wave slots again while they wait at the barriers, and a commitment queued
    // behind this one runs slower for it (three streams of 4096 x 4096 commitments: 6220 against 6550 Mpoints/s)
    if (alone && geom::tree_reduction(rows, lg_lpr, nparts)) {
        commit_reduce_tree_kernel<AFFINE><<<(unsigned)((rows + kTreeRows - 1) / kTreeRows), geom::kTreeThreads, 0, s>>>(out, partial, rows, nparts);
        return;
    }
    const size_t per_wave = (size_t)64 >> lg_lpr;
    commit_reduce_kernel<AFFINE><<<(unsigned)((rows + per_wave - 1) / per_wave), 64, 0, s>>>(out, partial, rows, nparts, lg_lpr);
}

template <bool FR>
static int commit_wide_impl(uint32_t* out, const void* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t N,
                            uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st, int* caller_flag = nullptr) {
    if (size == 0) return GRAPE_OK;                      // no rows: nothing is read or written
    GRAPE_REQUIRE(size <= kMaxCommitScalars, "more than 2^28 scalars in one call: commit the rows in several calls");
    CHECK_PTR16(out); CHECK_PTR16(scalars); CHECK_PTR16(table);
    GRAPE_REQUIRE(rowlen >= 1 && size % rowlen == 0, "size must be a multiple of rowlen");
    GRAPE_REQUIRE(rowlen <= N, "row longer than the generator set");
    // a single-window table may hold fewer than 2^(c-1) multiples (the indexed commitments: K table
    // rows, digits 1..K); a digit above K is caught on the device
    GRAPE_REQUIRE(c >= 2 && c <= (FR ? 16u : 24u) && nw >= 1 && K >= 1 && (K >= (1u << (c - 1)) || (!FR && nw == 1)),
                  "need 2 <= c <= 16 (24 for int32) and K >= 2^(c-1) (any K >= 1 with one window of int32 digits)");
    if (FR) GRAPE_REQUIRE((uint64_t)nw * c >= 255, "Fr scalars need nw*c >= 255");
    const size_t rows = size / rowlen;
    if (rows == 0) return GRAPE_OK;
    hipStream_t s = as_stream(st);
    // rows go through in slabs so that the per-lane partial sums stay within 512 MiB whatever the
    // number of rows (a row segment leaves 64 partial sums of 256 bytes)
    const geom::WidePlan plan = geom::wide_plan(size, rowlen, geom::kSlabSegments);
    const uint32_t lg_lpr = plan.lg_lpr, nseg = plan.nseg, seg = plan.seg;
    const size_t slab = plan.slab, partial_bytes = plan.partial_bytes;
    void* ws;
    const size_t tmp_bytes = reduce_tmp_bytes(slab, nseg * 64);
    int rc = scratch_get(kSlotMsm, partial_bytes + tmp_bytes + 64, &ws, s);
    if (rc) return rc;
    uint32_t* red_tmp = (uint32_t*)((char*)ws + partial_bytes);
    // the digit-range flag: the call's own (cleared here, read back at the end), or one the caller
    // owns, has cleared and reads when it likes - then nothing here waits for the stream
    int* err = caller_flag ? caller_flag : (int*)((char*)ws + partial_bytes + tmp_bytes);
    if (!caller_flag) {
        rc = zero_fill(err, sizeof(int), s);
        if (rc) return rc;
    }
    const size_t elem_words = FR ? 8 : 1;
    profile_begin();
    for (size_t r0 = 0; r0 < rows; r0 += slab) {
        const size_t nr = rows - r0 < slab ? rows - r0 : slab;
        const uint32_t* sc = (const uint32_t*)scalars + r0 * rowlen * elem_words;
        profile_mark(s);
        commit_wide_kernel<FR><<<blocks_for(nr * nseg * 64), kBlock, 0, s>>>((uint32_t*)ws, sc, rowlen, nr, seg, nseg, table, N, c, nw, K, err);
        profile_mark(s);
        launch_reduce<true>(out + r0 * (size_t)(2 * FW), (const uint32_t*)ws, nr, nseg * 64, lg_lpr, red_tmp, s, caller_flag == nullptr);
        profile_mark(s);
    }
    GRAPE_LAUNCH_CHECK();
    if (caller_flag) return GRAPE_OK;
    int h_err = 0;
    GRAPE_HIP_CHECK(hipMemcpyAsync(&h_err, err, sizeof(int), hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    if (h_err) {
        set_error("commit: a scalar does not fit the table's digit range (c=%u, nw=%u, K=%u)", c, nw, K);
        return GRAPE_EINVAL;
    }
    return GRAPE_OK;
}

template <bool FR>
static int commit_ref_impl(uint32_t* out, const void* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t npoints,
                           grape_stream_t st) {
    if (size == 0) return GRAPE_OK;                      // no rows: nothing is read or written
    GRAPE_REQUIRE(size <= kMaxCommitScalars, "more than 2^28 scalars in one call: commit the rows in several calls");
    CHECK_PTR16(out); CHECK_PTR16(scalars); CHECK_PTR16(table);
    GRAPE_REQUIRE(rowlen >= 1 && size % rowlen == 0 && rowlen <= npoints, "bad shape");
    const size_t rows = size / rowlen;
    if (rows == 0) return GRAPE_OK;
    hipStream_t s = as_stream(st);
    const uint32_t nwin = FR ? 32 : 4;
    // column segments: enough waves to fill the chip, at least one 64-column sweep each, and chains
    // of at most 128 partial sums per reducing lane
    const uint32_t lg_lpr = reduce_lanes_log2(rows * nwin);
    uint32_t nseg = 1;
    while (rows * nwin * nseg < 8192 && rowlen / (nseg * 2) >= 64 && nseg * 2 <= (2u << lg_lpr)) nseg *= 2;
    const uint32_t seg = (rowlen + nseg - 1) / nseg;
    // rows go through in slabs so that the per-lane partial sums stay within 512 MiB
    size_t slab = 32768 / ((size_t)nwin * nseg);
    if (slab < 1) slab = 1;
    if (slab > rows) slab = rows;
    const size_t partial_bytes = slab * nwin * nseg * 64 * (size_t)(4 * kPartialWords);
    void* ws;
    const size_t sums_bytes = (slab * nwin * (size_t)(8 * FW) + 255) & ~(size_t)255;
    int rc = scratch_get(kSlotMsm, partial_bytes + sums_bytes + reduce_tmp_bytes(slab * nwin, nseg * 64) + 64, &ws, s);
    if (rc) return rc;
    uint32_t* sums = (uint32_t*)((char*)ws + partial_bytes);
    uint32_t* red_tmp = (uint32_t*)((char*)ws + partial_bytes + sums_bytes);
    const size_t elem_words = FR ? 8 : 1;
    for (size_t r0 = 0; r0 < rows; r0 += slab) {
        const size_t nr = rows - r0 < slab ? rows - r0 : slab;
        const size_t units = nr * nwin * nseg;
        const uint32_t* sc = (const uint32_t*)scalars + r0 * rowlen * elem_words;
        commit_ref28_kernel<FR><<<blocks_for(units * 64), kBlock, 0, s>>>((uint32_t*)ws, sc, rowlen, nr, seg, nseg, table, npoints);
        launch_reduce<true>(sums, (const uint32_t*)ws, nr * nwin, nseg * 64, lg_lpr, red_tmp, s);
        commit_ref_horner_kernel<<<blocks_for(nr, 64), 64, 0, s>>>(out + r0 * (size_t)(2 * FW), sums, nr, nwin);
    }
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

extern "C" {

int grape_g1_generator(uint32_t* out) {
    GRAPE_REQUIRE(out != nullptr, "null output");
    for (int i = 0; i < FW; i++) {
        out[i] = g1_gen_x(i);
        out[FW + i] = g1_gen_y(i);
    }
    return GRAPE_OK;
}

int grape_g1_scalar_mul_base(uint32_t* out, const uint32_t* k, const uint32_t* base, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(k); CHECK_PTR16(base);
    scalar_mul_base_kernel<<<blocks_for(n, 64), 64, 0, as_stream(st)>>>(out, k, base, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

static int wide_table_gen_impl(uint32_t* table, const uint32_t* gens, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st);

// The multiples come from the level-wise generator of the wide tables (one window, K = W - 1), a
// slab of generators at a time through a staging table of at most 1 GiB, and are then rewritten in
// the reference's layout and limb form.
int grape_g1_table_gen(uint32_t* table, const uint32_t* gens, size_t N, uint32_t W, grape_stream_t st) {
    if (N == 0 || W == 0) return GRAPE_OK;
    CHECK_PTR16(table); CHECK_PTR16(gens);
    GRAPE_REQUIRE(W <= (1u << 16), "bad table shape");
    hipStream_t s = as_stream(st);
    const uint32_t K = W > 1 ? W - 1 : 1;
    size_t slab = ((size_t)1 << 30) / ((size_t)K * 4 * kWideEntryWords);
    if (slab < 64) slab = 64;
    if (slab > N) slab = N;
    void* stage;
    int rc = scratch_get(kSlotTable, slab * K * 4 * kWideEntryWords, &stage, s);
    if (rc) return rc;
    for (size_t i0 = 0; i0 < N; i0 += slab) {
        const size_t ns = N - i0 < slab ? N - i0 : slab;
        if (W > 1) {
            rc = wide_table_gen_impl((uint32_t*)stage, gens + i0 * (size_t)(2 * FW), ns, 1, 1, K, st);
            if (rc) return rc;
        }
        ref_from_wide_kernel<<<blocks_for(ns * W), kBlock, 0, s>>>(table, (const uint32_t*)stage, N, i0, ns, W);
        GRAPE_LAUNCH_CHECK();
    }
    return GRAPE_OK;
}

size_t grape_g1_wide_table_bytes(size_t N, uint32_t nw, uint32_t K) { return (size_t)nw * K * N * 4 * kWideEntryWords; }

// table[(w*K + k-1)*N + i] = k * 2^(spacing*w) * G_i for k = 1..K, w < nw
static int wide_table_gen_impl(uint32_t* table, const uint32_t* gens, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st) {
    hipStream_t s = as_stream(st);
    const size_t per_chunk = (size_t)nw * N;
    // the first CH multiples of every base as a chain of mixed additions, normalised together;
    // everything above them level by level from the entries below (wide_extend_kernel)
    uint32_t CH = kFirstChain;
    if (K < CH) CH = K;
    void* ws;
    const size_t bases_bytes = per_chunk * (8 * FW);
    const size_t tmp_bytes = (size_t)CH * per_chunk * (16 * FW);
    int rc = scratch_get(kSlotMsm, bases_bytes + tmp_bytes + 256, &ws, s);
    if (rc) return rc;
    uint32_t* bases = (uint32_t*)ws;
    uint32_t* tmp = (uint32_t*)((char*)ws + bases_bytes);
    int* degenerate = (int*)((char*)ws + bases_bytes + tmp_bytes);
    rc = zero_fill(degenerate, sizeof(int), s);
    if (rc) return rc;
    window_bases_kernel<<<blocks_for(N, 64), 64, 0, s>>>(bases, gens, N, c, nw);
    GRAPE_LAUNCH_CHECK();
    {
        wide_chain_kernel<<<blocks_for(per_chunk, 64), 64, 0, s>>>(tmp, bases, N, nw, K, CH, 0, 1);
        const size_t n_entries = (size_t)CH * per_chunk;
        const size_t nthr2 = (n_entries + kNormChunk - 1) / kNormChunk;
        wide_normalize_kernel<<<blocks_for(nthr2, 64), 64, 0, s>>>(table, tmp, N, nw, K, CH, 0, n_entries);
        GRAPE_LAUNCH_CHECK();
    }
    for (uint32_t have = CH; have < K;) {
        const uint32_t cnt = K - have < have ? K - have : have;
        const uint32_t run = cnt < kExtendRun ? cnt : kExtendRun;
        const size_t nthreads = per_chunk * ((cnt + run - 1) / run);
        const size_t exact_want = (per_chunk * cnt + 63) / 64;
        const unsigned exact_blocks = (unsigned)(exact_want < 16384 ? exact_want : 16384);   // a no-op unless the flag is up
        wide_extend_kernel<<<blocks_for(nthreads), kBlock, 0, s>>>(table, N, nw, K, have, cnt, run, degenerate);
        wide_extend_exact_kernel<<<exact_blocks, 64, 0, s>>>(table, N, nw, K, have, cnt, degenerate);
        GRAPE_LAUNCH_CHECK();
        have += cnt;
    }
    return GRAPE_OK;
}

int grape_g1_wide_table_gen(uint32_t* table, const uint32_t* gens, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st) {
    CHECK_PTR16(table); CHECK_PTR16(gens);
    GRAPE_REQUIRE(N >= 1 && c >= 1 && c <= 16 && nw >= 1 && K >= 1 && K <= (1u << 16), "bad table shape");
    return wide_table_gen_impl(table, gens, N, c, nw, K, st);
}

int grape_g1_strided_table_gen(uint32_t* table, const uint32_t* gens, size_t N, uint32_t c, uint32_t J, uint32_t nsets, grape_stream_t st) {
    CHECK_PTR16(table); CHECK_PTR16(gens);
    GRAPE_REQUIRE(N >= 1 && c >= 2 && c <= 18 && J >= 1 && nsets >= 1 && (uint64_t)c * J * (nsets - 1) < 256, "bad table shape");
    return wide_table_gen_impl(table, gens, N, c * J, nsets, 1u << (c - 1), st);
}

// Full-width scalars through a strided table (see commit_strided_kernel): nw = ceil(255 / c) windows,
// J residues, nsets = ceil(nw / J) table sets of K = 2^(c-1) multiples.
int grape_commit_fr_strided(uint32_t* out, const uint32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t N,
                            uint32_t c, uint32_t J, uint32_t nsets, grape_stream_t st) {
    if (size == 0) return GRAPE_OK;
    GRAPE_REQUIRE(size <= kMaxCommitScalars, "more than 2^28 scalars in one call: commit the rows in several calls");
    CHECK_PTR16(out); CHECK_PTR16(scalars); CHECK_PTR16(table);
    GRAPE_REQUIRE(rowlen >= 1 && size % rowlen == 0, "size must be a multiple of rowlen");
    GRAPE_REQUIRE(rowlen <= N, "row longer than the generator set");
    GRAPE_REQUIRE(c >= 2 && c <= 18 && J >= 1, "need 2 <= c <= 18 and J >= 1");
    const uint32_t nw = (255 + c - 1) / c, K = 1u << (c - 1);
    GRAPE_REQUIRE(J <= nw && (uint64_t)nsets * J >= nw, "nsets * J must cover ceil(255 / c) windows");
    const size_t rows = size / rowlen;
    hipStream_t s = as_stream(st);
    // (row, residue) pairs are the rows of the accumulation and reduction launches
    const geom::WidePlan plan = geom::wide_plan(rows * J * (size_t)rowlen, rowlen, geom::kSlabSegments);
    const uint32_t lg_lpr = plan.lg_lpr, nseg = plan.nseg, seg = plan.seg;
    size_t slab = plan.slab / J;                              // whole rows per launch
    if (slab < 1) slab = 1;
    if (slab > rows) slab = rows;
    const size_t partial_bytes = slab * J * nseg * 64 * (size_t)(4 * kPartialWords);
    const size_t sums_bytes = slab * J * (size_t)(4 * kPartialWords);
    void* ws;
    int rc = scratch_get(kSlotMsm, partial_bytes + sums_bytes + reduce_tmp_bytes(slab * J, nseg * 64), &ws, s);
    if (rc) return rc;
    uint32_t* sums = (uint32_t*)((char*)ws + partial_bytes);
    uint32_t* red_tmp = (uint32_t*)((char*)ws + partial_bytes + sums_bytes);
    profile_begin();
    for (size_t r0 = 0; r0 < rows; r0 += slab) {
        const size_t nr = rows - r0 < slab ? rows - r0 : slab;
        const uint32_t* sc = scalars + r0 * rowlen * 8;
        profile_mark(s);
        commit_strided_kernel<<<blocks_for(nr * J * nseg * 64), kBlock, 0, s>>>((uint32_t*)ws, sc, rowlen, nr, seg, nseg, table, N, c, nw, K, J, nsets);
        profile_mark(s);
        launch_reduce<false>(sums, (const uint32_t*)ws, nr * J, nseg * 64, lg_lpr, red_tmp, s);
        strided_horner_kernel<<<blocks_for(nr, 64), 64, 0, s>>>(out + r0 * (size_t)(2 * FW), sums, nr, J, c);
        profile_mark(s);
    }
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_g1_scaled_table_gen(uint32_t* out, const uint32_t* scalars, size_t len, size_t ncols, const uint32_t* table, size_t N,
                              uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st) {
    CHECK_PTR16(out); CHECK_PTR16(scalars); CHECK_PTR16(table);
    GRAPE_REQUIRE(len >= 1 && ncols >= 1 && ncols <= N, "bad shape");
    GRAPE_REQUIRE(c >= 2 && c <= 16 && (uint64_t)nw * c >= 255 && K >= (1u << (c - 1)), "need a full-width wide table");
    hipStream_t s = as_stream(st);
    // slabs of scalars so that the XYZZ staging buffer stays near 1.5 GiB
    size_t slab = ((size_t)3 << 29) / (ncols * (16 * FW));
    if (slab < 1) slab = 1;
    if (slab > len) slab = len;
    void* ws;
    int rc = scratch_get(kSlotMsm, slab * ncols * (16 * FW) + 64, &ws, s);
    if (rc) return rc;
    int* err = (int*)((char*)ws + slab * ncols * (16 * FW));
    rc = zero_fill(err, sizeof(int), s);
    if (rc) return rc;
    for (size_t t0 = 0; t0 < len; t0 += slab) {
        size_t nt = len - t0 < slab ? len - t0 : slab;
        size_t n_entries = nt * ncols;
        scaled_chain_kernel<<<blocks_for(n_entries), kBlock, 0, s>>>((uint32_t*)ws, scalars, t0, nt, ncols, table, N, c, nw, K, err);
        size_t nthr = (n_entries + kNormChunk - 1) / kNormChunk;
        scaled_normalize_kernel<<<blocks_for(nthr, 64), 64, 0, s>>>(out, (const uint32_t*)ws, t0 * ncols, n_entries);
        GRAPE_LAUNCH_CHECK();
    }
    int h_err = 0;
    GRAPE_HIP_CHECK(hipMemcpyAsync(&h_err, err, sizeof(int), hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    if (h_err) {
        set_error("scaled table: a scalar digit exceeds the wide table's range");
        return GRAPE_EINVAL;
    }
    return GRAPE_OK;
}

int grape_commit_fr_sparse(uint32_t* out, const uint32_t* scalars, const int32_t* skip, size_t size, uint32_t rowlen,
                           const uint32_t* table, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st) {
    if (size == 0) return GRAPE_OK;
    GRAPE_REQUIRE(size <= kMaxCommitScalars, "more than 2^28 scalars in one call: commit the rows in several calls");
    CHECK_PTR16(out); CHECK_PTR16(scalars); CHECK_PTR16(table);
    GRAPE_REQUIRE(skip != nullptr, "no flag array");
    GRAPE_REQUIRE(rowlen >= 1 && size % rowlen == 0, "size must be a multiple of rowlen");
    GRAPE_REQUIRE(rowlen <= N, "row longer than the generator set");
    GRAPE_REQUIRE(c >= 2 && c <= 16 && (uint64_t)nw * c >= 255 && K >= (1u << (c - 1)), "need a full-width wide table");
    const size_t rows = size / rowlen;
    hipStream_t s = as_stream(st);
    const size_t slab = rows < geom::kSlabSegments ? rows : geom::kSlabSegments;
    const size_t partial_bytes = slab * geom::kWaveLanes * (size_t)(4 * geom::kPartialWords);
    void* ws;
    int rc = scratch_get(kSlotMsm, partial_bytes + 64, &ws, s);
    if (rc) return rc;
    int* err = (int*)((char*)ws + partial_bytes);
    rc = zero_fill(err, sizeof(int), s);
    if (rc) return rc;
    for (size_t r0 = 0; r0 < rows; r0 += slab) {
        const size_t nr = rows - r0 < slab ? rows - r0 : slab;
        const uint32_t lg_lpr = reduce_lanes_log2(nr);
        const size_t rows_per_wave = (size_t)64 >> lg_lpr;
        // many rows: half a wave per row, so that a thinly populated row still fills its batch
        const bool narrow = nr >= 4096;
        if (narrow)
            commit_sparse_fr_kernel<32><<<(unsigned)((nr + 1) / 2), 64, 0, s>>>((uint32_t*)ws, scalars + r0 * rowlen * 8, skip + r0 * rowlen, rowlen, nr,
                                                                              table, N, c, nw, K, err);
        else
            commit_sparse_fr_kernel<64><<<(unsigned)nr, 64, 0, s>>>((uint32_t*)ws, scalars + r0 * rowlen * 8, skip + r0 * rowlen, rowlen, nr, table, N,
                                                                   c, nw, K, err);
        commit_reduce_kernel<true><<<(unsigned)((nr + rows_per_wave - 1) / rows_per_wave), 64, 0, s>>>(out + r0 * (size_t)(2 * FW),
                                                                                                  (const uint32_t*)ws, nr, narrow ? 32 : 64, lg_lpr);
    }
    GRAPE_LAUNCH_CHECK();
    int h_err = 0;
    GRAPE_HIP_CHECK(hipMemcpyAsync(&h_err, err, sizeof(int), hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    if (h_err) {
        set_error("sparse commit: a scalar digit exceeds the wide table's range");
        return GRAPE_EINVAL;
    }
    return GRAPE_OK;
}

int grape_commit_i32(uint32_t* out, const int32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t N,
                     uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st) {
    return commit_wide_impl<false>(out, scalars, size, rowlen, table, N, c, nw, K, st);
}
int grape_commit_i32_nowait(uint32_t* out, const int32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t N,
                            uint32_t c, uint32_t nw, uint32_t K, int32_t* d_flag, grape_stream_t st) {
    GRAPE_REQUIRE(d_flag != nullptr, "the caller's flag is required");
    return commit_wide_impl<false>(out, scalars, size, rowlen, table, N, c, nw, K, st, d_flag);
}
int grape_commit_fr(uint32_t* out, const uint32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t N,
                    uint32_t c, uint32_t nw, uint32_t K, grape_stream_t st) {
    return commit_wide_impl<true>(out, scalars, size, rowlen, table, N, c, nw, K, st);
}
int grape_commit_fr_nowait(uint32_t* out, const uint32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table, size_t N,
                           uint32_t c, uint32_t nw, uint32_t K, int32_t* d_flag, grape_stream_t st) {
    GRAPE_REQUIRE(d_flag != nullptr, "the caller's flag is required");
    return commit_wide_impl<true>(out, scalars, size, rowlen, table, N, c, nw, K, st, d_flag);
}

int grape_commit_i32_ref_table(uint32_t* out, const int32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table,
                               size_t npoints, grape_stream_t st) {
    return commit_ref_impl<false>(out, scalars, size, rowlen, table, npoints, st);
}
int grape_commit_fr_ref_table(uint32_t* out, const uint32_t* scalars, size_t size, uint32_t rowlen, const uint32_t* table,
                              size_t npoints, grape_stream_t st) {
    return commit_ref_impl<true>(out, scalars, size, rowlen, table, npoints, st);
}

int grape_g1_affine_to_jacobian(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in);
    affine_to_jac_kernel<<<blocks_for(n, 64), 64, 0, as_stream(st)>>>(out, in, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_g1_jacobian_to_affine(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in);
    jac_to_affine_kernel<<<blocks_for(n, 64), 64, 0, as_stream(st)>>>(out, in, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_g1_affine_add(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(a); CHECK_PTR16(b);
    affine_add_kernel<<<blocks_for(n, 64), 64, 0, as_stream(st)>>>(out, a, b, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

}  // extern "C"
