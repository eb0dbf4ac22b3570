/*
 * TEST INFRASTRUCTURE — CPU oracle for the Grape proving hot path (see grape_oracle.h).
 * Not part of the product: the shipped library never links or loads this file.
 *
 * Every function restates a piece of the reference and says which; the reference's own host
 * arithmetic (libff) is not in the tree, so each one is pinned by independent checks held in
 * tests/ (Python big integers, textbook affine chord-tangent arithmetic, brute force):
 *
 *   field ops ........ closed forms a*b*R^-1 mod m etc., edge vectors      (test_oracle_field.py)
 *   G1 law ........... textbook affine arithmetic on Python integers,
 *                      on-curve, r*G = infinity                             (test_oracle_curve.py)
 *   table, commits ... naive sum_i s_i*G_i; int path == Fr path; linearity  (test_oracle_curve.py)
 *   fold / MLE ....... brute-force sum_i t[i]*prod_j eq(bit_j(i),u_j),
 *                      incl. non-power-of-two extents                       (test_oracle_fold.py)
 *   sumcheck ......... brute-force round polynomials p(0),p(1),p(2);
 *                      first claim = Y(u) of an exact integer matmul        (test_oracle_sumcheck.py)
 *   eleMul, claims ... brute-force round polynomials at t = 0..3, returned
 *                      values = multilinear extensions at v                 (test_oracle_elemul.py)
 *   all of the above . known-answer vectors written from the definitions    (test_golden.py)
 *   logUp ............ numpy.bincount; sum A = sum m*B; S(v) by brute force (test_oracle_tlookup.py)
 *
 * Citations are to files under the reference's root.
 */
#include "grape_oracle.h"
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef unsigned __int128 u128;
typedef uint64_t u64;

/* limbs of 64 bits of a base-field element: 6 for BLS12-381 (default), 4 for BN254 (-DORC_BN254) */
#if defined(ORC_BN254)
#define FPL 4
/* ------------------------------------------------------------------------------------------ */
/* constants: include/field/alt_bn128.cuh:11-45, re-derived from closed forms (2^k mod m);      */
/* curve y^2 = x^3 + 3 with generator (1, 2)                                                    */
/* ------------------------------------------------------------------------------------------ */
static const u64 FR_MOD[4] = {0x43e1f593f0000001ull, 0x2833e84879b97091ull, 0xb85045b68181585dull, 0x30644e72e131a029ull};
static const u64 FR_ONE[4] = {0xac96341c4ffffffbull, 0x36fc76959f60cd29ull, 0x666ea36f7879462eull, 0x0e0a77c19a07df2full};
static const u64 FR_RR[4] = {0x1bb8e645ae216da7ull, 0x53fe3ab1e35c59e3ull, 0x8c49833d53bb8085ull, 0x0216d0b17f4e44a5ull};
static const u64 FR_PM2[4] = {0x43e1f593efffffffull, 0x2833e84879b97091ull, 0xb85045b68181585dull, 0x30644e72e131a029ull};
#define FR_M0 0xc2e1f593efffffffull
static const u64 FP_MOD[FPL] = {0x3c208c16d87cfd47ull, 0x97816a916871ca8dull, 0xb85045b68181585dull, 0x30644e72e131a029ull};
static const u64 FP_ONE[FPL] = {0xd35d438dc58f0d9dull, 0x0a78eb28f5c70b3dull, 0x666ea36f7879462cull, 0x0e0a77c19a07df2full};
static const u64 FP_RR[FPL] = {0xf32cfc5b538afa89ull, 0xb5e71911d44501fbull, 0x47ab1eff0a417ff6ull, 0x06d89f71cab8351full};
static const u64 FP_PM2[FPL] = {0x3c208c16d87cfd45ull, 0x97816a916871ca8dull, 0xb85045b68181585dull, 0x30644e72e131a029ull};
#define FP_M0 0x87d20782e4866389ull
static const u64 G1_GX[FPL] = {0xd35d438dc58f0d9dull, 0x0a78eb28f5c70b3dull, 0x666ea36f7879462cull, 0x0e0a77c19a07df2full};
static const u64 G1_GY[FPL] = {0xa6ba871b8b1e1b3aull, 0x14f1d651eb8e167bull, 0xccdd46def0f28c58ull, 0x1c14ef83340fbe5eull};
static const u64 G1_B[FPL] = {0x7a17caa950ad28d7ull, 0x1f6ac17ae15521b9ull, 0x334bea4e696bd284ull, 0x2a1f6744ce179d8eull};

#else
#define FPL 6
/* ------------------------------------------------------------------------------------------ */
/* constants: include/field/bls12-381.cuh:7-45, re-derived from closed forms (2^k mod m)        */
/* ------------------------------------------------------------------------------------------ */
static const u64 FR_MOD[4] = {0xffffffff00000001ull, 0x53bda402fffe5bfeull, 0x3339d80809a1d805ull,
                              0x73eda753299d7d48ull};
static const u64 FR_ONE[4] = {0x00000001fffffffeull, 0x5884b7fa00034802ull, 0x998c4fefecbc4ff5ull,
                              0x1824b159acc5056full};
static const u64 FR_RR[4] = {0xc999e990f3f29c6dull, 0x2b6cedcb87925c23ull, 0x05d314967254398full,
                             0x0748d9d99f59ff11ull};
static const u64 FR_PM2[4] = {0xfffffffeffffffffull, 0x53bda402fffe5bfeull, 0x3339d80809a1d805ull,
                              0x73eda753299d7d48ull};
#define FR_M0 0xfffffffeffffffffull

static const u64 FP_MOD[FPL] = {0xb9feffffffffaaabull, 0x1eabfffeb153ffffull, 0x6730d2a0f6b0f624ull,
                              0x64774b84f38512bfull, 0x4b1ba7b6434bacd7ull, 0x1a0111ea397fe69aull};
static const u64 FP_ONE[FPL] = {0x760900000002fffdull, 0xebf4000bc40c0002ull, 0x5f48985753c758baull,
                              0x77ce585370525745ull, 0x5c071a97a256ec6dull, 0x15f65ec3fa80e493ull};
static const u64 FP_RR[FPL] = {0xf4df1f341c341746ull, 0x0a76e6a609d104f1ull, 0x8de5476c4c95b6d5ull,
                             0x67eb88a9939d83c0ull, 0x9a793e85b519952dull, 0x11988fe592cae3aaull};
static const u64 FP_PM2[FPL] = {0xb9feffffffffaaa9ull, 0x1eabfffeb153ffffull, 0x6730d2a0f6b0f624ull,
                              0x64774b84f38512bfull, 0x4b1ba7b6434bacd7ull, 0x1a0111ea397fe69aull};
#define FP_M0 0x89f3fffcfffcfffdull
/* standard G1 generator, Montgomery form */
static const u64 G1_GX[FPL] = {0x5cb38790fd530c16ull, 0x7817fc679976fff5ull, 0x154f95c7143ba1c1ull,
                             0xf0ae6acdf3d0e747ull, 0xedce6ecc21dbf440ull, 0x120177419e0bfb75ull};
static const u64 G1_GY[FPL] = {0xbaac93d50ce72271ull, 0x8c22631a7918fd8eull, 0xdd595f13570725ceull,
                             0x51ac582950405194ull, 0x0e1c8c3fad0059c0ull, 0x0bbc3efc5008a26aull};
static const u64 G1_B[FPL] = {0xaa270000000cfff3ull, 0x53cc0032fc34000aull, 0x478fe97a6b0a807full,
                            0xb1d37ebee6ba24d7ull, 0x8ec9733bbf78ab2full, 0x09d645513d83de7eull};

#endif

/* ------------------------------------------------------------------------------------------ */
/* generic n-limb Montgomery arithmetic (semantics of include/field/mont_t.cuh: canonical       */
/* results; + :225, - :277, * :406-427, cneg :303, to :453, from :483, 1/0 = 0 :1113)           */
/* ------------------------------------------------------------------------------------------ */
#define MAXL 6

static inline int ge_mod(const u64 *a, const u64 *mod, int n) {
    for (int i = n - 1; i >= 0; i--) {
        if (a[i] > mod[i]) return 1;
        if (a[i] < mod[i]) return 0;
    }
    return 1;
}
static inline u64 sub_n(u64 *r, const u64 *a, const u64 *b, int n) {
    u64 borrow = 0;
    for (int i = 0; i < n; i++) {
        u128 t = (u128)a[i] - b[i] - borrow;
        r[i] = (u64)t;
        borrow = (u64)(t >> 64) & 1;
    }
    return borrow;
}
static inline u64 add_n(u64 *r, const u64 *a, const u64 *b, int n) {
    u64 c = 0;
    for (int i = 0; i < n; i++) {
        u128 t = (u128)a[i] + b[i] + c;
        r[i] = (u64)t;
        c = (u64)(t >> 64);
    }
    return c;
}
static inline int is_zero_n(const u64 *a, int n) {
    u64 acc = 0;
    for (int i = 0; i < n; i++) acc |= a[i];
    return acc == 0;
}
static inline void mod_add(u64 *r, const u64 *a, const u64 *b, const u64 *mod, int n) {
    u64 s[MAXL];
    u64 c = add_n(s, a, b, n);
    if (c || ge_mod(s, mod, n)) sub_n(r, s, mod, n);
    else memcpy(r, s, 8 * n);
}
static inline void mod_sub(u64 *r, const u64 *a, const u64 *b, const u64 *mod, int n) {
    u64 d[MAXL];
    u64 borrow = sub_n(d, a, b, n);
    if (borrow) add_n(r, d, mod, n);
    else memcpy(r, d, 8 * n);
}
static inline void mod_neg(u64 *r, const u64 *a, const u64 *mod, int n) {
    if (is_zero_n(a, n)) memset(r, 0, 8 * n);
    else sub_n(r, mod, a, n);
}
static inline void mont_mul_n(u64 *r, const u64 *a, const u64 *b, const u64 *mod, u64 m0, int n) {
    u64 t[MAXL + 2];
    memset(t, 0, sizeof t);
    for (int i = 0; i < n; i++) {
        u64 c = 0;
        for (int j = 0; j < n; j++) {
            u128 acc = (u128)a[j] * b[i] + t[j] + c;
            t[j] = (u64)acc;
            c = (u64)(acc >> 64);
        }
        u128 s = (u128)t[n] + c;
        t[n] = (u64)s;
        t[n + 1] = (u64)(s >> 64);
        u64 m = t[0] * m0;
        u128 acc = (u128)m * mod[0] + t[0];
        c = (u64)(acc >> 64);
        for (int j = 1; j < n; j++) {
            acc = (u128)m * mod[j] + t[j] + c;
            t[j - 1] = (u64)acc;
            c = (u64)(acc >> 64);
        }
        s = (u128)t[n] + c;
        t[n - 1] = (u64)s;
        t[n] = t[n + 1] + (u64)(s >> 64);
    }
    if (t[n] || ge_mod(t, mod, n)) sub_n(r, t, mod, n);
    else memcpy(r, t, 8 * n);
}
/* a^(m-2) by square-and-multiply */
static void mont_inv_n(u64 *r, const u64 *a, const u64 *mod, u64 m0, const u64 *one,
                       const u64 *pm2, int n) {
    u64 acc[MAXL], base[MAXL];
    memcpy(acc, one, 8 * n);
    memcpy(base, a, 8 * n);
    for (int i = 0; i < 64 * n; i++) {
        if ((pm2[i / 64] >> (i % 64)) & 1) mont_mul_n(acc, acc, base, mod, m0, n);
        mont_mul_n(base, base, base, mod, m0, n);
    }
    memcpy(r, acc, 8 * n);
}

/* ---- Fr ---- */
static inline void fr_add(u64 *r, const u64 *a, const u64 *b) { mod_add(r, a, b, FR_MOD, 4); }
static inline void fr_sub(u64 *r, const u64 *a, const u64 *b) { mod_sub(r, a, b, FR_MOD, 4); }
static inline void fr_mul(u64 *r, const u64 *a, const u64 *b) { mont_mul_n(r, a, b, FR_MOD, FR_M0, 4); }
static inline void fr_neg(u64 *r, const u64 *a) { mod_neg(r, a, FR_MOD, 4); }
static inline void fr_inv(u64 *r, const u64 *a) { mont_inv_n(r, a, FR_MOD, FR_M0, FR_ONE, FR_PM2, 4); }
static inline void fr_cpy(u64 *r, const u64 *a) { memcpy(r, a, 32); }
static inline void fr_zero(u64 *r) { memset(r, 0, 32); }
static inline int fr_eq(const u64 *a, const u64 *b) { return memcmp(a, b, 32) == 0; }
static void fr_from_i64(u64 *r, int64_t x) {
    u64 t[4] = {x < 0 ? (u64)0 - (u64)x : (u64)x, 0, 0, 0};
    fr_mul(r, t, FR_RR);
    if (x < 0) fr_neg(r, r);
}
/* ---- Fp ---- */
static inline void fp_add(u64 *r, const u64 *a, const u64 *b) { mod_add(r, a, b, FP_MOD, FPL); }
static inline void fp_sub(u64 *r, const u64 *a, const u64 *b) { mod_sub(r, a, b, FP_MOD, FPL); }
static inline void fp_mul(u64 *r, const u64 *a, const u64 *b) { mont_mul_n(r, a, b, FP_MOD, FP_M0, FPL); }
static inline void fp_sqr(u64 *r, const u64 *a) { mont_mul_n(r, a, a, FP_MOD, FP_M0, FPL); }
static inline void fp_neg(u64 *r, const u64 *a) { mod_neg(r, a, FP_MOD, FPL); }
static inline void fp_inv(u64 *r, const u64 *a) { mont_inv_n(r, a, FP_MOD, FP_M0, FP_ONE, FP_PM2, FPL); }
static inline void fp_cpy(u64 *r, const u64 *a) { memcpy(r, a, 8 * FPL); }
static inline int fp_is_zero(const u64 *a) { return is_zero_n(a, FPL); }

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ceil(log2 n), Log2(0) = Log2(1) = 0: src/ioutils.cu:173-190 */
uint32_t orc_log2(uint32_t n) {
    if (n == 0) return 0;
    n--;
    uint32_t r = 0;
    while (n > 0) {
        n >>= 1;
        r++;
    }
    return r;
}

void orc_fr_add(u64 *r, const u64 *a, const u64 *b) { fr_add(r, a, b); }
void orc_fr_sub(u64 *r, const u64 *a, const u64 *b) { fr_sub(r, a, b); }
void orc_fr_mul(u64 *r, const u64 *a, const u64 *b) { fr_mul(r, a, b); }
void orc_fr_neg(u64 *r, const u64 *a) { fr_neg(r, a); }
void orc_fr_inv(u64 *r, const u64 *a) { fr_inv(r, a); }
void orc_fr_to_mont(u64 *r, const u64 *a) { fr_mul(r, a, FR_RR); }
void orc_fr_from_mont(u64 *r, const u64 *a) {
    u64 one[4] = {1, 0, 0, 0};
    fr_mul(r, a, one);
}
void orc_fr_from_i64(u64 *r, int64_t x) { fr_from_i64(r, x); }
void orc_fp_add(u64 *r, const u64 *a, const u64 *b) { fp_add(r, a, b); }
void orc_fp_sub(u64 *r, const u64 *a, const u64 *b) { fp_sub(r, a, b); }
void orc_fp_mul(u64 *r, const u64 *a, const u64 *b) { fp_mul(r, a, b); }
void orc_fp_neg(u64 *r, const u64 *a) { fp_neg(r, a); }
void orc_fp_inv(u64 *r, const u64 *a) { fp_inv(r, a); }
void orc_fp_to_mont(u64 *r, const u64 *a) { fp_mul(r, a, FP_RR); }
void orc_fp_from_mont(u64 *r, const u64 *a) {
    u64 one[FPL] = {1};
    fp_mul(r, a, one);
}

/* ------------------------------------------------------------------------------------------ */
/* Fr tensors: src/fr-tensor.cu kernels, one OpenMP loop per kernel                             */
/* ------------------------------------------------------------------------------------------ */
#define VEC2(NAME, OP)                                                         \
    void NAME(u64 *r, const u64 *a, const u64 *b, uint64_t n) {                \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t i = 0; i < (int64_t)n; i++) OP(r + 4 * i, a + 4 * i, b + 4 * i); \
    }
VEC2(orc_fr_vec_add, fr_add) /* Fr_elementwise_add :74-79 */
VEC2(orc_fr_vec_sub, fr_sub) /* Fr_elementwise_sub :81-86 */
VEC2(orc_fr_vec_mul, fr_mul) /* Fr_elementwise_mul :96-101 */

void orc_fr_vec_bcast_add(u64 *r, const u64 *a, const u64 *x, uint64_t n) { /* :88-93 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) fr_add(r + 4 * i, a + 4 * i, x);
}
void orc_fr_vec_bcast_mul(u64 *r, const u64 *a, const u64 *x, uint64_t n) { /* :103-108 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) fr_mul(r + 4 * i, a + 4 * i, x);
}
void orc_fr_vec_from_i32(u64 *r, const int32_t *x, uint64_t n) { /* int_to_fr :30-39 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) fr_from_i64(r + 4 * i, x[i]);
}
void orc_fr_vec_from_u32(u64 *r, const uint32_t *x, uint64_t n) { /* uint_to_fr :41-46 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) fr_from_i64(r + 4 * i, (int64_t)x[i]);
}
void orc_fr_vec_to_mont(u64 *r, const u64 *a, uint64_t n) { /* to_kernel :116-120 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) orc_fr_to_mont(r + 4 * i, a + 4 * i);
}
void orc_fr_vec_from_mont(u64 *r, const u64 *a, uint64_t n) { /* from_kernel :110-114 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) orc_fr_from_mont(r + 4 * i, a + 4 * i);
}
void orc_fr_vec_inv(u64 *r, const u64 *a, uint64_t n) { /* inverse_kernel :122-126 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) fr_inv(r + 4 * i, a + 4 * i);
}
/* FrTensor::sum(sz) :415-440 (the value; the tree order is irrelevant in a field) */
void orc_fr_sum(u64 *r, const u64 *a, uint64_t n) {
    int nt = orc_num_threads();
    u64(*part)[4] = calloc((size_t)nt, 32);
#pragma omp parallel
    {
#ifdef _OPENMP
        int t = omp_get_thread_num();
#else
        int t = 0;
#endif
        u64 acc[4] = {0, 0, 0, 0};
#pragma omp for schedule(static)
        for (int64_t i = 0; i < (int64_t)n; i++) fr_add(acc, acc, a + 4 * i);
        fr_cpy(part[t], acc);
    }
    u64 acc[4] = {0, 0, 0, 0};
    for (int t = 0; t < nt; t++) fr_add(acc, acc, part[t]);
    fr_cpy(r, acc);
    free(part);
}
/* sum_by_dim_kernel :155-163: each row's sum broadcast back over the row */
void orc_fr_sum_by_dim(u64 *out, const u64 *in, uint64_t rows, uint64_t dim) {
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)rows; g++) {
        u64 s[4] = {0, 0, 0, 0};
        for (uint64_t i = 0; i < dim; i++) fr_add(s, s, in + 4 * (g * dim + i));
        for (uint64_t i = 0; i < dim; i++) fr_cpy(out + 4 * (g * dim + i), s);
    }
}
/* pad_fr_kernel :24-28 */
void orc_fr_pad(u64 *out, const u64 *in, uint32_t N, uint32_t pad_N, uint64_t pad_size,
                const u64 *pad_val) {
    for (uint64_t g = 0; g < pad_size; g++) {
        if (g % pad_N < N) fr_cpy(out + 4 * g, in + 4 * ((g / pad_N) * N + g % pad_N));
        else fr_cpy(out + 4 * g, pad_val);
    }
}
/* pad_int_kernel :18-22 */
void orc_i32_pad(int32_t *out, const int32_t *in, uint32_t N, uint32_t pad_N, uint64_t pad_size) {
    for (uint64_t g = 0; g < pad_size; g++)
        out[g] = (g % pad_N >= N) ? 0 : in[(g / pad_N) * N + g % pad_N];
}

/* Fr_partial_me :168-188 with Fr_partial_eval_kernel :53-72 — one pass per round, in place */
static void fr_partial_me(uint64_t N, u64 *t, const u64 *x, uint32_t id, uint32_t cur_dim,
                          uint32_t window_size) {
    uint64_t out_size = N;
    uint64_t gap = window_size;
    uint32_t count = orc_log2(cur_dim);
    uint64_t cur_in = cur_dim;
    uint64_t dim = (uint64_t)cur_dim * window_size;
    while (count--) {
        uint64_t cur_out = (cur_in + 1) / 2;
        uint64_t other = out_size / (cur_in * window_size);
        out_size = other * cur_out * window_size;
        const u64 *xr = x + 4 * id;
#pragma omp parallel for schedule(static)
        for (int64_t gid = 0; gid < (int64_t)out_size; gid++) {
            uint64_t ind0 = gid / (cur_out * window_size);
            uint64_t ind1 = (gid / window_size) % cur_out;
            uint64_t ind2 = gid % window_size;
            u64 *p0 = t + 4 * (ind0 * dim + (2 * ind1) * gap + ind2);
            u64 d[4];
            if (2 * ind1 + 1 < cur_in) {
                const u64 *p1 = t + 4 * (ind0 * dim + (2 * ind1 + 1) * gap + ind2);
                fr_sub(d, p1, p0);
                fr_mul(d, xr, d);
                fr_add(p0, p0, d);
            } else {
                fr_mul(d, xr, p0);
                fr_sub(p0, p0, d);
            }
        }
        id += 1;
        gap <<= 1;
        cur_in = cur_out;
    }
}
/* FrTensor::partial_eval :330-344: fold, then compact the survivors to the front
 * (out of place in effect; the reference's in-place Memory_alignment :48-51 means this) */
void orc_fr_partial_eval(u64 *t, uint64_t N, const u64 *x, uint32_t c, uint32_t id, uint32_t gap) {
    fr_partial_me(N, t, x, id, c, gap);
    if (gap == 1 && N != c) {
        for (uint64_t g = 1; g < N / c; g++) fr_cpy(t + 4 * g, t + 4 * (g * c));
    } else if (gap != 1) {
        for (uint64_t i = 1; i < N / gap / c; i++)
            memmove(t + 4 * (i * gap), t + 4 * (i * (uint64_t)c * gap), 32 * (size_t)gap);
    }
}
/* FrTensor::operator()(u) :346-369, including its 11008-column special case */
void orc_fr_mle_eval(u64 *out, u64 *t, uint64_t size, const u64 *u, uint32_t nu) {
    if (size < ((uint64_t)1 << nu)) {
        fr_partial_me(size, t, u, orc_log2(11008), (uint32_t)(size / 11008), 11008);
        fr_partial_me(11008, t, u, 0, 11008, 1);
    } else {
        fr_partial_me(size, t, u, 0, (uint32_t)size, 1);
    }
    fr_cpy(out, t);
}

/* ------------------------------------------------------------------------------------------ */
/* G1: include/curve/{affine_t,jacobian_t,xyzz_t}.cuh                                           */
/* ------------------------------------------------------------------------------------------ */
typedef struct { u64 x[FPL], y[FPL]; } aff_t;
typedef struct { u64 x[FPL], y[FPL], zz[FPL], zzz[FPL]; } xyzz_t;

static inline int aff_is_inf(const aff_t *p) { return fp_is_zero(p->x) && fp_is_zero(p->y); }
static inline int xyzz_is_inf(const xyzz_t *p) { return fp_is_zero(p->zz); }
static inline void xyzz_set_inf(xyzz_t *p) { memset(p, 0, sizeof *p); }

/* acc += +-p: xyzz_t::add(affine, subtract) xyzz_t.cuh:363-441 */
static void xyzz_madd(xyzz_t *acc, const aff_t *p, int subtract) {
    if (aff_is_inf(p)) return;
    u64 py[FPL];
    if (subtract) fp_neg(py, p->y);
    else fp_cpy(py, p->y);
    if (xyzz_is_inf(acc)) {
        fp_cpy(acc->x, p->x);
        fp_cpy(acc->y, py);
        fp_cpy(acc->zz, FP_ONE);
        fp_cpy(acc->zzz, FP_ONE);
        return;
    }
    u64 P[FPL], R[FPL], PP[FPL], PPP[FPL], Q[FPL], X3[FPL], t[FPL];
    fp_mul(P, p->x, acc->zz);
    fp_sub(P, P, acc->x);
    fp_mul(R, py, acc->zzz);
    fp_sub(R, R, acc->y);
    if (!fp_is_zero(P)) {
        fp_sqr(PP, P);
        fp_mul(PPP, P, PP);
        fp_mul(Q, acc->x, PP);
        fp_sqr(X3, R);
        fp_sub(X3, X3, PPP);
        fp_sub(X3, X3, Q);
        fp_sub(X3, X3, Q);
        fp_sub(t, Q, X3);
        fp_mul(t, t, R);
        fp_mul(acc->y, acc->y, PPP);
        fp_sub(acc->y, t, acc->y);
        fp_cpy(acc->x, X3);
        fp_mul(acc->zz, acc->zz, PP);
        fp_mul(acc->zzz, acc->zzz, PPP);
    } else if (fp_is_zero(R)) {
        u64 U[FPL], V[FPL], W[FPL], S[FPL], M[FPL];
        fp_add(U, py, py);
        fp_sqr(V, U);
        fp_mul(W, U, V);
        fp_mul(S, p->x, V);
        fp_sqr(M, p->x);
        fp_add(t, M, M);
        fp_add(M, t, M);
        fp_sqr(X3, M);
        fp_sub(X3, X3, S);
        fp_sub(X3, X3, S);
        fp_sub(t, S, X3);
        fp_mul(t, t, M);
        fp_mul(acc->y, W, py);
        fp_sub(acc->y, t, acc->y);
        fp_cpy(acc->x, X3);
        fp_cpy(acc->zz, V);
        fp_cpy(acc->zzz, W);
    } else {
        xyzz_set_inf(acc);
    }
}
/* acc = 2*acc (dbl-2008-s-1 as in xyzz_t.cuh:170-200) */
static void xyzz_dbl(xyzz_t *acc) {
    if (xyzz_is_inf(acc)) return;
    u64 U[FPL], V[FPL], W[FPL], S[FPL], M[FPL], X3[FPL], t[FPL];
    fp_add(U, acc->y, acc->y);
    fp_sqr(V, U);
    fp_mul(W, U, V);
    fp_mul(S, acc->x, V);
    fp_sqr(M, acc->x);
    fp_add(t, M, M);
    fp_add(M, t, M);
    fp_sqr(X3, M);
    fp_sub(X3, X3, S);
    fp_sub(X3, X3, S);
    fp_sub(t, S, X3);
    fp_mul(t, t, M);
    fp_mul(acc->y, W, acc->y);
    fp_sub(acc->y, t, acc->y);
    fp_cpy(acc->x, X3);
    fp_mul(acc->zz, V, acc->zz);
    fp_mul(acc->zzz, W, acc->zzz);
}
/* acc += q: xyzz_t::add(xyzz) xyzz_t.cuh:129-212 */
static void xyzz_add(xyzz_t *acc, const xyzz_t *q) {
    if (xyzz_is_inf(q)) return;
    if (xyzz_is_inf(acc)) {
        *acc = *q;
        return;
    }
    u64 U1[FPL], S1[FPL], P[FPL], R[FPL], PP[FPL], PPP[FPL], Q[FPL], X3[FPL], t[FPL];
    fp_mul(U1, acc->x, q->zz);
    fp_mul(S1, acc->y, q->zzz);
    fp_mul(P, q->x, acc->zz);
    fp_sub(P, P, U1);
    fp_mul(R, q->y, acc->zzz);
    fp_sub(R, R, S1);
    if (!fp_is_zero(P)) {
        fp_sqr(PP, P);
        fp_mul(PPP, P, PP);
        fp_mul(Q, U1, PP);
        fp_sqr(X3, R);
        fp_sub(X3, X3, PPP);
        fp_sub(X3, X3, Q);
        fp_sub(X3, X3, Q);
        fp_sub(t, Q, X3);
        fp_mul(t, t, R);
        fp_mul(acc->y, S1, PPP);
        fp_sub(acc->y, t, acc->y);
        fp_cpy(acc->x, X3);
        fp_mul(acc->zz, acc->zz, q->zz);
        fp_mul(acc->zz, acc->zz, PP);
        fp_mul(acc->zzz, acc->zzz, q->zzz);
        fp_mul(acc->zzz, acc->zzz, PPP);
    } else if (fp_is_zero(R)) {
        xyzz_dbl(acc);
    } else {
        xyzz_set_inf(acc);
    }
}
/* xyzz_t -> affine, xyzz_t.cuh:89-97: x = X/ZZ, y = Y/ZZZ; infinity -> (0,0) */
static void xyzz_to_affine(aff_t *r, const xyzz_t *p) {
    if (xyzz_is_inf(p)) {
        memset(r, 0, sizeof *r);
        return;
    }
    u64 zi[FPL], zzi[FPL];
    fp_inv(zi, p->zzz);       /* 1/ZZZ */
    fp_mul(r->y, p->y, zi);
    fp_mul(zzi, zi, p->zz);   /* 1/Z */
    fp_sqr(zzi, zzi);         /* 1/ZZ */
    fp_mul(r->x, p->x, zzi);
}
static void xyzz_from_affine(xyzz_t *r, const aff_t *p) {
    xyzz_set_inf(r);
    xyzz_madd(r, p, 0);
}
/* k*P by left-to-right double-and-add over the 256-bit canonical scalar */
static void g1_scalar_mul(aff_t *out, const aff_t *p, const u64 *k) {
    xyzz_t acc;
    xyzz_set_inf(&acc);
    for (int i = 255; i >= 0; i--) {
        xyzz_dbl(&acc);
        if ((k[i / 64] >> (i % 64)) & 1) xyzz_madd(&acc, p, 0);
    }
    xyzz_to_affine(out, &acc);
}

void orc_g1_generator(u64 *out) {
    memcpy(out, G1_GX, 8 * FPL);
    memcpy(out + FPL, G1_GY, 8 * FPL);
}
int orc_g1_on_curve(const u64 *p) {
    const aff_t *a = (const aff_t *)p;
    if (aff_is_inf(a)) return 1;
    u64 l[FPL], r[FPL];
    fp_sqr(l, a->y);
    fp_sqr(r, a->x);
    fp_mul(r, r, a->x);
    fp_add(r, r, G1_B);
    return memcmp(l, r, 8 * FPL) == 0;
}
void orc_g1_add_affine(u64 *out, const u64 *a, const u64 *b) {
    xyzz_t acc;
    xyzz_from_affine(&acc, (const aff_t *)a);
    xyzz_madd(&acc, (const aff_t *)b, 0);
    xyzz_to_affine((aff_t *)out, &acc);
}
void orc_g1_scalar_mul(u64 *out, const u64 *p, const u64 *k) {
    g1_scalar_mul((aff_t *)out, (const aff_t *)p, k);
}
void orc_g1_make_generators(u64 *out, const u64 *k, uint64_t n) {
    aff_t g;
    orc_g1_generator((u64 *)&g);
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t i = 0; i < (int64_t)n; i++) g1_scalar_mul((aff_t *)(out + 2 * FPL * i), &g, k + 4 * i);
}
/* jacobian_t -> affine, jacobian_t.cuh:33-41 */
void orc_g1_jac_to_affine(u64 *out, const u64 *in, uint64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) {
        const u64 *X = in + 3 * FPL * i, *Y = X + FPL, *Z = X + 2 * FPL;
        aff_t *r = (aff_t *)(out + 2 * FPL * i);
        if (fp_is_zero(Z)) {
            memset(r, 0, sizeof *r);
            continue;
        }
        u64 zi[FPL], zi2[FPL], zi3[FPL];
        fp_inv(zi, Z);
        fp_sqr(zi2, zi);
        fp_mul(zi3, zi2, zi);
        fp_mul(r->x, X, zi2);
        fp_mul(r->y, Y, zi3);
    }
}
/* naive_msm src/ec_operation.cu:15-27: out[w*N+i] = w*G_i by repeated addition; w = 0 is (0,0) */
void orc_g1_table(u64 *table, const u64 *gens, uint64_t N, uint32_t W) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)N; i++) {
        const aff_t *g = (const aff_t *)(gens + 2 * FPL * i);
        xyzz_t res;
        xyzz_set_inf(&res);
        for (uint32_t w = 0; w < W; w++) {
            xyzz_to_affine((aff_t *)(table + 2 * FPL * ((uint64_t)w * N + i)), &res);
            xyzz_madd(&res, g, 0);
        }
    }
}
/*
 * Hyrax::commit(int*) src/Hyrax.cu:312-333 with int_windows_sum :46-65 and int_windows_reduce
 * :67-87: per row, for byte window w of |s| gather table[byte*npoints + i], negate for s < 0,
 * accumulate; the row value is sum_w 2^(8w) * S_w.  Output as affine.
 */
void orc_commit_i32(u64 *out, const int32_t *scalars, const u64 *table, uint64_t size,
                    uint32_t rowlen, uint64_t npoints) {
    uint64_t rows = size / rowlen;
    const aff_t *tb = (const aff_t *)table;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t r = 0; r < (int64_t)rows; r++) {
        xyzz_t total;
        xyzz_set_inf(&total);
        for (int w = 3; w >= 0; w--) {
            xyzz_t sum;
            xyzz_set_inf(&sum);
            for (uint32_t i = 0; i < rowlen; i++) {
                int32_t s = scalars[r * rowlen + i];
                uint32_t a = s < 0 ? (uint32_t)0 - (uint32_t)s : (uint32_t)s;
                uint32_t idx = (a >> (8 * w)) & 255u;
                xyzz_madd(&sum, &tb[(uint64_t)idx * npoints + i], s < 0);
            }
            for (int d = 0; d < 8; d++) xyzz_dbl(&total);
            xyzz_add(&total, &sum);
        }
        xyzz_to_affine((aff_t *)(out + 2 * FPL * r), &total);
    }
}
/*
 * Hyrax::commit(FrTensor&) src/Hyrax.cu:335-359 with many_windows_sum :128-144 and
 * many_windows_reduce :146-167: scalars leave Montgomery form, 32 byte windows each.
 */
void orc_commit_fr(u64 *out, const u64 *scalars, const u64 *table, uint64_t size, uint32_t rowlen,
                   uint64_t npoints) {
    uint64_t rows = size / rowlen;
    const aff_t *tb = (const aff_t *)table;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t r = 0; r < (int64_t)rows; r++) {
        xyzz_t total;
        xyzz_set_inf(&total);
        for (int w = 31; w >= 0; w--) {
            xyzz_t sum;
            xyzz_set_inf(&sum);
            for (uint32_t i = 0; i < rowlen; i++) {
                u64 k[4];
                orc_fr_from_mont(k, scalars + 4 * (r * rowlen + i));
                uint32_t idx = (uint32_t)(k[w / 8] >> (8 * (w % 8))) & 255u;
                xyzz_madd(&sum, &tb[(uint64_t)idx * npoints + i], 0);
            }
            for (int d = 0; d < 8; d++) xyzz_dbl(&total);
            xyzz_add(&total, &sum);
        }
        xyzz_to_affine((aff_t *)(out + 2 * FPL * r), &total);
    }
}
/* brute force sum_i s_i*G_i by double-and-add (the check commented out at test/HyraxTest.cu:146-178) */
void orc_msm_naive_i64(u64 *out, const int64_t *scalars, const u64 *gens, uint64_t n) {
    xyzz_t total;
    xyzz_set_inf(&total);
    for (uint64_t i = 0; i < n; i++) {
        int64_t s = scalars[i];
        u64 k[4] = {s < 0 ? (u64)0 - (u64)s : (u64)s, 0, 0, 0};
        aff_t t;
        g1_scalar_mul(&t, (const aff_t *)(gens + 2 * FPL * i), k);
        xyzz_madd(&total, &t, s < 0);
    }
    xyzz_to_affine((aff_t *)out, &total);
}

/* ------------------------------------------------------------------------------------------ */
/* sumcheck: src/prove.cu, src/polynomial.cu                                                    */
/* ------------------------------------------------------------------------------------------ */
typedef struct { u64 c[4][4]; int deg; } poly_t; /* coefficients low to high */

static void poly_zero(poly_t *p, int deg) {
    memset(p, 0, sizeof *p);
    p->deg = deg;
}
/* Polynomial::eq(u) src/polynomial.cu:40-45: (1-u) + (2u-1) t */
static void poly_eq(poly_t *p, const u64 *u) {
    poly_zero(p, 1);
    fr_sub(p->c[0], FR_ONE, u);
    fr_add(p->c[1], u, u);
    fr_sub(p->c[1], p->c[1], FR_ONE);
}
/* Polynomial::eq(u,v) :47-53: 2uv - u - v + 1 */
static void eq2(u64 *r, const u64 *u, const u64 *v) {
    u64 t[4], s[4];
    fr_mul(t, u, v);
    fr_add(t, t, t);
    fr_add(s, u, v);
    fr_sub(t, t, s);
    fr_add(r, t, FR_ONE);
}
static void poly_mul(poly_t *r, const poly_t *a, const poly_t *b) { /* operator* :100-107 */
    poly_t o;
    poly_zero(&o, a->deg + b->deg);
    for (int i = 0; i <= a->deg; i++)
        for (int j = 0; j <= b->deg; j++) {
            u64 t[4];
            fr_mul(t, a->c[i], b->c[j]);
            fr_add(o.c[i + j], o.c[i + j], t);
        }
    *r = o;
}
static void poly_scale(poly_t *p, const u64 *s) {
    for (int i = 0; i <= p->deg; i++) fr_mul(p->c[i], p->c[i], s);
}
static void poly_add(poly_t *r, const poly_t *a, const poly_t *b) { /* operator+ :69-80 */
    poly_t o;
    int d = a->deg > b->deg ? a->deg : b->deg;
    poly_zero(&o, d);
    for (int i = 0; i <= d; i++) {
        if (i <= a->deg) fr_add(o.c[i], o.c[i], a->c[i]);
        if (i <= b->deg) fr_add(o.c[i], o.c[i], b->c[i]);
    }
    *r = o;
}
static void poly_sub(poly_t *r, const poly_t *a, const poly_t *b) { /* operator- :82-93 */
    poly_t o;
    int d = a->deg > b->deg ? a->deg : b->deg;
    poly_zero(&o, d);
    for (int i = 0; i <= d; i++) {
        if (i <= a->deg) fr_add(o.c[i], o.c[i], a->c[i]);
        if (i <= b->deg) fr_sub(o.c[i], o.c[i], b->c[i]);
    }
    *r = o;
}
static void poly_eval(u64 *r, const poly_t *p, const u64 *x) { /* Horner :136-145 */
    u64 acc[4];
    fr_cpy(acc, p->c[p->deg]);
    for (int i = p->deg - 1; i >= 0; i--) {
        fr_mul(acc, acc, x);
        fr_add(acc, acc, p->c[i]);
    }
    fr_cpy(r, acc);
}
static void poly_eval01sum(u64 *r, const poly_t *p) { /* p(0) + p(1), :127-134 */
    u64 s[4];
    fr_cpy(s, p->c[0]);
    for (int i = 0; i <= p->deg; i++) fr_add(s, s, p->c[i]);
    fr_cpy(r, s);
}
static void transcript_put(u64 *transcript, uint32_t round, const poly_t *p) {
    memset(transcript + 16 * round, 0, 128);
    for (int i = 0; i <= p->deg; i++) fr_cpy(transcript + 16 * round + 4 * i, p->c[i]);
}

/* sumcheck_kernel (two tensors) src/prove.cu:29-46 */
void orc_sumcheck_round2(u64 *A, u64 *B, u64 *a, u64 *b, u64 *c, uint32_t in_size,
                         uint32_t out_size, const u64 *v) {
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)out_size; g++) {
        u64 Aa[4], Ab[4], Ba[4], Bb[4], t[4], s[4];
        fr_cpy(Ab, A + 4 * g);
        fr_cpy(Bb, B + 4 * g);
        if ((uint64_t)g + out_size < in_size) {
            fr_sub(Aa, A + 4 * (g + out_size), Ab);
            fr_sub(Ba, B + 4 * (g + out_size), Bb);
        } else {
            fr_neg(Aa, Ab);
            fr_neg(Ba, Bb);
        }
        fr_mul(t, Aa, v);
        fr_add(A + 4 * g, t, Ab);
        fr_mul(t, Ba, v);
        fr_add(B + 4 * g, t, Bb);
        fr_mul(c + 4 * g, Ab, Bb);
        fr_mul(t, Aa, Bb);
        fr_mul(s, Ab, Ba);
        fr_add(b + 4 * g, t, s);
        fr_mul(a + 4 * g, Aa, Ba);
    }
}

/* prove_matmul src/prove.cu:175-210 with matmul_sumcheck_phase1 :49-85 and phase2 :87-117 */
int orc_prove_matmul(u64 *A, u64 *B, uint32_t L, uint32_t N, uint32_t M, uint32_t K, const u64 *u,
                     uint32_t nu, const u64 *v, uint32_t nv, u64 *claim, u64 *transcript,
                     uint32_t *n_rounds, u64 *A_claim, u64 *B_claim) {
    (void)nu;
    (void)nv;
    uint32_t round = 0;
    int status = 0;
    orc_fr_partial_eval(A, (uint64_t)L * N * K, u, N, orc_log2(M), K);
    orc_fr_partial_eval(B, (uint64_t)L * M * K, u, M, 0, K);
    uint64_t LK = (uint64_t)L * K;
    u64 *a = malloc(32 * LK), *b = malloc(32 * LK), *c = malloc(32 * LK);
    u64 eq_acc[4];
    fr_cpy(eq_acc, FR_ONE);
    /* phase 1: bind layer bits, challenges from the back of v */
    {
        const u64 *uend = u + 4 * orc_log2(L * N * M);
        const u64 *vend = v + 4 * orc_log2(L * K);
        uint32_t rounds = orc_log2((uint32_t)(LK / K));
        uint32_t in = (uint32_t)LK, out = in / 2;
        for (uint32_t i = 0; i < rounds; i++) {
            const u64 *v_now = vend - 4 * (i + 1);
            const u64 *u_now = uend - 4 * (i + 1);
            orc_sumcheck_round2(A, B, a, b, c, in, out, v_now);
            orc_fr_partial_eval(a, out, uend - 4 * rounds, out / K, 0, K);
            orc_fr_partial_eval(b, out, uend - 4 * rounds, out / K, 0, K);
            orc_fr_partial_eval(c, out, uend - 4 * rounds, out / K, 0, K);
            poly_t p, e;
            poly_zero(&p, 2);
            orc_fr_sum(p.c[0], c, K);
            orc_fr_sum(p.c[1], b, K);
            orc_fr_sum(p.c[2], a, K);
            poly_eq(&e, u_now);
            poly_scale(&e, eq_acc);
            poly_mul(&p, &p, &e);
            transcript_put(transcript, round++, &p);
            u64 s[4];
            poly_eval01sum(s, &p);
            if (!fr_eq(s, claim) && !status) status = 1;
            poly_eval(claim, &p, v_now);
            in = out;
            out = out / 2;
            u64 t[4];
            eq2(t, u_now, v_now); /* (1-v)(1-u) + vu */
            fr_mul(eq_acc, eq_acc, t);
        }
    }
    /* phase 2: bind k bits */
    {
        const u64 *vend = v + 4 * orc_log2(K);
        uint32_t rounds = orc_log2(K);
        uint32_t in = K, out = rounds ? (1u << (rounds - 1)) : 0;
        for (uint32_t i = 0; i < rounds; i++) {
            const u64 *v_now = vend - 4 * (i + 1);
            orc_sumcheck_round2(A, B, a, b, c, in, out, v_now);
            poly_t p;
            poly_zero(&p, 2);
            orc_fr_sum(p.c[0], c, out);
            orc_fr_sum(p.c[1], b, out);
            orc_fr_sum(p.c[2], a, out);
            poly_scale(&p, eq_acc);
            transcript_put(transcript, round++, &p);
            u64 s[4];
            poly_eval01sum(s, &p);
            if (!fr_eq(s, claim) && !status) status = 2;
            poly_eval(claim, &p, v_now);
            in = out;
            out = out / 2;
        }
    }
    fr_cpy(A_claim, A);
    fr_cpy(B_claim, B);
    u64 t[4];
    fr_mul(t, A_claim, B_claim);
    fr_mul(t, t, eq_acc);
    if (!fr_eq(t, claim) && !status) status = 3;
    *n_rounds = round;
    free(a);
    free(b);
    free(c);
    return status;
}

/* sumcheck_kernel (one tensor) src/prove.cu:14-27 */
static void sumcheck_round1(u64 *X, u64 *a, u64 *b, uint32_t in_size, uint32_t out_size, const u64 *v) {
    for (uint32_t g = 0; g < out_size; g++) {
        u64 Xa[4], Xb[4], t[4];
        fr_cpy(Xb, X + 4 * (uint64_t)g);
        if ((uint64_t)g + out_size < in_size) fr_sub(Xa, X + 4 * ((uint64_t)g + out_size), Xb);
        else fr_neg(Xa, Xb);
        fr_mul(t, Xa, v);
        fr_add(X + 4 * (uint64_t)g, t, Xb);
        fr_cpy(b + 4 * (uint64_t)g, Xb);
        fr_cpy(a + 4 * (uint64_t)g, Xa);
    }
}

/* prove_eleMul src/prove.cu:212-243 with eleMul_sumcheck :119-172.  A, B: L*M*N elements, are
 * folded in place.  Status 1: a round check failed, 3: final product check failed, 4: first_size
 * (= L*M) is not a power of two (the reference throws). */
int orc_prove_elemul(u64 *A, u64 *B, uint32_t L, uint32_t M, uint32_t N, const u64 *u, uint32_t nu,
                     const u64 *v, uint32_t nv, u64 *claim, u64 *transcript, uint32_t *n_rounds,
                     u64 *A_claim, u64 *B_claim) {
    (void)nu;
    (void)nv;
    const uint32_t size = L * M * N, first_size = L * M;
    *n_rounds = 0;
    if ((1u << orc_log2(first_size)) != first_size) return 4;
    const u64 *uend = u + 4 * orc_log2(L * N * M);
    const u64 *vend = v + 4 * orc_log2(L * M * N);
    const uint32_t second_size = size / first_size;
    const uint32_t rounds = orc_log2(size);
    uint32_t in = size, out = size / 2;
    uint64_t cap = size / 2 ? size / 2 : 1;
    u64 *a = malloc(32 * cap), *b = malloc(32 * cap), *c = malloc(32 * cap);
    u64 eq_acc[4];
    fr_cpy(eq_acc, FR_ONE);
    int status = 0;
    for (uint32_t i = 0; i < rounds; i++) {
        const u64 *v_now = vend - 4 * (i + 1);
        const u64 *u_now = uend - 4 * (i + 1);
        orc_sumcheck_round2(A, B, a, b, c, in, out, v_now);
        u64 *arr[3] = {a, b, c};
        for (int k = 0; k < 3; k++) {
            if (in > second_size) {
                orc_fr_partial_eval(arr[k], out, uend - 4 * orc_log2(first_size), out / second_size, 0, second_size);
                orc_fr_partial_eval(arr[k], second_size, uend - 4 * orc_log2(size), second_size, 0, 1);
            } else {
                orc_fr_partial_eval(arr[k], out, uend - 4 * orc_log2(size), out, 0, 1);
            }
        }
        poly_t p, e;
        poly_zero(&p, 2);
        fr_cpy(p.c[0], c);
        fr_cpy(p.c[1], b);
        fr_cpy(p.c[2], a);
        poly_eq(&e, u_now);
        poly_scale(&e, eq_acc);
        poly_mul(&p, &p, &e);
        transcript_put(transcript, i, &p);
        u64 s[4], t[4];
        poly_eval01sum(s, &p);
        if (!fr_eq(s, claim) && !status) status = 1;
        poly_eval(claim, &p, v_now);
        in = out;
        out = (out == second_size) ? (1u << (orc_log2(out) - 1)) : out / 2;
        eq2(t, u_now, v_now);
        fr_mul(eq_acc, eq_acc, t);
    }
    *n_rounds = rounds;
    fr_cpy(A_claim, A);
    fr_cpy(B_claim, B);
    u64 t[4];
    fr_mul(t, A_claim, B_claim);
    fr_mul(t, t, eq_acc);
    if (!fr_eq(t, claim) && !status) status = 3;
    free(a);
    free(b);
    free(c);
    return status;
}

/* combine_claims src/prove.cu:245-301: merges `num` claims X(u_j) = claims[j] into one claim
 * X(v).  u holds num rows of nv challenges.  Returns X(v) in ret and every round polynomial
 * (degree 2) in transcript.  Status 1: a round check failed, 3: the final check failed. */
int orc_combine_claims(u64 *X, uint32_t size, const u64 *claims, uint32_t num, const u64 *u,
                       const u64 *v, uint32_t nv, u64 *transcript, u64 *ret) {
    u64 claim[4];
    fr_zero(claim);
    for (uint32_t j = 0; j < num; j++) fr_add(claim, claim, claims + 4 * j);
    uint64_t cap = size / 2 ? size / 2 : 1;
    u64 *a = malloc(32 * cap), *b = malloc(32 * cap), *ta = malloc(32 * cap), *tb = malloc(32 * cap);
    u64 *eq_acc = malloc(32 * (size_t)(num ? num : 1));
    for (uint32_t j = 0; j < num; j++) fr_cpy(eq_acc + 4 * j, FR_ONE);
    uint32_t in = size, out = size / 2;
    int status = 0;
    for (uint32_t i = 0; i < nv; i++) {
        const uint32_t left = nv - 1 - i;          /* challenges still unbound after this round */
        const u64 *v_now = v + 4 * left;           /* new_v.back() */
        sumcheck_round1(X, a, b, in, out, v_now);
        poly_t p;
        poly_zero(&p, 2);
        for (uint32_t j = 0; j < num; j++) {
            const u64 *uj = u + 4 * (uint64_t)j * nv;
            const u64 *now_u = uj + 4 * left;      /* new_u[j].back() */
            memcpy(ta, a, 32 * (size_t)out);
            memcpy(tb, b, 32 * (size_t)out);
            poly_t p1, e;
            poly_zero(&p1, 1);
            orc_fr_mle_eval(p1.c[0], tb, out, uj, left);
            orc_fr_mle_eval(p1.c[1], ta, out, uj, left);
            poly_eq(&e, now_u);
            poly_mul(&p1, &p1, &e);
            poly_scale(&p1, eq_acc + 4 * j);
            poly_add(&p, &p, &p1);
            u64 t[4];
            eq2(t, now_u, v_now);
            fr_mul(eq_acc + 4 * j, eq_acc + 4 * j, t);
        }
        transcript_put(transcript, i, &p);
        u64 s[4];
        poly_eval01sum(s, &p);
        if (!fr_eq(s, claim) && !status) status = 1;
        poly_eval(claim, &p, v_now);
        in = out;
        out = out / 2;
    }
    fr_cpy(ret, X);
    u64 sum[4], t[4];
    fr_zero(sum);
    for (uint32_t j = 0; j < num; j++) {
        fr_mul(t, eq_acc + 4 * j, ret);
        fr_add(sum, sum, t);
    }
    if (!fr_eq(sum, claim) && !status) status = 3;
    free(a);
    free(b);
    free(ta);
    free(tb);
    free(eq_acc);
    return status;
}

/* ------------------------------------------------------------------------------------------ */
/* tlookup / logUp: src/tlookup.cu                                                              */
/* ------------------------------------------------------------------------------------------ */
/* get_histogram_kernel :5-14: index = low limb of the canonical value of (v - low) */
void orc_histogram(uint32_t *hist, const u64 *vals, uint64_t n, int32_t low, uint32_t len) {
    u64 lowf[4];
    fr_from_i64(lowf, low);
    memset(hist, 0, 4 * (size_t)len);
    for (uint64_t i = 0; i < n; i++) {
        u64 t[4], k[4];
        fr_sub(t, vals + 4 * i, lowf);
        orc_fr_from_mont(k, t);
        uint32_t idx = (uint32_t)k[0];
        if (idx < len) hist[idx]++;
    }
}
/* tLookupRange::prep :265-286: histogram, the pad-count fix-up for a witness whose length is not
 * a power of two (the padding value 0 is counted into bin -low), then uint -> Fr */
void orc_tlookup_prep(u64 *m, const u64 *vals, uint64_t n, int32_t low, uint32_t len) {
    uint32_t *hist = malloc(4 * (size_t)len);
    orc_histogram(hist, vals, n, low, len);
    uint64_t padded = (uint64_t)1 << orc_log2((uint32_t)n);
    if (n != padded) hist[-low] += (uint32_t)(padded - n);
    orc_fr_vec_from_u32(m, hist, len);
    free(hist);
}
/* tlookuprange_init_kernel :16-31 and tLookupRangeMapping_init_kernel :33-50 */
void orc_tlookup_init(u64 *T, u64 *B, int32_t low, uint32_t len, const u64 *beta, const u64 *map,
                      const u64 *r) {
    u64 lowf[4];
    fr_from_i64(lowf, low);
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)len; g++) {
        u64 t[4], s[4];
        fr_from_i64(t, g);
        fr_add(t, t, lowf);
        if (map) {
            fr_mul(s, map + 4 * g, r);
            fr_add(t, t, s);
        }
        fr_cpy(T + 4 * g, t);
        fr_add(t, t, beta);
        fr_inv(B + 4 * g, t);
    }
}
/* tLookup_poly_kernel :64-78 */
static void tl_poly(const u64 *A, const u64 *S, const u64 *beta, u64 *o0, u64 *o1, u64 *o2,
                    uint64_t n_out) {
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < (int64_t)n_out; t++) {
        u64 c00[4], c01[4], c10[4], c11[4], x[4], y[4];
        fr_cpy(c00, A + 4 * t);
        fr_sub(c01, A + 4 * (t + n_out), A + 4 * t);
        fr_add(c10, S + 4 * t, beta);
        fr_sub(c11, S + 4 * (t + n_out), S + 4 * t);
        fr_mul(o0 + 4 * t, c00, c10);
        fr_mul(x, c01, c10);
        fr_mul(y, c00, c11);
        fr_add(o1 + 4 * t, x, y);
        fr_mul(o2 + 4 * t, c01, c11);
    }
}
/* tLookup_poly_sum_kernel :80-88 */
static void tl_poly_sum(const u64 *A, u64 *o0, u64 *o1, uint64_t n_out) {
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < (int64_t)n_out; t++) {
        fr_cpy(o0 + 4 * t, A + 4 * t);
        fr_sub(o1 + 4 * t, A + 4 * (t + n_out), A + 4 * t);
    }
}
static void mle_at(u64 *out, u64 *tmp, uint64_t n, const u64 *u, uint32_t nu) {
    orc_fr_mle_eval(out, tmp, n, u, nu);
}
/* MSB-split fold t[g] += v*(t[g+h]-t[g]) == partial_eval(size, v, 2, 0, size/2), :235-238 */
static void fold_msb(u64 *dst, const u64 *src, uint64_t h, const u64 *v) {
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)h; g++) {
        u64 d[4];
        fr_sub(d, src + 4 * (g + h), src + 4 * g);
        fr_mul(d, v, d);
        fr_add(dst + 4 * g, src + 4 * g, d);
    }
}

/* tLookupRange::prove :288-343 after prep/pad/inverse, with tLookup_phase1 :216-244,
 * tLookup_phase1_step_poly :117-151, tLookup_phase2 :192-214, tLookup_phase2_step_poly :153-190 */
int orc_tlookup_prove(u64 *S, uint64_t D, const u64 *T_in, const u64 *B_in, const u64 *m_in,
                      uint32_t len, const u64 *alpha_in, const u64 *beta, const u64 *u_in,
                      const u64 *v, uint32_t nuv, u64 *transcript, uint32_t *n_rounds,
                      u64 *S_claim) {
    int status = 0;
    uint32_t round = 0;
    uint64_t Nt = len;
    uint32_t logN = orc_log2(len);
    /* A = 1/(S + beta): tlookup_inv_kernel :52-62 */
    u64 *A = malloc(32 * D);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)D; i++) {
        u64 t[4];
        fr_add(t, S + 4 * i, beta);
        fr_inv(A + 4 * i, t);
    }
    u64 *T = malloc(32 * Nt), *B = malloc(32 * Nt), *m = malloc(32 * Nt);
    memcpy(T, T_in, 32 * Nt);
    memcpy(B, B_in, 32 * Nt);
    memcpy(m, m_in, 32 * Nt);
    u64 alpha[4], alpha_sq[4], C[4], claim[4], ratio[4], two_inv[4], t[4];
    fr_cpy(alpha, alpha_in);
    fr_mul(alpha_sq, alpha, alpha);
    { /* C = alpha^2 - sum(B*m) :324-325 */
        u64 *Bm = malloc(32 * Nt);
        orc_fr_vec_mul(Bm, B, m, Nt);
        orc_fr_sum(t, Bm, Nt);
        free(Bm);
        fr_sub(C, alpha_sq, t);
    }
    fr_add(claim, alpha, alpha_sq);
    { /* N/D :331 */
        u64 nf[4], df[4];
        fr_from_i64(nf, (int64_t)Nt);
        fr_from_i64(df, (int64_t)D);
        fr_inv(df, df);
        fr_mul(ratio, nf, df);
    }
    fr_from_i64(two_inv, 2);
    fr_inv(two_inv, two_inv);

    uint32_t nu = nuv;         /* live length of u */
    uint32_t nv1 = nuv - logN; /* v1 = v[logN:], v2 = v[:logN] :333-334 */
    uint32_t nv2 = logN;
    uint64_t half_max = D / 2 > 1 ? D / 2 : 1;
    u64 *t0 = malloc(32 * half_max), *t1 = malloc(32 * half_max), *t2 = malloc(32 * half_max);
    uint64_t cur = D;
    /* phase 1 */
    while (nv1 > 0) {
        uint64_t h = cur / 2;
        const u64 *u_top = u_in + 4 * (nu - 1);
        const u64 *v_top = v + 4 * (logN + nv1 - 1);
        poly_t p0, p1, e, p;
        tl_poly(A, S, beta, t0, t1, t2, h);
        poly_zero(&p0, 2);
        mle_at(p0.c[0], t0, h, u_in, nu - 1);
        mle_at(p0.c[1], t1, h, u_in, nu - 1);
        mle_at(p0.c[2], t2, h, u_in, nu - 1);
        poly_scale(&p0, alpha);
        poly_eq(&e, u_top);
        poly_mul(&p0, &p0, &e);
        tl_poly_sum(A, t0, t1, h);
        poly_zero(&p1, 1);
        orc_fr_sum(p1.c[0], t0, h);
        orc_fr_sum(p1.c[1], t1, h);
        poly_add(&p, &p0, &p1);
        fr_mul(t, C, two_inv);
        fr_add(p.c[0], p.c[0], t);
        transcript_put(transcript, round++, &p);
        u64 s[4];
        poly_eval01sum(s, &p);
        if (!fr_eq(s, claim) && !status) status = 1;
        poly_eval(claim, &p, v_top);
        fold_msb(A, A, h, v_top);
        fold_msb(S, S, h, v_top);
        eq2(t, u_top, v_top);
        fr_mul(alpha, alpha, t);
        fr_mul(C, C, two_inv);
        cur = h;
        nu--;
        nv1--;
    }
    /* phase 2 */
    while (nv2 > 0) {
        uint64_t h = Nt / 2;
        const u64 *u_top = u_in + 4 * (nu - 1);
        const u64 *v_top = v + 4 * (nv2 - 1);
        poly_t p0, q, p1, p2, e, p;
        u64 zero[4] = {0, 0, 0, 0}, coef[4];
        tl_poly(A, S, beta, t0, t1, t2, h);
        poly_zero(&p0, 2);
        mle_at(p0.c[0], t0, h, u_in, nu - 1);
        mle_at(p0.c[1], t1, h, u_in, nu - 1);
        mle_at(p0.c[2], t2, h, u_in, nu - 1);
        poly_scale(&p0, alpha);
        fr_mul(coef, ratio, alpha_sq);
        tl_poly(B, T, beta, t0, t1, t2, h);
        poly_zero(&q, 2);
        mle_at(q.c[0], t0, h, u_in, nu - 1);
        mle_at(q.c[1], t1, h, u_in, nu - 1);
        mle_at(q.c[2], t2, h, u_in, nu - 1);
        poly_scale(&q, coef);
        poly_add(&p0, &p0, &q);
        tl_poly_sum(A, t0, t1, h);
        poly_zero(&p1, 1);
        orc_fr_sum(p1.c[0], t0, h);
        orc_fr_sum(p1.c[1], t1, h);
        tl_poly(m, B, zero, t0, t1, t2, h);
        poly_zero(&p2, 2);
        orc_fr_sum(p2.c[0], t0, h);
        orc_fr_sum(p2.c[1], t1, h);
        orc_fr_sum(p2.c[2], t2, h);
        poly_scale(&p2, ratio);
        poly_eq(&e, u_top);
        poly_mul(&p, &e, &p0);
        poly_add(&p, &p, &p1);
        poly_sub(&p, &p, &p2);
        transcript_put(transcript, round++, &p);
        u64 s[4];
        poly_eval01sum(s, &p);
        if (!fr_eq(s, claim) && !status) status = 2;
        poly_eval(claim, &p, v_top);
        fold_msb(A, A, h, v_top);
        fold_msb(S, S, h, v_top);
        fold_msb(B, B, h, v_top);
        fold_msb(T, T, h, v_top);
        fold_msb(m, m, h, v_top);
        eq2(t, u_top, v_top);
        fr_mul(alpha, alpha, t);
        fr_mul(alpha_sq, alpha_sq, t);
        Nt = h;
        nu--;
        nv2--;
    }
    fr_cpy(S_claim, S);
    *n_rounds = round;
    free(A);
    free(T);
    free(B);
    free(m);
    free(t0);
    free(t1);
    free(t2);
    return status;
}
