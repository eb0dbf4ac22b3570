/*
 * TEST INFRASTRUCTURE — CPU oracle for the Grape proving hot path.
 *
 * A plain-C restatement of the reference's algorithms (field, curve, commitment, fold, sumcheck,
 * logUp) on 64-bit limbs.  It exists to check the HIP implementation and to serve as the
 * reported CPU baseline; nothing in the shipped library may call, link or load it.  Only the
 * test-suite, the smoke check and the benchmark's cpu_baseline leg use it.
 *
 * Memory formats are the reference's: an Fr element is 4 x u64 little-endian limbs holding the
 * canonical Montgomery residue x*2^256 mod r; an Fp element is 6 x u64 (x*2^384 mod p); an affine
 * G1 point is (x, y) = 12 x u64 with infinity = all zero; a Jacobian point is 18 x u64.
 * Compiled with -DORC_BN254 the same code is the BN254 instantiation (the reference's
 * include/field/alt_bn128.cuh): Fp is 4 x u64 (x*2^256 mod p), an affine point 8 x u64, a
 * Jacobian point 12 x u64, the curve y^2 = x^3 + 3 with generator (1, 2).
 *
 * How each function is pinned (what independent check guards it) is listed in grape_oracle.c.
 */
#ifndef GRAPE_ORACLE_H
#define GRAPE_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t orc_fr[4];
#if defined(ORC_BN254)
typedef uint64_t orc_fp[4];
#else
typedef uint64_t orc_fp[6];
#endif

int orc_num_threads(void);
uint32_t orc_log2(uint32_t n);

/* ---- field scalars ---- */
void orc_fr_add(uint64_t *r, const uint64_t *a, const uint64_t *b);
void orc_fr_sub(uint64_t *r, const uint64_t *a, const uint64_t *b);
void orc_fr_mul(uint64_t *r, const uint64_t *a, const uint64_t *b);
void orc_fr_neg(uint64_t *r, const uint64_t *a);
void orc_fr_inv(uint64_t *r, const uint64_t *a);
void orc_fr_to_mont(uint64_t *r, const uint64_t *a);
void orc_fr_from_mont(uint64_t *r, const uint64_t *a);
void orc_fr_from_i64(uint64_t *r, int64_t x);
void orc_fp_add(uint64_t *r, const uint64_t *a, const uint64_t *b);
void orc_fp_sub(uint64_t *r, const uint64_t *a, const uint64_t *b);
void orc_fp_mul(uint64_t *r, const uint64_t *a, const uint64_t *b);
void orc_fp_neg(uint64_t *r, const uint64_t *a);
void orc_fp_inv(uint64_t *r, const uint64_t *a);
void orc_fp_to_mont(uint64_t *r, const uint64_t *a);
void orc_fp_from_mont(uint64_t *r, const uint64_t *a);

/* ---- Fr tensors (arrays of n elements) ---- */
void orc_fr_vec_add(uint64_t *r, const uint64_t *a, const uint64_t *b, uint64_t n);
void orc_fr_vec_sub(uint64_t *r, const uint64_t *a, const uint64_t *b, uint64_t n);
void orc_fr_vec_mul(uint64_t *r, const uint64_t *a, const uint64_t *b, uint64_t n);
void orc_fr_vec_bcast_add(uint64_t *r, const uint64_t *a, const uint64_t *x, uint64_t n);
void orc_fr_vec_bcast_mul(uint64_t *r, const uint64_t *a, const uint64_t *x, uint64_t n);
void orc_fr_vec_from_i32(uint64_t *r, const int32_t *x, uint64_t n);
void orc_fr_vec_from_u32(uint64_t *r, const uint32_t *x, uint64_t n);
void orc_fr_vec_to_mont(uint64_t *r, const uint64_t *a, uint64_t n);
void orc_fr_vec_from_mont(uint64_t *r, const uint64_t *a, uint64_t n);
void orc_fr_vec_inv(uint64_t *r, const uint64_t *a, uint64_t n);
void orc_fr_sum(uint64_t *r, const uint64_t *a, uint64_t n);
void orc_fr_sum_by_dim(uint64_t *out, const uint64_t *in, uint64_t rows, uint64_t dim);
void orc_fr_pad(uint64_t *out, const uint64_t *in, uint32_t N, uint32_t pad_N, uint64_t pad_size,
                const uint64_t *pad_val);
void orc_i32_pad(int32_t *out, const int32_t *in, uint32_t N, uint32_t pad_N, uint64_t pad_size);
/* in-place fold + compaction, FrTensor::partial_eval */
void orc_fr_partial_eval(uint64_t *t, uint64_t N, const uint64_t *x, uint32_t c, uint32_t id,
                         uint32_t gap);
/* full multilinear evaluation (destroys t), FrTensor::operator()(u) */
void orc_fr_mle_eval(uint64_t *out, uint64_t *t, uint64_t size, const uint64_t *u, uint32_t nu);

/* ---- G1 ---- */
void orc_g1_generator(uint64_t *out_affine);
int orc_g1_on_curve(const uint64_t *p_affine);
void orc_g1_add_affine(uint64_t *out_affine, const uint64_t *a_affine, const uint64_t *b_affine);
/* out = k*P for a canonical (non-Montgomery) 256-bit k */
void orc_g1_scalar_mul(uint64_t *out_affine, const uint64_t *p_affine, const uint64_t *k_plain);
/* n generators k_i * G, k_i canonical scalars */
void orc_g1_make_generators(uint64_t *out_affine, const uint64_t *k_plain, uint64_t n);
void orc_g1_jac_to_affine(uint64_t *out_affine, const uint64_t *in_jac, uint64_t n);
/* table[w*N + i] = w * G_i, w < W (precompute_generators / naive_msm) */
void orc_g1_table(uint64_t *table_affine, const uint64_t *gens_affine, uint64_t N, uint32_t W);
/* Hyrax::commit(int*,...): rows = size/rowlen, byte windows of |s|, table stride npoints */
void orc_commit_i32(uint64_t *out_affine, const int32_t *scalars, const uint64_t *table_affine,
                    uint64_t size, uint32_t rowlen, uint64_t npoints);
/* Hyrax::commit(FrTensor&,...): 32 byte windows of the canonical scalar */
void orc_commit_fr(uint64_t *out_affine, const uint64_t *scalars_mont, const uint64_t *table_affine,
                   uint64_t size, uint32_t rowlen, uint64_t npoints);
/* plain double-and-add sum_i s_i * G_i, the brute-force check of the two above */
void orc_msm_naive_i64(uint64_t *out_affine, const int64_t *scalars, const uint64_t *gens_affine,
                       uint64_t n);

/* ---- sumcheck ---- */
/* One fused round of the two-tensor kernel: folds A,B in place, writes coefficient arrays. */
void orc_sumcheck_round2(uint64_t *A, uint64_t *B, uint64_t *a, uint64_t *b, uint64_t *c,
                         uint32_t in_size, uint32_t out_size, const uint64_t *v);
/*
 * prove_matmul.  A is L*N*K, B is L*M*K (both consumed).  transcript receives, per round,
 * 4 coefficients (low to high, unused high ones zero); n_rounds the number of rounds written.
 * Returns 0, or 1/2/3 when the phase-1 / phase-2 / final consistency check fails.
 */
int orc_prove_matmul(uint64_t *A, uint64_t *B, uint32_t L, uint32_t N, uint32_t M, uint32_t K,
                     const uint64_t *u, uint32_t nu, const uint64_t *v, uint32_t nv,
                     uint64_t *claim, uint64_t *transcript, uint32_t *n_rounds,
                     uint64_t *A_claim, uint64_t *B_claim);

/*
 * prove_eleMul (src/prove.cu:212-243, eleMul_sumcheck :119-172).  A, B: L*M*N elements, consumed.
 * Transcript as above (degree 3).  Returns 0, 1 (round check), 3 (final check) or 4 (L*M is not
 * a power of two).
 */
int orc_prove_elemul(uint64_t *A, uint64_t *B, uint32_t L, uint32_t M, uint32_t N, const uint64_t *u,
                     uint32_t nu, const uint64_t *v, uint32_t nv, uint64_t *claim, uint64_t *transcript,
                     uint32_t *n_rounds, uint64_t *A_claim, uint64_t *B_claim);
/*
 * combine_claims (src/prove.cu:245-301): u holds num rows of nv challenges; X (size = 2^nv
 * elements) is consumed; ret receives X(v).  Returns 0, 1 (round check) or 3 (final check).
 */
int orc_combine_claims(uint64_t *X, uint32_t size, const uint64_t *claims, uint32_t num, const uint64_t *u,
                       const uint64_t *v, uint32_t nv, uint64_t *transcript, uint64_t *ret);

/* ---- tlookup / logUp ---- */
void orc_histogram(uint32_t *hist, const uint64_t *vals_mont, uint64_t n, int32_t low, uint32_t len);
void orc_tlookup_prep(uint64_t *m_mont, const uint64_t *vals_mont, uint64_t n, int32_t low,
                      uint32_t len);
/* T[i] = low + i (+ r*map[i] when map != NULL), B[i] = 1/(T[i] + beta) */
void orc_tlookup_init(uint64_t *T, uint64_t *B, int32_t low, uint32_t len, const uint64_t *beta,
                      const uint64_t *map_mont, const uint64_t *r);
/*
 * tLookupRange::prove after prep: S (size D, a power of two here) is consumed.  m is the
 * multiplicity tensor (len entries, Montgomery), T,B the table and its inverses.
 * transcript: 4 coefficients per round; returns 0 or 1/2 for a phase-1 / phase-2 check failure.
 */
int orc_tlookup_prove(uint64_t *S, uint64_t D, const uint64_t *T, const uint64_t *B,
                      const uint64_t *m, uint32_t len, const uint64_t *alpha, const uint64_t *beta,
                      const uint64_t *u, const uint64_t *v, uint32_t nuv, uint64_t *transcript,
                      uint32_t *n_rounds, uint64_t *S_claim);

#ifdef __cplusplus
}
#endif
#endif
