/*
 * C entry points over the C++ host classes (FrTensor, Hyrax, prove_matmul, tLookupRange, ...),
 * for callers without a C++ toolchain (the Python test-suite and benchmark bind these with
 * ctypes).  Every function returns 0 on success and 1 after a C++ exception, whose message
 * grape_host_last_error() returns.  Pointers named d_* are device memory; field elements in
 * host memory are 8 x u32 Montgomery limbs, affine points 24 x u32.
 */
#ifndef GRAPE_HOST_CAPI_H
#define GRAPE_HOST_CAPI_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char *grape_host_last_error(void);
void grape_host_seed(uint64_t seed);
/* tLookupRange objects made by the wrappers below commit A through the scaled table (1) or as a
 * full-width tensor (0); default 1. */
void grape_host_set_indexed_commit(int on);
/* What the tensor arguments d_A, d_B, d_T, d_S, d_S_in, d_S_out, d_tensor of the calls below point
 * to: 0 (default) field elements of 32 bytes; 1 int32 values, which the call embeds into a tensor of
 * its own with FrTensor::get_data as the reference's drivers do (test/llm.cu:77).  Returns 1 for an
 * unknown format. */
int grape_host_set_input_format(int fmt);
/* With int32 inputs, grape_host_hyrax_open and grape_host_mle_eval fold the integers directly and the lookup provers
 * index the integer witness (1, default: Hyrax::open(const int*, ...), FrTensor::eval_ints, tLookupRange::prove(const int*, ...),
 * tLookupRangeMapping::prove(const int*, const int*, ...)), or every call embeds its tensors first (0). */
void grape_host_set_int_folds(int on);

/* prove_matmul on copies of the device tensors d_A (L*N*K) and d_B (L*M*K).  transcript receives
 * 4 coefficients (8 u32 each) per round. */
int grape_host_prove_matmul(const uint32_t *d_A, const uint32_t *d_B, int L, int N, int M, int K, const uint32_t *u,
                            uint32_t nu, const uint32_t *v, uint32_t nv, uint32_t *claim_inout, uint32_t *transcript,
                            uint32_t *n_rounds, uint32_t *A_claim, uint32_t *B_claim);
/* Seconds spent inside the most recent prove_matmul / tLookup prove proper (copies of the inputs
 * and allocations made by these wrappers excluded), device synchronised on both sides. */
double grape_host_last_prove_seconds(void);
/* Of which, for the lookup provers, seconds spent committing A and m. */
double grape_host_last_commit_seconds(void);
int grape_host_prove_elemul(const uint32_t *d_A, const uint32_t *d_B, int L, int M, int N, const uint32_t *u, uint32_t nu,
                            const uint32_t *v, uint32_t nv, uint32_t *claim_inout, uint32_t *transcript,
                            uint32_t *n_rounds, uint32_t *A_claim, uint32_t *B_claim);
/* combine_claims: num claims about d_X (size elements) at points u (num x nv elements, row-major). */
int grape_host_combine_claims(const uint32_t *d_X, uint32_t size, const uint32_t *claims, uint32_t num, const uint32_t *u,
                              const uint32_t *v, uint32_t nv, uint32_t *transcript, uint32_t *n_rounds, uint32_t *result);
/* FrTensor::operator()(u) on a copy of d_T. */
int grape_host_mle_eval(const uint32_t *d_T, uint32_t size, const uint32_t *u, uint32_t nu, uint32_t *out);

/* Hyrax over a reference-format device table (k*G_i, k < 256, stride npoints_total).
 * Commits d_scalars (int32) and writes rows = size/(N*com_scale) affine points to out_affine (host). */
int grape_host_hyrax_commit_i32(const int32_t *d_scalars, uint32_t size, uint32_t N, const uint32_t *d_table,
                                uint32_t npoints, uint32_t com_scale, uint32_t layer_num, uint32_t *out_affine);
int grape_host_hyrax_commit_fr(const uint32_t *d_scalars, uint32_t size, uint32_t N, const uint32_t *d_table,
                               uint32_t npoints, uint32_t com_scale, uint32_t layer_num, uint32_t *out_affine);
/* commit + open at eval_point with blinding challenge c, then verify; *verified = 1/0,
 * result = the opened evaluation, which also equals the multilinear extension at eval_point. */
int grape_host_hyrax_open_verify(const uint32_t *d_tensor, uint32_t size, uint32_t N, const uint32_t *d_table,
                                 uint32_t npoints, uint32_t com_scale, uint32_t layer_num, const uint32_t *eval_point,
                                 uint32_t n_eval, const uint32_t *c, uint32_t *result, int *verified);
/* Hyrax::open alone on a copy of the tensor: result = the opened evaluation.  The time of the
 * opening (between two device synchronisations) is what grape_host_last_prove_seconds() returns. */
int grape_host_hyrax_open(const uint32_t *d_tensor, uint32_t size, uint32_t N, const uint32_t *d_table, uint32_t npoints,
                          uint32_t com_scale, uint32_t layer_num, const uint32_t *eval_point, uint32_t n_eval,
                          const uint32_t *c, uint32_t *result);

/*
 * tLookupRange(low, len).prove on a copy of the witness d_S (D elements).  alpha, u, v are host
 * values (u, v: nuv elements).  Outputs: multiplicities as len Fr elements (host), the
 * transcript, S(v), and the commitments of A and m (affine, host; pass NULL to skip).
 * d_table/npoints/com_scale describe the Hyrax used for those commitments.
 */
int grape_host_tlookup_range_prove(const uint32_t *d_S, uint32_t D, int32_t low, uint32_t len, const uint32_t *alpha,
                                   const uint32_t *u, const uint32_t *v, uint32_t nuv, const uint32_t *d_table,
                                   uint32_t npoints, uint32_t com_scale, uint32_t msm_size, uint32_t *m_out,
                                   uint32_t *transcript, uint32_t *n_rounds, uint32_t *S_claim, uint32_t *com_A_out,
                                   uint32_t *com_m_out, double *commit_seconds);
/* tLookupRangeMapping with table map[len] (host int32) and random combiner r. */
int grape_host_tlookup_mapping_prove(const uint32_t *d_S_in, const uint32_t *d_S_out, uint32_t D, int32_t low,
                                     uint32_t len, const int32_t *map, const uint32_t *alpha, const uint32_t *r,
                                     const uint32_t *u, const uint32_t *v, uint32_t nuv, const uint32_t *d_table,
                                     uint32_t npoints, uint32_t com_scale, uint32_t msm_size, uint32_t *transcript,
                                     uint32_t *n_rounds, uint32_t *S_claim);
/* The same, with the count from which a table entry gets a row of the per-proof table B[t]*G_i
 * (0 = the break-even count), the commitment of A (affine, D / (msm_size*com_scale) points) and
 * hot_stats[0] = entries that got a row, hot_stats[1] = elements committed as full-width scalars
 * (both zero when the plain path was taken), hot_stats[2] = 1 when the rows were found in place:
 * lookup objects persist across calls (keyed by range, r, the mapped values and the generators) as the
 * reference's driver keeps them across the layers of a model, and the rows of an earlier proof serve
 * a later one while they cover its witness; a call with hot_min_count != 0 builds its own rows and
 * keeps none. */
int grape_host_tlookup_mapping_prove_ex(const uint32_t *d_S_in, const uint32_t *d_S_out, uint32_t D, int32_t low,
                                        uint32_t len, const int32_t *map, const uint32_t *alpha, const uint32_t *r,
                                        const uint32_t *u, const uint32_t *v, uint32_t nuv, const uint32_t *d_table,
                                        uint32_t npoints, uint32_t com_scale, uint32_t msm_size, uint32_t *transcript,
                                        uint32_t *n_rounds, uint32_t *S_claim, uint32_t hot_min_count, uint32_t *com_A_out,
                                        uint64_t *hot_stats);
/* Host-side scalar arithmetic checks: out = a op b with op in {0:+, 1:-, 2:*, 3: a^-1}. */
int grape_host_fr_op(int op, const uint32_t *a, const uint32_t *b, uint32_t *out);
/* k * G as a host computation (affine out) */
int grape_host_g1_mul_generator(const uint32_t *k_mont, uint32_t *out_affine);

/* single_commit (src/Hyrax.cu:176-185): one row of N full-width scalars against the reference-format
 * table; the Jacobian result is returned in affine form on the host. */
int grape_host_single_commit(const uint32_t *d_scalars, uint32_t N, const uint32_t *d_table, uint32_t npoints,
                             uint32_t *out_affine);
/* File helpers (ioutils.hpp): op 0 = savebin, 1 = loadbin of `size` bytes at ptr (device memory
 * when is_gpu != 0); findsize; load_data into a fresh device buffer (*d_out, *n elements);
 * generate_data (std::mt19937(123456) int32) into a fresh device buffer. */
int grape_host_bin_io(int op, const char *filename, void *ptr, size_t size, int is_gpu);
unsigned long grape_host_findsize(const char *filename);
int grape_host_load_data(const char *filename, int32_t **d_out, uint32_t *n);
int grape_host_generate_data(int32_t **d_out, uint32_t size);

/* Quantised-layer witness generator (witness.hpp; zzllama/llama/model.py).  d_weights9: device int32
 * pointers in the order Q, K, V, O, gate, up, down, NormFirst, NormSecond.  _names writes the tensor
 * names separated by '\n' into buf (NUL-terminated); _tensor returns the device pointer and element
 * count of one tensor; _save appends all tensors to <dir>/<W|Q|R>/<name>-<group>.bin. */
int grape_host_layer_witness_new(void **handle, uint32_t seq_len, uint32_t dim, uint32_t hidden);
int grape_host_layer_witness_generate(void *handle, const int32_t *d_x, const int32_t *const *d_weights9, const int32_t *d_exp,
                                      const int32_t *d_silu, double eps);
int grape_host_layer_witness_names(void *handle, char *buf, size_t cap);
int grape_host_layer_witness_tensor(void *handle, const char *name, const int32_t **d_ptr, size_t *size);
int grape_host_layer_witness_save(void *handle, const char *dir, uint32_t group);
int grape_host_layer_witness_free(void *handle);
/* The exp (2^20 entries) and SiLU (2^19 entries) tables into host arrays; round-to-nearest-even float16. */
int grape_host_witness_tables(int32_t *exp_out, int32_t *silu_out);
double grape_host_to_float16(double x);

#ifdef __cplusplus
}
#endif
#endif
