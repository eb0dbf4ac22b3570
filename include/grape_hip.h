/*
 * grape_hip.h — C ABI of the MI355X (gfx950) kernels behind Grape's proving hot path.
 *
 * Everything the host-side classes (FrTensor, Hyrax, prove_matmul, tLookupRange, ...) need from
 * the GPU goes through these functions; they are the only place HIP is used.  Conventions:
 *
 *   - every pointer named d_* is DEVICE memory, everything else is host memory;
 *   - an Fr element is 8 x u32 little-endian limbs (32 bytes, 32-byte aligned arrays) holding the
 *     canonical Montgomery residue x*2^256 mod r — the reference's fr_t image
 *     (include/field/mont_t.cuh:33, include/field/bls12-381.cuh:24-45), which is also the image
 *     of the host Fr (4 x u64), so values move between host and device by plain copies as in
 *     src/fr-tensor.cu:214,352,437;
 *   - an Fp element is 12 x u32 (x*2^384 mod p); an affine G1 point is {x,y} = 96 bytes with
 *     infinity = all zero (include/curve/affine_t.cuh:28-39); a Jacobian point is {X,Y,Z} = 144
 *     bytes with Z = 0 for infinity; an XYZZ accumulator is {X,Y,ZZ,ZZZ} = 192 bytes.  These are
 *     the sizes of the BLS12-381 library; the BN254 build of the same sources (libgrape_hip_bn254.so,
 *     include/field/alt_bn128.cuh) has Fp = 8 x u32 (x*2^256 mod p) and points of 64 / 96 / 128 bytes;
 *   - every function returns 0 on success and a negative GRAPE_E* code otherwise;
 *     grape_last_error() gives the message.  Nothing is printed, nothing throws;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Kernels are only
 *     enqueued; results are ready after grape_stream_sync(stream).  Functions that return a value
 *     to the host say so and synchronise the stream themselves;
 *   - one host thread per stream.  Internal scratch memory (partial sums, fold buffers, MSM
 *     partials) is pooled per stream, so calls on DIFFERENT streams - from one host thread or from
 *     several - never share it and may overlap; calls on the same stream are ordered by the
 *     stream.  A buffer of the pool grows on demand (hipMalloc after waiting for its stream), so a
 *     caller who captures a stream into a graph runs each shape once before capturing;
 *   - grape_free does NOT wait for the device the way cudaFree / hipFree do: it only hands the block
 *     to the allocation cache described below, and the wait happens when that block is handed out
 *     again.  A caller that relied on cudaFree as a synchronisation point calls grape_stream_sync.
 */
#ifndef GRAPE_HIP_H
#define GRAPE_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GRAPE_OK 0
#define GRAPE_EINVAL (-1)   /* bad argument (null pointer, size mismatch, unsupported shape) */
#define GRAPE_EHIP (-2)     /* a HIP runtime call failed */
#define GRAPE_ENOMEM (-3)   /* device allocation failed */

typedef void *grape_stream_t;

/* ------------------------------------------------------------------ runtime ------------------ */
/* Select the device and create the per-device scratch pool.  Must be called once before use. */
int grape_init(int device);
const char *grape_last_error(void);
int grape_stream_sync(grape_stream_t stream);
/* Thin allocation / copy helpers so host code needs no HIP headers (replace the reference's
 * direct cudaMalloc / cudaMemcpy / cudaFree calls, e.g. src/fr-tensor.cu:371-374,322-328). */
int grape_malloc(void **d_ptr, size_t bytes);
int grape_free(void *d_ptr);
/* grape_free keeps the block for grape_malloc to hand out again (to a request of exactly the same
 * size; up to GRAPE_ALLOC_CACHE_GIB in total, default 32, 0 switches it off): the host classes
 * allocate and free a tensor per call as the reference does, and the driver's allocation calls
 * cost tens of microseconds for small blocks and milliseconds and more for multi-GiB ones.  This gives every kept block back to the
 * driver (it also happens by itself when an allocation fails).  No counterpart in the reference. */
int grape_alloc_cache_release(size_t *bytes_released);
/* Host to device, ordered like any other work on `stream`; the host buffer may be reused as soon as
 * the call returns.  At most 1 KiB (a scalar, a vector of challenges) is carried by a small kernel
 * as its argument and the call does not wait; a longer copy waits for the stream. */
int grape_memcpy_h2d(void *d_dst, const void *src, size_t bytes, grape_stream_t stream);
int grape_memcpy_d2h(void *dst, const void *d_src, size_t bytes, grape_stream_t stream); /* syncs */
int grape_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes, grape_stream_t stream);
int grape_memset_zero(void *d_ptr, size_t bytes, grape_stream_t stream);

/* ------------------------------------------------------------------ Fr tensors --------------- */
/* out[i] = a[i] (+,-,*) b[i]; out may alias a or b.
 * Fr_elementwise_add/sub/mul, src/fr-tensor.cu:74-101. */
int grape_fr_add(uint32_t *d_out, const uint32_t *d_a, const uint32_t *d_b, size_t n, grape_stream_t stream);
int grape_fr_sub(uint32_t *d_out, const uint32_t *d_a, const uint32_t *d_b, size_t n, grape_stream_t stream);
int grape_fr_mul(uint32_t *d_out, const uint32_t *d_a, const uint32_t *d_b, size_t n, grape_stream_t stream);
/* out[i] = a[i] (+,*) x[0], x one device element.  Fr_broadcast_add/mul, src/fr-tensor.cu:88-108. */
int grape_fr_bcast_add(uint32_t *d_out, const uint32_t *d_a, const uint32_t *d_x, size_t n, grape_stream_t stream);
int grape_fr_bcast_mul(uint32_t *d_out, const uint32_t *d_a, const uint32_t *d_x, size_t n, grape_stream_t stream);
/* out[i] = x[i] + r * y[i] with one device scalar r (out may alias x or y): the combined witness
 * S_in + r*S_out of a mapping lookup in one pass (src/tlookup.cu:407-410 takes three). */
int grape_fr_axpy(uint32_t *d_out, const uint32_t *d_x, const uint32_t *d_r, const uint32_t *d_y, size_t n, grape_stream_t stream);
/* Integer embedding, negatives as r-|v|.  int_to_fr / uint_to_fr, src/fr-tensor.cu:30-46. */
int grape_fr_from_i32(uint32_t *d_out, const int32_t *d_in, size_t n, grape_stream_t stream);
int grape_fr_from_u32(uint32_t *d_out, const uint32_t *d_in, size_t n, grape_stream_t stream);
/* Enter / leave Montgomery form, in place allowed.  to_kernel / from_kernel, src/fr-tensor.cu:110-120. */
int grape_fr_to_mont(uint32_t *d_out, const uint32_t *d_in, size_t n, grape_stream_t stream);
int grape_fr_from_mont(uint32_t *d_out, const uint32_t *d_in, size_t n, grape_stream_t stream);
/* out[i] = 1/in[i], 1/0 = 0, by batched Montgomery inversion (same values as the per-element
 * reciprocal of inverse_kernel, src/fr-tensor.cu:122-126).  out may alias in. */
int grape_fr_batch_inverse(uint32_t *d_out, const uint32_t *d_in, size_t n, grape_stream_t stream);
/* out[i] = 1/(in[i] + beta[0]).  tlookup_inv_kernel, src/tlookup.cu:52-62. */
int grape_fr_shift_inverse(uint32_t *d_out, const uint32_t *d_in, const uint32_t *d_beta, size_t n, grape_stream_t stream);
/* d_out[0] = sum of the first n elements; the input is left untouched (the reference's
 * FrTensor::sum, src/fr-tensor.cu:415-440, clobbers it for n > 256 — not reproduced). */
int grape_fr_sum(uint32_t *d_out, const uint32_t *d_in, size_t n, grape_stream_t stream);
/* Row sums broadcast back over each row of `dim` columns.  sum_by_dim_kernel, src/fr-tensor.cu:155-163. */
int grape_fr_sum_by_dim(uint32_t *d_out, const uint32_t *d_in, size_t rows, size_t dim, grape_stream_t stream);
/* Row padding N -> pad_N columns, pad_size output elements.  pad_fr_kernel / pad_int_kernel,
 * src/fr-tensor.cu:18-28.  out must not alias in. */
int grape_fr_pad(uint32_t *d_out, const uint32_t *d_in, uint32_t N, uint32_t pad_N, size_t pad_size,
                 const uint32_t *d_pad_val, grape_stream_t stream);
int grape_i32_pad(int32_t *d_out, const int32_t *d_in, uint32_t N, uint32_t pad_N, size_t pad_size, grape_stream_t stream);
/* The same with a fill value other than zero (pads the table indices of a lookup witness with the
 * index of the padding value). */
int grape_i32_pad_fill(int32_t *d_out, const int32_t *d_in, uint32_t N, uint32_t pad_N, size_t pad_size, int32_t fill,
                       grape_stream_t stream);
/*
 * Fold (partial multilinear evaluation) in place: view the first N elements of t as
 * [N/(c*gap)][c][gap], bind the c axis with challenges x[id], x[id+1], ... (index bit j of the
 * axis pairs with x[id+j]; a missing partner of an odd tail counts as zero) and leave the
 * [N/(c*gap)][gap] result contiguous at the front of t.
 * FrTensor::partial_eval, src/fr-tensor.cu:330-344 with Fr_partial_me :168-188 and
 * Fr_partial_eval_kernel :53-72.  x is a device array of challenges.
 */
int grape_fr_fold(uint32_t *d_t, size_t N, const uint32_t *d_x, uint32_t c, uint32_t id, uint32_t gap, grape_stream_t stream);
/*
 * The same fold of a tensor of N 32-bit integers, i.e. of the field tensor that FrTensor::get_data
 * (src/fr-tensor.cu:30-39: |x| as a residue, negated for x < 0) would make of d_in - without making it:
 * the first pass reads the integers and writes field elements into d_out, the later passes work there.
 * The [N/(c*gap)][gap] result is left at the front of d_out, which must hold
 * grape_fr_fold_i32_elems(N, c, gap) elements; d_in is not modified.  For the reference's drivers'
 * get_data + partial_eval / operator() / Hyrax::open on an integer tensor (test/llm.cu:99-125).
 */
size_t grape_fr_fold_i32_elems(size_t N, uint32_t c, uint32_t gap);
int grape_fr_fold_i32(uint32_t *d_out, const int32_t *d_in, size_t N, const uint32_t *d_x, uint32_t c, uint32_t id, uint32_t gap,
                      grape_stream_t stream);

/* ------------------------------------------------------------------ sumcheck ----------------- */
/*
 * One round of the two-tensor sumcheck kernel (sumcheck_kernel, src/prove.cu:29-46) fused with the
 * three reductions the reference runs afterwards (src/prove.cu:101-105): for g < out_size with
 * hi = X[g+out_size] (zero when g+out_size >= in_size): Xa = hi - X[g], Xb = X[g];
 * A[g] = Aa*v + Ab, B[g] = Ba*v + Bb (in place) and
 * d_sums[0] = sum Ab*Bb, d_sums[1] = sum (Aa*Bb + Ab*Ba), d_sums[2] = sum Aa*Ba.
 */
int grape_sumcheck_round2(uint32_t *d_A, uint32_t *d_B, uint32_t in_size, uint32_t out_size,
                          const uint32_t *d_v, uint32_t *d_sums, grape_stream_t stream);
/* The same round when the caller holds the running claim: the sum of a round's polynomial over
 * {0, 1} equals the value the previous round's polynomial took at its challenge (the check
 * src/prove.cu:107 makes), so with that value in *d_claim (device, one element) the kernel sums only
 * c0 and c2 and takes c1 = claim - 2 c0 - c2 - one limb product per index pair fewer, which is what a
 * long round is bound by.  d_sums receives (c0, c1, c2) as above and *d_claim the next round's claim
 * c0 + c1 v + c2 v^2, so a chain of rounds needs the claim only once.  A caller that uses it gives up
 * the per-round check of the sums against the claim; the check of the final claim against the folded
 * values (src/prove.cu:204) still covers the whole chain. */
int grape_sumcheck_round2_claim(uint32_t *d_A, uint32_t *d_B, uint32_t in_size, uint32_t out_size, const uint32_t *d_v,
                                uint32_t *d_claim, uint32_t *d_sums, grape_stream_t stream);
/* The same round for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * results as grape_sumcheck_round2, but the per-workgroup partial sums go to a fixed 384 KiB array
 * inside the library's code object instead of the growing scratch pool, so the call never calls
 * hipMalloc / hipFree; out_size is limited to 2^26 indices (GRAPE_EINVAL beyond).  grape_init looks the
 * array's address up for its device (a call on a device grape_init has not seen does so itself on
 * first use).  Every call on one GPU shares that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe. */
int grape_sumcheck_round2_noalloc(uint32_t *d_A, uint32_t *d_B, uint32_t in_size, uint32_t out_size,
                                  const uint32_t *d_v, uint32_t *d_sums, grape_stream_t stream);
/* The last rounds of the same sumcheck in one launch (one workgroup, a barrier between rounds):
 * `rounds` successive rounds starting from in_size <= 512 elements, out_size = 2^(ceil(log2 in_size) - 1)
 * and halving from there; round i takes its challenge from d_v_end[-(i+1)] (the reference walks
 * its challenge array backwards, src/prove.cu:101) and leaves its three sums in d_sums[3i..3i+2].
 * Same results as `rounds` calls of grape_sumcheck_round2. */
int grape_sumcheck_round2_tail(uint32_t *d_A, uint32_t *d_B, uint32_t in_size, uint32_t rounds,
                               const uint32_t *d_v_end, uint32_t *d_sums, grape_stream_t stream);
/* As above but also materialises the coefficient arrays a, b, c (needed by phase 1, which folds
 * them over the remaining layer bits, src/prove.cu:64-66).  d_sums may be NULL. */
int grape_sumcheck_round2_coeffs(uint32_t *d_A, uint32_t *d_B, uint32_t *d_a, uint32_t *d_b, uint32_t *d_c,
                                 uint32_t in_size, uint32_t out_size, const uint32_t *d_v,
                                 uint32_t *d_sums, grape_stream_t stream);
/* Single-tensor round (sumcheck_kernel, src/prove.cu:14-27): X[g] = Xa*v + Xb, a[g] = Xa, b[g] = Xb. */
int grape_sumcheck_round1(uint32_t *d_X, uint32_t *d_a, uint32_t *d_b, uint32_t in_size, uint32_t out_size,
                          const uint32_t *d_v, grape_stream_t stream);

/* ------------------------------------------------------------------ eq-weighted rounds -------- */
/*
 * Pyramid of eq tables for nu challenges u (device array): level j (2^j elements) starts at element
 * offset 2^j - 1 and holds eq(u[0..j-1], i) = prod_{b<j} (u_b if bit_b(i) else 1 - u_b), for
 * j = 0..nu; grape_eq_pyramid_elems(nu) = 2^(nu+1) - 1 elements in all.  A sumcheck that binds the
 * top variable first uses level nu-1 in its first round, nu-2 in the second, ...: no table is
 * recomputed or halved between rounds (the reference folds its coefficient arrays over the
 * remaining variables of u in every round instead: src/prove.cu:64-66,142-154, src/tlookup.cu:129-138).
 */
size_t grape_eq_pyramid_elems(uint32_t nu);
int grape_eq_pyramid(uint32_t *d_pyr, const uint32_t *d_u, uint32_t nu, grape_stream_t stream);
/*
 * One round of a sumcheck over sum_x e[x] * A(x) * (S(x) + beta), fused with the fold of both
 * tensors: for g < n_out, with X0 = X[g], X1 = X[g + n_out] (zero when g + n_out >= in_size),
 *   d_sums[0..2] = sum_g e[g'] * coefficients (low to high) of (A0 + t(A1-A0)) * (S0 + beta + t(S1-S0))
 *   d_sums[3], d_sums[4] = sum_g A0, sum_g (A1 - A0)                    (only when plain_sums != 0)
 *   A[g] = A0 + v(A1 - A0), S[g] = S0 + v(S1 - S0)                      (in place)
 * d_beta may be NULL (beta = 0).  d_e is the weight table of this round (a level of the pyramid above).
 * When the tensors' rows hold rowlen elements but the weights live on rows padded to rowpad entries
 * (rows of 11008 with weights over 16384), g' = g + (g / rowlen) * (rowpad - rowlen); otherwise pass
 * rowlen = rowpad and g' = g.  d_sums holds 3 (5 with plain_sums) elements.
 * plain_sums == 2 (with rowlen == rowpad and in_size == 2 n_out) is the round of a caller that knows
 * A[i] * (S[i] + beta) = 1 at every index and weights that sum to one - the first round of a logUp
 * proof over A = 1/(S + beta): d_sums[0] = 1 and d_sums[1] = -d_sums[2] then follow without being
 * summed, and the pass takes one weight product per index instead of two.  The five sums equal those
 * of plain_sums == 1 whenever the statement holds.
 * plain_sums == 3 (d_beta given, n_out >= 2^16) leaves the middle coefficient out: d_sums[1] = 0 and the
 * other four sums as with plain_sums == 1.  It is for a caller that holds the round's claim - the sum of
 * the round polynomial over {0, 1}, src/tlookup.cu:228 - from which the middle coefficient follows.
 * One pass replaces sumcheck_kernel + three folds of coefficient arrays per round in eleMul_sumcheck
 * (src/prove.cu:119-172) and tLookup_poly_kernel + three multilinear evaluations +
 * tLookup_poly_sum_kernel + two sums + the reduce kernel in tLookup_phase1 (src/tlookup.cu:117-151,216-244).
 */
int grape_wround2(uint32_t *d_A, uint32_t *d_S, const uint32_t *d_beta, const uint32_t *d_e, uint32_t in_size, uint32_t n_out,
                  uint32_t rowlen, uint32_t rowpad, const uint32_t *d_v, int plain_sums, uint32_t *d_sums, grape_stream_t stream);
/*
 * grape_wround2 in two halves, for a prover that queues all rounds of a proof and reads their sums once at the
 * end (the reference's tLookup_phase1 loop, src/tlookup.cu:216-244, copies and waits once per round): the finishing of
 * a round's sums is then not part of the chain of rounds and may run on another stream, and the tables of the
 * challenges' multiples are made by one launch for the whole proof.
 *   grape_fold_tables:  d_tabs + GRAPE_FOLD_TABLE_WORDS * k (int32 words) receives the table of d_v[k], k < count <= 64.
 *   grape_wround2_queue: the pass over the operands of grape_wround2 (same arguments and folds); the round's
 *     per-workgroup sums go to d_partial (grape_wround2_partial_bytes(n_out) bytes, 16-byte aligned, the
 *     caller's own for as long as the round is unfinished).  d_tab: the table of *d_v made by grape_fold_tables
 *     (rounds of n_out >= 2^16; plain_sums == 3 requires it) or NULL for the single-product fold.
 *   grape_wround2_finish: d_sums[0..4] (d_sums[0..2] with plain_sums == 0) from d_partial, as grape_wround2 leaves
 *     them; n_out and plain_sums as given to grape_wround2_queue.
 */
#define GRAPE_FOLD_TABLE_WORDS 100 /* int32 words of one challenge's table */
size_t grape_wround2_partial_bytes(uint32_t n_out);
int grape_fold_tables(int32_t *d_tabs, const uint32_t *d_v, uint32_t count, grape_stream_t stream);
int grape_wround2_queue(uint32_t *d_A, uint32_t *d_S, const uint32_t *d_beta, const uint32_t *d_e, uint32_t in_size, uint32_t n_out,
                        uint32_t rowlen, uint32_t rowpad, const uint32_t *d_v, int plain_sums, const int32_t *d_tab,
                        uint32_t *d_partial, grape_stream_t stream);
int grape_wround2_finish(uint32_t *d_sums, const uint32_t *d_partial, uint32_t n_out, int plain_sums, grape_stream_t stream);
/*
 * grape_wround2_queue with plain_sums == 2 for a logUp tensor that was never written out: the first round of a
 * lookup over 2 n_out elements reads d_A[i] as d_B[d_idx1[i] - 1] (d_idx1 as grape_tlookup_index_inverse leaves it with
 * d_A == NULL and no unmatched element; an index 0 reads entry 0) and writes the folded tensor to d_A[0 .. n_out);
 * d_S is folded in place.  d_tab is required (n_out >= 2^16).  Finished by grape_wround2_finish(.., plain_sums = 2).
 * Together with the pass over the witness this leaves out one write and one read of the whole tensor
 * (tlookup_inv_kernel's output, src/tlookup.cu:52-62, as the first round's input, :117-151).
 */
int grape_wround2_queue_indexed(uint32_t *d_A, uint32_t *d_S, const int32_t *d_idx1, const uint32_t *d_B, uint32_t len,
                                const uint32_t *d_beta, const uint32_t *d_e, uint32_t n_out, const uint32_t *d_v, const int32_t *d_tab,
                                uint32_t *d_partial, grape_stream_t stream);
/*
 * One round of matmul_sumcheck_phase1 (src/prove.cu:49-85): grape_sumcheck_round2 on indices
 * g = seg * seglen + k where every index of a segment carries the weight d_e[seg]
 * (out_size / seglen segments): d_sums[t] = sum_seg d_e[seg] * sum_k coefficient_t(seg, k); A and B
 * are folded in place.
 */
int grape_sumcheck_round2_seg(uint32_t *d_A, uint32_t *d_B, uint32_t in_size, uint32_t out_size, uint32_t seglen,
                              const uint32_t *d_e, const uint32_t *d_v, uint32_t *d_sums, grape_stream_t stream);
/*
 * Weighted sums of one tensor against several weight tables at once (combine_claims,
 * src/prove.cu:245-300, evaluates the two coefficient arrays at the remaining variables of every
 * claim's point): for j < num (at most 16),
 *   d_sums[2j] = sum_g e_j[g] * X0,  d_sums[2j+1] = sum_g e_j[g] * (X1 - X0),   g < n_out.
 * e_tables is a host array of num device pointers.  X is not modified.
 */
int grape_wsum1_multi(const uint32_t *d_X, const uint32_t *const *e_tables, uint32_t num, uint32_t in_size, uint32_t n_out,
                      uint32_t *d_sums, grape_stream_t stream);

/* ------------------------------------------------------------------ tlookup / logUp ---------- */
/* hist[(v - low) as integer] += 1 for n values (Montgomery Fr); hist has `len` u32 counters and
 * is NOT cleared here.  Values outside [low, low+len) are ignored.
 * get_histogram_kernel, src/tlookup.cu:5-14. */
int grape_tlookup_hist(uint32_t *d_hist, const uint32_t *d_vals, size_t n, int32_t low, uint32_t len, grape_stream_t stream);
/* out[i] = (v_i - low) + 1 as an int32 for n values (Montgomery Fr) inside [low, low+len), 0 for a
 * value outside: the table index of each witness element, shifted by one (the index the
 * reference derives inside get_histogram_kernel, src/tlookup.cu:9-12).  Feeds the indexed
 * commitment of A = 1/(S+beta) below. */
int grape_tlookup_index(int32_t *d_out, const uint32_t *d_vals, size_t n, int32_t low, uint32_t len, grape_stream_t stream);
/* Index and logUp tensor in one pass over the witness: d_idx1 as grape_tlookup_index makes it from
 * d_key (the witness of a range lookup, the input component of a mapping lookup), and
 * d_A[i] = d_B[index] = 1/(T[index] + beta) where the element matches its table entry: for a range
 * lookup (d_cmp = d_cmp_table = NULL) every key inside the table does; for a mapping lookup the
 * output component must equal the table's, d_cmp[i] == d_cmp_table[index].  Other elements are
 * left unwritten and counted in *mismatches (host; the call synchronises), as
 * grape_tlookup_inverse_by_table does.  Replaces grape_tlookup_index + that call (src/tlookup.cu:9-12
 * and :52-62) where the witness needs no padding. */
int grape_tlookup_index_inverse(int32_t *d_idx1, uint32_t *d_A, const uint32_t *d_key, size_t n, int32_t low, uint32_t len,
                                const uint32_t *d_B, const uint32_t *d_cmp, const uint32_t *d_cmp_table, size_t *mismatches,
                                grape_stream_t stream);
/* The same pass queued without waiting: the count of unmatched elements is left in the device word
 * d_mismatches (cleared by the call), for a caller that has more to queue before it reads the count.
 * d_A == NULL: indices and the count only (a caller whose first round gathers d_B[index] itself,
 * grape_wround2_queue_indexed). */
int grape_tlookup_index_inverse_nowait(int32_t *d_idx1, uint32_t *d_A, const uint32_t *d_key, size_t n, int32_t low, uint32_t len,
                                       const uint32_t *d_B, const uint32_t *d_cmp, const uint32_t *d_cmp_table,
                                       uint32_t *d_mismatches, grape_stream_t stream);
/* The pass over a witness that is still a tensor of 32-bit integers (what a driver would embed with
 * FrTensor::get_data first, test/llm.cu:77): indices, check, count and d_A as above (d_A may be NULL), and the
 * witness as field elements in d_S: d_S[i] = key_i for a range lookup (d_cmp = d_cmp_table = d_r = NULL),
 * d_S[i] = key_i + r * cmp_i for a mapping lookup (src/tlookup.cu:407-410), whose second components are
 * compared with the INTEGER table d_cmp_table[index].  Queued without waiting, as the call above. */
int grape_tlookup_index_embed_i32_nowait(int32_t *d_idx1, uint32_t *d_A, uint32_t *d_S, const int32_t *d_key, const int32_t *d_cmp,
                                         size_t n, int32_t low, uint32_t len, const uint32_t *d_B, const int32_t *d_cmp_table,
                                         const uint32_t *d_r, uint32_t *d_mismatches, grape_stream_t stream);
/* The same histogram from indices already made by grape_tlookup_index (d_idx1[i] = index + 1,
 * 0 = outside the table): hist[d_idx1[i] - 1] += 1. */
int grape_tlookup_hist_index(uint32_t *d_hist, const int32_t *d_idx1, size_t n, uint32_t len, grape_stream_t stream);
/* A = 1/(S + beta) read from the lookup table instead of computed (tlookup_inv_kernel,
 * src/tlookup.cu:52-62, is an inversion per element): where S[i] equals the table entry
 * T[d_idx1[i] - 1], A[i] = B[d_idx1[i] - 1] with B = 1/(T + beta).  Elements outside the table or
 * different from their entry are left unwritten and counted in *mismatches (host; the call
 * synchronises); a caller that sees mismatches != 0 inverts the tensor with
 * grape_fr_shift_inverse instead. */
int grape_tlookup_inverse_by_table(uint32_t *d_A, const uint32_t *d_S, const int32_t *d_idx1, const uint32_t *d_T,
                                   const uint32_t *d_B, size_t n, uint32_t len, size_t *mismatches, grape_stream_t stream);
/*
 * Occupied-entry selection for the commitment of a logUp tensor A = B[index] whose table is too
 * large for a table of B[t]*G_i over every entry t (the mapping lookups' 2^19..2^20 entries): the
 * elements of A take only the values of the entries that occur in the witness, and activations
 * concentrate on few of them.  Entries with d_hist[t] >= min_count get a slot, in table order, at
 * most max_hot of them: d_slot1[t] = slot + 1 (0 for the others), d_hot_list[slot] = t.
 * info (HOST, two words; the call synchronises): info[0] = number of slots given, info[1] =
 * number of witness elements whose entry got none.  The committer then builds the scaled table of
 * B[d_hot_list[.]] (grape_fr_gather + grape_g1_scaled_table_gen), commits the slotted elements at
 * one addition each (grape_tlookup_hot_index + grape_commit_i32) and the others as full-width
 * scalars (grape_fr_mask_cold + grape_commit_fr*), and adds the two (grape_g1_affine_add).  The
 * reference commits A as a full-width tensor (src/tlookup.cu:320, :433); the group elements are
 * the same.  No counterpart in the reference.
 */
int grape_tlookup_hot_select(const uint32_t *d_hist, uint32_t len, uint32_t min_count, uint32_t max_hot, int32_t *d_slot1,
                             uint32_t *d_hot_list, uint64_t *info, grape_stream_t stream);
/* A slot assignment kept from an earlier witness of the same table (the rows of B[t]*G_i it stands
 * for are kept with it): *cold_elements (HOST; the call synchronises) = number of elements of the
 * witness counted in d_hist whose entry has no slot in d_slot1, i.e. what would have to be
 * committed as full-width scalars if the rows were used again.  No counterpart in the reference. */
int grape_tlookup_hot_coverage(const uint32_t *d_hist, uint32_t len, const int32_t *d_slot1, uint64_t *cold_elements,
                               grape_stream_t stream);
/* out[i] = d_slot1[d_idx1[i] - 1] (0 when d_idx1[i] is 0 or above len). */
int grape_tlookup_hot_index(int32_t *d_out, const int32_t *d_idx1, size_t n, const int32_t *d_slot1, uint32_t len,
                            grape_stream_t stream);
/* out[i] = X[i] where d_hot1[i] == 0, zero elsewhere (n field elements). */
int grape_fr_mask_cold(uint32_t *d_out, const uint32_t *d_X, const int32_t *d_hot1, size_t n, grape_stream_t stream);
/* out[i] = src[d_list[i]] (n field elements). */
int grape_fr_gather(uint32_t *d_out, const uint32_t *d_src, const uint32_t *d_list, size_t n, grape_stream_t stream);
/* T[i] = low + i (+ r*map[i] when d_map != NULL), B[i] = 1/(T[i] + beta).
 * tlookuprange_init_kernel / tLookupRangeMapping_init_kernel, src/tlookup.cu:16-50. */
int grape_tlookup_init(uint32_t *d_T, uint32_t *d_B, int32_t low, uint32_t len, const uint32_t *d_beta,
                       const uint32_t *d_map, const uint32_t *d_r, grape_stream_t stream);
/* out0 = A0*(S0+beta), out1 = A1*(S0+beta) + A0*S1, out2 = A1*S1 with X0 = X[t], X1 = X[t+n_out]-X[t].
 * tLookup_poly_kernel, src/tlookup.cu:64-78.  d_beta may be NULL (beta = 0, as :181). */
int grape_tlookup_poly(const uint32_t *d_A, const uint32_t *d_S, const uint32_t *d_beta, uint32_t *d_out0,
                       uint32_t *d_out1, uint32_t *d_out2, size_t n_out, grape_stream_t stream);
/* out0 = A[t], out1 = A[t+n_out] - A[t].  tLookup_poly_sum_kernel, src/tlookup.cu:80-88. */
int grape_tlookup_poly_sum(const uint32_t *d_A, uint32_t *d_out0, uint32_t *d_out1, size_t n_out, grape_stream_t stream);
/*
 * Fused round of the logUp sumcheck: with X_t = X0 + t*X1 on the MSB split of size n_out and
 * e[x] = eq(u_low, x) held in d_eq (n_out entries), writes into d_sums (8 elements):
 *   [0..2] sum_x e[x] * coefficients of (A0 + tA1)(S0 + beta + tS1)      (src/tlookup.cu:129-138)
 *   [3..4] sum_x A0, sum_x A1                                           (:142-146)
 * Nothing is modified.  This replaces tLookup_poly_kernel + three full multilinear evaluations
 * + tLookup_poly_sum_kernel + two sums of the reference with one pass over A, S and e.
 */
int grape_tlookup_round_sums(const uint32_t *d_A, const uint32_t *d_S, const uint32_t *d_beta, const uint32_t *d_eq,
                             size_t n_out, uint32_t *d_sums, grape_stream_t stream);
/* d_sums[0..2] = sums of the coefficients of (m0 + t m1)(B0 + t B1) (src/tlookup.cu:180-185). */
int grape_tlookup_mb_sums(const uint32_t *d_m, const uint32_t *d_B, size_t n_out, uint32_t *d_sums, grape_stream_t stream);
/*
 * One round of the table side of the logUp sumcheck (the terms over B, T and m of tLookup_phase2,
 * src/tlookup.cu:153-190) in one launch: d_sums[0..4] as grape_tlookup_round_sums(B, T, beta, eq),
 * d_sums[5..7] as grape_tlookup_mb_sums(m, B), then B, T and m are folded in place by the challenge
 * d_v as grape_fr_fold_msb_multi does (their first n_out elements are the folded tensors).
 */
int grape_tlookup_table_round(uint32_t *d_B, uint32_t *d_T, uint32_t *d_m, const uint32_t *d_beta, const uint32_t *d_eq,
                              size_t n_out, const uint32_t *d_v, uint32_t *d_sums, grape_stream_t stream);
/* e[i] = prod_j (u_j if bit_j(i) else 1 - u_j) for i < 2^nu; u is a device array of nu challenges. */
int grape_eq_table(uint32_t *d_eq, const uint32_t *d_u, uint32_t nu, grape_stream_t stream);
/* e'[x] = e[x] + e[x + n_out] for x < n_out: the table of the remaining variables after the
 * top one is dropped. */
int grape_eq_table_halve(uint32_t *d_eq, size_t n_out, grape_stream_t stream);
/* MSB fold of k tensors at once: X[g] = X[g] + v*(X[g+n_out]-X[g]) for each of the k device
 * pointers in d_ptrs (host array of device pointers), in place.
 * tLookup_phase2_reduce_kernel, src/tlookup.cu:100-113; FrTensor::partial_eval(size,v,2,0,size/2). */
int grape_fr_fold_msb_multi(uint32_t *const *ptrs, uint32_t k, size_t n_out, const uint32_t *d_v, grape_stream_t stream);

/* ------------------------------------------------------------------ G1 / Hyrax --------------- */
/* The standard BLS12-381 G1 generator, affine Montgomery, to host memory (96 bytes). */
int grape_g1_generator(uint32_t *out_affine);
/* out[i] = k[i] * base for n canonical (non-Montgomery) 256-bit scalars k and one affine base
 * point; used to derive seeded generators (the reference draws bn128::random_element(),
 * src/ec_operation.cu:31-36). */
int grape_g1_scalar_mul_base(uint32_t *d_out_affine, const uint32_t *d_k_plain, const uint32_t *d_base_affine,
                             size_t n, grape_stream_t stream);
/* The reference's generator table: table[w*N + i] = w*G_i for w < W as affine points, entry
 * w = 0 is infinity.  precompute_generators + naive_msm, src/ec_operation.cu:15-49. */
int grape_g1_table_gen(uint32_t *d_table_affine, const uint32_t *d_gens_affine, size_t N, uint32_t W, grape_stream_t stream);
/*
 * Wide fixed-base table for the commitment kernels:
 *   table[(w*K + (k-1))*N + i] = k * 2^(c*w) * G_i,  k = 1..K, w < nw
 * With c = 16, nw = 1, K = 32768 a signed 16-bit scalar is ONE mixed addition; with c = 8,
 * nw = 32, K = 128 a 255-bit scalar is 32 signed-digit additions into a single accumulator.
 * The table is private to this library (only the commitment entry points read it): each entry
 * holds the affine coordinates in the working form of the commitment kernels - on BLS12-381
 * 2 x 14 limbs of 28 bits (Montgomery radix 2^392) padded to 128 bytes, so a gather is exactly one
 * cache line; on BN254 2 x 10 limbs (radix 2^280) stored dense in 80 bytes.
 * Size: grape_g1_wide_table_bytes(N, nw, K) = nw*K*N entries of 128 bytes (80 in the BN254 build).
 */
int grape_g1_wide_table_gen(uint32_t *d_table_affine, const uint32_t *d_gens_affine, size_t N, uint32_t c, uint32_t nw,
                            uint32_t K, grape_stream_t stream);
size_t grape_g1_wide_table_bytes(size_t N, uint32_t nw, uint32_t K);
/*
 * Scaled table out[t*ncols + i] = s_t * G_i for `len` scalars s_t (device, Montgomery Fr) and the
 * first ncols generators, computed through a full-width wide table (c, nw, K as built above).
 * Same entry format, so grape_commit_i32(out, idx, size, rowlen, table = this, N = ncols,
 * c = log2(len)+1, nw = 1, K = len) with idx = t+1 gives sum_i s_{t_i} * G_i at ONE addition per
 * element.  Used for the logUp commitment of A = 1/(S+beta): its elements take only `len`
 * distinct values B[t] (the reference commits A as a full-width tensor, src/tlookup.cu:320).
 * No counterpart in the reference.  Size: grape_g1_wide_table_bytes(ncols, 1, len) bytes.
 */
int grape_g1_scaled_table_gen(uint32_t *d_out, const uint32_t *d_scalars_mont, size_t len, size_t ncols,
                              const uint32_t *d_wide_table, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t stream);
/*
 * Row commitments of an integer matrix: for each of size/rowlen rows,
 * C_row = sum_i s[row*rowlen + i] * G_i, i < rowlen, written as AFFINE points (96 bytes each).
 * Hyrax::commit(int*, size, N), src/Hyrax.cu:312-333 (int_windows_sum :46-65, int_windows_reduce
 * :67-87); rowlen is the reference's N*com_scale.  The wide table must have been built for
 * N >= rowlen generators with radix 2^c, nw windows and K >= 2^(c-1) (with nw = 1 any K >= 1: the
 * indexed commitments pass digits 1..K, and a larger digit returns GRAPE_EINVAL); scalars are recoded into
 * signed radix-2^c digits (2 <= c <= 24 here), so any int32 is accepted when nw*c >= 33, and the
 * int16 fast path (c = 16, nw = 1) requires -32768 <= s <= 32767 (checked on device: returns
 * GRAPE_EINVAL after synchronising if violated).  One call takes at most 2^28 scalars (GRAPE_EINVAL
 * beyond; every commitment entry point has this bound): rows are independent, so a longer tensor is
 * committed in several calls, as the host class Hyrax does.
 */
int grape_commit_i32(uint32_t *d_out_affine, const int32_t *d_scalars, size_t size, uint32_t rowlen,
                     const uint32_t *d_wide_table, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t stream);
/* grape_commit_i32 without the wait at its end: the kernels are queued and the call returns.  The
 * digit-range check lands in *d_flag (device int32 the caller owns and has cleared: set to 1 when a
 * scalar did not fit, in which case the outputs are meaningless); the caller reads it after
 * synchronising the stream.  For callers that queue other work while the commitment runs (the
 * lookups' rounds on streams of their own). */
int grape_commit_i32_nowait(uint32_t *d_out_affine, const int32_t *d_scalars, size_t size, uint32_t rowlen,
                            const uint32_t *d_wide_table, size_t N, uint32_t c, uint32_t nw, uint32_t K, int32_t *d_flag,
                            grape_stream_t stream);
/* Same for full-width Fr scalars (Montgomery form in, left untouched — the reference's
 * tensor.from()/to() round trip of src/Hyrax.cu:347,356 is not needed).
 * Hyrax::commit(FrTensor&, size, N), src/Hyrax.cu:335-359. Requires nw*c >= 255: a scalar in the
 * upper half of the field is taken as -(r - k), so magnitudes stay below 2^254 and the top window
 * never carries out. */
int grape_commit_fr(uint32_t *d_out_affine, const uint32_t *d_scalars_mont, size_t size, uint32_t rowlen,
                    const uint32_t *d_wide_table, size_t N, uint32_t c, uint32_t nw, uint32_t K, grape_stream_t stream);
/* grape_commit_fr without the wait at its end, *d_flag as in grape_commit_i32_nowait: for Hyrax::open
 * (src/Hyrax.cu:237-305), whose blinding row is committed beside the folds of the opened tensor. */
int grape_commit_fr_nowait(uint32_t *d_out_affine, const uint32_t *d_scalars_mont, size_t size, uint32_t rowlen,
                           const uint32_t *d_wide_table, size_t N, uint32_t c, uint32_t nw, uint32_t K, int32_t *d_flag,
                           grape_stream_t stream);
/*
 * Strided fixed-base table: table[(q*K + (k-1))*N + i] = k * 2^(c*J*q) * G_i, k = 1..K = 2^(c-1), q < nsets
 * (the same entry format as the wide table; size grape_g1_wide_table_bytes(N, nsets, K)), and the
 * commitment of full-width scalars through it: window w = q*J + j of a scalar is looked up in set q,
 * the J residues j are summed apart and combined per row as sum_j 2^(c*j) * A_j by (J-1)*c doublings.
 * For the same bytes as a per-window table this affords wider windows: 16 additions per scalar
 * (c = 16, J = 4, 68 GB for 4096 generators) against 19 (c = 14, 82 GB), and it reaches generator sets
 * no per-window table fits (262144 generators: c = 12, J = 22, one set, 68 GB, 22 additions against
 * the 32 of the reference's byte windows).  Requires nsets * J >= ceil(255 / c), 2 <= c <= 18.
 * Same results as grape_commit_fr.  Hyrax::commit(FrTensor&, size, N), src/Hyrax.cu:335-359.
 */
int grape_g1_strided_table_gen(uint32_t *d_table, const uint32_t *d_gens_affine, size_t N, uint32_t c, uint32_t J, uint32_t nsets,
                               grape_stream_t stream);
int grape_commit_fr_strided(uint32_t *d_out_affine, const uint32_t *d_scalars_mont, size_t size, uint32_t rowlen,
                            const uint32_t *d_table, size_t N, uint32_t c, uint32_t J, uint32_t nsets, grape_stream_t stream);
/* Commitments through the reference-format table (k*G_i, k < 256, byte windows of |s| resp. of
 * the canonical scalar) — the reference's own algorithm, kept for tables loaded from its
 * points.bin.  Output affine. */
int grape_commit_i32_ref_table(uint32_t *d_out_affine, const int32_t *d_scalars, size_t size, uint32_t rowlen,
                               const uint32_t *d_table_affine, size_t npoints, grape_stream_t stream);
int grape_commit_fr_ref_table(uint32_t *d_out_affine, const uint32_t *d_scalars_mont, size_t size, uint32_t rowlen,
                              const uint32_t *d_table_affine, size_t npoints, grape_stream_t stream);
/* Format conversions for callers that keep the reference's jacob_t arrays. */
/* Row commitments of the elements of a full-width tensor whose flag is zero (d_skip[i] != 0 leaves
 * element i out): C_row = sum_{i : d_skip[row*rowlen+i] == 0} s[row*rowlen+i] * G_i, through a
 * per-window full-width table (grape_g1_wide_table_gen with nw*c >= 255).  Made for tensors of
 * which a small share is live (the elements of a logUp tensor that the occupied-entry table of
 * grape_tlookup_hot_select does not cover): live columns are queued per row and worked on in dense
 * batches.  No counterpart in the reference (it commits the whole tensor, src/tlookup.cu:320). */
int grape_commit_fr_sparse(uint32_t *d_out_affine, const uint32_t *d_scalars_mont, const int32_t *d_skip, size_t size,
                           uint32_t rowlen, const uint32_t *d_wide_table, size_t N, uint32_t c, uint32_t nw, uint32_t K,
                           grape_stream_t stream);
/* out[i] = a[i] + b[i] for n affine points (infinity, equal and opposite operands included); the
 * group law of include/curve/xyzz_t.cuh.  Combines two partial row commitments. */
int grape_g1_affine_add(uint32_t *d_out_affine, const uint32_t *d_a_affine, const uint32_t *d_b_affine, size_t n,
                        grape_stream_t stream);
int grape_g1_affine_to_jacobian(uint32_t *d_out_jac, const uint32_t *d_in_affine, size_t n, grape_stream_t stream);
int grape_g1_jacobian_to_affine(uint32_t *d_out_affine, const uint32_t *d_in_jac, size_t n, grape_stream_t stream);

/* ------------------------------------------------------------------ witness generation ------- */
/* The fixed-point rules of the reference's witness generator (zzllama/llama/model.py) on int32
 * device tensors.  Conditions the reference asserts or assumes (table index in range, quotient
 * fits int32, row sum positive, sum of squares below 2^64) do not fail the call: they set bits of a
 * sticky per-device status word, see grape_wit_status.
 *
 * Y[l][n][m] = sum_k a[l][n][k] * b[l][m][k] exactly (64-bit), then q = floor((Y + scale/2) / scale)
 * and r = Y - q*scale (1 <= scale <= 2^31); d_r may be NULL; transpose_out writes [l][m][n].  The matrix products and
 * rescalings of model.py:485-491, :547-550, :574-583, :646-658, :683-686. */
int grape_wit_matmul_rescale(int32_t *d_q, int32_t *d_r, const int32_t *d_a, const int32_t *d_b, uint32_t L, uint32_t N,
                             uint32_t M, uint32_t K, int64_t scale, int transpose_out, grape_stream_t stream);
/* Two implementations give the same (exact) result: 64-bit multiply-add kernels for any shape, and,
 * for one batch of 16-byte aligned operands with K a multiple of 4 and magnitudes below 2^22, int8
 * matrix-core products of signed byte planes (this path reads the operands' ranges back and so
 * synchronises the stream).  method 0 = choose (matrix cores from 2^26 multiply-adds), 1 = multiply-add
 * kernels only, 2 = matrix cores or GRAPE_EINVAL.  With grape_profile_enable, grape_profile_last()
 * gives [0] the product kernel, or, on the matrix cores, [0] the plane split of both operands (which also
 * finds their ranges), [1] the host's read of the ranges and [2] the product kernel. */
int grape_wit_set_matmul_method(int method);
/* q, r of a[i] * b[i] (d_r may be NULL).  model.py:673-675. */
int grape_wit_elemul_rescale(int32_t *d_q, int32_t *d_r, const int32_t *d_a, const int32_t *d_b, size_t n, int64_t scale,
                             grape_stream_t stream);
/* out[i] = table[in[i] - low] for in[i] in [low, low + len).  my_silu, model.py:118-149 (low = -2^18, len = 2^19). */
int grape_wit_table_lookup(int32_t *d_out, const int32_t *d_in, size_t n, int32_t low, uint32_t len, const int32_t *d_table,
                           grape_stream_t stream);
/* out[i] = a[i] + b[i] (the two skip connections, model.py:764-771). */
int grape_wit_add_i32(int32_t *d_out, const int32_t *d_a, const int32_t *d_b, size_t n, grape_stream_t stream);
/* Row-wise table softmax, my_softmax, model.py:76-116: max[rows], shifted = x - max, exp =
 * table[shifted + 2^bit_shift - 1] (table of 2^index_bits entries), sum[rows] (low 32 bits, as the
 * reference stores it), prob = floor((exp*scale + floor(sum/2)) / sum), query = 2*scale*exp -
 * sum*(2*prob - 1); all outputs rows x cols int32 except max and sum. */
int grape_wit_softmax(int32_t *d_max, int32_t *d_shifted, int32_t *d_exp, int32_t *d_sum, int32_t *d_prob, int32_t *d_query,
                      const int32_t *d_scores, uint32_t rows, uint32_t cols, const int32_t *d_table, uint32_t bit_shift,
                      uint32_t index_bits, int64_t scale, grape_stream_t stream);
/* out[row] = sum of x[row][c]^2 as an exact 64-bit integer: the integer part of RMSNorm's mean
 * square (model.py:193); the float16 reciprocal root is taken on the host from this sum. */
int grape_wit_row_sumsq(uint64_t *d_out, const int32_t *d_x, uint32_t rows, uint32_t cols, grape_stream_t stream);
/* RMSNorm.forward, model.py:228-234, given rms_int per row: (q,r)_rmsw = rescale(rms[row] * w[col]),
 * (q,r)_out = rescale(q_rmsw * x). */
int grape_wit_rmsnorm_apply(int32_t *d_q_rmsw, int32_t *d_r_rmsw, int32_t *d_q_out, int32_t *d_r_out, const int32_t *d_x,
                            const int32_t *d_rms, const int32_t *d_w, uint32_t rows, uint32_t cols, int64_t scale,
                            grape_stream_t stream);
/* Synchronises, returns the status bits set since the last call and clears them: 1 = a quotient left
 * int32, 2 = a table index out of range (the reference's assertions, model.py:86-87, :137-138),
 * 4 = a softmax row summed to zero or met a negative table entry, 8 = a sum of squares left 64 bits. */
#define GRAPE_WIT_QUOTIENT 1u
#define GRAPE_WIT_INDEX 2u
#define GRAPE_WIT_SUM 4u
#define GRAPE_WIT_SQUARES 8u
int grape_wit_status(uint32_t *flags, grape_stream_t stream);

/* ------------------------------------------------------------------ measurement -------------- */
/* Device-to-device copy of `bytes` with the library's own streaming kernel, `iters` times;
 * returns the average time per copy in milliseconds in *ms (HIP events on `stream`). */
int grape_bench_copy(void *d_dst, const void *d_src, size_t bytes, int iters, float *ms, grape_stream_t stream);
/* The same for an Fr tensor of n elements moved with the tensors' own access pattern (one 32-byte
 * element per lane as two 16-byte accesses). */
int grape_bench_copy_fr(uint32_t *d_out, const uint32_t *d_in, size_t n, int iters, float *ms, grape_stream_t stream);
/* Dependency-free v_mad_u64_u32 throughput: every lane of `blocks` x 256 threads runs
 * `inner` x 64 multiply-adds; *mads_per_s receives lane-level 32x32 multiplies per second. */
int grape_bench_mad_u64_u32(int blocks, int inner, int iters, double *mads_per_s, grape_stream_t stream);
/* Kernel-level timing: when enabled, the commitment entry points bracket each kernel they launch
 * with HIP events on the caller's stream.  grape_profile_last() synchronises and returns the
 * durations (ms) of the kernels of the most recent call, in launch order (for grape_commit_*:
 * [0] accumulation kernel, [1] row-reduction kernel; for grape_fr_fold: [0] weight kernel, then
 * one entry per pass); *n receives how many were written. */
int grape_profile_enable(int on);
int grape_profile_last(float *ms, int cap, int *n);
/* A second stream for work that is independent of the caller's (the host classes run the table side
 * of a lookup's rounds on one, beside the witness side): default priority, no implicit
 * synchronisation with the default stream; order across streams with grape_event_record +
 * grape_stream_wait_event.  Scratch memory is per stream, so calls on different streams never share
 * any; grape_stream_destroy waits for the stream and frees its scratch. */
int grape_stream_create(grape_stream_t *out);
int grape_stream_destroy(grape_stream_t stream);
int grape_stream_wait_event(grape_stream_t stream, void *ev);
/* Event helpers on a stream (HIP events): ordering between streams, and timing for benchmarks that
 * live above this ABI. */
int grape_event_create(void **ev);
int grape_event_destroy(void *ev);
int grape_event_record(void *ev, grape_stream_t stream);
int grape_event_elapsed_ms(float *ms, void *ev_start, void *ev_stop); /* syncs on ev_stop */

#ifdef __cplusplus
}
#endif
#endif
