// Sumcheck rounds whose terms carry an eq(u, x) weight: the element-product sumcheck (src/prove.cu:
// 119-172), phase 1 of the matmul sumcheck (:49-85), the claim-merging sumcheck (:245-300) and the
// logUp rounds of tLookup (src/tlookup.cu:117-244).  The reference materialises coefficient arrays
// and folds each of them over the remaining variables of u in every round; here a round is ONE
// pass over the operands: the weights come from a pyramid of eq tables built once per proof (no
// per-round halving), the operands are folded in place by the same pass, and the weighted sums
// leave the kernel as per-workgroup partial sums that a one-block kernel finishes.  Challenges are
// known before the first round, so the host queues all rounds and reads the sums once.
#include "fr_device.hpp"

namespace grape {

// ---------------------------------------------------------------- eq pyramid
// Level j (2^j entries) sits at element offset 2^j - 1; level j holds eq(u[0..j-1], i), bit b of i
// paired with u[b].  Level j+1 from level j: hi = lo * u[j], lo' = lo - hi.
constexpr uint32_t kPyrHeadLevels = 9;   // levels 0..9 built by one workgroup (512 threads' worth at the top)

__global__ void __launch_bounds__(kBlock) eq_pyramid_head_kernel(uint32_t* pyr, const uint32_t* u, uint32_t levels) {
    if (threadIdx.x == 0) st_fr(pyr, 0, Fr::one());
    __syncthreads();
    for (uint32_t j = 0; j < levels; j++) {
        const size_t half = (size_t)1 << j, src = half - 1, dst = 2 * half - 1;
        const Fr uj = ld_fr(u, j);
        for (size_t i = threadIdx.x; i < half; i += kBlock) {
            const Fr lo = ld_fr(pyr, src + i);
            const Fr hi = fr26::mulc(lo, uj);
            st_fr(pyr, dst + i + half, hi);
            st_fr(pyr, dst + i, sub(lo, hi));
        }
        __threadfence_block();
        __syncthreads();
    }
}
__global__ void __launch_bounds__(kBlock) eq_pyramid_level_kernel(uint32_t* pyr, const uint32_t* u, uint32_t j) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t half = (size_t)1 << j;
    if (i >= half) return;
    const Fr lo = ld_fr(pyr, half - 1 + i);
    const Fr hi = fr26::mulc(lo, ld_fr(u, j));
    st_fr(pyr, 2 * half - 1 + i + half, hi);
    st_fr(pyr, 2 * half - 1 + i, sub(lo, hi));
}

// ---------------------------------------------------------------- weighted two-tensor round
// One thread runs at most kWIters indices; the three weighted sums are double-width column
// accumulators reduced once per thread.  Per index (e = weight, x0/x1 = halves of the MSB split,
// d = x1 - x0, S' = S + beta):
//   ea0 = e*a0 in (0, 1.46 r), ead = e*da in (0.54 r, 2.46 r)        (limbs normalised, below 2^26)
//   W0 += ea0 * s0'        < 2.92 r^2         s0' < 2r, limbs < 2^27
//   W2 += ead * ds         < 2.46 r^2         |ds| < r, |limb| < 2^26
//   WQ += (ea0+ead) * s1'  < 7.84 r^2         s1' < 2r, limbs < 2^27 -> a column grows by < 2^57.4
// so 24 indices keep a column below 2^62 and the sums within +-5.4 r of their offsets.  The sums
// leave the thread WITHOUT the radix factor 16 (value / 2^260, canonical); the finishing kernel
// applies it once.  The middle coefficient is WQ - W0 - W2 (one product instead of two).
constexpr int kWIters = 24;

// a finished column sum -> canonical element of value V / 2^260 + (a multiple of r)
__device__ __forceinline__ Fr reduce_to_fr(fr26::Acc& C, int lo_r) {
    return fr26::unpack(fr26::canon_wide(fr26::reduce(C, lo_r)));
}

// sums[0..2] = 16 * (W0, WQ - W0 - W2, W2); with PLAIN sums[3] = sum A0, sums[4] = sum A1 - sum A0
// UNIT (weights that sum to one, A * (S + beta) = 1 everywhere): sums[0] = 1, sums[1] = -sums[2]
// NOMID (the caller takes the middle coefficient from its running claim): sums[1] = 0
template <bool PLAIN, bool UNIT, bool NOMID>
__device__ __forceinline__ void wround2_result(uint32_t* out, const Fr* acc) {
    Fr w[3] = {acc[0], NOMID ? Fr::zero() : sub(sub(acc[1], acc[0]), acc[2]), acc[2]};
#pragma unroll
    for (int k = 0; k < 3; k++) {
        Fr t = w[k];
#pragma unroll
        for (int d = 0; d < 4; d++) t = add(t, t);
        w[k] = t;
    }
    if (UNIT) {
        w[0] = Fr::one();
        w[1] = sub(Fr::zero(), w[2]);
    }
#pragma unroll
    for (int k = 0; k < 3; k++) st_fr(out, k, w[k]);
    if (PLAIN) {
        st_fr(out, 3, acc[3]);
        st_fr(out, 4, sub(acc[4], acc[3]));
    }
}

// UNIT: the caller states that A[i] * (S[i] + beta) = 1 at every index (the first round of a logUp
// proof, where A was made as the inverse of S + beta).  Then the constant coefficient is the sum of
// the weights and the value at t = 1 equals it, so only the top coefficient sum_g e * dA * dS is
// taken: one weight product and one accumulation per index instead of two and three.
// TAB: the folds go through the table of the challenge's multiples (fr26::fold_table; long rounds).
// NOMID: the sum of the round polynomial over {0, 1} is known to the caller (the value the previous
// round's polynomial took at its challenge), which fixes the middle coefficient: the value at t = 1
// is not accumulated - one product and one double-width accumulator less per index.
// IDX: A is not read but gathered, A[i] = Bt[idx1[i] - 1] (in_size == 2 n_out): the first round of a lookup whose
// logUp tensor was never written out - the pass over the witness left the table indices only.
template <bool BETA, bool PLAIN, bool UNIT, bool TAB, bool NOMID = false, bool IDX = false>
__global__ void __launch_bounds__(kBlock, 2) wround2_kernel(uint32_t* A, uint32_t* S, const uint32_t* beta, const uint32_t* E,
                                                         uint32_t in_size, uint32_t n_out, uint32_t rowlen, uint32_t rowpad,
                                                         const uint32_t* v, const int32_t* __restrict__ tab, uint32_t* partial,
                                                         const int32_t* __restrict__ idx1 = nullptr, const uint32_t* Bt = nullptr) {
    constexpr int NV = PLAIN ? 5 : 3;
    __shared__ Fr lds[NV * (kBlock / 64)];
    fr26::Limbs w1;
    if (!TAB) w1 = fr26::weight16(ld_fr(v, 0));
    fr26::Limbs bt;
    if (BETA) bt = fr26::pack(ld_fr(beta, 0));
    fr26::Acc W0, WQ, W2;
    fr26::acc_zero(W0);
    fr26::acc_zero(WQ);
    fr26::acc_zero(W2);
    fr26::Limbs sa0, sa1;                       // plain limb-wise sums of A's halves (24 terms below 2^26)
#pragma unroll
    for (int k = 0; k < fr26::N; k++) sa0.v[k] = sa1.v[k] = 0;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x; g < n_out; g += stride) {
        // weights live on rows of `rowpad` entries when the tensors' rows hold `rowlen` < rowpad
        const size_t ei = rowlen == rowpad ? g : g + (size_t)((uint32_t)g / rowlen) * (rowpad - rowlen);
        const fr26::Limbs e16 = fr26::pack16(ld_fr(E, ei));
        fr26::Limbs a0, a1;
        if (IDX) {
            const uint32_t j0 = (uint32_t)idx1[g], j1 = (uint32_t)idx1[g + n_out];     // 0 marks an element outside the table
            a0 = ld_l26(Bt, j0 ? j0 - 1 : 0);
            a1 = ld_l26(Bt, j1 ? j1 - 1 : 0);
        } else {
            a0 = ld_l26(A, g);
            a1 = ld_hi26(A, g, n_out, in_size);
        }
        const fr26::Limbs da = fr26::sub(a1, a0);
        fr26::Acc T;
        fr26::Limbs ea0;
        if (!UNIT) {
            fr26::acc_zero(T);
            fr26::mac(T, e16, a0);
            ea0 = fr26::reduce(T, 0);
        }
        fr26::acc_zero(T);
        fr26::mac(T, e16, da);
        const fr26::Limbs ead = fr26::reduce(T, 1);
        if (PLAIN) {
            sa0 = fr26::add(sa0, a0);
            sa1 = fr26::add(sa1, a1);
        }
        st_fr(A, g, TAB ? foldt1(tab, a0, da) : fold1(w1, a0, da));
        const fr26::Limbs s0r = ld_l26(S, g);
        const fr26::Limbs s1r = ld_hi26(S, g, n_out, in_size);
        const fr26::Limbs ds = fr26::sub(s1r, s0r);
        st_fr(S, g, TAB ? foldt1(tab, s0r, ds) : fold1(w1, s0r, ds));
        fr26::mac(W2, ead, ds);
        if (UNIT) {
            // W0 and WQ stay zero: the finishing kernel writes the coefficients they would give
        } else if (BETA) {
            fr26::mac(W0, ea0, fr26::add(s0r, bt));
            if (!NOMID) fr26::mac(WQ, fr26::add(ea0, ead), fr26::add(s1r, bt));
        } else {
            fr26::mac(W0, ea0, s0r);
            if (!NOMID) fr26::mac(WQ, fr26::add(ea0, ead), s1r);
        }
    }
    // offsets: |W0| < 71 r^2 -> within 2 r, |W2| < 60 r^2 -> within 1.7 r, |WQ| < 189 r^2 -> within 5.4 r
    Fr acc[NV];
    acc[0] = reduce_to_fr(W0, 3);
    acc[1] = NOMID ? Fr::zero() : reduce_to_fr(WQ, 6);
    acc[2] = reduce_to_fr(W2, 3);
    if (PLAIN) {
        acc[3] = fr26::limb_sum_to_fr(sa0, 0);      // below 24 r
        acc[4] = fr26::limb_sum_to_fr(sa1, 0);
    }
    block_sum<NV>(acc, lds);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < NV; k++) st_fr(partial, (size_t)blockIdx.x * NV + k, acc[k]);
    }
}
template <bool PLAIN, bool UNIT, bool NOMID, int BLOCK>
__global__ void __launch_bounds__(BLOCK) wround2_final_kernel(uint32_t* out, const uint32_t* partial, unsigned nblocks) {
    constexpr int NV = PLAIN ? 5 : 3;
    __shared__ uint32_t lds9[NV * (BLOCK / 64) * 9];
    Fr tot[NV];
    workgroup_totals<NV, BLOCK, NOMID ? 2u : 0u>(tot, partial, nblocks, lds9);
    if (threadIdx.x == 0) wround2_result<PLAIN, UNIT, NOMID>(out, tot);
}

// ---------------------------------------------------------------- matmul phase 1: weights per segment
// Indices g = seg * seglen + k; every index of a segment shares the weight e[seg], so the three
// sums are taken per (segment, chunk) without weights and the finishing kernel applies e[seg].
__global__ void __launch_bounds__(kBlock) sumcheck2_seg_kernel(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t out_size,
                                                               uint32_t seglen, uint32_t seg0, const uint32_t* v, uint32_t* partial) {
    __shared__ Fr lds[3 * (kBlock / 64)];
    const fr26::Limbs w1 = fr26::weight16(ld_fr(v, 0));
    fr26::Acc C0, Q, C2;
    fr26::acc_zero(C0);
    fr26::acc_zero(Q);
    fr26::acc_zero(C2);
    const uint32_t seg = seg0 + blockIdx.y;            // a launch covers at most 65535 segments (the grid's y extent)
    const uint32_t stride = gridDim.x * kBlock;      // the host keeps seglen / stride <= 64
    for (uint32_t k = blockIdx.x * kBlock + threadIdx.x; k < seglen; k += stride) {
        const size_t g = (size_t)seg * seglen + k;
        if (g >= out_size) break;
        const fr26::Limbs a0 = ld_l26(A, g), b0 = ld_l26(B, g);
        const fr26::Limbs a1 = ld_hi26(A, g, out_size, in_size), b1 = ld_hi26(B, g, out_size, in_size);
        const fr26::Limbs da = fr26::sub(a1, a0), db = fr26::sub(b1, b0);
        st_fr(A, g, fold1(w1, a0, da));
        st_fr(B, g, fold1(w1, b0, db));
        fr26::mac(C0, a0, b0);
        fr26::mac(Q, a1, b1);
        fr26::mac(C2, da, db);
    }
    const Fr c0 = fr26::finish_sum(C0, 2), c2 = fr26::finish_sum(C2, 2), q1 = fr26::finish_sum(Q, 2);
    Fr acc[3] = {c0, sub(sub(q1, c0), c2), c2};
    block_sum<3>(acc, lds);
    if (threadIdx.x == 0) {
        const size_t slot = (size_t)seg * gridDim.x + blockIdx.x;
#pragma unroll
        for (int t = 0; t < 3; t++) st_fr(partial, slot * 3 + t, acc[t]);
    }
}
// sums[t] = sum_seg e[seg] * sum_chunk partial[seg][chunk][t]
__global__ void __launch_bounds__(kBlock) seg_final_kernel(uint32_t* out, const uint32_t* partial, const uint32_t* e, uint32_t nseg,
                                                           uint32_t nchunk) {
    __shared__ Fr lds[3 * (kBlock / 64)];
    Fr acc[3] = {Fr::zero(), Fr::zero(), Fr::zero()};
    for (uint32_t s = threadIdx.x; s < nseg; s += kBlock) {
        Fr t[3] = {Fr::zero(), Fr::zero(), Fr::zero()};
        for (uint32_t c = 0; c < nchunk; c++) {
#pragma unroll
            for (int k = 0; k < 3; k++) t[k] = add(t[k], ld_fr(partial, ((size_t)s * nchunk + c) * 3 + k));
        }
        const Fr w = ld_fr(e, s);
#pragma unroll
        for (int k = 0; k < 3; k++) acc[k] = add(acc[k], fr26::mulc(w, t[k]));
    }
    block_sum<3>(acc, lds);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 3; k++) st_fr(out, k, acc[k]);
    }
}

// ---------------------------------------------------------------- claim merging: one tensor, several weight tables
// For claim j (blockIdx.y) with weights e_j: sums[2j] = sum_x e_j[x] X0[x], sums[2j+1] = sum_x e_j[x] (X1[x] - X0[x]).
// Nothing is modified (the fold is a separate launch: every claim reads the unfolded tensor).
struct PyrPack { const uint32_t* p[16]; };
__global__ void __launch_bounds__(kBlock) wsum1_kernel(const uint32_t* X, PyrPack E, uint32_t in_size, uint32_t n_out, uint32_t* partial) {
    __shared__ Fr lds[2 * (kBlock / 64)];
    const uint32_t* e = E.p[blockIdx.y];
    fr26::Acc C0, C1;
    fr26::acc_zero(C0);
    fr26::acc_zero(C1);
    const size_t stride = (size_t)gridDim.x * kBlock;
    // 64 indices per thread at most: e, x0 below 2^26 per limb -> a column grows by < 2^55.4 per index
    for (size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x; g < n_out; g += stride) {
        const fr26::Limbs w = ld_l26(e, g);
        const fr26::Limbs x0 = ld_l26(X, g);
        const fr26::Limbs x1 = ld_hi26(X, g, n_out, in_size);
        fr26::mac(C0, w, x0);
        fr26::mac(C1, w, fr26::sub(x1, x0));
    }
    // |sum| < 64 r^2 -> within 1.82 r of the offset; the factor 16 is applied by the finishing kernel
    Fr acc[2] = {reduce_to_fr(C0, 2), reduce_to_fr(C1, 2)};
    block_sum<2>(acc, lds);
    if (threadIdx.x == 0) {
        const size_t slot = (size_t)blockIdx.y * gridDim.x + blockIdx.x;
        st_fr(partial, slot * 2, acc[0]);
        st_fr(partial, slot * 2 + 1, acc[1]);
    }
}
__global__ void __launch_bounds__(kBlock) wsum1_final_kernel(uint32_t* out, const uint32_t* partial, uint32_t nblocks) {
    __shared__ Fr lds[2 * (kBlock / 64)];
    const uint32_t j = blockIdx.x;
    Fr acc[2] = {Fr::zero(), Fr::zero()};
    for (uint32_t b = threadIdx.x; b < nblocks; b += kBlock) {
        acc[0] = add(acc[0], ld_fr(partial, ((size_t)j * nblocks + b) * 2));
        acc[1] = add(acc[1], ld_fr(partial, ((size_t)j * nblocks + b) * 2 + 1));
    }
    block_sum<2>(acc, lds);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
            Fr t = acc[k];
#pragma unroll
            for (int d = 0; d < 4; d++) t = add(t, t);
            st_fr(out, 2 * (size_t)j + k, t);
        }
    }
}

}  // namespace grape

using namespace grape;

extern "C" {

size_t grape_eq_pyramid_elems(uint32_t nu) { return ((size_t)2 << nu) - 1; }

int grape_eq_pyramid(uint32_t* pyr, const uint32_t* u, uint32_t nu, grape_stream_t st) {
    CHECK_PTR16(pyr);
    GRAPE_REQUIRE(nu <= 30, "too many variables");
    if (nu) CHECK_PTR16(u);
    hipStream_t s = as_stream(st);
    const uint32_t head = nu < kPyrHeadLevels ? nu : kPyrHeadLevels;
    eq_pyramid_head_kernel<<<1, kBlock, 0, s>>>(pyr, u, head);
    for (uint32_t j = head; j < nu; j++) eq_pyramid_level_kernel<<<blocks_for((size_t)1 << j), kBlock, 0, s>>>(pyr, u, j);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

// workgroups of a weighted round over n_out index pairs
static unsigned wround2_blocks(uint32_t n_out) {
    unsigned nb = blocks_for(n_out);
    if (nb > (unsigned)kNumCU * 4) {
        const unsigned need = blocks_for(n_out, kBlock * kWIters);
        nb = need > (unsigned)kNumCU * 4 ? need : (unsigned)kNumCU * 4;
    }
    return nb;
}

// The two launches of a weighted round: the pass over the operands (partial sums per workgroup; `tab`: the table of
// the challenge's multiples, or nullptr for the single-product fold) and the kernel that finishes the sums.
static int wround2_main(uint32_t* A, uint32_t* S, const uint32_t* beta, const uint32_t* E, uint32_t in_size, uint32_t n_out,
                        uint32_t rowlen, uint32_t rowpad, const uint32_t* v, int plain_sums, const int32_t* tab, uint32_t* partial,
                        hipStream_t s) {
    const unsigned nb = wround2_blocks(n_out);
    const bool use_tab = tab != nullptr;
// five sums and three accumulators leave no registers for the table fold's columns (it spills: 1.16 against
    // 1.10 ms at 2^24 index pairs), so that form keeps the single-product fold at every size
#define GRAPE_WROUND2(B, P, U)                                                                                        \
    do {                                                                                                              \
        if (use_tab && !((P) && !(U)))                                                                                \
            wround2_kernel<B, P, U, !((P) && !(U))><<<nb, kBlock, 0, s>>>(A, S, beta, E, in_size, n_out, rowlen, rowpad, v, tab, partial); \
        else wround2_kernel<B, P, U, false><<<nb, kBlock, 0, s>>>(A, S, beta, E, in_size, n_out, rowlen, rowpad, v, nullptr, partial);    \
    } while (0)
    if (plain_sums == 3) {
        // the middle coefficient is left to the caller (sums[1] = 0); long rounds of a logUp proof
        GRAPE_REQUIRE(beta != nullptr && use_tab, "the round without its middle coefficient is built for logUp rounds of 2^16 index pairs and more");
        wround2_kernel<true, true, false, true, true><<<nb, kBlock, 0, s>>>(A, S, beta, E, in_size, n_out, rowlen, rowpad, v, tab, partial);
    } else if (plain_sums == 2) {
        GRAPE_REQUIRE(rowlen == rowpad && in_size == 2 * (uint64_t)n_out,
                      "the inverse-pair round needs whole pairs and unpadded rows (weights that sum to one)");
        if (beta) GRAPE_WROUND2(true, true, true);
        else GRAPE_WROUND2(false, true, true);
    } else if (beta && plain_sums) {
        GRAPE_WROUND2(true, true, false);
    } else if (beta) {
        GRAPE_WROUND2(true, false, false);
    } else if (plain_sums) {
        GRAPE_WROUND2(false, true, false);
    } else {
        GRAPE_WROUND2(false, false, false);
    }
#undef GRAPE_WROUND2
    return GRAPE_OK;
}
static void wround2_final(uint32_t* sums, const uint32_t* partial, uint32_t n_out, int plain_sums, hipStream_t s) {
    const unsigned nb = wround2_blocks(n_out);
#define GRAPE_WFINAL(P, U, M)                                                                                    \
    do {                                                                                                         \
        if (nb >= kFinalWideMin) wround2_final_kernel<P, U, M, kFinalBlock><<<1, kFinalBlock, 0, s>>>(sums, partial, nb); \
        else wround2_final_kernel<P, U, M, kBlock><<<1, kBlock, 0, s>>>(sums, partial, nb);                      \
    } while (0)
    if (plain_sums == 3) GRAPE_WFINAL(true, false, true);
    else if (plain_sums == 2) GRAPE_WFINAL(true, true, false);
    else if (plain_sums) GRAPE_WFINAL(true, false, false);
    else GRAPE_WFINAL(false, false, false);
#undef GRAPE_WFINAL
}
#define GRAPE_WROUND2_CHECKS()                                                                                              \
    CHECK_PTR16(A); CHECK_PTR16(S); CHECK_PTR16(E); CHECK_PTR16(v);                                                        \
    GRAPE_REQUIRE(n_out >= 1 && in_size >= n_out && in_size <= 2 * (uint64_t)n_out, "need n_out <= in_size <= 2*n_out"); \
    GRAPE_REQUIRE(rowlen >= 1 && rowlen <= rowpad, "need 1 <= rowlen <= rowpad");                                        \
    if (beta) CHECK_PTR16(beta)

int grape_wround2(uint32_t* A, uint32_t* S, const uint32_t* beta, const uint32_t* E, uint32_t in_size, uint32_t n_out,
                  uint32_t rowlen, uint32_t rowpad, const uint32_t* v, int plain_sums, uint32_t* sums, grape_stream_t st) {
    GRAPE_WROUND2_CHECKS();
    CHECK_PTR16(sums);
    hipStream_t s = as_stream(st);
    void* ws;
    const size_t partial_bytes = (size_t)wround2_blocks(n_out) * (plain_sums ? 5 : 3) * 32;
    int rc = scratch_get(kSlotReduce, partial_bytes + kFoldTableBytes, &ws, s);
    if (rc) return rc;
    uint32_t* partial = (uint32_t*)ws;
    // long rounds fold through the table of the challenge's multiples (one more small launch)
    int32_t* tab = nullptr;
    if (n_out >= kTableFoldMinOut) {
        tab = (int32_t*)((char*)ws + partial_bytes);
        fold_tables_kernel<<<1, 64, 0, s>>>(tab, v, 1);
    }
    rc = wround2_main(A, S, beta, E, in_size, n_out, rowlen, rowpad, v, plain_sums, tab, partial, s);
    if (rc) return rc;
    wround2_final(sums, partial, n_out, plain_sums, s);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

size_t grape_wround2_partial_bytes(uint32_t n_out) { return (size_t)wround2_blocks(n_out ? n_out : 1) * 5 * 32; }

static_assert(GRAPE_FOLD_TABLE_WORDS == fr26::kFoldTableWords, "the header's table size is the kernels'");
int grape_fold_tables(int32_t* tabs, const uint32_t* v, uint32_t count, grape_stream_t st) {
    GRAPE_REQUIRE(tabs != nullptr && (reinterpret_cast<uintptr_t>(tabs) & 3) == 0, "tabs must be 4-byte aligned");
    GRAPE_REQUIRE(count >= 1 && count <= 64, "1..64 challenges");
    CHECK_PTR16(v);
    fold_tables_kernel<<<1, 64, 0, as_stream(st)>>>(tabs, v, count);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wround2_queue(uint32_t* A, uint32_t* S, const uint32_t* beta, const uint32_t* E, uint32_t in_size, uint32_t n_out,
                        uint32_t rowlen, uint32_t rowpad, const uint32_t* v, int plain_sums, const int32_t* tab, uint32_t* partial,
                        grape_stream_t st) {
    GRAPE_WROUND2_CHECKS();
    CHECK_PTR16(partial);
    GRAPE_REQUIRE(tab == nullptr || n_out >= kTableFoldMinOut, "the table fold is built for rounds of 2^16 index pairs and more");
    int rc = wround2_main(A, S, beta, E, in_size, n_out, rowlen, rowpad, v, plain_sums, tab, partial, as_stream(st));
    if (rc) return rc;
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wround2_queue_indexed(uint32_t* A, uint32_t* S, const int32_t* idx1, const uint32_t* Bt, uint32_t len, const uint32_t* beta,
                                const uint32_t* E, uint32_t n_out, const uint32_t* v, const int32_t* tab, uint32_t* partial,
                                grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(S); CHECK_PTR16(E); CHECK_PTR16(v); CHECK_PTR16(Bt); CHECK_PTR16(beta); CHECK_PTR16(partial);
    GRAPE_REQUIRE(idx1 != nullptr && len >= 1, "bad arguments");
    GRAPE_REQUIRE(tab != nullptr && n_out >= kTableFoldMinOut && n_out <= (1u << 30), "built for first rounds of 2^16 index pairs and more");
    wround2_kernel<true, true, true, true, false, true><<<wround2_blocks(n_out), kBlock, 0, as_stream(st)>>>(
        A, S, beta, E, 2 * n_out, n_out, 1, 1, v, tab, partial, idx1, Bt);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wround2_finish(uint32_t* sums, const uint32_t* partial, uint32_t n_out, int plain_sums, grape_stream_t st) {
    CHECK_PTR16(sums); CHECK_PTR16(partial);
    GRAPE_REQUIRE(n_out >= 1, "need n_out >= 1");
    wround2_final(sums, partial, n_out, plain_sums, as_stream(st));
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
#undef GRAPE_WROUND2_CHECKS

int grape_sumcheck_round2_seg(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t out_size, uint32_t seglen, const uint32_t* e,
                              const uint32_t* v, uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(B); CHECK_PTR16(e); CHECK_PTR16(v); CHECK_PTR16(sums);
    GRAPE_REQUIRE(out_size >= 1 && in_size >= out_size && in_size <= 2 * (uint64_t)out_size, "need out_size <= in_size <= 2*out_size");
    GRAPE_REQUIRE(seglen >= 1 && out_size % seglen == 0, "out_size must be a whole number of segments");
    const uint32_t nseg = out_size / seglen;
    hipStream_t s = as_stream(st);
    // chunks per segment: one index per thread until the grid is large, never more than 64 per thread
    uint32_t nchunk = blocks_for(seglen);
    const uint32_t cap = nseg >= 2048 ? 1 : 2048 / nseg;
    if (nchunk > cap) nchunk = cap;
    const uint32_t need = blocks_for(seglen, kBlock * 64);
    if (nchunk < need) nchunk = need;
    void* ws;
    int rc = scratch_get(kSlotReduce, (size_t)nseg * nchunk * 3 * 32, &ws, s);
    if (rc) return rc;
    for (uint32_t seg0 = 0; seg0 < nseg; seg0 += 65535) {
        const uint32_t ns = nseg - seg0 < 65535 ? nseg - seg0 : 65535;
        sumcheck2_seg_kernel<<<dim3(nchunk, ns), kBlock, 0, s>>>(A, B, in_size, out_size, seglen, seg0, v, (uint32_t*)ws);
    }
    seg_final_kernel<<<1, kBlock, 0, s>>>(sums, (const uint32_t*)ws, e, nseg, nchunk);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wsum1_multi(const uint32_t* X, const uint32_t* const* e_tables, uint32_t num, uint32_t in_size, uint32_t n_out,
                      uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(X); CHECK_PTR16(sums);
    GRAPE_REQUIRE(e_tables != nullptr && num >= 1 && num <= 16, "1..16 weight tables");
    GRAPE_REQUIRE(n_out >= 1 && in_size >= n_out && in_size <= 2 * (uint64_t)n_out, "need n_out <= in_size <= 2*n_out");
    PyrPack pk;
    for (uint32_t j = 0; j < 16; j++) pk.p[j] = j < num ? e_tables[j] : nullptr;
    for (uint32_t j = 0; j < num; j++) CHECK_PTR16(pk.p[j]);
    hipStream_t s = as_stream(st);
    unsigned nb = blocks_for(n_out);
    if (nb > (unsigned)kNumCU * 4) {
        const unsigned need = blocks_for(n_out, kBlock * 64);
        nb = need > (unsigned)kNumCU * 4 ? need : (unsigned)kNumCU * 4;
    }
    void* ws;
    int rc = scratch_get(kSlotReduce, (size_t)nb * num * 2 * 32, &ws, s);
    if (rc) return rc;
    wsum1_kernel<<<dim3(nb, num), kBlock, 0, s>>>(X, pk, in_size, n_out, (uint32_t*)ws);
    wsum1_final_kernel<<<num, kBlock, 0, s>>>(sums, (const uint32_t*)ws, nb);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

}  // extern "C"
