#include "prove.hpp"
#include <cassert>
#include <memory>
#include "../../include/grape_hip.h"

using grape_host::check;
static inline uint32_t* W(fr_t* p) { return reinterpret_cast<uint32_t*>(p); }

static void record(SumcheckTranscript* t, const Polynomial& p, const Fr& claim) {
    if (t) {
        t->rounds.push_back(p);
        t->claims.push_back(claim);
    }
}
static void read3(fr_t* d_sums, Fr out[3]) {
    check(grape_memcpy_d2h(out, d_sums, 3 * sizeof(fr_t), nullptr), "grape_memcpy_d2h");
}

namespace {
// device buffer released on scope exit
struct DeviceBuf {
    void* p = nullptr;
    explicit DeviceBuf(size_t bytes) { check(grape_malloc(&p, bytes ? bytes : 1), "grape_malloc"); }
    ~DeviceBuf() { grape_free(p); }
    DeviceBuf(const DeviceBuf&) = delete;
    DeviceBuf& operator=(const DeviceBuf&) = delete;
    fr_t* fr() const { return static_cast<fr_t*>(p); }
};
// eq tables of every prefix of `nvars` device challenges starting at d_u (level j at offset 2^j - 1)
struct EqPyramid {
    DeviceBuf buf;
    EqPyramid(const fr_t* d_u, uint nvars) : buf(sizeof(fr_t) * grape_eq_pyramid_elems(nvars)) {
        check(grape_eq_pyramid(W(buf.fr()), reinterpret_cast<const uint32_t*>(d_u), nvars, nullptr), "grape_eq_pyramid");
    }
    fr_t* level(uint j) const { return buf.fr() + (((size_t)1 << j) - 1); }
};
std::vector<Fr> download_vec(const fr_t* d, size_t n) {
    std::vector<Fr> out(n);
    if (n) check(grape_memcpy_d2h(out.data(), d, sizeof(fr_t) * n, nullptr), "grape_memcpy_d2h");
    return out;
}
}  // namespace

// Phase 1 of the matmul sumcheck (src/prove.cu:49-85) binds the batch variables l of
// sum_l eq(u_l, l) sum_k A[l][k] B[l][k].  The reference writes three coefficient arrays per round,
// folds each over the remaining l-bits of u and sums the K survivors; here every round is one
// launch that folds A and B and takes the three sums per batch row, weighted by that row's
// eq(u_low, l') from a table built once.  The rounds are queued back to back (the challenges
// are known up front) and their sums read with one copy.
Fr matmul_sumcheck_phase1(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* u, fr_t* v, uint K, uint size,
                          Fr& claim, SumcheckTranscript* transcript) {
    (void)a;
    (void)b;
    (void)c;
    const uint rounds = Log2(size / K);
    Fr eq_accumulate = Fr::one();
    if (rounds == 0) return eq_accumulate;
    if (size != (K << rounds)) throw std::runtime_error("matmul_phase1: the batch extent must be a power of two");
    const std::vector<Fr> us = download_vec(u - rounds, rounds), vs = download_vec(v - rounds, rounds);
    EqPyramid eq(u - rounds, rounds - 1);
    FrTensor sums(3 * rounds);
    uint in = size;
    for (uint i = 0; i < rounds; i++) {
        const uint out = in / 2;
        check(grape_sumcheck_round2_seg(W(A.gpu_data), W(B.gpu_data), in, out, K, W(eq.level(rounds - 1 - i)), W(v - i - 1),
                                        W(sums.gpu_data + 3 * i), nullptr),
              "grape_sumcheck_round2_seg");
        in = out;
    }
    const std::vector<Fr> s = download_vec(sums.gpu_data, 3 * (size_t)rounds);
    for (uint i = 0; i < rounds; i++) {
        const Fr &u_now = us[rounds - 1 - i], &v_now = vs[rounds - 1 - i];
        Polynomial p({s[3 * i], s[3 * i + 1], s[3 * i + 2]});
        p *= (Polynomial::eq(u_now) * eq_accumulate);
        if (p(0) + p(1) != claim) throw std::runtime_error("matmul_phase1: claim != p(0) + p(1)");
        claim = p(v_now);
        record(transcript, p, claim);
        eq_accumulate *= Polynomial::eq(u_now, v_now);
    }
    return eq_accumulate;
}

// rounds of at least this many index pairs take their middle coefficient from the running claim
static constexpr uint kClaimRoundMinOut = 1u << 16;

// src/prove.cu:87-117, with the three reductions fused into the round kernel
void matmul_sumcheck_phase2(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* v, uint K, Fr& claim,
                            Fr& eq_accumulate, SumcheckTranscript* transcript) {
    (void)a;
    (void)b;
    (void)c;
    uint rounds = Log2(K);
    if (rounds == 0) return;
    uint inputsize = K;
    uint outputsize = 1u << (rounds - 1);
    // all challenges of this phase in one copy
    std::vector<Fr> vs(rounds);
    check(grape_memcpy_d2h(vs.data(), v - rounds, sizeof(fr_t) * rounds, nullptr), "grape_memcpy_d2h");
    // The challenges are known before the first round, so all rounds are queued back to back,
    // each leaving its three sums in its own slot, and read with one copy at the end (the
    // reference copies and synchronises after every round).
    FrTensor sums(3 * rounds);
    // Long rounds (2^16 index pairs and more) are bound by their limb products, and one of the three
    // per pair can go when the round is given the running claim: p(0) + p(1) = claim fixes the middle
    // coefficient.  The claim the kernels chain is the one of the bare sums (without eq_accumulate).
    fr_t* d_claim = nullptr;
    if (outputsize >= kClaimRoundMinOut && !(eq_accumulate == Fr::zero())) {
        d_claim = grape_host::upload(std::vector<Fr>{claim * eq_accumulate.inverse()});
    }
    struct Release {
        fr_t*& p;
        ~Release() { grape_free(p); }
    } release{d_claim};
    for (uint i = 0; i < rounds; i++) {
        if (d_claim && outputsize >= kClaimRoundMinOut) {
            check(grape_sumcheck_round2_claim(W(A.gpu_data), W(B.gpu_data), inputsize, outputsize, W(v - i - 1), W(d_claim),
                                              W(sums.gpu_data + 3 * i), nullptr),
                  "grape_sumcheck_round2_claim");
            inputsize = outputsize;
            outputsize = outputsize / 2;
            continue;
        }
        if (inputsize <= 512) {
            // short tensors: all remaining rounds in one launch
            check(grape_sumcheck_round2_tail(W(A.gpu_data), W(B.gpu_data), inputsize, rounds - i, W(v - i), W(sums.gpu_data + 3 * i), nullptr),
                  "grape_sumcheck_round2_tail");
            break;
        }
        check(grape_sumcheck_round2(W(A.gpu_data), W(B.gpu_data), inputsize, outputsize, W(v - i - 1), W(sums.gpu_data + 3 * i), nullptr),
              "grape_sumcheck_round2");
        inputsize = outputsize;
        outputsize = outputsize / 2;
    }
    std::vector<Fr> s(3 * (size_t)rounds);
    check(grape_memcpy_d2h(s.data(), sums.gpu_data, sizeof(fr_t) * 3 * rounds, nullptr), "grape_memcpy_d2h");
    for (uint i = 0; i < rounds; i++) {
        Polynomial p({s[3 * i] * eq_accumulate, s[3 * i + 1] * eq_accumulate, s[3 * i + 2] * eq_accumulate});
        if (p(0) + p(1) != claim) throw std::runtime_error("matmul_phase2: claim != p(0) + p(1)");
        const Fr& v_now = vs[rounds - 1 - i];
        claim = p(v_now);
        record(transcript, p, claim);
    }
}

// src/prove.cu:175-210
std::pair<Fr, Fr> prove_matmul(FrTensor& A, FrTensor& B, int L, int N, int M, int K, const std::vector<Fr> u,
                               const std::vector<Fr> v, Fr& claim, SumcheckTranscript* transcript) {
    // The point u is read as log2(M) variables of the column index, log2(N) of the row index and log2(L)
    // of the batch index, while the reference finds the end of the batch variables at Log2(L*N*M)
    // (src/prove.cu:198): the two agree only when the padded extents multiply to the padded product.
    // A shape like N = 3, M = 5 (Log2(15) = 4, but 2 + 3 variables) has no defined reading - the
    // reference's folds would run past the end of u - and is refused, as is a point that is too short.
    const uint lu = Log2((uint)L) + Log2((uint)N) + Log2((uint)M);
    if (L < 1 || N < 1 || M < 1 || K < 1 || Log2((uint)(L * N * M)) != lu || u.size() < lu || v.size() < Log2((uint)(L * K)))
        throw std::runtime_error("prove_matmul: Incompatible dimensions");
    return prove_matmul_impl(&A, &B, nullptr, nullptr, L, N, M, K, u, v, claim, transcript);
}
std::pair<Fr, Fr> prove_matmul(const int* device_int_A, const int* device_int_B, int L, int N, int M, int K, const std::vector<Fr> u,
                               const std::vector<Fr> v, Fr& claim, SumcheckTranscript* transcript) {
    const uint lu = Log2((uint)L) + Log2((uint)N) + Log2((uint)M);
    if (L < 1 || N < 1 || M < 1 || K < 1 || Log2((uint)(L * N * M)) != lu || u.size() < lu || v.size() < Log2((uint)(L * K)))
        throw std::runtime_error("prove_matmul: Incompatible dimensions");
    return prove_matmul_impl(nullptr, nullptr, device_int_A, device_int_B, L, N, M, K, u, v, claim, transcript);
}
// A_in / B_in, or the integer tensors read as FrTensor::get_data would embed them: the folds over the row variables, which
// read each operand once, then read the integers themselves
std::pair<Fr, Fr> prove_matmul_impl(FrTensor* A_in, FrTensor* B_in, const int* A_ints, const int* B_ints, int L, int N, int M, int K,
                                    const std::vector<Fr>& u, const std::vector<Fr>& v, Fr& claim, SumcheckTranscript* transcript) {
    fr_t* U = grape_host::upload(u);
    fr_t* V = grape_host::upload(v);
    std::pair<Fr, Fr> ret;
    try {
        std::unique_ptr<FrTensor> A_own, B_own;
        if (A_ints) {
            A_own.reset(new FrTensor(FrTensor::folded_from_ints(A_ints, (uint)(L * N * K), U, N, Log2(M), K)));
            B_own.reset(new FrTensor(FrTensor::folded_from_ints(B_ints, (uint)(L * M * K), U, M, 0, K)));
        } else {
            A_in->partial_eval(A_in->size, U, N, Log2(M), K);
            B_in->partial_eval(B_in->size, U, M, 0, K);
        }
        FrTensor& A = A_ints ? *A_own : *A_in;
        FrTensor& B = A_ints ? *B_own : *B_in;
        FrTensor a(1), b(1), c(1);      // the reference's coefficient arrays (src/prove.cu:190-192): not used by the fused rounds
        Fr eq_accumulate = matmul_sumcheck_phase1(A, B, a, b, c, U + Log2(L * N * M), V + Log2(L * K), K, K * L, claim, transcript);
        matmul_sumcheck_phase2(A, B, a, b, c, V + Log2(K), K, claim, eq_accumulate, transcript);
        Fr A_claim = grape_host::download(A.gpu_data);
        Fr B_claim = grape_host::download(B.gpu_data);
        if (A_claim * B_claim * eq_accumulate != claim) throw std::runtime_error("prove_matmul: A(v) * B(v) * eq != claim");
        ret = {A_claim, B_claim};
    } catch (...) {
        grape_free(V);
        grape_free(U);
        throw;
    }
    grape_free(V);
    grape_free(U);
    return ret;
}

// The element-product sumcheck (src/prove.cu:119-172) proves sum_x eq(u, x) A(x) B(x) over tensors
// of first_size rows of second_size = size / first_size elements, the row index bound first
// (rows are not padded; a last row extent that is no power of two reads as zero-extended).  The
// reference writes three coefficient arrays per round and folds each over the remaining variables
// of u; here a round is one launch that folds A and B and takes the three sums weighted by
// eq(u_low, x) from a pyramid of tables built once - on rows padded to a power of two, which is
// where the variables of u live.
Fr eleMul_sumcheck(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* u, fr_t* v, uint first_size, uint size,
                   Fr& claim, SumcheckTranscript* transcript) {
    (void)a;
    (void)b;
    (void)c;
    if ((1u << Log2(first_size)) != first_size) throw std::runtime_error("eleMul_sumcheck: first_size is illegal");
    const uint second_size = size / first_size;
    const uint rounds = Log2(size);
    Fr eq_accumulate = Fr::one();
    if (rounds == 0) return eq_accumulate;
    const uint row_pad = 1u << Log2(second_size);
    const std::vector<Fr> us = download_vec(u - rounds, rounds), vs = download_vec(v - rounds, rounds);
    EqPyramid eq(u - rounds, rounds - 1);
    FrTensor sums(3 * rounds);
    uint in = size, out = size / 2;
    for (uint i = 0; i < rounds; i++) {
        // while whole rows are paired the weights are addressed on padded rows
        const bool rows = in > second_size && second_size != row_pad;
        check(grape_wround2(W(A.gpu_data), W(B.gpu_data), nullptr, W(eq.level(rounds - 1 - i)), in, out, rows ? second_size : 1,
                            rows ? row_pad : 1, W(v - i - 1), 0, W(sums.gpu_data + 3 * i), nullptr),
              "grape_wround2");
        in = out;
        out = out == second_size ? (1u << (Log2(out) - 1)) : out / 2;
        if (out == 0) out = 1;
    }
    const std::vector<Fr> s = download_vec(sums.gpu_data, 3 * (size_t)rounds);
    for (uint i = 0; i < rounds; i++) {
        const Fr &u_now = us[rounds - 1 - i], &v_now = vs[rounds - 1 - i];
        Polynomial p({s[3 * i], s[3 * i + 1], s[3 * i + 2]});
        p *= (Polynomial::eq(u_now) * eq_accumulate);
        if (p(0) + p(1) != claim) throw std::runtime_error("ele_Mul: claim != p(0) + p(1)");
        claim = p(v_now);
        record(transcript, p, claim);
        eq_accumulate *= Polynomial::eq(u_now, v_now);
    }
    return eq_accumulate;
}

// src/prove.cu:212-243
std::pair<Fr, Fr> prove_eleMul(FrTensor& A, FrTensor& B, int L, int M, int N, const std::vector<Fr> u, const std::vector<Fr> v,
                               Fr& claim, SumcheckTranscript* transcript) {
    fr_t* U = grape_host::upload(u);
    fr_t* V = grape_host::upload(v);
    std::pair<Fr, Fr> ret;
    try {
        FrTensor a(1), b(1), c(1);      // the reference's coefficient arrays (src/prove.cu:224-226): not used by the fused rounds
        Fr eq_accumulate = eleMul_sumcheck(A, B, a, b, c, U + Log2(L * N * M), V + Log2(L * M * N), L * M, L * M * N, claim, transcript);
        Fr A_claim = grape_host::download(A.gpu_data);
        Fr B_claim = grape_host::download(B.gpu_data);
        if (A_claim * B_claim * eq_accumulate != claim) throw std::runtime_error("prove_eleMul: A(v) * B(v) * eq != claim");
        ret = {A_claim, B_claim};
    } catch (...) {
        grape_free(V);
        grape_free(U);
        throw;
    }
    grape_free(V);
    grape_free(U);
    return ret;
}

// combine_claims (src/prove.cu:245-300) merges several claims X(u_j) = claim_j about one tensor into
// one claim X(v) by a sumcheck over sum_j sum_x eq(u_j, x) X(x).  Per round the reference copies
// the two coefficient arrays once per claim and evaluates each copy at the remaining variables of
// u_j; here the weights of every claim come from its own eq pyramid (built once), one launch takes
// all 2*num weighted sums of the round from a single read of X per claim, a second folds X, and
// the rounds are queued without copies in between.
Fr combine_claims(FrTensor& X, const std::vector<Fr>& claims, const std::vector<std::vector<Fr>>& u, const std::vector<Fr>& v,
                  const uint size, SumcheckTranscript* transcript) {
    if (size != (1u << Log2(size))) throw std::runtime_error("combine_claims: size must be a power of two");
    const uint num = (uint)claims.size();
    for (uint i = 0; i < num; i++)
        if (u[i].size() != v.size()) throw std::runtime_error("combine_claims: point sizes differ");
    if ((1u << v.size()) != size) throw std::runtime_error("combine_claims: 2^|v| != size");
    Fr claim = Fr::zero();
    for (uint i = 0; i < num; i++) claim += claims[i];
    const uint rounds = (uint)v.size();
    std::vector<Fr> eq_accumulate(num, Fr::one());
    if (rounds > 0 && num > 0) {
        fr_t* d_v = grape_host::upload(v);
        std::vector<std::unique_ptr<EqPyramid>> eq;
        std::vector<fr_t*> d_u(num, nullptr);
        FrTensor sums(2 * num * rounds);
        try {
            for (uint j = 0; j < num; j++) {
                d_u[j] = grape_host::upload(u[j]);
                eq.emplace_back(new EqPyramid(d_u[j], rounds - 1));
            }
            uint in = size;
            for (uint i = 0; i < rounds; i++) {
                const uint out = in / 2;
                // one launch weighs the tensor against up to 16 tables: more claims go in groups of 16
                for (uint j0 = 0; j0 < num; j0 += 16) {
                    const uint nj = num - j0 < 16 ? num - j0 : 16;
                    const uint32_t* tables[16];
                    for (uint j = 0; j < nj; j++) tables[j] = W(eq[j0 + j]->level(rounds - 1 - i));
                    check(grape_wsum1_multi(W(X.gpu_data), tables, nj, in, out, W(sums.gpu_data + 2 * ((size_t)num * i + j0)), nullptr),
                          "grape_wsum1_multi");
                }
                uint32_t* ptrs[1] = {W(X.gpu_data)};
                check(grape_fr_fold_msb_multi(ptrs, 1, out, W(d_v + (rounds - 1 - i)), nullptr), "grape_fr_fold_msb_multi");
                in = out;
            }
            const std::vector<Fr> s = download_vec(sums.gpu_data, 2 * (size_t)num * rounds);
            for (uint i = 0; i < rounds; i++) {
                const Fr& v_now = v[rounds - 1 - i];
                Polynomial p(2);
                for (uint j = 0; j < num; j++) {
                    const Fr& now_u = u[j][rounds - 1 - i];
                    const Fr* sj = &s[2 * ((size_t)num * i + j)];
                    Polynomial p1({sj[0], sj[1]});
                    p1 *= Polynomial::eq(now_u);
                    p1 *= eq_accumulate[j];
                    p += p1;
                    eq_accumulate[j] *= Polynomial::eq(now_u, v_now);
                }
                if (p(0) + p(1) != claim) throw std::runtime_error("combine_claims: claim != p(0) + p(1)");
                claim = p(v_now);
                record(transcript, p, claim);
            }
        } catch (...) {
            check(grape_stream_sync(nullptr), "sync");
            for (fr_t* d : d_u) grape_free(d);
            grape_free(d_v);
            throw;
        }
        check(grape_stream_sync(nullptr), "sync");
        for (fr_t* d : d_u) grape_free(d);
        grape_free(d_v);
    }
    Fr ret = X(0u);
    Fr sum = Fr::zero();
    for (uint i = 0; i < num; i++) sum += eq_accumulate[i] * ret;
    if (sum != claim) throw std::runtime_error("combine_claims: final check failed");
    return ret;
}
