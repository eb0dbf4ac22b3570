#include "prove.hpp"
#include <cassert>
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

// src/prove.cu:49-85
Fr matmul_sumcheck_phase1(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* u, fr_t* v, uint K, uint size,
                          Fr& claim, SumcheckTranscript* transcript) {
    uint rounds = Log2(size / K);
    uint inputsize = size;
    uint outputsize = inputsize / 2;
    Fr eq_accumulate = Fr::one();
    for (uint i = 0; i < rounds; i++) {
        check(grape_sumcheck_round2_coeffs(W(A.gpu_data), W(B.gpu_data), W(a.gpu_data), W(b.gpu_data), W(c.gpu_data), inputsize,
                                           outputsize, W(v - i - 1), nullptr, nullptr),
              "grape_sumcheck_round2_coeffs");
        a.partial_eval(outputsize, u - rounds, outputsize / K, 0, K);
        b.partial_eval(outputsize, u - rounds, outputsize / K, 0, K);
        c.partial_eval(outputsize, u - rounds, outputsize / K, 0, K);
        Polynomial p({c.sum(K), b.sum(K), a.sum(K)});
        Fr u_now = grape_host::download(u - i - 1);
        p *= (Polynomial::eq(u_now) * eq_accumulate);
        if (p(0) + p(1) != claim) throw std::runtime_error("matmul_phase1: claim != p(0) + p(1)");
        Fr v_now = grape_host::download(v - i - 1);
        claim = p(v_now);
        record(transcript, p, claim);
        inputsize = outputsize;
        outputsize = outputsize / 2;
        eq_accumulate *= (Fr::one() - v_now) * (Fr::one() - u_now) + v_now * u_now;
    }
    return eq_accumulate;
}

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
    for (uint i = 0; i < rounds; i++) {
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
    fr_t* U = grape_host::upload(u);
    fr_t* V = grape_host::upload(v);
    std::pair<Fr, Fr> ret;
    try {
        A.partial_eval(A.size, U, N, Log2(M), K);
        B.partial_eval(B.size, U, M, 0, K);
        uint LK = (uint)L * (uint)K;
        FrTensor a(LK < 3 ? 3 : LK), b(LK), c(LK);
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

// src/prove.cu:119-172
Fr eleMul_sumcheck(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* u, fr_t* v, uint first_size, uint size,
                   Fr& claim, SumcheckTranscript* transcript) {
    if ((1u << Log2(first_size)) != first_size) throw std::runtime_error("eleMul_sumcheck: first_size is illegal");
    uint second_size = size / first_size;
    uint rounds = Log2(size);
    uint inputsize = size;
    uint outputsize = size / 2;
    Fr eq_accumulate = Fr::one();
    for (uint i = 0; i < rounds; i++) {
        check(grape_sumcheck_round2_coeffs(W(A.gpu_data), W(B.gpu_data), W(a.gpu_data), W(b.gpu_data), W(c.gpu_data), inputsize,
                                           outputsize, W(v - i - 1), nullptr, nullptr),
              "grape_sumcheck_round2_coeffs");
        if (inputsize > second_size) {
            for (FrTensor* t : {&a, &b, &c}) {
                t->partial_eval(outputsize, u - Log2(first_size), outputsize / second_size, 0, second_size);
                t->partial_eval(second_size, u - Log2(size), second_size, 0, 1);
            }
        } else {
            for (FrTensor* t : {&a, &b, &c}) t->partial_eval(outputsize, u - Log2(size), outputsize, 0, 1);
        }
        Polynomial p({c(0u), b(0u), a(0u)});
        Fr u_now = grape_host::download(u - i - 1);
        p *= (Polynomial::eq(u_now) * eq_accumulate);
        if (p(0) + p(1) != claim) throw std::runtime_error("ele_Mul: claim != p(0) + p(1)");
        Fr v_now = grape_host::download(v - i - 1);
        claim = p(v_now);
        record(transcript, p, claim);
        inputsize = outputsize;
        outputsize = outputsize == second_size ? (1u << (Log2(outputsize) - 1)) : outputsize / 2;
        eq_accumulate *= ((Fr::one() - v_now) * (Fr::one() - u_now) + v_now * u_now);
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
        uint half = (uint)(L * M * N / 2);
        FrTensor a(half ? half : 1), b(half ? half : 1), c(half ? half : 1);
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

// src/prove.cu:245-300: several claims X(u_j) = claim_j about one tensor reduced to one claim X(v)
Fr combine_claims(FrTensor& X, const std::vector<Fr>& claims, const std::vector<std::vector<Fr>>& u, const std::vector<Fr>& v,
                  const uint size, SumcheckTranscript* transcript) {
    if (size != (1u << Log2(size))) throw std::runtime_error("combine_claims: size must be a power of two");
    uint num = (uint)claims.size();
    for (uint i = 0; i < num; i++)
        if (u[i].size() != v.size()) throw std::runtime_error("combine_claims: point sizes differ");
    if ((1u << v.size()) != size) throw std::runtime_error("combine_claims: 2^|v| != size");
    Fr claim = Fr::zero();
    for (uint i = 0; i < num; i++) claim += claims[i];
    uint rounds = (uint)v.size();
    uint half = size / 2 ? size / 2 : 1;
    FrTensor a(half), b(half), tmp_a(half), tmp_b(half);
    uint input_size = size, output_size = size / 2;
    std::vector<std::vector<Fr>> new_u = u;
    std::vector<Fr> new_v = v;
    std::vector<Fr> eq_accumulate(num, Fr::one());
    for (uint i = 0; i < rounds; i++) {
        a.set_size(output_size);
        b.set_size(output_size);
        tmp_a.set_size(output_size);
        tmp_b.set_size(output_size);
        fr_t* d_v = grape_host::device_scalar(new_v.back());
        check(grape_sumcheck_round1(W(X.gpu_data), W(a.gpu_data), W(b.gpu_data), input_size, output_size, W(d_v), nullptr),
              "grape_sumcheck_round1");
        Polynomial p(2);
        for (uint j = 0; j < num; j++) {
            Fr now_u = new_u[j].back();
            new_u[j].pop_back();
            tmp_a = a;
            tmp_b = b;
            Polynomial p1({tmp_b(new_u[j]), tmp_a(new_u[j])});
            p1 *= Polynomial::eq(now_u);
            p1 *= eq_accumulate[j];
            p += p1;
            eq_accumulate[j] *= Polynomial::eq(now_u, new_v.back());
        }
        if (p(0) + p(1) != claim) throw std::runtime_error("combine_claims: claim != p(0) + p(1)");
        claim = p(new_v.back());
        record(transcript, p, claim);
        new_v.pop_back();
        input_size = output_size;
        output_size = output_size / 2;
    }
    Fr ret = X(0u);
    Fr sum = Fr::zero();
    for (uint i = 0; i < num; i++) sum += eq_accumulate[i] * ret;
    if (sum != claim) throw std::runtime_error("combine_claims: final check failed");
    return ret;
}
