// Sumcheck provers: the interface of the reference's include/prove.cuh:36-54.
// Every entry point takes one extra, optional argument that records the round polynomials
// (the reference keeps no transcript; a drop-in call site simply omits it).
#pragma once
#include <utility>
#include <vector>
#include "fr_tensor.hpp"
#include "polynomial.hpp"

struct SumcheckTranscript {
    std::vector<Polynomial> rounds;   // one polynomial per round, coefficients low to high
    std::vector<Fr> claims;           // running claim after each round
};

// Work tensors a driver keeps across the sumchecks of one layer (include/prove.cuh:13-26):
// a, b, c hold tokens_size * 2^13 elements each, tmpw one FFN row of 11008.
struct SumcheckWorkTmp {
    FrTensor tmpw;
    FrTensor a;
    FrTensor b;
    FrTensor c;
    size_t tokens_size;

    explicit SumcheckWorkTmp(size_t tokens_size_)
        : tmpw(11008), a((uint)(tokens_size_ * (1u << 13))), b((uint)(tokens_size_ * (1u << 13))),
          c((uint)(tokens_size_ * (1u << 13))), tokens_size(tokens_size_) {}
    SumcheckWorkTmp(const SumcheckWorkTmp&) = delete;
    SumcheckWorkTmp& operator=(const SumcheckWorkTmp&) = delete;
};

Fr matmul_sumcheck_phase1(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* u, fr_t* v, uint K,
                          uint size, Fr& claim, SumcheckTranscript* transcript = nullptr);
void matmul_sumcheck_phase2(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* v, uint K, Fr& claim,
                            Fr& eq_accumulate, SumcheckTranscript* transcript = nullptr);
Fr eleMul_sumcheck(FrTensor& A, FrTensor& B, FrTensor& a, FrTensor& b, FrTensor& c, fr_t* u, fr_t* v, uint first_size,
                   uint size, Fr& claim, SumcheckTranscript* transcript = nullptr);

// A is L x N x K, B is L x M x K (k fastest); both are consumed.  u = (m bits | n bits | l bits),
// v = (k bits | l bits), claim in/out.  Returns (A(v_k,u_n,v_l), B(v_k,u_m,v_l)).
std::pair<Fr, Fr> prove_matmul(FrTensor& A, FrTensor& B, int L, int N, int M, int K, const std::vector<Fr> u,
                               const std::vector<Fr> v, Fr& claim, SumcheckTranscript* transcript = nullptr);
// addition: prove_matmul for the tensors FrTensor::get_data would make of the device integers (the reference's drivers embed
// the operands and prove, test/llm.cu:85-95): the folds over the row variables read the integers
std::pair<Fr, Fr> prove_matmul(const int* device_int_A, const int* device_int_B, int L, int N, int M, int K, const std::vector<Fr> u,
                               const std::vector<Fr> v, Fr& claim, SumcheckTranscript* transcript = nullptr);
std::pair<Fr, Fr> prove_matmul_impl(FrTensor* A, FrTensor* B, const int* A_ints, const int* B_ints, int L, int N, int M, int K,
                                    const std::vector<Fr>& u, const std::vector<Fr>& v, Fr& claim, SumcheckTranscript* transcript);
std::pair<Fr, Fr> prove_eleMul(FrTensor& A, FrTensor& B, int L, int M, int N, const std::vector<Fr> u,
                               const std::vector<Fr> v, Fr& claim, SumcheckTranscript* transcript = nullptr);
Fr combine_claims(FrTensor& X, const std::vector<Fr>& claims, const std::vector<std::vector<Fr>>& u,
                  const std::vector<Fr>& v, const uint size, SumcheckTranscript* transcript = nullptr);
