#include "ec_operation.hpp"
#include <algorithm>
#include "../../include/grape_hip.h"

using grape_host::check;

std::vector<bn128> precompute_generators(uint N, uint W, affine_t* out) {
    grape_host::ensure_init();
    // scalars on the host, points on the device; the scalars (the generators' discrete logarithms,
    // which would break the binding of every commitment) are wiped on both sides once used
    std::vector<uint32_t> k(8 * (size_t)N);
    for (uint i = 0; i < N; i++) Fr::random_element().to_plain(&k[8 * (size_t)i]);
    uint32_t* d_k = nullptr;
    affine_t *d_base = nullptr, *d_gens = nullptr;
    check(grape_malloc((void**)&d_k, 32 * (size_t)N), "grape_malloc");
    check(grape_malloc((void**)&d_base, sizeof(affine_t)), "grape_malloc");
    check(grape_malloc((void**)&d_gens, sizeof(affine_t) * (size_t)N), "grape_malloc");
    affine_t base;
    check(grape_g1_generator(reinterpret_cast<uint32_t*>(&base)), "grape_g1_generator");
    check(grape_memcpy_h2d(d_k, k.data(), 32 * (size_t)N, nullptr), "h2d");
    check(grape_memcpy_h2d(d_base, &base, sizeof(affine_t), nullptr), "h2d");
    check(grape_g1_scalar_mul_base(reinterpret_cast<uint32_t*>(d_gens), d_k, reinterpret_cast<uint32_t*>(d_base), N, nullptr),
          "grape_g1_scalar_mul_base");
    check(grape_g1_table_gen(reinterpret_cast<uint32_t*>(out), reinterpret_cast<uint32_t*>(d_gens), N, W, nullptr), "grape_g1_table_gen");
    std::vector<affine_t> host(N);
    check(grape_memcpy_d2h(host.data(), d_gens, sizeof(affine_t) * (size_t)N, nullptr), "d2h");
    check(grape_memset_zero(d_k, 32 * (size_t)N, nullptr), "grape_memset_zero");
    check(grape_stream_sync(nullptr), "sync");
    {
        volatile uint32_t* w = k.data();
        for (size_t i = 0; i < k.size(); i++) w[i] = 0;
    }
    grape_free(d_k);
    grape_free(d_base);
    grape_free(d_gens);
    std::vector<bn128> gens(N);
    for (uint i = 0; i < N; i++) gens[i] = bn128(host[i]);
    return gens;
}

std::vector<Fr> random_vec(uint len) {
    std::vector<Fr> out(len);
    for (uint i = 0; i < len; i++) out[i] = Fr::random_element();
    return out;
}

void generate_random_eval_points(size_t data_size, std::vector<Fr>& eval_point) {
    size_t log_size = Log2((uint)data_size);
    if (eval_point.size() != log_size) eval_point.resize(log_size);
    for (size_t i = 0; i < log_size; i++) eval_point[i] = Fr::random_element();
}

// first  <- second[:same] | first[last : last+first_size] | second[same:]
// second <- second[:same] | first[:last]                  | second[same:]
void ReassembleVectors(std::vector<Fr>& first, std::vector<Fr>& second, size_t first_size, size_t same_size, size_t last_size) {
    std::vector<Fr> r1, r2;
    r1.insert(r1.end(), second.begin(), second.begin() + same_size);
    r1.insert(r1.end(), first.begin() + last_size, first.begin() + last_size + first_size);
    r1.insert(r1.end(), second.begin() + same_size, second.end());
    r2.insert(r2.end(), second.begin(), second.begin() + same_size);
    r2.insert(r2.end(), first.begin(), first.begin() + last_size);
    r2.insert(r2.end(), second.begin() + same_size, second.end());
    second = r2;
    first = r1;
}
