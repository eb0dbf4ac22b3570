#include "host_capi.h"
#include "ioutils.hpp"
#include <cstring>
#include <string>
#include "../../include/grape_hip.h"
#include "ec_operation.hpp"
#include "fr_tensor.hpp"
#include "hyrax.hpp"
#include "prove.hpp"
#include "tlookup.hpp"
#include "witness.hpp"

static thread_local std::string g_err;
static double g_last_prove_s = 0;
static bool g_indexed_commit = true;
static double g_last_commit_s = 0;
#include <chrono>
struct ProveTimer {
    std::chrono::steady_clock::time_point t0;
    ProveTimer() {
        grape_stream_sync(nullptr);
        t0 = std::chrono::steady_clock::now();
    }
    ~ProveTimer() {
        grape_stream_sync(nullptr);
        g_last_prove_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    }
};

#define GUARD_BEGIN try {
#define GUARD_END                      \
    }                                  \
    catch (const std::exception& e) {  \
        g_err = e.what();              \
        return 1;                      \
    }                                  \
    return 0;

#include <map>
#include <array>
#include <memory>
#include <tuple>
// Hyrax objects persist across calls (keyed by their table), so the wide fixed-base tables
// they build are generated once per generator set, as in a long-running prover.
static void drop_lookup_objects();   // they hold tables tied to a Hyrax object: gone before it goes
static Hyrax& hyrax_for(const uint32_t* d_table, uint32_t npoints, uint32_t com_scale, uint32_t layer_num) {
    typedef std::tuple<const uint32_t*, uint32_t, uint32_t, uint32_t> Key;
    static std::map<Key, std::unique_ptr<Hyrax>> cache;
    static bn128 G = bn128::one();
    Key k(d_table, npoints, com_scale, layer_num);
    auto it = cache.find(k);
    if (it == cache.end()) {
        if (cache.size() >= 4) {                // bounded: drop old tables
            drop_lookup_objects();
            cache.clear();
        }
        it = cache.emplace(k, std::unique_ptr<Hyrax>(new Hyrax(layer_num, npoints / com_scale, (affine_t*)d_table, G, com_scale))).first;
    }
    return *it->second;
}

static std::vector<Fr> vec_from(const uint32_t* p, uint32_t n) {
    std::vector<Fr> v(n);
    if (n) std::memcpy(v.data(), p, 32 * (size_t)n);
    return v;
}
static Fr fr_from(const uint32_t* p) {
    Fr x;
    std::memcpy(&x, p, 32);
    return x;
}
static void fr_to(uint32_t* p, const Fr& x) { std::memcpy(p, &x, 32); }
static int g_input_format = 0;      // 0: field elements, 1: int32 values (grape_host_set_input_format)
static bool g_int_folds = true;     // integer inputs of an opening or an evaluation are folded from the integers (grape_host_set_int_folds)
static FrTensor tensor_from_device(const uint32_t* d, uint32_t n, uint32_t capacity = 0) {
    FrTensor t(capacity > n ? capacity : n);
    if (g_input_format == 1) {
        // as the reference's drivers hand integers to a tensor: FrTensor::get_data (test/llm.cu:77)
        t.get_data(n, reinterpret_cast<int*>(const_cast<uint32_t*>(d)));
        return t;
    }
    t.set_size(n);
    grape_host::check(grape_memcpy_d2d(t.gpu_data, d, 32 * (size_t)n, nullptr), "grape_memcpy_d2d");
    return t;
}
static void put_transcript(const SumcheckTranscript& tr, uint32_t* out, uint32_t* n_rounds) {
    *n_rounds = (uint32_t)tr.rounds.size();
    for (size_t r = 0; r < tr.rounds.size(); r++) {
        std::memset(out + 32 * r, 0, 128);
        const auto& c = tr.rounds[r].coefficients();
        for (size_t i = 0; i < c.size() && i < 4; i++) fr_to(out + 32 * r + 8 * i, c[i]);
    }
}

extern "C" {

const char* grape_host_last_error(void) { return g_err.c_str(); }
double grape_host_last_prove_seconds(void) { return g_last_prove_s; }
double grape_host_last_commit_seconds(void) { return g_last_commit_s; }
void grape_host_seed(uint64_t seed) { Fr::seed(seed); }
void grape_host_set_indexed_commit(int on) { g_indexed_commit = on != 0; }
int grape_host_set_input_format(int fmt) {
    if (fmt != 0 && fmt != 1) return 1;
    g_input_format = fmt;
    return 0;
}
void grape_host_set_int_folds(int on) { g_int_folds = on != 0; }

int grape_host_prove_matmul(const uint32_t* d_A, const uint32_t* d_B, int L, int N, int M, int K, const uint32_t* u, uint32_t nu,
                            const uint32_t* v, uint32_t nv, uint32_t* claim_inout, uint32_t* transcript, uint32_t* n_rounds,
                            uint32_t* A_claim, uint32_t* B_claim) {
    GUARD_BEGIN
    Fr claim = fr_from(claim_inout);
    SumcheckTranscript tr;
    std::pair<Fr, Fr> res;
    if (g_input_format == 1 && g_int_folds) {
        ProveTimer timer;
        res = prove_matmul(reinterpret_cast<const int*>(d_A), reinterpret_cast<const int*>(d_B), L, N, M, K, vec_from(u, nu), vec_from(v, nv),
                           claim, &tr);
    } else {
        FrTensor A = tensor_from_device(d_A, (uint32_t)(L * N * K));
        FrTensor B = tensor_from_device(d_B, (uint32_t)(L * M * K));
        ProveTimer timer;
        res = prove_matmul(A, B, L, N, M, K, vec_from(u, nu), vec_from(v, nv), claim, &tr);
    }
    fr_to(claim_inout, claim);
    fr_to(A_claim, res.first);
    fr_to(B_claim, res.second);
    put_transcript(tr, transcript, n_rounds);
    GUARD_END
}

int grape_host_prove_elemul(const uint32_t* d_A, const uint32_t* d_B, int L, int M, int N, const uint32_t* u, uint32_t nu,
                            const uint32_t* v, uint32_t nv, uint32_t* claim_inout, uint32_t* transcript, uint32_t* n_rounds,
                            uint32_t* A_claim, uint32_t* B_claim) {
    GUARD_BEGIN
    FrTensor A = tensor_from_device(d_A, (uint32_t)(L * M * N));
    FrTensor B = tensor_from_device(d_B, (uint32_t)(L * M * N));
    Fr claim = fr_from(claim_inout);
    SumcheckTranscript tr;
    std::pair<Fr, Fr> res;
    {
        ProveTimer timer;
        res = prove_eleMul(A, B, L, M, N, vec_from(u, nu), vec_from(v, nv), claim, &tr);
    }
    fr_to(claim_inout, claim);
    fr_to(A_claim, res.first);
    fr_to(B_claim, res.second);
    put_transcript(tr, transcript, n_rounds);
    GUARD_END
}

int grape_host_combine_claims(const uint32_t* d_X, uint32_t size, const uint32_t* claims, uint32_t num, const uint32_t* u,
                              const uint32_t* v, uint32_t nv, uint32_t* transcript, uint32_t* n_rounds, uint32_t* result) {
    GUARD_BEGIN
    FrTensor X = tensor_from_device(d_X, size);
    std::vector<std::vector<Fr>> us(num);
    for (uint32_t j = 0; j < num; j++) us[j] = vec_from(u + 8 * (size_t)j * nv, nv);
    SumcheckTranscript tr;
    Fr r;
    {
        ProveTimer timer;
        r = combine_claims(X, vec_from(claims, num), us, vec_from(v, nv), size, &tr);
    }
    fr_to(result, r);
    put_transcript(tr, transcript, n_rounds);
    GUARD_END
}

int grape_host_mle_eval(const uint32_t* d_T, uint32_t size, const uint32_t* u, uint32_t nu, uint32_t* out) {
    GUARD_BEGIN
    if (g_input_format == 1 && g_int_folds) {
        fr_to(out, FrTensor::eval_ints(reinterpret_cast<const int*>(d_T), size, vec_from(u, nu)));
    } else {
        FrTensor T = tensor_from_device(d_T, size);
        fr_to(out, T(vec_from(u, nu)));
    }
    GUARD_END
}

int grape_host_hyrax_commit_i32(const int32_t* d_scalars, uint32_t size, uint32_t N, const uint32_t* d_table, uint32_t npoints,
                                uint32_t com_scale, uint32_t layer_num, uint32_t* out_affine) {
    GUARD_BEGIN
    Hyrax& hyrax = hyrax_for(d_table, npoints, com_scale, layer_num);
    affine_t* c = hyrax.commit_affine(const_cast<int*>(d_scalars), size, N);
    uint32_t rows = size / (N * com_scale);
    grape_host::check(grape_memcpy_d2h(out_affine, c, sizeof(affine_t) * (size_t)rows, nullptr), "d2h");
    grape_free(c);
    GUARD_END
}

int grape_host_hyrax_commit_fr(const uint32_t* d_scalars, uint32_t size, uint32_t N, const uint32_t* d_table, uint32_t npoints,
                               uint32_t com_scale, uint32_t layer_num, uint32_t* out_affine) {
    GUARD_BEGIN
    Hyrax& hyrax = hyrax_for(d_table, npoints, com_scale, layer_num);
    FrTensor t = tensor_from_device(d_scalars, size);
    // through the Jacobian-returning entry point, to cover the reference's return format
    jacob_t* cj = hyrax.commit(t, size, N);
    uint32_t rows = size / (N * com_scale);
    affine_t* ca = nullptr;
    grape_host::check(grape_malloc((void**)&ca, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    grape_host::check(grape_g1_jacobian_to_affine((uint32_t*)ca, (const uint32_t*)cj, rows, nullptr), "jac->affine");
    grape_host::check(grape_memcpy_d2h(out_affine, ca, sizeof(affine_t) * (size_t)rows, nullptr), "d2h");
    grape_free(ca);
    grape_free(cj);
    GUARD_END
}

int grape_host_hyrax_open_verify(const uint32_t* d_tensor, uint32_t size, uint32_t N, const uint32_t* d_table, uint32_t npoints,
                                 uint32_t com_scale, uint32_t layer_num, const uint32_t* eval_point, uint32_t n_eval,
                                 const uint32_t* c, uint32_t* result, int* verified) {
    GUARD_BEGIN
    Hyrax& hyrax = hyrax_for(d_table, npoints, com_scale, layer_num);
    FrTensor t = tensor_from_device(d_tensor, size);
    jacob_t* com = hyrax.commit(t, size, N);
    std::vector<Fr> pt = vec_from(eval_point, n_eval);
    Hyrax_proof proof = hyrax.open(t, pt, fr_from(c), size, N);
    fr_to(result, proof.result);
    *verified = hyrax.verify(proof, com, pt, fr_from(c), size, N) ? 1 : 0;
    grape_free(com);
    GUARD_END
}

// Hyrax::open alone (src/Hyrax.cu:237-305): the opening a prover runs after a sub-proof, timed like the provers
int grape_host_hyrax_open(const uint32_t* d_tensor, uint32_t size, uint32_t N, const uint32_t* d_table, uint32_t npoints,
                          uint32_t com_scale, uint32_t layer_num, const uint32_t* eval_point, uint32_t n_eval, const uint32_t* c,
                          uint32_t* result) {
    GUARD_BEGIN
    Hyrax& hyrax = hyrax_for(d_table, npoints, com_scale, layer_num);
    if (g_input_format == 1 && g_int_folds) {
        ProveTimer timer;
        Hyrax_proof proof = hyrax.open(reinterpret_cast<const int*>(d_tensor), vec_from(eval_point, n_eval), fr_from(c), size, N);
        fr_to(result, proof.result);
    } else {
        FrTensor t = tensor_from_device(d_tensor, size);
        ProveTimer timer;
        Hyrax_proof proof = hyrax.open(t, vec_from(eval_point, n_eval), fr_from(c), size, N);
        fr_to(result, proof.result);
    }
    GUARD_END
}

extern "C++" {
// Lookup objects persist across calls like the reference's driver keeps them across the layers of a
// model (test/llm.cu:57-64): the tables tied to them (B[t]*G_i over every entry of a range table,
// over the occupied entries of a mapping table) are built by the first proof.
typedef std::tuple<int32_t, uint32_t, Hyrax*> LKey;
static std::map<LKey, std::unique_ptr<tLookupRange>> g_range_lookups;
// a mapping lookup with its r pinned (the constructor draws r; the table is rebuilt with the given one)
struct PinnedMapping : tLookupRangeMapping {
    PinnedMapping(int low, uint len, const int* map, const Fr& r_) : tLookupRangeMapping(low, len, map) {
        r = r_;
        grape_host::check(grape_tlookup_init((uint32_t*)T.gpu_data, (uint32_t*)B.gpu_data, low, len,
                                             (uint32_t*)grape_host::device_scalar(beta), (uint32_t*)mapped_vals.gpu_data,
                                             (uint32_t*)grape_host::device_scalar(r), nullptr),
                          "grape_tlookup_init");
    }
};
// keyed by range, r, a hash of the mapped values and the Hyrax object
typedef std::tuple<int32_t, uint32_t, std::array<uint64_t, 4>, uint64_t, Hyrax*> MKey;
static std::map<MKey, std::unique_ptr<PinnedMapping>> g_mapping_lookups;
static void drop_lookup_objects() {
    g_range_lookups.clear();
    g_mapping_lookups.clear();
}
static uint64_t hash_ints(const int32_t* p, size_t n) {
    uint64_t h = 1469598103934665603ull;                 // FNV-1a over the words
    for (size_t i = 0; i < n; i++) {
        h ^= (uint32_t)p[i];
        h *= 1099511628211ull;
    }
    return h;
}
}  // extern "C++"

int grape_host_tlookup_range_prove(const uint32_t* d_S, uint32_t D, int32_t low, uint32_t len, const uint32_t* alpha,
                                   const uint32_t* u, const uint32_t* v, uint32_t nuv, const uint32_t* d_table, uint32_t npoints,
                                   uint32_t com_scale, uint32_t msm_size, uint32_t* m_out, uint32_t* transcript, uint32_t* n_rounds,
                                   uint32_t* S_claim, uint32_t* com_A_out, uint32_t* com_m_out, double* commit_seconds) {
    GUARD_BEGIN
    Hyrax& hyrax = hyrax_for(d_table, npoints, com_scale, 1);
    // lookup objects persist like Hyrax objects: their scaled table is built once
    LKey lkey(low, len, &hyrax);
    auto lit = g_range_lookups.find(lkey);
    if (lit == g_range_lookups.end()) {
        if (g_range_lookups.size() >= 2) g_range_lookups.clear();
        lit = g_range_lookups.emplace(lkey, std::unique_ptr<tLookupRange>(new tLookupRange(low, len))).first;
    }
    tLookupRange& lk = *lit->second;
    lk.set_indexed_commit(g_indexed_commit);
    lk.alpha = fr_from(alpha);
    lk.set_u(vec_from(u, nuv));
    uint32_t Dp = 1u << Log2(D);
    FrTensor A(Dp);
    double ct = 0;
    Fr sc;
    if (g_input_format == 1 && g_int_folds) {
        // the witness stays a tensor of integers: the prover's pass over it embeds it on the way
        FrTensor S(Dp);
        S.set_size(D);
        ProveTimer timer;
        sc = lk.prove(reinterpret_cast<const int*>(d_S), S, A, vec_from(v, nuv), hyrax, msm_size, ct);
    } else {
        FrTensor S = tensor_from_device(d_S, D, Dp);
        ProveTimer timer;
        sc = lk.prove(S, A, vec_from(v, nuv), hyrax, msm_size, ct);
    }
    fr_to(S_claim, sc);
    put_transcript(lk.last_transcript, transcript, n_rounds);
    if (m_out) grape_host::check(grape_memcpy_d2h(m_out, lk.m.gpu_data, 32 * (size_t)lk.m.size, nullptr), "d2h");
    if (com_A_out) grape_host::check(grape_memcpy_d2h(com_A_out, lk.com_A, sizeof(affine_t) * (size_t)lk.com_A_rows, nullptr), "d2h");
    if (com_m_out) grape_host::check(grape_memcpy_d2h(com_m_out, lk.com_m, sizeof(affine_t) * (size_t)lk.com_m_rows, nullptr), "d2h");
    g_last_commit_s = ct;
    if (commit_seconds) *commit_seconds = ct;
    GUARD_END
}

static void mapping_prove_impl(const uint32_t* d_S_in, const uint32_t* d_S_out, uint32_t D, int32_t low, uint32_t len,
                               const int32_t* map, const uint32_t* alpha, const uint32_t* r, const uint32_t* u,
                               const uint32_t* v, uint32_t nuv, const uint32_t* d_table, uint32_t npoints, uint32_t com_scale,
                               uint32_t msm_size, uint32_t* transcript, uint32_t* n_rounds, uint32_t* S_claim,
                               uint32_t hot_min_count, uint32_t* com_A_out, uint64_t* hot_stats) {
    Hyrax& hyrax = hyrax_for(d_table, npoints, com_scale, 1);
    std::array<uint64_t, 4> rk;
    std::memcpy(rk.data(), r, 32);
    MKey mkey(low, len, rk, hash_ints(map, len), &hyrax);
    auto mit = g_mapping_lookups.find(mkey);
    if (mit == g_mapping_lookups.end()) {
        if (g_mapping_lookups.size() >= 4) g_mapping_lookups.clear();
        mit = g_mapping_lookups.emplace(mkey, std::unique_ptr<PinnedMapping>(new PinnedMapping(low, len, map, fr_from(r)))).first;
    }
    PinnedMapping& lk = *mit->second;
    lk.set_indexed_commit(g_indexed_commit);
    lk.set_hot_min_count(hot_min_count);
    lk.alpha = fr_from(alpha);
    lk.set_u(vec_from(u, nuv));
    uint32_t Dp = 1u << Log2(D);
    FrTensor A(Dp);
    double ct = 0;
    Fr sc;
    if (g_input_format == 1 && g_int_folds) {
        ProveTimer timer;
        sc = lk.prove(reinterpret_cast<const int*>(d_S_in), reinterpret_cast<const int*>(d_S_out), D, A, vec_from(v, nuv), hyrax, msm_size, ct);
    } else {
        FrTensor S_in = tensor_from_device(d_S_in, D);
        FrTensor S_out = tensor_from_device(d_S_out, D);
        ProveTimer timer;
        sc = lk.prove(S_in, S_out, A, vec_from(v, nuv), hyrax, msm_size, ct);
    }
    g_last_commit_s = ct;
    fr_to(S_claim, sc);
    put_transcript(lk.last_transcript, transcript, n_rounds);
    if (com_A_out) grape_host::check(grape_memcpy_d2h(com_A_out, lk.com_A, sizeof(affine_t) * (size_t)lk.com_A_rows, nullptr), "d2h");
    if (hot_stats) {
        hot_stats[0] = lk.hot_entries();
        hot_stats[1] = lk.cold_elements();
        hot_stats[2] = lk.hot_rows_reused() ? 1 : 0;
    }
}

int grape_host_tlookup_mapping_prove(const uint32_t* d_S_in, const uint32_t* d_S_out, uint32_t D, int32_t low, uint32_t len,
                                     const int32_t* map, const uint32_t* alpha, const uint32_t* r, const uint32_t* u,
                                     const uint32_t* v, uint32_t nuv, const uint32_t* d_table, uint32_t npoints, uint32_t com_scale,
                                     uint32_t msm_size, uint32_t* transcript, uint32_t* n_rounds, uint32_t* S_claim) {
    GUARD_BEGIN
    mapping_prove_impl(d_S_in, d_S_out, D, low, len, map, alpha, r, u, v, nuv, d_table, npoints, com_scale, msm_size, transcript,
                       n_rounds, S_claim, 0, nullptr, nullptr);
    GUARD_END
}

int grape_host_tlookup_mapping_prove_ex(const uint32_t* d_S_in, const uint32_t* d_S_out, uint32_t D, int32_t low, uint32_t len,
                                        const int32_t* map, const uint32_t* alpha, const uint32_t* r, const uint32_t* u,
                                        const uint32_t* v, uint32_t nuv, const uint32_t* d_table, uint32_t npoints,
                                        uint32_t com_scale, uint32_t msm_size, uint32_t* transcript, uint32_t* n_rounds,
                                        uint32_t* S_claim, uint32_t hot_min_count, uint32_t* com_A_out, uint64_t* hot_stats) {
    GUARD_BEGIN
    mapping_prove_impl(d_S_in, d_S_out, D, low, len, map, alpha, r, u, v, nuv, d_table, npoints, com_scale, msm_size, transcript,
                       n_rounds, S_claim, hot_min_count, com_A_out, hot_stats);
    GUARD_END
}

int grape_host_fr_op(int op, const uint32_t* a, const uint32_t* b, uint32_t* out) {
    GUARD_BEGIN
    Fr x = fr_from(a), y = b ? fr_from(b) : Fr::zero(), r;
    switch (op) {
        case 0: r = x + y; break;
        case 1: r = x - y; break;
        case 2: r = x * y; break;
        case 3: r = x.inverse(); break;
        default: throw std::runtime_error("bad op");
    }
    fr_to(out, r);
    GUARD_END
}

int grape_host_g1_mul_generator(const uint32_t* k_mont, uint32_t* out_affine) {
    GUARD_BEGIN
    bn128 p = fr_from(k_mont) * bn128::one();
    affine_t a = p.to_affine();
    std::memcpy(out_affine, &a, sizeof a);
    GUARD_END
}

int grape_host_single_commit(const uint32_t* d_scalars, uint32_t N, const uint32_t* d_table, uint32_t npoints, uint32_t* out_affine) {
    GUARD_BEGIN
    jacob_t* com = nullptr;
    grape_host::check(grape_malloc((void**)&com, sizeof(jacob_t)), "grape_malloc");
    single_commit((fr_t*)d_scalars, (affine_t*)d_table, com, N, npoints);
    affine_t* aff = nullptr;
    grape_host::check(grape_malloc((void**)&aff, sizeof(affine_t)), "grape_malloc");
    grape_host::check(grape_g1_jacobian_to_affine((uint32_t*)aff, (const uint32_t*)com, 1, nullptr), "grape_g1_jacobian_to_affine");
    grape_host::check(grape_memcpy_d2h(out_affine, aff, sizeof(affine_t), nullptr), "grape_memcpy_d2h");
    grape_free(aff);
    grape_free(com);
    GUARD_END
}
int grape_host_bin_io(int op, const char* filename, void* ptr, size_t size, int is_gpu) {
    GUARD_BEGIN
    if (op == 0) savebin(filename, ptr, size, is_gpu != 0);
    else loadbin(filename, ptr, size, is_gpu != 0);
    GUARD_END
}
unsigned long grape_host_findsize(const char* filename) { return findsize(filename); }
int grape_host_load_data(const char* filename, int32_t** d_out, uint32_t* n) {
    GUARD_BEGIN
    int* p = nullptr;
    *n = load_data(filename, &p);
    *d_out = p;
    GUARD_END
}
int grape_host_generate_data(int32_t** d_out, uint32_t size) {
    GUARD_BEGIN
    int* p = nullptr;
    generate_data(&p, size);
    *d_out = p;
    GUARD_END
}


int grape_host_layer_witness_new(void** handle, uint32_t seq_len, uint32_t dim, uint32_t hidden) {
    GUARD_BEGIN
    *handle = new LayerWitness(seq_len, dim, hidden);
    GUARD_END
}
int grape_host_layer_witness_generate(void* handle, const int32_t* d_x, const int32_t* const* w, const int32_t* d_exp,
                                      const int32_t* d_silu, double eps) {
    GUARD_BEGIN
    LayerWitness::Weights ws{w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7], w[8]};
    LayerWitness::Tables tb{d_exp, d_silu};
    ProveTimer timer;
    static_cast<LayerWitness*>(handle)->generate(d_x, ws, tb, eps);
    GUARD_END
}
int grape_host_layer_witness_names(void* handle, char* buf, size_t cap) {
    GUARD_BEGIN
    std::string all;
    for (const auto& n : static_cast<LayerWitness*>(handle)->names()) all += n + "\n";
    if (all.size() + 1 > cap) throw std::length_error("name buffer too small");
    std::memcpy(buf, all.c_str(), all.size() + 1);
    GUARD_END
}
int grape_host_layer_witness_tensor(void* handle, const char* name, const int32_t** d_ptr, size_t* size) {
    GUARD_BEGIN
    const LayerWitness* lw = static_cast<LayerWitness*>(handle);
    *d_ptr = lw->tensor(name);
    *size = lw->tensor_size(name);
    GUARD_END
}
int grape_host_layer_witness_save(void* handle, const char* dir, uint32_t group) {
    GUARD_BEGIN
    static_cast<LayerWitness*>(handle)->save(dir, group);
    GUARD_END
}
int grape_host_layer_witness_free(void* handle) {
    GUARD_BEGIN
    delete static_cast<LayerWitness*>(handle);
    GUARD_END
}
int grape_host_witness_tables(int32_t* exp_out, int32_t* silu_out) {
    GUARD_BEGIN
    if (exp_out) {
        std::vector<int> t = LayerWitness::make_exp_table();
        std::memcpy(exp_out, t.data(), sizeof(int) * t.size());
    }
    if (silu_out) {
        std::vector<int> t = LayerWitness::make_silu_table();
        std::memcpy(silu_out, t.data(), sizeof(int) * t.size());
    }
    GUARD_END
}
double grape_host_to_float16(double x) { return LayerWitness::to_float16(x); }

}  // extern "C"
