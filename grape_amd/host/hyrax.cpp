#include "hyrax.hpp"
#include <cstdlib>
#include <cassert>
#include <map>
#include <utility>
#include "../../include/grape_hip.h"

using grape_host::check;
static inline uint32_t* W(void* p) { return reinterpret_cast<uint32_t*>(p); }
static inline const uint32_t* W(const void* p) { return reinterpret_cast<const uint32_t*>(p); }

Hyrax_proof::Hyrax_proof(Fr result_, size_t z_len, bn128 commit_d_, bn128 commit_ad_)
    : z_size(z_len), result(result_), commit_d(commit_d_), commit_ad(commit_ad_) {
    z = new Fr[z_size];
}
Hyrax_proof::~Hyrax_proof() { delete[] z; }
Hyrax_proof::Hyrax_proof(const Hyrax_proof& o) : z_size(o.z_size), result(o.result), commit_d(o.commit_d), commit_ad(o.commit_ad) {
    z = new Fr[z_size];
    for (size_t i = 0; i < z_size; i++) z[i] = o.z[i];
}
Hyrax_proof& Hyrax_proof::operator=(const Hyrax_proof& o) {
    if (this != &o) {
        delete[] z;
        z_size = o.z_size;
        result = o.result;
        commit_d = o.commit_d;
        commit_ad = o.commit_ad;
        z = new Fr[z_size];
        for (size_t i = 0; i < z_size; i++) z[i] = o.z[i];
    }
    return *this;
}

Hyrax::Hyrax(uint layer_num_, uint npoints_, affine_t* g, bn128& G_, uint com_scale_)
    : com_scale(com_scale_), layer_num(layer_num_), npoints(npoints_ * com_scale_), G(G_), g_affine(g) {
    grape_host::ensure_init();
    // GRAPE_TABLE_BUDGET_GIB overrides the default budget of the fixed-base tables
    if (const char* e = std::getenv("GRAPE_TABLE_BUDGET_GIB")) {
        char* end = nullptr;
        unsigned long long gib = std::strtoull(e, &end, 10);
        if (end != e) table_budget_ = (size_t)gib << 30;
    }
}
// scaled tables handed out: table -> (the Hyrax object whose budget holds it, bytes).  Never
// destroyed: lookup objects with static lifetime release their tables while the process exits.
static std::map<const void*, std::pair<Hyrax*, size_t>>& scaled_registry() {
    static auto* r = new std::map<const void*, std::pair<Hyrax*, size_t>>();
    return *r;
}

Hyrax::~Hyrax() {
    for (auto& e : scaled_registry())
        if (e.second.first == this) e.second.first = nullptr;
    grape_free(int16_table_.d);
    grape_free(int16x2_table_.d);
    grape_free(int32_table_.d);
    grape_free(fr_table_.d);
}

// src/Hyrax.cu:314-315 / :337-338
void Hyrax::check_shape(uint size, uint N) const {
    if (size / N / com_scale < layer_num) throw std::runtime_error("Size too small: size < N * com_scale * layer_num");
    if (N != (1u << Log2(N))) throw std::runtime_error("N must be a power of 2");
}

// Builds (once) the wide table over the first `rowlen` generators; false when it exceeds the budget.
bool Hyrax::ensure_table(WideTable& t, uint rowlen, uint c, uint nw, uint K) {
    if (t.d && t.ngen >= rowlen && t.c == c && t.nw == nw) return true;
    size_t bytes = grape_g1_wide_table_bytes(rowlen, nw, K);
    if (bytes > table_budget_) return false;
    if (rowlen > npoints) throw std::runtime_error("row longer than the generator set");
    grape_free(t.d);
    t = WideTable();
    check(grape_malloc((void**)&t.d, bytes), "grape_malloc");
    // generators are row k = 1 of the reference-format table
    check(grape_g1_wide_table_gen(W(t.d), W(g_affine + npoints), rowlen, c, nw, K, nullptr), "grape_g1_wide_table_gen");
    t.ngen = rowlen;
    t.c = c;
    t.nw = nw;
    t.K = K;
    return true;
}

affine_t* Hyrax::commit_affine(int* tensor, uint size, uint N) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    const uint rows = size / rowlen;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    // small-scalar fast paths: one signed 16-bit digit per scalar (one mixed addition per element)
    // when that table fits the budget, else two signed 9-bit digits (two additions; 17 GB instead of
    // 275 GB for the 262144-column rows of the reference's com_scale = 16 shapes)
    if (int16_ok_) {
        WideTable* t = nullptr;
        if (ensure_table(int16_table_, rowlen, 16, 1, 32768)) t = &int16_table_;
        else if (ensure_table(int16x2_table_, rowlen, 9, 2, 256)) t = &int16x2_table_;
        if (t) {
            int rc = grape_commit_i32(W(out), tensor, size, rowlen, W(t->d), t->ngen, t->c, t->nw, t->K, nullptr);
            if (rc == GRAPE_OK) return out;
            if (rc != GRAPE_EINVAL) check(rc, "grape_commit_i32");
            int16_ok_ = false;   // a scalar outside int16: use the general tables from now on
        }
    }
    if (ensure_table(int32_table_, rowlen, 8, 5, 128)) {
        check(grape_commit_i32(W(out), tensor, size, rowlen, W(int32_table_.d), int32_table_.ngen, 8, 5, 128, nullptr), "grape_commit_i32");
    } else {
        check(grape_commit_i32_ref_table(W(out), tensor, size, rowlen, W(g_affine), npoints, nullptr), "grape_commit_i32_ref_table");
    }
    return out;
}

// Full-width scalars cost ceil(256/c) additions each, so the widest radix whose table fits the
// budget is used (from c = 10 up).  For 4096 generators: c = 14 is 19 additions per element (82 GB, what the
// default budget allows next to the other tables), c = 13 is 20 (43 GB), c = 15 is 17.5 on average
// (155 GB; measured no faster than c = 14, its gathers miss more), against 32 plus a doubling
// chain for the reference's byte windows.
bool Hyrax::ensure_fr_table(uint rowlen, bool build) {
    if (fr_table_.d && fr_table_.ngen >= rowlen) return true;
    if (!build) return false;
    size_t used = 0;
    if (int16_table_.d) used += grape_g1_wide_table_bytes(int16_table_.ngen, int16_table_.nw, int16_table_.K);
    if (int16x2_table_.d) used += grape_g1_wide_table_bytes(int16x2_table_.ngen, int16x2_table_.nw, int16x2_table_.K);
    if (int32_table_.d) used += grape_g1_wide_table_bytes(int32_table_.ngen, int32_table_.nw, int32_table_.K);
    // ceil(255 / c) windows: the kernel takes a scalar of the upper half as -(r - k), so magnitudes
    // stay below 2^254 and the top signed digit never carries out (c = 15: 17 windows, not 18).
    // Below c = 10 a wide table (32 additions per element at c = 8) saves nothing over the
    // reference-format table, whose path needs no build, so very long rows (the reference's
    // com_scale = 16 shapes: 65536 to 262144 columns) stay on that path.
    for (uint c = 15; c >= 10; c--) {
        uint nw = (255 + c - 1) / c, K = 1u << (c - 1);
        if (used + grape_g1_wide_table_bytes(rowlen, nw, K) <= table_budget_) return ensure_table(fr_table_, rowlen, c, nw, K);
    }
    return false;
}

affine_t* Hyrax::commit_affine(FrTensor& tensor, uint size, uint N) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    const uint rows = size / rowlen;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    if (ensure_fr_table(rowlen)) {
        check(grape_commit_fr(W(out), W(tensor.gpu_data), size, rowlen, W(fr_table_.d), fr_table_.ngen, fr_table_.c, fr_table_.nw,
                              fr_table_.K, nullptr),
              "grape_commit_fr");
    } else {
        check(grape_commit_fr_ref_table(W(out), W(tensor.gpu_data), size, rowlen, W(g_affine), npoints, nullptr), "grape_commit_fr_ref_table");
    }
    return out;
}

affine_t* Hyrax::build_scaled_table(const FrTensor& scalars, uint ncols) {
    if (ncols > npoints) throw std::runtime_error("row longer than the generator set");
    if (!ensure_fr_table(ncols)) return nullptr;
    size_t bytes = grape_g1_wide_table_bytes(ncols, 1, scalars.size);   // one entry per (scalar, column)
    size_t used = scaled_bytes_ + grape_g1_wide_table_bytes(fr_table_.ngen, fr_table_.nw, fr_table_.K);
    if (int16_table_.d) used += grape_g1_wide_table_bytes(int16_table_.ngen, int16_table_.nw, int16_table_.K);
    if (int16x2_table_.d) used += grape_g1_wide_table_bytes(int16x2_table_.ngen, int16x2_table_.nw, int16x2_table_.K);
    if (int32_table_.d) used += grape_g1_wide_table_bytes(int32_table_.ngen, int32_table_.nw, int32_table_.K);
    if (used + bytes > table_budget_) return nullptr;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, bytes), "grape_malloc");
    check(grape_g1_scaled_table_gen(W(out), W(scalars.gpu_data), scalars.size, ncols, W(fr_table_.d), fr_table_.ngen, fr_table_.c,
                                    fr_table_.nw, fr_table_.K, nullptr),
          "grape_g1_scaled_table_gen");
    scaled_bytes_ += bytes;
    scaled_registry()[out] = std::make_pair(this, bytes);
    return out;
}

void Hyrax::release_scaled_table(affine_t* table) {
    if (!table) return;
    auto it = scaled_registry().find(table);
    if (it != scaled_registry().end()) {
        if (it->second.first) it->second.first->scaled_bytes_ -= it->second.second;
        scaled_registry().erase(it);
    }
    grape_free(table);
}

affine_t* Hyrax::commit_indexed_affine(int* idx_plus1, uint size, uint N, affine_t* scaled_table, uint ncols, uint len) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    if (rowlen > ncols) throw std::runtime_error("row longer than the scaled table");
    const uint rows = size / rowlen;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    // one unsigned "digit" idx+1 in [1, len]: radix 2^(log2(len)+1) keeps it below the sign threshold
    const uint c = Log2(len) + 1;
    check(grape_commit_i32(W(out), idx_plus1, size, rowlen, W(scaled_table), ncols, c, 1, len, nullptr), "grape_commit_i32 (indexed)");
    return out;
}

void single_commit(fr_t* d, affine_t* g, jacob_t* com, uint N, uint npoints) {
    grape_host::ensure_init();
    affine_t* a = nullptr;
    check(grape_malloc((void**)&a, sizeof(affine_t)), "grape_malloc");
    check(grape_commit_fr_ref_table(W(a), W(d), N, N, W(g), npoints, nullptr), "grape_commit_fr_ref_table");
    check(grape_g1_affine_to_jacobian(W(com), W(a), 1, nullptr), "grape_g1_affine_to_jacobian");
    check(grape_stream_sync(nullptr), "sync");
    grape_free(a);
}

static jacob_t* to_jacobian(affine_t* aff, uint rows) {
    jacob_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(jacob_t) * (size_t)rows), "grape_malloc");
    check(grape_g1_affine_to_jacobian(W(out), W(aff), rows, nullptr), "grape_g1_affine_to_jacobian");
    check(grape_stream_sync(nullptr), "sync");
    grape_free(aff);
    return out;
}
jacob_t* Hyrax::commit(int* tensor, uint size, uint N) {
    affine_t* a = commit_affine(tensor, size, N);
    return to_jacobian(a, size / (N * com_scale));
}
jacob_t* Hyrax::commit(FrTensor& tensor, uint size, uint N) {
    affine_t* a = commit_affine(tensor, size, N);
    return to_jacobian(a, size / (N * com_scale));
}

// Hyrax::open, src/Hyrax.cu:237-305: fold the tensor down to one row x of length new_N at the
// outer variables of the point, blind it as z = c*x + d with a random row d, commit d, and send
// <a,d>*G where a is the eq-vector of the inner variables.
Hyrax_proof Hyrax::open(FrTensor& tensor, const std::vector<Fr> eval_point_, Fr c, uint size, uint N) {
    if (size / N / com_scale < layer_num) throw std::runtime_error("Size too small: size < N * com_scale * layer_num");
    uint pad_N = 1u << Log2(N);
    uint new_N = pad_N * com_scale;
    assert(eval_point_.size() == Log2(size));
    last_open_point_ = eval_point_;
    fr_t* eval_point = grape_host::upload(eval_point_);

    std::vector<Fr> host_d(new_N);
    for (uint i = 0; i < new_N; i++) host_d[i] = Fr::random_element();
    FrTensor d = FrTensor::from_host(host_d);

    // commitment of d: one row of new_N full-width scalars (single_commit, src/Hyrax.cu:176-185)
    affine_t* com_d_dev = nullptr;
    check(grape_malloc((void**)&com_d_dev, sizeof(affine_t)), "grape_malloc");
    // one row only: a table that is already there is used, none is built for it
    if (ensure_fr_table(new_N, false)) {
        check(grape_commit_fr(W(com_d_dev), W(d.gpu_data), new_N, new_N, W(fr_table_.d), fr_table_.ngen, fr_table_.c, fr_table_.nw,
                              fr_table_.K, nullptr),
              "grape_commit_fr");
    } else {
        check(grape_commit_fr_ref_table(W(com_d_dev), W(d.gpu_data), new_N, new_N, W(g_affine), npoints, nullptr), "grape_commit_fr_ref_table");
    }

    FrTensor x(new_N);
    tensor.partial_eval(size, eval_point, (size / layer_num) / (N * com_scale), Log2(N * com_scale), N * com_scale);
    tensor.partial_eval((N * com_scale) * layer_num, eval_point, layer_num, Log2(size / layer_num), N * com_scale);
    x = tensor;
    if (pad_N != N) x.pad(tensor, N, pad_N, new_N, Fr::zero());

    tensor.partial_eval(new_N, eval_point, new_N, 0, 1);
    Fr result = grape_host::download(tensor.gpu_data);

    FrTensor z(new_N);
    z = x;
    z *= c;
    z += d;

    d.partial_eval(d.size, eval_point, new_N, 0, 1);
    Fr sum_ad = grape_host::download(d.gpu_data);
    bn128 commit_ad = sum_ad * G;

    affine_t host_com_d;
    check(grape_memcpy_d2h(&host_com_d, com_d_dev, sizeof(affine_t), nullptr), "d2h");
    Hyrax_proof proof(result, new_N, bn128(host_com_d), commit_ad);
    check(grape_memcpy_d2h(proof.z, z.gpu_data, sizeof(fr_t) * (size_t)new_N, nullptr), "d2h");
    grape_free(com_d_dev);
    grape_free(eval_point);
    return proof;
}

// The driver-side verification of test/HyraxTest.cu:87-125: fold the row commitments at the outer
// variables, then check  c*C + com_d == com(z)  and  (c*result)*G + com_ad == <a,z>*G.
bool Hyrax::verify(Hyrax_proof& proof, jacob_t* commitment, const std::vector<Fr>& eval_point, Fr c, uint size, uint N) {
    const uint rowlen = N * com_scale;
    const uint rows = size / rowlen;
    const uint new_N = (uint)proof.z_size;
    std::vector<jacob_t> raw(rows);
    check(grape_memcpy_d2h(raw.data(), commitment, sizeof(jacob_t) * (size_t)rows, nullptr), "d2h");
    std::vector<bn128> coms(rows);
    for (uint i = 0; i < rows; i++) coms[i] = bn128(raw[i]);
    const uint inner = Log2(rowlen);
    bn128 C = host_partial_me<bn128>(coms.data(), rows, eval_point.begin() + inner, eval_point.end());
    // com(z) on the device
    std::vector<Fr> zv(proof.z, proof.z + new_N);
    FrTensor z = FrTensor::from_host(zv);
    affine_t* com_z_dev = nullptr;
    check(grape_malloc((void**)&com_z_dev, sizeof(affine_t)), "grape_malloc");
    if (ensure_fr_table(new_N)) {
        check(grape_commit_fr(W(com_z_dev), W(z.gpu_data), new_N, new_N, W(fr_table_.d), fr_table_.ngen, fr_table_.c, fr_table_.nw,
                              fr_table_.K, nullptr),
              "grape_commit_fr");
    } else {
        check(grape_commit_fr_ref_table(W(com_z_dev), W(z.gpu_data), new_N, new_N, W(g_affine), npoints, nullptr), "grape_commit_fr_ref_table");
    }
    affine_t com_z;
    check(grape_memcpy_d2h(&com_z, com_z_dev, sizeof(affine_t), nullptr), "d2h");
    grape_free(com_z_dev);
    if (!(c * C + proof.commit_d == bn128(com_z))) return false;
    std::vector<Fr> inner_point(eval_point.begin(), eval_point.begin() + inner);
    Fr az = z(inner_point);
    return (c * proof.result) * G + proof.commit_ad == az * G;
}

void Hyrax::verify(Hyrax_proof& proof, jacob_t* commitment, Fr c, uint size, uint N) {
    if (last_open_point_.size() != Log2(size)) throw std::runtime_error("Hyrax::verify: no opening of this size was made by this object");
    if (!verify(proof, commitment, last_open_point_, c, size, N)) throw std::runtime_error("Hyrax::verify: the opening does not match the commitment");
}
