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
    grape_free(fr_strided_.d);
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
    // against what every other table of this object holds (the one being replaced gives its bytes back)
    const size_t others = table_bytes_in_use() - (t.d ? grape_g1_wide_table_bytes(t.ngen, t.nw, t.K) : 0);
    if (others + bytes > table_budget_) return false;
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

namespace {
// One C-ABI commitment call takes at most 2^28 scalars (the largest single call that is tested on the
// GPU); longer tensors go through in whole rows, each call writing its own rows of the output.
constexpr size_t kMaxScalarsPerCall = (size_t)1 << 28;
// fn(first_element, elements, first_row) -> status; stops at the first non-zero status
template <class F>
int for_row_chunks(size_t size, uint rowlen, F fn) {
    size_t rows_per_call = kMaxScalarsPerCall / rowlen;
    if (rows_per_call < 1) rows_per_call = 1;
    const size_t rows = size / rowlen;
    for (size_t r0 = 0; r0 < rows; r0 += rows_per_call) {
        const size_t nr = rows - r0 < rows_per_call ? rows - r0 : rows_per_call;
        int rc = fn(r0 * rowlen, nr * rowlen, r0);
        if (rc != GRAPE_OK) return rc;
    }
    return GRAPE_OK;
}
}  // namespace

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
            int rc = for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
                return grape_commit_i32(W(out + r0), tensor + e0, n, rowlen, W(t->d), t->ngen, t->c, t->nw, t->K, nullptr);
            });
            if (rc == GRAPE_OK) return out;
            if (rc != GRAPE_EINVAL) check(rc, "grape_commit_i32");
            int16_ok_ = false;   // a scalar outside int16: use the general tables from now on
        }
    }
    commit_i32_rows(out, tensor, size, rowlen, nullptr);
    return out;
}

// any int32 scalars: five signed 8-bit digits per scalar through a small table, or the reference's
// byte windows when even that table is over budget
void Hyrax::commit_i32_rows(affine_t* out, int* tensor, size_t size, uint rowlen, int* d_flag, void* stream) {
    if (!d_flag) stream = nullptr;                       // a call that waits for its result runs on the default stream
    const affine_t* had = int32_table_.d;
    if (ensure_table(int32_table_, rowlen, 8, 5, 128)) {
        // a table built just now was built on the default stream: another stream may read it only once it is there
        if (stream && int32_table_.d != had) check(grape_stream_sync(nullptr), "sync");
        check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
                  if (d_flag)
                      return grape_commit_i32_nowait(W(out + r0), tensor + e0, n, rowlen, W(int32_table_.d), int32_table_.ngen, 8, 5, 128,
                                                     d_flag, stream);
                  return grape_commit_i32(W(out + r0), tensor + e0, n, rowlen, W(int32_table_.d), int32_table_.ngen, 8, 5, 128, nullptr);
              }),
              "grape_commit_i32");
    } else {
        check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
                  return grape_commit_i32_ref_table(W(out + r0), tensor + e0, n, rowlen, W(g_affine), npoints, stream);
              }),
              "grape_commit_i32_ref_table");
    }
}

affine_t* Hyrax::commit_affine_i32(int* tensor, uint size, uint N, int* d_flag, void* stream) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)(size / rowlen)), "grape_malloc");
    commit_i32_rows(out, tensor, size, rowlen, d_flag, stream);
    return out;
}

size_t Hyrax::table_bytes_in_use() const {
    size_t used = scaled_bytes_;
    for (const WideTable* t : {&int16_table_, &int16x2_table_, &int32_table_, &fr_table_})
        if (t->d) used += grape_g1_wide_table_bytes(t->ngen, t->nw, t->K);
    if (fr_strided_.d) used += grape_g1_wide_table_bytes(fr_strided_.ngen, fr_strided_.nsets, 1u << (fr_strided_.c - 1));
    return used;
}

// A per-window table for full-width scalars (every window has its own set of multiples, so a
// scalar multiple needs additions only and one accumulator per lane): what the scaled table
// B[t] * G_i of a lookup object is built through and what the sparse commitment reads, at one
// addition per window (c = 13: 20 additions from 43 GB for 4096 generators; the widest window whose
// table stays below its cap and inside the budget is taken - the table itself is generated in a
// tenth of a second).  Multi-row commitments do not use it when a strided table exists.
bool Hyrax::ensure_fr_table(uint rowlen, bool build) {
    if (fr_table_.d && fr_table_.ngen >= rowlen) return true;
    if (!build) return false;
    const size_t used = table_bytes_in_use();
    for (uint c = 13; c >= 8; c--) {
        const uint nw = (255 + c - 1) / c, K = 1u << (c - 1);
        const size_t bytes = grape_g1_wide_table_bytes(rowlen, nw, K);
        // wide windows may take 48 GB, narrow ones (which lose to the strided table anyway) 16 GB
        const size_t cap = (size_t)(c >= 12 ? 48 : 16) << 30;
        if (bytes <= cap && used + bytes <= table_budget_) return ensure_table(fr_table_, rowlen, c, nw, K);
    }
    return false;
}

// Full-width scalars cost one addition per c-bit window, so the table that leaves the fewest
// additions per scalar within its share of the budget is built: windows of c bits, every J-th
// window set kept, the J residue sums combined by (J-1)*c doublings per row.  Measured cost per
// scalar, in additions: ceil(255/c) + 0.3 J (each residue recodes the scalar again).  Half of the
// budget at most goes to this table - the rest is for the int16 table and the lookups' scaled
// tables.  4096 generators: c = 16, J = 4, 4 sets, 69 GB, 16 additions (a per-window table of the
// same bytes has c = 14 and 19); 65536 generators: c = 13, J = 10; 262144: c = 11, J = 12, against
// 32 additions plus a doubling chain per row for the reference's byte windows.
bool Hyrax::ensure_strided_table(uint rowlen, bool build) {
    if (fr_strided_.d && fr_strided_.ngen >= rowlen) return true;
    if (!build) return false;
    if (rowlen > npoints) throw std::runtime_error("row longer than the generator set");
    const size_t used = table_bytes_in_use() - (fr_strided_.d ? grape_g1_wide_table_bytes(fr_strided_.ngen, fr_strided_.nsets, 1u << (fr_strided_.c - 1)) : 0);
    size_t cap = table_budget_ / 2;
    if (used + cap > table_budget_) cap = table_budget_ > used ? table_budget_ - used : 0;
    // the cheapest table over `ngen` generators within the cap: cost per scalar, c, J, number of sets
    struct Choice { double cost; uint c, J, nsets; };
    auto choose = [&](uint ngen) {
        Choice best{30.0, 0, 0, 0};       // a table that does not beat 30 additions per scalar is not worth building
        for (uint c = 8; c <= 17; c++) {
            const uint nw = (255 + c - 1) / c;
            for (uint J = 1; J <= nw; J++) {
                const uint nsets = (nw + J - 1) / J;
                if ((nsets - 1) * J * c >= 256) continue;
                const size_t bytes = grape_g1_wide_table_bytes(ngen, nsets, 1u << (c - 1));
                if (bytes > cap) continue;
                const double cost = nw + 0.3 * J + (double)bytes / 1e12;
                if (cost < best.cost) best = Choice{cost, c, J, nsets};
            }
        }
        return best;
    };
    // one table over every generator serves all row lengths; it is preferred to a table over the
    // first `rowlen` generators (which a longer row would have to replace, at half a second per
    // build) unless that costs over a quarter more additions per scalar
    Choice pick = choose(rowlen);
    uint ngen = rowlen;
    if (npoints > rowlen) {
        const Choice all = choose(npoints);
        if (all.c != 0 && (pick.c == 0 || all.cost <= 1.25 * pick.cost)) {
            pick = all;
            ngen = npoints;
        }
    }
    const uint bc = pick.c, bj = pick.J, bs = pick.nsets;
    if (bc == 0) return false;
    grape_free(fr_strided_.d);
    fr_strided_ = StridedTable();
    check(grape_malloc((void**)&fr_strided_.d, grape_g1_wide_table_bytes(ngen, bs, 1u << (bc - 1))), "grape_malloc");
    check(grape_g1_strided_table_gen(W(fr_strided_.d), W(g_affine + npoints), ngen, bc, bj, bs, nullptr), "grape_g1_strided_table_gen");
    fr_strided_.ngen = ngen;
    fr_strided_.c = bc;
    fr_strided_.J = bj;
    fr_strided_.nsets = bs;
    return true;
}

bool Hyrax::commit_fr_rows(affine_t* out, fr_t* scalars, size_t size, uint rowlen, bool may_build, void* stream, int* d_flag) {
    // one row only (an opening's blinding row): a table that is already there is used, none is built for it,
    // and the per-window table is preferred - its 20 additions per scalar are nothing for one row, while the
    // strided table's (J-1)*c doublings per row are a chain of half a millisecond on one lane
    const bool single = size == rowlen;
    if (single && ensure_fr_table(rowlen, false)) {
        const WideTable& t = fr_table_;
        if (d_flag) {
            check(grape_commit_fr_nowait(W(out), W(scalars), size, rowlen, W(t.d), t.ngen, t.c, t.nw, t.K, d_flag, stream), "grape_commit_fr_nowait");
            return true;
        }
        check(grape_commit_fr(W(out), W(scalars), size, rowlen, W(t.d), t.ngen, t.c, t.nw, t.K, stream), "grape_commit_fr");
    } else if (ensure_strided_table(rowlen, may_build)) {
        const StridedTable& t = fr_strided_;
        check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
                  return grape_commit_fr_strided(W(out + r0), W(scalars + e0), n, rowlen, W(t.d), t.ngen, t.c, t.J, t.nsets, stream);
              }),
              "grape_commit_fr_strided");
    } else if (ensure_fr_table(rowlen, false)) {
        const WideTable& t = fr_table_;
        check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
                  return grape_commit_fr(W(out + r0), W(scalars + e0), n, rowlen, W(t.d), t.ngen, t.c, t.nw, t.K, stream);
              }),
              "grape_commit_fr");
    } else {
        check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
                  return grape_commit_fr_ref_table(W(out + r0), W(scalars + e0), n, rowlen, W(g_affine), npoints, stream);
              }),
              "grape_commit_fr_ref_table");
    }
    return false;
}

affine_t* Hyrax::commit_affine(FrTensor& tensor, uint size, uint N) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    const uint rows = size / rowlen;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    commit_fr_rows(out, tensor.gpu_data, size, rowlen, rows > 1);
    return out;
}

bool Hyrax::prepare_scaled_tables(uint ncols) { return ensure_fr_table(ncols); }

affine_t* Hyrax::build_scaled_table(const FrTensor& scalars, uint ncols) {
    if (ncols > npoints) throw std::runtime_error("row longer than the generator set");
    size_t bytes = grape_g1_wide_table_bytes(ncols, 1, scalars.size);   // one entry per (scalar, column)
    if (table_bytes_in_use() + bytes > table_budget_) return nullptr;      // before the per-window table is built for nothing
    if (!ensure_fr_table(ncols)) return nullptr;
    if (table_bytes_in_use() + bytes > table_budget_) return nullptr;
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

bool Hyrax::owns_scaled_table(const affine_t* table) const {
    auto it = scaled_registry().find(table);
    return it != scaled_registry().end() && it->second.first == this;
}

affine_t* Hyrax::commit_indexed_affine(int* idx_plus1, uint size, uint N, affine_t* scaled_table, uint ncols, uint len, int* d_flag) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    if (rowlen > ncols) throw std::runtime_error("row longer than the scaled table");
    const uint rows = size / rowlen;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    // one unsigned "digit" idx+1 in [1, len]: radix 2^(log2(len)+1) keeps it below the sign threshold
    const uint c = Log2(len) + 1 < 2 ? 2 : Log2(len) + 1;
    check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
              if (d_flag) return grape_commit_i32_nowait(W(out + r0), idx_plus1 + e0, n, rowlen, W(scaled_table), ncols, c, 1, len, d_flag, nullptr);
              return grape_commit_i32(W(out + r0), idx_plus1 + e0, n, rowlen, W(scaled_table), ncols, c, 1, len, nullptr);
          }),
          "grape_commit_i32 (indexed)");
    return out;
}

affine_t* Hyrax::commit_sparse_affine(FrTensor& tensor, int* skip, uint size, uint N) {
    check_shape(size, N);
    const uint rowlen = N * com_scale;
    if (!ensure_fr_table(rowlen, false)) return nullptr;
    const WideTable& t = fr_table_;
    const uint rows = size / rowlen;
    affine_t* out = nullptr;
    check(grape_malloc((void**)&out, sizeof(affine_t) * (size_t)rows), "grape_malloc");
    check(for_row_chunks(size, rowlen, [&](size_t e0, size_t n, size_t r0) {
              return grape_commit_fr_sparse(W(out + r0), W(tensor.gpu_data + e0), skip + e0, n, rowlen, W(t.d), t.ngen, t.c, t.nw, t.K, nullptr);
          }),
          "grape_commit_fr_sparse");
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
    return open_impl(&tensor, nullptr, eval_point_, c, size, N);
}
Hyrax_proof Hyrax::open(const int* device_int_data, const std::vector<Fr> eval_point_, Fr c, uint size, uint N) {
    return open_impl(nullptr, device_int_data, eval_point_, c, size, N);
}
// tensor_in, or the integer tensor `ints` read as FrTensor::get_data would embed it: its fold over the rows then reads the
// integers directly (4 bytes per element where embedding and folding move 68)
Hyrax_proof Hyrax::open_impl(FrTensor* tensor_in, const int* ints, const std::vector<Fr>& eval_point_, Fr c, uint size, uint N) {
    if (size / N / com_scale < layer_num) throw std::runtime_error("Size too small: size < N * com_scale * layer_num");
    uint pad_N = 1u << Log2(N);
    uint new_N = pad_N * com_scale;
    assert(eval_point_.size() == Log2(size));
    last_open_point_ = eval_point_;
    fr_t* eval_point = grape_host::upload(eval_point_);

    std::vector<Fr> host_d(new_N);
    for (uint i = 0; i < new_N; i++) host_d[i] = Fr::random_element();
    FrTensor d = FrTensor::from_host(host_d);

    // commitment of d: one row of new_N full-width scalars (single_commit, src/Hyrax.cu:176-185).  A short
    // accumulation and then a latency chain (the row's reduction), so it runs on a stream of its own beside the folds
    // of the tensor below; nothing below writes to d.
    static grape_stream_t open_stream = nullptr;      // lives as long as the process
    static void* d_uploaded = nullptr;
    if (!open_stream) {
        check(grape_stream_create(&open_stream), "grape_stream_create");
        check(grape_event_create(&d_uploaded), "grape_event_create");
    }
    check(grape_event_record(d_uploaded, nullptr), "grape_event_record");        // a short d travels as a queued launch
    check(grape_stream_wait_event(open_stream, d_uploaded), "grape_stream_wait_event");
    // (the point and, behind it, the digit-range flag of a commitment queued without waiting)
    affine_t* com_d_dev = nullptr;
    check(grape_malloc((void**)&com_d_dev, sizeof(affine_t) + 16), "grape_malloc");
    int* d_flag = reinterpret_cast<int*>(com_d_dev + 1);
    check(grape_memset_zero(d_flag, sizeof(int), open_stream), "grape_memset_zero");
    const bool flag_used = commit_fr_rows(com_d_dev, d.gpu_data, new_N, new_N, false, open_stream, d_flag);

    FrTensor x(new_N);
    std::unique_ptr<FrTensor> rows_of_ints;
    if (ints) {
        rows_of_ints.reset(new FrTensor(FrTensor::folded_from_ints(ints, size, eval_point, (size / layer_num) / (N * com_scale),
                                                                    Log2(N * com_scale), N * com_scale)));
    } else {
        tensor_in->partial_eval(size, eval_point, (size / layer_num) / (N * com_scale), Log2(N * com_scale), N * com_scale);
    }
    FrTensor& tensor = ints ? *rows_of_ints : *tensor_in;
    tensor.partial_eval((N * com_scale) * layer_num, eval_point, layer_num, Log2(size / layer_num), N * com_scale);
    x = tensor;
    if (pad_N != N) x.pad(tensor, N, pad_N, new_N, Fr::zero());

    tensor.partial_eval(new_N, eval_point, new_N, 0, 1);
    Fr result = grape_host::download(tensor.gpu_data);

    FrTensor z(new_N);
    z = x;
    z *= c;
    z += d;

    FrTensor d_fold(d);                         // folded in place: a copy, the commitment may still be reading d
    d_fold.partial_eval(d_fold.size, eval_point, new_N, 0, 1);
    Fr sum_ad = grape_host::download(d_fold.gpu_data);
    if (!G_multiples_) G_multiples_.reset(new G1FixedBase(G));
    bn128 commit_ad = G_multiples_->mul(sum_ad);

    struct { affine_t p; int flag[4]; } com_d_host;
    static_assert(sizeof(com_d_host) == sizeof(affine_t) + 16, "point and flag travel together");
    check(grape_memcpy_d2h(&com_d_host, com_d_dev, sizeof(com_d_host), open_stream), "d2h");     // waits for the commitment
    if (flag_used && com_d_host.flag[0]) {
        grape_free(com_d_dev);
        grape_free(eval_point);
        throw std::runtime_error("Hyrax::open: a blinding scalar does not fit the table's digit range");
    }
    const affine_t& host_com_d = com_d_host.p;
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
    commit_fr_rows(com_z_dev, z.gpu_data, new_N, new_N, false);
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
