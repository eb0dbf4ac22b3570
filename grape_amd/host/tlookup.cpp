#include "tlookup.hpp"
#include <cassert>
#include <chrono>
#include <cstdio>
#include <functional>
#include "../../include/grape_hip.h"

using grape_host::check;
static inline uint32_t* W(fr_t* p) { return reinterpret_cast<uint32_t*>(p); }
static inline const uint32_t* W(const fr_t* p) { return reinterpret_cast<const uint32_t*>(p); }

// src/tlookup.cu:247: beta is the table size, alpha is random
tLookup::tLookup(const uint size) : alpha(Fr::random_element()), beta(Fr((long)size)), T(size), B(size), m(size) {}
tLookup::~tLookup() {
    grape_free(com_A);
    grape_free(com_m);
    Hyrax::release_scaled_table(scaled_table_);
    Hyrax::release_scaled_table(hot_table_);
    grape_free(hot_slot1_);
    grape_free(d_idx_);
}

void tLookup::make_index(const FrTensor& vals, int low_) {
    drop_index();
    check(grape_malloc((void**)&d_idx_, sizeof(int) * (size_t)(vals.size ? vals.size : 1)), "grape_malloc");
    check(grape_tlookup_index(d_idx_, W(vals.gpu_data), vals.size, low_, T.size, nullptr), "grape_tlookup_index");
}
void tLookup::make_index_and_A(const FrTensor& key, int low_, FrTensor& A, const FrTensor* cmp, const FrTensor* cmp_table, bool write_A) {
    drop_index();
    a_ready_ = false;
    a_deferred_ = false;
    check(grape_malloc((void**)&d_idx_, sizeof(int) * (size_t)(key.size ? key.size : 1)), "grape_malloc");
    // The pass over the witness is queued first and its count of unmatched elements read last: in between the
    // host queues the proof's weights (a dozen small launches on the second stream) while the chip is busy.
    uint32_t* d_count = nullptr;
    check(grape_malloc((void**)&d_count, sizeof(uint32_t)), "grape_malloc");
    uint32_t mismatches = 1;
    try {
        check(grape_tlookup_index_inverse_nowait(d_idx_, write_A ? W(A.gpu_data) : nullptr, W(key.gpu_data), key.size, low_, T.size, W(B.gpu_data),
                                                 cmp ? W(cmp->gpu_data) : nullptr, cmp_table ? W(cmp_table->gpu_data) : nullptr, d_count,
                                                 nullptr),
              "grape_tlookup_index_inverse_nowait");
        start_weights(1u << Log2(key.size));
        check(grape_memcpy_d2h(&mismatches, d_count, sizeof(uint32_t), nullptr), "grape_memcpy_d2h");
    } catch (...) {
        grape_stream_sync(nullptr);
        grape_free(d_count);
        throw;
    }
    grape_free(d_count);
    a_ready_ = write_A && mismatches == 0;
    a_deferred_ = !write_A && mismatches == 0;
}
void tLookup::make_index_and_A_from_ints(const int* key, const int* cmp, uint n, int low_, FrTensor& S, FrTensor& A, const int* cmp_table,
                                         const Fr* r, bool write_A) {
    drop_index();
    a_ready_ = false;
    a_deferred_ = false;
    check(grape_malloc((void**)&d_idx_, sizeof(int) * (size_t)(n ? n : 1)), "grape_malloc");
    uint32_t* d_count = nullptr;
    check(grape_malloc((void**)&d_count, sizeof(uint32_t)), "grape_malloc");
    uint32_t mismatches = 1;
    try {
        check(grape_tlookup_index_embed_i32_nowait(d_idx_, write_A ? W(A.gpu_data) : nullptr, W(S.gpu_data), key, cmp, n, low_, T.size,
                                                   W(B.gpu_data), cmp_table, r ? W(grape_host::device_scalar(*r)) : nullptr, d_count, nullptr),
              "grape_tlookup_index_embed_i32_nowait");
        S.set_size(n);
        start_weights(1u << Log2(n));
        check(grape_memcpy_d2h(&mismatches, d_count, sizeof(uint32_t), nullptr), "grape_memcpy_d2h");
    } catch (...) {
        grape_stream_sync(nullptr);
        grape_free(d_count);
        throw;
    }
    grape_free(d_count);
    a_ready_ = write_A && mismatches == 0;
    a_deferred_ = !write_A && mismatches == 0;
}
void tLookup::pad_index(uint N, uint pad_N, uint pad_size, int fill) {
    if (!d_idx_ || N == pad_N) return;
    int* padded = nullptr;
    check(grape_malloc((void**)&padded, sizeof(int) * (size_t)pad_size), "grape_malloc");
    check(grape_i32_pad_fill(padded, d_idx_, N, pad_N, pad_size, fill, nullptr), "grape_i32_pad_fill");
    grape_free(d_idx_);                       // grape_free hands a block out again only after the work queued so far
    d_idx_ = padded;
}
void tLookup::drop_index() {
    if (d_idx_ || d_hist_) {
        grape_free(d_idx_);
        grape_free(d_hist_);
        d_idx_ = nullptr;
        d_hist_ = nullptr;
    }
}
// multiplicities from the indices (get_histogram_kernel, src/tlookup.cu:5-14, with the padding
// rule of :276-281)
void tLookup::index_to_m(uint witness_size, int low_, void* stream) {
    m_pending_ = false;
    uint32_t* hist = nullptr;
    check(grape_malloc((void**)&hist, sizeof(uint32_t) * (size_t)m.size), "grape_malloc");
    check(grape_memset_zero(hist, sizeof(uint32_t) * (size_t)m.size, stream), "grape_memset_zero");
    check(grape_tlookup_hist_index(hist, d_idx_, witness_size, m.size, stream), "grape_tlookup_hist_index");
    if (witness_size != (1u << Log2(witness_size))) {
        uint32_t zero_count = 0;
        check(grape_memcpy_d2h(&zero_count, hist + (-low_), sizeof(uint32_t), stream), "d2h");
        zero_count += (1u << Log2(witness_size)) - witness_size;
        check(grape_memcpy_h2d(hist + (-low_), &zero_count, sizeof(uint32_t), stream), "h2d");
    }
    check(grape_fr_from_u32(W(m.gpu_data), hist, m.size, stream), "grape_fr_from_u32");
    grape_free(d_hist_);
    d_hist_ = hist;                           // kept for the proof in flight: the commitment of A picks its table entries by count
}

// com(A) through the entries that occur often.  A[i] = B[index_i]; an entry t that occurs n_t times
// costs n_t full-width scalars (16 to 20 additions each) on the plain path, or one row B[t]*G_i of
// the scaled table (rowlen entries at 20 additions and a normalisation each, built for this proof
// only) plus n_t single additions.  So an entry is worth a row when n_t exceeds rowlen by a factor
// somewhat above one; 1.8 is taken (the proof's time is flat from 1.2 to 2.2), and with the
// activations of a transformer layer nearly all elements sit on such entries.  Elements of the
// other entries keep their scalars and are committed on the plain path; the two sums are added.
// Returns false (nothing committed) when no entry qualifies or the table does not fit.
void tLookup::drop_hot_rows() {
    Hyrax::release_scaled_table(hot_table_);
    grape_free(hot_slot1_);
    hot_table_ = nullptr;
    hot_slot1_ = nullptr;
    hot_rows_ = hot_cols_ = 0;
    hot_for_ = nullptr;
}

bool tLookup::commit_A_by_occupancy(FrTensor& A, uint D, uint msm_size, Hyrax& hyrax) {
    const uint N = T.size;
    const uint rowlen = msm_size * hyrax.com_scale;
    const uint rows = D / rowlen;
    const uint min_count = hot_min_count_ ? hot_min_count_ : (uint)(1.8 * rowlen) + 1;
    hot_reused_ = false;
    uint64_t cold = 0;
    // rows kept from an earlier proof: used again when the elements they leave out (20 additions
    // each instead of one) cost less than building rows anew (rowlen entries of 20 additions and a
    // normalisation per row)
    if (hot_table_ && (hot_for_ != &hyrax || hot_cols_ != rowlen || !hyrax.owns_scaled_table(hot_table_))) drop_hot_rows();
    if (hot_table_ && hot_min_count_ == 0) {
        check(grape_tlookup_hot_coverage(d_hist_, N, hot_slot1_, &cold, nullptr), "grape_tlookup_hot_coverage");
        if ((double)cold * 19.0 <= (double)hot_rows_ * rowlen * 23.0) hot_reused_ = true;
    }
    if (!hot_reused_) {
        drop_hot_rows();
        const size_t row_bytes = grape_g1_wide_table_bytes(rowlen, 1, 1);
        // the per-window table the rows are built through comes first: it takes its share of the budget
        if (!hyrax.prepare_scaled_tables(rowlen)) return false;
        size_t max_hot = hyrax.table_bytes_free() / row_bytes;
        if (max_hot > N) max_hot = N;
        if (max_hot == 0) return false;
        uint32_t* d_list = nullptr;
        try {
            check(grape_malloc((void**)&hot_slot1_, sizeof(int) * (size_t)N), "grape_malloc");
            check(grape_malloc((void**)&d_list, sizeof(uint32_t) * (size_t)N), "grape_malloc");
            uint64_t info[2] = {0, 0};
            check(grape_tlookup_hot_select(d_hist_, N, min_count, (uint32_t)max_hot, hot_slot1_, d_list, info, nullptr), "grape_tlookup_hot_select");
            const uint n_hot = (uint)info[0];
            cold = info[1];
            if (n_hot != 0) {
                FrTensor Bhot(n_hot);
                check(grape_fr_gather(W(Bhot.gpu_data), W(B.gpu_data), d_list, n_hot, nullptr), "grape_fr_gather");
                hot_table_ = hyrax.build_scaled_table(Bhot, rowlen);
            }
            hot_rows_ = n_hot;
            hot_cols_ = rowlen;
            hot_for_ = &hyrax;
        } catch (...) {
            grape_stream_sync(nullptr);
            grape_free(d_list);
            drop_hot_rows();
            throw;
        }
        grape_free(d_list);
        if (!hot_table_) {
            drop_hot_rows();
            return false;
        }
    }
    int* d_hot = nullptr;
    affine_t* com_cold = nullptr;
    try {
        check(grape_malloc((void**)&d_hot, sizeof(int) * (size_t)D), "grape_malloc");
        check(grape_tlookup_hot_index(d_hot, d_idx_, D, hot_slot1_, N, nullptr), "grape_tlookup_hot_index");
        com_A = hyrax.commit_indexed_affine(d_hot, D, msm_size, hot_table_, rowlen, hot_rows_);
        if (cold != 0) {
            // the elements without a table row: queued per row and committed as full-width scalars
            com_cold = hyrax.commit_sparse_affine(A, d_hot, D, msm_size);
            if (!com_cold) {
                FrTensor Acold(D);
                check(grape_fr_mask_cold(W(Acold.gpu_data), W(A.gpu_data), d_hot, D, nullptr), "grape_fr_mask_cold");
                com_cold = hyrax.commit_affine(Acold, D, msm_size);
            }
            check(grape_g1_affine_add((uint32_t*)com_A, (const uint32_t*)com_A, (const uint32_t*)com_cold, rows, nullptr),
                  "grape_g1_affine_add");
        }
        hot_entries_ = hot_rows_;
        cold_elements_ = cold;
        check(grape_stream_sync(nullptr), "sync");
    } catch (...) {
        grape_stream_sync(nullptr);
        grape_free(d_hot); grape_free(com_cold);
        throw;
    }
    grape_free(d_hot); grape_free(com_cold);
    // a caller that pins the count threshold is measuring one selection: nothing is kept for the next proof
    if (hot_min_count_ != 0) drop_hot_rows();
    return true;
}

namespace {
// A witness round over at least this many index pairs runs before the commitments of its proof, a
// shorter one (launch-bound) beside them.
constexpr uint kLongRoundPairs = 1u << 16;
// A stream beside the default one (two per process, created on first use) and the two events that order it against
// the default stream: begin() makes it wait for what the default stream has queued, end() makes the
// default stream wait for it.  If the scope is left by an exception the destructor waits for the
// stream, so nothing it still reads is freed under it.
grape_stream_t g_side_stream[2] = {nullptr, nullptr};
void* g_side_event[2][2] = {{nullptr, nullptr}, {nullptr, nullptr}};
void* g_commit_event[2] = {nullptr, nullptr};
// (never destroyed: they live as long as the process, like the HIP runtime's own default stream)
struct SideChain {
    grape_stream_t stream = nullptr;
    bool open = false;
    explicit SideChain(int which) {
        if (!g_side_stream[which]) {
            check(grape_stream_create(&g_side_stream[which]), "grape_stream_create");
            check(grape_event_create(&g_side_event[which][0]), "grape_event_create");
            check(grape_event_create(&g_side_event[which][1]), "grape_event_create");
        }
        stream = g_side_stream[which];
        ev_begin = g_side_event[which][0];
        ev_end = g_side_event[which][1];
    }
    // `waiter` does not start what is queued on it from now on before what `other` holds at this moment is done
    static void order(grape_stream_t waiter, grape_stream_t other) {
        static void* ev = nullptr;
        if (!ev) check(grape_event_create(&ev), "grape_event_create");
        check(grape_event_record(ev, other), "grape_event_record");
        check(grape_stream_wait_event(waiter, ev), "grape_stream_wait_event");
    }
    void begin() {
        check(grape_event_record(ev_begin, nullptr), "grape_event_record");
        check(grape_stream_wait_event(stream, ev_begin), "grape_stream_wait_event");
        open = true;
    }
    void end() {
        check(grape_event_record(ev_end, stream), "grape_event_record");
        check(grape_stream_wait_event(nullptr, ev_end), "grape_stream_wait_event");
        open = false;
    }
    ~SideChain() {
        if (open) grape_stream_sync(stream);
    }
    void* ev_begin = nullptr;
    void* ev_end = nullptr;
};
// the two events that bracket the commitments queued beside the rounds
std::pair<void*, void*> commit_events() {
    if (!g_commit_event[0]) {
        check(grape_event_create(&g_commit_event[0]), "grape_event_create");
        check(grape_event_create(&g_commit_event[1]), "grape_event_create");
    }
    return {g_commit_event[0], g_commit_event[1]};
}
}  // namespace

void tLookup::start_weights(uint D) {
    const uint nu = Log2(D);
    u_ready_ = forced_u_.empty() ? random_vec(nu) : forced_u_;
    forced_u_.clear();
    E_ready_.reset();
    if (u_ready_.size() != nu) return;          // run() reports the mismatch
    E_ready_.reset(new FrTensor((uint)grape_eq_pyramid_elems(nu ? nu - 1 : 0)));
    // the point travels on the second stream too: on the default stream it would queue behind the pass over the
    // witness, and the pyramid with it
    SideChain side(0);
    fr_t* d_u = grape_host::upload(u_ready_, side.stream);
    check(grape_eq_pyramid(W(E_ready_->gpu_data), W(d_u), nu ? nu - 1 : 0, side.stream), "grape_eq_pyramid");
    grape_free(d_u);                            // handed out again only after what is queued here
}

static void histogram_to_m(FrTensor& m, const FrTensor& vals, int low) {
    uint32_t* hist = nullptr;
    check(grape_malloc((void**)&hist, sizeof(uint32_t) * (size_t)m.size), "grape_malloc");
    check(grape_memset_zero(hist, sizeof(uint32_t) * (size_t)m.size, nullptr), "grape_memset_zero");
    check(grape_tlookup_hist(hist, W(vals.gpu_data), vals.size, low, m.size, nullptr), "grape_tlookup_hist");
    // src/tlookup.cu:276-281: padding a witness of non-power-of-two length adds zeros
    if (vals.size != (1u << Log2(vals.size))) {
        uint32_t zero_count = 0;
        check(grape_memcpy_d2h(&zero_count, hist + (-low), sizeof(uint32_t), nullptr), "d2h");
        zero_count += (1u << Log2(vals.size)) - vals.size;
        check(grape_memcpy_h2d(hist + (-low), &zero_count, sizeof(uint32_t), nullptr), "h2d");
    }
    m.get_data(m.size, hist);
    check(grape_stream_sync(nullptr), "sync");
    grape_free(hist);
}

// src/tlookup.cu:250-263
tLookupRange::tLookupRange(int low_, uint len) : tLookup(1u << Log2(len)), low(low_) {
    index_known_ = true;
    index_low_ = low_;
    // the table always covers the whole power-of-two range T.size (the reference initialises
    // only the first len entries and leaves the rest unset)
    check(grape_tlookup_init(W(T.gpu_data), W(B.gpu_data), low, T.size, W(grape_host::device_scalar(beta)), nullptr, nullptr, nullptr),
          "grape_tlookup_init");
}
tLookupRange::~tLookupRange() {}

void tLookupRange::prep(const FrTensor& vals) { histogram_to_m(m, vals, low); }

// Shared body of tLookupRange::prove (src/tlookup.cu:288-343) and tLookupRangeMapping::prove
// (:397-456) from the inversion on, with tLookup_phase1 (:216-244) and tLookup_phase2 (:192-214).
// Per round the reference runs tLookup_poly_kernel, three full multilinear evaluations,
// tLookup_poly_sum_kernel and two sums (:117-151, :153-190); here one fused pass per operand
// pair produces the same coefficients, weighted by a table of eq(u_low, x) that is halved
// between rounds.
Fr tLookup::run(FrTensor& S, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size, double& commit_time) {
    const uint D = S.size;
    const uint N = T.size;
    // the point and its eq pyramid may have been started by prove() (start_weights)
    std::unique_ptr<FrTensor> E_early = std::move(E_ready_);
    std::vector<Fr> u;
    if (!u_ready_.empty() || E_early) {
        u = std::move(u_ready_);
        u_ready_.clear();
    } else {
        u = forced_u_.empty() ? random_vec(Log2(D)) : forced_u_;
        forced_u_.clear();
    }
    if (u.size() != Log2(D)) E_early.reset();
    if (u.size() != v.size()) throw std::runtime_error("u.size() != v.size()");
    if (v.size() != Log2(D)) throw std::runtime_error("u.size() != ceilLog2(D)");
    if (D % msm_size != 0) throw std::runtime_error("D % msm_size != 0");
    if (N > D) throw std::runtime_error("tLookup: the table is longer than the witness");   // phase 2 binds log2(N) of the log2(D) variables
    last_transcript = SumcheckTranscript();
    hot_entries_ = 0;                       // what THIS proof does with the occupied entries
    cold_elements_ = 0;
    hot_reused_ = false;

    // beta is read by kernels on the side streams until the end of the proof: a buffer of its own, not a
    // slot of the ring of grape_host::device_scalar (which is rewritten after 64 further scalars)
    grape_host::DeviceFr beta_buf(beta);
    fr_t* d_beta = beta_buf.get();
    // Commitments of A and m (kept, not dropped).  With the scaled table of a range lookup the
    // commitment of A reads only the indices, so it does not have to finish before the rounds start
    // folding A: the rounds are then queued first, on streams of their own, and the commitments run
    // beside them (the short rounds and the row reductions of the commitments are latency chains
    // that leave most of the chip idle on their own).  Otherwise the commitments come first.
    const uint rowlen = msm_size * hyrax.com_scale;
    auto timed = [&](const std::function<void()>& fn) {
        auto t0 = std::chrono::steady_clock::now();
        fn();
        commit_time += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    };
    timed([&] {
        if (indexed_commit_ && index_known_ &&
            (scaled_for_ != &hyrax || scaled_cols_ < rowlen || (scaled_table_ && !hyrax.owns_scaled_table(scaled_table_)))) {
            Hyrax::release_scaled_table(scaled_table_);
            scaled_table_ = hyrax.build_scaled_table(B, rowlen);   // nullptr when over budget
            scaled_cols_ = scaled_table_ ? rowlen : 0;
            scaled_for_ = &hyrax;
        }
    });
    const bool indexed = indexed_commit_ && index_known_ && scaled_table_;
    const bool overlap = indexed && d_idx_ != nullptr;
    // A = 1/(S + beta): read from B where the witness matches its table entry (every element of
    // a valid witness does), computed by batched inversion otherwise (tlookup_inv_kernel,
    // src/tlookup.cu:52-62, inverts per element).  When prove() found every element in the table and
    // left A unwritten, the first round gathers it from B - if that round is one of the long ones queued
    // beside the commitments; otherwise A is written out now.
    bool from_table = a_ready_;
    const bool gather_first = a_deferred_ && overlap && D == (1u << Log2(D)) && D / 2 >= kLongRoundPairs && A.size >= D;
    a_ready_ = false;
    a_deferred_ = false;
    if (gather_first) from_table = true;
    if (!from_table && d_idx_) {
        size_t mismatches = 0;
        check(grape_tlookup_inverse_by_table(W(A.gpu_data), W(S.gpu_data), d_idx_, W(T.gpu_data), W(B.gpu_data), D, N, &mismatches, nullptr),
              "grape_tlookup_inverse_by_table");
        from_table = mismatches == 0;
    }
    if (!from_table) check(grape_fr_shift_inverse(W(A.gpu_data), W(S.gpu_data), W(d_beta), D, nullptr), "grape_fr_shift_inverse");
    A.set_size(D);
    if (overlap) {
        // The previous proof's commitments go now, while the streams are idle: a block that is freed takes the
        // marks of what the streams hold at that moment, and the allocation that takes it over waits for those -
        // freed behind the long rounds, the commitments' output buffers would make the host wait for them.
        grape_free(com_A);
        grape_free(com_m);
        com_A = com_m = nullptr;
    }
    auto commit_all = [&] {
        grape_free(com_A);
        grape_free(com_m);
        com_A = com_m = nullptr;
        if (indexed) {
            int* d_idx = d_idx_;
            if (!d_idx) {
                check(grape_malloc((void**)&d_idx, sizeof(int) * (size_t)D), "grape_malloc");
                check(grape_tlookup_index(d_idx, W(S.gpu_data), D, index_low_, N, nullptr), "grape_tlookup_index");
            }
            com_A = hyrax.commit_indexed_affine(d_idx, D, msm_size, scaled_table_, scaled_cols_, N);
            check(grape_stream_sync(nullptr), "sync");
            if (d_idx != d_idx_) grape_free(d_idx);
        } else if (indexed_commit_ && from_table && d_idx_ && d_hist_ && D / rowlen > 1 && commit_A_by_occupancy(A, D, msm_size, hyrax)) {
            // committed through a table of the entries that occur often
        } else {
            com_A = hyrax.commit_affine(A, D, msm_size);
        }
        com_A_rows = D / (msm_size * hyrax.com_scale);
        uint m_N = 1u << (Log2(N) / 2);
        // the multiplicities are small integers: committed from the counters they were made from
        // (five 8-bit digits each) where those are at hand, as field elements otherwise
        if (d_hist_ && D < (1u << 31)) com_m = hyrax.commit_affine_i32(reinterpret_cast<int*>(d_hist_), N, m_N);
        else com_m = hyrax.commit_affine(m, N, m_N);
        com_m_rows = N / (m_N * hyrax.com_scale);
        check(grape_stream_sync(nullptr), "sync");
    };
    // multiplicities that prove() left to this point: counted now, on the default stream, unless the
    // commitments run beside the rounds - then the count, B * m and its sum follow the long rounds on the
    // second stream (whose table side and commitment of m are their only readers)
    if (m_pending_ && !overlap) index_to_m(m_pending_size_, m_pending_low_);
    const bool m_late = m_pending_;
    if (!overlap) timed(commit_all);

    FrTensor Bm(B);
    if (!m_late) Bm *= m;
    Fr alpha_sq = alpha * alpha;
    Fr claim = alpha + alpha_sq;
    Fr N_div_D = Fr((long)N) * Fr((long)D).invert();
    const Fr two_inv = Fr(2).invert();
    const uint logN = Log2(N);

    // eq tables of every prefix of u[0 .. nu-2]: round k (which binds variable nu-1-k) weights its
    // D / 2^(k+1) index pairs with level nu-1-k; nothing is halved between rounds
    const uint nu = (uint)u.size();
    std::unique_ptr<FrTensor> E_own;
    if (E_early) {
        SideChain early(0);
        SideChain::order(nullptr, early.stream);     // the default stream meets the finished pyramid
    } else {
        E_own.reset(new FrTensor((uint)grape_eq_pyramid_elems(nu ? nu - 1 : 0)));
        fr_t* d_u = grape_host::upload(u);
        check(grape_eq_pyramid(W(E_own->gpu_data), W(d_u), nu ? nu - 1 : 0, nullptr), "grape_eq_pyramid");
        grape_free(d_u);                    // no wait: the block is handed out again only after what is queued here
    }
    FrTensor& E = E_early ? *E_early : *E_own;
    // The prover's challenges are all known before the first round, so the rounds are queued
    // back to back: every round leaves its 13 sums in its own slot of one device buffer, which
    // is read once after the last round; the polynomials and the running claim follow on the
    // host.  (The reference interleaves a device-to-host copy and a sync with every round.)
    // (The sum of B * m, which only the host's constant term needs, travels with them.)
    const uint rounds = (uint)v.size();
    // (Three more slots travel with them: the sum of B * m, the last element left of S - the value the proof
    // returns - and the two digit-range flags of the commitments queued beside the rounds.)
    const size_t n_sums = 13 * (size_t)(rounds ? rounds : 1);
    FrTensor sums((uint)n_sums + 3);
    fr_t* const d_sum_Bm = sums.gpu_data + n_sums;
    fr_t* const d_S_last = sums.gpu_data + n_sums + 1;
    int* const d_flags = reinterpret_cast<int*>(sums.gpu_data + n_sums + 2);
    if (!m_late) check(grape_fr_sum(W(d_sum_Bm), W(Bm.gpu_data), N, nullptr), "grape_fr_sum");
    fr_t* d_v = grape_host::upload(v);
    Fr S_last;
    char* long_work = nullptr;             // partial sums of the long rounds and the challenges' tables (overlap mode)
    FrTensor Bw(B), Tw(T), mw(N);          // phase 2 binds copies; T, B, m of this object stay intact
    if (!m_late) check(grape_memcpy_d2d(mw.gpu_data, m.gpu_data, sizeof(fr_t) * (size_t)N, nullptr), "grape_memcpy_d2d");
    try {
        // The table side of phase 2 (B, T, m: sums and folds of the last log2(N) rounds) depends on
        // nothing the witness side produces, so it runs as a chain of its own on a second stream,
        // beside the rounds over A and S (the short rounds are launch- and latency-bound: five
        // small kernels per round on the table side, two on the witness side).
        SideChain side(0), witness(1);
        std::vector<char> mid_from_claim(rounds ? rounds : 1, 0);    // rounds whose middle coefficient follows from the claim
        side.begin();                       // the second stream waits for everything queued so far
        grape_stream_t ws = nullptr;        // where the short witness rounds run: the default stream, or one of its own beside the commitments
        uint cur = D;
        uint k = 0;
        int vi = (int)rounds - 1;
        size_t long_used = 0;
        int32_t* d_tabs = nullptr;
        // A and S: five sums and the fold of both tensors in one pass
        auto witness_round = [&](grape_stream_t st) {
            const uint half = cur / 2;
            fr_t* slot = sums.gpu_data + 13 * (size_t)k;
            const fr_t* e = E.gpu_data + (((size_t)1 << (nu - 1 - k)) - 1);
            // first round of a witness that sits on its table: A = B[index] is the exact inverse of S + beta at
            // every index (B holds the inverses of T + beta, none of which is zero for a range table and, for
            // a mapping table with its random r, except with probability 2^-235), and the weights of a full
            // level sum to one - the round then needs its top coefficient only
            int mode = (k == 0 && from_table && cur == 2 * half && (cur & (cur - 1)) == 0) ? 2 : 1;
            // a long round after the first: its middle coefficient is left to the host, which holds the
            // round's claim when it assembles the polynomials (one limb product per index pair less)
            if (mode == 1 && half >= kLongRoundPairs) {
                mode = 3;
                mid_from_claim[k] = 1;
            }
            if (long_work && half >= kLongRoundPairs) {
                // long round beside the commitments: only the pass over the operands stays on the chain of rounds; its
                // sums are finished on the stream of the short rounds, from a work buffer of the round's own
                uint32_t* partial = reinterpret_cast<uint32_t*>(long_work + long_used);
                long_used += grape_wround2_partial_bytes(half);
                if (k == 0 && gather_first)
                    check(grape_wround2_queue_indexed(W(A.gpu_data), W(S.gpu_data), d_idx_, W(B.gpu_data), N, W(d_beta), W(e), half, W(d_v + vi),
                                                      d_tabs + (size_t)GRAPE_FOLD_TABLE_WORDS * (size_t)vi, partial, st),
                          "grape_wround2_queue_indexed");
                else
                    check(grape_wround2_queue(W(A.gpu_data), W(S.gpu_data), W(d_beta), W(e), cur, half, 1, 1, W(d_v + vi), mode,
                                              d_tabs + (size_t)GRAPE_FOLD_TABLE_WORDS * (size_t)vi, partial, st),
                          "grape_wround2_queue");
                SideChain::order(witness.stream, st);
                check(grape_wround2_finish(W(slot), partial, half, mode, witness.stream), "grape_wround2_finish");
            } else {
                check(grape_wround2(W(A.gpu_data), W(S.gpu_data), W(d_beta), W(e), cur, half, 1, 1, W(d_v + vi), mode, W(slot), st), "grape_wround2");
            }
            A.set_size(half);
            S.set_size(half);
            cur = half;
            vi--;
            k++;
        };
        // the table side of phase 2: per round one launch for the five sums over (B, T), the three over
        // (m, B) and the fold of all three, and one finishing launch
        auto table_side = [&] {
            uint cur_t = N;
            for (int vt = (int)logN - 1; vt >= 0 && vt < (int)rounds; vt--) {
                const uint kt = rounds - 1 - (uint)vt;
                const uint half = cur_t / 2;
                fr_t* slot = sums.gpu_data + 13 * (size_t)kt;
                const fr_t* e = E.gpu_data + (((size_t)1 << (nu - 1 - kt)) - 1);
                check(grape_tlookup_table_round(W(Bw.gpu_data), W(Tw.gpu_data), W(mw.gpu_data), W(d_beta), W(e), half, W(d_v + vt),
                                                W(slot + 5), side.stream),
                      "grape_tlookup_table_round");
                cur_t = half;
            }
        };
        // overlap: the commitments are queued without waiting (their digit-range flags are read after
        // the rounds have been queued too), so the chip works on them while the host issues the
        // rounds' launches; everything that needs the host to wait on the default stream (the sums
        // above) is behind us.  The long witness rounds go first, on the default stream and so
        // BEFORE the commitments, not beside them: a round kernel and the commitment kernel each
        // fill the chip with two waves per SIMD, and side by side a SIMD holds one wave of each -
        // the commitment's wave then issues at the rate of a lone wave (half) while the round's
        // wave waits for memory, which made the pair slower than one after the other.  The short
        // rounds (launch-bound) do run beside the commitments, on a stream of their own.
        if (overlap) {
            // work memory of the long rounds (every round its own partial sums) and the tables of all challenges' multiples
            size_t need = 0;
            for (uint c = D; c / 2 >= kLongRoundPairs; c /= 2) need += grape_wround2_partial_bytes(c / 2);
            if (need) {
                check(grape_malloc((void**)&long_work, need + sizeof(int32_t) * GRAPE_FOLD_TABLE_WORDS * (size_t)rounds), "grape_malloc");
                d_tabs = reinterpret_cast<int32_t*>(long_work + need);
                for (uint k0 = 0; k0 < rounds; k0 += 64)
                    check(grape_fold_tables(d_tabs + (size_t)GRAPE_FOLD_TABLE_WORDS * k0, W(d_v + k0), std::min(64u, rounds - k0), nullptr), "grape_fold_tables");
            }
            while (vi >= 0 && cur / 2 >= kLongRoundPairs) witness_round(nullptr);
            // The table side and the commitment of m (a few rows: a short accumulation and a latency chain of a
            // row reduction) go to the second stream now, so that they run beside the long rounds and the
            // commitment of A instead of after them; the host gets through these launches while the chip
            // still works on the long rounds.
            check(grape_memset_zero(d_flags, 2 * sizeof(int), nullptr), "grape_memset_zero");
            if (m_late) {
                index_to_m(m_pending_size_, m_pending_low_, side.stream);
                check(grape_fr_mul(W(Bm.gpu_data), W(Bm.gpu_data), W(m.gpu_data), N, side.stream), "grape_fr_mul");
                check(grape_fr_sum(W(d_sum_Bm), W(Bm.gpu_data), N, side.stream), "grape_fr_sum");
                check(grape_memcpy_d2d(mw.gpu_data, m.gpu_data, sizeof(fr_t) * (size_t)N, side.stream), "grape_memcpy_d2d");
            }
            table_side();
            const uint m_N = 1u << (Log2(N) / 2);
            com_m_rows = N / (m_N * hyrax.com_scale);
            const bool m_aside = d_hist_ && D < (1u << 31);
            if (m_aside) {
                // d_flags was cleared on the default stream: the second stream meets that point first
                SideChain::order(side.stream, nullptr);
                com_m = hyrax.commit_affine_i32(reinterpret_cast<int*>(d_hist_), N, m_N, d_flags + 1, side.stream);
            }
            witness.begin();                // waits for what is queued so far (the long rounds) - not for the commitments, queued next
            ws = witness.stream;
            // commit_time of this mode: what the commitment of A takes on the default stream, between two events
            check(grape_event_record(commit_events().first, nullptr), "grape_event_record");
            timed([&] {
                com_A = hyrax.commit_indexed_affine(d_idx_, D, msm_size, scaled_table_, scaled_cols_, N, d_flags);
                com_A_rows = D / (msm_size * hyrax.com_scale);
                if (!m_aside) com_m = hyrax.commit_affine(m, N, m_N);
            });
            check(grape_event_record(commit_events().second, nullptr), "grape_event_record");
        }
        while (vi >= 0) witness_round(ws);
        check(grape_memcpy_d2d(d_S_last, S.gpu_data, sizeof(fr_t), ws), "grape_memcpy_d2d");   // S(v), behind the last round
        // without the overlap the table side is queued last: its small launches reach the chip while it
        // works on the first, long rounds of the witness side
        if (!overlap) table_side();
        if (overlap) witness.end();
        side.end();                         // the default stream waits for the table side
        // one copy brings everything the host still needs (and is where it waits for the proof's work)
        std::vector<Fr> h(n_sums + 3);
        check(grape_memcpy_d2h(h.data(), sums.gpu_data, sizeof(fr_t) * h.size(), nullptr), "d2h");
        if (overlap) {
            int flags[2];
            std::memcpy(flags, &h[n_sums + 2], sizeof flags);
            if (flags[0] || flags[1]) throw std::runtime_error("tLookup: a commitment inside the proof met a scalar outside its table's digits");
            float ms = 0;
            check(grape_event_elapsed_ms(&ms, commit_events().first, commit_events().second), "grape_event_elapsed_ms");
            commit_time += ms * 1e-3;
        }
        S_last = h[n_sums + 1];
        Fr C = alpha_sq - h[n_sums];
        grape_free(d_v);
        d_v = nullptr;
        grape_free(long_work);
        long_work = nullptr;

        Fr alpha_run = alpha, alpha_sq_run = alpha_sq;
        int ui = (int)nu - 1;      // index of the variable bound in this round (u.back())
        k = 0;
        for (int vi = (int)rounds - 1; vi >= 0; vi--, ui--, k++) {
            Fr* a3 = &h[13 * (size_t)k];
            const Fr* b3 = a3 + 5;
            const Fr* c3 = a3 + 10;
            const bool phase1 = vi >= (int)logN;
            // the round polynomial from the 13 sums (src/tlookup.cu:117-151, :153-190)
            auto round_poly = [&]() {
                Polynomial p0({a3[0], a3[1], a3[2]});
                p0 = p0 * alpha_run;
                Polynomial p1({a3[3], a3[4]});
                if (phase1) {
                    p0 *= Polynomial::eq(u[ui]);
                    return p0 + p1 + Polynomial(C * two_inv);
                }
                Fr coef = N_div_D * alpha_sq_run;
                p0 += Polynomial({b3[0] * coef, b3[1] * coef, b3[2] * coef});
                Polynomial p2({c3[0], c3[1], c3[2]});
                return Polynomial::eq(u[ui]) * p0 + p1 - p2 * N_div_D;
            };
            if (mid_from_claim[k]) {
                // the kernel left a3[1] = 0.  p(0) + p(1) is linear in it with slope eq(u, 1) * alpha_run = u * alpha_run
                // (only the value at t = 1 of the weighted term contains it), and must equal the claim
                const Fr slope = u[ui] * alpha_run;
                if (slope.is_zero()) throw std::runtime_error("tLookup: a challenge is zero, the round's middle coefficient is not determined by its claim");
                const Polynomial p_without = round_poly();
                a3[1] = (claim - (p_without(0) + p_without(1))) * slope.inverse();
            }
            Polynomial p = round_poly();
            if (claim != p(0) + p(1)) throw std::runtime_error(phase1 ? "tLookup_phase1: claim != p(0) + p(1)" : "tLookup_phase2: claim != p(0) + p(1)");
            if (phase1) C = C * two_inv;
            claim = p(v[vi]);
            last_transcript.rounds.push_back(p);
            last_transcript.claims.push_back(claim);
            Fr e = Polynomial::eq(u[ui], v[vi]);
            alpha_run *= e;
            if (vi < (int)logN) alpha_sq_run *= e;
        }
    } catch (...) {
        grape_free(d_v);
        grape_free(long_work);
        throw;
    }
    return S_last;
}

Fr tLookupRange::prove(FrTensor& S, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size, double& commit_time) {
    uint D = S.size;
    a_ready_ = false;
    if (D == (1u << Log2(D)) && A.size >= D) {
        // no padding: index and A = B[index] in one pass (starts the weights too); A stays unwritten where the
        // first round can gather it from B (a witness of 2^17 elements and more, committed through its indices)
        const bool gather = indexed_commit_ && index_known_ && D / 2 >= (1u << 16);
        make_index_and_A(S, low, A, nullptr, nullptr, !gather);
    } else {
        start_weights(1u << Log2(D));
        make_index(S, low);
    }
    // what prep(S) computes, from the shared indices; a witness that needs no padding leaves it to run()
    if (D == (1u << Log2(D)) && d_idx_) {
        m_pending_ = true;
        m_pending_size_ = D;
        m_pending_low_ = low;
    } else {
        index_to_m(D, low);
    }
    if (D != (1u << Log2(D))) {
        // src/tlookup.cu:299-305: rows of 11008 padded to 16384 with zeros
        Fr pad_value = Fr::zero();
        S.pad(A, 11008, 16384, 1u << Log2(D), pad_value);
        make_index(S, low);                   // indices of the padded witness
    }
    Fr ret;
    try {
        ret = run(S, A, v, hyrax, msm_size, commit_time);
    } catch (...) {
        m_pending_ = false;
        drop_index();
        throw;
    }
    drop_index();
    return ret;
}

Fr tLookupRange::prove(const int* device_int_S, FrTensor& S, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size,
                       double& commit_time) {
    const uint D = S.size;
    const uint Dp = 1u << Log2(D);
    if (D != Dp && D % 11008 == 0 && (uint64_t)(D / 11008) * 16384 <= Dp && low <= 0 && (int64_t)low + (int64_t)T.size > 0 && A.size >= Dp &&
        S.capacity() >= Dp) {
        // rows of 11008 (src/tlookup.cu:299-305): the INTEGERS are padded to rows of 16384 with zeros - the witness the reference
        // proves after its own padding, whose multiplicities are those of the unpadded one plus the padding's zeros
        // (:276-281) - and proved as a witness that needs none
        int* padded = nullptr;
        check(grape_malloc((void**)&padded, sizeof(int) * (size_t)Dp), "grape_malloc");
        Fr ret;
        try {
            check(grape_i32_pad(padded, device_int_S, 11008, 16384, Dp, nullptr), "grape_i32_pad");
            S.set_size(Dp);
            ret = prove(padded, S, A, v, hyrax, msm_size, commit_time);
        } catch (...) {
            grape_stream_sync(nullptr);
            grape_free(padded);
            throw;
        }
        grape_free(padded);
        return ret;
    }
    if (!(D == Dp && A.size >= D)) {
        // any other witness that needs padding goes the ordinary way
        S.get_data(D, const_cast<int*>(device_int_S));
        return prove(S, A, v, hyrax, msm_size, commit_time);
    }
    a_ready_ = false;
    const bool gather = indexed_commit_ && index_known_ && D / 2 >= (1u << 16);
    make_index_and_A_from_ints(device_int_S, nullptr, D, low, S, A, nullptr, nullptr, !gather);
    m_pending_ = true;
    m_pending_size_ = D;
    m_pending_low_ = low;
    Fr ret;
    try {
        ret = run(S, A, v, hyrax, msm_size, commit_time);
    } catch (...) {
        m_pending_ = false;
        drop_index();
        throw;
    }
    drop_index();
    return ret;
}

// ------------------------------------------------------------------ mapping lookup
void tLookupRangeMapping::init_from_host(const int* host_table, uint len) {
    if (len != (1u << Log2(len))) throw std::runtime_error("tLookupRangeMapping: len must be a power of two");
    int* d_int = nullptr;
    check(grape_malloc((void**)&d_int, sizeof(int) * (size_t)len), "grape_malloc");
    check(grape_memcpy_h2d(d_int, host_table, sizeof(int) * (size_t)len, nullptr), "h2d");
    mapped_vals.get_data(len, d_int);
    check(grape_tlookup_init(W(T.gpu_data), W(B.gpu_data), low, len, W(grape_host::device_scalar(beta)), W(mapped_vals.gpu_data),
                             W(grape_host::device_scalar(r)), nullptr),
          "grape_tlookup_init");
    check(grape_stream_sync(nullptr), "sync");
    grape_free(d_map_int_);
    d_map_int_ = d_int;                   // kept: a witness handed over as integers is checked against it
    have_map_zero_ = low <= 0 && (int64_t)low + (int64_t)len > 0;
    map_zero_ = have_map_zero_ ? host_table[-low] : 0;
}
tLookupRangeMapping::~tLookupRangeMapping() { grape_free(d_map_int_); }

// src/tlookup.cu:350-372
tLookupRangeMapping::tLookupRangeMapping(const int low_, const uint len, const std::string& filename)
    : tLookup(len), r(Fr::random_element()), low(low_), mapped_vals(len) {
    std::vector<int> host(len);
    FILE* f = std::fopen(filename.c_str(), "rb");
    if (!f) throw std::runtime_error("tLookupRangeMapping: cannot open " + filename);
    size_t got = std::fread(host.data(), sizeof(int), len, f);
    std::fclose(f);
    if (got != len) throw std::runtime_error("tLookupRangeMapping: short table file " + filename);
    init_from_host(host.data(), len);
}
tLookupRangeMapping::tLookupRangeMapping(const int low_, const uint len, const int* host_table)
    : tLookup(len), r(Fr::random_element()), low(low_), mapped_vals(len) {
    init_from_host(host_table, len);
}

void tLookupRangeMapping::prep(const FrTensor& vals) { histogram_to_m(m, vals, low); }

// src/tlookup.cu:397-456
Fr tLookupRangeMapping::prove(FrTensor& S_in, FrTensor& S_out, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax,
                              uint msm_size, double& commit_time) {
    uint D = S_in.size;
    a_ready_ = false;
    if (S_out.size != D) throw std::runtime_error("tLookupRangeMapping: S_in.size != S_out.size");
    // no padding: index, the check S_out = f(S_in) and A = B[index] in one pass (starts the weights too)
    if (D == (1u << Log2(D)) && A.size >= D) {
        make_index_and_A(S_in, low, A, &S_out, &mapped_vals);
    } else {
        start_weights(1u << Log2(D));
        make_index(S_in, low);
    }
    index_to_m(D, low);                       // what prep(S_in) computes, from the shared indices
    FrTensor S(1u << Log2(D));
    S.set_size(D);
    check(grape_fr_axpy(W(S.gpu_data), W(S_in.gpu_data), W(grape_host::device_scalar(r)), W(S_out.gpu_data), D, nullptr), "grape_fr_axpy");
    if (D != (1u << Log2(D))) {
        Fr pad_value = mapped_vals((uint)(-low)) * r;
        S.pad(A, 11008, 16384, 1u << Log2(D), pad_value);
        pad_index(11008, 16384, 1u << Log2(D), -low + 1);      // the padding value sits at table index -low
    }
    Fr ret;
    try {
        ret = run(S, A, v, hyrax, msm_size, commit_time);
    } catch (...) {
        drop_index();
        throw;
    }
    drop_index();
    return ret;
}

Fr tLookupRangeMapping::prove(const int* device_int_S_in, const int* device_int_S_out, uint D, FrTensor& A, const std::vector<Fr>& v,
                              Hyrax& hyrax, uint msm_size, double& commit_time) {
    const uint Dp = 1u << Log2(D);
    if (D != Dp && D % 11008 == 0 && (uint64_t)(D / 11008) * 16384 <= Dp && have_map_zero_ && A.size >= Dp) {
        // rows of 11008: both integer tensors are padded to rows of 16384 with the pair (0, f(0)) the reference pads with
        // (src/tlookup.cu:411-420) and proved as a witness that needs no padding
        int *pin = nullptr, *pout = nullptr;
        Fr ret;
        try {
            check(grape_malloc((void**)&pin, sizeof(int) * (size_t)Dp), "grape_malloc");
            check(grape_malloc((void**)&pout, sizeof(int) * (size_t)Dp), "grape_malloc");
            check(grape_i32_pad(pin, device_int_S_in, 11008, 16384, Dp, nullptr), "grape_i32_pad");
            check(grape_i32_pad_fill(pout, device_int_S_out, 11008, 16384, Dp, map_zero_, nullptr), "grape_i32_pad_fill");
            ret = prove(pin, pout, Dp, A, v, hyrax, msm_size, commit_time);
        } catch (...) {
            grape_stream_sync(nullptr);
            grape_free(pin);
            grape_free(pout);
            throw;
        }
        grape_free(pin);
        grape_free(pout);
        return ret;
    }
    if (!(D == Dp && A.size >= D)) {
        FrTensor S_in(D, const_cast<int*>(device_int_S_in)), S_out(D, const_cast<int*>(device_int_S_out));
        return prove(S_in, S_out, A, v, hyrax, msm_size, commit_time);
    }
    a_ready_ = false;
    // index, the check S_out = f(S_in) against the integer table, A = B[index] and the combined witness S_in + r * S_out in one
    // pass over the integers
    FrTensor S(D);
    make_index_and_A_from_ints(device_int_S_in, device_int_S_out, D, low, S, A, d_map_int_, &r, true);
    index_to_m(D, low);
    Fr ret;
    try {
        ret = run(S, A, v, hyrax, msm_size, commit_time);
    } catch (...) {
        drop_index();
        throw;
    }
    drop_index();
    return ret;
}

// ------------------------------------------------------------------ round-by-round form
namespace {
// coefficient arrays of (X0 + t X1)(Y0 + shift + t Y1) over the two halves of X and Y
// (tLookup_poly_kernel, src/tlookup.cu:64-81), each evaluated at the remaining variables
struct PolyArrays {
    FrTensor c0, c1, c2;
    explicit PolyArrays(uint n) : c0(n ? n : 1), c1(n ? n : 1), c2(n ? n : 1) {
        c0.set_size(n);
        c1.set_size(n);
        c2.set_size(n);
    }
    void products(const FrTensor& X, const FrTensor& Y, const Fr* shift, uint n) {
        const uint32_t* d_shift = shift ? W(grape_host::device_scalar(*shift)) : nullptr;
        check(grape_tlookup_poly(W(X.gpu_data), W(Y.gpu_data), d_shift, W(c0.gpu_data), W(c1.gpu_data), W(c2.gpu_data), n, nullptr),
              "grape_tlookup_poly");
    }
    void halves(const FrTensor& X, uint n) {     // c0 = X0, c1 = X1 - X0 (tLookup_poly_sum_kernel, :83-91)
        check(grape_tlookup_poly_sum(W(X.gpu_data), W(c0.gpu_data), W(c1.gpu_data), n, nullptr), "grape_tlookup_poly_sum");
    }
};
std::vector<Fr> without_last(const std::vector<Fr>& x) { return std::vector<Fr>(x.begin(), x.end() - (x.empty() ? 0 : 1)); }
}  // namespace

Polynomial tLookup_phase1_step_poly(const Fr& claim, const FrTensor& A, const FrTensor& S, const Fr& alpha, const Fr& beta, const Fr& C,
                                    const std::vector<Fr>& u) {
    (void)claim;
    if (A.size != S.size) throw std::runtime_error("A.size != S.size");
    if (u.empty()) throw std::runtime_error("tLookup_phase1_step_poly: no variable left");
    const uint half = A.size >> 1;
    const std::vector<Fr> rest = without_last(u);
    PolyArrays w(half);
    w.products(A, S, &beta, half);
    Polynomial weighted({w.c0(rest), w.c1(rest), w.c2(rest)});      // the evaluations consume the arrays
    weighted = weighted * alpha;
    weighted *= Polynomial::eq(u.back());
    w.halves(A, half);
    Polynomial plain({w.c0.sum(half), w.c1.sum(half)});
    return weighted + plain + Polynomial(C * Fr(2).invert());
}

Polynomial tLookup_phase2_step_poly(const FrTensor& A, const FrTensor& S, const FrTensor& B, const FrTensor& T, const FrTensor& m,
                                    const Fr& alpha_, const Fr& beta, const Fr& inv_size_ratio, const Fr& alpha_sq,
                                    const std::vector<Fr>& u) {
    if (u.empty()) throw std::runtime_error("tLookup_phase2_step_poly: no variable left");
    const uint half = m.size >> 1;
    const std::vector<Fr> rest = without_last(u);
    PolyArrays w(half);
    w.products(A, S, &beta, half);
    Polynomial weighted({w.c0(rest), w.c1(rest), w.c2(rest)});
    weighted = weighted * alpha_;
    const Fr coef = inv_size_ratio * alpha_sq;
    w.products(B, T, &beta, half);
    weighted += Polynomial({w.c0(rest) * coef, w.c1(rest) * coef, w.c2(rest) * coef});
    w.halves(A, half);
    Polynomial plain({w.c0.sum(half), w.c1.sum(half)});
    w.products(m, B, nullptr, half);
    Polynomial mb({w.c0.sum(half), w.c1.sum(half), w.c2.sum(half)});
    return Polynomial::eq(u.back()) * weighted + plain - mb * inv_size_ratio;
}

Fr tLookup_phase2(const Fr& claim, const FrTensor& A, const FrTensor& S, const FrTensor& B, const FrTensor& T, const FrTensor& m,
                  const Fr& alpha_, const Fr& beta, const Fr& inv_size_ratio, const Fr& alpha_sq, const std::vector<Fr>& u,
                  const std::vector<Fr>& v2) {
    // the reference recurses on fresh half-size tensors; here one set of working copies is bound in place
    FrTensor a(A), s(S), b(B), t(T), mm(m);
    Fr running = claim, weight = alpha_, weight_sq = alpha_sq;
    std::vector<Fr> uu(u), vv(v2);
    while (!vv.empty()) {
        const Polynomial p = tLookup_phase2_step_poly(a, s, b, t, mm, weight, beta, inv_size_ratio, weight_sq, uu);
        if (running != p(0) + p(1)) throw std::runtime_error("tLookup_phase2: claim != p(0) + p(1)");
        const uint half = a.size >> 1;
        uint32_t* ptrs[5] = {W(a.gpu_data), W(s.gpu_data), W(b.gpu_data), W(t.gpu_data), W(mm.gpu_data)};
        check(grape_fr_fold_msb_multi(ptrs, 5, half, W(grape_host::device_scalar(vv.back())), nullptr), "grape_fr_fold_msb_multi");
        check(grape_stream_sync(nullptr), "sync");
        for (FrTensor* x : {&a, &s, &b, &t, &mm}) x->set_size(half);
        running = p(vv.back());
        const Fr e = Polynomial::eq(uu.back(), vv.back());
        weight *= e;
        weight_sq *= e;
        uu.pop_back();
        vv.pop_back();
    }
    return s(0u);
}

Fr tLookup_phase1(const Fr& claim, FrTensor& A, FrTensor& S, const FrTensor& B, const FrTensor& T, FrTensor& m, const Fr& alpha,
                  const Fr& beta, const Fr& C, const Fr& inv_size_ratio, const Fr& alpha_sq, const std::vector<Fr>& u,
                  const std::vector<Fr>& v1, const std::vector<Fr>& v2) {
    Fr running = claim, weight = alpha, constant = C;
    std::vector<Fr> uu(u), vv(v1);
    const Fr two_inv = Fr(2).invert();
    while (!vv.empty()) {
        const Polynomial p = tLookup_phase1_step_poly(running, A, S, weight, beta, constant, uu);
        if (running != p(0) + p(1)) throw std::runtime_error("tLookup_phase1: claim != p(0) + p(1)");
        fr_t* d_v = grape_host::device_scalar(vv.back());
        A.partial_eval(A.size, d_v, 2, 0, A.size >> 1);
        A.set_size(A.size >> 1);
        S.partial_eval(S.size, d_v, 2, 0, S.size >> 1);
        S.set_size(S.size >> 1);
        running = p(vv.back());
        weight *= Polynomial::eq(uu.back(), vv.back());
        constant *= two_inv;
        uu.pop_back();
        vv.pop_back();
    }
    return tLookup_phase2(running, A, S, B, T, m, weight, beta, inv_size_ratio, alpha_sq, uu, v2);
}
