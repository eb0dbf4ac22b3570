// tlookup / logUp range and mapping proofs: the interface of the reference's
// include/tlookup.cuh:37-79.
#pragma once
#include <string>
#include <memory>
#include <vector>
#include "fr_tensor.hpp"
#include "hyrax.hpp"
#include "polynomial.hpp"
#include "prove.hpp"

class tLookup {
public:
    Fr alpha, beta;
    FrTensor T;
    FrTensor B;
    FrTensor m;

    tLookup(const uint size);

    // The reference draws the prover's point u inside prove() from an unseeded generator
    // (src/tlookup.cu:293); by default it comes from Fr::random_element (the OS generator unless seeded),
    // and a caller that needs a reproducible transcript can fix it here (consumed by the next prove).
    void set_u(const std::vector<Fr>& u) { forced_u_ = u; }
    // Round polynomials of the most recent prove (the reference keeps none).
    SumcheckTranscript last_transcript;
    // Device commitments of A and m made inside prove (affine points); the reference computes
    // and drops them (src/tlookup.cu:320-321).  Owned by this object.
    affine_t* com_A = nullptr;
    affine_t* com_m = nullptr;
    uint com_A_rows = 0, com_m_rows = 0;
    ~tLookup();
    // The elements of A = 1/(S+beta) take only T.size distinct values B[t].  When enabled (the
    // default) and the table fits the Hyrax object's budget, prove() commits A through a table of
    // B[t]*G_i built once per object - one addition per element instead of one per scalar digit.
    // The commitment is the same group element either way.
    void set_indexed_commit(bool on) { indexed_commit_ = on; }
    // Where no table over every entry fits (mapping lookups), A is committed through a table of
    // the entries that occur at least `n` times in the witness (0 = the break-even count, 1.8 times
    // the row length), built by the first proof that needs it and kept: a later proof uses the rows
    // again unless its elements outside them would cost more than new rows.  What the last prove()
    // did is reported below (hot_rows_reused: it found its rows in place).
    void set_hot_min_count(uint n) { hot_min_count_ = n; }
    uint hot_entries() const { return hot_entries_; }
    uint64_t cold_elements() const { return cold_elements_; }
    bool hot_rows_reused() const { return hot_reused_; }

protected:
    Fr run(FrTensor& S, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size, double& commit_time);
    std::vector<Fr> forced_u_;
    // The weights of a proof over a witness of D (padded) elements - the object's random point u and the pyramid of
    // its eq tables - started on the second stream before the witness is indexed and counted, so that they are
    // built beside those passes; run() takes them over.
    void start_weights(uint D);
    std::vector<Fr> u_ready_;
    std::unique_ptr<FrTensor> E_ready_;
    bool indexed_commit_ = true;
    bool index_known_ = false;          // set by tLookupRange: A's index is S - low
    int index_low_ = 0;
    // Table indices (+1, 0 = outside) of the witness of the proof in flight, made once by prove()
    // and used for the multiplicities, for A = B[index] and for the indexed commitment of A.
    // nullptr when the witness is padded (its indices then do not line up with the padded tensor).
    int* d_idx_ = nullptr;
    void make_index(const FrTensor& vals, int low_);
    // index and A = B[index] in one pass over a witness that needs no padding; cmp / cmp_table: the
    // second component of a mapping lookup and the table's.  Sets a_ready_ when every element matched.
    // write_A = false: the indices and the check only (a_deferred_ when every element matched); the first round then
    // gathers A from B, or run() writes it out where that round cannot.
    void make_index_and_A(const FrTensor& key, int low_, FrTensor& A, const FrTensor* cmp, const FrTensor* cmp_table, bool write_A = true);
    // the same pass over a witness that is still a tensor of integers: also leaves the witness as field elements in S
    // (key, or key + r * cmp with the integer table cmp_table of a mapping lookup)
    void make_index_and_A_from_ints(const int* key, const int* cmp, uint n, int low_, FrTensor& S, FrTensor& A, const int* cmp_table,
                                    const Fr* r, bool write_A);
    bool a_ready_ = false;              // A of the proof in flight already holds B[index]
    bool a_deferred_ = false;           // every element sits in the table, A not written yet
    void drop_index();
    void pad_index(uint N, uint pad_N, uint pad_size, int fill);   // rows of N indices -> rows of pad_N
    void index_to_m(uint witness_size, int low_, void* stream = nullptr);
    // prove() may leave the multiplicities to run(): when the commitments are queued beside the rounds, the
    // counting pass goes to the second stream (where everything that reads m runs) instead of standing between
    // the pass over the witness and the first round
    bool m_pending_ = false;
    uint m_pending_size_ = 0;
    int m_pending_low_ = 0;
    uint32_t* d_hist_ = nullptr;        // counts per table entry of the proof in flight (made by index_to_m)
    uint hot_min_count_ = 0;
    uint hot_entries_ = 0;
    uint64_t cold_elements_ = 0;
    bool hot_reused_ = false;
    bool commit_A_by_occupancy(FrTensor& A, uint D, uint msm_size, Hyrax& hyrax);
    // Rows B[t]*G_i of the entries that were occupied in an earlier witness, with their slot
    // assignment: B is fixed for the object's life (the reference keeps one lookup object for all
    // layers of a model, test/llm.cu:57-64), so the rows serve later proofs as long as they cover
    // the witness well enough.
    affine_t* hot_table_ = nullptr;
    int* hot_slot1_ = nullptr;          // entry -> slot + 1 (0 = no row), T.size entries
    uint hot_rows_ = 0, hot_cols_ = 0;
    Hyrax* hot_for_ = nullptr;
    void drop_hot_rows();
    affine_t* scaled_table_ = nullptr;  // B[t]*G_i, built on first use
    uint scaled_cols_ = 0;
    Hyrax* scaled_for_ = nullptr;
};

class tLookupRange : public tLookup {
public:
    const int low;

    tLookupRange(int low, uint len);
    ~tLookupRange();

    void prep(const FrTensor& vals);
    // Proves every element of S lies in [low, low+len); returns S(v).  S and A are scratch-mutated.
    Fr prove(FrTensor& S, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size, double& commit_time);
    // addition: the proof for the tensor that FrTensor::get_data would make of S.size device integers (the reference's
    // drivers embed the witness and prove it, test/llm.cu:77-104).  S is work memory of at least the padded size; the
    // pass that indexes the witness reads the integers and writes S.
    Fr prove(const int* device_int_S, FrTensor& S, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size, double& commit_time);
};

class tLookupRangeMapping : public tLookup {
public:
    Fr r;
    int low;
    FrTensor mapped_vals;

    // table_file holds len raw little-endian int32 values f(low), f(low+1), ...
    tLookupRangeMapping(const int low, const uint len, const std::string& table_file);
    // same from host memory
    tLookupRangeMapping(const int low, const uint len, const int* host_table);

    void prep(const FrTensor& vals);
    Fr prove(FrTensor& S_in, FrTensor& S_out, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax, uint msm_size,
             double& commit_time);
    // addition: the same for two tensors of D device integers (see tLookupRange::prove)
    Fr prove(const int* device_int_S_in, const int* device_int_S_out, uint D, FrTensor& A, const std::vector<Fr>& v, Hyrax& hyrax,
             uint msm_size, double& commit_time);
    ~tLookupRangeMapping();

private:
    void init_from_host(const int* host_table, uint len);
    int* d_map_int_ = nullptr;          // the table's second components as integers (for witnesses handed over as integers)
    bool have_map_zero_ = false;        // 0 is a table key ...
    int map_zero_ = 0;                  // ... and this its image f(0): the pair a padded witness is filled with
};

// The round-by-round form of the logUp sumcheck, as the reference exposes it
// (include/tlookup.cuh:22-34, src/tlookup.cu:117-244): one round polynomial per call from the
// coefficient arrays of (A0 + tA1)(S0 + beta + tS1), three multilinear evaluations and two sums;
// phase 1 binds the variables of D/N with v1 (from the back), phase 2 those of the table with v2.
// prove() does not go through these (its rounds are fused and queued); they give a caller the
// reference's own entry points and the tests an unfused restatement to compare with.
Polynomial tLookup_phase1_step_poly(const Fr& claim, const FrTensor& A, const FrTensor& S, const Fr& alpha, const Fr& beta, const Fr& C,
                                    const std::vector<Fr>& u);
Polynomial tLookup_phase2_step_poly(const FrTensor& A, const FrTensor& S, const FrTensor& B, const FrTensor& T, const FrTensor& m,
                                    const Fr& alpha_, const Fr& beta, const Fr& inv_size_ratio, const Fr& alpha_sq,
                                    const std::vector<Fr>& u);
Fr tLookup_phase2(const Fr& claim, const FrTensor& A, const FrTensor& S, const FrTensor& B, const FrTensor& T, const FrTensor& m,
                  const Fr& alpha_, const Fr& beta, const Fr& inv_size_ratio, const Fr& alpha_sq, const std::vector<Fr>& u,
                  const std::vector<Fr>& v2);
Fr tLookup_phase1(const Fr& claim, FrTensor& A, FrTensor& S, const FrTensor& B, const FrTensor& T, FrTensor& m, const Fr& alpha,
                  const Fr& beta, const Fr& C, const Fr& inv_size_ratio, const Fr& alpha_sq, const std::vector<Fr>& u,
                  const std::vector<Fr>& v1, const std::vector<Fr>& v2);
