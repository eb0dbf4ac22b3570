// Hyrax row commitments: the interface of the reference's include/Hyrax.cuh:57-86.
#pragma once
#include <memory>
#include <vector>
#include "ec_operation.hpp"
#include "fr_tensor.hpp"

class Hyrax_proof {
public:
    size_t z_size;
    Fr result;
    Fr* z;
    bn128 commit_d;
    bn128 commit_ad;

    Hyrax_proof(Fr result_, size_t z_len, bn128 commit_d_, bn128 commit_ad_);
    ~Hyrax_proof();
    Hyrax_proof(const Hyrax_proof& other);
    Hyrax_proof& operator=(const Hyrax_proof& other);
};

// com[0] = sum_i d[i] * G_i over the first N generators of the reference-format table g
// (entry w * npoints + i = w * G_i): the one-row commitment Hyrax::open makes of its blinding
// vector (single_commit, src/Hyrax.cu:176-185).  d: device, Montgomery form; com: device.
void single_commit(fr_t* d, affine_t* g, jacob_t* com, uint N, uint npoints);

class Hyrax {
public:
    uint com_scale;
    uint layer_num;
    uint npoints;          // generators available = npoints_ * com_scale (also the table stride)
    bn128 G;
    affine_t* g_affine;    // reference-format table: g_affine[k*npoints + i] = k*G_i, k < 256 (not owned)

    // com_scale is hard-wired to 16 in the reference (src/Hyrax.cu:229); it is a parameter here
    // with that default.
    Hyrax(uint layer_num_, uint npoints_, affine_t* g, bn128& G_, uint com_scale_ = 16);
    ~Hyrax();
    Hyrax(const Hyrax&) = delete;
    Hyrax& operator=(const Hyrax&) = delete;

    // Row commitments as a device array of Jacobian points (Z = 1); the caller frees it with
    // grape_free, as the reference's callers cudaFree it (test/commit.cu:72).
    jacob_t* commit(int* tensor, uint size, uint N);
    jacob_t* commit(FrTensor& tensor, uint size, uint N);
    // The same commitments as affine points (what the kernels produce).
    affine_t* commit_affine(int* tensor, uint size, uint N);
    affine_t* commit_affine(FrTensor& tensor, uint size, uint N);
    // Integers of any int32 magnitude, without trying the int16 table first (and without giving that
    // table up for this object when a value does not fit it): lookup multiplicities.
    // With d_flag (a device int the caller owns and has cleared) the call queues its kernels and returns
    // without waiting; the flag is 1 afterwards if a scalar did not fit the table's digits.
    // `stream` (a grape_stream_t; with d_flag only) is where the kernels are queued instead of the default stream.
    affine_t* commit_affine_i32(int* tensor, uint size, uint N, int* d_flag = nullptr, void* stream = nullptr);

    Hyrax_proof open(FrTensor& tensor, const std::vector<Fr> eval_point_, Fr c, uint size, uint N);
    // addition: the opening of the tensor that FrTensor::get_data would make of `size` device integers (the reference's
    // drivers embed an integer tensor and open it, test/llm.cu:99-104) - same proof, the integers are read directly
    Hyrax_proof open(const int* device_int_data, const std::vector<Fr> eval_point_, Fr c, uint size, uint N);
    // Checks an opening against row commitments (the equations of test/HyraxTest.cu:87-125);
    // the reference's own verify is an empty stub (src/Hyrax.cu:307-310).
    bool verify(Hyrax_proof& proof, jacob_t* commitment, const std::vector<Fr>& eval_point, Fr c, uint size, uint N);
    // The reference's signature (include/Hyrax.cuh:85), so that its call sites compile unchanged.  It
    // carries no evaluation point: the point of this object's most recent open() is used, and a
    // failed check (or a call before any open) throws std::runtime_error where the reference's
    // empty body returns silently.
    void verify(Hyrax_proof& proof, jacob_t* commitment, Fr c, uint size, uint N);

    // Scaled table out[t*ncols + i] = scalars[t] * G_i over the first ncols generators (device,
    // owned by the caller, freed with grape_free); nullptr when it would not fit the budget.
    // With it, a tensor whose elements are scalars[idx] commits at one addition per element:
    affine_t* build_scaled_table(const FrTensor& scalars, uint ncols);
    // Builds what build_scaled_table reads (the per-window table over the first ncols generators) if it is
    // not there yet, so that table_bytes_free() afterwards is what a scaled table may really take; false when
    // it does not fit the budget (build_scaled_table would return nullptr).
    bool prepare_scaled_tables(uint ncols);
    // frees a table that build_scaled_table returned and gives its bytes back to the budget of the
    // Hyrax object that built it, if that object still exists
    static void release_scaled_table(affine_t* table);
    // is `table` one that THIS object built and still accounts for?  (false once the object that
    // built it is gone, even if a new object sits at the same address)
    bool owns_scaled_table(const affine_t* table) const;
    // idx_plus1[j] = idx_j + 1 (0 = contributes nothing); rows of N*com_scale, affine output.
    affine_t* commit_indexed_affine(int* idx_plus1, uint size, uint N, affine_t* scaled_table, uint ncols, uint len, int* d_flag = nullptr);

    // Row commitments of the elements whose flag skip[j] is zero, the others left out; through the
    // per-window table that scaled tables are built with.  nullptr when that table does not exist.
    affine_t* commit_sparse_affine(FrTensor& tensor, int* skip, uint size, uint N);

    // Upper bound for the wide fixed-base tables this object may build (default 128 GiB of the 288 GB; GRAPE_TABLE_BUDGET_GIB overrides).  When a
    // table would not fit, commitments go through the reference-format table instead.
    void set_table_budget(size_t bytes) { table_budget_ = bytes; }
    // bytes of that budget not taken by tables that exist now
    size_t table_bytes_free() const {
        const size_t used = table_bytes_in_use();
        return used < table_budget_ ? table_budget_ - used : 0;
    }

private:
    struct WideTable {
        affine_t* d = nullptr;
        uint ngen = 0, c = 0, nw = 0, K = 0;
    };
    // every J-th window set of a full-width table: window w = q*J + j is looked up in set q
    struct StridedTable {
        affine_t* d = nullptr;
        uint ngen = 0, c = 0, J = 0, nsets = 0;
    };
    bool ensure_table(WideTable& t, uint rowlen, uint c, uint nw, uint K);
    bool ensure_fr_table(uint rowlen, bool build = true);       // small per-window table (scaled-table builds)
    bool ensure_strided_table(uint rowlen, bool build = true);  // the table full-width commitments go through
    size_t table_bytes_in_use() const;
    // commits `size` full-width scalars in rows of rowlen into out[0 .. size/rowlen)
    // d_flag (single rows through the per-window table only): queued without waiting, digit-range check left in *d_flag;
    // returns whether it was queued that way (false: the call has waited and checked)
    Hyrax_proof open_impl(FrTensor* tensor, const int* ints, const std::vector<Fr>& eval_point, Fr c, uint size, uint N);
    bool commit_fr_rows(affine_t* out, fr_t* scalars, size_t size, uint rowlen, bool may_build, void* stream = nullptr, int* d_flag = nullptr);
    void commit_i32_rows(affine_t* out, int* tensor, size_t size, uint rowlen, int* d_flag, void* stream = nullptr);
    void check_shape(uint size, uint N) const;
    WideTable int16_table_, int16x2_table_, int32_table_, fr_table_;
    StridedTable fr_strided_;
    bool int16_ok_ = true;
    size_t scaled_bytes_ = 0;
    std::vector<Fr> last_open_point_;
    std::unique_ptr<G1FixedBase> G_multiples_;      // built by the first opening
    size_t table_budget_ = (size_t)128 << 30;
};
