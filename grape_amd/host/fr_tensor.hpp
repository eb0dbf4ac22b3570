// FrTensor: a device array of Fr elements with the element-wise, reduction and fold operations of
// the reference's class (include/fr-tensor.cuh:36-76, src/fr-tensor.cu).  Same members, same
// argument meaning, same exceptions; kernels are reached through the C ABI only.
#pragma once
#include <stdexcept>
#include <string>
#include <vector>
#include "fr.hpp"

namespace grape_host {
// Throws std::runtime_error carrying grape_last_error() when a C-ABI call fails.
void check(int rc, const char* what);
// Uploads one scalar into a small ring of device slots and returns its device address
// (replaces the cudaMalloc + cudaMemcpy + cudaFree of a 32-byte scalar per call,
// src/fr-tensor.cu:212-218).  The slot is rewritten, on the default stream, once the calling thread has
// asked for 64 further scalars: the address is for kernels queued on the default stream right away.
// A scalar that other streams read, or that is read for long, gets a DeviceFr of its own.
fr_t* device_scalar(const Fr& x);
// One scalar in a device buffer of its own, freed when the object goes.
class DeviceFr {
public:
    explicit DeviceFr(const Fr& x);
    ~DeviceFr();
    DeviceFr(const DeviceFr&) = delete;
    DeviceFr& operator=(const DeviceFr&) = delete;
    fr_t* get() const { return p_; }

private:
    fr_t* p_ = nullptr;
};
// Uploads a challenge vector; the caller frees with grape_free.
fr_t* upload(const std::vector<Fr>& v, void* stream = nullptr);   // queued on `stream` (nullptr: the default stream)
Fr download(const fr_t* d_ptr);
void ensure_init();
}  // namespace grape_host

uint Log2(uint num);   // ceil(log2 num), Log2(0) = Log2(1) = 0 (src/ioutils.cu:173-190)
void pad_int(int** int_data, uint N, uint pad_N, uint pad_size);   // src/fr-tensor.cu:190-200

class FrTensor {
public:
    fr_t* gpu_data;
    uint size;

    FrTensor(uint size);
    FrTensor(const FrTensor& t);                 // deep copy
    FrTensor(uint size, int* device_int_data);   // embeds device int32 values
    ~FrTensor();

    FrTensor& operator=(const FrTensor& x);      // copies min(size) elements, never reallocates

    void set_size(uint sz);                      // relabels only; the allocation is unchanged
    void get_data(uint sz, int* device_int_data);
    void get_data(uint sz, uint* device_uint_data);
    void partial_eval(uint N, fr_t* x, uint c, uint id, uint gap);
    Fr operator()(const std::vector<Fr>& u);     // multilinear evaluation; destroys the contents
    void add_with_size(uint sz, const FrTensor& t);
    void mul_with_size(uint sz, const FrTensor& t);
    void mul_with_size(uint sz, fr_t* x);
    void mul_with_size(uint sz, Fr& x);
    void inverse();
    void from();
    void to();
    Fr sum(uint sz);                             // non-destructive (the reference clobbers the tensor)
    FrTensor sum(uint sz, uint N);
    Fr operator()(uint idx) const;
    void pad(FrTensor& tmp, uint N, uint pad_N, uint pad_size, const Fr& pad_val);

    FrTensor& operator+=(const FrTensor& t);
    FrTensor& operator+=(const int x);
    FrTensor& operator-=(const FrTensor& t);
    FrTensor& operator*=(const FrTensor& t);
    FrTensor& operator*=(fr_t* x);
    FrTensor& operator*=(const uint x);
    FrTensor& operator*=(Fr& x);

    static FrTensor random(uint size);

    // additions: an integer tensor folded or evaluated as the tensor get_data would make of it, without making
    // it (the first pass reads the integers): partial_eval(N, x, c, id, gap) of that tensor, compacted, and
    // operator()(u) for a power-of-two size
    static FrTensor folded_from_ints(const int* device_int_data, uint N, fr_t* x, uint c, uint id, uint gap);
    static Fr eval_ints(const int* device_int_data, uint size, const std::vector<Fr>& u);
    // additions: host <-> device transfer of whole tensors
    static FrTensor from_host(const std::vector<Fr>& v);
    std::vector<Fr> to_host() const;
    uint capacity() const { return capacity_; }

private:
    uint capacity_;
};

// The fold WITHOUT the compaction that FrTensor::partial_eval adds (src/fr-tensor.cu:168-188): the
// first N elements of t are read as [outer][cur_dim][window_size]; the cur_dim axis is bound with
// x[id], x[id+1], ... and the value of outer index o, inner index g is left at
// t[o * cur_dim * window_size + g], where the reference's in-place rounds leave it.  The other
// positions of the tensor, which hold intermediate values in the reference, keep their contents here.
void Fr_partial_me(uint N, FrTensor& t, fr_t* x, uint id, uint cur_dim, uint window_size);
