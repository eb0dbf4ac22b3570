#include "fr_tensor.hpp"
#include <algorithm>
#include <cassert>
#include "../../include/grape_hip.h"

namespace grape_host {

void check(int rc, const char* what) {
    if (rc != GRAPE_OK) throw std::runtime_error(std::string(what) + ": " + grape_last_error());
}

void ensure_init() {
    static bool done = false;
    if (!done) {
        check(grape_init(0), "grape_init");
        done = true;
    }
}

static constexpr int kSlots = 64;
namespace {
// the ring of one host thread, given back when the thread ends
struct ScalarRing {
    fr_t* p = nullptr;
    ~ScalarRing() { grape_free(p); }
};
}  // namespace
fr_t* device_scalar(const Fr& x) {
    // one ring per host thread: a slot is rewritten after kSlots further calls of the same thread,
    // never by another thread
    thread_local ScalarRing holder;
    thread_local int next = 0;
    ensure_init();
    if (!holder.p) check(grape_malloc((void**)&holder.p, sizeof(fr_t) * kSlots), "grape_malloc");
    fr_t* const ring = holder.p;
    fr_t* slot = ring + next;
    next = (next + 1) % kSlots;
    check(grape_memcpy_h2d(slot, &x, sizeof(fr_t), nullptr), "grape_memcpy_h2d");
    return slot;
}
DeviceFr::DeviceFr(const Fr& x) {
    ensure_init();
    check(grape_malloc((void**)&p_, sizeof(fr_t)), "grape_malloc");
    check(grape_memcpy_h2d(p_, &x, sizeof(fr_t), nullptr), "grape_memcpy_h2d");
}
DeviceFr::~DeviceFr() { grape_free(p_); }

fr_t* upload(const std::vector<Fr>& v, void* stream) {
    ensure_init();
    fr_t* d = nullptr;
    check(grape_malloc((void**)&d, sizeof(fr_t) * std::max<size_t>(v.size(), 1)), "grape_malloc");
    check(grape_memcpy_h2d(d, v.data(), sizeof(fr_t) * v.size(), stream), "grape_memcpy_h2d");
    return d;
}
Fr download(const fr_t* d_ptr) {
    Fr out;
    check(grape_memcpy_d2h(&out, d_ptr, sizeof(fr_t), nullptr), "grape_memcpy_d2h");
    return out;
}

}  // namespace grape_host

using grape_host::check;
static inline uint32_t* W(fr_t* p) { return reinterpret_cast<uint32_t*>(p); }
static inline const uint32_t* W(const fr_t* p) { return reinterpret_cast<const uint32_t*>(p); }

uint Log2(uint num) {
    if (num == 0) return 0;
    num--;
    uint r = 0;
    while (num > 0) {
        num >>= 1;
        r++;
    }
    return r;
}

void pad_int(int** int_data, uint N, uint pad_N, uint pad_size) {
    if (N == pad_N) return;
    int* old = *int_data;
    int* fresh = nullptr;
    check(grape_malloc((void**)&fresh, sizeof(int) * (size_t)pad_size), "grape_malloc");
    check(grape_i32_pad(fresh, old, N, pad_N, pad_size, nullptr), "grape_i32_pad");
    check(grape_stream_sync(nullptr), "sync");
    *int_data = fresh;
    check(grape_free(old), "grape_free");
}

FrTensor::FrTensor(uint size_) : gpu_data(nullptr), size(size_), capacity_(size_) {
    grape_host::ensure_init();
    check(grape_malloc((void**)&gpu_data, sizeof(fr_t) * (size_t)size), "grape_malloc");
}
FrTensor::FrTensor(const FrTensor& t) : gpu_data(nullptr), size(t.size), capacity_(t.size) {
    check(grape_malloc((void**)&gpu_data, sizeof(fr_t) * (size_t)size), "grape_malloc");
    check(grape_memcpy_d2d(gpu_data, t.gpu_data, sizeof(fr_t) * (size_t)size, nullptr), "grape_memcpy_d2d");
}
FrTensor::FrTensor(uint size_, int* int_data) : gpu_data(nullptr), size(size_), capacity_(size_) {
    grape_host::ensure_init();
    check(grape_malloc((void**)&gpu_data, sizeof(fr_t) * (size_t)size), "grape_malloc");
    check(grape_fr_from_i32(W(gpu_data), int_data, size, nullptr), "grape_fr_from_i32");
}
FrTensor::~FrTensor() {
    if (gpu_data != nullptr) {
        grape_free(gpu_data);
        gpu_data = nullptr;
    }
}
FrTensor& FrTensor::operator=(const FrTensor& t) {
    uint n = std::min(size, t.size);
    check(grape_memcpy_d2d(gpu_data, t.gpu_data, sizeof(fr_t) * (size_t)n, nullptr), "grape_memcpy_d2d");
    return *this;
}
void FrTensor::set_size(uint sz) {
    assert(gpu_data != nullptr);
    size = sz;
}
void FrTensor::get_data(uint sz, int* data) {
    size = sz;
    check(grape_fr_from_i32(W(gpu_data), data, size, nullptr), "grape_fr_from_i32");
}
void FrTensor::get_data(uint sz, uint* data) {
    size = sz;
    check(grape_fr_from_u32(W(gpu_data), data, size, nullptr), "grape_fr_from_u32");
}
void FrTensor::partial_eval(uint N, fr_t* x, uint c, uint id, uint gap) {
    check(grape_fr_fold(W(gpu_data), N, W(x), c, id, gap, nullptr), "grape_fr_fold");
}
// src/fr-tensor.cu:346-369, including the rows-of-11008 reading of a short tensor
Fr FrTensor::operator()(const std::vector<Fr>& u) {
    uint log_dim = (uint)u.size();
    fr_t* d_u = grape_host::upload(u);
    if ((uint64_t)size < ((uint64_t)1 << log_dim)) {
        check(grape_fr_fold(W(gpu_data), size, W(d_u), size / 11008, Log2(11008), 11008, nullptr), "grape_fr_fold");
        check(grape_fr_fold(W(gpu_data), 11008, W(d_u), 11008, 0, 1, nullptr), "grape_fr_fold");
    } else {
        check(grape_fr_fold(W(gpu_data), size, W(d_u), size, 0, 1, nullptr), "grape_fr_fold");
    }
    Fr ret = grape_host::download(gpu_data);
    grape_free(d_u);
    return ret;
}
void FrTensor::add_with_size(uint sz, const FrTensor& t) {
    check(grape_fr_add(W(gpu_data), W(gpu_data), W(t.gpu_data), sz, nullptr), "grape_fr_add");
}
void FrTensor::mul_with_size(uint sz, const FrTensor& t) {
    check(grape_fr_mul(W(gpu_data), W(gpu_data), W(t.gpu_data), sz, nullptr), "grape_fr_mul");
}
void FrTensor::mul_with_size(uint sz, fr_t* x) {
    check(grape_fr_bcast_mul(W(gpu_data), W(gpu_data), W(x), sz, nullptr), "grape_fr_bcast_mul");
}
void FrTensor::mul_with_size(uint sz, Fr& x) { mul_with_size(sz, grape_host::device_scalar(x)); }
void FrTensor::inverse() { check(grape_fr_batch_inverse(W(gpu_data), W(gpu_data), size, nullptr), "grape_fr_batch_inverse"); }
void FrTensor::from() { check(grape_fr_from_mont(W(gpu_data), W(gpu_data), size, nullptr), "grape_fr_from_mont"); }
void FrTensor::to() { check(grape_fr_to_mont(W(gpu_data), W(gpu_data), size, nullptr), "grape_fr_to_mont"); }
Fr FrTensor::sum(uint sz) {
    fr_t* slot = grape_host::device_scalar(Fr::zero());
    check(grape_fr_sum(W(slot), W(gpu_data), sz, nullptr), "grape_fr_sum");
    return grape_host::download(slot);
}
FrTensor FrTensor::sum(uint sz, uint N) {
    FrTensor out(sz);
    assert(sz % N == 0);
    check(grape_fr_sum_by_dim(W(out.gpu_data), W(gpu_data), size / N, N, nullptr), "grape_fr_sum_by_dim");
    return out;
}
Fr FrTensor::operator()(uint idx) const { return grape_host::download(gpu_data + idx); }
// src/fr-tensor.cu:459-467: pad through tmp, copy back, relabel
void FrTensor::pad(FrTensor& tmp, uint N, uint pad_N, uint pad_size, const Fr& pad_val) {
    if (N == pad_N) return;
    check(grape_fr_pad(W(tmp.gpu_data), W(gpu_data), N, pad_N, pad_size, W(grape_host::device_scalar(pad_val)), nullptr), "grape_fr_pad");
    check(grape_memcpy_d2d(gpu_data, tmp.gpu_data, sizeof(fr_t) * (size_t)pad_size, nullptr), "grape_memcpy_d2d");
    size = pad_size;
}
FrTensor& FrTensor::operator+=(const FrTensor& t) {
    if (size != t.size) throw std::runtime_error("Incompatible dimensions");
    check(grape_fr_add(W(gpu_data), W(gpu_data), W(t.gpu_data), size, nullptr), "grape_fr_add");
    return *this;
}
FrTensor& FrTensor::operator+=(const int x) {
    check(grape_fr_bcast_add(W(gpu_data), W(gpu_data), W(grape_host::device_scalar(Fr((long)x))), size, nullptr), "grape_fr_bcast_add");
    return *this;
}
FrTensor& FrTensor::operator-=(const FrTensor& t) {
    if (size != t.size) throw std::runtime_error("Incompatible dimensions");
    check(grape_fr_sub(W(gpu_data), W(gpu_data), W(t.gpu_data), size, nullptr), "grape_fr_sub");
    return *this;
}
FrTensor& FrTensor::operator*=(const FrTensor& t) {
    if (size != t.size) throw std::runtime_error("Incompatible dimensions");
    check(grape_fr_mul(W(gpu_data), W(gpu_data), W(t.gpu_data), size, nullptr), "grape_fr_mul");
    return *this;
}
FrTensor& FrTensor::operator*=(fr_t* x) {
    check(grape_fr_bcast_mul(W(gpu_data), W(gpu_data), W(x), size, nullptr), "grape_fr_bcast_mul");
    return *this;
}
FrTensor& FrTensor::operator*=(const uint x) { return *this *= grape_host::device_scalar(Fr((long)x)); }
FrTensor& FrTensor::operator*=(Fr& x) { return *this *= grape_host::device_scalar(x); }

FrTensor FrTensor::random(uint size) {
    std::vector<Fr> tmp(size);
    for (uint i = 0; i < size; i++) tmp[i] = Fr::random_element();
    return from_host(tmp);
}
FrTensor FrTensor::folded_from_ints(const int* device_int_data, uint N, fr_t* x, uint c, uint id, uint gap) {
    grape_host::ensure_init();
    const size_t elems = grape_fr_fold_i32_elems(N, c, gap);
    FrTensor out((uint)(elems ? elems : 1));
    check(grape_fr_fold_i32(W(out.gpu_data), device_int_data, N, W(x), c, id, gap, nullptr), "grape_fr_fold_i32");
    out.set_size(c && gap ? N / (c * gap) * gap : 0);
    return out;
}
Fr FrTensor::eval_ints(const int* device_int_data, uint size, const std::vector<Fr>& u) {
    if ((uint64_t)size != ((uint64_t)1 << u.size())) {
        // the rows-of-11008 reading of a short tensor (src/fr-tensor.cu:346-369) goes through the embedded tensor
        FrTensor t(size, const_cast<int*>(device_int_data));
        return t(u);
    }
    fr_t* d_u = grape_host::upload(u);
    FrTensor t = folded_from_ints(device_int_data, size, d_u, size, 0, 1);
    Fr ret = grape_host::download(t.gpu_data);
    grape_free(d_u);
    return ret;
}
FrTensor FrTensor::from_host(const std::vector<Fr>& v) {
    FrTensor out((uint)v.size());
    check(grape_memcpy_h2d(out.gpu_data, v.data(), sizeof(fr_t) * v.size(), nullptr), "grape_memcpy_h2d");
    return out;
}
std::vector<Fr> FrTensor::to_host() const {
    std::vector<Fr> v(size);
    check(grape_memcpy_d2h(v.data(), gpu_data, sizeof(fr_t) * (size_t)size, nullptr), "grape_memcpy_d2h");
    return v;
}

void Fr_partial_me(uint N, FrTensor& t, fr_t* x, uint id, uint cur_dim, uint window_size) {
    if (cur_dim <= 1 || N == 0) return;
    const size_t dim = (size_t)cur_dim * window_size;
    if (N % dim != 0) throw std::runtime_error("Fr_partial_me: N is not a multiple of cur_dim * window_size");
    const uint outer = (uint)(N / dim);
    FrTensor folded(N);
    check(grape_memcpy_d2d(folded.gpu_data, t.gpu_data, sizeof(fr_t) * (size_t)N, nullptr), "grape_memcpy_d2d");
    check(grape_fr_fold(W(folded.gpu_data), N, W(x), cur_dim, id, window_size, nullptr), "grape_fr_fold");
    for (uint o = 0; o < outer; o++)
        check(grape_memcpy_d2d(t.gpu_data + (size_t)o * dim, folded.gpu_data + (size_t)o * window_size, sizeof(fr_t) * (size_t)window_size, nullptr),
              "grape_memcpy_d2d");
    check(grape_stream_sync(nullptr), "sync");
}
