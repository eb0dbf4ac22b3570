#include "witness.hpp"
#include <cmath>
#include <cstdio>
#include <stdexcept>
#include "../../include/grape_hip.h"
#include "fr_tensor.hpp"

using grape_host::check;

LayerWitness::LayerWitness(uint seq_len_, uint dim_, uint hidden_)
    : seq_len(seq_len_), dim(dim_), hidden(hidden_), d_sumsq_(nullptr) {
    if (seq_len == 0 || dim == 0 || hidden == 0) throw std::invalid_argument("LayerWitness: empty shape");
    grape_host::ensure_init();
    const size_t TD = (size_t)seq_len * dim, TT = (size_t)seq_len * seq_len, TF = (size_t)seq_len * hidden;
    for (const char* n : {"Q/input", "Q/rmswFirst", "R/rmswFirst", "Q/normOutFirst", "R/normOutFirst", "Q/xq", "R/xq", "Q/xk", "R/xk", "Q/xv",
                          "R/xv", "Q/qkv", "R/qkv", "Q/atten_out", "R/atten_out", "Q/skip", "Q/rmswSecond", "R/rmswSecond",
                          "Q/normOutSecond", "R/normOutSecond", "Q/down_out", "R/down_out", "Q/output"})
        own(n, TD);
    for (const char* n : {"Q/scores", "R/scores", "Q/exp_input", "Q/exp_output", "Q/softmax_output", "Q/softmax_lookup_query"}) own(n, TT);
    for (const char* n : {"Q/up_out", "R/up_out", "Q/gate_out", "R/gate_out", "Q/silu_out", "Q/upSilu", "R/upSilu"}) own(n, TF);
    for (const char* n : {"Q/rmsFirst", "Q/rmsSecond", "Q/max", "Q/exp_sum"}) own(n, seq_len);
    check(grape_malloc((void**)&d_sumsq_, sizeof(unsigned long long) * (size_t)seq_len), "grape_malloc");
}

LayerWitness::~LayerWitness() {
    for (auto& kv : t_)
        if (kv.second.owned) grape_free(kv.second.owned);
    if (d_sumsq_) grape_free(d_sumsq_);
}

int* LayerWitness::own(const std::string& name, size_t size) {
    int* p = nullptr;
    check(grape_malloc((void**)&p, sizeof(int) * size), "grape_malloc");
    t_[name] = Slot{p, p, size};
    return p;
}

void LayerWitness::alias(const std::string& name, const int* p, size_t size) {
    auto it = t_.find(name);
    if (it != t_.end() && it->second.owned) grape_free(it->second.owned);
    t_[name] = Slot{nullptr, p, size};
}

std::vector<std::string> LayerWitness::names() const {
    std::vector<std::string> v;
    for (const auto& kv : t_) v.push_back(kv.first);
    return v;
}

const int* LayerWitness::tensor(const std::string& name) const {
    auto it = t_.find(name);
    if (it == t_.end()) throw std::out_of_range("LayerWitness: no tensor named " + name);
    return it->second.ptr;
}

size_t LayerWitness::tensor_size(const std::string& name) const {
    auto it = t_.find(name);
    if (it == t_.end()) throw std::out_of_range("LayerWitness: no tensor named " + name);
    return it->second.size;
}

double LayerWitness::to_float16(double x) {
    if (!(x == x)) throw std::domain_error("to_float16: not a number");
    const double ax = std::fabs(x);
    double r;
    if (ax < 6.103515625e-05) {                      // below 2^-14: subnormal spacing 2^-24
        r = std::nearbyint(ax * 16777216.0) / 16777216.0;
    } else {
        int e;
        const double m = std::frexp(ax, &e);          // ax = m * 2^e, m in [0.5, 1)
        r = std::ldexp(std::nearbyint(std::ldexp(m, 11)), e - 11);   // 11 significant bits, ties to even
    }
    if (r > 65504.0) throw std::overflow_error("to_float16: value beyond the float16 range");
    return x < 0 ? -r : r;
}

std::vector<int> LayerWitness::make_exp_table() {
    const int n = 1 << 20;
    std::vector<int> t(n);
    for (int i = 0; i < n; i++) t[i] = (int)std::nearbyint(std::exp((double)(i - (n - 1)) / 65536.0) * 65536.0);
    return t;
}

std::vector<int> LayerWitness::make_silu_table() {
    const int n = 1 << 19;
    std::vector<int> t(n);
    for (int i = 0; i < n; i++) {
        const double x = (double)(i - (1 << 18)) / 4096.0;
        t[i] = (int)std::nearbyint(x / (1.0 + std::exp(-x)) * 65536.0);
    }
    return t;
}

// model.py:216-257.  tag = "First" / "Second".
void LayerWitness::rmsnorm(const int* x, const int* w, const std::string& tag, double eps) {
    check(grape_wit_row_sumsq((uint64_t*)d_sumsq_, x, seq_len, dim, nullptr), "grape_wit_row_sumsq");
    std::vector<unsigned long long> ss(seq_len);
    check(grape_memcpy_d2h(ss.data(), d_sumsq_, sizeof(unsigned long long) * (size_t)seq_len, nullptr), "grape_memcpy_d2h");
    std::vector<int> rms(seq_len);
    for (uint i = 0; i < seq_len; i++) {
        const double t = (double)ss[i] / ((double)dim * 4294967296.0) + eps;
        const double h = to_float16(1.0 / std::sqrt(t));
        rms[i] = (int)std::nearbyint(h * 65536.0);
    }
    int* d_rms = const_cast<int*>(tensor("Q/rms" + tag));
    check(grape_memcpy_h2d(d_rms, rms.data(), sizeof(int) * (size_t)seq_len, nullptr), "grape_memcpy_h2d");
    check(grape_wit_rmsnorm_apply(const_cast<int*>(tensor("Q/rmsw" + tag)), const_cast<int*>(tensor("R/rmsw" + tag)),
                                  const_cast<int*>(tensor("Q/normOut" + tag)), const_cast<int*>(tensor("R/normOut" + tag)), x, d_rms, w,
                                  seq_len, dim, (int64_t)1 << SCALE_BITS, nullptr),
          "grape_wit_rmsnorm_apply");
}

void LayerWitness::generate(const int* x, const Weights& w, const Tables& tb, double eps) {
    if (!x || !w.Q || !w.K || !w.V || !w.O || !w.gate || !w.up || !w.down || !w.norm_first || !w.norm_second || !tb.exp || !tb.silu)
        throw std::invalid_argument("LayerWitness::generate: null input");
    const uint T = seq_len, D = dim, F = hidden;
    const int64_t S = (int64_t)1 << SCALE_BITS;
    auto m = [&](const char* n) { return const_cast<int*>(tensor(n)); };
    auto mm = [&](const char* q, const char* r, const int* a, const int* b, uint N, uint M, uint K, int bits, int tr) {
        check(grape_wit_matmul_rescale(m(q), m(r), a, b, 1, N, M, K, (int64_t)1 << bits, tr, nullptr), "grape_wit_matmul_rescale");
    };
    const size_t DD = (size_t)D * D, FD = (size_t)F * D;
    alias("W/Q", w.Q, DD); alias("W/K", w.K, DD); alias("W/V", w.V, DD); alias("W/O", w.O, DD);
    alias("W/gate", w.gate, FD); alias("W/up", w.up, FD); alias("W/down", w.down, FD);
    alias("W/NormFirst", w.norm_first, D); alias("W/NormSecond", w.norm_second, D);
    uint32_t flags = 0;
    check(grape_wit_status(&flags, nullptr), "grape_wit_status");      // forget what earlier callers left behind

    check(grape_memcpy_d2d(m("Q/input"), x, sizeof(int) * (size_t)T * D, nullptr), "grape_memcpy_d2d");
    rmsnorm(x, w.norm_first, "First", eps);
    // attention (model.py:473-590)
    const int* h1 = tensor("Q/normOutFirst");
    mm("Q/xq", "R/xq", h1, w.Q, T, D, D, SCALE_BITS, 0);
    mm("Q/xk", "R/xk", h1, w.K, T, D, D, SCALE_BITS, 0);
    mm("Q/xv", "R/xv", h1, w.V, T, D, D, SCALE_BITS, 1);               // kept transposed: [dim][seq], model.py:500-501
    mm("Q/scores", "R/scores", tensor("Q/xq"), tensor("Q/xk"), T, T, D, QK_SCALE_BITS, 0);
    check(grape_wit_softmax(m("Q/max"), m("Q/exp_input"), m("Q/exp_output"), m("Q/exp_sum"), m("Q/softmax_output"),
                            m("Q/softmax_lookup_query"), tensor("Q/scores"), T, T, tb.exp, 20, 20, S, nullptr),
          "grape_wit_softmax");
    mm("Q/qkv", "R/qkv", tensor("Q/softmax_output"), tensor("Q/xv"), T, D, T, SCALE_BITS, 0);
    mm("Q/atten_out", "R/atten_out", tensor("Q/qkv"), w.O, T, D, D, SCALE_BITS, 0);
    check(grape_wit_add_i32(m("Q/skip"), x, tensor("Q/atten_out"), (size_t)T * D, nullptr), "grape_wit_add_i32");
    // feed-forward (model.py:634-703)
    rmsnorm(tensor("Q/skip"), w.norm_second, "Second", eps);
    const int* h2 = tensor("Q/normOutSecond");
    alias("Q/ffn_input", h2, (size_t)T * D);
    mm("Q/up_out", "R/up_out", h2, w.up, T, F, D, SCALE_BITS, 0);
    mm("Q/gate_out", "R/gate_out", h2, w.gate, T, F, D, SWIGLU_SCALE_BITS, 0);
    check(grape_wit_table_lookup(m("Q/silu_out"), tensor("Q/gate_out"), (size_t)T * F, -(1 << 18), 1u << 19, tb.silu, nullptr),
          "grape_wit_table_lookup");
    check(grape_wit_elemul_rescale(m("Q/upSilu"), m("R/upSilu"), tensor("Q/silu_out"), tensor("Q/up_out"), (size_t)T * F, S, nullptr),
          "grape_wit_elemul_rescale");
    mm("Q/down_out", "R/down_out", tensor("Q/upSilu"), w.down, T, D, F, SCALE_BITS, 0);
    check(grape_wit_add_i32(m("Q/output"), tensor("Q/skip"), tensor("Q/down_out"), (size_t)T * D, nullptr), "grape_wit_add_i32");

    check(grape_wit_status(&flags, nullptr), "grape_wit_status");
    if (flags & GRAPE_WIT_INDEX) throw std::runtime_error("LayerWitness: a table index is out of range (the reference asserts here)");
    if (flags & GRAPE_WIT_QUOTIENT) throw std::runtime_error("LayerWitness: a rescaled value does not fit int32");
    if (flags & GRAPE_WIT_SUM) throw std::runtime_error("LayerWitness: a softmax row has no positive table entry");
    if (flags & GRAPE_WIT_SQUARES) throw std::runtime_error("LayerWitness: a row's sum of squares does not fit 64 bits");
}

void LayerWitness::save(const std::string& data_dir, uint group) const {
    std::vector<int> host;
    for (const auto& kv : t_) {
        host.resize(kv.second.size);
        check(grape_memcpy_d2h(host.data(), kv.second.ptr, sizeof(int) * kv.second.size, nullptr), "grape_memcpy_d2h");
        const std::string path = data_dir + "/" + kv.first + "-" + std::to_string(group) + ".bin";
        FILE* f = std::fopen(path.c_str(), "ab");
        if (!f) throw std::runtime_error("LayerWitness::save: cannot open " + path);
        const size_t n = std::fwrite(host.data(), sizeof(int), host.size(), f);
        std::fclose(f);
        if (n != host.size()) throw std::runtime_error("LayerWitness::save: short write to " + path);
    }
}
