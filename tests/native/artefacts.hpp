// The files the reference's programs exchange, written by this build's host classes for a model of
// chosen widths: public parameters as test/ppgen.cu writes them (points.bin: the 256 x n affine
// table; cpu_points.bin: the generators as Jacobian points), the lookup tables
// (table/exp-table.bin, table/swiglu-table.bin: raw int32) and the witness files of one transformer
// block as zzllama/llama/model.py writes them (W/, Q/, R/ <name>-0.bin, raw int32, from
// LayerWitness::save).  Shared by the C++ drivers beside it.
#pragma once
#include <sys/stat.h>
#include <cmath>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>
#include "../../include/grape_hip.h"
#include "../../grape_amd/host/ec_operation.hpp"
#include "../../grape_amd/host/ioutils.hpp"
#include "../../grape_amd/host/witness.hpp"

namespace artefacts {

inline void require(bool ok, const std::string& what) {
    if (!ok) throw std::runtime_error("artefacts: " + what);
}

// seeded, roughly normal integers (sum of four uniforms) of standard deviation sigma
struct Rng {
    unsigned long long s;
    explicit Rng(unsigned long long seed) : s(seed * 0x9e3779b97f4a7c15ull + 1) {}
    unsigned next() {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        return (unsigned)(s >> 32);
    }
    int gauss(double sigma) {
        double u = 0;
        for (int i = 0; i < 4; i++) u += (double)next() / 4294967296.0;
        return (int)((u - 2.0) * 1.7320508 * sigma);      // variance of the sum of four uniforms is 1/3
    }
};

inline int* upload(const std::vector<int>& h) {
    int* d = nullptr;
    require(grape_malloc((void**)&d, sizeof(int) * h.size()) == 0, "grape_malloc");
    require(grape_memcpy_h2d(d, h.data(), sizeof(int) * h.size(), nullptr) == 0, "h2d");
    return d;
}

inline int* device_ints(size_t n, Rng& rng, double sigma, int clip, int offset = 0) {
    std::vector<int> h(n);
    for (size_t i = 0; i < n; i++) {
        int v = rng.gauss(sigma);
        if (clip) v = v < -clip ? -clip : (v > clip - 1 ? clip - 1 : v);
        h[i] = v + offset;
    }
    return upload(h);
}

struct Shape {
    uint tokens, dim, hidden;      // the block: input_tokens x dim activations, hidden-wide feed-forward
    uint npoints, com_scale;       // npoints * com_scale generators (test/ppgen.cu:14-15)
};

// test/ppgen.cu:18-27; returns the table left on the device (256 * npoints * com_scale entries)
inline affine_t* write_parameters(const std::string& dir, const Shape& sh) {
    mkdir(dir.c_str(), 0755);
    const size_t ngen = (size_t)sh.npoints * sh.com_scale;
    affine_t* points = nullptr;
    require(grape_malloc((void**)&points, sizeof(affine_t) * 256 * ngen) == 0, "grape_malloc");
    std::vector<bn128> gens = precompute_generators((uint)ngen, 256, points);
    savebin(dir + "/points.bin", points, sizeof(affine_t) * 256 * ngen);
    savebin(dir + "/cpu_points.bin", gens.data(), gens.size() * sizeof(bn128), false);
    require(findsize(dir + "/points.bin") == sizeof(affine_t) * 256 * ngen, "points.bin size");
    require(findsize(dir + "/cpu_points.bin") == sizeof(bn128) * ngen, "cpu_points.bin size");
    return points;
}

// the two tables and the 50 witness files of one block with seeded weights (fan-in scaled so that
// activations keep unit variance) and a seeded input
inline void write_witness(const std::string& dir, const Shape& sh, unsigned long long seed) {
    for (const char* sub : {"", "/W", "/Q", "/R", "/table"}) mkdir((dir + sub).c_str(), 0755);
    Rng rng(seed);
    const size_t DD = (size_t)sh.dim * sh.dim, FD = (size_t)sh.hidden * sh.dim;
    const double sd = 65536.0 / std::sqrt((double)sh.dim), sf = 65536.0 / std::sqrt((double)sh.hidden);
    LayerWitness::Weights w;
    w.Q = device_ints(DD, rng, sd, 32768);
    w.K = device_ints(DD, rng, sd, 32768);
    w.V = device_ints(DD, rng, sd, 32768);
    w.O = device_ints(DD, rng, sd, 32768);
    w.gate = device_ints(FD, rng, sd, 32768);
    w.up = device_ints(FD, rng, sd, 32768);
    w.down = device_ints(FD, rng, sf, 32768);
    w.norm_first = device_ints(sh.dim, rng, 500, 0, 65536);
    w.norm_second = device_ints(sh.dim, rng, 500, 0, 65536);
    int* x = device_ints((size_t)sh.tokens * sh.dim, rng, 65536, 0);
    const std::vector<int> exp_table = LayerWitness::make_exp_table(), silu_table = LayerWitness::make_silu_table();
    savebin(dir + "/table/exp-table.bin", exp_table.data(), sizeof(int) * exp_table.size(), false);
    savebin(dir + "/table/swiglu-table.bin", silu_table.data(), sizeof(int) * silu_table.size(), false);
    LayerWitness::Tables tables{upload(exp_table), upload(silu_table)};
    LayerWitness lw(sh.tokens, sh.dim, sh.hidden);
    lw.generate(x, w, tables);
    lw.save(dir, 0);
    for (const int* p : {w.Q, w.K, w.V, w.O, w.gate, w.up, w.down, w.norm_first, w.norm_second, (const int*)x, tables.exp, tables.silu})
        grape_free(const_cast<int*>(p));
}

}  // namespace artefacts
