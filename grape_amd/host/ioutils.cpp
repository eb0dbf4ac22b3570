#include "ioutils.hpp"
#include <cstdio>
#include <cstdlib>
#include <limits>
#include <random>
#include <algorithm>
#include <stdexcept>
#include <vector>
#include "../../include/grape_hip.h"
#include "fr_tensor.hpp"

using grape_host::check;

namespace {
struct File {
    FILE* f;
    File(const std::string& name, const char* mode) : f(std::fopen(name.c_str(), mode)) {}
    ~File() { if (f) std::fclose(f); }
    explicit operator bool() const { return f != nullptr; }
};
}  // namespace

void savebin(const std::string& filename, const void* data, size_t size, bool is_gpu_data) {
    if (!data || size == 0) {
        std::fprintf(stderr, "Error: Invalid input parameters\n");
        return;
    }
    std::vector<char> staged;
    const void* src = data;
    if (is_gpu_data) {
        grape_host::ensure_init();
        staged.resize(size);
        check(grape_memcpy_d2h(staged.data(), data, size, nullptr), "grape_memcpy_d2h");
        src = staged.data();
    }
    File out(filename, "wb");
    if (!out) {
        std::fprintf(stderr, "Error: Failed to open file %s\n", filename.c_str());
        return;
    }
    if (std::fwrite(src, 1, size, out.f) != size) std::fprintf(stderr, "Error: short write to %s\n", filename.c_str());
}

ulong findsize(const std::string& filename) {
    File in(filename, "rb");
    if (!in) {
        std::fprintf(stderr, "Error: cannot open file %s\n", filename.c_str());
        return 0;
    }
    if (fseeko(in.f, 0, SEEK_END) != 0) {
        std::fprintf(stderr, "Error: fseeko failed\n");
        return 0;
    }
    const off_t size = ftello(in.f);
    if (size < 0) {
        std::fprintf(stderr, "Error: ftello failed\n");
        return 0;
    }
    return (ulong)size;
}

void loadbin(const std::string& filename, void* data, size_t size, bool is_gpu_data) {
    if (!data || size == 0) {
        std::fprintf(stderr, "Error: Invalid input parameters\n");
        return;
    }
    File in(filename, "rb");
    if (!in) {
        std::perror(("Error opening file " + filename).c_str());
        return;
    }
    // the destination is only written when the whole read succeeded, as in the reference
    std::vector<char> staged(size);
    const size_t got = std::fread(staged.data(), 1, size, in.f);
    if (got != size) {
        std::fprintf(stderr, "Error: Read %zu bytes, expected %zu\n", got, size);
        return;
    }
    if (is_gpu_data) {
        grape_host::ensure_init();
        check(grape_memcpy_h2d(data, staged.data(), size, nullptr), "grape_memcpy_h2d");
    } else {
        std::copy(staged.begin(), staged.end(), static_cast<char*>(data));
    }
}

static uint load_ints(const std::string& filename, int** gpu_ptr, std::vector<int>& host) {
    const size_t n = findsize(filename) / sizeof(int);
    File in(filename, "rb");
    if (!in) throw std::runtime_error("Error opening file " + filename);
    host.resize(n);
    if (n && std::fread(host.data(), sizeof(int), n, in.f) != n) throw std::runtime_error("short read of " + filename);
    grape_host::ensure_init();
    check(grape_malloc((void**)gpu_ptr, sizeof(int) * (n ? n : 1)), "grape_malloc");
    if (n) check(grape_memcpy_h2d(*gpu_ptr, host.data(), sizeof(int) * n, nullptr), "grape_memcpy_h2d");
    return (uint)n;
}

uint load_data(const std::string& filename, int** gpu_ptr) {
    if (*gpu_ptr != nullptr) {
        grape_free(*gpu_ptr);
        *gpu_ptr = nullptr;
    }
    std::vector<int> host;
    return load_ints(filename, gpu_ptr, host);
}

uint load_data(const std::string& filename, int** gpu_ptr, int** cpu_ptr) {
    std::vector<int> host;
    const uint n = load_ints(filename, gpu_ptr, host);
    *cpu_ptr = static_cast<int*>(std::malloc(sizeof(int) * (n ? n : 1)));   // the caller frees it with free()
    if (!*cpu_ptr) throw std::runtime_error("load_data: out of host memory");
    std::copy(host.begin(), host.end(), *cpu_ptr);
    return n;
}

void generate_data(int** out_ptr, uint size) {
    std::vector<int> host(size);
    std::mt19937 rng(123456);
    std::uniform_int_distribution<int> dist(std::numeric_limits<int>::min(), std::numeric_limits<int>::max());
    for (uint i = 0; i < size; i++) host[i] = dist(rng);
    grape_host::ensure_init();
    check(grape_malloc((void**)out_ptr, sizeof(int) * (size_t)(size ? size : 1)), "grape_malloc");
    if (size) check(grape_memcpy_h2d(*out_ptr, host.data(), sizeof(int) * (size_t)size, nullptr), "grape_memcpy_h2d");
}

const char* grape_host::device_checkpoint() {
    return grape_stream_sync(nullptr) == 0 ? "no error" : grape_last_error();
}
