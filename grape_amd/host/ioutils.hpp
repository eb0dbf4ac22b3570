// File helpers of the reference's drivers (include/ioutils.cuh:52-64, src/ioutils.cu:3-160): raw
// little-endian dumps of device or host buffers.  The formats are the reference's own:
//   * int tensors  (data/{W,Q,R}/*.bin): int32, row-major;
//   * Fr tensors:  fr_t[n], 32 bytes each, Montgomery form;
//   * points.bin:  affine_t[256 * npoints], entry w * npoints + i = w * G_i, 96 bytes each
//                  (64 in the BN254 build);
//   * commitments: jacob_t[rows], 144 bytes each (96 in the BN254 build).
// Point files are specific to the curve the library was built for; the BN254 build
// (-DGRAPE_CURVE_BN254) reads and writes the layout of the reference's own BN254 build.
#pragma once
#include <chrono>
#include <cstdio>
#include <string>

typedef unsigned int uint;
typedef unsigned long ulong;

// writes `size` bytes; device memory is staged through the host.  Errors are reported on stderr
// and the call returns, as in the reference.
void savebin(const std::string& filename, const void* data, size_t size, bool is_gpu_data = true);
// file size in bytes, 0 when the file cannot be read
ulong findsize(const std::string& filename);
// reads exactly `size` bytes into device (default) or host memory
void loadbin(const std::string& filename, void* data, size_t size, bool is_gpu_data = true);
// whole file of int32 into a fresh device buffer (an old *gpu_ptr is released first); returns the
// element count.  A missing file throws std::runtime_error (the reference calls exit(1)).
uint load_data(const std::string& filename, int** gpu_ptr);
uint load_data(const std::string& filename, int** gpu_ptr, int** cpu_ptr);
// `size` uniformly distributed int32 from std::mt19937(123456) into a fresh device buffer
void generate_data(int** out_ptr, uint size);

// The drivers' timing and checkpoint macros (include/ioutils.cuh:20-48), same names and output
// lines.  The reference times device work with events on stream 0; every public call of this build
// has finished its device work when it returns, so here both timer kinds read the host clock after
// waiting for the device.
namespace grape_host {
struct StopWatch {
    std::chrono::high_resolution_clock::time_point t0 = std::chrono::high_resolution_clock::now();
    double ms() const { return std::chrono::duration<double, std::milli>(std::chrono::high_resolution_clock::now() - t0).count(); }
};
// waits for the device and returns the text of its last error ("no error" when there is none)
const char* device_checkpoint();
}  // namespace grape_host
#define CUDA_DEBUG std::printf("%d %s\n", __LINE__, grape_host::device_checkpoint());
#define CUDA_TIMER_START(timer_name) \
    grape_host::device_checkpoint(); \
    grape_host::StopWatch timer_name##_watch;
#define CUDA_TIMER_STOP(timer_name)  \
    grape_host::device_checkpoint(); \
    std::printf("%s elapsed: %f ms\n", #timer_name, timer_name##_watch.ms());
#define CPU_TIMER_START(timer_name) grape_host::StopWatch timer_name##_watch;
#define CPU_TIMER_STOP(timer_name) std::printf("%s elapsed: %f ms\n", #timer_name, timer_name##_watch.ms())
