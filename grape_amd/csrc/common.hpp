// Shared host-side plumbing of the C-ABI translation units: error reporting, launch geometry
// and the per-device scratch pool.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/grape_hip.h"
#include "curve.hpp"
#include "field.hpp"

namespace grape {

void set_error(const char* fmt, ...);

#define GRAPE_HIP_CHECK(expr)                                                              \
    do {                                                                                   \
        hipError_t _e = (expr);                                                            \
        if (_e != hipSuccess) {                                                            \
            ::grape::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),      \
                               __FILE__, __LINE__);                                        \
            return GRAPE_EHIP;                                                             \
        }                                                                                  \
    } while (0)

#define GRAPE_REQUIRE(cond, msg)                                                           \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            ::grape::set_error("%s: %s", __func__, msg);                                   \
            return GRAPE_EINVAL;                                                           \
        }                                                                                  \
    } while (0)

#define GRAPE_LAUNCH_CHECK() GRAPE_HIP_CHECK(hipGetLastError())

// Tells the block cache of grape_malloc / grape_free which streams carry this library's work (see
// runtime.hip): the default stream and the streams made by grape_stream_create are known to it, any
// other stream makes it wait for the whole device again before a kept block is reused.
void note_stream(hipStream_t s);
static inline hipStream_t as_stream(grape_stream_t s) {
    hipStream_t h = reinterpret_cast<hipStream_t>(s);
    if (h) note_stream(h);
    return h;
}

constexpr int kBlock = 256;          // 4 wave64 per workgroup
constexpr int kNumCU = 256;          // MI355X
static inline unsigned blocks_for(size_t n, int per_block = kBlock) {
    return (unsigned)((n + per_block - 1) / per_block);
}

// Scratch pool: one growing device allocation per (stream, slot), reused across calls so the hot
// path never allocates once warm.  Slots are independent buffers (a call may use several at once);
// the buffer belongs to `stream`: only kernels launched on that stream may touch it.
enum ScratchSlot { kSlotReduce = 0, kSlotFold = 1, kSlotInv = 2, kSlotMsm = 3, kSlotMisc = 4, kSlotFoldW = 5, kSlotHistIdx = 6, kSlotHistPart = 7, kSlotWitA = 8, kSlotWitB = 9, kSlotTable = 10, kNumSlots = 11 };
int scratch_get(ScratchSlot slot, size_t bytes, void** out, hipStream_t stream);
// Zeroes device memory with a small fill kernel (word-sized regions) so that a caller who captures
// the stream into a graph records a kernel node, not a memset node.
int zero_fill(void* d_ptr, size_t bytes, hipStream_t s);
bool initialised();

// Optional per-kernel event timing (see grape_profile_enable).
bool profiling();
void profile_begin();                     // forget the previous call's marks
int profile_mark(hipStream_t s);          // record an event; kernels sit between consecutive marks

}  // namespace grape
