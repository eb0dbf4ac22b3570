// Launch geometry and address arithmetic of the wide-table commitment kernels, in one place so that
// the kernels, their launcher and a host build (tests/native/commit_geometry_host.cpp, which walks
// every wave of a shape and checks each offset against the size of the buffer it indexes) run the
// same expressions.  All element counts and offsets are size_t; only per-row quantities are 32-bit.
#pragma once
#include <stddef.h>
#include <stdint.h>
#include "field.hpp"

namespace grape {
namespace geom {

constexpr int kPartialWords = 64;      // one lane's partial accumulator: 256 bytes
constexpr int kWaveLanes = 64;
constexpr size_t kSlabSegments = 32768;   // row segments per launch: 512 MiB of partial sums

// Lanes that share a row in the one-wave row-reduction kernel: 8 when rows alone fill the chip (measured
// best for 4096 rows of 64 partials: 4 lanes +6 %, 16 +33 %, 32 +65 % - idle lanes of the tree steps cost
// more than shorter chains save), up to a whole wave when rows are few and the chain per lane is
// what takes the time (one row of 32768 partials: 150 ms with 8 lanes).  With 512 rows and more (a value
// below 6) a call that waits for its result takes the four-wave kernel instead, which hands partial sums
// between waves through LDS (tree_row / tree_share below); the value still bounds the column segments of a row.
GRAPE_HD uint32_t reduce_lanes_log2(size_t rows) {
    if (rows >= 2048) return 3;
    if (rows >= 1024) return 4;
    if (rows >= 512) return 5;
    return 6;
}

struct WidePlan {
    size_t rows;            // size / rowlen
    uint32_t lg_lpr;        // log2 of the lanes per row in the reduction
    uint32_t nseg, seg;     // column segments per row and their length
    size_t slab;            // rows per launch
    size_t partial_bytes;   // work buffer of one launch (slab * nseg * 64 lanes * 256 bytes)
};
// segments: enough waves to fill the chip (>= 4 per SIMD) but at least 64 columns per lane-sweep, and
// no more than leaves each reducing lane a chain of 128 partial sums; rows go through in slabs of
// slab_segments row segments
GRAPE_HD WidePlan wide_plan(size_t size, uint32_t rowlen, size_t slab_segments) {
    WidePlan p;
    p.rows = size / rowlen;
    p.lg_lpr = reduce_lanes_log2(p.rows);
    p.nseg = 1;
    while (p.rows * p.nseg < 4096 && rowlen / (p.nseg * 2) >= 64 && p.nseg * 2 <= (2u << p.lg_lpr)) p.nseg *= 2;
    p.seg = (rowlen + p.nseg - 1) / p.nseg;
    p.slab = slab_segments / (size_t)p.nseg;
    if (p.slab < 1) p.slab = 1;
    if (p.slab > p.rows) p.slab = p.rows;
    p.partial_bytes = p.slab * p.nseg * kWaveLanes * (size_t)(4 * kPartialWords);
    return p;
}

// what wave `wave` of a launch over `rows` rows works on
struct WaveSpan {
    size_t row;
    uint32_t s, col_end;
};
GRAPE_HD WaveSpan wave_span(size_t wave, uint32_t nseg, uint32_t seg, uint32_t rowlen) {
    WaveSpan w;
    w.row = wave / nseg;
    w.s = (uint32_t)(wave - w.row * nseg);
    w.col_end = (w.s + 1) * seg < rowlen ? (w.s + 1) * seg : rowlen;
    return w;
}
// element index of scalar (row, col) of a launch whose scalar pointer starts at its first row
GRAPE_HD size_t scalar_index(size_t row, uint32_t rowlen, uint32_t col) { return row * rowlen + col; }
// entry index of digit magnitude mag (1..K) of window w for generator col in a table over N generators
GRAPE_HD size_t table_entry(uint32_t w, uint32_t K, uint32_t mag, size_t N, uint32_t col) {
    return ((size_t)w * K + (mag - 1)) * N + col;
}
// 32-bit-word offset of partial accumulator i (i = wave * 64 + lane in the accumulation kernel,
// row * nparts + j in the reduction kernel)
GRAPE_HD size_t partial_word(size_t i) { return (size_t)kPartialWords * i; }
// reduction kernel: row of lane `lane` of workgroup `block`
GRAPE_HD size_t reduce_row(size_t block, int lane, uint32_t lg_lpr) { return block * (size_t)(kWaveLanes >> lg_lpr) + (size_t)(lane >> lg_lpr); }
// four-wave reduction kernel: a workgroup of 256 threads takes kTreeRows rows, 32 lanes a row; thread t works
// on row tree_row(block, t) and starts from partial sums tree_share(t), tree_share(t) + 32, ... of that row
constexpr int kTreeRows = 8;
constexpr int kTreeThreads = 256;
GRAPE_HD size_t tree_row(size_t block, int t) { return block * (size_t)kTreeRows + (size_t)(t & (kTreeRows - 1)); }
GRAPE_HD uint32_t tree_share(int t) { return (uint32_t)t >> 3; }
// taken for 512 to 4096 rows: up to 512 workgroups, which the chip holds all at once (two per compute unit) - with more
// rows the waves that idle at the kernel's barriers keep later workgroups out, and the one-wave kernel is faster
// (32 768 rows: 0.8 against 1.5 ms)
GRAPE_HD bool tree_reduction(size_t rows, uint32_t lg_lpr, uint32_t nparts) { return lg_lpr <= 5 && rows <= 4096 && nparts <= 4096; }
// workgroups of a launch of `threads` threads in groups of `per_block`
GRAPE_HD size_t blocks_needed(size_t threads, size_t per_block) { return (threads + per_block - 1) / per_block; }

}  // namespace geom
}  // namespace grape
