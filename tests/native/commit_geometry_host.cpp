// Host walk over the launch geometry of the wide-table commitment (grape_amd/csrc/commit_geometry.hpp,
// the expressions the kernels and their launcher use): every wave of every launch of a shape, its
// scalar reads, table gathers, partial-sum stores, the reduction kernel's loads and the output rows,
// each offset checked against the size of the buffer it indexes, every grid against the 32-bit limits
// of a launch.  Returns the number of violations; report[] receives the first one.
#include <cstdio>
#include <cstring>
#include <initializer_list>
#include "../../grape_amd/csrc/commit_geometry.hpp"
using namespace grape;

namespace {
struct Checker {
    long long bad = 0;
    char* report;
    size_t cap;
    void fail(const char* what, size_t got, size_t limit) {
        if (bad == 0 && report) snprintf(report, cap, "%s: %zu >= %zu", what, got, limit);
        bad++;
    }
    void lt(const char* what, size_t got, size_t limit) { if (!(got < limit)) fail(what, got, limit); }
    void le(const char* what, size_t got, size_t limit) { if (!(got <= limit)) fail(what, got, limit + 1); }
};
}  // namespace

extern "C" long long commit_geometry_check(size_t size, uint32_t rowlen, size_t N, uint32_t nw, uint32_t K, uint32_t elem_words,
                                           size_t slab_segments, uint32_t entry_words, uint32_t point_words, size_t* partial_bytes_out,
                                           size_t* launches_out, char* report, size_t report_cap) {
    Checker ck{0, report, report_cap};
    if (report && report_cap) report[0] = 0;
    const geom::WidePlan plan = geom::wide_plan(size, rowlen, slab_segments);
    if (partial_bytes_out) *partial_bytes_out = plan.partial_bytes;
    const size_t scalar_words = size * elem_words;                     // 32-bit words in the scalar buffer
    const size_t table_words = (size_t)nw * K * N * entry_words;
    const size_t partial_words = plan.partial_bytes / 4;
    const size_t out_words = plan.rows * point_words;
    const size_t rows_per_wave = (size_t)geom::kWaveLanes >> plan.lg_lpr;
    size_t launches = 0;
    for (size_t r0 = 0; r0 < plan.rows; r0 += plan.slab) {
        launches++;
        const size_t nr = plan.rows - r0 < plan.slab ? plan.rows - r0 : plan.slab;
        const size_t sc_base = r0 * rowlen * elem_words;               // word offset of this launch's scalars
        const size_t threads = nr * plan.nseg * geom::kWaveLanes;
        const size_t blocks = geom::blocks_needed(threads, 256);
        ck.le("accumulation grid (workgroups)", blocks, 0x7fffffffull);
        ck.le("accumulation grid (threads)", blocks * 256, 0xffffffffull);
        const size_t waves = blocks * 4;
        for (size_t wave = 0; wave < waves; wave++) {
            if (wave >= nr * plan.nseg) continue;                       // the kernel's own exit
            const geom::WaveSpan sp = geom::wave_span(wave, plan.nseg, plan.seg, rowlen);
            ck.lt("row of a wave", sp.row, nr);
            // first and last lane, first and last column each of them reads (incl. the two scalars kept in flight)
            for (int lane = 0; lane < geom::kWaveLanes; lane += geom::kWaveLanes - 1) {
                const uint32_t c0 = sp.s * plan.seg + (uint32_t)lane;
                if (c0 < sp.col_end) {
                    uint32_t last = c0 + ((sp.col_end - 1 - c0) / 64) * 64;
                    for (uint32_t col : {c0, last}) {
                        const size_t si = geom::scalar_index(sp.row, rowlen, col);
                        ck.lt("scalar word", sc_base + (si + 1) * elem_words - 1, scalar_words);
                        // extreme table entries this column can gather: window 0 / nw-1, magnitude 1 / K
                        ck.lt("table word", (geom::table_entry(nw - 1, K, K, N, col) + 1) * entry_words - 1, table_words);
                        ck.lt("table word (touch of the next column)", (geom::table_entry(0, K, K, N, col) + 1) * entry_words - 1, table_words);
                    }
                }
                ck.lt("partial word (store)", geom::partial_word(wave * 64 + lane) + geom::kPartialWords - 1, partial_words);
            }
        }
        // reduction kernel
        const size_t rblocks = (nr + rows_per_wave - 1) / rows_per_wave;
        ck.le("reduction grid (workgroups)", rblocks, 0x7fffffffull);
        ck.le("reduction grid (threads)", rblocks * 64, 0xffffffffull);
        const uint32_t nparts = plan.nseg * 64;
        if (geom::tree_reduction(nr, plan.lg_lpr, nparts)) {
            // four-wave kernel (calls that wait for their result): every thread's row and the last partial sum of its share
            const size_t tblocks = (nr + geom::kTreeRows - 1) / geom::kTreeRows;
            ck.le("tree reduction grid (workgroups)", tblocks, 0x7fffffffull);
            for (size_t b = 0; b < tblocks; b++) {
                for (int t = 0; t < geom::kTreeThreads; t++) {
                    const size_t row = geom::tree_row(b, t);
                    if (row >= nr) continue;
                    const uint32_t share = geom::tree_share(t);
                    ck.lt("share of a thread", share, 32);
                    if (share >= nparts) continue;
                    const uint32_t last = share + ((nparts - 1 - share) / 32) * 32;
                    ck.lt("partial sum of a row", last, nparts);
                    ck.lt("partial word (load)", geom::partial_word(row * nparts + last) + geom::kPartialWords - 1, partial_words);
                    ck.lt("output word", (r0 + row + 1) * point_words - 1, out_words);
                }
            }
        }
        // one-wave kernel (queued calls, and every call with few rows)
        for (size_t b = 0; b < rblocks; b++) {
            for (int lane = 0; lane < 64; lane++) {
                const size_t row = geom::reduce_row(b, lane, plan.lg_lpr);
                if (row >= nr) continue;
                ck.lt("partial word (load)", geom::partial_word(row * nparts + (nparts - 1)) + geom::kPartialWords - 1, partial_words);
                ck.lt("output word", (r0 + row + 1) * point_words - 1, out_words);
            }
        }
    }
    if (launches_out) *launches_out = launches;
    return ck.bad;
}
