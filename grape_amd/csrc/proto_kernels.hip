// Protocol kernels: fused sumcheck rounds (prove.cu) and the logUp / tlookup kernels (tlookup.cu).
// Every round kernel streams its operands once and leaves per-workgroup partial sums that a
// one-block kernel finishes; nothing here allocates.
#include <mutex>
#include "fr_device.hpp"

namespace grape {

// Iterations per thread of the round kernels: the coefficient sums are kept as double-width column
// accumulators across the grid-stride loop and reduced once per thread, which bounds how many
// products an accumulator may absorb: a column takes ten limb products below 2^52 per operand
// pair (2^55.4), so 64 pairs stay below 2^61.4, and |sum| < 64 r^2 leaves the reduction within
// (-1.82 r, 2.82 r) of its offset - inside the windows finish_sum is called with below.  The
// reduction and the workgroup tree that follow cost about five thousand instructions per thread:
// with 16 pairs per thread that was a quarter of the kernel, with 64 it is a fifteenth.
constexpr int kRoundIters = 64;

// CLAIM: the sum of the round polynomial over {0, 1} is known (it is the value the previous round's
// polynomial took at its challenge), so the value at t = 1 is not accumulated: the kernel leaves
// c0 and c2 and the finishing kernel takes c1 = claim - 2 c0 - c2.
template <bool COEFFS, bool TAB, bool CLAIM = false, bool PREFETCH = CLAIM>
__global__ void __launch_bounds__(kBlock, 2) sumcheck2_kernel(uint32_t* A, uint32_t* B, uint32_t* ca, uint32_t* cb, uint32_t* cc,
                                                           uint32_t in_size, uint32_t out_size, const uint32_t* v,
                                                           const int32_t* __restrict__ tab, uint32_t* partial) {
    __shared__ Fr lds[3 * (kBlock / 64)];
    fr26::Limbs w1;
    if (!TAB) w1 = fr26::weight16(ld_fr(v, 0));
    fr26::Acc C0, Q, C2;
    fr26::acc_zero(C0);
    fr26::acc_zero(Q);
    fr26::acc_zero(C2);
    const size_t stride = (size_t)gridDim.x * kBlock;
    size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x;
    // one index: fold both tensors in place and add the index's products to the coefficient sums
    auto step = [&](size_t i, const Fr& ra0, const Fr& rb0, const Fr& ra1, const Fr& rb1) __attribute__((always_inline)) {
        const fr26::Limbs a0 = fr26::pack(ra0), b0 = fr26::pack(rb0);
        const fr26::Limbs a1 = fr26::pack(ra1), b1 = fr26::pack(rb1);
        const fr26::Limbs da = fr26::sub(a1, a0), db = fr26::sub(b1, b0);   // signed, |limb| < 2^26
        // long rounds fold through the table of the challenge's multiples (no full reduction), short
        // ones through one limb product (no table to prepare)
        if (TAB) {
            Fr fa, fb;
            foldt2(tab, a0, da, b0, db, fa, fb);
            st_fr(A, i, fa);
            st_fr(B, i, fb);
        } else {
            st_fr(A, i, fold1(w1, a0, da));
            st_fr(B, i, fold1(w1, b0, db));
        }
        if (COEFFS) {
            // materialised coefficient arrays (phase 1 folds them further)
            fr26::Acc T;
            fr26::acc_zero(T);
            fr26::mac(T, a0, b0);
            const Fr c_ = fr26::finish_sum(T, 0);
            fr26::acc_zero(T);
            fr26::mac(T, da, db);
            const Fr a_ = fr26::finish_sum(T, 1);
            fr26::acc_zero(T);
            fr26::mac(T, a1, b1);
            st_fr(cc, i, c_);
            st_fr(cb, i, sub(sub(fr26::finish_sum(T, 0), c_), a_));
            st_fr(ca, i, a_);
        }
        // middle coefficient by Karatsuba: da*b0 + a0*db = a1*b1 - a0*b0 - da*db, so the value at
        // t = 1 is accumulated with one product instead of two
        fr26::mac(C0, a0, b0);
        if (!CLAIM) fr26::mac(Q, a1, b1);
        fr26::mac(C2, da, db);
    };
    if (!PREFETCH) {
        for (; g < out_size; g += stride)
            step(g, ld_fr(A, g), ld_fr(B, g), ld_hi(A, g, out_size, in_size), ld_hi(B, g, out_size, in_size));
    } else if (g < out_size) {
        // The next index's four operands are requested before this index's arithmetic starts, so a
        // wave's memory latency passes under its own ~3000 cycles of multiplies instead of under the
        // one other wave that the register budget leaves on the SIMD.  Two register sets take turns
        // (one is loaded while the other is worked on), so no copies stand between the loads and their
        // use.  All loads are unconditional, for the same reason: past the thread's last index they
        // repeat the current index (values unused), and an upper operand past the live extent is read
        // from the lower operand's address and replaced by zero when it is used.
        struct Set { Fr a0, b0, a1, b1; uint32_t hi_mask; };
        auto request = [&](Set& s, size_t i) __attribute__((always_inline)) {
            const bool hi_live = i + out_size < in_size;
            s.hi_mask = hi_live ? 0xffffffffu : 0u;
            const size_t ih = hi_live ? i + out_size : i;
            s.a0 = ld_fr(A, i), s.b0 = ld_fr(B, i), s.a1 = ld_fr(A, ih), s.b1 = ld_fr(B, ih);
        };
        auto work = [&](size_t i, const Set& s) __attribute__((always_inline)) {
            Fr a1 = s.a1, b1 = s.b1;
#pragma unroll
            for (int k = 0; k < 8; k++) a1.v[k] &= s.hi_mask, b1.v[k] &= s.hi_mask;
            step(i, s.a0, s.b0, a1, b1);
        };
        Set x, y;
        request(x, g);
        // the first operands are waited for here: a wait at the loop's head would also hold up every
        // later pass, whose operands arrived during the pass before
        arrived(x.a0), arrived(x.b0), arrived(x.a1), arrived(x.b1);
        for (;;) {
            size_t gn = g + stride;
            request(y, gn < out_size ? gn : g);
            work(g, x);
            if (gn >= out_size) break;
            g = gn, gn = g + stride;
            request(x, gn < out_size ? gn : g);
            work(g, y);
            if (gn >= out_size) break;
            g = gn;
        }
    }
    if (partial) {
        // at most kRoundIters = 64 products below r^2 in size: |sum| < 64 r^2 -> within (-1.82 r, 2.82 r) after the reduction
        const Fr c0 = fr26::finish_sum(C0, 2), c2 = fr26::finish_sum(C2, 2);
        Fr acc[3] = {c0, Fr::zero(), c2};
        if (!CLAIM) acc[1] = sub(sub(fr26::finish_sum(Q, 2), c0), c2);
        block_sum<3>(acc, lds);
        if (threadIdx.x == 0) {
            st_fr(partial, (size_t)blockIdx.x * 3 + 0, acc[0]);
            st_fr(partial, (size_t)blockIdx.x * 3 + 1, acc[1]);
            st_fr(partial, (size_t)blockIdx.x * 3 + 2, acc[2]);
        }
    }
}

// Finishes a round that was summed without its middle coefficient: out = (c0, claim - 2 c0 - c2, c2),
// and the claim of the next round, the polynomial's value at the challenge v, replaces *claim.
template <int BLOCK>
__global__ void __launch_bounds__(BLOCK) sumcheck2_claim_final_kernel(uint32_t* out, const uint32_t* partial, unsigned nblocks,
                                                                      uint32_t* claim, const uint32_t* v) {
    __shared__ uint32_t lds9[3 * (BLOCK / 64) * 9];
    Fr acc[3];
    workgroup_totals<3, BLOCK, 2u>(acc, partial, nblocks, lds9);       // the middle slot is not written by the round kernel
    if (threadIdx.x == 0) {
        const Fr c0 = acc[0], c2 = acc[2];
        const Fr c1 = sub(sub(sub(ld_fr(claim, 0), c0), c0), c2);
        const Fr vv = ld_fr(v, 0);
        st_fr(out, 0, c0);
        st_fr(out, 1, c1);
        st_fr(out, 2, c2);
        st_fr(claim, 0, add(c0, fr26::mulc(vv, add(c1, fr26::mulc(vv, c2)))));
    }
}

// The last rounds of a two-tensor sumcheck in ONE launch: once a round has at most kBlock output
// indices, one workgroup runs all remaining rounds back to back (a barrier between rounds
// instead of a launch and a finishing kernel per round).  Round i takes its challenge from
// v_end[-(i+1)] and leaves its three sums in sums[3i .. 3i+2].
__global__ void __launch_bounds__(kBlock) sumcheck2_tail_kernel(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t rounds,
                                                                const uint32_t* v_end, uint32_t* sums) {
    __shared__ Fr lds[3 * (kBlock / 64)];
    uint32_t in = in_size;
    uint32_t out = 1;
    while (2 * out < in) out *= 2;                    // 2^(ceil(log2 in) - 1), at most kBlock
    const uint32_t g = threadIdx.x;
    for (uint32_t i = 0; i < rounds; i++) {
        Fr acc[3] = {Fr::zero(), Fr::zero(), Fr::zero()};
        if (g < out) {
            const Fr vv = ld_fr(v_end - 8 * (size_t)(i + 1), 0);
            const fr26::Limbs w1 = fr26::weight16(vv);
            const Fr a0c = ld_fr(A, g), b0c = ld_fr(B, g);
            const Fr a1c = ld_hi(A, g, out, in), b1c = ld_hi(B, g, out, in);
            acc[0] = fr26::mulc(a0c, b0c);
            acc[2] = fr26::mulc(sub(a1c, a0c), sub(b1c, b0c));
            acc[1] = sub(sub(fr26::mulc(a1c, b1c), acc[0]), acc[2]);
            const fr26::Limbs a0 = fr26::pack(a0c), b0 = fr26::pack(b0c);
            st_fr(A, g, fold1(w1, a0, fr26::sub(fr26::pack(a1c), a0)));
            st_fr(B, g, fold1(w1, b0, fr26::sub(fr26::pack(b1c), b0)));
        }
        block_sum<3>(acc, lds);
        if (threadIdx.x == 0) {
#pragma unroll
            for (int k = 0; k < 3; k++) st_fr(sums, 3 * (size_t)i + k, acc[k]);
        }
        __syncthreads();                              // folded values and lds visible to the next round
        in = out;
        out = out / 2;
    }
}

__global__ void __launch_bounds__(kBlock) sumcheck1_kernel(uint32_t* X, uint32_t* a, uint32_t* b, uint32_t in_size,
                                                           uint32_t out_size, const uint32_t* v) {
    size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (g >= out_size) return;
    const Fr Xb = ld_fr(X, g);
    const Fr Xh = ld_hi(X, g, out_size, in_size);
    const fr26::Limbs lo = fr26::pack(Xb);
    st_fr(X, g, fold1(fr26::weight16(ld_fr(v, 0)), lo, fr26::sub(fr26::pack(Xh), lo)));
    st_fr(b, g, Xb);
    st_fr(a, g, sub(Xh, Xb));
}

// ---------------------------------------------------------------- tlookup
__global__ void __launch_bounds__(kBlock) hist_kernel(uint32_t* hist, const uint32_t* vals, size_t n, int32_t low, uint32_t len) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    bool valid = false;
    uint32_t idx = 0;
    if (i < n) {
        // (v - low) is a small non-negative integer for an in-range witness; leave Montgomery form
        // and take the low limb, rejecting anything with higher limbs set.
        Fr d = fr26::from_montc(sub(ld_fr(vals, i), fr26::from_i32c(low)));
        uint32_t hi = d.v[1] | d.v[2] | d.v[3] | d.v[4] | d.v[5] | d.v[6] | d.v[7];
        valid = hi == 0 && d.v[0] < len;
        idx = d.v[0];
    }
    // Wave-level aggregation: lanes holding the same bin are counted with one atomic.  Skewed
    // witnesses (clipped activations, padding zeros) otherwise serialise on a few counters.
    // Eight leaders are tried (enough to catch any bin that holds a sizeable share of the
    // wave); whatever is left is taken to be spread out and issues plain atomics.
    const int lane = threadIdx.x & 63;
    unsigned long long todo = __ballot(valid);
    for (int it = 0; it < 8 && todo != 0ull; it++) {
        const int leader = __ffsll((long long)todo) - 1;
        const uint32_t lidx = __shfl(idx, leader, 64);
        const unsigned long long same = __ballot(valid && idx == lidx) & todo;
        const int cnt = __popcll(same);
        if (lane == leader) atomicAdd(&hist[lidx], (uint32_t)cnt);
        todo &= ~same;
    }
    if (valid && ((todo >> lane) & 1ull)) atomicAdd(&hist[idx], 1u);
}

// Large histograms.  Device-wide atomics on a table of a million counters run at a few 10^9
// per second on this part (they are resolved on the memory side of the XCDs' L2 caches), so a
// long witness is counted in LDS instead: the witness is first reduced to 32-bit indices
// (index_kernel), workgroup (g, p) then streams chunk g of the indices and counts the bins of
// range p in LDS, and writes its counters with plain stores; a last kernel adds the chunks up.
// Every chunk is read once per bin range - 4 bytes per element and range, all of it streaming.
// Activations sit on a small part of a large table, so most (chunk, bin range) pairs hold nothing:
// a first pass over the indices leaves, per chunk, the set of bin ranges that occur in it (one bit
// each, at most 64 ranges), and the counting and merging kernels skip the pairs whose bit is clear.
// 2^27 softmax scores on a 2^20-entry table: 2 of 32 ranges per chunk, 4.6 ms -> 0.6 ms.
constexpr int kHistThreads = 1024;

__global__ void __launch_bounds__(kHistThreads) hist_ranges_kernel(unsigned long long* __restrict__ mask, const int32_t* __restrict__ idx1,
                                                                   size_t n, size_t per_chunk, uint32_t lg_bins) {
    __shared__ unsigned long long any;
    if (threadIdx.x == 0) any = 0ull;
    __syncthreads();
    const size_t lo = (size_t)blockIdx.x * per_chunk;            // per_chunk is a multiple of 4
    const size_t hi = lo + per_chunk < n ? lo + per_chunk : n;
    unsigned long long m = 0ull;
    for (size_t i = lo + 4 * (size_t)threadIdx.x; i < hi; i += 4 * kHistThreads) {
        int4 v = make_int4(0, 0, 0, 0);
        if (i + 4 <= hi) {
            v = *reinterpret_cast<const int4*>(idx1 + i);
        } else {
            v.x = idx1[i];
            if (i + 1 < hi) v.y = idx1[i + 1];
            if (i + 2 < hi) v.z = idx1[i + 2];
        }
        const int vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (vv[q] >= 1) m |= 1ull << (((uint32_t)(vv[q] - 1) >> lg_bins) & 63u);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m |= __shfl_xor(m, off, 64);
    if ((threadIdx.x & 63) == 0 && m) atomicOr(&any, m);
    __syncthreads();
    if (threadIdx.x == 0) mask[blockIdx.x] = any;
}

template <int BINS>
__global__ void __launch_bounds__(kHistThreads) hist_lds_kernel(uint32_t* __restrict__ partial, const int32_t* __restrict__ idx1,
                                                                size_t n, size_t per_chunk, uint32_t len,
                                                                const unsigned long long* __restrict__ mask) {
    extern __shared__ uint32_t bins[];
    if (mask && ((mask[blockIdx.x] >> blockIdx.y) & 1ull) == 0ull) return;   // nothing of this range in this chunk
    for (int k = threadIdx.x; k < BINS; k += kHistThreads) bins[k] = 0;
    __syncthreads();
    const uint32_t base = blockIdx.y * (uint32_t)BINS;
    const size_t lo = (size_t)blockIdx.x * per_chunk;            // per_chunk is a multiple of 4
    const size_t hi = lo + per_chunk < n ? lo + per_chunk : n;
    const int lane = threadIdx.x & 63;
    for (size_t i0 = lo + 4 * (size_t)(threadIdx.x & ~63); i0 < hi; i0 += 4 * kHistThreads) {
        // a wave takes 256 consecutive indices, four per lane (the trip count is wave-uniform)
        const size_t i = i0 + 4 * (size_t)lane;
        int4 v = make_int4(0, 0, 0, 0);
        if (i + 4 <= hi) {
            v = *reinterpret_cast<const int4*>(idx1 + i);
        } else {
            if (i < hi) v.x = idx1[i];
            if (i + 1 < hi) v.y = idx1[i + 1];
            if (i + 2 < hi) v.z = idx1[i + 2];
        }
        const int vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t b = (uint32_t)(vv[q] - 1) - base;      // 0 (out of range) wraps far away
            const bool in = b < (uint32_t)BINS;
            // lanes that share a bin are counted once: up to four leaders, then plain adds
            unsigned long long todo = __ballot(in);
            for (int it = 0; it < 4 && todo != 0ull; it++) {
                const int leader = __ffsll((long long)todo) - 1;
                const uint32_t lb = __shfl(b, leader, 64);
                const unsigned long long same = __ballot(in && b == lb) & todo;
                if (lane == leader) atomicAdd(&bins[lb], (uint32_t)__popcll(same));
                todo &= ~same;
            }
            if (in && ((todo >> lane) & 1ull)) atomicAdd(&bins[b], 1u);
        }
    }
    __syncthreads();
    uint32_t* dst = partial + (size_t)blockIdx.x * len + base;
    const uint32_t live = len - base < (uint32_t)BINS ? len - base : (uint32_t)BINS;
    for (uint32_t k = threadIdx.x; k < live; k += kHistThreads) dst[k] = bins[k];
}

__global__ void __launch_bounds__(kBlock) hist_merge_kernel(uint32_t* hist, const uint32_t* partial, uint32_t chunks, uint32_t len,
                                                            const unsigned long long* __restrict__ mask, uint32_t lg_bins) {
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= len) return;
    const uint32_t range = t >> lg_bins;
    uint32_t s = 0;
    for (uint32_t g = 0; g < chunks; g++)
        if (!mask || ((mask[g] >> range) & 1ull)) s += partial[(size_t)g * len + t];
    hist[t] += s;
}

// histogram of precomputed indices (idx1 = index + 1, 0 = outside the table), short witnesses
__global__ void __launch_bounds__(kBlock) hist_index_kernel(uint32_t* hist, const int32_t* idx1, size_t n, uint32_t len) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const uint32_t j = i < n ? (uint32_t)idx1[i] : 0u;
    const bool valid = j >= 1 && j <= len;
    const uint32_t idx = j - 1;
    const int lane = threadIdx.x & 63;
    unsigned long long todo = __ballot(valid);
    for (int it = 0; it < 8 && todo != 0ull; it++) {
        const int leader = __ffsll((long long)todo) - 1;
        const uint32_t lidx = __shfl(idx, leader, 64);
        const unsigned long long same = __ballot(valid && idx == lidx) & todo;
        if (lane == leader) atomicAdd(&hist[lidx], (uint32_t)__popcll(same));
        todo &= ~same;
    }
    if (valid && ((todo >> lane) & 1ull)) atomicAdd(&hist[idx], 1u);
}

// A[i] = 1 / (S[i] + beta) read from the table instead of computed: with B[t] = 1 / (T[t] + beta)
// and S[i] = T[idx_i], A[i] = B[idx_i].  Every element is checked against T; an element that is
// outside the table or differs from its entry is counted in *mismatches and left unwritten.
__global__ void __launch_bounds__(kBlock) inverse_by_table_kernel(uint32_t* A, const uint32_t* S, const int32_t* idx1, const uint32_t* T,
                                                                   const uint32_t* B, size_t n, uint32_t len, unsigned int* mismatches) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    bool bad = false;
    if (i < n) {
        const uint32_t j = (uint32_t)idx1[i];
        bad = !(j >= 1 && j <= len);
        if (!bad) {
            const Fr s = ld_fr(S, i), t = ld_fr(T, j - 1);
            uint32_t diff = 0;
#pragma unroll
            for (int k = 0; k < 8; k++) diff |= s.v[k] ^ t.v[k];
            bad = diff != 0;
            if (!bad) st_fr(A, i, ld_fr(B, j - 1));
        }
    }
    const unsigned long long b = __ballot(bad);
    if (b != 0ull && (threadIdx.x & 63) == 0) atomicAdd(mismatches, (unsigned int)__popcll(b));
}

// ---- occupied-entry ("hot") selection for the commitment of A = B[index]
// A logUp tensor A takes only the values B[t] of the entries that occur in the witness.  Entries
// that occur at least min_count times get a slot (in table order, at most max_hot of them): the
// committer builds B[t]*G_i for those entries only and adds one table point per element; the rest
// of the elements ("cold") keep their full-width scalars.  Three small launches: hot entries per tile
// of 1024, an exclusive scan of the tile counts, slots within every tile.
constexpr int kHotTile = 1024;          // entries per workgroup: 4 per thread
// pass 1: hot entries per tile
__global__ void __launch_bounds__(kBlock) hot_count_kernel(const uint32_t* __restrict__ hist, uint32_t len, uint32_t min_count,
                                                           uint32_t* __restrict__ tile_count) {
    __shared__ uint32_t wsum[kBlock / 64];
    const uint32_t base = blockIdx.x * kHotTile + threadIdx.x * 4;
    uint32_t mine = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) mine += (base + k < len && hist[base + k] >= min_count) ? 1u : 0u;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mine += __shfl_down(mine, off, 64);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) tile_count[blockIdx.x] = wsum[0] + wsum[1] + wsum[2] + wsum[3];
}
// pass 2 (one workgroup): tile_count -> exclusive prefix, in place; info[0] = slots given
__global__ void __launch_bounds__(kBlock) hot_scan_kernel(uint32_t* tile_count, uint32_t ntiles, uint32_t max_hot, unsigned long long* info) {
    __shared__ uint32_t part[kBlock];
    const uint32_t per = (ntiles + kBlock - 1) / kBlock;
    const uint32_t t0 = threadIdx.x * per, t1 = t0 + per < ntiles ? t0 + per : ntiles;
    uint32_t mine = 0;
    for (uint32_t t = t0; t < t1; t++) mine += tile_count[t];
    part[threadIdx.x] = mine;
    __syncthreads();
    for (int off = 1; off < kBlock; off <<= 1) {
        const uint32_t add = (int)threadIdx.x >= off ? part[threadIdx.x - off] : 0u;
        __syncthreads();
        part[threadIdx.x] += add;
        __syncthreads();
    }
    uint32_t run = part[threadIdx.x] - mine;
    for (uint32_t t = t0; t < t1; t++) {
        const uint32_t c = tile_count[t];
        tile_count[t] = run;
        run += c;
    }
    if (threadIdx.x == kBlock - 1) {
        const uint32_t total = part[kBlock - 1];
        info[0] = total < max_hot ? total : max_hot;
        info[1] = 0;
    }
}
// pass 3: slots in table order; info[1] += witness elements whose entry got none
__global__ void __launch_bounds__(kBlock) hot_assign_kernel(const uint32_t* __restrict__ hist, uint32_t len, uint32_t min_count,
                                                            uint32_t max_hot, const uint32_t* __restrict__ tile_base,
                                                            int32_t* __restrict__ slot1, uint32_t* __restrict__ hot_list,
                                                            unsigned long long* info) {
    __shared__ uint32_t wsum[kBlock / 64];
    __shared__ unsigned long long wcold[kBlock / 64];
    const uint32_t base = blockIdx.x * kHotTile + threadIdx.x * 4;
    uint32_t h[4];
    uint32_t mine = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        h[k] = base + k < len ? hist[base + k] : 0u;
        mine += (base + k < len && h[k] >= min_count) ? 1u : 0u;
    }
    // exclusive prefix of `mine` over the workgroup: inclusive scan within the wave, then the waves before
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    uint32_t slot = tile_base[blockIdx.x] + incl - mine;
    for (int w = 0; w < wave; w++) slot += wsum[w];
    unsigned long long cold = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        if (base + k >= len) break;
        const bool cand = h[k] >= min_count;
        const bool hot = cand && slot < max_hot;
        slot1[base + k] = hot ? (int32_t)(slot + 1) : 0;
        if (hot) hot_list[slot] = base + k;
        if (cand) slot++;
        if (!hot) cold += h[k];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) cold += __shfl_down(cold, off, 64);
    if (lane == 0) wcold[wave] = cold;
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned long long c = wcold[0] + wcold[1] + wcold[2] + wcold[3];
        if (c) atomicAdd(&info[1], c);
    }
}
// out[i] = slot + 1 of the element's entry (0: cold entry or outside the table)
__global__ void __launch_bounds__(kBlock) hot_index_kernel(int32_t* __restrict__ out, const int32_t* __restrict__ idx1, size_t n,
                                                           const int32_t* __restrict__ slot1, uint32_t len) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const uint32_t j = (uint32_t)idx1[i];
    out[i] = (j >= 1 && j <= len) ? slot1[j - 1] : 0;
}
// out[i] = X[i] where hot1[i] == 0, zero elsewhere
__global__ void __launch_bounds__(kBlock) mask_cold_kernel(uint32_t* out, const uint32_t* X, const int32_t* __restrict__ hot1, size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, hot1[i] == 0 ? ld_fr(X, i) : Fr::zero());
}
__global__ void __launch_bounds__(kBlock) gather_fr_kernel(uint32_t* out, const uint32_t* src, const uint32_t* __restrict__ list, size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, ld_fr(src, list[i]));
}

// Index and logUp tensor in one pass: idx1[i] = (key_i - low) + 1 for a key inside the table (0
// otherwise) and A[i] = B[index].  With `cmp` (mapping lookups) the element's second component must
// equal the table's (cmp[i] == cmp_table[index], i.e. S_out = f(S_in)); an element outside the table
// or with a wrong second component is counted in *mismatches and its A left unwritten.
__global__ void __launch_bounds__(kBlock) index_inverse_kernel(int32_t* idx1, uint32_t* A, const uint32_t* key, size_t n, int32_t low,
                                                                uint32_t len, const uint32_t* B, const uint32_t* cmp,
                                                                const uint32_t* cmp_table, unsigned int* mismatches) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    bool bad = false;
    if (i < n) {
        const Fr d = fr26::from_montc(sub(ld_fr(key, i), fr26::from_i32c(low)));
        const uint32_t hi = d.v[1] | d.v[2] | d.v[3] | d.v[4] | d.v[5] | d.v[6] | d.v[7];
        const bool inside = hi == 0 && d.v[0] < len;
        idx1[i] = inside ? (int32_t)(d.v[0] + 1) : 0;
        bad = !inside;
        if (inside && cmp) {
            const Fr a = ld_fr(cmp, i), b = ld_fr(cmp_table, d.v[0]);
            uint32_t diff = 0;
#pragma unroll
            for (int k = 0; k < 8; k++) diff |= a.v[k] ^ b.v[k];
            bad = diff != 0;
        }
        if (!bad && A) st_fr(A, i, ld_fr(B, d.v[0]));
    }
    const unsigned long long b = __ballot(bad);
    if (b != 0ull && (threadIdx.x & 63) == 0) atomicAdd(mismatches, (unsigned int)__popcll(b));
}

// The same pass over an INTEGER witness (the tensors a driver would first embed with FrTensor::get_data): besides the
// index, the check and A it leaves the witness itself as field elements - S[i] = key_i for a range lookup,
// S[i] = key_i + r * cmp_i (the combined witness, src/tlookup.cu:407-410) for a mapping lookup, whose table of second
// components is an integer table too.  8 bytes per element are read where embedding two tensors, indexing them and
// combining them move 270.
constexpr int kEmbedPerThread = 4;
__global__ void __launch_bounds__(kBlock) index_embed_i32_kernel(int32_t* idx1, uint32_t* A, uint32_t* S, const int32_t* __restrict__ key,
                                                                  const int32_t* __restrict__ cmp, size_t n, int32_t low, uint32_t len,
                                                                  const uint32_t* B, const int32_t* __restrict__ cmp_table, const uint32_t* r,
                                                                  unsigned int* mismatches) {
    // The witness element is ONE reduction of a two-term sum of plain integers against constants that carry the factors:
    // key * W + cmp * Wr with W = 16 * 2^512 and Wr = 16 * r * 2^512 (mod the modulus) reduces to (key + r * cmp) * 2^256,
    // the memory form.  An integer is two signed limbs, so a term is 20 multiply-adds.
    const fr26::Limbs w = fr26::weight16(Fr::rr());
    fr26::Limbs wr;
    if (cmp) wr = fr26::weight16(fr26::mulc(ld_fr(r, 0), Fr::rr()));
    auto mac_int = [](fr26::Acc& C, const fr26::Limbs& x, int32_t v) {
        const int64_t l0 = (int64_t)(v & (int32_t)fr26::MASK), l1 = (int64_t)(v >> fr26::W);
#pragma unroll
        for (int j = 0; j < fr26::N; j++) {
            C.c[j] += (int64_t)x.v[j] * l0;
            C.c[j + 1] += (int64_t)x.v[j] * l1;
        }
    };
    const size_t base = (size_t)blockIdx.x * (kBlock * kEmbedPerThread) + threadIdx.x;
    unsigned int nbad = 0;
#pragma unroll
    for (int q = 0; q < kEmbedPerThread; q++) {
        const size_t i = base + (size_t)q * kBlock;
        bool bad = false;
        if (i < n) {
            const int32_t k = key[i];
            const int64_t d = (int64_t)k - (int64_t)low;
            const bool inside = d >= 0 && d < (int64_t)len;
            idx1[i] = inside ? (int32_t)(d + 1) : 0;
            bad = !inside;
            fr26::Acc C;
            fr26::acc_zero(C);
            mac_int(C, w, k);
            if (cmp) {
                const int32_t c = cmp[i];
                if (inside) bad = c != cmp_table[d];
                mac_int(C, wr, c);
            }
            // |sum| < 2^32 * modulus: the reduced value plus one modulus lies in [0, 2 * modulus)
            st_fr(S, i, fr26::unpack(fr26::canon(fr26::reduce(C, 1), 1)));
            if (!bad && A) st_fr(A, i, ld_fr(B, (size_t)d));
        }
        nbad += (unsigned int)__popcll(__ballot(bad));
    }
    if (nbad != 0 && (threadIdx.x & 63) == 0) atomicAdd(mismatches, nbad);
}

// out[i] = (v_i - low) + 1 for an in-range value, 0 otherwise
__global__ void __launch_bounds__(kBlock) index_kernel(int32_t* out, const uint32_t* vals, size_t n, int32_t low, uint32_t len) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    Fr d = fr26::from_montc(sub(ld_fr(vals, i), fr26::from_i32c(low)));
    uint32_t hi = d.v[1] | d.v[2] | d.v[3] | d.v[4] | d.v[5] | d.v[6] | d.v[7];
    out[i] = (hi == 0 && d.v[0] < len) ? (int32_t)(d.v[0] + 1) : 0;
}

__global__ void __launch_bounds__(kBlock) tl_table_kernel(uint32_t* T, const uint32_t* map, const uint32_t* r, int32_t low, uint32_t len) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= len) return;
    Fr t = add(fr26::from_u32c((uint32_t)i), fr26::from_i32c(low));
    if (map) t = add(t, fr26::mulc(ld_fr(map, i), ld_fr(r, 0)));
    st_fr(T, i, t);
}

__global__ void __launch_bounds__(kBlock) tl_poly_kernel(const uint32_t* A, const uint32_t* S, const uint32_t* beta,
                                                         uint32_t* o0, uint32_t* o1, uint32_t* o2, size_t n_out) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= n_out) return;
    const Fr c00 = ld_fr(A, t);
    const Fr c01 = sub(ld_fr(A, t + n_out), c00);
    const Fr s0 = ld_fr(S, t);
    const Fr c10 = beta ? add(s0, ld_fr(beta, 0)) : s0;
    const Fr c11 = sub(ld_fr(S, t + n_out), s0);
    st_fr(o0, t, fr26::mulc(c00, c10));
    st_fr(o1, t, add(fr26::mulc(c01, c10), fr26::mulc(c00, c11)));
    st_fr(o2, t, fr26::mulc(c01, c11));
}

__global__ void __launch_bounds__(kBlock) tl_poly_sum_kernel(const uint32_t* A, uint32_t* o0, uint32_t* o1, size_t n_out) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= n_out) return;
    const Fr a0 = ld_fr(A, t);
    st_fr(o0, t, a0);
    st_fr(o1, t, sub(ld_fr(A, t + n_out), a0));
}

// 5 sums per round: eq-weighted coefficients of (A0+tA1)(S0+beta+tS1), and plain sums of A0, A1.
// e*A0 and e*A1 are reduced products; the three second-level products are accumulated
// double-width over the thread's iterations and reduced once.  This thread's share (the indices
// t = first, first + stride, ...; at most kLogUpIters of them) is left in acc[0..4].
__device__ __forceinline__ void tl_round_thread_sums(Fr* acc, const uint32_t* A, const uint32_t* S, const uint32_t* beta,
                                                     const uint32_t* eq, size_t n_out, size_t first, size_t stride) {
    const Fr btc = beta ? ld_fr(beta, 0) : Fr::zero();
    const fr26::Limbs bt = fr26::pack(btc);
    fr26::Acc C0, Q, C2;
    fr26::acc_zero(C0);
    fr26::acc_zero(Q);
    fr26::acc_zero(C2);
    // plain sums of A's halves as limb-wise sums (no carries: 16 terms of 26-bit limbs)
    fr26::Limbs sa0, sa1;
#pragma unroll
    for (int k = 0; k < fr26::N; k++) sa0.v[k] = sa1.v[k] = 0;
    for (size_t t = first; t < n_out; t += stride) {
        // operands are consumed as early as possible so that few of them are live beside the
        // three double-width accumulators
        const fr26::Limbs e16 = fr26::pack16(ld_fr(eq, t));         // limbs < 2^30: one product per column set
        const fr26::Limbs a0 = ld_l26(A, t);
        const fr26::Limbs s0r = ld_l26(S, t);
        const fr26::Limbs s1 = fr26::sub(ld_l26(S, t + n_out), s0r);   // signed
        const fr26::Limbs s0 = fr26::add(s0r, bt);                   // value < 2r, limbs < 2^27
        fr26::Acc T;
        fr26::acc_zero(T);
        fr26::mac(T, e16, a0);
        const fr26::Limbs ea0 = fr26::reduce(T, 0);                  // (0, 1.46 r)
        fr26::mac(C0, ea0, s0);
        const fr26::Limbs d1 = fr26::sub(ld_l26(A, t + n_out), a0);  // a1 - a0, signed
        sa0 = fr26::add(sa0, a0);
        sa1 = fr26::add(sa1, d1);
        fr26::acc_zero(T);
        fr26::mac(T, e16, d1);
        const fr26::Limbs ea1 = fr26::reduce(T, 1);                  // e*(a1-a0) in (0.54 r, 2.46 r)
        fr26::mac(C2, ea1, s1);
        // middle coefficient by Karatsuba: e*a0*s1 + e*(a1-a0)*s0 = (e*a1)*(s0+s1) - c0 - c2,
        // so Q accumulates the value at t = 1 with one product instead of two
        fr26::mac(Q, fr26::add(ea0, ea1), fr26::add(s0, s1));        // (0.54 r, 3.92 r) * (-r, 3r)
    }
    // per iteration |Q| grows by at most 3.92 * 3 r^2 = 11.8 r^2; 16 iterations -> below 189 r^2,
    // i.e. within 5.4 r of zero after the reduction: finish_sum's window of 34 r holds with lo_r = 6
    const Fr c0 = fr26::finish_sum(C0, 4), c2 = fr26::finish_sum(C2, 4), q1 = fr26::finish_sum(Q, 6);
    acc[0] = c0;
    acc[1] = sub(sub(q1, c0), c2);
    acc[2] = c2;
    acc[3] = fr26::limb_sum_to_fr(sa0, 0);
    acc[4] = fr26::limb_sum_to_fr(sa1, 16);
}
__global__ void __launch_bounds__(kBlock, 2) tl_round_kernel(const uint32_t* A, const uint32_t* S, const uint32_t* beta,
                                                          const uint32_t* eq, size_t n_out, uint32_t* partial) {
    __shared__ Fr lds[5 * (kBlock / 64)];
    Fr acc[5];
    tl_round_thread_sums(acc, A, S, beta, eq, n_out, (size_t)blockIdx.x * kBlock + threadIdx.x, (size_t)gridDim.x * kBlock);
    block_sum<5>(acc, lds);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 5; k++) st_fr(partial, (size_t)blockIdx.x * 5 + k, acc[k]);
    }
}

// the coefficient sums of (m0 + t m1)(B0 + t B1) over this thread's indices, left in acc[0..2]
__device__ __forceinline__ void tl_mb_thread_sums(Fr* acc, const uint32_t* m, const uint32_t* B, size_t n_out, size_t first, size_t stride) {
    fr26::Acc C0, Q, C2;
    fr26::acc_zero(C0);
    fr26::acc_zero(Q);
    fr26::acc_zero(C2);
    for (size_t t = first; t < n_out; t += stride) {
        const fr26::Limbs m0 = ld_l26(m, t), b0 = ld_l26(B, t);
        const fr26::Limbs mh = ld_l26(m, t + n_out), bh = ld_l26(B, t + n_out);
        const fr26::Limbs m1 = fr26::sub(mh, m0), b1 = fr26::sub(bh, b0);
        fr26::mac(C0, m0, b0);
        fr26::mac(Q, mh, bh);             // value at t = 1; the middle coefficient is Q - C0 - C2
        fr26::mac(C2, m1, b1);
    }
    const Fr c0 = fr26::finish_sum(C0, 2), c2 = fr26::finish_sum(C2, 2), q1 = fr26::finish_sum(Q, 2);
    acc[0] = c0;
    acc[1] = sub(sub(q1, c0), c2);
    acc[2] = c2;
}
__global__ void __launch_bounds__(kBlock) tl_mb_kernel(const uint32_t* m, const uint32_t* B, size_t n_out, uint32_t* partial) {
    __shared__ Fr lds[3 * (kBlock / 64)];
    Fr acc[3];
    tl_mb_thread_sums(acc, m, B, n_out, (size_t)blockIdx.x * kBlock + threadIdx.x, (size_t)gridDim.x * kBlock);
    block_sum<3>(acc, lds);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 3; k++) st_fr(partial, (size_t)blockIdx.x * 3 + k, acc[k]);
    }
}

// One round of the table side of a logUp proof (src/tlookup.cu:153-190: the terms over B, T and m of
// phase 2) as ONE launch: the five sums over (B, T + beta) with the round's weights, the three sums
// over (m, B), then the fold of the three tensors by the round's challenge - every index is read and
// folded by the thread that owns it, so the three steps need no barrier between them.  One finishing
// kernel adds up the workgroups' eight sums.  (The round was five launches: two sum kernels, their two
// finishing kernels and the fold.)
__global__ void __launch_bounds__(kBlock, 2) tl_table_round_kernel(uint32_t* B, uint32_t* T, uint32_t* m, const uint32_t* beta,
                                                                const uint32_t* eq, size_t n_out, const uint32_t* v, uint32_t* partial) {
    __shared__ Fr lds[8 * (kBlock / 64)];
    const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x, stride = (size_t)gridDim.x * kBlock;
    // the two groups of sums one after the other, each handed to the workgroup's sum before the next starts,
    // so that neither is held in registers beside the other's accumulators
    {
        Fr acc3[3];
        tl_mb_thread_sums(acc3, m, B, n_out, first, stride);
        block_sum<3>(acc3, lds);
        if (threadIdx.x == 0) {
#pragma unroll
            for (int k = 0; k < 3; k++) st_fr(partial, (size_t)blockIdx.x * 8 + 5 + k, acc3[k]);
        }
        __syncthreads();                   // lds is reused below
    }
    {
        Fr acc5[5];
        tl_round_thread_sums(acc5, B, T, beta, eq, n_out, first, stride);
        block_sum<5>(acc5, lds);
        if (threadIdx.x == 0) {
#pragma unroll
            for (int k = 0; k < 5; k++) st_fr(partial, (size_t)blockIdx.x * 8 + k, acc5[k]);
        }
    }
    const fr26::Limbs w1 = fr26::weight16(ld_fr(v, 0));
    auto fold_one = [&](uint32_t* X, size_t t) __attribute__((always_inline)) {
        const fr26::Limbs lo = ld_l26(X, t);
        st_fr(X, t, fold1(w1, lo, fr26::sub(ld_l26(X, t + n_out), lo)));
    };
    for (size_t t = first; t < n_out; t += stride) {
        fold_one(B, t);
        fold_one(T, t);
        fold_one(m, t);
    }
}

// eq table by doubling: level j turns e[0..2^j) into e[0..2^(j+1)) with
// e[i + 2^j] = e[i]*u_j, e[i] = e[i] - e[i + 2^j]   (= e[i]*(1-u_j))
__global__ void __launch_bounds__(kBlock) eq_level_kernel(uint32_t* e, const uint32_t* u, uint32_t j) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    size_t half = (size_t)1 << j;
    if (i >= half) return;
    const Fr lo = ld_fr(e, i);
    const Fr hi = fr26::mulc(lo, ld_fr(u, j));
    st_fr(e, i + half, hi);
    st_fr(e, i, sub(lo, hi));
}
__global__ void eq_init_kernel(uint32_t* e) {
    if (threadIdx.x == 0 && blockIdx.x == 0) st_fr(e, 0, Fr::one());
}
__global__ void __launch_bounds__(kBlock) eq_halve_kernel(uint32_t* e, size_t n_out) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_out) return;
    st_fr(e, i, add(ld_fr(e, i), ld_fr(e, i + n_out)));
}

struct PtrPack { uint32_t* p[8]; };
__global__ void __launch_bounds__(kBlock) fold_msb_multi_kernel(PtrPack pk, uint32_t k, size_t n_out, const uint32_t* v) {
    size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (g >= n_out) return;
    const fr26::Limbs w1 = fr26::weight16(ld_fr(v, 0));
    for (uint32_t j = 0; j < k; j++) {
        uint32_t* X = pk.p[j];
        const fr26::Limbs lo = ld_l26(X, g);
        st_fr(X, g, fold1(w1, lo, fr26::sub(ld_l26(X, g + n_out), lo)));
    }
}

// enough workgroups that no thread runs more than `iters` iterations, at most one element per
// thread while that still leaves every CU a few workgroups
static unsigned reduce_grid(size_t n, int iters = kRoundIters) {
    unsigned nb = blocks_for(n);
    unsigned cap = kNumCU * 4;
    if (nb <= cap) return nb;
    unsigned need = blocks_for(n, kBlock * iters);
    return need > cap ? need : cap;
}
// the logUp round sums grow faster per iteration (see tl_round_kernel)
constexpr int kLogUpIters = 16;

// ---------------------------------------------------------------- entry point that allocates nothing
// Partial sums of grape_sumcheck_round2_noalloc: a fixed array in the code object instead of a
// pool buffer, sized for the largest round that entry point accepts (kNoAllocMaxOut output indices
// -> at most kNoAllocMaxBlocks workgroups leaving three 32-byte sums each: 384 KiB per GPU, held
// until the process ends).  Host code never uses this name as an address: it asks the runtime for
// the array's device address once per device (noalloc_scratch) and passes that to the kernels.
constexpr uint32_t kNoAllocMaxOut = 1u << 26;
constexpr unsigned kNoAllocMaxBlocks = kNoAllocMaxOut / (kBlock * kRoundIters);
static __device__ __align__(256) uint32_t scratch[(size_t)kNoAllocMaxBlocks * 3 * 8 + kFoldTableBytes / 4];

constexpr int kMaxDevices = 64;
static uint32_t* g_noalloc_ptr[kMaxDevices] = {nullptr};
static std::mutex g_noalloc_mu;

// device address of `scratch` on the current device (looked up once per device)
static int noalloc_scratch(uint32_t** out) {
    int dev = -1;
    GRAPE_HIP_CHECK(hipGetDevice(&dev));
    GRAPE_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index out of range");
    std::lock_guard<std::mutex> lock(g_noalloc_mu);
    if (!g_noalloc_ptr[dev]) {
        void* p = nullptr;
        GRAPE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        GRAPE_REQUIRE(p != nullptr, "no device address for the static scratch array");
        g_noalloc_ptr[dev] = (uint32_t*)p;
    }
    *out = g_noalloc_ptr[dev];
    return GRAPE_OK;
}
// called by grape_init with its device current, so that the entry point's first call finds the
// address already there
int noalloc_setup() {
    uint32_t* p;
    return noalloc_scratch(&p);
}

}  // namespace grape

using namespace grape;

// defined in fr_kernels.hip
extern "C" int grape_fr_shift_inverse(uint32_t*, const uint32_t*, const uint32_t*, size_t, grape_stream_t);

template <bool COEFFS>
static int sumcheck2_impl(uint32_t* A, uint32_t* B, uint32_t* a, uint32_t* b, uint32_t* c, uint32_t in_size, uint32_t out_size,
                          const uint32_t* v, uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(B); CHECK_PTR16(v);
    GRAPE_REQUIRE(out_size >= 1 && in_size >= out_size && in_size <= 2 * out_size, "need out_size <= in_size <= 2*out_size");
    hipStream_t s = as_stream(st);
    unsigned nb = reduce_grid(out_size);
    uint32_t* partial = nullptr;
    if (sums) CHECK_PTR16(sums);
    // the partial sums, then the table of the challenge's multiples
    const size_t partial_bytes = (size_t)nb * 3 * 32;
    void* ws;
    int rc = scratch_get(kSlotReduce, partial_bytes + kFoldTableBytes, &ws, s);
    if (rc) return rc;
    if (sums) partial = (uint32_t*)ws;
    if (out_size >= kTableFoldMinOut) {
        int32_t* tab = (int32_t*)((char*)ws + partial_bytes);
        fold_tables_kernel<<<1, 64, 0, s>>>(tab, v, 1);
        sumcheck2_kernel<COEFFS, true><<<nb, kBlock, 0, s>>>(A, B, a, b, c, in_size, out_size, v, tab, partial);
    } else {
        sumcheck2_kernel<COEFFS, false><<<nb, kBlock, 0, s>>>(A, B, a, b, c, in_size, out_size, v, nullptr, partial);
    }
    if (sums) launch_final_sum<3>(sums, partial, nb, s);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

extern "C" {

int grape_sumcheck_round2_tail(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t rounds, const uint32_t* v_end, uint32_t* sums,
                               grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(B); CHECK_PTR16(v_end); CHECK_PTR16(sums);
    if (rounds == 0) return GRAPE_OK;
    GRAPE_REQUIRE(in_size >= 1 && in_size <= 2u * kBlock, "tail rounds start at 2 * 256 elements or fewer");
    uint32_t lg = 0;
    while ((1u << lg) < in_size) lg++;
    GRAPE_REQUIRE(rounds <= (lg ? lg : 1), "more rounds than variables");
    sumcheck2_tail_kernel<<<1, kBlock, 0, as_stream(st)>>>(A, B, in_size, rounds, v_end, sums);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_sumcheck_round2(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t out_size, const uint32_t* v, uint32_t* sums, grape_stream_t st) {
    GRAPE_REQUIRE(sums != nullptr, "d_sums is required");
    return sumcheck2_impl<false>(A, B, nullptr, nullptr, nullptr, in_size, out_size, v, sums, st);
}
int grape_sumcheck_round2_claim(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t out_size, const uint32_t* v, uint32_t* claim,
                                uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(B); CHECK_PTR16(v); CHECK_PTR16(claim); CHECK_PTR16(sums);
    GRAPE_REQUIRE(out_size >= 1 && in_size >= out_size && in_size <= 2 * out_size, "need out_size <= in_size <= 2*out_size");
    hipStream_t s = as_stream(st);
    const unsigned nb = reduce_grid(out_size);
    const size_t partial_bytes = (size_t)nb * 3 * 32;
    void* ws;
    int rc = scratch_get(kSlotReduce, partial_bytes + kFoldTableBytes, &ws, s);
    if (rc) return rc;
    uint32_t* partial = (uint32_t*)ws;
    if (out_size >= kTableFoldMinOut) {
        int32_t* tab = (int32_t*)((char*)ws + partial_bytes);
        fold_tables_kernel<<<1, 64, 0, s>>>(tab, v, 1);
        sumcheck2_kernel<false, true, true><<<nb, kBlock, 0, s>>>(A, B, nullptr, nullptr, nullptr, in_size, out_size, v, tab, partial);
    } else {
        sumcheck2_kernel<false, false, true><<<nb, kBlock, 0, s>>>(A, B, nullptr, nullptr, nullptr, in_size, out_size, v, nullptr, partial);
    }
    if (nb >= kFinalWideMin) sumcheck2_claim_final_kernel<kFinalBlock><<<1, kFinalBlock, 0, s>>>(sums, partial, nb, claim, v);
    else sumcheck2_claim_final_kernel<kBlock><<<1, kBlock, 0, s>>>(sums, partial, nb, claim, v);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_sumcheck_round2_noalloc(uint32_t* A, uint32_t* B, uint32_t in_size, uint32_t out_size, const uint32_t* v, uint32_t* sums,
                                  grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(B); CHECK_PTR16(v); CHECK_PTR16(sums);
    GRAPE_REQUIRE(out_size >= 1 && in_size >= out_size && in_size <= 2 * out_size, "need out_size <= in_size <= 2*out_size");
    if (out_size > kNoAllocMaxOut) {
        set_error("grape_sumcheck_round2_noalloc: out_size %u exceeds the limit of %u output indices of the static scratch array "
                  "(use grape_sumcheck_round2)", out_size, kNoAllocMaxOut);
        return GRAPE_EINVAL;
    }
    uint32_t* partial = nullptr;
    int rc = noalloc_scratch(&partial);
    if (rc) return rc;
    hipStream_t s = as_stream(st);
    const unsigned nb = reduce_grid(out_size);            // <= kNoAllocMaxBlocks for out_size <= kNoAllocMaxOut
    GRAPE_REQUIRE(nb <= kNoAllocMaxBlocks, "grid exceeds the static scratch array");
    // every workgroup writes its three partial sums and the finishing kernel reads exactly those, so
    // nothing of the previous call's contents is read and nothing has to be cleared
    if (out_size >= kTableFoldMinOut) {
        int32_t* tab = (int32_t*)(partial + (size_t)kNoAllocMaxBlocks * 3 * 8);   // behind the partial sums, rewritten by every call
        fold_tables_kernel<<<1, 64, 0, s>>>(tab, v, 1);
        sumcheck2_kernel<false, true><<<nb, kBlock, 0, s>>>(A, B, nullptr, nullptr, nullptr, in_size, out_size, v, tab, partial);
    } else {
        sumcheck2_kernel<false, false><<<nb, kBlock, 0, s>>>(A, B, nullptr, nullptr, nullptr, in_size, out_size, v, nullptr, partial);
    }
    launch_final_sum<3>(sums, partial, nb, s);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_sumcheck_round2_coeffs(uint32_t* A, uint32_t* B, uint32_t* a, uint32_t* b, uint32_t* c, uint32_t in_size,
                                 uint32_t out_size, const uint32_t* v, uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(a); CHECK_PTR16(b); CHECK_PTR16(c);
    return sumcheck2_impl<true>(A, B, a, b, c, in_size, out_size, v, sums, st);
}
int grape_sumcheck_round1(uint32_t* X, uint32_t* a, uint32_t* b, uint32_t in_size, uint32_t out_size, const uint32_t* v, grape_stream_t st) {
    CHECK_PTR16(X); CHECK_PTR16(a); CHECK_PTR16(b); CHECK_PTR16(v);
    GRAPE_REQUIRE(out_size >= 1 && in_size >= out_size && in_size <= 2 * out_size, "need out_size <= in_size <= 2*out_size");
    sumcheck1_kernel<<<blocks_for(out_size), kBlock, 0, as_stream(st)>>>(X, a, b, in_size, out_size, v);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

// LDS counting of n >= 2^20 precomputed indices (see hist_lds_kernel)
static int hist_lds_from_index(uint32_t* hist, const int32_t* idx, size_t n, uint32_t len, hipStream_t s) {
    // 32768 bins (128 KiB) per workgroup when the device grants that much dynamic LDS, else 16384
    static int bins = 0;
    if (bins == 0) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&hist_lds_kernel<32768>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 32768 * 4);
        if (e == hipSuccess) {
            bins = 32768;
        } else {
            (void)hipGetLastError();
            bins = 16384;
        }
    }
    const uint32_t ranges = (len + (uint32_t)bins - 1) / (uint32_t)bins;
    // chunks: enough workgroups to fill the chip, partial counters capped at 1 GiB
    size_t chunks = 256;
    while (chunks > 1 && chunks * (size_t)len * 4 > ((size_t)1 << 30)) chunks /= 2;
    while (chunks > 1 && n / chunks < ((size_t)1 << 16)) chunks /= 2;
    size_t per_chunk = (n + chunks - 1) / chunks;
    per_chunk = (per_chunk + 3) & ~(size_t)3;
    void* partial;
    const size_t partial_bytes = (chunks * (size_t)len * 4 + 7) & ~(size_t)7;
    int rc = scratch_get(kSlotHistPart, partial_bytes + chunks * sizeof(unsigned long long), &partial, s);
    if (rc) return rc;
    const uint32_t lg_bins = bins == 32768 ? 15u : 14u;
    unsigned long long* mask = nullptr;                    // which ranges occur in which chunk: worth a pass when there are several
    if (ranges >= 2 && ranges <= 64) {
        mask = (unsigned long long*)((char*)partial + partial_bytes);
        hist_ranges_kernel<<<(unsigned)chunks, kHistThreads, 0, s>>>(mask, idx, n, per_chunk, lg_bins);
    }
    const dim3 grid((unsigned)chunks, ranges);
    if (bins == 32768)
        hist_lds_kernel<32768><<<grid, kHistThreads, 32768 * 4, s>>>((uint32_t*)partial, idx, n, per_chunk, len, mask);
    else
        hist_lds_kernel<16384><<<grid, kHistThreads, 16384 * 4, s>>>((uint32_t*)partial, idx, n, per_chunk, len, mask);
    GRAPE_LAUNCH_CHECK();
    hist_merge_kernel<<<blocks_for(len), kBlock, 0, s>>>(hist, (const uint32_t*)partial, (uint32_t)chunks, len, mask, lg_bins);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_hist(uint32_t* hist, const uint32_t* vals, size_t n, int32_t low, uint32_t len, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    GRAPE_REQUIRE(hist != nullptr && len > 0, "bad histogram buffer");
    CHECK_PTR16(vals);
    hipStream_t s = as_stream(st);
    if (n < ((size_t)1 << 20)) {
        hist_kernel<<<blocks_for(n), kBlock, 0, s>>>(hist, vals, n, low, len);
        GRAPE_LAUNCH_CHECK();
        return GRAPE_OK;
    }
    void* idx;
    int rc = scratch_get(kSlotHistIdx, n * 4, &idx, s);
    if (rc) return rc;
    index_kernel<<<blocks_for(n), kBlock, 0, s>>>((int32_t*)idx, vals, n, low, len);
    GRAPE_LAUNCH_CHECK();
    return hist_lds_from_index(hist, (const int32_t*)idx, n, len, s);
}

int grape_tlookup_hist_index(uint32_t* hist, const int32_t* idx1, size_t n, uint32_t len, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    GRAPE_REQUIRE(hist != nullptr && idx1 != nullptr && len > 0, "bad arguments");
    GRAPE_REQUIRE((reinterpret_cast<uintptr_t>(idx1) & 15) == 0, "idx1 must be 16-byte aligned");
    hipStream_t s = as_stream(st);
    if (n < ((size_t)1 << 20)) {
        hist_index_kernel<<<blocks_for(n), kBlock, 0, s>>>(hist, idx1, n, len);
        GRAPE_LAUNCH_CHECK();
        return GRAPE_OK;
    }
    return hist_lds_from_index(hist, idx1, n, len, s);
}

int grape_tlookup_inverse_by_table(uint32_t* A, const uint32_t* S, const int32_t* idx1, const uint32_t* T, const uint32_t* B, size_t n,
                                   uint32_t len, size_t* mismatches, grape_stream_t st) {
    GRAPE_REQUIRE(mismatches != nullptr && idx1 != nullptr && len > 0, "bad arguments");
    *mismatches = 0;
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(A); CHECK_PTR16(S); CHECK_PTR16(T); CHECK_PTR16(B);
    hipStream_t s = as_stream(st);
    void* cnt;
    int rc = scratch_get(kSlotMisc, 64, &cnt, s);
    if (rc) return rc;
    rc = zero_fill(cnt, sizeof(unsigned int), s);
    if (rc) return rc;
    inverse_by_table_kernel<<<blocks_for(n), kBlock, 0, s>>>(A, S, idx1, T, B, n, len, (unsigned int*)cnt);
    GRAPE_LAUNCH_CHECK();
    unsigned int h = 0;
    GRAPE_HIP_CHECK(hipMemcpyAsync(&h, cnt, sizeof h, hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    *mismatches = h;
    return GRAPE_OK;
}

int grape_tlookup_index_inverse_nowait(int32_t* idx1, uint32_t* A, const uint32_t* key, size_t n, int32_t low, uint32_t len,
                                       const uint32_t* B, const uint32_t* cmp, const uint32_t* cmp_table, uint32_t* d_mismatches,
                                       grape_stream_t st) {
    GRAPE_REQUIRE(d_mismatches != nullptr && idx1 != nullptr && len > 0, "bad arguments");
    hipStream_t s = as_stream(st);
    int rc = zero_fill(d_mismatches, sizeof(uint32_t), s);
    if (rc) return rc;
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(key);
    if (A) { CHECK_PTR16(A); CHECK_PTR16(B); }       // A == nullptr: indices and the count only
    GRAPE_REQUIRE((cmp == nullptr) == (cmp_table == nullptr), "cmp and cmp_table go together");
    if (cmp) { CHECK_PTR16(cmp); CHECK_PTR16(cmp_table); }
    index_inverse_kernel<<<blocks_for(n), kBlock, 0, s>>>(idx1, A, key, n, low, len, B, cmp, cmp_table, (unsigned int*)d_mismatches);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_index_embed_i32_nowait(int32_t* idx1, uint32_t* A, uint32_t* S, const int32_t* key, const int32_t* cmp, size_t n, int32_t low,
                                         uint32_t len, const uint32_t* B, const int32_t* cmp_table, const uint32_t* r, uint32_t* d_mismatches,
                                         grape_stream_t st) {
    GRAPE_REQUIRE(d_mismatches != nullptr && idx1 != nullptr && len > 0, "bad arguments");
    hipStream_t s = as_stream(st);
    int rc = zero_fill(d_mismatches, sizeof(uint32_t), s);
    if (rc) return rc;
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(S);
    GRAPE_REQUIRE(key != nullptr, "null witness");
    if (A) { CHECK_PTR16(A); CHECK_PTR16(B); }       // A == nullptr: no logUp tensor written
    GRAPE_REQUIRE((cmp == nullptr) == (cmp_table == nullptr) && (cmp == nullptr) == (r == nullptr), "cmp, cmp_table and r go together");
    if (r) CHECK_PTR16(r);
    index_embed_i32_kernel<<<blocks_for(n, kBlock * kEmbedPerThread), kBlock, 0, s>>>(idx1, A, S, key, cmp, n, low, len, B, cmp_table, r,
                                                                                     (unsigned int*)d_mismatches);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_index_inverse(int32_t* idx1, uint32_t* A, const uint32_t* key, size_t n, int32_t low, uint32_t len,
                                const uint32_t* B, const uint32_t* cmp, const uint32_t* cmp_table, size_t* mismatches,
                                grape_stream_t st) {
    GRAPE_REQUIRE(mismatches != nullptr && idx1 != nullptr && len > 0, "bad arguments");
    *mismatches = 0;
    if (n == 0) return GRAPE_OK;
    hipStream_t s = as_stream(st);
    void* cnt;
    int rc = scratch_get(kSlotMisc, 64, &cnt, s);
    if (rc) return rc;
    rc = grape_tlookup_index_inverse_nowait(idx1, A, key, n, low, len, B, cmp, cmp_table, (uint32_t*)cnt, st);
    if (rc) return rc;
    unsigned int h = 0;
    GRAPE_HIP_CHECK(hipMemcpyAsync(&h, cnt, sizeof h, hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    *mismatches = h;
    return GRAPE_OK;
}

int grape_tlookup_index(int32_t* out, const uint32_t* vals, size_t n, int32_t low, uint32_t len, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    GRAPE_REQUIRE(out != nullptr && len > 0, "bad arguments");
    CHECK_PTR16(vals);
    index_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, vals, n, low, len);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_hot_select(const uint32_t* hist, uint32_t len, uint32_t min_count, uint32_t max_hot, int32_t* slot1,
                             uint32_t* hot_list, uint64_t* info, grape_stream_t st) {
    GRAPE_REQUIRE(hist != nullptr && slot1 != nullptr && hot_list != nullptr && info != nullptr && len > 0, "bad arguments");
    GRAPE_REQUIRE(min_count >= 1, "min_count must be at least 1");
    hipStream_t s = as_stream(st);
    const uint32_t ntiles = (len + kHotTile - 1) / kHotTile;
    void* ws;
    int rc = scratch_get(kSlotMisc, 64 + sizeof(uint32_t) * (size_t)ntiles, &ws, s);
    if (rc) return rc;
    unsigned long long* d_info = (unsigned long long*)ws;
    uint32_t* tiles = (uint32_t*)((char*)ws + 64);
    hot_count_kernel<<<ntiles, kBlock, 0, s>>>(hist, len, min_count, tiles);
    hot_scan_kernel<<<1, kBlock, 0, s>>>(tiles, ntiles, max_hot, d_info);
    hot_assign_kernel<<<ntiles, kBlock, 0, s>>>(hist, len, min_count, max_hot, tiles, slot1, hot_list, d_info);
    GRAPE_LAUNCH_CHECK();
    GRAPE_HIP_CHECK(hipMemcpyAsync(info, d_info, 2 * sizeof(uint64_t), hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    return GRAPE_OK;
}

// what a slot assignment made for an earlier witness leaves uncovered in this one
__global__ void __launch_bounds__(kBlock) hot_coverage_kernel(const uint32_t* __restrict__ hist, uint32_t len, const int32_t* __restrict__ slot1,
                                                              unsigned long long* info) {
    __shared__ unsigned long long part[kBlock / 64];
    unsigned long long cold = 0;
    for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < len; t += gridDim.x * kBlock)
        if (slot1[t] == 0) cold += hist[t];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) cold += __shfl_xor(cold, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = cold;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long sum = 0;
        for (int w = 0; w < kBlock / 64; w++) sum += part[w];
        if (sum) atomicAdd(info, sum);               // one atomic per workgroup
    }
}
int grape_tlookup_hot_coverage(const uint32_t* hist, uint32_t len, const int32_t* slot1, uint64_t* cold_elements, grape_stream_t st) {
    GRAPE_REQUIRE(hist != nullptr && slot1 != nullptr && cold_elements != nullptr && len > 0, "bad arguments");
    hipStream_t s = as_stream(st);
    void* ws;
    int rc = scratch_get(kSlotMisc, 64, &ws, s);
    if (rc) return rc;
    rc = zero_fill(ws, 8, s);
    if (rc) return rc;
    unsigned nb = blocks_for(len);
    if (nb > 256) nb = 256;
    hot_coverage_kernel<<<nb, kBlock, 0, s>>>(hist, len, slot1, (unsigned long long*)ws);
    GRAPE_LAUNCH_CHECK();
    GRAPE_HIP_CHECK(hipMemcpyAsync(cold_elements, ws, sizeof(uint64_t), hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    return GRAPE_OK;
}

int grape_tlookup_hot_index(int32_t* out, const int32_t* idx1, size_t n, const int32_t* slot1, uint32_t len, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    GRAPE_REQUIRE(out != nullptr && idx1 != nullptr && slot1 != nullptr && len > 0, "bad arguments");
    hot_index_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, idx1, n, slot1, len);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_fr_mask_cold(uint32_t* out, const uint32_t* X, const int32_t* hot1, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(X);
    GRAPE_REQUIRE(hot1 != nullptr, "bad arguments");
    mask_cold_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, X, hot1, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_fr_gather(uint32_t* out, const uint32_t* src, const uint32_t* list, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(src);
    GRAPE_REQUIRE(list != nullptr, "bad arguments");
    gather_fr_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, src, list, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_init(uint32_t* T, uint32_t* B, int32_t low, uint32_t len, const uint32_t* beta, const uint32_t* map,
                       const uint32_t* r, grape_stream_t st) {
    CHECK_PTR16(T); CHECK_PTR16(B); CHECK_PTR16(beta);
    GRAPE_REQUIRE(len > 0, "empty table");
    if (map) { CHECK_PTR16(map); CHECK_PTR16(r); }
    tl_table_kernel<<<blocks_for(len), kBlock, 0, as_stream(st)>>>(T, map, r, low, len);
    GRAPE_LAUNCH_CHECK();
    return grape_fr_shift_inverse(B, T, beta, len, st);
}

int grape_tlookup_poly(const uint32_t* A, const uint32_t* S, const uint32_t* beta, uint32_t* o0, uint32_t* o1, uint32_t* o2,
                       size_t n_out, grape_stream_t st) {
    if (n_out == 0) return GRAPE_OK;
    CHECK_PTR16(A); CHECK_PTR16(S); CHECK_PTR16(o0); CHECK_PTR16(o1); CHECK_PTR16(o2);
    tl_poly_kernel<<<blocks_for(n_out), kBlock, 0, as_stream(st)>>>(A, S, beta, o0, o1, o2, n_out);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_tlookup_poly_sum(const uint32_t* A, uint32_t* o0, uint32_t* o1, size_t n_out, grape_stream_t st) {
    if (n_out == 0) return GRAPE_OK;
    CHECK_PTR16(A); CHECK_PTR16(o0); CHECK_PTR16(o1);
    tl_poly_sum_kernel<<<blocks_for(n_out), kBlock, 0, as_stream(st)>>>(A, o0, o1, n_out);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_round_sums(const uint32_t* A, const uint32_t* S, const uint32_t* beta, const uint32_t* eq, size_t n_out,
                             uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(A); CHECK_PTR16(S); CHECK_PTR16(eq); CHECK_PTR16(sums);
    GRAPE_REQUIRE(n_out >= 1, "empty round");
    hipStream_t s = as_stream(st);
    unsigned nb = reduce_grid(n_out, kLogUpIters);
    void* ws;
    int rc = scratch_get(kSlotReduce, (size_t)nb * 5 * 32, &ws, s);
    if (rc) return rc;
    tl_round_kernel<<<nb, kBlock, 0, s>>>(A, S, beta, eq, n_out, (uint32_t*)ws);
    launch_final_sum<5>(sums, (const uint32_t*)ws, nb, s);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_tlookup_mb_sums(const uint32_t* m, const uint32_t* B, size_t n_out, uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(m); CHECK_PTR16(B); CHECK_PTR16(sums);
    GRAPE_REQUIRE(n_out >= 1, "empty round");
    hipStream_t s = as_stream(st);
    unsigned nb = reduce_grid(n_out);
    void* ws;
    int rc = scratch_get(kSlotReduce, (size_t)nb * 3 * 32, &ws, s);
    if (rc) return rc;
    tl_mb_kernel<<<nb, kBlock, 0, s>>>(m, B, n_out, (uint32_t*)ws);
    launch_final_sum<3>(sums, (const uint32_t*)ws, nb, s);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_tlookup_table_round(uint32_t* B, uint32_t* T, uint32_t* m, const uint32_t* beta, const uint32_t* eq, size_t n_out,
                              const uint32_t* v, uint32_t* sums, grape_stream_t st) {
    CHECK_PTR16(B); CHECK_PTR16(T); CHECK_PTR16(m); CHECK_PTR16(eq); CHECK_PTR16(v); CHECK_PTR16(sums);
    if (beta) CHECK_PTR16(beta);
    GRAPE_REQUIRE(n_out >= 1, "empty round");
    hipStream_t s = as_stream(st);
    const unsigned nb = reduce_grid(n_out, kLogUpIters);
    void* ws;
    int rc = scratch_get(kSlotReduce, (size_t)nb * 8 * 32, &ws, s);
    if (rc) return rc;
    tl_table_round_kernel<<<nb, kBlock, 0, s>>>(B, T, m, beta, eq, n_out, v, (uint32_t*)ws);
    launch_final_sum<8>(sums, (const uint32_t*)ws, nb, s);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_eq_table(uint32_t* e, const uint32_t* u, uint32_t nu, grape_stream_t st) {
    CHECK_PTR16(e);
    GRAPE_REQUIRE(nu <= 30, "too many variables");
    hipStream_t s = as_stream(st);
    eq_init_kernel<<<1, 64, 0, s>>>(e);
    if (nu) CHECK_PTR16(u);
    for (uint32_t j = 0; j < nu; j++) eq_level_kernel<<<blocks_for((size_t)1 << j), kBlock, 0, s>>>(e, u, j);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_eq_table_halve(uint32_t* e, size_t n_out, grape_stream_t st) {
    if (n_out == 0) return GRAPE_OK;
    CHECK_PTR16(e);
    eq_halve_kernel<<<blocks_for(n_out), kBlock, 0, as_stream(st)>>>(e, n_out);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_fr_fold_msb_multi(uint32_t* const* ptrs, uint32_t k, size_t n_out, const uint32_t* v, grape_stream_t st) {
    GRAPE_REQUIRE(ptrs != nullptr && k >= 1 && k <= 8, "1..8 tensors");
    CHECK_PTR16(v);
    if (n_out == 0) return GRAPE_OK;
    PtrPack pk;
    for (uint32_t j = 0; j < 8; j++) pk.p[j] = j < k ? ptrs[j] : nullptr;
    for (uint32_t j = 0; j < k; j++) CHECK_PTR16(pk.p[j]);
    fold_msb_multi_kernel<<<blocks_for(n_out), kBlock, 0, as_stream(st)>>>(pk, k, n_out, v);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

}  // extern "C"
