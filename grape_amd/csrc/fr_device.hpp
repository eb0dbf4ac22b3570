// Device-side helpers shared by the Fr kernels: 16-byte vector load/store of 32-byte elements
// and wave64 / workgroup tree sums.
#pragma once
#include "common.hpp"
#include "fr26.hpp"

namespace grape {

__device__ __forceinline__ Fr ld_fr(const uint32_t* base, size_t i) {
    const uint4* p = reinterpret_cast<const uint4*>(base) + 2 * i;
    uint4 lo = p[0], hi = p[1];
    Fr r;
    r.v[0] = lo.x; r.v[1] = lo.y; r.v[2] = lo.z; r.v[3] = lo.w;
    r.v[4] = hi.x; r.v[5] = hi.y; r.v[6] = hi.z; r.v[7] = hi.w;
    return r;
}
__device__ __forceinline__ void st_fr(uint32_t* base, size_t i, const Fr& a) {
    uint4* p = reinterpret_cast<uint4*>(base) + 2 * i;
    p[0] = make_uint4(a.v[0], a.v[1], a.v[2], a.v[3]);
    p[1] = make_uint4(a.v[4], a.v[5], a.v[6], a.v[7]);
}

// element as 26-bit working limbs straight from memory
// Marks an element as used at this point of the program, so that the wait for the loads that
// produce it is placed here.
__device__ __forceinline__ void arrived(Fr& a) {
    asm volatile("" : "+v"(a.v[0]), "+v"(a.v[1]), "+v"(a.v[2]), "+v"(a.v[3]), "+v"(a.v[4]), "+v"(a.v[5]), "+v"(a.v[6]), "+v"(a.v[7]));
}
__device__ __forceinline__ fr26::Limbs ld_l26(const uint32_t* base, size_t i) { return fr26::pack(ld_fr(base, i)); }

using fr26::fold1;

// Table folds of TWO elements by the same challenge, row by row of the table: the ten words of a row
// arrive through one scalar load and serve both elements, and the row pointer is re-derived from a
// value the previous row produced, so that the compiler keeps one or two rows in scalar registers
// instead of loading (and then spilling) all hundred words ahead of the loop.
typedef const __attribute__((address_space(4))) int32_t* FoldTabPtr;
__device__ __forceinline__ void foldt2(const int32_t* tab, const fr26::Limbs& lo_a, const fr26::Limbs& d_a, const fr26::Limbs& lo_b,
                                       const fr26::Limbs& d_b, Fr& out_a, Fr& out_b) {
    constexpr int N = fr26::N;
    int64_t ca[N + 2], cb[N + 2];
    ca[0] = ca[1] = cb[0] = cb[1] = 0;
#pragma unroll
    for (int k = 0; k < N; k++) {
        ca[k + 2] = (int64_t)(uint32_t)lo_a.v[k];
        cb[k + 2] = (int64_t)(uint32_t)lo_b.v[k];
    }
    // rows j and j + 1 are addressable from the start; the pointer of row j + 2 is released by a value
    // that row j has produced, so its scalar load is in flight while row j + 1 is multiplied
    FoldTabPtr row[N];
#pragma unroll
    for (int j = 0; j < N; j++) row[j] = (FoldTabPtr)(uintptr_t)(tab + j * N);
    asm volatile("" : "+s"(row[0]), "+s"(row[1]));
#pragma unroll
    for (int j = 0; j < N; j++) {
#pragma unroll
        for (int k = 0; k < N; k++) {
            const int32_t w = row[j][k];
            ca[k] += (int64_t)d_a.v[j] * (int64_t)w;
            cb[k] += (int64_t)d_b.v[j] * (int64_t)w;
        }
        if (j + 2 < N) asm volatile("" : "+s"(row[j + 2]) : "v"((uint32_t)ca[0]));
    }
    out_a = fr26::foldt_finish(ca);
    out_b = fr26::foldt_finish(cb);
}

// The table fold of ONE element, rows through scalar loads as in foldt2 (for kernels whose registers
// do not hold two sets of fold columns beside their accumulators).
__device__ __forceinline__ Fr foldt1(const int32_t* tab, const fr26::Limbs& lo, const fr26::Limbs& d) {
    constexpr int N = fr26::N;
    int64_t c[N + 2];
    c[0] = c[1] = 0;
#pragma unroll
    for (int k = 0; k < N; k++) c[k + 2] = (int64_t)(uint32_t)lo.v[k];
    FoldTabPtr row[N];
#pragma unroll
    for (int j = 0; j < N; j++) row[j] = (FoldTabPtr)(uintptr_t)(tab + j * N);
    asm volatile("" : "+s"(row[0]), "+s"(row[1]));
#pragma unroll
    for (int j = 0; j < N; j++) {
#pragma unroll
        for (int k = 0; k < N; k++) c[k] += (int64_t)d.v[j] * (int64_t)row[j][k];
        if (j + 2 < N) asm volatile("" : "+s"(row[j + 2]) : "v"((uint32_t)c[0]));
    }
    return fr26::foldt_finish(c);
}

// The ten multiples of a round's challenge that the table fold multiplies by (fr26::fold_table), for
// `count` <= 64 challenges: thread t writes the table of v[t] at tabs + 100 t.  (static: every
// source file that launches it gets its own copy)
static __global__ void __launch_bounds__(64) fold_tables_kernel(int32_t* tabs, const uint32_t* v, uint32_t count) {
    if (threadIdx.x < count) fr26::fold_table(tabs + (size_t)fr26::kFoldTableWords * threadIdx.x, ld_fr(v, threadIdx.x));
}
// Rounds of at least this many output indices fold through the table of the challenge's multiples
// (one more small launch per round); shorter rounds are launch-bound and keep the single product.
constexpr uint32_t kTableFoldMinOut = 1u << 16;
constexpr size_t kFoldTableBytes = 512;                  // 100 words, padded

// hi operand of the MSB split: X[g + h] or zero when that index is past the live extent
__device__ __forceinline__ Fr ld_hi(const uint32_t* X, size_t g, size_t h, size_t in_size) {
    return (g + h < in_size) ? ld_fr(X, g + h) : Fr::zero();
}

// hi operand as working limbs (zero past the live extent)
__device__ __forceinline__ fr26::Limbs ld_hi26(const uint32_t* X, size_t g, size_t h, size_t in_size) {
    return fr26::pack(ld_hi(X, g, h, in_size));
}

__device__ __forceinline__ Fr shfl_down_fr(const Fr& a, int off) {
    Fr r;
#pragma unroll
    for (int i = 0; i < 8; i++) r.v[i] = __shfl_down(a.v[i], off, 64);
    return r;
}
// wave64 tree: lane 0 ends with the sum of all 64 lanes
__device__ __forceinline__ Fr wave_sum(Fr a) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) a = add(a, shfl_down_fr(a, off));
    return a;
}
// Workgroup sum of NV values per thread; result valid in thread 0.  lds holds NV*(kBlock/64) Fr.
template <int NV>
__device__ __forceinline__ void block_sum(Fr* vals, Fr* lds) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int NW = kBlock / 64;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        Fr s = wave_sum(vals[k]);
        if (lane == 0) lds[k * NW + wave] = s;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < NV; k++) {
            Fr s = lds[k * NW];
            for (int w = 1; w < NW; w++) s = add(s, lds[k * NW + w]);
            vals[k] = s;
        }
    }
}

// ---- finishing kernels: ONE workgroup adds up the partial sums that the workgroups of a round left.
// A long round leaves up to eleven thousand partial sums per coefficient; read one at a time by 256
// threads that is a chain of 43 dependent loads (30-60 us, as much as the whole round of a short
// proof), so long lists go to a workgroup of 1024 threads, and every thread keeps two groups of loads
// in flight.  (Letting the last workgroup of the round kernel do this instead - an arrival counter
// behind a device-scope fence - was built and measured: the fence makes every workgroup write the
// folded tensors' dirty cache lines back before it may take its ticket, and the round kernels lost
// 5-12 % at 2^24 index pairs, more than the saved launch is worth.)
constexpr int kFinalBlock = 1024;
constexpr unsigned kFinalWideMin = 4 * kBlock;     // partial sums per coefficient from which the wide workgroup is used

// Plain integer sum of canonical elements (nine words: room for 2^32 terms): a step of a sum tree costs
// nine add-with-carry instead of the 24 instructions of a modular addition, and ONE reduction ends it.
struct Sum9 {
    uint32_t w[9];
};
__device__ __forceinline__ void sum9_zero(Sum9& s) {
#pragma unroll
    for (int i = 0; i < 9; i++) s.w[i] = 0;
}
__device__ __forceinline__ void sum9_add_fr(Sum9& s, const Fr& a) {
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) s.w[i] = detail::adc32(s.w[i], a.v[i], c);
    s.w[8] += c;
}
__device__ __forceinline__ void sum9_add(Sum9& s, const Sum9& t) {
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < 9; i++) s.w[i] = detail::adc32(s.w[i], t.w[i], c);
}
__device__ __forceinline__ Sum9 shfl_down_sum9(const Sum9& a, int off) {
    Sum9 r;
#pragma unroll
    for (int i = 0; i < 9; i++) r.w[i] = __shfl_down(a.w[i], off, 64);
    return r;
}
// lo + hi * 2^256 mod r: lo < 2^256 < 6 r loses r up to five times, and hi * 2^256 mod r is the memory
// form of the integer hi
__device__ __forceinline__ Fr sum9_to_fr(const Sum9& s) {
    Fr lo;
#pragma unroll
    for (int i = 0; i < 8; i++) lo.v[i] = s.w[i];
#pragma unroll
    for (int rep = 0; rep < 5; rep++) {
        Fr d;
        detail::final_sub<FrParams>(d.v, lo.v, 0);
        lo = d;
    }
    return add(lo, fr26::from_u32c(s.w[8]));
}

// tot[k] = sum over b < nblocks of partial[b*NV + k] for every k whose bit in SKIP is clear (the others
// are left zero), valid in thread 0 of a workgroup of BLOCK threads; lds9 holds NV * (BLOCK/64) * 9 words
template <int NV, int BLOCK, unsigned SKIP = 0>
__device__ __forceinline__ void workgroup_totals(Fr* tot, const uint32_t* partial, unsigned nblocks, uint32_t* lds9) {
    constexpr int NW = BLOCK / 64;
    Sum9 s[NV];
#pragma unroll
    for (int k = 0; k < NV; k++) sum9_zero(s[k]);
    unsigned b = threadIdx.x;
    for (; b + BLOCK < nblocks; b += 2 * BLOCK) {
        Fr t0[NV], t1[NV];
#pragma unroll
        for (int k = 0; k < NV; k++) {
            if (SKIP & (1u << k)) continue;
            t0[k] = ld_fr(partial, (size_t)b * NV + k);
            t1[k] = ld_fr(partial, (size_t)(b + BLOCK) * NV + k);
        }
#pragma unroll
        for (int k = 0; k < NV; k++) {
            if (SKIP & (1u << k)) continue;
            sum9_add_fr(s[k], t0[k]);
            sum9_add_fr(s[k], t1[k]);
        }
    }
    if (b < nblocks) {
#pragma unroll
        for (int k = 0; k < NV; k++) {
            if (SKIP & (1u << k)) continue;
            sum9_add_fr(s[k], ld_fr(partial, (size_t)b * NV + k));
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < NV; k++) {
        if (SKIP & (1u << k)) continue;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) sum9_add(s[k], shfl_down_sum9(s[k], off));
        if (lane == 0) {
#pragma unroll
            for (int i = 0; i < 9; i++) lds9[(k * NW + wave) * 9 + i] = s[k].w[i];
        }
    }
    __syncthreads();
    // thread k folds the waves' sums of value k and reduces it (the reductions side by side, not one
    // after the other on one thread), then thread 0 collects the NV results
    Fr mine = Fr::zero();
    const int k = threadIdx.x;
    if (k < NV && !((SKIP >> k) & 1u)) {
        Sum9 t;
        sum9_zero(t);
        for (int w = 0; w < NW; w++) {
            Sum9 o;
#pragma unroll
            for (int i = 0; i < 9; i++) o.w[i] = lds9[(k * NW + w) * 9 + i];
            sum9_add(t, o);
        }
        mine = sum9_to_fr(t);
    }
    __syncthreads();
    if (k < NV) {
#pragma unroll
        for (int i = 0; i < 8; i++) lds9[k * 8 + i] = mine.v[i];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int j = 0; j < NV; j++) {
#pragma unroll
            for (int i = 0; i < 8; i++) tot[j].v[i] = lds9[j * 8 + i];
        }
    }
}

// NV interleaved partial arrays: partial[b*NV + k]; out[k] = sum_b partial[b*NV + k]
template <int NV, int BLOCK = kBlock>
__global__ void __launch_bounds__(BLOCK) final_sum_kernel(uint32_t* out, const uint32_t* partial, unsigned nblocks) {
    __shared__ uint32_t lds9[NV * (BLOCK / 64) * 9];
    Fr acc[NV];
    workgroup_totals<NV, BLOCK>(acc, partial, nblocks, lds9);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < NV; k++) st_fr(out, k, acc[k]);
    }
}
template <int NV>
static inline void launch_final_sum(uint32_t* out, const uint32_t* partial, unsigned nblocks, hipStream_t s) {
    if (nblocks >= kFinalWideMin) final_sum_kernel<NV, kFinalBlock><<<1, kFinalBlock, 0, s>>>(out, partial, nblocks);
    else final_sum_kernel<NV, kBlock><<<1, kBlock, 0, s>>>(out, partial, nblocks);
}

#define CHECK_PTR16(p) GRAPE_REQUIRE((p) != nullptr && (reinterpret_cast<uintptr_t>(p) & 15) == 0, #p " must be a 16-byte aligned device pointer")

}  // namespace grape
