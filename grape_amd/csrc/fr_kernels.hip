// Fr tensor kernels: element-wise field ops, integer embedding, Montgomery in/out, padding,
// reductions, batched inversion and the multilinear fold.
//
// Layout: a tensor is an array of 32-byte elements (the reference's fr_t array); every lane moves
// one element with two 16-byte vector accesses, so a wave64 covers 2 KiB of contiguous memory per
// element index and both halves of every 128-byte line are consumed back to back.
#include "fr_device.hpp"
#include "divstep.hpp"

namespace grape {

// ------------------------------------------------------------------------------------------------
// element-wise
// ------------------------------------------------------------------------------------------------
enum BinOp { OP_ADD, OP_SUB, OP_MUL };

template <int OP>
__device__ __forceinline__ Fr apply(const Fr& a, const Fr& b) {
    if (OP == OP_ADD) return add(a, b);
    if (OP == OP_SUB) return sub(a, b);
    return fr26::mulc(a, b);
}

template <int OP>
__global__ void __launch_bounds__(kBlock) ew_kernel(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, apply<OP>(ld_fr(a, i), ld_fr(b, i)));
}

// plain copy with the tensors' access pattern (one 32-byte element per lane, two 16-byte accesses)
__global__ void __launch_bounds__(kBlock) copy_fr_kernel(uint32_t* out, const uint32_t* a, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, ld_fr(a, i));
}

template <int OP>
__global__ void __launch_bounds__(kBlock) bcast_kernel(uint32_t* out, const uint32_t* a, const uint32_t* x, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, apply<OP>(ld_fr(a, i), ld_fr(x, 0)));
}

// out = x + r * y with one scalar r (the combined witness of a mapping lookup, S_in + r * S_out,
// src/tlookup.cu:407-410, in one pass instead of a copy, a scalar product and a sum)
__global__ void __launch_bounds__(kBlock) axpy_kernel(uint32_t* out, const uint32_t* x, const uint32_t* r, const uint32_t* y, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, add(ld_fr(x, i), fr26::mulc(ld_fr(y, i), ld_fr(r, 0))));
}

__global__ void __launch_bounds__(kBlock) from_i32_kernel(uint32_t* out, const int32_t* in, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, fr26::from_i32c(in[i]));
}
__global__ void __launch_bounds__(kBlock) from_u32_kernel(uint32_t* out, const uint32_t* in, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    st_fr(out, i, fr26::from_u32c(in[i]));
}
template <bool TO>
__global__ void __launch_bounds__(kBlock) mont_kernel(uint32_t* out, const uint32_t* in, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    Fr a = ld_fr(in, i);
    st_fr(out, i, TO ? fr26::to_montc(a) : fr26::from_montc(a));
}

__global__ void __launch_bounds__(kBlock) pad_fr_kernel(uint32_t* out, const uint32_t* in, uint32_t N, uint32_t pad_N,
                                                        size_t size, const uint32_t* pad_val) {
    size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (g >= size) return;
    size_t row = g / pad_N;
    uint32_t col = (uint32_t)(g % pad_N);
    st_fr(out, g, col < N ? ld_fr(in, row * N + col) : ld_fr(pad_val, 0));
}
__global__ void __launch_bounds__(kBlock) pad_i32_kernel(int32_t* out, const int32_t* in, uint32_t N, uint32_t pad_N, size_t size,
                                                         int32_t fill) {
    size_t g = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (g >= size) return;
    size_t row = g / pad_N;
    uint32_t col = (uint32_t)(g % pad_N);
    out[g] = col < N ? in[row * N + col] : fill;
}

// ------------------------------------------------------------------------------------------------
// reductions
// ------------------------------------------------------------------------------------------------
// stage 1: grid-stride partial sums, one Fr per block; stage 2: the same kernel with one block.
__global__ void __launch_bounds__(kBlock) sum_kernel(uint32_t* out, const uint32_t* in, size_t n) {
    __shared__ Fr lds[kBlock / 64];
    Fr acc = Fr::zero();
    size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) acc = add(acc, ld_fr(in, i));
    block_sum<1>(&acc, lds);
    if (threadIdx.x == 0) st_fr(out, blockIdx.x, acc);
}

__global__ void __launch_bounds__(kBlock) sum_by_dim_kernel(uint32_t* out, const uint32_t* in, size_t rows, size_t dim) {
    // one wave per row: strided partial sums, wave tree, broadcast back
    const int lane = threadIdx.x & 63;
    size_t row = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
    if (row >= rows) return;
    Fr acc = Fr::zero();
    for (size_t i = lane; i < dim; i += 64) acc = add(acc, ld_fr(in, row * dim + i));
    acc = wave_sum(acc);
    Fr tot;
#pragma unroll
    for (int k = 0; k < 8; k++) tot.v[k] = __shfl(acc.v[k], 0, 64);
    for (size_t i = lane; i < dim; i += 64) st_fr(out, row * dim + i, tot);
}

// ------------------------------------------------------------------------------------------------
// batched inversion (Montgomery's trick), three levels:
//   chunk products -> (recursive inversion of the products) -> back-substitution.
// Zero inputs are skipped in the products and produce zero outputs.
// ------------------------------------------------------------------------------------------------
constexpr int kInvChunk = 8;

// prod[t] = product of the non-zero elements of chunk t (beta added first when given)
__global__ void __launch_bounds__(kBlock) inv_prod_kernel(uint32_t* prod, const uint32_t* in, const uint32_t* beta, size_t n) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    size_t nchunks = (n + kInvChunk - 1) / kInvChunk;
    if (t >= nchunks) return;
    Fr acc = Fr::one();
    Fr bt = beta ? ld_fr(beta, 0) : Fr::zero();
    // chunk t owns elements t, t + nchunks, t + 2*nchunks, ... so that lanes stay coalesced
#pragma unroll
    for (int k = 0; k < kInvChunk; k++) {
        size_t i = t + (size_t)k * nchunks;
        if (i < n) {
            Fr x = ld_fr(in, i);
            if (beta) x = add(x, bt);
            if (!x.is_zero()) acc = fr26::mulc(acc, x);
        }
    }
    st_fr(prod, t, acc);
}
// given inv_prod[t] = 1/prod[t], write the individual inverses.  Only the prefix products stay in
// registers (8 elements = 64 registers); the elements themselves are read again on the way back -
// holding both sets spilled to scratch memory, which cost 2.5 times the traffic of the second read.
__global__ void __launch_bounds__(kBlock) inv_back_kernel(uint32_t* out, const uint32_t* in, const uint32_t* beta,
                                                          const uint32_t* inv_prod, size_t n) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    size_t nchunks = (n + kInvChunk - 1) / kInvChunk;
    if (t >= nchunks) return;
    Fr bt = beta ? ld_fr(beta, 0) : Fr::zero();
    Fr pre[kInvChunk];   // pre[k] = product of non-zero x[0..k-1]
    Fr acc = Fr::one();
#pragma clang loop unroll(full)
    for (int k = 0; k < kInvChunk; k++) {
        size_t i = t + (size_t)k * nchunks;
        Fr x = Fr::zero();
        if (i < n) {
            x = ld_fr(in, i);
            if (beta) x = add(x, bt);
        }
        pre[k] = acc;
        if (!x.is_zero()) acc = fr26::mulc(acc, x);
    }
    Fr inv = ld_fr(inv_prod, t);   // 1 / product of all non-zero x
#pragma clang loop unroll(full)
    for (int k = kInvChunk - 1; k >= 0; k--) {
        size_t i = t + (size_t)k * nchunks;
        if (i < n) {
            Fr x = ld_fr(in, i);          // (out may be in: element i is read before it is written, by this thread only)
            if (beta) x = add(x, bt);
            if (x.is_zero()) {
                st_fr(out, i, Fr::zero());
            } else {
                st_fr(out, i, fr26::mulc(inv, pre[k]));
                inv = fr26::mulc(inv, x);
            }
        }
    }
}
// direct inversion, used for the last (small) level
__global__ void __launch_bounds__(kBlock) inv_direct_kernel(uint32_t* out, const uint32_t* in, const uint32_t* beta, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    Fr x = ld_fr(in, i);
    if (beta) x = add(x, ld_fr(beta, 0));
    st_fr(out, i, divstep::inverse_by(x));
}

// ------------------------------------------------------------------------------------------------
// fold.  One pass binds the TOP b bits of the folded axis (the multilinear extension does not
// care in which order variables are bound, and binding high bits keeps every access contiguous):
//   out[o][i_lo][g] = sum_{i_hi} w[i_hi] * t[o][i_hi*c_lo + i_lo][g],   i_hi*c_lo + i_lo < c
// with w[i_hi] = prod_k eq(x[k], bit_k(i_hi)) over the b challenges of those bits.
// ------------------------------------------------------------------------------------------------
constexpr int kFoldMaxBits = 8;      // bits bound by one pass (at most 64 products per thread)
constexpr int kFoldMaxPasses = 16;

struct FoldPlan {
    uint32_t npass;
    uint32_t lo[kFoldMaxPasses];      // the pass binds challenges lo .. lo+b-1
    uint32_t b[kFoldMaxPasses];
    uint32_t off[kFoldMaxPasses];     // first weight of the pass in the weight buffer
    uint32_t first_plain;             // pass 0 reads plain integers: its weights carry the factor 2^256 that brings
                                      // a product with a plain value into memory form
};

// Weights of every pass of a fold, in the 26-bit working form with the radix factor 16 folded
// in (reduced mod r): workgroup p writes w[i] = prod_k eq(x[lo+k], bit_k(i)) for i < 2^b.
__global__ void __launch_bounds__(kBlock) fold_weights_kernel(int32_t* wts, const uint32_t* x, FoldPlan plan) {
    const uint32_t p = blockIdx.x, b = plan.b[p];
    if (threadIdx.x >= (1u << b)) return;
    // all challenges first (one memory round trip), then a product tree of depth 3: the
    // factors of one level are independent, which a single wave needs to issue at full rate
    Fr f[kFoldMaxBits];
#pragma unroll
    for (uint32_t k = 0; k < (uint32_t)kFoldMaxBits; k++) f[k] = ld_fr(x, plan.lo[p] + (k < b ? k : 0));
#pragma unroll
    for (uint32_t k = 0; k < (uint32_t)kFoldMaxBits; k++)
        f[k] = k < b ? (((threadIdx.x >> k) & 1) ? f[k] : sub(Fr::one(), f[k])) : Fr::one();
#pragma unroll
    for (int width = kFoldMaxBits / 2; width >= 1; width /= 2) {
#pragma unroll
        for (int k = 0; k < width; k++) f[k] = fr26::mulc(f[2 * k], f[2 * k + 1]);
    }
    Fr acc = f[0];
    if (p == 0 && plan.first_plain) acc = fr26::mulc(acc, Fr::rr());
    const fr26::Limbs w = fr26::weight16(acc);
    int32_t* dst = wts + (size_t)fr26::N * (plan.off[p] + threadIdx.x);
#pragma unroll
    for (int k = 0; k < fr26::N; k++) dst[k] = w.v[k];
}

// One pass.  A workgroup is 4 waves: 4/S groups of 64 outputs, each output summed by S waves
// that take every S-th term; the partial sums meet in LDS.  The weight index is wave-uniform, so
// the weights arrive through scalar loads and cost no vector registers.
// I32: the input is a tensor of 32-bit integers (the value x stands for the field element x, negative values for
// r - |x|): an element is two signed limbs, a product 20 multiply-adds, and 4 bytes are read where the embedded
// tensor has 32 - the pass that folds an integer tensor without first writing it out as field elements.
template <int S, bool I32 = false>
__global__ void __launch_bounds__(kBlock) fold_pass_kernel(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                           const int32_t* __restrict__ wts, uint32_t n_hi_max,
                                                           uint32_t outer, uint32_t c, uint32_t lg_c_lo, uint32_t gap) {
    constexpr int IW = 4 / S;                       // output groups per workgroup
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int iw = wave % IW, part = wave / IW;
    // index arithmetic in 32 bits (the host checks that the output count fits)
    const uint32_t c_lo = 1u << lg_c_lo;
    const uint32_t c_out = c < c_lo ? c : c_lo;     // surviving extent of the axis
    const uint32_t inner = c_out * gap;             // outputs per outer index
    const uint32_t total = outer * inner;
    const uint32_t tid = ((uint32_t)blockIdx.x * IW + iw) * 64 + lane;
    const bool live = tid < total;
    const uint32_t o = live ? tid / inner : 0;
    const uint32_t p = live ? tid - o * inner : 0;  // i_lo*gap + g
    const uint32_t i_lo = p / gap;
    const uint32_t* src = in + (I32 ? 1 : 8) * ((size_t)o * c * gap + p);
    const int32_t* isrc = reinterpret_cast<const int32_t*>(src);
    const size_t hi_stride = (size_t)c_lo * gap;    // elements between consecutive i_hi
    // number of i_hi with i_hi*c_lo + i_lo < c (zero for a dead lane)
    const uint32_t n_hi = live ? (c - i_lo + c_lo - 1) >> lg_c_lo : 0;
    // One double-width accumulator per thread: at most 64 products of values below r, so the
    // column sums stay below 64 * 10 * 2^52 and the reduced value below 2.82 r.
    fr26::Acc C;
    fr26::acc_zero(C);
    // Terms below n_full = c / c_lo exist for every lane, so the main loop is branch-free with
    // wave-uniform offsets and four loads in flight per lane (a dead lane reads the terms of
    // output 0 and stores nothing).  A ragged last term (c not a multiple of c_lo) follows
    // under a lane predicate, in the part whose turn it is.
    constexpr int U = I32 ? 8 : 4;
    const uint32_t n_full = c >> lg_c_lo;
    uint32_t h = (uint32_t)part;
    // an integer x = l0 + 2^26 l1 with 0 <= l0 < 2^26, -32 <= l1 < 32: a column grows by < 2^53 per term
    auto mac_int = [&](const fr26::Limbs& w, int32_t xv) {
        const int64_t l0 = (int64_t)(xv & (int32_t)fr26::MASK), l1 = (int64_t)(xv >> fr26::W);
#pragma unroll
        for (int j = 0; j < fr26::N; j++) {
            C.c[j] += (int64_t)w.v[j] * l0;
            C.c[j + 1] += (int64_t)w.v[j] * l1;
        }
    };
    for (; h + (U - 1) * S < n_full; h += U * S) {
        Fr t[I32 ? 1 : U];
        int32_t ti[I32 ? U : 1];
#pragma unroll
        for (int k = 0; k < U; k++) {
            if (I32) ti[k] = isrc[(size_t)(h + k * S) * hi_stride];
            else t[k] = ld_fr(src, (size_t)(h + k * S) * hi_stride);
        }
#pragma unroll
        for (int k = 0; k < U; k++) {
            fr26::Limbs w;
#pragma unroll
            for (int j = 0; j < fr26::N; j++) w.v[j] = wts[(size_t)fr26::N * (h + k * S) + j];
            if (I32) mac_int(w, ti[k]);
            else fr26::mac(C, w, fr26::pack(t[k]));
        }
    }
    for (; h < n_hi_max; h += S) {
        if (h < n_hi) {
            fr26::Limbs w;
#pragma unroll
            for (int j = 0; j < fr26::N; j++) w.v[j] = wts[(size_t)fr26::N * h + j];
            if (I32) mac_int(w, isrc[(size_t)h * hi_stride]);
            else fr26::mac(C, w, ld_l26(src, (size_t)h * hi_stride));
        }
    }
    fr26::Limbs r = fr26::reduce(C, 0);
    if (S > 1) {
        __shared__ int32_t lds[fr26::N * (S > 1 ? S - 1 : 1) * IW * 64];
        if (part > 0) {
#pragma unroll
            for (int k = 0; k < fr26::N; k++) lds[((k * (S - 1) + part - 1) * IW + iw) * 64 + lane] = r.v[k];
        }
        __syncthreads();
        if (part == 0) {
#pragma unroll
            for (int q = 1; q < S; q++) {
#pragma unroll
                for (int k = 0; k < fr26::N; k++) r.v[k] += lds[((k * (S - 1) + q - 1) * IW + iw) * 64 + lane];
            }
            r = fr26::normalize(r);
        }
    }
    // below 2.82 S r <= 11.3 r
    if (part == 0 && live) st_fr(out, tid, fr26::unpack(fr26::canon_wide(r)));
}

// Small-tensor finish: one workgroup holds the whole [c][gap] slab of one outer index in LDS
// and binds the remaining bits top-down with a barrier per level.
constexpr int kFoldSmallElems = 2048;   // 64 KiB of LDS
constexpr int kFoldSmallMaxOuter = 256; // one workgroup per outer index: worth it only for few
static bool fold_small_fits(size_t outer, size_t c, size_t gap) {
    return c * gap <= (size_t)kFoldSmallElems && outer <= (size_t)kFoldSmallMaxOuter;
}

__global__ void __launch_bounds__(kBlock) fold_small_kernel(uint32_t* out, const uint32_t* in, const uint32_t* x,
                                                            uint32_t L, size_t c, size_t gap) {
    __shared__ Fr buf[kFoldSmallElems];
    const size_t o = blockIdx.x;
    const size_t n = c * gap;
    for (size_t i = threadIdx.x; i < n; i += kBlock) buf[i] = ld_fr(in, o * n + i);
    __syncthreads();
    size_t cur = c;
    for (int lvl = (int)L - 1; lvl >= 0; lvl--) {
        const size_t half = (size_t)1 << lvl;        // axis indices >= half fold onto [0, half)
        if (cur > half) {
            const Fr xv = ld_fr(x, lvl);
            const size_t nlow = half * gap;
            for (size_t i = threadIdx.x; i < nlow; i += kBlock) {
                const size_t j = i + nlow;
                Fr lo = buf[i];
                Fr hi = (j < cur * gap) ? buf[j] : Fr::zero();
                buf[i] = add(lo, fr26::mulc(xv, sub(hi, lo)));
            }
            cur = half;
        } else {
            // the whole upper half is padding: value *= (1 - x)
            const Fr xv = sub(Fr::one(), ld_fr(x, lvl));
            for (size_t i = threadIdx.x; i < cur * gap; i += kBlock) buf[i] = fr26::mulc(buf[i], xv);
        }
        __syncthreads();
    }
    for (size_t i = threadIdx.x; i < gap; i += kBlock) st_fr(out, o * gap + i, buf[i]);
}

static uint32_t log2ceil(size_t n) {
    uint32_t r = 0;
    while (((size_t)1 << r) < n) r++;
    return r;
}

}  // namespace grape

using namespace grape;


template <int OP>
static int launch_ew(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(a); CHECK_PTR16(b);
    ew_kernel<OP><<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, a, b, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
template <int OP>
static int launch_bcast(uint32_t* out, const uint32_t* a, const uint32_t* x, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(a); CHECK_PTR16(x);
    bcast_kernel<OP><<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, a, x, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

// shared by grape_fr_batch_inverse / grape_fr_shift_inverse
static int batch_inverse_impl(uint32_t* out, const uint32_t* in, const uint32_t* beta, size_t n, hipStream_t s) {
    if (n == 0) return GRAPE_OK;
    if (n <= 4096) {
        inv_direct_kernel<<<blocks_for(n), kBlock, 0, s>>>(out, in, beta, n);
        GRAPE_LAUNCH_CHECK();
        return GRAPE_OK;
    }
    // levels of chunk products live back to back in one scratch buffer
    size_t sizes[16];
    int levels = 0;
    size_t cur = n, total = 0;
    while (cur > 4096) {
        cur = (cur + kInvChunk - 1) / kInvChunk;
        sizes[levels++] = cur;
        total += cur;
    }
    void* ws;
    int rc = scratch_get(kSlotInv, total * 32, &ws, s);
    if (rc) return rc;
    uint32_t* lvl[16];
    {
        uint32_t* p = (uint32_t*)ws;
        for (int l = 0; l < levels; l++) {
            lvl[l] = p;
            p += 8 * sizes[l];
        }
    }
    // forward: products
    inv_prod_kernel<<<blocks_for(sizes[0]), kBlock, 0, s>>>(lvl[0], in, beta, n);
    for (int l = 1; l < levels; l++)
        inv_prod_kernel<<<blocks_for(sizes[l]), kBlock, 0, s>>>(lvl[l], lvl[l - 1], nullptr, sizes[l - 1]);
    // top: direct inversion in place
    inv_direct_kernel<<<blocks_for(sizes[levels - 1]), kBlock, 0, s>>>(lvl[levels - 1], lvl[levels - 1], nullptr, sizes[levels - 1]);
    // backward: each level's inverses from the level above (in place over the products)
    for (int l = levels - 1; l >= 1; l--)
        inv_back_kernel<<<blocks_for(sizes[l]), kBlock, 0, s>>>(lvl[l - 1], lvl[l - 1], nullptr, lvl[l], sizes[l - 1]);
    inv_back_kernel<<<blocks_for(sizes[0]), kBlock, 0, s>>>(out, in, beta, lvl[0], n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

extern "C" {

int grape_fr_add(uint32_t* o, const uint32_t* a, const uint32_t* b, size_t n, grape_stream_t s) { return launch_ew<OP_ADD>(o, a, b, n, s); }
int grape_fr_sub(uint32_t* o, const uint32_t* a, const uint32_t* b, size_t n, grape_stream_t s) { return launch_ew<OP_SUB>(o, a, b, n, s); }
int grape_fr_mul(uint32_t* o, const uint32_t* a, const uint32_t* b, size_t n, grape_stream_t s) { return launch_ew<OP_MUL>(o, a, b, n, s); }
int grape_fr_bcast_add(uint32_t* o, const uint32_t* a, const uint32_t* x, size_t n, grape_stream_t s) { return launch_bcast<OP_ADD>(o, a, x, n, s); }
int grape_fr_bcast_mul(uint32_t* o, const uint32_t* a, const uint32_t* x, size_t n, grape_stream_t s) { return launch_bcast<OP_MUL>(o, a, x, n, s); }

int grape_bench_copy_fr(uint32_t* out, const uint32_t* in, size_t n, int iters, float* ms, grape_stream_t st) {
    CHECK_PTR16(out); CHECK_PTR16(in);
    GRAPE_REQUIRE(n > 0 && iters > 0 && ms != nullptr, "bad arguments");
    hipStream_t s = as_stream(st);
    hipEvent_t e0, e1;
    GRAPE_HIP_CHECK(hipEventCreate(&e0));
    GRAPE_HIP_CHECK(hipEventCreate(&e1));
    copy_fr_kernel<<<blocks_for(n), kBlock, 0, s>>>(out, in, n);
    GRAPE_HIP_CHECK(hipEventRecord(e0, s));
    for (int i = 0; i < iters; i++) copy_fr_kernel<<<blocks_for(n), kBlock, 0, s>>>(out, in, n);
    GRAPE_HIP_CHECK(hipEventRecord(e1, s));
    GRAPE_HIP_CHECK(hipEventSynchronize(e1));
    GRAPE_LAUNCH_CHECK();
    float t;
    GRAPE_HIP_CHECK(hipEventElapsedTime(&t, e0, e1));
    *ms = t / iters;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return GRAPE_OK;
}

int grape_fr_axpy(uint32_t* out, const uint32_t* x, const uint32_t* r, const uint32_t* y, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(x); CHECK_PTR16(r); CHECK_PTR16(y);
    axpy_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, x, r, y, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_fr_from_i32(uint32_t* out, const int32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out);
    GRAPE_REQUIRE(in != nullptr, "null input");
    from_i32_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, in, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_fr_from_u32(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out);
    GRAPE_REQUIRE(in != nullptr, "null input");
    from_u32_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, in, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_fr_to_mont(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in);
    mont_kernel<true><<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, in, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_fr_from_mont(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in);
    mont_kernel<false><<<blocks_for(n), kBlock, 0, as_stream(st)>>>(out, in, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_fr_batch_inverse(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in);
    return batch_inverse_impl(out, in, nullptr, n, as_stream(st));
}
int grape_fr_shift_inverse(uint32_t* out, const uint32_t* in, const uint32_t* beta, size_t n, grape_stream_t st) {
    if (n == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in); CHECK_PTR16(beta);
    return batch_inverse_impl(out, in, beta, n, as_stream(st));
}

int grape_fr_sum(uint32_t* out, const uint32_t* in, size_t n, grape_stream_t st) {
    CHECK_PTR16(out);
    hipStream_t s = as_stream(st);
    if (n == 0) {
        return zero_fill(out, 32, s);
    }
    CHECK_PTR16(in);
    unsigned nb = blocks_for(n);
    if (nb > kNumCU * 8) nb = kNumCU * 8;
    if (nb == 1) {
        sum_kernel<<<1, kBlock, 0, s>>>(out, in, n);
    } else {
        void* ws;
        int rc = scratch_get(kSlotReduce, (size_t)nb * 32, &ws, s);
        if (rc) return rc;
        sum_kernel<<<nb, kBlock, 0, s>>>((uint32_t*)ws, in, n);
        launch_final_sum<1>(out, (const uint32_t*)ws, nb, s);
    }
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_fr_sum_by_dim(uint32_t* out, const uint32_t* in, size_t rows, size_t dim, grape_stream_t st) {
    if (rows == 0 || dim == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in);
    sum_by_dim_kernel<<<blocks_for(rows * 64), kBlock, 0, as_stream(st)>>>(out, in, rows, dim);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_fr_pad(uint32_t* out, const uint32_t* in, uint32_t N, uint32_t pad_N, size_t pad_size, const uint32_t* pad_val, grape_stream_t st) {
    if (pad_size == 0) return GRAPE_OK;
    CHECK_PTR16(out); CHECK_PTR16(in); CHECK_PTR16(pad_val);
    GRAPE_REQUIRE(N <= pad_N && pad_N > 0 && out != in, "need N <= pad_N and distinct buffers");
    pad_fr_kernel<<<blocks_for(pad_size), kBlock, 0, as_stream(st)>>>(out, in, N, pad_N, pad_size, pad_val);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_i32_pad(int32_t* out, const int32_t* in, uint32_t N, uint32_t pad_N, size_t pad_size, grape_stream_t st) {
    if (pad_size == 0) return GRAPE_OK;
    GRAPE_REQUIRE(out && in && N <= pad_N && pad_N > 0 && out != in, "need N <= pad_N and distinct buffers");
    pad_i32_kernel<<<blocks_for(pad_size), kBlock, 0, as_stream(st)>>>(out, in, N, pad_N, pad_size, 0);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}
int grape_i32_pad_fill(int32_t* out, const int32_t* in, uint32_t N, uint32_t pad_N, size_t pad_size, int32_t fill, grape_stream_t st) {
    if (pad_size == 0) return GRAPE_OK;
    GRAPE_REQUIRE(out && in && N <= pad_N && pad_N > 0 && out != in, "need N <= pad_N and distinct buffers");
    pad_i32_kernel<<<blocks_for(pad_size), kBlock, 0, as_stream(st)>>>(out, in, N, pad_N, pad_size, fill);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

// Plan of a fold's passes: each binds as many top bits as possible (6, or more when the outputs are
// too few to fill the chip and S waves share one output), until the slab of one outer index
// fits the LDS finish kernel.
struct FoldPass { uint32_t b, S, off; };
static int plan_fold(size_t outer, uint32_t c, uint32_t gap, uint32_t id, FoldPass* passes, FoldPlan& plan) {
    plan.npass = 0;
    plan.first_plain = 0;
    uint32_t l = log2ceil(c), off = 0;
    size_t cc = c;
    while (l > 0 && !fold_small_fits(outer, cc, gap)) {
        // Measured on MI355X: a pass streams fastest with one thread per output, 16 to 64
        // terms per thread and 2^20 threads; 2^19 threads come close.  Failing that, up to
        // four waves share an output to reach 2^19 threads.
        uint32_t S = 0, b = 0;
        auto items = [&](uint32_t tb) { return outer * gap * ((size_t)1 << (l - tb)); };
        for (uint32_t want = 20; want >= 19 && S == 0; want--) {
            for (uint32_t tb = l < 6 ? l : 6; tb >= 4 && S == 0; tb--) {
                if (items(tb) >= ((size_t)1 << want)) { S = 1; b = tb; }
            }
        }
        for (uint32_t tb = l < 8 ? l : 8; tb >= 4 && S == 0; tb--) {
            const uint32_t ts = items(tb) * 2 >= ((size_t)1 << 19) ? 2 : 4;
            if (items(tb) * ts >= ((size_t)1 << 19) && (1u << tb) <= 64 * ts) { S = ts; b = tb; }
        }
        if (S == 0) {
            // too few outputs to fill the chip whatever the split: four waves per output and
            // at most 32 terms per thread keep the pass short
            S = 4; b = l <= 7 ? l : 6;
            // few, short slabs: stop as soon as the LDS finish kernel can take over
            if (outer <= (size_t)kFoldSmallMaxOuter && gap <= (size_t)kFoldSmallElems) {
                uint32_t keep = 0;      // bits the finish kernel can bind
                while (keep < l && (((size_t)2 << keep) * gap) <= (size_t)kFoldSmallElems) keep++;
                if (l > keep && l - keep < b) b = l - keep;
            }
        }
        GRAPE_REQUIRE(plan.npass < (uint32_t)kFoldMaxPasses, "fold: too many passes");
        passes[plan.npass] = {b, S, off};
        plan.lo[plan.npass] = id + (l - b);
        plan.b[plan.npass] = b;
        plan.off[plan.npass] = off;
        plan.npass++;
        off += 1u << b;
        l -= b;
        const size_t c_lo = (size_t)1 << l;
        cc = cc < c_lo ? cc : c_lo;
    }
    return GRAPE_OK;
}

// grape_fr_fold on t, or - with `ints` - the fold of the integer tensor `ints` left in t: the first pass reads the
// integers (4 bytes per element) and writes field elements, the later passes work on those as before.
static int fold_impl(uint32_t* t, const int32_t* ints, size_t N, const uint32_t* x, uint32_t c, uint32_t id, uint32_t gap, grape_stream_t st) {
    if (N == 0) return GRAPE_OK;
    CHECK_PTR16(t); CHECK_PTR16(x);
    GRAPE_REQUIRE(c >= 1 && gap >= 1 && N >= (size_t)c * gap && N % ((size_t)c * gap) == 0, "N must be a multiple of c*gap");
    hipStream_t s = as_stream(st);
    const size_t outer = N / ((size_t)c * gap);
    uint32_t L = log2ceil(c);
    FoldPass passes[kFoldMaxPasses];
    FoldPlan plan;
    int prc = plan_fold(outer, c, gap, id, passes, plan);
    if (prc) return prc;
    if (ints && (L == 0 || plan.npass == 0)) {
        // nothing to bind, or a tensor small enough for the finish kernel alone: embedded first (N elements of t)
        from_i32_kernel<<<blocks_for(N), kBlock, 0, s>>>(t, ints, N);
        GRAPE_LAUNCH_CHECK();
        ints = nullptr;
    }
    if (L == 0) return GRAPE_OK;   // c == 1: nothing to bind, data already compact
    plan.first_plain = ints ? 1u : 0u;
    const uint32_t* xs = x + 8 * (size_t)id;
    size_t cur_c = c;
    const uint32_t* src = ints ? reinterpret_cast<const uint32_t*>(ints) : t;
    // With a single outer index a pass can run in place (thread p reads p + k*stride only).
    // Otherwise passes ping-pong through scratch and the result is copied to the front.
    uint32_t* ws[2] = {nullptr, nullptr};
    int which = 0;
    const int32_t* wts = nullptr;
    if (plan.npass) {
        void* p;
        int rc = scratch_get(kSlotFoldW, ((size_t)kFoldMaxPasses * (1u << kFoldMaxBits) + 64) * fr26::N * 4, &p, s);
        if (rc) return rc;
        profile_begin();
        profile_mark(s);
        fold_weights_kernel<<<plan.npass, kBlock, 0, s>>>((int32_t*)p, x, plan);
        GRAPE_LAUNCH_CHECK();
        profile_mark(s);               // profiled intervals: the weight kernel, then one per pass
        wts = (const int32_t*)p;
    }
    uint32_t pi = 0;
    while (L > 0) {
        if (fold_small_fits(outer, cur_c, gap)) {
            uint32_t* dst = t;
            if (outer > 1 && src == t) {
                // reading slabs o*cur_c*gap while writing o*gap would race across workgroups
                void* p;
                int rc = scratch_get(kSlotFold, outer * gap * 32 * 2 + 64, &p, s);
                if (rc) return rc;
                dst = (uint32_t*)p;
            }
            fold_small_kernel<<<(unsigned)outer, kBlock, 0, s>>>(dst, src, xs, L, cur_c, gap);
            GRAPE_LAUNCH_CHECK();
            if (dst != t) GRAPE_HIP_CHECK(hipMemcpyAsync(t, dst, outer * gap * 32, hipMemcpyDeviceToDevice, s));
            return GRAPE_OK;
        }
        const FoldPass& ps = passes[pi++];
        const uint32_t b = ps.b;
        const size_t c_lo = (size_t)1 << (L - b);
        const size_t c_out = cur_c < c_lo ? cur_c : c_lo;
        uint32_t* dst;
        if (outer == 1) {
            dst = t;   // in place (src == t always holds here)
        } else {
            if (!ws[0]) {
                void* p;
                // two buffers, each large enough for the first pass output
                size_t each = outer * c_out * gap * 32;
                int rc = scratch_get(kSlotFold, 2 * each + 64, &p, s);
                if (rc) return rc;
                ws[0] = (uint32_t*)p;
                ws[1] = (uint32_t*)((char*)p + each);
            }
            dst = ws[which];
            which ^= 1;
        }
        const size_t total = outer * c_out * gap;
        GRAPE_REQUIRE(total < ((size_t)1 << 32) - 256, "fold: more than 2^32 outputs in one pass");
        const uint32_t n_hi_max = (uint32_t)((cur_c + c_lo - 1) / c_lo);
        const int32_t* w = wts + (size_t)fr26::N * ps.off;
        const bool plain = ints != nullptr && pi == 1;      // the first pass of a fold of integers
#define GRAPE_FOLD_PASS(SS, PER)                                                                                                    \
    do {                                                                                                                            \
        if (plain) fold_pass_kernel<SS, true><<<blocks_for(total, PER), kBlock, 0, s>>>(dst, src, w, n_hi_max, (uint32_t)outer, (uint32_t)cur_c, L - b, gap); \
        else fold_pass_kernel<SS, false><<<blocks_for(total, PER), kBlock, 0, s>>>(dst, src, w, n_hi_max, (uint32_t)outer, (uint32_t)cur_c, L - b, gap);     \
    } while (0)
        if (ps.S == 1) GRAPE_FOLD_PASS(1, 256);
        else if (ps.S == 2) GRAPE_FOLD_PASS(2, 128);
        else GRAPE_FOLD_PASS(4, 64);
#undef GRAPE_FOLD_PASS
        GRAPE_LAUNCH_CHECK();
        profile_mark(s);
        src = dst;
        cur_c = c_out;
        L -= b;
    }
    if (src != t) GRAPE_HIP_CHECK(hipMemcpyAsync(t, src, outer * gap * 32, hipMemcpyDeviceToDevice, s));
    return GRAPE_OK;
}

int grape_fr_fold(uint32_t* t, size_t N, const uint32_t* x, uint32_t c, uint32_t id, uint32_t gap, grape_stream_t st) {
    return fold_impl(t, nullptr, N, x, c, id, gap, st);
}

size_t grape_fr_fold_i32_elems(size_t N, uint32_t c, uint32_t gap) {
    if (N == 0 || c == 0 || gap == 0 || N % ((size_t)c * gap) != 0) return N;
    const size_t outer = N / ((size_t)c * gap);
    FoldPass passes[kFoldMaxPasses];
    FoldPlan plan;
    if (plan_fold(outer, c, gap, 0, passes, plan) != GRAPE_OK || plan.npass == 0) return N;
    if (outer > 1) return outer * gap;                 // the passes go through work memory of the library
    const size_t c_lo = (size_t)1 << (log2ceil(c) - passes[0].b);
    return (c < c_lo ? c : c_lo) * gap;                // one outer index: the first pass writes into d_out
}

int grape_fr_fold_i32(uint32_t* out, const int32_t* in, size_t N, const uint32_t* x, uint32_t c, uint32_t id, uint32_t gap, grape_stream_t st) {
    GRAPE_REQUIRE(in != nullptr || N == 0, "null input");
    return fold_impl(out, in, N, x, c, id, gap, st);
}

}  // extern "C"
