// Quantised-layer witness generation on the GPU: the fixed-point rules of the reference's Python
// generator (zzllama/llama/model.py) as integer kernels.  Every product is exact (64-bit
// accumulation of 32 x 32-bit products: v_mad_i64_i32 issues at the rate of an addition on gfx950),
// every rescaling is q = floor((y + S/2) / S), r = y - q*S (model.py:489-491), and the epilogue of
// a matrix product writes quotient and remainder directly, so the 64-bit products never reach
// memory.
//
// Conditions the reference asserts (table indices in range, model.py:86-87) or silently assumes
// (quotients fit 32 bits) are recorded in a sticky device-side status word, read and cleared by
// grape_wit_status().
#include "common.hpp"

namespace grape {

enum WitFlag : uint32_t { kWitQuotient = 1, kWitIndex = 2, kWitSum = 4, kWitSquares = 8 };

// floor((y + s/2) / s) and the centred remainder; s > 0, sh = log2(s) or -1 when s is no power of 2
__device__ __forceinline__ void rescale64(int64_t y, int64_t s, int sh, int32_t& q, int32_t& r, uint32_t& bad) {
    const int64_t t = y + (s >> 1);
    int64_t qq;
    if (sh >= 0) {
        qq = t >> sh;                         // arithmetic shift floors
    } else {
        qq = t / s;
        if ((t % s != 0) && (t < 0)) qq -= 1;  // C division truncates; floor wanted
    }
    bad |= (qq != (int64_t)(int32_t)qq) ? (uint32_t)kWitQuotient : 0u;
    q = (int32_t)qq;
    r = (int32_t)(y - qq * s);
}

// ------------------------------------------------------------------------------------------------
// Y[l][n][m] = sum_k A[l][n][k] * B[l][m][k], rescaled.  Tile 128 x 128 x 32 per workgroup of 256
// threads; each thread owns the 8 x 8 outputs (ty + 16 i, tx + 16 j).  Tiles sit in LDS row-major
// with a row stride of 36 words, which makes the 16-byte fragment reads of 16 consecutive rows hit
// 16 disjoint groups of 4 banks.  The next tile travels from memory into registers while the
// current one is multiplied.
// ------------------------------------------------------------------------------------------------
constexpr int kTM = 128, kTK = 32, kLd = 36;

struct MatmulArgs {
    int32_t* q;
    int32_t* r;          // may be null
    const int32_t* a;
    const int32_t* b;
    uint32_t N, M, K;
    int64_t scale;
    int shift;           // log2(scale) or -1
    int transpose_out;   // write [m][n] instead of [n][m]
    uint32_t tiles_n, tiles_m;
    uint32_t* status;
};

__global__ void __launch_bounds__(256, 2) wit_matmul_tiled_kernel(MatmulArgs p) {
    __shared__ __attribute__((aligned(16))) int32_t As[kTM * kLd];
    __shared__ __attribute__((aligned(16))) int32_t Bs[kTM * kLd];
    // consecutive workgroups go to different XCDs; give each XCD a contiguous run of tiles so
    // that the tiles sharing rows of A and of B meet in the same L2
    uint32_t bid = blockIdx.x;
    const uint32_t nb = gridDim.x;
    if ((nb & 7u) == 0) bid = (bid & 7u) * (nb >> 3) + (bid >> 3);
    const uint32_t tn = bid / p.tiles_m, tm = bid - tn * p.tiles_m;
    const uint32_t l = blockIdx.y;
    const int32_t* A = p.a + (size_t)l * p.N * p.K;
    const int32_t* B = p.b + (size_t)l * p.M * p.K;
    const uint32_t n0 = tn * kTM, m0 = tm * kTM;
    const uint32_t t = threadIdx.x, tx = t & 15u, ty = t >> 4;

    // staging: 4 + 4 vectors of 4 words per thread; vector v = t + 256 p covers row v / 8, words 4 (v % 8)
    uint4 sa[4], sb[4];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int pp = 0; pp < 4; pp++) {
            const uint32_t v = t + 256u * pp, row = v >> 3, kk = k0 + 4u * (v & 7u);
            const bool ka = kk < p.K;     // K is a multiple of 4: a vector is inside or outside as a whole
            const uint32_t ra = n0 + row < p.N ? n0 + row : p.N - 1, rb = m0 + row < p.M ? m0 + row : p.M - 1;
            const uint32_t kc = ka ? kk : 0;
            uint4 va = *reinterpret_cast<const uint4*>(A + (size_t)ra * p.K + kc);
            uint4 vb = *reinterpret_cast<const uint4*>(B + (size_t)rb * p.K + kc);
            const bool oka = ka && (n0 + row < p.N), okb = ka && (m0 + row < p.M);
            sa[pp] = oka ? va : make_uint4(0, 0, 0, 0);
            sb[pp] = okb ? vb : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int pp = 0; pp < 4; pp++) {
            const uint32_t v = t + 256u * pp, row = v >> 3, c = 4u * (v & 7u);
            *reinterpret_cast<uint4*>(&As[row * kLd + c]) = sa[pp];
            *reinterpret_cast<uint4*>(&Bs[row * kLd + c]) = sb[pp];
        }
    };

    int64_t acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[i][j] = 0;

    fetch(0);
    for (uint32_t k0 = 0; k0 < p.K; k0 += kTK) {
        __syncthreads();                 // everyone is done with the previous tile
        stage();
        __syncthreads();
        if (k0 + kTK < p.K) fetch(k0 + kTK);
#pragma unroll 1
        for (int kk = 0; kk < kTK; kk += 4) {
            int32_t fa[8][4];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int4 v = *reinterpret_cast<const int4*>(&As[(ty + 16 * i) * kLd + kk]);
                fa[i][0] = v.x; fa[i][1] = v.y; fa[i][2] = v.z; fa[i][3] = v.w;
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int4 v = *reinterpret_cast<const int4*>(&Bs[(tx + 16 * j) * kLd + kk]);
                const int32_t fb[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int c = 0; c < 4; c++)
#pragma unroll
                    for (int i = 0; i < 8; i++) acc[i][j] += (int64_t)fa[i][c] * (int64_t)fb[c];
            }
        }
    }

    uint32_t bad = 0;
    int32_t* Q = p.q + (size_t)l * p.N * p.M;
    int32_t* R = p.r ? p.r + (size_t)l * p.N * p.M : nullptr;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t n = n0 + ty + 16 * i;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t m = m0 + tx + 16 * j;
            if (n < p.N && m < p.M) {
                int32_t q, r;
                rescale64(acc[i][j], p.scale, p.shift, q, r, bad);
                const size_t o = p.transpose_out ? (size_t)m * p.N + n : (size_t)n * p.M + m;
                Q[o] = q;
                if (R) R[o] = r;
            }
        }
    }
    if (bad) atomicOr(p.status, bad);
}

// any shape: one thread per output, used when K is no multiple of 4 or a row is not 16-byte aligned
__global__ void __launch_bounds__(kBlock) wit_matmul_simple_kernel(MatmulArgs p, uint32_t L) {
    const size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t per = (size_t)p.N * p.M;
    if (idx >= per * L) return;
    const uint32_t l = (uint32_t)(idx / per);
    const size_t nm = idx - (size_t)l * per;
    const uint32_t n = (uint32_t)(nm / p.M), m = (uint32_t)(nm - (size_t)n * p.M);
    const int32_t* a = p.a + ((size_t)l * p.N + n) * p.K;
    const int32_t* b = p.b + ((size_t)l * p.M + m) * p.K;
    int64_t acc = 0;
    for (uint32_t k = 0; k < p.K; k++) acc += (int64_t)a[k] * (int64_t)b[k];
    uint32_t bad = 0;
    int32_t q, r;
    rescale64(acc, p.scale, p.shift, q, r, bad);
    const size_t o = (size_t)l * per + (p.transpose_out ? (size_t)m * p.N + n : (size_t)n * p.M + m);
    p.q[o] = q;
    if (p.r) p.r[o] = r;
    if (bad) atomicOr(p.status, bad);
}

// ------------------------------------------------------------------------------------------------
// The same product on the matrix cores.  An int32 operand is split into P planes of signed bytes
// (balanced radix-256 digits, x = sum_p d_p 256^p, d_p in [-128, 127]); the product is the sum over
// plane pairs of int8 x int8 -> int32 matrix products (v_mfma_i32_32x32x32_i8), and pairs with the
// same p + q share an accumulator.  All of it is exact: a digit product is at most 2^14 and a
// group absorbs at most min(PA, PB) * K of them, kept below 2^31 by the host.  The groups are
// recombined as 64-bit integers in the epilogue and rescaled like in the kernel above.
//
// Workgroup tile 64 (rows of a) x 128 (rows of b), K step 64 bytes; four waves, each 32 x 64 (two
// MFMA tiles); the 16-byte chunks of an LDS row are permuted by the row number so that fragment
// reads and staging writes are both free of bank conflicts; the next K step travels through
// registers while this one multiplies.  Products with at least one 128 x 128 tile per CU take
// the eight-wave kernel further down.
// ------------------------------------------------------------------------------------------------
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));
constexpr int kMfTN = 64, kMfTM = 128, kMfK = 64, kMfLd = 64;
constexpr int kBgT = 128;      // rows of a and rows of b per workgroup of the large-tile kernel

// planes[p][row][k] for k < Kp (zero beyond K) for three planes, and the largest magnitude of x folded
// into *mx with an atomic maximum (one per workgroup): the caller learns from it how many of the
// planes are non-zero.  A thread takes 4 consecutive k at a time, the grid strides over the tensor.
__global__ void __launch_bounds__(kBlock) wit_split_kernel(int8_t* planes, uint32_t* mx, const int32_t* x, uint32_t R, uint32_t K, uint32_t Kp) {
    const uint32_t per_row = Kp / 4;
    const size_t total = (size_t)R * per_row, stride = (size_t)gridDim.x * kBlock;
    const size_t plane = (size_t)R * Kp;
    uint32_t m = 0;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += stride) {
        const uint32_t row = (uint32_t)(idx / per_row), k = 4u * (uint32_t)(idx - (size_t)row * per_row);
        int32_t v[4] = {0, 0, 0, 0};
        if (k < K) {      // K is a multiple of 4
            const int4 t = *reinterpret_cast<const int4*>(x + (size_t)row * K + k);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t a = v[j] < 0 ? 0u - (uint32_t)v[j] : (uint32_t)v[j];
            m = a > m ? a : m;
        }
#pragma unroll
        for (int p = 0; p < 3; p++) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int32_t d = (int32_t)(int8_t)(v[j] & 0xff);
                // (v - d) is a multiple of 256; the subtraction cannot wrap (|d| <= 128 towards zero)
                v[j] = (int32_t)(((int64_t)v[j] - d) >> 8);
                w |= ((uint32_t)d & 0xffu) << (8 * j);
            }
            *reinterpret_cast<uint32_t*>(planes + p * plane + (size_t)row * Kp + k) = w;
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t o = __shfl_xor(m, off, 64);
        m = o > m ? o : m;
    }
    // one atomic per workgroup: atomics on one address are served one after the other
    __shared__ uint32_t sh[kBlock / 64];
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kBlock / 64; w++) m = sh[w] > m ? sh[w] : m;
        if (m) atomicMax(mx, m);
    }
}

struct MfmaArgs {
    int32_t* q;
    int32_t* r;
    const int8_t* a;     // [PA][N][Kp]
    const int8_t* b;     // [PB][M][Kp]
    uint32_t N, M, Kp;
    int64_t scale;
    int shift, transpose_out;
    uint32_t tiles_n, tiles_m;
    uint32_t* status;
};

// Which tile a workgroup takes.  Workgroups are dealt to the eight XCDs in turn, so workgroup b is the
// (b / 8)-th of XCD b % 8; every XCD gets a contiguous run of the tile order, and the order walks
// panels of eight tile columns row by row: the 64 workgroups an XCD runs at a time then share the
// operand rows of 8 x 8 tiles (a step's distinct bytes are an eighth of what they request) and find
// them in that XCD's L2 instead of streaming whole rows of tiles past it.
__device__ __forceinline__ void mfma_tile_of(uint32_t b, uint32_t nb, uint32_t tiles_n, uint32_t tiles_m, uint32_t& tn, uint32_t& tm) {
    constexpr uint32_t W = 8;
    const uint32_t x = b & 7u, per = nb >> 3, extra = nb & 7u;
    uint32_t l = x * per + (x < extra ? x : extra) + (b >> 3);
    const uint32_t full = tiles_m / W, in_full = full * tiles_n * W;
    if (l < in_full) {
        const uint32_t pnl = l / (tiles_n * W), r = l - pnl * tiles_n * W;
        tn = r / W;
        tm = pnl * W + (r - tn * W);
    } else {
        l -= in_full;
        const uint32_t wr = tiles_m - full * W;
        tn = l / wr;
        tm = full * W + (l - tn * wr);
    }
}

template <int PA, int PB>
__global__ void __launch_bounds__(256, 2) wit_matmul_mfma_kernel(MfmaArgs p) {
    constexpr int G = PA + PB - 1;
    constexpr int CR = kMfK / 16;                     // 16-byte chunks in a row of one K step
    constexpr int RP = 256 / CR;                      // rows one staging pass of the workgroup covers
    constexpr int NA = kMfTN / RP, NB = kMfTM / RP;   // passes per plane
    __shared__ __attribute__((aligned(16))) int8_t As[PA * kMfTN * kMfLd];
    __shared__ __attribute__((aligned(16))) int8_t Bs[PB * kMfTM * kMfLd];
    uint32_t tn, tm;
    mfma_tile_of(blockIdx.x, gridDim.x, p.tiles_n, p.tiles_m, tn, tm);
    const uint32_t n0 = tn * kMfTN, m0 = tm * kMfTM;
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    const uint32_t wn = (wave & 1u) * 32u, wm = (wave >> 1) * 64u;

    // staging: thread t carries chunk t % CR of rows t / CR + RP h of every plane (fully unrolled: registers)
    const uint32_t lr = t / CR, ck = 16u * (t % CR);
    v4i_t sa[PA][NA], sb[PB][NB];
    const int8_t *ga[NA], *gb[NB];
#pragma unroll
    for (int h = 0; h < NA; h++) {
        const uint32_t r = n0 + lr + RP * h;
        ga[h] = p.a + (size_t)(r < p.N ? r : p.N - 1) * p.Kp + ck;
    }
#pragma unroll
    for (int h = 0; h < NB; h++) {
        const uint32_t r = m0 + lr + RP * h;
        gb[h] = p.b + (size_t)(r < p.M ? r : p.M - 1) * p.Kp + ck;
    }
    const size_t pla = (size_t)p.N * p.Kp, plb = (size_t)p.M * p.Kp;     // plane strides
    v16i_t acc[G][2];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[g][tt][i] = 0;

    // LDS rows are kMfK bytes with no padding; the 16-byte chunk c of row r sits at chunk position
    // c ^ ((r / RL) % CR) (RL = rows per 128 bytes), so that eight consecutive rows' equal chunks
    // (the fragment reads) and the consecutive chunks of one or two rows (the staging writes) both
    // spread over all banks
    constexpr int RL = 8 / CR;
    const uint32_t frow = lane & 31u;
    const uint32_t fx = 16u * ((lane >> 5) ^ ((frow / RL) % CR));     // fragment of k offset kk + 16 (lane / 32): byte kk ^ fx
    const uint32_t wx = 16u * ((t % CR) ^ ((lr / RL) % CR));
#define WIT_LD16(ptr) (*reinterpret_cast<const v4i_t*>(ptr))
#define WIT_ST16(arr, row, v) (*reinterpret_cast<v4i_t*>(&arr[(row) * kMfLd + wx]) = (v))
    auto fetch = [&](uint32_t k) {
#pragma unroll
        for (int pa = 0; pa < PA; pa++)
#pragma unroll
            for (int h = 0; h < NA; h++) sa[pa][h] = WIT_LD16(ga[h] + pa * pla + k);
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int h = 0; h < NB; h++) sb[pb][h] = WIT_LD16(gb[h] + pb * plb + k);
    };
    fetch(0);
    for (uint32_t k0 = 0; k0 < p.Kp; k0 += kMfK) {
        __syncthreads();
#pragma unroll
        for (int pa = 0; pa < PA; pa++)
#pragma unroll
            for (int h = 0; h < NA; h++) WIT_ST16(As, pa * kMfTN + RP * h + lr, sa[pa][h]);
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int h = 0; h < NB; h++) WIT_ST16(Bs, pb * kMfTM + RP * h + lr, sb[pb][h]);
        __syncthreads();
        if (k0 + kMfK < p.Kp) fetch(k0 + kMfK);
#pragma unroll
        for (int kk = 0; kk < kMfK; kk += 32) {
            v4i_t fa[PA], fb[PB][2];
#pragma unroll
            for (int pa = 0; pa < PA; pa++)
                fa[pa] = *reinterpret_cast<const v4i_t*>(&As[(pa * kMfTN + wn + frow) * kMfLd + (kk ^ fx)]);
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int tt = 0; tt < 2; tt++)
                    fb[pb][tt] = *reinterpret_cast<const v4i_t*>(&Bs[(pb * kMfTM + wm + 32 * tt + frow) * kMfLd + (kk ^ fx)]);
#pragma unroll
            for (int pa = 0; pa < PA; pa++)
#pragma unroll
                for (int pb = 0; pb < PB; pb++)
#pragma unroll
                    for (int tt = 0; tt < 2; tt++)
                        acc[pa + pb][tt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[pa], fb[pb][tt], acc[pa + pb][tt], 0, 0, 0);
        }
    }

#undef WIT_LD16
#undef WIT_ST16
    // accumulator register i of lane l holds row 8 (i / 4) + 4 (l / 32) + i % 4, column l % 32
    uint32_t bad = 0;
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
        const uint32_t m = m0 + wm + 32 * tt + (lane & 31u);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t n = n0 + wn + 8 * (i / 4) + 4 * (lane >> 5) + (i % 4);
            int64_t y = 0;
#pragma unroll
            for (int g = G - 1; g >= 0; g--) y = y * 256 + (int64_t)acc[g][tt][i];
            if (n < p.N && m < p.M) {
                int32_t q, r;
                rescale64(y, p.scale, p.shift, q, r, bad);
                const size_t o = p.transpose_out ? (size_t)m * p.N + n : (size_t)n * p.M + m;
                p.q[o] = q;
                if (p.r) p.r[o] = r;
            }
        }
    }
    if (bad) atomicOr(p.status, bad);
}

// The same product with a workgroup tile of 128 x 128 and eight waves (4 x 2, each 32 x 64 as above):
// a workgroup then asks L2 for 40 KB per K step and 192 matrix instructions where two workgroups of
// the kernel above ask for 56 KB, and L2 bandwidth is what the smaller tile runs into.  One workgroup
// fills a CU (two waves per SIMD), so the K steps alternate between two LDS stages with one barrier
// per step: a wave writes the operands of step k + 1 (in registers since step k - 1) to the other
// stage, requests those of step k + 2, and multiplies step k.  The products are v_mfma_i32_16x16x64_i8
// (2 x 4 tiles of 16 x 16 per wave, one instruction per tile, plane pair and K step): same
// fragments, registers and operations as with the 32 x 32 x 32 form, but the chip holds a higher
// clock under it (2.0 against 1.76 GHz in a loop of nothing else on random bytes).  Launched when
// the product has at least one such tile per CU.
template <int PA, int PB>
__global__ void __launch_bounds__(512, 2) wit_matmul_mfma_big_kernel(MfmaArgs p) {
    constexpr int G = PA + PB - 1;
    constexpr int CR = kMfK / 16, RL = 8 / CR;
    static_assert(512 / CR == kBgT, "one staging pass covers the tile's rows");
    constexpr int kStageA = PA * kBgT * kMfK, kStageB = PB * kBgT * kMfK;
    __shared__ __attribute__((aligned(16))) int8_t As[2 * kStageA];
    __shared__ __attribute__((aligned(16))) int8_t Bs[2 * kStageB];
    uint32_t tn, tm;
    mfma_tile_of(blockIdx.x, gridDim.x, p.tiles_n, p.tiles_m, tn, tm);
    const uint32_t n0 = tn * kBgT, m0 = tm * kBgT;
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    const uint32_t wn = (wave & 3u) * 32u, wm = (wave >> 2) * 64u;

    const uint32_t lr = t / CR, ck = 16u * (t % CR);
    v4i_t sa[PA], sb[PB];
    const uint32_t ra = n0 + lr, rb = m0 + lr;
    const int8_t* ga = p.a + (size_t)(ra < p.N ? ra : p.N - 1) * p.Kp + ck;
    const int8_t* gb = p.b + (size_t)(rb < p.M ? rb : p.M - 1) * p.Kp + ck;
    const size_t pla = (size_t)p.N * p.Kp, plb = (size_t)p.M * p.Kp;
    // v_mfma_i32_16x16x64_i8: one K step is one instruction deep; 2 x 4 tiles of 16 x 16 per wave
    v4i_t acc[G][2][4];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int ti = 0; ti < 2; ti++)
#pragma unroll
            for (int tj = 0; tj < 4; tj++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[g][ti][tj][i] = 0;

    // same chunk positions in LDS as in the kernel above
    const uint32_t frow = lane & 15u;
    const uint32_t fx = 16u * ((lane >> 4) ^ ((frow / RL) % CR));      // lane l holds row l % 16, bytes 16 (l / 16) .. + 16 of the step
    const uint32_t wx = 16u * ((t % CR) ^ ((lr / RL) % CR));
#define WIT_FETCH(k)                                                                                          \
    {                                                                                                         \
        _Pragma("unroll") for (int pa = 0; pa < PA; pa++) sa[pa] = *reinterpret_cast<const v4i_t*>(ga + pa * pla + (k)); \
        _Pragma("unroll") for (int pb = 0; pb < PB; pb++) sb[pb] = *reinterpret_cast<const v4i_t*>(gb + pb * plb + (k)); \
    }
#define WIT_STAGE(st)                                                                                         \
    {                                                                                                         \
        _Pragma("unroll") for (int pa = 0; pa < PA; pa++)                                                     \
            *reinterpret_cast<v4i_t*>(&As[(st) * kStageA + (pa * kBgT + lr) * kMfK + wx]) = sa[pa];           \
        _Pragma("unroll") for (int pb = 0; pb < PB; pb++)                                                     \
            *reinterpret_cast<v4i_t*>(&Bs[(st) * kStageB + (pb * kBgT + lr) * kMfK + wx]) = sb[pb];           \
    }
    WIT_FETCH(0);
    WIT_STAGE(0);
    if (kMfK < p.Kp) WIT_FETCH(kMfK);
    __syncthreads();
    uint32_t cur = 0;
    static_assert(kMfK == 64, "a K step is one matrix instruction deep");
    for (uint32_t k0 = 0; k0 < p.Kp; k0 += kMfK) {
        const int8_t* Ac = As + cur * kStageA;
        const int8_t* Bc = Bs + cur * kStageB;
        // this step's fragments are requested before the staging writes, which would otherwise queue ahead of them
        v4i_t fa[PA][2];
#pragma unroll
        for (int pa = 0; pa < PA; pa++)
#pragma unroll
            for (int ti = 0; ti < 2; ti++)
                fa[pa][ti] = *reinterpret_cast<const v4i_t*>(&Ac[(pa * kBgT + wn + 16 * ti + frow) * kMfK + fx]);
        if constexpr (PA + PB < 6) {
            v4i_t fb[PB][4];
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int tj = 0; tj < 4; tj++)
                    fb[pb][tj] = *reinterpret_cast<const v4i_t*>(&Bc[(pb * kBgT + wm + 16 * tj + frow) * kMfK + fx]);
            if (k0 + kMfK < p.Kp) {
                WIT_STAGE(cur ^ 1u);
                if (k0 + 2 * kMfK < p.Kp) WIT_FETCH(k0 + 2 * kMfK);
            }
#pragma unroll
            for (int ti = 0; ti < 2; ti++)
#pragma unroll
                for (int pa = 0; pa < PA; pa++)
#pragma unroll
                    for (int pb = 0; pb < PB; pb++)
#pragma unroll
                        for (int tj = 0; tj < 4; tj++)
                            acc[pa + pb][ti][tj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[pa][ti], fb[pb][tj], acc[pa + pb][ti][tj], 0, 0, 0);
        } else {
            // three planes on both sides: the fragments of b one tile column at a time, or the 160 accumulator
            // registers and 18 fragments do not fit
            if (k0 + kMfK < p.Kp) {
                WIT_STAGE(cur ^ 1u);
                if (k0 + 2 * kMfK < p.Kp) WIT_FETCH(k0 + 2 * kMfK);
            }
#pragma unroll
            for (int tj = 0; tj < 4; tj++) {
                v4i_t fb[PB];
#pragma unroll
                for (int pb = 0; pb < PB; pb++) fb[pb] = *reinterpret_cast<const v4i_t*>(&Bc[(pb * kBgT + wm + 16 * tj + frow) * kMfK + fx]);
#pragma unroll
                for (int ti = 0; ti < 2; ti++)
#pragma unroll
                    for (int pa = 0; pa < PA; pa++)
#pragma unroll
                        for (int pb = 0; pb < PB; pb++)
                            acc[pa + pb][ti][tj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[pa][ti], fb[pb], acc[pa + pb][ti][tj], 0, 0, 0);
            }
        }
        __syncthreads();
        cur ^= 1u;
    }
#undef WIT_FETCH
#undef WIT_STAGE

    // accumulator register i of lane l holds row 4 (l / 16) + i, column l % 16 of its tile
    uint32_t bad = 0;
#pragma unroll
    for (int ti = 0; ti < 2; ti++)
#pragma unroll
        for (int tj = 0; tj < 4; tj++) {
            const uint32_t m = m0 + wm + 16 * tj + (lane & 15u);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t n = n0 + wn + 16 * ti + 4 * (lane >> 4) + i;
                int64_t y = 0;
#pragma unroll
                for (int g = G - 1; g >= 0; g--) y = y * 256 + (int64_t)acc[g][ti][tj][i];
                if (n < p.N && m < p.M) {
                    int32_t q, r;
                    rescale64(y, p.scale, p.shift, q, r, bad);
                    const size_t o = p.transpose_out ? (size_t)m * p.N + n : (size_t)n * p.M + m;
                    p.q[o] = q;
                    if (p.r) p.r[o] = r;
                }
            }
        }
    if (bad) atomicOr(p.status, bad);
}

__global__ void __launch_bounds__(kBlock) wit_elemul_rescale_kernel(int32_t* q, int32_t* r, const int32_t* a, const int32_t* b, size_t n,
                                                                    int64_t scale, int shift, uint32_t* status) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    uint32_t bad = 0;
    int32_t qq, rr;
    rescale64((int64_t)a[i] * (int64_t)b[i], scale, shift, qq, rr, bad);
    q[i] = qq;
    if (r) r[i] = rr;
    if (bad) atomicOr(status, bad);
}

__global__ void __launch_bounds__(kBlock) wit_lookup_kernel(int32_t* out, const int32_t* in, size_t n, int32_t low, uint32_t len,
                                                            const int32_t* table, uint32_t* status) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t idx = (int64_t)in[i] - (int64_t)low;
    const bool ok = idx >= 0 && idx < (int64_t)len;
    out[i] = table[ok ? idx : 0];
    if (!ok) atomicOr(status, (uint32_t)kWitIndex);
}

__global__ void __launch_bounds__(kBlock) wit_add_kernel(int32_t* out, const int32_t* a, const int32_t* b, size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = (int32_t)((uint32_t)a[i] + (uint32_t)b[i]);
}

// block-wide reductions over 256 threads (4 waves)
__device__ __forceinline__ int32_t block_max_i32(int32_t v, int32_t* sh) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const int32_t o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    int32_t m = sh[0];
#pragma unroll
    for (int w = 1; w < kBlock / 64; w++) m = sh[w] > m ? sh[w] : m;
    __syncthreads();
    return m;
}
__device__ __forceinline__ uint64_t block_sum_u64(uint64_t v, uint64_t* sh) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor((unsigned long long)v, off, 64);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    uint64_t s = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) s += sh[w];
    __syncthreads();
    return s;
}

// One workgroup per row of the scores (model.py:76-116).
__global__ void __launch_bounds__(kBlock) wit_softmax_kernel(int32_t* out_max, int32_t* out_shift, int32_t* out_exp, int32_t* out_sum,
                                                             int32_t* out_prob, int32_t* out_query, const int32_t* scores, uint32_t cols,
                                                             const int32_t* table, uint32_t offset, uint32_t len, int64_t scale,
                                                             uint32_t* status) {
    __shared__ int32_t sh_i[kBlock / 64];
    __shared__ uint64_t sh_u[kBlock / 64];
    const size_t row = blockIdx.x;
    const int32_t* x = scores + row * cols;
    int32_t mx = INT32_MIN;
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock) mx = x[c] > mx ? x[c] : mx;
    mx = block_max_i32(mx, sh_i);
    uint64_t sum = 0;
    uint32_t bad = 0;
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock) {
        const int64_t d = (int64_t)x[c] - (int64_t)mx;               // <= 0
        const int64_t idx = d + (int64_t)offset;
        const bool ok = idx >= 0 && idx < (int64_t)len;
        const int32_t e = table[ok ? idx : 0];
        bad |= ok ? 0u : (uint32_t)kWitIndex;
        bad |= e < 0 ? (uint32_t)kWitSum : 0u;
        out_shift[row * cols + c] = (int32_t)d;
        out_exp[row * cols + c] = e;
        sum += (uint64_t)(uint32_t)(e < 0 ? 0 : e);
    }
    sum = block_sum_u64(sum, sh_u);
    if (sum == 0) {
        bad |= (uint32_t)kWitSum;
        sum = 1;
    }
    if (threadIdx.x == 0) {
        out_max[row] = mx;
        out_sum[row] = (int32_t)sum;            // the reference stores the 64-bit sum as int32 (model.py:103)
    }
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock) {
        const uint64_t e = (uint64_t)(uint32_t)out_exp[row * cols + c];   // this thread's own earlier store
        const uint64_t o = (e * (uint64_t)scale + (sum >> 1)) / sum;
        out_prob[row * cols + c] = (int32_t)o;
        out_query[row * cols + c] = (int32_t)((int64_t)(e * 2u * (uint64_t)scale) - (int64_t)sum * (2 * (int64_t)o - 1));
    }
    if (bad) atomicOr(status, bad);
}

// per row: exact sum of squares as a 64-bit integer (status flag when it leaves 64 bits)
__global__ void __launch_bounds__(kBlock) wit_row_sumsq_kernel(uint64_t* out, const int32_t* x, uint32_t cols, uint32_t* status) {
    __shared__ uint64_t sh_u[kBlock / 64];
    const size_t row = blockIdx.x;
    uint64_t lo = 0, hi = 0;
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock) {
        const int64_t v = x[row * cols + c];
        const uint64_t sq = (uint64_t)(v * v);
        lo += sq;
        hi += lo < sq ? 1u : 0u;
    }
    // the high parts and the low parts are summed separately; low parts are split so that their
    // block sum cannot wrap (256 values below 2^56 each)
    const uint64_t lo_lo = lo & 0x00ffffffffffffffull, lo_hi = lo >> 56;
    const uint64_t s_lo = block_sum_u64(lo_lo, sh_u);
    const uint64_t s_hi = block_sum_u64(lo_hi + (hi << 8), sh_u);     // units of 2^56
    if (threadIdx.x == 0) {
        const uint64_t top = s_hi + (s_lo >> 56);                      // total = top * 2^56 + (s_lo mod 2^56)
        if (top >> 8) atomicOr(status, (uint32_t)kWitSquares);
        out[row] = (top << 56) | (s_lo & 0x00ffffffffffffffull);
    }
}

// model.py:228-234: rms_w = rescale(rms[row] * w[col]); out = rescale(rms_w.q * x)
__global__ void __launch_bounds__(kBlock) wit_rmsnorm_apply_kernel(int32_t* q_rmsw, int32_t* r_rmsw, int32_t* q_out, int32_t* r_out,
                                                                   const int32_t* x, const int32_t* rms, const int32_t* w, size_t n,
                                                                   uint32_t cols, int64_t scale, int shift, uint32_t* status) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const size_t row = i / cols;
    const uint32_t col = (uint32_t)(i - row * cols);
    uint32_t bad = 0;
    int32_t q1, r1, q2, r2;
    rescale64((int64_t)rms[row] * (int64_t)w[col], scale, shift, q1, r1, bad);
    rescale64((int64_t)q1 * (int64_t)x[i], scale, shift, q2, r2, bad);
    q_rmsw[i] = q1;
    r_rmsw[i] = r1;
    q_out[i] = q2;
    r_out[i] = r2;
    if (bad) atomicOr(status, bad);
}

__global__ void wit_status_clear_kernel(uint32_t* status) { *status = 0; }

static uint32_t* g_status[16] = {nullptr};

static int status_word(uint32_t** out, hipStream_t s) {
    int dev = 0;
    GRAPE_HIP_CHECK(hipGetDevice(&dev));
    GRAPE_REQUIRE(dev >= 0 && dev < 16, "device index out of range");
    if (!g_status[dev]) {
        GRAPE_HIP_CHECK(hipMalloc((void**)&g_status[dev], 256));
        wit_status_clear_kernel<<<1, 1, 0, s>>>(g_status[dev]);
        GRAPE_LAUNCH_CHECK();
        GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    }
    *out = g_status[dev];
    return GRAPE_OK;
}

static int g_matmul_method = 0;   // 0 = choose, 1 = multiply-add kernels only, 2 = matrix cores or fail

// signed byte planes needed for magnitudes up to maxabs (one spare bit keeps the top digit small)
static int planes_for(uint32_t maxabs) {
    if (maxabs < (1u << 6)) return 1;
    if (maxabs < (1u << 14)) return 2;
    if (maxabs < (1u << 22)) return 3;
    if (maxabs < (1u << 30)) return 4;
    return 5;
}

static int log2_exact(int64_t s) {
    if (s <= 0 || (s & (s - 1)) != 0) return -1;
    int sh = 0;
    while ((((int64_t)1) << sh) != s) sh++;
    return sh;
}

}  // namespace grape

using namespace grape;

#define CHECK_PTR(p) GRAPE_REQUIRE((p) != nullptr, #p " is null")

extern "C" {

int grape_wit_matmul_rescale(int32_t* d_q, int32_t* d_r, const int32_t* d_a, const int32_t* d_b, uint32_t L, uint32_t N, uint32_t M,
                             uint32_t K, int64_t scale, int transpose_out, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    GRAPE_REQUIRE(scale >= 1 && scale <= ((int64_t)1 << 31), "scale must be in 1..2^31 (the remainder is stored as int32)");
    if (L == 0 || N == 0 || M == 0) return GRAPE_OK;
    CHECK_PTR(d_q); CHECK_PTR(d_a); CHECK_PTR(d_b);
    GRAPE_REQUIRE(K >= 1, "empty inner dimension");
    GRAPE_REQUIRE((uint64_t)L * N * M < ((uint64_t)1 << 40) && (uint64_t)N * K < ((uint64_t)1 << 40) && (uint64_t)M * K < ((uint64_t)1 << 40),
                  "tensor too large");
    hipStream_t s = as_stream(st);
    MatmulArgs p;
    p.q = d_q; p.r = d_r; p.a = d_a; p.b = d_b;
    p.N = N; p.M = M; p.K = K;
    p.scale = scale;
    p.shift = log2_exact(scale);
    p.transpose_out = transpose_out ? 1 : 0;
    p.tiles_n = (N + kTM - 1) / kTM;
    p.tiles_m = (M + kTM - 1) / kTM;
    int rc = status_word(&p.status, s);
    if (rc) return rc;
    const bool aligned = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_a) | reinterpret_cast<uintptr_t>(d_b)) & 15) == 0;
    // matrix-core path: one batch, aligned rows, operands of at most three byte planes each.  The split into
    // three planes also reports the operands' largest magnitudes; planes that turn out to be zero are left
    // out of the product, and operands beyond three planes go to the multiply-add kernel.
    bool use_mfma = false;
    int PA = 0, PB = 0;
    const uint32_t Kp = (K + kMfK - 1) / kMfK * kMfK;
    void *pa = nullptr, *pb = nullptr;
    if (g_matmul_method != 1 && L == 1 && aligned && (g_matmul_method == 2 || (uint64_t)N * M * K >= ((uint64_t)1 << 26))) {
        void* mx;
        rc = scratch_get(kSlotMisc, 64, &mx, s);
        if (rc) return rc;
        rc = scratch_get(kSlotWitA, (size_t)3 * N * Kp, &pa, s);
        if (rc) return rc;
        rc = scratch_get(kSlotWitB, (size_t)3 * M * Kp, &pb, s);
        if (rc) return rc;
        uint32_t* d_mx = (uint32_t*)mx;
        if (profiling()) {
            profile_begin();
            profile_mark(s);
        }
        wit_status_clear_kernel<<<1, 1, 0, s>>>(d_mx);
        wit_status_clear_kernel<<<1, 1, 0, s>>>(d_mx + 1);
        // at least 8 groups of 4 per thread, at most 2048 workgroups (one atomic each)
        const size_t ga_ = ((size_t)N * (Kp / 4) + kBlock * 8 - 1) / (kBlock * 8), gb_ = ((size_t)M * (Kp / 4) + kBlock * 8 - 1) / (kBlock * 8);
        wit_split_kernel<<<(unsigned)(ga_ < 2048 ? ga_ : 2048), kBlock, 0, s>>>((int8_t*)pa, d_mx, d_a, N, K, Kp);
        wit_split_kernel<<<(unsigned)(gb_ < 2048 ? gb_ : 2048), kBlock, 0, s>>>((int8_t*)pb, d_mx + 1, d_b, M, K, Kp);
        GRAPE_LAUNCH_CHECK();
        if (profiling()) profile_mark(s);
        uint32_t h_mx[2] = {0, 0};
        GRAPE_HIP_CHECK(hipMemcpyAsync(h_mx, d_mx, sizeof(h_mx), hipMemcpyDeviceToHost, s));
        GRAPE_HIP_CHECK(hipStreamSynchronize(s));
        if (profiling()) profile_mark(s);      // intervals: the split, the host's read of the magnitudes, the product
        PA = planes_for(h_mx[0]);
        PB = planes_for(h_mx[1]);
        if (PA < 2) PA = 2;
        if (PB < 2) PB = 2;
        const int pmin = PA < PB ? PA : PB;
        use_mfma = PA <= 3 && PB <= 3 && (uint64_t)Kp * pmin < 131072;   // a group stays below 2^31
    }
    GRAPE_REQUIRE(!(g_matmul_method == 2 && !use_mfma), "the matrix-core path needs one batch, K a multiple of 4, 16-byte aligned rows and operands below 2^22");
    if (profiling() && !use_mfma) {
        profile_begin();
        profile_mark(s);
    }
    if (use_mfma) {
        MfmaArgs m;
        m.q = d_q; m.r = d_r; m.a = (const int8_t*)pa; m.b = (const int8_t*)pb;
        m.N = N; m.M = M; m.Kp = Kp;
        m.scale = scale; m.shift = p.shift; m.transpose_out = p.transpose_out;
        m.status = p.status;
        const uint64_t big_tiles = (uint64_t)((N + kBgT - 1) / kBgT) * ((M + kBgT - 1) / kBgT);
        if (big_tiles >= (uint64_t)kNumCU) {
            m.tiles_n = (N + kBgT - 1) / kBgT;
            m.tiles_m = (M + kBgT - 1) / kBgT;
            const unsigned grid = (unsigned)big_tiles;
            if (PA == 2 && PB == 2) wit_matmul_mfma_big_kernel<2, 2><<<grid, 512, 0, s>>>(m);
            else if (PA == 3 && PB == 2) wit_matmul_mfma_big_kernel<3, 2><<<grid, 512, 0, s>>>(m);
            else if (PA == 2 && PB == 3) wit_matmul_mfma_big_kernel<2, 3><<<grid, 512, 0, s>>>(m);
            else wit_matmul_mfma_big_kernel<3, 3><<<grid, 512, 0, s>>>(m);
        } else {
            m.tiles_n = (N + kMfTN - 1) / kMfTN;
            m.tiles_m = (M + kMfTM - 1) / kMfTM;
            const unsigned grid = m.tiles_n * m.tiles_m;
            if (PA == 2 && PB == 2) wit_matmul_mfma_kernel<2, 2><<<grid, 256, 0, s>>>(m);
            else if (PA == 3 && PB == 2) wit_matmul_mfma_kernel<3, 2><<<grid, 256, 0, s>>>(m);
            else if (PA == 2 && PB == 3) wit_matmul_mfma_kernel<2, 3><<<grid, 256, 0, s>>>(m);
            else wit_matmul_mfma_kernel<3, 3><<<grid, 256, 0, s>>>(m);
        }
    } else if (aligned && L <= 65535) {
        dim3 grid(p.tiles_n * p.tiles_m, L);
        wit_matmul_tiled_kernel<<<grid, 256, 0, s>>>(p);
    } else {
        wit_matmul_simple_kernel<<<blocks_for((size_t)L * N * M), kBlock, 0, s>>>(p, L);
    }
    GRAPE_LAUNCH_CHECK();
    if (profiling()) profile_mark(s);
    return GRAPE_OK;
}

int grape_wit_set_matmul_method(int method) {
    GRAPE_REQUIRE(method >= 0 && method <= 2, "method must be 0 (choose), 1 (multiply-add kernels) or 2 (matrix cores)");
    g_matmul_method = method;
    return GRAPE_OK;
}

int grape_wit_elemul_rescale(int32_t* d_q, int32_t* d_r, const int32_t* d_a, const int32_t* d_b, size_t n, int64_t scale, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    GRAPE_REQUIRE(scale >= 1 && scale <= ((int64_t)1 << 31), "scale must be in 1..2^31 (the remainder is stored as int32)");
    if (n == 0) return GRAPE_OK;
    CHECK_PTR(d_q); CHECK_PTR(d_a); CHECK_PTR(d_b);
    hipStream_t s = as_stream(st);
    uint32_t* status;
    int rc = status_word(&status, s);
    if (rc) return rc;
    wit_elemul_rescale_kernel<<<blocks_for(n), kBlock, 0, s>>>(d_q, d_r, d_a, d_b, n, scale, log2_exact(scale), status);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wit_table_lookup(int32_t* d_out, const int32_t* d_in, size_t n, int32_t low, uint32_t len, const int32_t* d_table, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    GRAPE_REQUIRE(len >= 1, "empty table");
    if (n == 0) return GRAPE_OK;
    CHECK_PTR(d_out); CHECK_PTR(d_in); CHECK_PTR(d_table);
    hipStream_t s = as_stream(st);
    uint32_t* status;
    int rc = status_word(&status, s);
    if (rc) return rc;
    wit_lookup_kernel<<<blocks_for(n), kBlock, 0, s>>>(d_out, d_in, n, low, len, d_table, status);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wit_add_i32(int32_t* d_out, const int32_t* d_a, const int32_t* d_b, size_t n, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    if (n == 0) return GRAPE_OK;
    CHECK_PTR(d_out); CHECK_PTR(d_a); CHECK_PTR(d_b);
    wit_add_kernel<<<blocks_for(n), kBlock, 0, as_stream(st)>>>(d_out, d_a, d_b, n);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wit_softmax(int32_t* d_max, int32_t* d_shifted, int32_t* d_exp, int32_t* d_sum, int32_t* d_prob, int32_t* d_query,
                      const int32_t* d_scores, uint32_t rows, uint32_t cols, const int32_t* d_table, uint32_t bit_shift,
                      uint32_t index_bits, int64_t scale, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    GRAPE_REQUIRE(bit_shift >= 1 && bit_shift <= 30 && index_bits >= 1 && index_bits <= 30, "bit_shift and index_bits must be in 1..30");
    GRAPE_REQUIRE(scale >= 1 && scale <= ((int64_t)1 << 30), "scale must be in 1..2^30");
    if (rows == 0) return GRAPE_OK;
    GRAPE_REQUIRE(cols >= 1, "empty rows");
    CHECK_PTR(d_max); CHECK_PTR(d_shifted); CHECK_PTR(d_exp); CHECK_PTR(d_sum); CHECK_PTR(d_prob); CHECK_PTR(d_query);
    CHECK_PTR(d_scores); CHECK_PTR(d_table);
    hipStream_t s = as_stream(st);
    uint32_t* status;
    int rc = status_word(&status, s);
    if (rc) return rc;
    wit_softmax_kernel<<<rows, kBlock, 0, s>>>(d_max, d_shifted, d_exp, d_sum, d_prob, d_query, d_scores, cols, d_table,
                                               (1u << bit_shift) - 1u, 1u << index_bits, scale, status);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wit_row_sumsq(uint64_t* d_out, const int32_t* d_x, uint32_t rows, uint32_t cols, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    if (rows == 0) return GRAPE_OK;
    GRAPE_REQUIRE(cols >= 1, "empty rows");
    CHECK_PTR(d_out); CHECK_PTR(d_x);
    hipStream_t s = as_stream(st);
    uint32_t* status;
    int rc = status_word(&status, s);
    if (rc) return rc;
    wit_row_sumsq_kernel<<<rows, kBlock, 0, s>>>(d_out, d_x, cols, status);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wit_rmsnorm_apply(int32_t* d_q_rmsw, int32_t* d_r_rmsw, int32_t* d_q_out, int32_t* d_r_out, const int32_t* d_x,
                            const int32_t* d_rms, const int32_t* d_w, uint32_t rows, uint32_t cols, int64_t scale, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    GRAPE_REQUIRE(scale >= 1 && scale <= ((int64_t)1 << 31), "scale must be in 1..2^31 (the remainder is stored as int32)");
    if (rows == 0) return GRAPE_OK;
    GRAPE_REQUIRE(cols >= 1, "empty rows");
    CHECK_PTR(d_q_rmsw); CHECK_PTR(d_r_rmsw); CHECK_PTR(d_q_out); CHECK_PTR(d_r_out); CHECK_PTR(d_x); CHECK_PTR(d_rms); CHECK_PTR(d_w);
    hipStream_t s = as_stream(st);
    uint32_t* status;
    int rc = status_word(&status, s);
    if (rc) return rc;
    const size_t n = (size_t)rows * cols;
    wit_rmsnorm_apply_kernel<<<blocks_for(n), kBlock, 0, s>>>(d_q_rmsw, d_r_rmsw, d_q_out, d_r_out, d_x, d_rms, d_w, n, cols, scale,
                                                              log2_exact(scale), status);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

int grape_wit_status(uint32_t* flags, grape_stream_t st) {
    GRAPE_REQUIRE(initialised(), "grape_init has not been called");
    CHECK_PTR(flags);
    hipStream_t s = as_stream(st);
    uint32_t* status;
    int rc = status_word(&status, s);
    if (rc) return rc;
    GRAPE_HIP_CHECK(hipMemcpyAsync(flags, status, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    wit_status_clear_kernel<<<1, 1, 0, s>>>(status);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

}  // extern "C"
