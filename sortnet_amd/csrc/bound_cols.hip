// Interval-bound forward from per-weight-row candidate tables (see bound_cols.h).
#include "bound_cols.h"

namespace sd {

namespace {

constexpr int kChunk = kColsChunk;   // inputs per table word
constexpr int kTileB = 128;          // batch rows of a tile: 64 lanes x 2
constexpr int kTileW = 128;          // weight rows of a workgroup of the main kernel: 16 wavefronts x 8
constexpr int kLowSlices = 8;        // slices of the input range in the two table kernels
constexpr int kStage = 64;           // inputs of one LDS stage of the per-weight-row main kernel (two table words)

inline size_t align256(size_t b) { return (b + 255) / 256 * 256; }
inline int tiles_b(int B) { return (B + kTileB - 1) / kTileB; }
inline int mpad_of(int M) { return (M + kTileW - 1) / kTileW * kTileW; }

struct Carve {
    float* xr;        // [S][4][N]  per batch tile and input: min l, max l, min u, max u over the tile's rows (repaired)
    float* wr;        // [T][2][N]  per weight tile and input: min w, max w over the tile's rows
    float* low;       // [S][2][Mp] (or [T][2][Bp]) lower bounds of the upper / lower result of every output of the table's rows
    float* stat;      // two sums of col_range_kernel's probe, directly behind `low` (one fill clears both)
    unsigned long long* count;   // [0] marks of the per-weight-row table, [1] of the per-batch-row table, [2] every-term kernel's turn
    uint32_t* bits;   // [S][NCH][Mp] (or [T][Bp][NCH]): bit i of a word = input 32 c + i may hold a maximum of that row in that tile
    uint32_t* partial;   // marks per wavefront of the table kernel
    uint32_t* order;  // [S][Mp] per batch tile and block of 128 weight rows: the row (0..127) at each place of the block
    float* xt;        // [S][N][64][4] per batch tile and input: (l, l', u, u') of the tile's rows i and i + 64, repaired
    float* wt;        // [T][N][128] per weight tile and input: the weights of the tile's rows (the per-batch-row kernel walks these)
};

inline int bpad_of(int B) { return (B + kTileB - 1) / kTileB * kTileB; }
inline size_t maxz(size_t a, size_t b) { return a > b ? a : b; }

size_t carve_sizes(int B, int M, int N, size_t (&sz)[9]) {
    const size_t S = tiles_b(B), Mp = mpad_of(M), Bp = bpad_of(B), T = Mp / kTileW, NCH = N / kChunk;
    sz[0] = align256(S * 4 * N * 4);                               // xr
    sz[1] = align256(T * 2 * N * 4);                               // wr
    sz[2] = align256(maxz(S * 2 * Mp, T * 2 * Bp) * 4 + 8);        // low + stat
    sz[3] = 256;                                                   // count
    sz[4] = align256(maxz(S * NCH * Mp, T * NCH * Bp) * 4);        // bits
    sz[5] = align256(maxz(Mp / 64, Bp / 64 * ((T + 3) / 4)) * kLowSlices * 4 * 4);   // partial
    sz[6] = align256(S * N * 1024);                                // xt
    sz[7] = align256(S * Mp * 4);                                  // order
    sz[8] = align256(Mp * N * 4);                                  // wt
    return sz[0] + sz[1] + sz[2] + sz[3] + sz[4] + sz[5] + sz[6] + sz[7] + sz[8];
}

Carve carve(void* ws, int B, int M, int N) {
    size_t sz[9];
    carve_sizes(B, M, N, sz);
    const size_t S = tiles_b(B), Mp = mpad_of(M), Bp = bpad_of(B), T = Mp / kTileW;
    char* p = static_cast<char*>(ws);
    Carve c;
    c.xr = reinterpret_cast<float*>(p); p += sz[0];
    c.wr = reinterpret_cast<float*>(p); p += sz[1];
    c.low = reinterpret_cast<float*>(p);
    c.stat = c.low + maxz(S * 2 * Mp, T * 2 * Bp);
    p += sz[2];
    c.count = reinterpret_cast<unsigned long long*>(p); p += sz[3];
    c.bits = reinterpret_cast<uint32_t*>(p); p += sz[4];
    c.partial = reinterpret_cast<uint32_t*>(p); p += sz[5];
    c.xt = reinterpret_cast<float*>(p); p += sz[6];
    c.order = reinterpret_cast<uint32_t*>(p); p += sz[7];
    c.wt = reinterpret_cast<float*>(p);
    return c;
}

// inverted intervals become their midpoint (core/cuda/bound_inf_dist_cuda.cu:63)
__device__ __forceinline__ void repair(float& l, float& u) {
    if (l > u) l = u = (l + u) * 0.5f;
}

// ---- tables ----------------------------------------------------------------------------------
// Also answers whether the table is worth building: it can only prune when the rows of a batch tile are alike
// compared with the entries of a weight row.  stat[0] collects the widths of the column ranges of l and u over all
// tiles and columns, stat[1] the ranges of the same columns over the first 16 weight rows (added once, by the
// workgroups of tile 0); see rows_decide().
__global__ void __launch_bounds__(256) col_range_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                        const float* __restrict__ w, int B, int M, int N,
                                                        float* __restrict__ xr, float* __restrict__ stat) {
    // 64 inputs x 4 groups of 32 rows per workgroup, combined through LDS
    __shared__ float part[4][5][64];
    __shared__ float wpart[4][2][64];
    const int nl = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + nl, s = blockIdx.y;
    const int r0 = s * kTileB + grp * (kTileB / 4);
    const int r1 = r0 + kTileB / 4 < B ? r0 + kTileB / 4 : B;
    float lmin = __builtin_inff(), lmax = -__builtin_inff(), umin = __builtin_inff(), umax = -__builtin_inff();
    float wlo = __builtin_inff(), whi = -__builtin_inff();
    float odd = 0.f;   // stays 0 while every l and u of the column is finite
    if (n < N) {
        #pragma unroll 4
        for (int r = r0; r < r1; r++) {
            float l = xl[(size_t)r * N + n], u = xu[(size_t)r * N + n];
            odd += (l - l) + (u - u);
            repair(l, u);
            lmin = fminf(lmin, l); lmax = fmaxf(lmax, l);
            umin = fminf(umin, u); umax = fmaxf(umax, u);
        }
        if (s == 0) {
            #pragma unroll
            for (int k = 0; k < 4; k++) {
                const int m = grp * 4 + k;
                if (m < M) { const float v = w[(size_t)m * N + n]; wlo = fminf(wlo, v); whi = fmaxf(whi, v); }
            }
        }
    }
    part[grp][0][nl] = lmin; part[grp][1][nl] = lmax; part[grp][2][nl] = umin; part[grp][3][nl] = umax;
    part[grp][4][nl] = odd;
    wpart[grp][0][nl] = wlo; wpart[grp][1][nl] = whi;
    __syncthreads();
    if (grp == 0) {
        float bw = 0.f, ww = 0.f;
        if (n < N) {
            #pragma unroll
            for (int g = 1; g < 4; g++) {
                lmin = fminf(lmin, part[g][0][nl]); lmax = fmaxf(lmax, part[g][1][nl]);
                umin = fminf(umin, part[g][2][nl]); umax = fmaxf(umax, part[g][3][nl]);
                wlo = fminf(wlo, wpart[g][0][nl]); whi = fmaxf(whi, wpart[g][1][nl]);
                odd += part[g][4][nl];
            }
            // A row whose l or u is undefined or infinite at this input drops terms the other rows keep, so nothing
            // may be concluded from the column: its range becomes everything (no lower bound, always a candidate).
            if (!(odd == 0.f)) { lmin = umin = -__builtin_inff(); lmax = umax = __builtin_inff(); }
            float* o = xr + (size_t)s * 4 * N + n;
            o[0] = lmin; o[N] = lmax; o[2 * (size_t)N] = umin; o[3 * (size_t)N] = umax;
            bw = fmaxf(lmax - lmin, umax - umin);
            if (s == 0) ww = whi - wlo;
            if (!(bw < 3.0e38f)) bw = 3.0e38f;   // infinite or undefined widths count as very wide
        }
        #pragma unroll
        for (int o = 32; o; o >>= 1) { bw += __shfl_xor(bw, o); ww += __shfl_xor(ww, o); }
        if (nl == 0) {
            unsafeAtomicAdd(stat, bw);
            if (s == 0) unsafeAtomicAdd(stat + 1, ww);
        }
    }
}

// The batch rows of a tile differ by more than kProbeRatio times what 16 entries of a weight column do (images
// against small weights: ratio 15; the bounds of hidden layers: below 1): a table per weight row would mark every
// input, because it is the batch row that decides where the maximum sits.  Then the table is built the other way
// round, per batch row and tile of 128 weight rows (row_* kernels below); otherwise per weight row (col_*).
constexpr float kProbeRatio = 2.5f;
__device__ __forceinline__ bool rows_decide(const float* stat, int S) {
    return stat[0] > kProbeRatio * (float)S * stat[1];
}

// The two table kernels share their tiling: a workgroup takes 64 weight rows (one per lane) and a slice of the
// inputs; wavefront v works on batch tile v (+ 4, + 8, ...), for which the column ranges are wave-uniform
// (LDS broadcasts); the weights go through LDS, 64 x 32 at a time, so that a lane can own a row.
//   LOW:  lower bounds of the results, max_n of the smallest each term can be over the rows of the tile
//         (fp32 subtraction is monotone, so the bound holds for the rounded terms), merged over the slices by
//         atomic maximum of the bit patterns (all values >= 1e-10 > 0 on zero-filled memory);
//   else: one table word per (tile, chunk, weight row): bit n set when the largest the term can be reaches the
//         lower bound of the upper or of the lower result; the marks are counted.
// Within a block of 128 weight rows the words are not stored in the order of the rows.  The main kernel gives each
// of its 16 wavefronts eight places of a block and a workgroup ends with its slowest wavefront, while the marks of a
// row vary several-fold around their mean (with consecutive rows the fullest wavefront carries 1.2-1.35 times the
// mean).  A row's lower bounds tell how many marks it will get (the smaller of the two ranks the rows of a block
// nearly as their mark counts do), so the rows are ranked by it, smallest (most marks) first, and dealt back and
// forth: ranks 0..15 to wavefronts 0..15, ranks 16..31 to wavefronts 15..0, and so on.  order[] names the row at
// each place.
template <bool LOW>
__device__ __forceinline__ void col_table_body(const float* __restrict__ w, const float* __restrict__ xr,
                                               int M, int N, int S, int Mp, float* __restrict__ low,
                                               uint32_t* __restrict__ bits, uint32_t* __restrict__ partial,
                                               uint32_t* __restrict__ order, int bx, int by, int gx, int gy) {
    // row stride 36 words: 16-byte rows, and the 128-bit reads of 16 consecutive lanes fall on disjoint banks
    __shared__ __attribute__((aligned(16))) float wt[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float xs[4][4][kChunk];   // column ranges of the four batch tiles of this pass, current chunk
    __shared__ float keys[LOW ? 1 : 4][LOW ? 1 : kTileW];            // per batch tile of this pass: what the rows of the block are ranked by
    const int tid = threadIdx.x, r = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = bx * 64, NCH = N / kChunk;
    const int per = (NCH + gy - 1) / gy;
    const int c_lo = by * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;
    const int lrow = tid >> 2, q = tid & 3;
    const int mload = m0 + lrow < M ? m0 + lrow : M - 1;
    const bool valid = m0 + r < M;
    // this work-item's two values of xs: tile tid / 64 of the pass, range tid / 16 % 4, inputs 2 (tid % 16), + 1
    const int xt = tid >> 6, xk = (tid >> 4) & 3, xn = 2 * (tid & 15);
    int marks = 0;
    for (int sb = 0; sb < S; sb += 4) {
        const int s = sb + wave;
        const bool active = s < S;
        float LU = kEps, LL = kEps;
        int wordrow = m0 + r;   // where this row's words go: its place within its block of 128
        if (!LOW && active) {
            LU = fmaxf(kEps, low[(size_t)(s * 2) * Mp + m0 + r]);
            LL = fmaxf(kEps, low[(size_t)(s * 2 + 1) * Mp + m0 + r]);
            const int mb = m0 & ~(kTileW - 1), mine = m0 - mb + r;
            #pragma unroll
            for (int j = r; j < kTileW; j += 64) {
                const float a = fmaxf(kEps, low[(size_t)(s * 2) * Mp + mb + j]);
                const float b = fmaxf(kEps, low[(size_t)(s * 2 + 1) * Mp + mb + j]);
                keys[wave][j] = mb + j < M ? fminf(a, b) : __builtin_inff();   // rows past the last one have no marks
            }
            __builtin_amdgcn_wave_barrier();   // LDS operations of one wavefront complete in order
            const float key = keys[wave][mine];
            int rank = 0;
            for (int j = 0; j < kTileW; j++) {
                const float other = keys[wave][j];
                rank += (other < key || (other == key && j < mine)) ? 1 : 0;
            }
            const int k = rank >> 4, j = rank & 15;
            wordrow = mb + ((k & 1) ? 15 - j : j) * 8 + k;
            if (by == 0) order[(size_t)s * Mp + wordrow] = (uint32_t)mine;
        }
        // the weights and ranges of the next chunk are fetched while the current one is used
        float4 pa, pb;
        float2 px;
        const float* xsrc = xr + ((size_t)(sb + xt < S ? sb + xt : S - 1) * 4 + xk) * N + xn;
        auto fetch = [&](int c) {
            const int cc = c < c_hi ? c : c_hi - 1;
            const float* src = w + (size_t)mload * N + cc * kChunk + 8 * q;
            pa = *reinterpret_cast<const float4*>(src); pb = *reinterpret_cast<const float4*>(src + 4);
            px = *reinterpret_cast<const float2*>(xsrc + cc * kChunk);
        };
        if (c_lo < c_hi) fetch(c_lo);
        for (int c = c_lo; c < c_hi; c++) {
            {
                *reinterpret_cast<float4*>(&wt[lrow][8 * q]) = pa;
                *reinterpret_cast<float4*>(&wt[lrow][8 * q + 4]) = pb;
                *reinterpret_cast<float2*>(&xs[xt][xk][xn]) = px;
            }
            fetch(c + 1);
            __syncthreads();
            if (active) {
                uint32_t word = 0;
                #pragma unroll
                for (int n4 = 0; n4 < kChunk; n4 += 4) {
                    const float4 wv4 = *reinterpret_cast<const float4*>(&wt[r][n4]);
                    const float4 a4 = *reinterpret_cast<const float4*>(&xs[wave][0][n4]);   // min l
                    const float4 b4 = *reinterpret_cast<const float4*>(&xs[wave][1][n4]);   // max l
                    const float4 c4 = *reinterpret_cast<const float4*>(&xs[wave][2][n4]);   // min u
                    const float4 d4 = *reinterpret_cast<const float4*>(&xs[wave][3][n4]);   // max u
                    const float wv[4] = {wv4.x, wv4.y, wv4.z, wv4.w};
                    const float lmin[4] = {a4.x, a4.y, a4.z, a4.w}, lmax[4] = {b4.x, b4.y, b4.z, b4.w};
                    const float umin[4] = {c4.x, c4.y, c4.z, c4.w}, umax[4] = {d4.x, d4.y, d4.z, d4.w};
                    #pragma unroll
                    for (int k = 0; k < 4; k++) {
                        if (LOW) {
                            LU = fmaxf(fmaxf(LU, umin[k] - wv[k]), wv[k] - lmax[k]);
                            LL = fmaxf(fmaxf(LL, lmin[k] - wv[k]), wv[k] - umax[k]);
                        } else {
                            const float capU = fmaxf(wv[k] - lmin[k], umax[k] - wv[k]);
                            const float capL = fmaxf(lmax[k] - wv[k], wv[k] - umin[k]);
                            word |= (uint32_t)(!(capU < LU) || !(capL < LL)) << (n4 + k);   // undefined counts as a candidate
                        }
                    }
                }
                if (!LOW) {
                    if (!valid) word = 0u;
                    bits[((size_t)s * NCH + c) * Mp + wordrow] = word;
                    marks += __builtin_popcount(word);
                }
            }
            __syncthreads();
        }
        if (LOW && active && valid) {
            atomicMax(reinterpret_cast<int*>(low + (size_t)(s * 2) * Mp + m0 + r), __float_as_int(LU));
            atomicMax(reinterpret_cast<int*>(low + (size_t)(s * 2 + 1) * Mp + m0 + r), __float_as_int(LL));
        }
    }
    if (!LOW) {
        // one number per wavefront for sum_tables_kernel (atomics on one address would serialise)
        #pragma unroll
        for (int o = 32; o; o >>= 1) marks += __shfl_xor(marks, o);
        if (r == 0) partial[((size_t)by * gx + bx) * 4 + wave] = (uint32_t)marks;
    }
}

// ---- main kernel --------------------------------------------------------------------------
// A workgroup of 16 wavefronts owns 128 batch rows x 128 weight rows and a slice of the inputs.  Lane l holds the
// batch rows l and l + 64; wavefront v the weight rows 8 v .. 8 v + 7: 32 running minima / maxima per lane.  The
// inputs go by in stages of 64.  The (l, l', u, u') words of a lane's two rows come from a copy that xt_kernel has
// laid out per tile and input the way they lie in LDS (repaired, 1 KB per input), so staging is four 16-byte copies
// per work-item, fetched while the previous stage is used.  A wavefront's weights never enter LDS: lane n of register
// r holds w[row r][input n of the stage], and a marked input's weight is read from its lane.  The two table words of
// a (stage, weight row) are scalar loads.  A marked (weight row, input) pair then costs one 16-byte LDS read, one
// lane read and the eight vector instructions of the terms; the operands of a row's next mark are fetched while the
// current one is used.  The results leave through an LDS transpose (coalesced along the weight rows) and merge over
// the slices by atomic maximum.
constexpr int kStageFloats = kStage * 256;   // (l, l', u, u') of 64 lanes per input
// (two stages of inputs; with positions the results leave through two planes of 128 x 129 words)
constexpr int kLdsWords = 2 * kStageFloats > 2 * kTileB * (kTileW + 1) ? 2 * kStageFloats : 2 * kTileB * (kTileW + 1);

// (l, l', u, u') of the batch rows i and i + 64 of every tile, per input, repaired: the layout the main kernel keeps
// in LDS, so that it stages a tile with 16-byte copies.  16 inputs per workgroup.
__global__ void __launch_bounds__(256) xt_kernel(const float* __restrict__ xl, const float* __restrict__ xu, int B, int N,
                                                 const unsigned long long* __restrict__ count,
                                                 unsigned long long limit_col, float* __restrict__ xT) {
    if (count[0] > limit_col) return;
    __shared__ __attribute__((aligned(16))) float t[16 * 256];
    const int n0 = blockIdx.x * 16, s = blockIdx.y;
    const int row = threadIdx.x >> 1, half = threadIdx.x & 1;
    const int b = s * kTileB + row < B ? s * kTileB + row : B - 1;
    const float* pl = xl + (size_t)b * N + n0 + 8 * half;
    const float* pu = xu + (size_t)b * N + n0 + 8 * half;
    float4 l0 = *reinterpret_cast<const float4*>(pl), l1 = *reinterpret_cast<const float4*>(pl + 4);
    float4 u0 = *reinterpret_cast<const float4*>(pu), u1 = *reinterpret_cast<const float4*>(pu + 4);
    repair(l0.x, u0.x); repair(l0.y, u0.y); repair(l0.z, u0.z); repair(l0.w, u0.w);
    repair(l1.x, u1.x); repair(l1.y, u1.y); repair(l1.z, u1.z); repair(l1.w, u1.w);
    const float l[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
    const float u[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
    float* d = t + (8 * half) * 256 + 4 * (row & 63) + (row >> 6);
    #pragma unroll
    for (int k = 0; k < 8; k++) { d[k * 256] = l[k]; d[k * 256 + 2] = u[k]; }
    __syncthreads();
    float4* dst = reinterpret_cast<float4*>(xT + ((size_t)s * N + n0) * 256);
    const float4* src = reinterpret_cast<const float4*>(t);
    #pragma unroll
    for (int k = 0; k < 4; k++) dst[threadIdx.x + 256 * k] = src[threadIdx.x + 256 * k];
}

// POS: for the forward that also returns positions.  Every output then carries, next to its running minimum / maximum,
// the number (within the slice, 8 bits) of the 32-input chunk whose mark last raised it - the marks of a row go by in
// the order of the inputs and only a strictly better term replaces, so this is the chunk of the first input that
// attains the result, as the every-term kernel's chunk tracking finds it - and the slices merge as that kernel's do:
// 64-bit atomic maximum of (value bits << 32 | ~chunk) into packedL / packedU, from which resolve_bound_kernel takes
// values and positions.  Outputs that no term raised above the 1e-10 start write nothing.
template <bool POS>
__device__ __forceinline__ void bound_cols_body(const float* __restrict__ xT, const float* __restrict__ w,
                                                const uint32_t* __restrict__ bits, const uint32_t* __restrict__ order,
                                                int B, int M, int Mp, int N, int nsplit, float* __restrict__ yL,
                                                float* __restrict__ yU, unsigned long long* __restrict__ packedL,
                                                unsigned long long* __restrict__ packedU, float* smem) {
    constexpr int TW = 8;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int TM = (M + kTileW - 1) / kTileW, SB = (B + kTileB - 1) / kTileB, NCH = N / kChunk;
    const int NST = (NCH + 1) / 2;
    const int mt = blockIdx.x % TM, s = (blockIdx.x / TM) % SB, split = blockIdx.x / (TM * SB);
    const int m0 = mt * kTileW, b0 = s * kTileB;
    const int per = (NST + nsplit - 1) / nsplit;
    const int st_lo = split * per, st_hi = st_lo + per < NST ? st_lo + per : NST;

    float lo[TW][2], hi[TW][2];
    uint32_t cw[TW];   // POS: chunk numbers of (lower, lower', upper, upper') of a weight row, one byte each, 255 = none
    #pragma unroll
    for (int r = 0; r < TW; r++) { lo[r][0] = lo[r][1] = -kEps; hi[r][0] = hi[r][1] = kEps; cw[r] = 0xffffffffu; }

    // the rows at this wavefront's eight places of the block (wave-uniform)
    int row[TW];
    #pragma unroll
    for (int r = 0; r < TW; r++) row[r] = (int)order[(size_t)s * Mp + m0 + wave * TW + r];

    if (st_lo < st_hi) {
        const float* __restrict__ xsrc = xT + (size_t)s * N * 256;
        const size_t xlast = (size_t)N * 256 - 4;                       // the tile's last 16-byte word
        const uint32_t* __restrict__ bw = bits + (size_t)s * NCH * Mp + m0 + wave * TW;   // words of chunk c: bw[c * Mp + r]
        size_t wrow[TW];
        #pragma unroll
        for (int r = 0; r < TW; r++) wrow[r] = (size_t)(m0 + row[r] < M ? m0 + row[r] : M - 1) * N;

        auto load_x = [&](int st, float4 (&v)[4]) __attribute__((always_inline)) {
            #pragma unroll
            for (int k = 0; k < 4; k++) {
                size_t off = (size_t)st * kStageFloats + 4 * (size_t)(tid + 1024 * k);
                if (off > xlast) off = xlast;                            // half stage at the end of the inputs
                v[k] = *reinterpret_cast<const float4*>(xsrc + off);
            }
        };
        auto store_x = [&](int buf, const float4 (&v)[4]) __attribute__((always_inline)) {
            float4* d = reinterpret_cast<float4*>(smem + buf * kStageFloats);
            #pragma unroll
            for (int k = 0; k < 4; k++) d[tid + 1024 * k] = v[k];
        };
        auto load_w = [&](int st, float (&v)[TW]) __attribute__((always_inline)) {
            const int n = st * kStage + lane < N ? st * kStage + lane : N - 1;
            #pragma unroll
            for (int r = 0; r < TW; r++) v[r] = w[wrow[r] + n];
        };
        auto load_words = [&](int st, uint32_t (&a)[TW], uint32_t (&b)[TW]) __attribute__((always_inline)) {
            const int c0 = 2 * st, c1 = 2 * st + 1 < NCH ? 2 * st + 1 : 2 * st;
            const uint32_t keep = 2 * st + 1 < NCH ? 0xffffffffu : 0u;
            #pragma unroll
            for (int r = 0; r < TW; r++) {
                a[r] = bw[(size_t)c0 * Mp + r];
                b[r] = bw[(size_t)c1 * Mp + r] & keep;
            }
        };
        // kl4: the chunk number of the mark within the slice in all four bytes
        auto term = [&](float (&l2)[2], float (&h2)[2], uint32_t& c4, const float4& x, float wv, uint32_t kl4)
                        __attribute__((always_inline)) {
            const float a1 = wv - x.x, a2 = x.z - wv, b1 = wv - x.y, b2 = x.w - wv;
            if (POS) {
                const float m0 = fminf(a1, a2), M0 = fmaxf(a1, a2), m1 = fminf(b1, b2), M1 = fmaxf(b1, b2);
                const bool w0 = m0 < l2[0], w1 = m1 < l2[1], w2 = M0 > h2[0], w3 = M1 > h2[1];
                l2[0] = w0 ? m0 : l2[0]; l2[1] = w1 ? m1 : l2[1];
                h2[0] = w2 ? M0 : h2[0]; h2[1] = w3 ? M1 : h2[1];
                c4 = w0 ? ((c4 & 0xffffff00u) | (kl4 & 0x000000ffu)) : c4;
                c4 = w1 ? ((c4 & 0xffff00ffu) | (kl4 & 0x0000ff00u)) : c4;
                c4 = w2 ? ((c4 & 0xff00ffffu) | (kl4 & 0x00ff0000u)) : c4;
                c4 = w3 ? ((c4 & 0x00ffffffu) | (kl4 & 0xff000000u)) : c4;
            } else {
                l2[0] = fminf(fminf(l2[0], a1), a2);
                h2[0] = fmaxf(fmaxf(h2[0], a1), a2);
                l2[1] = fminf(fminf(l2[1], b1), b2);
                h2[1] = fmaxf(fmaxf(h2[1], b1), b2);
            }
        };
        // a weight row's marks of the stage, in order; the operands of the next mark are on their way while the
        // current one is used
        auto compute = [&](int buf, int st, const float (&wv)[TW], const uint32_t (&wa)[TW], const uint32_t (&wb2)[TW])
                           __attribute__((always_inline)) {
            const float* X = smem + buf * kStageFloats + 4 * lane;
            const uint32_t k0 = (uint32_t)(2 * (st - st_lo));
            auto kl4 = [&](int n) __attribute__((always_inline)) { return (k0 + (uint32_t)(n >> 5)) * 0x01010101u; };
            #pragma unroll
            for (int r = 0; r < TW; r++) {
                unsigned long long bm = ((unsigned long long)wb2[r] << 32) | (unsigned long long)wa[r];
                if (bm) {
                    int n = __builtin_ctzll(bm);
                    bm &= bm - 1;
                    float4 xa = *reinterpret_cast<const float4*>(X + n * 256), xb;
                    float va = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv[r]), n)), vb;
                    uint32_t ka = kl4(n), kb;
                    while (true) {
                        if (!bm) { term(lo[r], hi[r], cw[r], xa, va, ka); break; }
                        n = __builtin_ctzll(bm);
                        bm &= bm - 1;
                        xb = *reinterpret_cast<const float4*>(X + n * 256);
                        vb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv[r]), n));
                        kb = kl4(n);
                        term(lo[r], hi[r], cw[r], xa, va, ka);
                        if (!bm) { term(lo[r], hi[r], cw[r], xb, vb, kb); break; }
                        n = __builtin_ctzll(bm);
                        bm &= bm - 1;
                        xa = *reinterpret_cast<const float4*>(X + n * 256);
                        va = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv[r]), n));
                        ka = kl4(n);
                        term(lo[r], hi[r], cw[r], xb, vb, kb);
                    }
                }
            }
        };

        float4 xs[4];
        float wc[TW], wn[TW];
        uint32_t a0[TW], a1[TW], n0[TW], n1[TW];
        load_x(st_lo, xs); load_w(st_lo, wc); load_words(st_lo, a0, a1);
        store_x(0, xs);
        __syncthreads();
        for (int st = st_lo; st < st_hi; st++) {
            const int buf = (st - st_lo) & 1;
            const int nx = st + 1 < st_hi ? st + 1 : st;   // the last stage is fetched once more rather than behind a test
            load_x(nx, xs); load_w(nx, wn); load_words(nx, n0, n1);
            compute(buf, st, wc, a0, a1);
            store_x(buf ^ 1, xs);
            #pragma unroll
            for (int r = 0; r < TW; r++) { wc[r] = wn[r]; a0[r] = n0[r]; a1[r] = n1[r]; }
            __syncthreads();
        }
    }

    if (POS) {
        // (value, chunk) pairs: [batch row][weight row] through LDS, lower then upper, values and chunk numbers side by side
        float* tv = smem;
        uint32_t* tc = reinterpret_cast<uint32_t*>(smem) + kTileB * (kTileW + 1);
        const uint32_t c_first = (uint32_t)(2 * st_lo);
        #pragma unroll
        for (int which = 0; which < 2; which++) {
            __syncthreads();
            #pragma unroll
            for (int r = 0; r < TW; r++) {
                #pragma unroll
                for (int j = 0; j < 2; j++) {
                    tv[(lane + 64 * j) * (kTileW + 1) + row[r]] = which == 0 ? -lo[r][j] : hi[r][j];
                    tc[(lane + 64 * j) * (kTileW + 1) + row[r]] = (cw[r] >> (16 * which + 8 * j)) & 0xffu;
                }
            }
            __syncthreads();
            unsigned long long* y = which == 0 ? packedL : packedU;
            for (int e = tid; e < kTileB * kTileW; e += 1024) {
                const int bl = e >> 7, ml = e & (kTileW - 1);
                const uint32_t kl = tc[bl * (kTileW + 1) + ml];
                if (b0 + bl < B && m0 + ml < M && kl != 0xffu) {
                    const unsigned long long key =
                        ((unsigned long long)__float_as_uint(tv[bl * (kTileW + 1) + ml]) << 32) |
                        (unsigned long long)(0xffffffffu - (c_first + kl));
                    atomicMax(y + (size_t)(b0 + bl) * M + m0 + ml, key);
                }
            }
        }
        return;
    }
    // results: [batch row][weight row] through LDS, lower then upper
    float* tr = smem;
    #pragma unroll
    for (int which = 0; which < 2; which++) {
        __syncthreads();
        #pragma unroll
        for (int r = 0; r < TW; r++) {
            #pragma unroll
            for (int j = 0; j < 2; j++)
                tr[(lane + 64 * j) * (kTileW + 1) + row[r]] = which == 0 ? -lo[r][j] : hi[r][j];
        }
        __syncthreads();
        float* y = which == 0 ? yL : yU;
        for (int e = tid; e < kTileB * kTileW; e += 1024) {
            const int bl = e >> 7, ml = e & (kTileW - 1);
            if (b0 + bl < B && m0 + ml < M) {
                const float v = tr[bl * (kTileW + 1) + ml];
                float* dst = y + (size_t)(b0 + bl) * M + m0 + ml;
                // both results are >= 1e-10 > 0, so their bit patterns order like integers
                if (nsplit > 1) atomicMax(reinterpret_cast<int*>(dst), __float_as_int(v));
                else *dst = v;
            }
        }
    }
}

// ---- the other orientation: tables per batch row and tile of 128 weight rows ----------------------
// Over a tile of 128 weight rows the terms of (b, n) are bracketed by the column minimum and maximum of the weights.
// Same three steps with the roles exchanged: ranges of W per (tile, input), lower bounds of the results per
// (tile, batch row), marks per (tile, chunk, batch row).  All of them return at once unless rows_decide().
__global__ void __launch_bounds__(256) row_range_kernel(const float* __restrict__ w, int M, int N, int S,
                                                        float* __restrict__ wr, float* __restrict__ wt,
                                                        const float* __restrict__ stat) {
    if (!rows_decide(stat, S)) return;
    __shared__ float part[4][3][64];
    const int nl = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + nl, t = blockIdx.y;
    const int r0 = t * kTileW + grp * (kTileW / 4);
    float lo = __builtin_inff(), hi = -__builtin_inff(), odd = 0.f;
    if (n < N) {
        // also the transposed copy the main kernel walks: wt[(t N + n) 128 + row of the tile] (rows past the last: 0)
        float v[kTileW / 4];
        #pragma unroll
        for (int i = 0; i < kTileW / 4; i++) v[i] = r0 + i < M ? w[(size_t)(r0 + i) * N + n] : 0.f;
        #pragma unroll
        for (int i = 0; i < kTileW / 4; i++) {
            if (r0 + i < M) { lo = fminf(lo, v[i]); hi = fmaxf(hi, v[i]); odd += v[i] - v[i]; }
        }
        float4* dst = reinterpret_cast<float4*>(wt + ((size_t)t * N + n) * kTileW + grp * (kTileW / 4));
        #pragma unroll
        for (int i = 0; i < kTileW / 16; i++) dst[i] = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    }
    part[grp][0][nl] = lo; part[grp][1][nl] = hi; part[grp][2][nl] = odd;
    __syncthreads();
    if (grp == 0 && n < N) {
        #pragma unroll
        for (int g = 1; g < 4; g++) { lo = fminf(lo, part[g][0][nl]); hi = fmaxf(hi, part[g][1][nl]); odd += part[g][2][nl]; }
        // an undefined or infinite weight drops terms its neighbours keep: the column's range becomes everything
        if (!(odd == 0.f)) { lo = -__builtin_inff(); hi = __builtin_inff(); }
        wr[(size_t)(t * 2) * N + n] = lo;
        wr[(size_t)(t * 2 + 1) * N + n] = hi;
    }
}

// a workgroup takes 64 batch rows (one per lane; l and u through LDS, repaired) and a slice of the inputs; wavefront
// v works on weight tile 4 blockIdx.z + v, whose column ranges are LDS broadcasts
template <bool LOW>
__device__ __forceinline__ void row_table_body(const float* __restrict__ xl, const float* __restrict__ xu,
                                               const float* __restrict__ wr, int B, int N, int T, int Bp,
                                               float* __restrict__ low, uint32_t* __restrict__ bits,
                                               uint32_t* __restrict__ partial, int bx, int by, int bz, int gx, int gy) {
    __shared__ __attribute__((aligned(16))) float lt[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float ut[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float ws[4][2][kChunk];   // min w, max w of the four weight tiles of this pass
    const int tid = threadIdx.x, r = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b0 = bx * 64, NCH = N / kChunk;
    const int per = (NCH + gy - 1) / gy;
    const int c_lo = by * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;
    const int lrow = tid >> 2, q = tid & 3;
    const int bload = b0 + lrow < B ? b0 + lrow : B - 1;
    const bool valid = b0 + r < B;
    const int xt = tid >> 6, xk = (tid >> 5) & 1, xn = tid & 31;   // this work-item's value of ws
    int marks = 0;
    {
        const int tb = bz * 4;
        const int t = tb + wave;
        const bool active = t < T;
        float LU = kEps, LL = kEps;
        if (!LOW && active) {
            LU = fmaxf(kEps, low[(size_t)(t * 2) * Bp + b0 + r]);
            LL = fmaxf(kEps, low[(size_t)(t * 2 + 1) * Bp + b0 + r]);
        }
        float4 la, lb, ua, ub;
        float px;
        const float* wsrc = wr + ((size_t)(tb + xt < T ? tb + xt : T - 1) * 2 + xk) * N + xn;
        auto fetch = [&](int c) {
            const int cc = c < c_hi ? c : c_hi - 1;
            const size_t off = (size_t)bload * N + cc * kChunk + 8 * q;
            la = *reinterpret_cast<const float4*>(xl + off); lb = *reinterpret_cast<const float4*>(xl + off + 4);
            ua = *reinterpret_cast<const float4*>(xu + off); ub = *reinterpret_cast<const float4*>(xu + off + 4);
            px = wsrc[cc * kChunk];
        };
        if (c_lo < c_hi) fetch(c_lo);
        for (int c = c_lo; c < c_hi; c++) {
            {
                float4 a = la, b = lb, d = ua, e = ub;
                repair(a.x, d.x); repair(a.y, d.y); repair(a.z, d.z); repair(a.w, d.w);
                repair(b.x, e.x); repair(b.y, e.y); repair(b.z, e.z); repair(b.w, e.w);
                *reinterpret_cast<float4*>(&lt[lrow][8 * q]) = a; *reinterpret_cast<float4*>(&lt[lrow][8 * q + 4]) = b;
                *reinterpret_cast<float4*>(&ut[lrow][8 * q]) = d; *reinterpret_cast<float4*>(&ut[lrow][8 * q + 4]) = e;
                ws[xt][xk][xn] = px;
            }
            fetch(c + 1);
            __syncthreads();
            if (active) {
                uint32_t word = 0;
                #pragma unroll
                for (int n4 = 0; n4 < kChunk; n4 += 4) {
                    const float4 l4 = *reinterpret_cast<const float4*>(&lt[r][n4]);
                    const float4 u4 = *reinterpret_cast<const float4*>(&ut[r][n4]);
                    const float4 a4 = *reinterpret_cast<const float4*>(&ws[wave][0][n4]);   // min w
                    const float4 b4 = *reinterpret_cast<const float4*>(&ws[wave][1][n4]);   // max w
                    const float l[4] = {l4.x, l4.y, l4.z, l4.w}, u[4] = {u4.x, u4.y, u4.z, u4.w};
                    const float wmin[4] = {a4.x, a4.y, a4.z, a4.w}, wmax[4] = {b4.x, b4.y, b4.z, b4.w};
                    #pragma unroll
                    for (int k = 0; k < 4; k++) {
                        if (LOW) {
                            LU = fmaxf(fmaxf(LU, wmin[k] - l[k]), u[k] - wmax[k]);
                            LL = fmaxf(fmaxf(LL, l[k] - wmax[k]), wmin[k] - u[k]);
                        } else {
                            const float capU = fmaxf(wmax[k] - l[k], u[k] - wmin[k]);
                            const float capL = fmaxf(l[k] - wmin[k], wmax[k] - u[k]);
                            word |= (uint32_t)(!(capU < LU) || !(capL < LL)) << (n4 + k);   // undefined counts as a candidate
                        }
                    }
                }
                if (!LOW) {
                    if (!valid) word = 0u;
                    bits[((size_t)t * Bp + b0 + r) * NCH + c] = word;   // a row's words side by side
                    marks += __builtin_popcount(word);
                }
            }
            __syncthreads();
        }
        if (LOW && active && valid) {
            atomicMax(reinterpret_cast<int*>(low + (size_t)(t * 2) * Bp + b0 + r), __float_as_int(LU));
            atomicMax(reinterpret_cast<int*>(low + (size_t)(t * 2 + 1) * Bp + b0 + r), __float_as_int(LL));
        }
    }
    if (!LOW) {
        #pragma unroll
        for (int o = 32; o; o >>= 1) marks += __shfl_xor(marks, o);
        if (r == 0)
            partial[(((size_t)bz * gy + by) * gx + bx) * 4 + wave] = (uint32_t)marks;
    }
}

// Both table steps as one launch each: the probe picks the orientation, and workgroups beyond the grid of that
// orientation return at once.
template <bool LOW>
__global__ void __launch_bounds__(256) table_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                    const float* __restrict__ w, const float* __restrict__ xr,
                                                    const float* __restrict__ wr, int B, int M, int N, int S, int T,
                                                    int Mp, int Bp, int slices, float* __restrict__ low,
                                                    uint32_t* __restrict__ bits, uint32_t* __restrict__ partial,
                                                    uint32_t* __restrict__ order, const float* __restrict__ stat) {
    const int id = blockIdx.x;
    if (rows_decide(stat, S)) {
        const int gx = Bp / 64, gy = slices, gz = (T + 3) / 4;
        if (id >= gx * gy * gz) return;
        row_table_body<LOW>(xl, xu, wr, B, N, T, Bp, low, bits, partial, id % gx, (id / gx) % gy, id / (gx * gy), gx, gy);
    } else {
        const int gx = Mp / 64, gy = slices;
        if (id >= gx * gy) return;
        col_table_body<LOW>(w, xr, M, N, S, Mp, low, bits, partial, order, id % gx, id / gx, gx, gy);
    }
}

// count[0] = marks of the table per weight row, count[1] = of the table per batch row (the one that was not built
// counts as full), count[2] = 1 when neither is below its limit, which is what the every-term kernel waits for,
// count[3] = 1 when the per-weight-row marks are below a sixteenth of their limit (for the caller's choice of kernel),
// count[4] = 1 when the kernel of the tables per batch row runs (with positions it stores the final results itself)
__global__ void __launch_bounds__(1024) sum_tables_kernel(const uint32_t* __restrict__ partial, size_t n_col,
                                                          size_t n_row, unsigned long long* __restrict__ count,
                                                          const float* __restrict__ stat, int S,
                                                          unsigned long long limit_col, unsigned long long limit_row) {
    __shared__ unsigned long long acc[1024];
    const bool rows = rows_decide(stat, S);
    const size_t n = rows ? n_row : n_col;
    unsigned long long s0 = 0;
    for (size_t i = threadIdx.x; i < n; i += 1024) s0 += partial[i];
    acc[threadIdx.x] = s0;
    __syncthreads();
    for (int o = 512; o; o >>= 1) {
        if ((int)threadIdx.x < o) acc[threadIdx.x] += acc[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const unsigned long long c = rows ? ~0ull : acc[0], r = rows ? acc[0] : ~0ull;
        count[0] = c;
        count[1] = r;
        count[2] = (c > limit_col && r > limit_row) ? 1ull : 0ull;
        // so few marks per weight row that staging tiles through LDS is most of the main kernel's time
        count[3] = c <= limit_col / 16 ? 1ull : 0ull;
        count[4] = (c > limit_col && r <= limit_row) ? 1ull : 0ull;
    }
}

// Main kernel of this orientation.  A wavefront takes one batch row against the tile's 128 weight rows (lane l holds the
// rows l and l + 64): it reads the row's table words 64 chunks at a time, lists the marked inputs in LDS and walks the
// list four marks at a time with the loads of the next four in flight: lane l fetches the number and the (l, u) of mark
// l % 4 (read back lane by lane, so they are scalar operands of the terms), every lane its two weights from the
// transposed copy (two coalesced 256-byte loads per mark).  No tile is staged and no barrier is met; the workgroups of a
// tile (eight wavefronts = eight batch rows each) are dealt to one die, whose cache then holds the tile's transposed
// weights.  Every load is issued unconditionally (groups past the end of the list repeat its last mark and are not
// used).  One wavefront sees every input of its outputs, so the results are stored, not merged.
// POS: the mark that last improved a bound strictly is the first input attaining it (the marks go by in input order,
// and every input that attains a bound is marked), so values and positions are stored as they are
// (core/cuda/bound_inf_dist_cuda.cu:176-212: position = input | bit 31 when w - l > u - w; a lower bound that never
// left its floor keeps 0xffffffff) and the resolve pass is told to skip the call (count[4]).
constexpr int kWalkWaves = 8;        // wavefronts of a workgroup
constexpr int kWalkBatch = 64;       // chunks whose table words a wavefront reads at a time, one per lane
constexpr int kWalkListCap = 2304;   // entries of a wavefront's list of marked inputs (16-bit input numbers)

template <bool POS>
__global__ void __launch_bounds__(64 * kWalkWaves)
bound_rows_walk_kernel(const float* __restrict__ xl, const float* __restrict__ xu, const float* __restrict__ wt,
                       const uint32_t* __restrict__ bits, const unsigned long long* __restrict__ count,
                       unsigned long long limit_col, unsigned long long limit_row, int B, int Bp, int M, int N,
                       float* __restrict__ yL, float* __restrict__ yU, int* __restrict__ posL, int* __restrict__ posU) {
    if (count[0] <= limit_col || count[1] > limit_row) return;   // the other table's turn, or the every-term kernel's
    __shared__ uint16_t list[kWalkWaves][kWalkListCap];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int NCH = N / kChunk, BG = (B + kWalkWaves - 1) / kWalkWaves;
    int item = blockIdx.x;
    if (gridDim.x % 8 == 0) item = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int bg = item % BG, t = item / BG;
    const int b = bg * kWalkWaves + wave;
    if (b >= B) return;   // wave-uniform
    const float* __restrict__ wcol = wt + (size_t)t * N * kTileW + lane;
    uint16_t* mine = list[wave];
    const uint32_t* __restrict__ rowbits = bits + ((size_t)t * Bp + b) * NCH;
    const float* __restrict__ xlrow = xl + (size_t)b * N;
    const float* __restrict__ xurow = xu + (size_t)b * N;
    float lo[2] = {-kEps, -kEps}, hi[2] = {kEps, kEps};
    int pl[2] = {-1, -1}, pu[2] = {0, 0};   // POS: the input that last improved the bound, with its flag
    int cnt = 0;   // marks in the list
    float lreg[2], ureg[2];
    int nreg[2];
    float wa[2][4], wb[2][4];
    auto load = [&](int buf, int k0, int total) __attribute__((always_inline)) {
        int k = k0 + (lane & 3);
        k = k < total ? k : total - 1;
        const int nn = (int)mine[k];
        float l = xlrow[nn], u = xurow[nn];
        repair(l, u);
        lreg[buf] = l; ureg[buf] = u; nreg[buf] = nn;
        #pragma unroll
        for (int i = 0; i < 4; i++) {
            const int n = __builtin_amdgcn_readlane(nn, i);
            wa[buf][i] = wcol[(size_t)n * kTileW];
            wb[buf][i] = wcol[(size_t)n * kTileW + 64];
        }
    };
    auto compute = [&](int buf, int k0, int total) __attribute__((always_inline)) {
        #pragma unroll
        for (int i = 0; i < 4; i++) {
            if (k0 + i < total) {   // wave-uniform
                const float li = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, lreg[buf]), i));
                const float ui = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ureg[buf]), i));
                const float a1 = wa[buf][i] - li, a2 = ui - wa[buf][i], b1 = wb[buf][i] - li, b2 = ui - wb[buf][i];
                if constexpr (POS) {
                    const int n = __builtin_amdgcn_readlane(nreg[buf], i);
                    const int p0 = a1 <= a2 ? n : n | (int)0x80000000, p1 = b1 <= b2 ? n : n | (int)0x80000000;
                    const float v0 = fminf(a1, a2), V0 = fmaxf(a1, a2), v1 = fminf(b1, b2), V1 = fmaxf(b1, b2);
                    const bool w0 = v0 < lo[0], w1 = v1 < lo[1], w2 = V0 > hi[0], w3 = V1 > hi[1];
                    lo[0] = w0 ? v0 : lo[0]; lo[1] = w1 ? v1 : lo[1];
                    hi[0] = w2 ? V0 : hi[0]; hi[1] = w3 ? V1 : hi[1];
                    pl[0] = w0 ? p0 : pl[0]; pl[1] = w1 ? p1 : pl[1];
                    pu[0] = w2 ? p0 : pu[0]; pu[1] = w3 ? p1 : pu[1];
                } else {
                    lo[0] = fminf(fminf(lo[0], a1), a2);
                    hi[0] = fmaxf(fmaxf(hi[0], a1), a2);
                    lo[1] = fminf(fminf(lo[1], b1), b2);
                    hi[1] = fmaxf(fmaxf(hi[1], b1), b2);
                }
            }
        }
    };
    auto walk = [&](int total) __attribute__((always_inline)) {
        if (total == 0) return;
        load(0, 0, total);
        for (int k0 = 0; k0 < total; k0 += 8) {
            load(1, k0 + 4, total);
            compute(0, k0, total);
            load(0, k0 + 8, total);
            compute(1, k0 + 4, total);
        }
    };
    uint32_t next = lane < NCH ? rowbits[lane] : 0u;
    for (int c0 = 0; c0 < NCH; c0 += kWalkBatch) {
        uint32_t word = next;
        if (c0 + kWalkBatch < NCH) next = c0 + kWalkBatch + lane < NCH ? rowbits[c0 + kWalkBatch + lane] : 0u;
        // every lane appends the marks of its word behind those of the lanes before it
        const int mine_n = __builtin_popcount(word);
        int incl = mine_n;
        #pragma unroll
        for (int o = 1; o < kWalkBatch; o <<= 1) {
            const int v = __shfl_up(incl, o);
            if (lane >= o) incl += v;
        }
        int off = cnt + incl - mine_n;
        cnt += __builtin_amdgcn_readlane(incl, kWalkBatch - 1);
        while (word) {
            const int i = __builtin_ctz(word);
            word &= word - 1;
            mine[off++] = (uint16_t)(((c0 + lane) << 5) | i);   // the input's number (rows of at most 65536 inputs)
        }
        // a row's marks are walked in one go unless the list could overflow with the next chunks
        if (cnt > kWalkListCap - kWalkBatch * kChunk || c0 + kWalkBatch >= NCH) {
            __builtin_amdgcn_wave_barrier();
            walk(cnt);
            cnt = 0;
            __builtin_amdgcn_wave_barrier();   // the reads of the list come before the next marks
        }
    }
    #pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = t * kTileW + lane + 64 * j;
        if (col < M) {
            const size_t o = (size_t)b * M + col;
            yL[o] = -lo[j]; yU[o] = hi[j];
            if constexpr (POS) { posL[o] = pl[j]; posU[o] = pu[j]; }
        }
    }
}

// The kernel of the tables per weight row (the tables per batch row have bound_rows_walk_kernel)
template <bool POS>
__global__ void __launch_bounds__(1024, 1)
bound_table_kernel(const float* __restrict__ w, const float* __restrict__ xT, const uint32_t* __restrict__ bits,
                   const uint32_t* __restrict__ order, const unsigned long long* __restrict__ count,
                   unsigned long long limit_col, int B, int M, int Mp, int N, int nsplit, float* __restrict__ yL,
                   float* __restrict__ yU, unsigned long long* __restrict__ packedL,
                   unsigned long long* __restrict__ packedU) {
    __shared__ __attribute__((aligned(16))) float lds[kLdsWords];
    if (count[0] <= limit_col) bound_cols_body<POS>(xT, w, bits, order, B, M, Mp, N, nsplit, yL, yU, packedL, packedU, lds);
}

}  // namespace

size_t bound_cols_workspace(int B, int CO, int CI) {
    size_t sz[9];
    return carve_sizes(B, CO, CI, sz);
}

int bound_cols_forward(const float* xl, const float* xu, const float* w, int B, int CO, int CI, float* outL,
                       float* outU, unsigned long long* packedL, unsigned long long* packedU, int* posL, int* posU,
                       void* ws, float density, float density_rows, const unsigned long long** gate,
                       unsigned long long* gate_limit, hipStream_t st) {
    const bool with_pos = packedL != nullptr;
    if (CI % kChunk != 0 || B < 1 || CO < 1) { set_error("bound_cols_forward: shape not supported"); return SD_ERR_ARG; }
    const Carve c = carve(ws, B, CO, CI);
    const int S = tiles_b(B), Mp = mpad_of(CO), Bp = bpad_of(B), T = Mp / kTileW, NCH = CI / kChunk;
    const size_t lown = maxz((size_t)S * 2 * Mp, (size_t)T * 2 * Bp);
    int rc;
    if ((rc = fill_zero(c.low, lown + 2, st))) return rc;   // the lower bounds and the two sums behind them
    hipLaunchKernelGGL(col_range_kernel, dim3((CI + 63) / 64, S), dim3(256), 0, st, xl, xu, w, B, CO, CI, c.xr, c.stat);
    if ((rc = check_launch("col_range_kernel"))) return rc;
    const int slices = NCH < kLowSlices ? NCH : kLowSlices;
    const float d = density < 0.f ? 0.f : density > 1.f ? 1.f : density;
    const float dr = density_rows < 0.f ? 0.f : density_rows > 1.f ? 1.f : density_rows;
    const unsigned long long limit_col = (unsigned long long)((double)S * CO * CI * d);
    // (the kernel of the tables per batch row lists 16-bit input numbers)
    const unsigned long long limit_row = CI <= 65536 ? (unsigned long long)((double)T * B * CI * dr) : 0ull;
    // ranges of W per tile of weight rows and the transposed copy: only when the probe picks the tables per batch row
    hipLaunchKernelGGL(row_range_kernel, dim3((CI + 63) / 64, T), dim3(256), 0, st, w, CO, CI, S, c.wr, c.wt, c.stat);
    if ((rc = check_launch("row_range_kernel"))) return rc;
    const int wg_col = (Mp / 64) * slices, wg_row = (Bp / 64) * slices * ((T + 3) / 4);
    const int wg_tab = wg_col > wg_row ? wg_col : wg_row;
    hipLaunchKernelGGL(table_kernel<true>, dim3(wg_tab), dim3(256), 0, st, xl, xu, w, c.xr, c.wr, B, CO, CI, S, T, Mp, Bp,
                       slices, c.low, c.bits, c.partial, c.order, c.stat);
    if ((rc = check_launch("table_kernel<low>"))) return rc;
    hipLaunchKernelGGL(table_kernel<false>, dim3(wg_tab), dim3(256), 0, st, xl, xu, w, c.xr, c.wr, B, CO, CI, S, T, Mp, Bp,
                       slices, c.low, c.bits, c.partial, c.order, c.stat);
    if ((rc = check_launch("table_kernel<bits>"))) return rc;
    hipLaunchKernelGGL(sum_tables_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)wg_col * 4, (size_t)wg_row * 4,
                       c.count, c.stat, S, limit_col, limit_row);
    if ((rc = check_launch("sum_tables_kernel"))) return rc;
    // the every-term kernel runs when count[2] > 0
    *gate = c.count + 2;
    *gate_limit = 0ull;
    note_term_counts(c.count, 2, (double)S * CO * CI, (double)T * B * CI, limit_col);
    // a few workgroups per compute unit over the run: the work of a workgroup follows the marks of its rows
    hipLaunchKernelGGL(xt_kernel, dim3(CI / 16, S), dim3(256), 0, st, xl, xu, B, CI, c.count, limit_col, c.xt);
    if ((rc = check_launch("xt_kernel"))) return rc;
    // Slices of the input range.  A workgroup takes a whole compute unit and stays for its whole run, so the launch
    // proceeds in rounds of num_cus() workgroups and 2.5 rounds cost three: the count with the least time by that
    // model, each further slice priced at 4 % (its share of the merge), is taken.
    const long long wgs = (long long)T * S, cus = num_cus();
    int nsplit = 1;
    double best = 0.0;
    for (int n = 1; n <= 16 && (n == 1 || n <= NCH / 8); n++) {
        const double cost = (double)((wgs * n + cus - 1) / cus) / n * (1.0 + 0.04 * n);
        if (n == 1 || cost < best) { best = cost; nsplit = n; }
    }
    const int BG = (B + kWalkWaves - 1) / kWalkWaves;
    if (with_pos) {
        // chunk numbers within a slice take 8 bits (255 = none)
        while ((((NCH + 1) / 2 + nsplit - 1) / nsplit) * 2 > 254) nsplit++;
        hipLaunchKernelGGL(bound_table_kernel<true>, dim3((unsigned)(wgs * nsplit)), dim3(1024), 0, st, w, c.xt, c.bits,
                           c.order, c.count, limit_col, B, CO, Mp, CI, nsplit, nullptr, nullptr, packedL, packedU);
        if ((rc = check_launch("bound_table_kernel"))) return rc;
        hipLaunchKernelGGL(bound_rows_walk_kernel<true>, dim3((unsigned)(T * BG)), dim3(64 * kWalkWaves), 0, st, xl, xu, c.wt,
                           c.bits, c.count, limit_col, limit_row, B, Bp, CO, CI, outL, outU, posL, posU);
        return check_launch("bound_rows_walk_kernel");
    }
    hipLaunchKernelGGL(bound_table_kernel<false>, dim3((unsigned)(wgs * nsplit)), dim3(1024), 0, st, w, c.xt, c.bits, c.order,
                       c.count, limit_col, B, CO, Mp, CI, nsplit, outL, outU, nullptr, nullptr);
    if ((rc = check_launch("bound_table_kernel"))) return rc;
    hipLaunchKernelGGL(bound_rows_walk_kernel<false>, dim3((unsigned)(T * BG)), dim3(64 * kWalkWaves), 0, st, xl, xu, c.wt, c.bits,
                       c.count, limit_col, limit_row, B, Bp, CO, CI, outL, outU, nullptr, nullptr);
    return check_launch("bound_rows_walk_kernel");
}

}  // namespace sd
