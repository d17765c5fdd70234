// Sort neuron and its interval bounds from per-weight-row candidate tables (see sort_cols.h).
#include "sort_cols.h"
#include <type_traits>
#include <utility>
#include "fwd_tile.h"

namespace sd {

namespace {

constexpr int kChunk = kSortColsChunk;
constexpr int kTileB = 128;          // batch rows of a tile: 64 lanes x 2
constexpr int kRowPad = 128;         // weight rows are padded to a multiple of this in the tables
constexpr int kMaxPer = 32;          // most chunks a slice of the table kernels covers
constexpr int kMainWaves = 8;        // wavefronts of a workgroup of the main kernel
constexpr int kMainRows = 1;         // weight rows a wavefront of the main kernel takes, one after the other
constexpr int kMainTile = kMainWaves * kMainRows;   // weight rows of a workgroup: its results leave 128 bytes wide
constexpr int kBatch = 64;           // chunks whose table words a wavefront reads at a time, one per lane
constexpr int kListCap = 2304;       // entries of a wavefront's list of marked inputs (16-bit input numbers)

inline size_t align256(size_t b) { return (b + 255) / 256 * 256; }
inline int tiles_b(int B) { return (B + kTileB - 1) / kTileB; }
inline int mpad_of(int M) { return (M + kRowPad - 1) / kRowPad * kRowPad; }
inline int slices_of(int NCH) {
    int s = (NCH + kMaxPer - 1) / kMaxPer;
    if (s < 16) s = 16;
    return s < NCH ? s : NCH;
}

struct Carve {
    float* xr;        // [S][4][N]   per batch tile and input: min l, max l, min u, max u over the tile's rows
    float* xT;        // [N][Bp]     the inputs transposed ((l, u) pairs in the interval form), intervals repaired
    float* lists;     // [S][slices][2][K][Mp]  K largest chunk maxima of the lower bounds of a weight row's terms within a slice
    float* low;       // [S][2][Mp]  K-th largest of them over all slices: upper list, lower list
    uint32_t* bits;   // [S][Mp][NCH] bit i of a word = input 32 c + i may be among the K largest of that row in that tile
    uint32_t* partial;   // marks per wavefront of the table kernel
    unsigned long long* count;
    float* stat;      // two sums of sc_range_kernel's probe, 16 bytes behind the count and its flag (one fill clears all of it)
};

size_t carve_sizes(int B, int M, int N, int K, size_t (&sz)[7]) {
    const size_t S = tiles_b(B), Bp = S * kTileB, Mp = mpad_of(M), NCH = N / kChunk, slices = slices_of((int)NCH);
    sz[0] = align256(S * 4 * N * 4);
    sz[1] = align256((size_t)N * Bp * 8);
    sz[2] = align256(S * slices * 2 * K * Mp * 4);
    sz[3] = align256(S * 2 * Mp * 4);
    sz[4] = align256(S * Mp * NCH * 4);
    sz[5] = align256(Mp / 64 * slices * 4 * 4);
    sz[6] = 256;
    size_t t = 0;
    for (size_t v : sz) t += v;
    return t;
}

Carve carve(void* ws, int B, int M, int N, int K) {
    size_t sz[7];
    carve_sizes(B, M, N, K, sz);
    char* p = static_cast<char*>(ws);
    Carve c;
    c.xr = reinterpret_cast<float*>(p); p += sz[0];
    c.xT = reinterpret_cast<float*>(p); p += sz[1];
    c.lists = reinterpret_cast<float*>(p); p += sz[2];
    c.low = reinterpret_cast<float*>(p); p += sz[3];
    c.bits = reinterpret_cast<uint32_t*>(p); p += sz[4];
    c.partial = reinterpret_cast<uint32_t*>(p); p += sz[5];
    c.count = reinterpret_cast<unsigned long long*>(p);
    c.stat = reinterpret_cast<float*>(p + 16);
    return c;
}

// inverted intervals become their midpoint (core/cuda/sort_neuron.cu:262)
__device__ __forceinline__ void repair(float& l, float& u) {
    if (l > u) l = u = (l + u) * 0.5f;
}

// Top-K lists are kept as the bit patterns of their values (all >= 0, where signed integers order like the
// floats): new[k] = max(res[k], min(res[k+1], v)) (core/cuda/sort_neuron.cu:76-77) = the median of the three, one integer
// instruction per slot.  A negative v (sign bit set: a negative integer) is below every entry and changes nothing;
// an undefined v with a clear sign bit would order above every number, so callers hand over defined values only.
__device__ __forceinline__ int imed3(int a, int b, int c) {
    int r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
template <int K>
__device__ __forceinline__ void insert_bits(int (&res)[K], float value) {
    const int v = __builtin_bit_cast(int, value);
    #pragma unroll
    for (int k = 0; k < K - 1; k++) res[k] = imed3(res[k], v, res[k + 1]);
    res[K - 1] = max(res[K - 1], v);
}
template <int K>
__device__ __forceinline__ float geo_sum_bits(const int (&res)[K], float q) {
    float f[K];
    #pragma unroll
    for (int k = 0; k < K; k++) f[k] = __builtin_bit_cast(float, res[k]);
    return geo_sum<K>(f, q);
}

// ---- tables ----------------------------------------------------------------------------------
// Column ranges of a tile of 128 batch rows x 64 inputs, and the transposed copy of the tile the main kernel reads
// (one row of 128 values per input).  Value form: l = u = x.
// Also answers whether the table is worth building: it can only prune when the rows of a batch tile are alike
// compared with the entries of a weight row.  stat[0] collects the widths of the column ranges over all tiles and
// columns, stat[1] the ranges of the same columns over the first 16 weight rows (added once, by the workgroups of
// tile 0); see table_pointless().
// MASKED (value form only): xkeep holds one word per (batch row, 32 inputs); an input a row does not keep takes no
// part in the ranges and is undefined in the transposed copy, so that its term never wins a comparison.  A column no
// row of the tile keeps has neither a lower bound nor a candidate.
template <bool IV, bool MASKED>
__global__ void __launch_bounds__(256) sc_range_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                       const float* __restrict__ w, const uint32_t* __restrict__ xkeep,
                                                       int B, int M, int N, int Bp, float* __restrict__ xr,
                                                       float* __restrict__ xT, float* __restrict__ stat) {
    static_assert(!(IV && MASKED), "the factored mask belongs to the value form");
    __shared__ float part[4][5][64];
    __shared__ float wpart[4][2][64];
    __shared__ float tl[64][kTileB + 1];
    __shared__ float tu[IV ? 64 : 1][kTileB + 1];
    const int tid = threadIdx.x, nl = tid & 63, grp = tid >> 6;
    const int n0 = blockIdx.x * 64, n = n0 + nl, s = blockIdx.y;
    float lmin = __builtin_inff(), lmax = -__builtin_inff(), umin = __builtin_inff(), umax = -__builtin_inff();
    float odd = 0.f;   // stays 0 while every value of the column is finite
    #pragma unroll 4
    for (int r = 0; r < kTileB / 4; r++) {
        const int col = grp * (kTileB / 4) + r, row = s * kTileB + col;
        float l = 0.f, u = 0.f;
        if (n < N && row < B) {
            l = xl[(size_t)row * N + n];
            u = IV ? xu[(size_t)row * N + n] : l;
            bool kept = true;
            if constexpr (MASKED) kept = (xkeep[(size_t)row * (N / kChunk) + (n >> 5)] >> (n & 31)) & 1u;
            if (kept) {
                odd += (l - l) + (u - u);
                if (IV) repair(l, u);
                lmin = fminf(lmin, l); lmax = fmaxf(lmax, l);
                umin = fminf(umin, u); umax = fmaxf(umax, u);
            } else l = u = __builtin_nanf("");
        }
        tl[nl][col] = l;
        if (IV) tu[nl][col] = u;
    }
    // the probe: ranges of the same columns over the first 16 weight rows (tile 0 only)
    float wlo = __builtin_inff(), whi = -__builtin_inff();
    if (s == 0 && n < N) {
        #pragma unroll
        for (int k = 0; k < 4; k++) {
            const int m = grp * 4 + k;
            if (m < M) { const float v = w[(size_t)m * N + n]; wlo = fminf(wlo, v); whi = fmaxf(whi, v); }
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
            // A row whose value is undefined or infinite at this input drops terms the other rows keep, so nothing
            // may be concluded from the column: its range becomes everything (no lower bound, always a candidate).
            if (!(odd == 0.f)) { lmin = umin = -__builtin_inff(); lmax = umax = __builtin_inff(); }
            const bool empty = lmin > lmax;   // no row of the tile keeps this input
            bw = empty ? 0.f : fmaxf(lmax - lmin, umax - umin);
            // empty: w - max l = -inf and min u - w = -inf (no lower bound); w - min l = -inf and max u - w = -inf (no candidate)
            if (empty) { lmin = lmax = __builtin_inff(); umin = umax = -__builtin_inff(); }
            float* o = xr + (size_t)s * 4 * N + n;
            o[0] = lmin; o[N] = lmax; o[2 * (size_t)N] = umin; o[3 * (size_t)N] = umax;
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
    for (int e = tid; e < 64 * kTileB; e += 256) {
        const int nn = e >> 7, col = e & (kTileB - 1);
        if (n0 + nn < N) {
            const size_t o = (size_t)(n0 + nn) * Bp + s * kTileB + col;
            if (IV) reinterpret_cast<float2*>(xT)[o] = make_float2(tl[nn][col], tu[nn][col]);
            else xT[o] = tl[nn][col];
        }
    }
}

// The batch rows of a tile differ by more than kProbeRatio times what 16 entries of a weight column do (images
// against small weights): the table would mark nearly every input, so it is not built and reported as full.
constexpr float kProbeRatio = 2.5f;
__device__ __forceinline__ bool table_pointless(const float* stat, int S) {
    return stat[0] > kProbeRatio * (float)S * stat[1];
}

// The two table kernels share their tiling: a workgroup takes 64 weight rows (one per lane) and a slice of the
// inputs; wavefront v works on batch tile v (+ 4, + 8, ...), for which the column ranges are wave-uniform (LDS
// broadcasts); the weights go through LDS, 64 x 32 at a time, so that a lane can own a row.
// Lower bounds.  The smallest a term can be over the rows of the tile bounds it from below in every row (fp32
// subtraction is monotone, so this holds for the rounded terms), and K chunks of inputs whose largest such bound is
// at least t hold K terms that are at least t in every row: the kernel keeps the K largest chunk maxima of the slice
// (one insertion per 32 inputs), whose K-th largest over all slices bounds the K-th largest term.
// WMASK: wkeep holds one word per (weight row, 32 inputs); an input a weight row does not keep has no term.
template <int K, bool IV, bool WMASK>
__global__ void __launch_bounds__(256) sc_low_kernel(const float* __restrict__ w, const float* __restrict__ xr,
                                                     const uint32_t* __restrict__ wkeep, int M, int N, int S, int Mp,
                                                     float* __restrict__ lists, const float* __restrict__ stat) {
    if (table_pointless(stat, S)) return;
    __shared__ __attribute__((aligned(16))) float wt[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float xs[4][4][kChunk];
    const int tid = threadIdx.x, r = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = blockIdx.x * 64, NCH = N / kChunk;
    const int slices = gridDim.y, slice = blockIdx.y;
    const int per = (NCH + slices - 1) / slices;
    const int c_lo = slice * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;
    const int lrow = tid >> 2, q = tid & 3;
    const int mload = m0 + lrow < M ? m0 + lrow : M - 1;
    const int xt = tid >> 6, xk = (tid >> 4) & 3, xn = 2 * (tid & 15);
    for (int sb = 0; sb < S; sb += 4) {
        const int s = sb + wave;
        const bool active = s < S;
        int hi[K], lo[IV ? K : 1];
        #pragma unroll
        for (int k = 0; k < K; k++) { hi[k] = 0; if constexpr (IV) lo[k] = 0; }
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
            *reinterpret_cast<float4*>(&wt[lrow][8 * q]) = pa;
            *reinterpret_cast<float4*>(&wt[lrow][8 * q + 4]) = pb;
            *reinterpret_cast<float2*>(&xs[xt][xk][xn]) = px;
            fetch(c + 1);
            __syncthreads();
            if (active) {
                // largest lower bound of the chunk: fmaxf drops undefined differences (an undefined weight: the term
                // is undefined in every row), and the lists start at 0
                float cu = 0.f, cl = 0.f;
                uint32_t kw = ~0u;
                if constexpr (WMASK) kw = wkeep[(size_t)(m0 + r < M ? m0 + r : M - 1) * NCH + c];
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
                        if constexpr (WMASK) {
                            const float a = fmaxf(wv[k] - lmax[k], umin[k] - wv[k]);
                            cu = fmaxf(cu, ((kw >> (n4 + k)) & 1u) ? a : 0.f);
                        } else cu = fmaxf(fmaxf(cu, wv[k] - lmax[k]), umin[k] - wv[k]);
                        if constexpr (IV) cl = fmaxf(fmaxf(cl, lmin[k] - wv[k]), wv[k] - umax[k]);
                    }
                }
                insert_bits<K>(hi, cu);
                if constexpr (IV) insert_bits<K>(lo, cl);
            }
            __syncthreads();
        }
        if (active) {
            float* dst = lists + (((size_t)s * slices + slice) * 2) * K * Mp + m0 + r;
            #pragma unroll
            for (int k = 0; k < K; k++) {
                dst[(size_t)k * Mp] = __builtin_bit_cast(float, hi[k]);
                if constexpr (IV) dst[(size_t)(K + k) * Mp] = __builtin_bit_cast(float, lo[k]);
            }
        }
    }
}

// K-th largest of the slices' lists (0 when fewer than K lower bounds are positive)
template <int K>
__global__ void __launch_bounds__(256) sc_merge_kernel(const float* __restrict__ lists, int slices, int Mp, int nw,
                                                       float* __restrict__ low, const float* __restrict__ stat) {
    if (table_pointless(stat, gridDim.y / nw)) return;
    const int m = blockIdx.x * 256 + threadIdx.x;
    if (m >= Mp) return;
    const int s = blockIdx.y / nw, which = blockIdx.y % nw;
    int res[K];
    #pragma unroll
    for (int k = 0; k < K; k++) res[k] = 0;
    for (int slice = 0; slice < slices; slice++) {
        const float* src = lists + ((((size_t)s * slices + slice) * 2 + which) * K) * Mp + m;
        #pragma unroll
        for (int k = 0; k < K; k++) insert_bits<K>(res, src[(size_t)k * Mp]);
    }
    low[((size_t)s * 2 + which) * Mp + m] = __builtin_bit_cast(float, res[0]);
}

// One table word per (tile, weight row, chunk): bit n set when the largest the term of input n can be over the rows
// of the tile reaches the bound of its list and is positive (the lists start at 0 and take larger values only).
// The words of a wavefront's 64 rows are gathered in LDS and leave row by row, so that the main kernel finds the
// words of a weight row side by side.  The marks are counted per wavefront.
template <bool IV, bool WMASK>
__global__ void __launch_bounds__(256) sc_bits_kernel(const float* __restrict__ w, const float* __restrict__ xr,
                                                      const float* __restrict__ low,
                                                      const uint32_t* __restrict__ wkeep, int M, int N, int S, int Mp,
                                                      uint32_t* __restrict__ bits, uint32_t* __restrict__ partial,
                                                      const float* __restrict__ stat) {
    if (table_pointless(stat, S)) return;
    __shared__ __attribute__((aligned(16))) float wt[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float xs[4][4][kChunk];
    __shared__ uint32_t wd[4][64][kMaxPer + 1];
    const int tid = threadIdx.x, r = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = blockIdx.x * 64, NCH = N / kChunk;
    const int slices = gridDim.y, slice = blockIdx.y;
    const int per = (NCH + slices - 1) / slices;   // at most kMaxPer (slices_of)
    const int c_lo = slice * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;
    const int lrow = tid >> 2, q = tid & 3;
    const int mload = m0 + lrow < M ? m0 + lrow : M - 1;
    const bool valid = m0 + r < M;
    const int xt = tid >> 6, xk = (tid >> 4) & 3, xn = 2 * (tid & 15);
    int marks = 0;
    for (int sb = 0; sb < S; sb += 4) {
        const int s = sb + wave;
        const bool active = s < S;
        float LU = 0.f, LL = 0.f;
        if (active) {
            LU = low[(size_t)(s * 2) * Mp + m0 + r];
            if (IV) LL = low[(size_t)(s * 2 + 1) * Mp + m0 + r];
        }
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
            *reinterpret_cast<float4*>(&wt[lrow][8 * q]) = pa;
            *reinterpret_cast<float4*>(&wt[lrow][8 * q + 4]) = pb;
            *reinterpret_cast<float2*>(&xs[xt][xk][xn]) = px;
            fetch(c + 1);
            __syncthreads();
            if (active) {
                uint32_t word = 0;
                #pragma unroll
                for (int n4 = 0; n4 < kChunk; n4 += 4) {
                    const float4 wv4 = *reinterpret_cast<const float4*>(&wt[r][n4]);
                    const float4 a4 = *reinterpret_cast<const float4*>(&xs[wave][0][n4]);
                    const float4 b4 = *reinterpret_cast<const float4*>(&xs[wave][1][n4]);
                    const float4 c4 = *reinterpret_cast<const float4*>(&xs[wave][2][n4]);
                    const float4 d4 = *reinterpret_cast<const float4*>(&xs[wave][3][n4]);
                    const float wv[4] = {wv4.x, wv4.y, wv4.z, wv4.w};
                    const float lmin[4] = {a4.x, a4.y, a4.z, a4.w}, lmax[4] = {b4.x, b4.y, b4.z, b4.w};
                    const float umin[4] = {c4.x, c4.y, c4.z, c4.w}, umax[4] = {d4.x, d4.y, d4.z, d4.w};
                    #pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const float capU = fmaxf(wv[k] - lmin[k], umax[k] - wv[k]);
                        bool mark = capU >= LU && capU > 0.f;
                        if (IV) {
                            const float capL = fmaxf(lmax[k] - wv[k], wv[k] - umin[k]);
                            mark = mark || (capL >= LL && capL > 0.f);
                        }
                        word |= (uint32_t)mark << (n4 + k);
                    }
                }
                if (!valid) word = 0u;
                if constexpr (WMASK) word &= wkeep[(size_t)(m0 + r < M ? m0 + r : M - 1) * NCH + c];
                wd[wave][r][c - c_lo] = word;
                marks += __builtin_popcount(word);
            }
            __syncthreads();
        }
        if (active) {
            // the wavefront's own words: row by row, the chunks of the slice side by side
            for (int row = 0; row < 64; row++)
                if (r < c_hi - c_lo) bits[((size_t)s * Mp + m0 + row) * NCH + c_lo + r] = wd[wave][row][r];
        }
    }
    #pragma unroll
    for (int o = 32; o; o >>= 1) marks += __shfl_xor(marks, o);
    if (r == 0) partial[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 4 + wave] = (uint32_t)marks;
}

// count[0] = marks (a table that was not built counts as full), count[1] = 1 when that is above the limit
__global__ void __launch_bounds__(1024) sc_sum_kernel(const uint32_t* __restrict__ partial, size_t n,
                                                      unsigned long long* __restrict__ count,
                                                      const float* __restrict__ stat, int S, unsigned long long limit) {
    if (table_pointless(stat, S)) { if (threadIdx.x == 0) { count[0] = ~0ull; count[1] = 1ull; } return; }
    __shared__ unsigned long long acc[1024];
    unsigned long long s0 = 0;
    for (size_t i = threadIdx.x; i < n; i += 1024) s0 += partial[i];
    acc[threadIdx.x] = s0;
    __syncthreads();
    for (int o = 512; o; o >>= 1) {
        if ((int)threadIdx.x < o) acc[threadIdx.x] += acc[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) { count[0] = acc[0]; count[1] = acc[0] > limit ? 1ull : 0ull; }
}

// ---- main kernel -------------------------------------------------------------------------------
// A workgroup takes 32 weight rows and one batch tile; each of its wavefronts takes four of the rows, one after the
// other, with lane l holding the batch rows l and l + 64 of the tile.  For a row the wavefront reads the row's
// table words 64 chunks at a time, lists the marked inputs in LDS and walks the list four marks at a time (the
// loads of the next four in flight): per mark one weight (a wave-uniform load), one transposed row of inputs (two
// coalesced loads) and the insertions into the top-K lists, which are the single-pass kernel's (branch-free medians; same terms, same lists).  The
// results of the workgroup leave through LDS, 128 bytes wide.
// MAXFORM (K = 1, interval form): the lists are the running maxima of the interval bounds of the l-inf distance
// (core/cuda/bound_inf_dist_cuda.cu:15-118), which leave as max(1e-10, .) instead of through the geometric sum.
template <int K, bool IV, bool MAXFORM = false>
__global__ void __launch_bounds__(64 * kMainWaves)
sc_main_kernel(const float* __restrict__ xT, const float* __restrict__ w, const uint32_t* __restrict__ bits,
               const unsigned long long* __restrict__ count, unsigned long long limit, int B, int Bp, int M, int Mp,
               int N, float q, float* __restrict__ yL, float* __restrict__ yU) {
    if (gate_closed(count, limit, 0)) return;
    __shared__ uint16_t list[kMainWaves][kListCap];
    __shared__ float stage[IV ? 2 : 1][kTileB][kMainTile + 1];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int MB = Mp / kMainTile, NCH = N / kChunk;
    // Workgroups go to the chip's eight dies in turn, each with a cache of its own: consecutive (tile, rows) pairs
    // are dealt out so that a die sees few batch tiles, whose transposed inputs (1 KiB per marked input) it re-reads
    int item = blockIdx.x;
    if (gridDim.x % 8 == 0) item = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int mb = item % MB, s = item / MB;
    using X = typename std::conditional<IV, float2, float>::type;
    const X* __restrict__ xcol = reinterpret_cast<const X*>(xT) + (size_t)s * kTileB + lane;
    uint16_t* mine = list[wave];

    for (int rr = 0; rr < kMainRows; rr++) {
        const int ml = wave * kMainRows + rr, m = mb * kMainTile + ml;
        if (m >= M) break;   // wave-uniform; the rows of a wavefront ascend
        int hi[2][K], lo[IV ? 2 : 1][IV ? K : 1];
        #pragma unroll
        for (int k = 0; k < K; k++) {
            hi[0][k] = hi[1][k] = 0;
            if constexpr (IV) lo[0][k] = lo[1][k] = 0;
        }
        const uint32_t* __restrict__ rowbits = bits + ((size_t)s * Mp + m) * NCH;
        const float* __restrict__ wrow = w + (size_t)m * N;
        // One group of four marks: lane l fetches the number and the weight of mark l % 4 (read back lane by lane,
        // so the weight is a scalar operand of the terms), every lane its two entries of the four transposed input
        // rows.  Groups past the end of the list repeat its last mark and are not used: every load is issued
        // unconditionally, so that the waits the compiler places cover exactly the group that is used next.
        int cnt = 0;   // marks in the list
        float wreg[2];
        X xa[2][4], xb[2][4];
        auto load = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            int k = k0 + (lane & 3);
            k = k < total ? k : total - 1;
            const int nn = (int)mine[k];
            wreg[buf] = wrow[nn];
            #pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = __builtin_amdgcn_readlane(nn, i);
                xa[buf][i] = xcol[(size_t)n * Bp];
                xb[buf][i] = xcol[(size_t)n * Bp + 64];
            }
        };
        auto compute = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            #pragma unroll
            for (int i = 0; i < 4; i++) {
                if (k0 + i < total) {   // wave-uniform
                    const float wi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wreg[buf]), i));
                    if constexpr (IV && MAXFORM) {
                        // a term with an undefined operand is dropped (min / max keep the defined one, as the
                        // reference's do; the final max with 0 drops a term that is undefined altogether)
                        const float a1 = wi - xa[buf][i].x, a2 = xa[buf][i].y - wi;
                        const float b1 = wi - xb[buf][i].x, b2 = xb[buf][i].y - wi;
                        insert_bits<K>(lo[0], fmaxf(-fminf(a1, a2), 0.f));
                        insert_bits<K>(hi[0], fmaxf(fmaxf(a1, a2), 0.f));
                        insert_bits<K>(lo[1], fmaxf(-fminf(b1, b2), 0.f));
                        insert_bits<K>(hi[1], fmaxf(fmaxf(b1, b2), 0.f));
                    } else if constexpr (IV) {
                        const float a1 = wi - xa[buf][i].x, a2 = xa[buf][i].y - wi;
                        const float b1 = wi - xb[buf][i].x, b2 = xb[buf][i].y - wi;
                        // (the maximum with -1 turns a term that is undefined altogether, whose bit pattern would
                        // order above every number, into a negative one, which the lists ignore; three-operand
                        // maxima, so it costs no instruction)
                        insert_bits<K>(lo[0], fmaxf(fmaxf(-a1, -a2), -1.f));
                        insert_bits<K>(hi[0], fmaxf(fmaxf(a1, a2), -1.f));
                        insert_bits<K>(lo[1], fmaxf(fmaxf(-b1, -b2), -1.f));
                        insert_bits<K>(hi[1], fmaxf(fmaxf(b1, b2), -1.f));
                    } else {
                        // (the same for the value form: the maximum stands where the absolute value's own
                        // instruction stood)
                        insert_bits<K>(hi[0], fmaxf(fabsf(xa[buf][i] - wi), -1.f));
                        insert_bits<K>(hi[1], fmaxf(fabsf(xb[buf][i] - wi), -1.f));
                    }
                }
            }
        };
        // walks the list, the loads of a group in flight while the group before it is used
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
        for (int c0 = 0; c0 < NCH; c0 += kBatch) {
            uint32_t word = next;
            if (c0 + kBatch < NCH) next = c0 + kBatch + lane < NCH ? rowbits[c0 + kBatch + lane] : 0u;
            // every lane appends the marks of its word behind those of the lanes before it
            const int mine_n = __builtin_popcount(word);
            int incl = mine_n;
            #pragma unroll
            for (int o = 1; o < kBatch; o <<= 1) {
                const int t = __shfl_up(incl, o);
                if (lane >= o) incl += t;
            }
            int off = cnt + incl - mine_n;
            cnt += __builtin_amdgcn_readlane(incl, kBatch - 1);
            while (word) {
                const int i = __builtin_ctz(word);
                word &= word - 1;
                mine[off++] = (uint16_t)(((c0 + lane) << 5) | i);   // the input's number (CI <= 65536)
            }
            // a row's marks are walked in one go unless the list could overflow with the next chunks
            if (cnt > kListCap - kBatch * kChunk || c0 + kBatch >= NCH) {
                __builtin_amdgcn_wave_barrier();
                walk(cnt);
                cnt = 0;
                __builtin_amdgcn_wave_barrier();   // the reads of the list come before the next marks
            }
        }
        #pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (MAXFORM) {
                static_assert(!MAXFORM || (K == 1 && IV), "the maximum form is the interval form with one entry");
                stage[0][lane + 64 * j][ml] = fmaxf(__builtin_bit_cast(float, hi[j][0]), kEps);
                stage[1][lane + 64 * j][ml] = fmaxf(__builtin_bit_cast(float, lo[j][0]), kEps);
            } else {
                stage[0][lane + 64 * j][ml] = geo_sum_bits<K>(hi[j], q);
                if constexpr (IV) stage[1][lane + 64 * j][ml] = geo_sum_bits<K>(lo[j], q);
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < kTileB * kMainTile; e += 64 * kMainWaves) {
        const int bl = e / kMainTile, mloc = e % kMainTile;
        const int b = s * kTileB + bl, m = mb * kMainTile + mloc;
        if (b < B && m < M) {
            yU[(size_t)b * M + m] = stage[0][bl][mloc];
            if constexpr (IV) yL[(size_t)b * M + m] = stage[1][bl][mloc];
        }
    }
}

// l-inf distance (maximum and where it sits) from the same tables, value form, optionally under the factored mask.
// As sc_main_kernel, with the running maximum and its position (input number, bit 31 = the difference is negative;
// the marks are walked in ascending input order and only a larger term replaces the maximum, so the first of
// equal terms wins as in core/cuda/inf_dist_cuda.cu:176-190) instead of the top-K lists.  `low` holds the bound the
// marks were taken against: every unmarked input's term is below it in every row, so a maximum that reaches it is
// the maximum over all inputs.  Under the mask a row may keep none of the inputs the bound rests on; if any row of
// the wavefront ends below the bound, the wavefront walks the weight row again over every input it keeps (`wkeep`
// words; all inputs without a mask), which costs that wavefront what the every-term kernel costs it.
template <bool POS>
__global__ void __launch_bounds__(64 * kMainWaves)
mc_main_kernel(const float* __restrict__ xT, const float* __restrict__ w, const uint32_t* __restrict__ bits,
               const uint32_t* __restrict__ wkeep, const float* __restrict__ low,
               const unsigned long long* __restrict__ count, unsigned long long limit, int B, int Bp, int M, int Mp,
               int N, float* __restrict__ y, int* __restrict__ pos) {
    if (gate_closed(count, limit, 0)) return;
    __shared__ uint16_t list[kMainWaves][kListCap];
    __shared__ float stage_y[kTileB][kMainTile + 1];
    __shared__ int stage_p[POS ? kTileB : 1][kMainTile + 1];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int MB = Mp / kMainTile, NCH = N / kChunk;
    int item = blockIdx.x;
    if (gridDim.x % 8 == 0) item = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int mb = item % MB, s = item / MB;
    const float* __restrict__ xcol = xT + (size_t)s * kTileB + lane;
    uint16_t* mine = list[wave];
    const int m = mb * kMainTile + wave;
    if (m < M) {   // wave-uniform
        const float* __restrict__ wrow = w + (size_t)m * N;
        // per batch row of the lane: the difference of largest magnitude so far (its sign is the position's flag)
        // and the input it sits at; without positions only the magnitude
        float best[2];
        int where[2];
        float wreg[2];
        int nreg[2];
        float xa[2][4], xb[2][4];
        auto load = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            int k = k0 + (lane & 3);
            k = k < total ? k : total - 1;
            const int nn = (int)mine[k];
            nreg[buf] = nn;
            wreg[buf] = wrow[nn];
            #pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = __builtin_amdgcn_readlane(nn, i);
                xa[buf][i] = xcol[(size_t)n * Bp];
                xb[buf][i] = xcol[(size_t)n * Bp + 64];
            }
        };
        auto compute = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            #pragma unroll
            for (int i = 0; i < 4; i++) {
                if (k0 + i < total) {   // wave-uniform
                    const float wi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wreg[buf]), i));
                    const int n = __builtin_amdgcn_readlane(nreg[buf], i);
                    const float d0 = xa[buf][i] - wi, d1 = xb[buf][i] - wi;
                    // an undefined difference (an input the row does not keep) never compares greater
                    if constexpr (POS) {
                        const bool g0 = fabsf(d0) > fabsf(best[0]), g1 = fabsf(d1) > fabsf(best[1]);
                        best[0] = g0 ? d0 : best[0]; where[0] = g0 ? n : where[0];
                        best[1] = g1 ? d1 : best[1]; where[1] = g1 ? n : where[1];
                    } else {
                        best[0] = fmaxf(best[0], fabsf(d0));
                        best[1] = fmaxf(best[1], fabsf(d1));
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
        // one pass over the weight row: `words` = its table words, or (second pass) the inputs it keeps
        auto pass = [&](const uint32_t* __restrict__ words) __attribute__((always_inline)) {
            best[0] = best[1] = kEps;
            where[0] = where[1] = 0;
            int cnt = 0;
            uint32_t next = lane < NCH ? (words ? words[lane] : ~0u) : 0u;
            for (int c0 = 0; c0 < NCH; c0 += kBatch) {
                uint32_t word = next;
                if (c0 + kBatch < NCH) next = c0 + kBatch + lane < NCH ? (words ? words[c0 + kBatch + lane] : ~0u) : 0u;
                const int mine_n = __builtin_popcount(word);
                int incl = mine_n;
                #pragma unroll
                for (int o = 1; o < kBatch; o <<= 1) {
                    const int t = __shfl_up(incl, o);
                    if (lane >= o) incl += t;
                }
                int off = cnt + incl - mine_n;
                cnt += __builtin_amdgcn_readlane(incl, kBatch - 1);
                while (word) {
                    const int i = __builtin_ctz(word);
                    word &= word - 1;
                    mine[off++] = (uint16_t)(((c0 + lane) << 5) | i);
                }
                if (cnt > kListCap - kBatch * kChunk || c0 + kBatch >= NCH) {
                    __builtin_amdgcn_wave_barrier();
                    walk(cnt);
                    cnt = 0;
                    __builtin_amdgcn_wave_barrier();
                }
            }
        };
        pass(bits + ((size_t)s * Mp + m) * NCH);
        const float bound = low[(size_t)(s * 2) * Mp + m];
        const int b0 = s * kTileB + lane;
        const bool short0 = b0 < B && fabsf(best[0]) < bound, short1 = b0 + 64 < B && fabsf(best[1]) < bound;
        if (__builtin_amdgcn_ballot_w64(short0 || short1) != 0ull) pass(wkeep ? wkeep + (size_t)m * NCH : nullptr);
        #pragma unroll
        for (int j = 0; j < 2; j++) {
            stage_y[lane + 64 * j][wave] = fabsf(best[j]);
            if (POS) stage_p[lane + 64 * j][wave] = where[j] | (best[j] >= 0.f ? 0 : (int)kSign);
        }
    }
    __syncthreads();
    for (int e = tid; e < kTileB * kMainTile; e += 64 * kMainWaves) {
        const int bl = e / kMainTile, mloc = e % kMainTile;
        const int b = s * kTileB + bl, mm = mb * kMainTile + mloc;
        if (b < B && mm < M) {
            y[(size_t)b * M + mm] = stage_y[bl][mloc];
            if (POS) pos[(size_t)b * M + mm] = stage_p[bl][mloc];
        }
    }
}

template <int K, bool WMASK>
int run_max(const float* x, const float* w, const uint32_t* xkeep, const uint32_t* wkeep, int B, int M, int N, float* y,
            int* pos, const Carve& c, unsigned long long limit, hipStream_t st) {
    const int S = tiles_b(B), Bp = S * kTileB, Mp = mpad_of(M), NCH = N / kChunk, slices = slices_of(NCH);
    int rc;
    if ((rc = fill_zero(c.count, 8, st))) return rc;   // the count, its flag and the two sums of the probe behind them
    if (WMASK) hipLaunchKernelGGL((sc_range_kernel<false, true>), dim3((N + 63) / 64, S), dim3(256), 0, st, x, nullptr, w, xkeep, B, M, N, Bp, c.xr, c.xT, c.stat);
    else hipLaunchKernelGGL((sc_range_kernel<false, false>), dim3((N + 63) / 64, S), dim3(256), 0, st, x, nullptr, w, nullptr, B, M, N, Bp, c.xr, c.xT, c.stat);
    if ((rc = check_launch("sc_range_kernel"))) return rc;
    hipLaunchKernelGGL((sc_low_kernel<K, false, WMASK>), dim3(Mp / 64, slices), dim3(256), 0, st, w, c.xr, wkeep, M, N, S, Mp, c.lists, c.stat);
    if ((rc = check_launch("sc_low_kernel"))) return rc;
    hipLaunchKernelGGL((sc_merge_kernel<K>), dim3((Mp + 255) / 256, S), dim3(256), 0, st, c.lists, slices, Mp, 1, c.low, c.stat);
    if ((rc = check_launch("sc_merge_kernel"))) return rc;
    hipLaunchKernelGGL((sc_bits_kernel<false, WMASK>), dim3(Mp / 64, slices), dim3(256), 0, st, w, c.xr, c.low, wkeep, M, N, S, Mp, c.bits, c.partial, c.stat);
    if ((rc = check_launch("sc_bits_kernel"))) return rc;
    hipLaunchKernelGGL(sc_sum_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)(Mp / 64) * slices * 4, c.count, c.stat, S, limit);
    if ((rc = check_launch("sc_sum_kernel"))) return rc;
    const dim3 grid((unsigned)(S * (Mp / kMainTile)));
    if (pos) hipLaunchKernelGGL((mc_main_kernel<true>), grid, dim3(64 * kMainWaves), 0, st, c.xT, w, c.bits, wkeep, c.low, c.count, limit, B, Bp, M, Mp, N, y, pos);
    else hipLaunchKernelGGL((mc_main_kernel<false>), grid, dim3(64 * kMainWaves), 0, st, c.xT, w, c.bits, wkeep, c.low, c.count, limit, B, Bp, M, Mp, N, y, pos);
    return check_launch("mc_main_kernel");
}

template <class F, int... R>
__device__ __forceinline__ void static_for(F&& f, std::integer_sequence<int, R...>) {
    (f(std::integral_constant<int, R>{}), ...);
}

// Value form with positions (core/cuda/sort_neuron.cu:111-214): as sc_main_kernel, with the ordered insertion that
// carries the input numbers.  The marks of a row are walked in ascending input order, and every term that is at
// least the final K-th largest value of an output is marked, so these terms meet the list in the order and against
// the entries they meet in the scan over all inputs: same values and same positions, ties included.  pos is
// (K, B, M) with slot 0 = largest; the K planes leave through LDS one after the other.
template <int K>
__global__ void __launch_bounds__(64 * kMainWaves)
sp_main_kernel(const float* __restrict__ xT, const float* __restrict__ w, const uint32_t* __restrict__ bits,
               const unsigned long long* __restrict__ count, unsigned long long limit, int B, int Bp, int M, int Mp,
               int N, float q, float* __restrict__ y, int* __restrict__ pos) {
    if (gate_closed(count, limit, 0)) return;
    __shared__ uint16_t list[kMainWaves][kListCap];
    __shared__ int stage[kTileB][kMainTile + 1];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int MB = Mp / kMainTile, NCH = N / kChunk;
    int item = blockIdx.x;
    if (gridDim.x % 8 == 0) item = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int mb = item % MB, s = item / MB;
    const float* __restrict__ xcol = xT + (size_t)s * kTileB + lane;
    uint16_t* mine = list[wave];
    const int m = mb * kMainTile + wave;
    float res[2][K];
    int idx[2][K];
    #pragma unroll
    for (int k = 0; k < K; k++) { res[0][k] = res[1][k] = 0.f; idx[0][k] = idx[1][k] = 0; }
    if (m < M) {   // wave-uniform
        const float* __restrict__ wrow = w + (size_t)m * N;
        const uint32_t* __restrict__ rowbits = bits + ((size_t)s * Mp + m) * NCH;
        float wreg[2];
        int nreg[2];
        float xa[2][4], xb[2][4];
        auto load = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            int k = k0 + (lane & 3);
            k = k < total ? k : total - 1;
            const int nn = (int)mine[k];
            nreg[buf] = nn;
            wreg[buf] = wrow[nn];
            #pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = __builtin_amdgcn_readlane(nn, i);
                xa[buf][i] = xcol[(size_t)n * Bp];
                xb[buf][i] = xcol[(size_t)n * Bp + 64];
            }
        };
        auto compute = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            #pragma unroll
            for (int i = 0; i < 4; i++) {
                if (k0 + i < total) {   // wave-uniform
                    const float wi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wreg[buf]), i));
                    const int n = __builtin_amdgcn_readlane(nreg[buf], i);
                    const float d0 = xa[buf][i] - wi, d1 = xb[buf][i] - wi;
                    if (fabsf(d0) > res[0][0]) topk_insert<K>(res[0], idx[0], fabsf(d0), n | (d0 >= 0.f ? 0 : (int)kSign));
                    if (fabsf(d1) > res[1][0]) topk_insert<K>(res[1], idx[1], fabsf(d1), n | (d1 >= 0.f ? 0 : (int)kSign));
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
        int cnt = 0;
        uint32_t next = lane < NCH ? rowbits[lane] : 0u;
        for (int c0 = 0; c0 < NCH; c0 += kBatch) {
            uint32_t word = next;
            if (c0 + kBatch < NCH) next = c0 + kBatch + lane < NCH ? rowbits[c0 + kBatch + lane] : 0u;
            const int mine_n = __builtin_popcount(word);
            int incl = mine_n;
            #pragma unroll
            for (int o = 1; o < kBatch; o <<= 1) {
                const int t = __shfl_up(incl, o);
                if (lane >= o) incl += t;
            }
            int off = cnt + incl - mine_n;
            cnt += __builtin_amdgcn_readlane(incl, kBatch - 1);
            while (word) {
                const int i = __builtin_ctz(word);
                word &= word - 1;
                mine[off++] = (uint16_t)(((c0 + lane) << 5) | i);
            }
            if (cnt > kListCap - kBatch * kChunk || c0 + kBatch >= NCH) {
                __builtin_amdgcn_wave_barrier();
                walk(cnt);
                cnt = 0;
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
    const size_t plane = (size_t)B * M;
    // the values, then the K planes of positions (slot 0 = largest = res[K-1]); the rounds are expanded at compile
    // time so that the lists are only ever indexed with constants and stay in registers
    static_for([&](auto R) __attribute__((always_inline)) {
        constexpr int round = decltype(R)::value;
        if (m < M) {
            #pragma unroll
            for (int j = 0; j < 2; j++) {
                if constexpr (round == 0) stage[lane + 64 * j][wave] = __builtin_bit_cast(int, geo_sum<K>(res[j], q));
                else stage[lane + 64 * j][wave] = idx[j][K - round];
            }
        }
        __syncthreads();
        for (int e = tid; e < kTileB * kMainTile; e += 64 * kMainWaves) {
            const int bl = e / kMainTile, mloc = e % kMainTile;
            const int b = s * kTileB + bl, mm = mb * kMainTile + mloc;
            if (b < B && mm < M) {
                const size_t o = (size_t)b * M + mm;
                if constexpr (round == 0) y[o] = __builtin_bit_cast(float, stage[bl][mloc]);
                else pos[(size_t)(round - 1) * plane + o] = stage[bl][mloc];
            }
        }
        __syncthreads();
    }, std::make_integer_sequence<int, K + 1>{});
}

template <int K, bool IV, bool MAXFORM = false>
int run(const float* xl, const float* xu, const float* w, int B, int M, int N, float q, float* outL, float* outU,
        int* pos, const Carve& c, unsigned long long limit, hipStream_t st) {
    const int S = tiles_b(B), Bp = S * kTileB, Mp = mpad_of(M), NCH = N / kChunk, slices = slices_of(NCH);
    int rc;
    if ((rc = fill_zero(c.count, 8, st))) return rc;   // the count and the two sums of the probe behind it
    hipLaunchKernelGGL((sc_range_kernel<IV, false>), dim3((N + 63) / 64, S), dim3(256), 0, st, xl, xu, w, nullptr, B, M, N, Bp, c.xr, c.xT, c.stat);
    if ((rc = check_launch("sc_range_kernel"))) return rc;
    hipLaunchKernelGGL((sc_low_kernel<K, IV, false>), dim3(Mp / 64, slices), dim3(256), 0, st, w, c.xr, nullptr, M, N, S, Mp, c.lists, c.stat);
    if ((rc = check_launch("sc_low_kernel"))) return rc;
    const int nw = IV ? 2 : 1;
    hipLaunchKernelGGL((sc_merge_kernel<K>), dim3((Mp + 255) / 256, S * nw), dim3(256), 0, st, c.lists, slices, Mp, nw, c.low, c.stat);
    if ((rc = check_launch("sc_merge_kernel"))) return rc;
    hipLaunchKernelGGL((sc_bits_kernel<IV, false>), dim3(Mp / 64, slices), dim3(256), 0, st, w, c.xr, c.low, nullptr, M, N, S, Mp, c.bits, c.partial, c.stat);
    if ((rc = check_launch("sc_bits_kernel"))) return rc;
    hipLaunchKernelGGL(sc_sum_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)(Mp / 64) * slices * 4, c.count, c.stat, S, limit);
    if ((rc = check_launch("sc_sum_kernel"))) return rc;
    if constexpr (!IV) {
        if (pos) {
            hipLaunchKernelGGL((sp_main_kernel<K>), dim3((unsigned)(S * (Mp / kMainTile))), dim3(64 * kMainWaves), 0, st,
                               c.xT, w, c.bits, c.count, limit, B, Bp, M, Mp, N, q, outU, pos);
            return check_launch("sp_main_kernel");
        }
    }
    hipLaunchKernelGGL((sc_main_kernel<K, IV, MAXFORM>), dim3((unsigned)(S * (Mp / kMainTile))), dim3(64 * kMainWaves), 0, st,
                       c.xT, w, c.bits, c.count, limit, B, Bp, M, Mp, N, q, outL, outU);
    return check_launch("sc_main_kernel");
}

}  // namespace

size_t sort_cols_workspace(int B, int CO, int CI, int K) {
    size_t sz[7];
    return carve_sizes(B, CO, CI, K, sz);
}

#define SD_SORT_COLS_K(X) \
    X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16) X(17) \
    X(18) X(19) X(20) X(21) X(22) X(23) X(24) X(25)

int sort_cols_forward(const float* xl, const float* xu, const float* w, int B, int CO, int CI, float q, int K,
                      float* outL, float* outU, int* pos, void* ws, float density, const unsigned long long** gate,
                      unsigned long long* gate_limit, hipStream_t st) {
    if (CI % kChunk != 0 || CI > 65536 || B < 1 || CO < 1) {
        set_error("sort_cols_forward: shape not supported");
        return SD_ERR_ARG;
    }
    const Carve c = carve(ws, B, CO, CI, K);
    const float d = density < 0.f ? 0.f : density > 1.f ? 1.f : density;
    const unsigned long long limit = (unsigned long long)((double)tiles_b(B) * CO * CI * d);
    *gate = c.count;
    *gate_limit = limit;
    note_term_counts(c.count, 1, (double)tiles_b(B) * CO * CI, 1.0, 0ull);
    if (K == 1 && xu) return run<1, true, true>(xl, xu, w, B, CO, CI, q, outL, outU, nullptr, c, limit, st);
    switch (K) {
#define X(k) case k: return xu ? run<k, true>(xl, xu, w, B, CO, CI, q, outL, outU, nullptr, c, limit, st) \
                               : run<k, false>(xl, nullptr, w, B, CO, CI, q, outL, outU, pos, c, limit, st);
        SD_SORT_COLS_K(X)
#undef X
    }
    set_error("sort_cols_forward: K=%d outside 2..25", K);
    return SD_ERR_ARG;
}


int max_cols_depth(float keep_x) {
    if (keep_x >= 1.f) return 1;
    // inputs the bound rests on such that a row keeps none of them less often than once in 10^4 outputs (such an
    // output costs its wavefront a second pass over every input; more inputs lower the bound and mark more)
    const int need = (int)ceilf(logf(1e-4f) / logf(1.f - keep_x));
    for (int k : {8, 12, 16, 20, 24}) if (need <= k) return k;
    return 0;
}

size_t max_cols_workspace(int B, int CO, int CI, int K) { return sort_cols_workspace(B, CO, CI, K); }

int max_cols_forward(const float* x, const float* w, const uint32_t* xkeep, const uint32_t* wkeep, int B, int CO, int CI,
                     int K, float* y, int* pos, void* ws, float density, const unsigned long long** gate,
                     unsigned long long* gate_limit, hipStream_t st) {
    if (CI % kChunk != 0 || CI > 65536 || B < 1 || CO < 1 || (xkeep == nullptr) != (wkeep == nullptr)) {
        set_error("max_cols_forward: shape not supported");
        return SD_ERR_ARG;
    }
    const Carve c = carve(ws, B, CO, CI, K);
    const float d = density < 0.f ? 0.f : density > 1.f ? 1.f : density;
    const unsigned long long limit = (unsigned long long)((double)tiles_b(B) * CO * CI * d);
    *gate = c.count;
    *gate_limit = limit;
    note_term_counts(c.count, 1, (double)tiles_b(B) * CO * CI, 1.0, 0ull);
    if (!xkeep) {
        if (K == 1) return run_max<1, false>(x, w, nullptr, nullptr, B, CO, CI, y, pos, c, limit, st);
    } else switch (K) {
#define X(k) case k: return run_max<k, true>(x, w, xkeep, wkeep, B, CO, CI, y, pos, c, limit, st);
        X(8) X(12) X(16) X(20) X(24)
#undef X
    }
    set_error("max_cols_forward: depth %d not supported", K);
    return SD_ERR_ARG;
}

}  // namespace sd
