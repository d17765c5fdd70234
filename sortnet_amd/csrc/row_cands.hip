// Sort neuron, its interval bounds and the l-inf forward from candidate tables per batch row (see row_cands.h).
#include "row_cands.h"
#include <type_traits>
#include <utility>
#include "fwd_tile.h"

namespace sd {

namespace {

constexpr int kChunk = kRowCandsChunk;
constexpr int kTileW = 128;          // weight rows of a tile: 64 lanes x 2
constexpr int kBPad = 128;           // batch rows are padded to a multiple of this in the tables
constexpr int kMaxPer = 32;          // most chunks a slice of the table kernels covers
constexpr int kWaves = 16;           // wavefronts of a workgroup of the main kernel
constexpr int kSeg = 64;             // chunks whose table words the main kernel keeps in LDS at a time
constexpr int kWRow = 2 * 64 + 4;    // floats per input in the staged weight tile: 64 lanes x (w, w')

inline size_t align256(size_t b) { return (b + 255) / 256 * 256; }
inline int tiles_w(int M) { return (M + kTileW - 1) / kTileW; }
inline int bpad_of(int B) { return (B + kBPad - 1) / kBPad * kBPad; }
inline int slices_of(int NCH) {
    int s = (NCH + kMaxPer - 1) / kMaxPer;
    if (s < 16) s = 16;
    return s < NCH ? s : NCH;
}

// The value and interval forms of the sort neuron walk a transposed copy of the weights, wavefront by wavefront,
// without LDS tiles or barriers (rt_main_kernel); the forms with positions and the l-inf forms stage tiles
// (rc_main_kernel).
constexpr bool walks_transposed(int form) { return form == kRowsSortValues || form == kRowsSortInterval; }

struct Carve {
    float* wr;        // [T][2][N]  per tile of weight rows and input: min w, max w over the rows that keep the input
    float* lists;     // [T][slices][nw][K][Bp]  K largest chunk maxima of the lower bounds of a batch row's terms within a slice
    float* low;       // [T][nw][Bp]  K-th largest of them over all slices: upper list, lower list
    uint32_t* bits;   // [T][NCH][Bp] bit i of a word = input 32 c + i may be among the K largest of that batch row in that tile
    uint32_t* partial;            // marks per wavefront of the table kernel
    unsigned long long* count;    // [0] marks, [1] every-term kernels run, [2] this table's kernel runs, [3] marks per weight row (copy), [4] outputs to recompute
    uint32_t* fix;    // [B * M] outputs of the masked l-inf form whose bound did not hold (recomputed from every input)
    float* wt;        // [T][N][128] the weights of a tile, one 512-byte row per input (forms walked without LDS tiles)
};

size_t carve_sizes(int form, int B, int M, int N, int K, size_t (&sz)[8]) {
    const size_t T = tiles_w(M), Bp = bpad_of(B), NCH = N / kChunk, slices = slices_of((int)NCH);
    const size_t nw = form == kRowsSortInterval ? 2 : 1;
    sz[0] = align256(T * 2 * N * 4);
    sz[1] = align256(T * slices * nw * K * Bp * 4);
    sz[2] = align256(T * nw * Bp * 4);
    sz[3] = align256(T * NCH * Bp * 4);
    sz[4] = align256(Bp / 64 * slices * ((T + 3) / 4) * 4 * 4);
    sz[5] = 256;
    sz[6] = form == kRowsMax ? align256((size_t)B * M * 4) : 0;
    sz[7] = walks_transposed(form) ? align256(T * N * kTileW * 4) : 0;
    size_t t = 0;
    for (size_t v : sz) t += v;
    return t;
}

Carve carve(void* ws, int form, int B, int M, int N, int K) {
    size_t sz[8];
    carve_sizes(form, B, M, N, K, sz);
    char* p = static_cast<char*>(ws);
    Carve c;
    c.wr = reinterpret_cast<float*>(p); p += sz[0];
    c.lists = reinterpret_cast<float*>(p); p += sz[1];
    c.low = reinterpret_cast<float*>(p); p += sz[2];
    c.bits = reinterpret_cast<uint32_t*>(p); p += sz[3];
    c.partial = reinterpret_cast<uint32_t*>(p); p += sz[4];
    c.count = reinterpret_cast<unsigned long long*>(p); p += sz[5];
    c.fix = reinterpret_cast<uint32_t*>(p); p += sz[6];
    c.wt = reinterpret_cast<float*>(p);
    return c;
}

// inverted intervals become their midpoint (core/cuda/sort_neuron.cu:262)
__device__ __forceinline__ void repair(float& l, float& u) {
    if (l > u) l = u = (l + u) * 0.5f;
}

// The probe of sort_cols.hip (same constant): the batch rows of a tile differ by more than 2.5 times what 16 entries
// of a weight column do.  stat[0] = widths of the input columns over all batch tiles, stat[1] = widths of the same
// columns over 16 weight rows.
// `ratio` is kProbeRatio for the sort-neuron forms.  The l-inf form asks for more (kProbeRatioMax): its kernel only pays
// below about 4 % of marks, and on inputs spread evenly over their range the marked share is about 1.5 / (that ratio), so
// its tables are not even built unless the probe promises that few.
constexpr float kProbeRatio = 2.5f, kProbeRatioMax = 40.f;
__device__ __forceinline__ bool rows_decide(const float* stat, int S, float ratio) {
    return stat[0] > ratio * (float)S * stat[1];
}

// Top-K lists hold their values ascending (res[K-1] largest) and start at 0: new[k] = max(res[k], min(res[k+1], v))
// (core/cuda/sort_neuron.cu:76-77) = the median of the three.  An undefined v leaves the list unchanged (the
// median instruction then returns the smallest defined operand), a negative one as well.
template <int K>
__device__ __forceinline__ void insert_value(float (&res)[K], float v) {
    #pragma unroll
    for (int k = 0; k < K - 1; k++) res[k] = __builtin_amdgcn_fmed3f(res[k], v, res[k + 1]);
    res[K - 1] = __builtin_amdgcn_fmed3f(res[K - 1], v, __builtin_inff());
}
// The same with +infinity held in a register the compiler cannot see through: with the literal it rewrites the last
// median as a maximum and adds an instruction that quiets res[K - 1] first (two instructions per list and mark).
template <int K>
__device__ __forceinline__ void insert_value(float (&res)[K], float v, float inf) {
    #pragma unroll
    for (int k = 0; k < K - 1; k++) res[k] = __builtin_amdgcn_fmed3f(res[k], v, res[k + 1]);
    res[K - 1] = __builtin_amdgcn_fmed3f(res[K - 1], v, inf);
}

template <class F, int... R>
__device__ __forceinline__ void static_for(F&& f, std::integer_sequence<int, R...>) {
    (f(std::integral_constant<int, R>{}), ...);
}

// ---- tables ----------------------------------------------------------------------------------
// Column ranges of the weights over a tile of 128 weight rows (WMASK: over the rows that keep the input; a column
// that no row keeps, or that holds an undefined or infinite weight, becomes (-inf, +inf): no lower bound, always a
// candidate).  64 inputs x 4 groups of 32 rows per workgroup.
template <bool WMASK, bool WT = false>
__global__ void __launch_bounds__(256) rc_range_kernel(const float* __restrict__ w, const uint32_t* __restrict__ wkeep,
                                                       int M, int N, int S, float* __restrict__ wr,
                                                       const float* __restrict__ stat, float ratio,
                                                       float* __restrict__ wt = nullptr) {
    if (!rows_decide(stat, S, ratio)) return;
    __shared__ float part[4][3][64];
    const int nl = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + nl, t = blockIdx.y;
    const int r0 = t * kTileW + grp * (kTileW / 4);
    const int r1 = r0 + kTileW / 4 < M ? r0 + kTileW / 4 : M;
    float lo = __builtin_inff(), hi = -__builtin_inff(), odd = 0.f;
    if constexpr (WT) {
        // WT: also the transposed copy, wt[(t N + n) 128 + row of the tile] (rows past the last: zero, not used)
        static_assert(!WMASK, "the transposed copy is for the forms without a mask");
        if (n < N) {
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
    } else if (n < N) {
        #pragma unroll 4
        for (int m = r0; m < r1; m++) {
            bool kept = true;
            if constexpr (WMASK) kept = (wkeep[(size_t)m * (N / kChunk) + (n >> 5)] >> (n & 31)) & 1u;
            if (kept) {
                const float v = w[(size_t)m * N + n];
                lo = fminf(lo, v); hi = fmaxf(hi, v); odd += v - v;
            }
        }
    }
    part[grp][0][nl] = lo; part[grp][1][nl] = hi; part[grp][2][nl] = odd;
    __syncthreads();
    if (grp == 0 && n < N) {
        #pragma unroll
        for (int g = 1; g < 4; g++) { lo = fminf(lo, part[g][0][nl]); hi = fmaxf(hi, part[g][1][nl]); odd += part[g][2][nl]; }
        if (!(odd == 0.f) || lo > hi) { lo = -__builtin_inff(); hi = __builtin_inff(); }
        wr[(size_t)(t * 2) * N + n] = lo;
        wr[(size_t)(t * 2 + 1) * N + n] = hi;
    }
}

// The two table kernels share their tiling: a workgroup takes 64 batch rows (one per lane; l and u through LDS,
// repaired) and a slice of the inputs; wavefront v works on weight tile 4 blockIdx.z + v, whose column ranges are
// LDS broadcasts.
// Lower bounds.  The smallest a term can be over the weight rows of the tile bounds it from below for every one of
// them (fp32 subtraction is monotone, so this holds for the rounded terms), and K chunks of inputs whose largest
// such bound is at least t hold K terms that are at least t for every weight row: the kernel keeps the K largest
// chunk maxima of the slice (one insertion per 32 inputs), whose K-th largest over all slices bounds the K-th
// largest term.  Value form: l = u = x.
// XMASK (l-inf form under the factored mask): xkeep holds one word per (batch row, 32 inputs); an input the batch row
// does not keep has no term.
template <int K, bool IV, bool XMASK>
__global__ void __launch_bounds__(256) rc_low_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                     const uint32_t* __restrict__ xkeep, const float* __restrict__ wr,
                                                     int B, int N, int T, int Bp, int S, float* __restrict__ lists,
                                                     const float* __restrict__ stat, float ratio) {
    if (!rows_decide(stat, S, ratio)) return;
    __shared__ __attribute__((aligned(16))) float lt[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float ut[IV ? 64 : 1][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float ws[4][2][kChunk];
    const int tid = threadIdx.x, r = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b0 = blockIdx.x * 64, NCH = N / kChunk;
    const int slices = gridDim.y, slice = blockIdx.y;
    const int per = (NCH + slices - 1) / slices;
    const int c_lo = slice * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;
    const int lrow = tid >> 2, q = tid & 3;
    const int bload = b0 + lrow < B ? b0 + lrow : B - 1;
    const int brow = b0 + r < B ? b0 + r : B - 1;
    const int xt = tid >> 6, xk = (tid >> 5) & 1, xn = tid & 31;   // this work-item's value of ws
    const int tb = blockIdx.z * 4, t = tb + wave;
    const bool active = t < T;
    constexpr int nw = IV ? 2 : 1;
    float hi[K], lo[IV ? K : 1];
    #pragma unroll
    for (int k = 0; k < K; k++) { hi[k] = 0.f; if constexpr (IV) lo[k] = 0.f; }
    float4 la, lb, ua, ub;
    float px;
    const float* wsrc = wr + ((size_t)(tb + xt < T ? tb + xt : T - 1) * 2 + xk) * N + xn;
    auto fetch = [&](int c) {
        const int cc = c < c_hi ? c : c_hi - 1;
        const size_t off = (size_t)bload * N + cc * kChunk + 8 * q;
        la = *reinterpret_cast<const float4*>(xl + off); lb = *reinterpret_cast<const float4*>(xl + off + 4);
        if constexpr (IV) { ua = *reinterpret_cast<const float4*>(xu + off); ub = *reinterpret_cast<const float4*>(xu + off + 4); }
        px = wsrc[cc * kChunk];
    };
    if (c_lo < c_hi) fetch(c_lo);
    for (int c = c_lo; c < c_hi; c++) {
        {
            float4 a = la, b = lb;
            if constexpr (IV) {
                float4 d = ua, e = ub;
                repair(a.x, d.x); repair(a.y, d.y); repair(a.z, d.z); repair(a.w, d.w);
                repair(b.x, e.x); repair(b.y, e.y); repair(b.z, e.z); repair(b.w, e.w);
                *reinterpret_cast<float4*>(&ut[lrow][8 * q]) = d; *reinterpret_cast<float4*>(&ut[lrow][8 * q + 4]) = e;
            }
            *reinterpret_cast<float4*>(&lt[lrow][8 * q]) = a; *reinterpret_cast<float4*>(&lt[lrow][8 * q + 4]) = b;
            ws[xt][xk][xn] = px;
        }
        fetch(c + 1);
        __syncthreads();
        if (active) {
            // largest lower bound of the chunk: fmaxf drops undefined differences, and the lists start at 0
            float cu = 0.f, cl = 0.f;
            uint32_t kx = ~0u;
            if constexpr (XMASK) kx = xkeep[(size_t)brow * NCH + c];
            #pragma unroll
            for (int n4 = 0; n4 < kChunk; n4 += 4) {
                const float4 l4 = *reinterpret_cast<const float4*>(&lt[r][n4]);
                const float4 u4 = IV ? *reinterpret_cast<const float4*>(&ut[IV ? r : 0][n4]) : l4;
                const float4 a4 = *reinterpret_cast<const float4*>(&ws[wave][0][n4]);   // min w
                const float4 b4 = *reinterpret_cast<const float4*>(&ws[wave][1][n4]);   // max w
                const float l[4] = {l4.x, l4.y, l4.z, l4.w}, u[4] = {u4.x, u4.y, u4.z, u4.w};
                const float wmin[4] = {a4.x, a4.y, a4.z, a4.w}, wmax[4] = {b4.x, b4.y, b4.z, b4.w};
                #pragma unroll
                for (int k = 0; k < 4; k++) {
                    if constexpr (XMASK) {
                        const float a = fmaxf(wmin[k] - l[k], u[k] - wmax[k]);
                        cu = fmaxf(cu, ((kx >> (n4 + k)) & 1u) ? a : 0.f);
                    } else cu = fmaxf(fmaxf(cu, wmin[k] - l[k]), u[k] - wmax[k]);
                    if constexpr (IV) cl = fmaxf(fmaxf(cl, l[k] - wmax[k]), wmin[k] - u[k]);
                }
            }
            insert_value<K>(hi, cu);
            if constexpr (IV) insert_value<K>(lo, cl);
        }
        __syncthreads();
    }
    if (active) {
        float* dst = lists + (((size_t)t * slices + slice) * nw) * K * Bp + b0 + r;
        #pragma unroll
        for (int k = 0; k < K; k++) {
            dst[(size_t)k * Bp] = hi[k];
            if constexpr (IV) dst[(size_t)(K + k) * Bp] = lo[k];
        }
    }
}

// K-th largest of the slices' lists (0 when fewer than K lower bounds are positive); grid.y = T * nw
template <int K>
__global__ void __launch_bounds__(256) rc_merge_kernel(const float* __restrict__ lists, int slices, int Bp, int nw, int S,
                                                       float* __restrict__ low, const float* __restrict__ stat, float ratio) {
    if (!rows_decide(stat, S, ratio)) return;
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= Bp) return;
    const int t = blockIdx.y / nw, which = blockIdx.y % nw;
    float res[K];
    #pragma unroll
    for (int k = 0; k < K; k++) res[k] = 0.f;
    for (int slice = 0; slice < slices; slice++) {
        const float* src = lists + ((((size_t)t * slices + slice) * nw + which) * K) * Bp + b;
        #pragma unroll
        for (int k = 0; k < K; k++) insert_value<K>(res, src[(size_t)k * Bp]);
    }
    low[((size_t)t * nw + which) * Bp + b] = res[0];
}

// One table word per (tile, chunk, batch row): bit n set when the largest the term of input n can be over the weight
// rows of the tile reaches the bound of its list and is positive (the lists start at 0 and take larger values only;
// an undefined bound or term compares false: an undefined term is left out of every list).  Marks counted per
// wavefront.
// BYROW: the words of a (tile, batch row) lie side by side over the chunks, bits[(t Bp + b) NCH + c] (rt_main_kernel
// reads a row's words 64 at a time); otherwise those of a (tile, chunk) over the batch rows, bits[(t NCH + c) Bp + b].
template <bool IV, bool XMASK, bool BYROW = false>
__global__ void __launch_bounds__(256) rc_bits_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                      const uint32_t* __restrict__ xkeep, const float* __restrict__ wr,
                                                      const float* __restrict__ low, int B, int N, int T, int Bp, int S,
                                                      uint32_t* __restrict__ bits, uint32_t* __restrict__ partial,
                                                      const float* __restrict__ stat, float ratio) {
    if (!rows_decide(stat, S, ratio)) return;
    __shared__ __attribute__((aligned(16))) float lt[64][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float ut[IV ? 64 : 1][kChunk + 4];
    __shared__ __attribute__((aligned(16))) float ws[4][2][kChunk];
    const int tid = threadIdx.x, r = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b0 = blockIdx.x * 64, NCH = N / kChunk;
    const int slices = gridDim.y, slice = blockIdx.y;
    const int per = (NCH + slices - 1) / slices;
    const int c_lo = slice * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;
    const int lrow = tid >> 2, q = tid & 3;
    const int bload = b0 + lrow < B ? b0 + lrow : B - 1;
    const int brow = b0 + r < B ? b0 + r : B - 1;
    const bool valid = b0 + r < B;
    const int xt = tid >> 6, xk = (tid >> 5) & 1, xn = tid & 31;
    const int tb = blockIdx.z * 4, t = tb + wave;
    const bool active = t < T;
    constexpr int nw = IV ? 2 : 1;
    int marks = 0;
    float LU = 0.f, LL = 0.f;
    if (active) {
        LU = low[((size_t)t * nw) * Bp + b0 + r];
        if constexpr (IV) LL = low[((size_t)t * nw + 1) * Bp + b0 + r];
    }
    float4 la, lb, ua, ub;
    float px;
    const float* wsrc = wr + ((size_t)(tb + xt < T ? tb + xt : T - 1) * 2 + xk) * N + xn;
    auto fetch = [&](int c) {
        const int cc = c < c_hi ? c : c_hi - 1;
        const size_t off = (size_t)bload * N + cc * kChunk + 8 * q;
        la = *reinterpret_cast<const float4*>(xl + off); lb = *reinterpret_cast<const float4*>(xl + off + 4);
        if constexpr (IV) { ua = *reinterpret_cast<const float4*>(xu + off); ub = *reinterpret_cast<const float4*>(xu + off + 4); }
        px = wsrc[cc * kChunk];
    };
    if (c_lo < c_hi) fetch(c_lo);
    for (int c = c_lo; c < c_hi; c++) {
        {
            float4 a = la, b = lb;
            if constexpr (IV) {
                float4 d = ua, e = ub;
                repair(a.x, d.x); repair(a.y, d.y); repair(a.z, d.z); repair(a.w, d.w);
                repair(b.x, e.x); repair(b.y, e.y); repair(b.z, e.z); repair(b.w, e.w);
                *reinterpret_cast<float4*>(&ut[lrow][8 * q]) = d; *reinterpret_cast<float4*>(&ut[lrow][8 * q + 4]) = e;
            }
            *reinterpret_cast<float4*>(&lt[lrow][8 * q]) = a; *reinterpret_cast<float4*>(&lt[lrow][8 * q + 4]) = b;
            ws[xt][xk][xn] = px;
        }
        fetch(c + 1);
        __syncthreads();
        if (active) {
            uint32_t word = 0;
            #pragma unroll
            for (int n4 = 0; n4 < kChunk; n4 += 4) {
                const float4 l4 = *reinterpret_cast<const float4*>(&lt[r][n4]);
                const float4 u4 = IV ? *reinterpret_cast<const float4*>(&ut[IV ? r : 0][n4]) : l4;
                const float4 a4 = *reinterpret_cast<const float4*>(&ws[wave][0][n4]);
                const float4 b4 = *reinterpret_cast<const float4*>(&ws[wave][1][n4]);
                const float l[4] = {l4.x, l4.y, l4.z, l4.w}, u[4] = {u4.x, u4.y, u4.z, u4.w};
                const float wmin[4] = {a4.x, a4.y, a4.z, a4.w}, wmax[4] = {b4.x, b4.y, b4.z, b4.w};
                #pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float capU = fmaxf(wmax[k] - l[k], u[k] - wmin[k]);
                    bool mark = capU >= LU && capU > 0.f;
                    if constexpr (IV) {
                        const float capL = fmaxf(l[k] - wmin[k], wmax[k] - u[k]);
                        mark = mark || (capL >= LL && capL > 0.f);
                    }
                    word |= (uint32_t)mark << (n4 + k);
                }
            }
            if (!valid) word = 0u;
            if constexpr (XMASK) word &= xkeep[(size_t)brow * NCH + c];
            if constexpr (BYROW) bits[((size_t)t * Bp + b0 + r) * NCH + c] = word;
            else bits[((size_t)t * NCH + c) * Bp + b0 + r] = word;
            marks += __builtin_popcount(word);
        }
        __syncthreads();
    }
    #pragma unroll
    for (int o = 32; o; o >>= 1) marks += __shfl_xor(marks, o);
    if (r == 0) partial[(((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 4 + wave] = (uint32_t)marks;
}

// count[0] = marks (all ones when the table was not built), count[1] = 1 when the kernels that evaluate every term
// are to run (neither table is below its limit), count[2] = 1 when this table's kernel runs, count[3] = marks per
// weight row (copy), count[4] = 0 (the main kernel counts the outputs to recompute there)
__global__ void __launch_bounds__(1024) rc_sum_kernel(const uint32_t* __restrict__ partial, size_t n,
                                                      unsigned long long* __restrict__ count,
                                                      const unsigned long long* __restrict__ col_count,
                                                      const float* __restrict__ stat, int S, unsigned long long limit,
                                                      float ratio) {
    __shared__ unsigned long long acc[1024];
    const bool rows = rows_decide(stat, S, ratio);
    unsigned long long s0 = 0;
    if (rows) for (size_t i = threadIdx.x; i < n; i += 1024) s0 += partial[i];
    acc[threadIdx.x] = s0;
    __syncthreads();
    for (int o = 512; o; o >>= 1) {
        if ((int)threadIdx.x < o) acc[threadIdx.x] += acc[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const bool run = rows && acc[0] <= limit;
        count[0] = rows ? acc[0] : ~0ull;
        count[1] = (col_count[1] != 0ull && !run) ? 1ull : 0ull;
        count[2] = run ? 1ull : 0ull;
        count[3] = col_count[0];
        count[4] = 0ull;
    }
}

// ---- main kernel -------------------------------------------------------------------------------
// A workgroup of 16 wavefronts owns 128 weight rows (lane l holds the rows l and l + 64 of the tile) and a group of
// `rows` <= 16 TR batch rows, dealt evenly to its wavefronts (at most TR each).  The group size is chosen on the host
// so that the workgroups fill whole rounds of the chip's compute units.  The inputs go by in stages of 64.  The
// weight tile of a stage (128 x 64) goes through LDS, where an input's (w, w') of a lane is one 8-byte word; the
// tiles of the next two stages are on their way while the current one is used.  A wavefront keeps the inputs of its
// own rows in registers (lane i holds input i of the stage; the next stage's are fetched a stage ahead), so a marked
// input's value reaches the terms as a lane read and no barrier stands between a wavefront and its inputs.  The table
// words of 32 stages at a time are copied to LDS ahead of the loop over them; a stage nobody marks is not staged.  One
// loop per batch row over that row's own marks, so that the top-K lists are only ever indexed with constants; the
// marks are taken four at a time, the weights of all four requested before the first term is formed (the walk is
// bound by the latency of its LDS reads otherwise).  The results are written along the weight rows as they are.
constexpr int kStage = 2 * kChunk;   // inputs of a stage: two table words per batch row

struct MainArgs {
    const float* xl; const float* xu; const float* w;
    const uint32_t* xkeep; const uint32_t* wkeep;   // factored mask (l-inf form), or null
    const uint32_t* bits; const float* low;
    unsigned long long* count;
    uint32_t* fix;
    int B, Bp, M, N;
    int rows;                                        // batch rows of a workgroup
    float q;
    float* outL; float* outU; int* pos;
};

template <int FORM, int K, int TR, bool POS, bool MASKED>
__global__ void __launch_bounds__(64 * kWaves, 1) rc_main_kernel(MainArgs a) {
    if (a.count[2] == 0ull) return;
    constexpr bool IV = FORM == kRowsSortInterval;
    constexpr int ROWS = kWaves * TR;                 // most batch rows of a workgroup
    constexpr int TILE = kStage * kWRow;              // floats of one buffer
    extern __shared__ __attribute__((aligned(16))) float smem[];
    uint32_t* wb = reinterpret_cast<uint32_t*>(smem + 2 * TILE);   // [kSeg][ROWS]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this wavefront's lists of the marked inputs of its rows in one stage (two entries past a full list are read)
    // (off: byte offset of the input's weights in the tile; un: the row's upper end in the interval form, the input's
    // number within the stage, as bits, in the others)
    struct Entry { int off; float l, un; };
    Entry* marks = reinterpret_cast<Entry*>(wb + kSeg * ROWS) + wave * (TR * kStage + 2);
    const int B = a.B, Bp = a.Bp, M = a.M, N = a.N, NCH = N / kChunk;
    const int rows = a.rows, BG = (B + rows - 1) / rows;
    // Workgroups go to the chip's eight dies in turn, each with a cache of its own: consecutive (tile, batch rows)
    // pairs are dealt out so that the workgroups of a tile of weight rows, which all stream that tile, share a die
    int item = blockIdx.x;
    if (gridDim.x % 8 == 0) item = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int bg = item % BG, t = item / BG;
    const int m0 = t * kTileW, b0 = bg * rows;
    // this wavefront's rows of the group: r_lo .. r_lo + nr - 1 (nr <= TR)
    const int r_lo = wave * rows / kWaves, nr = (wave + 1) * rows / kWaves - r_lo;
    auto wt = [&](int buf) { return smem + buf * TILE; };

    // the lists of marks start as zeros: entries past the end of a list are read (and not used)
    for (int i = lane; i < (TR * kStage + 2) * 3; i += 64) reinterpret_cast<uint32_t*>(marks)[i] = 0u;
    float inf = __builtin_inff();
    asm volatile("" : "+v"(inf));                     // (see insert_value)

    // state of the wavefront's rows x the lane's two weight rows
    constexpr bool LISTS = FORM != kRowsMax;
    float hi[TR][2][LISTS ? K : 1];
    float lo[IV ? TR : 1][2][IV ? K : 1];
    int idx[(FORM == kRowsSortPos || (FORM == kRowsMax && POS)) ? TR : 1][2][FORM == kRowsSortPos ? K : 1];
    #pragma unroll
    for (int r = 0; r < TR; r++) {
        #pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (LISTS) {
                #pragma unroll
                for (int k = 0; k < K; k++) {
                    hi[r][j][k] = 0.f;
                    if constexpr (IV) lo[r][j][k] = 0.f;
                    if constexpr (FORM == kRowsSortPos) idx[r][j][k] = 0;
                }
            } else {
                hi[r][j][0] = kEps;
                if constexpr (POS) idx[r][j][0] = 0;
            }
        }
    }

    // word of (chunk c, batch row b0 + i): bw[c * Bp + i]; rows past the batch, up to the padded count, hold zero
    const uint32_t* __restrict__ bw = a.bits + (size_t)t * NCH * Bp + b0;
    int seg_lo = 0;                                   // first chunk (of 32 inputs) whose words are in LDS
    auto marked = [&](int st) {
        const uint32_t* q = wb + (2 * st - seg_lo) * ROWS;
        uint32_t v = lane < rows ? (q[lane] | q[ROWS + lane]) : 0u;
        if constexpr (ROWS > 64) v |= lane + 64 < rows ? (q[lane + 64] | q[ROWS + lane + 64]) : 0u;
        return __builtin_amdgcn_ballot_w64(v != 0u) != 0ull;
    };
    // weight tile: work-item (frow, fq) carries inputs 4 fq .. + 3 and 32 + 4 fq .. + 3 of weight row frow of the stage
    const int frow = tid >> 3, fq = tid & 7;
    const int fm = m0 + frow < M ? m0 + frow : M - 1;
    struct Piece { float4 a, b; uint32_t ka, kb; };
    auto fetch = [&](int st, bool need, Piece& p) __attribute__((always_inline)) {
        const int c0 = 2 * st, c1 = 2 * st + 1 < NCH ? 2 * st + 1 : 2 * st;   // the last stage may be half a stage
        const float* src = a.w + (size_t)fm * N + 4 * fq;
        p.a = *reinterpret_cast<const float4*>(need ? src + (size_t)c0 * kChunk : a.w);
        p.b = *reinterpret_cast<const float4*>(need ? src + (size_t)c1 * kChunk : a.w);
        if constexpr (MASKED) {
            p.ka = need ? a.wkeep[(size_t)fm * NCH + c0] : 0u;
            p.kb = need ? a.wkeep[(size_t)fm * NCH + c1] : 0u;
        }
    };
    auto stash = [&](int buf, const Piece& p) __attribute__((always_inline)) {
        float4 u = p.a, v = p.b;
        if constexpr (MASKED) {
            // dropped weights become undefined: their terms never compare greater
            const float qn = __builtin_nanf("");
            const uint32_t ba = p.ka >> (4 * fq), bb = p.kb >> (4 * fq);
            u.x = (ba & 1u) ? u.x : qn; u.y = (ba & 2u) ? u.y : qn; u.z = (ba & 4u) ? u.z : qn; u.w = (ba & 8u) ? u.w : qn;
            v.x = (bb & 1u) ? v.x : qn; v.y = (bb & 2u) ? v.y : qn; v.z = (bb & 4u) ? v.z : qn; v.w = (bb & 8u) ? v.w : qn;
        }
        // weight row frow belongs to lane frow % 64, slot frow / 64
        float* dw = wt(buf) + (4 * fq) * kWRow + 2 * (frow & 63) + (frow >> 6);
        dw[0] = u.x; dw[kWRow] = u.y; dw[2 * kWRow] = u.z; dw[3 * kWRow] = u.w;
        dw += kChunk * kWRow;
        dw[0] = v.x; dw[kWRow] = v.y; dw[2 * kWRow] = v.z; dw[3 * kWRow] = v.w;
    };
    // inputs of the wavefront's rows: lane i holds input i of the stage (repaired, dropped inputs undefined)
    uint32_t xoff[TR];   // (B x N stays below 2^31 elements)
    #pragma unroll
    for (int r = 0; r < TR; r++) {
        const int row = b0 + r_lo + (r < nr ? r : 0);
        xoff[r] = (uint32_t)(row < B ? row : B - 1) * (uint32_t)N;
    }
    auto load_x = [&](int st, float (&xl_)[TR], float (&xu_)[IV ? TR : 1]) __attribute__((always_inline)) {
        int n = st * kStage + lane;
        const bool in = n < N;
        n = in ? n : N - 1;
        #pragma unroll
        for (int r = 0; r < TR; r++) {
            float l = a.xl[xoff[r] + n];
            if constexpr (IV) {
                float u = a.xu[xoff[r] + n];
                repair(l, u);
                xu_[r] = u;
            }
            if constexpr (MASKED) {
                const uint32_t kx = a.xkeep[xoff[r] / (uint32_t)kChunk + (uint32_t)(n >> 5)];   // (N is a multiple of 32)
                l = ((kx >> (n & 31)) & 1u) ? l : __builtin_nanf("");
            }
            xl_[r] = l;
        }
    };
    // one marked input of row r: ww = the lane's two weights, (xa, xb) = the row's value and the input's number within
    // the stage as bits (or its l and u), n0 = the first input of the stage
    auto term = [&](auto R, const float2& ww, float xa, float xb, int n0) __attribute__((always_inline)) {
        constexpr int r = decltype(R)::value;
        [[maybe_unused]] const int n = n0 + __float_as_int(xb);   // (forms without an interval)
        if constexpr (IV) {
            const float a1 = ww.x - xa, a2 = xb - ww.x, b1 = ww.y - xa, b2 = xb - ww.y;
            insert_value<K>(lo[r][0], -fminf(a1, a2), inf);
            insert_value<K>(hi[r][0], fmaxf(a1, a2), inf);
            insert_value<K>(lo[r][1], -fminf(b1, b2), inf);
            insert_value<K>(hi[r][1], fmaxf(b1, b2), inf);
        } else {
            const float d0 = xa - ww.x, d1 = xa - ww.y;
            if constexpr (FORM == kRowsSortValues) {
                insert_value<K>(hi[r][0], fabsf(d0), inf);
                insert_value<K>(hi[r][1], fabsf(d1), inf);
            } else if constexpr (FORM == kRowsSortPos) {
                // the marks of a row go by in ascending input order: the ordered insertion of the scan over
                // all inputs (core/cuda/sort_neuron.cu:108-113, 176-185), ties included
                if (fabsf(d0) > hi[r][0][0]) topk_insert<K>(hi[r][0], idx[r][0], fabsf(d0), n | (d0 >= 0.f ? 0 : (int)kSign));
                if (fabsf(d1) > hi[r][1][0]) topk_insert<K>(hi[r][1], idx[r][1], fabsf(d1), n | (d1 >= 0.f ? 0 : (int)kSign));
            } else {
                // running maximum; only a larger term replaces it, so the first of equal terms keeps the
                // position (core/cuda/inf_dist_cuda.cu:176-190); an undefined term never compares greater
                const bool g0 = fabsf(d0) > hi[r][0][0], g1 = fabsf(d1) > hi[r][1][0];
                hi[r][0][0] = g0 ? fabsf(d0) : hi[r][0][0];
                hi[r][1][0] = g1 ? fabsf(d1) : hi[r][1][0];
                if constexpr (POS) {
                    idx[r][0][0] = g0 ? (n | (d0 >= 0.f ? 0 : (int)kSign)) : idx[r][0][0];
                    idx[r][1][0] = g1 ? (n | (d1 >= 0.f ? 0 : (int)kSign)) : idx[r][1][0];
                }
            }
        }
    };
    // The marks of the wavefront's rows in the stage are first compacted by the lanes themselves: lane i, which holds
    // input i, finds its place among the marked lanes of a row with a bit count and posts (i, value) in that row's
    // list.  The walk over a list then costs one broadcast read per mark and no bit scanning (the scalar unit, which
    // all sixteen wavefronts share, only keeps the loop's count), and it is software-pipelined: while the terms of
    // mark k are formed, the weights of mark k + 1 and the entry of mark k + 2 are on their way (an entry must have
    // arrived before its weights can be asked for: two dependent LDS reads per mark otherwise).  The rows' lists lie
    // end to end, so the pipeline is filled once per stage and runs on across the rows.
    auto compute = [&](int buf, int st, const float (&xl_)[TR], const float (&xu_)[IV ? TR : 1]) __attribute__((always_inline)) {
        const char* W = reinterpret_cast<const char*>(wt(buf) + 2 * lane);
        const uint32_t* words = wb + (2 * st - seg_lo) * ROWS + r_lo;
        uint32_t wa[TR], wc[TR];
        #pragma unroll
        for (int r = 0; r < TR; r++) { wa[r] = words[r < nr ? r : 0]; wc[r] = words[ROWS + (r < nr ? r : 0)]; }
        int end[TR];                                      // one past row r's last entry in the wavefront's list
        __builtin_amdgcn_wave_barrier();                 // the walk of the stage before this one has read its entries
        int filled = 0;
        #pragma unroll
        for (int r = 0; r < TR; r++) {
            uint32_t mlo = 0u, mhi = 0u;
            if (r < nr) { mlo = (uint32_t)__builtin_amdgcn_readfirstlane(wa[r]); mhi = (uint32_t)__builtin_amdgcn_readfirstlane(wc[r]); }
            const uint32_t mine = ((lane < 32 ? mlo : mhi) >> (lane & 31)) & 1u;
            const int rank = (int)__builtin_amdgcn_mbcnt_hi(mhi, __builtin_amdgcn_mbcnt_lo(mlo, 0u));
            if (mine) marks[filled + rank] = Entry{lane * (kWRow * 4), xl_[r], IV ? xu_[IV ? r : 0] : __int_as_float(lane)};
            filled += __builtin_popcount(mlo) + __builtin_popcount(mhi);
            end[r] = filled;
        }
        __builtin_amdgcn_wave_barrier();                 // LDS operations of one wavefront complete in order
        if (filled == 0) return;
        const int n0 = st * kStage;
        // (past the end of the list the entries are stale, from an earlier stage or the zeros the lists start with:
        // their offsets lie in the tile and what is read through them is not used)
        Entry e = marks[0], e1 = marks[1];
        float2 ww = *reinterpret_cast<const float2*>(W + e.off);
        int k = 0;
        static_for([&](auto R) __attribute__((always_inline)) {
            constexpr int r = decltype(R)::value;
            for (; k < end[r]; k++) {
                const float2 w1 = *reinterpret_cast<const float2*>(W + e1.off);
                const Entry e2 = marks[k + 2];
                term(R, ww, e.l, e.un, n0);
                e = e1; ww = w1; e1 = e2;
            }
        }, std::make_integer_sequence<int, TR>{});
    };

    float xc[TR], xcu[IV ? TR : 1], xn[TR], xnu[IV ? TR : 1];
    for (; seg_lo < NCH; seg_lo += kSeg) {
        const int seg_hi = seg_lo + kSeg < NCH ? seg_lo + kSeg : NCH;      // chunks [seg_lo, seg_hi), seg_lo even
        const int st_lo = seg_lo / 2, st_hi = (seg_hi + 1) / 2;
        __syncthreads();
        for (int e = tid; e < kSeg * ROWS; e += 64 * kWaves) {
            const int i = e % ROWS, c = seg_lo + e / ROWS;
            wb[e] = (i < rows && c < seg_hi) ? bw[(size_t)c * Bp + i] : 0u;
        }
        __syncthreads();
        // stage st is used from LDS while the pieces of stages st + 1 and st + 2 are on their way
        Piece pa, pb;
        pa.ka = pa.kb = pb.ka = pb.kb = 0u;
        bool n0 = marked(st_lo), n1 = st_lo + 1 < st_hi ? marked(st_lo + 1) : false;
        fetch(st_lo, n0, pa);
        fetch(st_lo + 1 < st_hi ? st_lo + 1 : st_lo, n1, pb);
        load_x(st_lo, xc, xcu);
        if (n0) stash(0, pa);
        __syncthreads();
        for (int st = st_lo; st < st_hi; st += 2) {
            const bool n2 = st + 2 < st_hi ? marked(st + 2) : false;
            fetch(st + 2 < st_hi ? st + 2 : st, n2, pa);
            load_x(st + 1 < st_hi ? st + 1 : st, xn, xnu);
            if (n0) compute(0, st, xc, xcu);
            if (n1) stash(1, pb);
            __syncthreads();
            if (st + 1 >= st_hi) break;
            const bool n3 = st + 3 < st_hi ? marked(st + 3) : false;
            fetch(st + 3 < st_hi ? st + 3 : st, n3, pb);
            load_x(st + 2 < st_hi ? st + 2 : st, xc, xcu);
            if (n1) compute(1, st + 1, xn, xnu);
            if (n2) stash(0, pa);
            __syncthreads();
            n0 = n2; n1 = n3;
        }
    }

    const size_t plane = (size_t)B * M;
    static_for([&](auto R) __attribute__((always_inline)) {
        constexpr int r = decltype(R)::value;
        const int row = b0 + r_lo + r;
        if (r < nr && row < B) {
            float bound = 0.f;
            if constexpr (MASKED) bound = a.low[(size_t)t * Bp + row];   // wave-uniform
            #pragma unroll
            for (int j = 0; j < 2; j++) {
                const int col = m0 + lane + 64 * j;
                if (col < M) {
                    const size_t o = (size_t)row * M + col;
                    if constexpr (FORM == kRowsSortValues) {
                        a.outU[o] = geo_sum<K>(hi[r][j], a.q);
                    } else if constexpr (IV) {
                        a.outL[o] = geo_sum<K>(lo[r][j], a.q);
                        a.outU[o] = geo_sum<K>(hi[r][j], a.q);
                    } else if constexpr (FORM == kRowsSortPos) {
                        a.outU[o] = geo_sum<K>(hi[r][j], a.q);
                        #pragma unroll
                        for (int k = 0; k < K; k++) a.pos[(size_t)(K - 1 - k) * plane + o] = idx[r][j][k];   // plane 0 = largest
                    } else {
                        a.outU[o] = hi[r][j][0];
                        if constexpr (POS) a.pos[o] = idx[r][j][0];
                        if constexpr (MASKED) {
                            // The bound rests on K inputs that the batch row keeps; a weight row that keeps none of them
                            // may have its maximum at an unmarked input: such an output is recomputed from every input.
                            if (!(hi[r][j][0] >= bound)) a.fix[atomicAdd(a.count + 4, 1ull)] = (uint32_t)o;
                        }
                    }
                }
            }
        }
    }, std::make_integer_sequence<int, TR>{});
}

// ---- main kernel without tiles -------------------------------------------------------------------
// Values and interval bounds of the sort neuron.  A wavefront takes one batch row at a time against the tile's 128
// weight rows (lane l holds the rows l and l + 64): it reads the row's table words 64 chunks at a time, lists the
// marked inputs in LDS and walks the list four marks at a time with the loads of the next four in flight: lane l
// fetches the number and the row's value(s) of mark l % 4 (read back lane by lane, so they are scalar operands of the
// terms), every lane its two weights from the transposed copy (two coalesced 256-byte loads per mark).  No tile is
// staged and no barrier is met, so a wavefront with many marks holds nobody up; the tile's transposed weights
// (2.6 MB at 5120 inputs) stay in the cache of the die its workgroups are dealt to.  Every load is issued
// unconditionally (groups past the end of the list repeat its last mark and are not used), so that the waits the
// compiler places cover exactly the group that is used next.
constexpr int kRtWaves = 8;          // wavefronts of a workgroup
constexpr int kRtRows = 1;           // batch rows a wavefront takes, one after the other
constexpr int kRtBatch = 64;         // chunks whose table words a wavefront reads at a time, one per lane
constexpr int kRtListCap = 2304;     // entries of a wavefront's list of marked inputs (16-bit input numbers)

struct RtArgs {
    const float* xl; const float* xu; const float* wt;
    const uint32_t* bits;
    const unsigned long long* count;
    int B, Bp, M, N;
    float q;
    float* outL; float* outU;
};

template <int K, bool IV>
__global__ void __launch_bounds__(64 * kRtWaves) rt_main_kernel(RtArgs a) {
    if (a.count[2] == 0ull) return;
    __shared__ uint16_t list[kRtWaves][kRtListCap];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int B = a.B, M = a.M, N = a.N, NCH = N / kChunk;
    const int BG = (B + kRtWaves * kRtRows - 1) / (kRtWaves * kRtRows);
    // consecutive (tile, batch rows) pairs are dealt out so that the workgroups of a tile share a die and its cache
    int item = blockIdx.x;
    if (gridDim.x % 8 == 0) item = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int bg = item % BG, t = item / BG;
    const float* __restrict__ wcol = a.wt + (size_t)t * N * kTileW + lane;
    uint16_t* mine = list[wave];
    float inf = __builtin_inff();
    asm volatile("" : "+v"(inf));                     // (see insert_value)

    for (int rr = 0; rr < kRtRows; rr++) {
        const int b = (bg * kRtWaves + wave) * kRtRows + rr;
        if (b >= B) break;   // wave-uniform; the rows of a wavefront ascend
        float hi[2][K], lo[IV ? 2 : 1][IV ? K : 1];
        #pragma unroll
        for (int k = 0; k < K; k++) {
            hi[0][k] = hi[1][k] = 0.f;
            if constexpr (IV) lo[0][k] = lo[1][k] = 0.f;
        }
        const uint32_t* __restrict__ rowbits = a.bits + ((size_t)t * a.Bp + b) * NCH;
        const float* __restrict__ xlrow = a.xl + (size_t)b * N;
        const float* __restrict__ xurow = IV ? a.xu + (size_t)b * N : nullptr;
        int cnt = 0;   // marks in the list
        float xreg[2], ureg[IV ? 2 : 1];
        float wa[2][4], wb[2][4];
        auto load = [&](int buf, int k0, int total) __attribute__((always_inline)) {
            int k = k0 + (lane & 3);
            k = k < total ? k : total - 1;
            const int nn = (int)mine[k];
            float l = xlrow[nn];
            if constexpr (IV) {
                float u = xurow[nn];
                repair(l, u);
                ureg[buf] = u;
            }
            xreg[buf] = l;
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
                    const float xi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xreg[buf]), i));
                    if constexpr (IV) {
                        const float ui = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ureg[buf]), i));
                        const float a1 = wa[buf][i] - xi, a2 = ui - wa[buf][i];
                        const float b1 = wb[buf][i] - xi, b2 = ui - wb[buf][i];
                        insert_value<K>(lo[0], -fminf(a1, a2), inf);
                        insert_value<K>(hi[0], fmaxf(a1, a2), inf);
                        insert_value<K>(lo[1], -fminf(b1, b2), inf);
                        insert_value<K>(hi[1], fmaxf(b1, b2), inf);
                    } else {
                        insert_value<K>(hi[0], fabsf(xi - wa[buf][i]), inf);
                        insert_value<K>(hi[1], fabsf(xi - wb[buf][i]), inf);
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
        for (int c0 = 0; c0 < NCH; c0 += kRtBatch) {
            uint32_t word = next;
            if (c0 + kRtBatch < NCH) next = c0 + kRtBatch + lane < NCH ? rowbits[c0 + kRtBatch + lane] : 0u;
            // every lane appends the marks of its word behind those of the lanes before it
            const int mine_n = __builtin_popcount(word);
            int incl = mine_n;
            #pragma unroll
            for (int o = 1; o < kRtBatch; o <<= 1) {
                const int v = __shfl_up(incl, o);
                if (lane >= o) incl += v;
            }
            int off = cnt + incl - mine_n;
            cnt += __builtin_amdgcn_readlane(incl, kRtBatch - 1);
            while (word) {
                const int i = __builtin_ctz(word);
                word &= word - 1;
                mine[off++] = (uint16_t)(((c0 + lane) << 5) | i);   // the input's number (rows of at most 65536 inputs)
            }
            // a row's marks are walked in one go unless the list could overflow with the next chunks
            if (cnt > kRtListCap - kRtBatch * kChunk || c0 + kRtBatch >= NCH) {
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
                a.outU[o] = geo_sum<K>(hi[j], a.q);
                if constexpr (IV) a.outL[o] = geo_sum<K>(lo[j], a.q);
            }
        }
    }
}

// Outputs of the masked l-inf form whose maximum stayed below the bound their marks were taken against: one
// wavefront per output over every input that both rows keep, lowest input first among equal terms.
template <bool POS>
__global__ void __launch_bounds__(256) rc_fix_kernel(MainArgs a) {
    if (a.count[2] == 0ull) return;
    const unsigned long long total = a.count[4];
    const int lane = threadIdx.x & 63;
    const int N = a.N, NCH = N / kChunk;
    for (unsigned long long e = (unsigned long long)blockIdx.x * 4 + (threadIdx.x >> 6); e < total; e += (unsigned long long)gridDim.x * 4) {
        const uint32_t o = a.fix[e];
        const int b = (int)(o / (uint32_t)a.M), m = (int)(o % (uint32_t)a.M);
        const float* xr = a.xl + (size_t)b * N;
        const float* wrow = a.w + (size_t)m * N;
        float best = kEps;
        int where = 0;
        for (int n = lane; n < N; n += 64) {
            const uint32_t keep = a.xkeep[(size_t)b * NCH + (n >> 5)] & a.wkeep[(size_t)m * NCH + (n >> 5)];
            const float d = xr[n] - wrow[n];
            if (((keep >> (n & 31)) & 1u) && fabsf(d) > best) { best = fabsf(d); where = n | (d >= 0.f ? 0 : (int)kSign); }
        }
        #pragma unroll
        for (int s = 32; s; s >>= 1) {
            const float ob = __shfl_xor(best, s);
            const int ow = __shfl_xor(where, s);
            // a lane that found nothing keeps (1e-10, 0) and loses to any term; equal terms: the lower input
            const bool take = ob > best || (ob == best && ob > kEps && (ow & 0x7fffffff) < (where & 0x7fffffff));
            best = take ? ob : best;
            where = take ? ow : where;
        }
        if (lane == 0) {
            a.outU[o] = best;
            if constexpr (POS) a.pos[o] = where;
        }
    }
}

// Batch rows of a workgroup (at most `cap`): the workgroups stay for their whole run, one per compute unit, so the
// launch proceeds in rounds of num_cus() workgroups and a partly filled last round costs a whole one.  Among the group
// counts from the fewest that `cap` allows up to twice as many, the one that wastes least is taken (more groups also
// stage the weight tiles more often, so the fewest wins ties).
inline int rows_per_group(int B, int T, int cap) {
    const long long cus = num_cus();
    const int g_min = (B + cap - 1) / cap;
    int best_g = g_min;
    double best = 0.0;
    for (int g = g_min; g <= 2 * g_min && g <= B; g++) {
        const long long wgs = (long long)g * T, rounds = (wgs + cus - 1) / cus;
        const int rows = (B + g - 1) / g;
        // time ~ rounds x rows of a group (+ a fixed share per round for staging the tiles)
        const double cost = (double)rounds * (rows + 0.15 * cap);
        if (g == g_min || cost < best * 0.98) { best = cost; best_g = g; }
    }
    return (B + best_g - 1) / best_g;
}

template <int FORM, int K, int TR, bool POS, bool MASKED>
int launch_main(MainArgs a, hipStream_t st) {
    constexpr int ROWS = kWaves * TR;
    constexpr size_t lds = (size_t)(2 * kStage * kWRow + kSeg * ROWS) * 4 + (size_t)kWaves * TR * (kStage + 2) * 12;
    static_assert(lds <= 160 * 1024, "LDS of the main kernel");
    auto kern = rc_main_kernel<FORM, K, TR, POS, MASKED>;
    static bool attr_done = false;   // once per instantiation (benign if two threads both set it)
    if (!attr_done) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            set_error("row_cands: cannot reserve %zu bytes of LDS", lds);
            return SD_ERR_HIP;
        }
        attr_done = true;
    }
    const int T = tiles_w(a.M);
    a.rows = rows_per_group(a.B, T, ROWS);
    const int BG = (a.B + a.rows - 1) / a.rows;
    hipLaunchKernelGGL(kern, dim3((unsigned)(T * BG)), dim3(64 * kWaves), lds, st, a);
    return check_launch("rc_main_kernel");
}

// Batch rows per wavefront: as many as keep the top-K lists of its rows x the lane's two weight rows (2 K registers per
// row for values, 4 K with the second list or the positions) within about 64 of the 128 registers that 16 wavefronts
// per compute unit allow; the rest go to the 24 staging registers of the two chunks in flight, the operands of four
// marks and addresses (checked with the compiler's resource report: no instantiation spills).
constexpr int tr_for(int form, int K) {
    const int per = (form == kRowsSortValues ? 2 : 4) * K;
    // (the ordered insertion with positions needs the most temporaries, the two-list form a few more than the values)
    const int tr = (form == kRowsSortValues ? 64 : form == kRowsSortInterval ? 80 : 40) / per;
    if (form == kRowsSortInterval && tr >= 4) return tr > 5 ? 4 : 3;   // (four and five rows of two lists spill)
    return tr > 5 ? 5 : tr < 1 ? 1 : tr;
}

template <int FORM, int K>
int run(const float* xl, const float* xu, const float* w, int B, int M, int N, float q, float* outL, float* outU, int* pos,
        const Carve& c, unsigned long long limit, const float* col_stat, const unsigned long long* col_count, hipStream_t st) {
    constexpr bool IV = FORM == kRowsSortInterval;
    constexpr bool WT = walks_transposed(FORM);
    const int T = tiles_w(M), Bp = bpad_of(B), NCH = N / kChunk, slices = slices_of(NCH), S = (B + 127) / 128;
    int rc;
    hipLaunchKernelGGL((rc_range_kernel<false, WT>), dim3((N + 63) / 64, T), dim3(256), 0, st, w, nullptr, M, N, S, c.wr, col_stat,
                       kProbeRatio, WT ? c.wt : nullptr);
    if ((rc = check_launch("rc_range_kernel"))) return rc;
    const dim3 tgrid(Bp / 64, slices, (T + 3) / 4);
    hipLaunchKernelGGL((rc_low_kernel<K, IV, false>), tgrid, dim3(256), 0, st, xl, xu, nullptr, c.wr, B, N, T, Bp, S, c.lists, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_low_kernel"))) return rc;
    constexpr int nw = IV ? 2 : 1;
    hipLaunchKernelGGL((rc_merge_kernel<K>), dim3((Bp + 255) / 256, T * nw), dim3(256), 0, st, c.lists, slices, Bp, nw, S, c.low, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_merge_kernel"))) return rc;
    hipLaunchKernelGGL((rc_bits_kernel<IV, false, WT>), tgrid, dim3(256), 0, st, xl, xu, nullptr, c.wr, c.low, B, N, T, Bp, S, c.bits, c.partial, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_bits_kernel"))) return rc;
    hipLaunchKernelGGL(rc_sum_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)tgrid.x * tgrid.y * tgrid.z * 4, c.count, col_count, col_stat, S, limit, kProbeRatio);
    if ((rc = check_launch("rc_sum_kernel"))) return rc;
    if constexpr (WT) {
        RtArgs a{xl, xu, c.wt, c.bits, c.count, B, Bp, M, N, q, outL, outU};
        const int BG = (B + kRtWaves * kRtRows - 1) / (kRtWaves * kRtRows);
        hipLaunchKernelGGL((rt_main_kernel<K, IV>), dim3((unsigned)(T * BG)), dim3(64 * kRtWaves), 0, st, a);
        return check_launch("rt_main_kernel");
    } else {
        MainArgs a{xl, xu, w, nullptr, nullptr, c.bits, c.low, c.count, c.fix, B, Bp, M, N, 0, q, outL, outU, pos};
        return launch_main<FORM, K, tr_for(FORM, K), false, false>(a, st);
    }
}

template <int K, bool MASKED>
int run_max(const float* x, const float* w, const uint32_t* xkeep, const uint32_t* wkeep, int B, int M, int N, float* y,
            int* pos, const Carve& c, unsigned long long limit, const float* col_stat, const unsigned long long* col_count,
            float ratio, hipStream_t st) {
    const int T = tiles_w(M), Bp = bpad_of(B), NCH = N / kChunk, slices = slices_of(NCH), S = (B + 127) / 128;
    int rc;
    hipLaunchKernelGGL((rc_range_kernel<MASKED>), dim3((N + 63) / 64, T), dim3(256), 0, st, w, wkeep, M, N, S, c.wr, col_stat, ratio);
    if ((rc = check_launch("rc_range_kernel"))) return rc;
    const dim3 tgrid(Bp / 64, slices, (T + 3) / 4);
    hipLaunchKernelGGL((rc_low_kernel<K, false, MASKED>), tgrid, dim3(256), 0, st, x, nullptr, xkeep, c.wr, B, N, T, Bp, S, c.lists, col_stat, ratio);
    if ((rc = check_launch("rc_low_kernel"))) return rc;
    hipLaunchKernelGGL((rc_merge_kernel<K>), dim3((Bp + 255) / 256, T), dim3(256), 0, st, c.lists, slices, Bp, 1, S, c.low, col_stat, ratio);
    if ((rc = check_launch("rc_merge_kernel"))) return rc;
    hipLaunchKernelGGL((rc_bits_kernel<false, MASKED>), tgrid, dim3(256), 0, st, x, nullptr, xkeep, c.wr, c.low, B, N, T, Bp, S, c.bits, c.partial, col_stat, ratio);
    if ((rc = check_launch("rc_bits_kernel"))) return rc;
    hipLaunchKernelGGL(rc_sum_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)tgrid.x * tgrid.y * tgrid.z * 4, c.count, col_count, col_stat, S, limit, ratio);
    if ((rc = check_launch("rc_sum_kernel"))) return rc;
    MainArgs a{x, nullptr, w, xkeep, wkeep, c.bits, c.low, c.count, c.fix, B, Bp, M, N, 0, 0.f, nullptr, y, pos};
    // (four rows per wavefront: their mark lists share the LDS with the weight tiles)
    if (pos) rc = launch_main<kRowsMax, 1, 4, true, MASKED>(a, st);
    else rc = launch_main<kRowsMax, 1, 4, false, MASKED>(a, st);
    if (rc || !MASKED) return rc;
    if (pos) hipLaunchKernelGGL((rc_fix_kernel<true>), dim3(256), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((rc_fix_kernel<false>), dim3(256), dim3(256), 0, st, a);
    return check_launch("rc_fix_kernel");
}

}  // namespace

size_t row_cands_workspace(int form, int B, int CO, int CI, int K) {
    size_t sz[8];
    return carve_sizes(form, B, CO, CI, K, sz);
}

bool row_cands_supported(int form, int K) {
    switch (form) {
        case kRowsSortValues: return K >= 2 && K <= 25;
        case kRowsSortInterval: return K >= 2 && K <= 18;
        case kRowsSortPos: return K >= 2 && K <= 12;
        case kRowsMax: return K == 1 || K == 8 || K == 12 || K == 16 || K == 20 || K == 24;
    }
    return false;
}

#define SD_ROWS_K12(X) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12)
#define SD_ROWS_K18(X) SD_ROWS_K12(X) X(13) X(14) X(15) X(16) X(17) X(18)
#define SD_ROWS_K25(X) SD_ROWS_K18(X) X(19) X(20) X(21) X(22) X(23) X(24) X(25)

int row_cands_forward(int form, const float* xl, const float* xu, const float* w, const uint32_t* xkeep,
                      const uint32_t* wkeep, int B, int CO, int CI, float q, int K, float* outL, float* outU, int* pos,
                      void* ws, float density, bool forced, const float* col_stat, const unsigned long long* col_count,
                      const unsigned long long** every, hipStream_t st) {
    const float ratio_max = forced ? kProbeRatio : kProbeRatioMax;
    if (CI % kChunk != 0 || B < 1 || CO < 1 || !row_cands_supported(form, K) || (xkeep == nullptr) != (wkeep == nullptr) ||
        (long long)B * CO >= (1ll << 32)) {
        set_error("row_cands_forward: shape or form not supported");
        return SD_ERR_ARG;
    }
    if (walks_transposed(form) && CI > 65536) {   // (16-bit input numbers in the lists of marks)
        set_error("row_cands_forward: rows of more than 65536 inputs");
        return SD_ERR_ARG;
    }
    const Carve c = carve(ws, form, B, CO, CI, K);
    const float d = density < 0.f ? 0.f : density > 1.f ? 1.f : density;
    const unsigned long long limit = (unsigned long long)((double)tiles_w(CO) * B * CI * d);
    *every = c.count + 1;
    switch (form) {
        case kRowsSortValues:
            switch (K) {
#define X(k) case k: return run<kRowsSortValues, k>(xl, nullptr, w, B, CO, CI, q, outL, outU, nullptr, c, limit, col_stat, col_count, st);
                SD_ROWS_K25(X)
#undef X
            }
            break;
        case kRowsSortInterval:
            switch (K) {
#define X(k) case k: return run<kRowsSortInterval, k>(xl, xu, w, B, CO, CI, q, outL, outU, nullptr, c, limit, col_stat, col_count, st);
                SD_ROWS_K18(X)
#undef X
            }
            break;
        case kRowsSortPos:
            switch (K) {
#define X(k) case k: return run<kRowsSortPos, k>(xl, nullptr, w, B, CO, CI, q, outL, outU, pos, c, limit, col_stat, col_count, st);
                SD_ROWS_K12(X)
#undef X
            }
            break;
        case kRowsMax:
            if (!xkeep) return run_max<1, false>(xl, w, nullptr, nullptr, B, CO, CI, outU, pos, c, limit, col_stat, col_count, ratio_max, st);
            switch (K) {
#define X(k) case k: return run_max<k, true>(xl, w, xkeep, wkeep, B, CO, CI, outU, pos, c, limit, col_stat, col_count, ratio_max, st);
                X(8) X(12) X(16) X(20) X(24)
#undef X
            }
            break;
    }
    set_error("row_cands_forward: K=%d not supported for form %d", K, form);
    return SD_ERR_ARG;
}

}  // namespace sd
