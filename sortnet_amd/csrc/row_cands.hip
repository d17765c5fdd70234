// Sort neuron, its interval bounds and the l-inf forward from candidate tables per batch row (see row_cands.h).
#include "row_cands.h"
#include "fwd_tile.h"

namespace sd {

namespace {

constexpr int kChunk = kRowCandsChunk;
constexpr int kTileW = 128;          // weight rows of a tile: 64 lanes x 2
constexpr int kBPad = 128;           // batch rows are padded to a multiple of this in the tables
constexpr int kMaxPer = 32;          // most chunks a slice of the table kernels covers

inline size_t align256(size_t b) { return (b + 255) / 256 * 256; }
inline int tiles_w(int M) { return (M + kTileW - 1) / kTileW; }
inline int bpad_of(int B) { return (B + kBPad - 1) / kBPad * kBPad; }
inline int slices_of(int NCH) {
    int s = (NCH + kMaxPer - 1) / kMaxPer;
    if (s < 16) s = 16;
    return s < NCH ? s : NCH;
}

struct Carve {
    float* wr;        // [T][2][N]  per tile of weight rows and input: min w, max w over the rows that keep the input
    float* lists;     // [T][slices][nw][K][Bp]  K largest chunk maxima of the lower bounds of a batch row's terms within a slice
    float* low;       // [T][nw][Bp]  K-th largest of them over all slices: upper list, lower list
    uint32_t* bits;   // [T][Bp][NCH] bit i of a word = input 32 c + i may be among the K largest of that batch row in that tile
    uint32_t* partial;            // marks per wavefront of the table kernel
    unsigned long long* count;    // [0] marks, [1] every-term kernels run, [2] this table's kernel runs, [3] marks per weight row (copy), [4] outputs to recompute
    uint32_t* fix;    // [B * M] outputs of the masked l-inf form whose bound did not hold (recomputed from every input)
    float* wt;        // [T][N][128] the weights of a tile, one 512-byte row per input (dropped weights undefined)
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
    sz[7] = align256(T * N * kTileW * 4);
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
// below about 10 % of marks, and on inputs spread evenly over their range the marked share is about 1 / (that ratio), so
// its tables are not even built unless the probe promises that few.
constexpr float kProbeRatio = 2.5f, kProbeRatioMax = 10.f;
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

// ---- tables ----------------------------------------------------------------------------------
// Column ranges of the weights over a tile of 128 weight rows (WMASK: over the rows that keep the input; a column
// that no row keeps, or that holds an undefined or infinite weight, becomes (-inf, +inf): no lower bound, always a
// candidate).  64 inputs x 4 groups of 32 rows per workgroup.
template <bool WMASK>
__global__ void __launch_bounds__(256) rc_range_kernel(const float* __restrict__ w, const uint32_t* __restrict__ wkeep,
                                                       int M, int N, int S, float* __restrict__ wr, float* __restrict__ wt,
                                                       const float* __restrict__ stat, float ratio) {
    if (!rows_decide(stat, S, ratio)) return;
    __shared__ float part[4][3][64];
    const int nl = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + nl, t = blockIdx.y;
    const int r0 = t * kTileW + grp * (kTileW / 4);
    float lo = __builtin_inff(), hi = -__builtin_inff(), odd = 0.f;
    if (n < N) {
        float v[kTileW / 4];
        #pragma unroll
        for (int i = 0; i < kTileW / 4; i++) v[i] = r0 + i < M ? w[(size_t)(r0 + i) * N + n] : 0.f;
        #pragma unroll
        for (int i = 0; i < kTileW / 4; i++) {
            bool kept = r0 + i < M;
            if constexpr (WMASK) {
                if (kept) kept = (wkeep[(size_t)(r0 + i) * (N / kChunk) + (n >> 5)] >> (n & 31)) & 1u;
            }
            if (kept) { lo = fminf(lo, v[i]); hi = fmaxf(hi, v[i]); odd += v[i] - v[i]; }
            else if (WMASK) v[i] = __builtin_nanf("");
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
// The words of a (tile, batch row) lie side by side over the chunks, bits[(t Bp + b) NCH + c]: the main kernel reads a
// row's words 64 at a time.
template <bool IV, bool XMASK>
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
            bits[((size_t)t * Bp + b0 + r) * NCH + c] = word;
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
// A wavefront takes one batch row at a time against the tile's 128 weight rows (lane l holds the rows l and l + 64):
// it reads the row's table words 64 chunks at a time, lists the marked inputs in LDS and walks the list four marks at
// a time with the loads of the next four in flight: lane l fetches the number and the row's value(s) of mark l % 4
// (read back lane by lane, so they are scalar operands of the terms), every lane its two weights from the transposed
// copy (two coalesced 256-byte loads per mark).  No tile is staged and no barrier is met, so a wavefront with many
// marks holds nobody up; a workgroup is eight wavefronts = eight batch rows, and the workgroups of a tile are dealt to
// one die, so that the tile's transposed weights (2.6 MB at 5120 inputs) stay in that die's cache while its 64
// resident workgroups walk them.  Every load is issued unconditionally (groups past the end of the list repeat its last
// mark and are not used), so that the waits the compiler places cover exactly the group that is used next.
// Forms: top-K lists of values (branch-free median insertion), of both interval bounds, of values with the input
// numbers (the reference's ordered insertion: the marks go by in ascending input order), and the l-inf distance (the
// difference of largest magnitude and, optionally, its input; under the factored mask the dropped weights of the
// transposed copy are undefined, the table holds no input the batch row drops, and an output that ends below the bound
// its marks were taken against is listed for rc_fix_kernel).
constexpr int kRtWaves = 8;          // wavefronts of a workgroup
constexpr int kRtRows = 1;           // batch rows a wavefront takes, one after the other
constexpr int kRtBatch = 64;         // chunks whose table words a wavefront reads at a time, one per lane
constexpr int kRtListCap = 2304;     // entries of a wavefront's list of marked inputs (16-bit input numbers)

struct RtArgs {
    const float* xl; const float* xu; const float* wt;
    const uint32_t* bits; const float* low;
    unsigned long long* count;
    uint32_t* fix;
    int B, Bp, M, N;
    float q;
    float* outL; float* outU; int* pos;
};

template <int FORM, int K, bool POS, bool MASKED>
__global__ void __launch_bounds__(64 * kRtWaves) rt_main_kernel(RtArgs a) {
    if (a.count[2] == 0ull) return;
    constexpr bool IV = FORM == kRowsSortInterval;
    constexpr bool LISTS = FORM != kRowsMax;
    constexpr bool IDX = FORM == kRowsSortPos || (FORM == kRowsMax && POS);
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
    const size_t plane = (size_t)B * M;

    for (int rr = 0; rr < kRtRows; rr++) {
        const int b = (bg * kRtWaves + wave) * kRtRows + rr;
        if (b >= B) break;   // wave-uniform; the rows of a wavefront ascend
        // state of the row x the lane's two weight rows: top-K lists (ascending), or the difference of largest magnitude
        float hi[2][LISTS ? K : 1], lo[IV ? 2 : 1][IV ? K : 1];
        int idx[IDX ? 2 : 1][FORM == kRowsSortPos ? K : 1];
        #pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (LISTS) {
                #pragma unroll
                for (int k = 0; k < K; k++) {
                    hi[j][k] = 0.f;
                    if constexpr (IV) lo[j][k] = 0.f;
                    if constexpr (FORM == kRowsSortPos) idx[j][k] = 0;
                }
            } else {
                hi[j][0] = kEps;
                if constexpr (POS) idx[j][0] = 0;
            }
        }
        const uint32_t* __restrict__ rowbits = a.bits + ((size_t)t * a.Bp + b) * NCH;
        const float* __restrict__ xlrow = a.xl + (size_t)b * N;
        const float* __restrict__ xurow = IV ? a.xu + (size_t)b * N : nullptr;
        int cnt = 0;   // marks in the list
        float xreg[2], ureg[IV ? 2 : 1];
        int nreg[IDX ? 2 : 1];
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
            if constexpr (IDX) nreg[buf] = nn;
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
                        const float d0 = xi - wa[buf][i], d1 = xi - wb[buf][i];
                        [[maybe_unused]] int n = 0;
                        if constexpr (IDX) n = __builtin_amdgcn_readlane(nreg[IDX ? buf : 0], i);
                        if constexpr (FORM == kRowsSortValues) {
                            insert_value<K>(hi[0], fabsf(d0), inf);
                            insert_value<K>(hi[1], fabsf(d1), inf);
                        } else if constexpr (FORM == kRowsSortPos) {
                            // the marks of a row go by in ascending input order: the ordered insertion of the scan
                            // over all inputs (core/cuda/sort_neuron.cu:108-113, 176-185), ties included
                            if (fabsf(d0) > hi[0][0]) topk_insert<K>(hi[0], idx[0], fabsf(d0), n | (d0 >= 0.f ? 0 : (int)kSign));
                            if (fabsf(d1) > hi[1][0]) topk_insert<K>(hi[1], idx[1], fabsf(d1), n | (d1 >= 0.f ? 0 : (int)kSign));
                        } else {
                            // running maximum; only a larger term replaces it, so the first of equal terms keeps the
                            // position (core/cuda/inf_dist_cuda.cu:176-190); an undefined term (a weight the row of
                            // the mask drops) never compares greater
                            // (the difference itself is kept: its magnitude is the maximum, its sign the flag of
                            // the position)
                            const bool g0 = fabsf(d0) > fabsf(hi[0][0]), g1 = fabsf(d1) > fabsf(hi[1][0]);
                            hi[0][0] = g0 ? d0 : hi[0][0];
                            hi[1][0] = g1 ? d1 : hi[1][0];
                            if constexpr (POS) {
                                idx[0][0] = g0 ? n : idx[0][0];
                                idx[1][0] = g1 ? n : idx[1][0];
                            }
                        }
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
        float bound = 0.f;
        if constexpr (MASKED) bound = a.low[(size_t)t * a.Bp + b];   // wave-uniform
        #pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = t * kTileW + lane + 64 * j;
            if (col < M) {
                const size_t o = (size_t)b * M + col;
                if constexpr (LISTS) {
                    a.outU[o] = geo_sum<K>(hi[j], a.q);
                    if constexpr (IV) a.outL[o] = geo_sum<K>(lo[j], a.q);
                    if constexpr (FORM == kRowsSortPos) {
                        #pragma unroll
                        for (int k = 0; k < K; k++) a.pos[(size_t)(K - 1 - k) * plane + o] = idx[j][k];   // plane 0 = largest
                    }
                } else {
                    a.outU[o] = fabsf(hi[j][0]);
                    if constexpr (POS) a.pos[o] = idx[j][0] | (hi[j][0] >= 0.f ? 0 : (int)kSign);
                    if constexpr (MASKED) {
                        // The bound rests on K inputs that the batch row keeps; a weight row that keeps none of them
                        // may have its maximum at an unmarked input: such an output is recomputed from every input.
                        if (!(fabsf(hi[j][0]) >= bound)) a.fix[atomicAdd(a.count + 4, 1ull)] = (uint32_t)o;
                    }
                }
            }
        }
    }
}

struct FixArgs {
    const float* xl; const float* w;
    const uint32_t* xkeep; const uint32_t* wkeep;
    const unsigned long long* count;
    const uint32_t* fix;
    int M, N;
    float* outU; int* pos;
};

// Outputs of the masked l-inf form whose maximum stayed below the bound their marks were taken against: one
// wavefront per output over every input that both rows keep, lowest input first among equal terms.
template <bool POS>
__global__ void __launch_bounds__(256) rc_fix_kernel(FixArgs a) {
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

template <int FORM, int K, bool POS, bool MASKED>
int launch_rt(const RtArgs& a, hipStream_t st) {
    const int T = tiles_w(a.M), BG = (a.B + kRtWaves * kRtRows - 1) / (kRtWaves * kRtRows);
    hipLaunchKernelGGL((rt_main_kernel<FORM, K, POS, MASKED>), dim3((unsigned)(T * BG)), dim3(64 * kRtWaves), 0, st, a);
    return check_launch("rt_main_kernel");
}

template <int FORM, int K>
int run(const float* xl, const float* xu, const float* w, int B, int M, int N, float q, float* outL, float* outU, int* pos,
        const Carve& c, unsigned long long limit, const float* col_stat, const unsigned long long* col_count, hipStream_t st) {
    constexpr bool IV = FORM == kRowsSortInterval;
    const int T = tiles_w(M), Bp = bpad_of(B), NCH = N / kChunk, slices = slices_of(NCH), S = (B + 127) / 128;
    int rc;
    hipLaunchKernelGGL((rc_range_kernel<false>), dim3((N + 63) / 64, T), dim3(256), 0, st, w, nullptr, M, N, S, c.wr, c.wt, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_range_kernel"))) return rc;
    const dim3 tgrid(Bp / 64, slices, (T + 3) / 4);
    hipLaunchKernelGGL((rc_low_kernel<K, IV, false>), tgrid, dim3(256), 0, st, xl, xu, nullptr, c.wr, B, N, T, Bp, S, c.lists, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_low_kernel"))) return rc;
    constexpr int nw = IV ? 2 : 1;
    hipLaunchKernelGGL((rc_merge_kernel<K>), dim3((Bp + 255) / 256, T * nw), dim3(256), 0, st, c.lists, slices, Bp, nw, S, c.low, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_merge_kernel"))) return rc;
    hipLaunchKernelGGL((rc_bits_kernel<IV, false>), tgrid, dim3(256), 0, st, xl, xu, nullptr, c.wr, c.low, B, N, T, Bp, S, c.bits, c.partial, col_stat, kProbeRatio);
    if ((rc = check_launch("rc_bits_kernel"))) return rc;
    hipLaunchKernelGGL(rc_sum_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)tgrid.x * tgrid.y * tgrid.z * 4, c.count, col_count, col_stat, S, limit, kProbeRatio);
    if ((rc = check_launch("rc_sum_kernel"))) return rc;
    RtArgs a{xl, xu, c.wt, c.bits, c.low, c.count, c.fix, B, Bp, M, N, q, outL, outU, pos};
    return launch_rt<FORM, K, false, false>(a, st);
}

template <int K, bool MASKED>
int run_max(const float* x, const float* w, const uint32_t* xkeep, const uint32_t* wkeep, int B, int M, int N, float* y,
            int* pos, const Carve& c, unsigned long long limit, const float* col_stat, const unsigned long long* col_count,
            float ratio, hipStream_t st) {
    const int T = tiles_w(M), Bp = bpad_of(B), NCH = N / kChunk, slices = slices_of(NCH), S = (B + 127) / 128;
    int rc;
    hipLaunchKernelGGL((rc_range_kernel<MASKED>), dim3((N + 63) / 64, T), dim3(256), 0, st, w, wkeep, M, N, S, c.wr, c.wt, col_stat, ratio);
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
    RtArgs a{x, nullptr, c.wt, c.bits, c.low, c.count, c.fix, B, Bp, M, N, 0.f, nullptr, y, pos};
    if (pos) rc = launch_rt<kRowsMax, 1, true, MASKED>(a, st);
    else rc = launch_rt<kRowsMax, 1, false, MASKED>(a, st);
    if (rc || !MASKED) return rc;
    const FixArgs f{x, w, xkeep, wkeep, c.count, c.fix, M, N, y, pos};
    if (pos) hipLaunchKernelGGL((rc_fix_kernel<true>), dim3(256), dim3(256), 0, st, f);
    else hipLaunchKernelGGL((rc_fix_kernel<false>), dim3(256), dim3(256), 0, st, f);
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
        case kRowsSortInterval: return K >= 2 && K <= 25;
        case kRowsSortPos: return K >= 2 && K <= 25;
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
    if (CI > 65536) {   // (16-bit input numbers in the lists of marks)
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
                SD_ROWS_K25(X)
#undef X
            }
            break;
        case kRowsSortPos:
            switch (K) {
#define X(k) case k: return run<kRowsSortPos, k>(xl, nullptr, w, B, CO, CI, q, outL, outU, pos, c, limit, col_stat, col_count, st);
                SD_ROWS_K25(X)
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
