// l-p norm distance at large p from per-row candidate tables (see lp_rows.h).
#include <cmath>
#include "lp_rows.h"

namespace sd {

namespace {

constexpr int kTileM = 256;               // output channels of a tile: 64 lanes x 4
constexpr int kChunk = kRowsChunk;        // inputs per table word
constexpr int WS = kChunk + 1;            // LDS row stride of the weight tile: lanes read one input of 64 rows
constexpr int XS = kChunk + 4;            // LDS row stride of the input tile (16-byte rows, broadcast reads)
// slack of the candidate test over the roundings of the test it stands in for
constexpr float kMargin = 1.f + 1.f / 1048576.f;

inline size_t align256(size_t b) { return (b + 255) / 256 * 256; }
inline int tiles_of(int M) { return (M + kTileM - 1) / kTileM; }
inline int bpad_of(int B) { return (B + 63) / 64 * 64; }

struct Carve {
    float* wabs;      // [T][N]      max |w| over the tile's output channels
    float* ymin;      // [T][Bpad]   min scale over the tile's output channels
    uint32_t* bits;   // [T][NCH][Bpad] candidate inputs, bit i of word (t, c, b) = input 32 c + i of row b
    unsigned long long* count;   // marks in the table
    uint32_t* partial;           // marks per wavefront of cand_bits_kernel
    float* extra;     // what follows
};

Carve carve(void* ws, int B, int M, int N) {
    const int T = tiles_of(M), Bp = bpad_of(B), NCH = N / kChunk;
    char* p = static_cast<char*>(ws);
    Carve c;
    c.wabs = reinterpret_cast<float*>(p); p += align256((size_t)T * N * 4);
    c.ymin = reinterpret_cast<float*>(p); p += align256((size_t)T * Bp * 4);
    c.bits = reinterpret_cast<uint32_t*>(p); p += align256((size_t)T * NCH * Bp * 4);
    c.count = reinterpret_cast<unsigned long long*>(p); p += 256;
    c.partial = reinterpret_cast<uint32_t*>(p); p += align256((size_t)NCH * (Bp / 64) * 4 * 4);
    c.extra = reinterpret_cast<float*>(p);
    return c;
}

// ---- candidate tables ------------------------------------------------------------------------
__global__ void __launch_bounds__(256) tile_wabs_kernel(const float* __restrict__ w, int M, int N,
                                                        float* __restrict__ wabs) {
    const int n = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
    if (n >= N) return;
    const int m0 = t * kTileM, m1 = m0 + kTileM < M ? m0 + kTileM : M;
    float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
    float odd = 0.f;   // stays 0 while every weight of the column is finite
    int m = m0;
    for (; m + 4 <= m1; m += 4) {
        const float a = w[(size_t)m * N + n], b = w[(size_t)(m + 1) * N + n];
        const float c = w[(size_t)(m + 2) * N + n], d = w[(size_t)(m + 3) * N + n];
        v0 = fmaxf(v0, fabsf(a)); v1 = fmaxf(v1, fabsf(b)); v2 = fmaxf(v2, fabsf(c)); v3 = fmaxf(v3, fabsf(d));
        odd += ((a - a) + (b - b)) + ((c - c) + (d - d));
    }
    for (; m < m1; m++) { const float a = w[(size_t)m * N + n]; v0 = fmaxf(v0, fabsf(a)); odd += a - a; }
    // an undefined weight must reach the outputs it belongs to: the column's bound becomes undefined, which
    // cand_bits_kernel takes for a candidate in every row
    wabs[(size_t)t * N + n] = fmaxf(fmaxf(v0, v1), fmaxf(v2, v3)) + odd;
}

// one wavefront per (row, tile): smallest scale of the tile's outputs; RECIP also writes 1 / v for every output
template <bool RECIP>
__global__ void __launch_bounds__(256) tile_rowmin_kernel(const float* __restrict__ v, int B, int M, int T, int Bp,
                                                          float* __restrict__ ymin, float* __restrict__ rv) {
    const int wave = (int)((blockIdx.x * 256u + threadIdx.x) >> 6), lane = threadIdx.x & 63;
    if (wave >= B * T) return;
    const int b = wave / T, t = wave - b * T;
    float r = __builtin_inff();
    float odd = 0.f;   // stays 0 while every scale of the tile is finite
    #pragma unroll
    for (int j = 0; j < kTileM / 64; j++) {
        const int m = t * kTileM + lane + 64 * j;
        if (m < M) {
            const float y = v[(size_t)b * M + m];
            r = fminf(r, y);
            odd += y - y;
            if (RECIP) rv[(size_t)b * M + m] = 1.f / y;
        }
    }
    #pragma unroll
    for (int o = 32; o; o >>= 1) { r = fminf(r, __shfl_xor(r, o)); odd += __shfl_xor(odd, o); }
    // an undefined or infinite scale makes the row's terms of the tile undefined: the bound becomes undefined, which
    // cand_bits_kernel takes for a candidate at every input
    if (lane == 0) ymin[(size_t)t * Bp + b] = r + odd;
}

// one wavefront per (row, tile): a lower bound of the largest |x[b,n] - w[m,n]| of every output channel m of the
// tile, max_n (|x[b,n]| - max_m |w[m,n]|), at least the 1e-10 floor of a distance
__global__ void __launch_bounds__(256) tile_rowlow_kernel(const float* __restrict__ x, const float* __restrict__ wabs,
                                                          int B, int N, int T, int Bp, float* __restrict__ low) {
    const int wave = (int)((blockIdx.x * 256u + threadIdx.x) >> 6), lane = threadIdx.x & 63;
    if (wave >= B * T) return;
    const int b = wave / T, t = wave - b * T;
    float r = kEps;
    for (int n = lane; n < N; n += 64) r = fmaxf(r, fabsf(x[(size_t)b * N + n]) - wabs[(size_t)t * N + n]);
    #pragma unroll
    for (int o = 32; o; o >>= 1) r = fmaxf(r, __shfl_xor(r, o));
    if (lane == 0) low[(size_t)t * Bp + b] = r;
}

// bit (t, b, n): some output channel m of tile t may have |x[b,n] - w[m,n]| > thr * scale[b,m].  A workgroup takes
// 64 rows x 32 inputs (one table word per row and tile): |x| goes through LDS so that a work-item can own a row
// and the words of 64 rows leave as one coalesced store; wavefront v handles the tiles v, v + 4, ...  Every
// wavefront leaves the number of its marks in partial[] for sum_marks_kernel.
__global__ void __launch_bounds__(256) cand_bits_kernel(const float* __restrict__ x, const float* __restrict__ wabs,
                                                        const float* __restrict__ ymin, float thr, int B, int Bp,
                                                        int N, int T, uint32_t* __restrict__ bits,
                                                        uint32_t* __restrict__ partial) {
    __shared__ float xs[64][kChunk + 1];
    const int c = blockIdx.x, b0 = blockIdx.y * 64, tid = threadIdx.x, NCH = N / kChunk;
    {
        const int row = tid >> 2, q = tid & 3, b = b0 + row;
        #pragma unroll
        for (int k = 0; k < 8; k++) xs[row][8 * q + k] = b < B ? fabsf(x[(size_t)b * N + c * kChunk + 8 * q + k]) : 0.f;
    }
    __syncthreads();
    const int r = tid & 63, b = b0 + r;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int marks = 0;
    for (int t = wave; t < T; t += 4) {
        // (an infinite bound - an infinite input - becomes undefined: every input of the row is a candidate, so the
        // outputs come out undefined as they do when every term is formed)
        const float s = ymin[(size_t)t * Bp + b];
        const float lim = b < B ? thr * ((s - s) + s) : __builtin_inff();
        const float* __restrict__ wa = wabs + (size_t)t * N + c * kChunk;
        uint32_t word = 0;
        #pragma unroll
        for (int n = 0; n < kChunk; n++) word |= (uint32_t)(!((xs[r][n] + wa[n]) * kMargin <= lim)) << n;   // undefined counts
        if (b >= B) word = 0u;
        bits[((size_t)t * NCH + c) * Bp + b] = word;
        marks += __builtin_popcount(word);
    }
    #pragma unroll
    for (int o = 32; o; o >>= 1) marks += __shfl_xor(marks, o);
    if ((tid & 63) == 0) partial[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 4 + wave] = (uint32_t)marks;
}

__global__ void __launch_bounds__(1024) sum_marks_kernel(const uint32_t* __restrict__ partial, size_t n,
                                                         unsigned long long* __restrict__ count) {
    __shared__ unsigned long long acc[1024];
    unsigned long long s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    size_t i = threadIdx.x;
    for (; i + 3072 < n; i += 4096) { s0 += partial[i]; s1 += partial[i + 1024]; s2 += partial[i + 2048]; s3 += partial[i + 3072]; }
    for (; i < n; i += 1024) s0 += partial[i];
    acc[threadIdx.x] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    for (int o = 512; o; o >>= 1) {
        if ((int)threadIdx.x < o) acc[threadIdx.x] += acc[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) *count = acc[0];
}

int build_tables(const Carve& c, const float* x, const float* w, const float* scale, float* recip, int B, int M,
                 int N, float thr, hipStream_t st) {
    const int T = tiles_of(M), Bp = bpad_of(B);
    hipLaunchKernelGGL(tile_wabs_kernel, dim3((N + 255) / 256, T), dim3(256), 0, st, w, M, N, c.wabs);
    int rc = check_launch("tile_wabs_kernel");
    if (rc) return rc;
    const unsigned waves = (unsigned)B * T;
    if (!scale) hipLaunchKernelGGL(tile_rowlow_kernel, dim3((waves + 3) / 4), dim3(256), 0, st, x, c.wabs, B, N, T, Bp, c.ymin);
    else if (recip) hipLaunchKernelGGL(tile_rowmin_kernel<true>, dim3((waves + 3) / 4), dim3(256), 0, st, scale, B, M, T, Bp, c.ymin, recip);
    else hipLaunchKernelGGL(tile_rowmin_kernel<false>, dim3((waves + 3) / 4), dim3(256), 0, st, scale, B, M, T, Bp, c.ymin, recip);
    if ((rc = check_launch("tile_rowmin_kernel"))) return rc;
    const int NCH = N / kChunk;
    hipLaunchKernelGGL(cand_bits_kernel, dim3(NCH, Bp / 64), dim3(256), 0, st, x, c.wabs, c.ymin, thr, B, Bp, N, T, c.bits, c.partial);
    if ((rc = check_launch("cand_bits_kernel"))) return rc;
    hipLaunchKernelGGL(sum_marks_kernel, dim3(1), dim3(1024), 0, st, c.partial, (size_t)NCH * (Bp / 64) * 4, c.count);
    return check_launch("sum_marks_kernel");
}

// ---- forward ------------------------------------------------------------------------------
// A workgroup of NW wavefronts owns 8 NW batch rows x 256 output channels and a slice of the inputs; wavefront v
// owns rows 8 v .. 8 v + 7, lane l the columns l + 64 j (j < 4): 32 sums and 32 reciprocal scales in registers.
// The inputs go by in chunks of 32: the weight tile (256 x 32) and the input tile (8 NW x 32) of the next-but-one
// chunk are in flight while the current one is used from LDS; a chunk that the table marks for none of the rows is
// not fetched.  Within a chunk the wavefront takes its rows one after the other and walks each row's own marks:
// the input of the row as an LDS broadcast, the four weights of the lane's columns, four terms.
// ONLINE: no maxima are given; every sum is kept relative to the largest term met so far and rescaled when a
// larger one comes (core/cuda/norm_dist_cuda.cu:36-160), with 1 / maximum in place of the given reciprocal scale.
// The slice results are (sum, maximum) pairs in part[slice] and part[nsplit + slice].
template <int NW, bool ONLINE>   // wavefronts per workgroup: 4 or 16
__global__ void __launch_bounds__(64 * NW, (NW == 4 ? 2 : 1))
lp_rows_fwd_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ maxv,
                   const uint32_t* __restrict__ bits, const unsigned long long* __restrict__ count,
                   unsigned long long limit, int B, int Bp, int M, int N, int nsplit, float p, float inv_p,
                   float* __restrict__ y, float* __restrict__ part) {
    constexpr int TB = 8, ROWS = TB * NW, NT = 64 * NW;   // rows per wavefront / workgroup, work-items
    constexpr int WV = kTileM * 8 / NT;                    // 16-byte pieces of the weight tile per work-item
    static_assert(ROWS <= 128 && ROWS * 8 == NT, "one 16-byte piece of the input tile per work-item");
    if (gate_closed(count, limit, 0)) return;
    __shared__ float wt[2][kTileM * WS];
    __shared__ float xt[2][ROWS * XS];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = (M + kTileM - 1) / kTileM, RT = (B + ROWS - 1) / ROWS;
    const int u = blockIdx.x / RT, t = u % T, split = u / T, r0 = (blockIdx.x % RT) * ROWS;
    const int m0 = t * kTileM, NCH = N / kChunk;
    const int per = (NCH + nsplit - 1) / nsplit;
    const int c_lo = split * per, c_hi = c_lo + per < NCH ? c_lo + per : NCH;

    float rinv[TB][4], acc[TB][4];
    #pragma unroll
    for (int r = 0; r < TB; r++) {
        #pragma unroll
        for (int j = 0; j < 4; j++) {
            const int row = r0 + wave * TB + r, col = m0 + lane + 64 * j;
            if (ONLINE) {
                // the virtual term of size 1e-10 (1 relative to a maximum of 1e-10) belongs to slice 0 only
                rinv[r][j] = 1.f / kEps;
                acc[r][j] = split == 0 ? 1.f : 0.f;
            } else {
                const float mv = (row < B && col < M) ? maxv[(size_t)row * M + col] : 1.f;
                rinv[r][j] = 1.f / mv;
                acc[r][j] = split == 0 ? __builtin_amdgcn_exp2f(p * __builtin_amdgcn_logf(kEps * rinv[r][j])) : 0.f;
            }
        }
    }

    // word of (chunk c, row r0 + i): bw[c * Bp + i]; rows past the batch, up to the padded count, hold zero words
    const uint32_t* __restrict__ bw = bits + (size_t)t * NCH * Bp + r0;
    const int rows_here = Bp - r0 < ROWS ? Bp - r0 : ROWS;
    // The words of up to SEG chunks are copied to LDS ahead of the loop over them (zero for rows past the padded
    // count), so that no global load sits between two chunks.
    constexpr int SEG = NW == 16 ? 64 : 32;
    __shared__ uint32_t wb[SEG * ROWS];
    int seg_lo = c_lo;
    auto marked = [&](int c) {   // anything marked in chunk c for the rows of the workgroup
        const uint32_t* q = wb + (c - seg_lo) * ROWS;
        uint32_t v = lane < ROWS ? q[lane < ROWS ? lane : 0] : 0u;
        if (ROWS > 64) v |= q[lane + 64];
        return __builtin_amdgcn_ballot_w64(v != 0u) != 0ull;
    };
    // always issued, so that the number of loads in flight is the same on every path (the waits the compiler places
    // in front of a stash then leave the younger fetch in flight); a chunk that nobody needs re-reads one hot line
    auto fetch = [&](int c, bool need, float4 (&wr)[WV], float4& xr) {
        const int n0 = c * kChunk;
        #pragma unroll
        for (int i = 0; i < WV; i++) {
            const int e = tid + NT * i, col = e >> 3, q = e & 7;
            const int m = m0 + col < M ? m0 + col : M - 1;
            wr[i] = *reinterpret_cast<const float4*>(need ? w + (size_t)m * N + n0 + 4 * q : w);
        }
        const int row = tid >> 3, q = tid & 7;
        const int rr = r0 + row < B ? r0 + row : B - 1;
        xr = *reinterpret_cast<const float4*>(need ? x + (size_t)rr * N + n0 + 4 * q : x);
    };
    auto stash = [&](int buf, const float4 (&wr)[WV], const float4& xr) {
        #pragma unroll
        for (int i = 0; i < WV; i++) {
            const int e = tid + NT * i, col = e >> 3, q = e & 7;
            float* d = &wt[buf][col * WS + 4 * q];
            d[0] = wr[i].x; d[1] = wr[i].y; d[2] = wr[i].z; d[3] = wr[i].w;
        }
        *reinterpret_cast<float4*>(&xt[buf][(tid >> 3) * XS + 4 * (tid & 7)]) = xr;
    };
    // The scalar unit is shared by the wavefronts of a compute unit, so the walk spends as few scalar instructions
    // per marked input as it can: one loop per row over that row's own marks (find-first-set, clear, branch).
    auto compute = [&](int buf, int c) {
        #pragma unroll
        for (int r = 0; r < TB; r++) {
            uint32_t bm = __builtin_amdgcn_readfirstlane(wb[(c - seg_lo) * ROWS + wave * TB + r]);
            while (bm) {
                const int n = __builtin_ctz(bm);
                bm &= bm - 1;
                const float xv = xt[buf][(wave * TB + r) * XS + n];
                // every term of a marked input is evaluated: on data that the table suits, most of them count
                #pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float d = fabsf(xv - wt[buf][(lane + 64 * j) * WS + n]);
                    const float lg = p * __builtin_amdgcn_logf(d * rinv[r][j]);
                    if (ONLINE) {
                        // ratio above 1: a new maximum; the old sum shrinks by ratio^-p and the new term is 1.
                        // The reciprocal need not be exact: the result is the sum's root divided by the same
                        // reciprocal, whatever it is; only the rescaling sees its error, p times, and the root
                        // takes that back.
                        const bool up = lg > 0.f;
                        const float e = __builtin_amdgcn_exp2f(up ? -lg : lg);
                        acc[r][j] = up ? fmaf(acc[r][j], e, 1.f) : acc[r][j] + e;
                        rinv[r][j] = up ? __builtin_amdgcn_rcpf(d) : rinv[r][j];
                    } else acc[r][j] += __builtin_amdgcn_exp2f(lg);
                }
            }
        }
    };

    // Two chunks are in flight: while chunk c is used from LDS, chunk c + 1 waits in registers and chunk c + 2 is
    // being fetched; a chunk's registers go to the LDS buffer that the chunk before the previous one has left.
    for (; seg_lo < c_hi; seg_lo += SEG) {
        const int seg_hi = seg_lo + SEG < c_hi ? seg_lo + SEG : c_hi;
        __syncthreads();   // the previous segment's words and tiles are no longer read
        for (int e = tid; e < (seg_hi - seg_lo) * ROWS; e += NT) {
            const int i = e % ROWS;
            wb[e] = i < rows_here ? bw[(size_t)(seg_lo + e / ROWS) * Bp + i] : 0u;
        }
        __syncthreads();
        float4 wa[WV], xa, wc[WV], xc;
        bool n0 = marked(seg_lo), n1 = seg_lo + 1 < seg_hi ? marked(seg_lo + 1) : false;
        fetch(seg_lo, n0, wa, xa);
        fetch(seg_lo + 1 < seg_hi ? seg_lo + 1 : seg_lo, n1, wc, xc);
        if (n0) stash(0, wa, xa);
        __syncthreads();
        for (int c = seg_lo; c < seg_hi; c += 2) {
            const bool n2 = c + 2 < seg_hi ? marked(c + 2) : false;
            fetch(c + 2 < seg_hi ? c + 2 : c, n2, wa, xa);
            if (n0) compute(0, c);
            if (n1) stash(1, wc, xc);
            __syncthreads();
            if (c + 1 >= seg_hi) break;
            const bool n3 = c + 3 < seg_hi ? marked(c + 3) : false;
            fetch(c + 3 < seg_hi ? c + 3 : c, n3, wc, xc);
            if (n1) compute(1, c + 1);
            if (n2) stash(0, wa, xa);
            __syncthreads();
            n0 = n2; n1 = n3;
        }
    }

    #pragma unroll
    for (int r = 0; r < TB; r++) {
        #pragma unroll
        for (int j = 0; j < 4; j++) {
            const int row = r0 + wave * TB + r, col = m0 + lane + 64 * j;
            if (row < B && col < M) {
                const size_t o = (size_t)row * M + col;
                if (ONLINE) {
                    const float mx = 1.f / rinv[r][j];
                    if (nsplit > 1) {
                        part[(size_t)split * B * M + o] = acc[r][j];
                        part[(size_t)(nsplit + split) * B * M + o] = mx;
                    } else y[o] = powf(acc[r][j], inv_p) * mx;
                } else if (nsplit > 1) part[(size_t)split * B * M + o] = acc[r][j];
                else y[o] = powf(acc[r][j], inv_p) * maxv[o];
            }
        }
    }
}

// ---- backward -----------------------------------------------------------------------------
// sum over the 64 lanes; the total is valid in lanes 0..15
template <int CTRL>
__device__ __forceinline__ float dpp_get(float a) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_get<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_get<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_get<0x141>(v);   // row_half_mirror
    v += dpp_get<0x140>(v);   // row_mirror: every lane holds the sum of its row of 16
    auto lane_of = [](float a, int l) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, a), l));
    };
    const float s1 = lane_of(v, 16), s2 = lane_of(v, 32), s3 = lane_of(v, 48);
    return ((v + s1) + s2) + s3;
}

// A workgroup owns 256 output channels and 32 inputs; its four wavefronts work on their own: wavefront v owns
// inputs n0 = 32 c + 8 v .. n0 + 7 for all 256 channels (lane l: columns l + 64 j), with those 32 weights and 32
// grad_weight sums in registers, and walks the batch rows that mark one of its inputs (byte v of the table words
// of chunk c).  The marked rows of a block of 512 are first collected into a list in LDS, so that the
// operands of the next row on the list (grad_output, 1 / y, eight inputs) are in flight while the current row is
// worked on.  Per marked input of a row: four terms per lane through the significance test, their sum over the
// wavefront added to grad_input with one atomic.  grad_weight needs no atomics: the wavefront sees every row.
template <bool WGRAD>
__global__ void __launch_bounds__(256, 2)
lp_rows_bwd_kernel(const float* __restrict__ gy, const float* __restrict__ x, const float* __restrict__ w,
                   const float* __restrict__ ry, const uint32_t* __restrict__ bits,
                   const unsigned long long* __restrict__ count, unsigned long long limit, int B, int Bp, int M, int N,
                   int groups, float pm1, float* __restrict__ gx, float* __restrict__ gw) {
    constexpr int kListRows = 512;
    if (gate_closed(count, limit, 0)) return;
    __shared__ uint32_t list[4][kListRows];   // row | byte << 24
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups go to the eight XCDs in turn.  The chunks of a column tile are cut in `groups` runs; all
    // workgroups of one (tile, run) unit are given to one XCD, next to each other in launch order, so that the
    // grad_output and 1 / y columns of the tile stay in that XCD's L2.
    const int NCH = N / kChunk, T = (M + kTileM - 1) / kTileM, cpu = (NCH + groups - 1) / groups;
    const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
    const int u = (jj / cpu) * 8 + xcd;
    const int t = u / groups, c = (u % groups) * cpu + jj % cpu;
    if (u >= T * groups || c >= NCH) return;
    const int m0 = t * kTileM, n0 = c * kChunk + 8 * wave;
    int col[4];
    bool colok[4];
    float wv[4][8], gwa[4][8];
    #pragma unroll
    for (int j = 0; j < 4; j++) {
        colok[j] = m0 + lane + 64 * j < M;
        col[j] = colok[j] ? m0 + lane + 64 * j : M - 1;
        const float4 a = *reinterpret_cast<const float4*>(w + (size_t)col[j] * N + n0);
        const float4 b = *reinterpret_cast<const float4*>(w + (size_t)col[j] * N + n0 + 4);
        wv[j][0] = a.x; wv[j][1] = a.y; wv[j][2] = a.z; wv[j][3] = a.w;
        wv[j][4] = b.x; wv[j][5] = b.y; wv[j][6] = b.z; wv[j][7] = b.w;
        #pragma unroll
        for (int k = 0; k < 8; k++) gwa[j][k] = 0.f;
    }
    const uint32_t* __restrict__ bw = bits + ((size_t)t * NCH + c) * Bp;

    struct RowOps { float g[4], r[4]; float4 x0, x1; uint32_t e; };
    auto load = [&](uint32_t e, RowOps& d) {
        const int row = (int)(e & 0xffffffu);
        d.e = e;
        #pragma unroll
        for (int j = 0; j < 4; j++) {
            const float gv = gy[(size_t)row * M + col[j]];
            d.g[j] = colok[j] ? gv : 0.f;
            d.r[j] = ry[(size_t)row * M + col[j]];
        }
        d.x0 = *reinterpret_cast<const float4*>(x + (size_t)row * N + n0);
        d.x1 = *reinterpret_cast<const float4*>(x + (size_t)row * N + n0 + 4);
    };
    auto work = [&](const RowOps& d) {
        const int row = (int)(d.e & 0xffffffu);
        const uint32_t rb = d.e >> 24;
        const float xv[8] = {d.x0.x, d.x0.y, d.x0.z, d.x0.w, d.x1.x, d.x1.y, d.x1.z, d.x1.w};
        #pragma unroll
        for (int k = 0; k < 8; k++) {
            if ((rb >> k) & 1u) {
                // every term of a marked input is evaluated: on data that the table suits, most of them count
                float sum = 0.f;
                #pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float sr = (xv[k] - wv[j][k]) * d.r[j];
                    const float pw = __builtin_amdgcn_exp2f(pm1 * __builtin_amdgcn_logf(fabsf(sr)));
                    const float u = d.g[j] * __builtin_copysignf(pw, sr);
                    if (WGRAD) gwa[j][k] += u;
                    sum += u;
                }
                sum = wave_sum(sum);
                if (lane == 0) unsafeAtomicAdd(gx + (size_t)row * N + n0 + k, sum);
            }
        }
    };

    for (int sb = 0; sb < Bp; sb += kListRows) {
        // marked rows of this block, in row order
        int cnt = 0;
        #pragma unroll 1
        for (int k = 0; k < kListRows && sb + k < Bp; k += 64) {
            const int row = sb + k + lane;   // Bp is a multiple of 64
            const uint32_t byte = (bw[row] >> (8 * wave)) & 0xffu;
            const unsigned long long mk = __builtin_amdgcn_ballot_w64(byte != 0u);
            const int before = __builtin_amdgcn_mbcnt_hi((uint32_t)(mk >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mk, 0u));
            if (byte != 0u) list[wave][cnt + before] = (uint32_t)row | (byte << 24);
            cnt += __builtin_popcountll(mk);
        }
        cnt = __builtin_amdgcn_readfirstlane(cnt);
        // the operands of the two rows after the current one are in flight; past the end of the list the last entry
        // is loaded again, so that the number of loads in flight is the same on every path
        if (cnt > 0) {
            auto entry = [&](int i) { return __builtin_amdgcn_readfirstlane(list[wave][i < cnt ? i : cnt - 1]); };
            RowOps a, b, d;
            load(entry(0), a);
            load(entry(1), b);
            for (int i = 0; i < cnt; i += 3) {
                load(entry(i + 2), d);
                work(a);
                load(entry(i + 3), a);
                if (i + 1 < cnt) work(b);
                load(entry(i + 4), b);
                if (i + 2 < cnt) work(d);
            }
        }
    }
    if (WGRAD) {
        #pragma unroll
        for (int j = 0; j < 4; j++) {
            if (colok[j]) {
                float* dst = gw + (size_t)col[j] * N + n0;
                *reinterpret_cast<float4*>(dst) = make_float4(-gwa[j][0], -gwa[j][1], -gwa[j][2], -gwa[j][3]);
                *reinterpret_cast<float4*>(dst + 4) = make_float4(-gwa[j][4], -gwa[j][5], -gwa[j][6], -gwa[j][7]);
            }
        }
    }
}

}  // namespace

size_t lp_rows_workspace(int B, int CO, int CI) {
    const int T = tiles_of(CO), Bp = bpad_of(B), NCH = CI / kChunk;
    return align256((size_t)T * CI * 4) + align256((size_t)T * Bp * 4) + align256((size_t)T * NCH * Bp * 4) + 256 +
           align256((size_t)NCH * (Bp / 64) * 4 * 4);
}

// rows per forward workgroup: 128 (16 wavefronts share a weight tile) unless the batch is small
static int fwd_rows(int B) { return B > 64 ? 128 : 32; }

int lp_rows_forward_nsplit(int B, int CO, int CI) {
    // one round of workgroups when the tiles alone do not fill the device, else no cut
    const int rows = fwd_rows(B);
    const long long wgs = (long long)tiles_of(CO) * ((B + rows - 1) / rows);
    const long long slots = (long long)num_cus() * (rows == 128 ? 1 : 2);
    int ns = (int)(slots / wgs);
    const int NCH = CI / kChunk;
    if (ns > NCH / 8) ns = NCH / 8;   // slices of at least 8 chunks
    if (ns > 16) ns = 16;
    return ns < 1 ? 1 : ns;
}

static unsigned long long mark_limit(int B, int CO, int CI, float density) {
    const double all = (double)tiles_of(CO) * B * CI;
    return (unsigned long long)(all * (density < 0.f ? 0.f : density > 1.f ? 1.f : density));
}

int lp_rows_forward(const float* x, const float* w, const float* maxv, int B, int CO, int CI, float p, float thr,
                    int nsplit, float* y, float* part, void* ws, float density,
                    const unsigned long long** gate, unsigned long long* gate_limit, hipStream_t st) {
    if (CI % kChunk != 0 || B < 1 || B >= (1 << 22) || CO < 1) { set_error("lp_rows_forward: shape not supported"); return SD_ERR_ARG; }
    const Carve c = carve(ws, B, CO, CI);
    int rc = build_tables(c, x, w, maxv, nullptr, B, CO, CI, thr, st);
    if (rc) return rc;
    *gate = c.count;
    *gate_limit = mark_limit(B, CO, CI, density);
    const int rows = fwd_rows(B), units = tiles_of(CO) * nsplit, RT = (B + rows - 1) / rows;
    dim3 grid((unsigned)(units * RT));
    const int Bp = bpad_of(B);
    const float ip = 1.f / p;
#define SD_ROWS_FWD(NW, ON) hipLaunchKernelGGL((lp_rows_fwd_kernel<NW, ON>), grid, dim3(64 * NW), 0, st, x, w, maxv, c.bits, \
                                               c.count, *gate_limit, B, Bp, CO, CI, nsplit, p, ip, y, part)
    if (rows == 128) { if (maxv) SD_ROWS_FWD(16, false); else SD_ROWS_FWD(16, true); }
    else { if (maxv) SD_ROWS_FWD(4, false); else SD_ROWS_FWD(4, true); }
#undef SD_ROWS_FWD
    return check_launch("lp_rows_fwd_kernel");
}

int lp_rows_backward(const float* gy, const float* x, const float* w, const float* y, int B, int CO, int CI,
                     float pm1, float thr, float* gx, float* gw, void* ws, float density, const float** recip,
                     const unsigned long long** gate, unsigned long long* gate_limit, hipStream_t st) {
    if (CI % kChunk != 0 || B < 1 || B >= (1 << 22) || CO < 1) { set_error("lp_rows_backward: shape not supported"); return SD_ERR_ARG; }
    const Carve c = carve(ws, B, CO, CI);
    float* ry = c.extra;
    int rc = build_tables(c, x, w, y, ry, B, CO, CI, thr, st);
    if (rc) return rc;
    if ((rc = fill_zero(gx, (size_t)B * CI, st))) return rc;
    *recip = ry;
    *gate = c.count;
    *gate_limit = mark_limit(B, CO, CI, density);
    const int T = tiles_of(CO), NCH = CI / kChunk;
    int groups = 1;
    while (groups < 8 && (T * groups) % 8 != 0 && NCH / (2 * groups) >= 8) groups *= 2;
    const int cpu = (NCH + groups - 1) / groups;
    dim3 grid((unsigned)(8 * ((T * groups + 7) / 8) * cpu));
    if (gw) hipLaunchKernelGGL((lp_rows_bwd_kernel<true>), grid, dim3(256), 0, st, gy, x, w, ry, c.bits, c.count, *gate_limit, B, bpad_of(B), CO, CI, groups, pm1, gx, gw);
    else hipLaunchKernelGGL((lp_rows_bwd_kernel<false>), grid, dim3(256), 0, st, gy, x, w, ry, c.bits, c.count, *gate_limit, B, bpad_of(B), CO, CI, groups, pm1, gx, gw);
    return check_launch("lp_rows_bwd_kernel");
}

}  // namespace sd
