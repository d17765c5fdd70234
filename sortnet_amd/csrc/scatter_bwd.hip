// Backward of the arg-max style ops (l-inf, sort neuron, interval bounds): every output sends its
// upstream gradient to the saved input position(s) of grad_input and grad_weight
// (core/cuda/inf_dist_cuda.cu:214-271, sort_neuron.cu:316-375, bound_inf_dist_cuda.cu:240-299).
// Dense layers accumulate both gradients in LDS row histograms and write every row once; index lists and
// very long rows fall back to a zero-fill pass and hardware fp32 atomic adds on device memory.
#include <cmath>
#include "common.h"

namespace sd {

struct BwdArgs {
    const float* g0; const float* g1;    // upstream gradient (lower / upper for the interval op)
    const int* p0; const int* p1;        // saved positions
    float* gx0; float* gx1; float* gw;   // gw may be null
    const int* ci_idx; const int* co_idx;
    int B, HW, G, COg, CIg, W_COg, W_CIg;
    int K;                               // slots per output (1 for l-inf)
    float q, coef0;                      // sort neuron: first coefficient 1/(1-(1-q)^K) and ratio
    long long total;                     // B * CO * HW
};

// l-inf (K = 1, unit coefficient) and sort neuron (K slots, geometric coefficients)
template <bool SORT, bool HAS_W>
__global__ void __launch_bounds__(256) scatter_bwd_kernel(BwdArgs a) {
    long long o = (long long)blockIdx.x * 256 + threadIdx.x;
    if (o >= a.total) return;
    int hw = (int)(o % a.HW);
    long long t = o / a.HW;
    int c = (int)(t % (a.G * a.COg));
    int b = (int)(t / (a.G * a.COg));
    int g = c / a.COg, m = c - g * a.COg;
    int s = b / kSubBatch;
    float grad = a.g0[o];
    float coef = a.coef0;
    size_t xbase = ((size_t)(b * a.G + g) * a.CIg) * a.HW + hw;
    size_t wrow = 0;
    if (HAS_W) {
        int mm = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
        wrow = (size_t)(g * a.W_COg + mm) * a.W_CIg;
    }
    const int K = SORT ? a.K : 1;
    for (int k = 0; k < K; k++) {
        int pr = a.p0[(size_t)k * a.total + o];
        int n = pr & 0x7fffffff;
        float v = pr >= 0 ? grad : -grad;
        if (SORT) { v = v * coef * a.q; coef *= 1.f - a.q; }
        unsafeAtomicAdd(a.gx0 + xbase + (size_t)n * a.HW, v);
        if (HAS_W) {
            int nn = a.ci_idx ? a.ci_idx[(s * a.G + g) * a.CIg + n] : n;
            unsafeAtomicAdd(a.gw + wrow + nn, -v);
        }
    }
}

template <bool HAS_W>
__global__ void __launch_bounds__(256) bound_bwd_kernel(BwdArgs a) {
    long long o = (long long)blockIdx.x * 256 + threadIdx.x;
    if (o >= a.total) return;
    int hw = (int)(o % a.HW);
    long long t = o / a.HW;
    int c = (int)(t % (a.G * a.COg));
    int b = (int)(t / (a.G * a.COg));
    int g = c / a.COg;
    size_t xbase = ((size_t)(b * a.G + g) * a.CIg) * a.HW + hw;
    size_t wrow = (size_t)c * a.CIg;
    int pl = a.p0[o], pu = a.p1[o];
    float gl = a.g0[o], gu = a.g1[o];
    int nl = pl & 0x7fffffff, nu = pu & 0x7fffffff;
    float vl = pl >= 0 ? gl : -gl, vu = pu >= 0 ? gu : -gu;
    if ((uint32_t)pl != kNanId) {
        unsafeAtomicAdd((pl >= 0 ? a.gx0 : a.gx1) + xbase + (size_t)nl * a.HW, vl);
        if (HAS_W) unsafeAtomicAdd(a.gw + wrow + nl, -vl);
    }
    unsafeAtomicAdd((pu >= 0 ? a.gx1 : a.gx0) + xbase + (size_t)nu * a.HW, vu);
    if (HAS_W) unsafeAtomicAdd(a.gw + wrow + nu, -vu);
}

// Row-histogram variants: one workgroup owns one (sample, group, position) row of grad_input,
// accumulates it in LDS (colliding adds stay on chip) and writes it out once, so grad_input needs
// neither a zero-fill pass nor global atomics.  grad_weight is still scattered with atomics.
constexpr int kMaxRowLds = 12288;   // floats of LDS one row histogram may take

template <bool SORT, bool HAS_W>
__global__ void __launch_bounds__(1024) scatter_bwd_rows_kernel(BwdArgs a) {
    extern __shared__ float hist[];
    const int row = blockIdx.x;                 // ((b * G) + g) * HW + hw
    const int hw = row % a.HW;
    const int bg = row / a.HW;
    const int g = bg % a.G, b = bg / a.G;
    const int s = b / kSubBatch;
    for (int n = threadIdx.x; n < a.CIg; n += blockDim.x) hist[n] = 0.f;
    __syncthreads();
    const size_t obase = ((size_t)(b * a.G + g) * a.COg) * a.HW + hw;
    const int K = SORT ? a.K : 1;
    for (int m = threadIdx.x; m < a.COg; m += blockDim.x) {
        size_t o = obase + (size_t)m * a.HW;
        float grad = a.g0[o];
        float coef = a.coef0;
        size_t wrow = 0;
        if (HAS_W) {
            int mm = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
            wrow = (size_t)(g * a.W_COg + mm) * a.W_CIg;
        }
        for (int k = 0; k < K; k++) {
            int pr = a.p0[(size_t)k * a.total + o];
            int n = pr & 0x7fffffff;
            float v = pr >= 0 ? grad : -grad;
            if (SORT) { v = v * coef * a.q; coef *= 1.f - a.q; }
            atomicAdd(&hist[n], v);
            if (HAS_W) {
                int nn = a.ci_idx ? a.ci_idx[(s * a.G + g) * a.CIg + n] : n;
                unsafeAtomicAdd(a.gw + wrow + nn, -v);
            }
        }
    }
    __syncthreads();
    const size_t xbase = ((size_t)(b * a.G + g) * a.CIg) * a.HW + hw;
    for (int n = threadIdx.x; n < a.CIg; n += blockDim.x) a.gx0[xbase + (size_t)n * a.HW] = hist[n];
}

template <bool HAS_W>
__global__ void __launch_bounds__(256) bound_bwd_rows_kernel(BwdArgs a) {
    extern __shared__ float hist[];             // [0, CIg) lower, [CIg, 2 CIg) upper
    const int row = blockIdx.x;
    const int hw = row % a.HW;
    const int bg = row / a.HW;
    const int g = bg % a.G, b = bg / a.G;
    for (int n = threadIdx.x; n < 2 * a.CIg; n += 256) hist[n] = 0.f;
    __syncthreads();
    const size_t obase = ((size_t)(b * a.G + g) * a.COg) * a.HW + hw;
    for (int m = threadIdx.x; m < a.COg; m += 256) {
        size_t o = obase + (size_t)m * a.HW;
        size_t wrow = (size_t)(g * a.COg + m) * a.CIg;
        int pl = a.p0[o], pu = a.p1[o];
        float gl = a.g0[o], gu = a.g1[o];
        int nl = pl & 0x7fffffff, nu = pu & 0x7fffffff;
        float vl = pl >= 0 ? gl : -gl, vu = pu >= 0 ? gu : -gu;
        if ((uint32_t)pl != kNanId) {
            atomicAdd(&hist[(pl >= 0 ? 0 : a.CIg) + nl], vl);
            if (HAS_W) unsafeAtomicAdd(a.gw + wrow + nl, -vl);
        }
        atomicAdd(&hist[(pu >= 0 ? a.CIg : 0) + nu], vu);
        if (HAS_W) unsafeAtomicAdd(a.gw + wrow + nu, -vu);
    }
    __syncthreads();
    const size_t xbase = ((size_t)(b * a.G + g) * a.CIg) * a.HW + hw;
    for (int n = threadIdx.x; n < a.CIg; n += 256) {
        a.gx0[xbase + (size_t)n * a.HW] = hist[n];
        a.gx1[xbase + (size_t)n * a.HW] = hist[a.CIg + n];
    }
}

// grad_weight by rows (dense layers, no index lists): one workgroup owns WR consecutive weight rows,
// accumulates in LDS whatever any (sample, position, slot) sends into them and writes the rows out once, so
// grad_weight needs neither a zero-fill pass nor global atomics.  Work-item = (row j = tid % WR, batch rows
// tid / WR + i * 256 / WR): the WR positions of one batch row are adjacent in memory when HW == 1.
// MODE 0: l-inf, 1: sort neuron (K slots, geometric coefficients), 2: interval bounds (two positions).
// A workgroup reads WR adjacent entries of every row of pos and grad_output, so one 64-byte piece of those rows is
// shared by 16 / WR workgroups.  Workgroups go to the chip's eight dies in turn, each
// with a cache of its own: eight consecutive row blocks are given to one die, next to each other in launch order, so
// that a piece is fetched from memory by one die, once, instead of by all eight.
constexpr int kMaxWRowsLds = 15360;   // floats of LDS the weight-row histograms of one workgroup may take

template <int MODE>
__global__ void __launch_bounds__(256) wrows_bwd_kernel(BwdArgs a, int WR) {
    extern __shared__ float hist[];             // [WR][CIg]
    const int CO = a.G * a.COg;
    const int die = blockIdx.x & 7, k = blockIdx.x >> 3;
    const int c0 = ((((k >> 3) * 8 + die) << 3) + (k & 7)) * WR;
    if (c0 >= CO) return;                       // the grid is rounded up to 64 row blocks
    const int nrows = CO - c0 < WR ? CO - c0 : WR;
    for (int n = threadIdx.x; n < WR * a.CIg; n += 256) hist[n] = 0.f;
    __syncthreads();
    const int j = threadIdx.x % WR, rstep = 256 / WR;
    const int R = a.B * a.HW;
    if (j < nrows) {
        float* h = hist + (size_t)j * a.CIg;
        for (int r = threadIdx.x / WR; r < R; r += rstep) {
            int b = r, hw = 0;
            if (a.HW > 1) { b = r / a.HW; hw = r - b * a.HW; }
            const size_t o = ((size_t)b * CO + c0 + j) * a.HW + hw;
            if (MODE == 2) {
                int pl = a.p0[o], pu = a.p1[o];
                float gl = a.g0[o], gu = a.g1[o];
                if ((uint32_t)pl != kNanId) atomicAdd(&h[pl & 0x7fffffff], pl >= 0 ? -gl : gl);
                atomicAdd(&h[pu & 0x7fffffff], pu >= 0 ? -gu : gu);
            } else {
                const float grad = a.g0[o];
                float coef = a.coef0;
                const int K = MODE == 1 ? a.K : 1;
                for (int k = 0; k < K; k++) {
                    int pr = a.p0[(size_t)k * a.total + o];
                    float v = pr >= 0 ? grad : -grad;
                    if (MODE == 1) { v = v * coef * a.q; coef *= 1.f - a.q; }
                    atomicAdd(&h[pr & 0x7fffffff], -v);
                }
            }
        }
    }
    __syncthreads();
    float* out = a.gw + (size_t)c0 * a.CIg;
    for (int n = threadIdx.x; n < nrows * a.CIg; n += 256) out[n] = hist[n];
}

// The same for the l-inf layer with index lists (core/cuda/inf_dist_cuda.cu:214-275 scatters with global atomics into a
// zero-filled grad_weight).  A weight row r receives from sub-batch s only when r is in that sub-batch's list of kept
// outputs, from the output at r's place in the list: row_place_kernel writes the place of every weight row per
// (sub-batch, group), -1 for rows not kept, so that a workgroup can again own WR weight rows, collect them in LDS over
// all samples (the position is a place in the sub-batch's list of kept inputs, whose entry is the column) and write
// them out once, rows nobody kept as zeros.
__global__ void __launch_bounds__(256) row_place_kernel(const int* __restrict__ co_idx, int COg, int W_COg,
                                                        int* __restrict__ place) {
    const int sg = blockIdx.x;                      // sub-batch * G + group
    int* p = place + (size_t)sg * W_COg;
    for (int r = threadIdx.x; r < W_COg; r += 256) p[r] = -1;
    __syncthreads();                                // the fills of this workgroup are ordered before its entries
    for (int m = threadIdx.x; m < COg; m += 256) {
        const int r = co_idx[(size_t)sg * COg + m];
        if (r >= 0 && r < W_COg) p[r] = m;
    }
}

__global__ void __launch_bounds__(256) wrows_lists_bwd_kernel(BwdArgs a, int WR, const int* __restrict__ place) {
    extern __shared__ float hist[];             // [WR][W_CIg]
    const int rows_total = a.G * a.W_COg;
    const int die = blockIdx.x & 7, k = blockIdx.x >> 3;
    const int c0 = ((((k >> 3) * 8 + die) << 3) + (k & 7)) * WR;      // as in wrows_bwd_kernel
    if (c0 >= rows_total) return;
    const int nrows = rows_total - c0 < WR ? rows_total - c0 : WR;
    for (int n = threadIdx.x; n < WR * a.W_CIg; n += 256) hist[n] = 0.f;
    __syncthreads();
    const int j = threadIdx.x % WR, rstep = 256 / WR;
    const int R = a.B * a.HW;
    if (j < nrows) {
        const int g = (c0 + j) / a.W_COg, rr = (c0 + j) - g * a.W_COg;
        float* h = hist + (size_t)j * a.W_CIg;
        for (int r = threadIdx.x / WR; r < R; r += rstep) {
            int b = r, hw = 0;
            if (a.HW > 1) { b = r / a.HW; hw = r - b * a.HW; }
            const int sg = (b / kSubBatch) * a.G + g;
            const int m = place ? place[(size_t)sg * a.W_COg + rr] : rr;
            if (m < 0) continue;
            const size_t o = ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw;
            const float grad = a.g0[o];
            const int pr = a.p0[o];
            const int n = pr & 0x7fffffff;
            if (n >= a.CIg) continue;                // a position outside the list: not followed into LDS
            const int col = a.ci_idx ? a.ci_idx[(size_t)sg * a.CIg + n] : n;
            if ((unsigned)col < (unsigned)a.W_CIg) atomicAdd(&h[col], pr >= 0 ? -grad : grad);
        }
    }
    __syncthreads();
    float* out = a.gw + (size_t)c0 * a.W_CIg;
    for (int n = threadIdx.x; n < nrows * a.W_CIg; n += 256) out[n] = hist[n];
}

// launches wrows_bwd_kernel when the layer is dense and a row fits; returns false when the caller has to
// take the zero-fill + atomics path for grad_weight
template <int MODE>
static bool launch_wrows(const BwdArgs& a, hipStream_t st) {
    if ((a.ci_idx || a.co_idx) && MODE == 0 && a.W_CIg <= kMaxWRowsLds) {
        int* place = nullptr;
        if (a.co_idx) {
            const int SG = (a.B + kSubBatch - 1) / kSubBatch * a.G;
            place = static_cast<int*>(workspace((size_t)SG * a.W_COg * sizeof(int), st));   // the only request of the call
            if (!place) return false;
            hipLaunchKernelGGL(row_place_kernel, dim3((unsigned)SG), dim3(256), 0, st, a.co_idx, a.COg, a.W_COg, place);
        }
        int WR = 1;
        while (WR < 8 && 2 * WR * a.W_CIg <= kMaxWRowsLds) WR *= 2;
        const int blocks = (a.G * a.W_COg + WR - 1) / WR;
        hipLaunchKernelGGL(wrows_lists_bwd_kernel, dim3((unsigned)((blocks + 63) / 64 * 64)), dim3(256),
                           (size_t)WR * a.W_CIg * sizeof(float), st, a, WR, place);
        return true;
    }
    if (a.ci_idx || a.co_idx || a.CIg > kMaxWRowsLds) return false;
    int WR = 1;
    while (WR < 8 && 2 * WR * a.CIg <= kMaxWRowsLds) WR *= 2;
    const int CO = a.G * a.COg;
    const int blocks = (CO + WR - 1) / WR;
    hipLaunchKernelGGL((wrows_bwd_kernel<MODE>), dim3((unsigned)((blocks + 63) / 64 * 64)), dim3(256),
                       (size_t)WR * a.CIg * sizeof(float), st, a, WR);
    return true;
}

static int make_bwd_args(BwdArgs& a, const char* who, int B, int CO, int CI, int G, int HW,
                         const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    SD_REQUIRE(B > 0 && CO > 0 && CI > 0 && G > 0 && HW > 0, "%s: sizes must be positive", who);
    SD_REQUIRE(CO % G == 0 && CI % G == 0, "%s: CO=%d and CI=%d must be multiples of G=%d", who, CO, CI, G);
    SD_REQUIRE((long long)B * CO * HW < (1ll << 31) && (long long)B * CI * HW < (1ll << 31),
               "%s: tensor too large for 32-bit indexing", who);
    a = BwdArgs{};
    a.B = B; a.HW = HW; a.G = G; a.COg = CO / G; a.CIg = CI / G;
    a.ci_idx = ci_idx; a.co_idx = co_idx;
    if (co_idx) { SD_REQUIRE(W_CO > 0 && W_CO % G == 0, "%s: bad W_CO=%d", who, W_CO); a.W_COg = W_CO / G; }
    else a.W_COg = a.COg;
    if (ci_idx) { SD_REQUIRE(W_CI > 0 && W_CI % G == 0, "%s: bad W_CI=%d", who, W_CI); a.W_CIg = W_CI / G; }
    else a.W_CIg = a.CIg;
    a.K = 1; a.q = 1.f; a.coef0 = 1.f;
    a.total = (long long)B * CO * HW;
    return SD_OK;
}

template <bool SORT>
static int run_scatter(BwdArgs& a, hipStream_t st) {
    int rc;
    float* gw_atomic = a.gw;      // grad_weight target of the atomics path, null once the row kernel has taken it
    if (a.gw && launch_wrows<SORT ? 1 : 0>(a, st)) {
        if ((rc = check_launch("wrows_bwd_kernel"))) return rc;
        gw_atomic = nullptr;
    }
    if (gw_atomic && (rc = fill_zero(gw_atomic, (size_t)a.G * a.W_COg * a.W_CIg, st))) return rc;
    BwdArgs x = a;
    x.gw = gw_atomic;
    if (a.CIg <= kMaxRowLds) {
        dim3 rows((unsigned)(a.B * a.G * a.HW));
        size_t lds = (size_t)a.CIg * sizeof(float);
        // few rows: more work-items per row, so that enough position / index loads are in flight
        const dim3 block(rows.x < 4u * (unsigned)num_cus() ? 1024 : 256);
        if (x.gw) hipLaunchKernelGGL((scatter_bwd_rows_kernel<SORT, true>), rows, block, lds, st, x);
        else hipLaunchKernelGGL((scatter_bwd_rows_kernel<SORT, false>), rows, block, lds, st, x);
        return check_launch("scatter_bwd_rows_kernel");
    }
    if ((rc = fill_zero(a.gx0, (size_t)a.B * a.G * a.CIg * a.HW, st))) return rc;
    dim3 grid((unsigned)((a.total + 255) / 256));
    if (x.gw) hipLaunchKernelGGL((scatter_bwd_kernel<SORT, true>), grid, dim3(256), 0, st, x);
    else hipLaunchKernelGGL((scatter_bwd_kernel<SORT, false>), grid, dim3(256), 0, st, x);
    return check_launch("scatter_bwd_kernel");
}

}  // namespace sd

using namespace sd;

extern "C" int sd_inf_dist_backward_input(const float* grad_output, const int* pos,
                                          int B, int CO, int CI, int G, int HW, float* grad_input, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    BwdArgs a;
    int rc = make_bwd_args(a, "inf_dist_backward_input", B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(grad_output && pos && grad_input, "inf_dist_backward_input: null pointer");
    a.g0 = grad_output; a.p0 = pos; a.gx0 = grad_input;
    return run_scatter<false>(a, static_cast<hipStream_t>(stream));
}

extern "C" int sd_inf_dist_backward_input_weight(const float* grad_output, const int* pos,
                                                 int B, int CO, int CI, int G, int HW, float* grad_input,
                                                 float* grad_weight, const int* w_index_ci, const int* w_index_co,
                                                 int W_CO, int W_CI, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    BwdArgs a;
    int rc = make_bwd_args(a, "inf_dist_backward_input_weight", B, CO, CI, G, HW, w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(grad_output && pos && grad_input && grad_weight, "inf_dist_backward_input_weight: null pointer");
    a.g0 = grad_output; a.p0 = pos; a.gx0 = grad_input; a.gw = grad_weight;
    return run_scatter<false>(a, static_cast<hipStream_t>(stream));
}

static int sort_bwd(const char* who, const float* grad_output, const int* pos, int B, int CO, int CI, int G, int HW,
                    float* grad_input, float* grad_weight, float q, int K, sd_stream_t stream) {
    BwdArgs a;
    int rc = make_bwd_args(a, who, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(grad_output && pos && grad_input, "%s: null pointer", who);
    SD_REQUIRE(K >= 1 && K <= 25, "%s: K=%d outside 1..25", who, K);
    SD_REQUIRE(q > 0.f && q <= 1.f, "%s: q=%g outside (0, 1]", who, (double)q);
    a.g0 = grad_output; a.p0 = pos; a.gx0 = grad_input; a.gw = grad_weight;
    a.K = K; a.q = q;
    float r = powf(1.f - q, (float)K);          // core/cuda/sort_neuron.cu:322
    a.coef0 = 1.f + r / (1.f - r);
    return run_scatter<true>(a, static_cast<hipStream_t>(stream));
}

extern "C" int sd_sort_neuron_backward_input(const float* grad_output, const int* pos,
                                             int B, int CO, int CI, int G, int HW, float* grad_input,
                                             float q, int K, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    return sort_bwd("sort_neuron_backward_input", grad_output, pos, B, CO, CI, G, HW, grad_input, nullptr, q, K, stream);
}

extern "C" int sd_sort_neuron_backward_input_weight(const float* grad_output, const int* pos,
                                                    int B, int CO, int CI, int G, int HW, float* grad_input,
                                                    float* grad_weight, float q, int K, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    SD_REQUIRE(grad_weight, "sort_neuron_backward_input_weight: null grad_weight");
    return sort_bwd("sort_neuron_backward_input_weight", grad_output, pos, B, CO, CI, G, HW, grad_input, grad_weight,
                    q, K, stream);
}

static int bound_bwd(const char* who, const float* gL, const float* gU, const int* posL, const int* posU,
                     int B, int CO, int CI, int G, int HW, float* gxL, float* gxU, float* gw, sd_stream_t stream) {
    BwdArgs a;
    int rc = make_bwd_args(a, who, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(gL && gU && posL && posU && gxL && gxU, "%s: null pointer", who);
    a.g0 = gL; a.g1 = gU; a.p0 = posL; a.p1 = posU; a.gx0 = gxL; a.gx1 = gxU; a.gw = gw;
    hipStream_t st = static_cast<hipStream_t>(stream);
    size_t nx = (size_t)B * CI * HW;
    if (gw && launch_wrows<2>(a, st)) {
        if ((rc = check_launch("wrows_bwd_kernel"))) return rc;
        a.gw = gw = nullptr;
    }
    if (gw && (rc = fill_zero(gw, (size_t)CO * a.CIg, st))) return rc;
    if (2 * a.CIg <= kMaxRowLds) {
        dim3 rows((unsigned)(B * G * HW));
        size_t lds = (size_t)2 * a.CIg * sizeof(float);
        if (gw) hipLaunchKernelGGL((bound_bwd_rows_kernel<true>), rows, dim3(256), lds, st, a);
        else hipLaunchKernelGGL((bound_bwd_rows_kernel<false>), rows, dim3(256), lds, st, a);
        return check_launch("bound_bwd_rows_kernel");
    }
    if ((rc = fill_zero(gxL, nx, st))) return rc;
    if ((rc = fill_zero(gxU, nx, st))) return rc;
    dim3 grid((unsigned)((a.total + 255) / 256));
    if (gw) hipLaunchKernelGGL((bound_bwd_kernel<true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((bound_bwd_kernel<false>), grid, dim3(256), 0, st, a);
    return check_launch("bound_bwd_kernel");
}

extern "C" int sd_bound_inf_dist_backward_input(const float* grad_outputL, const float* grad_outputU,
                                                const int* posL, const int* posU, int B, int CO, int CI, int G, int HW,
                                                float* grad_inputL, float* grad_inputU, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    return bound_bwd("bound_inf_dist_backward_input", grad_outputL, grad_outputU, posL, posU, B, CO, CI, G, HW,
                     grad_inputL, grad_inputU, nullptr, stream);
}

extern "C" int sd_bound_inf_dist_backward_input_weight(const float* grad_outputL, const float* grad_outputU,
                                                       const int* posL, const int* posU, int B, int CO, int CI, int G,
                                                       int HW, float* grad_inputL, float* grad_inputU,
                                                       float* grad_weight, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    SD_REQUIRE(grad_weight, "bound_inf_dist_backward_input_weight: null grad_weight");
    return bound_bwd("bound_inf_dist_backward_input_weight", grad_outputL, grad_outputU, posL, posU, B, CO, CI, G, HW,
                     grad_inputL, grad_inputU, grad_weight, stream);
}
