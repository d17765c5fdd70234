// l-p norm distance: forward entry points and the fused backward kernel.
#include <atomic>
#include <cstdlib>
#include "fwd_tile.h"
#include "fwd_args.h"
#include "lp_rows.h"

namespace sd {

// integral 0 <= p <= 8 selects a multiply chain, anything else the transcendental path
// (core/cuda/norm_dist.cpp:17-38)
// smallest thresholds from which the significance tests paid at B = 512, M = N = 5120 (p of about 32 for the
// vector-load forward, about 77 for the two-pass forward of the index lists)
constexpr float kLpSkipFrom = 0.5f, kLpSkipFromOnline = 0.75f;
// backward: the dense both-gradient kernel (p of about 65) and the general kernel (p of about 80)
constexpr float kLpSkipFromFused = 0.68f, kLpSkipFromGeneral = 0.73f;

// largest share of marked (tile, row, input) triples at which the candidate-table kernels run instead of the
// kernels that evaluate every term (sd_set_lp_candidate_density); negative: the built-in limits below
static std::atomic<float> g_rows_density{-1.f};
// Measured at B = 512, M = N = 5120 on three kinds of data (normal or uniform inputs against small weights,
// normal inputs against weights of the same size), in ms against the marked share d:
//   forward   table kernel 0.2 + 3.6 d    every term 2.8, with wave-level significance tests 1.3 .. 3.6
//   backward  both gradients 0.13 + 6 d   every term 3.5, with tests 2.8 .. 4.8
//             grad_input only 0.09 + 5 d  every term 3.15, with tests 1.45 .. 4.3
// The limits sit near where the table kernel meets the fastest case of the kernel it replaces: a little above it
// where that kernel's slow cases are far slower than its fast ones.
constexpr float kRowsCapForward = 0.55f, kRowsCapForwardSkip = 0.3f;
constexpr float kRowsCapBackward = 0.5f, kRowsCapBackwardSkip = 0.4f;
constexpr float kRowsCapBackwardInput = 0.55f, kRowsCapBackwardInputSkip = 0.3f;
// below this threshold (p of about 12 forward, 20 backward) most inputs are marked on all three
constexpr float kRowsFromThr = 0.15f;
static inline float rows_cap(float builtin, float thr) {
    const float density = g_rows_density.load(std::memory_order_relaxed);
    if (density >= 0.f) return density;
    return thr >= kRowsFromThr ? builtin : 0.f;
}

static inline int int_power(float p) {
    if (p == (float)(int)p && p >= 0.f && p <= 8.f) return (int)p;
    return -1;
}

// ratio below which a term of r^p is dropped (see lp_add_significant); 0 when it is below `from`, i.e. when too
// many terms would pass for the wavefront-level tests to pay
static inline float lp_skip_threshold(float drop, float p, float from) {
    // the test only makes sense for an exponent above 1: then 0 < thr < 1 and ratios below it are small.  For
    // an exponent of at most 1 (backward with p <= 2) drop^(1/p) is no threshold at all (it exceeds 1 for
    // negative exponents) and every term is evaluated.
    if (!(p > 1.f)) return 0.f;
    const float thr = powf(drop, 1.f / p);
    return (thr >= from && thr < 1.f) ? thr : 0.f;
}

template <template <int> class Pol, int TB, int TM>
static int launch_lp(int ip, const FwdArgs& a, hipStream_t st) {
    switch (ip) {
        case 1: return launch_fwd<Pol<1>, TB, TM>(a, st);
        case 2: return launch_fwd<Pol<2>, TB, TM>(a, st);
        case 3: return launch_fwd<Pol<3>, TB, TM>(a, st);
        case 4: return launch_fwd<Pol<4>, TB, TM>(a, st);
        case 5: return launch_fwd<Pol<5>, TB, TM>(a, st);
        case 6: return launch_fwd<Pol<6>, TB, TM>(a, st);
        case 7: return launch_fwd<Pol<7>, TB, TM>(a, st);
        case 8: return launch_fwd<Pol<8>, TB, TM>(a, st);
        default: return launch_fwd<Pol<-1>, TB, TM>(a, st);
    }
}

// merges the split-N slices of the l-p forward in slice order (deterministic) and takes the root:
// plain sums, sums relative to a known maximum (scale), or (sum, running maximum) pairs of the online form
__global__ void __launch_bounds__(256) lp_finalize_kernel(const float* __restrict__ part0, const float* __restrict__ part1,
                                                          const float* __restrict__ scale,
                                                          int nsplit, size_t total, float p, float inv_p,
                                                          float* __restrict__ y, const unsigned long long* gate,
                                                          unsigned long long gate_limit, int gate_above) {
    size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= total || gate_closed(gate, gate_limit, gate_above)) return;
    if (part1 == nullptr) {
        float s = 0.f;
        for (int k = 0; k < nsplit; k++) s += part0[(size_t)k * total + o];
        y[o] = scale ? powf(s, inv_p) * scale[o] : powf(fmaxf(s, FLT_MIN), inv_p);
    } else {
        float M = kEps;
        for (int k = 0; k < nsplit; k++) M = fmaxf(M, part1[(size_t)k * total + o]);
        float s = 0.f;
        for (int k = 0; k < nsplit; k++) {
            float Mk = part1[(size_t)k * total + o];
            s += part0[(size_t)k * total + o] * __builtin_amdgcn_exp2f(p * __builtin_amdgcn_logf(Mk / M));
        }
        y[o] = powf(s, inv_p) * M;
    }
}

// cuts the reduction range when the output tiles alone cannot fill the device; partial sums go to the
// library workspace and are merged by lp_finalize_kernel
static int lp_split_setup(FwdArgs& a, int BB, int BM, bool online, hipStream_t st) {
    a.nsplit = pick_nsplit(a, BB, BM);
    if (a.nsplit > 1) {
        a.part_stride = (size_t)a.R * a.G * a.COg;
        a.part0 = static_cast<float*>(workspace(a.part_stride * a.nsplit * (online ? 2 : 1) * sizeof(float), st));
        if (!a.part0) return SD_ERR_HIP;
        a.part1 = online ? a.part0 + a.part_stride * a.nsplit : nullptr;
    }
    return SD_OK;
}

static int lp_split_finish(const FwdArgs& a, hipStream_t st) {
    if (a.nsplit <= 1) return SD_OK;
    hipLaunchKernelGGL(lp_finalize_kernel, dim3((unsigned)((a.part_stride + 255) / 256)), dim3(256), 0, st,
                       a.part0, a.part1, a.part1 ? nullptr : a.aux, a.nsplit, a.part_stride, a.p, a.inv_p, a.y0,
                       a.gate, a.gate_limit, a.gate_above);
    return check_launch("lp_finalize_kernel");
}

// General p on the vector path: the exact maximum of |x - w| per output first (l-inf kernel, 1.5
// instructions per term), then one pass of sums relative to it, instead of the online form's two passes over
// every LDS chunk.  Workspace: the maxima, then the partial sums of the split reduction.
static int lp_forward_max_first(FwdArgs& a, bool small, hipStream_t st) {
    const size_t total = (size_t)a.R * a.G * a.COg;
    // dense single-group layers: a kernel that works from per-row candidate tables and finds the maxima as it goes
    // is queued in front of the two steps below, and a count taken on the device decides which of the two runs
    const float thr_rows = powf(1e-6f / (float)a.CIg, 1.f / a.p);
    const float cap = rows_cap(a.skip_thr > 0.f ? kRowsCapForwardSkip : kRowsCapForward, thr_rows);
    const bool rows = cap > 0.f && a.G == 1 && a.HW == 1 && !a.ci_idx && !a.co_idx && a.W_CIg == a.CIg &&
                      a.CIg % kRowsChunk == 0 && a.R < (1 << 22) && thr_rows > 0.f && thr_rows < 1.f;
    FwdArgs m = a;
    m.nsplit = pick_nsplit(m, small ? 32 : 64, 128);
    a.nsplit = m.nsplit;
    const int ns_rows = rows ? lp_rows_forward_nsplit(a.R, a.COg, a.CIg) : 1;
    // maxima, then the slice results of whichever sum kernel runs (the table kernel leaves two values per slice)
    const int slots = a.nsplit > 1 ? a.nsplit : 0, slots_rows = ns_rows > 1 ? 2 * ns_rows : 0;
    const size_t head = total * (size_t)(1 + (slots > slots_rows ? slots : slots_rows)) * sizeof(float);
    const size_t head_al = (head + 255) / 256 * 256;
    float* base = static_cast<float*>(workspace(head_al + (rows ? lp_rows_workspace(a.R, a.COg, a.CIg) : 0), st));
    if (!base) return SD_ERR_HIP;
    int rc;
    if (rows) {
        FwdArgs r = a;
        r.nsplit = ns_rows;
        r.part_stride = total;
        r.part0 = ns_rows > 1 ? base + total : nullptr;
        r.part1 = ns_rows > 1 ? base + total * (size_t)(1 + ns_rows) : nullptr;
        rc = lp_rows_forward(a.x0, a.w, nullptr, a.R, a.COg, a.CIg, a.p, thr_rows, ns_rows, a.y0, r.part0,
                             reinterpret_cast<char*>(base) + head_al, cap, &r.gate, &r.gate_limit, st);
        if (rc) return rc;
        r.gate_above = 0;
        if ((rc = lp_split_finish(r, st))) return rc;
        a.gate = r.gate; a.gate_limit = r.gate_limit; a.gate_above = 1;
        m.gate = r.gate; m.gate_limit = r.gate_limit; m.gate_above = 1;
    }
    m.y0 = base;
    if (m.nsplit > 1 && (rc = fill_zero(base, total, st))) return rc;
    if (rows) rc = small ? launch_fwd<LinfNogradGated, 2, 8>(m, st) : launch_fwd<LinfNogradGated, 4, 8>(m, st);
    else rc = small ? launch_fwd<LinfNograd, 2, 8>(m, st) : launch_fwd<LinfNograd, 4, 8>(m, st);
    if (rc) return rc;
    a.aux = base;
    a.part_stride = total;
    a.part0 = a.nsplit > 1 ? base + total : nullptr;
    a.part1 = nullptr;
    if (a.skip_thr > 0.f) rc = small ? launch_fwd<LpWithMaxSkip, 2, 8>(a, st) : launch_fwd<LpWithMaxSkip, 4, 8>(a, st);
    else rc = small ? launch_fwd<LpWithMax<-1>, 2, 8>(a, st) : launch_fwd<LpWithMax<-1>, 4, 8>(a, st);
    if (rc) return rc;
    return lp_split_finish(a, st);
}

// ---- backward -------------------------------------------------------------------------------
// u(b,m,n) = g[b,m] sgn(d) (|d| / y[b,m])^(p-1), d = x[b,n] - w[m,n]
// grad_x[b,n] = sum_m u,  grad_w[m,n] = - sum_b u      (core/cuda/norm_dist_cuda.cu:261-504)
//
// A workgroup owns 256 consecutive input channels (one per work-item) and RB = 32 batch rows.
// Each work-item keeps its 32 inputs and 32 grad_x partial sums in registers and walks all
// output channels in chunks of MC; per output channel it needs its own w[m,n] and the 32 wave-uniform
// pairs (g, 1/y), which are staged in LDS and read as broadcasts.  Everything a chunk needs is
// requested one chunk ahead, so that no load latency sits between two chunks: the weight rows of the
// next chunk (index lists: the row numbers of the chunk after it, one per lane, handed out with
// v_readlane), its weights (MC independent loads into registers) and its (g, 1/y) pairs (into the other
// half of the LDS buffer, one barrier per chunk).  The sum over the 32 rows of grad_w is formed in
// registers and added to memory with one coalesced atomic per work-item and output channel.
constexpr int RB = 32;   // batch rows per workgroup (= one index-list sub-batch)
constexpr int MC = 8;    // output channels per chunk (the chunk body is unrolled: weights sit in named registers)
static_assert(MC * RB == 256, "one (g, 1/y) pair per work-item and chunk");

struct LpBwdArgs {
    const float* gy; const float* x; const float* w; const float* y;
    float* gx; float* gw;
    const int* ci_idx; const int* co_idx;
    int B, R, HW, G, COg, CIg, W_COg, W_CIg;
    float pm1;   // p - 1
    float skip_thr;  // general p: |d| / y below this cannot change the sums (0 = every term is evaluated)
    const unsigned long long* gate;   // see FwdArgs::gate
    unsigned long long gate_limit;
    int gate_above;
    const float* ry;                  // 1 / y when the caller already holds it, else null
    bool gx_is_zero;                  // grad_input was zero-filled by the caller
    int zsplit;  // slices of the output-channel range (grad_input then merges with atomic adds)
};

template <int IP>
__device__ __forceinline__ float signed_pow(float d, float ry, float pm1) {
    float sr = d * ry;   // signed ratio
    float t1;
    switch (IP) {
        case 0: return d >= 0.f ? 1.f : -1.f;
        case 1: return sr;
        case 2: return fabsf(sr) * sr;
        case 3: return sr * sr * sr;
        case 4: t1 = sr * sr; return fabsf(sr) * sr * t1;
        case 5: t1 = sr * sr; return sr * t1 * t1;
        case 6: t1 = sr * sr; return fabsf(sr) * sr * t1 * t1;
        case 7: t1 = sr * sr; return sr * t1 * t1 * t1;
        case 8: t1 = sr * sr; return fabsf(sr) * sr * t1 * (t1 * t1);
        default: {
            float pw = __builtin_amdgcn_exp2f(pm1 * __builtin_amdgcn_logf(fabsf(sr)));
            return __builtin_copysignf(pw, sr);   // 1/y > 0: the ratio carries the sign of d (one v_bfi)
        }
    }
}

// general p from the signed ratio sr = d / y
__device__ __forceinline__ float signed_pow_ratio(float sr, float pm1) {
    float pw = __builtin_amdgcn_exp2f(pm1 * __builtin_amdgcn_logf(fabsf(sr)));
    return __builtin_copysignf(pw, sr);
}

// terms of output channel k of a chunk: FULL = all RB rows present
template <int IP, bool WGRAD, bool SKIP, bool FULL>
__device__ __forceinline__ void lp_bwd_channel(const LpBwdArgs& a, const float2 (&gr)[RB], const float (&xr)[RB],
                                               float (&acc)[RB], float wk, int rows, int row, bool n_ok,
                                               float* __restrict__ gwcol) {
    float wsum = 0.f;
    if (SKIP) {
        // large p: the two transcendentals only where some lane of the wavefront has a term that counts,
        // tested for eight batch rows together first (padded rows have x = 0, g = 0 and 1/y = 0)
        #pragma unroll
        for (int i0 = 0; i0 < RB; i0 += 8) {
            float sr[8], big = 0.f;
            #pragma unroll
            for (int e = 0; e < 8; e++) { sr[e] = (xr[i0 + e] - wk) * gr[i0 + e].y; big = fmaxf(big, fabsf(sr[e])); }
            if (__builtin_amdgcn_ballot_w64(big > a.skip_thr) == 0ull) continue;
            #pragma unroll
            for (int e = 0; e < 8; e++) {
                if (__builtin_amdgcn_ballot_w64(fabsf(sr[e]) > a.skip_thr) != 0ull) {
                    float u = gr[i0 + e].x * signed_pow_ratio(sr[e], a.pm1);
                    acc[i0 + e] += u;
                    wsum += u;
                }
            }
        }
    } else {
        #pragma unroll
        for (int i = 0; i < RB; i++) {
            if (FULL || i < rows) {
                float2 t = gr[i];
                float pw = signed_pow<IP>(xr[i] - wk, t.y, a.pm1);
                acc[i] = fmaf(t.x, pw, acc[i]);
                wsum = fmaf(t.x, pw, wsum);
            }
        }
    }
    if (WGRAD && n_ok) unsafeAtomicAdd(gwcol + (size_t)row * a.W_CIg, -wsum);
}

// one chunk.  The multiply-chain and plain general-p forms unroll the channels (weights in named registers); the
// significance-test form is branchy and large, so it loops and picks its weight with selects.
template <int IP, bool WGRAD, bool SKIP, bool FULL>
__device__ __forceinline__ void lp_bwd_chunk(const LpBwdArgs& a, const float2 (&gr)[MC][RB], const float (&xr)[RB],
                                             float (&acc)[RB], const float (&wv)[MC], int rows, int mcount,
                                             int rowv, bool n_ok, float* __restrict__ gwcol) {
    if (SKIP) {
        #pragma unroll 1
        for (int k = 0; k < mcount; k++) {
            float wk = wv[0];
            #pragma unroll
            for (int j = 1; j < MC; j++) wk = k == j ? wv[j] : wk;
            lp_bwd_channel<IP, WGRAD, SKIP, FULL>(a, gr[k], xr, acc, wk, rows, __builtin_amdgcn_readlane(rowv, k), n_ok, gwcol);
        }
    } else {
        #pragma unroll
        for (int k = 0; k < MC; k++) {
            if (k < mcount)
                lp_bwd_channel<IP, WGRAD, SKIP, FULL>(a, gr[k], xr, acc, wv[k], rows, __builtin_amdgcn_readlane(rowv, k), n_ok, gwcol);
        }
    }
}

template <int IP, bool WGRAD, bool SKIP = false>
__global__ void __launch_bounds__(256, (SKIP ? 4 : 1)) lp_bwd_kernel(LpBwdArgs a) {
    __shared__ float2 gr[2][MC][RB];   // (g, 1/y) of output channel m0+k, row r0+i; two chunks
    if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return;

    const int tid = threadIdx.x;
    const int g = blockIdx.z % a.G, slice = blockIdx.z / a.G;
    // output channels of this slice, whole chunks
    const int per = ((a.COg + a.zsplit - 1) / a.zsplit + MC - 1) / MC * MC;
    const int m_lo = slice * per, m_hi = m_lo + per < a.COg ? m_lo + per : a.COg;
    if (m_lo >= m_hi) return;   // whole workgroup; grad_input of a sliced launch is zero-filled beforehand
    const int r0 = blockIdx.y * RB;
    const int n = blockIdx.x * 256 + tid;
    const bool n_ok = n < a.CIg;
    const int s = (r0 / a.HW) / kSubBatch;
    int rows = a.R - r0;
    if (rows > RB) rows = RB;

    const int wcol = n_ok ? (a.ci_idx ? a.ci_idx[(s * a.G + g) * a.CIg + n] : n) : 0;
    const int* __restrict__ co = a.co_idx ? a.co_idx + (size_t)(s * a.G + g) * a.COg : nullptr;
    const float* __restrict__ wcolp = a.w + (size_t)g * a.W_COg * a.W_CIg + wcol;
    float* __restrict__ gwcol = WGRAD ? a.gw + (size_t)g * a.W_COg * a.W_CIg + wcol : nullptr;
    // weight row of output channel m0 + (lane mod MC), clamped into the slice so that every load stays inside W
    const int kl = tid & (MC - 1);
    auto row_of = [&](int m0) {
        int m = m0 + kl;
        m = m < m_hi ? m : m_hi - 1;
        return co ? co[m] : m;
    };
    // (g, 1/y) pair number tid of the chunk at m0: consecutive work-items take consecutive channels of one row
    const int sk = tid % MC, si = tid / MC;
    // returns (g, y); the reciprocal is taken when the pair is written to LDS, after the chunk's arithmetic, so
    // that nothing waits for these loads early (padding: g = 0, y = inf, i.e. 1/y = 0)
    auto pair_of = [&](int m0) {
        float2 v = make_float2(0.f, __builtin_inff());
        const int m = m0 + sk, r = r0 + si;
        if (m < m_hi && si < rows) {
            int b = r / a.HW, hw = r - b * a.HW;
            size_t o = ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw;
            v.x = a.gy[o];
            v.y = a.y[o];
        }
        return v;
    };

    float xr[RB], acc[RB];
    #pragma unroll
    for (int i = 0; i < RB; i++) {
        int r = r0 + i;
        float v = 0.f;
        if (n_ok && i < rows) {
            int b = r / a.HW, hw = r - b * a.HW;
            v = a.x[((size_t)(b * a.G + g) * a.CIg + n) * a.HW + hw];
        }
        xr[i] = v;
        acc[i] = 0.f;
    }

    int rowv = row_of(m_lo), rown = row_of(m_lo + MC);
    float wv[MC];
    #pragma unroll
    for (int k = 0; k < MC; k++) wv[k] = wcolp[(size_t)__builtin_amdgcn_readlane(rowv, k) * a.W_CIg];
    {
        const float2 p0 = pair_of(m_lo);
        gr[0][sk][si] = make_float2(p0.x, 1.f / p0.y);
    }
    __syncthreads();

    int buf = 0;
    for (int m0 = m_lo; m0 < m_hi; m0 += MC, buf ^= 1) {
        // requests for the next chunk (clamped rows: always inside W) and the row numbers of the one after it
        float wn[MC];
        #pragma unroll
        for (int k = 0; k < MC; k++) wn[k] = wcolp[(size_t)__builtin_amdgcn_readlane(rown, k) * a.W_CIg];
        const int rownn = row_of(m0 + 2 * MC);
        const float2 pn = pair_of(m0 + MC);

        const int mcount = m_hi - m0 < MC ? m_hi - m0 : MC;
        if (rows == RB) lp_bwd_chunk<IP, WGRAD, SKIP, true>(a, gr[buf], xr, acc, wv, rows, mcount, rowv, n_ok, gwcol);
        else lp_bwd_chunk<IP, WGRAD, SKIP, false>(a, gr[buf], xr, acc, wv, rows, mcount, rowv, n_ok, gwcol);

        gr[buf ^ 1][sk][si] = make_float2(pn.x, 1.f / pn.y);   // last read in the previous iteration, before its barrier
        __syncthreads();
        #pragma unroll
        for (int k = 0; k < MC; k++) wv[k] = wn[k];
        rowv = rown;
        rown = rownn;
    }
    if (n_ok) {
        #pragma unroll
        for (int i = 0; i < RB; i++) {
            if (i < rows) {
                int r = r0 + i;
                int b = r / a.HW, hw = r - b * a.HW;
                float* dst = a.gx + ((size_t)(b * a.G + g) * a.CIg + n) * a.HW + hw;
                if (a.zsplit > 1) unsafeAtomicAdd(dst, acc[i]);
                else *dst = acc[i];
            }
        }
    }
}

// ---- backward, dense single-group case with grad_weight and large p ------------------------------
// Fused dense backward for grad_input AND grad_weight: u(b, m, n) is formed once and feeds both sums.
// A workgroup owns FN = 8 consecutive input channels and a range of at most FMR weight rows; its 256
// work-items are 16 (row of W: m = tm + 16 j) x 16 (batch row: b = tb + 16 i) with a 4 x 2 x 8 block of terms
// each per (batch tile, weight tile) pair.  Outer loop = batch tiles, inner loop = weight tiles:
//   grad_x partial sums of the 4 batch rows stay in registers across the inner loop, are reduced over the 16
//   work-items that share the rows and added to memory (one atomic per row and channel and weight range);
//   grad_w partial sums of a pair are combined through LDS into an accumulator that covers the whole weight
//   range and is written out once at the end (the workgroup sees every batch row, so grad_weight needs no
//   global atomics).
// All operands sit in vector registers; the only LDS traffic is that combination.
constexpr int FN = 8, FMR = 1024;

__global__ void __launch_bounds__(256) lp_recip_kernel(const float* __restrict__ y, size_t n, float* __restrict__ ry) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) ry[i] = 1.f / y[i];
}

template <int IP, bool SKIP>
__global__ void __launch_bounds__(256, 3) lp_bwd_fused_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                              const float* __restrict__ g, const float* __restrict__ ry,
                                                              int B, int M, int N, int mr, float pm1, float skip_thr,
                                                              float* __restrict__ gx, float* __restrict__ gw,
                                                              const unsigned long long* gate, unsigned long long gate_limit,
                                                              int gate_above) {
    constexpr int TI = 4, TJ = 2;                 // batch rows / weight rows per work-item
    constexpr int PSTRIDE = FN * 16 * TJ + 16;    // plane of one batch-row group, skewed by 16 banks
    constexpr int GSTRIDE = FMR + 32;
    static_assert(FN * 16 * TJ == 256, "one accumulator per work-item and weight tile");
    __shared__ float gwl[FN * GSTRIDE];
    __shared__ float part[16 * PSTRIDE];
    if (gate_closed(gate, gate_limit, gate_above)) return;
    const int tid = threadIdx.x, tm = tid & 15, tb = tid >> 4;
    const int n0 = blockIdx.x * FN;
    const int m_lo = blockIdx.y * mr, m_hi = m_lo + mr < M ? m_lo + mr : M;
    for (int e = tid; e < FN * GSTRIDE; e += 256) gwl[e] = 0.f;
    __syncthreads();

    for (int b0 = 0; b0 < B; b0 += 16 * TI) {
        float xr[TI][FN], gxp[TI][FN];
        int bi[TI];
        #pragma unroll
        for (int i = 0; i < TI; i++) {
            int b = b0 + tb + 16 * i;
            bi[i] = b < B ? b : -1;
            const float* xp = x + (size_t)(b < B ? b : B - 1) * N + n0;
            float4 v0 = *reinterpret_cast<const float4*>(xp), v1 = *reinterpret_cast<const float4*>(xp + 4);
            xr[i][0] = v0.x; xr[i][1] = v0.y; xr[i][2] = v0.z; xr[i][3] = v0.w;
            xr[i][4] = v1.x; xr[i][5] = v1.y; xr[i][6] = v1.z; xr[i][7] = v1.w;
            #pragma unroll
            for (int t = 0; t < FN; t++) gxp[i][t] = 0.f;
        }
        for (int m0 = m_lo; m0 < m_hi; m0 += 16 * TJ) {
            float wr[TJ][FN], gwp[TJ][FN];
            int mj[TJ];
            #pragma unroll
            for (int j = 0; j < TJ; j++) {
                int m = m0 + tm + 16 * j;
                mj[j] = m < m_hi ? m : -1;
                const float* wp = w + (size_t)(m < m_hi ? m : m_hi - 1) * N + n0;
                float4 v0 = *reinterpret_cast<const float4*>(wp), v1 = *reinterpret_cast<const float4*>(wp + 4);
                wr[j][0] = v0.x; wr[j][1] = v0.y; wr[j][2] = v0.z; wr[j][3] = v0.w;
                wr[j][4] = v1.x; wr[j][5] = v1.y; wr[j][6] = v1.z; wr[j][7] = v1.w;
                #pragma unroll
                for (int t = 0; t < FN; t++) gwp[j][t] = 0.f;
            }
            // (g, 1/y) of the TI x TJ pairs first, so that the branches below do not serialise their loads
            float gvs[TI][TJ], rvs[TI][TJ];
            #pragma unroll
            for (int i = 0; i < TI; i++) {
                #pragma unroll
                for (int j = 0; j < TJ; j++) {
                    const bool ok = bi[i] >= 0 && mj[j] >= 0;
                    // padded rows reuse the last valid row of x / w and its own 1/y, so the ratio stays <= 1
                    const size_t o = (size_t)(bi[i] >= 0 ? bi[i] : B - 1) * M + (mj[j] >= 0 ? mj[j] : m_hi - 1);
                    gvs[i][j] = ok ? g[o] : 0.f;
                    rvs[i][j] = ry[o];
                }
            }
            #pragma unroll
            for (int i = 0; i < TI; i++) {
                #pragma unroll
                for (int j = 0; j < TJ; j++) {
                    const float gv = gvs[i][j], rv = rvs[i][j];
                    if (SKIP) {
                        // large p: transcendentals only where some lane of the wavefront has a term that counts,
                        // tested for the eight channels together first
                        float sr[FN], big = 0.f;
                        #pragma unroll
                        for (int t = 0; t < FN; t++) { sr[t] = (xr[i][t] - wr[j][t]) * rv; big = fmaxf(big, fabsf(sr[t])); }
                        if (__builtin_amdgcn_ballot_w64(big > skip_thr) != 0ull) {
                            #pragma unroll
                            for (int t = 0; t < FN; t++) {
                                if (__builtin_amdgcn_ballot_w64(fabsf(sr[t]) > skip_thr) != 0ull) {
                                    float pw = signed_pow_ratio(sr[t], pm1);
                                    gxp[i][t] = fmaf(gv, pw, gxp[i][t]);
                                    gwp[j][t] = fmaf(gv, pw, gwp[j][t]);
                                }
                            }
                        }
                        continue;
                    }
                    #pragma unroll
                    for (int t = 0; t < FN; t++) {
                        float pw = signed_pow<IP>(xr[i][t] - wr[j][t], rv, pm1);
                        gxp[i][t] = fmaf(gv, pw, gxp[i][t]);
                        gwp[j][t] = fmaf(gv, pw, gwp[j][t]);
                    }
                }
            }
            // the 16 work-items that share a weight row publish their partial sums; work-item (t, row) of the
            // tile then adds the 16 of them to the accumulator it owns (LDS float atomics are far too slow)
            #pragma unroll
            for (int j = 0; j < TJ; j++) {
                #pragma unroll
                for (int t = 0; t < FN; t++) part[tb * PSTRIDE + t * (16 * TJ) + tm + 16 * j] = gwp[j][t];
            }
            __syncthreads();
            {
                const int t = tid / (16 * TJ), ml = tid % (16 * TJ);
                float sum = 0.f;
                #pragma unroll
                for (int k = 0; k < 16; k++) sum += part[k * PSTRIDE + t * (16 * TJ) + ml];
                if (m0 + ml < m_hi) gwl[t * GSTRIDE + (m0 - m_lo) + ml] += sum;
            }
            __syncthreads();
        }
        // sum over the 16 work-items that share the batch rows, then one atomic per row and channel
        #pragma unroll
        for (int i = 0; i < TI; i++) {
            #pragma unroll
            for (int t = 0; t < FN; t++) {
                float v = gxp[i][t];
                v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4); v += __shfl_xor(v, 8);
                gxp[i][t] = v;
            }
        }
        if (tm == 0) {
            #pragma unroll
            for (int i = 0; i < TI; i++) {
                if (bi[i] >= 0) {
                    #pragma unroll
                    for (int t = 0; t < FN; t++) unsafeAtomicAdd(gx + (size_t)bi[i] * N + n0 + t, gxp[i][t]);
                }
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < (m_hi - m_lo) * 2; e += 256) {
        int row = e >> 1, h = (e & 1) * 4;
        const float* src = gwl + h * GSTRIDE + row;
        *reinterpret_cast<float4*>(gw + (size_t)(m_lo + row) * N + n0 + h) =
            make_float4(-src[0], -src[GSTRIDE], -src[2 * GSTRIDE], -src[3 * GSTRIDE]);
    }
}

static int launch_lp_bwd_fused(int ip, const LpBwdArgs& a, hipStream_t st) {
    const int B = a.R, M = a.COg, N = a.CIg;
    const size_t n = (size_t)B * M;
    int rc;
    const float* ry = a.ry;   // with it comes a zero-filled grad_input
    if (!ry) {
        float* buf = static_cast<float*>(workspace(n * sizeof(float), st));
        if (!buf) return SD_ERR_HIP;
        hipLaunchKernelGGL(lp_recip_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a.y, n, buf);
        if ((rc = check_launch("lp_recip_kernel"))) return rc;
        if ((rc = fill_zero(a.gx, (size_t)B * N, st))) return rc;
        ry = buf;
    }
    const int ranges = (M + FMR - 1) / FMR;
    const int mr = (((M + ranges - 1) / ranges) + 31) / 32 * 32;   // equal ranges, whole weight tiles
    dim3 grid(N / FN, (M + mr - 1) / mr);
    (void)ip;
    hipLaunchKernelGGL((lp_bwd_fused_kernel<-1, true>), grid, dim3(256), 0, st, a.x, a.w, a.gy, ry, B, M, N, mr, a.pm1,
                       a.skip_thr, a.gx, a.gw, a.gate, a.gate_limit, a.gate_above);
    return check_launch("lp_bwd_fused_kernel");
}

template <bool WGRAD>
static int launch_lp_bwd(int ip, const LpBwdArgs& a_in, hipStream_t st) {
    // a workgroup covers 256 input channels x 32 rows and walks the output channels; when that leaves the
    // device mostly idle (index lists: a few hundred kept inputs per sub-batch) the output-channel range is
    // cut in slices that merge into grad_input with atomic adds
    LpBwdArgs a = a_in;
    const long long blocks = (long long)((a.CIg + 255) / 256) * ((a.R + RB - 1) / RB) * a.G;
    // workgroups run in rounds of (resident workgroups per CU) x CUs: take the slice count whose last round
    // is fullest, a smaller count unless a larger one gains 3 %, slices of at least 64 channels
    const double slots = (double)((a.skip_thr > 0.f ? 4 : 3) * num_cus());
    double best = 0.0;
    a.zsplit = 1;
    for (int z = 1; z <= 16 && (z == 1 || a.COg / z >= 64); z++) {
        const double rounds = (double)blocks * z / slots, eff = rounds / std::ceil(rounds);
        if (eff > best * 1.03) { best = eff; a.zsplit = z; }
    }
    int rc;
    if (a.zsplit > 1 && !a.gx_is_zero && (rc = fill_zero(a.gx, (size_t)a.R * a.G * a.CIg, st))) return rc;
    dim3 grid((a.CIg + 255) / 256, (a.R + RB - 1) / RB, a.G * a.zsplit);
#define SD_CASE(k) case k: hipLaunchKernelGGL((lp_bwd_kernel<k, WGRAD>), grid, dim3(256), 0, st, a); break;
    switch (ip) {
        SD_CASE(0) SD_CASE(1) SD_CASE(2) SD_CASE(3) SD_CASE(4) SD_CASE(5) SD_CASE(6) SD_CASE(7) SD_CASE(8)
        default:
            if (a.skip_thr > 0.f) hipLaunchKernelGGL((lp_bwd_kernel<-1, WGRAD, true>), grid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((lp_bwd_kernel<-1, WGRAD>), grid, dim3(256), 0, st, a);
            break;
    }
#undef SD_CASE
    return check_launch("lp_bwd_kernel");
}

static int lp_backward(const char* who, const float* grad_output, const float* input, const float* weight,
                       const float* output, int B, int CO, int CI, int G, int HW, float* grad_input,
                       float* grad_weight, float p, const int* ci_idx, const int* co_idx, int W_CO, int W_CI,
                       sd_stream_t stream) {
    FwdArgs f;
    int rc = make_fwd_args(f, who, input, nullptr, weight, B, CO, CI, G, HW, ci_idx, co_idx, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(grad_output && output && grad_input, "%s: null pointer", who);
    SD_REQUIRE(p > 0.f && !std::isinf(p), "%s: p=%g must be positive and finite", who, (double)p);
    LpBwdArgs a{};
    a.gy = grad_output; a.x = input; a.w = weight; a.y = output; a.gx = grad_input; a.gw = grad_weight;
    a.ci_idx = ci_idx; a.co_idx = co_idx;
    a.B = B; a.R = f.R; a.HW = HW; a.G = G; a.COg = f.COg; a.CIg = f.CIg; a.W_COg = f.W_COg; a.W_CIg = f.W_CIg;
    a.pm1 = p - 1.f;
    // a dropped term has (|d| / y)^(p-1) < 1e-16: the reference trains with AdamW at eps = 1e-10 (main.py:38,432), which
    // turns gradient entries far below the parity bar into full-size updates, so the cut sits where even the sum of
    // all dropped terms of an entry (at most 1e-16 x terms x |grad_output|) cannot move such an update visibly
    a.skip_thr = int_power(p - 1.f) < 0 ? lp_skip_threshold(1e-16f, p - 1.f, kLpSkipFrom) : 0.f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int ip = int_power(p - 1.f);
    // large p with both gradients in the dense single-group case: the kernel that forms every term once for both
    // sums and owns its grad_weight block tests significance more cheaply than the general kernel, whose
    // test only pays from a higher threshold; everything else goes through the general kernel
    const bool dense = G == 1 && HW == 1 && !ci_idx && !co_idx && f.CIg % FN == 0 && aligned16(input) &&
                       aligned16(weight) && aligned16(grad_weight);
    // dense layers at general p: a kernel that works from per-row candidate tables is queued in front of the one
    // that evaluates every term, and a count taken on the device decides which of the two runs
    const float thr_rows = (ip < 0 && a.pm1 > 1.f) ? powf(1e-16f, 1.f / a.pm1) : 0.f;
    bool zero_gx = false;
    // which kernel evaluates every term, and whether it runs its own wave-level tests
    const bool fused = dense && grad_weight && a.skip_thr >= kLpSkipFromFused;
    const bool tests = fused || a.skip_thr >= kLpSkipFromGeneral;
    const float cap = rows_cap(grad_weight ? (tests ? kRowsCapBackwardSkip : kRowsCapBackward)
                                           : (tests ? kRowsCapBackwardInputSkip : kRowsCapBackwardInput), thr_rows);
    if (cap > 0.f && dense && thr_rows > 0.f && thr_rows < 1.f && f.CIg % kRowsChunk == 0 && f.W_CIg == f.CIg &&
        B < (1 << 22)) {
        void* ws = workspace(lp_rows_workspace(f.R, f.COg, f.CIg) + (size_t)f.R * f.COg * sizeof(float), st);
        if (!ws) return SD_ERR_HIP;
        // the general kernel adds to a zero-filled grad_weight, which the table kernel must not find cleared after it ran
        if (grad_weight && !fused && (rc = fill_zero(grad_weight, (size_t)G * f.W_COg * f.W_CIg, st))) return rc;
        if ((rc = lp_rows_backward(grad_output, input, weight, output, f.R, f.COg, f.CIg, a.pm1, thr_rows, grad_input,
                                   grad_weight, ws, cap, &a.ry, &a.gate, &a.gate_limit, st))) return rc;
        a.gate_above = 1;
        zero_gx = true;
    }
    if (dense && grad_weight && a.skip_thr >= kLpSkipFromFused) return launch_lp_bwd_fused(ip, a, st);
    if (a.skip_thr < kLpSkipFromGeneral) a.skip_thr = 0.f;
    a.gx_is_zero = zero_gx;
    if (grad_weight) {
        if (!zero_gx && (rc = fill_zero(grad_weight, (size_t)G * f.W_COg * f.W_CIg, st))) return rc;
        return launch_lp_bwd<true>(ip, a, st);
    }
    return launch_lp_bwd<false>(ip, a, st);
}

}  // namespace sd

using namespace sd;

extern "C" int sd_set_lp_candidate_density(float density) {
    SD_REQUIRE(density <= 1.f, "set_lp_candidate_density: %g is above 1", (double)density);
    g_rows_density = density;
    return SD_OK;
}

extern "C" int sd_norm_dist_forward(const float* input, const float* weight,
                                    int B, int CO, int CI, int G, int HW, float* output, float p,
                                    const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                    sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "norm_dist_forward", input, nullptr, weight, B, CO, CI, G, HW,
                           w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(output, "norm_dist_forward: null output");
    SD_REQUIRE(p > 0.f && !std::isinf(p), "norm_dist_forward: p=%g must be positive and finite", (double)p);
    a.y0 = output; a.p = p; a.inv_p = 1.f / p;
    hipStream_t st = static_cast<hipStream_t>(stream);
    static const int kTb42[] = {4, 2};
    const bool small = w_index_ci || w_index_co || pick_tb(a, kTb42, 2, 128) == 2;
    const bool online = p > 10.f;   // core/cuda/norm_dist.cpp:4,51-55
    const bool lists = w_index_ci || w_index_co;
    // p > 10: the exact maximum per output first, then one pass of sums relative to it.  On the vector path, and with
    // index lists as well: there the gather kernel's two passes over every LDS chunk (the online form) cost more than
    // a second launch (index-list training step at keep 0.75: 17.6 -> 13.7 ms at p = 256, 20.4 -> 20.1 at p = 24).
    const bool max_first = online && ((a.fast_x && a.fast_w && !w_index_co) || (lists && a.HW == 1));
    a.skip_thr = lp_skip_threshold(1e-6f / (float)a.CIg, p, max_first ? kLpSkipFrom : kLpSkipFromOnline);
    if (max_first) return lp_forward_max_first(a, small, st);
    if ((rc = lp_split_setup(a, small ? 32 : 64, 128, online, st))) return rc;
    if (!online) {
        int ip = int_power(p);
        rc = small ? launch_lp<LpPlain, 2, 8>(ip, a, st) : launch_lp<LpPlain, 4, 8>(ip, a, st);
    } else {
        if (a.skip_thr > 0.f) rc = small ? launch_fwd<LpOnlineSkip, 2, 8>(a, st) : launch_fwd<LpOnlineSkip, 4, 8>(a, st);
        else rc = small ? launch_fwd<LpOnline<-1>, 2, 8>(a, st) : launch_fwd<LpOnline<-1>, 4, 8>(a, st);
    }
    if (rc) return rc;
    return lp_split_finish(a, st);
}

extern "C" int sd_norm_dist_forward_with_max(const float* input, const float* weight, const float* max_output,
                                             int B, int CO, int CI, int G, int HW, float* output, float p,
                                             const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                             sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "norm_dist_forward_with_max", input, nullptr, weight, B, CO, CI, G, HW,
                           w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(output && max_output, "norm_dist_forward_with_max: null output or max_output");
    SD_REQUIRE(p > 0.f && !std::isinf(p), "norm_dist_forward_with_max: p=%g must be positive and finite", (double)p);
    a.y0 = output; a.aux = max_output; a.p = p; a.inv_p = 1.f / p;
    return launch_lp<LpWithMax, 2, 8>(int_power(p), a, static_cast<hipStream_t>(stream));
}

extern "C" int sd_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                           const float* output, int B, int CO, int CI, int G, int HW,
                                           float* grad_input, float p,
                                           const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                           sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    return lp_backward("norm_dist_backward_input", grad_output, input, weight, output, B, CO, CI, G, HW,
                       grad_input, nullptr, p, w_index_ci, w_index_co, W_CO, W_CI, stream);
}

extern "C" int sd_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                                  const float* output, int B, int CO, int CI, int G, int HW,
                                                  float* grad_input, float* grad_weight, float p,
                                                  const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                                  sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    SD_REQUIRE(grad_weight, "norm_dist_backward_input_weight: null grad_weight");
    return lp_backward("norm_dist_backward_input_weight", grad_output, input, weight, output, B, CO, CI, G, HW,
                       grad_input, grad_weight, p, w_index_ci, w_index_co, W_CO, W_CI, stream);
}
