/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of the SortNet distance-neuron
 * hot path.  Nothing in the shipped package may call into this file; only tests/, the
 * smoke check and the cpu_baseline leg of the benchmark do.
 *
 * Each function restates, in plain scalar C, what one row of the reference extension
 * computes (reference citations are relative to the upstream repository root):
 *
 *   sdo_inf_dist_forward          core/cuda/inf_dist_cuda.cu:110-212 (and :17-107 without pos)
 *   sdo_inf_dist_backward         core/cuda/inf_dist_cuda.cu:214-271
 *   sdo_bound_inf_dist_forward    core/cuda/bound_inf_dist_cuda.cu:15-238
 *   sdo_bound_inf_dist_backward   core/cuda/bound_inf_dist_cuda.cu:240-299
 *   sdo_sort_neuron_forward       core/cuda/sort_neuron.cu:16-214
 *   sdo_sort_neuron_backward      core/cuda/sort_neuron.cu:316-375
 *   sdo_bound_sort_neuron_forward core/cuda/sort_neuron.cu:216-314
 *   sdo_norm_dist_forward         core/cuda/norm_dist_cuda.cu:36-259 (closed form, see below)
 *   sdo_norm_dist_backward        core/cuda/norm_dist_cuda.cu:261-504
 *   sdo_masked_inf_dist_forward   no reference symbol: max over a Bernoulli-kept subset with
 *                                 the mask drawn from the counter RNG defined in this file
 *   sdo_rng_word                  the counter RNG itself
 *
 * Tensor layout (same as the reference): x is (B, CI, HW) with CI = G * CIg, weight is
 * (W_CO, W_CIg), outputs are (B, CO, HW) with CO = G * COg, all contiguous fp32; pos is int32.
 * Optional index lists w_index_ci (S, G, CIg) and w_index_co (S, G, COg), S = ceil(B/32),
 * select the weight sub-matrix used by the 32-sample sub-batch s = b / 32
 * (core/cuda/inf_dist_cuda.cu:123-127,163-172).
 *
 * Pinning status (see tests/test_oracle_pins.py):
 *   l-inf forward / argmax / sign   pinned: torch.cdist(p=inf), brute force, tie fixtures
 *   l-inf, bound, sort backward     pinned: torch autograd through a gather-based forward
 *   IBP l-inf forward               pinned: closed form of the reference's torch fallback
 *                                   (core/norm_dist.py:251-259), interval invariants
 *   sort neuron / IBP sort forward  pinned: torch.topk + geometric weights
 *                                   (core/norm_dist.py:226-230), q->1 and K=1 limits
 *   l-p forward / backward          pinned: torch.cdist(p), fp64 autograd, Euler identity
 *   masked neuron                   pinned: brute force with the mask recomputed in numpy
 *   Exact fp32 bit patterns of the reference's sort-neuron sums, l-p results and atomic
 *   gradient sums are NOT reproducible off an NVIDIA GPU (nvcc FMA contraction, __powf,
 *   __frcp_rn, atomic ordering): those are "parity unpinned" at the bit level and are
 *   compared at rel 1e-5.
 *
 * The l-p functions evaluate the reference's formulas in double precision (the reference
 * itself is only accurate to ~1e-6 relative: its running maximum is refreshed only when it
 * grows by more than 1+1e-6, core/cuda/norm_dist_cuda.cu:119-129).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>

#define SDO_EPS 1e-10f
#define SDO_SUB_BATCH 32
#define SDO_SIGN 0x80000000u
#define SDO_NAN_ID 0xffffffffu

/* ------------------------------------------------------------------------------------------
 * Counter RNG.  word = mix(mix(seed ^ stream * C1 + row) + (col + 1) * C2) with
 * mix = the "lowbias32" integer finaliser (xorshift-multiply, two rounds).
 * ---------------------------------------------------------------------------------------- */
static inline uint32_t sdo_mix(uint32_t h) {
    h ^= h >> 16; h *= 0x21f0aaadu;
    h ^= h >> 15; h *= 0x735a2d97u;
    h ^= h >> 15;
    return h;
}
static inline uint32_t sdo_row_key(uint32_t seed, uint32_t stream, uint32_t row) {
    return sdo_mix((seed ^ (stream * 0x9e3779b9u)) + row);
}
static inline uint32_t sdo_word(uint32_t key, uint32_t col) {
    return sdo_mix(key + (col + 1u) * 0x85ebca6bu);
}
uint32_t sdo_rng_word(uint32_t seed, uint32_t stream, uint32_t row, uint32_t col) {
    return sdo_word(sdo_row_key(seed, stream, row), col);
}

/* mask modes of the masked neuron */
#define SDO_MASK_TERM 0      /* independent draw per (b, m, n): 8-bit lanes of word(row=b*CO*HW.., col=n/4) */
#define SDO_MASK_FACTORED 1  /* keep(b,m,n) = kx(b,n) & kw(m,n), 16-bit thresholds ~ sqrt(q) each */

/* thresholds derived from q, shared with the device code (same integer arithmetic) */
uint32_t sdo_mask_threshold8(float q) { /* keep iff byte < T8 */
    double t = floor((double)q * 256.0 + 0.5);
    if (t < 0) t = 0;
    if (t > 256) t = 256;
    return (uint32_t)t;
}
uint32_t sdo_mask_threshold16(float q) { /* keep iff half-word < T16, T16 ~ sqrt(q) * 65536 */
    double t = floor(sqrt((double)q) * 65536.0 + 0.5);
    if (t < 0) t = 0;
    if (t > 65536) t = 65536;
    return (uint32_t)t;
}

typedef struct {
    int B, CO, CI, G, HW, COg, CIg, W_COg, W_CIg;
    const int *ci_idx, *co_idx;
} sdo_dims;

static sdo_dims sdo_make(int B, int CO, int CI, int G, int HW,
                         const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    sdo_dims d;
    d.B = B; d.CO = CO; d.CI = CI; d.G = G; d.HW = HW;
    d.COg = CO / G; d.CIg = CI / G;
    d.ci_idx = ci_idx; d.co_idx = co_idx;
    d.W_COg = co_idx ? W_CO / G : d.COg;
    d.W_CIg = ci_idx ? W_CI / G : d.CIg;
    return d;
}
/* row of the weight matrix used by sample b, group g, (compact) output channel m */
static inline int sdo_wrow(const sdo_dims* d, int b, int g, int m) {
    int s = b / SDO_SUB_BATCH;
    int mm = d->co_idx ? d->co_idx[(s * d->G + g) * d->COg + m] : m;
    return g * d->W_COg + mm;
}
static inline int sdo_wcol(const sdo_dims* d, int b, int g, int n) {
    int s = b / SDO_SUB_BATCH;
    return d->ci_idx ? d->ci_idx[(s * d->G + g) * d->CIg + n] : n;
}

/* ------------------------------------------------------------------------------------------
 * l-inf distance forward.  pos may be NULL (nograd form).
 * ---------------------------------------------------------------------------------------- */
void sdo_inf_dist_forward(const float* x, const float* w, int B, int CO, int CI, int G, int HW,
                          float* y, int* pos,
                          const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, ci_idx, co_idx, W_CO, W_CI);
    #pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg, m = c % d.COg;
        const float* wr = w + (size_t)sdo_wrow(&d, b, g, m) * d.W_CIg;
        for (int hw = 0; hw < HW; hw++) {
            const float* xr = x + ((size_t)(b * G + g) * d.CIg) * HW + hw;
            float best = SDO_EPS; uint32_t p = 0;
            if (!ci_idx) {
                for (int n = 0; n < d.CIg; n++) {
                    float t = xr[(size_t)n * HW] - wr[n], a = fabsf(t);
                    if (a > best) { best = a; p = (uint32_t)n | (t >= 0 ? 0u : SDO_SIGN); }
                }
            } else {
                for (int n = 0; n < d.CIg; n++) {
                    float t = xr[(size_t)n * HW] - wr[sdo_wcol(&d, b, g, n)], a = fabsf(t);
                    if (a > best) { best = a; p = (uint32_t)n | (t >= 0 ? 0u : SDO_SIGN); }
                }
            }
            size_t o = ((size_t)b * CO + c) * HW + hw;
            y[o] = best;
            if (pos) pos[o] = (int)p;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Masked order-statistic neuron: l-inf forward over the kept terms only.
 * keep bits come from the counter RNG; pos may be NULL.
 * ---------------------------------------------------------------------------------------- */
void sdo_masked_inf_dist_forward(const float* x, const float* w, int B, int CO, int CI, int G, int HW,
                                 float* y, int* pos, float q, uint32_t seed, int mode) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, NULL, NULL, CO, CI);
    uint32_t t8 = sdo_mask_threshold8(q), t16 = sdo_mask_threshold16(q);
    #pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg, m = c % d.COg;
        const float* wr = w + (size_t)(g * d.COg + m) * d.CIg;
        for (int hw = 0; hw < HW; hw++) {
            const float* xr = x + ((size_t)(b * G + g) * d.CIg) * HW + hw;
            size_t o = ((size_t)b * CO + c) * HW + hw;
            uint32_t key_t = sdo_row_key(seed, 0u, (uint32_t)o);
            uint32_t key_x = sdo_row_key(seed, 1u, (uint32_t)((b * G + g) * HW + hw));
            uint32_t key_w = sdo_row_key(seed, 2u, (uint32_t)c);
            float best = SDO_EPS; uint32_t p = 0;
            for (int n = 0; n < d.CIg; n++) {
                int keep;
                if (mode == SDO_MASK_TERM) {
                    uint32_t word = sdo_word(key_t, (uint32_t)(n >> 2));
                    keep = ((word >> (8 * (n & 3))) & 0xffu) < t8;
                } else {
                    keep = (sdo_word(key_x, (uint32_t)n) >> 16) < t16 &&
                           (sdo_word(key_w, (uint32_t)n) >> 16) < t16;
                }
                if (!keep) continue;
                float t = xr[(size_t)n * HW] - wr[n], a = fabsf(t);
                if (a > best) { best = a; p = (uint32_t)n | (t >= 0 ? 0u : SDO_SIGN); }
            }
            y[o] = best;
            if (pos) pos[o] = (int)p;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Scatter backward shared by the l-inf, sort and bound kernels.  Accumulates in double so the
 * result does not depend on summation order; serial over the scattered rows of grad_w.
 * ---------------------------------------------------------------------------------------- */
static void sdo_store_double(const double* acc, float* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = (float)acc[i];
}

void sdo_inf_dist_backward(const float* gy, const int* pos, int B, int CO, int CI, int G, int HW,
                           float* grad_x, float* grad_w,
                           const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, ci_idx, co_idx, W_CO, W_CI);
    size_t nx = (size_t)B * CI * HW, nw = (size_t)G * d.W_COg * d.W_CIg;
    double* ax = (double*)calloc(nx, sizeof(double));
    double* aw = grad_w ? (double*)calloc(nw, sizeof(double)) : NULL;
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg, m = c % d.COg;
        for (int hw = 0; hw < HW; hw++) {
            size_t o = ((size_t)b * CO + c) * HW + hw;
            uint32_t p = (uint32_t)pos[o];
            int n = (int)(p & ~SDO_SIGN);
            double v = (p & SDO_SIGN) ? -(double)gy[o] : (double)gy[o];
            ax[((size_t)(b * G + g) * d.CIg + n) * HW + hw] += v;
            if (aw) aw[(size_t)sdo_wrow(&d, b, g, m) * d.W_CIg + sdo_wcol(&d, b, g, n)] -= v;
        }
    }
    sdo_store_double(ax, grad_x, nx); free(ax);
    if (aw) { sdo_store_double(aw, grad_w, nw); free(aw); }
}

/* ------------------------------------------------------------------------------------------
 * Interval bound propagation through the l-inf layer.  posL/posU may both be NULL.
 * ---------------------------------------------------------------------------------------- */
void sdo_bound_inf_dist_forward(const float* xL, const float* xU, const float* w,
                                int B, int CO, int CI, int G, int HW,
                                float* yL, float* yU, int* posL, int* posU) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, NULL, NULL, CO, CI);
    #pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg;
        const float* wr = w + (size_t)c * d.CIg;
        for (int hw = 0; hw < HW; hw++) {
            size_t xo = ((size_t)(b * G + g) * d.CIg) * HW + hw;
            float lo = -SDO_EPS, hi = SDO_EPS; uint32_t pl = SDO_NAN_ID, pu = 0;
            for (int n = 0; n < d.CIg; n++) {
                float l = xL[xo + (size_t)n * HW], u = xU[xo + (size_t)n * HW];
                if (l > u) l = u = (l + u) * 0.5f;
                float t1 = wr[n] - l, t2 = u - wr[n];
                /* min / max of the device code return the defined operand when the other is undefined
                   (bound_inf_dist_cuda.cu:95-96, 204); an undefined result fails the strict compares below */
                float a = fminf(t1, t2), bb = fmaxf(t1, t2);
                uint32_t p = (uint32_t)n | (t1 <= t2 ? 0u : SDO_SIGN);
                if (a < lo) { lo = a; pl = p; }
                if (bb > hi) { hi = bb; pu = p; }
            }
            size_t o = ((size_t)b * CO + c) * HW + hw;
            yL[o] = -lo; yU[o] = hi;
            if (posL) posL[o] = (int)pl;
            if (posU) posU[o] = (int)pu;
        }
    }
}

void sdo_bound_inf_dist_backward(const float* gL, const float* gU, const int* posL, const int* posU,
                                 int B, int CO, int CI, int G, int HW,
                                 float* grad_xL, float* grad_xU, float* grad_w) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, NULL, NULL, CO, CI);
    size_t nx = (size_t)B * CI * HW, nw = (size_t)CO * d.CIg;
    double* aL = (double*)calloc(nx, sizeof(double));
    double* aU = (double*)calloc(nx, sizeof(double));
    double* aw = grad_w ? (double*)calloc(nw, sizeof(double)) : NULL;
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg;
        for (int hw = 0; hw < HW; hw++) {
            size_t o = ((size_t)b * CO + c) * HW + hw;
            uint32_t pl = (uint32_t)posL[o], pu = (uint32_t)posU[o];
            int nl = (int)(pl & ~SDO_SIGN), nu = (int)(pu & ~SDO_SIGN);
            double vl = (pl & SDO_SIGN) ? -(double)gL[o] : (double)gL[o];
            double vu = (pu & SDO_SIGN) ? -(double)gU[o] : (double)gU[o];
            size_t base = ((size_t)(b * G + g) * d.CIg) * HW + hw;
            if (pl != SDO_NAN_ID) {
                ((pl & SDO_SIGN) ? aU : aL)[base + (size_t)nl * HW] += vl;
                if (aw) aw[(size_t)c * d.CIg + nl] -= vl;
            }
            ((pu & SDO_SIGN) ? aL : aU)[base + (size_t)nu * HW] += vu;
            if (aw) aw[(size_t)c * d.CIg + nu] -= vu;
        }
    }
    sdo_store_double(aL, grad_xL, nx); free(aL);
    sdo_store_double(aU, grad_xU, nx); free(aU);
    if (aw) { sdo_store_double(aw, grad_w, nw); free(aw); }
}

/* ------------------------------------------------------------------------------------------
 * Sort neuron (top-K of |x-w| with geometric weights).  res[] is kept ascending
 * (res[K-1] = largest) exactly as the reference does; a new value enters only if it is
 * strictly greater than res[0] and is placed above equal values.  pos may be NULL;
 * pos is (K, B, CO, HW) with slot 0 = largest.  All arithmetic of the weighted sum is fp32 in
 * the reference's order: ans += (res * c) * q ; c *= 1 - q ; y = ans / (1 - c).
 * ---------------------------------------------------------------------------------------- */
#define SDO_MAX_K 25

static inline void sdo_insert(float* res, uint32_t* idx, int K, float v, uint32_t p) {
    if (!(v > res[0])) return;
    int k;
    for (k = 0; k < K - 1; k++) {
        if (v < res[k + 1]) { res[k] = v; idx[k] = p; return; }
        res[k] = res[k + 1]; idx[k] = idx[k + 1];
    }
    res[K - 1] = v; idx[K - 1] = p;
}

static inline float sdo_geo_sum(const float* res, int K, float q, float init, float* c_out) {
    /* built with -ffp-contract=off: every product and sum below rounds to fp32 separately */
    float ans = init, c = 1.0f;
    for (int k = K - 1; k >= 0; k--) {
        ans += res[k] * c * q;
        c *= 1.0f - q;
    }
    *c_out = c;
    return ans;
}

int sdo_sort_neuron_forward(const float* x, const float* w, int B, int CO, int CI, int G, int HW,
                            float* y, int* pos, float q, int K) {
    if (K < 1 || K > SDO_MAX_K) return 1;
    sdo_dims d = sdo_make(B, CO, CI, G, HW, NULL, NULL, CO, CI);
    size_t size = (size_t)B * CO * HW;
    #pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg;
        const float* wr = w + (size_t)c * d.CIg;
        for (int hw = 0; hw < HW; hw++) {
            const float* xr = x + ((size_t)(b * G + g) * d.CIg) * HW + hw;
            float res[SDO_MAX_K]; uint32_t idx[SDO_MAX_K];
            for (int k = 0; k < K; k++) { res[k] = 0; idx[k] = 0; }
            for (int n = 0; n < d.CIg; n++) {
                float t = xr[(size_t)n * HW] - wr[n];
                sdo_insert(res, idx, K, fabsf(t), (uint32_t)n | (t >= 0 ? 0u : SDO_SIGN));
            }
            size_t o = ((size_t)b * CO + c) * HW + hw;
            float cfin;
            float ans = sdo_geo_sum(res, K, q, SDO_EPS, &cfin);
            y[o] = ans / (1.0f - cfin);
            if (pos) for (int k = K - 1; k >= 0; k--) pos[(size_t)(K - 1 - k) * size + o] = (int)idx[k];
        }
    }
    return 0;
}

void sdo_sort_neuron_backward(const float* gy, const int* pos, int B, int CO, int CI, int G, int HW,
                              float* grad_x, float* grad_w, float q, int K) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, NULL, NULL, CO, CI);
    size_t nx = (size_t)B * CI * HW, nw = (size_t)CO * d.CIg, size = (size_t)B * CO * HW;
    double* ax = (double*)calloc(nx, sizeof(double));
    double* aw = grad_w ? (double*)calloc(nw, sizeof(double)) : NULL;
    double r = pow(1.0 - (double)q, (double)K);
    double norm = 1.0 + r / (1.0 - r);
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg;
        for (int hw = 0; hw < HW; hw++) {
            size_t o = ((size_t)b * CO + c) * HW + hw;
            double coef = norm;
            for (int k = 0; k < K; k++) {
                uint32_t p = (uint32_t)pos[(size_t)k * size + o];
                int n = (int)(p & ~SDO_SIGN);
                double v = ((p & SDO_SIGN) ? -(double)gy[o] : (double)gy[o]) * coef * (double)q;
                ax[((size_t)(b * G + g) * d.CIg + n) * HW + hw] += v;
                if (aw) aw[(size_t)c * d.CIg + n] -= v;
                coef *= 1.0 - (double)q;
            }
        }
    }
    sdo_store_double(ax, grad_x, nx); free(ax);
    if (aw) { sdo_store_double(aw, grad_w, nw); free(aw); }
}

int sdo_bound_sort_neuron_forward(const float* xL, const float* xU, const float* w,
                                  int B, int CO, int CI, int G, int HW,
                                  float* yL, float* yU, float q, int K) {
    if (K < 1 || K > SDO_MAX_K) return 1;
    sdo_dims d = sdo_make(B, CO, CI, G, HW, NULL, NULL, CO, CI);
    #pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg;
        const float* wr = w + (size_t)c * d.CIg;
        for (int hw = 0; hw < HW; hw++) {
            size_t xo = ((size_t)(b * G + g) * d.CIg) * HW + hw;
            /* resU ascending top-K of max(t1,t2); resL holds -(K most negative of min(t1,t2)),
               also ascending, so one insertion routine serves both */
            float resL[SDO_MAX_K], resU[SDO_MAX_K]; uint32_t dummy[SDO_MAX_K];
            for (int k = 0; k < K; k++) { resL[k] = 0; resU[k] = 0; }
            for (int n = 0; n < d.CIg; n++) {
                float l = xL[xo + (size_t)n * HW], u = xU[xo + (size_t)n * HW];
                if (l > u) l = u = (l + u) * 0.5f;
                float t1 = wr[n] - l, t2 = u - wr[n];
                /* min / max as on the device (sort_neuron.cu:280).  A term whose operands are both undefined is
                   dropped here, while the reference's min/max insertion (:283-287) then duplicates the largest
                   entry of the list: undefined inputs to the sort neuron are outside what this restatement pins. */
                float a = fminf(t1, t2), bb = fmaxf(t1, t2);
                sdo_insert(resL, dummy, K, -a, 0);
                sdo_insert(resU, dummy, K, bb, 0);
            }
            size_t o = ((size_t)b * CO + c) * HW + hw;
            float cfin;
            /* lower: -( -EPS + sum resL_j c q ) with resL_j <= 0 in the reference == EPS + sum(-resL_j) c q */
            float aL = sdo_geo_sum(resL, K, q, SDO_EPS, &cfin);
            float aU = sdo_geo_sum(resU, K, q, SDO_EPS, &cfin);
            yL[o] = aL / (1.0f - cfin);
            yU[o] = aU / (1.0f - cfin);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * l-p norm distance, evaluated in double precision.
 *   p <= 10 : y = max(sum |d|^p, FLT_MIN)^(1/p)                 (norm_dist_cuda.cu:238,253)
 *   p  > 10 : y = M (sum (|d|/M)^p + (EPS/M)^p)^(1/p), M = max(EPS, max|d|)   (:61-154)
 * ---------------------------------------------------------------------------------------- */
void sdo_norm_dist_forward(const float* x, const float* w, int B, int CO, int CI, int G, int HW,
                           float* y, float p,
                           const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, ci_idx, co_idx, W_CO, W_CI);
    double dp = (double)p;
    #pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
    for (int c = 0; c < CO; c++) {
        int g = c / d.COg, m = c % d.COg;
        const float* wr = w + (size_t)sdo_wrow(&d, b, g, m) * d.W_CIg;
        for (int hw = 0; hw < HW; hw++) {
            const float* xr = x + ((size_t)(b * G + g) * d.CIg) * HW + hw;
            double ans;
            if (p <= 10.0f) {
                double s = 0;
                for (int n = 0; n < d.CIg; n++)
                    s += pow(fabs((double)(xr[(size_t)n * HW] - wr[sdo_wcol(&d, b, g, n)])), dp);
                if (s < (double)FLT_MIN) s = (double)FLT_MIN;
                ans = pow(s, 1.0 / dp);
            } else {
                double M = (double)SDO_EPS;
                for (int n = 0; n < d.CIg; n++) {
                    double a = fabs((double)(xr[(size_t)n * HW] - wr[sdo_wcol(&d, b, g, n)]));
                    if (a > M) M = a;
                }
                double s = pow((double)SDO_EPS / M, dp);
                for (int n = 0; n < d.CIg; n++)
                    s += pow(fabs((double)(xr[(size_t)n * HW] - wr[sdo_wcol(&d, b, g, n)])) / M, dp);
                ans = pow(s, 1.0 / dp) * M;
            }
            y[((size_t)b * CO + c) * HW + hw] = (float)ans;
        }
    }
}

/* u = g * sgn(d) * (|d| / y)^(p-1) ; grad_x[b,n] = sum_m u ; grad_w[m,n] = - sum_b u
 * (norm_dist_cuda.cu:261-266,349,456-461).  y is the saved forward output. */
void sdo_norm_dist_backward(const float* gy, const float* x, const float* w, const float* y,
                            int B, int CO, int CI, int G, int HW,
                            float* grad_x, float* grad_w, float p,
                            const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    sdo_dims d = sdo_make(B, CO, CI, G, HW, ci_idx, co_idx, W_CO, W_CI);
    size_t nx = (size_t)B * CI * HW, nw = (size_t)G * d.W_COg * d.W_CIg;
    double pm1 = (double)p - 1.0;
    double* ax = (double*)calloc(nx, sizeof(double));
    double* aw = grad_w ? (double*)calloc(nw, sizeof(double)) : NULL;
    /* parallel over input channels: each (g, n) owns its grad_x column and grad_w column */
    #pragma omp parallel for collapse(2) schedule(static)
    for (int g = 0; g < G; g++)
    for (int n = 0; n < d.CIg; n++) {
        for (int b = 0; b < B; b++) {
            int wc = sdo_wcol(&d, b, g, n);
            for (int hw = 0; hw < HW; hw++) {
                size_t xi = ((size_t)(b * G + g) * d.CIg + n) * HW + hw;
                double s = 0;
                for (int m = 0; m < d.COg; m++) {
                    size_t o = ((size_t)b * CO + g * d.COg + m) * HW + hw;
                    size_t wi = (size_t)sdo_wrow(&d, b, g, m) * d.W_CIg + wc;
                    float tf = x[xi] - w[wi];
                    double t = (double)tf;
                    double r = fabs(t) / (double)y[o];
                    double u = (double)gy[o] * pow(r, pm1) * (t >= 0 ? 1.0 : -1.0);
                    s += u;
                    if (aw) {
                        /* with index lists different n of one sub-batch never alias, but different
                           sub-batches can hit the same weight column from different n */
                        if (d.ci_idx) {
                            #pragma omp atomic
                            aw[wi] -= u;
                        } else aw[wi] -= u;
                    }
                }
                ax[xi] = s;
            }
        }
    }
    sdo_store_double(ax, grad_x, nx); free(ax);
    if (aw) { sdo_store_double(aw, grad_w, nw); free(aw); }
}

/* ------------------------------------------------------------------------------------------
 * Mean shift over batch and spatial positions (training form, no index list):
 * mean[c] = mean_{b,hw} x ; out = x - mean   (core/models/bound_basic_module.py:142,155)
 * ---------------------------------------------------------------------------------------- */
void sdo_mean_shift(const float* x, int B, int C, int HW, float* mean, float* out) {
    #pragma omp parallel for schedule(static)
    for (int c = 0; c < C; c++) {
        double s = 0;
        for (int b = 0; b < B; b++)
            for (int hw = 0; hw < HW; hw++) s += (double)x[((size_t)b * C + c) * HW + hw];
        mean[c] = (float)(s / ((double)B * HW));
    }
    #pragma omp parallel for schedule(static)
    for (int b = 0; b < B; b++)
        for (int c = 0; c < C; c++)
            for (int hw = 0; hw < HW; hw++) {
                size_t i = ((size_t)b * C + c) * HW + hw;
                out[i] = x[i] - mean[c];
            }
}

/* ------------------------------------------------------------------------------------------
 * Mask sampling of the index-list form (core/models/norm_dist.py:14-17 restated on the counter RNG):
 * count = #{c : word(key(3,0), c) < q 2^32}; list (s,g) = the `count` channels with the smallest
 * 48-bit keys (word(key(4, s G + g), c) << 16) | c, ascending channel order.
 * ---------------------------------------------------------------------------------------- */
int sdo_mask_count(uint32_t seed, int C, float q) {
    double t = floor((double)q * 4294967296.0 + 0.5);
    if (t < 0) t = 0;
    if (t > 4294967296.0) t = 4294967296.0;
    uint64_t thr = (uint64_t)t;
    uint32_t key = sdo_row_key(seed, 3u, 0u);
    int n = 0;
    for (int c = 0; c < C; c++) n += (uint64_t)sdo_word(key, (uint32_t)c) < thr;
    return n;
}

static int sdo_cmp_u64(const void* a, const void* b) {
    uint64_t x = *(const uint64_t*)a, y = *(const uint64_t*)b;
    return x < y ? -1 : x > y;
}

void sdo_sample_index_lists(uint32_t seed, int S, int G, int C, int count, int* out) {
    uint64_t* keys = (uint64_t*)malloc((size_t)C * sizeof(uint64_t));
    uint64_t* sorted = (uint64_t*)malloc((size_t)C * sizeof(uint64_t));
    for (int r = 0; r < S * G; r++) {
        uint32_t rk = sdo_row_key(seed, 4u, (uint32_t)r);
        for (int c = 0; c < C; c++) keys[c] = ((uint64_t)sdo_word(rk, (uint32_t)c) << 16) | (uint64_t)c;
        memcpy(sorted, keys, (size_t)C * sizeof(uint64_t));
        qsort(sorted, (size_t)C, sizeof(uint64_t), sdo_cmp_u64);
        int k = 0;
        if (count > 0) {
            uint64_t last = sorted[count - 1];
            for (int c = 0; c < C; c++) if (keys[c] <= last) out[(size_t)r * count + k++] = c;
        }
    }
    free(keys); free(sorted);
}
