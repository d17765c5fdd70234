// l-p norm distance: forward entry points and the fused backward kernel.
#include "fwd_tile.h"
#include "fwd_args.h"

namespace sd {

// integral 0 <= p <= 8 selects a multiply chain, anything else the transcendental path
// (core/cuda/norm_dist.cpp:17-38)
static inline int int_power(float p) {
    if (p == (float)(int)p && p >= 0.f && p <= 8.f) return (int)p;
    return -1;
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

// ---- backward -------------------------------------------------------------------------------
// u(b,m,n) = g[b,m] sgn(d) (|d| / y[b,m])^(p-1), d = x[b,n] - w[m,n]
// grad_x[b,n] = sum_m u,  grad_w[m,n] = - sum_b u      (core/cuda/norm_dist_cuda.cu:261-504)
//
// A workgroup owns 256 consecutive input channels (one per work-item) and RB = 32 batch rows.
// Each work-item keeps its 32 inputs and 32 grad_x partial sums in registers and walks all
// output channels; per output channel it needs its own w[m,n] (coalesced global load) and the
// 32 wave-uniform pairs (g, 1/y), which are staged in LDS in chunks of MC channels and read as
// broadcasts.  The sum over the 32 rows of grad_w is formed in registers and added to memory
// with one coalesced atomic per work-item and output channel.
constexpr int RB = 32;   // batch rows per workgroup (= one index-list sub-batch)
constexpr int MC = 16;   // output channels per LDS chunk

struct LpBwdArgs {
    const float* gy; const float* x; const float* w; const float* y;
    float* gx; float* gw;
    const int* ci_idx; const int* co_idx;
    int B, R, HW, G, COg, CIg, W_COg, W_CIg;
    float pm1;   // p - 1
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
            return d >= 0.f ? pw : -pw;
        }
    }
}

template <int IP, bool WGRAD>
__global__ void __launch_bounds__(256) lp_bwd_kernel(LpBwdArgs a) {
    __shared__ float2 gr[MC][RB];   // (g, 1/y) of output channel m0+k, row r0+i

    const int tid = threadIdx.x;
    const int g = blockIdx.z;
    const int r0 = blockIdx.y * RB;
    const int n = blockIdx.x * 256 + tid;
    const bool n_ok = n < a.CIg;
    const int s = (r0 / a.HW) / kSubBatch;
    int rows = a.R - r0;
    if (rows > RB) rows = RB;

    const int wcol = n_ok ? (a.ci_idx ? a.ci_idx[(s * a.G + g) * a.CIg + n] : n) : 0;

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

    for (int m0 = 0; m0 < a.COg; m0 += MC) {
        __syncthreads();
        // stage (g, 1/y): MC * RB = 512 pairs, two per work-item; consecutive work-items take
        // consecutive channels of one row when HW == 1
        #pragma unroll
        for (int e = tid; e < MC * RB; e += 256) {
            int k = e % MC, i = e / MC;
            int m = m0 + k, r = r0 + i;
            float2 v = make_float2(0.f, 0.f);
            if (m < a.COg && i < rows) {
                int b = r / a.HW, hw = r - b * a.HW;
                size_t o = ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw;
                v.x = a.gy[o];
                v.y = 1.f / a.y[o];
            }
            gr[k][i] = v;
        }
        float wv[MC];
        #pragma unroll
        for (int k = 0; k < MC; k++) {
            int m = m0 + k;
            float v = 0.f;
            if (n_ok && m < a.COg) {
                int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
                v = a.w[(size_t)(g * a.W_COg + wrow) * a.W_CIg + wcol];
            }
            wv[k] = v;
        }
        __syncthreads();
        const int mcount = a.COg - m0 < MC ? a.COg - m0 : MC;
        for (int k = 0; k < mcount; k++) {
            float wsum = 0.f;
            if (rows == RB) {
                #pragma unroll
                for (int i = 0; i < RB; i++) {
                    float2 t = gr[k][i];
                    float u = t.x * signed_pow<IP>(xr[i] - wv[k], t.y, a.pm1);
                    acc[i] += u;
                    wsum += u;
                }
            } else {
                #pragma unroll
                for (int i = 0; i < RB; i++) {
                    if (i < rows) {
                        float2 t = gr[k][i];
                        float u = t.x * signed_pow<IP>(xr[i] - wv[k], t.y, a.pm1);
                        acc[i] += u;
                        wsum += u;
                    }
                }
            }
            if (WGRAD && n_ok) {
                int m = m0 + k;
                int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
                unsafeAtomicAdd(a.gw + (size_t)(g * a.W_COg + wrow) * a.W_CIg + wcol, -wsum);
            }
        }
    }
    if (n_ok) {
        #pragma unroll
        for (int i = 0; i < RB; i++) {
            if (i < rows) {
                int r = r0 + i;
                int b = r / a.HW, hw = r - b * a.HW;
                a.gx[((size_t)(b * a.G + g) * a.CIg + n) * a.HW + hw] = acc[i];
            }
        }
    }
}

template <bool WGRAD>
static int launch_lp_bwd(int ip, const LpBwdArgs& a, hipStream_t st) {
    dim3 grid((a.CIg + 255) / 256, (a.R + RB - 1) / RB, a.G);
#define SD_CASE(k) case k: hipLaunchKernelGGL((lp_bwd_kernel<k, WGRAD>), grid, dim3(256), 0, st, a); break;
    switch (ip) {
        SD_CASE(0) SD_CASE(1) SD_CASE(2) SD_CASE(3) SD_CASE(4) SD_CASE(5) SD_CASE(6) SD_CASE(7) SD_CASE(8)
        default: hipLaunchKernelGGL((lp_bwd_kernel<-1, WGRAD>), grid, dim3(256), 0, st, a); break;
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
    hipStream_t st = static_cast<hipStream_t>(stream);
    int ip = int_power(p - 1.f);
    if (grad_weight) {
        if ((rc = fill_zero(grad_weight, (size_t)G * f.W_COg * f.W_CIg, st))) return rc;
        return launch_lp_bwd<true>(ip, a, st);
    }
    return launch_lp_bwd<false>(ip, a, st);
}

}  // namespace sd

using namespace sd;

extern "C" int sd_norm_dist_forward(const float* input, const float* weight,
                                    int B, int CO, int CI, int G, int HW, float* output, float p,
                                    const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                    sd_stream_t stream) {
    FwdArgs a;
    int rc = make_fwd_args(a, "norm_dist_forward", input, nullptr, weight, B, CO, CI, G, HW,
                           w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(output, "norm_dist_forward: null output");
    SD_REQUIRE(p > 0.f && !std::isinf(p), "norm_dist_forward: p=%g must be positive and finite", (double)p);
    a.y0 = output; a.p = p; a.inv_p = 1.f / p;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = w_index_ci || w_index_co || a.R <= 32;
    if (p <= 10.f) {   // core/cuda/norm_dist.cpp:4,51-55
        int ip = int_power(p);
        return small ? launch_lp<LpPlain, 2, 8>(ip, a, st) : launch_lp<LpPlain, 4, 8>(ip, a, st);
    }
    return small ? launch_fwd<LpOnline<-1>, 2, 8>(a, st) : launch_fwd<LpOnline<-1>, 4, 8>(a, st);
}

extern "C" int sd_norm_dist_forward_with_max(const float* input, const float* weight, const float* max_output,
                                             int B, int CO, int CI, int G, int HW, float* output, float p,
                                             const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                             sd_stream_t stream) {
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
    return lp_backward("norm_dist_backward_input", grad_output, input, weight, output, B, CO, CI, G, HW,
                       grad_input, nullptr, p, w_index_ci, w_index_co, W_CO, W_CI, stream);
}

extern "C" int sd_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                                  const float* output, int B, int CO, int CI, int G, int HW,
                                                  float* grad_input, float* grad_weight, float p,
                                                  const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                                  sd_stream_t stream) {
    SD_REQUIRE(grad_weight, "norm_dist_backward_input_weight: null grad_weight");
    return lp_backward("norm_dist_backward_input_weight", grad_output, input, weight, output, B, CO, CI, G, HW,
                       grad_input, grad_weight, p, w_index_ci, w_index_co, W_CO, W_CI, stream);
}
