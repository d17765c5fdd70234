// Mean shift over batch and spatial positions, the step that follows every distance layer
// (core/models/bound_basic_module.py:106-157, training form without index list):
//   mean[c] = mean_{b,hw} x[b,c,hw];  running = (1 - momentum) running + momentum mean;  y = x - mean[c]
// the plain per-channel shift y = x - shift[c] used in evaluation mode and for a bias, and the training form
// with a kept-channel index list per 32-sample sub-batch.
#include "common.h"

namespace sd {

// One workgroup owns 64 channels (HW == 1) or one channel (HW > 1); 16 groups of 64 work-items walk
// the batch in parallel, partial sums meet in LDS, the sum order is fixed (deterministic result).
__global__ void __launch_bounds__(1024) channel_mean_kernel(const float* __restrict__ x, int B, int C, int HW,
                                                            float* __restrict__ mean, float* __restrict__ running,
                                                            float momentum) {
    __shared__ float part[16][64];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    float s = 0.f;
    if (HW == 1) {
        const int c = blockIdx.x * 64 + lane;
        if (c < C)
            for (int b = grp; b < B; b += 16) s += x[(size_t)b * C + c];
        part[grp][lane] = s;
        __syncthreads();
        if (grp == 0 && c < C) {
            float t = 0.f;
            #pragma unroll
            for (int k = 0; k < 16; k++) t += part[k][lane];
            float m = t / (float)B;
            mean[c] = m;
            if (running) running[c] = (1.f - momentum) * running[c] + momentum * m;
        }
    } else {
        const int c = blockIdx.x;
        const long long n = (long long)B * HW;
        for (long long i = threadIdx.x; i < n; i += 1024) {
            long long b = i / HW, hw = i - b * HW;
            s += x[((size_t)b * C + c) * HW + hw];
        }
        part[grp][lane] = s;
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = 0.f;
            for (int k = 0; k < 16; k++)
                for (int l = 0; l < 64; l++) t += part[k][l];
            float m = t / (float)n;
            mean[c] = m;
            if (running) running[c] = (1.f - momentum) * running[c] + momentum * m;
        }
    }
}

__global__ void __launch_bounds__(256) channel_shift_kernel(const float* __restrict__ x, const float* __restrict__ shift,
                                                            long long total, int C, int HW, float sign,
                                                            float* __restrict__ y) {
    long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    if (HW == 1 && C % 4 == 0 && i + 3 < total) {
        float4 v = *reinterpret_cast<const float4*>(x + i);
        float4 sh = *reinterpret_cast<const float4*>(shift + (i % C));
        v.x += sign * sh.x; v.y += sign * sh.y; v.z += sign * sh.z; v.w += sign * sh.w;
        *reinterpret_cast<float4*>(y + i) = v;
    } else {
        for (int k = 0; k < 4 && i + k < total; k++) {
            long long j = i + k;
            int c = (int)((j / HW) % C);
            y[j] = x[j] + sign * shift[c];
        }
    }
}

// ---- index-list form: the input holds, for every 32-sample sub-batch s, only the channels index[s, g, :] ----

// column sums of one sub-batch: work-item = one kept channel j of (s, g); the sum lands in the slot of the
// full channel it stands for.  A sub-batch lists a channel at most once, so slots are written at most once.
__global__ void __launch_bounds__(256) index_colsum_kernel(const float* __restrict__ x, const int* __restrict__ index,
                                                           int B, int G, int cnt, int Cg, int HW,
                                                           float* __restrict__ part, float* __restrict__ rows) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    const int sg = blockIdx.y, s = sg / G, g = sg - s * G;
    if (j >= cnt) return;
    const int b0 = s * kSubBatch, b1 = b0 + kSubBatch < B ? b0 + kSubBatch : B;
    float t = 0.f;
    if (HW == 1) {
        const float* src = x + (size_t)g * cnt + j;
        const size_t stride = (size_t)G * cnt;
        #pragma unroll 8
        for (int b = b0; b < b1; b++) t += src[b * stride];      // independent loads, added in sample order
    } else {
        for (int b = b0; b < b1; b++) {
            const float* src = x + ((size_t)(b * G + g) * cnt + j) * HW;
            for (int hw = 0; hw < HW; hw++) t += src[hw];
        }
    }
    const size_t slot = (size_t)s * G * Cg + (size_t)g * Cg + index[(size_t)sg * cnt + j];
    part[slot] = t;
    rows[slot] = (float)(b1 - b0);
}

// mean of every full channel over the sub-batches that kept it, in sub-batch order (deterministic)
__global__ void __launch_bounds__(256) index_mean_kernel(const float* __restrict__ part, const float* __restrict__ rows,
                                                         int S, int C, int HW, float* __restrict__ mean,
                                                         float* __restrict__ running, float momentum) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    float total = 0.f, seen = 1e-10f;
    for (int s = 0; s < S; s++) { total += part[(size_t)s * C + c]; seen += rows[(size_t)s * C + c]; }
    const float m = total / (seen * (float)HW);
    mean[c] = m;
    if (running) running[c] = (1.f - momentum) * running[c] + momentum * m;
}

__global__ void __launch_bounds__(256) index_shift_kernel(const float* __restrict__ x, const int* __restrict__ index,
                                                          const float* __restrict__ mean, long long total,
                                                          int G, int cnt, int Cg, int HW, float* __restrict__ y) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long long t = i / HW;
    const int j = (int)(t % cnt);
    const long long bg = t / cnt;
    const int g = (int)(bg % G), b = (int)(bg / G);
    const int s = b / kSubBatch;
    y[i] = x[i] - mean[g * Cg + index[(size_t)(s * G + g) * cnt + j]];
}

static int check_dims(const char* who, int B, int C, int HW) {
    SD_REQUIRE(B > 0 && C > 0 && HW > 0, "%s: sizes must be positive", who);
    SD_REQUIRE((long long)B * C * HW < (1ll << 31), "%s: tensor too large for 32-bit indexing", who);
    return SD_OK;
}

}  // namespace sd

using namespace sd;

extern "C" int sd_mean_shift_forward(const float* input, int B, int C, int HW, float* mean, float* running_mean,
                                     float momentum, float* output, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    int rc = check_dims("mean_shift_forward", B, C, HW);
    if (rc) return rc;
    SD_REQUIRE(input && mean && output, "mean_shift_forward: null pointer");
    SD_REQUIRE(reinterpret_cast<uintptr_t>(input) % 16 == 0 && reinterpret_cast<uintptr_t>(output) % 16 == 0 &&
               reinterpret_cast<uintptr_t>(mean) % 16 == 0, "mean_shift_forward: buffers must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 grid(HW == 1 ? (C + 63) / 64 : C);
    hipLaunchKernelGGL(channel_mean_kernel, grid, dim3(1024), 0, st, input, B, C, HW, mean, running_mean, momentum);
    if ((rc = check_launch("channel_mean_kernel"))) return rc;
    long long total = (long long)B * C * HW;
    hipLaunchKernelGGL(channel_shift_kernel, dim3((unsigned)((total / 4 + 255) / 256 + 1)), dim3(256), 0, st,
                       input, mean, total, C, HW, -1.f, output);
    return check_launch("channel_shift_kernel");
}

extern "C" int sd_channel_shift(const float* input, const float* shift, int B, int C, int HW, float sign,
                                float* output, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    int rc = check_dims("channel_shift", B, C, HW);
    if (rc) return rc;
    SD_REQUIRE(input && shift && output, "channel_shift: null pointer");
    SD_REQUIRE(reinterpret_cast<uintptr_t>(input) % 16 == 0 && reinterpret_cast<uintptr_t>(output) % 16 == 0 &&
               reinterpret_cast<uintptr_t>(shift) % 16 == 0, "channel_shift: buffers must be 16-byte aligned");
    long long total = (long long)B * C * HW;
    hipLaunchKernelGGL(channel_shift_kernel, dim3((unsigned)((total / 4 + 255) / 256 + 1)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), input, shift, total, C, HW, sign, output);
    return check_launch("channel_shift_kernel");
}

extern "C" int sd_mean_shift_index_forward(const float* input, const int* index, int B, int G, int cnt, int Cg, int HW,
                                           float* mean, float* running_mean, float momentum, float* output,
                                           sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    SD_REQUIRE(G > 0 && cnt > 0 && Cg >= cnt, "mean_shift_index_forward: need G > 0 and 0 < cnt <= Cg (cnt=%d Cg=%d)", cnt, Cg);
    SD_REQUIRE((long long)G * cnt < (1ll << 31) && (long long)G * Cg < (1ll << 31), "mean_shift_index_forward: too many channels");
    int rc = check_dims("mean_shift_index_forward", B, G * cnt, HW);
    if (rc) return rc;
    SD_REQUIRE(input && index && mean && output, "mean_shift_index_forward: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int S = (B + kSubBatch - 1) / kSubBatch, C = G * Cg;
    float* part = static_cast<float*>(workspace((size_t)2 * S * C * sizeof(float), st));
    if (!part) return SD_ERR_HIP;
    float* rows = part + (size_t)S * C;
    if ((rc = fill_zero(part, (size_t)2 * S * C, st))) return rc;
    hipLaunchKernelGGL(index_colsum_kernel, dim3((cnt + 255) / 256, S * G), dim3(256), 0, st,
                       input, index, B, G, cnt, Cg, HW, part, rows);
    if ((rc = check_launch("index_colsum_kernel"))) return rc;
    hipLaunchKernelGGL(index_mean_kernel, dim3((C + 255) / 256), dim3(256), 0, st, part, rows, S, C, HW, mean,
                       running_mean, momentum);
    if ((rc = check_launch("index_mean_kernel"))) return rc;
    const long long total = (long long)B * G * cnt * HW;
    hipLaunchKernelGGL(index_shift_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                       input, index, mean, total, G, cnt, Cg, HW, output);
    return check_launch("index_shift_kernel");
}
