// Device-side replacement of the reference's host-side mask sampling
// (core/models/norm_dist.py:14-17: count = (rand(C) < q).sum(); per (sub-batch, group) a uniformly random
// subset of exactly `count` channels, returned as ascending int32 indices).  Built on the library's
// stateless counter RNG, so the kept count can be evaluated on the host without touching the GPU and the
// index lists on the device without any host synchronisation.
//   count            = #{ c < C : word(key(3, 0), c) < q * 2^32 }
//   list (s, g)      = the `count` channels with the smallest 48-bit keys
//                      (word(key(4, s * G + g), c) << 16) | c, in ascending channel order
#include <cmath>
#include "common.h"

namespace sd {

__host__ __device__ __forceinline__ unsigned long long sample_key(uint32_t rowkey, uint32_t c) {
    return ((unsigned long long)rng_word(rowkey, c) << 16) | (unsigned long long)c;
}

__global__ void __launch_bounds__(256) sample_index_lists_kernel(uint32_t seed, int C, int count, int* __restrict__ out) {
    __shared__ int red[256];
    __shared__ unsigned long long s_lo, s_hi;
    const int tid = threadIdx.x;
    const uint32_t rowkey = rng_row_key(seed, 4u, blockIdx.x);
    // smallest T with #{keys < T} >= count, by bisection on the 48-bit key range (keys are distinct)
    if (tid == 0) { s_lo = 0ull; s_hi = 1ull << 48; }
    __syncthreads();
    for (int it = 0; it < 48; it++) {
        const unsigned long long lo = s_lo, hi = s_hi;
        const unsigned long long mid = lo + ((hi - lo) >> 1);
        int cnt = 0;
        for (int c = tid; c < C; c += 256) cnt += sample_key(rowkey, (uint32_t)c) < mid ? 1 : 0;
        red[tid] = cnt;
        __syncthreads();
        for (int s = 128; s > 0; s >>= 1) {
            if (tid < s) red[tid] += red[tid + s];
            __syncthreads();
        }
        if (tid == 0) {
            if (red[0] >= count) s_hi = mid; else s_lo = mid + 1;
        }
        __syncthreads();
    }
    const unsigned long long T = s_hi;    // #{keys < T} == count
    // ordered compaction: work-item t owns channels [t * per, (t + 1) * per)
    const int per = (C + 255) / 256;
    const int c0 = tid * per, c1 = c0 + per < C ? c0 + per : C;
    int mine = 0;
    for (int c = c0; c < c1; c++) mine += sample_key(rowkey, (uint32_t)c) < T ? 1 : 0;
    red[tid] = mine;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int t = 0; t < 256; t++) { int v = red[t]; red[t] = run; run += v; }
    }
    __syncthreads();
    int pos = red[tid];
    int* dst = out + (size_t)blockIdx.x * count;
    for (int c = c0; c < c1; c++)
        if (sample_key(rowkey, (uint32_t)c) < T) dst[pos++] = c;
}

}  // namespace sd

using namespace sd;

extern "C" int sd_mask_count(uint32_t seed, int C, float q) {
    if (C <= 0) return 0;
    double t = std::floor((double)q * 4294967296.0 + 0.5);
    if (t < 0) t = 0;
    if (t > 4294967296.0) t = 4294967296.0;
    const unsigned long long thr = (unsigned long long)t;
    const uint32_t key = rng_row_key(seed, 3u, 0u);
    int n = 0;
    for (int c = 0; c < C; c++) n += (unsigned long long)rng_word(key, (uint32_t)c) < thr ? 1 : 0;
    return n;
}

extern "C" int sd_sample_index_lists(uint32_t seed, int S, int G, int C, int count, int* out, sd_stream_t stream) {
    SD_REQUIRE(S > 0 && G > 0 && C > 0 && C < 65536, "sample_index_lists: need S, G > 0 and 0 < C < 65536");
    SD_REQUIRE(count >= 0 && count <= C, "sample_index_lists: count=%d outside 0..C=%d", count, C);
    if (count == 0) return SD_OK;
    SD_REQUIRE(out, "sample_index_lists: null output");
    hipLaunchKernelGGL(sample_index_lists_kernel, dim3(S * G), dim3(256), 0, static_cast<hipStream_t>(stream),
                       seed, C, count, out);
    return check_launch("sample_index_lists_kernel");
}
