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

// sum of one wave-uniform value per wavefront over the four wavefronts of a workgroup.  `part` holds one slot
// per wavefront and call parity, so one barrier per call is enough.
__device__ __forceinline__ int block_sum_uniform(int v, int (*part)[4], int parity) {
    if ((threadIdx.x & 63) == 0) part[parity][threadIdx.x >> 6] = v;
    __syncthreads();
    return part[parity][0] + part[parity][1] + part[parity][2] + part[parity][3];
}
__device__ __forceinline__ int wave_sum(int v) {
    #pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}
// exclusive prefix over the 256 work-items in work-item order
__device__ __forceinline__ int block_exclusive_scan(int mine, int* wave_total) {
    const int tid = threadIdx.x;
    int incl = mine;
    #pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int v = __shfl_up(incl, off);
        if ((tid & 63) >= off) incl += v;
    }
    if ((tid & 63) == 63) wave_total[tid >> 6] = incl;
    __syncthreads();
    int before = incl - mine;
    for (int w = 0; w < (tid >> 6); w++) before += wave_total[w];
    return before;
}

// One workgroup per (sub-batch, group); work-item t owns the channels [t * per, (t + 1) * per).
// The `count` smallest 48-bit keys (word << 16 | channel) are the keys whose word is below the count-th smallest
// word w, plus the lowest channels among the keys whose word equals w.
//
// CACHED (C <= 256 * kCached): the words stay in registers; w is found by a radix selection over the 32-bit word
// range (three LDS histograms: bits 31..20, 19..8, 7..0, each followed by a scan that names the bin holding the
// count-th smallest word among those that match the bins chosen so far), and ties on w are ranked by the ordered
// scan.  (A bisection over the word range, 32 rounds of counting with a barrier each, took 60 us and more for 16
// sub-batches of 5120 channels: the kernel occupies 16 compute units and every round is latency.)
// Otherwise the words are recomputed and the threshold is found by bisection over the whole 48-bit key range.
constexpr int kCached = 32;

template <bool CACHED>
__global__ void __launch_bounds__(256) sample_index_lists_kernel(uint32_t seed, int C, int count, int* __restrict__ out) {
    __shared__ int part[2][4];
    __shared__ int wave_total[4];
    __shared__ int hist[CACHED ? 4096 : 1];
    __shared__ int sel[2];
    const int tid = threadIdx.x;
    const uint32_t rowkey = rng_row_key(seed, 4u, blockIdx.x);
    const int per = (C + 255) / 256;
    const int c0 = tid * per, c1 = c0 + per < C ? c0 + per : C;
    int* dst = out + (size_t)blockIdx.x * count;
    if (CACHED) {
        uint32_t word[kCached];
        #pragma unroll
        for (int i = 0; i < kCached; i++) word[i] = rng_word(rowkey, (uint32_t)(c0 + i));
        // smallest w with #{word <= w} >= count: its bits from the top, `remaining` = its rank among the words
        // that share the bits found so far
        uint32_t w = 0u;
        int remaining = count;
        #pragma unroll
        for (int level = 0; level < 3; level++) {
            const int shift = level == 0 ? 20 : level == 1 ? 8 : 0;
            const int nbins = level == 2 ? 256 : 4096, own = nbins / 256;
            for (int k = tid; k < nbins; k += 256) hist[k] = 0;
            __syncthreads();
            #pragma unroll
            for (int i = 0; i < kCached; i++) {
                const bool match = level == 0 || (level == 1 ? (word[i] >> 20) == (w >> 20) : (word[i] >> 8) == (w >> 8));
                if (c0 + i < c1 && match) atomicAdd(&hist[(word[i] >> shift) & (uint32_t)(nbins - 1)], 1);
            }
            __syncthreads();
            int local = 0;
            for (int k = 0; k < own; k++) local += hist[tid * own + k];
            int running = block_exclusive_scan(local, wave_total);
            for (int k = 0; k < own; k++) {
                const int h = hist[tid * own + k];
                if (running < remaining && running + h >= remaining) { sel[0] = tid * own + k; sel[1] = running; }
                running += h;
            }
            __syncthreads();
            w |= (uint32_t)sel[0] << shift;
            remaining -= sel[1];
            __syncthreads();   // sel, hist and wave_total are rewritten by the next level
        }
        int below = 0, ties = 0;
        #pragma unroll
        for (int i = 0; i < kCached; i++) {
            below += (c0 + i < c1 && word[i] < w) ? 1 : 0;
            ties += (c0 + i < c1 && word[i] == w) ? 1 : 0;
        }
        const int all_below = block_sum_uniform(wave_sum(below), part, 0);     // parity 0 was last written 2 calls ago
        const int take = count - all_below;                                    // ties to keep, >= 1
        const int before = block_exclusive_scan(below | (ties << 16), wave_total);
        int tie_rank = before >> 16;
        int pos = (before & 0xffff) + (tie_rank < take ? tie_rank : take);
        #pragma unroll
        for (int i = 0; i < kCached; i++) {
            if (c0 + i < c1) {
                bool keep = word[i] < w;
                if (word[i] == w) keep = tie_rank++ < take;
                if (keep) dst[pos++] = c0 + i;
            }
        }
    } else {
        auto below = [&](unsigned long long T) {
            int cnt = 0;
            for (int c = c0; c < c1; c++) cnt += sample_key(rowkey, (uint32_t)c) < T ? 1 : 0;
            return cnt;
        };
        // smallest T with #{keys < T} >= count (keys are distinct); every work-item follows the same interval
        unsigned long long lo = 0ull, hi = 1ull << 48;
        for (int it = 0; it < 48; it++) {
            const unsigned long long mid = lo + ((hi - lo) >> 1);
            if (block_sum_uniform(wave_sum(below(mid)), part, it & 1) >= count) hi = mid; else lo = mid + 1;
        }
        int pos = block_exclusive_scan(below(hi), wave_total);
        for (int c = c0; c < c1; c++)
            if (sample_key(rowkey, (uint32_t)c) < hi) dst[pos++] = c;
    }
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
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    SD_REQUIRE(S > 0 && G > 0 && C > 0 && C < 65536, "sample_index_lists: need S, G > 0 and 0 < C < 65536");
    SD_REQUIRE(count >= 0 && count <= C, "sample_index_lists: count=%d outside 0..C=%d", count, C);
    if (count == 0) return SD_OK;
    SD_REQUIRE(out, "sample_index_lists: null output");
    if (C <= 256 * kCached)
        hipLaunchKernelGGL(sample_index_lists_kernel<true>, dim3(S * G), dim3(256), 0, static_cast<hipStream_t>(stream),
                           seed, C, count, out);
    else
        hipLaunchKernelGGL(sample_index_lists_kernel<false>, dim3(S * G), dim3(256), 0, static_cast<hipStream_t>(stream),
                           seed, C, count, out);
    return check_launch("sample_index_lists_kernel");
}
