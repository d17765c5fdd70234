// Shared definitions of the gfx950 distance-neuron kernels: argument block, counter RNG,
// error reporting and small utility kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/sortdist.h"

namespace sd {

constexpr float kEps = 1e-10f;            // floor of every distance (core/cuda/inf_dist_cuda.cu:14)
constexpr uint32_t kSign = 0x80000000u;   // bit 31 of pos
constexpr uint32_t kNanId = 0xffffffffu;  // "no lower-bound gradient" sentinel (bound_inf_dist_cuda.cu:12)
constexpr int kSubBatch = 32;             // samples sharing one index list (inf_dist_cuda.cu:8)

// ---- counter RNG: word = mix(mix((seed ^ stream * C1) + row) + (col + 1) * C2) ------------------
__host__ __device__ __forceinline__ uint32_t rng_mix(uint32_t h) {
    h ^= h >> 16; h *= 0x21f0aaadu;
    h ^= h >> 15; h *= 0x735a2d97u;
    h ^= h >> 15;
    return h;
}
__host__ __device__ __forceinline__ uint32_t rng_row_key(uint32_t seed, uint32_t stream, uint32_t row) {
    return rng_mix((seed ^ (stream * 0x9e3779b9u)) + row);
}
__host__ __device__ __forceinline__ uint32_t rng_word(uint32_t key, uint32_t col) {
    return rng_mix(key + (col + 1u) * 0x85ebca6bu);
}

// ---- arguments shared by every forward tile kernel -------------------------------------------
struct FwdArgs {
    const float* x0;      // input, or lower bound
    const float* x1;      // upper bound (interval kernels)
    const float* w;
    const float* aux;     // max_output of the with-max l-p forward
    float* y0;            // output, or lower output
    float* y1;            // upper output
    int* p0;              // pos / posL / sort pos (K, B, CO, HW)
    int* p1;              // posU
    unsigned long long* packed0;  // (value bits << 32 | ~chunk) merge buffer of split-N position kernels
    unsigned long long* packed1;  // same for the upper bound of the interval kernel
    float* part0;         // split-N partial sums of the l-p forward, [nsplit][part_stride]
    float* part1;         // split-N partial maxima (online form)
    size_t part_stride;   // B * CO * HW
    const uint32_t* xmask;  // factored mask: keep bits of x rows, one word per (row, chunk), or null
    const uint32_t* wmask;  // same for w rows
    const int* ci_idx;    // (S, G, CIg) or null
    const int* co_idx;    // (S, G, COg) or null
    int B, R, HW, G;      // R = B * HW rows of the batch tile
    int COg, CIg;         // per-group output / input channels (compact sizes with index lists)
    int W_COg, W_CIg;     // per-group rows / row length of the weight tensor
    int nsplit;           // number of slices the reduction range is cut in (grid.z = G * nsplit)
    int fast_x, fast_w;   // 128-bit loads allowed for the x / w tiles
    float p, inv_p, q;
    float skip_thr;       // l-p, large p: ratios to the running scale below this cannot change the fp32 result (0 = unused)
    uint32_t seed, t8, t16;
    int mask_mode;        // -1 none, SD_MASK_TERM, SD_MASK_FACTORED
    // device-side choice between two kernels queued for the same result (gated policies only): the kernel runs
    // when gate is null or (*gate > gate_limit) == gate_above, and returns at once otherwise
    const unsigned long long* gate;
    unsigned long long gate_limit;
    int gate_above;
    // interval forward with positions: non-null and non-zero on the device when a table kernel has already stored the
    // final values and positions, so that resolve_bound_kernel has nothing to do
    const unsigned long long* resolved;
};

__device__ __forceinline__ bool gate_closed(const unsigned long long* gate, unsigned long long limit, int above) {
    return gate != nullptr && (*gate > limit) != (above != 0);
}

// ---- error reporting ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);
// records which forward tile kernel the calling thread dispatched last (sd_last_forward_kernel)
void note_forward_kernel(const char* kind, int tb, int tm);
// With sd_time_forward_kernels(1): an event on `stream` before and after a forward tile kernel's launch, for
// sd_last_forward_kernel_ms.  Nothing while the stream is being captured.
void forward_kernel_timer(hipStream_t stream, bool after);

// What sd_last_forward_term_share reads: where the candidate-table counters of the calling thread's last forward
// call lie on the device and how to turn them into the share of the terms that the call formed.
//   kind 0: no tables were queued (every term is formed)
//   kind 1: counts[0] = marked (tile, weight row, input) triples of denom0, counts[1] != 0 when the every-term kernel ran
//   kind 2: counts[0] / counts[1] = marks of the table per weight row (of denom0) / per batch row (of denom1),
//           counts[2] != 0 when the every-term kernel ran, else the per-weight-row table served iff counts[0] <= limit0
//   kind 3: counts[0] = marks of the table per batch row (of denom0), counts[1] != 0 when the every-term kernels ran,
//           counts[2] != 0 when the per-batch-row table served, counts[3] = marks of the table per weight row (of denom1)
void note_term_counts(const unsigned long long* counts, int kind, double denom0, double denom1, unsigned long long limit0);

#define SD_REQUIRE(cond, ...)                                   \
    do {                                                        \
        if (!(cond)) { sd::set_error(__VA_ARGS__); return SD_ERR_ARG; } \
    } while (0)

// number of compute units of the current device (cached)
int num_cus();

// grow-only scratch buffer owned by the library, one per (device, stream): split-N merges, bit masks, partial
// sums.  Work queued on different streams never shares one; calls on ONE stream use it in queue order.
// Growing waits for that stream and re-allocates (bytes == 0 returns the current buffer).
void* workspace(size_t bytes, hipStream_t stream);

// Held by an entry point while it queues its kernels.  The calls of several host threads then reach their streams
// one after the other, whole, so that a stream's workspace is used in call order even when threads share the stream
// (as they do by default); only the queueing is serialised, the work of different streams still overlaps.
class CallGuard {
public:
    CallGuard();
    ~CallGuard();
    CallGuard(const CallGuard&) = delete;
    CallGuard& operator=(const CallGuard&) = delete;
};

// Whether a call site's candidate tables have paid lately.  Calls that queue a table kernel and an every-term kernel
// for one result let the device choose, and report afterwards which ran (hint_record: an 8-byte copy of the device's
// flag into pinned host memory, read by a later call once its event has completed; nothing waits).  When the every-term
// kernel ran kHintStreak times in a row for a (site, weight matrix, shape) - a layer - the next kHintSkip calls do not build tables at all
// (hint_build_tables returns false), then one call probes again.  A performance hint only: results do not depend on
// it.  Neither function does anything while `stream` is being captured (tables are then always built).
constexpr int kHintStreak = 3, kHintSkip = 31;
bool hint_build_tables(int site, const void* weight, int B, int CO, int CI, hipStream_t stream);
void hint_record(int site, const void* weight, int B, int CO, int CI, const unsigned long long* every_term_ran,
                 hipStream_t stream);

// zero-fill n floats on `stream` with a kernel (graph-capture friendly, no memset node)
int fill_zero(void* ptr, size_t n_words, hipStream_t stream);
// the same for two buffers with one launch
int fill_zero2(void* a, size_t na_words, void* b, size_t nb_words, hipStream_t stream);

}  // namespace sd
