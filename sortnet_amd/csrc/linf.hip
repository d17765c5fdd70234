// l-inf distance, masked order-statistic neuron and interval-bound forward entry points.
#include "fwd_tile.h"
#include "fwd_args.h"
#include "bound_cols.h"
#include "sort_cols.h"
#include "row_cands.h"
#include <atomic>
#include <mutex>
#include <type_traits>

using namespace sd;

// largest share of marked (tile, weight row, input) triples at which the candidate-table kernel of the interval
// forward runs instead of the kernel that evaluates every term (sd_set_bound_candidate_density); negative: built-in
static std::atomic<float> g_bound_density{-1.f};
// measured at B = 512, M = N = 5120: the table kernel takes 0.09 + 2.6 x share ms (about 60 SIMD cycles per marked
// (tile, weight row, input)) after 0.10 ms for the tables, against 1.03-1.09 ms for every term; the kernel of the
// tables per batch row 0.14 + 3.3 x share ms.  The tables are paid for by the time the choice is made, so the limits
// sit a little below where the table kernel alone meets the every-term kernel.
constexpr float kBoundColsCap = 0.30f, kBoundRowsCap = 0.26f;
// With the built-in limits, layers below this many terms go without tables: building them and starting the table
// kernel takes about 0.19 ms, which is what the every-term kernel needs for 2.4 G terms (512 x 10 x 5120: 0.06 ms
// for every term against 0.10 ms from tables).
constexpr long long kBoundColsMinTerms = 1ll << 31;
// The forward that also returns positions: its table kernel spends about twice as long per mark (a compare and two
// selects per output instead of a three-operand minimum or maximum) and the every-term kernel 1.5 times as long per
// term, so the limit is lower.
constexpr float kBoundPosColsCap = 0.15f;
constexpr int kHintSiteBound = 1, kHintSiteBoundSparse = 8, kHintSiteBoundPos = 9;
constexpr float kBoundSparseCap = 0.03f;   // marked share up to which the kernel without LDS staging runs
static std::atomic<int> g_bound_form{0};            // 0: chosen per layer, 1: staged tiles, 2: transposed-row walk

// The l-inf forward (plain, and under the factored mask) on dense single-group layers queues a kernel that works from
// per-weight-row candidate tables in front of the kernels that evaluate every term; a count taken on the device
// decides which runs.  Negative g_linf_density: built-in limit, layers of at least kMaxColsMinTerms terms, and not
// where the tables have not paid lately (hint_build_tables); 0 never; up to 1: that share, at any size.
static std::atomic<float> g_linf_density{-1.f};
static std::atomic<int> g_linf_depth{0};   // under the mask: inputs the bound of a weight row rests on (0 = from the keep probability)
constexpr float kMaxColsCap = 0.10f;
constexpr long long kMaxColsMinTerms = 1ll << 31;   // below, the tables cost more than evaluating every term
constexpr int kHintSiteLinf = 4, kHintSiteMasked = 5;

// Depth of the tables' bound for this shape and mask (0 = the call is not served from tables), by shape and size
// alone: the workspace is sized by this, so that a call under graph capture (which always builds tables) never needs
// more than the eager call before it did.
static int max_cols_eligible(const FwdArgs& a, float keep_x, int B, int CO, int CI, int G, int HW) {
    const float density = g_linf_density.load(std::memory_order_relaxed);
    const int depth = g_linf_depth.load(std::memory_order_relaxed);
    if (density == 0.f || G != 1 || HW != 1 || CI % kSortColsChunk != 0 || CI > 65536 || !a.fast_x || !a.fast_w ||
        a.ci_idx || a.co_idx) return 0;
    int K = max_cols_depth(keep_x);
    if (depth > 0 && keep_x < 1.f) K = depth;
    if (K == 0 || density > 0.f) return K;
    return (long long)B * CO * CI >= kMaxColsMinTerms ? K : 0;
}
// eligible depth `K`, or 0 when (with the built-in limit) the layer's tables have not paid lately
static int max_cols_wanted(const FwdArgs& a, int K, int site, int B, int CO, int CI, hipStream_t st) {
    if (K == 0 || g_linf_density.load(std::memory_order_relaxed) > 0.f) return K;
    return hint_build_tables(site, a.w, B, CO, CI, st) ? K : 0;
}

// Largest share of marked (tile of 128 weight rows, batch row, input) triples at which the l-inf kernel of the tables
// per batch row runs, and the smallest layer (in terms) given such tables under the built-in limit.  Measured on inputs
// in [0, 1] against weights ~ N(0, 1/N) (6.5 to 8.4 % marked): 512 x 5120 x 5120 0.34 ms (0.36 with positions; 0.15 ms
// of it tables and the transposed copy of the weights) against 0.49 (0.61) for every term, 256 x 12288 x 10240 0.86
// (0.89) against 1.28 (1.30), 512 x 3072 x 5120 0.26 (0.27) against 0.27 (0.43), 256 x 4096 x 2048 0.13 (0.13)
// against 0.09 (0.12): the main kernel's time grows with the marks, so the limit sits where the two would meet at the
// large sizes.  With the 512 x 3072 x 5120 layer served from tables the benchmark step gained 0.1 ms on one stream and
// lost 0.05 ms on three (presumably the table passes and the transposed copy, which stream the operands through
// memory, meet the traffic of the optimizer and the backward on the other streams), so the size limit sits above
// that layer.
constexpr float kMaxRowsCap = 0.10f;
constexpr long long kMaxRowsMinTerms = 1ll << 33;

// bytes of both tables' workspace for one call: per weight row first, per batch row behind it
static size_t max_tables_bytes(int B, int CO, int CI, int K) {
    const size_t cols = (max_cols_workspace(B, CO, CI, K) + 255) / 256 * 256;
    return cols + (row_cands_supported(kRowsMax, K) ? (row_cands_workspace(kRowsMax, B, CO, CI, K) + 255) / 256 * 256 : 0);
}

// `ws`: max_tables_bytes() bytes.  Afterwards a.gate[0] is non-zero when the every-term kernels are to run.
static int queue_max_cols(FwdArgs& a, int K, int B, int CO, int CI, void* ws, hipStream_t st) {
    const float density = g_linf_density.load(std::memory_order_relaxed);
    const float cap = density > 0.f ? density : kMaxColsCap;
    // depth 1: the mask keeps everything
    const uint32_t* xkeep = K == 1 ? nullptr : a.xmask;
    const uint32_t* wkeep = K == 1 ? nullptr : a.wmask;
    int rc = max_cols_forward(a.x0, a.w, xkeep, wkeep, B, CO, CI, K, a.y0, a.p0, ws, cap, &a.gate, &a.gate_limit, st);
    a.gate_above = 1;
    const bool rows = row_cands_supported(kRowsMax, K) && (density > 0.f || (long long)B * CO * CI >= kMaxRowsMinTerms);
    if (rc || !rows) {
        if (!rc) { a.gate = a.gate + 1; a.gate_limit = 0ull; }   // the flag behind the counter, as with both tables
        return rc;
    }
    const unsigned long long* col_count = a.gate;
    char* rows_ws = static_cast<char*>(ws) + (max_cols_workspace(B, CO, CI, K) + 255) / 256 * 256;
    const unsigned long long* every = nullptr;
    rc = row_cands_forward(kRowsMax, a.x0, nullptr, a.w, xkeep, wkeep, B, CO, CI, 0.f, K, nullptr, a.y0, a.p0, rows_ws,
                           density > 0.f ? density : kMaxRowsCap, density > 0.f, sort_cols_probe_sums(col_count), col_count, &every, st);
    if (rc) return rc;
    a.gate = every;
    a.gate_limit = 0ull;
    note_term_counts(every - 1, 3, (double)((CO + 127) / 128) * B * CI, (double)((B + 127) / 128) * CO * CI, 0ull);
    return SD_OK;
}

static void max_cols_report(const FwdArgs& a, int site, int B, int CO, int CI, hipStream_t st) {
    if (g_linf_density.load(std::memory_order_relaxed) < 0.f && a.gate) hint_record(site, a.w, B, CO, CI, a.gate, st);
}

extern "C" int sd_set_linf_candidate_density(float density) {
    SD_REQUIRE(density <= 1.f, "set_linf_candidate_density: %g is above 1", (double)density);
    g_linf_density = density;
    return SD_OK;
}

extern "C" int sd_set_linf_candidate_depth(int depth) {
    SD_REQUIRE(depth == 0 || depth == 8 || depth == 12 || depth == 16 || depth == 20 || depth == 24,
               "set_linf_candidate_depth: %d is not one of 0, 8, 12, 16, 20, 24", depth);
    g_linf_depth = depth;
    return SD_OK;
}

// One work-item per (row, chunk): the 32 keep bits of the factored mask for inputs
// chunk*32 .. chunk*32+31 of an x row (stream 1) or a w row (stream 2).
static __global__ void __launch_bounds__(256) build_masks_kernel(uint32_t* __restrict__ out, long long rows, int nchunks,
                                                          int CIg, uint32_t seed, uint32_t stream, uint32_t t16) {
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * nchunks) return;
    uint32_t row = (uint32_t)(i / nchunks);
    int chunk = (int)(i - (long long)row * nchunks);
    uint32_t key = rng_row_key(seed, stream, row);
    uint32_t bits = 0;
    #pragma unroll 8
    for (int k = 0; k < KT; k++) {
        int n = chunk * KT + k;
        if (n < CIg && (rng_word(key, (uint32_t)n) >> 16) < t16) bits |= 1u << k;
    }
    out[i] = bits;
}

// forward with positions: chunk-tracking kernel (split-N through the packed workspace when the
// grid would otherwise be too small) followed by the position resolve pass
// merge_buf / merge_cap: caller-supplied memory for the split-N merge instead of the library workspace (the entry
// point that allocates nothing); a problem that needs more than merge_cap bytes is rejected
template <class P>
static int run_chunk_pos(FwdArgs& a, bool index_lists, hipStream_t st, void* merge_buf = nullptr, size_t merge_cap = 0) {
    // with index lists a batch tile must stay inside one 32-sample sub-batch
    static const int kTb42[] = {4, 2};
    const int TB = index_lists ? 2 : pick_tb(a, kTb42, 2, 16 * P::WIDE_TM);
    const bool gather = index_lists && !(a.fast_x && a.fast_w);      // served by the scalar-load kernel
    a.nsplit = TB == 2 ? pick_nsplit(a, 32, gather ? 128 : 16 * P::WIDE_TM, gather ? 1 : 8) : pick_nsplit(a, 16 * P::WIDE_TB, 16 * P::WIDE_TM);
    // dense exact tiles of the l-inf policy: LDS-direct kernel with 4 x 8 outputs per work-item and the chunk numbers
    // packed four to a register (same (value, chunk) results, so the same resolve pass follows)
    bool packed_direct = false;
    if constexpr (std::is_same<P, LinfChunk>::value) {
        if (TB == 4 && direct_ok<4, 8>(a)) {
            const int ns = pick_nsplit(a, 64, 128);
            if ((a.CIg / KT + ns - 1) / ns <= LinfChunkPacked::MAX_CHUNKS) { packed_direct = true; a.nsplit = ns; }
        }
    }
    int rc;
    if (a.nsplit > 1) {
        // the merge buffer sits at the start of the workspace; a factored-mask call has already sized
        // the workspace for it and placed its bit masks behind it
        size_t n = (size_t)a.R * a.G * a.COg;
        if (merge_buf) {
            SD_REQUIRE(n * 8 <= merge_cap, "inf_dist_forward_noalloc: %zu outputs need %zu bytes of merge scratch, the "
                       "built-in buffer holds %zu (at most %zu outputs)", n, n * 8, merge_cap, merge_cap / 8);
            a.packed0 = static_cast<unsigned long long*>(merge_buf);
        } else a.packed0 = static_cast<unsigned long long*>(a.xmask ? workspace(0, st) : workspace(n * 8, st));
        if (!a.packed0) return SD_ERR_HIP;
        if ((rc = fill_zero(a.packed0, n * 2, st))) return rc;
    }
    if (packed_direct) {
        forward_kernel_timer(st, false);
        rc = launch_fwd_direct<LinfChunkPacked, 4, 8>(a, st);
        forward_kernel_timer(st, true);
    }
    else if (TB == 2) rc = gather ? launch_fwd<P, 2, 8>(a, st) : launch_fwd<P, 2, P::WIDE_TM>(a, st);
    else rc = launch_fwd<P, P::WIDE_TB, P::WIDE_TM>(a, st);
    if (rc) return rc;
    return launch_resolve(a, st);
}

extern "C" int sd_inf_dist_forward_nograd(const float* input, const float* weight,
                                          int B, int CO, int CI, int G, int HW, float* output, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "inf_dist_forward_nograd", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(output, "inf_dist_forward_nograd: null output");
    a.y0 = output;
    hipStream_t st = static_cast<hipStream_t>(stream);
    static const int kTb42[] = {4, 2};   // 8 rows per work-item measured slower (168 registers, three waves per SIMD)
    const int TB = pick_tb(a, kTb42, 2, 128);
    a.nsplit = pick_nsplit(a, 16 * TB, 128);
    if (a.nsplit > 1 && (rc = fill_zero(output, (size_t)B * CO * HW, st))) return rc;
    const int KE = max_cols_eligible(a, 1.f, B, CO, CI, G, HW);
    const int K = max_cols_wanted(a, KE, kHintSiteLinf, B, CO, CI, st);
    if (KE) {
        void* ws = workspace(max_tables_bytes(B, CO, CI, KE), st);   // the only request of this call
        if (!ws) return SD_ERR_HIP;
        if (K && (rc = queue_max_cols(a, K, B, CO, CI, ws, st))) return rc;
    }
    rc = TB == 2 ? launch_fwd<LinfNograd, 2, 8>(a, st) : launch_fwd<LinfNograd, 4, 8>(a, st);
    if (K && rc == SD_OK) max_cols_report(a, kHintSiteLinf, B, CO, CI, st);
    return rc;
}

extern "C" int sd_inf_dist_forward(const float* input, const float* weight,
                                   int B, int CO, int CI, int G, int HW, float* output, int* pos,
                                   const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                   sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "inf_dist_forward", input, nullptr, weight, B, CO, CI, G, HW,
                           w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(output && pos, "inf_dist_forward: null output or pos");
    a.y0 = output; a.p0 = pos;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int KE = max_cols_eligible(a, 1.f, B, CO, CI, G, HW);
    if (!KE) return run_chunk_pos<LinfChunk>(a, w_index_ci || w_index_co, st);
    const int K = max_cols_wanted(a, KE, kHintSiteLinf, B, CO, CI, st);
    // one workspace request for both users: the split-N merge buffer first, the tables (with the counter the gates
    // read) behind it
    const size_t merge = (((size_t)B * CO * 8) + 255) / 256 * 256;
    char* base = static_cast<char*>(workspace(merge + max_tables_bytes(B, CO, CI, KE), st));
    if (!base) return SD_ERR_HIP;
    if (K && (rc = queue_max_cols(a, K, B, CO, CI, base + merge, st))) return rc;
    rc = run_chunk_pos<LinfChunk>(a, false, st, base, merge);
    if (K && rc == SD_OK) max_cols_report(a, kHintSiteLinf, B, CO, CI, st);
    return rc;
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// Same operation as sd_inf_dist_forward for callers that cannot call hipMalloc (code under graph capture,
// serving loops, harnesses that forbid allocation).  The split-N merge buffer, which sd_inf_dist_forward takes
// from the grow-only library workspace, lives in a file-scope device array instead.  Every GPU holds its own
// copy of the array at its own address: the address is looked up once per device with hipGetSymbolAddress and
// only that pointer is ever handed to kernels.  All calls on one GPU share the array, so calls that overlap on
// one GPU (different streams or threads) race; the part a call uses is cleared by a fill kernel first.
constexpr size_t kScratchBytes = (size_t)32 << 20;   // 4 Mi outputs of 8 bytes: covers 512 x 5120 outputs
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

static int scratch_address(void** out) {
    static std::mutex mu;
    static void* ptrs[64] = {nullptr};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        set_error("inf_dist_forward_noalloc: no current device");
        return SD_ERR_HIP;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            set_error("inf_dist_forward_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return SD_ERR_HIP;
        }
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return SD_OK;
}

extern "C" int sd_inf_dist_forward_noalloc(const float* input, const float* weight,
                                           int B, int CO, int CI, int G, int HW, float* output, int* pos,
                                           const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                           sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "inf_dist_forward_noalloc", input, nullptr, weight, B, CO, CI, G, HW,
                           w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(output && pos, "inf_dist_forward_noalloc: null output or pos");
    a.y0 = output; a.p0 = pos;
    const size_t outputs = (size_t)B * CO * HW;
    SD_REQUIRE(outputs * 8 <= kScratchBytes, "inf_dist_forward_noalloc: %zu outputs exceed the maximum of %zu "
               "(8 bytes of built-in merge scratch per output, %zu bytes in all); use sd_inf_dist_forward",
               outputs, kScratchBytes / 8, kScratchBytes);
    void* buf = nullptr;
    if ((rc = scratch_address(&buf))) return rc;
    return run_chunk_pos<LinfChunk>(a, w_index_ci || w_index_co, static_cast<hipStream_t>(stream), buf, kScratchBytes);
}

extern "C" int sd_masked_inf_dist_forward(const float* input, const float* weight,
                                          int B, int CO, int CI, int G, int HW, float* output, int* pos,
                                          float q, uint32_t seed, int mode, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "masked_inf_dist_forward", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(output, "masked_inf_dist_forward: null output");
    SD_REQUIRE(q >= 0.f && q <= 1.f, "masked_inf_dist_forward: q=%g outside [0, 1]", (double)q);
    SD_REQUIRE(mode == SD_MASK_TERM || mode == SD_MASK_FACTORED, "masked_inf_dist_forward: unknown mask mode %d", mode);
    a.y0 = output; a.p0 = pos;
    a.q = q; a.seed = seed; a.mask_mode = mode;
    a.t8 = sd_mask_threshold8(q); a.t16 = sd_mask_threshold16(q);
    const bool small = a.R <= 32;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == SD_MASK_TERM) {
        if (pos) return run_chunk_pos<MaskedTermChunk>(a, false, st);
        a.nsplit = pick_nsplit(a, small ? 32 : 64, 128);
        if (a.nsplit > 1 && (rc = fill_zero(output, (size_t)B * CO * HW, st))) return rc;
        return small ? launch_fwd<MaskedTermMax, 2, 8>(a, st) : launch_fwd<MaskedTermMax, 4, 8>(a, st);
    }
    // factored mask: dropped inputs / weights are replaced by NaN while staging the tiles and
    // NaN terms never win the maximum, so the plain l-inf policies apply unchanged.  On the
    // vector-load path the keep bits are built once per call into the library workspace.
    size_t packed_bytes = 0;
    int K = 0;          // depth of the candidate tables' bound (0: no tables)
    void* tables = nullptr;
    if (a.fast_x && a.fast_w) {
        const int nchunks = (a.CIg + KT - 1) / KT;
        const long long xrows = (long long)a.R * G, wrows = (long long)CO;
        packed_bytes = pos ? (((size_t)a.R * CO * 8 + 255) / 256) * 256 : 0;
        // one request for every user of the workspace: merge buffer, keep bits, candidate tables
        const size_t mask_bytes = ((size_t)(xrows + wrows) * nchunks * 4 + 255) / 256 * 256;
        const int KE = max_cols_eligible(a, (float)a.t16 / 65536.f, B, CO, CI, G, HW);
        K = max_cols_wanted(a, KE, kHintSiteMasked, B, CO, CI, st);
        char* base = static_cast<char*>(workspace(packed_bytes + mask_bytes + (KE ? max_tables_bytes(B, CO, CI, KE) : 0), st));
        if (!base) return SD_ERR_HIP;
        tables = base + packed_bytes + mask_bytes;
        uint32_t* xm = reinterpret_cast<uint32_t*>(base + packed_bytes);
        uint32_t* wm = xm + xrows * nchunks;
        hipLaunchKernelGGL(build_masks_kernel, dim3((unsigned)((xrows * nchunks + 255) / 256)), dim3(256), 0, st,
                           xm, xrows, nchunks, a.CIg, seed, 1u, a.t16);
        hipLaunchKernelGGL(build_masks_kernel, dim3((unsigned)((wrows * nchunks + 255) / 256)), dim3(256), 0, st,
                           wm, wrows, nchunks, a.CIg, seed, 2u, a.t16);
        if ((rc = check_launch("build_masks_kernel"))) return rc;
        a.xmask = xm; a.wmask = wm;
    }
    if (pos) {
        if (K && (rc = queue_max_cols(a, K, B, CO, CI, tables, st))) return rc;
        rc = run_chunk_pos<LinfChunk>(a, false, st);
        if (K && rc == SD_OK) max_cols_report(a, kHintSiteMasked, B, CO, CI, st);
        return rc;
    }
    static const int kTb42[] = {4, 2};   // 8 rows per work-item measured slower (168 registers, three waves per SIMD)
    const int TB = pick_tb(a, kTb42, 2, 128);
    a.nsplit = pick_nsplit(a, 16 * TB, 128);
    if (a.nsplit > 1 && (rc = fill_zero(output, (size_t)B * CO * HW, st))) return rc;
    if (K && (rc = queue_max_cols(a, K, B, CO, CI, tables, st))) return rc;
    rc = TB == 2 ? launch_fwd<LinfNograd, 2, 8>(a, st) : launch_fwd<LinfNograd, 4, 8>(a, st);
    if (K && rc == SD_OK) max_cols_report(a, kHintSiteMasked, B, CO, CI, st);
    return rc;
}

extern "C" int sd_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight,
                                                int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                                sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    SD_REQUIRE(inputU, "bound_inf_dist_forward_nograd: null upper input");
    int rc = make_fwd_args(a, "bound_inf_dist_forward_nograd", inputL, inputU, weight, B, CO, CI, G, HW,
                           nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(outputL && outputU, "bound_inf_dist_forward_nograd: null output");
    a.y0 = outputL; a.y1 = outputU;
    hipStream_t st = static_cast<hipStream_t>(stream);
    static const int kTb42[] = {4, 2};
    const int TB = pick_tb(a, kTb42, 2, 128);
    a.nsplit = pick_nsplit(a, 16 * TB, 16 * 8);
    // dense single-group layers: a kernel that works from per-weight-row candidate tables is queued in front of the
    // one that evaluates every term, and a count taken on the device decides which of the two runs
    const float bound_density = g_bound_density.load(std::memory_order_relaxed);
    const int bound_form = g_bound_form.load(std::memory_order_relaxed);
    const float cap = bound_density >= 0.f ? bound_density : kBoundColsCap;
    bool cols = cap > 0.f && G == 1 && HW == 1 && CI % kColsChunk == 0 && a.fast_x && a.fast_w &&
                (bound_density >= 0.f || (long long)B * CO * CI >= kBoundColsMinTerms);
    // The workspace is sized by shape alone (whatever the hints below decide), so that a call under graph capture,
    // which always builds the staged tables, never needs more than the eager call before it did.
    char* wsbase = nullptr;
    if (cols) {
        const size_t staged = bound_cols_workspace(B, CO, CI), walk = CI <= 65536 ? sort_cols_workspace(B, CO, CI, 1) : 0;
        wsbase = static_cast<char*>(workspace(staged > walk ? staged : walk, st));   // the only request of this call
        if (!wsbase) return SD_ERR_HIP;
    }
    // with the built-in limit, a layer whose tables have not paid lately is not given any for a while
    const bool hinted = cols && bound_density < 0.f;
    if (hinted && !hint_build_tables(kHintSiteBound, weight, B, CO, CI, st)) cols = false;
    // Very few marks (weights of unit scale against rows that are alike: below 1 %): the staged kernel would spend its
    // time moving tiles through LDS, and the kernel that walks a weight row's marks over a transposed copy of the
    // inputs serves better.  Chosen by hand (sd_set_bound_candidate_form) or, with the built-in limit, for a layer
    // whose last three staged calls reported that few marks ("not building" the staged tables, in the hint's terms).
    bool sparse = cols && bound_form == 2 && CI <= 65536;
    if (cols && bound_form == 0 && hinted && CI <= 65536)
        sparse = !hint_build_tables(kHintSiteBoundSparse, weight, B, CO, CI, st);
    if (sparse) {
        void* ws = wsbase;
        if (a.nsplit > 1) {   // the every-term kernel, should it run, merges its slices into zeros
            if ((rc = fill_zero2(outputL, (size_t)B * CO * HW, outputU, (size_t)B * CO * HW, st))) return rc;
        }
        if ((rc = sort_cols_forward(inputL, inputU, weight, B, CO, CI, 0.f, 1, outputL, outputU, nullptr, ws,
                                    bound_density > 0.f ? bound_density : kBoundSparseCap, &a.gate, &a.gate_limit, st)))
            return rc;
        a.gate_above = 1;
        return TB == 2 ? launch_fwd<BoundNogradGated, 2, 8>(a, st) : launch_fwd<BoundNogradGated, 4, 8>(a, st);
    }
    if (a.nsplit > 1 || cols) {
        if ((rc = fill_zero2(outputL, (size_t)B * CO * HW, outputU, (size_t)B * CO * HW, st))) return rc;
    }
    if (cols) {
        void* ws = wsbase;
        if ((rc = bound_cols_forward(inputL, inputU, weight, B, CO, CI, outputL, outputU, nullptr, nullptr, nullptr, nullptr, ws, cap,
                                     bound_density >= 0.f ? bound_density : kBoundRowsCap, &a.gate, &a.gate_limit, st)))
            return rc;
        a.gate_above = 1;
        rc = TB == 2 ? launch_fwd<BoundNogradGated, 2, 8>(a, st) : launch_fwd<BoundNogradGated, 4, 8>(a, st);
        if (hinted && rc == SD_OK) {
            hint_record(kHintSiteBound, weight, B, CO, CI, a.gate, st);   // the gate is 1 when every term ran
            if (bound_form == 0) hint_record(kHintSiteBoundSparse, weight, B, CO, CI, a.gate + 1, st);   // 1: very few marks
        }
        return rc;
    }
    if (TB == 2) return launch_fwd<BoundNograd, 2, 8>(a, st);
    return launch_fwd<BoundNograd, 4, 8>(a, st);
}

extern "C" int sd_set_bound_candidate_density(float density) {
    SD_REQUIRE(density <= 1.f, "set_bound_candidate_density: %g is above 1", (double)density);
    g_bound_density = density;
    return SD_OK;
}

extern "C" int sd_set_bound_candidate_form(int form) {
    SD_REQUIRE(form >= 0 && form <= 2, "set_bound_candidate_form: %d is not 0 (automatic), 1 (staged tiles) or 2 (row walk)", form);
    g_bound_form = form;
    return SD_OK;
}

extern "C" int sd_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight,
                                         int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                         int* posL, int* posU, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    SD_REQUIRE(inputU, "bound_inf_dist_forward: null upper input");
    int rc = make_fwd_args(a, "bound_inf_dist_forward", inputL, inputU, weight, B, CO, CI, G, HW,
                           nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(outputL && outputU && posL && posU, "bound_inf_dist_forward: null output or pos");
    a.y0 = outputL; a.y1 = outputU; a.p0 = posL; a.p1 = posU;
    hipStream_t st = static_cast<hipStream_t>(stream);
    static const int kTb42[] = {4, 2};
    const int TB = pick_tb(a, kTb42, 2, 64);
    a.nsplit = pick_nsplit(a, 16 * TB, 64);
    // dense single-group layers: the table kernel, tracking the chunk of every result, is queued in front
    // of the every-term kernel as for the forward without positions; both leave (value, chunk) pairs for the resolve
    const float bound_density = g_bound_density.load(std::memory_order_relaxed);
    const float cap = bound_density >= 0.f ? bound_density : kBoundPosColsCap;
    bool cols = cap > 0.f && G == 1 && HW == 1 && CI % kColsChunk == 0 && a.fast_x && a.fast_w &&
                (bound_density >= 0.f || (long long)B * CO * CI >= kBoundColsMinTerms);
    const bool elig = cols;   // by shape alone: what the workspace is sized by (a captured call always builds tables)
    const bool hinted = cols && bound_density < 0.f;
    if (hinted && !hint_build_tables(kHintSiteBoundPos, weight, B, CO, CI, st)) cols = false;
    if (cols && a.nsplit < 2) a.nsplit = 2;   // both kernels merge into the packed pairs
    if (a.nsplit > 1 || elig) {
        size_t n = (size_t)a.R * a.G * a.COg;
        const size_t pairs = (n * 16 + 255) / 256 * 256;
        char* ws = static_cast<char*>(workspace(pairs + (elig ? bound_cols_workspace(B, CO, CI) : 0), st));   // the only request
        if (!ws) return SD_ERR_HIP;
        a.packed0 = reinterpret_cast<unsigned long long*>(ws);
        a.packed1 = a.packed0 + n;
        if (a.nsplit > 1 && (rc = fill_zero(a.packed0, n * 4, st))) return rc;
        if (cols) {
            if ((rc = bound_cols_forward(inputL, inputU, weight, B, CO, CI, outputL, outputU, a.packed0, a.packed1, posL, posU,
                                         ws + pairs, cap, cap, &a.gate, &a.gate_limit, st)))
                return rc;
            a.gate_above = 1;
            a.resolved = a.gate + 2;   // the tables per batch row store final values and positions themselves
        }
    }
    // exact dense tiles: the LDS-direct kernel with the chunk numbers packed (same (value, chunk) pairs, same resolve)
    if (TB == 4 && a.nsplit > 1 && direct_ok<4, 4>(a) && (a.CIg / KT + a.nsplit - 1) / a.nsplit <= BoundChunkPacked::MAX_CHUNKS)
        rc = launch_fwd_direct<BoundChunkPacked, 4, 4>(a, st);
    else rc = TB == 2 ? launch_fwd<BoundChunk, 2, 4>(a, st) : launch_fwd<BoundChunk, 4, 4>(a, st);
    if (rc) return rc;
    if (hinted && cols) hint_record(kHintSiteBoundPos, weight, B, CO, CI, a.gate, st);   // the gate is 1 when every term ran
    return launch_resolve_bound(a, st);
}
