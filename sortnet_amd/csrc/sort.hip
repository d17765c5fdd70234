// Sort-neuron forward entry points (top-K order statistics with geometric weights), K = 2..25 as
// in the reference's instantiation table (core/cuda/sort_neuron.cu:403-534).
#include "fwd_tile.h"
#include "fwd_args.h"
#include "sort_cols.h"
#include "row_cands.h"
#include <atomic>

using namespace sd;

#define SD_FOR_EACH_K(X) \
    X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16) X(17) \
    X(18) X(19) X(20) X(21) X(22) X(23) X(24) X(25)

static int check_qk(const char* who, float q, int K, int CIg) {
    SD_REQUIRE(K >= 2 && K <= 25, "%s: K=%d outside 2..25", who, K);
    SD_REQUIRE(q > 0.f && q <= 1.f, "%s: q=%g outside (0, 1]", who, (double)q);
    (void)CIg;
    return SD_OK;
}

// Second pass of the two-level sort neuron.  One workgroup per weight row: the row is staged in LDS once
// (chunks of KT floats, each followed by 4 floats of padding so that work-items reading different chunks hit
// different banks) and every work-item resolves one output of that row at a time, reading the candidate
// chunks of its input row (128-bit loads) against the staged weights.  VALUES: the K largest candidate values
// by branch-free insertion; otherwise the reference's ordered insertion with indices over the candidates in
// ascending input order (the chunk numbers are sorted first), which ends in the same list as the scan over
// all inputs because every left-out term is smaller than the final K-th value.
constexpr int kSortRowMax = 12288;   // inputs per weight row this path stages
constexpr int kChunkPad = KT + 4;

template <int K, bool VALUES>
__global__ void __launch_bounds__(256) sort_rows_kernel(FwdArgs a, const int* __restrict__ keys) {
    constexpr int KP = K + kKeySlack;
    extern __shared__ __attribute__((aligned(16))) float wrow[];
    if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return;   // one of two queued for the result
    const int c = blockIdx.x;                      // g * COg + m
    const int g = c / a.COg;
    const float* wsrc = a.w + (size_t)c * a.CIg;
    for (int n = threadIdx.x * 4; n < a.CIg; n += 1024)
        *reinterpret_cast<float4*>(wrow + (n / KT) * kChunkPad + (n % KT)) = *reinterpret_cast<const float4*>(wsrc + n);
    __syncthreads();
    const size_t size = (size_t)a.B * a.G * a.COg;
    const int nchunks = (a.CIg + KT - 1) / KT;
    for (int b = threadIdx.x; b < a.B; b += 256) {
        const size_t o = (size_t)b * a.G * a.COg + c;
        const float* xr = a.x0 + (size_t)(b * a.G + g) * a.CIg;
        float res[K];
        int idx[K];
        #pragma unroll
        for (int k = 0; k < K; k++) { res[k] = 0.f; idx[k] = 0; }
        auto chunk = [&](int cid) {
            const int n0 = cid * KT;
            const float* wc = wrow + cid * kChunkPad;
            #pragma unroll
            for (int q4 = 0; q4 < KT / 4; q4++) {
                int n = n0 + 4 * q4;
                const bool in = n < a.CIg;           // CIg is a multiple of 4 on this path
                if (!in) n = a.CIg - 4;
                const float4 xv = *reinterpret_cast<const float4*>(xr + n);
                const float4 wv = *reinterpret_cast<const float4*>(wc + (n - n0));
                const float d[4] = {xv.x - wv.x, xv.y - wv.y, xv.z - wv.z, xv.w - wv.w};
                #pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float v = in ? fabsf(d[e]) : 0.f;
                    if (VALUES) topk_insert_values<K>(res, v);
                    else if (v > res[0]) topk_insert<K>(res, idx, v, (n + e) | (d[e] >= 0.f ? 0 : (int)kSign));
                }
            }
        };
        uint32_t key[KP];
        #pragma unroll
        for (int k = 0; k < KP; k++) key[k] = (uint32_t)keys[((size_t)k * a.G * a.COg + c) * a.B + b];
        // keys ascend: key[KP - K] is the K-th largest; chunks whose truncated maximum reaches it are candidates
        const uint32_t cut = key[KP - K] >> kKeyIdBits;
        if (cut != 0u && (key[0] >> kKeyIdBits) == cut) {
            for (int cid = 0; cid < nchunks; cid++) chunk(cid);     // too many chunks share the cut value
        } else {
            int ids[KP];
            #pragma unroll
            for (int k = 0; k < KP; k++) {
                const uint32_t bucket = key[k] >> kKeyIdBits;
                ids[k] = (bucket != 0u && bucket >= cut) ? (int)(key[k] & ((1u << kKeyIdBits) - 1u)) : 0x7fffffff;
            }
            if (!VALUES) {
                // ascending chunk numbers (odd-even transposition network; skipped slots sort to the end)
                #pragma unroll
                for (int i = 0; i < KP; i++) {
                    #pragma unroll
                    for (int k = i & 1; k + 1 < KP; k += 2) {
                        int lo = min(ids[k], ids[k + 1]), hi = max(ids[k], ids[k + 1]);
                        ids[k] = lo; ids[k + 1] = hi;
                    }
                }
            }
            #pragma unroll
            for (int k = 0; k < KP; k++) {
                if (ids[k] < nchunks) chunk(ids[k]);
            }
        }
        a.y0[o] = geo_sum<K>(res, a.q);
        if (!VALUES) {
            #pragma unroll
            for (int k = K - 1; k >= 0; k--) a.p0[(size_t)(K - 1 - k) * size + o] = idx[k];
        }
    }
}

// two-level path: dense vector-load case with a reduction long enough for the chunk lists to pay
static bool two_level_ok(const FwdArgs& a, int K) {
    const int nchunks = (a.CIg + KT - 1) / KT;
    return a.HW == 1 && a.fast_x && a.fast_w && a.CIg <= kSortRowMax && K <= 12 && nchunks >= 4 * K &&
           nchunks <= (1 << kKeyIdBits);
}

// bytes of the two-level path's key lists
static size_t two_level_bytes(const FwdArgs& a, int K) {
    return (size_t)(K + kKeySlack) * ((size_t)a.R * a.G * a.COg) * sizeof(int);
}

// `keys`: two_level_bytes() of workspace
template <int K, bool VALUES>
static int run_two_level(FwdArgs& a, bool small, int* keys, hipStream_t st) {
    FwdArgs t = a;
    t.p0 = keys;
    int rc = small ? launch_fwd<SortChunkKeys<K>, 1, 2>(t, st) : launch_fwd<SortChunkKeys<K>, 2, 4>(t, st);
    if (rc) return rc;
    const int nchunks = (a.CIg + KT - 1) / KT;
    hipLaunchKernelGGL((sort_rows_kernel<K, VALUES>), dim3((unsigned)(a.G * a.COg)), dim3(256),
                       (size_t)nchunks * kChunkPad * sizeof(float), st, a, keys);
    return check_launch("sort_rows_kernel");
}

// Dense single-group layers: a kernel that works from per-weight-row candidate tables is queued in front of the
// kernels that evaluate every term, and a count taken on the device decides which of the two runs (at most
// kSortColsCap of the terms marked: the table kernel).  Negative g_sort_density: built-in limit, and only layers
// large enough for the tables to pay; 0 never; up to 1: that share, at any size.
static std::atomic<float> g_sort_density{-1.f};
constexpr float kSortColsCap = 0.10f;
constexpr long long kSortColsMinTerms = 1ll << 24;

// `site`: which entry point asks (with the built-in limit, a layer whose tables have not paid lately is not given
// any for a while, see hint_build_tables)
constexpr int kHintSiteSort = 2, kHintSiteBoundSort = 3, kHintSiteSortPos = 6;
// shape and size alone: the workspace is sized by this, so that a call under graph capture (which always builds
// tables) never needs more than the eager call before it did
static bool sort_cols_eligible(const FwdArgs& a, int B, int CO, int CI, int G, int HW) {
    const float density = g_sort_density.load(std::memory_order_relaxed);
    // the mark lists of the table kernels hold 16-bit input numbers
    if (density == 0.f || G != 1 || HW != 1 || CI % kSortColsChunk != 0 || CI > 65536 || !a.fast_x || !a.fast_w) return false;
    return density > 0.f || (long long)B * CO * CI >= kSortColsMinTerms;
}
// eligible, and (with the built-in limit) the layer's tables have paid lately
static bool sort_cols_ok(const FwdArgs& a, int site, int B, int CO, int CI, hipStream_t st) {
    return g_sort_density.load(std::memory_order_relaxed) > 0.f || hint_build_tables(site, a.w, B, CO, CI, st);
}
// after the every-term kernels have been queued behind the table kernel
static void sort_cols_report(const FwdArgs& a, int site, int B, int CO, int CI, hipStream_t st) {
    if (g_sort_density.load(std::memory_order_relaxed) < 0.f && a.gate) hint_record(site, a.w, B, CO, CI, a.gate, st);
}

// Largest share of marked (tile of 128 weight rows, batch row, input) triples at which the kernel of the tables per
// batch row runs.  Measured per 512 x 5120 x 5120 layer at K = 10 on inputs in [0, 1] against weights ~ N(0, 1/N)
// (7.2 % marked): values 0.58 ms against 1.9 ms for every term, interval bounds 0.95 against 3.3, values with positions
// 0.83 against 2.4; 0.16 ms of that are tables and the transposed copy of the weights, the rest grows with the marks
// (the two would meet at 25 to 30 %).
constexpr float kSortRowsCap = 0.22f;
// Smallest layers (in terms) given tables per batch row under the built-in limit (128 x 3072 x 1024, 0.4 G terms:
// values 0.12 ms from tables against 0.14 ms for every term, with positions 0.16 against 0.19, interval bounds 0.17
// against 0.32)
constexpr long long kSortRowsMinTerms = 1ll << 28;

// bytes of both tables' workspace for one call: per weight row first (with the probe and the counter the per-batch-row
// tables read), per batch row behind it
static size_t sort_tables_bytes(int form, int B, int CO, int CI, int K) {
    const size_t cols = (sort_cols_workspace(B, CO, CI, K) + 255) / 256 * 256;
    return cols + (row_cands_supported(form, K) ? (row_cands_workspace(form, B, CO, CI, K) + 255) / 256 * 256 : 0);
}

// `ws`: sort_tables_bytes() bytes.  The gate it leaves in `a` points into `ws`: the kernels queued behind it must
// not be given memory that overlaps it, and `ws` must stay allocated until they have run (one workspace request
// per call, carved by the caller).  Afterwards a.gate[0] is non-zero when the every-term kernels are to run.
static int queue_sort_cols(FwdArgs& a, int form, const float* xl, const float* xu, const float* w, int B, int CO, int CI,
                           float q, int K, float* outL, float* outU, int* pos, void* ws, hipStream_t st) {
    const float density = g_sort_density.load(std::memory_order_relaxed);
    const float cap = density > 0.f ? density : kSortColsCap;
    int rc = sort_cols_forward(xl, xu, w, B, CO, CI, q, K, outL, outU, pos, ws, cap, &a.gate, &a.gate_limit, st);
    a.gate_above = 1;
    const long long terms = (long long)B * CO * CI;
    const bool rows = row_cands_supported(form, K) &&
                      (density > 0.f || terms >= kSortRowsMinTerms);
    if (rc || !rows) {
        // the every-term kernels read the flag behind the counter, as with both tables
        if (!rc) { a.gate = a.gate + 1; a.gate_limit = 0ull; }
        return rc;
    }
    const unsigned long long* col_count = a.gate;
    char* rows_ws = static_cast<char*>(ws) + (sort_cols_workspace(B, CO, CI, K) + 255) / 256 * 256;
    const unsigned long long* every = nullptr;
    rc = row_cands_forward(form, xl, xu, w, nullptr, nullptr, B, CO, CI, q, K, outL, outU, pos, rows_ws,
                           density > 0.f ? density : kSortRowsCap, density > 0.f, sort_cols_probe_sums(col_count), col_count, &every, st);
    if (rc) return rc;
    a.gate = every;
    a.gate_limit = 0ull;
    note_term_counts(every - 1, 3, (double)((CO + 127) / 128) * B * CI, (double)((B + 127) / 128) * CO * CI, 0ull);
    return SD_OK;
}

extern "C" int sd_set_sort_candidate_density(float density) {
    SD_REQUIRE(density <= 1.f, "set_sort_candidate_density: %g is above 1", (double)density);
    g_sort_density = density;
    return SD_OK;
}

// few output tiles: 16 x 32 tiles instead of 32 x 64 (the top-K lists do not merge across a split reduction)
static bool few_tiles(const FwdArgs& a, int BB, int BM) {
    long long tiles = (long long)((a.R + BB - 1) / BB) * ((a.COg + BM - 1) / BM) * a.G;
    return tiles < 2ll * num_cus();
}

extern "C" int sd_sort_neuron_forward_nograd(const float* input, const float* weight,
                                             int B, int CO, int CI, int G, int HW, float* output, float q, int K,
                                             sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "sort_neuron_forward_nograd", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    if ((rc = check_qk("sort_neuron_forward_nograd", q, K, a.CIg))) return rc;
    SD_REQUIRE(output, "sort_neuron_forward_nograd: null output");
    a.y0 = output; a.q = q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = few_tiles(a, 32, 64);
    const bool two = K <= 12 && two_level_ok(a, K), elig = sort_cols_eligible(a, B, CO, CI, G, HW);
    const bool cols = elig && sort_cols_ok(a, kHintSiteSort, B, CO, CI, st);
    // one request for both users of the workspace: the tables (with the counter the gates read) first, the key
    // lists of the two-level path behind them
    const size_t tbytes = elig ? sort_tables_bytes(kRowsSortValues, B, CO, CI, K) : 0;
    char* base = nullptr;
    if (elig || two) {
        base = static_cast<char*>(workspace(tbytes + (two ? two_level_bytes(a, K) : 0), st));
        if (!base) return SD_ERR_HIP;
    }
    int* keys = reinterpret_cast<int*>(base + tbytes);
    if (cols && (rc = queue_sort_cols(a, kRowsSortValues, input, nullptr, weight, B, CO, CI, q, K, nullptr, output, nullptr, base, st))) return rc;
    rc = SD_ERR_ARG;
    switch (K) {
#define X(k) case k: if (k <= 12 && two) rc = run_two_level<(k <= 12 ? k : 2), true>(a, small, keys, st); \
                     else rc = small ? launch_fwd<SortNograd<k>, 1, 2>(a, st) : launch_fwd<SortNograd<k>, 2, 4>(a, st); \
                     break;
        SD_FOR_EACH_K(X)
#undef X
    }
    if (cols && rc == SD_OK) sort_cols_report(a, kHintSiteSort, B, CO, CI, st);
    return rc;
}

extern "C" int sd_sort_neuron_forward(const float* input, const float* weight,
                                      int B, int CO, int CI, int G, int HW, float* output, int* pos, float q, int K,
                                      sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    int rc = make_fwd_args(a, "sort_neuron_forward", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    if ((rc = check_qk("sort_neuron_forward", q, K, a.CIg))) return rc;
    SD_REQUIRE(output && pos, "sort_neuron_forward: null output or pos");
    SD_REQUIRE((long long)K * B * CO * HW < (1ll << 31), "sort_neuron_forward: pos too large for 32-bit indexing");
    a.y0 = output; a.p0 = pos; a.q = q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = few_tiles(a, 32, 32);
    const bool two = K <= 12 && two_level_ok(a, K);
    const bool elig = sort_cols_eligible(a, B, CO, CI, G, HW);
    const bool cols = elig && sort_cols_ok(a, kHintSiteSortPos, B, CO, CI, st);
    // one request for both users of the workspace, as in sd_sort_neuron_forward_nograd
    const size_t tbytes = elig ? sort_tables_bytes(kRowsSortPos, B, CO, CI, K) : 0;
    char* base = nullptr;
    if (elig || two) {
        base = static_cast<char*>(workspace(tbytes + (two ? two_level_bytes(a, K) : 0), st));
        if (!base) return SD_ERR_HIP;
    }
    int* keys = reinterpret_cast<int*>(base + tbytes);
    if (cols && (rc = queue_sort_cols(a, kRowsSortPos, input, nullptr, weight, B, CO, CI, q, K, nullptr, output, pos, base, st))) return rc;
    rc = SD_ERR_ARG;
    switch (K) {
#define X(k) case k: if (k <= 12 && two) rc = run_two_level<(k <= 12 ? k : 2), false>(a, few_tiles(a, 32, 64), keys, st); \
                     else rc = small ? launch_fwd<SortPos<k>, 1, 2>(a, st) : launch_fwd<SortPos<k>, 2, 2>(a, st); \
                     break;
        SD_FOR_EACH_K(X)
#undef X
    }
    if (cols && rc == SD_OK) sort_cols_report(a, kHintSiteSortPos, B, CO, CI, st);
    return rc;
}

extern "C" int sd_bound_sort_neuron_forward(const float* inputL, const float* inputU, const float* weight,
                                            int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                            float q, int K, sd_stream_t stream) {
    sd::CallGuard call_guard;   // calls of several host threads reach a stream one after the other, whole
    FwdArgs a;
    SD_REQUIRE(inputU, "bound_sort_neuron_forward: null upper input");
    int rc = make_fwd_args(a, "bound_sort_neuron_forward", inputL, inputU, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    if ((rc = check_qk("bound_sort_neuron_forward", q, K, a.CIg))) return rc;
    SD_REQUIRE(outputL && outputU, "bound_sort_neuron_forward: null output");
    a.y0 = outputL; a.y1 = outputU; a.q = q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = few_tiles(a, 32, 32);
    const bool elig = sort_cols_eligible(a, B, CO, CI, G, HW);
    const bool cols = elig && sort_cols_ok(a, kHintSiteBoundSort, B, CO, CI, st);
    if (elig) {
        void* ws = workspace(sort_tables_bytes(kRowsSortInterval, B, CO, CI, K), st);   // the only request of this call
        if (!ws) return SD_ERR_HIP;
        if (cols && (rc = queue_sort_cols(a, kRowsSortInterval, inputL, inputU, weight, B, CO, CI, q, K, outputL, outputU, nullptr, ws, st))) return rc;
    }
    rc = SD_ERR_ARG;
    switch (K) {
#define X(k) case k: rc = small ? launch_fwd<BoundSort<k>, 1, 2>(a, st) : launch_fwd<BoundSort<k>, 2, 2>(a, st); break;
        SD_FOR_EACH_K(X)
#undef X
    }
    if (cols && rc == SD_OK) sort_cols_report(a, kHintSiteBoundSort, B, CO, CI, st);
    return rc;
}
