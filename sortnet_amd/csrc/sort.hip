// Sort-neuron forward entry points (top-K order statistics with geometric weights), K = 2..25 as
// in the reference's instantiation table (core/cuda/sort_neuron.cu:403-534).
#include "fwd_tile.h"
#include "fwd_args.h"

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

// few output tiles: 16 x 32 tiles instead of 32 x 64 (the top-K lists do not merge across a split reduction)
static bool few_tiles(const FwdArgs& a, int BB, int BM) {
    long long tiles = (long long)((a.R + BB - 1) / BB) * ((a.COg + BM - 1) / BM) * a.G;
    return tiles < 2ll * num_cus();
}

extern "C" int sd_sort_neuron_forward_nograd(const float* input, const float* weight,
                                             int B, int CO, int CI, int G, int HW, float* output, float q, int K,
                                             sd_stream_t stream) {
    FwdArgs a;
    int rc = make_fwd_args(a, "sort_neuron_forward_nograd", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    if ((rc = check_qk("sort_neuron_forward_nograd", q, K, a.CIg))) return rc;
    SD_REQUIRE(output, "sort_neuron_forward_nograd: null output");
    a.y0 = output; a.q = q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = few_tiles(a, 32, 64);
    switch (K) {
#define X(k) case k: return small ? launch_fwd<SortNograd<k>, 1, 2>(a, st) : launch_fwd<SortNograd<k>, 2, 4>(a, st);
        SD_FOR_EACH_K(X)
#undef X
    }
    return SD_ERR_ARG;
}

extern "C" int sd_sort_neuron_forward(const float* input, const float* weight,
                                      int B, int CO, int CI, int G, int HW, float* output, int* pos, float q, int K,
                                      sd_stream_t stream) {
    FwdArgs a;
    int rc = make_fwd_args(a, "sort_neuron_forward", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    if ((rc = check_qk("sort_neuron_forward", q, K, a.CIg))) return rc;
    SD_REQUIRE(output && pos, "sort_neuron_forward: null output or pos");
    SD_REQUIRE((long long)K * B * CO * HW < (1ll << 31), "sort_neuron_forward: pos too large for 32-bit indexing");
    a.y0 = output; a.p0 = pos; a.q = q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = few_tiles(a, 32, 32);
    switch (K) {
#define X(k) case k: return small ? launch_fwd<SortPos<k>, 1, 2>(a, st) : launch_fwd<SortPos<k>, 2, 2>(a, st);
        SD_FOR_EACH_K(X)
#undef X
    }
    return SD_ERR_ARG;
}

extern "C" int sd_bound_sort_neuron_forward(const float* inputL, const float* inputU, const float* weight,
                                            int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                            float q, int K, sd_stream_t stream) {
    FwdArgs a;
    SD_REQUIRE(inputU, "bound_sort_neuron_forward: null upper input");
    int rc = make_fwd_args(a, "bound_sort_neuron_forward", inputL, inputU, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    if ((rc = check_qk("bound_sort_neuron_forward", q, K, a.CIg))) return rc;
    SD_REQUIRE(outputL && outputU, "bound_sort_neuron_forward: null output");
    a.y0 = outputL; a.y1 = outputU; a.q = q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = few_tiles(a, 32, 32);
    switch (K) {
#define X(k) case k: return small ? launch_fwd<BoundSort<k>, 1, 2>(a, st) : launch_fwd<BoundSort<k>, 2, 2>(a, st);
        SD_FOR_EACH_K(X)
#undef X
    }
    return SD_ERR_ARG;
}
