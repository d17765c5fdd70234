// l-inf distance, masked order-statistic neuron and interval-bound forward entry points.
#include "fwd_tile.h"
#include "fwd_args.h"

using namespace sd;

// forward with positions: chunk-tracking kernel (split-N through the packed workspace when the
// grid would otherwise be too small) followed by the position resolve pass
template <class P>
static int run_chunk_pos(FwdArgs& a, bool index_lists, hipStream_t st) {
    // with index lists a batch tile must stay inside one 32-sample sub-batch
    const int TB = (index_lists || a.R <= 32) ? 2 : 4;
    a.nsplit = pick_nsplit(a, 16 * TB, 128);
    int rc;
    if (a.nsplit > 1) {
        size_t n = (size_t)a.R * a.G * a.COg;
        a.packed0 = static_cast<unsigned long long*>(workspace(n * 8));
        if (!a.packed0) return SD_ERR_HIP;
        if ((rc = fill_zero(a.packed0, n * 2, st))) return rc;
    }
    rc = TB == 2 ? launch_fwd<P, 2, 8>(a, st) : launch_fwd<P, 4, 8>(a, st);
    if (rc) return rc;
    return launch_resolve(a, st);
}

extern "C" int sd_inf_dist_forward_nograd(const float* input, const float* weight,
                                          int B, int CO, int CI, int G, int HW, float* output, sd_stream_t stream) {
    FwdArgs a;
    int rc = make_fwd_args(a, "inf_dist_forward_nograd", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(output, "inf_dist_forward_nograd: null output");
    a.y0 = output;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int TB = a.R <= 32 ? 2 : a.R <= 64 ? 4 : 8;
    a.nsplit = pick_nsplit(a, 16 * TB, 128);
    if (a.nsplit > 1 && (rc = fill_zero(output, (size_t)B * CO * HW, st))) return rc;
    if (TB == 2) return launch_fwd<LinfNograd, 2, 8>(a, st);
    if (TB == 4) return launch_fwd<LinfNograd, 4, 8>(a, st);
    return launch_fwd<LinfNograd, 8, 8>(a, st);
}

extern "C" int sd_inf_dist_forward(const float* input, const float* weight,
                                   int B, int CO, int CI, int G, int HW, float* output, int* pos,
                                   const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                   sd_stream_t stream) {
    FwdArgs a;
    int rc = make_fwd_args(a, "inf_dist_forward", input, nullptr, weight, B, CO, CI, G, HW,
                           w_index_ci, w_index_co, W_CO, W_CI);
    if (rc) return rc;
    SD_REQUIRE(output && pos, "inf_dist_forward: null output or pos");
    a.y0 = output; a.p0 = pos;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return run_chunk_pos<LinfChunk>(a, w_index_ci || w_index_co, st);
}

extern "C" int sd_masked_inf_dist_forward(const float* input, const float* weight,
                                          int B, int CO, int CI, int G, int HW, float* output, int* pos,
                                          float q, uint32_t seed, int mode, sd_stream_t stream) {
    FwdArgs a;
    int rc = make_fwd_args(a, "masked_inf_dist_forward", input, nullptr, weight, B, CO, CI, G, HW, nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(output, "masked_inf_dist_forward: null output");
    SD_REQUIRE(q >= 0.f && q <= 1.f, "masked_inf_dist_forward: q=%g outside [0, 1]", (double)q);
    SD_REQUIRE(mode == SD_MASK_TERM || mode == SD_MASK_FACTORED, "masked_inf_dist_forward: unknown mask mode %d", mode);
    a.y0 = output; a.p0 = pos;
    a.q = q; a.seed = seed; a.mask_mode = mode;
    a.t8 = sd_mask_threshold8(q); a.t16 = sd_mask_threshold16(q);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = a.R <= 32;
    if (mode == SD_MASK_TERM) {
        if (pos) return run_chunk_pos<MaskedTermChunk>(a, false, st);
        return small ? launch_fwd<MaskedTerm<false>, 2, 8>(a, st) : launch_fwd<MaskedTerm<false>, 4, 8>(a, st);
    }
    // factored mask: dropped inputs / weights are replaced by NaN while staging the tiles and
    // NaN terms never win the maximum, so the plain l-inf policies apply unchanged
    if (pos) return run_chunk_pos<LinfChunk>(a, false, st);
    const int TB = a.R <= 32 ? 2 : a.R <= 64 ? 4 : 8;
    a.nsplit = pick_nsplit(a, 16 * TB, 128);
    if (a.nsplit > 1 && (rc = fill_zero(output, (size_t)B * CO * HW, st))) return rc;
    if (TB == 2) return launch_fwd<LinfNograd, 2, 8>(a, st);
    if (TB == 4) return launch_fwd<LinfNograd, 4, 8>(a, st);
    return launch_fwd<LinfNograd, 8, 8>(a, st);
}

extern "C" int sd_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight,
                                                int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                                sd_stream_t stream) {
    FwdArgs a;
    SD_REQUIRE(inputU, "bound_inf_dist_forward_nograd: null upper input");
    int rc = make_fwd_args(a, "bound_inf_dist_forward_nograd", inputL, inputU, weight, B, CO, CI, G, HW,
                           nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(outputL && outputU, "bound_inf_dist_forward_nograd: null output");
    a.y0 = outputL; a.y1 = outputU;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int TB = a.R <= 32 ? 2 : 4;
    a.nsplit = pick_nsplit(a, 16 * TB, 128);
    if (a.nsplit > 1) {
        if ((rc = fill_zero(outputL, (size_t)B * CO * HW, st))) return rc;
        if ((rc = fill_zero(outputU, (size_t)B * CO * HW, st))) return rc;
    }
    if (TB == 2) return launch_fwd<BoundNograd, 2, 8>(a, st);
    return launch_fwd<BoundNograd, 4, 8>(a, st);
}

extern "C" int sd_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight,
                                         int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                         int* posL, int* posU, sd_stream_t stream) {
    FwdArgs a;
    SD_REQUIRE(inputU, "bound_inf_dist_forward: null upper input");
    int rc = make_fwd_args(a, "bound_inf_dist_forward", inputL, inputU, weight, B, CO, CI, G, HW,
                           nullptr, nullptr, 0, 0);
    if (rc) return rc;
    SD_REQUIRE(outputL && outputU && posL && posU, "bound_inf_dist_forward: null output or pos");
    a.y0 = outputL; a.y1 = outputU; a.p0 = posL; a.p1 = posU;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a.R <= 32) return launch_fwd<BoundPos, 2, 4>(a, st);
    return launch_fwd<BoundPos, 4, 4>(a, st);
}
