// Host-side validation and FwdArgs construction shared by the forward entry points.
#pragma once
#include <cmath>
#include "common.h"

namespace sd {

inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// Validates the common shape arguments and fills the shape part of FwdArgs.
// Returns SD_OK or SD_ERR_ARG (message set).
inline int make_fwd_args(FwdArgs& a, const char* who, const float* x0, const float* x1, const float* w,
                         int B, int CO, int CI, int G, int HW,
                         const int* ci_idx, const int* co_idx, int W_CO, int W_CI) {
    SD_REQUIRE(x0 && w, "%s: null input or weight pointer", who);
    SD_REQUIRE(B > 0 && CO > 0 && CI > 0 && G > 0 && HW > 0, "%s: sizes must be positive (B=%d CO=%d CI=%d G=%d HW=%d)",
               who, B, CO, CI, G, HW);
    SD_REQUIRE(CO % G == 0 && CI % G == 0, "%s: CO=%d and CI=%d must be multiples of G=%d", who, CO, CI, G);
    SD_REQUIRE((long long)B * HW < (1ll << 31) && (long long)B * CO * HW < (1ll << 31) &&
               (long long)B * CI * HW < (1ll << 31), "%s: tensor too large for 32-bit indexing", who);
    a = FwdArgs{};
    note_term_counts(nullptr, 0, 1.0, 1.0, 0ull);   // until a table kernel is queued for this call
    a.x0 = x0; a.x1 = x1; a.w = w;
    a.ci_idx = ci_idx; a.co_idx = co_idx;
    a.B = B; a.R = B * HW; a.HW = HW; a.G = G;
    a.COg = CO / G; a.CIg = CI / G;
    if (co_idx) {
        SD_REQUIRE(W_CO > 0 && W_CO % G == 0, "%s: W_CO=%d must be a positive multiple of G", who, W_CO);
        a.W_COg = W_CO / G;
    } else a.W_COg = a.COg;
    if (ci_idx) {
        SD_REQUIRE(W_CI > 0 && W_CI % G == 0, "%s: W_CI=%d must be a positive multiple of G", who, W_CI);
        a.W_CIg = W_CI / G;
    } else a.W_CIg = a.CIg;
    SD_REQUIRE((long long)G * a.W_COg * a.W_CIg < (1ll << 31), "%s: weight too large for 32-bit indexing", who);
    a.nsplit = 1;
    a.mask_mode = -1;
    bool vec = HW == 1 && a.CIg % 4 == 0;
    a.fast_x = vec && aligned16(x0) && (!x1 || aligned16(x1));
    a.fast_w = !ci_idx && a.CIg % 4 == 0 && a.W_CIg % 4 == 0 && aligned16(w);
    return SD_OK;
}

// how many slices to cut the reduction range in.  A compute unit holds two to four of these
// workgroups at a time and a workgroup runs about as long alone as with neighbours, so the last,
// partly filled round of workgroups costs a full round: eight workgroups per compute unit keep that
// tail below a fifth of the run.  A slice keeps at least four LDS chunks (128 inputs).  The index-list
// kernels are bound by their gather loads, not by the tail, and pay for every slice with merge traffic: they
// ask for one workgroup per compute unit (per_cu).
inline int pick_nsplit(const FwdArgs& a, int BB, int BM, int per_cu = 8) {
    long long tiles = (long long)((a.R + BB - 1) / BB) * ((a.COg + BM - 1) / BM) * a.G;
    int chunks = (a.CIg + 31) / 32;
    long long want = (long long)per_cu * num_cus();
    int max_ns = chunks / 4;
    if (max_ns > 16) max_ns = 16;
    int ns = 1;
    while (ns * 2 <= max_ns && tiles * ns < want) ns *= 2;
    return ns;
}

// rows per work-item (batch tile = 16 * TB rows): the largest candidate whose tiles, after split-N,
// still give the device about four workgroups per compute unit; small problems fall to the smallest
inline int pick_tb(const FwdArgs& a, const int* candidates, int n, int BM) {
    for (int k = 0; k < n; k++) {
        int BB = 16 * candidates[k];
        if (a.R <= BB / 2 && k + 1 < n) continue;   // tile mostly padding
        long long tiles = (long long)((a.R + BB - 1) / BB) * ((a.COg + BM - 1) / BM) * a.G;
        if (tiles * pick_nsplit(a, BB, BM) >= 4ll * num_cus()) return candidates[k];
    }
    return candidates[n - 1];
}

}  // namespace sd
