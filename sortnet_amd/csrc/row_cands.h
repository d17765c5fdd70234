// Sort neuron, its interval bounds and the l-inf forward (plain and under the factored mask) of dense single-group
// layers from candidate tables built per BATCH ROW and tile of 128 weight rows: the orientation for inputs whose
// spread over the inputs of a row is large against the weights (images in [0, 1] against weights ~ N(0, 1/N)).
//
// Over a tile of weight rows the term |x[b,n] - w[m,n]| is bracketed by the column minimum and maximum of the
// weights, so the K largest terms of (b, m) sit, for every m of the tile, at the few inputs where x[b, .] is
// extreme.  A bit table (tile, batch row, 32 inputs) marks the inputs whose term can reach a lower bound of the
// K-th largest; the main kernel gives a wavefront one batch row (lane l holds the weight rows l and l + 64 of the
// tile), lists the row's marks and walks them against a transposed copy of the tile's weights, so an unmarked input
// costs nothing.  Same bits as the kernels that evaluate every term
// (core/cuda/sort_neuron.cu:16-314, core/cuda/inf_dist_cuda.cu:110-212 semantics).
//
// This orientation is queued behind the per-weight-row tables of sort_cols.h and shares their probe: its kernels
// return at once unless the probe found that the batch rows differ by more than the weights do.
#pragma once
#include "common.h"

namespace sd {

// inputs of one bit-table word; CI must be a multiple of it
constexpr int kRowCandsChunk = 32;

enum RowCandsForm {
    kRowsSortValues = 0,     // sort neuron, values
    kRowsSortInterval = 1,   // interval bounds of the sort neuron
    kRowsSortPos = 2,        // sort neuron, values and the K planes of positions
    kRowsMax = 3,            // l-inf distance (K = depth of the bound: 1 without a mask), optionally positions
};

// bytes of workspace row_cands_forward needs
size_t row_cands_workspace(int form, int B, int CO, int CI, int K);

// True when this build has a main kernel for (form, K): the sort-neuron forms for K = 2 .. 25, the l-inf form for the
// depths of max_cols_depth.
bool row_cands_supported(int form, int K);

// Queues the tables per batch row and the main kernel that works from them.
//   col_stat / col_count: the probe sums and the counter words that sort_cols_forward / max_cols_forward left for
//     the same call (col_count[1] != 0: the per-weight-row tables are above their limit).  Everything here returns
//     at once unless the probe says that the batch decides.
//   density: largest share of marked (tile of weight rows, batch row, input) triples at which the main kernel runs;
//     forced: the caller's limit was set by hand (then the l-inf form builds its tables whenever the batch decides,
//     instead of only where the probe promises very few marks).
//   *every: device word that is non-zero when neither table serves the call, i.e. when the kernels that evaluate
//     every term are to run (their gate: run when *every > 0); (*every)[-1] holds the marks of this table,
//     (*every)[1] is non-zero when this table's kernel runs, (*every)[2] the marks per weight row (copied).
//   xkeep / wkeep (kRowsMax only, both or neither): keep bits of the factored mask, one word per (row, 32 inputs).
//   outL / outU / pos as in sort_cols_forward / max_cols_forward (values go to outU).
int row_cands_forward(int form, const float* xl, const float* xu, const float* w, const uint32_t* xkeep,
                      const uint32_t* wkeep, int B, int CO, int CI, float q, int K, float* outL, float* outU, int* pos,
                      void* ws, float density, bool forced, const float* col_stat, const unsigned long long* col_count,
                      const unsigned long long** every, hipStream_t st);

}  // namespace sd
