// Sort neuron (values only) and its interval bounds for dense single-group layers, from per-weight-row candidate
// tables.
//
// Both are sums over the K largest terms of a row of terms (core/cuda/sort_neuron.cu:16-109, 216-314), so an input
// whose term cannot reach a lower bound of the K-th largest term can be left out without changing a bit.  Over a
// tile of 128 batch rows the terms of (m, n) are bracketed by the column minima / maxima of the inputs; when the
// rows of a tile are alike compared with the entries of a weight row (weights of unit scale against activations
// that a mean shift has centred), the same few dozen inputs per weight row hold the K largest terms of every batch
// row.  A bit table (tile, weight row, 32 inputs) marks them, and a wavefront that owns a weight row and 128 batch
// rows (two per lane) walks the row's marks, fetching one weight and one transposed row of inputs per mark.
#pragma once
#include "common.h"

namespace sd {

// inputs of one bit-table word; CI must be a multiple of it
constexpr int kSortColsChunk = 32;

// bytes of workspace sort_cols_forward needs
size_t sort_cols_workspace(int B, int CO, int CI, int K);

// Builds the table, counts its marks on the device and queues the table kernel so that it runs only when at most
// `density` of all (tile, weight row, input) triples are marked; the caller queues the kernels that evaluate every
// term with the opposite condition on the same counter (*gate, *gate_limit); (*gate)[1] is 1 when those are to run.
//   xu != nullptr: interval form, outL / outU receive the bounds; with K = 1 these are the interval bounds of the
//   l-inf distance (maxima with the 1e-10 floor, q unused), for layers whose marks are too few to stage tiles for;
//   xu == nullptr: value form on xl, outU receives the values (outL is not used) and pos, if not null, the K planes
//   of positions (K, B, CO), largest first.
int sort_cols_forward(const float* xl, const float* xu, const float* w, int B, int CO, int CI, float q, int K,
                      float* outL, float* outU, int* pos, void* ws, float density, const unsigned long long** gate,
                      unsigned long long* gate_limit, hipStream_t st);

// The two sums of the probe that sort_cols_forward / max_cols_forward leave behind the counter words *gate points at
// (widths of the input columns over all batch tiles; widths of the same columns over 16 weight rows), for the tables
// of the other orientation (row_cands.h), which are queued behind these and decide from the same sums.
inline const float* sort_cols_probe_sums(const unsigned long long* gate) { return reinterpret_cast<const float*>(gate + 2); }

// l-inf distance forward (maximum and, if pos is not null, its position) from the same kind of table, optionally
// under the factored mask (xkeep: one word per (batch row, 32 inputs), wkeep: per (weight row, 32 inputs); both or
// neither).  K = max_cols_depth(probability that a row keeps an input): how many inputs the bound of a weight row
// rests on (1 without a mask; 0 = the mask keeps too little for a table).  Same contract as sort_cols_forward.
int max_cols_depth(float keep_x);
size_t max_cols_workspace(int B, int CO, int CI, int K);
int max_cols_forward(const float* x, const float* w, const uint32_t* xkeep, const uint32_t* wkeep, int B, int CO, int CI,
                     int K, float* y, int* pos, void* ws, float density, const unsigned long long** gate,
                     unsigned long long* gate_limit, hipStream_t st);

}  // namespace sd
