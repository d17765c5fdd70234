// Interval-bound forward (values only) of dense single-group layers from per-weight-row candidate tables.
//
// yL[b,m] = max(1e-10, max_n max(l[b,n] - w[m,n], w[m,n] - u[b,n])) and yU[b,m] = max(1e-10, max_n max(w[m,n] - l[b,n],
// u[b,n] - w[m,n])) (core/cuda/bound_inf_dist_cuda.cu:15-118) are maxima, so an input n whose term cannot reach a
// lower bound of the result can be left out without changing a bit.  Over a tile of 128 batch rows the terms of
// (m, n) are bracketed by the column minima / maxima of l and u: when the rows of the tile are alike (the bounds
// of hidden layers) and the weights of a row are not, few inputs per weight row can hold the maximum.  A bit table
// (tile, 32 inputs, weight row) marks them; the kernel gives a wavefront one weight row at a time (64 lanes =
// 64 batch rows x 2), so the table is read with scalar instructions and an unmarked input costs nothing.
#pragma once
#include "common.h"

namespace sd {

// inputs of one bit-table word; CI must be a multiple of it
constexpr int kColsChunk = 32;

// bytes of workspace bound_cols_forward needs
size_t bound_cols_workspace(int B, int CO, int CI);

// Builds the table, counts its marks on the device and queues the table kernel so that it runs only when at most
// `density` of all (tile, weight row, input) triples are marked (`density_rows` of all (tile of weight rows, batch
// row, input) triples where the table is built per batch row); the caller queues the kernel that evaluates every
// term with the opposite condition on the same counter (*gate, *gate_limit).  outL / outU must be zero-filled:
// the slices of the input range merge by atomic maximum.  (*gate)[1] (the word behind the gate) is 1 when the marks
// per weight row are so few (below a sixteenth of the limit) that a kernel without LDS staging would serve better.
// With packedL / packedU (B x CO words each, zero-filled) and posL / posU: the forward with positions.  The kernel of
// the tables per weight row leaves (value bits << 32 | ~chunk of 32 inputs) per output in packedL / packedU, merged by
// atomic maximum, as the every-term kernel with chunk tracking does (fwd_tile.h: store_chunk_winner), for
// resolve_bound_kernel to take values and positions from; the kernel of the tables per batch row stores final values
// and positions in outL / outU / posL / posU itself and sets (*gate)[2], which the resolve pass must be given as
// FwdArgs::resolved.
int bound_cols_forward(const float* xl, const float* xu, const float* w, int B, int CO, int CI, float* outL,
                       float* outU, unsigned long long* packedL, unsigned long long* packedU, int* posL, int* posU,
                       void* ws, float density, float density_rows, const unsigned long long** gate,
                       unsigned long long* gate_limit, hipStream_t st);

}  // namespace sd
