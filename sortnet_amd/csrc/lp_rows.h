// l-p norm distance at large p, dense single-group form: kernels that work from per-row candidate lists.
//
// At large p only terms with |x[b,n] - w[m,n]| close to the scale of output (b, m) change the fp32 result
// (core/cuda/norm_dist_cuda.cu:36-160 evaluates all of them).  Whether a term can count is bounded from above
// by |x[b,n]| + max_m |w[m,n]| over a tile of output channels, which depends on the row and the input only: a
// bit table (tile, 32 inputs, row) marks the inputs of every row that can hold a term that counts for some
// output channel of the tile.  The kernels give a wavefront one batch row at a time (64 lanes = 64 output
// channels), so the table is read with scalar instructions and an input that is not marked costs nothing.
#pragma once
#include "common.h"

namespace sd {

// inputs of one bit-table word; CI must be a multiple of it
constexpr int kRowsChunk = 32;

// Both calls below build the table, count its marks on the device and queue their kernel so that it runs only when
// at most `density` of all (tile, row, input) triples are marked (the kernel that evaluates every term is queued by
// the caller with the opposite condition on the same counter, returned in *gate / *gate_limit).

// bytes of workspace the two calls below need beyond their arguments
size_t lp_rows_workspace(int B, int CO, int CI);

// number of slices the input range of the forward is cut in (partial sums go to `part`)
int lp_rows_forward_nsplit(int B, int CO, int CI);

// sums of (|x - w| / maxv)^p relative to the given maxima.  nsplit == 1: y = maxv * sum^(1/p); otherwise the
// slice sums go to part[slice][B * CO] for the caller to merge.  maxv == nullptr: the kernel finds the maxima itself
// as it goes (the table then comes from a lower bound of them), and the slices leave (sum, maximum) pairs in
// part[slice] and part[nsplit + slice].  ws: lp_rows_workspace bytes.
int lp_rows_forward(const float* x, const float* w, const float* maxv, int B, int CO, int CI, float p, float thr,
                    int nsplit, float* y, float* part, void* ws, float density,
                    const unsigned long long** gate, unsigned long long* gate_limit, hipStream_t st);

// grad_input (always; zero-filled here) and grad_weight (if non-null) of the l-p distance from its output y;
// terms with |d| / y <= thr are dropped.  ws: lp_rows_workspace bytes followed by B * CO floats, which receive
// 1 / y (*recip) for the caller's own kernel.
int lp_rows_backward(const float* gy, const float* x, const float* w, const float* y, int B, int CO, int CI,
                     float pm1, float thr, float* gx, float* gw, void* ws, float density, const float** recip,
                     const unsigned long long** gate, unsigned long long* gate_limit, hipStream_t st);

}  // namespace sd
