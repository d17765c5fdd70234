/*
 * sortdist -- plain C ABI of the MI355X (gfx950) distance-neuron kernels.
 *
 * Every entry point replaces one static launcher of the reference extension
 * (core/cuda/norm_dist.h, cited per function) one level below its pybind layer
 * (core/cuda/norm_dist.cpp:294-317): raw device pointers and sizes in, nothing returned
 * but a status.  Differences from the reference launchers, all additive:
 *   - a trailing `stream` argument (a hipStream_t passed as void*; NULL = the null stream);
 *     the reference always used the legacy default stream;
 *   - an int status instead of void: 0 = ok, SD_ERR_ARG = rejected arguments,
 *     SD_ERR_HIP = a HIP call or kernel launch failed; sd_last_error() returns the message
 *     of the calling thread's last failure.
 *
 * Conventions (same as the reference): all tensors are contiguous fp32 device memory,
 * indices are int32.  input is (B, CI, HW), weight is (W_CO, W_CI / G), output is
 * (B, CO, HW); CI and CO count all groups.  B, CO, CI, HW are what the reference's pybind
 * layer derives from the tensor sizes.  The optional index lists w_index_ci (S, G, CI/G) and
 * w_index_co (S, G, CO/G), S = ceil(B/32), select for each 32-sample sub-batch the rows and
 * columns of weight that the (already compacted) input and output refer to; pass NULL for
 * the dense case, in which W_CO, W_CI are ignored.  The callee zero-fills every buffer it
 * scatters into (grad_input, grad_weight), as the reference launchers do, and owns no
 * caller-visible memory.  pos packs the arg-max input index in bits 0..30 and a branch/sign
 * flag in bit 31.
 *
 * The backward entry points trust pos: bits 0..30 must be below CI / G (the forward entry points
 * only write such values); an index outside that range is read or written out of bounds, as in
 * the reference.
 *
 * Scratch memory: the library keeps one device buffer per (GPU, stream) for partial results
 * (split reductions, mask bits, candidate lists, per-slice sums) and grows it on demand with
 * hipMalloc; growing waits for that stream first.  Calls are asynchronous on `stream`; calls
 * on different streams never share a buffer and may overlap, calls on one stream use it in
 * queue order.  Host threads: every entry point may be called from any thread at any time; while
 * a call queues its kernels it holds a library-wide lock, so the calls of several threads reach
 * a shared stream whole, one after the other, and each gets the results it would get alone.
 * The sd_set_* limits are process-wide atomics that a call reads once when it starts; per-layer
 * table hints (which of two queued kernels has been running lately) are kept for the 256 most
 * recently used (entry point, weight pointer, shape) triples and never change a result.  A call that would have to grow the buffer while its stream is being captured
 * into a graph fails with SD_ERR_HIP: run it once on that stream before the capture.
 * Outputs that are zero-filled or merged with 128-bit stores must be 16-byte aligned.
 */
#ifndef SORTDIST_H
#define SORTDIST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SD_OK 0
#define SD_ERR_ARG 1
#define SD_ERR_HIP 2

#define SD_MASK_TERM 0      /* independent Bernoulli draw for every (b, m, n) term */
#define SD_MASK_FACTORED 1  /* keep(b,m,n) = keep_x(b,n) & keep_w(m,n), each with probability sqrt(q) */

typedef void* sd_stream_t;

/* library / error reporting (no reference counterpart) */
int sd_version(void);
const char* sd_last_error(void);
/* Which forward tile kernel the calling thread's last forward call dispatched, with its register tile, e.g.
 * "fwd_kernel_direct<4,8>" (global -> LDS loads), "fwd_kernel_pipe<4,8>" (register-staged), "fwd_kernel_lists<2,8>"
 * (gather loads), "fwd_kernel<2,4>" (general): for tests and benchmarks that must know which path they measured. */
const char* sd_last_forward_kernel(void);
/* For benchmarks that must report a tile kernel's own duration rather than an entry point's (which also queues fill,
 * table and resolve kernels): after sd_time_forward_kernels(1) every forward entry point called by this thread records
 * an event on its stream before and after the launch of its forward tile kernel, and sd_last_forward_kernel_ms() waits
 * for the later one and returns the milliseconds between them (-1 when there is none).  Off by default; nothing is
 * recorded on a stream that is being captured. */
int sd_time_forward_kernels(int on);
float sd_last_forward_kernel_ms(void);
/* For benchmarks that must say how much arithmetic a call really did: the share (0..1] of its B * CO * CI / G terms that
 * the calling thread's last l-inf, masked (factored), interval or sort-neuron forward call formed.  Waits for `stream`
 * (the one the call was queued on; call this before queueing anything else there) and reads the call's candidate-table
 * counters: the marked share when a table kernel served the call, 1 when every term was evaluated or no table was
 * queued (index lists, groups, small layers, l-p calls); -1 on a HIP error.  No reference counterpart. */
float sd_last_forward_term_share(sd_stream_t stream);
/* Dense single-group l-p calls at general p queue two kernels for the same result: one that evaluates every term
 * and one that works from a table of the inputs that can hold a term that counts (per output-channel tile and batch
 * row).  The share of marked table entries, counted on the device, decides which of the two runs: the table kernel
 * when it is at most `density` (0 never builds the table, 1 always uses it, negative = the built-in limits, which
 * are the default: 0.05 to 0.2 depending on the call).  Process-wide; no reference counterpart
 * (core/cuda/norm_dist_cuda.cu evaluates every term). */
int sd_set_lp_candidate_density(float density);
/* The same for sd_bound_inf_dist_forward_nograd and sd_bound_inf_dist_forward on dense single-group layers (CI a multiple of 32): a kernel that works
 * from a table of the inputs that can hold the maximum of a weight row over a tile of 128 batch rows, and the kernel
 * that evaluates every term; both give the same bits.  Built-in limits: 0.30 (0.26 where the table is built per batch
 * row and tile of 128 weight rows instead, which the call decides from its operands), layers of at least 2^31 terms;
 * a `density` of 0 or more applies at any size.  The form with positions has a built-in limit of 0.15; values and
 * positions are the every-term kernel's.  No reference counterpart
 * (core/cuda/bound_inf_dist_cuda.cu evaluates every term). */
int sd_set_bound_candidate_density(float density);
/* Which table kernel serves sd_bound_inf_dist_forward_nograd: 1 = the one that stages tiles of inputs and weights
 * through LDS (marked shares of a few per cent and more), 2 = the one that walks a weight row's marks over a
 * transposed copy of the inputs (marked shares below about 1 %: weights of unit scale against batch rows that are
 * alike), 0 (default) = 1 until a layer has reported that few marks three calls in a row, then 2 for 31 calls.  Same
 * bits whichever runs. */
int sd_set_bound_candidate_form(int form);
/* The same for sd_sort_neuron_forward[_nograd] and sd_bound_sort_neuron_forward on dense single-group layers (CI a
 * multiple of 32): a kernel that works from a table of the inputs that can be among the K largest terms of a weight
 * row over a tile of 128 batch rows, and the kernels that evaluate every term; both give the same bits (positions
 * included).  Built-in limit 0.10, and the table is only built for layers of at least 2^24 terms; a positive `density` applies at any
 * size.  No reference counterpart (core/cuda/sort_neuron.cu evaluates every term). */
int sd_set_sort_candidate_density(float density);
/* The same for sd_inf_dist_forward[_nograd] (no index lists) and sd_masked_inf_dist_forward (factored mask) on dense
 * single-group layers (CI a multiple of 32, at most 65536): a kernel that works from a table of the inputs that can hold
 * the maximum of a weight row over a tile of 128 batch rows, and the kernels that evaluate every term; same values and
 * positions either way.  Built-in limit 0.10, layers of at least 2^31 terms.  Under the mask the table's bound rests on
 * `depth` inputs per weight row, chosen so that a batch row keeps none of them less than once in 10^4 outputs (such an
 * output is recomputed from every input); sd_set_linf_candidate_depth overrides the choice (0 = automatic; 8, 12, 16,
 * 20 or 24).  No reference counterpart (core/cuda/inf_dist_cuda.cu evaluates every term). */
int sd_set_linf_candidate_density(float density);
int sd_set_linf_candidate_depth(int depth);

/* ---- l-inf distance: struct inf_dist, core/cuda/norm_dist.h:20-31 ---- */

/* inf_dist::forward_nograd (norm_dist.h:21-22; core/cuda/inf_dist_cuda.cu:277-304):
 * output = max(1e-10, max_n |input - weight|). */
int sd_inf_dist_forward_nograd(const float* input, const float* weight,
                               int B, int CO, int CI, int G, int HW, float* output, sd_stream_t stream);

/* inf_dist::forward (norm_dist.h:23-25; inf_dist_cuda.cu:306-323): as above plus
 * pos = lowest arg-max index | (input - weight < 0) << 31; optional index lists. */
int sd_inf_dist_forward(const float* input, const float* weight,
                        int B, int CO, int CI, int G, int HW, float* output, int* pos,
                        const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI, sd_stream_t stream);

/* No counterpart in the reference.  sd_inf_dist_forward for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments and
 * results, but the scratch of its split reduction lives in a 32 MiB device array built into the library
 * instead of the grow-only workspace, and the call performs no hipMalloc / hipFree.  At most
 * 4 194 304 outputs (B * CO * HW); larger calls return SD_ERR_ARG.  The first call on a GPU looks the
 * array's address up (make it before any capture).  All calls on one GPU share the array: calls that
 * overlap on one GPU (other streams or threads) race. */
int sd_inf_dist_forward_noalloc(const float* input, const float* weight,
                                int B, int CO, int CI, int G, int HW, float* output, int* pos,
                                const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                sd_stream_t stream);

/* inf_dist::backward_input (norm_dist.h:26-27; inf_dist_cuda.cu:325-336). */
int sd_inf_dist_backward_input(const float* grad_output, const int* pos,
                               int B, int CO, int CI, int G, int HW, float* grad_input, sd_stream_t stream);

/* inf_dist::backward_input_weight (norm_dist.h:28-30; inf_dist_cuda.cu:338-354).
 * With index lists grad_weight has the full (W_CO, W_CI / G) shape. */
int sd_inf_dist_backward_input_weight(const float* grad_output, const int* pos,
                                      int B, int CO, int CI, int G, int HW, float* grad_input, float* grad_weight,
                                      const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                      sd_stream_t stream);

/* ---- interval bounds through the l-inf layer: struct bound_inf_dist, norm_dist.h:33-45 ---- */

/* bound_inf_dist::forward_nograd (norm_dist.h:34-35; core/cuda/bound_inf_dist_cuda.cu:314-328). */
int sd_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight,
                                     int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                     sd_stream_t stream);

/* bound_inf_dist::forward (norm_dist.h:36-37; bound_inf_dist_cuda.cu:330-346). */
int sd_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight,
                              int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                              int* posL, int* posU, sd_stream_t stream);

/* bound_inf_dist::backward_input (norm_dist.h:38-40; bound_inf_dist_cuda.cu:362-371). */
int sd_bound_inf_dist_backward_input(const float* grad_outputL, const float* grad_outputU,
                                     const int* posL, const int* posU, int B, int CO, int CI, int G, int HW,
                                     float* grad_inputL, float* grad_inputU, sd_stream_t stream);

/* bound_inf_dist::backward_input_weight (norm_dist.h:41-44; bound_inf_dist_cuda.cu:373-383). */
int sd_bound_inf_dist_backward_input_weight(const float* grad_outputL, const float* grad_outputU,
                                            const int* posL, const int* posU, int B, int CO, int CI, int G, int HW,
                                            float* grad_inputL, float* grad_inputU, float* grad_weight,
                                            sd_stream_t stream);

/* ---- sort neuron: struct sort_neuron, norm_dist.h:47-57; K in 2..25 ----
 * Undefined (NaN) terms: a term |input - weight| that is NaN is LEFT OUT of the K largest here (values, positions and
 * interval form alike), whichever kernel serves the call.  The reference's insertion max(res[k], min(res[k+1], v))
 * (core/cuda/sort_neuron.cu:73-77, 283-287) instead shifts its list down by one on such a term, i.e. counts the
 * largest entry so far twice; that behaviour depends on the order in which the inputs are scanned and is not
 * reproduced.  Finite inputs, +-inf included, give the reference's results.  (The l-inf and interval-bound entry points
 * drop NaN terms exactly as the reference's strict comparisons and fminf / fmaxf do.) */

/* sort_neuron::forward_nograd (norm_dist.h:48-49; core/cuda/sort_neuron.cu:387-434). */
int sd_sort_neuron_forward_nograd(const float* input, const float* weight,
                                  int B, int CO, int CI, int G, int HW, float* output, float q, int K,
                                  sd_stream_t stream);

/* sort_neuron::forward (norm_dist.h:50-51; sort_neuron.cu:437-485); pos is (K, B, CO, HW). */
int sd_sort_neuron_forward(const float* input, const float* weight,
                           int B, int CO, int CI, int G, int HW, float* output, int* pos, float q, int K,
                           sd_stream_t stream);

/* sort_neuron::backward_input (norm_dist.h:52-53; sort_neuron.cu:536-547). */
int sd_sort_neuron_backward_input(const float* grad_output, const int* pos,
                                  int B, int CO, int CI, int G, int HW, float* grad_input, float q, int K,
                                  sd_stream_t stream);

/* sort_neuron::backward_input_weight (norm_dist.h:54-56; sort_neuron.cu:549-562). */
int sd_sort_neuron_backward_input_weight(const float* grad_output, const int* pos,
                                         int B, int CO, int CI, int G, int HW, float* grad_input,
                                         float* grad_weight, float q, int K, sd_stream_t stream);

/* bound_sort_neuron_forward_cuda (norm_dist.h:60-61; sort_neuron.cu:487-534). */
int sd_bound_sort_neuron_forward(const float* inputL, const float* inputU, const float* weight,
                                 int B, int CO, int CI, int G, int HW, float* outputL, float* outputU,
                                 float q, int K, sd_stream_t stream);

/* ---- l-p norm distance: template struct norm_dist<ip>, norm_dist.h:4-18.  The dispatch on p
 * that the reference does in its pybind layer (norm_dist.cpp:4,17-38,51-60) happens inside.
 * Undefined (NaN) and infinite operands: the reference sums every term, so an output that meets such an operand is
 * undefined there.  Here the forward never returns a finite value for such an output, whichever kernel serves the
 * call (undefined, or infinite where a kernel leaves out the undefined term inf / inf), and every other output is
 * unaffected.  The backward kernels leave out terms whose ratio to the output does not compare as significant, an
 * undefined ratio among them, so the gradients that belong to a non-finite output are only partly undefined:
 * callers detect such a state from the forward's output. ---- */

/* norm_dist<ip>::forward / forward_with_max(max_output = nullptr) as selected by
 * norm_dist_forward (core/cuda/norm_dist.cpp:43-61; norm_dist_cuda.cu:512-552). */
int sd_norm_dist_forward(const float* input, const float* weight,
                         int B, int CO, int CI, int G, int HW, float* output, float p,
                         const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI, sd_stream_t stream);

/* norm_dist<ip>::forward_with_max with a caller-supplied max_output (norm_dist.h:8-10;
 * norm_dist.cpp:67-80). */
int sd_norm_dist_forward_with_max(const float* input, const float* weight, const float* max_output,
                                  int B, int CO, int CI, int G, int HW, float* output, float p,
                                  const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                  sd_stream_t stream);

/* norm_dist<ip>::backward_input (norm_dist.h:11-13; norm_dist.cpp:86-102). */
int sd_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                const float* output, int B, int CO, int CI, int G, int HW,
                                float* grad_input, float p,
                                const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                sd_stream_t stream);

/* norm_dist<ip>::backward_input_weight (norm_dist.h:14-17; norm_dist.cpp:108-125). */
int sd_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                       const float* output, int B, int CO, int CI, int G, int HW,
                                       float* grad_input, float* grad_weight, float p,
                                       const int* w_index_ci, const int* w_index_co, int W_CO, int W_CI,
                                       sd_stream_t stream);

/* ---- masked order-statistic neuron (no reference launcher: the reference builds its training
 * mask on the host, core/models/norm_dist.py:14-17, and hands index lists to inf_dist::forward).
 * output = max(1e-10, max over kept n of |input - weight|) where term (b, m, n) is kept with
 * probability q, decided by a stateless counter RNG of (seed, b, m, n); pos may be NULL. ---- */
int sd_masked_inf_dist_forward(const float* input, const float* weight,
                               int B, int CO, int CI, int G, int HW, float* output, int* pos,
                               float q, uint32_t seed, int mode, sd_stream_t stream);

/* ---- mean shift, the step after every distance layer (MeanShiftDropout without index list,
 * core/models/bound_basic_module.py:123-157; done with torch ops in the reference) ---- */

/* Training form: mean[c] = mean over (b, hw) of input; running_mean (may be NULL) is updated in place as
 * (1 - momentum) running_mean + momentum mean; output = input - mean[c].  Applied to an upstream
 * gradient with running_mean = NULL it is also the backward of itself. */
int sd_mean_shift_forward(const float* input, int B, int C, int HW, float* mean, float* running_mean,
                          float momentum, float* output, sd_stream_t stream);

/* output = input + sign * shift[c]: evaluation-mode mean shift (sign = -1) and bias add (sign = +1),
 * core/models/bound_basic_module.py:155 and core/models/norm_dist.py:102-103. */
int sd_channel_shift(const float* input, const float* shift, int B, int C, int HW, float sign,
                     float* output, sd_stream_t stream);

/* Training-mode mean shift when every 32-sample sub-batch keeps its own channel subset
 * (core/models/bound_basic_module.py:125-137,146-153, done there with torch ops).  input / output are
 * (B, G * cnt, HW), already compacted; index is (S, G, cnt), S = ceil(B / 32), ascending channel numbers below
 * Cg for every (sub-batch, group).  mean (G * Cg) receives, for every full channel, the mean over the samples
 * and positions of the sub-batches that kept it (0 for a channel nobody kept); running_mean (G * Cg, may be
 * NULL) is updated as above; output = input - mean[index].  Partial sums are added in sub-batch order, so
 * the result is deterministic.  With running_mean = NULL it is also the backward of itself. */
int sd_mean_shift_index_forward(const float* input, const int* index, int B, int G, int cnt, int Cg, int HW,
                                float* mean, float* running_mean, float momentum, float* output,
                                sd_stream_t stream);

/* ---- device-side mask sampling for the index-list form (replaces sample_mask,
 * core/models/norm_dist.py:14-17, which draws on the host with a device synchronisation) ---- */

/* Host-only, touches no GPU: the number of kept channels, count = #{c < C : u_c < q} with u_c from
 * the counter RNG (the reference's (rand(C) < q).sum()). */
int sd_mask_count(uint32_t seed, int C, float q);

/* out (S, G, count) int32: for every (sub-batch, group) a uniformly random subset of exactly `count`
 * of the C channels, ascending (the reference's sort(topk(rand(S, G, C), count).indices)). */
int sd_sample_index_lists(uint32_t seed, int S, int G, int C, int count, int* out, sd_stream_t stream);

/* The counter RNG and the thresholds it is compared with, exposed for verification. */
uint32_t sd_rng_word(uint32_t seed, uint32_t stream_id, uint32_t row, uint32_t col);
uint32_t sd_mask_threshold8(float q);
uint32_t sd_mask_threshold16(float q);

#ifdef __cplusplus
}
#endif
#endif /* SORTDIST_H */
