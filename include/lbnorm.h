/* lbnorm.h — C ABI of the MI355X (gfx950) normalization and softmax kernels.
 *
 * Each entry point is the device compute of one LBANN layer's fp_compute() or
 * bp_compute() on LOCAL matrices: column-major, element (r,c) at buf[r + c*ld],
 * one column per mini-batch sample (El::Matrix<T,Device>: Height/Width/LDim/Buffer).
 * A call only enqueues work on `stream`: it allocates and frees no memory, reads
 * no results back, and does not wait for the device (one exception, described under
 * "Waits across workgroups": a cluster kernel that follows one enqueued on another
 * host thread's hipStreamPerThread waits for the device once).  All pointers are device
 * pointers that must stay valid until the stream work completes.  Every output
 * element is overwritten (outputs may be uninitialised on entry); nothing is
 * accumulated into.  Calls with width == 0 or an empty sample return LBN_OK
 * without launching.
 *
 * Return value: LBN_OK, a negative LBN_ERR_* code for a rejected argument, or a
 * positive hipError_t from the launch.  No C++ exception crosses this boundary.
 * An entry point clears the calling thread's pending HIP error (hipGetLastError)
 * when it starts, so that the status it returns reports its own launches only: a
 * caller that wants to see an error left by its own earlier HIP calls reads it
 * before calling in.
 *
 * Scratch memory ("workspace") is always caller-provided.  The matching
 * *_workspace_bytes() function returns the size needed for a given shape
 * (possibly 0, in which case NULL may be passed).  A workspace only carries data
 * between the kernels of one call.
 *
 * HIP graphs: the compute entry points may be called on a stream that is recording
 * (hipStreamBeginCapture); they record kernel launches only.  The kernels in which
 * workgroups wait for each other tell one call's partial results from another's by
 * a tag; a recorded call repeats its arguments, so while recording such a kernel is
 * preceded by a one-thread kernel that advances a counter in the workspace, which
 * the tag takes in.  The workspace passed while recording is therefore part of the
 * graph's state: keep it allocated, and do not run two replays that share it at the
 * same time.
 *
 * Waits across workgroups.  Those kernels ("cluster kernels": batch norm, softmax and
 * layer norm over rows too long for one workgroup) size their grid to the workgroups the
 * idle device holds at once, so that all members of a cluster are resident together and
 * every wait ends.  Two things this rests on are assumptions about the hardware, not
 * guarantees of the HIP API: the occupancy query describes a device that runs nothing
 * else, and workgroups are dispatched in block order (members of a cluster are
 * consecutive blocks, so a launch that shares the device still has at most one partly
 * resident cluster, whose missing members are the next to start).  Two cluster kernels must
 * not share the device: each could hold part of it and wait for workgroups that cannot
 * start.  The library sees to that for eager calls itself: a cluster kernel whose
 * predecessor went to another stream is made to wait for it with an event (processes that
 * use one stream for these calls pay nothing; the first call from a second stream records
 * the event behind its predecessor, and only when that predecessor went to another host
 * thread's hipStreamPerThread, a stream this thread cannot name, does it wait for the device,
 * once), and launches from several host threads queue up behind a mutex.  Should the order
 * not be established at all (event and device wait both refused, e.g. while another thread
 * records a graph in global capture mode), the call runs its multi-kernel path instead.
 * What it cannot order are replays of HIP graphs that contain cluster kernels: do not
 * replay two such graphs, or one next to eager cluster calls of another stream, at the same
 * time (or set LBN_NO_CLUSTER=1 in the environment, which selects the multi-kernel paths
 * everywhere), and other work that occupies the device while a cluster kernel starts
 * shrinks what the occupancy query promised.  Every wait is bounded: a wait that runs out raises
 * a sticky error word in the workspace's first 64 bytes (written by nothing else), the
 * kernel ends normally with undefined results, and the entry point has long returned 0.
 * lbn_workspace_timed_out() reads that word; a caller who wants to rely on it clears the
 * first 64 bytes of a workspace once after allocating it (recycled memory may hold
 * anything) and checks where results are consumed.  The two host-side mirrors of the
 * layer classes do both.
 *
 * Process-wide state of the library: the counter the per-call tags are drawn from (an
 * atomic), the cached occupancy figures per kernel and device and compute-unit counts per
 * device, per device the stream of the
 * last cluster kernel with its mutex and (once a second stream has been seen) one event,
 * and the environment switches, each read once.  Nothing else outlives a call.
 */
#ifndef LBNORM_H_INCLUDED
#define LBNORM_H_INCLUDED

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* lbn_stream_t; /* a hipStream_t; NULL is the default stream */

#define LBN_OK 0
#define LBN_ERR_INVALID_ARGUMENT (-1) /* negative size, ld < height, NULL matrix, ... */
#define LBN_ERR_WORKSPACE (-2)        /* workspace NULL or smaller than *_workspace_bytes() */
#define LBN_ERR_UNSUPPORTED (-3)      /* shape outside what the kernels index (e.g. > 2^31 rows) */

/* Statistics formula selector for the `flags` argument of the normalization forwards.
 * LBN_STATS_TWO_PASS (default): mean first, then the mean of squared deviations.
 * LBN_STATS_SUMSQ: E[x^2] - mean^2 from running sums, the formula of the reference
 * CPU code (layer_norm.cpp:99-112, batch_normalization.cpp:124-128), including its
 * cancellation error. */
#define LBN_STATS_TWO_PASS 0
#define LBN_STATS_SUMSQ 1
/* LBN_STATS_REFERENCE_ORDER: for parity tests only, never a default.  The statistics are
 * formed as the reference CPU code forms them: ONE sequential fp32 sum of x and of x*x
 * per row (layer norm, layer_norm.cpp:77-88) or per channel (batch norm, columns outer,
 * rows inner, batch_normalization.cpp:70-85), separate multiplications and additions,
 * then the reference's expression for mean and variance operation for operation.  Mean
 * and variance then equal the CPU code's bit for bit, which shows that the order of
 * summation is all that separates the default modes from it.  One lane per row or
 * channel does the adding: thousands of times slower than the default, and rejected with
 * LBN_ERR_UNSUPPORTED for tensors of more than 2^27 entries.  The layer-norm output is
 * written with the reference's operations as well; batch norm applies the statistics
 * with the kernel that inference uses.  lbn_batch_norm_bwd_reference_order_f32 is the
 * matching backward. */
#define LBN_STATS_REFERENCE_ORDER 2

int lbn_version(void);
const char* lbn_status_string(int status);

/* Diagnostic, not part of any layer: the batch-norm and wide-softmax kernels in which
 * several workgroups share a channel or a row wait for each other with a bounded
 * number of polls; a wait that runs out raises a sticky flag in the workspace and the
 * results of that call are then undefined.  This call waits for `stream`, copies the
 * flag of `workspace` (the pointer that was passed to the compute call) to the host
 * and stores it in *timed_out (0 or 1).  It is the only entry point that synchronises.
 * It has no counterpart in the reference, whose kernels do not wait across workgroups. */
int lbn_workspace_timed_out(lbn_stream_t stream, const void* workspace, int* timed_out);

/* Diagnostic: exercises the designed exit of a wait that cannot end.  Launches ONE
 * workgroup that acts as member 0 of a cluster of two, publishes its pair (1, 2) and polls
 * for a member 1 that does not exist; after max_polls (1..65536) rounds the wait gives up,
 * raises the error word of `workspace` (at least 128 bytes, 16-byte aligned) and the
 * kernel ends like any other.  out4 (4 floats, device) receives member 0's pair and the
 * stand-in (-1, -1) of the absent member.  Afterwards lbn_workspace_timed_out() reports 1
 * for this workspace until its header is cleared.  workspace == NULL (workspace_bytes
 * ignored) runs the same on the library-owned array of lbn_softmax_fwd_static_scratch_f32,
 * whose word lbn_softmax_fwd_static_scratch_timed_out() reads.  No counterpart in the
 * reference. */
int lbn_selftest_cluster_wait_gives_up(lbn_stream_t stream, void* workspace, size_t workspace_bytes,
                                       int max_polls, float* out4);

/* Diagnostic, no counterpart in the reference: copies x to y (num_channels channels of
 * channel_size entries per column, `width` columns; channel_size a multiple of 4, buffers and
 * leading dimensions on the 16-byte grid, else LBN_ERR_UNSUPPORTED) through the register
 * pipeline of the batch-norm kernels in which workgroups share a channel (persistent workgroups
 * of 512 threads, three tiles of four 16-byte vectors per thread in rotation, non-temporal
 * stores) without any arithmetic and without any exchange between workgroups.  channel_major
 * != 0 walks the matrix in the order of those kernels, channel after channel with every
 * channel's `width` segments cut into the workgroups' shares; 0 walks contiguous tiles.
 * The time of this call is what the memory system gives that order of accesses; bench.py
 * --pattern-yardstick reports it beside the batch-norm figures. */
int lbn_selftest_copy_pipeline_f32(lbn_stream_t stream, int64_t num_channels, int64_t channel_size, int64_t width,
                                   const float* x, int64_t ldx, float* y, int64_t ldy, int channel_major);

/* ------------------------------------------------------------------ layer norm
 * Replaces layer_norm_layer::fp_compute / bp_compute
 * (src/layers/regularizers/layer_norm.cpp:263-290, :292-348; math :41-136, :139-258).
 * A sample holds `num_groups` groups (get_normdims, layer_norm.hpp:362-405: product
 * of dims before start_dim) of `norm_size` contiguous entries, group g starting at
 * row g*norm_stride.  stats is (2*num_groups x width): rows [0,G) mean, [G,2G)
 * variance (biased, clamped at 0; 1 when norm_size <= 1); stats_grad likewise holds
 * dL/dmean and dL/dvar.  scale/bias (length norm_size, fp32) may be NULL.
 * Backward overwrites dscale/dbias (length norm_size) when they are non-NULL;
 * dscale != NULL requires scale != NULL.  The _f16 variants store x, y, dy, dx as
 * IEEE binary16 and compute in fp32; statistics, scale, bias and their gradients
 * stay fp32.
 * Forward scratch is optional: it is only used for groups too long for one workgroup's
 * registers (tens of thousands of entries: the layer's default, start_dim = 0,
 * normalises over a whole sample), which are then shared by several workgroups and
 * read once; with workspace == NULL such groups are read twice by one workgroup
 * each.  lbn_layer_norm_fwd_workspace_bytes() is 0 for every other shape. */
size_t lbn_layer_norm_fwd_workspace_bytes(int64_t num_groups, int64_t norm_size,
                                          int64_t width, int elem_bytes);
int lbn_layer_norm_fwd_f32(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon,
                           const float* x, int64_t ldx, float* y, int64_t ldy,
                           float* stats, int64_t ld_stats,
                           const float* scale, const float* bias,
                           void* workspace, size_t workspace_bytes, int flags);
int lbn_layer_norm_fwd_f16(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon,
                           const void* x, int64_t ldx, void* y, int64_t ldy,
                           float* stats, int64_t ld_stats,
                           const float* scale, const float* bias,
                           void* workspace, size_t workspace_bytes, int flags);
size_t lbn_layer_norm_bwd_workspace_bytes(int64_t num_groups, int64_t norm_size,
                                          int64_t width, int has_weight_grads,
                                          int elem_bytes);
int lbn_layer_norm_bwd_f32(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon,
                           const float* x, int64_t ldx, const float* dy, int64_t lddy,
                           float* dx, int64_t lddx,
                           const float* stats, int64_t ld_stats,
                           float* stats_grad, int64_t ld_stats_grad,
                           const float* scale, float* dscale, float* dbias,
                           void* workspace, size_t workspace_bytes);
int lbn_layer_norm_bwd_f16(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon,
                           const void* x, int64_t ldx, const void* dy, int64_t lddy,
                           void* dx, int64_t lddx,
                           const float* stats, int64_t ld_stats,
                           float* stats_grad, int64_t ld_stats_grad,
                           const float* scale, float* dscale, float* dbias,
                           void* workspace, size_t workspace_bytes);

/* --------------------------------------------------------------- instance norm
 * Replaces instance_norm_layer::fp_compute / bp_compute
 * (src/layers/regularizers/instance_norm.cpp:47-127, :137-245; GPU code
 * instance_norm.cu).  A sample is `channels` contiguous slabs of `channel_size`
 * entries; every (sample, channel) slab is normalised on its own with the biased
 * variance, no scale or bias.  stats is the layer's workspace matrix
 * (2*channels x width): the reference keeps sum(x) and sum(x^2) there
 * (instance_norm.cpp:72-89), this library keeps the mean in rows [0,C) and the
 * variance in rows [C,2C); the matrix is private to the layer, which only hands it
 * from forward to backward.  channel_size <= 1: y = 0 and dx = 0
 * (instance_norm.cpp:65-68, :164-167).  The backward workspace takes the place of
 * the reference's local statistics-gradient matrix (instance_norm.cpp:173-174).
 * Forward scratch is optional and only non-zero for channels of tens of thousands
 * of entries (volumes), as for layer norm. */
size_t lbn_instance_norm_fwd_workspace_bytes(int64_t channels, int64_t channel_size,
                                             int64_t width);
int lbn_instance_norm_fwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                              int64_t width, float epsilon,
                              const float* x, int64_t ldx, float* y, int64_t ldy,
                              float* stats, int64_t ld_stats,
                              void* workspace, size_t workspace_bytes);
size_t lbn_instance_norm_bwd_workspace_bytes(int64_t channels, int64_t channel_size,
                                             int64_t width);
int lbn_instance_norm_bwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                              int64_t width, float epsilon,
                              const float* x, int64_t ldx, const float* dy, int64_t lddy,
                              float* dx, int64_t lddx,
                              const float* stats, int64_t ld_stats,
                              void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------- entry-wise batch norm
 * Replaces entrywise_batch_normalization_layer::fp_compute / bp_compute
 * (src/layers/regularizers/entrywise_batch_normalization.cpp:52-202, :210-414; GPU
 * code entrywise_batch_normalization.cu).  Every entry of the sample tensor (matrix
 * row) has its own statistics over the mini-batch (matrix columns): the variance is
 * Bessel corrected (times n/(n-1)), there is no scale or bias.  stats and stats_grad
 * are (height x 2): column 0 mean resp. dL/dmean, column 1 variance resp. dL/dvar
 * (m_batch_statistics, m_batch_statistics_gradient).  training != 0: statistics from
 * the mini-batch, running_mean / running_var (the layer's two weights, length height)
 * updated with `decay` when width > 1; a single sample gives variance 1, y = 0 and
 * dx = 0.  training == 0: forward normalises with the running statistics and writes
 * neither them nor stats; backward is dx = dy / sqrt(running_var + epsilon) and reads
 * neither x nor stats (both may be NULL).  Statistics are over the local width: with
 * several ranks the reference sums them across the mini-batch (:97-100, :301-303):
 * use the split entry points below.  Where the reference's E[x^2] - mean^2 can come out
 * negative, the variance here is clamped at zero.
 * The workspace is optional (NULL: none): with it, a mini-batch of more than 256 samples
 * whose samples have few entries (4096 x 2048, say) is cut into column slabs that are
 * summed side by side instead of by one workgroup per 64 rows. */
size_t lbn_entrywise_batch_norm_workspace_bytes(int64_t height, int64_t width);
int lbn_entrywise_batch_norm_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                     float decay, float epsilon, int training,
                                     const float* x, int64_t ldx, float* y, int64_t ldy,
                                     float* stats, int64_t ld_stats,
                                     float* running_mean, float* running_var,
                                     void* workspace, size_t workspace_bytes);
/* Parity tests only (compare LBN_STATS_REFERENCE_ORDER): the training-mode forward with the CPU
 * code's own arithmetic (entrywise_batch_normalization.cpp:77-124, :136-163): per entry ONE
 * sequential fp32 sum of x and of x * x over the columns in order, variance = (sqsum / n -
 * mean * mean) * n / (n - 1) with no clamp, so that a negative value gives NaN outputs as it does
 * there.  Results equal the CPU layer's bit for bit.  No workspace; tensors of more than 2^27
 * entries are refused with LBN_ERR_UNSUPPORTED.  No counterpart of its own in the reference: it
 * is the reference's arithmetic on the GPU. */
int lbn_entrywise_batch_norm_fwd_reference_order_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                                     float decay, float epsilon,
                                                     const float* x, int64_t ldx, float* y, int64_t ldy,
                                                     float* stats, int64_t ld_stats,
                                                     float* running_mean, float* running_var);
int lbn_entrywise_batch_norm_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                     float epsilon, int training,
                                     const float* x, int64_t ldx, const float* dy, int64_t lddy,
                                     float* dx, int64_t lddx,
                                     const float* stats, int64_t ld_stats,
                                     float* stats_grad, int64_t ld_stats_grad,
                                     const float* running_var,
                                     void* workspace, size_t workspace_bytes);

/* The same computation cut where the reference places its all-reduces, for callers whose
 * mini-batch is spread over several ranks (entrywise_batch_normalization.cpp:97-100 and
 * :301-303): local sums -> [caller's all-reduce of the (height x 2) matrix] -> statistics
 * -> apply.  `width` is the local number of columns, `statistics_count` the global one
 * (input.Width() in the reference, :101 and :267).
 * fwd_sums writes per-row sum(x) into column 0 of stats and sum(x^2) into column 1
 * (:78-95; zeros for width == 0); fwd_stats turns the reduced sums into mean and variance
 * in place and updates the running statistics (:101-125; statistics_count <= 1: variance 1,
 * running statistics untouched); fwd_apply normalises with any (mean, var) pair of
 * vectors: the two stats columns in training, the running statistics in inference
 * (:131-160).  bwd_sums writes the local parts of dL/dmean, dL/dvar into stats_grad
 * (:275-299); bwd_apply forms dx from the reduced stats_grad (:305-335;
 * statistics_count <= 1: dx = 0). */
int lbn_entrywise_batch_norm_fwd_sums_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                          const float* x, int64_t ldx,
                                          float* stats, int64_t ld_stats);
int lbn_entrywise_batch_norm_fwd_stats_f32(lbn_stream_t stream, int64_t height,
                                           int64_t statistics_count, float decay,
                                           float* stats, int64_t ld_stats,
                                           float* running_mean, float* running_var);
int lbn_entrywise_batch_norm_fwd_apply_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                           float epsilon, const float* x, int64_t ldx,
                                           float* y, int64_t ldy,
                                           const float* mean, const float* var);
int lbn_entrywise_batch_norm_bwd_sums_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                          float epsilon, const float* x, int64_t ldx,
                                          const float* dy, int64_t lddy,
                                          const float* stats, int64_t ld_stats,
                                          float* stats_grad, int64_t ld_stats_grad);
int lbn_entrywise_batch_norm_bwd_apply_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                           int64_t statistics_count, float epsilon,
                                           const float* x, int64_t ldx,
                                           const float* dy, int64_t lddy, float* dx, int64_t lddx,
                                           const float* stats, int64_t ld_stats,
                                           const float* stats_grad, int64_t ld_stats_grad);

/* ------------------------------------------------------------------ batch norm
 * Replaces batch_normalization_layer::fp_compute / bp_compute
 * (src/layers/regularizers/batch_normalization.cpp:37-175, :178-329).
 * A sample is `channels` contiguous slabs of `channel_size` entries (NCHW flattened:
 * channel c = rows [c*cs,(c+1)*cs) of every column).  mean/var (length channels) are
 * the layer's m_mean_and_var columns; scale, bias, running_mean, running_var are
 * weights 0..3.  training != 0 computes batch statistics over channel_size*width
 * values (local statistics, statistics_group_size == 1), writes mean/var and updates
 * the running statistics with `decay`; training == 0 normalises with the running
 * statistics and leaves mean/var untouched.  bessel != 0 scales the variance by
 * n/(n-1) (the reference default).  The variance is clamped below at epsilon and
 * epsilon is added again under the square root, as the reference does.  The _f16
 * variants store x, y, dy, dx as IEEE binary16 and compute in fp32, with statistics,
 * weights and their gradients in fp32 (the accumulation type the reference's GPU code
 * uses for half data, BNAcc, batch_normalization.hpp:60-71). */
size_t lbn_batch_norm_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width);
int lbn_batch_norm_fwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                           int64_t width, int bessel, float epsilon, float decay,
                           int training, const float* x, int64_t ldx, float* y, int64_t ldy,
                           float* mean, float* var, const float* scale, const float* bias,
                           float* running_mean, float* running_var,
                           void* workspace, size_t workspace_bytes, int flags);
int lbn_batch_norm_bwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                           int64_t width, int bessel, float epsilon, int training,
                           const float* x, int64_t ldx, const float* dy, int64_t lddy,
                           float* dx, int64_t lddx, const float* mean, const float* var,
                           const float* running_mean, const float* running_var,
                           const float* scale, float* dscale, float* dbias,
                           float* dmean, float* dvar,
                           void* workspace, size_t workspace_bytes);
/* For parity tests only: lbn_batch_norm_bwd_f32 with the four per-channel gradients
 * accumulated as the reference CPU code does (batch_normalization.cpp:211-245: one
 * sequential fp32 sum each per channel, columns outer, rows inner, the reference's
 * per-entry expressions without fused multiply-adds), then the ordinary dx kernel on
 * those values.  With the statistics of an LBN_STATS_REFERENCE_ORDER forward, dscale,
 * dbias, dmean and dvar equal the CPU code's bit for bit.  Same arguments, workspace and
 * size limit (2^27 entries) as described for that flag. */
int lbn_batch_norm_bwd_reference_order_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                           int64_t width, int bessel, float epsilon, int training,
                                           const float* x, int64_t ldx, const float* dy, int64_t lddy,
                                           float* dx, int64_t lddx, const float* mean, const float* var,
                                           const float* running_mean, const float* running_var,
                                           const float* scale, float* dscale, float* dbias,
                                           float* dmean, float* dvar,
                                           void* workspace, size_t workspace_bytes);
int lbn_batch_norm_fwd_f16(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                           int64_t width, int bessel, float epsilon, float decay,
                           int training, const void* x, int64_t ldx, void* y, int64_t ldy,
                           float* mean, float* var, const float* scale, const float* bias,
                           float* running_mean, float* running_var,
                           void* workspace, size_t workspace_bytes, int flags);
int lbn_batch_norm_bwd_f16(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                           int64_t width, int bessel, float epsilon, int training,
                           const void* x, int64_t ldx, const void* dy, int64_t lddy,
                           void* dx, int64_t lddx, const float* mean, const float* var,
                           const float* running_mean, const float* running_var,
                           const float* scale, float* dscale, float* dbias,
                           float* dmean, float* dvar,
                           void* workspace, size_t workspace_bytes);

/* The same computation cut where the reference places its all-reduces, for callers
 * that aggregate statistics over several ranks (batch_normalization.cpp:87-115 and
 * :248-263): local sums -> [caller's all-reduce] -> statistics -> apply.
 * fwd_sums writes per-channel sum(x) into `mean` and sum(x^2) into `var`;
 * fwd_stats turns those sums over `num_per_sum` values into mean/variance in place
 * and updates the running statistics; fwd_apply normalises.  bwd_sums writes dscale,
 * dbias and the local parts of dmean, dvar; bwd_apply forms dx from the (reduced)
 * dmean, dvar and the global `num_per_sum`. */
int lbn_batch_norm_fwd_sums_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                int64_t width, const float* x, int64_t ldx,
                                float* mean, float* var,
                                void* workspace, size_t workspace_bytes);
int lbn_batch_norm_fwd_stats_f32(lbn_stream_t stream, int64_t channels, int64_t num_per_sum,
                                 int bessel, float epsilon, float decay,
                                 float* mean, float* var,
                                 float* running_mean, float* running_var);
int lbn_batch_norm_fwd_apply_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                 int64_t width, float epsilon, const float* x, int64_t ldx,
                                 float* y, int64_t ldy, const float* mean, const float* var,
                                 const float* scale, const float* bias);
int lbn_batch_norm_bwd_sums_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                int64_t width, float epsilon,
                                const float* x, int64_t ldx, const float* dy, int64_t lddy,
                                const float* mean, const float* var, const float* scale,
                                float* dscale, float* dbias, float* dmean, float* dvar,
                                void* workspace, size_t workspace_bytes);
int lbn_batch_norm_bwd_apply_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                 int64_t width, int64_t num_per_sum, int bessel, float epsilon,
                                 const float* x, int64_t ldx, const float* dy, int64_t lddy,
                                 float* dx, int64_t lddx, const float* mean, const float* var,
                                 const float* scale, const float* dmean, const float* dvar);

/* --------------------------------------------------------------------- softmax
 * Replaces softmax_layer::fp_compute / bp_compute on the data-parallel layout
 * (src/layers/activations/softmax.cpp:157-234), whose CPU arithmetic is
 * openmp_backend::softmax_forward / softmax_backward
 * (include/lbann/utils/dnn_lib/openmp/softmax.hpp:39-117, :119-181), mode INSTANCE:
 * softmax over each column.  Results that are not normal floats (zero, denormal, NaN)
 * are written as 0, as that code does.  y may alias x and dx may alias dy (the layer
 * can run in place, softmax.hpp:134).  Any height, leading dimension and 4-byte aligned
 * pointer is accepted.  Fastest: columns that start on 16-byte boundaries and a height
 * that is a multiple of 4.  Columns off that grid move one float at a time, except that
 * columns of 8000 entries or more still move as 16-byte vectors when the tensors of the
 * call (x and y; y, dy and dx) have pointers that agree modulo 16 bytes and leading
 * dimensions that agree modulo 4 entries. */
size_t lbn_softmax_workspace_bytes(int64_t height, int64_t width);
int lbn_softmax_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                        const float* x, int64_t ldx, float* y, int64_t ldy,
                        void* workspace, size_t workspace_bytes);
int lbn_softmax_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                        const float* y, int64_t ldy, const float* dy, int64_t lddy,
                        float* dx, int64_t lddx, void* workspace, size_t workspace_bytes);

/* For parity tests only (see LBN_STATS_REFERENCE_ORDER): softmax forward with the column's
 * denominator formed as the reference CPU code forms it (openmp/softmax.hpp:75-95: ONE
 * sequential fp32 sum of exp(x - max) in row order), and log-softmax backward with the
 * column's sum of dy formed likewise (log_softmax.cpp:108-118).  What the default kernels
 * add as trees then agrees with the CPU code to the last bits (the log-softmax sum bit for
 * bit; the softmax denominator up to the 1-ulp difference between two accurate exponential
 * functions).  One wave per column, one lane adding: rejected with LBN_ERR_UNSUPPORTED
 * above 2^27 entries.  No workspace. */
int lbn_softmax_fwd_reference_order_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                        const float* x, int64_t ldx, float* y, int64_t ldy);
int lbn_log_softmax_bwd_reference_order_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                            const float* y, int64_t ldy, const float* dy, int64_t lddy,
                                            float* dx, int64_t lddx);

/* Softmax forward for callers that cannot allocate device memory or hand over a
 * workspace: code running under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, results
 * and kernels as lbn_softmax_fwd_f32, but the scratch is an array that is part of the
 * library's code object (lbn_softmax_fwd_static_scratch_max_bytes() bytes, 1 MiB, held
 * by every GPU the library runs on until the process ends); the call itself allocates
 * and frees nothing.  Shapes with lbn_softmax_workspace_bytes(height, width) above that
 * size are rejected with LBN_ERR_UNSUPPORTED before anything is launched.  All calls on
 * one GPU share the array: two such calls that overlap in time on one GPU (different
 * streams, or concurrent graph replays) race on it and are not supported; calls on one
 * stream are ordered and safe.  Nothing in the array has to start at zero.
 *
 * The first call on a device looks up the array's address and creates the event that
 * orders cluster kernels across streams; neither may happen while a stream is recording
 * a graph, so callers that record call lbn_softmax_fwd_static_scratch_prepare() once per
 * device beforehand, with that device current (it launches nothing; calling it again is
 * harmless).  The array's first 64 bytes hold the sticky word of the bounded waits like any
 * workspace's; the caller never sees the array, so
 * lbn_softmax_fwd_static_scratch_timed_out() reads that word for the current device
 * (waits for `stream`, stores 0 or 1 in *timed_out) and clears it when it was raised.
 * lbn_selftest_cluster_wait_gives_up() with a NULL workspace raises it on purpose. */
size_t lbn_softmax_fwd_static_scratch_max_bytes(void);
int lbn_softmax_fwd_static_scratch_prepare(void);
int lbn_softmax_fwd_static_scratch_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                       const float* x, int64_t ldx, float* y, int64_t ldy);
int lbn_softmax_fwd_static_scratch_timed_out(lbn_stream_t stream, int* timed_out);

/* ----------------------------------------------------------------- log-softmax
 * Replaces log_softmax_layer::fp_compute / bp_compute
 * (src/layers/activations/log_softmax.cpp:35-93, :95-136, :140-156).
 * y = x - max - log(sum(exp(x - max))); dx = dy - exp(y) * sum(dy).  In place allowed
 * (log_softmax.hpp:101).  Shares lbn_softmax_workspace_bytes(). */
int lbn_log_softmax_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                            const float* x, int64_t ldx, float* y, int64_t ldy,
                            void* workspace, size_t workspace_bytes);
int lbn_log_softmax_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                            const float* y, int64_t ldy, const float* dy, int64_t lddy,
                            float* dx, int64_t lddx, void* workspace, size_t workspace_bytes);

/* fp16 storage for the two layers above: the reference instantiates softmax_layer and
 * log_softmax_layer for half precision too (src/layers/activations/softmax.cpp:236-243,
 * log_softmax.cpp:160-167, LBANN_INSTANTIATE_CPU_HALF / GPU_HALF).  x, y, dy, dx are IEEE
 * binary16 in memory; all arithmetic (maximum, exponentials, sums) is fp32, where the
 * reference's half instantiation also accumulates in half (the exponential is evaluated to a
 * relative error of about |x - max| * 3e-8, far inside binary16's rounding); results are rounded to nearest
 * even on store, and softmax's flush of non-normal results applies to the fp32 value before
 * rounding (binary16 denormals are kept).  Same arguments as the _f32 entry points (leading
 * dimensions in elements); the workspace is not used and may be NULL.  In place allowed. */
int lbn_softmax_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width,
                        const void* x, int64_t ldx, void* y, int64_t ldy,
                        void* workspace, size_t workspace_bytes);
int lbn_softmax_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width,
                        const void* y, int64_t ldy, const void* dy, int64_t lddy,
                        void* dx, int64_t lddx, void* workspace, size_t workspace_bytes);
int lbn_log_softmax_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width,
                            const void* x, int64_t ldx, void* y, int64_t ldy,
                            void* workspace, size_t workspace_bytes);
int lbn_log_softmax_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width,
                            const void* y, int64_t ldy, const void* dy, int64_t lddy,
                            void* dx, int64_t lddx, void* workspace, size_t workspace_bytes);

/* --------------------------------------------------------- channelwise softmax
 * Replaces channelwise_softmax_layer::fp_compute / bp_compute
 * (src/layers/misc/channelwise_softmax.cpp:41-113, :121-184).  Each sample holds
 * `channels` windows of `channel_size` contiguous entries, window j starting at row
 * j*channel_stride (get_channel_size_and_stride, channelwise_softmax_impl.hpp:58-104);
 * a softmax is taken inside every window.  No flush of denormal results.  In place
 * allowed (channelwise_softmax.hpp:78) when windows do not overlap. */
size_t lbn_channelwise_softmax_workspace_bytes(int64_t channels, int64_t channel_size,
                                               int64_t width);
int lbn_channelwise_softmax_fwd_f32(lbn_stream_t stream, int64_t channels,
                                    int64_t channel_size, int64_t channel_stride,
                                    int64_t width, const float* x, int64_t ldx,
                                    float* y, int64_t ldy,
                                    void* workspace, size_t workspace_bytes);
int lbn_channelwise_softmax_bwd_f32(lbn_stream_t stream, int64_t channels,
                                    int64_t channel_size, int64_t channel_stride,
                                    int64_t width, const float* y, int64_t ldy,
                                    const float* dy, int64_t lddy, float* dx, int64_t lddx,
                                    void* workspace, size_t workspace_bytes);

/* --------------------------------------------------------------- cross entropy
 * The layer that consumes the softmax output.  Replaces
 * cross_entropy_layer::local_fp_compute / local_bp_compute
 * (src/layers/loss/cross_entropy.cpp:35-73, :75-120; GPU code cross_entropy.cu).
 * loss[c*ld_loss] = -sum over rows with xhat > 0 of xhat * log(prediction) for column c
 * (the layer's 1 x width workspace matrix, before its sum across ranks,
 * cross_entropy_impl.hpp:186-201).  Backward: dprediction = -dloss * xhat / prediction
 * where xhat > 0 and 0 elsewhere; dground_truth = -dloss * log(prediction), with
 * dloss[c*ld_dloss] the gradient w.r.t. column c's loss.
 * use_labels == 0: ground_truth has the shape of prediction.  use_labels != 0: it
 * holds one class index per spatial position, stored as a floating-point number in rows
 * [0, spatial_size) of its column; row r of prediction is class r / spatial_size at
 * position r % spatial_size and xhat(r) = 1 where the position's label, converted to
 * int, equals the class, else 0; dground_truth is not written and may be NULL (with a dense
 * ground truth it is written unless it is NULL).
 * spatial_size is ignored when use_labels == 0. */
size_t lbn_cross_entropy_fwd_workspace_bytes(int64_t height, int64_t width);
int lbn_cross_entropy_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size,
                              const float* prediction, int64_t ld_prediction,
                              const float* ground_truth, int64_t ld_ground_truth,
                              float* loss, int64_t ld_loss,
                              void* workspace, size_t workspace_bytes);
int lbn_cross_entropy_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size,
                              const float* prediction, int64_t ld_prediction,
                              const float* ground_truth, int64_t ld_ground_truth,
                              const float* dloss, int64_t ld_dloss,
                              float* dprediction, int64_t ld_dprediction,
                              float* dground_truth, int64_t ld_dground_truth);

/* fp16 storage: the reference instantiates cross_entropy_layer for half precision too
 * (src/layers/loss/cross_entropy.cpp:157-166, LBANN_INSTANTIATE_CPU_HALF).  Every matrix
 * (prediction, ground truth, loss, dloss and the two gradients) is IEEE binary16 in memory;
 * logarithms, products and the sum over a column are fp32, where the reference's half
 * instantiation also accumulates in half; results are rounded to nearest even on store (a
 * loss or gradient beyond 65504 becomes infinite).  Labels are class indices stored as
 * binary16, exact up to 2048.  Same arguments as the _f32 entry points, leading dimensions
 * in elements; the workspace (fp32 partial sums) has the same size. */
int lbn_cross_entropy_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size,
                              const void* prediction, int64_t ld_prediction,
                              const void* ground_truth, int64_t ld_ground_truth,
                              void* loss, int64_t ld_loss,
                              void* workspace, size_t workspace_bytes);
int lbn_cross_entropy_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size,
                              const void* prediction, int64_t ld_prediction,
                              const void* ground_truth, int64_t ld_ground_truth,
                              const void* dloss, int64_t ld_dloss,
                              void* dprediction, int64_t ld_dprediction,
                              void* dground_truth, int64_t ld_dground_truth);

/* Softmax forward and the cross-entropy forward of its output in one pass: y as
 * lbn_softmax_fwd_f32 writes it (softmax.cpp:43-109, flush included) and loss as
 * lbn_cross_entropy_fwd_f32(prediction = y) gives it (cross_entropy.cpp:35-73), for the
 * softmax -> cross_entropy pair that ends the reference's classification models.  The
 * results are those of the two calls made one after the other; the cross entropy reads y
 * from registers instead of from memory.  Rows that fit a workgroup's registers
 * (height a multiple of 4, 16-byte aligned columns, at most 32768 entries) with a dense
 * ground truth, or labels with spatial_size == 1, take the fused kernel; every other shape
 * runs the two layers' kernels back to back inside this call.  The workspace serves both.
 *
 * Backward of the same pair: dx, the gradient with respect to the softmax input, from y, the
 * ground truth and dloss (the gradient of column c's loss at dloss[c*ld_dloss]), i.e. what
 * lbn_cross_entropy_bwd_f32 (cross_entropy.cpp:75-120) followed by lbn_softmax_bwd_f32
 * (openmp/softmax.hpp:119-181) computes, with the same operations, without writing the
 * gradient with respect to the prediction in between (three tensors of traffic instead of
 * seven).  dground_truth (dense ground truth only) is written when it is not NULL.  Shapes
 * outside the fused kernel run the two kernels inside the call, the first leaving its result
 * in dx and the second working in place on it; workspace as for lbn_softmax_bwd_f32
 * (lbn_softmax_workspace_bytes). */
size_t lbn_softmax_cross_entropy_fwd_workspace_bytes(int64_t height, int64_t width);
int lbn_softmax_cross_entropy_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                                      int64_t spatial_size,
                                      const float* x, int64_t ldx,
                                      const float* ground_truth, int64_t ld_ground_truth,
                                      float* y, int64_t ldy,
                                      float* loss, int64_t ld_loss,
                                      void* workspace, size_t workspace_bytes);
int lbn_softmax_cross_entropy_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                                      int64_t spatial_size,
                                      const float* y, int64_t ldy,
                                      const float* ground_truth, int64_t ld_ground_truth,
                                      const float* dloss, int64_t ld_dloss,
                                      float* dx, int64_t lddx,
                                      float* dground_truth, int64_t ld_dground_truth,
                                      void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------- scale and bias layers
 * The learned affine layers that follow a normalization layer without one.  Replace
 * entrywise_scale_bias_layer::fp_compute / bp_compute
 * (src/layers/learning/entrywise_scale_bias.cpp:35-60, :62-113) and
 * channelwise_scale_bias_layer::fp_compute / bp_compute
 * (src/layers/learning/channelwise_scale_bias.cpp:33-73, :75-135).
 * y = a*x + b; dx = a*dy; da = sum(x*dy), db = sum(dy) over everything that shares the
 * pair (a, b): one pair per matrix row over the mini-batch (entry-wise), or one per
 * channel = rows [c*channel_size, (c+1)*channel_size) of every column (channel-wise).
 * weights is the layer's single weights matrix, (height x 2) resp. (channels x 2):
 * column 0 scale, column 1 bias; weights_grad has the same shape and is overwritten
 * (the caller adds it to the optimizer's gradient, entrywise_scale_bias.cpp:139-145). */
int lbn_entrywise_scale_bias_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                     const float* x, int64_t ldx, float* y, int64_t ldy,
                                     const float* weights, int64_t ld_weights);
size_t lbn_entrywise_scale_bias_bwd_workspace_bytes(int64_t height, int64_t width);
int lbn_entrywise_scale_bias_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                     const float* x, int64_t ldx, const float* dy, int64_t lddy,
                                     float* dx, int64_t lddx,
                                     const float* weights, int64_t ld_weights,
                                     float* weights_grad, int64_t ld_weights_grad,
                                     void* workspace, size_t workspace_bytes);
int lbn_channelwise_scale_bias_fwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                       int64_t width, const float* x, int64_t ldx,
                                       float* y, int64_t ldy,
                                       const float* weights, int64_t ld_weights);
size_t lbn_channelwise_scale_bias_bwd_workspace_bytes(int64_t channels, int64_t channel_size,
                                                      int64_t width);
int lbn_channelwise_scale_bias_bwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                       int64_t width, const float* x, int64_t ldx,
                                       const float* dy, int64_t lddy, float* dx, int64_t lddx,
                                       const float* weights, int64_t ld_weights,
                                       float* weights_grad, int64_t ld_weights_grad,
                                       void* workspace, size_t workspace_bytes);

/* ------------------------------------------------ the optimizer's gradient buffer
 * Where dscale / dbias / weights_grad go next.  Replaces the Scale + Axpy pair of
 * optimizer::add_to_gradient (include/lbann/optimizers/optimizer_impl.hpp:207-217) on
 * the local (height x width, column-major) matrices:
 *   gradient = buf_scale * gradient + in_scale * contribution
 * with buf_scale and in_scale as get_gradient_buffer (:219-288) picks them from the
 * buffer's status (cleared: 0 and 1; ready: 1 and 1), in_scale already multiplied by
 * add_to_gradient's scale argument.  buf_scale == 0 overwrites: the buffer's previous
 * contents are not read (they may never have been initialised).  Each product and the
 * sum are rounded separately, like the two library calls. */
int lbn_gradient_sink_f32(lbn_stream_t stream, int64_t height, int64_t width, float buf_scale,
                          float in_scale, const float* contribution, int64_t ld_contribution,
                          float* gradient, int64_t ld_gradient);

/* ------------------------------------------- the five layers for double precision
 * The reference instantiates its layers for TensorDataType = double when it is built with
 * LBANN_HAS_DOUBLE (include/lbann/macros/instantiate.hpp:28-30,
 * src/layers/regularizers/layer_norm_builder.cpp:48-54, batch_normalization_builder.cpp,
 * softmax.cpp / log_softmax.cpp / channelwise_softmax.cpp instantiations).  These entry points
 * are the _f32 ones with every matrix, statistic, weight and epsilon in binary64 and all
 * arithmetic in binary64; arguments mean what they mean there (sizes, leading dimensions in
 * elements, NULL rules, in-place rules, LBN_STATS_TWO_PASS / LBN_STATS_SUMSQ).  Differences:
 * the softmax family and the layer-norm forward use no scratch (no workspace arguments);
 * layer-norm backward needs lbn_layer_norm_bwd_workspace_bytes_f64() only for weight
 * gradients; batch norm always needs lbn_batch_norm_workspace_bytes_f64() in training mode
 * and in backward.  Workspaces are 16-byte aligned.  No kernel here waits across workgroups.
 * Batch norm channels are limited to 2^31 - 1 entries (channel_size * width). */
int lbn_softmax_fwd_f64(lbn_stream_t stream, int64_t height, int64_t width,
                        const double* x, int64_t ldx, double* y, int64_t ldy);
int lbn_softmax_bwd_f64(lbn_stream_t stream, int64_t height, int64_t width,
                        const double* y, int64_t ldy, const double* dy, int64_t lddy,
                        double* dx, int64_t lddx);
int lbn_log_softmax_fwd_f64(lbn_stream_t stream, int64_t height, int64_t width,
                            const double* x, int64_t ldx, double* y, int64_t ldy);
int lbn_log_softmax_bwd_f64(lbn_stream_t stream, int64_t height, int64_t width,
                            const double* y, int64_t ldy, const double* dy, int64_t lddy,
                            double* dx, int64_t lddx);
int lbn_channelwise_softmax_fwd_f64(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width,
                                    const double* x, int64_t ldx, double* y, int64_t ldy);
int lbn_channelwise_softmax_bwd_f64(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width,
                                    const double* y, int64_t ldy, const double* dy, int64_t lddy,
                                    double* dx, int64_t lddx);
int lbn_layer_norm_fwd_f64(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, double epsilon,
                           const double* x, int64_t ldx, double* y, int64_t ldy,
                           double* stats, int64_t ld_stats,
                           const double* scale, const double* bias, int flags);
size_t lbn_layer_norm_bwd_workspace_bytes_f64(int64_t num_groups, int64_t norm_size,
                                              int64_t width, int has_weight_grads);
int lbn_layer_norm_bwd_f64(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, double epsilon,
                           const double* x, int64_t ldx, const double* dy, int64_t lddy,
                           double* dx, int64_t lddx, const double* stats, int64_t ld_stats,
                           double* stats_grad, int64_t ld_stats_grad,
                           const double* scale, double* dscale, double* dbias,
                           void* workspace, size_t workspace_bytes);
size_t lbn_batch_norm_workspace_bytes_f64(int64_t channels, int64_t channel_size, int64_t width);
int lbn_batch_norm_fwd_f64(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                           int64_t width, int bessel, double epsilon, double decay,
                           int training, const double* x, int64_t ldx, double* y, int64_t ldy,
                           double* mean, double* var, const double* scale, const double* bias,
                           double* running_mean, double* running_var,
                           void* workspace, size_t workspace_bytes, int flags);
int lbn_batch_norm_bwd_f64(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                           int64_t width, int bessel, double epsilon, int training,
                           const double* x, int64_t ldx, const double* dy, int64_t lddy,
                           double* dx, int64_t lddx, const double* mean, const double* var,
                           const double* running_mean, const double* running_var,
                           const double* scale, double* dscale, double* dbias,
                           double* dmean, double* dvar,
                           void* workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* LBNORM_H_INCLUDED */
