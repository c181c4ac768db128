// Entry-wise batch norm over a mini-batch wider than the register tiles when the matrix has
// too few rows to fill the device with one workgroup per 64 rows (4096 entries x 2048
// samples: 64 workgroups): the columns are cut into slabs that sum side by side, the slabs'
// partial sums are added in slab order, and the output is written on a (row blocks x column
// chunks) grid.  These are the kernels of the forward -> [all-reduce] -> apply cut
// (entrywise_batch_norm_split.hip), with the reference's own formula for the statistics
// (entrywise_batch_normalization.cpp:101-125).  Needs scratch for the partial sums.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace lbn {

// Scratch the slab path wants for an (h x w) problem; 0: the path does not apply.
size_t ebn_slab_workspace_bytes(int64_t h, int64_t w);

// Both return false when the shape, the alignment or the scratch does not allow the path
// (nothing was launched; the caller goes on to its own kernels).
bool ebn_slab_fwd(hipStream_t st, int64_t h, int64_t w, float eps, float decay, const float* x, int64_t ldx, float* y,
                  int64_t ldy, float* stats, int64_t ld_stats, float* running_mean, float* running_var, void* ws,
                  size_t ws_bytes);
bool ebn_slab_bwd(hipStream_t st, int64_t h, int64_t w, float eps, const float* x, int64_t ldx, const float* dy,
                  int64_t lddy, float* dx, int64_t lddx, const float* stats, int64_t ld_stats, float* stats_grad,
                  int64_t ld_stats_grad, void* ws, size_t ws_bytes);

// Outside training: y = (x - running_mean) / sqrt(running_var + eps) and dx = dy / sqrt(running_var
// + eps) (entrywise_batch_normalization.cpp:131-160, :352-392) on a (row blocks x column chunks)
// grid, whatever the alignment.  (One thread per row walking every column left a 4096-row
// matrix with 16 workgroups: 89 us for 4096 x 2048.)
void ebn_inference_fwd(hipStream_t st, int64_t h, int64_t w, float eps, const float* x, int64_t ldx, float* y,
                       int64_t ldy, const float* running_mean, const float* running_var);
void ebn_inference_bwd(hipStream_t st, int64_t h, int64_t w, float eps, const float* dy, int64_t lddy, float* dx,
                       int64_t lddx, const float* running_var);

}  // namespace lbn
