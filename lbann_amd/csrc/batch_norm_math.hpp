// Per-channel batch-norm formulas shared by the kernels of batch_norm.hip and
// batch_norm_rows.hpp.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace lbn {

// Mean / variance from sums about pivot K over n values, with the reference's Bessel
// factor and epsilon floor (batch_normalization.cpp:118-131).
__device__ __forceinline__ void stats_from_sums(float s, float q, float K, int64_t n, int bessel,
                                                float eps, float& mean, float& var)
{
  const float nf = static_cast<float>(n);
  const float dm = s / nf;
  const float sqmean = q / nf;
  mean = K + dm;
  var = nf * (sqmean - dm * dm) / (nf - static_cast<float>(bessel ? 1 : 0));
  var = fmaxf(var, eps);
}

// The four gradients of a channel from A = sum(dy) and B = sum(dy * (x - mean))
// (batch_normalization.cpp:211-245).
__device__ __forceinline__ void grads_from_sums(float A, float B, float scale, float inv_stdev,
                                                float& dscale, float& dbias, float& dmean,
                                                float& dvar)
{
  dscale = B * inv_stdev;
  dbias = A;
  dmean = -(scale * inv_stdev) * A;
  dvar = -scale * B * (inv_stdev * inv_stdev * inv_stdev / 2);
}

}  // namespace lbn
