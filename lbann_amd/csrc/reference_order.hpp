// Statistics in the reference's own order of summation, for parity tests only.
//
// The reference CPU code forms every per-channel (batch norm) or per-row (layer norm) sum as ONE
// sequential fp32 accumulation in loop order (batch_normalization.cpp:70-85 and :211-245: columns
// outer, rows of the channel inner; layer_norm.cpp:77-88: the row's entries in order).  The
// production kernels add the same terms as trees, which is more accurate and differs from the
// reference by the reference's own rounding error (1e-5 to 1e-4 over 2e5 terms).  The kernels
// here redo those sums the reference's way: one wave per channel or row loads 256 entries at a
// time (coalesced), parks them in LDS, and a single lane adds them in index order with separate
// multiplications and additions (no fused multiply-add, as the reference is compiled), then
// finishes the statistics with the reference's expression, operation for operation.  With them
// the statistics agree with the CPU code bit for bit, which shows that summation order is all
// that separates the two.  Selected only by LBN_STATS_REFERENCE_ORDER / the *_reference_order
// entry point, never by default, and rejected above kRefOrderMaxEntries entries per tensor:
// one lane per channel is thousands of times slower than the production kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cfloat>
#include <cstdint>

#include "device_utils.hpp"

namespace lbn {

constexpr int64_t kRefOrderMaxEntries = int64_t(1) << 27;
constexpr int kRefChunk = 4 * kWave;  // entries parked in LDS per round: four per lane

// Visits entries 0 .. total-1 of an item in order.  load(idx, out[NT]) fetches the NT values of
// entry idx (all lanes, any order); add(v[NT]) is called by lane 0 alone, once per entry, in
// index order.  `buf` is NT x kRefChunk floats of LDS.  Called by the one wave of a workgroup.
template <int NT, typename Load, typename Add>
__device__ __forceinline__ void ref_order_walk(int64_t total, float (*buf)[kRefChunk], Load load, Add add)
{
  const int lane = threadIdx.x;
  float r[4][NT];
  auto fetch = [&](int64_t base) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t idx = base + kWave * j + lane;
#pragma unroll
      for (int t = 0; t < NT; ++t) r[j][t] = 0.f;
      if (idx < total) load(idx, r[j]);
    }
  };
  fetch(0);
  for (int64_t base = 0; base < total; base += kRefChunk) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < NT; ++t) buf[t][kWave * j + lane] = r[j][t];
    __syncthreads();
    if (base + kRefChunk < total) fetch(base + kRefChunk);  // in flight while lane 0 adds
    if (lane == 0) {
      const int cnt = total - base < kRefChunk ? static_cast<int>(total - base) : kRefChunk;
      for (int i = 0; i < cnt; ++i) {
        float v[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) v[t] = buf[t][i];
        add(v);
      }
    }
    __syncthreads();
  }
}

// The reference's arithmetic, one IEEE operation at a time: the pragma keeps the compiler from
// contracting a multiplication and an addition into a fused multiply-add, in these functions and
// wherever they are inlined.  Division and square root are the correctly rounded ones (hipcc's
// default for fp32).
__device__ __forceinline__ float ref_add(float a, float b)
{
#pragma clang fp contract(off)
  return a + b;
}
__device__ __forceinline__ float ref_sub(float a, float b)
{
#pragma clang fp contract(off)
  return a - b;
}
__device__ __forceinline__ float ref_mul(float a, float b)
{
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float ref_div(float a, float b)
{
#pragma clang fp contract(off)
  return a / b;
}

// 1 / sqrt(var + eps) as the reference writes it.
__device__ __forceinline__ float ref_inv_stdev(float var, float eps)
{
  return ref_div(1.f, sqrtf(ref_add(var, eps)));
}

// ------------------------------------------------------------------- batch norm
// Forward statistics of channel blockIdx.x (batch_normalization.cpp:70-85, :118-138): writes
// mean, var and updates the running statistics.
template <typename S>
__global__ void __launch_bounds__(kWave)
bn_ref_order_fwd_stats(const S* __restrict__ x, int64_t ldx, int64_t cs, int64_t w, int bessel, float eps,
                       float decay, float* __restrict__ mean, float* __restrict__ var,
                       float* __restrict__ rmean, float* __restrict__ rvar)
{
  __shared__ float buf[1][kRefChunk];
  const int64_t c = blockIdx.x;
  const S* xc = x + c * cs;
  const int64_t total = cs * w;
  float sum = 0.f, sqsum = 0.f;
  ref_order_walk<1>(
    total, buf,
    [&](int64_t idx, float (&v)[1]) {
      const int64_t col = idx / cs;
      v[0] = Vec16<S>::load1(xc + col * ldx + (idx - col * cs));
    },
    [&](const float (&v)[1]) {
      sum = ref_add(sum, v[0]);
      sqsum = ref_add(sqsum, ref_mul(v[0], v[0]));
    });
  if (threadIdx.x != 0) return;
  if (total <= 1) {  // :119-121: the variance is set to one, the "mean" stays the sum
    mean[c] = sum;
    var[c] = 1.f;
    return;
  }
  const float nf = static_cast<float>(total);
  const float m = ref_div(sum, nf);
  const float sqmean = ref_div(sqsum, nf);
  float v = ref_div(ref_mul(nf, ref_sub(sqmean, ref_mul(m, m))),
                      ref_sub(nf, static_cast<float>(bessel ? 1 : 0)));
  v = fmaxf(v, eps);
  mean[c] = m;
  var[c] = v;
  const float keep = ref_sub(1.f, decay);
  rmean[c] = ref_add(ref_mul(decay, rmean[c]), ref_mul(keep, m));
  rvar[c] = ref_add(ref_mul(decay, rvar[c]), ref_mul(keep, v));
}

// The four per-channel gradients of channel blockIdx.x (batch_normalization.cpp:211-245).
template <typename S>
__global__ void __launch_bounds__(kWave)
bn_ref_order_bwd_sums(const S* __restrict__ x, const S* __restrict__ dy, int64_t ldx, int64_t lddy, int64_t cs,
                      int64_t w, float eps, int training, const float* __restrict__ mean_in,
                      const float* __restrict__ var_in, const float* __restrict__ gamma,
                      float* __restrict__ dscale_out, float* __restrict__ dbias_out,
                      float* __restrict__ dmean_out, float* __restrict__ dvar_out)
{
  __shared__ float buf[2][kRefChunk];
  const int64_t c = blockIdx.x;
  const S* xc = x + c * cs;
  const S* gc = dy + c * cs;
  const int64_t total = cs * w;
  const float mean = mean_in[c];
  const float scale = gamma[c];
  const float inv_stdev = ref_inv_stdev(var_in[c], eps);
  const float dvar_factor = ref_div(ref_mul(ref_mul(inv_stdev, inv_stdev), inv_stdev), 2.f);
  float dmean = 0.f, dvar = 0.f, dscale = 0.f, dbias = 0.f;
  ref_order_walk<2>(
    total, buf,
    [&](int64_t idx, float (&v)[2]) {
      const int64_t col = idx / cs;
      const int64_t row = idx - col * cs;
      v[0] = Vec16<S>::load1(xc + col * ldx + row);
      v[1] = Vec16<S>::load1(gc + col * lddy + row);
    },
    [&](const float (&v)[2]) {
      const float d = ref_sub(v[0], mean);
      const float xhat = ref_mul(d, inv_stdev);
      const float g = v[1];
      dscale = ref_add(dscale, ref_mul(g, xhat));
      dbias = ref_add(dbias, g);
      const float ndxhat = -ref_mul(g, scale);
      dmean = ref_add(dmean, ref_mul(ndxhat, inv_stdev));
      dvar = ref_add(dvar, ref_mul(ref_mul(ndxhat, d), dvar_factor));
    });
  if (threadIdx.x != 0) return;
  dscale_out[c] = dscale;
  dbias_out[c] = dbias;
  dmean_out[c] = training ? dmean : 0.f;  // :262-265: dropped outside training
  dvar_out[c] = training ? dvar : 0.f;
}

// ------------------------------------------------------------------- layer norm
// Statistics of row blockIdx.x (layer_norm.cpp:77-112) and the row's output (:117-135), the
// latter by all lanes with the reference's operations in its order (scale, then bias).
template <typename T, typename Map>
__global__ void __launch_bounds__(kWave)
ln_ref_order_fwd(const T* __restrict__ x, T* __restrict__ y, int64_t ldx, int64_t ldy, Map map, int64_t n,
                 float eps, float* __restrict__ stats, int64_t ld_stats, const float* __restrict__ gamma,
                 const float* __restrict__ beta)
{
  __shared__ float buf[1][kRefChunk];
  __shared__ float result[2];
  const int64_t row = blockIdx.x;
  int64_t col, g;
  map.split(row, col, g);
  const T* xr = x + g * map.stride + col * ldx;
  T* yr = y + g * map.stride + col * ldy;
  float sum = 0.f, sqsum = 0.f;
  ref_order_walk<1>(
    n, buf, [&](int64_t idx, float (&v)[1]) { v[0] = Vec16<T>::load1(xr + idx); },
    [&](const float (&v)[1]) {
      sum = ref_add(sum, v[0]);
      sqsum = ref_add(sqsum, ref_mul(v[0], v[0]));
    });
  if (threadIdx.x == 0) {
    float mean = sum, var = 1.f;  // :92-95: a row of one entry keeps its sum and a variance of one
    if (n > 1) {
      const float nf = static_cast<float>(n);
      mean = ref_div(sum, nf);
      var = fmaxf(ref_sub(ref_div(sqsum, nf), ref_mul(mean, mean)), 0.f);
    }
    stats[g + col * ld_stats] = mean;
    stats[map.groups + g + col * ld_stats] = var;
    result[0] = mean;
    result[1] = var;
  }
  __syncthreads();
  const float mean = result[0];
  const float inv_stdev = ref_inv_stdev(result[1], eps);
  for (int64_t k = threadIdx.x; k < n; k += kWave) {
    float r = ref_mul(ref_sub(Vec16<T>::load1(xr + k), mean), inv_stdev);
    if (gamma) r = ref_mul(r, gamma[k]);
    if (beta) r = ref_add(r, beta[k]);
    Vec16<T>::store1(yr + k, r);
  }
}

// ------------------------------------------------------------------- softmax family
// Softmax forward of column blockIdx.x as openmp/softmax.hpp:39-117 computes it: the column's
// maximum, then ONE sequential fp32 sum of exp(x - max) in row order (the exponentials themselves
// are evaluated by all lanes, with the accurate library exponential), then y = (1 / sum) * exp,
// non-normal results flushed to zero.
static __global__ void __launch_bounds__(kWave)
sm_ref_order_fwd(const float* __restrict__ x, float* __restrict__ y, int64_t ldx, int64_t ldy, int64_t h)
{
  __shared__ float buf[1][kRefChunk];
  __shared__ float result;
  const float* xc = x + static_cast<int64_t>(blockIdx.x) * ldx;
  float* yc = y + static_cast<int64_t>(blockIdx.x) * ldy;
  float m = -FLT_MAX;
  for (int64_t r = threadIdx.x; r < h; r += kWave) m = fmaxf(m, xc[r]);
  m = wave_max(m);
  float sum = 0.f;
  ref_order_walk<1>(
    h, buf,
    [&](int64_t idx, float (&v)[1]) {
      v[0] = expf(ref_sub(xc[idx], m));
      yc[idx] = v[0];  // in place safe: x[idx] is not read again
    },
    [&](const float (&v)[1]) { sum = ref_add(sum, v[0]); });
  if (threadIdx.x == 0) result = ref_div(1.f, sum);
  __syncthreads();
  const float scale = result;
  for (int64_t r = threadIdx.x; r < h; r += kWave) {
    const float t = ref_mul(scale, yc[r]);
    yc[r] = __builtin_isnormal(t) ? t : 0.f;
  }
}

// Log-softmax backward of column blockIdx.x as log_softmax.cpp:95-136 computes it: ONE sequential
// fp32 sum of dy in row order, then dx = dy - exp(y) * sum.
static __global__ void __launch_bounds__(kWave)
lsm_ref_order_bwd(const float* __restrict__ y, const float* __restrict__ dy, float* __restrict__ dx, int64_t ldy,
                  int64_t lddy, int64_t lddx, int64_t h)
{
  __shared__ float buf[1][kRefChunk];
  __shared__ float result;
  const float* yc = y + static_cast<int64_t>(blockIdx.x) * ldy;
  const float* gc = dy + static_cast<int64_t>(blockIdx.x) * lddy;
  float* dc = dx + static_cast<int64_t>(blockIdx.x) * lddx;
  float sum = 0.f;
  ref_order_walk<1>(
    h, buf, [&](int64_t idx, float (&v)[1]) { v[0] = gc[idx]; },
    [&](const float (&v)[1]) { sum = ref_add(sum, v[0]); });
  if (threadIdx.x == 0) result = sum;
  __syncthreads();
  const float s = result;
  for (int64_t r = threadIdx.x; r < h; r += kWave) dc[r] = ref_sub(gc[r], ref_mul(expf(yc[r]), s));
}

// Entry-wise batch norm forward (training) as the CPU code computes it
// (entrywise_batch_normalization.cpp:77-124, :136-163): per entry one sequential sum of x and of
// x * x over the columns in order, mean = sum / w, variance = (sqsum / w - mean * mean) * w / (w - 1)
// WITHOUT a clamp (a negative value then gives NaN outputs, as it does there), running statistics,
// y = (x - mean) * (1 / sqrt(var + eps)).  One thread per entry: consecutive lanes read consecutive
// rows of a column.
static __global__ void __launch_bounds__(256)
ebn_ref_order_fwd(int64_t h, int64_t w, float decay, float eps, const float* __restrict__ x, int64_t ldx,
                  float* __restrict__ y, int64_t ldy, float* __restrict__ stats, int64_t ld_stats,
                  float* __restrict__ rmean, float* __restrict__ rvar)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= h) return;
  float sum = 0.f, sqsum = 0.f;
  for (int64_t c = 0; c < w; ++c) {
    const float v = x[r + c * ldx];
    sum = ref_add(sum, v);
    sqsum = ref_add(sqsum, ref_mul(v, v));
  }
  float mean = sum, var = 1.f;
  if (w > 1) {
    const float wf = static_cast<float>(w);
    mean = ref_div(sum, wf);
    const float sqmean = ref_div(sqsum, wf);
    var = ref_div(ref_mul(ref_sub(sqmean, ref_mul(mean, mean)), wf), ref_sub(wf, 1.f));
    const float keep = ref_sub(1.f, decay);
    rmean[r] = ref_add(ref_mul(decay, rmean[r]), ref_mul(keep, mean));
    rvar[r] = ref_add(ref_mul(decay, rvar[r]), ref_mul(keep, var));
  }
  stats[r] = mean;
  stats[r + ld_stats] = var;
  const float inv_stdev = ref_inv_stdev(var, eps);
  for (int64_t c = 0; c < w; ++c) y[r + c * ldy] = ref_mul(ref_sub(x[r + c * ldx], mean), inv_stdev);
}

}  // namespace lbn
