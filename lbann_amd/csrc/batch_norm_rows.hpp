// Batch norm for channels that are not a whole number of 16-byte vectors (channel_size
// 1 after a fully-connected layer, 49 for 7 x 7 feature maps, ...), fp32.  The kernels of
// batch_norm.hip walk a channel's segments, which then start at odd offsets and, for tiny
// channels, are a few bytes per column; here lanes run along consecutive matrix ROWS
// instead (row_tiles.hpp), whatever channel a row belongs to:
//
//   bn_rt_*_sums    per-row partial pairs over the columns of a slab -> part[slab][row]
//   bn_rt_*_stats   one wave per channel adds the pairs of its rows and slabs in a fixed
//                   order and finishes the channel: statistics and running statistics
//                   (forward), dscale, dbias, dmean, dvar (backward)
//   bn_rt_*_apply   elementwise pass with per-row coefficients looked up by row / cs
//
// Math, formulas and special cases as in batch_norm.hip (batch_normalization.cpp:37-175,
// :178-329).  x (and dy) are read twice; the second read comes from the caches when the
// tensors fit.
#pragma once

#include "batch_norm_math.hpp"
#include "device_utils.hpp"
#include "row_tiles.hpp"

namespace lbn {

struct BnRtArgs {
  int64_t h, w, cs;
  const float* x;
  const float* dy;
  float* out;  // y or dx
  int64_t ldx, lddy, ldo;
  int64_t slab_width;
  float2* part;  // [slabs][h]
  int use_pivot;
  float eps;
  const float* mean;
  const float* var;
  const float* scale;
  const float* bias;
  const float* dmean;
  const float* dvar;
  float count;         // n = channel_size * width
  float count_bessel;  // n - 1 with Bessel's correction, else n
  int zero;            // n <= 1: dx = 0
};

// Forward: (s, q) = sums of (x - K) and (x - K)^2 with K the first entry of the row's
// channel (0 for the reference's E[x^2] - mean^2 formula).  Backward: (A, B) = sums of dy
// and dy * (x - mean).
template <int GW, bool BWD>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_sums(BnRtArgs a)
{
  using P = RowTilePos<GW>;
  __shared__ float lds[kRowTileWaves][P::kRows][2];
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  const bool row_ok = r0 < a.h;  // h is a multiple of 4
  const int64_t rr = row_ok ? r0 : 0;
  const int64_t c0 = static_cast<int64_t>(blockIdx.y) * a.slab_width;
  const int64_t c1 = row_ok ? imin64(c0 + a.slab_width, a.w) : 0;
  float K[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t ch = (rr + r) / a.cs;
    K[r] = BWD ? a.mean[ch] : (a.use_pivot ? a.x[ch * a.cs] : 0.f);
  }
  float sa[4] = {0.f, 0.f, 0.f, 0.f}, sb[4] = {0.f, 0.f, 0.f, 0.f};
  auto add = [&](const float (&v)[4], const float (&g)[4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float d = v[r] - K[r];
      if (BWD) {
        sa[r] += g[r];
        sb[r] = __builtin_fmaf(g[r], d, sb[r]);
      }
      else {
        sa[r] += d;
        sb[r] = __builtin_fmaf(d, d, sb[r]);
      }
    }
  };
  int64_t c = c0 + p.g;
  for (; c + P::kGroups < c1; c += 2 * P::kGroups) {
    float v[2][4], g[2][4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Vec16<float>::load(a.x + rr + (c + j * P::kGroups) * a.ldx, v[j]);
      if (BWD) Vec16<float>::load(a.dy + rr + (c + j * P::kGroups) * a.lddy, g[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) add(v[j], g[j]);
  }
  for (; c < c1; c += P::kGroups) {
    float v[4], g[4];
    Vec16<float>::load(a.x + rr + c * a.ldx, v);
    if (BWD) Vec16<float>::load(a.dy + rr + c * a.lddy, g);
    add(v, g);
  }
  row_tile_merge<GW>(sa, sb, lds, p);
  if (p.g != 0 || !row_ok) return;
  float2* dst = a.part + static_cast<int64_t>(blockIdx.y) * a.h + r0;
#pragma unroll
  for (int r = 0; r < 4; ++r) dst[r] = make_float2(sa[r], sb[r]);
}

// Totals of channel c: lane-strided over its cs rows x slabs entries, then one wave sum;
// every lane gets them.
__device__ __forceinline__ float2 bn_rt_channel_total(const float2* part, int64_t h, int slabs, int64_t cs,
                                                      int64_t c)
{
  const int lane = threadIdx.x & (kWave - 1);
  float a = 0.f, b = 0.f;
  for (int s = 0; s < slabs; ++s) {
    const float2* row = part + static_cast<int64_t>(s) * h + c * cs;
    for (int64_t i = lane; i < cs; i += kWave) {
      const float2 v = row[i];
      a += v.x;
      b += v.y;
    }
  }
  return make_float2(wave_sum(a), wave_sum(b));
}

// One wave per channel (4 channels per workgroup).
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_fwd_stats(int64_t C, int64_t cs, int64_t w, int64_t h, int slabs, const float2* __restrict__ part,
                const float* __restrict__ x, int use_pivot, int bessel, float eps, float decay,
                float* __restrict__ mean, float* __restrict__ var, float* __restrict__ rmean,
                float* __restrict__ rvar)
{
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kRowTileWaves + wave_index();
  if (c >= C) return;
  const float2 t = bn_rt_channel_total(part, h, slabs, cs, c);
  if ((threadIdx.x & (kWave - 1)) != 0) return;
  const int64_t n = cs * w;
  if (n <= 1) {  // batch_normalization.cpp:118-120: the mean holds x, the variance is 1
    mean[c] = x[c * cs];
    var[c] = 1.f;
    return;
  }
  const float K = use_pivot ? x[c * cs] : 0.f;
  float m, v;
  stats_from_sums(t.x, t.y, K, n, bessel, eps, m, v);
  mean[c] = m;
  var[c] = v;
  rmean[c] = decay * rmean[c] + (1.f - decay) * m;
  rvar[c] = decay * rvar[c] + (1.f - decay) * v;
}

__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_bwd_stats(int64_t C, int64_t cs, int64_t h, int slabs, const float2* __restrict__ part, float eps,
                int training, const float* __restrict__ var, const float* __restrict__ scale,
                float* __restrict__ dscale, float* __restrict__ dbias, float* __restrict__ dmean,
                float* __restrict__ dvar)
{
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kRowTileWaves + wave_index();
  if (c >= C) return;
  const float2 t = bn_rt_channel_total(part, h, slabs, cs, c);
  if ((threadIdx.x & (kWave - 1)) != 0) return;
  const float inv_stdev = 1.0f / sqrtf(var[c] + eps);
  float ds, db, dm, dv;
  grads_from_sums(t.x, t.y, scale[c], inv_stdev, ds, db, dm, dv);
  dscale[c] = ds;
  dbias[c] = db;
  dmean[c] = training ? dm : 0.f;  // statistics are constants outside training
  dvar[c] = training ? dv : 0.f;
}

// Forward: y = scale * ((x - mean) * inv_stdev) + bias.
// Backward: dx = dy * scale * inv_stdev + dmean / n + dvar * 2 / (n - bessel) * (x - mean).
template <int GW, bool BWD>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_apply(BnRtArgs a)
{
  using P = RowTilePos<GW>;
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  if (r0 >= a.h) return;
  const int64_t c0 = static_cast<int64_t>(blockIdx.y) * a.slab_width;
  const int64_t c1 = imin64(c0 + a.slab_width, a.w);
  float mean[4], k0[4], k1[4], k2[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t ch = (r0 + r) / a.cs;
    mean[r] = a.mean[ch];
    const float inv_stdev = 1.0f / sqrtf(a.var[ch] + a.eps);
    if (BWD) {
      k0[r] = a.scale[ch] * inv_stdev;
      k1[r] = a.dmean[ch] / a.count;
      k2[r] = a.dvar[ch] * 2.f / a.count_bessel;
    }
    else {
      k0[r] = inv_stdev;
      k1[r] = a.scale[ch];
      k2[r] = a.bias[ch];
    }
  }
  auto finish = [&](float (&v)[4], const float (&g)[4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (BWD) v[r] = a.zero ? 0.f : g[r] * k0[r] + k1[r] + k2[r] * (v[r] - mean[r]);
      else v[r] = k1[r] * ((v[r] - mean[r]) * k0[r]) + k2[r];
    }
  };
  int64_t c = c0 + p.g;
  for (; c + P::kGroups < c1; c += 2 * P::kGroups) {
    float v[2][4], g[2][4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Vec16<float>::load(a.x + r0 + (c + j * P::kGroups) * a.ldx, v[j]);
      if (BWD) Vec16<float>::load(a.dy + r0 + (c + j * P::kGroups) * a.lddy, g[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      finish(v[j], g[j]);
      Vec16<float>::store(a.out + r0 + (c + j * P::kGroups) * a.ldo, v[j]);
    }
  }
  for (; c < c1; c += P::kGroups) {
    float v[4], g[4];
    Vec16<float>::load(a.x + r0 + c * a.ldx, v);
    if (BWD) Vec16<float>::load(a.dy + r0 + c * a.lddy, g);
    finish(v, g);
    Vec16<float>::store(a.out + r0 + c * a.ldo, v);
  }
}

inline size_t bn_rt_workspace_bytes(int64_t h, int64_t w)
{
  const RowTilePlan p = row_tile_plan(h, w);
  return static_cast<size_t>(p.slabs) * static_cast<size_t>(h) * sizeof(float2);
}

}  // namespace lbn
