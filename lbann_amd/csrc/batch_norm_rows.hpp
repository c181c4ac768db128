// Batch norm for channels that are not a whole number of 16-byte vectors (channel_size
// 1 after a fully-connected layer, 49 for 7 x 7 feature maps, ...), fp32 or fp16 storage.  The kernels of
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

// S: storage type with four entries per access (float: 16 bytes; f16x4: 8 bytes of fp16).
template <typename S>
struct BnRtArgs {
  int64_t h, w, cs;
  const S* x;
  const S* dy;
  S* out;  // y or dx
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
template <typename S, int GW, bool BWD>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_sums(BnRtArgs<S> a)
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
    K[r] = BWD ? a.mean[ch] : (a.use_pivot ? Vec16<S>::load1(a.x + ch * a.cs) : 0.f);
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
      Vec16<S>::load(a.x + rr + (c + j * P::kGroups) * a.ldx, v[j]);
      if (BWD) Vec16<S>::load(a.dy + rr + (c + j * P::kGroups) * a.lddy, g[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) add(v[j], g[j]);
  }
  for (; c < c1; c += P::kGroups) {
    float v[4], g[4];
    Vec16<S>::load(a.x + rr + c * a.ldx, v);
    if (BWD) Vec16<S>::load(a.dy + rr + c * a.lddy, g);
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
  double a = 0., b = 0.;  // a lane adds up to slabs x cs / 64 partials in sequence
  for (int s = 0; s < slabs; ++s) {
    const float2* row = part + static_cast<int64_t>(s) * h + c * cs;
    for (int64_t i = lane; i < cs; i += kWave) {
      const float2 v = row[i];
      a += static_cast<double>(v.x);
      b += static_cast<double>(v.y);
    }
  }
  return make_float2(wave_sum(static_cast<float>(a)), wave_sum(static_cast<float>(b)));
}

// The same by a whole workgroup, for channels of many rows (a 111 x 111 map: 12321 rows, which
// one wave walked for 58 us): thread-strided with four independent loads in flight, waves added
// through LDS in order.  Thread 0 gets the totals.
constexpr int64_t kBnRtWideChannel = 256;  // rows x slabs from which a channel takes a workgroup

__device__ __forceinline__ float2 bn_rt_channel_total_wide(const float2* part, int64_t h, int slabs, int64_t cs,
                                                           int64_t c)
{
  __shared__ float2 red[kRowTileWaves];
  constexpr int U = 4;
  double a[U] = {0., 0., 0., 0.}, b[U] = {0., 0., 0., 0.};
  for (int s = 0; s < slabs; ++s) {
    const float2* row = part + static_cast<int64_t>(s) * h + c * cs;
    for (int64_t i0 = threadIdx.x; i0 < cs; i0 += U * kRowTileThreads) {
      float2 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = i0 + u * kRowTileThreads;
        v[u] = i < cs ? row[i] : make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        a[u] += static_cast<double>(v[u].x);
        b[u] += static_cast<double>(v[u].y);
      }
    }
  }
  const float ta = wave_sum(static_cast<float>((a[0] + a[1]) + (a[2] + a[3])));
  const float tb = wave_sum(static_cast<float>((b[0] + b[1]) + (b[2] + b[3])));
  if ((threadIdx.x & (kWave - 1)) == 0) red[wave_index()] = make_float2(ta, tb);
  __syncthreads();
  float2 t = red[0];
#pragma unroll
  for (int k = 1; k < kRowTileWaves; ++k) {
    t.x += red[k].x;
    t.y += red[k].y;
  }
  return t;
}

// Channels of a few rows (batch norm behind a fully connected layer: 16384 channels of one row):
// one thread per channel adds its rows x slabs partials, instead of a wave per channel with one
// busy lane (16384 channels x 512 columns: 8 us of a 29 us forward pass that way).
constexpr int64_t kBnRtThinChannel = 8;  // rows x slabs up to which a channel takes one thread

__device__ __forceinline__ float2 bn_rt_channel_total_thin(const float2* part, int64_t h, int slabs, int64_t cs,
                                                           int64_t c)
{
  double a = 0., b = 0.;
  for (int s = 0; s < slabs; ++s) {
    const float2* row = part + static_cast<int64_t>(s) * h + c * cs;
    for (int64_t i = 0; i < cs; ++i) {
      a += static_cast<double>(row[i].x);
      b += static_cast<double>(row[i].y);
    }
  }
  return make_float2(static_cast<float>(a), static_cast<float>(b));
}

// How a channel's partials are added up: by one wave (4 channels per workgroup), by a whole
// workgroup, or by one thread (256 channels per workgroup).
constexpr int kBnRtWave = 0, kBnRtWide = 1, kBnRtThin = 2;

inline int bn_rt_stats_mode(int64_t cs, int slabs)
{
  const int64_t parts = cs * slabs;
  return parts >= kBnRtWideChannel ? kBnRtWide : parts <= kBnRtThinChannel ? kBnRtThin : kBnRtWave;
}

inline unsigned bn_rt_stats_grid(int mode, int64_t C)
{
  const int64_t per = mode == kBnRtWide ? 1 : mode == kBnRtThin ? kRowTileThreads : kRowTileWaves;
  return static_cast<unsigned>((C + per - 1) / per);
}

template <int MODE>
__device__ __forceinline__ bool bn_rt_stats_channel(int64_t C, int64_t& c)
{
  c = MODE == kBnRtWide   ? static_cast<int64_t>(blockIdx.x)
      : MODE == kBnRtThin ? static_cast<int64_t>(blockIdx.x) * kRowTileThreads + threadIdx.x
                          : static_cast<int64_t>(blockIdx.x) * kRowTileWaves + wave_index();
  return c < C;
}

// The thread that holds a channel's totals and writes its results.
template <int MODE>
__device__ __forceinline__ bool bn_rt_stats_writer()
{
  return MODE == kBnRtWide ? threadIdx.x == 0 : MODE == kBnRtThin ? true : (threadIdx.x & (kWave - 1)) == 0;
}

template <int MODE>
__device__ __forceinline__ float2 bn_rt_stats_total(const float2* part, int64_t h, int slabs, int64_t cs, int64_t c)
{
  if constexpr (MODE == kBnRtWide) return bn_rt_channel_total_wide(part, h, slabs, cs, c);
  else if constexpr (MODE == kBnRtThin) return bn_rt_channel_total_thin(part, h, slabs, cs, c);
  else return bn_rt_channel_total(part, h, slabs, cs, c);
}

template <typename S, int MODE>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_fwd_stats(int64_t C, int64_t cs, int64_t w, int64_t h, int slabs, const float2* __restrict__ part,
                const S* __restrict__ x, int use_pivot, int bessel, float eps, float decay,
                float* __restrict__ mean, float* __restrict__ var, float* __restrict__ rmean,
                float* __restrict__ rvar)
{
  int64_t c;
  if (!bn_rt_stats_channel<MODE>(C, c)) return;  // (whole workgroups or waves in the modes that use barriers or wave sums)
  const float2 t = bn_rt_stats_total<MODE>(part, h, slabs, cs, c);
  if (!bn_rt_stats_writer<MODE>()) return;
  const int64_t n = cs * w;
  if (n <= 1) {  // batch_normalization.cpp:118-120: the mean holds x, the variance is 1
    mean[c] = Vec16<S>::load1(x + c * cs);
    var[c] = 1.f;
    return;
  }
  const float K = use_pivot ? Vec16<S>::load1(x + c * cs) : 0.f;
  float m, v;
  stats_from_sums(t.x, t.y, K, n, bessel, eps, m, v);
  mean[c] = m;
  var[c] = v;
  rmean[c] = decay * rmean[c] + (1.f - decay) * m;
  rvar[c] = decay * rvar[c] + (1.f - decay) * v;
}

template <int MODE>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_bwd_stats(int64_t C, int64_t cs, int64_t h, int slabs, const float2* __restrict__ part, float eps,
                int training, const float* __restrict__ var, const float* __restrict__ scale,
                float* __restrict__ dscale, float* __restrict__ dbias, float* __restrict__ dmean,
                float* __restrict__ dvar)
{
  int64_t c;
  if (!bn_rt_stats_channel<MODE>(C, c)) return;  // (whole workgroups or waves in the modes that use barriers or wave sums)
  const float2 t = bn_rt_stats_total<MODE>(part, h, slabs, cs, c);
  if (!bn_rt_stats_writer<MODE>()) return;
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
template <typename S, int GW, bool BWD>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_apply(BnRtArgs<S> a)
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
      Vec16<S>::load(a.x + r0 + (c + j * P::kGroups) * a.ldx, v[j]);
      if (BWD) Vec16<S>::load(a.dy + r0 + (c + j * P::kGroups) * a.lddy, g[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      finish(v[j], g[j]);
      Vec16<S>::store(a.out + r0 + (c + j * P::kGroups) * a.ldo, v[j]);
    }
  }
  for (; c < c1; c += P::kGroups) {
    float v[4], g[4];
    Vec16<S>::load(a.x + r0 + c * a.ldx, v);
    if (BWD) Vec16<S>::load(a.dy + r0 + c * a.lddy, g);
    finish(v, g);
    Vec16<S>::store(a.out + r0 + c * a.ldo, v);
  }
}


// ---- register-resident variant for mini-batches of at most 256 columns ------------------
// A workgroup keeps (rows x all columns) in registers (the entry-wise batch norm tiling:
// 256 rows x <= 64 columns with GW = 1, 64 rows x <= 256 columns with GW = 4) and owns
// whole channels: it takes `rows_eff` rows, the largest multiple of lcm(cs, 4) that fits.
// Per-row pairs are merged over the column groups in LDS, one thread per channel adds its
// cs rows and finishes the channel, and the output is written from registers: one kernel,
// x (and dy) read once.
template <typename S>
struct BnRtTileArgs {
  int64_t h, w, cs, n;  // n = cs * w
  int rows_eff;         // rows per workgroup: a multiple of cs and of 4
  const S* x;
  const S* dy;
  S* out;
  int64_t ldx, lddy, ldo;
  int use_pivot, bessel, training;
  float eps, decay;
  float* mean;    // forward: written; backward: read
  float* var;
  const float* scale;
  const float* bias;
  float* rmean;
  float* rvar;
  float* dscale;
  float* dbias;
  float* dmean;
  float* dvar;
};

// Shared front end: merges the per-row pairs (a, b) of the column groups and returns, in
// chan[c][0..1], the totals of local channel c (c < nch) of this workgroup.
template <int GW>
__device__ __forceinline__ void bn_rt_tile_channel_totals(float (&a)[4], float (&b)[4],
                                                          float (*lds)[RowTilePos<GW>::kRows][2],
                                                          float (*chan)[4], const RowTilePos<GW>& p, int cs,
                                                          int nch)
{
  using P = RowTilePos<GW>;
  if (GW == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      a[r] += __shfl_xor(a[r], 16);
      b[r] += __shfl_xor(b[r], 16);
      a[r] += __shfl_xor(a[r], 32);
      b[r] += __shfl_xor(b[r], 32);
    }
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  if (lane < P::kQuads) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      lds[wave][4 * p.q + r][0] = a[r];
      lds[wave][4 * p.q + r][1] = b[r];
    }
  }
  __syncthreads();
  const int c = threadIdx.x;
  if (c < nch) {
    // one thread adds cs x waves partials in sequence: in double, so that sums about a pivot
    // far from the mean (large partials, small total) lose nothing here
    double sa = 0., sb = 0.;
    for (int i = c * cs; i < (c + 1) * cs; ++i) {
#pragma unroll
      for (int k = 0; k < kRowTileWaves; ++k) {
        sa += static_cast<double>(lds[k][i][0]);
        sb += static_cast<double>(lds[k][i][1]);
      }
    }
    chan[c][0] = static_cast<float>(sa);
    chan[c][1] = static_cast<float>(sb);
  }
  __syncthreads();
}

template <typename S, int CPT, int GW>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_fwd_tile(BnRtTileArgs<S> a)
{
  using P = RowTilePos<GW>;
  __shared__ float lds[kRowTileWaves][P::kRows][2];
  __shared__ float chan[P::kRows][4];
  const P p;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * a.rows_eff;
  const int local = 4 * p.q;
  const int64_t rows_here = imin64(a.rows_eff, a.h - base);  // a multiple of cs and of 4
  const bool row_ok = local < rows_here;
  const int64_t r0 = base + (row_ok ? local : 0);
  const int cs = static_cast<int>(a.cs);
  const int nch = static_cast<int>(rows_here / cs);

  float K[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) K[r] = a.use_pivot ? Vec16<S>::load1(a.x + ((r0 + r) / cs) * cs) : 0.f;
  float v[CPT][4];
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (row_ok && c < a.w) {
      Vec16<S>::load(a.x + r0 + c * a.ldx, v[j]);
    }
    else {
#pragma unroll
      for (int r = 0; r < 4; ++r) v[j][r] = K[r];
    }
  }
  float s[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < CPT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float d = v[j][r] - K[r];
      s[r] += d;
      sq[r] = __builtin_fmaf(d, d, sq[r]);
    }
  bn_rt_tile_channel_totals<GW>(s, sq, lds, chan, p, cs, nch);
  // one thread per channel finishes it and leaves (mean, 1/stdev) for the rows
  if (static_cast<int>(threadIdx.x) < nch) {
    const int64_t ch = base / cs + threadIdx.x;
    float m, var;
    if (a.n <= 1) {  // batch_normalization.cpp:118-120
      m = Vec16<S>::load1(a.x + ch * cs);
      var = 1.f;
    }
    else {
      const float Kc = a.use_pivot ? Vec16<S>::load1(a.x + ch * cs) : 0.f;
      stats_from_sums(chan[threadIdx.x][0], chan[threadIdx.x][1], Kc, a.n, a.bessel, a.eps, m, var);
      a.rmean[ch] = a.decay * a.rmean[ch] + (1.f - a.decay) * m;
      a.rvar[ch] = a.decay * a.rvar[ch] + (1.f - a.decay) * var;
    }
    a.mean[ch] = m;
    a.var[ch] = var;
    chan[threadIdx.x][2] = m;
    chan[threadIdx.x][3] = 1.0f / sqrtf(var + a.eps);
  }
  __syncthreads();
  if (!row_ok) return;
  float mean[4], inv[4], sc[4], bi[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int lc = (local + r) / cs;
    mean[r] = chan[lc][2];
    inv[r] = chan[lc][3];
    sc[r] = a.scale[base / cs + lc];
    bi[r] = a.bias[base / cs + lc];
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (c < a.w) {
#pragma unroll
      for (int r = 0; r < 4; ++r) v[j][r] = sc[r] * ((v[j][r] - mean[r]) * inv[r]) + bi[r];
      Vec16<S>::store(a.out + r0 + c * a.ldo, v[j]);
    }
  }
}

template <typename S, int CPT, int GW>
__global__ void __launch_bounds__(kRowTileThreads)
bn_rt_bwd_tile(BnRtTileArgs<S> a)
{
  using P = RowTilePos<GW>;
  __shared__ float lds[kRowTileWaves][P::kRows][2];
  __shared__ float chan[P::kRows][4];
  const P p;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * a.rows_eff;
  const int local = 4 * p.q;
  const int64_t rows_here = imin64(a.rows_eff, a.h - base);
  const bool row_ok = local < rows_here;
  const int64_t r0 = base + (row_ok ? local : 0);
  const int cs = static_cast<int>(a.cs);
  const int nch = static_cast<int>(rows_here / cs);

  float mean[4], k0[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t ch = (r0 + r) / cs;
    mean[r] = a.mean[ch];
    k0[r] = a.scale[ch] * (1.0f / sqrtf(a.var[ch] + a.eps));
  }
  float xc[CPT][4], g[CPT][4];
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (row_ok && c < a.w) {
      Vec16<S>::load(a.x + r0 + c * a.ldx, xc[j]);
      Vec16<S>::load(a.dy + r0 + c * a.lddy, g[j]);
#pragma unroll
      for (int r = 0; r < 4; ++r) xc[j][r] -= mean[r];
    }
    else {
#pragma unroll
      for (int r = 0; r < 4; ++r) xc[j][r] = g[j][r] = 0.f;
    }
  }
  float sa[4] = {0.f, 0.f, 0.f, 0.f}, sb[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < CPT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      sa[r] += g[j][r];
      sb[r] = __builtin_fmaf(g[j][r], xc[j][r], sb[r]);
    }
  bn_rt_tile_channel_totals<GW>(sa, sb, lds, chan, p, cs, nch);
  if (static_cast<int>(threadIdx.x) < nch) {
    const int64_t ch = base / cs + threadIdx.x;
    const float inv_stdev = 1.0f / sqrtf(a.var[ch] + a.eps);
    float ds, db, dm, dv;
    grads_from_sums(chan[threadIdx.x][0], chan[threadIdx.x][1], a.scale[ch], inv_stdev, ds, db, dm, dv);
    if (!a.training) dm = dv = 0.f;  // statistics are constants outside training
    a.dscale[ch] = ds;
    a.dbias[ch] = db;
    a.dmean[ch] = dm;
    a.dvar[ch] = dv;
    chan[threadIdx.x][2] = dm / static_cast<float>(a.n);
    chan[threadIdx.x][3] = dv * 2.f / static_cast<float>(a.n - (a.bessel ? 1 : 0));
  }
  __syncthreads();
  if (!row_ok) return;
  float k1[4], k2[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int lc = (local + r) / cs;
    k1[r] = chan[lc][2];
    k2[r] = chan[lc][3];
  }
  const bool zero = a.n <= 1;
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (c < a.w) {
#pragma unroll
      for (int r = 0; r < 4; ++r) g[j][r] = zero ? 0.f : g[j][r] * k0[r] + k1[r] + k2[r] * xc[j][r];
      Vec16<S>::store(a.out + r0 + c * a.ldo, g[j]);
    }
  }
}

// Rows a workgroup of the register-resident variant takes: the largest multiple of
// lcm(cs, 4) within `rows` (0: channels too long for a workgroup).
inline int bn_rt_tile_rows(int64_t cs, int rows)
{
  int64_t l = cs;
  while (l % 4 != 0) l += cs;  // lcm(cs, 4)
  if (l > rows) return 0;
  return static_cast<int>((rows / l) * l);
}

inline size_t bn_rt_workspace_bytes(int64_t h, int64_t w)
{
  // (the query does not know the storage type: the larger of the two plans)
  const int a = row_tile_plan(h, w, 4).slabs, b = row_tile_plan(h, w, 2).slabs;
  return static_cast<size_t>(a > b ? a : b) * static_cast<size_t>(h) * sizeof(float2);
}

}  // namespace lbn
