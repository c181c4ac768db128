// Layer-norm kernels for rows too long for the register-resident kernels (more than
// 16384 entries, e.g. layer norm over a whole image sample or instance norm over a large
// channel).  Math as in layer_norm.hip (layer_norm.cpp:41-136, :139-258).
//
//  * ln_fwd_long / ln_bwd_long: one 1024-thread workgroup per row, two passes over the
//    row with 16-byte accesses, four vectors per thread in flight.  The second pass
//    re-reads what the first one just streamed, so for rows that fit the caches (a
//    row is at most a few MiB) the tensor crosses HBM about once.  Statistics are
//    taken about the row's first entry (no E[x^2] - mean^2 cancellation); the
//    reference's formula (LBN_STATS_SUMSQ) is the same code with pivot 0.
//  * ln_wgrad_columns: weight gradients are sums over rows.  A thread owns one 16-byte
//    vector of feature positions and walks the rows of its slab (grid.y slabs, so that
//    short and wide problems still fill the device); the slabs' partial rows are added
//    by ln_wgrad_reduce in a fixed order.  VEC = false is the scalar variant for
//    unaligned shapes.
#pragma once

#include "device_utils.hpp"

namespace lbn {

constexpr int kLongThreads = 1024;
constexpr int kLongWaves = kLongThreads / kWave;
constexpr int kLongUnroll = 4;

template <typename T>
__global__ void __launch_bounds__(kLongThreads)
ln_fwd_long(const T* __restrict__ x, T* __restrict__ y, int64_t ldx, int64_t ldy, RowMap map,
            int64_t nvec, int tail, float inv_n, float eps, float* __restrict__ stats, int64_t ld_stats,
            const float* __restrict__ gamma, const float* __restrict__ beta, int sumsq)
{
  // tail: entries after the nvec whole vectors (rows of f32u data whose length is not a multiple
  // of 4), one per thread of the first `tail` threads; 0 for every other storage type.
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  __shared__ float red[2 * kLongWaves];
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const int64_t row = blockIdx.x;
  int64_t col, g;
  map.split(row, col, g);
  const T* xr = x + g * map.stride + col * ldx;
  T* yr = y + g * map.stride + col * ldy;
  const float K = sumsq ? 0.f : IO::load1(xr);

  float s = 0.f, q = 0.f;
  const bool has_tail = static_cast<int>(threadIdx.x) < tail;
  const int64_t tail_at = VE * nvec + threadIdx.x;
  float tv = 0.f;
  if (has_tail) {
    tv = IO::load1(xr + tail_at);
    const float d = tv - K;
    s = d;
    q = d * d;
  }
  int64_t j = threadIdx.x;
  for (; j + (kLongUnroll - 1) * kLongThreads < nvec; j += kLongUnroll * kLongThreads) {
    float v[kLongUnroll][VE];
#pragma unroll
    for (int u = 0; u < kLongUnroll; ++u) IO::load(xr + VE * (j + u * kLongThreads), v[u]);
#pragma unroll
    for (int u = 0; u < kLongUnroll; ++u)
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        const float d = v[u][k] - K;
        s += d;
        q = __builtin_fmaf(d, d, q);
      }
  }
  for (; j < nvec; j += kLongThreads) {
    float v[VE];
    IO::load(xr + VE * j, v);
#pragma unroll
    for (int k = 0; k < VE; ++k) {
      const float d = v[k] - K;
      s += d;
      q = __builtin_fmaf(d, d, q);
    }
  }
  team_sum2<kLongWaves>(s, q, red, wv, lane);
  float dm = s * inv_n;
  float var = fmaxf(__builtin_fmaf(-dm, dm, q * inv_n), 0.f);
  if (sumsq) {  // the reference's own expression: true divisions, no fused multiply-add
    const float nf = static_cast<float>(nvec * VE + tail);
    dm = s / nf;
    var = fmaxf(__fsub_rn(q / nf, __fmul_rn(dm, dm)), 0.f);
  }
  const float mean = K + dm;
  const float inv_stdev = 1.0f / sqrtf(var + eps);
  if (threadIdx.x == 0) {
    stats[g + col * ld_stats] = mean;
    stats[map.groups + g + col * ld_stats] = var;
  }

  auto apply = [&](int64_t jj, float (&v)[VE]) {
    float ga[VE], be[VE];
#pragma unroll
    for (int k4 = 0; k4 < VE; k4 += 4) {
      float w[4] = {1.f, 1.f, 1.f, 1.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
      if (gamma) load_weights4<T>(gamma + VE * jj + k4, w);
      if (beta) load_weights4<T>(beta + VE * jj + k4, b);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        ga[k4 + k] = w[k];
        be[k4 + k] = b[k];
      }
    }
#pragma unroll
    for (int k = 0; k < VE; ++k) v[k] = __builtin_fmaf((v[k] - mean) * inv_stdev, ga[k], be[k]);
    IO::store(yr + VE * jj, v);
  };
  if (has_tail)
    IO::store1(yr + tail_at, __builtin_fmaf((tv - mean) * inv_stdev, gamma ? gamma[tail_at] : 1.f,
                                            beta ? beta[tail_at] : 0.f));
  j = threadIdx.x;
  for (; j + (kLongUnroll - 1) * kLongThreads < nvec; j += kLongUnroll * kLongThreads) {
    float v[kLongUnroll][VE];
#pragma unroll
    for (int u = 0; u < kLongUnroll; ++u) IO::load(xr + VE * (j + u * kLongThreads), v[u]);
#pragma unroll
    for (int u = 0; u < kLongUnroll; ++u) apply(j + u * kLongThreads, v[u]);
  }
  for (; j < nvec; j += kLongThreads) {
    float v[VE];
    IO::load(xr + VE * j, v);
    apply(j, v);
  }
}

template <typename T>
__global__ void __launch_bounds__(kLongThreads)
ln_bwd_long(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ dx, int64_t ldx,
            int64_t lddy, int64_t lddx, RowMap map, int64_t nvec, int tail, float inv_n, float eps,
            const float* __restrict__ stats, int64_t ld_stats, float* __restrict__ sgrad,
            int64_t ld_sgrad, const float* __restrict__ gamma)
{
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  constexpr int U = kLongUnroll / 2;  // two tensors per step
  __shared__ float red[2 * kLongWaves];
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const int64_t row = blockIdx.x;
  int64_t col, g;
  map.split(row, col, g);
  const T* xr = x + g * map.stride + col * ldx;
  const T* gr = dy + g * map.stride + col * lddy;
  T* dr = dx + g * map.stride + col * lddx;
  const float mean = stats[g + col * ld_stats];
  const float inv_stdev = 1.0f / sqrtf(stats[map.groups + g + col * ld_stats] + eps);

  // on return v holds xh = (x - mean) / stdev and d holds dy * scale
  auto prepare = [&](int64_t jj, float (&v)[VE], float (&d)[VE]) {
#pragma unroll
    for (int k4 = 0; k4 < VE; k4 += 4) {
      float w[4] = {1.f, 1.f, 1.f, 1.f};
      if (gamma) load_weights4<T>(gamma + VE * jj + k4, w);
#pragma unroll
      for (int k = 0; k < 4; ++k) d[k4 + k] *= w[k];
    }
#pragma unroll
    for (int k = 0; k < VE; ++k) v[k] = (v[k] - mean) * inv_stdev;
  };

  float a = 0.f, b = 0.f;
  // (tail: as in ln_fwd_long) the thread's entry as xh and dy * scale
  const bool has_tail = static_cast<int>(threadIdx.x) < tail;
  const int64_t tail_at = VE * nvec + threadIdx.x;
  float tx = 0.f, td = 0.f;
  if (has_tail) {
    tx = (IO::load1(xr + tail_at) - mean) * inv_stdev;
    td = IO::load1(gr + tail_at) * (gamma ? gamma[tail_at] : 1.f);
    a = td;
    b = td * tx;
  }
  int64_t j = threadIdx.x;
  for (; j + (U - 1) * kLongThreads < nvec; j += U * kLongThreads) {
    float v[U][VE], d[U][VE];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      IO::load(xr + VE * (j + u * kLongThreads), v[u]);
      IO::load(gr + VE * (j + u * kLongThreads), d[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      prepare(j + u * kLongThreads, v[u], d[u]);
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        a += d[u][k];
        b = __builtin_fmaf(d[u][k], v[u][k], b);
      }
    }
  }
  for (; j < nvec; j += kLongThreads) {
    float v[VE], d[VE];
    IO::load(xr + VE * j, v);
    IO::load(gr + VE * j, d);
    prepare(j, v, d);
#pragma unroll
    for (int k = 0; k < VE; ++k) {
      a += d[k];
      b = __builtin_fmaf(d[k], v[k], b);
    }
  }
  team_sum2<kLongWaves>(a, b, red, wv, lane);
  const float dmean = -a * inv_stdev;
  const float dvar = -b * inv_stdev * inv_stdev * 0.5f;
  if (threadIdx.x == 0) {
    sgrad[g + col * ld_sgrad] = dmean;
    sgrad[map.groups + g + col * ld_sgrad] = dvar;
  }
  const float c0 = dmean * inv_n;
  const float c1 = -b * inv_stdev * inv_n;  // dvar * 2 / n per unit of xh

  if (has_tail) IO::store1(dr + tail_at, __builtin_fmaf(td, inv_stdev, __builtin_fmaf(c1, tx, c0)));
  j = threadIdx.x;
  for (; j + (U - 1) * kLongThreads < nvec; j += U * kLongThreads) {
    float v[U][VE], d[U][VE];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      IO::load(xr + VE * (j + u * kLongThreads), v[u]);
      IO::load(gr + VE * (j + u * kLongThreads), d[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      prepare(j + u * kLongThreads, v[u], d[u]);
#pragma unroll
      for (int k = 0; k < VE; ++k) d[u][k] = __builtin_fmaf(d[u][k], inv_stdev, __builtin_fmaf(c1, v[u][k], c0));
      IO::store(dr + VE * (j + u * kLongThreads), d[u]);
    }
  }
  for (; j < nvec; j += kLongThreads) {
    float v[VE], d[VE];
    IO::load(xr + VE * j, v);
    IO::load(gr + VE * j, d);
    prepare(j, v, d);
#pragma unroll
    for (int k = 0; k < VE; ++k) d[k] = __builtin_fmaf(d[k], inv_stdev, __builtin_fmaf(c1, v[k], c0));
    IO::store(dr + VE * j, d);
  }
}

// Partial weight gradients of row slab blockIdx.y: 2*n floats at wpart + blockIdx.y*2*n,
// the dscale row followed by the dbias row (the layout ln_wgrad_reduce adds up).
// units = n / VE (VEC) or n (scalar).
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
ln_wgrad_columns(const T* __restrict__ x, const T* __restrict__ dy, int64_t ldx, int64_t lddy,
                 RowMap map, int64_t rows, int64_t units, int64_t n, float eps,
                 const float* __restrict__ stats, int64_t ld_stats, float* __restrict__ wpart, int tail = 0)
{
  // tail (VEC only, f32u data): features after the `units` whole vectors; the thread after the
  // last vector takes them entry by entry.
  using IO = Vec16<T>;
  constexpr int VE = VEC ? IO::N : 1;
  const int64_t k = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t per = (rows + gridDim.y - 1) / gridDim.y;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * per;
  const int64_t r1 = imin64(r0 + per, rows);
  const bool partial = VEC && tail > 0 && k == units;
  const bool ok = k < units || partial;
  const int64_t off = ok ? VE * k : 0;
  const int mine = partial ? tail : VE;  // entries of this thread's access unit
  float dg[VE], db[VE];
#pragma unroll
  for (int e = 0; e < VE; ++e) dg[e] = db[e] = 0.f;
#pragma unroll 4
  for (int64_t r = r0; r < r1; ++r) {
    int64_t col, g;
    map.split(r, col, g);  // block-uniform
    const float mean = stats[g + col * ld_stats];
    const float inv_stdev = 1.0f / sqrtf(stats[map.groups + g + col * ld_stats] + eps);
    float v[VE], d[VE];
    if constexpr (VEC) {
      if (!partial) {
        IO::load(x + g * map.stride + col * ldx + off, v);
        IO::load(dy + g * map.stride + col * lddy + off, d);
      }
      else {
#pragma unroll
        for (int e = 0; e < VE; ++e) {
          v[e] = e < tail ? IO::load1(x + g * map.stride + col * ldx + off + e) : 0.f;
          d[e] = e < tail ? IO::load1(dy + g * map.stride + col * lddy + off + e) : 0.f;
        }
      }
    }
    else {
      v[0] = IO::load1(x + g * map.stride + col * ldx + off);
      d[0] = IO::load1(dy + g * map.stride + col * lddy + off);
    }
#pragma unroll
    for (int e = 0; e < VE; ++e) {
      db[e] += d[e];
      dg[e] = __builtin_fmaf(d[e], (v[e] - mean) * inv_stdev, dg[e]);
    }
  }
  if (!ok) return;
  float* out = wpart + static_cast<int64_t>(blockIdx.y) * 2 * n;
#pragma unroll
  for (int e = 0; e < VE; ++e) {
    if (e < mine) {
      out[off + e] = dg[e];
      out[n + off + e] = db[e];
    }
  }
}

// Scalar companion of ln_wgrad_reduce for n that is not a multiple of 4.  A workgroup takes
// 32 features of one of the two rows (blockIdx.y: dscale, dbias): thread (c, g) adds the partial
// rows g, g + 8, ... of feature c with eight loads in flight, and the eight groups are added
// through LDS in a fixed order.  (One thread per feature walking all P rows by itself left a
// 1001-feature problem with four workgroups: 107 us for 256 partial rows.)
constexpr int kWgradScalarCols = 32;
__global__ void __launch_bounds__(256)
ln_wgrad_reduce_scalar(const float* __restrict__ part, int64_t P, int64_t n, float* __restrict__ dscale,
                       float* __restrict__ dbias)
{
  constexpr int C = kWgradScalarCols, G = 256 / C, U = 8;
  __shared__ float sm[G][C + 1];
  float* out = blockIdx.y == 0 ? dscale : dbias;
  if (!out) return;
  const int c = threadIdx.x % C, g = threadIdx.x / C;
  const int64_t k = static_cast<int64_t>(blockIdx.x) * C + c;
  float acc = 0.f;
  if (k < n) {
    const float* src = part + blockIdx.y * n + k;
    for (int64_t p0 = g; p0 < P; p0 += static_cast<int64_t>(G) * U) {
      float w[U];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const int64_t q = p0 + static_cast<int64_t>(G) * j;
        w[j] = q < P ? src[q * 2 * n] : 0.f;
      }
      acc += ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7]));
    }
  }
  sm[g][c] = acc;
  __syncthreads();
  if (threadIdx.x < C) {
    const int64_t kc = static_cast<int64_t>(blockIdx.x) * C + threadIdx.x;
    if (kc < n) {
      const int t = threadIdx.x;
      out[kc] = ((sm[0][t] + sm[1][t]) + (sm[2][t] + sm[3][t])) + ((sm[4][t] + sm[5][t]) + (sm[6][t] + sm[7][t]));
    }
  }
}

}  // namespace lbn
