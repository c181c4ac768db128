// Layer norm over rows too long for one workgroup's registers (a whole image sample:
// the layer's default is to normalise over every entry of a sample), when there are
// too few rows to fill the device with one workgroup per row.  Math as in
// layer_norm.hip (layer_norm.cpp:41-136, :139-258).
//
// A cluster of M workgroups of 1024 threads shares a row (cluster_sync.hpp): workgroup k
// keeps vectors [k*1024*V, (k+1)*1024*V) in registers, the cluster exchanges one pair of
// partial sums per row and every workgroup finishes its share from registers, so x (and
// dy) cross HBM once.  The grid is persistent (cluster cl takes rows cl, cl + nclusters,
// ...) and rotates three register tiles like the batch-norm and softmax cluster kernels:
// in a step a workgroup reduces the tile loaded a step earlier and publishes its sums,
// issues the loads of the tile after that, then collects the sums of the oldest tile and
// writes its output.
//
// A workgroup always owns the same feature positions, so it copies its slice of scale and
// bias into LDS once (thread-private cells) instead of fetching 8 bytes of weights per
// entry and row from the caches.
//
// Backward with weight gradients: for the same reason
// it accumulates its slice of dscale / dbias over all its rows in LDS (thread-private
// cells again, no synchronisation) and writes one partial row per cluster at the end;
// ln_wgrad_reduce adds the clusters' rows in a fixed order.
#pragma once

#include <type_traits>

#include "cluster_sync.hpp"
#include "device_utils.hpp"

namespace lbn {

constexpr int kLnClThreads = 1024;
constexpr int kLnClWaves = kLnClThreads / kWave;
constexpr int kLnClMaxM = kClusterMaxSumM;  // a wave polls two slots per lane
constexpr int kLnClFwdUnits = 16384;  // entries per workgroup in forward: 2 x 64 KiB of LDS for scale and bias
constexpr int kLnClBwdUnits = 8192;   // in backward: 2 x 32 KiB of LDS accumulators and 32 KiB for the scale

template <typename T>
struct LnClArgs {
  const T* x;
  const T* dy;  // backward only
  T* out;       // forward: y; backward: dx
  int64_t ldx, lddy, ldo;
  RowMap map;
  int64_t rows;
  int64_t n;
  unsigned nvec;
  unsigned per_wg;  // vectors per workgroup: workgroup k owns [k * per_wg, (k + 1) * per_wg) of a row
  int M, sumsq;
  float inv_n, eps;
  float* stats;  // forward: written; backward: read
  int64_t ld_stats;
  float* sgrad;  // backward: written
  int64_t ld_sgrad;
  const float* gamma;
  const float* beta;
  float* wpart;  // backward with weight gradients: one row of 2n floats per cluster
  ClusterWorkspace cw;
  ClusterTag tag;
  __device__ __forceinline__ unsigned long long* slots(int64_t row) const { return cw.slots + row * M * 2; }
};

// cluster_collect_sums() restated with the two slots written out: these kernels sit at the
// 128-register limit of 1024-thread workgroups, and this form leaves the register allocator
// two registers more than the shared template does (7 % of the backward time on 64 rows of
// 802816 entries).
__device__ __forceinline__ void ln_cl_collect(unsigned long long* slots, int M, ClusterTag tag, int* error_word,
                                              float& ta, float& tb)
{
  const int lane = threadIdx.x & 63;
  unsigned long long w[2][2] = {{0, 0}, {0, 0}};
  bool have[2] = {false, false};
  int polls = 0;
  for (;;) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int j = lane + 64 * h;
      if (j < M && !have[h]) {
        w[h][0] = __hip_atomic_load(slots + 2 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        w[h][1] = __hip_atomic_load(slots + 2 * j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        have[h] = static_cast<unsigned>(w[h][0] >> 32) == tag.lo && static_cast<unsigned>(w[h][1] >> 32) == tag.hi;
      }
    }
    if (__all((have[0] || lane >= M) && (have[1] || lane + 64 >= M))) break;
    if (++polls > kClusterMaxPolls) {
      if (lane == 0) __hip_atomic_store(error_word, kClusterTimedOut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  float a = 0.f, b = 0.f;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (have[h]) {
      a += __uint_as_float(static_cast<unsigned>(w[h][0]));
      b += __uint_as_float(static_cast<unsigned>(w[h][1]));
    }
  }
  ta = wave_sum(a);
  tb = wave_sum(b);
}

// Copies this thread's V vectors of a weight array (or `fill` when there is none) into its
// LDS cells: cell i of thread t is cells[(i * 1024 + t) * VE ...].
template <typename T, int V>
__device__ __forceinline__ void ln_cl_stage_weights(const float* w, float fill, unsigned base, unsigned nvec,
                                                    float* cells)
{
  constexpr int VE = Vec16<T>::N;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kLnClThreads;
    float v[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) v[e] = fill;
    if (w && idx < nvec) load_f32_run<VE>(w + VE * static_cast<int64_t>(idx), v);
    float* cell = cells + (i * kLnClThreads + threadIdx.x) * VE;
#pragma unroll
    for (int e = 0; e < VE; ++e) cell[e] = v[e];
  }
}

// ------------------------------------------------------------------------ forward
template <typename T, int V>
struct LnClFwdTile {
  typename Vec16<T>::raw_t v[V];
  float K;  // pivot of the sums: the row's first entry, or 0 for the reference's formula
};

template <typename T, int V>
__device__ __forceinline__ void ln_cl_fwd_load(LnClFwdTile<T, V>& t, const LnClArgs<T>& a, int64_t row, unsigned base)
{
  using IO = Vec16<T>;
  const T* xr = a.x + a.map.offset(row, a.ldx);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kLnClThreads;
    t.v[i] = typename IO::raw_t{};
    if (idx < a.nvec) t.v[i] = IO::load_raw(xr + IO::N * static_cast<int64_t>(idx));
  }
  t.K = a.sumsq ? 0.f : IO::load1(xr);
}

template <typename T, int V>
__device__ __forceinline__ void ln_cl_fwd_reduce(const LnClArgs<T>& a, int64_t row, int k, unsigned base,
                                                 const LnClFwdTile<T, V>& t, float* red)
{
  using IO = Vec16<T>;
  float s = 0.f, q = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (base + i * kLnClThreads < a.nvec) {
      float v[IO::N];
      IO::unpack(t.v[i], v);
#pragma unroll
      for (int e = 0; e < IO::N; ++e) {
        const float d = v[e] - t.K;
        s += d;
        q = __builtin_fmaf(d, d, q);
      }
    }
  }
  team_sum2<kLnClWaves>(s, q, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) cluster_publish(s, q, a.slots(row), k, a.tag);
}

template <typename T, int V, bool AFFINE>
__device__ __forceinline__ void ln_cl_fwd_finish(const LnClArgs<T>& a, int64_t row, int k, unsigned base,
                                                 const LnClFwdTile<T, V>& t, float* bc, const float* wts)
{
  using IO = Vec16<T>;
  if (threadIdx.x < kWave) {
    float ts, tq;
    ln_cl_collect(a.slots(row), a.M, a.tag, a.cw.error, ts, tq);
    if (threadIdx.x == 0) {
      float dm = ts * a.inv_n;
      float var = fmaxf(__builtin_fmaf(-dm, dm, tq * a.inv_n), 0.f);
      if (a.sumsq) {  // the reference's own expression (layer_norm.cpp:99-112): true divisions, no fused multiply-add
        const float nf = static_cast<float>(a.n);
        dm = ts / nf;
        var = fmaxf(__fsub_rn(tq / nf, __fmul_rn(dm, dm)), 0.f);
      }
      const float mean = t.K + dm;
      bc[0] = mean;
      bc[1] = 1.0f / sqrtf(var + a.eps);
      if (k == 0) {
        int64_t col, g;
        a.map.split(row, col, g);
        a.stats[g + col * a.ld_stats] = mean;
        a.stats[a.map.groups + g + col * a.ld_stats] = var;
      }
    }
  }
  __syncthreads();
  const float mean = bc[0];
  const float inv_stdev = bc[1];
  T* yr = a.out + a.map.offset(row, a.ldo);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kLnClThreads;
    if (idx < a.nvec) {
      float v[IO::N];
      IO::unpack(t.v[i], v);
      if (AFFINE) {
        const float* ga = wts + (i * kLnClThreads + threadIdx.x) * IO::N;
        const float* be = ga + kLnClThreads * V * IO::N;
#pragma unroll
        for (int e = 0; e < IO::N; ++e) v[e] = __builtin_fmaf((v[e] - mean) * inv_stdev, ga[e], be[e]);
      }
      else {
#pragma unroll
        for (int e = 0; e < IO::N; ++e) v[e] = (v[e] - mean) * inv_stdev;
      }
      IO::store(yr + IO::N * static_cast<int64_t>(idx), v);
    }
  }
}

template <typename T, int V, bool AFFINE>
__device__ __forceinline__ void ln_cl_fwd_step(const LnClArgs<T>& a, int64_t row, int64_t nc, int k, unsigned base,
                                               LnClFwdTile<T, V>& F, LnClFwdTile<T, V>& R, LnClFwdTile<T, V>& L,
                                               float* red, float* bc, const float* wts)
{
  if (row + nc < a.rows) ln_cl_fwd_reduce<T, V>(a, row + nc, k, base, R, red);
  if (row + 2 * nc < a.rows) ln_cl_fwd_load<T, V>(L, a, row + 2 * nc, base);
  asm volatile("" ::: "memory");  // keep the loads above the wait below
  ln_cl_fwd_finish<T, V, AFFINE>(a, row, k, base, F, bc, wts);
}

template <typename T, int V, bool AFFINE>
__global__ void __launch_bounds__(kLnClThreads)
ln_fwd_cluster(LnClArgs<T> a)
{
  static_assert(kLnClThreads * V * Vec16<T>::N <= kLnClFwdUnits, "a workgroup's share of scale and bias must fit LDS");
  __shared__ float red[2 * kLnClWaves];
  __shared__ float bc[3][2];
  __shared__ float wts[AFFINE ? 2 * kLnClThreads * V * Vec16<T>::N : 1];  // scale cells, then bias cells
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  const unsigned base = static_cast<unsigned>(k) * a.per_wg + threadIdx.x;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  {  // from here on `nvec` is the end of this workgroup's share
    const unsigned end = (static_cast<unsigned>(k) + 1) * a.per_wg;
    if (end < a.nvec) a.nvec = end;
  }
  if (AFFINE) {  // read back by the same thread only: no barrier needed
    ln_cl_stage_weights<T, V>(a.gamma, 1.f, base, a.nvec, wts);
    ln_cl_stage_weights<T, V>(a.beta, 0.f, base, a.nvec, wts + kLnClThreads * V * Vec16<T>::N);
  }
  LnClFwdTile<T, V> t0, t1, t2;
  ln_cl_fwd_load<T, V>(t0, a, cl, base);
  if (cl + nc < a.rows) ln_cl_fwd_load<T, V>(t1, a, cl + nc, base);
  ln_cl_fwd_reduce<T, V>(a, cl, k, base, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  // one broadcast pair per position of the rotation: a step without a reduction has no
  // barrier between the reads of one finish and the write of the next
  for (int64_t row = cl; row < a.rows; row += 3 * nc) {
    ln_cl_fwd_step<T, V, AFFINE>(a, row, nc, k, base, t0, t1, t2, red, bc[0], wts);
    if (row + nc < a.rows) ln_cl_fwd_step<T, V, AFFINE>(a, row + nc, nc, k, base, t1, t2, t0, red, bc[1], wts);
    if (row + 2 * nc < a.rows) ln_cl_fwd_step<T, V, AFFINE>(a, row + 2 * nc, nc, k, base, t2, t0, t1, red, bc[2], wts);
  }
}

// ----------------------------------------------------------------------- backward
template <typename T, int V>
struct LnClBwdTile {
  typename Vec16<T>::raw_t x[V];
  typename Vec16<T>::raw_t g[V];
  float mean, inv_stdev;
};

template <typename T, int V>
__device__ __forceinline__ void ln_cl_bwd_load(LnClBwdTile<T, V>& t, const LnClArgs<T>& a, int64_t row, unsigned base)
{
  using IO = Vec16<T>;
  int64_t col, g;
  a.map.split(row, col, g);
  const T* xr = a.x + g * a.map.stride + col * a.ldx;
  const T* gr = a.dy + g * a.map.stride + col * a.lddy;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kLnClThreads;
    t.x[i] = typename IO::raw_t{};
    t.g[i] = typename IO::raw_t{};
    if (idx < a.nvec) {
      t.x[i] = IO::load_raw(xr + IO::N * static_cast<int64_t>(idx));
      t.g[i] = IO::load_raw(gr + IO::N * static_cast<int64_t>(idx));
    }
  }
  t.mean = a.stats[g + col * a.ld_stats];
  t.inv_stdev = 1.0f / sqrtf(a.stats[a.map.groups + g + col * a.ld_stats] + a.eps);
}

// A = sum(dy * scale), B = sum(dy * scale * xh) with xh = (x - mean) / stdev.
template <typename T, int V>
__device__ __forceinline__ void ln_cl_bwd_reduce(const LnClArgs<T>& a, int64_t row, int k, unsigned base,
                                                 const LnClBwdTile<T, V>& t, float* red, const float* scale_cells)
{
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kLnClThreads;
    if (idx < a.nvec) {
      float x[VE], g[VE];
      IO::unpack(t.x[i], x);
      IO::unpack(t.g[i], g);
      const float* ga = scale_cells + (i * kLnClThreads + threadIdx.x) * VE;
#pragma unroll
      for (int e = 0; e < VE; ++e) {
        const float xh = (x[e] - t.mean) * t.inv_stdev;
        const float gs = g[e] * ga[e];
        sa += gs;
        sb = __builtin_fmaf(gs, xh, sb);
      }
    }
  }
  team_sum2<kLnClWaves>(sa, sb, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) cluster_publish(sa, sb, a.slots(row), k, a.tag);
}

// dx from the cluster's sums; the weight gradients dscale += dy * xh, dbias += dy go to this
// thread's cells of `acc` here, after the rendezvous, where nobody waits for them.
template <typename T, int V, bool WGRAD>
__device__ __forceinline__ void ln_cl_bwd_finish(const LnClArgs<T>& a, int64_t row, int k, unsigned base,
                                                 const LnClBwdTile<T, V>& t, float* bc, const float* scale_cells,
                                                 float* acc)
{
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  const float inv_stdev = t.inv_stdev;
  int64_t col, g;
  a.map.split(row, col, g);
  if (threadIdx.x < kWave) {
    float ta, tb;
    ln_cl_collect(a.slots(row), a.M, a.tag, a.cw.error, ta, tb);
    if (threadIdx.x == 0) {
      const float dmean = -ta * inv_stdev;
      const float dvar = -tb * inv_stdev * inv_stdev * 0.5f;
      bc[0] = dmean * a.inv_n;
      bc[1] = -tb * inv_stdev * a.inv_n;  // dvar * 2 / n per unit of xh
      if (k == 0) {
        a.sgrad[g + col * a.ld_sgrad] = dmean;
        a.sgrad[a.map.groups + g + col * a.ld_sgrad] = dvar;
      }
    }
  }
  __syncthreads();
  const float c0 = bc[0];
  const float c1 = bc[1];
  T* dr = a.out + g * a.map.stride + col * a.ldo;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kLnClThreads;
    if (idx < a.nvec) {
      float x[VE], d[VE];
      IO::unpack(t.x[i], x);
      IO::unpack(t.g[i], d);
      const float* ga = scale_cells + (i * kLnClThreads + threadIdx.x) * VE;
      float* cell = acc + (i * kLnClThreads + threadIdx.x) * VE;
#pragma unroll
      for (int e = 0; e < VE; ++e) {
        const float xh = (x[e] - t.mean) * inv_stdev;
        if (WGRAD) {
          cell[e] = __builtin_fmaf(d[e], xh, cell[e]);
          cell[kLnClBwdUnits + e] += d[e];
        }
        d[e] = __builtin_fmaf(d[e] * ga[e], inv_stdev, __builtin_fmaf(c1, xh, c0));
      }
      IO::store(dr + VE * static_cast<int64_t>(idx), d);
    }
  }
}

template <typename T, int V, bool WGRAD>
__device__ __forceinline__ void ln_cl_bwd_step(const LnClArgs<T>& a, int64_t row, int64_t nc, int k, unsigned base,
                                               LnClBwdTile<T, V>& F, LnClBwdTile<T, V>& R, LnClBwdTile<T, V>& L,
                                               float* red, float* bc, float* acc, const float* scale_cells)
{
  if (row + nc < a.rows) ln_cl_bwd_reduce<T, V>(a, row + nc, k, base, R, red, scale_cells);
  if (row + 2 * nc < a.rows) ln_cl_bwd_load<T, V>(L, a, row + 2 * nc, base);
  asm volatile("" ::: "memory");
  ln_cl_bwd_finish<T, V, WGRAD>(a, row, k, base, F, bc, scale_cells, acc);
}

template <typename T, int V, bool WGRAD>
__global__ void __launch_bounds__(kLnClThreads)
ln_bwd_cluster(LnClArgs<T> a)
{
  constexpr int VE = Vec16<T>::N;
  static_assert(kLnClThreads * V * VE <= kLnClBwdUnits, "a workgroup's share must fit the LDS accumulators");
  __shared__ float red[2 * kLnClWaves];
  __shared__ float bc[3][2];
  __shared__ float acc[WGRAD ? 2 * kLnClBwdUnits : 1];
  __shared__ float scale_cells[kLnClThreads * V * VE];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  const unsigned base = static_cast<unsigned>(k) * a.per_wg + threadIdx.x;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  {  // from here on `nvec` is the end of this workgroup's share
    const unsigned end = (static_cast<unsigned>(k) + 1) * a.per_wg;
    if (end < a.nvec) a.nvec = end;
  }
  if (WGRAD) {
    for (int p = threadIdx.x; p < 2 * kLnClBwdUnits; p += kLnClThreads) acc[p] = 0.f;  // each thread clears its own cells
  }
  ln_cl_stage_weights<T, V>(a.gamma, 1.f, base, a.nvec, scale_cells);  // read back by the same thread only
  LnClBwdTile<T, V> t0, t1, t2;
  ln_cl_bwd_load<T, V>(t0, a, cl, base);
  if (cl + nc < a.rows) ln_cl_bwd_load<T, V>(t1, a, cl + nc, base);
  if (WGRAD) __syncthreads();  // the clearing loop above is strided differently from the cells' owners
  ln_cl_bwd_reduce<T, V>(a, cl, k, base, t0, red, scale_cells);
  __syncthreads();
  for (int64_t row = cl; row < a.rows; row += 3 * nc) {
    ln_cl_bwd_step<T, V, WGRAD>(a, row, nc, k, base, t0, t1, t2, red, bc[0], acc, scale_cells);
    if (row + nc < a.rows)
      ln_cl_bwd_step<T, V, WGRAD>(a, row + nc, nc, k, base, t1, t2, t0, red, bc[1], acc, scale_cells);
    if (row + 2 * nc < a.rows)
      ln_cl_bwd_step<T, V, WGRAD>(a, row + 2 * nc, nc, k, base, t2, t0, t1, red, bc[2], acc, scale_cells);
  }
  if (WGRAD) {
    // this cluster's partial row: 2n floats, dscale then dbias
    float* out = a.wpart + cl * 2 * a.n;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = base + i * kLnClThreads;
      if (idx < a.nvec) {
        const float* cell = acc + (i * kLnClThreads + threadIdx.x) * VE;
        float dg[VE], db[VE];
#pragma unroll
        for (int e = 0; e < VE; ++e) {
          dg[e] = cell[e];
          db[e] = cell[kLnClBwdUnits + e];
        }
        store_f32_run<VE>(out + VE * static_cast<int64_t>(idx), dg);
        store_f32_run<VE>(out + a.n + VE * static_cast<int64_t>(idx), db);
      }
    }
  }
}

// Adds the P partial rows (2n floats each: dscale then dbias) that the clusters wrote, in
// order.  Long rows and few partials: a thread owns four consecutive positions and walks
// the rows, so every access is a coalesced 16-byte one.  n is a multiple of 4.
__global__ void __launch_bounds__(256)
ln_wgrad_reduce_wide(const float* __restrict__ part, int64_t P, int64_t n, float* __restrict__ dscale,
                     float* __restrict__ dbias)
{
  const int64_t q = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (q >= n / 2) return;  // 2n / 4 quads
  const int64_t j = 4 * q;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int64_t p = 0; p < P; ++p) {
    float w[4];
    Vec16<float>::load(part + p * 2 * n + j, w);
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] += w[c];
  }
  float* out = j < n ? dscale : dbias;
  if (!out) return;
  const int64_t k = j < n ? j : j - n;
#pragma unroll
  for (int c = 0; c < 4; ++c) out[k + c] = acc[c];
}

// ------------------------------------------------------------------------ host side
// Cluster shape for rows of nvec vectors with at most max_v vectors per thread: the fewest
// workgroups per row that hold it (what the workspace query plans with).
inline ClusterPlan plan_ln_cluster(int64_t nvec, int max_v)
{
  const int64_t per = kLnClThreads;
  const int64_t M = (nvec + per * max_v - 1) / (per * max_v);
  if (M < 1 || M > kLnClMaxM) return {0, 0};
  return {static_cast<int>((nvec + per * M - 1) / (per * M)), static_cast<int>(M)};
}

// What a launch uses on a device that holds `cap` workgroups: as many clusters as the
// minimal shape allows, then the workgroups that would stay idle are given to the clusters
// (a row of 98 shares on 256 compute units runs as 2 clusters of 128 instead of 2 of 98).
struct LnClusterLaunch {
  int M, V;
  int64_t clusters;
  unsigned per_wg;
};

inline LnClusterLaunch plan_ln_cluster_launch(int64_t nvec, int64_t rows, ClusterPlan min_plan, int64_t cap,
                                              int64_t max_clusters)
{
  LnClusterLaunch l{0, 0, 0, 0};
  if (!min_plan.M) return l;
  int64_t nc = cap / min_plan.M;
  if (nc > rows) nc = rows;
  if (nc > max_clusters) nc = max_clusters;
  if (nc < 1) return l;
  nc = (rows + (rows + nc - 1) / nc - 1) / ((rows + nc - 1) / nc);  // every cluster walks the same number of rows
  int64_t M = cap / nc;
  if (M > kLnClMaxM) M = kLnClMaxM;
  if (M < min_plan.M) M = min_plan.M;
  const int64_t per_wg = (nvec + M - 1) / M;
  M = (nvec + per_wg - 1) / per_wg;  // drop workgroups that would own nothing
  l.M = static_cast<int>(M);
  l.V = static_cast<int>((per_wg + kLnClThreads - 1) / kLnClThreads);
  l.clusters = nc;
  l.per_wg = static_cast<unsigned>(per_wg);
  return l;
}

// Clusters a launch may use: bounded by what the workspace query assumes (it cannot ask the
// device), by the rows and by the workgroups the device holds at once.
inline int64_t ln_cluster_count_bound(int64_t rows, int M)
{
  int64_t nc = 512 / M;
  if (nc > rows) nc = rows;
  return nc < 1 ? 1 : nc;
}

}  // namespace lbn

// ------------------------------------------------- rows beyond the register clusters
// Rows of millions of entries (instance norm over volumes: 256^3 is 16.8 M entries per
// channel): a workgroup's share no longer fits its registers, and there are so few rows that
// one workgroup per row would leave most of the device idle.  As in batch_norm_stream.hpp a
// cluster shares a row and every workgroup streams its share twice, the second time from
// the caches; persistent over rows.  Weight gradients are not produced here (a slice of
// dscale / dbias of this size fits neither registers nor LDS): layer norm with weights on
// such rows keeps the two-pass kernels.
namespace lbn {

constexpr int kLnStreamThreads = 512;
constexpr int kLnStreamWaves = kLnStreamThreads / kWave;
constexpr int kLnStreamUnroll = 4;
// Vectors per thread at the head of a workgroup's share that stay in the workgroup between the
// two passes (16.8 M-entry rows over 128 workgroups are 64 vectors per thread, 4.1 M-entry rows
// 16: the latter are then read once).  Forward: half of them in registers, half parked in LDS by
// the thread that fetches them again (no barrier), 64 KiB per workgroup, so that two workgroups
// share a compute unit (all sixteen in registers took 136 of them: one workgroup per unit).
constexpr int kLnStreamKeepFwd = 8;
constexpr int kLnStreamLdsFwd = 16 - kLnStreamKeepFwd;
constexpr int kLnStreamKeepBwd = 8;
// Backward: eight vectors per thread and tensor in registers, the next eight parked in LDS by the
// thread that fetches them again (no barrier), 128 KiB per workgroup; the kernel's registers allow
// one workgroup per compute unit anyway.  4.1 M-entry rows over 128 workgroups (15.6 vectors per
// thread and tensor) are then read once: 346 -> 313 us (half as much parked: the same 313 us; two
// workgroups per unit with eight vectors per tensor kept in all: 339 us).
// Requesting the next row's head behind the stores that free its registers and slots (the slots
// filled from memory directly, global_load_lds_dwordx4) loses in both directions (16 x 160^3 x 2:
// forward 202 -> 223 us, backward 311 -> 351 us): the rendezvous keeps the workgroups of the device
// in step, so memory sees a phase of loads and then a phase of stores, and reads mixed into the
// stores cost more than the overlap returns.
constexpr int kLnStreamLdsBwd = 8;

template <int U, typename F>
__device__ __forceinline__ void ln_stream_walk(unsigned begin, unsigned end, F&& f)
{
  unsigned e = begin + threadIdx.x;
  for (; e + (U - 1) * kLnStreamThreads < end; e += U * kLnStreamThreads) f(e, std::integral_constant<int, U>{});
  for (; e < end; e += kLnStreamThreads) f(e, std::integral_constant<int, 1>{});
}

// AFFINE = false (instance norm, layer norm without weights): no loads, the fill value only.
template <typename T, bool AFFINE>
__device__ __forceinline__ void ln_stream_weights(const float* w, unsigned e, float fill, float (&out)[Vec16<T>::N])
{
  constexpr int VE = Vec16<T>::N;
#pragma unroll
  for (int k = 0; k < VE; ++k) out[k] = fill;
  if (AFFINE && w) load_f32_run<VE>(w + VE * static_cast<int64_t>(e), out);
}

template <typename T, bool AFFINE>
__global__ void __launch_bounds__(kLnStreamThreads)
ln_fwd_stream(LnClArgs<T> a)
{
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  // with weights the second pass also holds their loads: half the cache keeps it off the stack
  constexpr int KEEP = AFFINE ? kLnStreamKeepFwd / 2 : kLnStreamKeepFwd;
  constexpr int LK = kLnStreamLdsFwd;
  __shared__ float red[2 * kLnStreamWaves];
  __shared__ float bc[2];
  __shared__ typename IO::raw_t parked[LK > 0 ? LK : 1][kLnStreamThreads];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  const unsigned begin = static_cast<unsigned>(k) * a.per_wg;
  const unsigned end = begin + a.per_wg < a.nvec ? begin + a.per_wg : a.nvec;
  const unsigned parked_begin = begin + KEEP * kLnStreamThreads;
  const unsigned rest_fwd = parked_begin + LK * kLnStreamThreads;  // where streaming takes over
  for (int64_t row = cl; row < a.rows; row += nc) {
    const T* xr = a.x + a.map.offset(row, a.ldx);
    T* yr = a.out + a.map.offset(row, a.ldo);
    const float K = a.sumsq ? 0.f : IO::load1(xr);
    float s = 0.f, q = 0.f;
    // the head of the share stays in registers for the second pass
    typename IO::raw_t kept[KEEP];
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const unsigned e = begin + threadIdx.x + i * kLnStreamThreads;
      kept[i] = typename IO::raw_t{};
      if (e < end) kept[i] = IO::load_raw(xr + VE * static_cast<int64_t>(e));
    }
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      if (begin + threadIdx.x + i * kLnStreamThreads < end) {
        float v[VE];
        IO::unpack(kept[i], v);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float d = v[j] - K;
          s += d;
          q = __builtin_fmaf(d, d, q);
        }
      }
    }
    if constexpr (LK > 0) {  // the next vectors of the share: summed now, parked in LDS for the second pass
      typename IO::raw_t pv[LK];
#pragma unroll
      for (int i = 0; i < LK; ++i) {
        const unsigned e = parked_begin + threadIdx.x + i * kLnStreamThreads;
        pv[i] = typename IO::raw_t{};
        if (e < end) pv[i] = IO::load_raw(xr + VE * static_cast<int64_t>(e));
      }
#pragma unroll
      for (int i = 0; i < LK; ++i) {
        if (parked_begin + threadIdx.x + i * kLnStreamThreads < end) {
          parked[i][threadIdx.x] = pv[i];
          float v[VE];
          IO::unpack(pv[i], v);
#pragma unroll
          for (int j = 0; j < VE; ++j) {
            const float d = v[j] - K;
            s += d;
            q = __builtin_fmaf(d, d, q);
          }
        }
      }
    }
    ln_stream_walk<kLnStreamUnroll>(rest_fwd, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float v[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) IO::load(xr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), v[u]);
#pragma unroll
      for (int u = 0; u < N; ++u)
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float d = v[u][j] - K;
          s += d;
          q = __builtin_fmaf(d, d, q);
        }
    });
    team_sum2<kLnStreamWaves>(s, q, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
    if (threadIdx.x == 0) cluster_publish(s, q, a.slots(row), k, a.tag);
    if (threadIdx.x < kWave) {
      float ts, tq;
      cluster_collect_sums<false>(a.slots(row), a.M, a.tag, a.cw.error, ts, tq);
      if (threadIdx.x == 0) {
        float dm = ts * a.inv_n;
        float var = fmaxf(__builtin_fmaf(-dm, dm, tq * a.inv_n), 0.f);
        if (a.sumsq) {  // the reference's own expression (layer_norm.cpp:99-112)
          const float nf = static_cast<float>(a.n);
          dm = ts / nf;
          var = fmaxf(__fsub_rn(tq / nf, __fmul_rn(dm, dm)), 0.f);
        }
        bc[0] = K + dm;
        bc[1] = 1.0f / sqrtf(var + a.eps);
        if (k == 0) {
          int64_t col, g;
          a.map.split(row, col, g);
          a.stats[g + col * a.ld_stats] = K + dm;
          a.stats[a.map.groups + g + col * a.ld_stats] = var;
        }
      }
    }
    __syncthreads();
    const float mean = bc[0];
    const float inv_stdev = bc[1];
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const unsigned e = begin + threadIdx.x + i * kLnStreamThreads;
      if (e < end) {
        float v[VE], ga[VE], be[VE];
        IO::unpack(kept[i], v);
        ln_stream_weights<T, AFFINE>(a.gamma, e, 1.f, ga);
        ln_stream_weights<T, AFFINE>(a.beta, e, 0.f, be);
#pragma unroll
        for (int j = 0; j < VE; ++j) v[j] = __builtin_fmaf((v[j] - mean) * inv_stdev, ga[j], be[j]);
        IO::store(yr + VE * static_cast<int64_t>(e), v);
      }
    }
    if constexpr (LK > 0) {
#pragma unroll
      for (int i = 0; i < LK; ++i) {
        const unsigned e = parked_begin + threadIdx.x + i * kLnStreamThreads;
        if (e < end) {
          float v[VE], ga[VE], be[VE];
          IO::unpack(parked[i][threadIdx.x], v);
          ln_stream_weights<T, AFFINE>(a.gamma, e, 1.f, ga);
          ln_stream_weights<T, AFFINE>(a.beta, e, 0.f, be);
#pragma unroll
          for (int j = 0; j < VE; ++j) v[j] = __builtin_fmaf((v[j] - mean) * inv_stdev, ga[j], be[j]);
          IO::store(yr + VE * static_cast<int64_t>(e), v);
        }
      }
    }
    ln_stream_walk<kLnStreamUnroll>(rest_fwd, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float v[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) IO::load(xr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), v[u]);
#pragma unroll
      for (int u = 0; u < N; ++u) {
        float ga[VE], be[VE];
        ln_stream_weights<T, AFFINE>(a.gamma, e + u * kLnStreamThreads, 1.f, ga);
        ln_stream_weights<T, AFFINE>(a.beta, e + u * kLnStreamThreads, 0.f, be);
#pragma unroll
        for (int j = 0; j < VE; ++j) v[u][j] = __builtin_fmaf((v[u][j] - mean) * inv_stdev, ga[j], be[j]);
        IO::store(yr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), v[u]);
      }
    });
    __syncthreads();  // bc and red are written again for the next row
  }
}

// Backward without weight gradients.
template <typename T, bool AFFINE>
__global__ void __launch_bounds__(kLnStreamThreads)
ln_bwd_stream(LnClArgs<T> a)
{
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  constexpr int U = kLnStreamUnroll / 2;  // two tensors per step
  __shared__ float red[2 * kLnStreamWaves];
  __shared__ float bc[2];
  __shared__ typename IO::raw_t parked_x[kLnStreamLdsBwd][kLnStreamThreads];
  __shared__ typename IO::raw_t parked_g[kLnStreamLdsBwd][kLnStreamThreads];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  const unsigned begin = static_cast<unsigned>(k) * a.per_wg;
  const unsigned end = begin + a.per_wg < a.nvec ? begin + a.per_wg : a.nvec;
  const unsigned parked_begin = begin + kLnStreamKeepBwd * kLnStreamThreads;
  const unsigned rest_bwd = parked_begin + kLnStreamLdsBwd * kLnStreamThreads;
  for (int64_t row = cl; row < a.rows; row += nc) {
    int64_t col, g;
    a.map.split(row, col, g);
    const T* xr = a.x + g * a.map.stride + col * a.ldx;
    const T* gr = a.dy + g * a.map.stride + col * a.lddy;
    T* dr = a.out + g * a.map.stride + col * a.ldo;
    const float mean = a.stats[g + col * a.ld_stats];
    const float inv_stdev = 1.0f / sqrtf(a.stats[a.map.groups + g + col * a.ld_stats] + a.eps);
    float sa = 0.f, sb = 0.f;
    typename IO::raw_t kept_x[kLnStreamKeepBwd], kept_g[kLnStreamKeepBwd];
#pragma unroll
    for (int i = 0; i < kLnStreamKeepBwd; ++i) {
      const unsigned e = begin + threadIdx.x + i * kLnStreamThreads;
      kept_x[i] = typename IO::raw_t{};
      kept_g[i] = typename IO::raw_t{};
      if (e < end) {
        kept_x[i] = IO::load_raw(xr + VE * static_cast<int64_t>(e));
        kept_g[i] = IO::load_raw(gr + VE * static_cast<int64_t>(e));
      }
    }
#pragma unroll
    for (int i = 0; i < kLnStreamKeepBwd; ++i) {
      const unsigned e = begin + threadIdx.x + i * kLnStreamThreads;
      if (e < end) {
        float x[VE], d[VE], ga[VE];
        IO::unpack(kept_x[i], x);
        IO::unpack(kept_g[i], d);
        ln_stream_weights<T, AFFINE>(a.gamma, e, 1.f, ga);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float gs = d[j] * ga[j];
          sa += gs;
          sb = __builtin_fmaf(gs, (x[j] - mean) * inv_stdev, sb);
        }
      }
    }
    // the next vectors of the share: summed now, parked in LDS for the second pass
#pragma unroll
    for (int i0 = 0; i0 < kLnStreamLdsBwd; i0 += 2) {  // two vectors of each tensor at a time
      typename IO::raw_t px[2], pg[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const unsigned e = parked_begin + threadIdx.x + (i0 + i) * kLnStreamThreads;
        px[i] = typename IO::raw_t{};
        pg[i] = typename IO::raw_t{};
        if (i0 + i < kLnStreamLdsBwd && e < end) {
          px[i] = IO::load_raw(xr + VE * static_cast<int64_t>(e));
          pg[i] = IO::load_raw(gr + VE * static_cast<int64_t>(e));
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const unsigned e = parked_begin + threadIdx.x + (i0 + i) * kLnStreamThreads;
        if (i0 + i < kLnStreamLdsBwd && e < end) {
          parked_x[i0 + i][threadIdx.x] = px[i];
          parked_g[i0 + i][threadIdx.x] = pg[i];
          float x[VE], d[VE], ga[VE];
          IO::unpack(px[i], x);
          IO::unpack(pg[i], d);
          ln_stream_weights<T, AFFINE>(a.gamma, e, 1.f, ga);
#pragma unroll
          for (int j = 0; j < VE; ++j) {
            const float gs = d[j] * ga[j];
            sa += gs;
            sb = __builtin_fmaf(gs, (x[j] - mean) * inv_stdev, sb);
          }
        }
      }
    }
    ln_stream_walk<U>(rest_bwd, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float x[N][VE], d[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) {
        IO::load(xr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), x[u]);
        IO::load(gr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), d[u]);
      }
#pragma unroll
      for (int u = 0; u < N; ++u) {
        float ga[VE];
        ln_stream_weights<T, AFFINE>(a.gamma, e + u * kLnStreamThreads, 1.f, ga);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float gs = d[u][j] * ga[j];
          sa += gs;
          sb = __builtin_fmaf(gs, (x[u][j] - mean) * inv_stdev, sb);
        }
      }
    });
    team_sum2<kLnStreamWaves>(sa, sb, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
    if (threadIdx.x == 0) cluster_publish(sa, sb, a.slots(row), k, a.tag);
    if (threadIdx.x < kWave) {
      float ta, tb;
      cluster_collect_sums<false>(a.slots(row), a.M, a.tag, a.cw.error, ta, tb);
      if (threadIdx.x == 0) {
        const float dmean = -ta * inv_stdev;
        const float dvar = -tb * inv_stdev * inv_stdev * 0.5f;
        bc[0] = dmean * a.inv_n;
        bc[1] = -tb * inv_stdev * a.inv_n;  // dvar * 2 / n per unit of xh
        if (k == 0) {
          a.sgrad[g + col * a.ld_sgrad] = dmean;
          a.sgrad[a.map.groups + g + col * a.ld_sgrad] = dvar;
        }
      }
    }
    __syncthreads();
    const float c0 = bc[0];
    const float c1 = bc[1];
#pragma unroll
    for (int i = 0; i < kLnStreamKeepBwd; ++i) {
      const unsigned e = begin + threadIdx.x + i * kLnStreamThreads;
      if (e < end) {
        float x[VE], d[VE], ga[VE];
        IO::unpack(kept_x[i], x);
        IO::unpack(kept_g[i], d);
        ln_stream_weights<T, AFFINE>(a.gamma, e, 1.f, ga);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float xh = (x[j] - mean) * inv_stdev;
          d[j] = __builtin_fmaf(d[j] * ga[j], inv_stdev, __builtin_fmaf(c1, xh, c0));
        }
        IO::store(dr + VE * static_cast<int64_t>(e), d);
      }
    }
#pragma unroll
    for (int i = 0; i < kLnStreamLdsBwd; ++i) {
      const unsigned e = parked_begin + threadIdx.x + i * kLnStreamThreads;
      if (e < end) {
        float x[VE], d[VE], ga[VE];
        IO::unpack(parked_x[i][threadIdx.x], x);
        IO::unpack(parked_g[i][threadIdx.x], d);
        ln_stream_weights<T, AFFINE>(a.gamma, e, 1.f, ga);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float xh = (x[j] - mean) * inv_stdev;
          d[j] = __builtin_fmaf(d[j] * ga[j], inv_stdev, __builtin_fmaf(c1, xh, c0));
        }
        IO::store(dr + VE * static_cast<int64_t>(e), d);
      }
    }
    ln_stream_walk<U>(rest_bwd, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float x[N][VE], d[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) {
        IO::load(xr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), x[u]);
        IO::load(gr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), d[u]);
      }
#pragma unroll
      for (int u = 0; u < N; ++u) {
        float ga[VE];
        ln_stream_weights<T, AFFINE>(a.gamma, e + u * kLnStreamThreads, 1.f, ga);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float xh = (x[u][j] - mean) * inv_stdev;
          d[u][j] = __builtin_fmaf(d[u][j] * ga[j], inv_stdev, __builtin_fmaf(c1, xh, c0));
        }
        IO::store(dr + VE * static_cast<int64_t>(e + u * kLnStreamThreads), d[u]);
      }
    });
    __syncthreads();
  }
}

}  // namespace lbn
