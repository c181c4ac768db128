// Batch normalization forward and backward for gfx950: fp32 storage, and IEEE binary16
// storage of x, y, dy, dx with all arithmetic, statistics and weights in fp32 (S is the
// storage type of every kernel below).
//
// Channel c of an NCHW mini-batch is the row range [c*cs, (c+1)*cs) of every matrix
// column, so a per-channel reduction crosses all columns: `width` segments of `cs`
// contiguous floats.  The reduction is split over P workgroups per channel
// (grid C x P) that walk the channel's segments with 128-bit coalesced loads and
// leave one partial pair per workgroup in the workspace; the apply kernel (same
// grid) merges the P partials in a fixed order in its prologue, workgroup 0 of each
// channel writes the statistics, and all P workgroups stream the channel once more
// to write the output.  No atomics: results are bitwise reproducible.
// Training-mode calls on aligned shapes take the single-pass register-resident
// cluster kernels further down; fp32 channels that are not a whole number of 16-byte
// vectors take the row-tile kernels of batch_norm_rows.hpp.
//
// Forward statistics are accumulated about a per-channel pivot (the channel's first
// entry), sum(x-K) and sum((x-K)^2), which removes the cancellation of
// E[x^2]-mean^2 when |mean| >> stdev at no extra cost; LBN_STATS_SUMSQ selects
// K = 0, the reference's formula (batch_normalization.cpp:70-85, :124-128).
#include <initializer_list>
#include <type_traits>
#include <utility>

#include "cluster_sync.hpp"
#include "device_utils.hpp"
#include "host_utils.hpp"
#include "batch_norm_math.hpp"
#include "batch_norm_rows.hpp"
#include "batch_norm_stream.hpp"
#include "reference_order.hpp"

namespace lbn {

constexpr int kBnThreads = 256;
constexpr int kBnMaxSplit = 1024;  // workgroups per channel; a wave merges a channel's partials (three channels of a
                                   // 299 x 299 image had been held to 64 workgroups each)

// Walks the elements of channel c owned by workgroup p: calls f(offset_in_x, offset_in_y...)
// through index arithmetic shared by all kernels.  `unit` = floats per access (4 or 1),
// `seg` = accesses per column segment (cs / unit).
struct ChannelWalk {
  int64_t cs;    // channel size in floats
  int64_t seg;   // accesses per segment
  int64_t total; // accesses per channel = seg * width
};

template <typename S, bool VEC>
__device__ __forceinline__ ChannelWalk make_walk(int64_t cs, int64_t w)
{
  const int64_t seg = VEC ? cs / Vec16<S>::N : cs;
  return {cs, seg, seg * w};
}

// ------------------------------------------------------------------ forward sums
template <typename S, bool VEC>
__global__ void __launch_bounds__(kBnThreads)
bn_fwd_sums(const S* __restrict__ x, int64_t ldx, int64_t cs, int64_t w, int use_pivot,
            float2* __restrict__ part)
{
  __shared__ float red[2 * (kBnThreads / kWave)];
  const int P = gridDim.y;
  const int p = blockIdx.y;
  const int64_t c = blockIdx.x;
  const ChannelWalk wk = make_walk<S, VEC>(cs, w);
  using IO = Vec16<S>;
  constexpr int VE = IO::N;
  const S* xc = x + c * cs;
  const float K = use_pivot ? IO::load1(xc) : 0.f;
  float s = 0.f, q = 0.f;
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const unsigned ucol = static_cast<unsigned>(j) / static_cast<unsigned>(wk.seg);  // j < 2^32 (host check)
    const int64_t col = ucol;
    const int64_t i = static_cast<unsigned>(j) - ucol * static_cast<unsigned>(wk.seg);
    if (VEC) {
      float v[VE];
      IO::load(xc + col * ldx + VE * i, v);
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        const float d = v[k] - K;
        s += d;
        q += d * d;
      }
    }
    else {
      const float d = IO::load1(xc + col * ldx + i) - K;
      s += d;
      q += d * d;
    }
  }
  team_sum2<kBnThreads / kWave>(s, q, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) part[c * P + p] = make_float2(s, q);
}

// Merges the P partial pairs of channel c; every lane of the calling wave gets the sums.
__device__ __forceinline__ float2 merge_partials(const float2* part, int64_t c, int P)
{
  const int lane = threadIdx.x & (kWave - 1);
  float a = 0.f, b = 0.f;
  for (int p = lane; p < P; p += kWave) {  // lane-strided, then the wave: a fixed order
    const float2 v = part[c * P + p];
    a += v.x;
    b += v.y;
  }
  return make_float2(wave_sum(a), wave_sum(b));
}

// Raw per-channel sums for callers that all-reduce them: mean[c] = sum, var[c] = sqsum.
__global__ void __launch_bounds__(kWave)
bn_store_sums(const float2* __restrict__ part, int P, float* __restrict__ mean,
              float* __restrict__ var)
{
  const int64_t c = blockIdx.x;
  const float2 r = merge_partials(part, c, P);
  if (threadIdx.x == 0) {
    mean[c] = r.x;
    var[c] = r.y;
  }
}

__global__ void __launch_bounds__(256)
bn_stats_from_sums(int64_t C, int64_t n, int bessel, float eps, float decay,
                   float* __restrict__ mean, float* __restrict__ var,
                   float* __restrict__ rmean, float* __restrict__ rvar)
{
  const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (c >= C) return;
  if (n <= 1) {
    var[c] = 1.f;
    return;
  }
  float m, v;
  stats_from_sums(mean[c], var[c], 0.f, n, bessel, eps, m, v);
  mean[c] = m;
  var[c] = v;
  rmean[c] = decay * rmean[c] + (1.f - decay) * m;
  rvar[c] = decay * rvar[c] + (1.f - decay) * v;
}

// ----------------------------------------------------------------- forward apply
// FROM_PART: statistics come from the partial sums in `part` (training, fused path)
// and workgroup 0 of each channel publishes them; otherwise mean/var are inputs.
template <typename S, bool VEC, bool FROM_PART>
__global__ void __launch_bounds__(kBnThreads)
bn_fwd_apply(const S* __restrict__ x, S* __restrict__ y, int64_t ldx, int64_t ldy,
             int64_t cs, int64_t w, int use_pivot, int bessel, float eps, float decay,
             const float2* __restrict__ part, float* __restrict__ mean_io,
             float* __restrict__ var_io, const float* __restrict__ gamma,
             const float* __restrict__ beta, float* __restrict__ rmean, float* __restrict__ rvar)
{
  const int P = gridDim.y;
  const int p = blockIdx.y;
  const int64_t c = blockIdx.x;
  const ChannelWalk wk = make_walk<S, VEC>(cs, w);
  using IO = Vec16<S>;
  constexpr int VE = IO::N;
  const S* xc = x + c * cs;
  S* yc = y + c * cs;
  float mean, var;
  if (FROM_PART) {
    const int64_t n = cs * w;
    if (n <= 1) {
      mean = IO::load1(xc);
      var = 1.f;
      if (p == 0 && threadIdx.x == 0) {
        mean_io[c] = mean;
        var_io[c] = var;
      }
    }
    else {
      const float K = use_pivot ? IO::load1(xc) : 0.f;
      const float2 r = merge_partials(part, c, P);
      stats_from_sums(r.x, r.y, K, n, bessel, eps, mean, var);
      if (p == 0 && threadIdx.x == 0) {
        mean_io[c] = mean;
        var_io[c] = var;
        rmean[c] = decay * rmean[c] + (1.f - decay) * mean;
        rvar[c] = decay * rvar[c] + (1.f - decay) * var;
      }
    }
  }
  else {
    mean = mean_io[c];
    var = var_io[c];
  }
  const float inv_stdev = 1.0f / sqrtf(var + eps);
  const float scale = gamma[c];
  const float bias = beta[c];
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const unsigned ucol = static_cast<unsigned>(j) / static_cast<unsigned>(wk.seg);  // j < 2^32 (host check)
    const int64_t col = ucol;
    const int64_t i = static_cast<unsigned>(j) - ucol * static_cast<unsigned>(wk.seg);
    if (VEC) {
      float v[VE];
      IO::load(xc + col * ldx + VE * i, v);
#pragma unroll
      for (int k = 0; k < VE; ++k) v[k] = scale * ((v[k] - mean) * inv_stdev) + bias;
      IO::store(yc + col * ldy + VE * i, v);
    }
    else {
      IO::store1(yc + col * ldy + i, scale * ((IO::load1(xc + col * ldx + i) - mean) * inv_stdev) + bias);
    }
  }
}

// ----------------------------------------------------------------- backward sums
// Two sums per channel carry all four gradients: A = sum(dy), B = sum(dy * (x - mean)).
// DX: outside training the statistics are constants, so dx = dy * scale / stdev needs none of
// the sums and is written in the same pass (three tensors of traffic instead of five).
template <typename S, bool VEC, bool DX = false>
__global__ void __launch_bounds__(kBnThreads)
bn_bwd_sums(const S* __restrict__ x, const S* __restrict__ dy, int64_t ldx, int64_t lddy,
            int64_t cs, int64_t w, const float* __restrict__ mean_in, float2* __restrict__ part,
            const float* __restrict__ var_in = nullptr, const float* __restrict__ gamma = nullptr, float eps = 0.f,
            S* dx = nullptr, int64_t lddx = 0)
{
  __shared__ float red[2 * (kBnThreads / kWave)];
  const int P = gridDim.y;
  const int p = blockIdx.y;
  const int64_t c = blockIdx.x;
  const ChannelWalk wk = make_walk<S, VEC>(cs, w);
  using IO = Vec16<S>;
  constexpr int VE = IO::N;
  const S* xc = x + c * cs;
  const S* gc = dy + c * cs;
  const float mean = mean_in[c];
  const float k0 = DX ? gamma[c] * (1.0f / sqrtf(var_in[c] + eps)) : 0.f;
  S* dc = DX ? dx + c * cs : nullptr;
  float a = 0.f, b = 0.f;
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const unsigned ucol = static_cast<unsigned>(j) / static_cast<unsigned>(wk.seg);  // j < 2^32 (host check)
    const int64_t col = ucol;
    const int64_t i = static_cast<unsigned>(j) - ucol * static_cast<unsigned>(wk.seg);
    if (VEC) {
      float v[VE], g[VE];
      IO::load(xc + col * ldx + VE * i, v);
      IO::load(gc + col * lddy + VE * i, g);
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        a += g[k];
        b += g[k] * (v[k] - mean);
      }
      if (DX) {  // in place (dx aliasing dy): the thread has read what it overwrites
#pragma unroll
        for (int k = 0; k < VE; ++k) g[k] *= k0;
        IO::store(dc + col * lddx + VE * i, g);
      }
    }
    else {
      const float g = IO::load1(gc + col * lddy + i);
      a += g;
      b += g * (IO::load1(xc + col * ldx + i) - mean);
      if (DX) IO::store1(dc + col * lddx + i, g * k0);
    }
  }
  team_sum2<kBnThreads / kWave>(a, b, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) part[c * P + p] = make_float2(a, b);
}

__global__ void __launch_bounds__(kWave)
bn_store_grads(const float2* __restrict__ part, int P, float eps, const float* __restrict__ mean,
               const float* __restrict__ var, const float* __restrict__ gamma,
               float* __restrict__ dscale, float* __restrict__ dbias, float* __restrict__ dmean,
               float* __restrict__ dvar, int training = 1)
{
  const int64_t c = blockIdx.x;
  const float2 r = merge_partials(part, c, P);
  if (threadIdx.x == 0) {
    const float inv_stdev = 1.0f / sqrtf(var[c] + eps);
    float ds, db, dm, dv;
    grads_from_sums(r.x, r.y, gamma[c], inv_stdev, ds, db, dm, dv);
    dscale[c] = ds;
    dbias[c] = db;
    dmean[c] = training ? dm : 0.f;  // statistics are constants outside training
    dvar[c] = training ? dv : 0.f;
  }
  (void)mean;
}

// ---------------------------------------------------------------- backward apply
// FROM_PART: gradients of the statistics come from the partial sums (fused path) and
// workgroup 0 of each channel publishes dscale, dbias, dmean, dvar; otherwise dmean
// and dvar are inputs (already reduced over ranks by the caller).
template <typename S, bool VEC, bool FROM_PART>
__global__ void __launch_bounds__(kBnThreads)
bn_bwd_apply(const S* __restrict__ x, const S* __restrict__ dy, S* __restrict__ dx,
             int64_t ldx, int64_t lddy, int64_t lddx, int64_t cs, int64_t w, int64_t num_per_sum,
             int bessel, float eps, int training, const float2* __restrict__ part,
             const float* __restrict__ mean_in, const float* __restrict__ var_in,
             const float* __restrict__ gamma, float* __restrict__ dscale,
             float* __restrict__ dbias, float* __restrict__ dmean_io, float* __restrict__ dvar_io)
{
  const int P = gridDim.y;
  const int p = blockIdx.y;
  const int64_t c = blockIdx.x;
  const ChannelWalk wk = make_walk<S, VEC>(cs, w);
  using IO = Vec16<S>;
  constexpr int VE = IO::N;
  const S* xc = x + c * cs;
  const S* gc = dy + c * cs;
  S* dc = dx + c * cs;
  const float mean = mean_in[c];
  const float inv_stdev = 1.0f / sqrtf(var_in[c] + eps);
  const float scale = gamma[c];
  float dmean, dvar;
  if (FROM_PART) {
    const float2 r = merge_partials(part, c, P);
    float ds, db;
    grads_from_sums(r.x, r.y, scale, inv_stdev, ds, db, dmean, dvar);
    if (!training) dmean = dvar = 0.f;  // statistics are constants outside training
    if (p == 0 && threadIdx.x == 0) {
      dscale[c] = ds;
      dbias[c] = db;
      dmean_io[c] = dmean;
      dvar_io[c] = dvar;
    }
  }
  else {
    dmean = dmean_io[c];
    dvar = dvar_io[c];
  }
  const bool zero = num_per_sum <= 1;
  const float k0 = scale * inv_stdev;
  const float dmean_term = dmean / static_cast<float>(num_per_sum);
  const float dvar_term = dvar * 2.f / static_cast<float>(num_per_sum - (bessel ? 1 : 0));
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const unsigned ucol = static_cast<unsigned>(j) / static_cast<unsigned>(wk.seg);  // j < 2^32 (host check)
    const int64_t col = ucol;
    const int64_t i = static_cast<unsigned>(j) - ucol * static_cast<unsigned>(wk.seg);
    if (VEC) {
      float v[VE], g[VE];
      if (!zero) {
        IO::load(xc + col * ldx + VE * i, v);
        IO::load(gc + col * lddy + VE * i, g);
      }
#pragma unroll
      for (int k = 0; k < VE; ++k) g[k] = zero ? 0.f : g[k] * k0 + dmean_term + dvar_term * (v[k] - mean);
      IO::store(dc + col * lddx + VE * i, g);
    }
    else {
      IO::store1(dc + col * lddx + i,
                 zero ? 0.f
                      : IO::load1(gc + col * lddy + i) * k0 + dmean_term +
                          dvar_term * (IO::load1(xc + col * ldx + i) - mean));
    }
  }
}


// ===================================================== register-resident clusters
// A channel (E = cs/VE * w 16-byte vectors of VE entries) is shared by a cluster of M workgroups of T
// threads; workgroup k keeps vectors [k*T*V, (k+1)*T*V) in registers.  The grid is
// persistent: cluster cl handles channels cl, cl + nclusters, ...
//
// The loop rotates three register tiles so that nothing waits on something issued
// in the same step: in step s a workgroup (1) reduces tile s+1, whose loads were
// issued a step earlier, and publishes its partial sums, (2) issues the loads of
// tile s+2, (3) collects the cluster's partials of tile s, published a step
// earlier, and finishes tile s from registers.  Loads, the rendezvous latency and
// stores of different channels overlap; every tensor crosses HBM once.
template <int V>
struct BnIndex {
  unsigned col[V], pos[V];
  bool ok[V];
};

template <int T, int V>
__device__ __forceinline__ BnIndex<V> bn_make_index(int k, unsigned seg, unsigned E, unsigned tid = threadIdx.x)
{
  BnIndex<V> ix;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned e = static_cast<unsigned>(k) * (T * V) + i * T + tid;
    ix.ok[i] = e < E;
    ix.col[i] = e / seg;
    ix.pos[i] = e - ix.col[i] * seg;
  }
  return ix;
}

// Tiles stay in registers as the raw vectors that were loaded (fp16 data stays packed: half
// the registers of its fp32 image, so twice the bytes in flight per thread) and are widened
// to fp32 vector by vector where they are used.
template <typename S, int V>
__device__ __forceinline__ void bn_tile_load(typename Vec16<S>::raw_t (&t)[V], const S* base, int64_t ld,
                                             const BnIndex<V>& ix)
{
  constexpr int VE = Vec16<S>::N;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    t[i] = typename Vec16<S>::raw_t{};
    if (ix.ok[i])
      t[i] = Vec16<S>::load_raw(base + static_cast<int64_t>(ix.col[i]) * ld + VE * static_cast<int64_t>(ix.pos[i]));
  }
}

template <typename S, int V>
__device__ __forceinline__ S* bn_tile_address(S* base, int64_t ld, const BnIndex<V>& ix, int i)
{
  return base + static_cast<int64_t>(ix.col[i]) * ld + Vec16<S>::N * static_cast<int64_t>(ix.pos[i]);
}

template <typename S>
struct BnFwdArgs {
  const S* x;
  S* y;
  int64_t ldx, ldy, cs;
  int C, M, use_pivot, bessel;
  float eps, decay;
  int64_t n;
  ClusterWorkspace cw;
  ClusterTag tag;
  float* mean_out;
  float* var_out;
  const float* gamma;
  const float* beta;
  float* rmean;
  float* rvar;
};

// A register tile: a workgroup's share of one channel plus the channel's scalars,
// all loaded at the same point of the pipeline so that no step waits on a load it
// issued itself.
template <typename S, int V>
struct BnFwdTile {
  typename Vec16<S>::raw_t v[V];
  float K, scale, bias;
};

template <typename S, int V>
__device__ __forceinline__ void bn_fwd_load(BnFwdTile<S, V>& t, const BnFwdArgs<S>& a, int ch,
                                            const BnIndex<V>& ix)
{
  const S* xc = a.x + static_cast<int64_t>(ch) * a.cs;
  bn_tile_load<S, V>(t.v, xc, a.ldx, ix);
  t.K = a.use_pivot ? Vec16<S>::load1(xc) : 0.f;
  t.scale = a.gamma[ch];
  t.bias = a.beta[ch];
}

// (1) of a step: partial sums of channel `ch` from tile `t`, published for the cluster.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_fwd_reduce(const BnFwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              const BnFwdTile<S, V>& t, float* red)
{
  const unsigned tid = threadIdx.x;
  const float K = t.K;
  float s = 0.f, q = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float v[Vec16<S>::N];
    Vec16<S>::unpack(t.v[i], v);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) {
      const float d = ix.ok[i] ? v[j] - K : 0.f;
      s += d;
      q += d * d;
    }
  }
  team_sum2<T / kWave>(s, q, red, tid / kWave, tid & (kWave - 1));
  if (tid == 0) cluster_publish(s, q, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, k, a.tag);
}

// (3) of a step: statistics of channel `ch` from the cluster's partials, output from tile `t`.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_fwd_finish(const BnFwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              BnFwdTile<S, V>& t, float* bc)
{
  const unsigned tid = threadIdx.x;
  if (tid < kWave) {
    float ts, tq;
    cluster_collect_sums(a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, a.M, a.tag, a.cw.error, ts, tq);
    if (tid == 0) {
      float mean, var;
      stats_from_sums(ts, tq, t.K, a.n, a.bessel, a.eps, mean, var);
      bc[0] = mean;
      bc[1] = 1.0f / sqrtf(var + a.eps);
      if (k == 0) {
        a.mean_out[ch] = mean;
        a.var_out[ch] = var;
        a.rmean[ch] = a.decay * a.rmean[ch] + (1.f - a.decay) * mean;
        a.rvar[ch] = a.decay * a.rvar[ch] + (1.f - a.decay) * var;
      }
    }
  }
  __syncthreads();
  const float mean = bc[0];
  const float inv_stdev = bc[1];
  S* yc = a.y + static_cast<int64_t>(ch) * a.cs;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (!ix.ok[i]) continue;
    float v[Vec16<S>::N];
    Vec16<S>::unpack(t.v[i], v);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) v[j] = t.scale * ((v[j] - mean) * inv_stdev) + t.bias;
    Vec16<S>::store(bn_tile_address<S, V>(yc, a.ldy, ix, i), v);
  }
}

// One step of the rotation: F finishes channel ch, R holds channel ch + nc, L
// receives channel ch + 2 nc.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_fwd_step(const BnFwdArgs<S>& a, const BnIndex<V>& ix, int ch, int nc, int k,
                                            BnFwdTile<S, V>& F, BnFwdTile<S, V>& R, BnFwdTile<S, V>& L,
                                            float* red, float* bc)
{
  if (ch + nc < a.C) bn_fwd_reduce<S, T, V>(a, ix, ch + nc, k, R, red);
  if (ch + 2 * nc < a.C) bn_fwd_load<S, V>(L, a, ch + 2 * nc, ix);
  asm volatile("" ::: "memory");  // keep the loads above the wait below
  bn_fwd_finish<S, T, V>(a, ix, ch, k, F, bc);
}

template <typename S, int T, int V>
__global__ void __launch_bounds__(T)
bn_fwd_cluster(BnFwdArgs<S> a, unsigned seg, unsigned E)
{
  __shared__ float red[2 * (T / kWave)];
  __shared__ float bc[3][2];
  const int nc = gridDim.x / a.M;
  const int cl = blockIdx.x / a.M;
  const int k = blockIdx.x - cl * a.M;
  const BnIndex<V> ix = bn_make_index<T, V>(k, seg, E);
  BnFwdTile<S, V> t0, t1, t2;
  if (cl >= a.C) return;
  cluster_resolve_tag(a.tag);
  bn_fwd_load<S, V>(t0, a, cl, ix);
  if (cl + nc < a.C) bn_fwd_load<S, V>(t1, a, cl + nc, ix);
  bn_fwd_reduce<S, T, V>(a, ix, cl, k, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  // Each position of the rotation has its own broadcast pair: a step without a reduction has
  // no barrier between the reads of one finish and the write of the next.
  for (int ch = cl; ch < a.C; ch += 3 * nc) {
    bn_fwd_step<S, T, V>(a, ix, ch, nc, k, t0, t1, t2, red, bc[0]);
    if (ch + nc < a.C) bn_fwd_step<S, T, V>(a, ix, ch + nc, nc, k, t1, t2, t0, red, bc[1]);
    if (ch + 2 * nc < a.C) bn_fwd_step<S, T, V>(a, ix, ch + 2 * nc, nc, k, t2, t0, t1, red, bc[2]);
  }
}

template <typename S>
struct BnBwdArgs {
  const S* x;
  const S* dy;
  S* dx;
  int64_t ldx, lddy, lddx, cs;
  int C, M, bessel;
  float eps;
  int64_t n;
  ClusterWorkspace cw;
  ClusterTag tag;
  const float* mean_in;
  const float* var_in;
  const float* gamma;
  float* dscale;
  float* dbias;
  float* dmean_out;
  float* dvar_out;
};

template <typename S, int V>
struct BnBwdTile {
  typename Vec16<S>::raw_t x[V];
  typename Vec16<S>::raw_t g[V];
  float mean, var, scale;
};

template <typename S, int V>
__device__ __forceinline__ void bn_bwd_load(BnBwdTile<S, V>& t, const BnBwdArgs<S>& a, int ch,
                                            const BnIndex<V>& ix)
{
  bn_tile_load<S, V>(t.x, a.x + static_cast<int64_t>(ch) * a.cs, a.ldx, ix);
  bn_tile_load<S, V>(t.g, a.dy + static_cast<int64_t>(ch) * a.cs, a.lddy, ix);
  t.mean = a.mean_in[ch];
  t.var = a.var_in[ch];
  t.scale = a.gamma[ch];
}

// Publishes A = sum(dy), B = sum(dy * (x - mean)); vectors past the end hold zeros in dy.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_bwd_reduce(const BnBwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              const BnBwdTile<S, V>& t, float* red)
{
  const unsigned tid = threadIdx.x;
  const float mean = t.mean;
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float x[Vec16<S>::N], g[Vec16<S>::N];
    Vec16<S>::unpack(t.x[i], x);
    Vec16<S>::unpack(t.g[i], g);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) {
      sa += g[j];
      sb += g[j] * (x[j] - mean);
    }
  }
  team_sum2<T / kWave>(sa, sb, red, tid / kWave, tid & (kWave - 1));
  if (tid == 0) cluster_publish(sa, sb, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, k, a.tag);
}

template <typename S, int T, int V>
__device__ __forceinline__ void bn_bwd_finish(const BnBwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              BnBwdTile<S, V>& t, float* bc)
{
  const unsigned tid = threadIdx.x;
  const float inv_stdev = 1.0f / sqrtf(t.var + a.eps);
  const float scale = t.scale;
  if (tid < kWave) {
    float ta, tb;
    cluster_collect_sums(a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, a.M, a.tag, a.cw.error, ta, tb);
    if (tid == 0) {
      float ds, db, dmean, dvar;
      grads_from_sums(ta, tb, scale, inv_stdev, ds, db, dmean, dvar);
      bc[0] = dmean / static_cast<float>(a.n);
      bc[1] = dvar * 2.f / static_cast<float>(a.n - (a.bessel ? 1 : 0));
      if (k == 0) {
        a.dscale[ch] = ds;
        a.dbias[ch] = db;
        a.dmean_out[ch] = dmean;
        a.dvar_out[ch] = dvar;
      }
    }
  }
  __syncthreads();
  const float dmean_term = bc[0];
  const float dvar_term = bc[1];
  const float k0 = scale * inv_stdev;
  const float mean = t.mean;
  S* dxc = a.dx + static_cast<int64_t>(ch) * a.cs;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (!ix.ok[i]) continue;
    float x[Vec16<S>::N], g[Vec16<S>::N];
    Vec16<S>::unpack(t.x[i], x);
    Vec16<S>::unpack(t.g[i], g);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) g[j] = g[j] * k0 + dmean_term + dvar_term * (x[j] - mean);
    Vec16<S>::store(bn_tile_address<S, V>(dxc, a.lddx, ix, i), g);
  }
}

template <typename S, int T, int V>
__device__ __forceinline__ void bn_bwd_step(const BnBwdArgs<S>& a, const BnIndex<V>& ix, int ch, int nc, int k,
                                            BnBwdTile<S, V>& F, BnBwdTile<S, V>& R, BnBwdTile<S, V>& L, float* red,
                                            float* bc)
{
  if (ch + nc < a.C) bn_bwd_reduce<S, T, V>(a, ix, ch + nc, k, R, red);
  if (ch + 2 * nc < a.C) bn_bwd_load<S, V>(L, a, ch + 2 * nc, ix);
  asm volatile("" ::: "memory");
  bn_bwd_finish<S, T, V>(a, ix, ch, k, F, bc);
}

// Backward in training mode: x and dy are read once, dx written once.
template <typename S, int T, int V>
__global__ void __launch_bounds__(T)
bn_bwd_cluster(BnBwdArgs<S> a, unsigned seg, unsigned E)
{
  __shared__ float red[2 * (T / kWave)];
  __shared__ float bc[3][2];
  const int nc = gridDim.x / a.M;
  const int cl = blockIdx.x / a.M;
  const int k = blockIdx.x - cl * a.M;
  const BnIndex<V> ix = bn_make_index<T, V>(k, seg, E);
  BnBwdTile<S, V> t0, t1, t2;
  if (cl >= a.C) return;
  cluster_resolve_tag(a.tag);
  bn_bwd_load<S, V>(t0, a, cl, ix);
  if (cl + nc < a.C) bn_bwd_load<S, V>(t1, a, cl + nc, ix);
  bn_bwd_reduce<S, T, V>(a, ix, cl, k, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  // Each position of the rotation has its own broadcast pair: a step without a reduction has
  // no barrier between the reads of one finish and the write of the next.
  for (int ch = cl; ch < a.C; ch += 3 * nc) {
    bn_bwd_step<S, T, V>(a, ix, ch, nc, k, t0, t1, t2, red, bc[0]);
    if (ch + nc < a.C) bn_bwd_step<S, T, V>(a, ix, ch + nc, nc, k, t1, t2, t0, red, bc[1]);
    if (ch + 2 * nc < a.C) bn_bwd_step<S, T, V>(a, ix, ch + 2 * nc, nc, k, t2, t0, t1, red, bc[2]);
  }
}

// ---------------------------------------------- a channel in one workgroup's registers
// Channels of up to 8192 vectors (late convolution stages: 14 x 14 or 28 x 28 maps), at least
// as many of them as fill the device: one short-lived workgroup per channel keeps the channel in
// registers between the sums and the output.  Nothing is exchanged between workgroups, so there
// is no rendezvous, no workspace and no tag; workgroups of different channels on a compute unit
// are in different phases, which is what overlaps loads, sums and stores.  Every thread forms the
// statistics from the workgroup's sums itself (one barrier per channel).
template <typename S, int T, int V>
__global__ void __launch_bounds__(T)
bn_fwd_channel(BnFwdArgs<S> a, unsigned seg, unsigned E)
{
  __shared__ float red[2 * (T / kWave)];
  const unsigned tid = threadIdx.x;
  // neighbouring channels, whose segments share cache lines, on one die
  const int ch = static_cast<int>(item_of_block_by_die(blockIdx.x, gridDim.x));
  // The columns and positions of a thread's vectors are formed once for the loads and once more
  // for the stores (kLeanIndex: from a copy of the thread index that the compiler cannot see
  // through): kept across the sums they take two registers per vector, which is what stands
  // between sixteen waves with eight 16-byte vectors each and two workgroups per compute unit.
  constexpr bool kLeanIndex = T == 1024 && V >= 8;
  BnFwdTile<S, V> t;
  {
    const BnIndex<V> ix = bn_make_index<T, V>(0, seg, E);
    bn_fwd_load<S, V>(t, a, ch, ix);
  }
  const float K = t.K;
  float s = 0.f, q = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float v[Vec16<S>::N];
    Vec16<S>::unpack(t.v[i], v);
    const bool in = i * T + tid < E;
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) {
      const float d = in ? v[j] - K : 0.f;
      s += d;
      q += d * d;
    }
  }
  team_sum2<T / kWave>(s, q, red, tid / kWave, tid & (kWave - 1));
  float mean, var;
  stats_from_sums(s, q, K, a.n, a.bessel, a.eps, mean, var);
  if (tid == 0) {
    a.mean_out[ch] = mean;
    a.var_out[ch] = var;
    a.rmean[ch] = a.decay * a.rmean[ch] + (1.f - a.decay) * mean;
    a.rvar[ch] = a.decay * a.rvar[ch] + (1.f - a.decay) * var;
  }
  const float inv_stdev = 1.0f / sqrtf(var + a.eps);
  S* yc = a.y + static_cast<int64_t>(ch) * a.cs;
  unsigned tid2 = tid;
  if (kLeanIndex) asm volatile("" : "+v"(tid2));
  const BnIndex<V> ix = bn_make_index<T, V>(0, seg, E, tid2);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (!ix.ok[i]) continue;
    float v[Vec16<S>::N];
    Vec16<S>::unpack(t.v[i], v);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) v[j] = t.scale * ((v[j] - mean) * inv_stdev) + t.bias;
    Vec16<S>::store(bn_tile_address<S, V>(yc, a.ldy, ix, i), v);
  }
}

template <typename S, int T, int V>
__global__ void __launch_bounds__(T)
bn_bwd_channel(BnBwdArgs<S> a, unsigned seg, unsigned E)
{
  __shared__ float red[2 * (T / kWave)];
  const unsigned tid = threadIdx.x;
  // neighbouring channels, whose segments share cache lines, on one die
  const int ch = static_cast<int>(item_of_block_by_die(blockIdx.x, gridDim.x));
  const BnIndex<V> ix = bn_make_index<T, V>(0, seg, E);
  BnBwdTile<S, V> t;
  bn_bwd_load<S, V>(t, a, ch, ix);
  const float mean = t.mean;
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {  // vectors past the end hold zeros in dy
    float x[Vec16<S>::N], g[Vec16<S>::N];
    Vec16<S>::unpack(t.x[i], x);
    Vec16<S>::unpack(t.g[i], g);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) {
      sa += g[j];
      sb += g[j] * (x[j] - mean);
    }
  }
  team_sum2<T / kWave>(sa, sb, red, tid / kWave, tid & (kWave - 1));
  const float inv_stdev = 1.0f / sqrtf(t.var + a.eps);
  const float scale = t.scale;
  float ds, db, dmean, dvar;
  grads_from_sums(sa, sb, scale, inv_stdev, ds, db, dmean, dvar);
  if (tid == 0) {
    a.dscale[ch] = ds;
    a.dbias[ch] = db;
    a.dmean_out[ch] = dmean;
    a.dvar_out[ch] = dvar;
  }
  const float dmean_term = dmean / static_cast<float>(a.n);
  const float dvar_term = dvar * 2.f / static_cast<float>(a.n - (a.bessel ? 1 : 0));
  const float k0 = scale * inv_stdev;
  S* dxc = a.dx + static_cast<int64_t>(ch) * a.cs;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (!ix.ok[i]) continue;
    float x[Vec16<S>::N], g[Vec16<S>::N];
    Vec16<S>::unpack(t.x[i], x);
    Vec16<S>::unpack(t.g[i], g);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) g[j] = g[j] * k0 + dmean_term + dvar_term * (x[j] - mean);
    Vec16<S>::store(bn_tile_address<S, V>(dxc, a.lddx, ix, i), g);
  }
}

// ------------------------------------------------ the same rotation without barriers
// Variant of the cluster kernels above in which the waves of a workgroup never meet at a
// barrier after the start-up (WaveMerge in cluster_sync.hpp): a wave adds its share, leaves
// the pair in LDS and counts itself in; the last wave to do so publishes the workgroup's
// sums; the first wave that needs the cluster's totals polls for them and hands them to the
// others through LDS.  Measured on 64 x 256 x 56 x 56: fp16 storage, whose steps are half as
// long, gains 6 % (91.7 against 97.7 us per step); fp32 loses 2.5 % (186 against 181 us), so
// the host side picks this variant for 16-bit storage only.  Letting every wave poll the
// cluster for itself was 30 % slower: a wave's polling loads return only after its earlier
// stores are acknowledged, and then all waves wait for that instead of one.
// (1) of a step: partial sums of channel `ch` from tile `t`; the wave that completes the
// workgroup's sums publishes them for the cluster.  No barrier: see WaveMerge.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_fwd_reduce_ws(const BnFwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              const BnFwdTile<S, V>& t, WaveMerge<T / kWave>& stage)
{
  const float K = t.K;
  float s = 0.f, q = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float v[Vec16<S>::N];
    Vec16<S>::unpack(t.v[i], v);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) {
      const float d = ix.ok[i] ? v[j] - K : 0.f;
      s += d;
      q += d * d;
    }
  }
  s = wave_sum_in_last(s);
  q = wave_sum_in_last(q);
  if (wave_merge_arrive(stage, s, q)) {
    wave_merge_read(stage, 0.f, 0.f, s, q);
    s = wave_sum_in_last(s);  // waves in index order: the same sum whichever wave came last
    q = wave_sum_in_last(q);
    if ((threadIdx.x & (kWave - 1)) == kWave - 1)
      cluster_publish(s, q, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, k, a.tag);
  }
}

// (3) of a step, per wave: statistics of channel `ch` from the cluster's partials (the
// first round of polling loads is already under way in `poll`), output from tile `t`.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_fwd_finish_ws(const BnFwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              BnFwdTile<S, V>& t, ClusterPollWide& poll,
                                              WaveMerge<T / kWave>& stage_f, bool poller, unsigned use)
{
  float ts, tq;
  if (poller) {
    cluster_poll_sums(poll, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, a.M, a.tag, a.cw.error, ts, tq);
    wave_merge_broadcast(stage_f, use, ts, tq);
  }
  else {
    wave_merge_wait(stage_f, use, a.cw.error, ts, tq);
  }
  float mean, var;
  stats_from_sums(ts, tq, t.K, a.n, a.bessel, a.eps, mean, var);
  const float inv_stdev = 1.0f / sqrtf(var + a.eps);
  if (k == 0 && threadIdx.x == 0) {
    a.mean_out[ch] = mean;
    a.var_out[ch] = var;
    a.rmean[ch] = a.decay * a.rmean[ch] + (1.f - a.decay) * mean;
    a.rvar[ch] = a.decay * a.rvar[ch] + (1.f - a.decay) * var;
  }
  S* yc = a.y + static_cast<int64_t>(ch) * a.cs;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (!ix.ok[i]) continue;
    float v[Vec16<S>::N];
    Vec16<S>::unpack(t.v[i], v);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) v[j] = t.scale * ((v[j] - mean) * inv_stdev) + t.bias;
    Vec16<S>::store(bn_tile_address<S, V>(yc, a.ldy, ix, i), v);
  }
}

// One step of the rotation: F finishes channel ch, R holds channel ch + nc, L
// receives channel ch + 2 nc.  The polling loads for F go out before the loads of L, so
// their words are back first and L's loads stay in flight while F is written.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_fwd_step_ws(const BnFwdArgs<S>& a, const BnIndex<V>& ix, int ch, int nc, int k,
                                            BnFwdTile<S, V>& F, BnFwdTile<S, V>& R, BnFwdTile<S, V>& L,
                                            WaveMerge<T / kWave>& stage_r, WaveMerge<T / kWave>& stage_f,
                                            unsigned use)
{
  if (ch + nc < a.C) bn_fwd_reduce_ws<S, T, V>(a, ix, ch + nc, k, R, stage_r);
  ClusterPollWide poll;
  const bool poller = wave_merge_claim(stage_f);
  if (poller) cluster_poll_issue(poll, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, a.M);
  asm volatile("" ::: "memory");  // polling loads first, then the tile
  if (ch + 2 * nc < a.C) bn_fwd_load<S, V>(L, a, ch + 2 * nc, ix);
  asm volatile("" ::: "memory");  // keep the loads above the wait below
  bn_fwd_finish_ws<S, T, V>(a, ix, ch, k, F, poll, stage_f, poller, use);
}

template <typename S, int T, int V>
__global__ void __launch_bounds__(T)
bn_fwd_cluster_ws(BnFwdArgs<S> a, unsigned seg, unsigned E)
{
  __shared__ WaveMerge<T / kWave> stage[3];  // one per position of the rotation
  const int nc = gridDim.x / a.M;
  const int cl = blockIdx.x / a.M;
  const int k = blockIdx.x - cl * a.M;
  const BnIndex<V> ix = bn_make_index<T, V>(k, seg, E);
  BnFwdTile<S, V> t0, t1, t2;
  if (cl >= a.C) return;
  cluster_resolve_tag(a.tag);
  bn_fwd_load<S, V>(t0, a, cl, ix);
  if (cl + nc < a.C) bn_fwd_load<S, V>(t1, a, cl + nc, ix);
  wave_merge_init(stage, 3);
  __syncthreads();  // the kernel's only barrier
  bn_fwd_reduce_ws<S, T, V>(a, ix, cl, k, t0, stage[0]);
  unsigned use = 0;
  for (int ch = cl; ch < a.C; ch += 3 * nc, ++use) {
    bn_fwd_step_ws<S, T, V>(a, ix, ch, nc, k, t0, t1, t2, stage[1], stage[0], use);
    if (ch + nc < a.C) bn_fwd_step_ws<S, T, V>(a, ix, ch + nc, nc, k, t1, t2, t0, stage[2], stage[1], use);
    if (ch + 2 * nc < a.C) bn_fwd_step_ws<S, T, V>(a, ix, ch + 2 * nc, nc, k, t2, t0, t1, stage[0], stage[2], use);
  }
}

// Publishes A = sum(dy), B = sum(dy * (x - mean)); vectors past the end hold zeros in dy.
template <typename S, int T, int V>
__device__ __forceinline__ void bn_bwd_reduce_ws(const BnBwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              const BnBwdTile<S, V>& t, WaveMerge<T / kWave>& stage)
{
  const float mean = t.mean;
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float x[Vec16<S>::N], g[Vec16<S>::N];
    Vec16<S>::unpack(t.x[i], x);
    Vec16<S>::unpack(t.g[i], g);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) {
      sa += g[j];
      sb += g[j] * (x[j] - mean);
    }
  }
  sa = wave_sum_in_last(sa);
  sb = wave_sum_in_last(sb);
  if (wave_merge_arrive(stage, sa, sb)) {
    wave_merge_read(stage, 0.f, 0.f, sa, sb);
    sa = wave_sum_in_last(sa);
    sb = wave_sum_in_last(sb);
    if ((threadIdx.x & (kWave - 1)) == kWave - 1)
      cluster_publish(sa, sb, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, k, a.tag);
  }
}

template <typename S, int T, int V>
__device__ __forceinline__ void bn_bwd_finish_ws(const BnBwdArgs<S>& a, const BnIndex<V>& ix, int ch, int k,
                                              BnBwdTile<S, V>& t, ClusterPollWide& poll,
                                              WaveMerge<T / kWave>& stage_f, bool poller, unsigned use)
{
  const float inv_stdev = 1.0f / sqrtf(t.var + a.eps);
  const float scale = t.scale;
  float ta, tb;
  if (poller) {
    cluster_poll_sums(poll, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, a.M, a.tag, a.cw.error, ta, tb);
    wave_merge_broadcast(stage_f, use, ta, tb);
  }
  else {
    wave_merge_wait(stage_f, use, a.cw.error, ta, tb);
  }
  float ds, db, dmean, dvar;
  grads_from_sums(ta, tb, scale, inv_stdev, ds, db, dmean, dvar);
  const float dmean_term = dmean / static_cast<float>(a.n);
  const float dvar_term = dvar * 2.f / static_cast<float>(a.n - (a.bessel ? 1 : 0));
  if (k == 0 && threadIdx.x == 0) {
    a.dscale[ch] = ds;
    a.dbias[ch] = db;
    a.dmean_out[ch] = dmean;
    a.dvar_out[ch] = dvar;
  }
  const float k0 = scale * inv_stdev;
  const float mean = t.mean;
  S* dxc = a.dx + static_cast<int64_t>(ch) * a.cs;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (!ix.ok[i]) continue;
    float x[Vec16<S>::N], g[Vec16<S>::N];
    Vec16<S>::unpack(t.x[i], x);
    Vec16<S>::unpack(t.g[i], g);
#pragma unroll
    for (int j = 0; j < Vec16<S>::N; ++j) g[j] = g[j] * k0 + dmean_term + dvar_term * (x[j] - mean);
    Vec16<S>::store(bn_tile_address<S, V>(dxc, a.lddx, ix, i), g);
  }
}

template <typename S, int T, int V>
__device__ __forceinline__ void bn_bwd_step_ws(const BnBwdArgs<S>& a, const BnIndex<V>& ix, int ch, int nc, int k,
                                            BnBwdTile<S, V>& F, BnBwdTile<S, V>& R, BnBwdTile<S, V>& L,
                                            WaveMerge<T / kWave>& stage_r, WaveMerge<T / kWave>& stage_f,
                                            unsigned use)
{
  if (ch + nc < a.C) bn_bwd_reduce_ws<S, T, V>(a, ix, ch + nc, k, R, stage_r);
  ClusterPollWide poll;
  const bool poller = wave_merge_claim(stage_f);
  if (poller) cluster_poll_issue(poll, a.cw.slots + static_cast<int64_t>(ch) * a.M * 2, a.M);
  asm volatile("" ::: "memory");
  if (ch + 2 * nc < a.C) bn_bwd_load<S, V>(L, a, ch + 2 * nc, ix);
  asm volatile("" ::: "memory");
  bn_bwd_finish_ws<S, T, V>(a, ix, ch, k, F, poll, stage_f, poller, use);
}

// Backward in training mode: x and dy are read once, dx written once.
template <typename S, int T, int V>
__global__ void __launch_bounds__(T)
bn_bwd_cluster_ws(BnBwdArgs<S> a, unsigned seg, unsigned E)
{
  __shared__ WaveMerge<T / kWave> stage[3];
  const int nc = gridDim.x / a.M;
  const int cl = blockIdx.x / a.M;
  const int k = blockIdx.x - cl * a.M;
  const BnIndex<V> ix = bn_make_index<T, V>(k, seg, E);
  BnBwdTile<S, V> t0, t1, t2;
  if (cl >= a.C) return;
  cluster_resolve_tag(a.tag);
  bn_bwd_load<S, V>(t0, a, cl, ix);
  if (cl + nc < a.C) bn_bwd_load<S, V>(t1, a, cl + nc, ix);
  wave_merge_init(stage, 3);
  __syncthreads();  // the kernel's only barrier
  bn_bwd_reduce_ws<S, T, V>(a, ix, cl, k, t0, stage[0]);
  unsigned use = 0;
  for (int ch = cl; ch < a.C; ch += 3 * nc, ++use) {
    bn_bwd_step_ws<S, T, V>(a, ix, ch, nc, k, t0, t1, t2, stage[1], stage[0], use);
    if (ch + nc < a.C) bn_bwd_step_ws<S, T, V>(a, ix, ch + nc, nc, k, t1, t2, t0, stage[2], stage[1], use);
    if (ch + 2 * nc < a.C) bn_bwd_step_ws<S, T, V>(a, ix, ch + 2 * nc, nc, k, t2, t0, t1, stage[0], stage[2], use);
  }
}

// Workgroup size and vectors per thread of a cluster launch for channels of E vectors.
struct BnClusterShape {
  int T, V, M;
};

// Larger workgroups pay the per-step costs (two barriers, one rendezvous) over more
// bytes: 512 threads are taken when that still splits a channel over at least 8
// workgroups (1024 measured the same), otherwise the smallest size that fits.
static BnClusterShape bn_cluster_shape(int64_t E, int max_v, int first_t)
{
  static const int force_t = std::getenv("LBN_BN_CLUSTER_T") ? std::atoi(std::getenv("LBN_BN_CLUSTER_T")) : 0;
  if (!force_t) {
    for (int T = 512; T >= first_t; T /= 2) {
      const ClusterPlan p = plan_cluster(E, max_v, T, kClusterMaxSumM);
      if (p.M >= 8) return {T, p.V, p.M};
    }
  }
  for (int T = force_t ? force_t : first_t; T <= 1024; T *= 2) {
    const ClusterPlan p = plan_cluster(E, max_v, T, kClusterMaxSumM);
    if (p.M) return {T, p.V, p.M};
    if (force_t) break;
  }
  return {0, 0, 0};
}

// Workgroup size and vectors per thread for a channel of E vectors held by one workgroup: the
// smallest workgroup whose threads hold at most eight vectors (of each tensor); T = 0 when the
// channel is too large or too small, or when C channels of that size leave compute units idle.
static BnClusterShape bn_channel_shape(int64_t E, int64_t C, int64_t max_e = 8192)
{
  static const bool disabled = std::getenv("LBN_BN_NO_CHANNEL") != nullptr;
  if (disabled || E < 512 || E > max_e) return {0, 0, 0};
  const int T = E <= 2048 ? 256 : E <= 4096 ? 512 : 1024;
  const int64_t per = ceil_div(E, T);
  const int V = per <= 2 ? 2 : per <= 4 ? 4 : 8;
  int cus = compute_units();
  if (cus < 1) cus = 256;
  // measured against the clusters on 14 x 14 to 32 x 32 maps: ahead by 5 to 40 % from 128 channels
  // on (256 of them when 256 threads hold a channel), level or behind with 64
  if (C * T < static_cast<int64_t>(cus) * 256 || 2 * C < cus) return {0, 0, 0};
  return {T, V, 1};
}

// The same for channels that are not a whole number of vectors (7 x 7 maps), held as single
// entries, up to sixteen per thread: consecutive lanes take consecutive entries, so a wave
// instruction reads 256 (fp16: 128) contiguous bytes wherever it does not cross from one sample to
// the next.
// Two-byte accesses move half as much per instruction: fp16 tensors beyond 4 M entries stay with
// the row tiles (128 x 2048 x 7 x 7: 68 us this way against 50; 64 x 512 x 7 x 7: 13.5 against 24.8).
static BnClusterShape bn_scalar_channel_shape(int64_t E, int64_t C, int elem_bytes)
{
  static const bool disabled = std::getenv("LBN_BN_NO_CHANNEL") != nullptr;
  if (disabled || E < 1024 || E > 16384) return {0, 0, 0};
  if (elem_bytes == 2 && E * C > (int64_t(4) << 20)) return {0, 0, 0};
  const int T = E <= 4096 ? 256 : E <= 8192 ? 512 : 1024;
  const int64_t per = ceil_div(E, T);
  const int V = per <= 4 ? 4 : per <= 8 ? 8 : 16;
  int cus = compute_units();
  if (cus < 1) cus = 256;
  if (C * T < static_cast<int64_t>(cus) * 256 || 2 * C < cus) return {0, 0, 0};
  return {T, V, 1};
}

// 16-bit storage runs the barrier-free variant of the cluster kernels, fp32 the one with
// barriers; LBN_BN_WAVE_SYNC=0|1 in the environment forces one of them for every type.
template <typename S>
static bool bn_wave_sync()
{
  static const int forced = std::getenv("LBN_BN_WAVE_SYNC") ? std::atoi(std::getenv("LBN_BN_WAVE_SYNC")) : -1;
  return forced >= 0 ? forced != 0 : sizeof(S) == 2;
}

// ==================================================================== host side
// Workgroups per channel: about 4096 workgroups in total, each with at least four
// accesses per thread, at most one wave's worth so a wave can merge the partials.
static int bn_split(int64_t C, int64_t cs, int64_t w)
{
  int64_t P = ceil_div(4096, C);
  const int64_t by_work = ceil_div(cs * w, 4 * 4 * kBnThreads);
  if (P > by_work) P = by_work;
  if (P > kBnMaxSplit) P = kBnMaxSplit;
  if (P < 1) P = 1;
  return static_cast<int>(P);
}

// Channels that are not whole vectors, and channels of one or two vectors, whose segments
// the channel walk would fetch one 16- or 32-byte piece per column (16384 x 4, w = 256:
// 450 us per step that way).
static bool bn_rt_shape(int64_t cs) { return cs % 4 != 0 || cs <= 8; }
constexpr int64_t kBnTileMaxCs = 16;  // aligned channels up to here still try the register-resident row tile

static size_t bn_workspace(int64_t C, int64_t cs, int64_t w)
{
  if (C <= 0 || cs <= 0 || w <= 0) return 0;
  const size_t split = kWorkspaceHeaderBytes + static_cast<size_t>(C) * bn_split(C, cs, w) * sizeof(float2);
  const size_t cluster = cluster_workspace_bytes(C, kClusterMaxSumM);
  size_t need = split > cluster ? split : cluster;
  if (bn_rt_shape(cs) && (C * cs) % 4 == 0) {  // the row-tile path of batch_norm_rows.hpp
    const size_t rows = kWorkspaceHeaderBytes + bn_rt_workspace_bytes(C * cs, w);
    if (rows > need) need = rows;
  }
  return need;
}

// Launches the register-resident forward when the shape allows it.  Returns false
// when the caller must use the two-kernel path.
template <typename S, int T, int V>
static bool bn_launch_fwd_cluster(hipStream_t st, const BnFwdArgs<S>& a, int64_t C, unsigned seg, unsigned E)
{
  const bool ws = bn_wave_sync<S>();
  const int cap = ws ? cluster_capacity(bn_fwd_cluster_ws<S, T, V>, T) : cluster_capacity(bn_fwd_cluster<S, T, V>, T);
  const int64_t ncl = cap / a.M < C ? cap / a.M : C;
  if (ncl < 1) return false;
  if (ws)
    hipLaunchKernelGGL((bn_fwd_cluster_ws<S, T, V>), dim3(static_cast<unsigned>(ncl * a.M)), dim3(T), 0, st, a, seg, E);
  else
    hipLaunchKernelGGL((bn_fwd_cluster<S, T, V>), dim3(static_cast<unsigned>(ncl * a.M)), dim3(T), 0, st, a, seg, E);
  return true;
}

template <typename S, int T, int V>
static bool bn_launch_bwd_cluster(hipStream_t st, const BnBwdArgs<S>& a, int64_t C, unsigned seg, unsigned E)
{
  const bool ws = bn_wave_sync<S>();
  const int cap = ws ? cluster_capacity(bn_bwd_cluster_ws<S, T, V>, T) : cluster_capacity(bn_bwd_cluster<S, T, V>, T);
  const int64_t ncl = cap / a.M < C ? cap / a.M : C;
  if (ncl < 1) return false;
  if (ws)
    hipLaunchKernelGGL((bn_bwd_cluster_ws<S, T, V>), dim3(static_cast<unsigned>(ncl * a.M)), dim3(T), 0, st, a, seg, E);
  else
    hipLaunchKernelGGL((bn_bwd_cluster<S, T, V>), dim3(static_cast<unsigned>(ncl * a.M)), dim3(T), 0, st, a, seg, E);
  return true;
}

template <typename S>
static bool bn_cluster_usable(int64_t C, int64_t cs, int64_t w, const void* ws)
{
  static const bool disabled = std::getenv("LBN_NO_CLUSTER") != nullptr;
  const int64_t E = cs / Vec16<S>::N * w;
  return !disabled && E < (int64_t(1) << 31) - 8192 && cs * w > 1 && C <= (1 << 24) && aligned16(ws);
}

// A thread keeps at most four raw vectors of a forward tile and two (four when a vector is 8
// bytes) of each tensor of a backward tile.
template <typename S>
static bool bn_try_fwd_cluster(hipStream_t st, int64_t C, int64_t cs, int64_t w, int pivot, int bessel,
                               float eps, float decay, const S* x, int64_t ldx, S* y, int64_t ldy,
                               float* mean, float* var, const float* scale, const float* bias,
                               float* rmean, float* rvar, void* ws)
{
  constexpr int VE = Vec16<S>::N;
  if (cs * w > 1 && C <= (1 << 24)) {
    // (vectors of eight halves, widened to fp32 where they are used: up to 4096 of them, which 512
    // threads hold; 64x512x28x28 in 1024 threads measured 3 % behind the clusters)
    BnClusterShape q = bn_channel_shape(cs / VE * w, C, VE == 8 ? 4096 : 8192);
    // forward, 4097 to 8192 vectors of 8 bytes: 512 threads with sixteen each, so that two workgroups
    // share a compute unit (128x1024x14x14 fp16: 55.0 -> 52.3 us per step; 16-byte vectors of fp32
    // then need 130 registers and lose, 93.0 -> 97.1 us)
    if (q.T == 1024 && sizeof(typename Vec16<S>::raw_t) == 8) q = BnClusterShape{512, 16, 1};
    if (q.T) {  // a channel per workgroup: no cluster, no workspace
      const BnFwdArgs<S> a{x, y, ldx, ldy, cs, static_cast<int>(C), 1, pivot, bessel, eps, decay, cs * w,
                           ClusterWorkspace{}, ClusterTag{}, mean, var, scale, bias, rmean, rvar};
      const unsigned seg = static_cast<unsigned>(cs / VE), Eu = static_cast<unsigned>(cs / VE * w);
#define X(TT, VV)                                                                                        \
  if (q.T == TT && q.V == VV) {                                                                          \
    hipLaunchKernelGGL((bn_fwd_channel<S, TT, VV>), dim3(static_cast<unsigned>(C)), dim3(TT), 0, st, a, seg, Eu); \
    return true;                                                                                         \
  }
      X(256, 2) X(256, 4) X(256, 8) X(512, 8)
      if constexpr (VE < 8) { X(1024, 8) }
      if constexpr (sizeof(typename Vec16<S>::raw_t) == 8) { X(512, 16) }
#undef X
    }
  }
  if (!bn_cluster_usable<S>(C, cs, w, ws)) return false;
  const int64_t E = cs / VE * w;
  const BnClusterShape p = bn_cluster_shape(E, 4, 256);
  if (!p.T) return false;
  ClusterLaunchGuard guard(st);
  if (guard.failed()) return false;
  const BnFwdArgs<S> a{x, y, ldx, ldy, cs, static_cast<int>(C), p.M, pivot, bessel, eps, decay, cs * w,
                       cluster_workspace(ws), cluster_call_tag(st, cluster_workspace(ws)), mean, var, scale, bias, rmean, rvar};
  const unsigned seg = static_cast<unsigned>(cs / VE), Eu = static_cast<unsigned>(E);
#define X(TT, VV) \
  if (p.T == TT && p.V == VV) return bn_launch_fwd_cluster<S, TT, VV>(st, a, C, seg, Eu);
  X(256, 1) X(256, 2) X(512, 1) X(512, 2) X(1024, 1) X(1024, 2)
  X(256, 3) X(256, 4) X(512, 3) X(512, 4) X(1024, 3) X(1024, 4)
#undef X
  return false;
}

template <typename S>
static bool bn_try_bwd_cluster(hipStream_t st, int64_t C, int64_t cs, int64_t w, int bessel, float eps,
                               const S* x, int64_t ldx, const S* dy, int64_t lddy, S* dx, int64_t lddx,
                               const float* mean, const float* var, const float* scale, float* dscale,
                               float* dbias, float* dmean, float* dvar, void* ws)
{
  constexpr int VE = Vec16<S>::N;
  if (cs * w > 1 && C <= (1 << 24)) {
    const BnClusterShape q = bn_channel_shape(cs / VE * w, C, VE == 8 ? 4096 : 8192);  // (as in the forward)
    if (q.T) {
      const BnBwdArgs<S> a{x, dy, dx, ldx, lddy, lddx, cs, static_cast<int>(C), 1, bessel, eps, cs * w,
                           ClusterWorkspace{}, ClusterTag{}, mean, var, scale, dscale, dbias, dmean, dvar};
      const unsigned seg = static_cast<unsigned>(cs / VE), Eu = static_cast<unsigned>(cs / VE * w);
#define X(TT, VV)                                                                                        \
  if (q.T == TT && q.V == VV) {                                                                          \
    hipLaunchKernelGGL((bn_bwd_channel<S, TT, VV>), dim3(static_cast<unsigned>(C)), dim3(TT), 0, st, a, seg, Eu); \
    return true;                                                                                         \
  }
      X(256, 2) X(256, 4) X(256, 8) X(512, 8)
      if constexpr (VE < 8) { X(1024, 8) }
#undef X
    }
  }
  if (!bn_cluster_usable<S>(C, cs, w, ws)) return false;
  const int64_t E = cs / VE * w;
  constexpr bool kShortVectors = sizeof(typename Vec16<S>::raw_t) == 8;
  const BnClusterShape p = bn_cluster_shape(E, kShortVectors ? 4 : 2, 256);
  if (!p.T) return false;
  ClusterLaunchGuard guard(st);
  if (guard.failed()) return false;
  const BnBwdArgs<S> a{x, dy, dx, ldx, lddy, lddx, cs, static_cast<int>(C), p.M, bessel, eps, cs * w,
                       cluster_workspace(ws), cluster_call_tag(st, cluster_workspace(ws)), mean, var, scale, dscale, dbias, dmean, dvar};
  const unsigned seg = static_cast<unsigned>(cs / VE), Eu = static_cast<unsigned>(E);
#define X(TT, VV) \
  if (p.T == TT && p.V == VV) return bn_launch_bwd_cluster<S, TT, VV>(st, a, C, seg, Eu);
  X(256, 1) X(512, 1) X(1024, 1) X(256, 2) X(512, 2) X(1024, 2)
  if constexpr (kShortVectors) { X(256, 3) X(512, 3) X(1024, 3) X(256, 4) X(512, 4) X(1024, 4) }
#undef X
  return false;
}

// Channels too large for the register-resident clusters: clusters that stream their share
// twice (batch_norm_stream.hpp).  False: the caller uses the sums -> apply kernels.
template <typename S, bool BWD>
static bool bn_try_stream(hipStream_t st, BnStreamArgs<S> a, int64_t C, int64_t cs, int64_t w, void* ws)
{
  static const bool disabled = std::getenv("LBN_NO_CLUSTER") != nullptr;
  constexpr int VE = Vec16<S>::N;
  const int64_t E = cs / VE * w;
  if (disabled || !aligned16(ws) || E >= (int64_t(1) << 31) || C > (1 << 24)) return false;
  const int cap = BWD ? cluster_capacity(bn_bwd_stream<S>, kBnStreamThreads)
                      : cluster_capacity(bn_fwd_stream<S>, kBnStreamThreads);
  int64_t M = cap < kClusterMaxSumM ? cap : kClusterMaxSumM;
  if (M < 1) return false;
  const int64_t share = ceil_div(E, M);
  M = ceil_div(E, share);
  static const int max_nc = std::getenv("LBN_BN_STREAM_CLUSTERS") ? std::atoi(std::getenv("LBN_BN_STREAM_CLUSTERS")) : 0;
  int64_t nc = cap / M;
  if (max_nc > 0 && nc > max_nc) nc = max_nc;
  if (nc > C) nc = C;
  if (nc < 1) return false;
  a.cs = cs, a.C = static_cast<int>(C), a.M = static_cast<int>(M), a.n = cs * w;
  a.seg = static_cast<unsigned>(cs / VE), a.E = static_cast<unsigned>(E), a.share = static_cast<unsigned>(share);
  a.cw = cluster_workspace(ws);
  ClusterLaunchGuard guard(st);
  if (guard.failed()) return false;
  a.tag = cluster_call_tag(st, a.cw);
  const dim3 grid(static_cast<unsigned>(nc * M));
  if (BWD) hipLaunchKernelGGL(bn_bwd_stream<S>, grid, dim3(kBnStreamThreads), 0, st, a);
  else hipLaunchKernelGGL(bn_fwd_stream<S>, grid, dim3(kBnStreamThreads), 0, st, a);
  return true;
}

static int bn_check(int64_t C, int64_t cs, int64_t w, const int64_t* lds, int nld)
{
  if (C < 0 || cs < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < C * cs) return LBN_ERR_INVALID_ARGUMENT;
  if (C >= (int64_t(1) << 31)) return LBN_ERR_UNSUPPORTED;  // channels ride on gridDim.x
  if (cs * w >= (int64_t(1) << 32)) return LBN_ERR_UNSUPPORTED;  // per-channel index fits 32 bits
  return LBN_OK;
}

template <typename S>
static bool bn_vec_ok(int64_t cs, int64_t w, const void* a, int64_t lda)
{
  constexpr int VE = Vec16<S>::N;
  constexpr uintptr_t bytes = VE * sizeof(S);  // 16, or 8 for fp16 in fours
  return cs % VE == 0 && reinterpret_cast<uintptr_t>(a) % bytes == 0 && (w <= 1 || lda % VE == 0);
}

// fp16 channels that are whole fours but not whole eights (196 = 14 x 14), or matrices aligned
// to 8 but not 16 bytes: the same kernels with 8-byte accesses instead of the scalar walk.
// The same storage tag also carries the row-tile kernels (channels of any odd size on a matrix
// whose rows come in aligned fours: 7 x 7 maps, single-entry channels).
static bool bn_f16_in_fours(int64_t C, int64_t cs, int64_t w,
                            std::initializer_list<std::pair<const void*, int64_t>> mats)
{
  bool eights = true, fours = true, tiles = cs % 4 != 0 || cs <= 8;
  for (const auto& m : mats) {
    eights = eights && bn_vec_ok<__half>(cs, w, m.first, m.second);
    fours = fours && bn_vec_ok<f16x4>(cs, w, m.first, m.second);
    tiles = tiles && row_quads_ok(C * cs, w, m.first, m.second, 2);
  }
  return !eights && (fours || tiles);
}

// ---- channels that are not whole 16-byte vectors, on a matrix whose row quads are aligned
// (batch_norm_rows.hpp).  Storage types with four entries per access: float and f16x4.
template <typename S>
static bool bn_rt_usable(int64_t C, int64_t cs, int64_t w, const void* a, int64_t lda)
{
  return bn_rt_shape(cs) && row_quads_ok(C * cs, w, a, lda, sizeof(S));
}

template <typename S, bool BWD>
static void bn_rt_launch_sums(hipStream_t st, const RowTilePlan& p, const BnRtArgs<S>& a)
{
  const dim3 grid(static_cast<unsigned>(p.tiles), static_cast<unsigned>(p.slabs));
  if (p.gw == 1) hipLaunchKernelGGL((bn_rt_sums<S, 1, BWD>), grid, dim3(kRowTileThreads), 0, st, a);
  else hipLaunchKernelGGL((bn_rt_sums<S, 4, BWD>), grid, dim3(kRowTileThreads), 0, st, a);
}

template <typename S, bool BWD>
static void bn_rt_launch_apply(hipStream_t st, const RowTilePlan& p, const BnRtArgs<S>& a)
{
  const dim3 grid(static_cast<unsigned>(p.tiles), static_cast<unsigned>(p.slabs));
  if (p.gw == 1) hipLaunchKernelGGL((bn_rt_apply<S, 1, BWD>), grid, dim3(kRowTileThreads), 0, st, a);
  else hipLaunchKernelGGL((bn_rt_apply<S, 4, BWD>), grid, dim3(kRowTileThreads), 0, st, a);
}

// Register-resident row tiles (one kernel, one read) for mini-batches of at most 256 columns
// whose channels fit a workgroup's rows; false: use the three-kernel row-tile path.
template <typename S, bool BWD>
static bool bn_rt_try_tile(hipStream_t st, BnRtTileArgs<S> a)
{
  int gw = 0, cpt = 0;
  if (a.w <= 256 && (a.rows_eff = bn_rt_tile_rows(a.cs, RowTilePos<4>::kRows)) > 0) {
    gw = 4;
    cpt = static_cast<int>(ceil_div(a.w, RowTilePos<4>::kGroups));
  }
  else if (a.w <= 64 && (a.rows_eff = bn_rt_tile_rows(a.cs, RowTilePos<1>::kRows)) > 0) {
    gw = 1;
    cpt = static_cast<int>(ceil_div(a.w, RowTilePos<1>::kGroups));
  }
  else {
    return false;
  }
  cpt = cpt <= 1 ? 1 : cpt <= 2 ? 2 : cpt <= 4 ? 4 : cpt <= 8 ? 8 : 16;
  const dim3 grid(static_cast<unsigned>(ceil_div(a.h, a.rows_eff)));
#define X(C, G)                                                                                         \
  if (cpt == C && gw == G) {                                                                            \
    if (BWD) hipLaunchKernelGGL((bn_rt_bwd_tile<S, C, G>), grid, dim3(kRowTileThreads), 0, st, a);         \
    else hipLaunchKernelGGL((bn_rt_fwd_tile<S, C, G>), grid, dim3(kRowTileThreads), 0, st, a);             \
    return true;                                                                                        \
  }
  X(1, 4) X(2, 4) X(4, 4) X(8, 4) X(16, 4) X(1, 1) X(2, 1) X(4, 1) X(8, 1) X(16, 1)
#undef X
  return false;
}

// Forward with given statistics (inference mode, and the last step of a caller that
// reduces the statistics over ranks itself).
template <typename S>
static int bn_fwd_apply_host(hipStream_t st, int64_t C, int64_t cs, int64_t w, float epsilon, const S* x,
                             int64_t ldx, S* y, int64_t ldy, const float* mean, const float* var,
                             const float* scale, const float* bias)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !y || !mean || !var || !scale || !bias) return LBN_ERR_INVALID_ARGUMENT;
  if constexpr (Vec16<S>::N == 4) {  // float or fp16 in fours: the row-tile kernels
    if (bn_rt_usable<S>(C, cs, w, x, ldx) && bn_rt_usable<S>(C, cs, w, y, ldy)) {
      const RowTilePlan p = row_tile_plan(C * cs, w, sizeof(S) == 2 ? 2 : 4);
      BnRtArgs<S> a{};
      a.h = C * cs, a.w = w, a.cs = cs, a.x = x, a.out = y, a.ldx = ldx, a.ldo = ldy;
      a.slab_width = p.slab_width, a.eps = epsilon, a.mean = mean, a.var = var, a.scale = scale, a.bias = bias;
      bn_rt_launch_apply<S, false>(st, p, a);
      return launch_status();
    }
  }
  const int P = bn_split(C, cs, w);
  const dim3 grid(static_cast<unsigned>(C), P);
  float* m = const_cast<float*>(mean);
  float* v = const_cast<float*>(var);
  if (bn_vec_ok<S>(cs, w, x, ldx) && bn_vec_ok<S>(cs, w, y, ldy))
    hipLaunchKernelGGL((bn_fwd_apply<S, true, false>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs,
                       w, 0, 0, epsilon, 0.f, nullptr, m, v, scale, bias, nullptr, nullptr);
  else
    hipLaunchKernelGGL((bn_fwd_apply<S, false, false>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs,
                       w, 0, 0, epsilon, 0.f, nullptr, m, v, scale, bias, nullptr, nullptr);
  return launch_status();
}

template <typename S>
static int bn_fwd_host(hipStream_t st, int64_t C, int64_t cs, int64_t w, int bessel, float epsilon,
                       float decay, int training, const S* x, int64_t ldx, S* y, int64_t ldy, float* mean,
                       float* var, const float* scale, const float* bias, float* running_mean,
                       float* running_var, void* workspace, size_t workspace_bytes, int flags)
{
  if (!training) {
    if (!running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
    return bn_fwd_apply_host<S>(st, C, cs, w, epsilon, x, ldx, y, ldy, running_mean, running_var, scale, bias);
  }
  const int64_t lds[2] = {ldx, ldy};
  if (int e = bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !y || !mean || !var || !scale || !bias || !running_mean || !running_var)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace_payload(workspace));
  const dim3 grid(static_cast<unsigned>(C), P);
  const int pivot = (flags & LBN_STATS_SUMSQ) ? 0 : 1;
  const bool vec = bn_vec_ok<S>(cs, w, x, ldx) && bn_vec_ok<S>(cs, w, y, ldy);
  if (flags & LBN_STATS_REFERENCE_ORDER) {
    // parity tests only: the statistics as one sequential fp32 sum per channel, then the apply
    // kernel that inference uses, on those statistics
    if (C * cs > kRefOrderMaxEntries / w || C > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
    if constexpr (std::is_same<S, f16x4>::value) return LBN_ERR_UNSUPPORTED;  // callers pass plain halves
    else {
      hipLaunchKernelGGL(bn_ref_order_fwd_stats<S>, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, x, ldx, cs, w,
                         bessel, epsilon, decay, mean, var, running_mean, running_var);
      if (vec)
        hipLaunchKernelGGL((bn_fwd_apply<S, true, false>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs, w, 0,
                           bessel, epsilon, decay, part, mean, var, scale, bias, running_mean, running_var);
      else
        hipLaunchKernelGGL((bn_fwd_apply<S, false, false>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs, w, 0,
                           bessel, epsilon, decay, part, mean, var, scale, bias, running_mean, running_var);
      return launch_status();
    }
  }
  {
    using S1 = typename std::conditional<sizeof(S) == 4, f32x1, f16x1>::type;
    if (!vec && cs * w > 1 && C <= (1 << 24)) {
      const BnClusterShape q = bn_scalar_channel_shape(cs * w, C, static_cast<int>(sizeof(S)));
      if (q.T) {  // a channel of single entries per workgroup
        const BnFwdArgs<S1> a{reinterpret_cast<const S1*>(x), reinterpret_cast<S1*>(y), ldx, ldy, cs,
                              static_cast<int>(C), 1, pivot, bessel, epsilon, decay, cs * w, ClusterWorkspace{},
                              ClusterTag{}, mean, var, scale, bias, running_mean, running_var};
        const unsigned seg = static_cast<unsigned>(cs), Eu = static_cast<unsigned>(cs * w);
#define X(TT, VV)                                                                                        \
  if (q.T == TT && q.V == VV) {                                                                          \
    hipLaunchKernelGGL((bn_fwd_channel<S1, TT, VV>), dim3(static_cast<unsigned>(C)), dim3(TT), 0, st, a, seg, Eu); \
    return launch_status();                                                                              \
  }
        X(256, 4) X(256, 8) X(256, 16) X(512, 16) X(1024, 16)
#undef X
      }
    }
  }
  if constexpr (Vec16<S>::N == 4) {  // float or fp16 in fours: the row-tile kernels
    // channels of three or four vectors: the register tile when the mini-batch fits it
    // (1024 x 16, w = 256: 19 us per step against 25 us for clusters), else clusters
    if (!bn_rt_shape(cs) && cs <= kBnTileMaxCs && row_quads_ok(C * cs, w, x, ldx, sizeof(S)) && row_quads_ok(C * cs, w, y, ldy, sizeof(S))) {
      BnRtTileArgs<S> t{};
      t.h = C * cs, t.w = w, t.cs = cs, t.n = cs * w, t.x = x, t.out = y, t.ldx = ldx, t.ldo = ldy;
      t.use_pivot = pivot, t.bessel = bessel, t.eps = epsilon, t.decay = decay, t.mean = mean, t.var = var;
      t.scale = scale, t.bias = bias, t.rmean = running_mean, t.rvar = running_var;
      if (bn_rt_try_tile<S, false>(st, t)) return launch_status();
    }
    if (bn_rt_usable<S>(C, cs, w, x, ldx) && bn_rt_usable<S>(C, cs, w, y, ldy) &&
        (reinterpret_cast<uintptr_t>(workspace) & 7u) == 0) {
      const int64_t h = C * cs;
      {
        BnRtTileArgs<S> t{};
        t.h = h, t.w = w, t.cs = cs, t.n = cs * w, t.x = x, t.out = y, t.ldx = ldx, t.ldo = ldy;
        t.use_pivot = pivot, t.bessel = bessel, t.eps = epsilon, t.decay = decay, t.mean = mean, t.var = var;
        t.scale = scale, t.bias = bias, t.rmean = running_mean, t.rvar = running_var;
        if (bn_rt_try_tile<S, false>(st, t)) return launch_status();
      }
      const RowTilePlan p = row_tile_plan(h, w, sizeof(S) == 2 ? 2 : 4);
      BnRtArgs<S> a{};
      a.h = h, a.w = w, a.cs = cs, a.x = x, a.out = y, a.ldx = ldx, a.ldo = ldy;
      a.slab_width = p.slab_width, a.part = part, a.use_pivot = pivot, a.eps = epsilon;
      a.mean = mean, a.var = var, a.scale = scale, a.bias = bias;
      bn_rt_launch_sums<S, false>(st, p, a);
      const int mode = bn_rt_stats_mode(cs, p.slabs);
      const dim3 sgrid(bn_rt_stats_grid(mode, C));
#define X(MODE)                                                                                              \
  if (mode == MODE)                                                                                          \
    hipLaunchKernelGGL((bn_rt_fwd_stats<S, MODE>), sgrid, dim3(kRowTileThreads), 0, st, C, cs, w, h, p.slabs, \
                       part, x, pivot, bessel, epsilon, decay, mean, var, running_mean, running_var);
      X(kBnRtWave) X(kBnRtWide) X(kBnRtThin)
#undef X
      bn_rt_launch_apply<S, false>(st, p, a);
      return launch_status();
    }
  }
  if (vec && bn_try_fwd_cluster<S>(st, C, cs, w, pivot, bessel, epsilon, decay, x, ldx, y, ldy, mean, var,
                                   scale, bias, running_mean, running_var, workspace))
    return launch_status();
  if (vec && cs * w > 1) {
    BnStreamArgs<S> sa{};
    sa.x = x, sa.out = y, sa.ldx = ldx, sa.ldo = ldy, sa.use_pivot = pivot, sa.bessel = bessel, sa.eps = epsilon;
    sa.decay = decay, sa.mean = mean, sa.var = var, sa.scale = scale, sa.bias = bias;
    sa.rmean = running_mean, sa.rvar = running_var;
    if (bn_try_stream<S, false>(st, sa, C, cs, w, workspace)) return launch_status();
  }
  if (vec) {
    hipLaunchKernelGGL((bn_fwd_sums<S, true>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, pivot, part);
    hipLaunchKernelGGL((bn_fwd_apply<S, true, true>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs, w,
                       pivot, bessel, epsilon, decay, part, mean, var, scale, bias, running_mean,
                       running_var);
  }
  else {
    hipLaunchKernelGGL((bn_fwd_sums<S, false>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, pivot, part);
    hipLaunchKernelGGL((bn_fwd_apply<S, false, true>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs, w,
                       pivot, bessel, epsilon, decay, part, mean, var, scale, bias, running_mean,
                       running_var);
  }
  return launch_status();
}

template <typename S>
static int bn_bwd_host(hipStream_t st, int64_t C, int64_t cs, int64_t w, int bessel, float epsilon,
                       int training, const S* x, int64_t ldx, const S* dy, int64_t lddy, S* dx,
                       int64_t lddx, const float* mean, const float* var, const float* running_mean,
                       const float* running_var, const float* scale, float* dscale, float* dbias,
                       float* dmean, float* dvar, void* workspace, size_t workspace_bytes,
                       bool reference_order = false)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = bn_check(C, cs, w, lds, 3)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  const float* use_mean = training ? mean : running_mean;
  const float* use_var = training ? var : running_var;
  if (!x || !dy || !dx || !use_mean || !use_var || !scale || !dscale || !dbias || !dmean || !dvar)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace_payload(workspace));
  const dim3 grid(static_cast<unsigned>(C), P);
  const int64_t n = cs * w;
  const bool vec = bn_vec_ok<S>(cs, w, x, ldx) && bn_vec_ok<S>(cs, w, dy, lddy) && bn_vec_ok<S>(cs, w, dx, lddx);
  if (reference_order) {
    // parity tests only: the four gradients as sequential fp32 sums per channel, then the apply
    // kernel of the several-rank cut, which takes dmean and dvar as inputs
    if (C * cs > kRefOrderMaxEntries / w || C > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
    if constexpr (std::is_same<S, f16x4>::value) return LBN_ERR_UNSUPPORTED;
    else {
      hipLaunchKernelGGL(bn_ref_order_bwd_sums<S>, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, x, dy, ldx, lddy,
                         cs, w, epsilon, training, use_mean, use_var, scale, dscale, dbias, dmean, dvar);
      if (vec)
        hipLaunchKernelGGL((bn_bwd_apply<S, true, false>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy, lddx,
                           cs, w, n, bessel, epsilon, training, part, use_mean, use_var, scale, dscale, dbias, dmean,
                           dvar);
      else
        hipLaunchKernelGGL((bn_bwd_apply<S, false, false>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy, lddx,
                           cs, w, n, bessel, epsilon, training, part, use_mean, use_var, scale, dscale, dbias, dmean,
                           dvar);
      return launch_status();
    }
  }
  {
    using S1 = typename std::conditional<sizeof(S) == 4, f32x1, f16x1>::type;
    if (!vec && training && n > 1 && C <= (1 << 24)) {
      const BnClusterShape q = bn_scalar_channel_shape(n, C, static_cast<int>(sizeof(S)));
      if (q.T) {
        const BnBwdArgs<S1> a{reinterpret_cast<const S1*>(x), reinterpret_cast<const S1*>(dy),
                              reinterpret_cast<S1*>(dx), ldx, lddy, lddx, cs, static_cast<int>(C), 1, bessel,
                              epsilon, n, ClusterWorkspace{}, ClusterTag{}, use_mean, use_var, scale, dscale, dbias,
                              dmean, dvar};
        const unsigned seg = static_cast<unsigned>(cs), Eu = static_cast<unsigned>(n);
#define X(TT, VV)                                                                                        \
  if (q.T == TT && q.V == VV) {                                                                          \
    hipLaunchKernelGGL((bn_bwd_channel<S1, TT, VV>), dim3(static_cast<unsigned>(C)), dim3(TT), 0, st, a, seg, Eu); \
    return launch_status();                                                                              \
  }
        X(256, 4) X(256, 8) X(256, 16) X(512, 16) X(1024, 16)
#undef X
      }
    }
  }
  if constexpr (Vec16<S>::N == 4) {  // float or fp16 in fours: the row-tile kernels
    if (!bn_rt_shape(cs) && cs <= kBnTileMaxCs && row_quads_ok(C * cs, w, x, ldx, sizeof(S)) && row_quads_ok(C * cs, w, dy, lddy, sizeof(S)) &&
        row_quads_ok(C * cs, w, dx, lddx, sizeof(S))) {
      BnRtTileArgs<S> t{};
      t.h = C * cs, t.w = w, t.cs = cs, t.n = n, t.x = x, t.dy = dy, t.out = dx, t.ldx = ldx, t.lddy = lddy, t.ldo = lddx;
      t.bessel = bessel, t.training = training, t.eps = epsilon;
      t.mean = const_cast<float*>(use_mean), t.var = const_cast<float*>(use_var), t.scale = scale;
      t.dscale = dscale, t.dbias = dbias, t.dmean = dmean, t.dvar = dvar;
      if (bn_rt_try_tile<S, true>(st, t)) return launch_status();
    }
    if (bn_rt_usable<S>(C, cs, w, x, ldx) && bn_rt_usable<S>(C, cs, w, dy, lddy) && bn_rt_usable<S>(C, cs, w, dx, lddx) &&
        (reinterpret_cast<uintptr_t>(workspace) & 7u) == 0) {
      const int64_t h = C * cs;
      {
        BnRtTileArgs<S> t{};
        t.h = h, t.w = w, t.cs = cs, t.n = n, t.x = x, t.dy = dy, t.out = dx, t.ldx = ldx, t.lddy = lddy, t.ldo = lddx;
        t.bessel = bessel, t.training = training, t.eps = epsilon;
        t.mean = const_cast<float*>(use_mean), t.var = const_cast<float*>(use_var), t.scale = scale;
        t.dscale = dscale, t.dbias = dbias, t.dmean = dmean, t.dvar = dvar;
        if (bn_rt_try_tile<S, true>(st, t)) return launch_status();
      }
      const RowTilePlan p = row_tile_plan(h, w, sizeof(S) == 2 ? 2 : 4);
      BnRtArgs<S> a{};
      a.h = h, a.w = w, a.cs = cs, a.x = x, a.dy = dy, a.out = dx, a.ldx = ldx, a.lddy = lddy, a.ldo = lddx;
      a.slab_width = p.slab_width, a.part = part, a.eps = epsilon;
      a.mean = use_mean, a.var = use_var, a.scale = scale, a.dmean = dmean, a.dvar = dvar;
      a.count = static_cast<float>(n), a.count_bessel = static_cast<float>(n - (bessel ? 1 : 0));
      a.zero = n <= 1;
      bn_rt_launch_sums<S, true>(st, p, a);
      const int mode = bn_rt_stats_mode(cs, p.slabs);
      const dim3 sgrid(bn_rt_stats_grid(mode, C));
#define X(MODE)                                                                                          \
  if (mode == MODE)                                                                                      \
    hipLaunchKernelGGL(bn_rt_bwd_stats<MODE>, sgrid, dim3(kRowTileThreads), 0, st, C, cs, h, p.slabs, part, \
                       epsilon, training, use_var, scale, dscale, dbias, dmean, dvar);
      X(kBnRtWave) X(kBnRtWide) X(kBnRtThin)
#undef X
      bn_rt_launch_apply<S, true>(st, p, a);
      return launch_status();
    }
  }
  if (training && vec &&
      bn_try_bwd_cluster<S>(st, C, cs, w, bessel, epsilon, x, ldx, dy, lddy, dx, lddx, use_mean, use_var,
                            scale, dscale, dbias, dmean, dvar, workspace))
    return launch_status();
  if (training && vec && n > 1) {
    BnStreamArgs<S> sa{};
    sa.x = x, sa.dy = dy, sa.out = dx, sa.ldx = ldx, sa.lddy = lddy, sa.ldo = lddx, sa.bessel = bessel;
    sa.eps = epsilon, sa.mean = const_cast<float*>(use_mean), sa.var = const_cast<float*>(use_var), sa.scale = scale;
    sa.dscale = dscale, sa.dbias = dbias, sa.dmean = dmean, sa.dvar = dvar;
    if (bn_try_stream<S, true>(st, sa, C, cs, w, workspace)) return launch_status();
  }
  if (!training && n > 1) {
    // statistics are constants: dx in the same pass as the sums, then the four gradients
    if (vec)
      hipLaunchKernelGGL((bn_bwd_sums<S, true, true>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, use_mean,
                         part, use_var, scale, epsilon, dx, lddx);
    else
      hipLaunchKernelGGL((bn_bwd_sums<S, false, true>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, use_mean,
                         part, use_var, scale, epsilon, dx, lddx);
    hipLaunchKernelGGL(bn_store_grads, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, part,
                       static_cast<int>(grid.y), epsilon, use_mean, use_var, scale, dscale, dbias, dmean, dvar, 0);
    return launch_status();
  }
  if (vec) {
    hipLaunchKernelGGL((bn_bwd_sums<S, true>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, use_mean, part);
    hipLaunchKernelGGL((bn_bwd_apply<S, true, true>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, n, bessel, epsilon, training, part, use_mean, use_var, scale, dscale,
                       dbias, dmean, dvar);
  }
  else {
    hipLaunchKernelGGL((bn_bwd_sums<S, false>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, use_mean, part);
    hipLaunchKernelGGL((bn_bwd_apply<S, false, true>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, n, bessel, epsilon, training, part, use_mean, use_var, scale, dscale,
                       dbias, dmean, dvar);
  }
  return launch_status();
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_batch_norm_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  return bn_workspace(channels, channel_size, width);
}

int lbn_batch_norm_fwd_sums_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                const float* x, int64_t ldx, float* mean, float* var,
                                void* workspace, size_t workspace_bytes)
{
  const int64_t lds[1] = {ldx};
  if (int e = bn_check(C, cs, w, lds, 1)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !mean || !var) return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace_payload(workspace));
  const dim3 grid(static_cast<unsigned>(C), P);
  hipStream_t st = as_stream(stream);
  if (bn_vec_ok<float>(cs, w, x, ldx))
    hipLaunchKernelGGL((bn_fwd_sums<float, true>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, 0, part);
  else
    hipLaunchKernelGGL((bn_fwd_sums<float, false>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, 0, part);
  hipLaunchKernelGGL(bn_store_sums, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, part, P, mean, var);
  return launch_status();
}

int lbn_batch_norm_fwd_stats_f32(lbn_stream_t stream, int64_t C, int64_t num_per_sum, int bessel,
                                 float epsilon, float decay, float* mean, float* var,
                                 float* running_mean, float* running_var)
{
  if (C < 0 || num_per_sum < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (C == 0) return LBN_OK;
  if (!mean || !var || !running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(bn_stats_from_sums, dim3(static_cast<unsigned>(ceil_div(C, 256))), dim3(256), 0,
                     as_stream(stream), C, num_per_sum, bessel, epsilon, decay, mean, var,
                     running_mean, running_var);
  return launch_status();
}

int lbn_batch_norm_fwd_apply_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                 float epsilon, const float* x, int64_t ldx, float* y, int64_t ldy,
                                 const float* mean, const float* var, const float* scale,
                                 const float* bias)
{
  return bn_fwd_apply_host<float>(as_stream(stream), C, cs, w, epsilon, x, ldx, y, ldy, mean, var, scale, bias);
}

int lbn_batch_norm_fwd_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                           float epsilon, float decay, int training, const float* x, int64_t ldx,
                           float* y, int64_t ldy, float* mean, float* var, const float* scale,
                           const float* bias, float* running_mean, float* running_var,
                           void* workspace, size_t workspace_bytes, int flags)
{
  return bn_fwd_host<float>(as_stream(stream), C, cs, w, bessel, epsilon, decay, training, x, ldx, y, ldy,
                            mean, var, scale, bias, running_mean, running_var, workspace, workspace_bytes,
                            flags);
}

int lbn_batch_norm_fwd_f16(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                           float epsilon, float decay, int training, const void* x, int64_t ldx,
                           void* y, int64_t ldy, float* mean, float* var, const float* scale,
                           const float* bias, float* running_mean, float* running_var,
                           void* workspace, size_t workspace_bytes, int flags)
{
  if (C > 0 && cs > 0 && w > 0 && !(flags & LBN_STATS_REFERENCE_ORDER) && bn_f16_in_fours(C, cs, w, {{x, ldx}, {y, ldy}}))
    return bn_fwd_host<f16x4>(as_stream(stream), C, cs, w, bessel, epsilon, decay, training,
                              static_cast<const f16x4*>(x), ldx, static_cast<f16x4*>(y), ldy, mean, var,
                              scale, bias, running_mean, running_var, workspace, workspace_bytes, flags);
  return bn_fwd_host<__half>(as_stream(stream), C, cs, w, bessel, epsilon, decay, training,
                             static_cast<const __half*>(x), ldx, static_cast<__half*>(y), ldy, mean, var,
                             scale, bias, running_mean, running_var, workspace, workspace_bytes, flags);
}

int lbn_batch_norm_bwd_sums_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                float epsilon, const float* x, int64_t ldx, const float* dy,
                                int64_t lddy, const float* mean, const float* var,
                                const float* scale, float* dscale, float* dbias, float* dmean,
                                float* dvar, void* workspace, size_t workspace_bytes)
{
  const int64_t lds[2] = {ldx, lddy};
  if (int e = bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !dy || !mean || !var || !scale || !dscale || !dbias || !dmean || !dvar)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace_payload(workspace));
  const dim3 grid(static_cast<unsigned>(C), P);
  hipStream_t st = as_stream(stream);
  if (bn_vec_ok<float>(cs, w, x, ldx) && bn_vec_ok<float>(cs, w, dy, lddy))
    hipLaunchKernelGGL((bn_bwd_sums<float, true>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, mean, part);
  else
    hipLaunchKernelGGL((bn_bwd_sums<float, false>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, mean, part);
  hipLaunchKernelGGL(bn_store_grads, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, part, P, epsilon,
                     mean, var, scale, dscale, dbias, dmean, dvar);
  return launch_status();
}

int lbn_batch_norm_bwd_apply_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                 int64_t num_per_sum, int bessel, float epsilon, const float* x,
                                 int64_t ldx, const float* dy, int64_t lddy, float* dx,
                                 int64_t lddx, const float* mean, const float* var,
                                 const float* scale, const float* dmean, const float* dvar)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = bn_check(C, cs, w, lds, 3)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !dy || !dx || !mean || !var || !scale || !dmean || !dvar) return LBN_ERR_INVALID_ARGUMENT;
  const int P = bn_split(C, cs, w);
  const dim3 grid(static_cast<unsigned>(C), P);
  hipStream_t st = as_stream(stream);
  float* dm = const_cast<float*>(dmean);
  float* dv = const_cast<float*>(dvar);
  if (bn_vec_ok<float>(cs, w, x, ldx) && bn_vec_ok<float>(cs, w, dy, lddy) && bn_vec_ok<float>(cs, w, dx, lddx))
    hipLaunchKernelGGL((bn_bwd_apply<float, true, false>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, num_per_sum, bessel, epsilon, 1, nullptr, mean, var, scale, nullptr,
                       nullptr, dm, dv);
  else
    hipLaunchKernelGGL((bn_bwd_apply<float, false, false>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, num_per_sum, bessel, epsilon, 1, nullptr, mean, var, scale, nullptr,
                       nullptr, dm, dv);
  return launch_status();
}

int lbn_batch_norm_bwd_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                           float epsilon, int training, const float* x, int64_t ldx,
                           const float* dy, int64_t lddy, float* dx, int64_t lddx,
                           const float* mean, const float* var, const float* running_mean,
                           const float* running_var, const float* scale, float* dscale,
                           float* dbias, float* dmean, float* dvar, void* workspace,
                           size_t workspace_bytes)
{
  return bn_bwd_host<float>(as_stream(stream), C, cs, w, bessel, epsilon, training, x, ldx, dy, lddy, dx, lddx,
                            mean, var, running_mean, running_var, scale, dscale, dbias, dmean, dvar, workspace,
                            workspace_bytes);
}

int lbn_batch_norm_bwd_reference_order_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                                           float epsilon, int training, const float* x, int64_t ldx,
                                           const float* dy, int64_t lddy, float* dx, int64_t lddx,
                                           const float* mean, const float* var, const float* running_mean,
                                           const float* running_var, const float* scale, float* dscale,
                                           float* dbias, float* dmean, float* dvar, void* workspace,
                                           size_t workspace_bytes)
{
  return bn_bwd_host<float>(as_stream(stream), C, cs, w, bessel, epsilon, training, x, ldx, dy, lddy, dx, lddx,
                            mean, var, running_mean, running_var, scale, dscale, dbias, dmean, dvar, workspace,
                            workspace_bytes, true);
}

int lbn_batch_norm_bwd_f16(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                           float epsilon, int training, const void* x, int64_t ldx, const void* dy,
                           int64_t lddy, void* dx, int64_t lddx, const float* mean, const float* var,
                           const float* running_mean, const float* running_var, const float* scale,
                           float* dscale, float* dbias, float* dmean, float* dvar, void* workspace,
                           size_t workspace_bytes)
{
  if (C > 0 && cs > 0 && w > 0 && bn_f16_in_fours(C, cs, w, {{x, ldx}, {dy, lddy}, {dx, lddx}}))
    return bn_bwd_host<f16x4>(as_stream(stream), C, cs, w, bessel, epsilon, training,
                              static_cast<const f16x4*>(x), ldx, static_cast<const f16x4*>(dy), lddy,
                              static_cast<f16x4*>(dx), lddx, mean, var, running_mean, running_var, scale,
                              dscale, dbias, dmean, dvar, workspace, workspace_bytes);
  return bn_bwd_host<__half>(as_stream(stream), C, cs, w, bessel, epsilon, training,
                             static_cast<const __half*>(x), ldx, static_cast<const __half*>(dy), lddy,
                             static_cast<__half*>(dx), lddx, mean, var, running_mean, running_var, scale,
                             dscale, dbias, dmean, dvar, workspace, workspace_bytes);
}

}  // extern "C"
