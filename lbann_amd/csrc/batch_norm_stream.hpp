// Batch norm for channels too large for the register-resident clusters of batch_norm.hip
// (more than about a million entries per channel: 112 x 112 maps at a mini-batch of 256,
// volumes).  Math as in batch_norm.hip (batch_normalization.cpp:37-175, :178-329).
//
// A cluster of M workgroups shares a channel as before, but a workgroup's share no longer
// fits its registers: it streams the share once for the sums, publishes them, collects the
// cluster's sums (cluster_sync.hpp) and streams the same share again for the output.  The
// second pass re-reads what the same workgroup read a moment ago: a cluster's channel is
// a few tens of MiB at most and only a few clusters are active, so it comes from the
// caches and x (and dy) cross HBM once, against twice for the sums -> apply kernels.
// Persistent grid: cluster cl takes channels cl, cl + nclusters, ...
#pragma once

#include <type_traits>

#include "batch_norm_math.hpp"
#include "cluster_sync.hpp"
#include "device_utils.hpp"

namespace lbn {

constexpr int kBnStreamThreads = 512;
constexpr int kBnStreamWaves = kBnStreamThreads / kWave;
constexpr int kBnStreamUnroll = 4;
// Vectors per thread at the head of a workgroup's share that stay in registers between the
// two passes (a 112 x 112 map at a mini-batch of 256 over 128 workgroups is 13 vectors per
// thread: read once).
// Half as many for the eight-entry vectors, whose unpacked form takes the registers.
// Further vectors are parked in LDS by the thread that fetches them again (no barrier).  Forward:
// two vectors in registers and eight in LDS (64 KiB), which fits two workgroups on a compute unit
// (sixteen in registers took 202 registers: one workgroup); backward: eight of each tensor in
// registers and four in LDS (its registers allow one workgroup per unit either way).  Measured,
// forward / backward us before -> after: 16 x 128 x 128 x 64 volumes (w = 4) 112 / 196 -> 103 / 176;
// 8 x 160^3 (w = 1) 56 / 80 -> 51 / 71; 64 x 112 x 112 (w = 256) 434 / 546 -> 402 / 546.
template <typename S> constexpr int kBnStreamKeepFwd = Vec16<S>::N > 4 ? 1 : 2;
template <typename S> constexpr int kBnStreamKeepBwd = Vec16<S>::N > 4 ? 4 : 8;
constexpr int kBnStreamLdsFwd = 8;
constexpr int kBnStreamLdsBwd = 4;

template <typename S>
struct BnStreamArgs {
  const S* x;
  const S* dy;  // backward only
  S* out;       // y or dx
  int64_t ldx, lddy, ldo, cs;
  int C, M, use_pivot, bessel, training;
  float eps, decay;
  int64_t n;       // entries per channel
  unsigned seg;    // vectors per column segment of a channel
  unsigned E;      // vectors per channel
  unsigned share;  // vectors per workgroup
  ClusterWorkspace cw;
  ClusterTag tag;
  float* mean;  // forward: written; backward: read
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

// Offset of vector e of a channel inside a matrix with leading dimension ld.
template <typename S>
__device__ __forceinline__ int64_t bn_stream_offset(unsigned e, unsigned seg, int64_t ld)
{
  const unsigned col = e / seg;
  return static_cast<int64_t>(col) * ld + Vec16<S>::N * static_cast<int64_t>(e - col * seg);
}

// Calls f(e, count) for this thread's vectors of the workgroup's share [begin, end): U
// vectors a workgroup-stride apart per call (the caller issues their loads together), then
// the leftovers one at a time.  `count` is a compile-time constant.
template <int U, typename F>
__device__ __forceinline__ void bn_stream_walk(unsigned begin, unsigned end, F&& f)
{
  unsigned e = begin + threadIdx.x;
  for (; e + (U - 1) * kBnStreamThreads < end; e += U * kBnStreamThreads) f(e, std::integral_constant<int, U>{});
  for (; e < end; e += kBnStreamThreads) f(e, std::integral_constant<int, 1>{});
}

template <typename S>
__global__ void __launch_bounds__(kBnStreamThreads)
bn_fwd_stream(BnStreamArgs<S> a)
{
  using IO = Vec16<S>;
  constexpr int VE = IO::N;
  __shared__ float red[2 * kBnStreamWaves];
  __shared__ float bc[2];
  __shared__ typename IO::raw_t parked[kBnStreamLdsFwd][kBnStreamThreads];
  const int nc = gridDim.x / a.M;
  const int cl = blockIdx.x / a.M;
  const int k = blockIdx.x - cl * a.M;
  if (cl >= a.C) return;
  cluster_resolve_tag(a.tag);
  const unsigned begin = static_cast<unsigned>(k) * a.share;
  const unsigned end = begin + a.share < a.E ? begin + a.share : a.E;
  const unsigned parked_begin = begin + kBnStreamKeepFwd<S> * kBnStreamThreads;
  const unsigned rest = parked_begin + kBnStreamLdsFwd * kBnStreamThreads;  // where streaming takes over
  for (int ch = cl; ch < a.C; ch += nc) {
    const S* xc = a.x + static_cast<int64_t>(ch) * a.cs;
    S* yc = a.out + static_cast<int64_t>(ch) * a.cs;
    const float K = a.use_pivot ? IO::load1(xc) : 0.f;
    float s = 0.f, q = 0.f;
    typename IO::raw_t kept[kBnStreamKeepFwd<S>];
#pragma unroll
    for (int i = 0; i < kBnStreamKeepFwd<S>; ++i) {
      const unsigned e = begin + threadIdx.x + i * kBnStreamThreads;
      kept[i] = typename IO::raw_t{};
      if (e < end) kept[i] = IO::load_raw(xc + bn_stream_offset<S>(e, a.seg, a.ldx));
    }
#pragma unroll
    for (int i = 0; i < kBnStreamKeepFwd<S>; ++i) {
      if (begin + threadIdx.x + i * kBnStreamThreads < end) {
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
    {  // the next vectors of the share: summed now, parked in LDS for the second pass
      typename IO::raw_t pv[kBnStreamLdsFwd];
#pragma unroll
      for (int i = 0; i < kBnStreamLdsFwd; ++i) {
        const unsigned e = parked_begin + threadIdx.x + i * kBnStreamThreads;
        pv[i] = typename IO::raw_t{};
        if (e < end) pv[i] = IO::load_raw(xc + bn_stream_offset<S>(e, a.seg, a.ldx));
      }
#pragma unroll
      for (int i = 0; i < kBnStreamLdsFwd; ++i) {
        if (parked_begin + threadIdx.x + i * kBnStreamThreads < end) {
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
    bn_stream_walk<kBnStreamUnroll>(rest, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float v[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) IO::load(xc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.ldx), v[u]);
#pragma unroll
      for (int u = 0; u < N; ++u) {
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const float d = v[u][j] - K;
          s += d;
          q = __builtin_fmaf(d, d, q);
        }
      }
    });
    team_sum2<kBnStreamWaves>(s, q, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
    unsigned long long* slots = a.cw.slots + static_cast<int64_t>(ch) * a.M * 2;
    if (threadIdx.x == 0) cluster_publish(s, q, slots, k, a.tag);
    if (threadIdx.x < kWave) {
      float ts, tq;
      cluster_collect_sums(slots, a.M, a.tag, a.cw.error, ts, tq);
      if (threadIdx.x == 0) {
        float mean, var;
        stats_from_sums(ts, tq, K, a.n, a.bessel, a.eps, mean, var);
        bc[0] = mean;
        bc[1] = 1.0f / sqrtf(var + a.eps);
        if (k == 0) {
          a.mean[ch] = mean;
          a.var[ch] = var;
          a.rmean[ch] = a.decay * a.rmean[ch] + (1.f - a.decay) * mean;
          a.rvar[ch] = a.decay * a.rvar[ch] + (1.f - a.decay) * var;
        }
      }
    }
    __syncthreads();
    const float mean = bc[0];
    const float inv_stdev = bc[1];
    const float scale = a.scale[ch], bias = a.bias[ch];
#pragma unroll
    for (int i = 0; i < kBnStreamKeepFwd<S>; ++i) {
      const unsigned e = begin + threadIdx.x + i * kBnStreamThreads;
      if (e < end) {
        float v[VE];
        IO::unpack(kept[i], v);
#pragma unroll
        for (int j = 0; j < VE; ++j) v[j] = scale * ((v[j] - mean) * inv_stdev) + bias;
        IO::store(yc + bn_stream_offset<S>(e, a.seg, a.ldo), v);
      }
    }
#pragma unroll
    for (int i = 0; i < kBnStreamLdsFwd; ++i) {
      const unsigned e = parked_begin + threadIdx.x + i * kBnStreamThreads;
      if (e < end) {
        float v[VE];
        IO::unpack(parked[i][threadIdx.x], v);
#pragma unroll
        for (int j = 0; j < VE; ++j) v[j] = scale * ((v[j] - mean) * inv_stdev) + bias;
        IO::store(yc + bn_stream_offset<S>(e, a.seg, a.ldo), v);
      }
    }
    bn_stream_walk<kBnStreamUnroll>(rest, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float v[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) IO::load(xc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.ldx), v[u]);
#pragma unroll
      for (int u = 0; u < N; ++u) {
#pragma unroll
        for (int j = 0; j < VE; ++j) v[u][j] = scale * ((v[u][j] - mean) * inv_stdev) + bias;
        IO::store(yc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.ldo), v[u]);
      }
    });
    __syncthreads();  // bc and red are written again for the next channel
  }
}

// Training-mode backward (statistics are variables of the loss).
template <typename S>
__global__ void __launch_bounds__(kBnStreamThreads)
bn_bwd_stream(BnStreamArgs<S> a)
{
  using IO = Vec16<S>;
  constexpr int VE = IO::N;
  constexpr int U = kBnStreamUnroll / 2;  // two tensors per step
  __shared__ float red[2 * kBnStreamWaves];
  __shared__ float bc[2];
  __shared__ typename IO::raw_t parked_x[kBnStreamLdsBwd][kBnStreamThreads];
  __shared__ typename IO::raw_t parked_g[kBnStreamLdsBwd][kBnStreamThreads];
  const int nc = gridDim.x / a.M;
  const int cl = blockIdx.x / a.M;
  const int k = blockIdx.x - cl * a.M;
  if (cl >= a.C) return;
  cluster_resolve_tag(a.tag);
  const unsigned begin = static_cast<unsigned>(k) * a.share;
  const unsigned end = begin + a.share < a.E ? begin + a.share : a.E;
  const unsigned parked_begin = begin + kBnStreamKeepBwd<S> * kBnStreamThreads;
  const unsigned rest = parked_begin + kBnStreamLdsBwd * kBnStreamThreads;
  for (int ch = cl; ch < a.C; ch += nc) {
    const S* xc = a.x + static_cast<int64_t>(ch) * a.cs;
    const S* gc = a.dy + static_cast<int64_t>(ch) * a.cs;
    S* dc = a.out + static_cast<int64_t>(ch) * a.cs;
    const float mean = a.mean[ch];
    const float inv_stdev = 1.0f / sqrtf(a.var[ch] + a.eps);
    const float scale = a.scale[ch];
    float sa = 0.f, sb = 0.f;
    typename IO::raw_t kept_x[kBnStreamKeepBwd<S>], kept_g[kBnStreamKeepBwd<S>];
#pragma unroll
    for (int i = 0; i < kBnStreamKeepBwd<S>; ++i) {
      const unsigned e = begin + threadIdx.x + i * kBnStreamThreads;
      kept_x[i] = typename IO::raw_t{};
      kept_g[i] = typename IO::raw_t{};
      if (e < end) {
        kept_x[i] = IO::load_raw(xc + bn_stream_offset<S>(e, a.seg, a.ldx));
        kept_g[i] = IO::load_raw(gc + bn_stream_offset<S>(e, a.seg, a.lddy));
      }
    }
#pragma unroll
    for (int i = 0; i < kBnStreamKeepBwd<S>; ++i) {
      if (begin + threadIdx.x + i * kBnStreamThreads < end) {
        float x[VE], g[VE];
        IO::unpack(kept_x[i], x);
        IO::unpack(kept_g[i], g);
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          sa += g[j];
          sb = __builtin_fmaf(g[j], x[j] - mean, sb);
        }
      }
    }
#pragma unroll
    for (int i0 = 0; i0 < kBnStreamLdsBwd; i0 += 2) {  // parked in LDS for the second pass, two vectors of each tensor at a time
      typename IO::raw_t px[2], pg[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const unsigned e = parked_begin + threadIdx.x + (i0 + i) * kBnStreamThreads;
        px[i] = typename IO::raw_t{};
        pg[i] = typename IO::raw_t{};
        if (e < end) {
          px[i] = IO::load_raw(xc + bn_stream_offset<S>(e, a.seg, a.ldx));
          pg[i] = IO::load_raw(gc + bn_stream_offset<S>(e, a.seg, a.lddy));
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (parked_begin + threadIdx.x + (i0 + i) * kBnStreamThreads < end) {
          parked_x[i0 + i][threadIdx.x] = px[i];
          parked_g[i0 + i][threadIdx.x] = pg[i];
          float x[VE], g[VE];
          IO::unpack(px[i], x);
          IO::unpack(pg[i], g);
#pragma unroll
          for (int j = 0; j < VE; ++j) {
            sa += g[j];
            sb = __builtin_fmaf(g[j], x[j] - mean, sb);
          }
        }
      }
    }
    bn_stream_walk<U>(rest, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float x[N][VE], g[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) {
        IO::load(xc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.ldx), x[u]);
        IO::load(gc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.lddy), g[u]);
      }
#pragma unroll
      for (int u = 0; u < N; ++u) {
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          sa += g[u][j];
          sb = __builtin_fmaf(g[u][j], x[u][j] - mean, sb);
        }
      }
    });
    team_sum2<kBnStreamWaves>(sa, sb, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
    unsigned long long* slots = a.cw.slots + static_cast<int64_t>(ch) * a.M * 2;
    if (threadIdx.x == 0) cluster_publish(sa, sb, slots, k, a.tag);
    if (threadIdx.x < kWave) {
      float ta, tb;
      cluster_collect_sums(slots, a.M, a.tag, a.cw.error, ta, tb);
      if (threadIdx.x == 0) {
        float ds, db, dmean, dvar;
        grads_from_sums(ta, tb, scale, inv_stdev, ds, db, dmean, dvar);
        bc[0] = dmean / static_cast<float>(a.n);
        bc[1] = dvar * 2.f / static_cast<float>(a.n - (a.bessel ? 1 : 0));
        if (k == 0) {
          a.dscale[ch] = ds;
          a.dbias[ch] = db;
          a.dmean[ch] = dmean;
          a.dvar[ch] = dvar;
        }
      }
    }
    __syncthreads();
    const float dmean_term = bc[0];
    const float dvar_term = bc[1];
    const float k0 = scale * inv_stdev;
#pragma unroll
    for (int i = 0; i < kBnStreamKeepBwd<S>; ++i) {
      const unsigned e = begin + threadIdx.x + i * kBnStreamThreads;
      if (e < end) {
        float x[VE], g[VE];
        IO::unpack(kept_x[i], x);
        IO::unpack(kept_g[i], g);
#pragma unroll
        for (int j = 0; j < VE; ++j) g[j] = g[j] * k0 + dmean_term + dvar_term * (x[j] - mean);
        IO::store(dc + bn_stream_offset<S>(e, a.seg, a.ldo), g);
      }
    }
#pragma unroll
    for (int i = 0; i < kBnStreamLdsBwd; ++i) {
      const unsigned e = parked_begin + threadIdx.x + i * kBnStreamThreads;
      if (e < end) {
        float x[VE], g[VE];
        IO::unpack(parked_x[i][threadIdx.x], x);
        IO::unpack(parked_g[i][threadIdx.x], g);
#pragma unroll
        for (int j = 0; j < VE; ++j) g[j] = g[j] * k0 + dmean_term + dvar_term * (x[j] - mean);
        IO::store(dc + bn_stream_offset<S>(e, a.seg, a.ldo), g);
      }
    }
    bn_stream_walk<U>(rest, end, [&](unsigned e, auto count) {
      constexpr int N = decltype(count)::value;
      float x[N][VE], g[N][VE];
#pragma unroll
      for (int u = 0; u < N; ++u) {
        IO::load(xc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.ldx), x[u]);
        IO::load(gc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.lddy), g[u]);
      }
#pragma unroll
      for (int u = 0; u < N; ++u) {
#pragma unroll
        for (int j = 0; j < VE; ++j) g[u][j] = g[u][j] * k0 + dmean_term + dvar_term * (x[u][j] - mean);
        IO::store(dc + bn_stream_offset<S>(e + u * kBnStreamThreads, a.seg, a.ldo), g[u]);
      }
    });
    __syncthreads();
  }
}

}  // namespace lbn
