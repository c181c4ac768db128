// Cross entropy between a predicted distribution x and a ground truth xhat, per sample
// (matrix column): loss = -sum over entries with xhat > 0 of xhat * log(x); backward
// gives dx = -dy * xhat / x where xhat > 0 (0 elsewhere) and dxhat = -dy * log(x).
// Reference CPU code: src/layers/loss/cross_entropy.cpp:35-73 (local_fp_cpu), :75-120
// (local_bp_cpu).
//
// Two ground-truth formats, as in the reference:
//  * dense: xhat has the shape of x.
//  * labels (use_labels): xhat holds one class index per spatial position, stored as a
//    floating-point number in rows [0, spatial) of its column; row r of x belongs to
//    class r / spatial at position r % spatial and xhat(r) is 1 where the position's
//    label equals the class, else 0.  The forward pass therefore needs one entry of x
//    per position: it gathers x(label*spatial + position) instead of streaming all of x.
//
// grid = (width, P): the P workgroups of a column stride over its 16-byte vectors
// (scalars for unaligned shapes); the forward pass reduces each workgroup's partial sum
// in a fixed order and, when P > 1, a one-wave kernel per column adds the P partials.
// No atomics.
#include <cmath>

#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {

constexpr int kCeThreads = 256;
constexpr int kCeWaves = kCeThreads / kWave;
constexpr int kCeMaxParts = 1024;      // workgroups per column (forward: their partial sums are merged by one wave)
constexpr int kCeMaxPartsBwd = 16384;  // backward: nothing to merge

// S: the storage type of every matrix of the layer (float, or __half with fp32 arithmetic).
template <typename S>
struct CeArgs {
  int64_t h, w, spatial;
  const S* x;
  const S* truth;
  int64_t ldx, ldt;
  S* loss;  // forward: element c at loss[c*ld_loss]
  int64_t ld_loss;
  const S* dy;  // backward: element c at dy[c*lddy]
  int64_t lddy;
  S* dx;
  S* dtruth;
  int64_t lddx, lddt;
  float* part;  // [w][P]
};

__device__ __forceinline__ float ce_term(float xhat, float x) { return xhat > 0.f ? -xhat * logf(x) : 0.f; }

// The class index a label entry stands for: conversion to int as in the reference
// (`const int truth_label = local_ground_truth(offset, col)`, cross_entropy.cpp:58).
__device__ __forceinline__ int64_t ce_label(float v) { return static_cast<int64_t>(static_cast<int>(v)); }

template <int T, typename S>
__device__ __forceinline__ void ce_store_partial(const CeArgs<S>& a, float sum, float* red)
{
  sum = team_sum<T / kWave>(sum, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) {
    const int64_t c = blockIdx.x;
    if (gridDim.y == 1) Vec16<S>::store1(a.loss + c * a.ld_loss, sum);
    else a.part[c * gridDim.y + blockIdx.y] = sum;
  }
}

// How a column is accessed: entry by entry, in aligned 16-byte vectors (columns of whole vectors
// on the 16-byte grid), or in 16-byte vectors at the alignment of one entry with the last
// h % VE entries apart (columns of odd height: 1001 classes x 16384 forward 22 us entry by entry).
constexpr int kCeScalar = 0, kCeVec = 1, kCeUnaligned = 2;

template <typename S> struct CeUnaligned;
template <> struct CeUnaligned<float> { using type = f32u; };
template <> struct CeUnaligned<__half> { using type = f16u; };

template <int VEC, typename S>
struct CeIO {
  using U = typename CeUnaligned<S>::type;
  static constexpr int N = Vec16<S>::N;
  static __device__ __forceinline__ void load(const S* p, float (&v)[N])
  {
    if constexpr (VEC == kCeUnaligned) Vec16<U>::load(reinterpret_cast<const U*>(p), v);
    else Vec16<S>::load(p, v);
  }
  static __device__ __forceinline__ void store(S* p, const float (&v)[N])
  {
    if constexpr (VEC == kCeUnaligned) Vec16<U>::store(reinterpret_cast<U*>(p), v);
    else Vec16<S>::store(p, v);
  }
};

template <int VEC, int T, typename S>
__global__ void __launch_bounds__(T)
ce_fwd_dense(CeArgs<S> a)
{
  constexpr int VE = Vec16<S>::N;
  __shared__ float red[T / kWave];
  const int64_t c = blockIdx.x;
  const S* xc = a.x + c * a.ldx;
  const S* tc = a.truth + c * a.ldt;
  const int64_t n = VEC ? a.h / VE : a.h;
  const int64_t step = static_cast<int64_t>(gridDim.y) * T;
  float sum = 0.f;
  for (int64_t j = static_cast<int64_t>(blockIdx.y) * T + threadIdx.x; j < n; j += step) {
    if (VEC) {
      float v[VE], t[VE];
      CeIO<VEC, S>::load(xc + VE * j, v);
      CeIO<VEC, S>::load(tc + VE * j, t);
#pragma unroll
      for (int k = 0; k < VE; ++k) sum += ce_term(t[k], v[k]);
    }
    else {
      sum += ce_term(Vec16<S>::load1(tc + j), Vec16<S>::load1(xc + j));
    }
  }
  if (VEC == kCeUnaligned && blockIdx.y == 0) {  // the entries behind the last whole vector
    const int64_t j = VE * n + threadIdx.x;
    if (j < a.h) sum += ce_term(Vec16<S>::load1(tc + j), Vec16<S>::load1(xc + j));
  }
  ce_store_partial<T>(a, sum, red);
}

// Columns of at most 64 entries (ten classes, say) when there are many of them: a team of 16
// lanes per column, four columns per wave, one entry per access (a wave still reads a
// contiguous run when the columns are packed).  One workgroup per column would leave 246 of
// its 256 threads idle: 21 classes x 1 M columns took 354 us forward that way.
constexpr int kCeShortMax = 64;
constexpr int kCeShortTeam = 16;
constexpr int kCeShortColumns = kCeThreads / kCeShortTeam;  // per workgroup

template <typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_fwd_dense_short(CeArgs<S> a)
{
  const int team = threadIdx.x / kCeShortTeam, l = threadIdx.x % kCeShortTeam;
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kCeShortColumns + team;
  if (c >= a.w) return;  // whole teams leave: the DPP sum below never reads another team's lanes
  const S* xc = a.x + c * a.ldx;
  const S* tc = a.truth + c * a.ldt;
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < kCeShortMax / kCeShortTeam; ++k) {
    const int64_t j = l + k * kCeShortTeam;
    if (j < a.h) sum += ce_term(Vec16<S>::load1(tc + j), Vec16<S>::load1(xc + j));
  }
  sum = row16_sum(sum);
  if (l == 0) Vec16<S>::store1(a.loss + c * a.ld_loss, sum);
}

template <typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_bwd_dense_short(CeArgs<S> a)
{
  const int team = threadIdx.x / kCeShortTeam, l = threadIdx.x % kCeShortTeam;
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kCeShortColumns + team;
  if (c >= a.w) return;
  const float g = Vec16<S>::load1(a.dy + c * a.lddy);
  const S* xc = a.x + c * a.ldx;
  const S* tc = a.truth + c * a.ldt;
  S* dxc = a.dx + c * a.lddx;
  S* dtc = a.dtruth + c * a.lddt;
#pragma unroll
  for (int k = 0; k < kCeShortMax / kCeShortTeam; ++k) {
    const int64_t j = l + k * kCeShortTeam;
    if (j < a.h) {
      const float v = Vec16<S>::load1(xc + j), t = Vec16<S>::load1(tc + j);
      if (a.dtruth) Vec16<S>::store1(dtc + j, -g * logf(v));
      Vec16<S>::store1(dxc + j, t > 0.f ? -g * t / v : 0.f);
    }
  }
}

// One thread per spatial position: gather the entry of x its label points at.
template <typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_fwd_labels(CeArgs<S> a)
{
  __shared__ float red[kCeWaves];
  const int64_t c = blockIdx.x;
  const S* xc = a.x + c * a.ldx;
  const S* tc = a.truth + c * a.ldt;
  const int64_t positions = a.spatial < a.h ? a.spatial : a.h;
  const int64_t step = static_cast<int64_t>(gridDim.y) * kCeThreads;
  float sum = 0.f;
  for (int64_t o = static_cast<int64_t>(blockIdx.y) * kCeThreads + threadIdx.x; o < positions; o += step) {
    const int64_t label = ce_label(Vec16<S>::load1(tc + o));
    const int64_t r = label * a.spatial + o;
    if (label >= 0 && r < a.h) sum += -logf(Vec16<S>::load1(xc + r));
  }
  ce_store_partial<kCeThreads>(a, sum, red);
}

template <typename S>
__global__ void __launch_bounds__(kWave)
ce_merge_parts(int P, const float* __restrict__ part, S* __restrict__ loss, int64_t ld_loss)
{
  const int64_t c = blockIdx.x;
  const int lane = threadIdx.x;
  float acc = 0.f;
  for (int p = lane; p < P; p += kWave) acc += part[c * P + p];  // lane-strided, then the wave: a fixed order
  const float v = wave_sum(acc);
  if (lane == 0) Vec16<S>::store1(loss + c * ld_loss, v);
}

template <int VEC, typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_bwd_dense(CeArgs<S> a)
{
  constexpr int VE = Vec16<S>::N;
  const int64_t c = blockIdx.x;
  const float g = Vec16<S>::load1(a.dy + c * a.lddy);
  const S* xc = a.x + c * a.ldx;
  const S* tc = a.truth + c * a.ldt;
  S* dxc = a.dx + c * a.lddx;
  S* dtc = a.dtruth + c * a.lddt;
  const int64_t n = VEC ? a.h / VE : a.h;
  const int64_t step = static_cast<int64_t>(gridDim.y) * kCeThreads;
  for (int64_t j = static_cast<int64_t>(blockIdx.y) * kCeThreads + threadIdx.x; j < n; j += step) {
    if (VEC) {
      float v[VE], t[VE], d[VE], dt[VE];
      CeIO<VEC, S>::load(xc + VE * j, v);
      CeIO<VEC, S>::load(tc + VE * j, t);
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        dt[k] = -g * logf(v[k]);
        d[k] = t[k] > 0.f ? -g * t[k] / v[k] : 0.f;
      }
      CeIO<VEC, S>::store(dxc + VE * j, d);
      if (a.dtruth) CeIO<VEC, S>::store(dtc + VE * j, dt);
    }
    else {
      const float v = Vec16<S>::load1(xc + j), t = Vec16<S>::load1(tc + j);
      if (a.dtruth) Vec16<S>::store1(dtc + j, -g * logf(v));
      Vec16<S>::store1(dxc + j, t > 0.f ? -g * t / v : 0.f);
    }
  }
  if (VEC == kCeUnaligned && blockIdx.y == 0) {  // the entries behind the last whole vector
    const int64_t j = VE * n + threadIdx.x;
    if (j < a.h) {
      const float v = Vec16<S>::load1(xc + j), t = Vec16<S>::load1(tc + j);
      if (a.dtruth) Vec16<S>::store1(dtc + j, -g * logf(v));
      Vec16<S>::store1(dxc + j, t > 0.f ? -g * t / v : 0.f);
    }
  }
}

// VEC: spatial is a multiple of the vector's entries, so the rows of a vector share a class.
template <bool VEC, typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_bwd_labels(CeArgs<S> a)
{
  constexpr int VE = Vec16<S>::N;
  const int64_t c = blockIdx.x;
  const float g = Vec16<S>::load1(a.dy + c * a.lddy);
  const S* xc = a.x + c * a.ldx;
  const S* tc = a.truth + c * a.ldt;
  S* dxc = a.dx + c * a.lddx;
  const int64_t n = VEC ? a.h / VE : a.h;
  const unsigned per_class = static_cast<unsigned>(VEC ? a.spatial / VE : a.spatial);  // < 2^32 (host check)
  const int64_t step = static_cast<int64_t>(gridDim.y) * kCeThreads;
  for (int64_t j = static_cast<int64_t>(blockIdx.y) * kCeThreads + threadIdx.x; j < n; j += step) {
    const unsigned cls = static_cast<unsigned>(j) / per_class;  // j < 2^32 (host check)
    const unsigned pos = static_cast<unsigned>(j) - cls * per_class;
    if (VEC) {
      float t[VE], d[VE];
      Vec16<S>::load(tc + VE * static_cast<int64_t>(pos), t);
      bool hit[VE];
      bool any = false;
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        d[k] = 0.f;
        hit[k] = ce_label(t[k]) == static_cast<int64_t>(cls);
        any |= hit[k];
      }
      if (any) {
        float v[VE];
        Vec16<S>::load(xc + VE * j, v);
#pragma unroll
        for (int k = 0; k < VE; ++k) d[k] = hit[k] ? -g / v[k] : 0.f;
      }
      Vec16<S>::store(dxc + VE * j, d);
    }
    else {
      Vec16<S>::store1(dxc + j, ce_label(Vec16<S>::load1(tc + pos)) == static_cast<int64_t>(cls)
                                    ? -g / Vec16<S>::load1(xc + j)
                                    : 0.f);
    }
  }
}

// Labels with one position per sample (plain classification: a column of `classes` entries and
// one label): every entry of dx is zero but the label's, so the column goes out in 16-byte
// stores at the alignment of one entry and x is read at the label only.  1000 classes x 65536:
// 100 us entry by entry.
template <typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_bwd_one_label(CeArgs<S> a)
{
  using U = typename CeUnaligned<S>::type;
  constexpr int VE = Vec16<S>::N;
  const int64_t c = blockIdx.x;
  const float g = Vec16<S>::load1(a.dy + c * a.lddy);
  const S* xc = a.x + c * a.ldx;
  S* dxc = a.dx + c * a.lddx;
  const int64_t label = ce_label(Vec16<S>::load1(a.truth + c * a.ldt));
  const float hit = (label >= 0 && label < a.h) ? -g / Vec16<S>::load1(xc + label) : 0.f;
  const int64_t n = a.h / VE;
  const int64_t step = static_cast<int64_t>(gridDim.y) * kCeThreads;
  for (int64_t j = static_cast<int64_t>(blockIdx.y) * kCeThreads + threadIdx.x; j < n; j += step) {
    float d[VE];
#pragma unroll
    for (int k = 0; k < VE; ++k) d[k] = (VE * j + k == label) ? hit : 0.f;
    Vec16<U>::store(reinterpret_cast<U*>(dxc + VE * j), d);
  }
  if (blockIdx.y == 0) {  // the entries behind the last whole vector
    const int64_t j = VE * n + threadIdx.x;
    if (j < a.h) Vec16<S>::store1(dxc + j, j == label ? hit : 0.f);
  }
}

// The same for many short columns: a workgroup takes eight of them, so that the chain of loads
// that ends in x[label] is waited for once per eight columns (one workgroup per column of 1000
// classes x 65536: 80 us, bound by that wait).
constexpr int kCeOneLabelColumns = 8;

template <typename S>
__global__ void __launch_bounds__(kCeThreads)
ce_bwd_one_label_columns(CeArgs<S> a)
{
  using U = typename CeUnaligned<S>::type;
  constexpr int VE = Vec16<S>::N;
  __shared__ float s_hit[kCeOneLabelColumns];
  __shared__ int64_t s_label[kCeOneLabelColumns];
  const int64_t c0 = static_cast<int64_t>(blockIdx.x) * kCeOneLabelColumns;
  if (threadIdx.x < kCeOneLabelColumns) {
    const int64_t c = c0 + threadIdx.x;
    int64_t label = -1;
    float hit = 0.f;
    if (c < a.w) {
      const float g = Vec16<S>::load1(a.dy + c * a.lddy);
      label = ce_label(Vec16<S>::load1(a.truth + c * a.ldt));
      if (label >= 0 && label < a.h) hit = -g / Vec16<S>::load1(a.x + c * a.ldx + label);
      else label = -1;
    }
    s_hit[threadIdx.x] = hit;
    s_label[threadIdx.x] = label;
  }
  __syncthreads();
  const int64_t n = a.h / VE;
  const int tail = static_cast<int>(a.h - VE * n);
#pragma unroll
  for (int k = 0; k < kCeOneLabelColumns; ++k) {
    const int64_t c = c0 + k;
    if (c >= a.w) break;  // block-uniform
    const int64_t label = s_label[k];
    const float hit = s_hit[k];
    S* dxc = a.dx + c * a.lddx;
    for (int64_t j = threadIdx.x; j < n; j += kCeThreads) {
      float d[VE];
#pragma unroll
      for (int e = 0; e < VE; ++e) d[e] = (VE * j + e == label) ? hit : 0.f;
      Vec16<U>::store(reinterpret_cast<U*>(dxc + VE * j), d);
    }
    if (static_cast<int>(threadIdx.x) < tail) {
      const int64_t j = VE * n + threadIdx.x;
      Vec16<S>::store1(dxc + j, j == label ? hit : 0.f);
    }
  }
}

// Workgroups of `threads` threads per column: about 2048 * 256 threads in total, each
// thread with at least four units.  (A single column of a segmentation map, 19 classes x
// 1024 x 2048 positions, had been held to 64 workgroups: 426 us backward.)
static int ce_parts(int64_t w, int64_t units_per_column, int threads = kCeThreads, int max_parts = kCeMaxParts)
{
  int64_t p = ceil_div(2048 * kCeThreads, w * threads);
  const int64_t most = ceil_div(units_per_column, 4 * threads);
  if (p > most) p = most;
  if (p > max_parts) p = max_parts;
  return static_cast<int>(p < 1 ? 1 : p);
}

// The most partial sums per column a forward call can ask for (what the workspace holds).
static int64_t ce_parts_bound(int64_t w)
{
  const int64_t p = ceil_div(2048, w);
  return p > kCeMaxParts ? kCeMaxParts : p;
}

static int ce_check(int64_t h, int64_t w, int use_labels, int64_t spatial, int64_t ldx, int64_t ldt)
{
  if (h < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (use_labels && spatial < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (w > 1 && (ldx < h || ldt < (use_labels ? (spatial < h ? spatial : h) : h))) return LBN_ERR_INVALID_ARGUMENT;
  if (h >= (int64_t(1) << 32) || w >= (int64_t(1) << 31) || (use_labels && spatial >= (int64_t(1) << 32)))
    return LBN_ERR_UNSUPPORTED;
  return LBN_OK;
}

// ve: entries per 16-byte vector.  A matrix that is not there (NULL) constrains nothing.
static bool ce_vec_ok(int64_t h, int64_t w, const void* p, int64_t ld, int ve)
{
  return h % ve == 0 && aligned16(p) && (!p || w <= 1 || ld % ve == 0);
}


template <typename S>
static int ce_fwd_impl(lbn_stream_t stream, int64_t height, int64_t width, int use_labels, int64_t spatial_size,
                       const S* prediction, int64_t ld_prediction, const S* ground_truth, int64_t ld_ground_truth,
                       S* loss, int64_t ld_loss, void* workspace, size_t workspace_bytes)
{
  constexpr int VE = Vec16<S>::N;
  if (int e = ce_check(height, width, use_labels, spatial_size, ld_prediction, ld_ground_truth)) return e;
  if (width == 0) return LBN_OK;
  if (!loss || ld_loss < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (height > 0 && (!prediction || !ground_truth)) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  CeArgs<S> a{};
  a.h = height, a.w = width, a.spatial = use_labels ? spatial_size : 1;
  a.x = prediction, a.truth = ground_truth, a.ldx = ld_prediction, a.ldt = ld_ground_truth;
  a.loss = loss, a.ld_loss = ld_loss, a.part = static_cast<float*>(workspace);
  if (!use_labels && height <= kCeShortMax && width >= 4096) {
    hipLaunchKernelGGL((ce_fwd_dense_short<S>), dim3(static_cast<unsigned>(ceil_div(width, kCeShortColumns))),
                       dim3(kCeThreads), 0, st, a);
    return launch_status();
  }
  const bool vec = !use_labels && ce_vec_ok(height, width, prediction, ld_prediction, VE) &&
                   ce_vec_ok(height, width, ground_truth, ld_ground_truth, VE);
  // columns off the 16-byte grid: 16-byte accesses at the alignment of one entry
  const bool unal = !use_labels && !vec && height >= 4 * VE;
  const int64_t units = use_labels ? (spatial_size < height ? spatial_size : height)
                                   : ((vec || unal) ? height / VE : height);
  // 1024-thread workgroups when that fills the device with one workgroup per column: no
  // partial sums to merge, so no second kernel
  const bool big = !use_labels && units >= 4 * 1024 && width >= 256;
  const int P = ce_parts(width, units, big ? 1024 : kCeThreads);
  if (P > 1 && (!workspace || workspace_bytes < static_cast<size_t>(width) * P * sizeof(float) ||
                (reinterpret_cast<uintptr_t>(workspace) & 3u)))
    return LBN_ERR_WORKSPACE;
  const dim3 grid(static_cast<unsigned>(width), static_cast<unsigned>(P));
  if (use_labels) hipLaunchKernelGGL((ce_fwd_labels<S>), grid, dim3(kCeThreads), 0, st, a);
  else if (vec && big) hipLaunchKernelGGL((ce_fwd_dense<kCeVec, 1024, S>), grid, dim3(1024), 0, st, a);
  else if (vec) hipLaunchKernelGGL((ce_fwd_dense<kCeVec, kCeThreads, S>), grid, dim3(kCeThreads), 0, st, a);
  else if (unal && big) hipLaunchKernelGGL((ce_fwd_dense<kCeUnaligned, 1024, S>), grid, dim3(1024), 0, st, a);
  else if (unal) hipLaunchKernelGGL((ce_fwd_dense<kCeUnaligned, kCeThreads, S>), grid, dim3(kCeThreads), 0, st, a);
  else if (big) hipLaunchKernelGGL((ce_fwd_dense<kCeScalar, 1024, S>), grid, dim3(1024), 0, st, a);
  else hipLaunchKernelGGL((ce_fwd_dense<kCeScalar, kCeThreads, S>), grid, dim3(kCeThreads), 0, st, a);
  if (P > 1)
    hipLaunchKernelGGL((ce_merge_parts<S>), dim3(static_cast<unsigned>(width)), dim3(kWave), 0, st, P, a.part, loss,
                       ld_loss);
  return launch_status();
}

template <typename S>
static int ce_bwd_impl(lbn_stream_t stream, int64_t height, int64_t width, int use_labels, int64_t spatial_size,
                       const S* prediction, int64_t ld_prediction, const S* ground_truth, int64_t ld_ground_truth,
                       const S* dloss, int64_t ld_dloss, S* dprediction, int64_t ld_dprediction, S* dground_truth,
                       int64_t ld_dground_truth)
{
  constexpr int VE = Vec16<S>::N;
  if (int e = ce_check(height, width, use_labels, spatial_size, ld_prediction, ld_ground_truth)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!prediction || !ground_truth || !dloss || !dprediction || ld_dloss < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (width > 1 && ld_dprediction < height) return LBN_ERR_INVALID_ARGUMENT;
  if (!use_labels && dground_truth && width > 1 && ld_dground_truth < height) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  CeArgs<S> a{};
  a.h = height, a.w = width, a.spatial = use_labels ? spatial_size : 1;
  a.x = prediction, a.truth = ground_truth, a.ldx = ld_prediction, a.ldt = ld_ground_truth;
  a.dy = dloss, a.lddy = ld_dloss, a.dx = dprediction, a.lddx = ld_dprediction;
  a.dtruth = dground_truth, a.lddt = ld_dground_truth;
  if (!use_labels && height <= kCeShortMax && width >= 4096) {
    hipLaunchKernelGGL((ce_bwd_dense_short<S>), dim3(static_cast<unsigned>(ceil_div(width, kCeShortColumns))),
                       dim3(kCeThreads), 0, st, a);
    return launch_status();
  }
  bool vec = ce_vec_ok(height, width, prediction, ld_prediction, VE) &&
             ce_vec_ok(height, width, dprediction, ld_dprediction, VE);
  if (use_labels)
    vec = vec && spatial_size % VE == 0 && aligned16(ground_truth) && (width <= 1 || ld_ground_truth % VE == 0);
  else
    vec = vec && ce_vec_ok(height, width, ground_truth, ld_ground_truth, VE) &&
          ce_vec_ok(height, width, dground_truth, ld_dground_truth, VE);
  const bool unal = !use_labels && !vec && height >= 4 * VE;
  const int P = ce_parts(width, (vec || unal) ? height / VE : height, kCeThreads, kCeMaxPartsBwd);
  const dim3 grid(static_cast<unsigned>(width), static_cast<unsigned>(P));
  if (use_labels && spatial_size == 1 && height >= 4 * VE) {
    const int P1 = ce_parts(width, height / VE, kCeThreads, kCeMaxPartsBwd);
    if (P1 == 1 && width >= 4096)
      hipLaunchKernelGGL((ce_bwd_one_label_columns<S>), dim3(static_cast<unsigned>(ceil_div(width, kCeOneLabelColumns))),
                         dim3(kCeThreads), 0, st, a);
    else
      hipLaunchKernelGGL((ce_bwd_one_label<S>), dim3(static_cast<unsigned>(width), static_cast<unsigned>(P1)),
                         dim3(kCeThreads), 0, st, a);
  }
  else if (use_labels) {
    if (vec) hipLaunchKernelGGL((ce_bwd_labels<true, S>), grid, dim3(kCeThreads), 0, st, a);
    else hipLaunchKernelGGL((ce_bwd_labels<false, S>), grid, dim3(kCeThreads), 0, st, a);
  }
  else {
    if (vec) hipLaunchKernelGGL((ce_bwd_dense<kCeVec, S>), grid, dim3(kCeThreads), 0, st, a);
    else if (unal) hipLaunchKernelGGL((ce_bwd_dense<kCeUnaligned, S>), grid, dim3(kCeThreads), 0, st, a);
    else hipLaunchKernelGGL((ce_bwd_dense<kCeScalar, S>), grid, dim3(kCeThreads), 0, st, a);
  }
  return launch_status();
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_cross_entropy_fwd_workspace_bytes(int64_t height, int64_t width)
{
  if (height <= 0 || width <= 0) return 0;
  return static_cast<size_t>(width) * ce_parts_bound(width) * sizeof(float);
}

int lbn_cross_entropy_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size, const float* prediction, int64_t ld_prediction,
                              const float* ground_truth, int64_t ld_ground_truth, float* loss,
                              int64_t ld_loss, void* workspace, size_t workspace_bytes)
{
  return ce_fwd_impl<float>(stream, height, width, use_labels, spatial_size, prediction, ld_prediction, ground_truth,
                            ld_ground_truth, loss, ld_loss, workspace, workspace_bytes);
}

int lbn_cross_entropy_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size, const float* prediction, int64_t ld_prediction,
                              const float* ground_truth, int64_t ld_ground_truth, const float* dloss,
                              int64_t ld_dloss, float* dprediction, int64_t ld_dprediction,
                              float* dground_truth, int64_t ld_dground_truth)
{
  return ce_bwd_impl<float>(stream, height, width, use_labels, spatial_size, prediction, ld_prediction, ground_truth,
                            ld_ground_truth, dloss, ld_dloss, dprediction, ld_dprediction, dground_truth,
                            ld_dground_truth);
}

int lbn_cross_entropy_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size, const void* prediction, int64_t ld_prediction,
                              const void* ground_truth, int64_t ld_ground_truth, void* loss, int64_t ld_loss,
                              void* workspace, size_t workspace_bytes)
{
  if ((reinterpret_cast<uintptr_t>(prediction) | reinterpret_cast<uintptr_t>(ground_truth) |
       reinterpret_cast<uintptr_t>(loss)) & 1u)
    return LBN_ERR_INVALID_ARGUMENT;
  return ce_fwd_impl<__half>(stream, height, width, use_labels, spatial_size, static_cast<const __half*>(prediction),
                             ld_prediction, static_cast<const __half*>(ground_truth), ld_ground_truth,
                             static_cast<__half*>(loss), ld_loss, workspace, workspace_bytes);
}

int lbn_cross_entropy_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                              int64_t spatial_size, const void* prediction, int64_t ld_prediction,
                              const void* ground_truth, int64_t ld_ground_truth, const void* dloss,
                              int64_t ld_dloss, void* dprediction, int64_t ld_dprediction, void* dground_truth,
                              int64_t ld_dground_truth)
{
  if ((reinterpret_cast<uintptr_t>(prediction) | reinterpret_cast<uintptr_t>(ground_truth) |
       reinterpret_cast<uintptr_t>(dloss) | reinterpret_cast<uintptr_t>(dprediction) |
       reinterpret_cast<uintptr_t>(dground_truth)) & 1u)
    return LBN_ERR_INVALID_ARGUMENT;
  return ce_bwd_impl<__half>(stream, height, width, use_labels, spatial_size, static_cast<const __half*>(prediction),
                             ld_prediction, static_cast<const __half*>(ground_truth), ld_ground_truth,
                             static_cast<const __half*>(dloss), ld_dloss, static_cast<__half*>(dprediction),
                             ld_dprediction, static_cast<__half*>(dground_truth), ld_dground_truth);
}

}  // extern "C"
