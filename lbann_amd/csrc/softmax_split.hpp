// Softmax family: the split ("chunked") kernels for rows that no register kernel takes, and the
// one-workgroup-per-row kernels for fp16 rows beyond the register kernels.  Included by softmax.hip.
#pragma once

#include "softmax_rows.hpp"

namespace lbn {

// ================================================================ split rows
// Block b handles chunk (b % S) of row (b / S); 256 threads per block.
constexpr int kChunkThreads = 256;
constexpr int kChunkUnroll = 4;

// Merges the online-softmax pairs (m, acc) of the 256 threads; every thread gets the result.
__device__ __forceinline__ void block_merge_max_sum(float& m, float& acc, float (*slot)[2])
{
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const float wm = wave_max(m);
  acc = wave_sum(acc * exp_fast(m - wm));
  if (lane == 0) {
    slot[wv][0] = wm;
    slot[wv][1] = acc;
  }
  __syncthreads();
  float bm = slot[0][0];
#pragma unroll
  for (int i = 1; i < kChunkThreads / kWave; ++i) bm = fmaxf(bm, slot[i][0]);
  float bs = 0.f;
#pragma unroll
  for (int i = 0; i < kChunkThreads / kWave; ++i) bs += slot[i][1] * exp_fast(slot[i][0] - bm);
  m = bm;
  acc = bs;
}

// A run of `len` floats at p, cut at 16-byte boundaries: `head` leading scalars, `nvec`
// aligned vectors, `tail` trailing scalars.  Rows whose starts are only 4-byte aligned
// (odd lengths, e.g. a vocabulary of 50257 entries) still move almost all of their bytes
// with 16-byte accesses this way.
struct Peel {
  int head, tail;
  int64_t nvec;
  // index (relative to p) of the edge scalar thread t handles, for t < head + tail
  __device__ __forceinline__ int64_t edge(int t) const { return t < head ? t : head + 4 * nvec + (t - head); }
};

__device__ __forceinline__ Peel peel16(const float* p, int64_t len)
{
  Peel r;
  r.head = static_cast<int>((4 - ((reinterpret_cast<uintptr_t>(p) >> 2) & 3)) & 3);
  if (r.head > len) r.head = static_cast<int>(len);
  r.nvec = (len - r.head) / 4;
  r.tail = static_cast<int>(len - r.head - 4 * r.nvec);
  return r;
}

__device__ __forceinline__ bool same_phase16(const void* a, const void* b)
{
  return ((reinterpret_cast<uintptr_t>(a) ^ reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
}

// Online (max, sum of exp) over nvec aligned vectors at base, strided over the workgroup;
// four independent 16-byte loads per thread are in flight before any is used.
__device__ __forceinline__ void sm_reduce_vectors(const float* base, int64_t nvec, float& m, float& acc)
{
  for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += kChunkUnroll * kChunkThreads) {
    float v[kChunkUnroll][4];
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int64_t i = i0 + u * kChunkThreads;
      if (i < nvec) {
        Vec16<float>::load(base + 4 * i, v[u]);
      }
      else {
#pragma unroll
        for (int k = 0; k < 4; ++k) v[u][k] = -FLT_MAX;
      }
    }
    float mn = m;
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u)
#pragma unroll
      for (int k = 0; k < 4; ++k) mn = fmaxf(mn, v[u][k]);
    float add = 0.f;
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const bool ok = i0 + u * kChunkThreads < nvec;
#pragma unroll
      for (int k = 0; k < 4; ++k) add += ok ? exp_fast(v[u][k] - mn) : 0.f;
    }
    acc = acc * exp_fast(m - mn) + add;
    m = mn;
  }
}

template <bool VEC>
__global__ void __launch_bounds__(kChunkThreads)
sm_fwd_partial(const float* x, int64_t ldx, RowMap map, int64_t n, int64_t chunk, int S,
               float2* part)
{
  __shared__ float slot[kChunkThreads / kWave][2];
  const int64_t row = blockIdx.x / S;
  const int s = blockIdx.x - row * S;
  const int64_t begin = s * chunk;
  const int64_t end = imin64(n, begin + chunk);
  const float* p = x + map.offset(row, ldx) + begin;
  float m = -FLT_MAX, acc = 0.f;
  if (VEC) {
    sm_reduce_vectors(p, (end - begin) / 4, m, acc);
  }
  else {
    const Peel pl = peel16(p, end - begin);
    if (static_cast<int>(threadIdx.x) < pl.head + pl.tail) {
      m = p[pl.edge(threadIdx.x)];
      acc = 1.f;
    }
    sm_reduce_vectors(p + pl.head, pl.nvec, m, acc);
  }
  block_merge_max_sum(m, acc, slot);
  if (threadIdx.x == 0) part[blockIdx.x] = make_float2(m, acc);
}

// out[i] = f(in[i]) over nvec aligned vectors, strided over the workgroup.
template <typename F>
__device__ __forceinline__ void sm_map_vectors(const float* in, float* out, int64_t nvec, F f)
{
  for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += kChunkUnroll * kChunkThreads) {
    float v[kChunkUnroll][4];
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int64_t i = i0 + u * kChunkThreads;
      if (i < nvec) Vec16<float>::load(in + 4 * i, v[u]);
    }
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int64_t i = i0 + u * kChunkThreads;
      if (i < nvec) {
#pragma unroll
        for (int k = 0; k < 4; ++k) v[u][k] = f(v[u][k]);
        Vec16<float>::store(out + 4 * i, v[u]);
      }
    }
  }
}

template <bool VEC, int KIND>
__global__ void __launch_bounds__(kChunkThreads)
sm_fwd_apply(const float* x, float* y, int64_t ldx, int64_t ldy, RowMap map, int64_t n,
             int64_t chunk, int S, const float2* part)
{
  const int64_t row = blockIdx.x / S;
  const int s = blockIdx.x - row * S;
  const int64_t begin = s * chunk;
  const int64_t end = imin64(n, begin + chunk);
  const int lane = threadIdx.x & (kWave - 1);
  // every wave merges the S <= 64 partials of the row on its own
  float pm = -FLT_MAX, ps = 0.f;
  if (lane < S) {
    const float2 p = part[row * S + lane];
    pm = p.x;
    ps = p.y;
  }
  const float m = wave_max(pm);
  const float sum = wave_sum(ps * exp_fast(pm - m));
  const float scale = 1.0f / sum;
  const float lse = (KIND == kLogSoftmax) ? log_of_sum(sum) : 0.f;
  const float* xp = x + map.offset(row, ldx) + begin;
  float* yp = y + map.offset(row, ldy) + begin;
  const int64_t len = end - begin;
  auto f = [&](float v) -> float {
    const float d = v - m;
    if (KIND == kLogSoftmax) return d - lse;
    const float r = scale * (KIND == kChannelwise ? exp_keep_denormals(d) : exp_fast(d));
    if (KIND == kSoftmax) return __builtin_isnormal(r) ? r : 0.f;
    return r;
  };
  if (VEC) {
    sm_map_vectors(xp, yp, len / 4, f);
  }
  else if (same_phase16(xp, yp)) {
    const Peel pl = peel16(xp, len);
    if (static_cast<int>(threadIdx.x) < pl.head + pl.tail) {
      const int64_t e = pl.edge(threadIdx.x);
      yp[e] = f(xp[e]);
    }
    sm_map_vectors(xp + pl.head, yp + pl.head, pl.nvec, f);
  }
  else {
    for (int64_t i = threadIdx.x; i < len; i += kChunkThreads) yp[i] = f(xp[i]);
  }
}

// sum of dy (log-softmax) or of y * dy over nvec aligned vectors, strided over the workgroup.
template <int KIND>
__device__ __forceinline__ float sm_dot_vectors(const float* yb, const float* gb, int64_t nvec)
{
  float acc = 0.f;
  for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += kChunkUnroll * kChunkThreads) {
    float a[kChunkUnroll][4], g[kChunkUnroll][4];
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int64_t i = i0 + u * kChunkThreads;
#pragma unroll
      for (int k = 0; k < 4; ++k) a[u][k] = g[u][k] = 0.f;
      if (i < nvec) {
        Vec16<float>::load(gb + 4 * i, g[u]);
        if (KIND != kLogSoftmax) Vec16<float>::load(yb + 4 * i, a[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      if (KIND == kLogSoftmax) acc += (g[u][0] + g[u][1]) + (g[u][2] + g[u][3]);
      else acc += (a[u][0] * g[u][0] + a[u][1] * g[u][1]) + (a[u][2] * g[u][2] + a[u][3] * g[u][3]);
    }
  }
  return acc;
}

template <bool VEC, int KIND>
__global__ void __launch_bounds__(kChunkThreads)
sm_bwd_partial(const float* y, const float* dy, int64_t ldy, int64_t lddy, RowMap map, int64_t n,
               int64_t chunk, int S, float* part)
{
  __shared__ float slot[kChunkThreads / kWave];
  const int64_t row = blockIdx.x / S;
  const int s = blockIdx.x - row * S;
  const int64_t begin = s * chunk;
  const int64_t end = imin64(n, begin + chunk);
  const float* yp = y + map.offset(row, ldy) + begin;
  const float* gp = dy + map.offset(row, lddy) + begin;
  const int64_t len = end - begin;
  float acc = 0.f;
  if (VEC) {
    acc = sm_dot_vectors<KIND>(yp, gp, len / 4);
  }
  else if (same_phase16(yp, gp)) {
    const Peel pl = peel16(gp, len);
    acc = sm_dot_vectors<KIND>(yp + pl.head, gp + pl.head, pl.nvec);
    if (static_cast<int>(threadIdx.x) < pl.head + pl.tail) {
      const int64_t e = pl.edge(threadIdx.x);
      acc += (KIND == kLogSoftmax) ? gp[e] : yp[e] * gp[e];
    }
  }
  else {
    for (int64_t i = threadIdx.x; i < len; i += kChunkThreads)
      acc += (KIND == kLogSoftmax) ? gp[i] : yp[i] * gp[i];
  }
  acc = team_sum<kChunkThreads / kWave>(acc, slot, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) part[blockIdx.x] = acc;
}

// out[i] = f(a[i], g[i]) over nvec aligned vectors, strided over the workgroup.
template <typename F>
__device__ __forceinline__ void sm_map2_vectors(const float* ab, const float* gb, float* out, int64_t nvec, F f)
{
  for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += kChunkUnroll * kChunkThreads) {
    float a[kChunkUnroll][4], g[kChunkUnroll][4];
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int64_t i = i0 + u * kChunkThreads;
      if (i < nvec) {
        Vec16<float>::load(ab + 4 * i, a[u]);
        Vec16<float>::load(gb + 4 * i, g[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int64_t i = i0 + u * kChunkThreads;
      if (i < nvec) {
#pragma unroll
        for (int k = 0; k < 4; ++k) g[u][k] = f(a[u][k], g[u][k]);
        Vec16<float>::store(out + 4 * i, g[u]);
      }
    }
  }
}

template <bool VEC, int KIND>
__global__ void __launch_bounds__(kChunkThreads)
sm_bwd_apply(const float* y, const float* dy, float* dx, int64_t ldy, int64_t lddy, int64_t lddx,
             RowMap map, int64_t n, int64_t chunk, int S, const float* part)
{
  const int64_t row = blockIdx.x / S;
  const int s = blockIdx.x - row * S;
  const int64_t begin = s * chunk;
  const int64_t end = imin64(n, begin + chunk);
  const int lane = threadIdx.x & (kWave - 1);
  const float sum = wave_sum(lane < S ? part[row * S + lane] : 0.f);
  const float* yp = y + map.offset(row, ldy) + begin;
  const float* gp = dy + map.offset(row, lddy) + begin;
  float* dp = dx + map.offset(row, lddx) + begin;
  const int64_t len = end - begin;
  auto f = [&](float a, float g) -> float {
    return (KIND == kLogSoftmax) ? g - exp_fast(a) * sum : a * (g - sum);
  };
  if (VEC) {
    sm_map2_vectors(yp, gp, dp, len / 4, f);
  }
  else if (same_phase16(yp, gp) && same_phase16(yp, dp)) {
    const Peel pl = peel16(yp, len);
    if (static_cast<int>(threadIdx.x) < pl.head + pl.tail) {
      const int64_t e = pl.edge(threadIdx.x);
      dp[e] = f(yp[e], gp[e]);
    }
    sm_map2_vectors(yp + pl.head, gp + pl.head, dp + pl.head, pl.nvec, f);
  }
  else {
    for (int64_t i = threadIdx.x; i < len; i += kChunkThreads) dp[i] = f(yp[i], gp[i]);
  }
}

// ============================================= fp16 rows beyond the register kernels
// One 256-thread workgroup per row, element-wise access, fp32 arithmetic: maximum, sum of
// exponentials, output (the input is read three times; rows this long in fp16 storage are
// rare, so this is the complete-coverage path, not a tuned one).
template <typename S, int KIND>
__global__ void __launch_bounds__(kChunkThreads)
sm_fwd_generic(const S* x, S* y, int64_t ldx, int64_t ldy, RowMap map, int64_t n)
{
  __shared__ float red[kChunkThreads / kWave];
  const int64_t row = blockIdx.x;
  const S* xr = x + map.offset(row, ldx);
  S* yr = y + map.offset(row, ldy);
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  float m = -FLT_MAX;
  for (int64_t i = threadIdx.x; i < n; i += kChunkThreads) m = fmaxf(m, RowLoad<S>::get(xr + i));
  m = team_max<kChunkThreads / kWave>(m, red, wv, lane);
  __syncthreads();
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += kChunkThreads) s += exp_fast(RowLoad<S>::get(xr + i) - m);
  s = team_sum<kChunkThreads / kWave>(s, red, wv, lane);
  const float f = 1.0f / s;
  const float lse = (KIND == kLogSoftmax) ? log_of_sum(s) : 0.f;
  for (int64_t i = threadIdx.x; i < n; i += kChunkThreads) {
    const float d = RowLoad<S>::get(xr + i) - m;
    float r;
    if (KIND == kLogSoftmax) {
      r = d - lse;
    }
    else {
      r = f * exp_fast(d);
      r = __builtin_isnormal(r) ? r : 0.f;
    }
    RowLoad<S>::put(yr + i, r);
  }
}

template <typename S, int KIND>
__global__ void __launch_bounds__(kChunkThreads)
sm_bwd_generic(const S* y, const S* dy, S* dx, int64_t ldy, int64_t lddy, int64_t lddx, RowMap map, int64_t n)
{
  __shared__ float red[kChunkThreads / kWave];
  const int64_t row = blockIdx.x;
  const S* yr = y + map.offset(row, ldy);
  const S* gr = dy + map.offset(row, lddy);
  S* dr = dx + map.offset(row, lddx);
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += kChunkThreads)
    s += (KIND == kLogSoftmax) ? RowLoad<S>::get(gr + i) : RowLoad<S>::get(yr + i) * RowLoad<S>::get(gr + i);
  s = team_sum<kChunkThreads / kWave>(s, red, wv, lane);
  // in place (dx aliasing dy): element i is read and written by the same thread, after the sum
  for (int64_t i = threadIdx.x; i < n; i += kChunkThreads) {
    const float a = RowLoad<S>::get(yr + i), g = RowLoad<S>::get(gr + i);
    RowLoad<S>::put(dr + i, (KIND == kLogSoftmax) ? g - exp_fast(a) * s : a * (g - s));
  }
}

// The same rows in packed 16-byte accesses: one 1024-thread workgroup per row, two passes.  The
// first takes the maximum and the sum of exponentials together (a thread rescales its sum when
// its maximum rises), the second writes the output; it finds the row in the last-level caches,
// so the input crosses HBM once.  16-bit storage: the two-operation exponential (sm_fwd_rows).
// FR: rows that start off the 16-byte grid (a vocabulary of 50257 entries) are cut per row into
// up to 7 leading entries, aligned vectors and up to 7 trailing entries; every tensor of the call
// starts each row at the same distance from a 16-byte boundary (checked on the host).
constexpr int kLongThreads = 1024;
constexpr int kLongUnroll = 4;

// The cut of one row of n 16-bit entries at p.
struct PackedRowCut {
  unsigned head, nvec, tail;
  // Entry handled by thread t < head + tail as a single value.
  __device__ __forceinline__ int64_t edge(unsigned t) const
  {
    return t < head ? t : static_cast<int64_t>(head) + 8 * static_cast<int64_t>(nvec) + (t - head);
  }
};

template <bool FR>
__device__ __forceinline__ PackedRowCut packed_row_cut(const void* p, int64_t n)
{
  if (!FR) return {0u, static_cast<unsigned>(n / 8), 0u};
  const unsigned shift = static_cast<unsigned>(reinterpret_cast<uintptr_t>(p) & 15u) / 2;
  unsigned head = (8 - shift) & 7;
  if (head > n) head = static_cast<unsigned>(n);
  const unsigned nvec = static_cast<unsigned>((n - head) / 8);
  return {head, nvec, static_cast<unsigned>(n - head - 8 * static_cast<int64_t>(nvec))};
}

template <typename S, int KIND, bool FR>
__global__ void __launch_bounds__(kLongThreads)
sm_fwd_long_packed(const S* x, S* y, int64_t ldx, int64_t ldy, RowMap map, int64_t n)
{
  static_assert(sizeof(S) == 2, "packed 16-bit rows");
  constexpr int W = Vec16<S>::N, NW = kLongThreads / kWave, U = kLongUnroll;
  static_assert(W == 8, "eight entries per vector");
  using raw_t = typename Vec16<S>::raw_t;
  __shared__ float red[2][NW];
  const int64_t row = blockIdx.x;
  const S* xr = x + map.offset(row, ldx);
  S* yr = y + map.offset(row, ldy);
  const PackedRowCut cut = packed_row_cut<FR>(xr, n);
  const S* xv = xr + cut.head;
  S* yv = yr + cut.head;
  const unsigned nvec = cut.nvec;
  const unsigned t = threadIdx.x;
  const int lane = t & (kWave - 1), wv = t / kWave;
  float m = -FLT_MAX, s = 0.f;
  const bool edge = FR && t < cut.head + cut.tail;
  float ev = 0.f;
  if (edge) {
    ev = Vec16<S>::load1(xr + cut.edge(t));
    m = fmaxf(m, ev);
    s = exp_quick(ev - m);
  }
  for (unsigned i0 = t; i0 < nvec; i0 += U * kLongThreads) {
    raw_t r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned idx = i0 + u * kLongThreads;
      r[u] = raw_t{};
      if (idx < nvec) r[u] = Vec16<S>::load_raw(xv + static_cast<int64_t>(W) * idx);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (i0 + u * kLongThreads >= nvec) continue;
      float v[W];
      Vec16<S>::unpack(r[u], v);
      float vm = v[0];
#pragma unroll
      for (int k = 1; k < W; ++k) vm = fmaxf(vm, v[k]);
      if (vm > m) {
        s *= exp_quick(m - vm);
        m = vm;
      }
#pragma unroll
      for (int k = 0; k < W; ++k) s += exp_quick(v[k] - m);
    }
  }
  float gm = wave_max(m);
  float gs = wave_sum(s * exp_fast(m - gm));
  if (lane == 0) {
    red[0][wv] = gm;
    red[1][wv] = gs;
  }
  __syncthreads();
  const float pm = lane < NW ? red[0][lane] : -FLT_MAX;
  const float ps = lane < NW ? red[1][lane] : 0.f;
  gm = wave_max(pm);
  gs = wave_sum(ps * exp_fast(pm - gm));
  const float f = 1.0f / gs;
  const float lse = (KIND == kLogSoftmax) ? log_of_sum(gs) : 0.f;
  auto result = [&](float v) {
    const float d = v - gm;
    if (KIND == kLogSoftmax) return d - lse;
    const float e = f * exp_quick(d);
    return __builtin_isnormal(e) ? e : 0.f;
  };
  // in place: a thread writes what it has read itself, and every read of the first pass lies
  // before the barrier above
  if (edge) Vec16<S>::store1(yr + cut.edge(t), result(ev));
  for (unsigned i0 = t; i0 < nvec; i0 += U * kLongThreads) {
    raw_t r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned idx = i0 + u * kLongThreads;
      r[u] = raw_t{};
      if (idx < nvec) r[u] = Vec16<S>::load_raw(xv + static_cast<int64_t>(W) * idx);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned idx = i0 + u * kLongThreads;
      if (idx >= nvec) continue;
      float v[W];
      Vec16<S>::unpack(r[u], v);
#pragma unroll
      for (int k = 0; k < W; ++k) v[k] = result(v[k]);
      Vec16<S>::store(yv + static_cast<int64_t>(W) * idx, v);
    }
  }
}

template <typename S, int KIND, bool FR>
__global__ void __launch_bounds__(kLongThreads)
sm_bwd_long_packed(const S* y, const S* dy, S* dx, int64_t ldy, int64_t lddy, int64_t lddx, RowMap map, int64_t n)
{
  static_assert(sizeof(S) == 2, "packed 16-bit rows");
  constexpr int W = Vec16<S>::N, NW = kLongThreads / kWave, U = kLongUnroll / 2;
  static_assert(W == 8, "eight entries per vector");
  using raw_t = typename Vec16<S>::raw_t;
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const S* yr = y + map.offset(row, ldy);
  const S* gr = dy + map.offset(row, lddy);
  S* dr = dx + map.offset(row, lddx);
  const PackedRowCut cut = packed_row_cut<FR>(yr, n);
  const S* yv = yr + cut.head;
  const S* gv = gr + cut.head;
  S* dv = dr + cut.head;
  const unsigned nvec = cut.nvec;
  const unsigned t = threadIdx.x;
  const int lane = t & (kWave - 1), wv = t / kWave;
  const bool edge = FR && t < cut.head + cut.tail;
  float ea = 0.f, eg = 0.f, s = 0.f;
  if (edge) {
    ea = Vec16<S>::load1(yr + cut.edge(t));
    eg = Vec16<S>::load1(gr + cut.edge(t));
    s = (KIND == kLogSoftmax) ? eg : ea * eg;
  }
  for (unsigned i0 = t; i0 < nvec; i0 += U * kLongThreads) {
    raw_t ra[U], rg[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned idx = i0 + u * kLongThreads;
      ra[u] = raw_t{};
      rg[u] = raw_t{};
      if (idx < nvec) {
        if (KIND != kLogSoftmax) ra[u] = Vec16<S>::load_raw(yv + static_cast<int64_t>(W) * idx);
        rg[u] = Vec16<S>::load_raw(gv + static_cast<int64_t>(W) * idx);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float a[W], g[W];  // vectors past the end hold zeros
      Vec16<S>::unpack(ra[u], a);
      Vec16<S>::unpack(rg[u], g);
#pragma unroll
      for (int k = 0; k < W; ++k) s += (KIND == kLogSoftmax) ? g[k] : a[k] * g[k];
    }
  }
  s = team_sum<NW>(s, red, wv, lane);
  auto result = [&](float a, float g) { return (KIND == kLogSoftmax) ? g - exp_quick(a) * s : a * (g - s); };
  // in place (dx aliasing dy or y): a thread writes what it has read itself, after the sum
  if (edge) Vec16<S>::store1(dr + cut.edge(t), result(ea, eg));
  for (unsigned i0 = t; i0 < nvec; i0 += U * kLongThreads) {
    raw_t ra[U], rg[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned idx = i0 + u * kLongThreads;
      ra[u] = raw_t{};
      rg[u] = raw_t{};
      if (idx < nvec) {
        ra[u] = Vec16<S>::load_raw(yv + static_cast<int64_t>(W) * idx);
        rg[u] = Vec16<S>::load_raw(gv + static_cast<int64_t>(W) * idx);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned idx = i0 + u * kLongThreads;
      if (idx >= nvec) continue;
      float a[W], g[W];
      Vec16<S>::unpack(ra[u], a);
      Vec16<S>::unpack(rg[u], g);
#pragma unroll
      for (int k = 0; k < W; ++k) g[k] = result(a[k], g[k]);
      Vec16<S>::store(dv + static_cast<int64_t>(W) * idx, g);
    }
  }
}

}  // namespace lbn
