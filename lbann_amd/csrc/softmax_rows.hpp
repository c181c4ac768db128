// Softmax family: the register-resident row kernels (one team of threads owns a row).
// Included by softmax.hip, whose header comment describes the three kernel families.
#pragma once

#include <type_traits>

#include "device_utils.hpp"

namespace lbn {


enum SmKind : int { kSoftmax = 0, kLogSoftmax = 1, kChannelwise = 2 };

constexpr int kMaxChunks = 64;  // S <= one wave, so a wave merges the partials of a row

// ======================================================= register-resident rows
// Access unit of the row kernels: W = 4 is a 16-byte vector (rows start on 16-byte
// boundaries and their length is a multiple of 4), W = 1 a single float for rows that are
// only 4-byte aligned (odd lengths such as 197 or 1001): a wave instruction then still
// reads 256 contiguous bytes.
template <typename S, int W>
struct RowIO;
template <>
struct RowIO<float, 4> {
  template <bool STREAM>
  static __device__ __forceinline__ void load(const float* p, float (&v)[4])
  {
    if (STREAM) Vec16<float>::load_stream(p, v);
    else Vec16<float>::load(p, v);
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { Vec16<float>::store(p, v); }
};
template <>
struct RowIO<float, 1> {
  template <bool STREAM>
  static __device__ __forceinline__ void load(const float* p, float (&v)[1])
  {
    v[0] = *p;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[1]) { *p = v[0]; }
};
// fp16 storage: 16-byte vectors of eight halves, or single halves for rows off the 16-byte
// grid; values are widened to fp32 on load and rounded to nearest even on store.
template <>
struct RowIO<__half, 8> {
  template <bool STREAM>
  static __device__ __forceinline__ void load(const __half* p, float (&v)[8])
  {
    Vec16<__half>::load(p, v);
  }
  static __device__ __forceinline__ void store(__half* p, const float (&v)[8]) { Vec16<__half>::store(p, v); }
};
template <>
struct RowIO<__half, 1> {
  template <bool STREAM>
  static __device__ __forceinline__ void load(const __half* p, float (&v)[1])
  {
    v[0] = __half2float(*p);
  }
  static __device__ __forceinline__ void store(__half* p, const float (&v)[1]) { *p = __float2half_rn(v[0]); }
};

// 16-byte accesses at the alignment of one entry (rows off the 16-byte grid); the hardware
// takes them at 93-95 % of the aligned rate.
template <typename S, int W>
struct RowIOUnaligned;
template <>
struct RowIOUnaligned<__half, 8> {
  static __device__ __forceinline__ void load(const __half* p, float (&v)[8])
  {
    Vec16<f16u>::load(reinterpret_cast<const f16u*>(p), v);
  }
  static __device__ __forceinline__ void store(__half* p, const float (&v)[8])
  {
    Vec16<f16u>::store(reinterpret_cast<f16u*>(p), v);
  }
};

template <>
struct RowIOUnaligned<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) { __builtin_memcpy(v, p, 16); }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { __builtin_memcpy(p, v, 16); }
};

template <typename S>
struct RowLoad {
  static __device__ __forceinline__ float get(const S* p) { float v[1]; RowIO<S, 1>::template load<false>(p, v); return v[0]; }
  static __device__ __forceinline__ void put(S* p, float r) { const float v[1] = {r}; RowIO<S, 1>::store(p, v); }
};

// Framed access: a row that starts off the 16-byte grid, addressed on it.  The frame begins at
// the 16-byte boundary at or below the row's first entry, `shift` (0..3) entries earlier;
// vector idx of the frame holds the row's entries 4 idx - shift ... 4 idx + 3 - shift.  Vectors
// that lie inside the row move as 16 bytes; the first and the last move entry by entry, and
// what lies outside the row is neither read nor written.  Every tensor of a call must have the
// same shift in every row (same_frames() on the host).
struct RowFrame {
  unsigned shift;
  unsigned nvec;  // vectors of the frame that hold entries of the row
};

__device__ __forceinline__ RowFrame row_frame(const float* rowp, unsigned n)
{
  const unsigned shift = (static_cast<unsigned>(reinterpret_cast<uintptr_t>(rowp)) >> 2) & 3u;
  return {shift, (shift + n + 3u) >> 2};
}

__device__ __forceinline__ void frame_load(const float* framep, unsigned idx, RowFrame fr, unsigned n, float fill,
                                           float (&v)[4])
{
  const unsigned e0 = 4u * idx;
  if (e0 >= fr.shift && e0 + 4u <= fr.shift + n) {
    Vec16<float>::load(framep + e0, v);
  }
  else {
#pragma unroll
    for (unsigned j = 0; j < 4; ++j) v[j] = (e0 + j >= fr.shift && e0 + j < fr.shift + n) ? framep[e0 + j] : fill;
  }
}

__device__ __forceinline__ void frame_store(float* framep, unsigned idx, RowFrame fr, unsigned n, const float (&v)[4])
{
  const unsigned e0 = 4u * idx;
  if (e0 >= fr.shift && e0 + 4u <= fr.shift + n) {
    Vec16<float>::store(framep + e0, v);
  }
  else {
#pragma unroll
    for (unsigned j = 0; j < 4; ++j)
      if (e0 + j >= fr.shift && e0 + j < fr.shift + n) framep[e0 + j] = v[j];
  }
}

// 1024-thread blocks are held to 64 registers so that two of them share a compute unit
// (not those with 32 accesses or more than 32 values per thread, which would spill).
// FR (fp32): framed access for rows off the 16-byte grid; `nvec` is then the row length in entries.
// UA: rows off the 16-byte grid in 16-byte accesses at the alignment of one entry; `nvec` is
// the row length in entries (at least W).  A last, partial vector is read as the row's last W
// entries, so it overlaps its neighbour: the entries the two share count as absent in the partial
// vector and are stored by the neighbour only.
template <typename S, int TPR, int V, int KIND, bool STREAM, int W = 16 / sizeof(S), bool FR = false, bool UA = false>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads, (TPR == 1024 && V <= 16 && V * W <= 32 ? 8 : 1))
sm_fwd_rows(const S* x, S* y, int64_t ldx, int64_t ldy, RowMap map, int64_t rows,
            unsigned nvec)
{
  static_assert(!FR || (std::is_same<S, float>::value && W == 4), "frames are made of 16-byte fp32 vectors");
  static_assert(!UA || (!FR && W == 16 / sizeof(S)), "unaligned access moves whole 16-byte vectors");
  using B = RowBlock<TPR>;
  constexpr bool kSub = TPR < kWave;  // short rows: 16 lanes own a row, four rows per wave
  static_assert(!kSub || TPR == 16, "sub-wave teams are one DPP row wide");
  constexpr int NW = kSub ? 1 : B::kWavesPerTeam;
  __shared__ float red[2][NW];
  const unsigned tid = threadIdx.x;
  // a team is a whole number of waves (then its index is wave-uniform) or a DPP row
  const int team = kSub ? static_cast<int>(tid) / TPR : wave_index() / NW;
  const unsigned t = tid - team * TPR;  // unsigned: addresses become scalar base + 32-bit offset
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * B::kTeams + team;
  if (B::kTeams > 1 && row >= rows) return;  // whole waves leave; no barrier below in that case

  const S* xr = x + map.offset(row, ldx);
  const unsigned n = nvec;
  RowFrame fr{0, nvec};
  if constexpr (FR) {
    fr = row_frame(xr, n);
    xr -= fr.shift;
    nvec = fr.nvec;
  }
  unsigned ua_skip = 0;  // UA: leading entries of the last vector that belong to its neighbour
  if constexpr (UA) {
    nvec = (n + W - 1) / W;
    ua_skip = nvec * W - n;
  }
  // entry offset of vector idx, and how many of its leading entries are not its own
  auto ua_off = [&](unsigned idx) { return (UA && idx == nvec - 1) ? n - W : unsigned(W) * idx; };
  auto ua_foreign = [&](unsigned idx) { return (UA && idx == nvec - 1) ? ua_skip : 0u; };
  float v[V][W];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
      if constexpr (FR) frame_load(xr, idx, fr, n, -FLT_MAX, v[i]);
      else if constexpr (UA) {
        RowIOUnaligned<S, W>::load(xr + ua_off(idx), v[i]);
        const unsigned foreign = ua_foreign(idx);
#pragma unroll
        for (int k = 0; k < W; ++k)
          if (unsigned(k) < foreign) v[i][k] = -FLT_MAX;
      }
      else RowIO<S, W>::template load<STREAM>(xr + unsigned(W) * idx, v[i]);
    }
    else {
#pragma unroll
      for (int k = 0; k < W; ++k) v[i][k] = -FLT_MAX;
    }
  }

  // Thread-local pass first: every thread takes the maximum of its own entries and
  // exponentiates against it as soon as its own loads have landed, without waiting
  // for the rest of the row; the (max, sum) pairs are then merged wave -> team with
  // a single barrier, and each thread rescales by exp(own max - row max) / row sum.
  float m = -FLT_MAX;  // starts from the lowest finite float like the reference
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int k = 0; k < W; ++k) m = fmaxf(m, v[i][k]);

  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const bool in_row = (t + i * TPR) < nvec;
    const unsigned foreign = ua_foreign(t + i * TPR);
#pragma unroll
    for (int k = 0; k < W; ++k) {
      const bool ok = in_row && !(UA && unsigned(k) < foreign);
      const float d = v[i][k] - m;
      float e;
      if (KIND == kLogSoftmax) e = exp_quick(d);  // only summed: x stays in the registers for the output
      else if (KIND == kChannelwise) e = exp_keep_denormals(d);
      // 16-bit storage rounds the result to 11 bits: the two-operation exponential (relative
      // error |d| * 3e-8) is exact enough there, and the kernel is bound by these operations,
      // not by memory, once an entry is two bytes
      else if (sizeof(S) == 2) e = exp_quick(d);
      else e = exp_fast(d);
      e = ok ? e : 0.f;
      s += e;
      if (KIND != kLogSoftmax) v[i][k] = e;
    }
  }

  // wave merge on the DPP path, then one LDS hop across the waves of the team
  float gm = kSub ? row16_max(m) : wave_max(m);
  float gs = kSub ? row16_sum(s * exp_fast(m - gm)) : wave_sum(s * exp_fast(m - gm));
  if (NW > 1) {
    if (lane == 0) {
      red[0][wv] = gm;
      red[1][wv] = gs;
    }
    __syncthreads();
    const float pm = lane < NW ? red[0][lane] : -FLT_MAX;
    const float ps = lane < NW ? red[1][lane] : 0.f;
    gm = wave_max(pm);
    gs = wave_sum(ps * exp_fast(pm - gm));
  }

  S* yr = y + map.offset(row, ldy);
  if constexpr (FR) yr -= fr.shift;  // the same frames as x (same_frames() on the host)
  const float shift = m - gm;  // <= 0
  const float f = exp_fast(shift) * (1.0f / gs);
  const float lse = (KIND == kLogSoftmax) ? log_of_sum(gs) : 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        if (KIND == kSoftmax) {
          const float r = f * v[i][k];
          v[i][k] = __builtin_isnormal(r) ? r : 0.f;
        }
        else if (KIND == kLogSoftmax) {
          v[i][k] = (v[i][k] - gm) - lse;
        }
        else {
          v[i][k] *= f;
        }
      }
      if constexpr (FR) frame_store(yr, idx, fr, n, v[i]);
      else if constexpr (UA) {
        const unsigned foreign = ua_foreign(idx);
        if (foreign) {
#pragma unroll
          for (int k = 0; k < W; ++k)
            if (unsigned(k) >= foreign) RowLoad<S>::put(yr + ua_off(idx) + k, v[i][k]);
        }
        else {
          RowIOUnaligned<S, W>::store(yr + ua_off(idx), v[i]);
        }
      }
      else RowIO<S, W>::store(yr + unsigned(W) * idx, v[i]);
    }
  }
}

// Forward over 16-bit rows of 1024 threads: with two bytes per entry the exponentials, not the
// memory, are what a compute unit spends its time on, and two workgroups that load, compute and
// store in step leave the memory idle while they compute.  Here one workgroup per compute unit
// walks rows b, b + grid, ...: the next row's packed vectors (16 bytes for 8 entries, so a
// second row costs few registers) are requested before the current row is unpacked, arrive while
// it is exponentiated, and its stores overlap the next row's arithmetic.
template <typename S, int V, int KIND>
__global__ void __launch_bounds__(1024)
sm_fwd_rows_walk(const S* x, S* y, int64_t ldx, int64_t ldy, RowMap map, int64_t rows, unsigned nvec)
{
  static_assert(sizeof(S) == 2, "packed 16-bit rows");
  constexpr int TPR = 1024, W = Vec16<S>::N, NW = TPR / kWave;
  using raw_t = typename Vec16<S>::raw_t;
  __shared__ float red[2][2][NW];
  const unsigned t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wv = wave_index();
  raw_t nx[V];
  auto request = [&](int64_t row) {
    const S* xr = x + map.offset(row, ldx);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      nx[i] = raw_t{};
      if (idx < nvec) nx[i] = Vec16<S>::load_raw(xr + unsigned(W) * idx);
    }
  };
  int64_t row = blockIdx.x;
  if (row >= rows) return;
  request(row);
  for (int it = 0; row < rows; row += gridDim.x, ++it) {
    float v[V][W];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      Vec16<S>::unpack(nx[i], v[i]);
      if (t + i * TPR >= nvec) {
#pragma unroll
        for (int k = 0; k < W; ++k) v[i][k] = -FLT_MAX;
      }
    }
    const int64_t next = row + gridDim.x;
    if (next < rows) request(next);
    asm volatile("" ::: "memory");  // the next row's loads go out ahead of this row's arithmetic

    float m = -FLT_MAX;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < W; ++k) m = fmaxf(m, v[i][k]);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const bool ok = (t + i * TPR) < nvec;
#pragma unroll
      for (int k = 0; k < W; ++k) {
        float e = exp_quick(v[i][k] - m);
        e = ok ? e : 0.f;
        s += e;
        if (KIND != kLogSoftmax) v[i][k] = e;
      }
    }
    float gm = wave_max(m);
    float gs = wave_sum(s * exp_fast(m - gm));
    float (&rd)[2][NW] = red[it & 1];  // the next row writes the other pair: one barrier per row
    if (lane == 0) {
      rd[0][wv] = gm;
      rd[1][wv] = gs;
    }
    __syncthreads();
    const float pm = lane < NW ? rd[0][lane] : -FLT_MAX;
    const float ps = lane < NW ? rd[1][lane] : 0.f;
    gm = wave_max(pm);
    gs = wave_sum(ps * exp_fast(pm - gm));

    S* yr = y + map.offset(row, ldy);
    const float f = exp_fast(m - gm) * (1.0f / gs);
    const float lse = (KIND == kLogSoftmax) ? log_of_sum(gs) : 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      if (idx < nvec) {
#pragma unroll
        for (int k = 0; k < W; ++k) {
          if (KIND == kSoftmax) {
            const float r = f * v[i][k];
            v[i][k] = __builtin_isnormal(r) ? r : 0.f;
          }
          else {
            v[i][k] = (v[i][k] - gm) - lse;
          }
        }
        Vec16<S>::store(yr + unsigned(W) * idx, v[i]);
      }
    }
  }
}

// Softmax forward with the cross entropy against a ground truth taken in the same pass
// (the consumer of the softmax output, src/layers/loss/cross_entropy.cpp:35-73): the row's
// outputs are written as sm_fwd_rows writes them, and loss = -sum over entries with
// xhat > 0 of xhat * log(y) is formed from the values that were just stored (flush included:
// an entry flushed to 0 under a positive xhat gives an infinite loss, as it does when the two
// layers run one after the other).  Saves the second layer's read of y.
// LABELS: the ground truth is one class index per column, stored as a float in row 0
// (use_labels with a spatial size of 1): xhat is 1 at that row and 0 elsewhere.
template <int TPR, int V, bool LABELS>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads)
sm_ce_fwd_rows(const float* x, const float* truth, float* y, float* loss, int64_t ldx, int64_t ldt, int64_t ldy,
               int64_t ld_loss, int64_t rows, unsigned nvec)
{
  using B = RowBlock<TPR>;
  constexpr int W = 4;
  constexpr bool kSub = TPR < kWave;
  static_assert(!kSub || TPR == 16, "sub-wave teams are one DPP row wide");
  constexpr int NW = kSub ? 1 : B::kWavesPerTeam;
  __shared__ float red[2][NW];
  __shared__ float red_loss[NW];
  const unsigned tid = threadIdx.x;
  const int team = kSub ? static_cast<int>(tid) / TPR : wave_index() / NW;
  const unsigned t = tid - team * TPR;
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * B::kTeams + team;
  if (B::kTeams > 1 && row >= rows) return;

  const float* xr = x + row * ldx;
  const float* tr = truth + row * ldt;
  float v[V][W], xh[LABELS ? 1 : V][W];
  int label = -1;
  if (LABELS) label = static_cast<int>(tr[0]);  // conversion to int as in the reference (cross_entropy.cpp:58)
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
      RowIO<float, W>::template load<false>(xr + unsigned(W) * idx, v[i]);
      if (!LABELS) RowIO<float, W>::template load<false>(tr + unsigned(W) * idx, xh[i]);
    }
    else {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        v[i][k] = -FLT_MAX;
        if (!LABELS) xh[i][k] = 0.f;
      }
    }
  }
  float m = -FLT_MAX;
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int k = 0; k < W; ++k) m = fmaxf(m, v[i][k]);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const bool ok = (t + i * TPR) < nvec;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      const float e = ok ? exp_fast(v[i][k] - m) : 0.f;
      s += e;
      v[i][k] = e;
    }
  }
  float gm = kSub ? row16_max(m) : wave_max(m);
  float gs = kSub ? row16_sum(s * exp_fast(m - gm)) : wave_sum(s * exp_fast(m - gm));
  if (NW > 1) {
    if (lane == 0) {
      red[0][wv] = gm;
      red[1][wv] = gs;
    }
    __syncthreads();
    const float pm = lane < NW ? red[0][lane] : -FLT_MAX;
    const float ps = lane < NW ? red[1][lane] : 0.f;
    gm = wave_max(pm);
    gs = wave_sum(ps * exp_fast(pm - gm));
  }
  float* yr = y + row * ldy;
  const float f = exp_fast(m - gm) * (1.0f / gs);
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        const float r = f * v[i][k];
        v[i][k] = __builtin_isnormal(r) ? r : 0.f;
        if (LABELS) {
          if (static_cast<int>(W * idx + k) == label) part += -logf(v[i][k]);
        }
        else if (xh[i][k] > 0.f) {
          part += -xh[i][k] * logf(v[i][k]);
        }
      }
      RowIO<float, W>::store(yr + unsigned(W) * idx, v[i]);
    }
  }
  part = kSub ? row16_sum(part) : team_sum<NW>(part, red_loss, wv, lane);
  if (t == 0) loss[row * ld_loss] = part;
}

// Backward of the softmax -> cross-entropy pair in one pass: the gradient with respect to the
// prediction, dp = -dloss * xhat / y where xhat > 0 and 0 elsewhere (cross_entropy.cpp:75-120), is
// formed in registers from the ground truth and goes straight into the softmax backward,
// dx = y * (dp - sum(y * dp)) (openmp/softmax.hpp:119-181), with the operations of the two kernels
// it replaces (a division, then the products), so a flushed y under a positive xhat gives the
// same NaN.  dp is never written; dtruth = -dloss * log(y) only when asked for (dense ground truth).
// LABELS as in sm_ce_fwd_rows.
template <int TPR, int V, bool LABELS>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads)
sm_ce_bwd_rows(const float* y, const float* truth, const float* dloss, float* dx, float* dtruth, int64_t ldy,
               int64_t ldt, int64_t ld_dloss, int64_t lddx, int64_t lddt, int64_t rows, unsigned nvec)
{
  using B = RowBlock<TPR>;
  constexpr int W = 4;
  constexpr bool kSub = TPR < kWave;
  static_assert(!kSub || TPR == 16, "sub-wave teams are one DPP row wide");
  constexpr int NW = kSub ? 1 : B::kWavesPerTeam;
  __shared__ float red[NW];
  const unsigned tid = threadIdx.x;
  const int team = kSub ? static_cast<int>(tid) / TPR : wave_index() / NW;
  const unsigned t = tid - team * TPR;
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * B::kTeams + team;
  if (B::kTeams > 1 && row >= rows) return;

  const float* yr = y + row * ldy;
  const float* tr = truth + row * ldt;
  const float gl = dloss[row * ld_dloss];
  float a[V][W], g[V][W];
  int label = -1;
  if (LABELS) label = static_cast<int>(tr[0]);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
      RowIO<float, W>::template load<false>(yr + unsigned(W) * idx, a[i]);
      if (!LABELS) RowIO<float, W>::template load<false>(tr + unsigned(W) * idx, g[i]);
    }
    else {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        a[i][k] = 1.f;  // never divided into: the matching xhat is 0
        g[i][k] = 0.f;
      }
    }
  }
  if (!LABELS && dtruth) {
    float* dtr = dtruth + row * lddt;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      if (idx < nvec) {
        float dt[W];
#pragma unroll
        for (int k = 0; k < W; ++k) dt[k] = -gl * logf(a[i][k]);
        RowIO<float, W>::store(dtr + unsigned(W) * idx, dt);
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      float dp;
      if (LABELS) dp = (idx < nvec && static_cast<int>(W * idx + k) == label) ? -gl / a[i][k] : 0.f;
      else dp = g[i][k] > 0.f ? -gl * g[i][k] / a[i][k] : 0.f;
      g[i][k] = dp;
      if (idx < nvec) s += a[i][k] * dp;
    }
  }
  s = kSub ? row16_sum(s) : team_sum<NW>(s, red, wv, lane);
  float* dr = dx + row * lddx;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
#pragma unroll
      for (int k = 0; k < W; ++k) g[i][k] = a[i][k] * (g[i][k] - s);
      RowIO<float, W>::store(dr + unsigned(W) * idx, g[i]);
    }
  }
}

// softmax / channelwise: dx = y * (dy - dot(y, dy));  log-softmax: dx = dy - exp(y) * sum(dy)
// STREAM: bit 0 streams y, bit 1 dy.  FR and UA as in sm_fwd_rows.
template <typename S, int TPR, int V, int KIND, int STREAM, int W = 16 / sizeof(S), bool FR = false, bool UA = false>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads)
sm_bwd_rows(const S* y, const S* dy, S* dx, int64_t ldy, int64_t lddy, int64_t lddx,
            RowMap map, int64_t rows, unsigned nvec)
{
  static_assert(!FR || (std::is_same<S, float>::value && W == 4), "frames are made of 16-byte fp32 vectors");
  static_assert(!UA || (!FR && W == 16 / sizeof(S)), "unaligned access moves whole 16-byte vectors");
  using B = RowBlock<TPR>;
  constexpr bool kSub = TPR < kWave;
  static_assert(!kSub || TPR == 16, "sub-wave teams are one DPP row wide");
  constexpr int NW = kSub ? 1 : B::kWavesPerTeam;
  __shared__ float red[NW];
  const unsigned tid = threadIdx.x;
  const int team = kSub ? static_cast<int>(tid) / TPR : wave_index() / NW;
  const unsigned t = tid - team * TPR;  // unsigned: addresses become scalar base + 32-bit offset
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * B::kTeams + team;
  if (B::kTeams > 1 && row >= rows) return;

  const S* yr = y + map.offset(row, ldy);
  const S* gr = dy + map.offset(row, lddy);
  const unsigned n = nvec;
  RowFrame fr{0, nvec};
  if constexpr (FR) {
    fr = row_frame(yr, n);
    yr -= fr.shift;
    gr -= fr.shift;
    nvec = fr.nvec;
  }
  unsigned ua_skip = 0;
  if constexpr (UA) {
    nvec = (n + W - 1) / W;
    ua_skip = nvec * W - n;
  }
  auto ua_off = [&](unsigned idx) { return (UA && idx == nvec - 1) ? n - W : unsigned(W) * idx; };
  auto ua_foreign = [&](unsigned idx) { return (UA && idx == nvec - 1) ? ua_skip : 0u; };
  float a[V][W], g[V][W];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
      if constexpr (FR) {
        frame_load(yr, idx, fr, n, 0.f, a[i]);
        frame_load(gr, idx, fr, n, 0.f, g[i]);
      }
      else if constexpr (UA) {
        RowIOUnaligned<S, W>::load(yr + ua_off(idx), a[i]);
        RowIOUnaligned<S, W>::load(gr + ua_off(idx), g[i]);
        const unsigned foreign = ua_foreign(idx);
#pragma unroll
        for (int k = 0; k < W; ++k)
          if (unsigned(k) < foreign) g[i][k] = 0.f;  // no share in the row sum (y is finite)
      }
      else {
        RowIO<S, W>::template load<(STREAM & 1) != 0>(yr + unsigned(W) * idx, a[i]);
        RowIO<S, W>::template load<(STREAM & 2) != 0>(gr + unsigned(W) * idx, g[i]);
      }
    }
    else {
#pragma unroll
      for (int k = 0; k < W; ++k) a[i][k] = g[i][k] = 0.f;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int k = 0; k < W; ++k) s += (KIND == kLogSoftmax) ? g[i][k] : a[i][k] * g[i][k];
  s = kSub ? row16_sum(s) : team_sum<NW>(s, red, wv, lane);

  S* dr = dx + map.offset(row, lddx);
  if constexpr (FR) dr -= fr.shift;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        // (16-bit storage: the two-operation exponential, as in the forward kernel)
        if (KIND == kLogSoftmax) g[i][k] = g[i][k] - (sizeof(S) == 2 ? exp_quick(a[i][k]) : exp_fast(a[i][k])) * s;
        else g[i][k] = a[i][k] * (g[i][k] - s);
      }
      if constexpr (FR) frame_store(dr, idx, fr, n, g[i]);
      else if constexpr (UA) {
        const unsigned foreign = ua_foreign(idx);
        if (foreign) {
#pragma unroll
          for (int k = 0; k < W; ++k)
            if (unsigned(k) >= foreign) RowLoad<S>::put(dr + ua_off(idx) + k, g[i][k]);
        }
        else {
          RowIOUnaligned<S, W>::store(dr + ua_off(idx), g[i]);
        }
      }
      else RowIO<S, W>::store(dr + unsigned(W) * idx, g[i]);
    }
  }
}


// Backward for rows that fill a 1024-thread workgroup's registers (two tensors of V vectors per
// thread: one workgroup per compute unit).  The grid is one resident wave of workgroups and a
// workgroup walks rows b, b + grid, ...: once dx of a row is formed in the registers that held dy,
// the registers that held y take the next row's y while dx is stored, and the next row's dy
// follows the stores, so a compute unit's loads overlap its stores instead of alternating with them.
// 32768 x 512: 50.9 us per step against 52.9 with one row per workgroup (log-softmax 51.5 against
// 54.8).  The same walk in the forward kernel, whose rows need half the registers so that two
// workgroups share a compute unit anyway, loses (53.0 against 51.2 us per step), and so does the
// walk over fp16 rows of this length (backward 19.9 against 18.8 us): fp32 rows of 8 vectors only.
// The fused softmax -> cross-entropy kernels, which hold two tensors each way, lose with it too: the
// division and the logarithms leave no registers for a second row (forward 47.8 against 35.8 us
// with 43 registers spilled, backward 38.8 against 37.0 us).
template <typename S, int V, int KIND, int STREAM>
__global__ void __launch_bounds__(1024)
sm_bwd_rows_walk(const S* y, const S* dy, S* dx, int64_t ldy, int64_t lddy, int64_t lddx,
                 RowMap map, int64_t rows, unsigned nvec)
{
  constexpr int TPR = 1024, W = 16 / sizeof(S), NW = TPR / kWave;
  __shared__ float red[2][NW];
  const unsigned t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wv = wave_index();
  float a[V][W], g[V][W];
  auto load_y = [&](int64_t row) {
    const S* yr = y + map.offset(row, ldy);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      if (idx < nvec) {
        RowIO<S, W>::template load<(STREAM & 1) != 0>(yr + unsigned(W) * idx, a[i]);
      }
      else {
#pragma unroll
        for (int k = 0; k < W; ++k) a[i][k] = 0.f;
      }
    }
  };
  auto load_dy = [&](int64_t row) {
    const S* gr = dy + map.offset(row, lddy);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      if (idx < nvec) {
        RowIO<S, W>::template load<(STREAM & 2) != 0>(gr + unsigned(W) * idx, g[i]);
      }
      else {
#pragma unroll
        for (int k = 0; k < W; ++k) g[i][k] = 0.f;
      }
    }
  };
  int64_t row = blockIdx.x;
  if (row >= rows) return;
  load_y(row);
  load_dy(row);
  for (int it = 0; row < rows; row += gridDim.x, ++it) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < W; ++k) s += (KIND == kLogSoftmax) ? g[i][k] : a[i][k] * g[i][k];
    s = team_sum<NW>(s, red[it & 1], wv, lane);
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < W; ++k) {
        if (KIND == kLogSoftmax) g[i][k] = g[i][k] - exp_fast(a[i][k]) * s;
        else g[i][k] = a[i][k] * (g[i][k] - s);
      }
    const int64_t next = row + gridDim.x;
    if (next < rows) load_y(next);
    asm volatile("" ::: "memory");  // y of the next row goes out ahead of this row's stores
    S* dr = dx + map.offset(row, lddx);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      if (idx < nvec) RowIO<S, W>::store(dr + unsigned(W) * idx, g[i]);
    }
    asm volatile("" ::: "memory");
    if (next < rows) load_dy(next);
  }
}

// The walk over 16-bit rows: both tensors of the next row wait as packed vectors (16 bytes for 8
// entries: 8 registers per thread and tensor at four vectors), so all of its loads go out before
// the current row is touched, arrive during its arithmetic and stores, and no wait for them
// stands behind a store.  (The fp32 walk above has no room for that and splits the next row's
// loads around the stores; 16-bit rows walked that way lose against one row per workgroup.)
template <typename S, int V, int KIND>
__global__ void __launch_bounds__(1024)
sm_bwd_rows_walk_packed(const S* y, const S* dy, S* dx, int64_t ldy, int64_t lddy, int64_t lddx, RowMap map,
                        int64_t rows, unsigned nvec)
{
  static_assert(sizeof(S) == 2, "packed 16-bit rows");
  constexpr int TPR = 1024, W = Vec16<S>::N, NW = TPR / kWave;
  using raw_t = typename Vec16<S>::raw_t;
  __shared__ float red[2][NW];
  const unsigned t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wv = wave_index();
  raw_t ny[V], ng[V];
  auto request = [&](int64_t row) {
    const S* yr = y + map.offset(row, ldy);
    const S* gr = dy + map.offset(row, lddy);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      ny[i] = raw_t{};
      ng[i] = raw_t{};
      if (idx < nvec) {
        ny[i] = Vec16<S>::load_raw(yr + unsigned(W) * idx);
        ng[i] = Vec16<S>::load_raw(gr + unsigned(W) * idx);
      }
    }
  };
  int64_t row = blockIdx.x;
  if (row >= rows) return;
  request(row);
  for (int it = 0; row < rows; row += gridDim.x, ++it) {
    float a[V][W], g[V][W];  // vectors past the end of the row hold zeros
#pragma unroll
    for (int i = 0; i < V; ++i) {
      Vec16<S>::unpack(ny[i], a[i]);
      Vec16<S>::unpack(ng[i], g[i]);
    }
    const int64_t next = row + gridDim.x;
    if (next < rows) request(next);
    asm volatile("" ::: "memory");  // the next row's loads go out ahead of this row's stores
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < W; ++k) s += (KIND == kLogSoftmax) ? g[i][k] : a[i][k] * g[i][k];
    s = team_sum<NW>(s, red[it & 1], wv, lane);
    S* dr = dx + map.offset(row, lddx);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const unsigned idx = t + i * TPR;
      if (idx < nvec) {
#pragma unroll
        for (int k = 0; k < W; ++k) {
          if (KIND == kLogSoftmax) g[i][k] = g[i][k] - exp_quick(a[i][k]) * s;
          else g[i][k] = a[i][k] * (g[i][k] - s);
        }
        Vec16<S>::store(dr + unsigned(W) * idx, g[i]);
      }
    }
  }
}

}  // namespace lbn
