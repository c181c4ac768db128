// Softmax, log-softmax and channelwise softmax, forward and backward, for gfx950.
//
// All three layers reduce over independent contiguous rows (a matrix column, or a
// channel window of a column).  Three kernel families cover every shape:
//
//  * register-resident row kernels: TPR threads (one wave, 256 or 1024 threads)
//    load a whole row with 128-bit coalesced loads, keep it in registers, reduce
//    on the wave64 DPP path (+ one LDS hop across waves), and store the result.
//    Each tensor is read once and written once.  Used when rows are 16-byte
//    aligned, a multiple of 4 long and at most 32768 entries; rows that are only
//    4-byte aligned (odd lengths) run the same kernels with one float per access up
//    to 8192 entries.
//  * register-resident clusters: rows too long for one workgroup whose tensors
//    exceed the caches are shared by a cluster of workgroups that exchange one
//    (max, sum) pair through memory.
//  * split ("chunked") kernels for the remaining long or unaligned rows: a row is cut
//    into S chunks, one workgroup each; chunks that start off a 16-byte boundary are
//    walked as leading scalars, aligned vectors and trailing scalars.  Kernel 1 leaves one partial reduction per chunk
//    in the workspace (for softmax an online (max, sum) pair), kernel 2 merges the
//    S partials and writes its chunk.  Kernel 1 reads everything before kernel 2
//    writes anything, so in-place operation stays safe with many workgroups per row.
//
// Numerics follow the reference CPU code: max-subtraction, exp at <= 2 ulp (exp_fast),
// reciprocal-then-multiply, and softmax (only) writes 0 for results that are not
// normal floats (include/lbann/utils/dnn_lib/openmp/softmax.hpp:107-116).
#include "cluster_sync.hpp"
#include "device_utils.hpp"
#include "host_utils.hpp"

#include <mutex>
#include <type_traits>

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
template <typename S, int TPR, int V, int KIND, bool STREAM, int W = 16 / sizeof(S), bool FR = false>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads, (TPR == 1024 && V <= 16 && V * W <= 32 ? 8 : 1))
sm_fwd_rows(const S* x, S* y, int64_t ldx, int64_t ldy, RowMap map, int64_t rows,
            unsigned nvec)
{
  static_assert(!FR || (std::is_same<S, float>::value && W == 4), "frames are made of 16-byte fp32 vectors");
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
  float v[V][W];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
      if constexpr (FR) frame_load(xr, idx, fr, n, -FLT_MAX, v[i]);
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
    const bool ok = (t + i * TPR) < nvec;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      const float d = v[i][k] - m;
      float e;
      if (KIND == kLogSoftmax) e = exp_quick(d);  // only summed: x stays in the registers for the output
      else if (KIND == kChannelwise) e = exp_keep_denormals(d);
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
      else RowIO<S, W>::store(yr + unsigned(W) * idx, v[i]);
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

// softmax / channelwise: dx = y * (dy - dot(y, dy));  log-softmax: dx = dy - exp(y) * sum(dy)
// STREAM: bit 0 streams y, bit 1 dy.  FR as in sm_fwd_rows.
template <typename S, int TPR, int V, int KIND, int STREAM, int W = 16 / sizeof(S), bool FR = false>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads)
sm_bwd_rows(const S* y, const S* dy, S* dx, int64_t ldy, int64_t lddy, int64_t lddx,
            RowMap map, int64_t rows, unsigned nvec)
{
  static_assert(!FR || (std::is_same<S, float>::value && W == 4), "frames are made of 16-byte fp32 vectors");
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
  float a[V][W], g[V][W];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = t + i * TPR;
    if (idx < nvec) {
      if constexpr (FR) {
        frame_load(yr, idx, fr, n, 0.f, a[i]);
        frame_load(gr, idx, fr, n, 0.f, g[i]);
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
        if (KIND == kLogSoftmax) g[i][k] = g[i][k] - exp_fast(a[i][k]) * s;
        else g[i][k] = a[i][k] * (g[i][k] - s);
      }
      if constexpr (FR) frame_store(dr, idx, fr, n, g[i]);
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

// Merges the online-softmax pairs (m, acc) of the 256 threads of a workgroup (defined
// with the split-row kernels below).
__device__ __forceinline__ void block_merge_max_sum(float& m, float& acc, float (*slot)[2]);

// ================================================ register-resident row clusters
// Rows too long for one workgroup's registers: a cluster of M workgroups shares a
// row, workgroup k keeps vectors [k*256*V, (k+1)*256*V) in registers, the cluster
// exchanges one (max, sum) pair per workgroup and every workgroup finishes from its
// registers.  One read and one write per element, and safe in place: a workgroup
// has read its whole share before it writes any of it, and shares are disjoint.
//
// The grid is persistent (cluster cl handles rows cl, cl + nclusters, ...) and rotates
// three register tiles so that nothing waits on something issued in the same step: in
// step s a workgroup (1) reduces tile s+1, whose loads were issued a step earlier, and
// publishes its partial pair, (2) issues the loads of tile s+2, (3) collects the
// cluster's partials of tile s, published a step earlier, and finishes tile s.
struct SmClusterArgs {
  const float* a;  // forward: x; backward: y
  const float* g;  // backward: dy
  float* out;
  int64_t lda, ldg, ldo;
  RowMap map;
  int64_t rows;
  unsigned nvec;
  unsigned n;  // framed access: entries per row (nvec is then the largest frame)
  int M;
  ClusterWorkspace cw;
  ClusterTag tag;
  __device__ __forceinline__ unsigned long long* slots(int64_t row) const { return cw.slots + row * M * 2; }
  // vectors of row `row` (every tensor has the same frames)
  template <bool FR>
  __device__ __forceinline__ unsigned row_nvec(int64_t row) const
  {
    return FR ? row_frame(a + map.offset(row, lda), n).nvec : nvec;
  }
};

template <int V, int W = 4>
struct SmFwdTile {
  float v[V][W];
  float m;  // the thread's own maximum: v holds exp(x - m) (or x - m for log-softmax)
};

template <int V, int W, bool FR = false>
__device__ __forceinline__ void sm_cl_load(float (&t)[V][W], const float* rowp, unsigned base,
                                           unsigned nvec, float fill, unsigned n = 0)
{
  static_assert(!FR || W == 4, "frames are made of 16-byte vectors");
  RowFrame fr{0, 0};
  if constexpr (FR) {
    fr = row_frame(rowp, n);
    rowp -= fr.shift;
    nvec = fr.nvec;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kClusterThreads;
    if (idx < nvec) {
      if constexpr (FR) frame_load(rowp, idx, fr, n, fill, t[i]);
      else RowIO<float, W>::template load<false>(rowp + W * static_cast<int64_t>(idx), t[i]);
    }
    else {
#pragma unroll
      for (int j = 0; j < W; ++j) t[i][j] = fill;
    }
  }
}

// The entries are exponentiated here, in front of the publication, and only rescaled after the
// exchange.  Summing a two-operation exponential here and exponentiating against the row's
// maximum afterwards (less work before the partials can leave) was measured: no gain on
// 262144 x 16 or 262144 x 256, and rows read one float at a time lose a third (50257 x 1024
// forward 137 against 87 us).
// (1) of a step: thread-local online softmax, one merge of the (max, sum) pairs of the
// workgroup, published for the cluster.
template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_fwd_reduce(const SmClusterArgs& a, int64_t row, int k, unsigned base,
                                                 SmFwdTile<V, W>& t, float (*red)[2])
{
  const unsigned nvec = a.row_nvec<FR>(row);
  float m = -FLT_MAX;
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int j = 0; j < W; ++j) m = fmaxf(m, t.v[i][j]);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const bool ok = base + i * kClusterThreads < nvec;
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const float d = t.v[i][j] - m;
      // (the entries of a frame's end vectors that lie outside the row hold -FLT_MAX: exp gives 0)
      const float e = ok ? (KIND == kChannelwise ? exp_keep_denormals(d) : exp_fast(d)) : 0.f;
      s += e;
      t.v[i][j] = (KIND == kLogSoftmax) ? d : e;
    }
  }
  t.m = m;
  block_merge_max_sum(m, s, red);
  if (threadIdx.x == 0) cluster_publish(m, s, a.slots(row), k, a.tag);
}

// (3) of a step.
// `poll` holds the polling loads for `row`, issued before the previous finish's stores (a wave's
// memory operations complete in order: a poll issued after stores waits for their acknowledgement);
// the loads for `next_row` (< 0: none) go out here, ahead of this row's stores.
template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_fwd_finish(const SmClusterArgs& a, int64_t row, unsigned base,
                                                 SmFwdTile<V, W>& t, float* bc, ClusterPoll<1>& poll, int64_t next_row)
{
  if (threadIdx.x < kWave) {
    float pm, ps;
    cluster_poll_pairs(poll, a.slots(row), a.M, a.tag, a.cw.error, -FLT_MAX, 0.f, pm, ps);
    const float gmax = wave_max(pm);
    const float gsum = wave_sum(ps * exp_fast(pm - gmax));
    if (threadIdx.x == 0) {
      bc[0] = gmax;
      bc[1] = gsum;
    }
  }
  __syncthreads();
  const float gm = bc[0];
  const float gs = bc[1];
  if (next_row >= 0 && threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(next_row), a.M);
  asm volatile("" ::: "memory");
  float* yr = a.out + a.map.offset(row, a.ldo);
  RowFrame fr{0, a.nvec};
  if constexpr (FR) {
    fr = row_frame(yr, a.n);
    yr -= fr.shift;
  }
  const float shift = t.m - gm;                     // <= 0: this thread's maximum against the row's
  const float f = exp_fast(shift) * (1.0f / gs);    // rescales exp(x - m) to exp(x - gm) / sum
  const float lse = (KIND == kLogSoftmax) ? log_of_sum(gs) : 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kClusterThreads;
    if (idx < fr.nvec) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        if (KIND == kSoftmax) {
          const float r = f * t.v[i][j];
          t.v[i][j] = __builtin_isnormal(r) ? r : 0.f;
        }
        else if (KIND == kLogSoftmax) {
          t.v[i][j] = (t.v[i][j] + shift) - lse;
        }
        else {
          t.v[i][j] *= f;
        }
      }
      if constexpr (FR) frame_store(yr, idx, fr, a.n, t.v[i]);
      else RowIO<float, W>::store(yr + W * static_cast<int64_t>(idx), t.v[i]);
    }
  }
}

template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_fwd_step(const SmClusterArgs& a, int64_t row, int64_t nc, int k,
                                               unsigned base, SmFwdTile<V, W>& F, SmFwdTile<V, W>& R,
                                               SmFwdTile<V, W>& L, float (*red)[2], float* bc,
                                               ClusterPoll<1>& poll)
{
  if (row + nc < a.rows) sm_cl_fwd_reduce<V, KIND, W, FR>(a, row + nc, k, base, R, red);
  if (row + 2 * nc < a.rows)
    sm_cl_load<V, W, FR>(L.v, a.a + a.map.offset(row + 2 * nc, a.lda), base, a.nvec, -FLT_MAX, a.n);
  asm volatile("" ::: "memory");  // keep the loads above the wait below
  sm_cl_fwd_finish<V, KIND, W, FR>(a, row, base, F, bc, poll, row + nc < a.rows ? row + nc : -1);
}

template <int V, int KIND, int W = 4, bool FR = false>
__global__ void __launch_bounds__(kClusterThreads)
sm_fwd_cluster(SmClusterArgs a)
{
  __shared__ float red[kClusterThreads / kWave][2];
  __shared__ float bc[3][2];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  const unsigned base = static_cast<unsigned>(k) * (kClusterThreads * V) + threadIdx.x;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  SmFwdTile<V, W> t0, t1, t2;
  sm_cl_load<V, W, FR>(t0.v, a.a + a.map.offset(cl, a.lda), base, a.nvec, -FLT_MAX, a.n);
  if (cl + nc < a.rows) sm_cl_load<V, W, FR>(t1.v, a.a + a.map.offset(cl + nc, a.lda), base, a.nvec, -FLT_MAX, a.n);
  sm_cl_fwd_reduce<V, KIND, W, FR>(a, cl, k, base, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  ClusterPoll<1> poll;
  if (threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(cl), a.M);
  // Each position of the rotation has its own broadcast slot: a step without a reduction has
  // no barrier between the reads of one finish and the write of the next.
  for (int64_t row = cl; row < a.rows; row += 3 * nc) {
    sm_cl_fwd_step<V, KIND, W, FR>(a, row, nc, k, base, t0, t1, t2, red, bc[0], poll);
    if (row + nc < a.rows) sm_cl_fwd_step<V, KIND, W, FR>(a, row + nc, nc, k, base, t1, t2, t0, red, bc[1], poll);
    if (row + 2 * nc < a.rows)
      sm_cl_fwd_step<V, KIND, W, FR>(a, row + 2 * nc, nc, k, base, t2, t0, t1, red, bc[2], poll);
  }
}

template <int V, int W = 4>
struct SmBwdTile {
  float a[V][W];
  float g[V][W];
};

template <int V, int KIND, int W = 4>
__device__ __forceinline__ void sm_cl_bwd_reduce(const SmClusterArgs& a, int64_t row, int k,
                                                 const SmBwdTile<V, W>& t, float* red)
{
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int j = 0; j < W; ++j) s += (KIND == kLogSoftmax) ? t.g[i][j] : t.a[i][j] * t.g[i][j];
  s = team_sum<kClusterThreads / kWave>(s, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) cluster_publish(s, 0.f, a.slots(row), k, a.tag);
}

template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_bwd_finish(const SmClusterArgs& a, int64_t row, unsigned base,
                                                 SmBwdTile<V, W>& t, float* bc, ClusterPoll<1>& poll, int64_t next_row)
{
  if (threadIdx.x < kWave) {
    float pt, unused;
    cluster_poll_pairs(poll, a.slots(row), a.M, a.tag, a.cw.error, 0.f, 0.f, pt, unused);
    pt = wave_sum(pt);
    if (threadIdx.x == 0) bc[0] = pt;
  }
  __syncthreads();
  const float tot = bc[0];
  if (next_row >= 0 && threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(next_row), a.M);
  asm volatile("" ::: "memory");
  float* dr = a.out + a.map.offset(row, a.ldo);
  RowFrame fr{0, a.nvec};
  if constexpr (FR) {
    fr = row_frame(dr, a.n);
    dr -= fr.shift;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kClusterThreads;
    if (idx < fr.nvec) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        if (KIND == kLogSoftmax) t.g[i][j] = t.g[i][j] - exp_fast(t.a[i][j]) * tot;
        else t.g[i][j] = t.a[i][j] * (t.g[i][j] - tot);
      }
      if constexpr (FR) frame_store(dr, idx, fr, a.n, t.g[i]);
      else RowIO<float, W>::store(dr + W * static_cast<int64_t>(idx), t.g[i]);
    }
  }
}

template <int V, int W, bool FR = false>
__device__ __forceinline__ void sm_cl_bwd_load(const SmClusterArgs& a, int64_t row, unsigned base,
                                               SmBwdTile<V, W>& t)
{
  sm_cl_load<V, W, FR>(t.a, a.a + a.map.offset(row, a.lda), base, a.nvec, 0.f, a.n);
  sm_cl_load<V, W, FR>(t.g, a.g + a.map.offset(row, a.ldg), base, a.nvec, 0.f, a.n);
}

template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_bwd_step(const SmClusterArgs& a, int64_t row, int64_t nc, int k,
                                               unsigned base, SmBwdTile<V, W>& F, SmBwdTile<V, W>& R,
                                               SmBwdTile<V, W>& L, float* red, float* bc, ClusterPoll<1>& poll)
{
  if (row + nc < a.rows) sm_cl_bwd_reduce<V, KIND, W>(a, row + nc, k, R, red);
  if (row + 2 * nc < a.rows) sm_cl_bwd_load<V, W, FR>(a, row + 2 * nc, base, L);
  asm volatile("" ::: "memory");
  sm_cl_bwd_finish<V, KIND, W, FR>(a, row, base, F, bc, poll, row + nc < a.rows ? row + nc : -1);
}

template <int V, int KIND, int W = 4, bool FR = false>
__global__ void __launch_bounds__(kClusterThreads)
sm_bwd_cluster(SmClusterArgs a)
{
  __shared__ float red[kClusterThreads / kWave];
  __shared__ float bc[3][1];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  const unsigned base = static_cast<unsigned>(k) * (kClusterThreads * V) + threadIdx.x;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  SmBwdTile<V, W> t0, t1, t2;
  sm_cl_bwd_load<V, W, FR>(a, cl, base, t0);
  if (cl + nc < a.rows) sm_cl_bwd_load<V, W, FR>(a, cl + nc, base, t1);
  sm_cl_bwd_reduce<V, KIND, W>(a, cl, k, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  ClusterPoll<1> poll;
  if (threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(cl), a.M);
  // Each position of the rotation has its own broadcast slot: a step without a reduction has
  // no barrier between the reads of one finish and the write of the next.
  for (int64_t row = cl; row < a.rows; row += 3 * nc) {
    sm_cl_bwd_step<V, KIND, W, FR>(a, row, nc, k, base, t0, t1, t2, red, bc[0], poll);
    if (row + nc < a.rows) sm_cl_bwd_step<V, KIND, W, FR>(a, row + nc, nc, k, base, t1, t2, t0, red, bc[1], poll);
    if (row + 2 * nc < a.rows)
      sm_cl_bwd_step<V, KIND, W, FR>(a, row + 2 * nc, nc, k, base, t2, t0, t1, red, bc[2], poll);
  }
}

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

// ==================================================================== host side
struct ChunkPlan {
  int S;
  int64_t chunk;
};

// Chunks per row for the split kernels: enough workgroups to occupy the device
// (about 4 per compute unit) without cutting rows into pieces shorter than 2048
// entries; chunk lengths are multiples of 4 so vector access stays aligned.
static ChunkPlan plan_chunks(int64_t n, int64_t rows)
{
  int64_t S = ceil_div(1024, rows);
  const int64_t by_len = ceil_div(n, 2048);
  if (S > by_len) S = by_len;
  if (S > kMaxChunks) S = kMaxChunks;
  if (S < 1) S = 1;
  int64_t chunk = ceil_div(ceil_div(n, S), 4) * 4;
  S = ceil_div(n, chunk);
  return {static_cast<int>(S), chunk};
}

constexpr int64_t kMaxScalarRow = 8192;   // the same in floats for rows accessed one float at a time
constexpr int64_t kMaxScalarLongRow = 32768;  // with 16 or 32 floats per thread: still one kernel, one read

// Rows of at most 64 access units, when there are many of them, go to teams of 16 lanes
// (four rows per wave) instead of leaving most of a wave idle: attention rows of 64
// entries (16 x 64 x 64 x 256) went from 124 to 54 us per step, 10-class rows from 78 to 21.
static RowConfig pick_sm_row_config(int64_t units, int64_t rows)
{
  if (units <= 64 && rows >= 4096) return {16, units <= 16 ? 1 : units <= 32 ? 2 : 4};
  return pick_row_config(units, rows);
}

static size_t sm_workspace_bytes(int64_t n, int64_t rows)
{
  if (n <= 0 || rows <= 0) return 0;
  const size_t chunked = kWorkspaceHeaderBytes + static_cast<size_t>(rows) * plan_chunks(n, rows).S * sizeof(float2);
  const size_t cluster = (n > kMaxScalarLongRow) ? cluster_workspace_bytes(rows) : 0;
  return chunked > cluster ? chunked : cluster;
}

// The register-resident cluster kernels read every element once but pay a rendezvous
// (a few microseconds) and a slot-reset launch; the two-kernel split path reads the
// input twice.  While the tensor fits the last-level caches the second read costs no
// HBM traffic, so the cluster path is used only for larger footprints.
constexpr int64_t kClusterMinBytes = int64_t(48) << 20;

// Streaming (non-temporal) loads keep a tensor that is read exactly once from pushing out
// lines that someone will read again.  Whether that pays depends on where the tensor is:
// measured on 32768 x 512 (64 MiB per tensor), us per step with the same buffers every step
// ("resident") / with every step's tensors rotated out of the caches ("cold"):
//   nothing streamed 52.8 / 62.7    backward streams y 52.3 / 60.9    y and dy 55.3 / 56.4
//   forward streams x 55.2 / 61.6   x and y 55.9 / 56.7               all three 54.5 / 58.4
// In a training step the forward input and the upstream gradient have just been written by
// the neighbouring layers and sit in the 256 MB Infinity Cache, while y was written a whole
// forward and backward sweep ago: y is streamed once a call moves more than a third of
// that cache, which costs nothing when the others are resident and helps when they are not.
// Calls that move more than the cache holds stream everything.
constexpr int64_t kStreamLoadMinBytes = int64_t(384) << 20;
constexpr int64_t kStreamOldInputMinBytes = int64_t(96) << 20;

static int stream_loads(int64_t rows, int64_t n, int tensors)
{
  static const int forced = std::getenv("LBN_STREAM_LOADS") ? std::atoi(std::getenv("LBN_STREAM_LOADS")) : -1;
  if (forced >= 0) return forced;
  return rows * n * 4 * tensors >= kStreamLoadMinBytes ? 1 : 0;
}

// A few very long rows whose tensors fit the caches (262144 x 16): one cluster kernel
// (20.6 us per step) against two split kernels per direction (22.7 us), except while a graph
// is recorded, where the cluster kernel needs a second node (24.1 us).
constexpr int64_t kFewRows = 64;

// Backward: bit 0 streams y, bit 1 streams dy (LBN_STREAM_LOADS_BWD overrides, for experiments).
static int stream_loads_bwd(int64_t rows, int64_t n)
{
  static const int forced = std::getenv("LBN_STREAM_LOADS_BWD") ? std::atoi(std::getenv("LBN_STREAM_LOADS_BWD")) : -1;
  if (forced >= 0) return forced & 3;
  if (stream_loads(rows, n, 3)) return 3;
  return rows * n * 4 * 3 >= kStreamOldInputMinBytes ? 1 : 0;
}

static bool cluster_enabled(hipStream_t st, int64_t rows, int64_t n)
{
  static const bool disabled = std::getenv("LBN_NO_CLUSTER") != nullptr;
  static const bool forced = std::getenv("LBN_FORCE_CLUSTER") != nullptr;
  if (disabled) return false;
  if (forced || rows * n * 4 >= kClusterMinBytes) return true;
  return rows <= kFewRows && !stream_is_capturing(st);
}

// Clusters of a launch that could hold `fit` of them at once.  Every cluster walks the same
// number of rows.  When all rows would fit at once (a few very long rows), a cluster still
// takes two rows as long as every compute unit keeps a workgroup: the second row's loads are
// in flight while the first row's partials cross the cluster, and the first row is written
// while the second one's do (262144 x 16: 13.1 against 14.7 us backward).  Four rows per
// cluster, all loaded up front by one workgroup per compute unit, were measured and are
// slower (forward 14.1 against 10.0 us per launch, backward the same 10.6): one wave per
// SIMD cannot overlap the exponentials of one row with the loads of the next.
static int64_t cluster_count(int64_t rows, int64_t fit, int M)
{
  int64_t per = ceil_div(rows, fit);
  if (per == 1 && rows >= 2 && ceil_div(rows, 2) * M >= 256) per = 2;
  return ceil_div(rows, per);
}

// Launch of the cluster kernels for rows of `units` accesses of W floats each.  Returns -1 when
// the plan or the device's capacity does not allow it (the caller goes on to the split
// kernels), otherwise the call's status.
// Framed access needs every tensor of the call to start each row at the same distance from a
// 16-byte boundary: the base pointers agree modulo 16 bytes and, with more than one column,
// so do the leading dimensions modulo 4 entries (the row stride inside a column is shared).
static bool same_frames(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t w)
{
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return (pa & 3u) == 0 && ((pa ^ pb) & 15u) == 0 && (w <= 1 || ((lda - ldb) & 3) == 0);
}

static bool framed_access()
{
  static const bool off = std::getenv("LBN_NO_FRAMED_ACCESS") != nullptr;
  return !off;
}

// FR: framed access (rows off the 16-byte grid moved as 16-byte vectors); `units` is then the
// largest frame, (n + 3 + 3) / 4 vectors, and `n` the row length.
template <int KIND, int W, bool FR = false>
static int sm_fwd_cluster_launch(hipStream_t st, ClusterPlan cp, int64_t units, int64_t rows, const float* x,
                                 int64_t ldx, float* y, int64_t ldy, RowMap map, void* ws, size_t ws_bytes,
                                 unsigned n = 0)
{
  if (!cp.M) return -1;
  if (!ws || ws_bytes < cluster_workspace_bytes(rows) || !aligned16(ws)) return LBN_ERR_WORKSPACE;
  const ClusterWorkspace cw = cluster_workspace(ws);
#define X(VV)                                                                                    \
  if (cp.V == VV) {                                                                              \
    const int cap = cluster_capacity(sm_fwd_cluster<VV, KIND, W, FR>, kClusterThreads);          \
    int64_t ncl = cap / cp.M < rows ? cap / cp.M : rows;                                         \
    if (ncl < 1) return -1;                                                                      \
    ncl = cluster_count(rows, ncl, cp.M);                                                        \
    ClusterLaunchGuard guard(st);                                                                \
    const SmClusterArgs a{x, nullptr, y, ldx, 0, ldy, map, rows, static_cast<unsigned>(units),   \
                          n, cp.M, cw, cluster_call_tag(st, cw)};                                \
    hipLaunchKernelGGL((sm_fwd_cluster<VV, KIND, W, FR>), dim3(static_cast<unsigned>(ncl * cp.M)), \
                       dim3(kClusterThreads), 0, st, a);                                         \
    return launch_status();                                                                      \
  }
  X(1) X(2) X(3) X(4)
  if constexpr (!FR) { X(5) X(6) X(7) X(8) }
#undef X
  return -1;
}

template <int KIND, int W, bool FR = false>
static int sm_bwd_cluster_launch(hipStream_t st, ClusterPlan cp, int64_t units, int64_t rows, const float* y,
                                 int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx, RowMap map,
                                 void* ws, size_t ws_bytes, unsigned n = 0)
{
  if (!cp.M) return -1;
  if (!ws || ws_bytes < cluster_workspace_bytes(rows) || !aligned16(ws)) return LBN_ERR_WORKSPACE;
  const ClusterWorkspace cw = cluster_workspace(ws);
#define X(VV)                                                                                    \
  if (cp.V == VV) {                                                                              \
    const int cap = cluster_capacity(sm_bwd_cluster<VV, KIND, W, FR>, kClusterThreads);          \
    int64_t ncl = cap / cp.M < rows ? cap / cp.M : rows;                                         \
    if (ncl < 1) return -1;                                                                      \
    ncl = cluster_count(rows, ncl, cp.M);                                                        \
    ClusterLaunchGuard guard(st);                                                                \
    const SmClusterArgs a{y, dy, dx, ldy, lddy, lddx, map, rows, static_cast<unsigned>(units),   \
                          n, cp.M, cw, cluster_call_tag(st, cw)};                                \
    hipLaunchKernelGGL((sm_bwd_cluster<VV, KIND, W, FR>), dim3(static_cast<unsigned>(ncl * cp.M)), \
                       dim3(kClusterThreads), 0, st, a);                                         \
    return launch_status();                                                                      \
  }
  X(1) X(2) X(3) X(4)
  if constexpr (W == 1) { X(5) X(6) X(7) X(8) }
#undef X
  return -1;
}

#define LBN_ROW_CASES(X)                                                                     \
  X(16, 1) X(16, 2) X(16, 4) X(64, 1) X(64, 2) X(64, 4) X(64, 8) X(256, 1) X(256, 2) X(256, 4) X(256, 8) X(1024, 1)      \
  X(1024, 2) X(1024, 4) X(1024, 8)

// Rows off the 16-byte grid that fit a workgroup's registers as a frame of 16-byte vectors
// (fp32 only).  False: not launched, the caller goes on to the one-float-per-access kernels.
// Measured, us per step framed / one float per access: 197 x 151296: 126 / 105; 1001 x 16384:
// 55 / 56; 4099 x 8192: 134 / 132; 8191 x 4096: 121 / 125; 16385 x 4096: 253 / 267;
// 30522 x 2048: 233 / 248.  The two end vectors of a row cost more than the wider accesses
// save until a row has a few thousand entries.
constexpr int64_t kFramedMinRow = 8000;

template <int KIND, typename S>
static bool sm_fwd_framed_rows(hipStream_t st, int64_t n, int64_t w, int64_t rows, const S* x, int64_t ldx, S* y,
                               int64_t ldy, RowMap map)
{
  if constexpr (!std::is_same<S, float>::value) {
    return false;
  }
  else {
    if (!framed_access() || n < kFramedMinRow || !same_frames(x, ldx, y, ldy, w)) return false;
    const RowConfig c = pick_sm_row_config((n + 6) / 4, rows);
    if (!c.tpr) return false;
#define X(TPR, V)                                                                                      \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                            \
    hipLaunchKernelGGL((sm_fwd_rows<float, TPR, V, KIND, false, 4, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                       x, y, ldx, ldy, map, rows, static_cast<unsigned>(n));                           \
    return true;                                                                                       \
  }
    LBN_ROW_CASES(X)
#undef X
    return false;
  }
}

template <int KIND, typename S>
static bool sm_bwd_framed_rows(hipStream_t st, int64_t n, int64_t w, int64_t rows, const S* y, int64_t ldy,
                               const S* dy, int64_t lddy, S* dx, int64_t lddx, RowMap map)
{
  if constexpr (!std::is_same<S, float>::value) {
    return false;
  }
  else {
    if (!framed_access() || n < kFramedMinRow || !same_frames(y, ldy, dy, lddy, w) ||
        !same_frames(y, ldy, dx, lddx, w))
      return false;
    const RowConfig c = pick_sm_row_config((n + 6) / 4, rows);
    if (!c.tpr) return false;
#define X(TPR, V)                                                                                      \
  if constexpr (!(TPR == 1024 && V > 8)) /* two tensors of more would not fit 128 registers */         \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                            \
    hipLaunchKernelGGL((sm_bwd_rows<float, TPR, V, KIND, 0, 4, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                       y, dy, dx, ldy, lddy, lddx, map, rows, static_cast<unsigned>(n));               \
    return true;                                                                                       \
  }
    LBN_ROW_CASES(X)
#undef X
    return false;
  }
}

template <int KIND, typename S = float>
static int sm_fwd(hipStream_t st, int64_t groups, int64_t n, int64_t stride, int64_t w,
                  const S* x, int64_t ldx, S* y, int64_t ldy, void* ws, size_t ws_bytes)
{
  constexpr int VE = 16 / sizeof(S);  // entries per 16-byte vector
  if (groups < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (groups == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !y) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = (groups - 1) * stride + n;
  if (w > 1 && (ldx < height || ldy < height)) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t rows = groups * w;
  if (rows > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  const RowMap map{groups, stride};
  const bool vec = (n % VE == 0) && rows_aligned16(x, stride, ldx, groups, w, sizeof(S)) &&
                   rows_aligned16(y, stride, ldy, groups, w, sizeof(S));
  if (vec) {
    const RowConfig c = pick_sm_row_config(n / VE, rows);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n / VE);
#define X(TPR, V)                                                                            \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    if (stream_loads(rows, n * sizeof(S) / 4, 2))                                            \
      hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                         x, y, ldx, ldy, map, rows, nvec);                                   \
    else                                                                                     \
      hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, false>), dim3(grid), dim3(B::kThreads), 0, st, \
                         x, y, ldx, ldy, map, rows, nvec);                                   \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X)
#undef X
    }
  }
  else if (sm_fwd_framed_rows<KIND>(st, n, w, rows, x, ldx, y, ldy, map)) {
    return launch_status();
  }
  else if (n <= kMaxScalarRow) {
    // rows that are only 4-byte aligned and short enough for registers: one float per access
    const RowConfig c = pick_sm_row_config(n, rows);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n);
#define X(TPR, V)                                                                            \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, false, 1>), dim3(grid), dim3(B::kThreads), 0, st, \
                       x, y, ldx, ldy, map, rows, nvec);                                     \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X)
#undef X
    }
  }
  else if (n <= kMaxScalarLongRow) {
    // the same up to 32768 entries (16385 x 4096: one kernel instead of partials + apply)
    const unsigned nvec = static_cast<unsigned>(n);
    const unsigned grid = static_cast<unsigned>(rows);
    if (n <= 16 * 1024)
      hipLaunchKernelGGL((sm_fwd_rows<S, 1024, 16, KIND, false, 1>), dim3(grid), dim3(1024), 0, st, x, y, ldx, ldy,
                         map, rows, nvec);
    else
      hipLaunchKernelGGL((sm_fwd_rows<S, 1024, 32, KIND, false, 1>), dim3(grid), dim3(1024), 0, st, x, y, ldx, ldy,
                         map, rows, nvec);
    return launch_status();
  }
  if constexpr (!std::is_same<S, float>::value) {
    // fp16 rows beyond the register kernels: one workgroup per row, three passes
    hipLaunchKernelGGL((sm_fwd_generic<S, KIND>), dim3(static_cast<unsigned>(rows)), dim3(kChunkThreads), 0, st, x, y,
                       ldx, ldy, map, n);
    return launch_status();
  }
  else {
    if (cluster_enabled(st, rows, n)) {
      int r = -1;
      if (vec && n / 4 < (int64_t(1) << 30)) {
        // four vectors per thread keep five workgroups per CU resident; eight only for rows that need it
        ClusterPlan cp = plan_cluster(n / 4, 4);
        if (!cp.M) cp = plan_cluster(n / 4, 8);
        r = sm_fwd_cluster_launch<KIND, 4>(st, cp, n / 4, rows, x, ldx, y, ldy, map, ws, ws_bytes);
      }
      else if (!vec) {
        // rows off the 16-byte grid (a vocabulary of 50257 entries): framed 16-byte access when both
        // tensors sit on the grid alike, else the same kernel with one float per access.  50257 x 1024,
        // us per step framed / one float per access: softmax 210 / 220, log-softmax 209 / 254
        const int64_t frame = (n + 6) / 4;
        if (framed_access() && same_frames(x, ldx, y, ldy, w) && n < (int64_t(1) << 31))
          r = sm_fwd_cluster_launch<KIND, 4, true>(st, plan_cluster(frame, 4), frame, rows, x, ldx, y, ldy, map, ws,
                                                   ws_bytes, static_cast<unsigned>(n));
        if (r < 0)
          r = sm_fwd_cluster_launch<KIND, 1>(st, plan_cluster(n, 8), n, rows, x, ldx, y, ldy, map, ws, ws_bytes);
      }
      if (r >= 0) return r;
    }
    const ChunkPlan p = plan_chunks(n, rows);
    if (rows * p.S > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
    if (!ws || ws_bytes < kWorkspaceHeaderBytes + static_cast<size_t>(rows) * p.S * sizeof(float2)) return LBN_ERR_WORKSPACE;
    float2* part = static_cast<float2*>(workspace_payload(ws));
    const dim3 grid(static_cast<unsigned>(rows * p.S)), block(kChunkThreads);
    if (vec) {
      hipLaunchKernelGGL((sm_fwd_partial<true>), grid, block, 0, st, x, ldx, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_fwd_apply<true, KIND>), grid, block, 0, st, x, y, ldx, ldy, map, n, p.chunk, p.S, part);
    }
    else {
      hipLaunchKernelGGL((sm_fwd_partial<false>), grid, block, 0, st, x, ldx, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_fwd_apply<false, KIND>), grid, block, 0, st, x, y, ldx, ldy, map, n, p.chunk, p.S, part);
    }
    return launch_status();
  }
}

// The walking backward kernel when the rows need more than one resident wave of workgroups.
template <int KIND, typename S>
static bool sm_bwd_walk(hipStream_t st, int hint, int64_t rows, unsigned nvec, const S* y, const S* dy,
                        S* dx, int64_t ldy, int64_t lddy, int64_t lddx, RowMap map)
{
  constexpr int V = 32 / (16 / sizeof(S));  // 32 values of each tensor per thread
  static const bool off = std::getenv("LBN_NO_BWD_WALK") != nullptr;
  if (off) return false;
#define W_(H)                                                                                          \
  if (hint == H) {                                                                                     \
    const int cap = resident_blocks(sm_bwd_rows_walk<S, V, KIND, H>, 1024);                            \
    if (cap < 1 || rows <= cap) return false;                                                          \
    hipLaunchKernelGGL((sm_bwd_rows_walk<S, V, KIND, H>), dim3(static_cast<unsigned>(cap)), dim3(1024), 0, st, y, dy, \
                       dx, ldy, lddy, lddx, map, rows, nvec);                                          \
    return true;                                                                                       \
  }
  W_(0) W_(1) W_(2) W_(3)
#undef W_
  return false;
}

template <int KIND, typename S = float>
static int sm_bwd(hipStream_t st, int64_t groups, int64_t n, int64_t stride, int64_t w,
                  const S* y, int64_t ldy, const S* dy, int64_t lddy, S* dx,
                  int64_t lddx, void* ws, size_t ws_bytes)
{
  constexpr int VE = 16 / sizeof(S);
  if (groups < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (groups == 0 || n == 0 || w == 0) return LBN_OK;
  if (!y || !dy || !dx) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = (groups - 1) * stride + n;
  if (w > 1 && (ldy < height || lddy < height || lddx < height)) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t rows = groups * w;
  if (rows > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  const RowMap map{groups, stride};
  const bool vec = (n % VE == 0) && rows_aligned16(y, stride, ldy, groups, w, sizeof(S)) &&
                   rows_aligned16(dy, stride, lddy, groups, w, sizeof(S)) &&
                   rows_aligned16(dx, stride, lddx, groups, w, sizeof(S));
  if (vec) {
    // two tensors live in registers: cap each at 4 vectors per thread when a row
    // still fits, so 1024-thread blocks keep two blocks per compute unit
    const RowConfig c = pick_sm_row_config(n / VE, rows);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n / VE);
#define X(TPR, V)                                                                            \
  if constexpr (!(TPR == 1024 && V * VE > 32)) /* two tensors of more would not fit 128 registers */ \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    const int hint = stream_loads_bwd(rows, n * sizeof(S) / 4);                              \
    if constexpr (std::is_same<S, float>::value && TPR == 1024 && V == 8) {                  \
      if (sm_bwd_walk<KIND>(st, hint, rows, nvec, y, dy, dx, ldy, lddy, lddx, map)) return launch_status(); \
    }                                                                                        \
    if (hint == 3)                                                                           \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 3>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    else if (hint == 1)                                                                      \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 1>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    else if (hint == 2)                                                                      \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 2>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    else                                                                                     \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 0>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X)
#undef X
    }
  }
  else if (sm_bwd_framed_rows<KIND>(st, n, w, rows, y, ldy, dy, lddy, dx, lddx, map)) {
    return launch_status();
  }
  else if (n <= kMaxScalarRow) {
    const RowConfig c = pick_sm_row_config(n, rows);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n);
#define X(TPR, V)                                                                            \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 0, 1>), dim3(grid), dim3(B::kThreads), 0, st, \
                       y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                         \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X)
#undef X
    }
  }
  else if (n <= (std::is_same<S, float>::value ? kMaxScalarLongRow : 16 * 1024)) {
    const unsigned nvec = static_cast<unsigned>(n);
    const unsigned grid = static_cast<unsigned>(rows);
    if (n <= 16 * 1024) {
      hipLaunchKernelGGL((sm_bwd_rows<S, 1024, 16, KIND, 0, 1>), dim3(grid), dim3(1024), 0, st, y, dy, dx, ldy,
                         lddy, lddx, map, rows, nvec);
    }
    else if constexpr (std::is_same<S, float>::value) {
      hipLaunchKernelGGL((sm_bwd_rows<S, 1024, 32, KIND, 0, 1>), dim3(grid), dim3(1024), 0, st, y, dy, dx, ldy,
                         lddy, lddx, map, rows, nvec);
    }
    return launch_status();
  }
  if constexpr (!std::is_same<S, float>::value) {
    hipLaunchKernelGGL((sm_bwd_generic<S, KIND>), dim3(static_cast<unsigned>(rows)), dim3(kChunkThreads), 0, st, y, dy,
                       dx, ldy, lddy, lddx, map, n);
    return launch_status();
  }
  else {
    if (cluster_enabled(st, rows, n)) {
      int r = -1;
      if (vec && n / 4 < (int64_t(1) << 30))
        r = sm_bwd_cluster_launch<KIND, 4>(st, plan_cluster(n / 4, 4), n / 4, rows, y, ldy, dy, lddy, dx, lddx, map, ws,
                                           ws_bytes);
      else if (!vec) {
        const int64_t frame = (n + 6) / 4;
        if (framed_access() && same_frames(y, ldy, dy, lddy, w) && same_frames(y, ldy, dx, lddx, w) &&
            n < (int64_t(1) << 31))
          r = sm_bwd_cluster_launch<KIND, 4, true>(st, plan_cluster(frame, 3), frame, rows, y, ldy, dy, lddy, dx, lddx,
                                                   map, ws, ws_bytes, static_cast<unsigned>(n));
        if (r < 0)
          r = sm_bwd_cluster_launch<KIND, 1>(st, plan_cluster(n, 8), n, rows, y, ldy, dy, lddy, dx, lddx, map, ws,
                                             ws_bytes);
      }
      if (r >= 0) return r;
    }
    const ChunkPlan p = plan_chunks(n, rows);
    if (rows * p.S > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
    if (!ws || ws_bytes < kWorkspaceHeaderBytes + static_cast<size_t>(rows) * p.S * sizeof(float2)) return LBN_ERR_WORKSPACE;
    float* part = static_cast<float*>(workspace_payload(ws));
    const dim3 grid(static_cast<unsigned>(rows * p.S)), block(kChunkThreads);
    if (vec) {
      hipLaunchKernelGGL((sm_bwd_partial<true, KIND>), grid, block, 0, st, y, dy, ldy, lddy, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_bwd_apply<true, KIND>), grid, block, 0, st, y, dy, dx, ldy, lddy, lddx, map, n, p.chunk, p.S, part);
    }
    else {
      hipLaunchKernelGGL((sm_bwd_partial<false, KIND>), grid, block, 0, st, y, dy, ldy, lddy, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_bwd_apply<false, KIND>), grid, block, 0, st, y, dy, dx, ldy, lddy, lddx, map, n, p.chunk, p.S, part);
    }
    return launch_status();
  }
}

// Softmax forward fused with the cross-entropy forward.  Returns -1 when the shape is not one
// the fused kernel takes (the caller then runs the two layers' kernels one after the other).
static int sm_ce_fwd_fused(hipStream_t st, int64_t n, int64_t w, int labels, const float* x, int64_t ldx,
                           const float* truth, int64_t ldt, float* y, int64_t ldy, float* loss, int64_t ld_loss)
{
  const bool vec = (n % 4 == 0) && rows_aligned16(x, n, ldx, 1, w, 4) && rows_aligned16(y, n, ldy, 1, w, 4) &&
                   (labels || rows_aligned16(truth, n, ldt, 1, w, 4));
  if (!vec) return -1;
  const RowConfig c = pick_sm_row_config(n / 4, w);
  if (!c.tpr) return -1;
  const unsigned nvec = static_cast<unsigned>(n / 4);
#define X(TPR, V)                                                                                      \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(w, B::kTeams));                               \
    if (labels)                                                                                        \
      hipLaunchKernelGGL((sm_ce_fwd_rows<TPR, V, true>), dim3(grid), dim3(B::kThreads), 0, st, x, truth, y, loss, \
                         ldx, ldt, ldy, ld_loss, w, nvec);                                             \
    else                                                                                               \
      hipLaunchKernelGGL((sm_ce_fwd_rows<TPR, V, false>), dim3(grid), dim3(B::kThreads), 0, st, x, truth, y, loss, \
                         ldx, ldt, ldy, ld_loss, w, nvec);                                             \
    return launch_status();                                                                            \
  }
  LBN_ROW_CASES(X)
#undef X
  return -1;
}

// ------------------------------------------------------------ library-owned scratch
// Scratch of the entry point that allocates nothing: one array per GPU, part of the code
// object, so it exists from the moment the library is loaded until the process ends.  The
// array's name is only a host-side handle: host code uses the address that
// hipGetSymbolAddress() reports for the current device, looked up once per device.
constexpr size_t kStaticScratchBytes = size_t(1) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;

// Device address of `scratch` on the current device; *out stays null on failure.
static int static_scratch_address(void** out)
{
  static std::mutex mu;
  static void* address[kMaxDevices] = {};
  *out = nullptr;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kMaxDevices) return LBN_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(mu);
  if (!address[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (!p) return static_cast<int>(hipErrorInvalidSymbol);
    address[dev] = p;
    // set-up, once per device: the event that orders cluster kernels across streams, so that
    // no later call of the entry point that allocates nothing has to create it
    ClusterLaunchGuard::prepare();
  }
  *out = address[dev];
  return LBN_OK;
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_softmax_workspace_bytes(int64_t height, int64_t width)
{
  return sm_workspace_bytes(height, width);
}

size_t lbn_channelwise_softmax_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  if (channels <= 0 || width <= 0) return 0;
  return sm_workspace_bytes(channel_size, channels * width);
}

int lbn_softmax_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                        int64_t ldx, float* y, int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy, workspace, workspace_bytes);
}

int lbn_softmax_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* y,
                        int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx,
                        void* workspace, size_t workspace_bytes)
{
  return sm_bwd<kSoftmax>(as_stream(stream), 1, height, height, width, y, ldy, dy, lddy, dx, lddx, workspace, workspace_bytes);
}

size_t lbn_softmax_fwd_static_scratch_max_bytes(void) { return kStaticScratchBytes; }

int lbn_softmax_fwd_static_scratch_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                                       int64_t ldx, float* y, int64_t ldy)
{
  if (height < 0 || width < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (sm_workspace_bytes(height, width) > kStaticScratchBytes) return LBN_ERR_UNSUPPORTED;
  void* ptr = nullptr;
  const int status = static_scratch_address(&ptr);
  if (status != LBN_OK) return status;
  return sm_fwd<kSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy, ptr, kStaticScratchBytes);
}

int lbn_log_softmax_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                            int64_t ldx, float* y, int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kLogSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy, workspace, workspace_bytes);
}

int lbn_log_softmax_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* y,
                            int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx,
                            void* workspace, size_t workspace_bytes)
{
  return sm_bwd<kLogSoftmax>(as_stream(stream), 1, height, height, width, y, ldy, dy, lddy, dx, lddx, workspace, workspace_bytes);
}

size_t lbn_softmax_cross_entropy_fwd_workspace_bytes(int64_t height, int64_t width)
{
  // the cross-entropy partial sums sit past the header that the softmax kernels keep their wait status in
  const size_t a = lbn_softmax_workspace_bytes(height, width);
  const size_t b = lbn_cross_entropy_fwd_workspace_bytes(height, width);
  return a > b + kWorkspaceHeaderBytes ? a : (b ? b + kWorkspaceHeaderBytes : a);
}

int lbn_softmax_cross_entropy_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                                      int64_t spatial_size, const float* x, int64_t ldx, const float* ground_truth,
                                      int64_t ld_truth, float* y, int64_t ldy, float* loss, int64_t ld_loss,
                                      void* workspace, size_t workspace_bytes)
{
  hipStream_t st = as_stream(stream);
  if (height < 0 || width < 0 || ld_loss < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (width == 0) return LBN_OK;
  if (height == 0)  // no softmax output; the loss of an empty column is 0
    return lbn_cross_entropy_fwd_f32(stream, height, width, use_labels, spatial_size, y, ldy, ground_truth, ld_truth,
                                     loss, ld_loss, nullptr, 0);
  if (!x || !ground_truth || !y || !loss || ld_loss < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (use_labels && spatial_size < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (width > 1 && (ldx < height || ldy < height || ld_truth < (use_labels ? 1 : height)))
    return LBN_ERR_INVALID_ARGUMENT;
  if (!use_labels || spatial_size == 1) {
    const int r = sm_ce_fwd_fused(st, height, width, use_labels ? 1 : 0, x, ldx, ground_truth, ld_truth, y, ldy,
                                  loss, ld_loss);
    if (r >= 0) return r;
  }
  // shapes the fused kernel does not take: the two layers' kernels one after the other
  const int status = sm_fwd<kSoftmax>(st, 1, height, height, width, x, ldx, y, ldy, workspace, workspace_bytes);
  if (status != LBN_OK) return status;
  const bool room = workspace && workspace_bytes > kWorkspaceHeaderBytes;
  return lbn_cross_entropy_fwd_f32(stream, height, width, use_labels, spatial_size, y, ldy, ground_truth, ld_truth,
                                   loss, ld_loss, room ? workspace_payload(workspace) : nullptr,
                                   room ? workspace_bytes - kWorkspaceHeaderBytes : 0);
}

// fp16 storage (IEEE binary16 in memory, fp32 arithmetic); the workspace arguments are there for
// symmetry with the fp32 entry points and are not used.
int lbn_softmax_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* x, int64_t ldx, void* y,
                        int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(x), ldx,
                                  static_cast<__half*>(y), ldy, workspace, workspace_bytes);
}

int lbn_softmax_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* y, int64_t ldy,
                        const void* dy, int64_t lddy, void* dx, int64_t lddx, void* workspace,
                        size_t workspace_bytes)
{
  return sm_bwd<kSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(y), ldy,
                                  static_cast<const __half*>(dy), lddy, static_cast<__half*>(dx), lddx, workspace,
                                  workspace_bytes);
}

int lbn_log_softmax_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* x, int64_t ldx,
                            void* y, int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kLogSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(x), ldx,
                                     static_cast<__half*>(y), ldy, workspace, workspace_bytes);
}

int lbn_log_softmax_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* y, int64_t ldy,
                            const void* dy, int64_t lddy, void* dx, int64_t lddx, void* workspace,
                            size_t workspace_bytes)
{
  return sm_bwd<kLogSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(y), ldy,
                                     static_cast<const __half*>(dy), lddy, static_cast<__half*>(dx), lddx, workspace,
                                     workspace_bytes);
}

int lbn_channelwise_softmax_fwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width, const float* x,
                                    int64_t ldx, float* y, int64_t ldy, void* workspace,
                                    size_t workspace_bytes)
{
  return sm_fwd<kChannelwise>(as_stream(stream), channels, channel_size, channel_stride, width, x, ldx, y, ldy, workspace, workspace_bytes);
}

int lbn_channelwise_softmax_bwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width, const float* y,
                                    int64_t ldy, const float* dy, int64_t lddy, float* dx,
                                    int64_t lddx, void* workspace, size_t workspace_bytes)
{
  return sm_bwd<kChannelwise>(as_stream(stream), channels, channel_size, channel_stride, width, y, ldy, dy, lddy, dx, lddx, workspace, workspace_bytes);
}

}  // extern "C"
