// Layer normalization forward and backward for gfx950, fp32 and fp16 storage
// (all arithmetic, statistics and weights in fp32).
//
// A row is one normalised group of one sample (layer_norm.hpp:362-405): n contiguous
// entries at row offset g*stride of column c.
//
//  * forward, register-resident: a team of 64/256/1024 threads loads the row once
//    with 128-bit loads, takes the mean, then the mean of squared deviations from
//    the registers (two-pass, no E[x^2]-mean^2 cancellation; the reference formula
//    is available through LBN_STATS_SUMSQ), writes the statistics and the output.
//  * backward, register-resident and persistent: each team walks over many rows,
//    keeps x and dy of the current row in registers, reduces the two row sums with
//    wave64 shuffles, writes dx, and accumulates its share of dscale/dbias in
//    registers across rows (a thread always owns the same feature positions).  The
//    teams of a block merge through LDS, every block leaves one partial row in the
//    workspace, and a second small kernel sums the partial rows in a fixed order:
//    no atomics, bitwise reproducible.
//  * rows off the 16-byte grid (odd lengths or leading dimensions) run the same register
//    kernels on other storage types: one float (f32x1) or one pair of halves (f16x2) per
//    access, or 16-byte accesses at the alignment of one entry (f32u, f16u), where the row's
//    last, partial vector is read as its last whole 16 bytes and the entries it shares with
//    its neighbour are masked out.  Which one serves a shape is measured, not derived:
//    ln_pairs_first, ln_vectors_first.
//  * rows longer than the register kernels hold: layer_norm_long.hpp.
//  * generic kernels (one 256-thread block per row, scalar access) cover what is left
//    (rows of fewer than 4 floats or 8 halves off the grid).
#include <type_traits>

#include "device_utils.hpp"
#include "host_utils.hpp"
#include "layer_norm_cluster.hpp"
#include "layer_norm_long.hpp"
#include "reference_order.hpp"

namespace lbn {

// ================================================================== forward
// A team of TPR threads owns a row in registers (V 16-byte vectors per thread) and
// walks the rows blockIdx.x*teams + team, + gridDim.x*teams, ...; the launch is one
// resident wave of blocks.  The team's next row is in flight, still packed, while the
// current one is processed, and threads that own at most 16 entries keep their scale
// and bias in registers across rows.
//
// Per element: one conversion, the sum, the centred value and its square (or, in
// sum-of-squares mode, the square of the raw value), then d * (1/stdev) and one
// multiply-add with scale and bias.  Means use a multiplication by 1/n.
template <typename T, int TPR, int V>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads)
ln_fwd_rows(const T* __restrict__ x, T* __restrict__ y, int64_t ldx, int64_t ldy, RowMap map,
            int64_t rows, int nvec, float inv_n, float eps, float* __restrict__ stats,
            int64_t ld_stats, const float* __restrict__ gamma, const float* __restrict__ beta,
            int sumsq, int tail = 0)
{
  using B = RowBlock<TPR>;
  using IO = Vec16<T>;
  using raw_t = typename IO::raw_t;
  constexpr int VE = IO::N;
  // Storage types whose 16-byte accesses need no alignment take rows of any length: nvec counts
  // a last vector of `tail` entries (0: none), which is read as the row's last VE entries,
  // overlapping its neighbour; the entries it shares count and are stored once, by the neighbour.
  constexpr bool kTail = UnalignedVec<T>::value;
  constexpr bool kSub = TPR < kWave;  // short rows: a team is one DPP row of 16 lanes, four rows per wave
  static_assert(!kSub || TPR == 16, "sub-wave teams are one DPP row wide");
  constexpr int NW = kSub ? 1 : B::kWavesPerTeam;
  constexpr bool kWeightsInRegs = V * VE <= 16;
  constexpr bool kPrefetch = V * VE < 32;  // wider rows: the registers only hold the current row
  constexpr int WV = kWeightsInRegs ? V : 1;
  __shared__ float red[4][B::kTeams][2 * NW];
  const int tid = threadIdx.x;
  // a team is a whole number of waves (then its index is wave-uniform) or a DPP row
  const int team = kSub ? tid / TPR : wave_index() / NW;
  const int t = tid - team * TPR;
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;

  // A vector past the end of the row re-reads vector 0 and is masked out of the sums.
  bool ok[V];
  int voff[V];
  int skip[V];  // leading entries of the vector that belong to its neighbour
#pragma unroll
  for (int i = 0; i < V; ++i) {
    ok[i] = t + i * TPR < nvec;
    voff[i] = ok[i] ? VE * (t + i * TPR) : 0;
    skip[i] = 0;
    if (kTail && tail && t + i * TPR == nvec - 1) {
      skip[i] = VE - tail;
      voff[i] -= skip[i];
    }
  }
  const int n_entries = (kTail && tail) ? (nvec - 1) * VE + tail : nvec * VE;
  auto load_weights = [&](const float* w, int i, float fill, float (&out)[VE]) {
#pragma unroll
    for (int k = 0; k < VE; ++k) out[k] = fill;
    if (w) {
      if constexpr (kTail) __builtin_memcpy(out, w + voff[i], sizeof(float) * VE);
      else load_f32_run<VE>(w + voff[i], out);
    }
  };
  float gam[WV][VE], bet[WV][VE];
  if constexpr (kWeightsInRegs) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      load_weights(gamma, i, 1.f, gam[i]);
      load_weights(beta, i, 0.f, bet[i]);
    }
  }

  const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * B::kTeams;
  const int64_t iters = (rows + rows_per_iter - 1) / rows_per_iter;
  const int64_t first_row = static_cast<int64_t>(blockIdx.x) * B::kTeams + team;
  raw_t q[V];  // the row in flight
  auto issue = [&](int64_t row) {
    const T* xr = x + map.offset(row < rows ? row : rows - 1, ldx);  // wave-uniform
#pragma unroll
    for (int i = 0; i < V; ++i) q[i] = IO::load_raw(xr + voff[i]);
  };

  // full: every thread owns V whole vectors, nothing is masked.
  auto process = [&](int64_t it, auto full) {
    constexpr bool kFull = decltype(full)::value;
    const int64_t row = it * rows_per_iter + first_row;
    if constexpr (!kPrefetch) issue(row);
    float v[V][VE];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      IO::unpack(q[i], v[i]);
      if (!kFull && !ok[i]) {
#pragma unroll
        for (int k = 0; k < VE; ++k) v[i][k] = 0.f;
      }
      if constexpr (kTail) {
#pragma unroll
        for (int k = 0; k < VE; ++k)
          if (k < skip[i]) v[i][k] = 0.f;
      }
    }
    if constexpr (kPrefetch) {
      if (it + 1 < iters) issue(row + rows_per_iter);
    }
    float* slots = red[2 * (it & 1)][team];
    float mean, var;
    if (sumsq) {
      float s = 0.f, sq = 0.f;
#pragma unroll
      for (int i = 0; i < V; ++i)
#pragma unroll
        for (int k = 0; k < VE; ++k) {
          s += v[i][k];
          sq = __builtin_fmaf(v[i][k], v[i][k], sq);
        }
      if constexpr (kSub) {
        s = row16_sum(s);
        sq = row16_sum(sq);
      }
      else {
        team_sum2<NW>(s, sq, slots, wv, lane);
      }
      // the reference's own expression (layer_norm.cpp:99-112): true divisions, no fused
      // multiply-add, so that its cancellation and clamp come out the same
      const float nf = static_cast<float>(n_entries);
      mean = s / nf;
      var = fmaxf(__fsub_rn(sq / nf, __fmul_rn(mean, mean)), 0.f);
#pragma unroll
      for (int i = 0; i < V; ++i)
#pragma unroll
        for (int k = 0; k < VE; ++k) v[i][k] -= mean;
    }
    else {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < V; ++i)
#pragma unroll
        for (int k = 0; k < VE; ++k) s += v[i][k];
      s = kSub ? row16_sum(s) : team_sum<NW>(s, slots, wv, lane);
      mean = s * inv_n;
      float sq = 0.f;
#pragma unroll
      for (int i = 0; i < V; ++i) {
#pragma unroll
        for (int k = 0; k < VE; ++k) {
          v[i][k] -= mean;
          const float d = ((kFull || ok[i]) && !(kTail && k < skip[i])) ? v[i][k] : 0.f;
          sq = __builtin_fmaf(d, d, sq);
        }
      }
      sq = kSub ? row16_sum(sq) : team_sum<NW>(sq, red[2 * (it & 1) + 1][team], wv, lane);
      var = sq * inv_n;
    }
    if (row < rows) {
      const float inv_stdev = rsqrt_refined(var + eps);
      int64_t col, g;
      map.split(row, col, g);
      if (t == 0) {
        stats[g + col * ld_stats] = mean;
        stats[map.groups + g + col * ld_stats] = var;
      }
      T* yr = y + g * map.stride + col * ldy;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (kFull || ok[i]) {
          if constexpr (kWeightsInRegs) {
#pragma unroll
            for (int k = 0; k < VE; ++k)
              v[i][k] = __builtin_fmaf(v[i][k] * inv_stdev, gam[i][k], bet[i][k]);
          }
          else {
            float gw[VE], bw[VE];
            load_weights(gamma, i, 1.f, gw);
            load_weights(beta, i, 0.f, bw);
#pragma unroll
            for (int k = 0; k < VE; ++k) v[i][k] = __builtin_fmaf(v[i][k] * inv_stdev, gw[k], bw[k]);
          }
          bool whole = true;
          if constexpr (kTail) {
            if (skip[i]) {
              whole = false;
#pragma unroll
              for (int k = 0; k < VE; ++k)
                if (k >= skip[i]) IO::store1(yr + voff[i] + k, v[i][k]);
            }
          }
          if (whole) IO::store(yr + voff[i], v[i]);
        }
      }
    }
  };

  if constexpr (kPrefetch) issue(first_row);
  if (nvec == TPR * V && !(kTail && tail)) {
    for (int64_t it = 0; it < iters; ++it) process(it, std::true_type{});
  }
  else {
    for (int64_t it = 0; it < iters; ++it) process(it, std::false_type{});
  }
}

// One 256-thread block per row, scalar access, any n >= 1.
template <typename T>
__global__ void __launch_bounds__(256)
ln_fwd_generic(const T* __restrict__ x, T* __restrict__ y, int64_t ldx, int64_t ldy, RowMap map,
               int64_t n, float eps, float* __restrict__ stats, int64_t ld_stats,
               const float* __restrict__ gamma, const float* __restrict__ beta, int sumsq)
{
  using IO = Vec16<T>;
  __shared__ float red[2][8];
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const int64_t row = blockIdx.x;
  const T* xr = x + map.offset(row, ldx);
  float mean, var;
  if (n <= 1) {
    mean = IO::load1(xr);
    var = 1.f;
  }
  else if (sumsq) {
    float s = 0.f, q = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
      const float a = IO::load1(xr + i);
      s += a;
      q += a * a;
    }
    team_sum2<4>(s, q, red[0], wv, lane);
    mean = s / static_cast<float>(n);
    var = fmaxf(q / static_cast<float>(n) - mean * mean, 0.f);
  }
  else {
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 256) s += IO::load1(xr + i);
    s = team_sum<4>(s, red[0], wv, lane);
    mean = s / static_cast<float>(n);
    float q = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
      const float d = IO::load1(xr + i) - mean;
      q += d * d;
    }
    q = team_sum<4>(q, red[1], wv, lane);
    var = q / static_cast<float>(n);
  }
  const float inv_stdev = 1.0f / sqrtf(var + eps);
  if (threadIdx.x == 0) {
    int64_t col, g;
    map.split(row, col, g);
    stats[g + col * ld_stats] = mean;
    stats[map.groups + g + col * ld_stats] = var;
  }
  T* yr = y + map.offset(row, ldy);
  for (int64_t i = threadIdx.x; i < n; i += 256) {
    float r = (IO::load1(xr + i) - mean) * inv_stdev;
    if (gamma) r *= gamma[i];
    if (beta) r += beta[i];
    IO::store1(yr + i, r);
  }
}

// Rows of a single entry (instance norm on 1 x 1 maps): the mean is the entry, the variance 1
// (layer_norm.cpp:70-77), one thread per row instead of a workgroup.
template <typename T>
__global__ void __launch_bounds__(256)
ln_fwd_single(const T* __restrict__ x, T* __restrict__ y, int64_t ldx, int64_t ldy, RowMap map, int64_t rows,
              float eps, float* __restrict__ stats, int64_t ld_stats, const float* __restrict__ gamma,
              const float* __restrict__ beta)
{
  using IO = Vec16<T>;
  const float inv_stdev = 1.0f / sqrtf(1.f + eps);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; row < rows;
       row += static_cast<int64_t>(gridDim.x) * 256) {
    int64_t col, g;
    map.split(row, col, g);
    const float v = IO::load1(x + g * map.stride + col * ldx);
    stats[g + col * ld_stats] = v;
    stats[map.groups + g + col * ld_stats] = 1.f;
    float r = (v - v) * inv_stdev;  // 0, or NaN for an entry that is not finite, as in the general kernel
    if (gamma) r *= gamma[0];
    if (beta) r += beta[0];
    IO::store1(y + g * map.stride + col * ldy, r);
  }
}

// ================================================================== backward
// Weight gradients of small problems without any exchange between workgroups: dscale and
// dbias of a feature depend on x, dy and the FORWARD statistics only (xh = (x - mean) /
// stdev needs nothing from this pass), so a workgroup can form them for a slice of eight
// access units of features over all rows by reading that column slice itself.  The tensors
// are read a second time, from the caches: worth it while they fit them, where it saves
// the partial rows, the reduction kernel and its launch (1024 x 128: three dependent
// kernels per step become two).  Threads = 8 access units x (threads / 8) row groups; the
// sums over rows and row groups run in a fixed order.
template <typename T>
struct LnColLoads {
  typename Vec16<T>::raw_t x[4], g[4];
  float mean[4], var[4];
};

template <typename T, int THREADS>
__device__ __forceinline__ void ln_cols_issue(LnColLoads<T>& c, const T* x, const T* dy, int64_t ldx, int64_t lddy,
                                              const RowMap& map, int64_t rows, int n, const float* stats,
                                              int64_t ld_stats, int64_t slice, int64_t row0)
{
  constexpr int VE = Vec16<T>::N;
  constexpr int RG = THREADS / 8;
  const int kq = threadIdx.x & 7, pg = threadIdx.x >> 3;
  int64_t k = (slice * 8 + kq) * VE;
  if (k >= n) k = 0;  // loads past the end re-read valid memory and are masked when used
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int64_t r = row0 + pg + RG * j;
    if (r >= rows) r = rows - 1;
    int64_t col, g;
    map.split(r, col, g);
    c.x[j] = Vec16<T>::load_raw(x + g * map.stride + col * ldx + k);
    c.g[j] = Vec16<T>::load_raw(dy + g * map.stride + col * lddy + k);
    c.mean[j] = stats[g + col * ld_stats];
    c.var[j] = stats[map.groups + g + col * ld_stats];
  }
}

template <typename T, int THREADS>
__device__ __forceinline__ void ln_cols_accumulate(const LnColLoads<T>& c, int64_t rows, int n, float eps,
                                                   int64_t slice, int64_t row0, float (&dg)[Vec16<T>::N],
                                                   float (&db)[Vec16<T>::N])
{
  constexpr int VE = Vec16<T>::N;
  constexpr int RG = THREADS / 8;
  const int kq = threadIdx.x & 7, pg = threadIdx.x >> 3;
  const bool col_ok = (slice * 8 + kq) * VE < n;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const bool use = col_ok && row0 + pg + RG * j < rows;
    const float inv_stdev = rsqrt_refined(c.var[j] + eps);
    float xv[VE], gv[VE];
    Vec16<T>::unpack(c.x[j], xv);
    Vec16<T>::unpack(c.g[j], gv);
#pragma unroll
    for (int e = 0; e < VE; ++e) {
      const float g = use ? gv[e] : 0.f;
      db[e] += g;
      dg[e] = __builtin_fmaf(g, (xv[e] - c.mean[j]) * inv_stdev, dg[e]);
    }
  }
}

// Adds the row groups' sums of a slice through LDS (sm: 2 x RG x (8 VE + 1) floats) and writes
// the slice's entries of dscale and dbias.
template <typename T, int THREADS>
__device__ __forceinline__ void ln_cols_finish(float* sm, int n, int64_t slice, const float (&dg)[Vec16<T>::N],
                                               const float (&db)[Vec16<T>::N], float* dscale, float* dbias)
{
  constexpr int VE = Vec16<T>::N;
  constexpr int RG = THREADS / 8;
  constexpr int W = 8 * VE + 1;
  const int kq = threadIdx.x & 7, pg = threadIdx.x >> 3;
#pragma unroll
  for (int e = 0; e < VE; ++e) {
    sm[pg * W + kq * VE + e] = dg[e];
    sm[(RG + pg) * W + kq * VE + e] = db[e];
  }
  __syncthreads();
  if (threadIdx.x < 2 * 8 * VE) {
    const int which = threadIdx.x / (8 * VE), c = threadIdx.x - which * (8 * VE);
    const float* col = sm + which * RG * W + c;
    float acc = 0.f;
#pragma unroll 8
    for (int r = 0; r < RG; r += 4) acc += (col[r * W] + col[(r + 1) * W]) + (col[(r + 2) * W] + col[(r + 3) * W]);
    const int64_t k = slice * 8 * VE + c;
    float* out = which == 0 ? dscale : dbias;
    if (out && k < n) out[k] = acc;
  }
  __syncthreads();  // the next slice writes sm again
}

// Partial weight gradients: block b writes 2*n floats at part + b*2*n (dscale row
// followed by dbias row).
//
// Per element the kernel spends 9 VALU operations before the row reduction and 4
// after it: with xh = (x - mean) / stdev,
//   dbias += dy;  dscale += dy * xh;  gs = dy * scale;  A += gs;  B += gs * xh
//   dx = gs / stdev + dmean / n + (dvar * 2 * stdev / n) * xh
// where dmean = -A / stdev and dvar = -B / (2 stdev^2)  (layer_norm.cpp:198-257).
//
// A team's next row is in flight, still packed, while the current one is processed,
// unless a thread owns 32 entries: then the registers only hold the current row.
//
// COLS (small problems, instead of WGRAD): the workgroup also forms dscale and dbias of its
// feature slices from the column slices of x and dy (ln_cols_*); `part` is unused and
// (dscale, dbias) are written directly.  The first column loads go out before the row work.
template <typename T, int TPR, int TEAMS, int V, bool WGRAD, bool COLS = false>
__global__ void __launch_bounds__((RowBlock<TPR, TEAMS>::kThreads))
ln_bwd_rows(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ dx, int64_t ldx,
            int64_t lddy, int64_t lddx, RowMap map, int64_t rows, int nvec, int n, float eps,
            const float* __restrict__ stats, int64_t ld_stats, float* __restrict__ sgrad,
            int64_t ld_sgrad, const float* __restrict__ gamma, float* __restrict__ part,
            float* __restrict__ dscale, float* __restrict__ dbias, int tail = 0, int col_blocks = 0)
{
  static_assert(!(WGRAD && COLS), "one way of forming the weight gradients");
  using B = RowBlock<TPR, TEAMS>;
  using IO = Vec16<T>;
  using raw_t = typename IO::raw_t;
  constexpr int VE = IO::N;
  // a last vector of `tail` entries, read as the row's last VE entries: see ln_fwd_rows
  constexpr bool kTail = UnalignedVec<T>::value;
  static_assert(!kTail || !COLS, "rows with a partial vector do not form weight gradients from column slices");
  constexpr bool kSub = TPR < kWave;
  static_assert(!kSub || TPR == 16, "sub-wave teams are one DPP row wide");
  constexpr int NW = kSub ? 1 : B::kWavesPerTeam;
  constexpr int kAccLds = (WGRAD && TEAMS > 1) ? 2 * TPR * V * VE : 1;
  constexpr bool kPrefetch = V * VE < 32;
  __shared__ float red[2][TEAMS][2 * NW];
  __shared__ float acc_lds[kAccLds];
  constexpr int kColLds = COLS ? 2 * (B::kThreads / 8) * (8 * VE + 1) : 1;
  __shared__ float col_lds[kColLds];
  const int tid = threadIdx.x;
  const int team = kSub ? tid / TPR : wave_index() / NW;
  const int t = tid - team * TPR;
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;

  // COLS: the last col_blocks workgroups of the grid form the weight gradients from column slices
  // and nothing else, the others walk rows and nothing else: neither waits for the other, since
  // both read inputs of the call only (col_blocks == 0: every workgroup does both, in turn).
  const int row_grid = COLS ? static_cast<int>(gridDim.x) - col_blocks : static_cast<int>(gridDim.x);
  const bool col_block = COLS && col_blocks > 0 && static_cast<int>(blockIdx.x) >= row_grid;
  const bool row_block = !col_block;
  const int64_t first_slice = col_block ? static_cast<int64_t>(blockIdx.x) - row_grid : blockIdx.x;
  const int64_t slice_step = (COLS && col_blocks > 0) ? col_blocks : gridDim.x;
  LnColLoads<T> cols;
  const int64_t col_slices = (n + 8 * VE - 1) / (8 * VE);
  if constexpr (COLS) {
    if (col_block || col_blocks == 0)
      ln_cols_issue<T, B::kThreads>(cols, x, dy, ldx, lddy, map, rows, n, stats, ld_stats, first_slice, 0);
  }

  // Loads are issued unconditionally: a row past the end re-reads the last row, a
  // vector past the end of a row re-reads vector 0.
  bool ok[V];
  int voff[V];
  int skip[V];  // leading entries of the vector that belong to its neighbour
#pragma unroll
  for (int i = 0; i < V; ++i) {
    ok[i] = t + i * TPR < nvec;
    voff[i] = ok[i] ? VE * (t + i * TPR) : 0;
    skip[i] = 0;
    if (kTail && tail && t + i * TPR == nvec - 1) {
      skip[i] = VE - tail;
      voff[i] -= skip[i];
    }
  }
  float gam[V][VE];
#pragma unroll
  for (int i = 0; i < V; ++i) {
#pragma unroll
    for (int k = 0; k < VE; ++k) gam[i][k] = 1.f;
    if (gamma && ok[i]) {
      if constexpr (kTail) __builtin_memcpy(gam[i], gamma + voff[i], sizeof(float) * VE);
      else load_f32_run<VE>(gamma + voff[i], gam[i]);
    }
  }
  float dg[WGRAD ? V : 1][VE], db[WGRAD ? V : 1][VE];
  if (WGRAD) {
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < VE; ++k) dg[i][k] = db[i][k] = 0.f;
  }

  // A row in flight: its still-packed 16-byte vectors and its two statistics.
  struct Slot {
    raw_t x[V], g[V];
    float mean, var;
  };
  // All row arithmetic is wave-uniform (scalar registers).
  auto issue = [&](Slot& s, int64_t row) {
    int64_t col, g;
    map.split(row < rows ? row : rows - 1, col, g);
    const T* xr = x + g * map.stride + col * ldx;
    const T* gr = dy + g * map.stride + col * lddy;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      s.x[i] = IO::load_raw(xr + voff[i]);
      using F = typename FreshInput<T>::type;  // dy through ordinary loads also beside a streamed x
      s.g[i] = Vec16<F>::load_raw(reinterpret_cast<const F*>(gr + voff[i]));
    }
    s.mean = stats[g + col * ld_stats];
    s.var = stats[map.groups + g + col * ld_stats];
  };

  const float inv_n = 1.0f / static_cast<float>(n);
  const int64_t rows_per_iter = static_cast<int64_t>(row_grid) * TEAMS;
  const int64_t iters = row_block ? (rows + rows_per_iter - 1) / rows_per_iter : 0;
  const int64_t first_row = static_cast<int64_t>(blockIdx.x) * TEAMS + team;

  // One row: s holds it on entry and, after its registers are unpacked, is refilled
  // (refill) with the team's next row, which stays in flight until its turn.
  // full: the row exists and every thread owns V whole vectors of it, so nothing is
  // masked.
  auto process = [&](Slot& s, int64_t it, auto refill, auto full) {
    constexpr bool kFull = decltype(full)::value;
    const int64_t row = it * rows_per_iter + first_row;
    const bool active = kFull || row < rows;
    if constexpr (!kPrefetch) issue(s, row);
    const float mean = s.mean;
    const float inv_stdev = rsqrt_refined(s.var + eps);
    float xh[V][VE], gs[V][VE];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      IO::unpack(s.x[i], xh[i]);
      IO::unpack(s.g[i], gs[i]);
    }
    if constexpr (kPrefetch && decltype(refill)::value) issue(s, row + rows_per_iter);
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const bool use_vec = kFull || (active && ok[i]);
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        // masked entries (re-read data of another vector or row) count as x = mean, dy = 0
        const bool use = use_vec && !(kTail && k < skip[i]);
        const float gv = use ? gs[i][k] : 0.f;
        xh[i][k] = use ? (xh[i][k] - mean) * inv_stdev : 0.f;  // subtract first: x*inv - mean*inv would cancel
        if (WGRAD) {
          db[i][k] += gv;
          dg[i][k] = __builtin_fmaf(gv, xh[i][k], dg[i][k]);
        }
        gs[i][k] = gv * gam[i][k];
        a += gs[i][k];
        b = __builtin_fmaf(gs[i][k], xh[i][k], b);
      }
    }
    if constexpr (kSub) {
      a = row16_sum(a);
      b = row16_sum(b);
    }
    else {
      team_sum2<NW>(a, b, red[it & 1][team], wv, lane);
    }
    if (active) {
      int64_t col, g;
      map.split(row, col, g);
      const float dmean = -a * inv_stdev;
      const float dvar = -b * inv_stdev * inv_stdev * 0.5f;
      if (t == 0) {
        sgrad[g + col * ld_sgrad] = dmean;
        sgrad[map.groups + g + col * ld_sgrad] = dvar;
      }
      const float c0 = dmean * inv_n;
      const float c1 = -b * inv_stdev * inv_n;  // dvar * 2 / n, per unit of xh = (x - mean) / stdev
      T* dr = dx + g * map.stride + col * lddx;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (kFull || ok[i]) {
#pragma unroll
          for (int k = 0; k < VE; ++k)
            gs[i][k] = __builtin_fmaf(gs[i][k], inv_stdev, __builtin_fmaf(c1, xh[i][k], c0));
          bool whole = true;
          if constexpr (kTail) {
            if (skip[i]) {
              whole = false;
#pragma unroll
              for (int k = 0; k < VE; ++k)
                if (k >= skip[i]) IO::store1(dr + voff[i] + k, gs[i][k]);
            }
          }
          if (whole) IO::store(dr + voff[i], gs[i]);
        }
      }
    }
  };

  // The main loop covers the iterations in which every team has a row; the last,
  // partly filled iteration is masked.
  Slot q;
  if constexpr (kPrefetch) {
    if (row_block) issue(q, first_row);
  }
  const int64_t full_iters = row_block ? rows / rows_per_iter : 0;
  int64_t it = 0;
  if (nvec == TPR * V && !(kTail && tail)) {
    for (; it < full_iters; ++it) process(q, it, std::true_type{}, std::true_type{});
  }
  else {
    for (; it < full_iters; ++it) process(q, it, std::true_type{}, std::false_type{});
  }
  if (it < iters) process(q, it, std::false_type{}, std::false_type{});

  if constexpr (COLS) {
    constexpr int64_t kRowsPerPass = 4 * (B::kThreads / 8);
    for (int64_t slice = first_slice; (col_block || col_blocks == 0) && slice < col_slices; slice += slice_step) {
      float cg[VE], cb[VE];
#pragma unroll
      for (int e = 0; e < VE; ++e) cg[e] = cb[e] = 0.f;
      for (int64_t row0 = 0; row0 < rows; row0 += kRowsPerPass) {
        if (slice != first_slice || row0 != 0)
          ln_cols_issue<T, B::kThreads>(cols, x, dy, ldx, lddy, map, rows, n, stats, ld_stats, slice, row0);
        ln_cols_accumulate<T, B::kThreads>(cols, rows, n, eps, slice, row0, cg, cb);
      }
      ln_cols_finish<T, B::kThreads>(col_lds, n, slice, cg, cb, dscale, dbias);
    }
  }

  if (WGRAD) {
    float* out = part + static_cast<int64_t>(blockIdx.x) * 2 * n;
    if (TEAMS > 1) {
      // teams add their register accumulators into LDS one after another
      float* lg = acc_lds;
      float* lb = acc_lds + TPR * V * VE;
      for (int tm = 0; tm < TEAMS; ++tm) {
        if (team == tm) {
#pragma unroll
          for (int i = 0; i < V; ++i)
#pragma unroll
            for (int k = 0; k < VE; ++k) {
              // (a vector past the end of the row keeps a slot of its own behind the row's entries)
              const int p = (kTail && ok[i]) ? voff[i] + k : (t + i * TPR) * VE + k;
              if (kTail && k < skip[i]) continue;  // the neighbour's entry
              if (tm == 0) {
                lg[p] = dg[i][k];
                lb[p] = db[i][k];
              }
              else {
                lg[p] += dg[i][k];
                lb[p] += db[i][k];
              }
            }
        }
        __syncthreads();
      }
      for (int p = tid; p < n; p += B::kThreads) {
        out[p] = lg[p];
        out[n + p] = lb[p];
      }
    }
    else {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (!ok[i]) continue;
        if constexpr (kTail) {
          if (skip[i]) {
#pragma unroll
            for (int k = 0; k < VE; ++k)
              if (k >= skip[i]) {
                out[voff[i] + k] = dg[i][k];
                out[n + voff[i] + k] = db[i][k];
              }
          }
          else {
            __builtin_memcpy(out + voff[i], dg[i], sizeof(float) * VE);
            __builtin_memcpy(out + n + voff[i], db[i], sizeof(float) * VE);
          }
        }
        else {
          store_f32_run<VE>(out + voff[i], dg[i]);
          store_f32_run<VE>(out + n + voff[i], db[i]);
        }
      }
    }
  }
}

// Sums P partial rows: grid (ceil(n/32), 2): y == 0 dscale, y == 1 dbias.  A block is
// 8 groups of four feature columns x 32 row groups; a thread has its (up to 8) 16-byte
// loads in flight together, so the kernel costs about one trip to memory.  The order
// of additions is fixed.  n is a multiple of 4 and part is 16-byte aligned.
__global__ void __launch_bounds__(256)
ln_wgrad_reduce(const float* __restrict__ part, int64_t P, int64_t n, float* __restrict__ dscale,
                float* __restrict__ dbias)
{
  __shared__ float sm[32][33];
  __shared__ float sm2[8][33];
  float* out = blockIdx.y == 0 ? dscale : dbias;
  if (!out) return;
  const int kq = threadIdx.x & 7;   // column quad
  const int pg = threadIdx.x >> 3;  // row group
  const int64_t k = static_cast<int64_t>(blockIdx.x) * 32 + 4 * kq;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (k < n) {
    const float* src = part + blockIdx.y * n + k;
    for (int64_t p0 = pg; p0 < P; p0 += 256) {
      float w[8][4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int64_t p = p0 + 32 * j;
        if (p < P) {
          Vec16<float>::load(src + p * 2 * n, w[j]);
        }
        else {
#pragma unroll
          for (int c = 0; c < 4; ++c) w[j][c] = 0.f;
        }
      }
#pragma unroll
      for (int c = 0; c < 4; ++c)
        acc[c] += ((w[0][c] + w[1][c]) + (w[2][c] + w[3][c])) + ((w[4][c] + w[5][c]) + (w[6][c] + w[7][c]));
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) sm[pg][4 * kq + c] = acc[c];
  __syncthreads();
  {
    const int c = threadIdx.x & 31, o = threadIdx.x >> 5;
    sm2[o][c] = (sm[4 * o][c] + sm[4 * o + 1][c]) + (sm[4 * o + 2][c] + sm[4 * o + 3][c]);
  }
  __syncthreads();
  if (threadIdx.x < 32) {
    const int c = threadIdx.x;
    const int64_t kc = static_cast<int64_t>(blockIdx.x) * 32 + c;
    if (kc < n)
      out[kc] = ((sm2[0][c] + sm2[1][c]) + (sm2[2][c] + sm2[3][c])) + ((sm2[4][c] + sm2[5][c]) + (sm2[6][c] + sm2[7][c]));
  }
}

// One 256-thread block per row, scalar access; weight gradients are left to
// ln_wgrad_generic.
template <typename T>
__global__ void __launch_bounds__(256)
ln_bwd_generic(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ dx, int64_t ldx,
               int64_t lddy, int64_t lddx, RowMap map, int64_t n, float eps,
               const float* __restrict__ stats, int64_t ld_stats, float* __restrict__ sgrad,
               int64_t ld_sgrad, const float* __restrict__ gamma)
{
  using IO = Vec16<T>;
  __shared__ float red[8];
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
  float a = 0.f, b = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 256) {
    float d = IO::load1(gr + i);
    if (gamma) d *= gamma[i];
    a += d;
    b += d * (IO::load1(xr + i) - mean);
  }
  team_sum2<4>(a, b, red, wv, lane);
  const float dmean = -a * inv_stdev;
  const float dvar = -b * inv_stdev * inv_stdev * inv_stdev / 2;
  if (threadIdx.x == 0) {
    sgrad[g + col * ld_sgrad] = dmean;
    sgrad[map.groups + g + col * ld_sgrad] = dvar;
  }
  const float nf = static_cast<float>(n);
  const float c0 = dmean / nf;
  const float c1 = dvar * 2.f / nf;
  for (int64_t i = threadIdx.x; i < n; i += 256) {
    float d = IO::load1(gr + i);
    if (gamma) d *= gamma[i];
    IO::store1(dr + i, d * inv_stdev + c0 + c1 * (IO::load1(xr + i) - mean));
  }
}

// dscale[k] = sum over rows of dy * (x - mean) / stdev, dbias[k] = sum of dy.
// One thread per feature k walks all rows (coalesced across k).
template <typename T>
__global__ void __launch_bounds__(256)
ln_wgrad_generic(const T* __restrict__ x, const T* __restrict__ dy, int64_t ldx, int64_t lddy,
                 RowMap map, int64_t rows, int64_t n, float eps, const float* __restrict__ stats,
                 int64_t ld_stats, float* __restrict__ dscale, float* __restrict__ dbias)
{
  using IO = Vec16<T>;
  const int64_t k = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (k >= n) return;
  float sg = 0.f, sb = 0.f;
  for (int64_t row = 0; row < rows; ++row) {
    int64_t col, g;
    map.split(row, col, g);
    const float mean = stats[g + col * ld_stats];
    const float inv_stdev = 1.0f / sqrtf(stats[map.groups + g + col * ld_stats] + eps);
    const float d = IO::load1(dy + g * map.stride + col * lddy + k);
    sb += d;
    sg += d * (IO::load1(x + g * map.stride + col * ldx + k) - mean) * inv_stdev;
  }
  if (dscale) dscale[k] = sg;
  if (dbias) dbias[k] = sb;
}

template <typename T>
__global__ void __launch_bounds__(256)
fill_matrix(T* p, int64_t h, int64_t w, int64_t ld, float value)
{
  const int64_t total = h * w;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t c = i / h;
    Vec16<T>::store1(p + (i - c * h) + c * ld, value);
  }
}

// ==================================================================== host side
// Shape of the persistent backward launch that produces weight gradients.
struct LnBwdPlan {
  int tpr, teams, v;
  int64_t blocks;  // == number of partial rows
};

// Persistent blocks: each leaves 2*n floats of partial sums, which are written once
// and read once, so fewer blocks mean less extra traffic, while more blocks hide more
// latency.  One block per compute unit (256) is the floor; the count doubles (up to
// 1024) as long as the partial sums stay below 1/20 of the tensor traffic.
constexpr int64_t kLnBwdMinBlocks = 256;
constexpr int64_t kLnBwdMaxBlocks = 1024;

static int64_t ln_bwd_block_limit(int64_t rows, int elem_bytes)
{
  static const int64_t forced = std::getenv("LBN_LN_BWD_BLOCKS") ? std::atoi(std::getenv("LBN_LN_BWD_BLOCKS")) : 0;
  if (forced > 0) return forced;
  // partial traffic / tensor traffic = blocks * 2n * 4 * 2 / (3 * rows * n * elem_bytes)
  int64_t blocks = kLnBwdMinBlocks;
  while (blocks < kLnBwdMaxBlocks && 2 * blocks * 16 * 20 <= 3 * rows * elem_bytes) blocks *= 2;
  return blocks;
}

// Blocks have at most 512 threads, which leaves every thread 256 registers: per owned
// entry a thread keeps the scale, two fp32 accumulators and two fp32 working values.
// Narrow teams with several vectors per thread spend the least on the row reduction,
// so the narrowest team that owns at most 16 entries per thread is taken; rows too
// long for that go to 512-thread teams with up to 32 entries per thread.
static LnBwdPlan plan_ln_bwd(int64_t nvec, int64_t rows, int ve, int elem_bytes, bool wgrad = true)
{
  static const int force_tpr = std::getenv("LBN_LN_BWD_TPR") ? std::atoi(std::getenv("LBN_LN_BWD_TPR")) : 0;
  static const int force_teams = std::getenv("LBN_LN_BWD_TEAMS") ? std::atoi(std::getenv("LBN_LN_BWD_TEAMS")) : 0;
  const int64_t max_blocks = ln_bwd_block_limit(rows, elem_bytes);
  LnBwdPlan p{0, 0, 0, 0};
  const int tprs[3] = {64, 256, 512};
  const int teams[3] = {4, 2, 1};
  // at most 8 access units per thread are instantiated
  const int v_pref = 16 / ve < 8 ? 16 / ve : 8, v_max = 32 / ve < 8 ? 32 / ve : 8;
  int pick = -1;
  for (int pass = 0; pass < 2 && pick < 0; ++pass)
    for (int i = 0; i < 3 && pick < 0; ++i) {
      if (force_tpr && tprs[i] != force_tpr) continue;
      const int64_t v = ceil_div(nvec, tprs[i]);
      // 32 entries per thread are instantiated for the widest team only
      if (v <= (pass == 0 ? v_pref : (tprs[i] == 512 || force_tpr ? v_max : v_pref))) pick = i;
    }
  if (pick < 0) return p;
  p.tpr = tprs[pick];
  p.teams = teams[pick];
  p.v = round_up_pow2_le8(ceil_div(nvec, p.tpr));
  if (!force_tpr && nvec <= (wgrad ? 32 : 64) && rows >= 4096) {
    // many short rows: teams of 16 lanes, four rows per wave (four vectors per lane only without
    // weight gradients, whose accumulators would double the registers: fp32 rows of 132 entries x
    // 131072 backward 41 -> 35 us without, 45 -> 48 us with them)
    p.tpr = 16;
    p.teams = 16;
    p.v = nvec <= 16 ? 1 : nvec <= 32 ? 2 : 4;
  }
  if (force_teams && force_teams <= p.teams) p.teams = force_teams;
  // spread small problems: fewer teams per block when rows are scarce
  while (p.teams > 1 && p.tpr * p.teams > 256 && ceil_div(rows, p.teams) < kLnBwdMinBlocks) p.teams /= 2;
  p.blocks = ceil_div(rows, p.teams);
  if (p.blocks > max_blocks) p.blocks = max_blocks;
  return p;
}

// Problems whose weight gradients the backward kernel forms itself from column slices (a
// second read of x and dy, served by the caches): few rows, and tensors that fit the caches.
static bool ln_bwd_small(int64_t rows, int64_t n, int elem_bytes)
{
  static const bool off = std::getenv("LBN_LN_NO_FUSED_WGRAD") != nullptr;
  // (us with / without, fp32: 1024 x 128 rows 4.3 / 7.0; 4096 x 512 8.5 / 13.7; 2048 x 1024 7.9 / 10.4;
  // 1024 x 1024 8.4 / 8.7; beyond 1024 rows the column walk is the longer chain: 1024 x 2048 16.1 / 9.5)
  return !off && rows <= 1024 && rows * n * elem_bytes <= (int64_t(8) << 20);
}

// Row slabs of ln_wgrad_columns: about 2048 workgroups in total, at most one slab per row.
static int64_t ln_wgrad_slabs(int64_t units, int64_t rows)
{
  int64_t s = ceil_div(2048, ceil_div(units, 256));
  if (s > rows) s = rows;
  if (s > 256) s = 256;
  return s < 1 ? 1 : s;
}

// fp16 rows that can be walked in 4-byte pairs: even offsets everywhere.
static bool rows_aligned4(const void* base, int64_t stride, int64_t ld, int64_t groups, int64_t width)
{
  return (reinterpret_cast<uintptr_t>(base) & 3u) == 0 && (groups <= 1 || stride % 2 == 0) &&
         (width <= 1 || ld % 2 == 0);
}

// LBN_LN_NO_UNALIGNED_ROWS=1 keeps rows off the 16-byte grid away from the register kernels
// with unaligned 16-byte accesses: single floats, pairs of halves, the two-pass kernels and
// the generic kernels serve them instead (for tests of those paths).
static bool ln_no_unaligned_rows()
{
  static const bool on = std::getenv("LBN_LN_NO_UNALIGNED_ROWS") != nullptr;
  return on;
}

// fp16 rows of even length on the 4-byte grid can be walked in pairs or in 16-byte vectors at
// 2-byte alignment.  Pairs give a short row more loads in flight per lane (258 x 65536 forward:
// 22 against 28 us) and are kept up to 512 entries and wherever weights have gradients (1002 x
// 16384 backward: 28 against 33 us); longer rows take the vectors (2050 x 8192 forward: 22
// against 45 us), and so do rows of 65 to 256 entries when there are many: 32 vectors hold them,
// a team of 16 lanes each (130 x 131072: 22 / 23 us against 32 / 37).
constexpr int64_t kLnPairsMaxFwd16 = 512;

static bool ln_pairs_first(int64_t n, int64_t rows)
{
  if (ln_no_unaligned_rows()) return true;
  return n <= kLnPairsMaxFwd16 && !(n > 64 && n <= 256 && rows >= 4096);
}

// With weight gradients the pairs stay, except where 16 vectors hold one of many rows
// (66 x 262144 backward: 46 against 78 us; 130 x 131072: 62 against 52 us).
static bool ln_pairs_first_wgrad(int64_t n, int64_t rows)
{
  if (ln_no_unaligned_rows()) return true;
  return !(n > 64 && n <= 128 && rows >= 4096);
}

// fp32 rows off the 16-byte grid can be walked one float at a time or in 16-byte vectors at
// 4-byte alignment (the last n % 4 entries in a vector that overlaps its neighbour).  Vectors
// win where 32 of them hold a row (teams of 16 lanes; 35 x 262144: 20 / 22 us against 49 / 62)
// and beyond `longer_than` entries (2049 x 8192 forward: 26 against 47 us; 1025 x 16384
// backward with weight gradients: 43 against 53 us); between, single floats are as fast or
// a little faster (1001 x 16384 backward: 32 against 34 us).
// team_units: the most vectors that a team of 16 lanes takes (64 forward, 32 with weight gradients).
static bool ln_vectors_first(int64_t n, int64_t longer_than, int64_t rows, int64_t team_units)
{
  if (n < 4 || ln_no_unaligned_rows()) return false;
  return (ceil_div(n, 4) <= team_units && rows >= 4096) || n > longer_than;
}

constexpr int64_t kLnLongMin16 = 4096;  // shortest fp16 row of odd length that takes a 1024-thread workgroup of its own (1001 entries: 75 against 40 us)
constexpr int64_t kLnMaxScalarRowFwd = 8192;  // rows accessed one float at a time: 1024 threads x 8
constexpr int64_t kLnMaxScalarRowBwd = 4096;  // 512 threads x 8

// ---- rows longer than the register kernels hold: clusters of workgroups (layer_norm_cluster.hpp)

static size_t ln_cluster_slot_bytes(int64_t rows, int M)
{
  return 64 + static_cast<size_t>(rows) * M * 2 * sizeof(unsigned long long);
}

// Partial rows of the weight gradients start on a 256-byte boundary behind the slots.
static size_t ln_cluster_part_offset(int64_t rows, int M) { return (ln_cluster_slot_bytes(rows, M) + 255) & ~size_t(255); }

// Workspace of the cluster path for rows of n entries (0: the shape does not take it).
static size_t ln_cluster_fwd_workspace(int64_t n, int64_t rows, int ve)
{
  if (n % ve != 0 || n / ve >= (int64_t(1) << 31)) return 0;
  // register clusters (a launch may widen them up to the maximum) or, beyond their reach, streaming clusters
  return ln_cluster_slot_bytes(rows, kLnClMaxM);
}

static size_t ln_cluster_bwd_workspace(int64_t n, int64_t rows, int ve)
{
  if (n % ve != 0) return 0;
  const ClusterPlan cp = plan_ln_cluster(n / ve, kLnClBwdUnits / (kLnClThreads * ve));
  if (!cp.M) return 0;  // rows beyond the register clusters keep the two-pass kernels when weights have gradients
  return ln_cluster_part_offset(rows, kLnClMaxM) +
         static_cast<size_t>(ln_cluster_count_bound(rows, cp.M)) * 2 * n * sizeof(float);
}

// ve: entries per 16-byte vector of the storage type (4: fp32, 8: fp16).  The size does not
// depend on pointers or leading dimensions, which the query does not see, so it covers
// every path the shape can take: 16-byte vectors, single floats, row slabs.
static size_t ln_bwd_workspace(int64_t n, int64_t rows, int ve)
{
  if (n <= 0 || rows <= 0) return 0;
  const int elem_bytes = 16 / ve;
  // partial rows of the multi-kernel paths sit behind the header that the cluster kernels own
  const size_t H = kWorkspaceHeaderBytes;
  size_t need = H + static_cast<size_t>(ln_wgrad_slabs(n, rows)) * 2 * n * sizeof(float);
  auto cover = [&](size_t bytes) { if (bytes > need) need = bytes; };
  if (n % ve == 0) {
    const LnBwdPlan p = plan_ln_bwd(n / ve, rows, ve, elem_bytes);
    if (p.tpr) cover(H + static_cast<size_t>(p.blocks) * 2 * n * sizeof(float));
    else cover(H + static_cast<size_t>(ln_wgrad_slabs(n / ve, rows)) * 2 * n * sizeof(float));
    if (!p.tpr) cover(ln_cluster_bwd_workspace(n, rows, ve));  // long rows: slots, then one partial row per cluster
  }
  if (ve == 4 && n <= kLnMaxScalarRowBwd) {  // fp32 rows off the 16-byte grid: one float per access
    const LnBwdPlan p = plan_ln_bwd(n, rows, 1, 4);
    if (p.tpr) cover(H + static_cast<size_t>(p.blocks) * 2 * n * sizeof(float));
  }
  if (n >= ve) {  // rows off the 16-byte grid: a last, partial vector counts as a unit
    const LnBwdPlan p = plan_ln_bwd(ceil_div(n, ve), rows, ve, elem_bytes);
    if (p.tpr) cover(H + static_cast<size_t>(p.blocks) * 2 * n * sizeof(float));
  }
  if (ve == 8 && n % 2 == 0 && n / 2 <= kLnMaxScalarRowBwd) {  // fp16 rows: one pair per access
    const LnBwdPlan p = plan_ln_bwd(n / 2, rows, 2, 2);
    if (p.tpr) cover(H + static_cast<size_t>(p.blocks) * 2 * n * sizeof(float));
  }
  return need;
}

// Workgroups of the row kernels that form no weight gradients, for `work` rows per team slot and
// `resident` workgroups that the device holds at once.  One resident wave of workgroups, each
// walking the same number of rows with the next row in flight, was the first design; workgroups
// that live for two rows only, far more than are resident, measure faster wherever that differs
// (forward, % of 8 TB/s with every call's tensors out of the caches, persistent -> two rows: rows of
// 64 / 256 / 1024 / 4096 floats at 64 MiB per tensor 74 / 79 / 78 / 80 -> 80 / 81 / 81 / 80, at
// 256 MiB 66 / 74 / 73 / 74 -> 74 / 76 / 76 / 75; fp16 4096 x 8192 on the same buffers 25.0 -> 24.0 us).
// Backward only gains on rows of up to 2 KiB (128- and 512-float rows at 196 MiB per tensor: 68 / 66
// -> 75 / 75) and loses on longer ones (3136 floats: 77 -> 64), which keep the resident wave.
static int64_t ln_row_grid(int64_t work, int64_t resident, bool short_lived)
{
  const int64_t rounds = ceil_div(work, resident);
  if (short_lived && rounds > 2) return ceil_div(work, 2);
  return ceil_div(work, rounds);
}

// Register-resident forward over rows of `units` access units (16-byte vectors, or single
// floats for ST = f32x1).  Returns 1 when launched, 0 when no configuration holds the row,
// -1 when the occupancy query fails.
template <typename ST>
static int ln_fwd_rows_launch(hipStream_t st, const ST* x, ST* y, int64_t ldx, int64_t ldy, RowMap map,
                              int64_t rows, int64_t units, float inv_n, float eps, float* stats, int64_t lds,
                              const float* gamma, const float* beta, int sumsq, int tail = 0)
{
  // tail: entries of a last, partial unit that `units` counts (storage types with unaligned access only)
  constexpr int VE = Vec16<ST>::N;
  RowConfig c = pick_row_config(units, rows, 8);
  // many short rows: teams of 16 lanes, four rows per wave, instead of mostly idle waves
  // (layer norm rows of 64 entries x 65536: 60 us per step against 150 us with one wave per row;
  // at 64 units per row the two shapes measure the same and the wave-wide team is kept)
  // (up to 64 units with four per lane: fp16 rows of 512 entries x 65536 26 -> 24 us, fp32 rows of
  // 132 x 131072 32 -> 27 us)
  if (units <= 64 && rows >= 4096) c = {16, units <= 16 ? 1 : units <= 32 ? 2 : 4};
  // single floats cost one register each: rows just past 256, 512 or 1024 entries stay with one
  // wave (or four) holding 8 or 16 of them instead of four (or sixteen) waves holding two
  // (257 x 65536: 59 us forward, 1025 x 16384: 81 us that way)
  // 16-bit rows of 8193 to 16384 entries: 512 threads with four vectors each, two workgroups per
  // compute unit, instead of 1024 threads with two, one workgroup per unit (4096 rows of 10240:
  // 98.3 -> 90.7 us per step; of 12288 and 16384: 1 %)
  if (VE == 8 && units > 1024 && units <= 2048 && rows >= 512) c = {512, 4};
  if (VE == 1 && rows >= 2048) {
    if (units > 256 && units <= 512) c = {64, 8};
    else if (units > 512 && units <= 1024) c = {64, 16};
    else if (units > 1024 && units <= 2048) c = {256, 8};
  }
  if (!c.tpr) return 0;
  const int nvec = static_cast<int>(units);
#define X(TPR, V)                                                                              \
  if (c.tpr == TPR && c.v == V) {                                                              \
    using B = RowBlock<TPR>;                                                                   \
    const int64_t work = ceil_div(rows, B::kTeams);                                            \
    const int64_t resident = resident_blocks(ln_fwd_rows<ST, TPR, V>, B::kThreads);            \
    if (resident <= 0) return -1;                                                              \
    const int64_t grid = ln_row_grid(work, resident, true);                                    \
    hipLaunchKernelGGL((ln_fwd_rows<ST, TPR, V>), dim3(static_cast<unsigned>(grid)),           \
                       dim3(B::kThreads), 0, st, x, y, ldx, ldy, map, rows, nvec, inv_n, eps,  \
                       stats, lds, gamma, beta, sumsq, tail);                                  \
    return 1;                                                                                  \
  }
  X(16, 1) X(16, 2) X(16, 4)
  X(64, 1) X(64, 2) X(64, 4) X(256, 1) X(256, 2) X(256, 4) X(1024, 1) X(1024, 2) X(1024, 4)
  X(64, 8) X(256, 8)
  if constexpr (VE == 8) { X(512, 4) }
  if constexpr (VE <= 4) { X(1024, 8) }
  if constexpr (VE == 1) { X(64, 16) }
#undef X
  return 0;
}

// Both return 1 when launched, 0 when the shape, the workspace or the device's capacity does
// not allow the cluster path (the caller goes on to the two-pass kernels).
template <typename T>
static int ln_fwd_cluster_launch(hipStream_t st, const T* x, T* y, int64_t ldx, int64_t ldy, RowMap map,
                                 int64_t rows, int64_t n, float eps, float* stats, int64_t lds,
                                 const float* gamma, const float* beta, int sumsq, void* ws, size_t ws_bytes)
{
  constexpr int VE = Vec16<T>::N;
  constexpr int kMaxV = kLnClFwdUnits / (kLnClThreads * VE);
  const ClusterPlan cp = plan_ln_cluster(n / VE, kMaxV);
  if (!cp.M || !ws || !aligned16(ws)) return 0;
  const ClusterWorkspace cw = cluster_workspace(ws);
  const bool affine = gamma || beta;
#define X(VV)                                                                                        \
  if (cp.V == VV) {                                                                                  \
    const int cap = affine ? cluster_capacity(ln_fwd_cluster<T, VV, true>, kLnClThreads)             \
                           : cluster_capacity(ln_fwd_cluster<T, VV, false>, kLnClThreads);           \
    const LnClusterLaunch l = plan_ln_cluster_launch(n / VE, rows, cp, cap, rows);                   \
    if (!l.M || l.V > VV || ws_bytes < ln_cluster_slot_bytes(rows, l.M)) return 0;                   \
    LnClArgs<T> a{};                                                                                 \
    a.x = x, a.out = y, a.ldx = ldx, a.ldo = ldy, a.map = map, a.rows = rows, a.n = n;               \
    a.nvec = static_cast<unsigned>(n / VE), a.per_wg = l.per_wg, a.M = l.M, a.sumsq = sumsq;         \
    a.inv_n = 1.0f / static_cast<float>(n), a.eps = eps, a.stats = stats, a.ld_stats = lds;          \
    ClusterLaunchGuard guard(st);                                                                    \
    if (guard.failed()) return 0;                                                                    \
    a.gamma = gamma, a.beta = beta, a.cw = cw, a.tag = cluster_call_tag(st, cw);                     \
    const dim3 grid(static_cast<unsigned>(l.clusters * l.M));                                        \
    if (affine) hipLaunchKernelGGL((ln_fwd_cluster<T, VV, true>), grid, dim3(kLnClThreads), 0, st, a); \
    else hipLaunchKernelGGL((ln_fwd_cluster<T, VV, false>), grid, dim3(kLnClThreads), 0, st, a);     \
    return 1;                                                                                        \
  }
  X(1) X(2)
  if constexpr (kMaxV >= 4) { X(3) X(4) }
#undef X
  return 0;
}

template <typename T>
static int ln_bwd_cluster_launch(hipStream_t st, bool wgrad, const T* x, const T* dy, T* dx, int64_t ldx,
                                 int64_t lddy, int64_t lddx, RowMap map, int64_t rows, int64_t n, float eps,
                                 const float* stats, int64_t lds, float* sgrad, int64_t ldsg,
                                 const float* gamma, float* dgamma, float* dbeta, void* ws, size_t ws_bytes)
{
  constexpr int VE = Vec16<T>::N;
  constexpr int kMaxV = kLnClBwdUnits / (kLnClThreads * VE);
  const ClusterPlan cp = plan_ln_cluster(n / VE, kMaxV);
  if (!cp.M || !ws || !aligned16(ws)) return 0;
  const size_t need = wgrad ? ln_cluster_bwd_workspace(n, rows, VE) : ln_cluster_slot_bytes(rows, kLnClMaxM);
  if (ws_bytes < need) return 0;
  const ClusterWorkspace cw = cluster_workspace(ws);
  float* wpart = reinterpret_cast<float*>(static_cast<char*>(ws) + ln_cluster_part_offset(rows, kLnClMaxM));
#define X(VV)                                                                                        \
  if (cp.V == VV) {                                                                                  \
    const int cap = wgrad ? cluster_capacity(ln_bwd_cluster<T, VV, true>, kLnClThreads)              \
                          : cluster_capacity(ln_bwd_cluster<T, VV, false>, kLnClThreads);            \
    const LnClusterLaunch l = plan_ln_cluster_launch(n / VE, rows, cp, cap, ln_cluster_count_bound(rows, cp.M)); \
    if (!l.M || l.V > VV) return 0;                                                                  \
    const int64_t nc = l.clusters;                                                                   \
    LnClArgs<T> a{};                                                                                 \
    a.x = x, a.dy = dy, a.out = dx, a.ldx = ldx, a.lddy = lddy, a.ldo = lddx, a.map = map;           \
    a.rows = rows, a.n = n, a.nvec = static_cast<unsigned>(n / VE), a.per_wg = l.per_wg, a.M = l.M;  \
    a.inv_n = 1.0f / static_cast<float>(n), a.eps = eps, a.stats = const_cast<float*>(stats);        \
    a.ld_stats = lds, a.sgrad = sgrad, a.ld_sgrad = ldsg, a.gamma = gamma, a.wpart = wpart;          \
    ClusterLaunchGuard guard(st);                                                                    \
    if (guard.failed()) return 0;                                                                    \
    a.cw = cw, a.tag = cluster_call_tag(st, cw);                                                     \
    const dim3 grid(static_cast<unsigned>(nc * l.M));                                                \
    if (wgrad) {                                                                                     \
      hipLaunchKernelGGL((ln_bwd_cluster<T, VV, true>), grid, dim3(kLnClThreads), 0, st, a);         \
      hipLaunchKernelGGL(ln_wgrad_reduce_wide, dim3(static_cast<unsigned>(ceil_div(n / 2, 256))), dim3(256), 0, \
                         st, wpart, nc, n, dgamma, dbeta);                                           \
    }                                                                                                \
    else {                                                                                           \
      hipLaunchKernelGGL((ln_bwd_cluster<T, VV, false>), grid, dim3(kLnClThreads), 0, st, a);        \
    }                                                                                                \
    return 1;                                                                                        \
  }
  X(1)
  if constexpr (kMaxV >= 2) { X(2) }
#undef X
  return 0;
}

// Rows beyond the register clusters: clusters that stream their share twice.  1: launched.
template <typename T, bool BWD>
static int ln_stream_launch(hipStream_t st, LnClArgs<T> a, int64_t rows, int64_t n, void* ws, size_t ws_bytes)
{
  static const bool disabled = std::getenv("LBN_NO_CLUSTER") != nullptr;
  constexpr int VE = Vec16<T>::N;
  const int64_t nvec = n / VE;
  if (disabled || !ws || !aligned16(ws) || nvec >= (int64_t(1) << 31)) return 0;
  const bool affine = a.gamma || a.beta;
  const int cap = BWD ? (affine ? cluster_capacity(ln_bwd_stream<T, true>, kLnStreamThreads)
                                : cluster_capacity(ln_bwd_stream<T, false>, kLnStreamThreads))
                      : (affine ? cluster_capacity(ln_fwd_stream<T, true>, kLnStreamThreads)
                                : cluster_capacity(ln_fwd_stream<T, false>, kLnStreamThreads));
  int64_t M = cap < kLnClMaxM ? cap : kLnClMaxM;
  if (M < 1) return 0;
  int64_t nc = cap / M;
  if (nc > rows) nc = rows;
  M = cap / nc < kLnClMaxM ? cap / nc : kLnClMaxM;  // few rows: wider clusters instead of idle workgroups
  const int64_t share = ceil_div(nvec, M);
  M = ceil_div(nvec, share);
  if (ws_bytes < ln_cluster_slot_bytes(rows, static_cast<int>(M))) return 0;
  a.rows = rows, a.n = n, a.nvec = static_cast<unsigned>(nvec), a.per_wg = static_cast<unsigned>(share);
  a.M = static_cast<int>(M), a.inv_n = 1.0f / static_cast<float>(n);
  a.cw = cluster_workspace(ws);
  ClusterLaunchGuard guard(st);
  if (guard.failed()) return 0;
  a.tag = cluster_call_tag(st, a.cw);
  const dim3 grid(static_cast<unsigned>(nc * M));
  if (BWD && affine) hipLaunchKernelGGL((ln_bwd_stream<T, true>), grid, dim3(kLnStreamThreads), 0, st, a);
  else if (BWD) hipLaunchKernelGGL((ln_bwd_stream<T, false>), grid, dim3(kLnStreamThreads), 0, st, a);
  else if (affine) hipLaunchKernelGGL((ln_fwd_stream<T, true>), grid, dim3(kLnStreamThreads), 0, st, a);
  else hipLaunchKernelGGL((ln_fwd_stream<T, false>), grid, dim3(kLnStreamThreads), 0, st, a);
  return 1;
}

template <typename T>
static int ln_fwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, float eps,
                  const T* x, int64_t ldx, T* y, int64_t ldy, float* stats, int64_t lds,
                  const float* gamma, const float* beta, void* ws, size_t ws_bytes, int flags)
{
  constexpr int VE = Vec16<T>::N;
  if (G < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (G == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !y || !stats) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = (G - 1) * stride + n;
  if (w > 1 && (ldx < height || ldy < height || lds < 2 * G)) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t rows = G * w;
  if (rows > (int64_t(1) << 30) || n > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  const RowMap map{G, stride};
  const int sumsq = (flags & LBN_STATS_SUMSQ) ? 1 : 0;
  const bool vec = (n % VE == 0) && rows_aligned16(x, stride, ldx, G, w, sizeof(T)) &&
                   rows_aligned16(y, stride, ldy, G, w, sizeof(T)) &&
                   (!gamma || aligned16(gamma)) && (!beta || aligned16(beta));
  const float inv_n = 1.0f / static_cast<float>(n);
  if (flags & LBN_STATS_REFERENCE_ORDER) {
    // parity tests only: one sequential fp32 sum per row, in the reference's order
    if (rows > kRefOrderMaxEntries / n) return LBN_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((ln_ref_order_fwd<T, RowMap>), dim3(static_cast<unsigned>(rows)), dim3(kWave), 0, st, x, y, ldx,
                       ldy, map, n, eps, stats, lds, gamma, beta);
    return launch_status();
  }
  if (n == 1) {
    const int64_t want = ceil_div(rows, 256);
    hipLaunchKernelGGL((ln_fwd_single<T>), dim3(static_cast<unsigned>(want > 8192 ? 8192 : want)), dim3(256), 0, st, x,
                       y, ldx, ldy, map, rows, eps, stats, lds, gamma, beta);
    return launch_status();
  }
  if (vec) {
    int r;
    if (stream_call_inputs(2 * rows * n * static_cast<int64_t>(sizeof(T)))) {
      using S = typename Streamed<T>::type;  // the same kernels with streaming loads of x
      r = ln_fwd_rows_launch<S>(st, reinterpret_cast<const S*>(x), reinterpret_cast<S*>(y), ldx, ldy, map, rows,
                                n / VE, inv_n, eps, stats, lds, gamma, beta, sumsq);
    }
    else {
      r = ln_fwd_rows_launch<T>(st, x, y, ldx, ldy, map, rows, n / VE, inv_n, eps, stats, lds, gamma, beta, sumsq);
    }
    if (r) return r < 0 ? LBN_ERR_UNSUPPORTED : launch_status();
    // longer than the register kernels hold: clusters when the caller gave scratch, else two passes
    if (ln_fwd_cluster_launch<T>(st, x, y, ldx, ldy, map, rows, n, eps, stats, lds, gamma, beta, sumsq, ws, ws_bytes))
      return launch_status();
    if (rows < 512) {  // few giant rows: one workgroup per row would leave most of the device idle
      LnClArgs<T> a{};
      a.x = x, a.out = y, a.ldx = ldx, a.ldo = ldy, a.map = map, a.sumsq = sumsq, a.eps = eps;
      a.stats = stats, a.ld_stats = lds, a.gamma = gamma, a.beta = beta;
      if (ln_stream_launch<T, false>(st, a, rows, n, ws, ws_bytes)) return launch_status();
    }
    hipLaunchKernelGGL((ln_fwd_long<T>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads), 0, st, x, y,
                       ldx, ldy, map, n / VE, 0, inv_n, eps, stats, lds, gamma, beta, sumsq);
    return launch_status();
  }
  if constexpr (std::is_same<T, __half>::value) {
    // fp16 rows off the 16-byte grid with an even length: the same kernels, one pair per access
    if (n % 2 == 0 && ln_pairs_first(n, rows) && rows_aligned4(x, stride, ldx, G, w) &&
        rows_aligned4(y, stride, ldy, G, w)) {
      if (int r = ln_fwd_rows_launch<f16x2>(st, reinterpret_cast<const f16x2*>(x), reinterpret_cast<f16x2*>(y),
                                            ldx, ldy, map, rows, n / 2, inv_n, eps, stats,
                                            lds, gamma, beta, sumsq))
        return r < 0 ? LBN_ERR_UNSUPPORTED : launch_status();
    }
  }
  if constexpr (std::is_same<T, float>::value) {
    if (n > 1 && n <= kLnMaxScalarRowFwd && !ln_vectors_first(n, 2048, rows, 64)) {  // rows off the 16-byte grid: the same kernels, one float per access
      if (int r = ln_fwd_rows_launch<f32x1>(st, reinterpret_cast<const f32x1*>(x), reinterpret_cast<f32x1*>(y),
                                            ldx, ldy, map, rows, n, inv_n, eps, stats, lds, gamma, beta, sumsq))
        return r < 0 ? LBN_ERR_UNSUPPORTED : launch_status();
    }
  }
  if constexpr (std::is_same<T, float>::value) {
    // longer fp32 rows off the 16-byte grid: 16-byte accesses at 4-byte alignment, the last n % 4
    // entries in a vector that overlaps its neighbour; first the register kernels, then two passes
    if (n >= 4 && !ln_no_unaligned_rows()) {  // (the partial vector reaches back four entries from the row's end)
      if (int r = ln_fwd_rows_launch<f32u>(st, reinterpret_cast<const f32u*>(x), reinterpret_cast<f32u*>(y), ldx, ldy,
                                           map, rows, ceil_div(n, 4), inv_n, eps, stats, lds, gamma, beta, sumsq,
                                           static_cast<int>(n % 4)))
        return r < 0 ? LBN_ERR_UNSUPPORTED : launch_status();
    }
    hipLaunchKernelGGL((ln_fwd_long<f32u>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads), 0, st,
                       reinterpret_cast<const f32u*>(x), reinterpret_cast<f32u*>(y), ldx, ldy, map, n / 4,
                       static_cast<int>(n % 4), inv_n, eps, stats, lds, gamma, beta, sumsq);
    return launch_status();
  }
  if constexpr (std::is_same<T, __half>::value) {
    // fp16 rows of odd length (or off the 4-byte grid): 16-byte accesses at 2-byte alignment, the last
    // n % 8 entries in a vector that overlaps its neighbour; first the register kernels
    if (n >= 8 && !ln_no_unaligned_rows()) {
      if (int r = ln_fwd_rows_launch<f16u>(st, reinterpret_cast<const f16u*>(x), reinterpret_cast<f16u*>(y), ldx, ldy,
                                           map, rows, ceil_div(n, 8), inv_n, eps, stats, lds, gamma, beta, sumsq,
                                           static_cast<int>(n % 8)))
        return r < 0 ? LBN_ERR_UNSUPPORTED : launch_status();
    }
    if (n >= kLnLongMin16) {
      hipLaunchKernelGGL((ln_fwd_long<f16u>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads), 0, st,
                         reinterpret_cast<const f16u*>(x), reinterpret_cast<f16u*>(y), ldx, ldy, map, n / 8,
                         static_cast<int>(n % 8), inv_n, eps, stats, lds, gamma, beta, sumsq);
      return launch_status();
    }
  }
  hipLaunchKernelGGL((ln_fwd_generic<T>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, st, x, y,
                     ldx, ldy, map, n, eps, stats, lds, gamma, beta, sumsq);
  return launch_status();
}

template <typename T, int TPR, int TEAMS, int V>
static void launch_ln_bwd_rows(hipStream_t st, bool wgrad, int64_t blocks, const T* x, const T* dy,
                               T* dx, int64_t ldx, int64_t lddy, int64_t lddx, RowMap map,
                               int64_t rows, int nvec, int n, float eps, const float* stats,
                               int64_t lds, float* sgrad, int64_t ldsg, const float* gamma,
                               float* part, int tail)
{
  using B = RowBlock<TPR, TEAMS>;
  const dim3 grid(static_cast<unsigned>(blocks)), block(B::kThreads);
  if (wgrad)
    hipLaunchKernelGGL((ln_bwd_rows<T, TPR, TEAMS, V, true>), grid, block, 0, st, x, dy, dx, ldx,
                       lddy, lddx, map, rows, nvec, n, eps, stats, lds, sgrad, ldsg, gamma, part, nullptr, nullptr,
                       tail);
  else {
    // nothing to accumulate across rows: one resident wave of blocks, each walking the
    // same number of rows with the next row in flight
    const int64_t units = ceil_div(rows, TEAMS);
    int64_t resident = resident_blocks(ln_bwd_rows<T, TPR, TEAMS, V, false>, B::kThreads);
    if (resident < 1) resident = 1;
    // (rows of up to 2 KiB: short-lived workgroups, see ln_row_grid)
    const dim3 all(static_cast<unsigned>(ln_row_grid(units, resident, static_cast<size_t>(n) * sizeof(T) <= 2048)));
    hipLaunchKernelGGL((ln_bwd_rows<T, TPR, TEAMS, V, false>), all, block, 0, st, x, dy, dx, ldx,
                       lddy, lddx, map, rows, nvec, n, eps, stats, lds, sgrad, ldsg, gamma, part, nullptr, nullptr,
                       tail);
  }
}

// Register-resident backward over rows of `units` access units, weight gradients included
// (partial rows in the workspace, then the fixed-order reduction).  Returns 1 when launched,
// 0 when no configuration holds the row, -1 when the workspace is missing or too small.
// tail: entries of a last, partial unit that `units` counts (storage types with unaligned access only).
template <typename ST>
static int ln_bwd_rows_launch(hipStream_t st, bool wgrad, const ST* x, const ST* dy, ST* dx, int64_t ldx,
                              int64_t lddy, int64_t lddx, RowMap map, int64_t rows, int64_t units, int64_t n,
                              int elem_bytes, float eps, const float* stats, int64_t lds, float* sgrad,
                              int64_t ldsg, const float* gamma, float* dgamma, float* dbeta, void* ws,
                              size_t ws_bytes, int tail = 0)
{
  constexpr int VE = Vec16<ST>::N;
  const LnBwdPlan p = plan_ln_bwd(units, rows, VE, elem_bytes, wgrad);
  if (!p.tpr) return 0;
  if constexpr (VE >= 4 && !UnalignedVec<ST>::value && !StreamedVec<ST>::value) {  // (small calls never stream)
    if (wgrad && ln_bwd_small(rows, n, elem_bytes)) {
      // tensors that fit the caches: weight gradients from column slices, in the same kernel, by
      // workgroups of their own beside those that walk the rows (1024 x 128: the kernel takes 3.x us
      // where one set of workgroups doing both in turn took 5.0)
      const int nvec_s = static_cast<int>(units);
      const int64_t slices = ceil_div(n, 8 * VE);
      const int col_blocks = static_cast<int>(slices < 256 ? slices : 256);
#define X(TPR, TEAMS, V)                                                                              \
  if (p.tpr == TPR && p.teams == TEAMS && p.v == V) {                                                 \
    using B = RowBlock<TPR, TEAMS>;                                                                   \
    hipLaunchKernelGGL((ln_bwd_rows<ST, TPR, TEAMS, V, false, true>),                                 \
                       dim3(static_cast<unsigned>(p.blocks + col_blocks)), dim3(B::kThreads), 0, st, x, dy, dx, ldx, \
                       lddy, lddx, map, rows, nvec_s, static_cast<int>(n), eps, stats, lds, sgrad, ldsg, gamma,  \
                       nullptr, dgamma, dbeta, 0, col_blocks);                                        \
    return 1;                                                                                         \
  }
      X(64, 4, 1) X(64, 4, 2) X(64, 4, 4) X(256, 2, 1) X(256, 2, 2) X(256, 1, 1) X(256, 1, 2)
      X(512, 1, 1) X(512, 1, 2)
      if constexpr (VE == 4) { X(256, 2, 4) X(256, 1, 4) X(512, 1, 4) }
#undef X
    }
  }
  float* part = nullptr;
  if (wgrad) {
    const size_t need = kWorkspaceHeaderBytes + static_cast<size_t>(p.blocks) * 2 * n * sizeof(float);
    if (!ws || ws_bytes < need || !aligned16(ws)) return -1;
    part = static_cast<float*>(workspace_payload(ws));
  }
  const int nvec = static_cast<int>(units);
  bool launched = false;
#define X(TPR, TEAMS, V)                                                                        \
  if (!launched && p.tpr == TPR && p.teams == TEAMS && p.v == V) {                              \
    launch_ln_bwd_rows<ST, TPR, TEAMS, V>(st, wgrad, p.blocks, x, dy, dx, ldx, lddy, lddx, map, \
                                          rows, nvec, static_cast<int>(n), eps, stats, lds,     \
                                          sgrad, ldsg, gamma, part, tail);                      \
    launched = true;                                                                            \
  }
  X(16, 16, 1) X(16, 16, 2) X(16, 16, 4)
  X(64, 4, 1) X(64, 4, 2) X(64, 4, 4) X(256, 2, 1) X(256, 2, 2) X(256, 1, 1) X(256, 1, 2)
  X(512, 1, 1) X(512, 1, 2) X(512, 1, 4)
  if constexpr (VE <= 4) { X(256, 2, 4) X(256, 1, 4) X(512, 1, 8) }
  if constexpr (VE <= 2) { X(64, 4, 8) X(256, 2, 8) X(256, 1, 8) }
#undef X
  if (!launched) return 0;
  if (wgrad) {
    if (n % 4 == 0)
      hipLaunchKernelGGL(ln_wgrad_reduce, dim3(static_cast<unsigned>(ceil_div(n, 32)), 2), dim3(256), 0, st,
                         part, p.blocks, n, dgamma, dbeta);
    else
      hipLaunchKernelGGL(ln_wgrad_reduce_scalar, dim3(static_cast<unsigned>(ceil_div(n, kWgradScalarCols)), 2), dim3(256), 0, st,
                         part, p.blocks, n, dgamma, dbeta);
  }
  return 1;
}

// Backward reads x a whole forward and backward sweep after the forward call did, and dy right
// after the next layer wrote it: from 160 MiB per call x goes through streaming loads and dy through
// ordinary ones.  Measured with the tensors of every call rotated out of the caches, rows of 4096
// floats, % of 8 TB/s with ordinary loads / with x streamed: 96 MiB per call 78 / 66, 120 MiB 74 / 70,
// 144 MiB 73 / 72, 168 MiB 71 / 74, 192 MiB 70 / 75, 384 MiB 70 / 74, 768 MiB 68 / 74 (dy streamed as
// well: 76 at both; not worth a third set of kernels).  A loop over the same buffers, where x is
// still cached from the forward call 30 us earlier, loses 9 % at 192 MiB.  With weight gradients
// fp32 calls gain as much (192 MiB per call, rows of 256 / 1024 / 4096 floats, rotated: 46.0 / 42.6 /
// 43.4 -> 41.9 / 37.9 / 39.5 us), 16-bit ones next to nothing below the general limit (4096 x 8192,
// 192 MiB per call, rotated: 67.5 -> 66.8 us per step; same buffers 59.8 -> 65.2), which they keep.
constexpr int64_t kLnStreamOldInputMinBytes = int64_t(160) << 20;

template <typename T>
static int ln_bwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, float eps,
                  const T* x, int64_t ldx, const T* dy, int64_t lddy, T* dx, int64_t lddx,
                  const float* stats, int64_t lds, float* sgrad, int64_t ldsg, const float* gamma,
                  float* dgamma, float* dbeta, void* ws, size_t ws_bytes)
{
  constexpr int VE = Vec16<T>::N;
  if (G < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (G == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !dy || !dx || !stats || !sgrad) return LBN_ERR_INVALID_ARGUMENT;
  if (dgamma && !gamma) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = (G - 1) * stride + n;
  if (w > 1 && (ldx < height || lddy < height || lddx < height || lds < 2 * G || ldsg < 2 * G))
    return LBN_ERR_INVALID_ARGUMENT;
  const int64_t rows = G * w;
  if (rows > (int64_t(1) << 30) || n > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  const RowMap map{G, stride};
  const bool wgrad = dgamma || dbeta;

  if (n <= 1) {
    // a single entry per group: the output is constant, every gradient is zero
    // (layer_norm.cpp:189-192; the weight-gradient buffers were zeroed at :300-309)
    const int64_t total = height * w;
    const int64_t want = ceil_div(total, 256);
    const unsigned grid = static_cast<unsigned>(want > 4096 ? 4096 : want);
    hipLaunchKernelGGL((fill_matrix<T>), dim3(grid), dim3(256), 0, st, dx, height, w, lddx, 0.f);
    if (dgamma) hipLaunchKernelGGL((fill_matrix<float>), dim3(1), dim3(256), 0, st, dgamma, n, 1, n, 0.f);
    if (dbeta) hipLaunchKernelGGL((fill_matrix<float>), dim3(1), dim3(256), 0, st, dbeta, n, 1, n, 0.f);
    return launch_status();
  }

  const bool vec = (n % VE == 0) && rows_aligned16(x, stride, ldx, G, w, sizeof(T)) &&
                   rows_aligned16(dy, stride, lddy, G, w, sizeof(T)) &&
                   rows_aligned16(dx, stride, lddx, G, w, sizeof(T)) &&
                   (!gamma || aligned16(gamma));
  if (vec) {
    int r;
    if (stream_call_inputs(3 * rows * n * static_cast<int64_t>(sizeof(T)),
                           (wgrad && sizeof(T) == 2) ? kStreamLoadMinBytes : kLnStreamOldInputMinBytes)) {
      using S = typename Streamed<T>::type;  // the same kernels with streaming loads of x
      r = ln_bwd_rows_launch<S>(st, wgrad, reinterpret_cast<const S*>(x), reinterpret_cast<const S*>(dy),
                                reinterpret_cast<S*>(dx), ldx, lddy, lddx, map, rows, n / VE, n, sizeof(T), eps,
                                stats, lds, sgrad, ldsg, gamma, dgamma, dbeta, ws, ws_bytes);
    }
    else {
      r = ln_bwd_rows_launch<T>(st, wgrad, x, dy, dx, ldx, lddy, lddx, map, rows, n / VE, n, sizeof(T), eps,
                                stats, lds, sgrad, ldsg, gamma, dgamma, dbeta, ws, ws_bytes);
    }
    if (r) return r < 0 ? LBN_ERR_WORKSPACE : launch_status();
    // longer than the register kernels hold: clusters (weight gradients included), else two passes
    if (ln_bwd_cluster_launch<T>(st, wgrad, x, dy, dx, ldx, lddy, lddx, map, rows, n, eps, stats, lds, sgrad, ldsg,
                                 gamma, dgamma, dbeta, ws, ws_bytes))
      return launch_status();
    if (!wgrad && rows < 512) {
      LnClArgs<T> a{};
      a.x = x, a.dy = dy, a.out = dx, a.ldx = ldx, a.lddy = lddy, a.ldo = lddx, a.map = map, a.eps = eps;
      a.stats = const_cast<float*>(stats), a.ld_stats = lds, a.sgrad = sgrad, a.ld_sgrad = ldsg, a.gamma = gamma;
      if (ln_stream_launch<T, true>(st, a, rows, n, ws, ws_bytes)) return launch_status();
    }
    hipLaunchKernelGGL((ln_bwd_long<T>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads), 0, st, x, dy,
                       dx, ldx, lddy, lddx, map, n / VE, 0, 1.0f / static_cast<float>(n), eps, stats, lds, sgrad,
                       ldsg, gamma);
  }
  else {
    if constexpr (std::is_same<T, __half>::value) {
      if (n % 2 == 0 && n / 2 <= kLnMaxScalarRowBwd && (wgrad ? ln_pairs_first_wgrad(n, rows) : ln_pairs_first(n, rows)) && rows_aligned4(x, stride, ldx, G, w) &&
          rows_aligned4(dy, stride, lddy, G, w) && rows_aligned4(dx, stride, lddx, G, w)) {
        if (int r = ln_bwd_rows_launch<f16x2>(st, wgrad, reinterpret_cast<const f16x2*>(x),
                                              reinterpret_cast<const f16x2*>(dy), reinterpret_cast<f16x2*>(dx),
                                              ldx, lddy, lddx, map, rows, n / 2, n, 2,
                                              eps, stats, lds, sgrad, ldsg, gamma, dgamma, dbeta, ws, ws_bytes))
          return r < 0 ? LBN_ERR_WORKSPACE : launch_status();
      }
    }
    if constexpr (std::is_same<T, __half>::value) {
      // fp16 rows of odd length (or off the 4-byte grid) in registers: 16-byte accesses at 2-byte
      // alignment, the last n % 8 entries in a vector that overlaps its neighbour
      if (n >= 8 && !ln_no_unaligned_rows()) {
        if (int r = ln_bwd_rows_launch<f16u>(st, wgrad, reinterpret_cast<const f16u*>(x),
                                             reinterpret_cast<const f16u*>(dy), reinterpret_cast<f16u*>(dx), ldx,
                                             lddy, lddx, map, rows, ceil_div(n, 8), n, 2, eps, stats, lds, sgrad, ldsg,
                                             gamma, dgamma, dbeta, ws, ws_bytes, static_cast<int>(n % 8)))
          return r < 0 ? LBN_ERR_WORKSPACE : launch_status();
      }
    }
    if constexpr (std::is_same<T, float>::value) {
      if (n <= kLnMaxScalarRowBwd && !ln_vectors_first(n, 1024, rows, wgrad ? 32 : 64)) {  // rows off the 16-byte grid: the same kernels, one float per access
        if (int r = ln_bwd_rows_launch<f32x1>(st, wgrad, reinterpret_cast<const f32x1*>(x),
                                              reinterpret_cast<const f32x1*>(dy), reinterpret_cast<f32x1*>(dx), ldx,
                                              lddy, lddx, map, rows, n, n, 4, eps, stats, lds, sgrad, ldsg, gamma,
                                              dgamma, dbeta, ws, ws_bytes))
          return r < 0 ? LBN_ERR_WORKSPACE : launch_status();
      }
    }
    if constexpr (std::is_same<T, float>::value) {
      if (n >= 4 && !ln_no_unaligned_rows()) {
        if (int r = ln_bwd_rows_launch<f32u>(st, wgrad, reinterpret_cast<const f32u*>(x),
                                             reinterpret_cast<const f32u*>(dy), reinterpret_cast<f32u*>(dx), ldx,
                                             lddy, lddx, map, rows, ceil_div(n, 4), n, 4, eps, stats, lds, sgrad, ldsg,
                                             gamma, dgamma, dbeta, ws, ws_bytes, static_cast<int>(n % 4)))
          return r < 0 ? LBN_ERR_WORKSPACE : launch_status();
      }
    }
    if constexpr (std::is_same<T, float>::value)
      hipLaunchKernelGGL((ln_bwd_long<f32u>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads), 0, st,
                         reinterpret_cast<const f32u*>(x), reinterpret_cast<const f32u*>(dy),
                         reinterpret_cast<f32u*>(dx), ldx, lddy, lddx, map, n / 4, static_cast<int>(n % 4),
                         1.0f / static_cast<float>(n), eps, stats, lds, sgrad, ldsg, gamma);
    else if (std::is_same<T, __half>::value && n >= kLnLongMin16)
      hipLaunchKernelGGL((ln_bwd_long<f16u>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads), 0, st,
                         reinterpret_cast<const f16u*>(x), reinterpret_cast<const f16u*>(dy),
                         reinterpret_cast<f16u*>(dx), ldx, lddy, lddx, map, n / 8, static_cast<int>(n % 8),
                         1.0f / static_cast<float>(n), eps, stats, lds, sgrad, ldsg, gamma);
    else
      hipLaunchKernelGGL((ln_bwd_generic<T>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, st, x, dy,
                         dx, ldx, lddy, lddx, map, n, eps, stats, lds, sgrad, ldsg, gamma);
  }
  if (wgrad) {
    // weight gradients of the two paths above: row slabs -> partial rows -> fixed-order sum
    const int64_t units = vec ? n / VE : n;
    const int64_t slabs = ln_wgrad_slabs(units, rows);
    if (ws && aligned16(ws) && ws_bytes >= kWorkspaceHeaderBytes + static_cast<size_t>(slabs) * 2 * n * sizeof(float)) {
      float* wpart = static_cast<float*>(workspace_payload(ws));
      const dim3 grid(static_cast<unsigned>(ceil_div(units, 256)), static_cast<unsigned>(slabs));
      if (vec)
        hipLaunchKernelGGL((ln_wgrad_columns<T, true>), grid, dim3(256), 0, st, x, dy, ldx, lddy, map, rows,
                           units, n, eps, stats, lds, wpart);
      else if (std::is_same<T, float>::value && n >= 64) {
        // fp32 rows off the 16-byte grid: 16-byte accesses at 4-byte alignment, the last n % 4 features apart
        const dim3 ugrid(static_cast<unsigned>(ceil_div(n / 4 + 1, 256)), static_cast<unsigned>(slabs));
        hipLaunchKernelGGL((ln_wgrad_columns<f32u, true>), ugrid, dim3(256), 0, st, reinterpret_cast<const f32u*>(x),
                           reinterpret_cast<const f32u*>(dy), ldx, lddy, map, rows, n / 4, n, eps, stats, lds, wpart,
                           static_cast<int>(n % 4));
      }
      else if (std::is_same<T, __half>::value && n >= 64) {
        // fp16 rows off the 16-byte grid: 16-byte accesses at 2-byte alignment, the last n % 8 features apart
        const dim3 ugrid(static_cast<unsigned>(ceil_div(n / 8 + 1, 256)), static_cast<unsigned>(slabs));
        hipLaunchKernelGGL((ln_wgrad_columns<f16u, true>), ugrid, dim3(256), 0, st, reinterpret_cast<const f16u*>(x),
                           reinterpret_cast<const f16u*>(dy), ldx, lddy, map, rows, n / 8, n, eps, stats, lds, wpart,
                           static_cast<int>(n % 8));
      }
      else
        hipLaunchKernelGGL((ln_wgrad_columns<T, false>), grid, dim3(256), 0, st, x, dy, ldx, lddy, map, rows,
                           units, n, eps, stats, lds, wpart);
      if (n % 4 == 0)
        hipLaunchKernelGGL(ln_wgrad_reduce, dim3(static_cast<unsigned>(ceil_div(n, 32)), 2), dim3(256), 0, st,
                           wpart, slabs, n, dgamma, dbeta);
      else
        hipLaunchKernelGGL(ln_wgrad_reduce_scalar, dim3(static_cast<unsigned>(ceil_div(n, kWgradScalarCols)), 2), dim3(256), 0,
                           st, wpart, slabs, n, dgamma, dbeta);
    }
    else {
      // no scratch: one thread per feature walks every row
      hipLaunchKernelGGL((ln_wgrad_generic<T>), dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256),
                         0, st, x, dy, ldx, lddy, map, rows, n, eps, stats, lds, dgamma, dbeta);
    }
  }
  return launch_status();
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_layer_norm_fwd_workspace_bytes(int64_t num_groups, int64_t norm_size, int64_t width, int elem_bytes)
{
  if (num_groups <= 0 || norm_size <= 0 || width <= 0) return 0;
  const int ve = elem_bytes == 2 ? 8 : 4;
  // only rows beyond the one-workgroup kernels use scratch
  if (norm_size % ve != 0 || pick_row_config(norm_size / ve, num_groups * width, 8).tpr) return 0;
  return ln_cluster_fwd_workspace(norm_size, num_groups * width, ve);
}

int lbn_layer_norm_fwd_f32(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon, const float* x,
                           int64_t ldx, float* y, int64_t ldy, float* stats, int64_t ld_stats,
                           const float* scale, const float* bias, void* workspace,
                           size_t workspace_bytes, int flags)
{
  return ln_fwd<float>(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon, x, ldx,
                       y, ldy, stats, ld_stats, scale, bias, workspace, workspace_bytes, flags);
}

int lbn_layer_norm_fwd_f16(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon, const void* x,
                           int64_t ldx, void* y, int64_t ldy, float* stats, int64_t ld_stats,
                           const float* scale, const float* bias, void* workspace,
                           size_t workspace_bytes, int flags)
{
  return ln_fwd<__half>(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon,
                        static_cast<const __half*>(x), ldx, static_cast<__half*>(y), ldy, stats,
                        ld_stats, scale, bias, workspace, workspace_bytes, flags);
}

size_t lbn_layer_norm_bwd_workspace_bytes(int64_t num_groups, int64_t norm_size, int64_t width,
                                          int has_weight_grads, int elem_bytes)
{
  if (num_groups <= 0 || norm_size <= 0 || width <= 0) return 0;
  const int ve = elem_bytes == 2 ? 8 : 4;
  const int64_t rows = num_groups * width;
  if (has_weight_grads) return ln_bwd_workspace(norm_size, rows, ve);
  // without weight gradients only the cluster kernels of long rows use scratch (their slots)
  if (norm_size % ve != 0 || plan_ln_bwd(norm_size / ve, rows, ve, elem_bytes == 2 ? 2 : 4).tpr) return 0;
  return norm_size / ve < (int64_t(1) << 31) ? ln_cluster_slot_bytes(rows, kLnClMaxM) : 0;
}

int lbn_layer_norm_bwd_f32(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon, const float* x,
                           int64_t ldx, const float* dy, int64_t lddy, float* dx, int64_t lddx,
                           const float* stats, int64_t ld_stats, float* stats_grad,
                           int64_t ld_stats_grad, const float* scale, float* dscale, float* dbias,
                           void* workspace, size_t workspace_bytes)
{
  return ln_bwd<float>(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon, x, ldx,
                       dy, lddy, dx, lddx, stats, ld_stats, stats_grad, ld_stats_grad, scale, dscale,
                       dbias, workspace, workspace_bytes);
}

int lbn_layer_norm_bwd_f16(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon, const void* x,
                           int64_t ldx, const void* dy, int64_t lddy, void* dx, int64_t lddx,
                           const float* stats, int64_t ld_stats, float* stats_grad,
                           int64_t ld_stats_grad, const float* scale, float* dscale, float* dbias,
                           void* workspace, size_t workspace_bytes)
{
  return ln_bwd<__half>(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon,
                        static_cast<const __half*>(x), ldx, static_cast<const __half*>(dy), lddy,
                        static_cast<__half*>(dx), lddx, stats, ld_stats, stats_grad, ld_stats_grad,
                        scale, dscale, dbias, workspace, workspace_bytes);
}

// Instance norm is layer norm over groups of channel_size entries without scale and
// bias (instance_norm.cpp:47-231 against layer_norm.cpp:41-258: the same statistics,
// the same 2/n factor in backward, the same constant output for single-entry groups).
size_t lbn_instance_norm_fwd_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  return lbn_layer_norm_fwd_workspace_bytes(channels, channel_size, width, 4);
}

int lbn_instance_norm_fwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                              int64_t width, float epsilon, const float* x, int64_t ldx, float* y,
                              int64_t ldy, float* stats, int64_t ld_stats, void* workspace,
                              size_t workspace_bytes)
{
  return ln_fwd<float>(as_stream(stream), channels, channel_size, channel_size, width, epsilon, x,
                       ldx, y, ldy, stats, ld_stats, nullptr, nullptr, workspace, workspace_bytes,
                       LBN_STATS_TWO_PASS);
}

// The scratch of the layer-norm kernels comes first (at least the 64-byte header, so that
// lbn_workspace_timed_out() finds the error word where it does for every other layer), the
// statistics gradients (2 * channels x width floats) behind it on a 256-byte boundary.
static size_t in_scratch_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  size_t b = lbn_layer_norm_bwd_workspace_bytes(channels, channel_size, width, 0, 4);
  if (b < kWorkspaceHeaderBytes) b = kWorkspaceHeaderBytes;
  return (b + 255) & ~size_t(255);
}

size_t lbn_instance_norm_bwd_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  if (channels <= 0 || channel_size <= 0 || width <= 0) return 0;
  return in_scratch_bytes(channels, channel_size, width) +
         static_cast<size_t>(2 * channels) * static_cast<size_t>(width) * sizeof(float);
}

int lbn_instance_norm_bwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                              int64_t width, float epsilon, const float* x, int64_t ldx,
                              const float* dy, int64_t lddy, float* dx, int64_t lddx,
                              const float* stats, int64_t ld_stats, void* workspace,
                              size_t workspace_bytes)
{
  if (channels < 0 || channel_size < 0 || width < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (channels == 0 || channel_size == 0 || width == 0) return LBN_OK;
  if (!workspace || workspace_bytes < lbn_instance_norm_bwd_workspace_bytes(channels, channel_size, width))
    return LBN_ERR_WORKSPACE;
  const size_t scratch = in_scratch_bytes(channels, channel_size, width);
  float* sgrad = reinterpret_cast<float*>(static_cast<char*>(workspace) + scratch);
  return ln_bwd<float>(as_stream(stream), channels, channel_size, channel_size, width, epsilon, x,
                       ldx, dy, lddy, dx, lddx, stats, ld_stats, sgrad, 2 * channels, nullptr, nullptr, nullptr,
                       workspace, scratch);
}

}  // extern "C"
