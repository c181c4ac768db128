// The five layers for TensorDataType = double (the reference instantiates its layers for double
// under LBANN_HAS_DOUBLE: include/lbann/macros/instantiate.hpp:28-30,
// src/layers/regularizers/layer_norm_builder.cpp:48-54).  Storage, statistics, weights and all
// arithmetic are binary64; every kernel is bound by HBM bandwidth at 8 bytes per entry.
//
// One family of row kernels serves layer norm, softmax, log-softmax and channelwise softmax: a
// team of 64, 256 or 1024 threads owns a row and keeps it in registers (V accesses of W = 2
// doubles, 16 bytes, per thread; W = 1 for rows off the 16-byte grid), so a tensor is read once
// and written once.  Teams walk rows b, b + grid, ... (the launch is a few workgroups per compute
// unit).  Rows beyond 32768 entries (16384 for W = 1) are streamed by one 1024-thread workgroup
// each, twice (the second pass re-reads what the first one left in the caches).  Layer-norm weight
// gradients are accumulated in registers across a team's rows and leave one partial row per team,
// added in a fixed order by a second kernel.  Batch norm reduces a channel (width segments of
// channel_size entries) over P workgroups into partial pairs and merges them, in a fixed order, in
// the prologue of the apply kernel.  No atomics: results are bitwise reproducible.
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cmath>
#include <cstdint>

#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {
namespace f64 {

constexpr int kMaxV = 16;
constexpr int kStreamThreads = 1024;
constexpr int kBnThreads = 256;
constexpr int kBnMaxSplit = 64;

enum { kSoftmax = 0, kLogSoftmax = 1, kChannelwise = 2 };

// ------------------------------------------------------------------ reductions
// Wave reductions of doubles on the DPP data path (the two halves of a double move with the same
// control; see the fp32 versions in device_utils.hpp): the wave's result is valid in lane 63.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ double dpp_move_d(double v, double old = 0.0)
{
  const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
  const unsigned long long o = __builtin_bit_cast(unsigned long long, old);
  const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_update_dpp(static_cast<int>(o), static_cast<int>(b), CTRL,
                                                                        ROW_MASK, 0xF, false));
  const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_update_dpp(static_cast<int>(o >> 32), static_cast<int>(b >> 32),
                                                                        CTRL, ROW_MASK, 0xF, false));
  return __builtin_bit_cast(double, (static_cast<unsigned long long>(hi) << 32) | lo);
}
__device__ __forceinline__ double read_lane_d(double v, int lane)
{
  const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
  const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b), lane));
  const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b >> 32), lane));
  return __builtin_bit_cast(double, (static_cast<unsigned long long>(hi) << 32) | lo);
}
__device__ __forceinline__ double wave_sum_in_last_d(double v)
{
  v += dpp_move_d<kDppQuadSwap1>(v);
  v += dpp_move_d<kDppQuadSwap2>(v);
  v += dpp_move_d<kDppHalfMirror>(v);
  v += dpp_move_d<kDppRowMirror>(v);
  v += dpp_move_d<kDppRowBcast15, 0xA>(v);  // rows 1 and 3 add rows 0 and 2; the others add 0
  v += dpp_move_d<kDppRowBcast31, 0xC>(v);  // row 3 adds rows 0 + 1
  return v;
}
__device__ __forceinline__ double wave_max_in_last_d(double v)
{
  v = fmax(v, dpp_move_d<kDppQuadSwap1>(v));
  v = fmax(v, dpp_move_d<kDppQuadSwap2>(v));
  v = fmax(v, dpp_move_d<kDppHalfMirror>(v));
  v = fmax(v, dpp_move_d<kDppRowMirror>(v));
  v = fmax(v, dpp_move_d<kDppRowBcast15, 0xA>(v, v));  // disabled rows keep their own value
  v = fmax(v, dpp_move_d<kDppRowBcast31, 0xC>(v, v));
  return v;
}

// Sum / maximum over a team of NW waves; every thread gets the result.  `slot` points to NW
// doubles of LDS private to the team and to this reduction; all threads of the workgroup call
// when NW > 1 (a team is then the whole workgroup).  Fixed order.
template <int NW>
__device__ __forceinline__ double team_sum_d(double v, double* slot)
{
  v = wave_sum_in_last_d(v);
  if constexpr (NW == 1) return read_lane_d(v, kWave - 1);
  if ((threadIdx.x & (kWave - 1)) == kWave - 1) slot[(threadIdx.x / kWave) % NW] = v;
  __syncthreads();
  double r = slot[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r += slot[i];
  return r;
}
template <int NW>
__device__ __forceinline__ double team_max_d(double v, double* slot)
{
  v = wave_max_in_last_d(v);
  if constexpr (NW == 1) return read_lane_d(v, kWave - 1);
  if ((threadIdx.x & (kWave - 1)) == kWave - 1) slot[(threadIdx.x / kWave) % NW] = v;
  __syncthreads();
  double r = slot[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = fmax(r, slot[i]);
  return r;
}

// ------------------------------------------------------------------ access
template <int W>
__device__ __forceinline__ void load_w(const double* p, double (&v)[W])
{
  if constexpr (W == 2) {
    const double2 t = *reinterpret_cast<const double2*>(p);
    v[0] = t.x;
    v[1] = t.y;
  }
  else {
    v[0] = *p;
  }
}
template <int W>
__device__ __forceinline__ void store_w(double* p, const double (&v)[W])
{
  if constexpr (W == 2) {
    typedef double v2d __attribute__((ext_vector_type(2)));
    v2d t;
    t.x = v[0];
    t.y = v[1];
    __builtin_nontemporal_store(t, reinterpret_cast<v2d*>(p));
  }
  else {
    __builtin_nontemporal_store(v[0], p);
  }
}

// A team's place in the launch: TPR threads per row, 256-thread workgroups hold 256 / TPR teams.
template <int TPR>
struct Team {
  static constexpr int kThreads = TPR < 256 ? 256 : TPR;
  static constexpr int kTeams = kThreads / TPR;
  static constexpr int kNW = TPR / kWave;
};

// Shapes of the register kernels.
struct RowShape {
  int tpr, v;
};
// The narrowest team whose threads own at most two accesses each (a thread's entries are doubles:
// registers run out quickly, and several small workgroups per compute unit overlap better than one
// large one); rows beyond 2048 accesses take 1024 threads with up to 16 accesses each.
inline RowShape pick_shape(int64_t units, int64_t rows)
{
  const int tprs[3] = {64, 256, 1024};
  for (int i = 0; i < 3; ++i) {
    const int64_t per = ceil_div(units, tprs[i]);
    if (per > (i == 2 ? kMaxV : 2)) continue;
    int v = 1;
    while (v < per) v *= 2;
    // few rows: a wider team keeps more of the device busy
    if (i < 2 && v > 1 && rows * (tprs[i] / kWave) < 2048) continue;
    return {tprs[i], v};
  }
  return {0, 0};
}

// Every register kernel: rows map to (column, group) as in the fp32 kernels.
struct RowArgs {
  const double* a;   // x (forward) or y / x (backward)
  const double* g;   // dy
  double* out;
  int64_t lda, ldg, ldo;
  RowMap map;
  int64_t rows;
  int units;         // accesses per row
  int n;             // entries per row
  double eps;
  double* stats;     // layer norm: (2G x w)
  int64_t ld_stats;
  double* sgrad;
  int64_t ld_sgrad;
  const double* gamma;
  const double* beta;
  double* part;      // layer norm backward: one partial (dscale | dbias) row of 2n per team
  int sumsq;
};

#define LBN_F64_ROW_PROLOGUE                                                         \
  using TM = Team<TPR>;                                                              \
  constexpr int NW = TM::kNW;                                                        \
  __shared__ double red[4][TM::kTeams][NW > 1 ? NW : 1];                             \
  const int team = threadIdx.x / TPR;                                                \
  const int t = threadIdx.x - team * TPR;                                            \
  const int64_t teams_total = static_cast<int64_t>(gridDim.x) * TM::kTeams;          \
  const int64_t first = static_cast<int64_t>(blockIdx.x) * TM::kTeams + team;        \
  const int64_t iters = (a.rows + teams_total - 1) / teams_total;                    \
  bool ok[V];                                                                        \
  int offs[V]; /* entry offset of access i; accesses past the row's end re-read access 0 */ \
  _Pragma("unroll") for (int i = 0; i < V; ++i) {                                    \
    ok[i] = t + i * TPR < a.units;                                                   \
    offs[i] = ok[i] ? W * (t + i * TPR) : 0;                                         \
  }                                                                                  \
  /* threads with many accesses form the offset anew at every use: held across the row loop the */ \
  /* offsets take V registers, and a spilled one is reloaded behind every load in flight */ \
  auto off_at = [&](int i) -> int {                                                  \
    if constexpr (V >= 8) {                                                          \
      int tv = t;                                                                    \
      asm volatile("" : "+v"(tv));                                                   \
      return tv + i * TPR < a.units ? W * (tv + i * TPR) : 0;                        \
    }                                                                                \
    else {                                                                           \
      return offs[i];                                                                \
    }                                                                                \
  };                                                                                 \
  /* row of iteration `it` (clamped to the last row: its loads are harmless, its stores skipped) */ \
  auto row_of = [&](int64_t it) {                                                    \
    const int64_t r = first + it * teams_total;                                      \
    return r < a.rows ? r : a.rows - 1;                                              \
  };

// ------------------------------------------------------------------ softmax family
// All of a row's loads are issued together, unconditionally; the row that a team takes next is
// requested while the current one is stored: every access is reloaded right behind its store, into
// the registers the store has just freed, so loads and stores of a compute unit overlap even
// when a row fills its registers (32768 doubles in a 1024-thread workgroup).
template <int KIND, int TPR, int V, int W>
__global__ void __launch_bounds__(Team<TPR>::kThreads)
sm_fwd_rows_f64(RowArgs a)
{
  LBN_F64_ROW_PROLOGUE
  double v[V][W];
  {
    const double* xr = a.a + a.map.offset(row_of(0), a.lda);
#pragma unroll
    for (int i = 0; i < V; ++i) load_w<W>(xr + off_at(i), v[i]);
  }
  for (int64_t it = 0; it < iters; ++it) {
    const int64_t row = first + it * teams_total;
    const bool live = row < a.rows;  // teams of a workgroup run the same number of iterations
    double m = -DBL_MAX;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int j = 0; j < W; ++j) m = fmax(m, ok[i] ? v[i][j] : -DBL_MAX);
    m = team_max_d<NW>(m, red[2 * (it & 1)][team]);
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        const double d = v[i][j] - m;
        const double e = exp(d);
        s += ok[i] ? e : 0.0;
        v[i][j] = KIND == kLogSoftmax ? d : e;
      }
    }
    s = team_sum_d<NW>(s, red[2 * (it & 1) + 1][team]);
    double* yr = a.out + a.map.offset(live ? row : a.rows - 1, a.ldo);
    const double* xn = a.a + a.map.offset(row_of(it + 1), a.lda);
    const bool more = it + 1 < iters;
    const double scale = 1.0 / s;
    const double lse = KIND == kLogSoftmax ? log(s) : 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        if (KIND == kSoftmax) {
          const double r2 = scale * v[i][j];
          v[i][j] = __builtin_isnormal(r2) ? r2 : 0.0;  // openmp/softmax.hpp:108-113
        }
        else if (KIND == kLogSoftmax) {
          v[i][j] -= lse;
        }
        else {
          v[i][j] /= s;  // channelwise_softmax.cpp:88-97: a division, denormals kept
        }
      }
      if (live && ok[i]) store_w<W>(yr + off_at(i), v[i]);
      if (more) load_w<W>(xn + off_at(i), v[i]);
    }
  }
}

template <int KIND, int TPR, int V, int W>
__global__ void __launch_bounds__(Team<TPR>::kThreads)
sm_bwd_rows_f64(RowArgs a)
{
  LBN_F64_ROW_PROLOGUE
  double y[V][W], g[V][W];
  {
    const int64_t r = row_of(0);
    const double* yr = a.a + a.map.offset(r, a.lda);
    const double* gr = a.g + a.map.offset(r, a.ldg);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      load_w<W>(yr + off_at(i), y[i]);
      load_w<W>(gr + off_at(i), g[i]);
    }
  }
  for (int64_t it = 0; it < iters; ++it) {
    const int64_t row = first + it * teams_total;
    const bool live = row < a.rows;
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int j = 0; j < W; ++j) s += ok[i] ? (KIND == kLogSoftmax ? g[i][j] : y[i][j] * g[i][j]) : 0.0;
    s = team_sum_d<NW>(s, red[it & 3][team]);
    double* dr = a.out + a.map.offset(live ? row : a.rows - 1, a.ldo);
    const int64_t rn = row_of(it + 1);
    const double* yn = a.a + a.map.offset(rn, a.lda);
    const double* gn = a.g + a.map.offset(rn, a.ldg);
    const bool more = it + 1 < iters;
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int j = 0; j < W; ++j)
        g[i][j] = KIND == kLogSoftmax ? g[i][j] - exp(y[i][j]) * s : y[i][j] * (g[i][j] - s);
      if (live && ok[i]) store_w<W>(dr + off_at(i), g[i]);
      if (more) {
        load_w<W>(yn + off_at(i), y[i]);
        load_w<W>(gn + off_at(i), g[i]);
      }
    }
  }
}

// Backward for rows of 16384 to 32768 doubles, whose y and dy are more than the registers of a
// 1024-thread workgroup hold (2 x 64 of 128 per thread): y stays in registers, of dy the first KR
// accesses per thread do and the other V - KR go from memory straight into LDS
// (global_load_lds_dwordx4: lane l of a wave fills the 16 bytes at the wave's base + 16 l, no
// registers in between), where each thread reads the slots that its own wave requested (no
// barrier).  Every entry is read once.  One workgroup per compute unit walks rows b, b + grid,
// ...; each access of the next row is requested right behind the store that frees its registers or
// its slot, so a compute unit's loads overlap its stores.
template <int KIND, int V, int KR>
__global__ void __launch_bounds__(1024)
sm_bwd_rows_parked_f64(RowArgs a)
{
  constexpr int TPR = 1024, NW = TPR / kWave, LK = V - KR;
  typedef double v2d __attribute__((ext_vector_type(2)));
  __shared__ v2d parked[LK][TPR];
  __shared__ double red[2][NW];
  const int t = threadIdx.x;
  auto live = [&](int i) { return t + i * TPR < a.units; };
  // Byte offset of access i in a row; accesses past the row's end repeat access 0 (every load is
  // unconditional, their values are left out of the sum and never stored).  A row's address is the
  // same for every thread: scalar registers, and one 32-bit offset per access.
  auto at = [&](const double* p, int i) {
    unsigned tv = t;
    asm volatile("" : "+v"(tv));  // formed anew at every use: sixteen offsets kept across the loop cost sixteen registers
    const unsigned off = tv + i * TPR < unsigned(a.units) ? 16u * (tv + i * TPR) : 16u * tv;
    return reinterpret_cast<const v2d*>(reinterpret_cast<const char*>(p) + off);
  };
  // access KR + j of a row of dy into slot j
  auto park = [&](const double* p, int j) {
    unsigned first = t;
    asm volatile("" : "+v"(first));  // as in at(): nine slot addresses would wait in registers otherwise
    first &= ~unsigned(kWave - 1);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)at(p, KR + j),
                                     (__attribute__((address_space(3))) void*)&parked[j][first], 16, 0, 0);
  };
  int64_t row = blockIdx.x;
  if (row >= a.rows) return;
  v2d y[V], g[KR];
  {
    const double* yr = a.a + a.map.offset(row, a.lda);
    const double* gr = a.g + a.map.offset(row, a.ldg);
#pragma unroll
    for (int j = 0; j < LK; ++j) park(gr, j);
#pragma unroll
    for (int i = 0; i < V; ++i) y[i] = *at(yr, i);
#pragma unroll
    for (int i = 0; i < KR; ++i) g[i] = *at(gr, i);
  }
  for (int it = 0; row < a.rows; row += gridDim.x, ++it) {
    // the slots are written by the memory system: everything this thread requested has arrived
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const v2d gi = i < KR ? g[i < KR ? i : 0] : parked[i < KR ? 0 : i - KR][t];
      const double part = KIND == kLogSoftmax ? gi.x + gi.y : y[i].x * gi.x + y[i].y * gi.y;
      s += live(i) ? part : 0.0;
      if (KIND == kLogSoftmax) {
        // exp(y) now, while no load is outstanding, and in place: its temporaries do not fit beside
        // the next row's requests in the loop of stores
        y[i].x = exp(y[i].x);
        y[i].y = exp(y[i].y);
      }
      if (i >= KR || KIND == kLogSoftmax) __builtin_amdgcn_sched_barrier(0);  // one access at a time: the registers are full
    }
    // team_sum_d with the partial sums fetched four at a time (it would hold all 16 at once)
    s = wave_sum_in_last_d(s);
    if ((t & (kWave - 1)) == kWave - 1) red[it & 1][t / kWave] = s;
    __syncthreads();
    s = 0.0;
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      s += red[it & 1][i];
      if (i % 4 == 3) __builtin_amdgcn_sched_barrier(0);
    }
    double* dr = a.out + a.map.offset(row, a.ldo);
    const int64_t next = row + gridDim.x;
    const bool more = next < a.rows;
    const double* yn = a.a + a.map.offset(more ? next : row, a.lda);
    const double* gn = a.g + a.map.offset(more ? next : row, a.ldg);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const v2d gi = i < KR ? g[i < KR ? i : 0] : parked[i < KR ? 0 : i - KR][t];
      v2d d;
      if (KIND == kLogSoftmax) {
        d.x = gi.x - y[i].x * s;
        d.y = gi.y - y[i].y * s;
      }
      else {
        d.x = y[i].x * (gi.x - s);
        d.y = y[i].y * (gi.y - s);
      }
      if (live(i)) __builtin_nontemporal_store(d, const_cast<v2d*>(at(dr, i)));
      asm volatile("" ::: "memory");  // the slot has been read before the next row's request overwrites it
      if (more) {
        y[i] = *at(yn, i);
        if (i < KR) g[i < KR ? i : 0] = *at(gn, i);
        else park(gn, i - KR);
      }
      __builtin_amdgcn_sched_barrier(0);  // one access at a time
    }
  }
}

// ------------------------------------------------------------------ layer norm
template <int TPR, int V, int W>
__global__ void __launch_bounds__(Team<TPR>::kThreads)
ln_fwd_rows_f64(RowArgs a)
{
  LBN_F64_ROW_PROLOGUE
  const double inv_n = 1.0 / static_cast<double>(a.n);
  // threads that own at most 8 entries keep their scale and bias in registers across rows
  constexpr bool kWeightsInRegs = V * W <= 8;
  double gam[kWeightsInRegs ? V : 1][W], bet[kWeightsInRegs ? V : 1][W];
  if constexpr (kWeightsInRegs) {
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int j = 0; j < W; ++j) {
        gam[i][j] = (a.gamma && ok[i]) ? a.gamma[off_at(i) + j] : 1.0;
        bet[i][j] = (a.beta && ok[i]) ? a.beta[off_at(i) + j] : 0.0;
      }
  }
  double v[V][W];
  {
    const double* xr = a.a + a.map.offset(row_of(0), a.lda);
#pragma unroll
    for (int i = 0; i < V; ++i) load_w<W>(xr + off_at(i), v[i]);
  }
  for (int64_t it = 0; it < iters; ++it) {
    const int64_t row = first + it * teams_total;
    const bool live = row < a.rows;
    double s = 0.0, q = 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int j = 0; j < W; ++j) {
        if (!ok[i]) v[i][j] = 0.0;
        s += v[i][j];
        q += v[i][j] * v[i][j];
      }
    s = team_sum_d<NW>(s, red[2 * (it & 1)][team]);
    double mean = s * inv_n;
    double var;
    if (a.sumsq) {  // the reference's expression (layer_norm.cpp:99-112)
      q = team_sum_d<NW>(q, red[2 * (it & 1) + 1][team]);
      const double nn = static_cast<double>(a.n);
      mean = s / nn;
      var = fmax(q / nn - mean * mean, 0.0);
    }
    else {
      double c = 0.0;
#pragma unroll
      for (int i = 0; i < V; ++i)
#pragma unroll
        for (int j = 0; j < W; ++j) {
          const double d = ok[i] ? v[i][j] - mean : 0.0;
          c += d * d;
        }
      var = team_sum_d<NW>(c, red[2 * (it & 1) + 1][team]) * inv_n;
    }
    int64_t col, g;
    a.map.split(live ? row : a.rows - 1, col, g);
    if (live && t == 0) {
      a.stats[g + col * a.ld_stats] = mean;
      a.stats[a.map.groups + g + col * a.ld_stats] = var;
    }
    const double inv_stdev = 1.0 / sqrt(var + a.eps);
    double* yr = a.out + g * a.map.stride + col * a.ldo;
    const double* xn = a.a + a.map.offset(row_of(it + 1), a.lda);
    const bool more = it + 1 < iters;
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        double y = (v[i][j] - mean) * inv_stdev;
        if constexpr (kWeightsInRegs) {
          y = y * gam[i][j] + bet[i][j];
        }
        else {
          if (a.gamma) y *= a.gamma[off_at(i) + j];
          if (a.beta) y += a.beta[off_at(i) + j];
        }
        v[i][j] = y;
      }
      if (live && ok[i]) store_w<W>(yr + off_at(i), v[i]);
      if (more) load_w<W>(xn + off_at(i), v[i]);
    }
  }
}

// WGRAD: dscale / dbias accumulate in registers across the team's rows (a thread always owns the
// same entries) and leave one partial row per team.  Measured and rejected for rows of 4096 doubles
// with weight gradients (8192 rows, 158 us): 512 threads with twice the entries each so that two
// workgroups share a compute unit (178 us: 18 registers spilled within 128), a second row
// requested ahead in 1024 threads (32 spilled), and 256 threads with eight accesses each, two
// workgroups per unit (157 us, no spill: the same time, so the kernel's shape is not what
// limits a call that moves 805 MB).
template <int TPR, int V, int W, bool WGRAD>
__global__ void __launch_bounds__(Team<TPR>::kThreads)
ln_bwd_rows_f64(RowArgs a)
{
  LBN_F64_ROW_PROLOGUE
  const double nn = static_cast<double>(a.n);
  double gam[V][W];
  double dg[WGRAD ? V : 1][W], db[WGRAD ? V : 1][W];
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int j = 0; j < W; ++j) {
      gam[i][j] = (a.gamma && ok[i]) ? a.gamma[off_at(i) + j] : 1.0;
      if (WGRAD) dg[i][j] = db[i][j] = 0.0;
    }
  double d[V][W], gs[V][W];
  double mean, var;
  auto issue = [&](int64_t it) {
    int64_t col, g;
    a.map.split(row_of(it), col, g);
    const double* xr = a.a + g * a.map.stride + col * a.lda;
    const double* gr = a.g + g * a.map.stride + col * a.ldg;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      load_w<W>(xr + off_at(i), d[i]);
      load_w<W>(gr + off_at(i), gs[i]);
    }
    mean = a.stats[g + col * a.ld_stats];
    var = a.stats[a.map.groups + g + col * a.ld_stats];
  };
  issue(0);
  for (int64_t it = 0; it < iters; ++it) {
    const int64_t row = first + it * teams_total;
    const bool live = row < a.rows;
    const double mu = mean;
    const double inv_stdev = 1.0 / sqrt(var + a.eps);
    double A = 0.0, B = 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        const bool use = ok[i] && live;
        const double gv = use ? gs[i][j] : 0.0;
        d[i][j] = use ? d[i][j] - mu : 0.0;
        if (WGRAD) {
          db[i][j] += gv;
          dg[i][j] += gv * d[i][j] * inv_stdev;
        }
        gs[i][j] = gv * gam[i][j];
        A += gs[i][j];
        B += gs[i][j] * d[i][j];
      }
    }
    A = team_sum_d<NW>(A, red[2 * (it & 1)][team]);
    B = team_sum_d<NW>(B, red[2 * (it & 1) + 1][team]);
    int64_t col, g;
    a.map.split(live ? row : a.rows - 1, col, g);
    const double dmean = -A * inv_stdev;
    const double dvar = -B * inv_stdev * inv_stdev * inv_stdev / 2;
    if (live && t == 0) {
      a.sgrad[g + col * a.ld_sgrad] = dmean;
      a.sgrad[a.map.groups + g + col * a.ld_sgrad] = dvar;
    }
    double* dr = a.out + g * a.map.stride + col * a.ldo;
    const double c0 = dmean / nn, c1 = dvar * 2 / nn;
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int j = 0; j < W; ++j) gs[i][j] = gs[i][j] * inv_stdev + c0 + c1 * d[i][j];
      if (live && ok[i]) store_w<W>(dr + off_at(i), gs[i]);
    }
    if (it + 1 < iters) issue(it + 1);
  }
  if (WGRAD) {
    double* out = a.part + first * 2 * a.n;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      if (!ok[i]) continue;
#pragma unroll
      for (int j = 0; j < W; ++j) {
        out[off_at(i) + j] = dg[i][j];
        out[a.n + off_at(i) + j] = db[i][j];
      }
    }
  }
}

// Adds P partial rows of 2n entries in a fixed order.  A workgroup takes 16 consecutive entries
// (128 contiguous bytes of every partial row); its 256 threads are 16 row groups x 16 entries, a
// thread adds rows g, g + 16, ... eight loads at a time, the groups are added through LDS.
__global__ void __launch_bounds__(256)
ln_wgrad_reduce_f64(const double* __restrict__ part, int64_t P, int64_t n, double* dscale, double* dbias)
{
  __shared__ double sm[16][17];
  const int e_in = threadIdx.x & 15, g = threadIdx.x >> 4;
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 16 + e_in;
  double acc = 0.0;
  if (e < 2 * n) {
    for (int64_t p0 = g; p0 < P; p0 += 16 * 8) {
      double w[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int64_t p = p0 + 16 * j;
        w[j] = p < P ? part[p * 2 * n + e] : 0.0;
      }
      acc += ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7]));
    }
  }
  sm[g][e_in] = acc;
  __syncthreads();
  if (threadIdx.x < 16 && e < 2 * n) {
    double r = 0.0;
#pragma unroll
    for (int k = 0; k < 16; ++k) r += sm[k][threadIdx.x];
    double* out = e < n ? dscale : dbias;
    if (out) out[e < n ? e : e - n] = r;
  }
}

// ------------------------------------------------------------------ long rows
// One 1024-thread workgroup per row, one double per access (512 contiguous bytes per wave), two
// passes; the second finds the row in the caches.  OP: 0 softmax family forward (KIND), 1 softmax
// family backward, 2 layer norm forward, 3 layer norm backward (weight gradients by the column
// kernel below).
template <int OP, int KIND>
__global__ void __launch_bounds__(kStreamThreads)
rows_stream_f64(RowArgs a)
{
  constexpr int NW = kStreamThreads / kWave;
  __shared__ double red[3][NW];
  const int64_t row = blockIdx.x;
  int64_t col, g;
  a.map.split(row, col, g);
  const int64_t off_a = g * a.map.stride + col * a.lda;
  const int64_t off_g = g * a.map.stride + col * a.ldg;
  const int64_t off_o = g * a.map.stride + col * a.ldo;
  const int t = threadIdx.x;
  const int64_t n = a.n;
  if (OP == 0) {
    const double* xr = a.a + off_a;
    // online, four entries at a time (their loads go out together, no data-dependent branch):
    // s = sum exp(x - m) over the thread's entries so far
    double m = -DBL_MAX, s = 0.0;
    for (int64_t k = t; k < n; k += 4 * kStreamThreads) {
      double x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t kk = k + u * kStreamThreads;
        x[u] = xr[kk < n ? kk : k];
      }
      const double mn = fmax(fmax(m, fmax(x[0], x[1])), fmax(x[2], x[3]));
      double add = 0.0;
#pragma unroll
      for (int u = 0; u < 4; ++u) add += k + u * kStreamThreads < n ? exp(x[u] - mn) : 0.0;
      s = s * exp(m - mn) + add;
      m = mn;
    }
    const double gm = team_max_d<NW>(m, red[0]);
    s = team_sum_d<NW>(s * exp(m - gm), red[1]);
    const double scale = 1.0 / s, lse = log(s);
    double* yr = a.out + off_o;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) {
      const double d = xr[k] - gm;
      double y;
      if (KIND == kLogSoftmax) y = d - lse;
      else if (KIND == kSoftmax) {
        y = scale * exp(d);
        y = __builtin_isnormal(y) ? y : 0.0;
      }
      else y = exp(d) / s;
      yr[k] = y;
    }
  }
  else if (OP == 1) {
    const double* yr = a.a + off_a;
    const double* gr = a.g + off_g;
    double s = 0.0;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) s += KIND == kLogSoftmax ? gr[k] : yr[k] * gr[k];
    s = team_sum_d<NW>(s, red[0]);
    double* dr = a.out + off_o;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) {
      const double y = yr[k], gg = gr[k];
      dr[k] = KIND == kLogSoftmax ? gg - exp(y) * s : y * (gg - s);
    }
  }
  else if (OP == 2) {
    const double* xr = a.a + off_a;
    const double K = a.sumsq ? 0.0 : xr[0];  // sums about the row's first entry: no cancellation
    double s = 0.0, q = 0.0;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) {
      const double d = xr[k] - K;
      s += d;
      q += d * d;
    }
    s = team_sum_d<NW>(s, red[0]);
    q = team_sum_d<NW>(q, red[1]);
    const double nn = static_cast<double>(n);
    const double dm = s / nn;
    const double mean = K + dm;
    const double var = n <= 1 ? 1.0 : fmax(q / nn - dm * dm, 0.0);
    if (t == 0) {
      a.stats[g + col * a.ld_stats] = mean;
      a.stats[a.map.groups + g + col * a.ld_stats] = var;
    }
    const double inv_stdev = 1.0 / sqrt(var + a.eps);
    double* yr = a.out + off_o;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) {
      double y = (xr[k] - mean) * inv_stdev;
      if (a.gamma) y *= a.gamma[k];
      if (a.beta) y += a.beta[k];
      yr[k] = y;
    }
  }
  else {
    const double* xr = a.a + off_a;
    const double* gr = a.g + off_g;
    const double mean = a.stats[g + col * a.ld_stats];
    const double var = a.stats[a.map.groups + g + col * a.ld_stats];
    const double inv_stdev = 1.0 / sqrt(var + a.eps);
    double A = 0.0, B = 0.0;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) {
      const double gg = a.gamma ? gr[k] * a.gamma[k] : gr[k];
      A += gg;
      B += gg * (xr[k] - mean);
    }
    A = team_sum_d<NW>(A, red[0]);
    B = team_sum_d<NW>(B, red[1]);
    const double dmean = -A * inv_stdev;
    const double dvar = -B * inv_stdev * inv_stdev * inv_stdev / 2;
    if (t == 0) {
      a.sgrad[g + col * a.ld_sgrad] = dmean;
      a.sgrad[a.map.groups + g + col * a.ld_sgrad] = dvar;
    }
    const double nn = static_cast<double>(n);
    const double c0 = dmean / nn, c1 = dvar * 2 / nn;
    double* dr = a.out + off_o;
#pragma unroll 4
    for (int64_t k = t; k < n; k += kStreamThreads) {
      const double gg = a.gamma ? gr[k] * a.gamma[k] : gr[k];
      dr[k] = gg * inv_stdev + c0 + c1 * (xr[k] - mean);
    }
  }
}

// Weight gradients of long rows: thread per entry k walks a slab of rows; grid (ceil(n/256), slabs);
// partial rows [slab][2n], added by ln_wgrad_reduce_f64.
__global__ void __launch_bounds__(256)
ln_wgrad_columns_f64(RowArgs a, int64_t rows_per_slab)
{
  const int64_t k = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (k >= a.n) return;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * rows_per_slab;
  const int64_t r1 = r0 + rows_per_slab < a.rows ? r0 + rows_per_slab : a.rows;
  double dg = 0.0, db = 0.0;
  for (int64_t row = r0; row < r1; ++row) {
    int64_t col, g;
    a.map.split(row, col, g);
    const double mean = a.stats[g + col * a.ld_stats];
    const double inv_stdev = 1.0 / sqrt(a.stats[a.map.groups + g + col * a.ld_stats] + a.eps);
    const double gg = a.g[g * a.map.stride + col * a.ldg + k];
    db += gg;
    dg += gg * (a.a[g * a.map.stride + col * a.lda + k] - mean) * inv_stdev;
  }
  double* out = a.part + static_cast<int64_t>(blockIdx.y) * 2 * a.n;
  out[k] = dg;
  out[a.n + k] = db;
}

__global__ void __launch_bounds__(256)
fill_f64(double* p, int64_t h, int64_t w, int64_t ld, double value)
{
  const int64_t total = h * w;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * 256)
    p[i % h + (i / h) * ld] = value;
}

// n == 1 (layer norm): mean = x, variance 1 (layer_norm.cpp:92-95), y from those.
__global__ void __launch_bounds__(256)
ln_fwd_single_f64(RowArgs a)
{
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (row >= a.rows) return;
  int64_t col, g;
  a.map.split(row, col, g);
  const double x = a.a[g * a.map.stride + col * a.lda];
  a.stats[g + col * a.ld_stats] = x;
  a.stats[a.map.groups + g + col * a.ld_stats] = 1.0;
  double y = (x - x) * (1.0 / sqrt(1.0 + a.eps));
  if (a.gamma) y *= a.gamma[0];
  if (a.beta) y += a.beta[0];
  a.out[g * a.map.stride + col * a.ldo] = y;
}

// ------------------------------------------------------------------ batch norm
struct BnArgs {
  const double* x;
  const double* dy;
  double* out;
  int64_t ldx, lddy, ldo, cs, w;
  int bessel, training, use_pivot;
  double eps, decay;
  double2* part;  // [C][P]
  int64_t part_channels;  // C, for the kernels that walk channels
  double* mean;
  double* var;
  const double* gamma;
  const double* beta;
  double* rmean;
  double* rvar;
  double* dscale;
  double* dbias;
  double* dmean;
  double* dvar;
};

// Entry j of channel c: column j / seg, position j % seg (seg = accesses per column segment).
// A thread's accesses are taken four at a time: load(u, column, position) for all four first, then
// use(u, column, position), so that four requests are in flight per thread.
constexpr int kBnUnroll = 4;

template <int W, typename Load, typename Use>
__device__ __forceinline__ void bn_walk(int64_t seg, int64_t w, int p, int P, Load load, Use use)
{
  // seg * w < 2^31 (host check): 32-bit division
  const unsigned total = static_cast<unsigned>(seg * w), useg = static_cast<unsigned>(seg);
  const unsigned step = static_cast<unsigned>(P) * kBnThreads;
  for (unsigned j0 = static_cast<unsigned>(p) * kBnThreads + threadIdx.x; j0 < total; j0 += kBnUnroll * step) {
    int64_t col[kBnUnroll], pos[kBnUnroll];
    bool in[kBnUnroll];
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      const unsigned j = j0 + u * step;
      in[u] = j < total && j >= j0;  // (the second test: no wrap-around near 2^32)
      const unsigned jj = in[u] ? j : j0;
      const unsigned c = jj / useg;
      col[u] = c;
      pos[u] = static_cast<int64_t>(W) * (jj - c * useg);
      load(u, col[u], pos[u]);
    }
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u)
      if (in[u]) use(u, col[u], pos[u]);
  }
}

template <int W, bool BWD>
__global__ void __launch_bounds__(kBnThreads)
bn_sums_f64(BnArgs a)
{
  __shared__ double red[2][kBnThreads / kWave];
  const int64_t c = blockIdx.x;
  const int P = gridDim.y, p = blockIdx.y;
  const double* xc = a.x + c * a.cs;
  const double* gc = BWD ? a.dy + c * a.cs : nullptr;
  const double K = BWD ? a.mean[c] : (a.use_pivot ? xc[0] : 0.0);
  double s = 0.0, q = 0.0;
  double v[kBnUnroll][W], g[kBnUnroll][W];
  bn_walk<W>(
    a.cs / W, a.w, p, P,
    [&](int u, int64_t col, int64_t pos) {
      load_w<W>(xc + col * a.ldx + pos, v[u]);
      if (BWD) load_w<W>(gc + col * a.lddy + pos, g[u]);
    },
    [&](int u, int64_t, int64_t) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        const double d = v[u][j] - K;
        if (BWD) {
          s += g[u][j];
          q += g[u][j] * d;
        }
        else {
          s += d;
          q += d * d;
        }
      }
    });
  s = team_sum_d<kBnThreads / kWave>(s, red[0]);
  q = team_sum_d<kBnThreads / kWave>(q, red[1]);
  if (threadIdx.x == 0) a.part[c * P + p] = make_double2(s, q);
}

// The P partial pairs of channel c, added in order by every thread (P <= 64, cached reads).
__device__ __forceinline__ double2 bn_merge(const double2* part, int64_t c, int P)
{
  double s = 0.0, q = 0.0;
  for (int p = 0; p < P; ++p) {
    const double2 v = part[c * P + p];
    s += v.x;
    q += v.y;
  }
  return make_double2(s, q);
}

// FROM_PART: training (statistics from the partial sums, published by workgroup 0 of the channel);
// otherwise mean / var are inputs (inference: the running statistics).
template <int W, bool FROM_PART>
__global__ void __launch_bounds__(kBnThreads)
bn_fwd_apply_f64(BnArgs a)
{
  const int64_t c = blockIdx.x;
  const int P = gridDim.y, p = blockIdx.y;
  const double* xc = a.x + c * a.cs;
  double* yc = a.out + c * a.cs;
  double mean, var;
  if (FROM_PART) {
    const int64_t n = a.cs * a.w;
    if (n <= 1) {
      mean = xc[0];
      var = 1.0;
      if (p == 0 && threadIdx.x == 0) {
        a.mean[c] = mean;
        a.var[c] = var;
      }
    }
    else {
      const double K = a.use_pivot ? xc[0] : 0.0;
      const double2 r = bn_merge(a.part, c, P);
      const double nn = static_cast<double>(n);
      const double dm = r.x / nn;
      mean = K + dm;
      var = fmax(nn * (r.y / nn - dm * dm) / (nn - (a.bessel ? 1 : 0)), a.eps);
      if (p == 0 && threadIdx.x == 0) {
        a.mean[c] = mean;
        a.var[c] = var;
        a.rmean[c] = a.decay * a.rmean[c] + (1.0 - a.decay) * mean;
        a.rvar[c] = a.decay * a.rvar[c] + (1.0 - a.decay) * var;
      }
    }
  }
  else {
    mean = a.mean[c];
    var = a.var[c];
  }
  const double inv_stdev = 1.0 / sqrt(var + a.eps);
  const double scale = a.gamma[c], bias = a.beta[c];
  double v[kBnUnroll][W];
  bn_walk<W>(
    a.cs / W, a.w, p, P, [&](int u, int64_t col, int64_t pos) { load_w<W>(xc + col * a.ldx + pos, v[u]); },
    [&](int u, int64_t col, int64_t pos) {
#pragma unroll
      for (int j = 0; j < W; ++j) v[u][j] = scale * ((v[u][j] - mean) * inv_stdev) + bias;
      store_w<W>(yc + col * a.ldo + pos, v[u]);
    });
}

template <int W>
__global__ void __launch_bounds__(kBnThreads)
bn_bwd_apply_f64(BnArgs a)
{
  const int64_t c = blockIdx.x;
  const int P = gridDim.y, p = blockIdx.y;
  const double* xc = a.x + c * a.cs;
  const double* gc = a.dy + c * a.cs;
  double* dc = a.out + c * a.cs;
  const int64_t n = a.cs * a.w;
  const double mean = a.mean[c];
  const double inv_stdev = 1.0 / sqrt(a.var[c] + a.eps);
  const double scale = a.gamma[c];
  const double2 r = bn_merge(a.part, c, P);  // A = sum dy, B = sum dy (x - mean)
  double dmean = -(scale * inv_stdev) * r.x;
  double dvar = -scale * r.y * (inv_stdev * inv_stdev * inv_stdev / 2);
  if (!a.training) dmean = dvar = 0.0;  // statistics are constants outside training
  if (p == 0 && threadIdx.x == 0) {
    a.dscale[c] = r.y * inv_stdev;
    a.dbias[c] = r.x;
    a.dmean[c] = dmean;
    a.dvar[c] = dvar;
  }
  const bool zero = n <= 1;
  const double k0 = scale * inv_stdev;
  const double c0 = dmean / static_cast<double>(n);
  const double c1 = dvar * 2 / static_cast<double>(n - (a.bessel ? 1 : 0));
  double v[kBnUnroll][W], g[kBnUnroll][W];
  bn_walk<W>(
    a.cs / W, a.w, p, P,
    [&](int u, int64_t col, int64_t pos) {
      load_w<W>(xc + col * a.ldx + pos, v[u]);
      load_w<W>(gc + col * a.lddy + pos, g[u]);
    },
    [&](int u, int64_t col, int64_t pos) {
#pragma unroll
      for (int j = 0; j < W; ++j) g[u][j] = zero ? 0.0 : g[u][j] * k0 + c0 + c1 * (v[u][j] - mean);
      store_w<W>(dc + col * a.ldo + pos, g[u]);
    });
}

// Training forward for channels of 128 KB to 400 KB (late convolution stages: many channels of few
// entries), one 1024-thread workgroup per channel: the channel waits in the workgroup between the
// statistics and the output (VR accesses of two doubles per thread in registers, LK more in LDS,
// filled from memory directly), so x crosses HBM once where bn_sums_f64 + bn_fwd_apply_f64 read it
// twice.  A workgroup walks channels c, c + grid, ...; each access of the next channel is
// requested behind the store that frees its registers or its slot.  Accesses past the channel's
// end repeat the thread's first access (every load is unconditional); they are left out of the
// sums and never stored.
constexpr int kBnChanRegs = 16;
constexpr int kBnChanLds = 9;
constexpr int kBnChanThreads = 1024;

__global__ void __launch_bounds__(kBnChanThreads)
bn_fwd_channel_f64(BnArgs a)
{
  constexpr int TPR = kBnChanThreads, NW = TPR / kWave, VR = kBnChanRegs, LK = kBnChanLds, V = VR + LK;
  typedef double v2d __attribute__((ext_vector_type(2)));
  __shared__ v2d parked[LK][TPR];
  __shared__ double red[2][NW];
  __shared__ double bc[2];
  const unsigned t = threadIdx.x;
  const unsigned seg = static_cast<unsigned>(a.cs / 2);             // accesses per column of the channel
  const unsigned total = seg * static_cast<unsigned>(a.w);
  const unsigned step_col = TPR / seg, step_pos = TPR % seg;        // access i + 1 from access i
  const unsigned col_first = t / seg, pos_first = t - col_first * seg;
  // f(i, column, position in the column in accesses, inside the channel) for the thread's accesses
  // in order; the chain of columns and positions is formed anew on every pass (kept across the
  // passes it would take two registers per access)
  auto for_each = [&](auto&& f) {
    unsigned col = col_first, pos = pos_first;
    asm volatile("" : "+v"(col), "+v"(pos));
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const bool in = t + i * TPR < total;
      f(i, in ? col : col_first, in ? pos : pos_first, in);
      col += step_col;
      pos += step_pos;
      if (pos >= seg) {
        pos -= seg;
        ++col;
      }
    }
  };
  auto slot = [&](int j) {
    unsigned first = t;
    asm volatile("" : "+v"(first));
    first &= ~unsigned(kWave - 1);
    return (__attribute__((address_space(3))) void*)&parked[j][first];
  };
  v2d xr[VR];
  auto request = [&](const double* xc) {
    for_each([&](int i, unsigned col, unsigned pos, bool) {
      const double* p = xc + col * a.ldx + 2 * pos;
      if (i < VR) xr[i < VR ? i : 0] = *reinterpret_cast<const v2d*>(p);
      else __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p, slot(i < VR ? 0 : i - VR), 16, 0, 0);
    });
  };
  int64_t c = blockIdx.x;
  if (c >= a.part_channels) return;
  request(a.x + c * a.cs);
  const double nn = static_cast<double>(a.cs * a.w);
  for (; c < a.part_channels; c += gridDim.x) {
    const double* xc = a.x + c * a.cs;
    double* yc = a.out + c * a.cs;
    const double K = a.use_pivot ? xc[0] : 0.0;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the slots in LDS are written by the memory system
    double s = 0.0, q = 0.0;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const v2d v = i < VR ? xr[i < VR ? i : 0] : parked[i < VR ? 0 : i - VR][t];
      const bool in = t + i * TPR < total;
      const double d0 = v.x - K, d1 = v.y - K;
      s += in ? d0 + d1 : 0.0;
      q += in ? d0 * d0 + d1 * d1 : 0.0;
      if (i >= VR) __builtin_amdgcn_sched_barrier(0);  // one slot at a time: the registers are full
    }
    s = wave_sum_in_last_d(s);
    q = wave_sum_in_last_d(q);
    if ((t & (kWave - 1)) == kWave - 1) {
      red[0][t / kWave] = s;
      red[1][t / kWave] = q;
    }
    __syncthreads();
    if (t == 0) {
      double ts = 0.0, tq = 0.0;
      for (int i = 0; i < NW; ++i) {
        ts += red[0][i];
        tq += red[1][i];
      }
      const double dm = ts / nn;
      const double mean = K + dm;
      const double var = fmax(nn * (tq / nn - dm * dm) / (nn - (a.bessel ? 1 : 0)), a.eps);
      bc[0] = mean;
      bc[1] = var;
      a.mean[c] = mean;
      a.var[c] = var;
      a.rmean[c] = a.decay * a.rmean[c] + (1.0 - a.decay) * mean;
      a.rvar[c] = a.decay * a.rvar[c] + (1.0 - a.decay) * var;
    }
    __syncthreads();
    const double mean = bc[0];
    const double inv_stdev = 1.0 / sqrt(bc[1] + a.eps);
    const double scale = a.gamma[c], bias = a.beta[c];
    const int64_t cn = c + gridDim.x;
    const bool more = cn < a.part_channels;
    const double* xn = a.x + (more ? cn : c) * a.cs;
    for_each([&](int i, unsigned col, unsigned pos, bool in) {
      v2d v = i < VR ? xr[i < VR ? i : 0] : parked[i < VR ? 0 : i - VR][t];
      v.x = scale * ((v.x - mean) * inv_stdev) + bias;
      v.y = scale * ((v.y - mean) * inv_stdev) + bias;
      if (in) __builtin_nontemporal_store(v, reinterpret_cast<v2d*>(yc + col * a.ldo + 2 * pos));
      asm volatile("" ::: "memory");  // the slot has been read before the next channel's request overwrites it
      if (more) {
        const double* p = xn + col * a.ldx + 2 * pos;
        if (i < VR) xr[i < VR ? i : 0] = *reinterpret_cast<const v2d*>(p);
        else __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p, slot(i < VR ? 0 : i - VR), 16, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);  // one access at a time
    });
    // bc and red are written again only after the next channel's first barrier
  }
}

// Backward for the same channels: dy waits in the workgroup (registers and LDS as x does in
// bn_fwd_channel_f64) while x streams through the registers twice, five accesses at a time: once
// for the two sums, once for dx.  Four passes over HBM (x, dy, x, dx) where bn_sums_f64 +
// bn_bwd_apply_f64 make five.  The next channel's dy is requested behind the stores of dx.
__global__ void __launch_bounds__(kBnChanThreads)
bn_bwd_channel_f64(BnArgs a)
{
  constexpr int TPR = kBnChanThreads, NW = TPR / kWave, VR = kBnChanRegs, LK = kBnChanLds, V = VR + LK, CH = 5;
  static_assert(V % CH == 0, "x streams through the registers CH accesses at a time");
  typedef double v2d __attribute__((ext_vector_type(2)));
  __shared__ v2d parked[LK][TPR];
  __shared__ double red[2][NW];
  __shared__ double bc[2];
  const unsigned t = threadIdx.x;
  const unsigned seg = static_cast<unsigned>(a.cs / 2);
  const unsigned total = seg * static_cast<unsigned>(a.w);
  const unsigned step_col = TPR / seg, step_pos = TPR % seg;
  const unsigned col_first = t / seg, pos_first = t - col_first * seg;
  auto advance = [&](unsigned& col, unsigned& pos) {
    col += step_col;
    pos += step_pos;
    if (pos >= seg) {
      pos -= seg;
      ++col;
    }
  };
  auto slot = [&](int j) {
    unsigned first = t;
    asm volatile("" : "+v"(first));
    first &= ~unsigned(kWave - 1);
    return (__attribute__((address_space(3))) void*)&parked[j][first];
  };
  v2d gr[VR];
  auto request_one = [&](const double* gc, int i, unsigned col, unsigned pos) {
    const double* p = gc + col * a.lddy + 2 * pos;
    if (i < VR) gr[i < VR ? i : 0] = *reinterpret_cast<const v2d*>(p);
    else __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p, slot(i < VR ? 0 : i - VR), 16, 0, 0);
  };
  int64_t c = blockIdx.x;
  if (c >= a.part_channels) return;
  {
    unsigned col = col_first, pos = pos_first;
    asm volatile("" : "+v"(col), "+v"(pos));
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const bool in = t + i * TPR < total;
      request_one(a.dy + c * a.cs, i, in ? col : col_first, in ? pos : pos_first);
      advance(col, pos);
    }
  }
  const int64_t n = a.cs * a.w;
  for (; c < a.part_channels; c += gridDim.x) {
    const double* xc = a.x + c * a.cs;
    double* dc = a.out + c * a.cs;
    const double mean = a.mean[c];
    const double inv_stdev = 1.0 / sqrt(a.var[c] + a.eps);
    const double scale = a.gamma[c];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the slots in LDS are written by the memory system
    double A = 0.0, B = 0.0;
    {
      unsigned col = col_first, pos = pos_first;
      asm volatile("" : "+v"(col), "+v"(pos));
#pragma unroll
      for (int i0 = 0; i0 < V; i0 += CH) {
        v2d xv[CH];
#pragma unroll
        for (int k = 0; k < CH; ++k) {
          const bool in = t + (i0 + k) * TPR < total;
          xv[k] = *reinterpret_cast<const v2d*>(xc + (in ? col : col_first) * a.ldx + 2 * (in ? pos : pos_first));
          advance(col, pos);
        }
#pragma unroll
        for (int k = 0; k < CH; ++k) {
          const int i = i0 + k;
          const v2d g = i < VR ? gr[i < VR ? i : 0] : parked[i < VR ? 0 : i - VR][t];
          const bool in = t + i * TPR < total;
          A += in ? g.x + g.y : 0.0;
          B += in ? g.x * (xv[k].x - mean) + g.y * (xv[k].y - mean) : 0.0;
        }
        __builtin_amdgcn_sched_barrier(0);  // one group of accesses at a time: the registers are full
      }
    }
    A = wave_sum_in_last_d(A);
    B = wave_sum_in_last_d(B);
    if ((t & (kWave - 1)) == kWave - 1) {
      red[0][t / kWave] = A;
      red[1][t / kWave] = B;
    }
    __syncthreads();
    if (t == 0) {
      double ta = 0.0, tb = 0.0;
      for (int i = 0; i < NW; ++i) {
        ta += red[0][i];
        tb += red[1][i];
      }
      double dmean = -(scale * inv_stdev) * ta;
      double dvar = -scale * tb * (inv_stdev * inv_stdev * inv_stdev / 2);
      if (!a.training) dmean = dvar = 0.0;  // statistics are constants outside training
      a.dscale[c] = tb * inv_stdev;
      a.dbias[c] = ta;
      a.dmean[c] = dmean;
      a.dvar[c] = dvar;
      bc[0] = dmean / static_cast<double>(n);
      bc[1] = dvar * 2 / static_cast<double>(n - (a.bessel ? 1 : 0));
    }
    __syncthreads();
    const double k0 = scale * inv_stdev, c0 = bc[0], c1 = bc[1];
    const int64_t cn = c + gridDim.x;
    const bool more = cn < a.part_channels;
    const double* gn = a.dy + (more ? cn : c) * a.cs;
    {
      unsigned col = col_first, pos = pos_first;
      asm volatile("" : "+v"(col), "+v"(pos));
#pragma unroll
      for (int i0 = 0; i0 < V; i0 += CH) {
        v2d xv[CH];
        unsigned ccol[CH], cpos[CH];
#pragma unroll
        for (int k = 0; k < CH; ++k) {
          const bool in = t + (i0 + k) * TPR < total;
          ccol[k] = in ? col : col_first;
          cpos[k] = in ? pos : pos_first;
          xv[k] = *reinterpret_cast<const v2d*>(xc + ccol[k] * a.ldx + 2 * cpos[k]);
          advance(col, pos);
        }
#pragma unroll
        for (int k = 0; k < CH; ++k) {
          const int i = i0 + k;
          const v2d g = i < VR ? gr[i < VR ? i : 0] : parked[i < VR ? 0 : i - VR][t];
          v2d d;
          d.x = g.x * k0 + c0 + c1 * (xv[k].x - mean);
          d.y = g.y * k0 + c0 + c1 * (xv[k].y - mean);
          if (t + i * TPR < total) __builtin_nontemporal_store(d, reinterpret_cast<v2d*>(dc + ccol[k] * a.ldo + 2 * cpos[k]));
        }
        asm volatile("" ::: "memory");  // the slots have been read before the next channel's requests overwrite them
        if (more) {
#pragma unroll
          for (int k = 0; k < CH; ++k) request_one(gn, i0 + k, ccol[k], cpos[k]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
}

// ================================================================== host side
static bool aligned_rows(const void* p, int64_t stride, int64_t ld, int64_t groups, int64_t w)
{
  return aligned16(p) && (groups <= 1 || stride % 2 == 0) && (w <= 1 || ld % 2 == 0);
}

// Workgroups of a row launch: a few per compute unit.  With weight gradients every team leaves a
// partial row of 2n doubles, so the launch is held to kWgradMaxGroups workgroups (at most
// 4 * kWgradMaxGroups partial rows, which is what the workspace is sized for).
constexpr int64_t kWgradMaxGroups = 512;

static int64_t row_grid(int64_t rows, int teams, bool wgrad = false)
{
  int cus = compute_units();
  if (cus < 1) cus = 256;
  const int64_t want = ceil_div(rows, teams);
  int64_t cap = static_cast<int64_t>(cus) * 8;
  if (wgrad && cap > kWgradMaxGroups) cap = kWgradMaxGroups;
  return want < cap ? want : cap;
}

#define LBN_F64_SHAPES(X, W)                                                                          \
  X(64, 1, W) X(64, 2, W) X(256, 1, W) X(256, 2, W)                                                   \
  X(1024, 1, W) X(1024, 2, W) X(1024, 4, W) X(1024, 8, W) X(1024, 16, W)

static int sm_check(int64_t G, int64_t n, int64_t stride, int64_t w, const int64_t* lds, int nld)
{
  if (G < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = G > 0 ? (G - 1) * stride + n : 0;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < height) return LBN_ERR_INVALID_ARGUMENT;
  if (G * w > (int64_t(1) << 30) || n > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  return LBN_OK;
}

template <int KIND>
static int sm_fwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, const double* x, int64_t ldx,
                  double* y, int64_t ldy)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = sm_check(G, n, stride, w, lds, 2)) return e;
  if (G == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !y) return LBN_ERR_INVALID_ARGUMENT;
  RowArgs a{};
  a.a = x, a.out = y, a.lda = ldx, a.ldo = ldy, a.map = RowMap{G, stride}, a.rows = G * w, a.n = static_cast<int>(n);
  const bool vec = n % 2 == 0 && aligned_rows(x, stride, ldx, G, w) && aligned_rows(y, stride, ldy, G, w);
  const int W = vec ? 2 : 1;
  a.units = static_cast<int>(n / W);
  const RowShape s = pick_shape(a.units, a.rows);
#define X(TPR, V, WW)                                                                                   \
  if (s.tpr == TPR && s.v == V && W == WW) {                                                            \
    int64_t grid = row_grid(a.rows, Team<TPR>::kTeams);                                                 \
    if (TPR == 1024 && V >= 16) {                                                                       \
      /* a row fills a compute unit's registers (one workgroup per unit): one resident wave of */       \
      /* workgroups, each walking its rows with the next row's loads behind the stores, instead of */   \
      /* one workgroup after another */                                                                 \
      const int cap = resident_blocks(sm_fwd_rows_f64<KIND, TPR, V, WW>, Team<TPR>::kThreads);          \
      if (cap >= 1 && cap <= compute_units() && grid > cap) grid = cap;                                 \
    }                                                                                                   \
    hipLaunchKernelGGL((sm_fwd_rows_f64<KIND, TPR, V, WW>), dim3(static_cast<unsigned>(grid)),          \
                       dim3(Team<TPR>::kThreads), 0, st, a);                                            \
    return launch_status();                                                                             \
  }
  LBN_F64_SHAPES(X, 1) LBN_F64_SHAPES(X, 2)
#undef X
  hipLaunchKernelGGL((rows_stream_f64<0, KIND>), dim3(static_cast<unsigned>(a.rows)), dim3(kStreamThreads), 0, st, a);
  return launch_status();
}

template <int KIND>
static int sm_bwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, const double* y, int64_t ldy,
                  const double* dy, int64_t lddy, double* dx, int64_t lddx)
{
  const int64_t lds[3] = {ldy, lddy, lddx};
  if (int e = sm_check(G, n, stride, w, lds, 3)) return e;
  if (G == 0 || n == 0 || w == 0) return LBN_OK;
  if (!y || !dy || !dx) return LBN_ERR_INVALID_ARGUMENT;
  RowArgs a{};
  a.a = y, a.g = dy, a.out = dx, a.lda = ldy, a.ldg = lddy, a.ldo = lddx, a.map = RowMap{G, stride};
  a.rows = G * w, a.n = static_cast<int>(n);
  const bool vec = n % 2 == 0 && aligned_rows(y, stride, ldy, G, w) && aligned_rows(dy, stride, lddy, G, w) &&
                   aligned_rows(dx, stride, lddx, G, w);
  const int W = vec ? 2 : 1;
  a.units = static_cast<int>(n / W);
  RowShape s = pick_shape(a.units, a.rows);
  if (s.v > 8) s = RowShape{0, 0};  // two tensors in registers: at most 8 accesses each
#define X(TPR, V, WW)                                                                                   \
  if (V <= 8 && s.tpr == TPR && s.v == V && W == WW) {                                                  \
    hipLaunchKernelGGL((sm_bwd_rows_f64<KIND, TPR, (V <= 8 ? V : 8), WW>),                              \
                       dim3(static_cast<unsigned>(row_grid(a.rows, Team<TPR>::kTeams))),                \
                       dim3(Team<TPR>::kThreads), 0, st, a);                                            \
    return launch_status();                                                                             \
  }
  LBN_F64_SHAPES(X, 1) LBN_F64_SHAPES(X, 2)
#undef X
  if (W == 2 && a.units <= 16 * 1024) {
    // up to 32768 doubles: y in registers, dy in registers and LDS, one workgroup per compute unit
    int cus = compute_units();
    if (cus < 1) cus = 256;
    const int64_t grid = a.rows < cus ? a.rows : cus;
    hipLaunchKernelGGL((sm_bwd_rows_parked_f64<KIND, 16, 7>), dim3(static_cast<unsigned>(grid)), dim3(1024), 0, st, a);
    return launch_status();
  }
  hipLaunchKernelGGL((rows_stream_f64<1, KIND>), dim3(static_cast<unsigned>(a.rows)), dim3(kStreamThreads), 0, st, a);
  return launch_status();
}

static size_t ln_bwd_workspace(int64_t n, int64_t rows)
{
  if (n <= 0 || rows <= 0) return 0;
  const int64_t teams = kWgradMaxGroups * 4;  // the largest launch: four teams per workgroup
  const int64_t parts = rows < teams ? rows : teams;
  return static_cast<size_t>(parts) * 2 * n * sizeof(double);
}

static int ln_fwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, double eps, const double* x,
                  int64_t ldx, double* y, int64_t ldy, double* stats, int64_t ld_stats, const double* gamma,
                  const double* beta, int flags)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = sm_check(G, n, stride, w, lds, 2)) return e;
  if (G == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !y || !stats || (w > 1 && ld_stats < 2 * G)) return LBN_ERR_INVALID_ARGUMENT;
  RowArgs a{};
  a.a = x, a.out = y, a.lda = ldx, a.ldo = ldy, a.map = RowMap{G, stride}, a.rows = G * w, a.n = static_cast<int>(n);
  a.eps = eps, a.stats = stats, a.ld_stats = ld_stats, a.gamma = gamma, a.beta = beta;
  a.sumsq = (flags & LBN_STATS_SUMSQ) ? 1 : 0;
  if (n == 1) {
    hipLaunchKernelGGL(ln_fwd_single_f64, dim3(static_cast<unsigned>(ceil_div(a.rows, 256))), dim3(256), 0, st, a);
    return launch_status();
  }
  const bool vec = n % 2 == 0 && aligned_rows(x, stride, ldx, G, w) && aligned_rows(y, stride, ldy, G, w);
  const int W = vec ? 2 : 1;
  a.units = static_cast<int>(n / W);
  const RowShape s = pick_shape(a.units, a.rows);
#define X(TPR, V, WW)                                                                                   \
  if (s.tpr == TPR && s.v == V && W == WW) {                                                            \
    hipLaunchKernelGGL((ln_fwd_rows_f64<TPR, V, WW>), dim3(static_cast<unsigned>(row_grid(a.rows, Team<TPR>::kTeams))), \
                       dim3(Team<TPR>::kThreads), 0, st, a);                                            \
    return launch_status();                                                                             \
  }
  LBN_F64_SHAPES(X, 1) LBN_F64_SHAPES(X, 2)
#undef X
  hipLaunchKernelGGL((rows_stream_f64<2, 0>), dim3(static_cast<unsigned>(a.rows)), dim3(kStreamThreads), 0, st, a);
  return launch_status();
}

static int ln_bwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, double eps, const double* x,
                  int64_t ldx, const double* dy, int64_t lddy, double* dx, int64_t lddx, const double* stats,
                  int64_t ld_stats, double* sgrad, int64_t ld_sgrad, const double* gamma, double* dgamma,
                  double* dbeta, void* ws, size_t ws_bytes)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = sm_check(G, n, stride, w, lds, 3)) return e;
  if (G == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !dy || !dx || !stats || !sgrad || (w > 1 && (ld_stats < 2 * G || ld_sgrad < 2 * G)))
    return LBN_ERR_INVALID_ARGUMENT;
  if (dgamma && !gamma) return LBN_ERR_INVALID_ARGUMENT;
  const bool wgrad = dgamma || dbeta;
  const int64_t rows = G * w;
  if (n <= 1) {
    // a single entry per group: the output is constant and every gradient zero
    // (layer_norm.cpp:189-192; the weight-gradient buffers were zeroed at :300-309)
    const int64_t height = (G - 1) * stride + n;
    const int64_t want = ceil_div(height * w, 256);
    hipLaunchKernelGGL(fill_f64, dim3(static_cast<unsigned>(want > 4096 ? 4096 : want)), dim3(256), 0, st, dx, height,
                       w, lddx, 0.0);
    if (dgamma) hipLaunchKernelGGL(fill_f64, dim3(1), dim3(256), 0, st, dgamma, n, int64_t(1), n, 0.0);
    if (dbeta) hipLaunchKernelGGL(fill_f64, dim3(1), dim3(256), 0, st, dbeta, n, int64_t(1), n, 0.0);
    return launch_status();
  }
  RowArgs a{};
  a.a = x, a.g = dy, a.out = dx, a.lda = ldx, a.ldg = lddy, a.ldo = lddx, a.map = RowMap{G, stride};
  a.rows = rows, a.n = static_cast<int>(n), a.eps = eps, a.stats = const_cast<double*>(stats), a.ld_stats = ld_stats;
  a.sgrad = sgrad, a.ld_sgrad = ld_sgrad, a.gamma = gamma, a.part = static_cast<double*>(ws);
  if (wgrad && (!ws || ws_bytes < ln_bwd_workspace(n, rows) || !aligned16(ws))) return LBN_ERR_WORKSPACE;
  const bool vec = n % 2 == 0 && aligned_rows(x, stride, ldx, G, w) && aligned_rows(dy, stride, lddy, G, w) &&
                   aligned_rows(dx, stride, lddx, G, w);
  const int W = vec ? 2 : 1;
  a.units = static_cast<int>(n / W);
  RowShape s = pick_shape(a.units, rows);
  if (s.v > 8) s = RowShape{0, 0};
#define X(TPR, V, WW)                                                                                   \
  if (V <= 8 && s.tpr == TPR && s.v == V && W == WW) {                                                  \
    constexpr int VV = V <= 8 ? V : 8;                                                                  \
    const int64_t grid = row_grid(rows, Team<TPR>::kTeams, wgrad);                                      \
    if (wgrad) {                                                                                        \
      hipLaunchKernelGGL((ln_bwd_rows_f64<TPR, VV, WW, true>), dim3(static_cast<unsigned>(grid)),       \
                         dim3(Team<TPR>::kThreads), 0, st, a);                                          \
      hipLaunchKernelGGL(ln_wgrad_reduce_f64, dim3(static_cast<unsigned>(ceil_div(2 * n, 16))), dim3(256), 0, st, \
                         a.part, grid * Team<TPR>::kTeams, n, dgamma, dbeta);                           \
    }                                                                                                   \
    else {                                                                                              \
      hipLaunchKernelGGL((ln_bwd_rows_f64<TPR, VV, WW, false>), dim3(static_cast<unsigned>(grid)),      \
                         dim3(Team<TPR>::kThreads), 0, st, a);                                          \
    }                                                                                                   \
    return launch_status();                                                                             \
  }
  LBN_F64_SHAPES(X, 1) LBN_F64_SHAPES(X, 2)
#undef X
  hipLaunchKernelGGL((rows_stream_f64<3, 0>), dim3(static_cast<unsigned>(rows)), dim3(kStreamThreads), 0, st, a);
  if (wgrad) {
    int64_t slabs = ceil_div(2048, ceil_div(n, 256));
    if (slabs > rows) slabs = rows;
    if (slabs > 256) slabs = 256;
    const int64_t per = ceil_div(rows, slabs);
    slabs = ceil_div(rows, per);
    hipLaunchKernelGGL(ln_wgrad_columns_f64, dim3(static_cast<unsigned>(ceil_div(n, 256)), static_cast<unsigned>(slabs)),
                       dim3(256), 0, st, a, per);
    hipLaunchKernelGGL(ln_wgrad_reduce_f64, dim3(static_cast<unsigned>(ceil_div(2 * n, 16))), dim3(256), 0, st, a.part,
                       slabs, n, dgamma, dbeta);
  }
  return launch_status();
}

static int bn_split(int64_t C, int64_t cs, int64_t w)
{
  int64_t P = ceil_div(2048, C);
  const int64_t most = ceil_div(cs * w, 2 * kBnThreads);
  if (P > most) P = most;
  if (P > kBnMaxSplit) P = kBnMaxSplit;
  return static_cast<int>(P < 1 ? 1 : P);
}

static int bn_check(int64_t C, int64_t cs, int64_t w, const int64_t* lds, int nld)
{
  if (C < 0 || cs < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < C * cs) return LBN_ERR_INVALID_ARGUMENT;
  if (C > (int64_t(1) << 30) || cs * w >= (int64_t(1) << 31)) return LBN_ERR_UNSUPPORTED;
  return LBN_OK;
}

static bool bn_vec(int64_t cs, int64_t w, const void* p, int64_t ld)
{
  return cs % 2 == 0 && aligned16(p) && (w <= 1 || ld % 2 == 0);
}

}  // namespace f64
}  // namespace lbn

using namespace lbn;
using namespace lbn::f64;

extern "C" {

int lbn_softmax_fwd_f64(lbn_stream_t stream, int64_t height, int64_t width, const double* x, int64_t ldx,
                        double* y, int64_t ldy)
{
  return f64::sm_fwd<kSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy);
}

int lbn_softmax_bwd_f64(lbn_stream_t stream, int64_t height, int64_t width, const double* y, int64_t ldy,
                        const double* dy, int64_t lddy, double* dx, int64_t lddx)
{
  return f64::sm_bwd<kSoftmax>(as_stream(stream), 1, height, height, width, y, ldy, dy, lddy, dx, lddx);
}

int lbn_log_softmax_fwd_f64(lbn_stream_t stream, int64_t height, int64_t width, const double* x, int64_t ldx,
                            double* y, int64_t ldy)
{
  return f64::sm_fwd<kLogSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy);
}

int lbn_log_softmax_bwd_f64(lbn_stream_t stream, int64_t height, int64_t width, const double* y, int64_t ldy,
                            const double* dy, int64_t lddy, double* dx, int64_t lddx)
{
  return f64::sm_bwd<kLogSoftmax>(as_stream(stream), 1, height, height, width, y, ldy, dy, lddy, dx, lddx);
}

int lbn_channelwise_softmax_fwd_f64(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width, const double* x, int64_t ldx,
                                    double* y, int64_t ldy)
{
  return f64::sm_fwd<kChannelwise>(as_stream(stream), channels, channel_size, channel_stride, width, x, ldx, y, ldy);
}

int lbn_channelwise_softmax_bwd_f64(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width, const double* y, int64_t ldy,
                                    const double* dy, int64_t lddy, double* dx, int64_t lddx)
{
  return f64::sm_bwd<kChannelwise>(as_stream(stream), channels, channel_size, channel_stride, width, y, ldy, dy, lddy,
                                   dx, lddx);
}

int lbn_layer_norm_fwd_f64(lbn_stream_t stream, int64_t num_groups, int64_t norm_size, int64_t norm_stride,
                           int64_t width, double epsilon, const double* x, int64_t ldx, double* y, int64_t ldy,
                           double* stats, int64_t ld_stats, const double* scale, const double* bias, int flags)
{
  return f64::ln_fwd(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon, x, ldx, y, ldy, stats,
                     ld_stats, scale, bias, flags);
}

size_t lbn_layer_norm_bwd_workspace_bytes_f64(int64_t num_groups, int64_t norm_size, int64_t width,
                                              int has_weight_grads)
{
  if (!has_weight_grads || num_groups <= 0 || width <= 0) return 0;
  return f64::ln_bwd_workspace(norm_size, num_groups * width);
}

int lbn_layer_norm_bwd_f64(lbn_stream_t stream, int64_t num_groups, int64_t norm_size, int64_t norm_stride,
                           int64_t width, double epsilon, const double* x, int64_t ldx, const double* dy,
                           int64_t lddy, double* dx, int64_t lddx, const double* stats, int64_t ld_stats,
                           double* stats_grad, int64_t ld_stats_grad, const double* scale, double* dscale,
                           double* dbias, void* workspace, size_t workspace_bytes)
{
  return f64::ln_bwd(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon, x, ldx, dy, lddy, dx, lddx,
                     stats, ld_stats, stats_grad, ld_stats_grad, scale, dscale, dbias, workspace, workspace_bytes);
}

size_t lbn_batch_norm_workspace_bytes_f64(int64_t channels, int64_t channel_size, int64_t width)
{
  if (channels <= 0 || channel_size <= 0 || width <= 0) return 0;
  return static_cast<size_t>(channels) * f64::kBnMaxSplit * sizeof(double2);
}

int lbn_batch_norm_fwd_f64(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel, double epsilon,
                           double decay, int training, const double* x, int64_t ldx, double* y, int64_t ldy,
                           double* mean, double* var, const double* scale, const double* bias,
                           double* running_mean, double* running_var, void* workspace, size_t workspace_bytes,
                           int flags)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = f64::bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !y || !scale || !bias || !running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
  if (training && (!mean || !var)) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  f64::BnArgs a{};
  a.x = x, a.out = y, a.ldx = ldx, a.ldo = ldy, a.cs = cs, a.w = w, a.bessel = bessel, a.training = training;
  a.use_pivot = (flags & LBN_STATS_SUMSQ) ? 0 : 1, a.eps = epsilon, a.decay = decay;
  a.gamma = scale, a.beta = bias, a.rmean = running_mean, a.rvar = running_var;
  const int P = f64::bn_split(C, cs, w);
  const dim3 grid(static_cast<unsigned>(C), P);
  const bool vec = f64::bn_vec(cs, w, x, ldx) && f64::bn_vec(cs, w, y, ldy);
  if (!training) {
    a.mean = running_mean, a.var = running_var;
    if (vec) hipLaunchKernelGGL((bn_fwd_apply_f64<2, false>), grid, dim3(f64::kBnThreads), 0, st, a);
    else hipLaunchKernelGGL((bn_fwd_apply_f64<1, false>), grid, dim3(f64::kBnThreads), 0, st, a);
    return launch_status();
  }
  if (!workspace || workspace_bytes < lbn_batch_norm_workspace_bytes_f64(C, cs, w) || !aligned16(workspace))
    return LBN_ERR_WORKSPACE;
  a.part = static_cast<double2*>(workspace), a.mean = mean, a.var = var;
  a.part_channels = C;
  {
    // channels that fit a compute unit's registers and LDS, at least one per unit: x is read once
    const int64_t accesses = cs / 2 * w;
    const int cus = compute_units();
    if (vec && cs * w > 1 && accesses >= 8 * f64::kBnChanThreads &&
        accesses <= (f64::kBnChanRegs + f64::kBnChanLds) * f64::kBnChanThreads && cus > 0 && C >= cus &&
        !std::getenv("LBN_F64_BN_TWO_PASS")) {
      hipLaunchKernelGGL(f64::bn_fwd_channel_f64, dim3(static_cast<unsigned>(cus)), dim3(f64::kBnChanThreads), 0, st, a);
      return launch_status();
    }
  }
  if (vec) {
    hipLaunchKernelGGL((bn_sums_f64<2, false>), grid, dim3(f64::kBnThreads), 0, st, a);
    hipLaunchKernelGGL((bn_fwd_apply_f64<2, true>), grid, dim3(f64::kBnThreads), 0, st, a);
  }
  else {
    hipLaunchKernelGGL((bn_sums_f64<1, false>), grid, dim3(f64::kBnThreads), 0, st, a);
    hipLaunchKernelGGL((bn_fwd_apply_f64<1, true>), grid, dim3(f64::kBnThreads), 0, st, a);
  }
  return launch_status();
}

int lbn_batch_norm_bwd_f64(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel, double epsilon,
                           int training, const double* x, int64_t ldx, const double* dy, int64_t lddy, double* dx,
                           int64_t lddx, const double* mean, const double* var, const double* running_mean,
                           const double* running_var, const double* scale, double* dscale, double* dbias,
                           double* dmean, double* dvar, void* workspace, size_t workspace_bytes)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = f64::bn_check(C, cs, w, lds, 3)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  const double* use_mean = training ? mean : running_mean;
  const double* use_var = training ? var : running_var;
  if (!x || !dy || !dx || !use_mean || !use_var || !scale || !dscale || !dbias || !dmean || !dvar)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < lbn_batch_norm_workspace_bytes_f64(C, cs, w) || !aligned16(workspace))
    return LBN_ERR_WORKSPACE;
  hipStream_t st = as_stream(stream);
  f64::BnArgs a{};
  a.x = x, a.dy = dy, a.out = dx, a.ldx = ldx, a.lddy = lddy, a.ldo = lddx, a.cs = cs, a.w = w, a.bessel = bessel;
  a.training = training, a.eps = epsilon, a.part = static_cast<double2*>(workspace);
  a.mean = const_cast<double*>(use_mean), a.var = const_cast<double*>(use_var), a.gamma = scale;
  a.dscale = dscale, a.dbias = dbias, a.dmean = dmean, a.dvar = dvar;
  const int P = f64::bn_split(C, cs, w);
  const dim3 grid(static_cast<unsigned>(C), P);
  const bool vec = f64::bn_vec(cs, w, x, ldx) && f64::bn_vec(cs, w, dy, lddy) && f64::bn_vec(cs, w, dx, lddx);
  a.part_channels = C;
  {
    // channels that fit a compute unit's registers and LDS, at least one per unit: dy is read once
    const int64_t accesses = cs / 2 * w;
    const int cus = compute_units();
    if (vec && cs * w > 1 && accesses >= 8 * f64::kBnChanThreads &&
        accesses <= (f64::kBnChanRegs + f64::kBnChanLds) * f64::kBnChanThreads && cus > 0 && C >= cus &&
        !std::getenv("LBN_F64_BN_TWO_PASS")) {
      hipLaunchKernelGGL(f64::bn_bwd_channel_f64, dim3(static_cast<unsigned>(cus)), dim3(f64::kBnChanThreads), 0, st, a);
      return launch_status();
    }
  }
  if (vec) {
    hipLaunchKernelGGL((bn_sums_f64<2, true>), grid, dim3(f64::kBnThreads), 0, st, a);
    hipLaunchKernelGGL((bn_bwd_apply_f64<2>), grid, dim3(f64::kBnThreads), 0, st, a);
  }
  else {
    hipLaunchKernelGGL((bn_sums_f64<1, true>), grid, dim3(f64::kBnThreads), 0, st, a);
    hipLaunchKernelGGL((bn_bwd_apply_f64<1>), grid, dim3(f64::kBnThreads), 0, st, a);
  }
  return launch_status();
}

}  // extern "C"
