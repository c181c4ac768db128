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
//  * generic kernels (one 256-thread block per row, scalar access) cover rows that
//    are unaligned, not a multiple of the vector length, or too long for registers.
#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {

// ================================================================== forward
template <typename T, int TPR, int V>
__global__ void __launch_bounds__(RowBlock<TPR>::kThreads)
ln_fwd_rows(const T* __restrict__ x, T* __restrict__ y, int64_t ldx, int64_t ldy, RowMap map,
            int64_t rows, int nvec, int n, float eps, float* __restrict__ stats,
            int64_t ld_stats, const float* __restrict__ gamma, const float* __restrict__ beta,
            int sumsq)
{
  using B = RowBlock<TPR>;
  using IO = Vec16<T>;
  constexpr int VE = IO::N;
  constexpr int NW = B::kWavesPerTeam;
  __shared__ float red[2][2 * NW];
  const int tid = threadIdx.x;
  const int team = wave_index() / NW;  // wave-uniform: a team is a whole number of waves
  const int t = tid - team * TPR;
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * B::kTeams + team;
  if (B::kTeams > 1 && row >= rows) return;

  const T* xr = x + map.offset(row, ldx);
  float v[V][VE];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int idx = t + i * TPR;
    if (idx < nvec) {
      IO::load(xr + VE * idx, v[i]);
    }
    else {
#pragma unroll
      for (int k = 0; k < VE; ++k) v[i][k] = 0.f;
    }
  }

  const float inv_n = 1.0f / static_cast<float>(n);
  float mean, var;
  if (sumsq) {
    float s = 0.f, q = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        s += v[i][k];
        q += v[i][k] * v[i][k];
      }
    team_sum2<NW>(s, q, red[0], wv, lane);
    mean = s / static_cast<float>(n);
    const float sqmean = q / static_cast<float>(n);
    var = fmaxf(sqmean - mean * mean, 0.f);
  }
  else {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < VE; ++k) s += v[i][k];
    s = team_sum<NW>(s, red[0], wv, lane);
    mean = s * inv_n;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const bool ok = (t + i * TPR) < nvec;
#pragma unroll
      for (int k = 0; k < VE; ++k) {
        const float d = v[i][k] - mean;
        q += ok ? d * d : 0.f;
      }
    }
    q = team_sum<NW>(q, red[1], wv, lane);
    var = q * inv_n;
  }
  const float inv_stdev = 1.0f / sqrtf(var + eps);

  if (t == 0) {
    int64_t col, g;
    map.split(row, col, g);
    stats[g + col * ld_stats] = mean;
    stats[map.groups + g + col * ld_stats] = var;
  }

  T* yr = y + map.offset(row, ldy);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int idx = t + i * TPR;
    if (idx < nvec) {
#pragma unroll
      for (int k = 0; k < VE; ++k) v[i][k] = (v[i][k] - mean) * inv_stdev;
      if (gamma) {
#pragma unroll
        for (int k4 = 0; k4 < VE; k4 += 4) {
          float w[4];
          Vec16<float>::load(gamma + VE * idx + k4, w);
#pragma unroll
          for (int k = 0; k < 4; ++k) v[i][k4 + k] *= w[k];
        }
      }
      if (beta) {
#pragma unroll
        for (int k4 = 0; k4 < VE; k4 += 4) {
          float w[4];
          Vec16<float>::load(beta + VE * idx + k4, w);
#pragma unroll
          for (int k = 0; k < 4; ++k) v[i][k4 + k] += w[k];
        }
      }
      IO::store(yr + VE * idx, v[i]);
    }
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

// ================================================================== backward
// Partial weight gradients: block b writes 2*n floats at part + b*2*n (dscale row
// followed by dbias row).
//
// Per element the kernel spends 9 VALU operations before the row reduction and 4
// after it: with xh = (x - mean) / stdev,
//   dbias += dy;  dscale += dy * xh;  gs = dy * scale;  A += gs;  B += gs * xh
//   dx = gs / stdev + dmean / n + (dvar * 2 * stdev / n) * xh
// where dmean = -A / stdev and dvar = -B / (2 stdev^2)  (layer_norm.cpp:198-257).
//
// DEPTH > 0: the still-packed 16-byte images of the next DEPTH rows of a team are in
// flight while the current row is processed.
template <typename T, int TPR, int TEAMS, int V, bool WGRAD, int DEPTH>
__global__ void __launch_bounds__((RowBlock<TPR, TEAMS>::kThreads))
ln_bwd_rows(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ dx, int64_t ldx,
            int64_t lddy, int64_t lddx, RowMap map, int64_t rows, int nvec, int n, float eps,
            const float* __restrict__ stats, int64_t ld_stats, float* __restrict__ sgrad,
            int64_t ld_sgrad, const float* __restrict__ gamma, float* __restrict__ part)
{
  using B = RowBlock<TPR, TEAMS>;
  using IO = Vec16<T>;
  using raw_t = typename IO::raw_t;
  constexpr int VE = IO::N;
  constexpr int NW = B::kWavesPerTeam;
  constexpr int kAccLds = (WGRAD && TEAMS > 1) ? 2 * TPR * V * VE : 1;
  constexpr int NQ = DEPTH > 0 ? DEPTH : 1;
  __shared__ float red[2][TEAMS][2 * NW];
  __shared__ float acc_lds[kAccLds];
  const int tid = threadIdx.x;
  const int team = wave_index() / NW;  // wave-uniform: a team is a whole number of waves
  const int t = tid - team * TPR;
  const int lane = tid & (kWave - 1);
  const int wv = t / kWave;

  float gam[V][VE];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int idx = t + i * TPR;
#pragma unroll
    for (int k = 0; k < VE; ++k) gam[i][k] = 1.f;
    if (gamma && idx < nvec) {
#pragma unroll
      for (int k4 = 0; k4 < VE; k4 += 4) {
        float w[4];
        Vec16<float>::load(gamma + VE * idx + k4, w);
#pragma unroll
        for (int k = 0; k < 4; ++k) gam[i][k4 + k] = w[k];
      }
    }
  }
  float dg[WGRAD ? V : 1][VE], db[WGRAD ? V : 1][VE];
  if (WGRAD) {
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
      for (int k = 0; k < VE; ++k) dg[i][k] = db[i][k] = 0.f;
  }

  raw_t qx[NQ][V], qg[NQ][V];  // rows in flight, packed
  // All row arithmetic is wave-uniform (scalar registers).
  auto issue = [&](raw_t (&rx)[V], raw_t (&rg)[V], int64_t row) {
    if (row < rows) {
      int64_t col, g;
      map.split(row, col, g);
      const T* xr = x + g * map.stride + col * ldx;
      const T* gr = dy + g * map.stride + col * lddy;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const int idx = t + i * TPR;
        if (idx < nvec) {
          rx[i] = IO::load_raw(xr + VE * idx);
          rg[i] = IO::load_raw(gr + VE * idx);
        }
      }
    }
  };

  const float inv_n = 1.0f / static_cast<float>(n);
  const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * TEAMS;
  const int64_t iters = (rows + rows_per_iter - 1) / rows_per_iter;
  const int64_t first_row = static_cast<int64_t>(blockIdx.x) * TEAMS + team;
  if (DEPTH > 0) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(qx[d], qg[d], first_row + d * rows_per_iter);
  }
  for (int64_t it = 0; it < iters; ++it) {
    const int64_t row = it * rows_per_iter + first_row;
    const bool active = row < rows;
    raw_t cx[V], cg[V];
    if (DEPTH > 0) {
      // take the oldest row in flight, shift the queue, refill its tail
#pragma unroll
      for (int i = 0; i < V; ++i) {
        cx[i] = qx[0][i];
        cg[i] = qg[0][i];
      }
#pragma unroll
      for (int d = 0; d + 1 < DEPTH; ++d)
#pragma unroll
        for (int i = 0; i < V; ++i) {
          qx[d][i] = qx[d + 1][i];
          qg[d][i] = qg[d + 1][i];
        }
      issue(qx[DEPTH - 1], qg[DEPTH - 1], row + DEPTH * rows_per_iter);
    }
    else {
      issue(cx, cg, row);
    }
    float inv_stdev = 0.f, mean = 0.f;
    int64_t col = 0, g = 0;
    if (active) {
      map.split(row, col, g);
      mean = stats[g + col * ld_stats];
      inv_stdev = rsqrt_refined(stats[map.groups + g + col * ld_stats] + eps);
    }
    float xh[V][VE], gs[V][VE];
    float a = 0.f, b = 0.f;
    if (active) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (t + i * TPR < nvec) {
          float xv[VE], gv[VE];
          IO::unpack(cx[i], xv);
          IO::unpack(cg[i], gv);
#pragma unroll
          for (int k = 0; k < VE; ++k) {
            xh[i][k] = (xv[k] - mean) * inv_stdev;  // subtract first: x*inv - mean*inv would cancel
            if (WGRAD) {
              db[i][k] += gv[k];
              dg[i][k] = __builtin_fmaf(gv[k], xh[i][k], dg[i][k]);
            }
            gs[i][k] = gv[k] * gam[i][k];
            a += gs[i][k];
            b = __builtin_fmaf(gs[i][k], xh[i][k], b);
          }
        }
        else {
#pragma unroll
          for (int k = 0; k < VE; ++k) xh[i][k] = gs[i][k] = 0.f;
        }
      }
    }
    team_sum2<NW>(a, b, red[it & 1][team], wv, lane);
    if (active) {
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
        const int idx = t + i * TPR;
        if (idx < nvec) {
#pragma unroll
          for (int k = 0; k < VE; ++k)
            gs[i][k] = __builtin_fmaf(gs[i][k], inv_stdev, __builtin_fmaf(c1, xh[i][k], c0));
          IO::store(dr + VE * idx, gs[i]);
        }
      }
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
              const int p = (t + i * TPR) * VE + k;
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
        const int idx = t + i * TPR;
        if (idx < nvec) {
#pragma unroll
          for (int k4 = 0; k4 < VE; k4 += 4) {
            float w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) w[k] = dg[i][k4 + k];
            Vec16<float>::store(out + VE * idx + k4, w);
#pragma unroll
            for (int k = 0; k < 4; ++k) w[k] = db[i][k4 + k];
            Vec16<float>::store(out + n + VE * idx + k4, w);
          }
        }
      }
    }
  }
}

// Sums P partial rows: grid (ceil(n/32), 2): y == 0 dscale, y == 1 dbias.  A block
// is 32 feature columns x 8 row groups; the order of additions is fixed.
__global__ void __launch_bounds__(256)
ln_wgrad_reduce(const float* __restrict__ part, int64_t P, int64_t n, float* __restrict__ dscale,
                float* __restrict__ dbias)
{
  __shared__ float sm[8][33];
  float* out = blockIdx.y == 0 ? dscale : dbias;
  if (!out) return;
  const int kx = threadIdx.x & 31;
  const int pg = threadIdx.x >> 5;
  const int64_t k = static_cast<int64_t>(blockIdx.x) * 32 + kx;
  const float* src = part + blockIdx.y * n + k;
  float acc = 0.f;
  if (k < n) {
    int64_t p = pg;
    for (; p + 24 < P; p += 32) {
      const float a0 = src[p * 2 * n];
      const float a1 = src[(p + 8) * 2 * n];
      const float a2 = src[(p + 16) * 2 * n];
      const float a3 = src[(p + 24) * 2 * n];
      acc += (a0 + a1) + (a2 + a3);
    }
    for (; p < P; p += 8) acc += src[p * 2 * n];
  }
  sm[pg][kx] = acc;
  __syncthreads();
  if (pg == 0 && k < n) {
    float r = sm[0][kx];
#pragma unroll
    for (int i = 1; i < 8; ++i) r += sm[i][kx];
    out[k] = r;
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
  int depth;       // rows in flight per team
};

// At most this many persistent blocks: each leaves 2*n floats of partial sums, so
// fewer blocks mean less extra traffic; 256 = one per compute unit.
constexpr int64_t kLnBwdMaxBlocks = 256;

static LnBwdPlan plan_ln_bwd(int64_t nvec, int64_t rows, int ve)
{
  static const int force_depth = std::getenv("LBN_LN_BWD_DEPTH") ? std::atoi(std::getenv("LBN_LN_BWD_DEPTH")) : -1;
  static const int force_tpr = std::getenv("LBN_LN_BWD_TPR") ? std::atoi(std::getenv("LBN_LN_BWD_TPR")) : 0;
  static const int force_teams = std::getenv("LBN_LN_BWD_TEAMS") ? std::atoi(std::getenv("LBN_LN_BWD_TEAMS")) : 0;
  static const int64_t max_blocks = std::getenv("LBN_LN_BWD_BLOCKS") ? std::atoi(std::getenv("LBN_LN_BWD_BLOCKS")) : kLnBwdMaxBlocks;
  // Registers per thread: two fp32 accumulators per owned entry plus the packed rows
  // in flight.  Few vectors per thread leave room for a deeper prefetch, so the
  // widest team that still keeps every thread busy is preferred.
  LnBwdPlan p{0, 0, 0, 0, 0};
  const int tprs[4] = {64, 256, 512, 1024};
  const int teams[4] = {4, 4, 2, 1};
  const int max_v = ve == 8 ? 2 : 4;
  int pick = -1;
  for (int i = 0; i < 4; ++i) {
    if (force_tpr && tprs[i] != force_tpr) continue;
    const int64_t v = ceil_div(nvec, tprs[i]);
    if (v > max_v) continue;
    if (pick < 0) pick = i;
    // prefer one vector per thread when the wider team is still fully used
    if (v == 1 && nvec * 2 > tprs[i]) { pick = i; break; }
  }
  if (pick < 0) return p;
  p.tpr = tprs[pick];
  p.teams = teams[pick];
  p.v = round_up_pow2_le8(ceil_div(nvec, p.tpr));
  if (p.tpr == 512 && p.v > 1) p.teams = 1;  // two such teams would not fit their LDS merge buffer
  if (force_teams && force_teams <= p.teams) p.teams = force_teams;
  // spread small problems: fewer teams per block when rows are scarce
  while (p.teams > 1 && p.tpr * p.teams > 256 && ceil_div(rows, p.teams) < max_blocks) p.teams /= 2;
  p.blocks = ceil_div(rows, p.teams);
  if (p.blocks > max_blocks) p.blocks = max_blocks;
  const int64_t rows_per_team = ceil_div(rows, p.blocks * p.teams);
  p.depth = p.v == 1 ? 3 : (p.v == 2 ? 1 : 0);
  if (rows_per_team <= 1) p.depth = 0;
  if (force_depth >= 0 && force_depth <= 3) p.depth = p.v > 2 ? 0 : (p.v == 2 && force_depth > 1 ? 1 : force_depth);
  return p;
}

static size_t ln_bwd_workspace(int64_t n, int64_t rows, int ve)
{
  if (n <= 0 || rows <= 0 || n % ve != 0) return 0;
  const LnBwdPlan p = plan_ln_bwd(n / ve, rows, ve);
  if (!p.tpr) return 0;
  return static_cast<size_t>(p.blocks) * 2 * n * sizeof(float);
}

template <typename T>
static int ln_fwd(hipStream_t st, int64_t G, int64_t n, int64_t stride, int64_t w, float eps,
                  const T* x, int64_t ldx, T* y, int64_t ldy, float* stats, int64_t lds,
                  const float* gamma, const float* beta, int flags)
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
  if (vec) {
    const RowConfig c = pick_row_config(n / VE, rows, 8);
    if (c.tpr) {
      const int nvec = static_cast<int>(n / VE);
#define X(TPR, V)                                                                              \
  if (c.tpr == TPR && c.v == V) {                                                              \
    using B = RowBlock<TPR>;                                                                   \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                    \
    hipLaunchKernelGGL((ln_fwd_rows<T, TPR, V>), dim3(grid), dim3(B::kThreads), 0, st, x, y,   \
                       ldx, ldy, map, rows, nvec, static_cast<int>(n), eps, stats, lds, gamma, \
                       beta, sumsq);                                                           \
    return launch_status();                                                                    \
  }
      X(64, 1) X(64, 2) X(64, 4) X(256, 1) X(256, 2) X(256, 4) X(1024, 1) X(1024, 2) X(1024, 4)
      X(64, 8) X(256, 8)
      if constexpr (VE == 4) { X(1024, 8) }
#undef X
    }
  }
  hipLaunchKernelGGL((ln_fwd_generic<T>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, st, x, y,
                     ldx, ldy, map, n, eps, stats, lds, gamma, beta, sumsq);
  return launch_status();
}

template <typename T, int TPR, int TEAMS, int V, int DEPTH>
static void launch_ln_bwd_rows(hipStream_t st, bool wgrad, int64_t blocks, const T* x, const T* dy,
                               T* dx, int64_t ldx, int64_t lddy, int64_t lddx, RowMap map,
                               int64_t rows, int nvec, int n, float eps, const float* stats,
                               int64_t lds, float* sgrad, int64_t ldsg, const float* gamma,
                               float* part)
{
  using B = RowBlock<TPR, TEAMS>;
  const dim3 grid(static_cast<unsigned>(blocks)), block(B::kThreads);
  if (wgrad)
    hipLaunchKernelGGL((ln_bwd_rows<T, TPR, TEAMS, V, true, DEPTH>), grid, block, 0, st, x, dy, dx, ldx,
                       lddy, lddx, map, rows, nvec, n, eps, stats, lds, sgrad, ldsg, gamma, part);
  else
    hipLaunchKernelGGL((ln_bwd_rows<T, TPR, TEAMS, V, false, 0>), grid, block, 0, st, x, dy, dx, ldx,
                       lddy, lddx, map, rows, nvec, n, eps, stats, lds, sgrad, ldsg, gamma, part);
}

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
    LnBwdPlan p = plan_ln_bwd(n / VE, rows, VE);
    if (p.tpr) {
      float* part = nullptr;
      if (wgrad) {
        const size_t need = static_cast<size_t>(p.blocks) * 2 * n * sizeof(float);
        if (!ws || ws_bytes < need || !aligned16(ws)) return LBN_ERR_WORKSPACE;
        part = static_cast<float*>(ws);
      }
      else {
        p.blocks = ceil_div(rows, p.teams);  // nothing to accumulate: one pass, all rows at once
      }
      const int nvec = static_cast<int>(n / VE);
      bool launched = false;
#define X(TPR, TEAMS, V, D)                                                                     \
  if (!launched && p.tpr == TPR && p.teams == TEAMS && p.v == V && p.depth == D) {              \
    launch_ln_bwd_rows<T, TPR, TEAMS, V, D>(st, wgrad, p.blocks, x, dy, dx, ldx, lddy, lddx,    \
                                            map, rows, nvec, static_cast<int>(n), eps, stats,   \
                                            lds, sgrad, ldsg, gamma, part);                     \
    launched = true;                                                                            \
  }
#define XD(TPR, TEAMS, V) X(TPR, TEAMS, V, 0) X(TPR, TEAMS, V, 1) X(TPR, TEAMS, V, 2) X(TPR, TEAMS, V, 3)
#define XS(TPR, TEAMS, V) X(TPR, TEAMS, V, 0) X(TPR, TEAMS, V, 1)
      XD(64, 4, 1) XS(64, 4, 2) XD(256, 1, 1) XS(256, 1, 2) XD(256, 2, 1) XS(256, 2, 2) XD(256, 4, 1)
      XS(256, 4, 2) XD(512, 1, 1) XS(512, 1, 2) XD(512, 2, 1) XD(1024, 1, 1) XS(1024, 1, 2)
      if constexpr (VE == 4) { X(64, 4, 4, 0) X(256, 1, 4, 0) X(256, 2, 4, 0) X(256, 4, 4, 0) X(512, 1, 4, 0) X(1024, 1, 4, 0) }
#undef XS
#undef XD
#undef X
      if (launched) {
        if (wgrad) {
          const dim3 grid(static_cast<unsigned>(ceil_div(n, 32)), 2);
          hipLaunchKernelGGL(ln_wgrad_reduce, grid, dim3(256), 0, st, part, p.blocks, n, dgamma, dbeta);
        }
        return launch_status();
      }
    }
  }
  hipLaunchKernelGGL((ln_bwd_generic<T>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, st, x, dy,
                     dx, ldx, lddy, lddx, map, n, eps, stats, lds, sgrad, ldsg, gamma);
  if (wgrad)
    hipLaunchKernelGGL((ln_wgrad_generic<T>), dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256),
                       0, st, x, dy, ldx, lddy, map, rows, n, eps, stats, lds, dgamma, dbeta);
  return launch_status();
}

}  // namespace lbn

using namespace lbn;

extern "C" {

int lbn_layer_norm_fwd_f32(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon, const float* x,
                           int64_t ldx, float* y, int64_t ldy, float* stats, int64_t ld_stats,
                           const float* scale, const float* bias, int flags)
{
  return ln_fwd<float>(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon, x, ldx,
                       y, ldy, stats, ld_stats, scale, bias, flags);
}

int lbn_layer_norm_fwd_f16(lbn_stream_t stream, int64_t num_groups, int64_t norm_size,
                           int64_t norm_stride, int64_t width, float epsilon, const void* x,
                           int64_t ldx, void* y, int64_t ldy, float* stats, int64_t ld_stats,
                           const float* scale, const float* bias, int flags)
{
  return ln_fwd<__half>(as_stream(stream), num_groups, norm_size, norm_stride, width, epsilon,
                        static_cast<const __half*>(x), ldx, static_cast<__half*>(y), ldy, stats,
                        ld_stats, scale, bias, flags);
}

size_t lbn_layer_norm_bwd_workspace_bytes(int64_t num_groups, int64_t norm_size, int64_t width,
                                          int has_weight_grads, int elem_bytes)
{
  if (!has_weight_grads || num_groups <= 0 || width <= 0) return 0;
  return ln_bwd_workspace(norm_size, num_groups * width, elem_bytes == 2 ? 8 : 4);
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

}  // extern "C"
