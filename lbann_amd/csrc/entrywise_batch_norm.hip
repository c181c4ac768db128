// Entry-wise batch normalization (entrywise_batch_normalization_layer): every entry of
// the sample tensor (a matrix row) is normalised with its own statistics over the
// mini-batch (the matrix columns), Bessel-corrected variance, no scale or bias.
// Reference CPU code: src/layers/regularizers/entrywise_batch_normalization.cpp:52-202
// (forward), :210-414 (backward).
//
// The reduction runs along the strided direction of the column-major matrix, so the
// roles of lanes and loops are swapped against layer norm: consecutive lanes take
// consecutive rows (16 bytes = 4 rows per lane, so a wave instruction reads whole
// cache lines of one column) and every thread owns a subset of the columns.
//
//  * ebn_*_tile<CPT,GW>: a 256-thread block owns 256/GW rows x all columns; a wave is
//    64/GW row quads x GW column groups (GW = 1 or 4), so the block has 4*GW column
//    groups and w <= 4*GW*CPT.  Thread (row quad q, column group g) keeps columns g,
//    g + 4*GW, ... of rows 4q..4q+3 in registers; the groups of a wave merge their
//    partial sums by lane exchange, the four waves through LDS (one barrier, fixed
//    order), and the block finishes from registers: x (and dy) are read once, y (dx)
//    written once.  Narrow mini-batches use GW = 1: a wave instruction then reads 1 KiB
//    of one column.  Sums are taken about the row's first column, which removes the
//    cancellation of E[x^2] - mean^2.
//  * ebn_*_generic: one thread per row, scalar but coalesced accesses, two passes
//    over the row: any shape and alignment, inference mode, and mini-batches wider
//    than 256 columns.
#include <cfloat>

#include "device_utils.hpp"
#include "entrywise_batch_norm_slabs.hpp"
#include "host_utils.hpp"
#include "reference_order.hpp"

namespace lbn {

constexpr int kEbnThreads = 256;
constexpr int kEbnWaves = kEbnThreads / kWave;

struct EbnArgs {
  int64_t h, w;
  float eps, decay;
  const float* x;
  const float* dy;
  float* out;  // y or dx
  int64_t ldx, lddy, ldo;
  float* stats;  // (h x 2): mean, variance
  int64_t ld_stats;
  float* sgrad;  // (h x 2): dL/dmean, dL/dvar
  int64_t ld_sgrad;
  float* rmean;
  float* rvar;
};

// mean and variance of a row from its sums about the pivot K: s = sum(x - K),
// q = sum((x - K)^2)  (entrywise_batch_normalization.cpp:109-124; one sample: variance 1).
__device__ __forceinline__ void ebn_stats_from_sums(float s, float q, float K, int64_t w, float& mean,
                                                    float& var)
{
  const float wf = static_cast<float>(w);
  const float dm = s / wf;
  mean = K + dm;
  var = w > 1 ? fmaxf(q - s * dm, 0.f) / (wf - 1.f) : 1.f;
}

// Position of a thread in its block's tile.
template <int GW>
struct EbnPos {
  static constexpr int kQuads = kWave / GW;            // row quads of a wave (and of the block)
  static constexpr int kRows = 4 * kQuads;             // rows of a block
  static constexpr int kGroups = kEbnWaves * GW;       // column groups of a block
  int q, g;
  bool writer;  // first column group of its wave: holds the wave's sums after the lane exchange
  __device__ __forceinline__ EbnPos()
  {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    q = lane & (kQuads - 1);
    g = lane / kQuads + GW * wave;
    writer = lane < kQuads;
  }
};

// Partial pairs of the block's column groups for each of its rows, merged in a fixed
// order: across the GW groups of a wave by lane exchange, across the waves through
// LDS.  Every thread gets the totals of its own 4 rows.
template <int GW>
__device__ __forceinline__ void ebn_merge(float (&a)[4], float (&b)[4],
                                          float (*lds)[EbnPos<GW>::kRows][2], const EbnPos<GW>& p)
{
  if (GW == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      a[r] += __shfl_xor(a[r], 16);
      b[r] += __shfl_xor(b[r], 16);
      a[r] += __shfl_xor(a[r], 32);
      b[r] += __shfl_xor(b[r], 32);
    }
  }
  const int wave = threadIdx.x / kWave;
  if (p.writer) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      lds[wave][4 * p.q + r][0] = a[r];
      lds[wave][4 * p.q + r][1] = b[r];
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int k = 0; k < kEbnWaves; ++k) {
      sa += lds[k][4 * p.q + r][0];
      sb += lds[k][4 * p.q + r][1];
    }
    a[r] = sa;
    b[r] = sb;
  }
}

// ST: inputs through streaming loads (calls that move more than the last-level cache holds).
template <int CPT, int GW, bool ST>
__global__ void __launch_bounds__(kEbnThreads)
ebn_fwd_tile(EbnArgs a)
{
  using P = EbnPos<GW>;
  __shared__ float lds[kEbnWaves][P::kRows][2];
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  const bool row_ok = r0 < a.h;  // h is a multiple of 4: a quad is inside or outside
  const int64_t rr = row_ok ? r0 : 0;

  float v[CPT][4];
  float K[4];
  Vec16<float>::load(a.x + rr, K);  // the rows' first column: the pivot of the sums
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (c < a.w) {
      if constexpr (ST) Vec16<float>::load_stream(a.x + rr + c * a.ldx, v[j]);
      else Vec16<float>::load(a.x + rr + c * a.ldx, v[j]);
    }
    else {
#pragma unroll
      for (int r = 0; r < 4; ++r) v[j][r] = K[r];
    }
  }
  float s[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < CPT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float d = v[j][r] - K[r];
      s[r] += d;
      sq[r] = __builtin_fmaf(d, d, sq[r]);
    }
  ebn_merge<GW>(s, sq, lds, p);
  if (!row_ok) return;
  float mean[4], var[4], inv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    ebn_stats_from_sums(s[r], sq[r], K[r], a.w, mean[r], var[r]);
    inv[r] = 1.0f / sqrtf(var[r] + a.eps);
  }
  if (p.g == 0) {
    Vec16<float>::store(a.stats + r0, mean);
    Vec16<float>::store(a.stats + r0 + a.ld_stats, var);
    if (a.w > 1) {  // entrywise_batch_normalization.cpp:121-122
      float rm[4], rv[4];
      Vec16<float>::load(a.rmean + r0, rm);
      Vec16<float>::load(a.rvar + r0, rv);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        rm[r] = a.decay * rm[r] + (1.f - a.decay) * mean[r];
        rv[r] = a.decay * rv[r] + (1.f - a.decay) * var[r];
      }
      Vec16<float>::store(a.rmean + r0, rm);
      Vec16<float>::store(a.rvar + r0, rv);
    }
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (c < a.w) {
#pragma unroll
      for (int r = 0; r < 4; ++r) v[j][r] = (v[j][r] - mean[r]) * inv[r];
      Vec16<float>::store(a.out + r0 + c * a.ldo, v[j]);
    }
  }
}

template <int CPT, int GW, bool ST>
__global__ void __launch_bounds__(kEbnThreads)
ebn_bwd_tile(EbnArgs a)
{
  using P = EbnPos<GW>;
  __shared__ float lds[kEbnWaves][P::kRows][2];
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  const bool row_ok = r0 < a.h;
  const int64_t rr = row_ok ? r0 : 0;

  float xc[CPT][4], gv[CPT][4];
  float mean[4], var[4], inv[4];
  Vec16<float>::load(a.stats + rr, mean);
  Vec16<float>::load(a.stats + rr + a.ld_stats, var);
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (c < a.w) {
      if constexpr (ST) {
        Vec16<float>::load_stream(a.x + rr + c * a.ldx, xc[j]);
        Vec16<float>::load_stream(a.dy + rr + c * a.lddy, gv[j]);
      }
      else {
        Vec16<float>::load(a.x + rr + c * a.ldx, xc[j]);
        Vec16<float>::load(a.dy + rr + c * a.lddy, gv[j]);
      }
    }
    else {
#pragma unroll
      for (int r = 0; r < 4; ++r) xc[j][r] = gv[j][r] = 0.f;
    }
  }
  float sa[4] = {0.f, 0.f, 0.f, 0.f}, sb[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int r = 0; r < 4; ++r) inv[r] = 1.0f / sqrtf(var[r] + a.eps);
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const bool ok = p.g + P::kGroups * j < a.w;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      xc[j][r] = ok ? xc[j][r] - mean[r] : 0.f;
      sa[r] += gv[j][r];
      sb[r] = __builtin_fmaf(gv[j][r], xc[j][r], sb[r]);
    }
  }
  ebn_merge<GW>(sa, sb, lds, p);
  if (!row_ok) return;
  // dL/dmean = -sum(dy) / stdev, dL/dvar = -sum(dy (x - mean)) / (2 stdev^3)
  // (entrywise_batch_normalization.cpp:264-296)
  const float wf = static_cast<float>(a.w);
  float dmean[4], dvar[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    dmean[r] = -sa[r] * inv[r];
    dvar[r] = -sb[r] * inv[r] * inv[r] * inv[r] * 0.5f;
  }
  if (p.g == 0) {
    Vec16<float>::store(a.sgrad + r0, dmean);
    Vec16<float>::store(a.sgrad + r0 + a.ld_sgrad, dvar);
  }
  float c0[4], c1[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    c0[r] = dmean[r] / wf;
    c1[r] = dvar[r] * 2.f / (wf - 1.f);
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int64_t c = p.g + P::kGroups * j;
    if (c < a.w) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        gv[j][r] = __builtin_fmaf(gv[j][r], inv[r], __builtin_fmaf(c1[r], xc[j][r], c0[r]));
      Vec16<float>::store(a.out + r0 + c * a.ldo, gv[j]);
    }
  }
}

// Mini-batches wider than the tile kernels hold in registers: the same tiling, two passes
// over the workgroup's rows x all columns (sums, then the output); the second pass re-reads
// what the first streamed.
template <int GW>
__global__ void __launch_bounds__(kEbnThreads)
ebn_fwd_wide(EbnArgs a)
{
  using P = EbnPos<GW>;
  __shared__ float lds[kEbnWaves][P::kRows][2];
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  const bool row_ok = r0 < a.h;
  const int64_t rr = row_ok ? r0 : 0;
  const int64_t w = row_ok ? a.w : 0;
  float K[4];
  Vec16<float>::load(a.x + rr, K);
  float s[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f};
  int64_t c = p.g;
  for (; c + P::kGroups < w; c += 2 * P::kGroups) {
    float v[2][4];
#pragma unroll
    for (int j = 0; j < 2; ++j) Vec16<float>::load(a.x + rr + (c + j * P::kGroups) * a.ldx, v[j]);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float d = v[j][r] - K[r];
        s[r] += d;
        sq[r] = __builtin_fmaf(d, d, sq[r]);
      }
  }
  for (; c < w; c += P::kGroups) {
    float v[4];
    Vec16<float>::load(a.x + rr + c * a.ldx, v);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float d = v[r] - K[r];
      s[r] += d;
      sq[r] = __builtin_fmaf(d, d, sq[r]);
    }
  }
  ebn_merge<GW>(s, sq, lds, p);
  if (!row_ok) return;
  float mean[4], var[4], inv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    ebn_stats_from_sums(s[r], sq[r], K[r], a.w, mean[r], var[r]);
    inv[r] = 1.0f / sqrtf(var[r] + a.eps);
  }
  if (p.g == 0) {
    Vec16<float>::store(a.stats + r0, mean);
    Vec16<float>::store(a.stats + r0 + a.ld_stats, var);
    float rm[4], rv[4];  // w > 1 here: entrywise_batch_normalization.cpp:121-122
    Vec16<float>::load(a.rmean + r0, rm);
    Vec16<float>::load(a.rvar + r0, rv);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      rm[r] = a.decay * rm[r] + (1.f - a.decay) * mean[r];
      rv[r] = a.decay * rv[r] + (1.f - a.decay) * var[r];
    }
    Vec16<float>::store(a.rmean + r0, rm);
    Vec16<float>::store(a.rvar + r0, rv);
  }
  for (c = p.g; c < w; c += P::kGroups) {
    float v[4];
    Vec16<float>::load(a.x + r0 + c * a.ldx, v);
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = (v[r] - mean[r]) * inv[r];
    Vec16<float>::store(a.out + r0 + c * a.ldo, v);
  }
}

template <int GW>
__global__ void __launch_bounds__(kEbnThreads)
ebn_bwd_wide(EbnArgs a)
{
  using P = EbnPos<GW>;
  __shared__ float lds[kEbnWaves][P::kRows][2];
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  const bool row_ok = r0 < a.h;
  const int64_t rr = row_ok ? r0 : 0;
  const int64_t w = row_ok ? a.w : 0;
  float mean[4], var[4], inv[4];
  Vec16<float>::load(a.stats + rr, mean);
  Vec16<float>::load(a.stats + rr + a.ld_stats, var);
#pragma unroll
  for (int r = 0; r < 4; ++r) inv[r] = 1.0f / sqrtf(var[r] + a.eps);
  float sa[4] = {0.f, 0.f, 0.f, 0.f}, sb[4] = {0.f, 0.f, 0.f, 0.f};
  for (int64_t c = p.g; c < w; c += P::kGroups) {
    float v[4], g[4];
    Vec16<float>::load(a.x + rr + c * a.ldx, v);
    Vec16<float>::load(a.dy + rr + c * a.lddy, g);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      sa[r] += g[r];
      sb[r] = __builtin_fmaf(g[r], v[r] - mean[r], sb[r]);
    }
  }
  ebn_merge<GW>(sa, sb, lds, p);
  if (!row_ok) return;
  const float wf = static_cast<float>(a.w);
  float dmean[4], dvar[4], c0[4], c1[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    dmean[r] = -sa[r] * inv[r];
    dvar[r] = -sb[r] * inv[r] * inv[r] * inv[r] * 0.5f;
    c0[r] = dmean[r] / wf;
    c1[r] = dvar[r] * 2.f / (wf - 1.f);
  }
  if (p.g == 0) {
    Vec16<float>::store(a.sgrad + r0, dmean);
    Vec16<float>::store(a.sgrad + r0 + a.ld_sgrad, dvar);
  }
  for (int64_t c = p.g; c < w; c += P::kGroups) {
    float v[4], g[4];
    Vec16<float>::load(a.x + r0 + c * a.ldx, v);
    Vec16<float>::load(a.dy + r0 + c * a.lddy, g);
#pragma unroll
    for (int r = 0; r < 4; ++r)
      g[r] = __builtin_fmaf(g[r], inv[r], __builtin_fmaf(c1[r], v[r] - mean[r], c0[r]));
    Vec16<float>::store(a.out + r0 + c * a.ldo, g);
  }
}

// Walks the w columns of a row eight at a time: f(c, u) first loads column c + u for all u in
// flight, g(c, u) then consumes them in order.  A thread of the kernels below owns one row and
// would otherwise wait for one 4-byte load per iteration.
template <typename Load, typename Use>
__device__ __forceinline__ void ebn_walk_columns(int64_t w, Load&& load, Use&& use)
{
  constexpr int U = 8;
  int64_t c = 0;
  for (; c + U <= w; c += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) load(c + u, u);
#pragma unroll
    for (int u = 0; u < U; ++u) use(c + u, u);
  }
  for (; c < w; ++c) {
    load(c, 0);
    use(c, 0);
  }
}

// One thread per row, training mode: statistics from the mini-batch (written to stats, running
// statistics updated).  (Outside training both directions are element-wise with per-row
// coefficients and run on a two-dimensional grid, entrywise_batch_norm_slabs.hpp.)
__global__ void __launch_bounds__(256)
ebn_fwd_generic(EbnArgs a)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= a.h) return;
  const float* xr = a.x + r;
  float mean, var;
  {
    const float K = xr[0];
    float s = 0.f, q = 0.f;
    float v[8];
    ebn_walk_columns(
      a.w, [&](int64_t c, int u) { v[u] = xr[c * a.ldx]; },
      [&](int64_t, int u) {
        const float d = v[u] - K;
        s += d;
        q = __builtin_fmaf(d, d, q);
      });
    ebn_stats_from_sums(s, q, K, a.w, mean, var);
    a.stats[r] = mean;
    a.stats[r + a.ld_stats] = var;
    if (a.w > 1) {
      a.rmean[r] = a.decay * a.rmean[r] + (1.f - a.decay) * mean;
      a.rvar[r] = a.decay * a.rvar[r] + (1.f - a.decay) * var;
    }
  }
  const float inv = 1.0f / sqrtf(var + a.eps);
  float* yr = a.out + r;
  float v[8];
  ebn_walk_columns(
    a.w, [&](int64_t c, int u) { v[u] = xr[c * a.ldx]; },
    [&](int64_t c, int u) { yr[c * a.ldo] = (v[u] - mean) * inv; });
}

__global__ void __launch_bounds__(256)
ebn_bwd_generic(EbnArgs a)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= a.h) return;
  const float* gr = a.dy + r;
  float* dr = a.out + r;
  const float* xr = a.x + r;
  const float mean = a.stats[r];
  const float inv = 1.0f / sqrtf(a.stats[r + a.ld_stats] + a.eps);
  float sa = 0.f, sb = 0.f;
  float g[8], v[8];
  ebn_walk_columns(
    a.w,
    [&](int64_t c, int u) {
      g[u] = gr[c * a.lddy];
      v[u] = xr[c * a.ldx];
    },
    [&](int64_t, int u) {
      sa += g[u];
      sb = __builtin_fmaf(g[u], v[u] - mean, sb);
    });
  const float wf = static_cast<float>(a.w);
  const float dmean = -sa * inv;
  const float dvar = -sb * inv * inv * inv * 0.5f;
  a.sgrad[r] = dmean;
  a.sgrad[r + a.ld_sgrad] = dvar;
  const float c0 = dmean / wf;
  const float c1 = dvar * 2.f / (wf - 1.f);
  // in place (dx aliasing dy or x): a thread writes a column's entry after reading it
  ebn_walk_columns(
    a.w,
    [&](int64_t c, int u) {
      g[u] = gr[c * a.lddy];
      v[u] = xr[c * a.ldx];
    },
    [&](int64_t c, int u) { dr[c * a.ldo] = __builtin_fmaf(g[u], inv, __builtin_fmaf(c1, v[u] - mean, c0)); });
}

__global__ void __launch_bounds__(256)
ebn_fill_zero(float* p, int64_t h, int64_t w, int64_t ld)
{
  const int64_t total = h * w;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t c = i / h;
    p[(i - c * h) + c * ld] = 0.f;
  }
}

// (columns per thread, column groups per wave) by mini-batch width: up to 64 columns
// a wave reads one column at a time, wider mini-batches put four columns in a wave.
constexpr int64_t kEbnMaxTileWidth = 256;
#define LBN_EBN_TILE_CASES(X) X(1, 1) X(2, 1) X(4, 1) X(8, 1) X(16, 1) X(8, 4) X(16, 4)

// 16-byte accesses need every column start aligned.
static bool ebn_vec_ok(int64_t h, int64_t w, const void* p, int64_t ld)
{
  return h % 4 == 0 && aligned16(p) && (w <= 1 || ld % 4 == 0);
}

static int ebn_check(int64_t h, int64_t w, const int64_t* lds, int nld)
{
  if (h < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < h) return LBN_ERR_INVALID_ARGUMENT;
  if (h > (int64_t(1) << 36)) return LBN_ERR_UNSUPPORTED;  // 64 rows per workgroup, gridDim.x < 2^31
  return LBN_OK;
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_entrywise_batch_norm_workspace_bytes(int64_t height, int64_t width)
{
  if (height <= 0 || width <= 0) return 0;
  return ebn_slab_workspace_bytes(height, width);
}

int lbn_entrywise_batch_norm_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, float decay,
                                     float epsilon, int training, const float* x, int64_t ldx,
                                     float* y, int64_t ldy, float* stats, int64_t ld_stats,
                                     float* running_mean, float* running_var, void* workspace,
                                     size_t workspace_bytes)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = ebn_check(height, width, lds, 2)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!x || !y || !running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
  if (training && (!stats || ld_stats < height)) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  const EbnArgs a{height, width, epsilon, decay, x, nullptr, y, ldx, 0, ldy, stats, ld_stats,
                  nullptr, 0, running_mean, running_var};
  const bool vec = ebn_vec_ok(height, width, x, ldx) && ebn_vec_ok(height, width, y, ldy) &&
                   aligned16(stats) && ld_stats % 4 == 0 && aligned16(running_mean) &&
                   aligned16(running_var);
  if (training && vec && width <= kEbnMaxTileWidth) {
    const bool stream = stream_call_inputs(2 * height * width * 4);
#define X(C, G)                                                                                  \
  if (width <= 4 * G * C) {                                                                      \
    const dim3 grid(static_cast<unsigned>(ceil_div(height, EbnPos<G>::kRows)));                  \
    if (stream) hipLaunchKernelGGL((ebn_fwd_tile<C, G, true>), grid, dim3(kEbnThreads), 0, st, a); \
    else hipLaunchKernelGGL((ebn_fwd_tile<C, G, false>), grid, dim3(kEbnThreads), 0, st, a);     \
    return launch_status();                                                                      \
  }
    LBN_EBN_TILE_CASES(X)
#undef X
  }
  if (training && vec) {  // wider than the register tiles
    // few rows: column slabs side by side when the caller gave scratch
    if (ebn_slab_fwd(st, height, width, epsilon, decay, x, ldx, y, ldy, stats, ld_stats, running_mean, running_var,
                     workspace, workspace_bytes))
      return launch_status();
    hipLaunchKernelGGL((ebn_fwd_wide<4>), dim3(static_cast<unsigned>(ceil_div(height, EbnPos<4>::kRows))),
                       dim3(kEbnThreads), 0, st, a);
    return launch_status();
  }
  const dim3 grid(static_cast<unsigned>(ceil_div(height, 256))), block(256);
  if (training) hipLaunchKernelGGL(ebn_fwd_generic, grid, block, 0, st, a);
  else ebn_inference_fwd(st, height, width, epsilon, x, ldx, y, ldy, running_mean, running_var);
  return launch_status();
}

int lbn_entrywise_batch_norm_fwd_reference_order_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                                     float decay, float epsilon, const float* x, int64_t ldx,
                                                     float* y, int64_t ldy, float* stats, int64_t ld_stats,
                                                     float* running_mean, float* running_var)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = ebn_check(height, width, lds, 2)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!x || !y || !running_mean || !running_var || !stats || ld_stats < height) return LBN_ERR_INVALID_ARGUMENT;
  if (height > kRefOrderMaxEntries / width) return LBN_ERR_UNSUPPORTED;
  hipStream_t st = as_stream(stream);
  hipLaunchKernelGGL(ebn_ref_order_fwd, dim3(static_cast<unsigned>(ceil_div(height, 256))), dim3(256), 0, st, height,
                     width, decay, epsilon, x, ldx, y, ldy, stats, ld_stats, running_mean, running_var);
  return launch_status();
}

int lbn_entrywise_batch_norm_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, float epsilon,
                                     int training, const float* x, int64_t ldx, const float* dy,
                                     int64_t lddy, float* dx, int64_t lddx, const float* stats,
                                     int64_t ld_stats, float* stats_grad, int64_t ld_stats_grad,
                                     const float* running_var, void* workspace, size_t workspace_bytes)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = ebn_check(height, width, lds, 3)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!dy || !dx) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  const EbnArgs a{height, width, epsilon, 0.f, x, dy, dx, ldx, lddy, lddx, const_cast<float*>(stats),
                  ld_stats, stats_grad, ld_stats_grad, nullptr, const_cast<float*>(running_var)};
  if (!training) {
    if (!running_var) return LBN_ERR_INVALID_ARGUMENT;
    ebn_inference_bwd(st, height, width, epsilon, dy, lddy, dx, lddx, running_var);
    return launch_status();
  }
  if (!x || !stats || !stats_grad || ld_stats < height || ld_stats_grad < height)
    return LBN_ERR_INVALID_ARGUMENT;
  if (width <= 1) {  // the output is constant: zero gradient (entrywise_batch_normalization.cpp:257-261)
    hipLaunchKernelGGL(ebn_fill_zero, dim3(static_cast<unsigned>(ceil_div(height * width, 256))),
                       dim3(256), 0, st, dx, height, width, lddx);
    return launch_status();
  }
  const bool vec = ebn_vec_ok(height, width, x, ldx) && ebn_vec_ok(height, width, dy, lddy) &&
                   ebn_vec_ok(height, width, dx, lddx) && aligned16(stats) && ld_stats % 4 == 0 &&
                   aligned16(stats_grad) && ld_stats_grad % 4 == 0;
  if (vec && width <= kEbnMaxTileWidth) {
    const bool stream = stream_call_inputs(3 * height * width * 4);
#define X(C, G)                                                                                  \
  if (width <= 4 * G * C) {                                                                      \
    const dim3 grid(static_cast<unsigned>(ceil_div(height, EbnPos<G>::kRows)));                  \
    if (stream) hipLaunchKernelGGL((ebn_bwd_tile<C, G, true>), grid, dim3(kEbnThreads), 0, st, a); \
    else hipLaunchKernelGGL((ebn_bwd_tile<C, G, false>), grid, dim3(kEbnThreads), 0, st, a);     \
    return launch_status();                                                                      \
  }
    LBN_EBN_TILE_CASES(X)
#undef X
  }
  if (vec) {  // wider than the register tiles
    if (ebn_slab_bwd(st, height, width, epsilon, x, ldx, dy, lddy, dx, lddx, stats, ld_stats, stats_grad,
                     ld_stats_grad, workspace, workspace_bytes))
      return launch_status();
    hipLaunchKernelGGL((ebn_bwd_wide<4>), dim3(static_cast<unsigned>(ceil_div(height, EbnPos<4>::kRows))),
                       dim3(kEbnThreads), 0, st, a);
    return launch_status();
  }
  hipLaunchKernelGGL(ebn_bwd_generic, dim3(static_cast<unsigned>(ceil_div(height, 256))),
                     dim3(256), 0, st, a);
  return launch_status();
}

}  // extern "C"
