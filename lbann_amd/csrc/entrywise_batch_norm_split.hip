// Entry-wise batch normalization cut where the reference places its all-reduces
// (src/layers/regularizers/entrywise_batch_normalization.cpp):
//   forward   local sums (:78-95) -> [all-reduce :97-100] -> statistics (:101-125) -> apply (:131-160)
//   backward  local dL/dmean, dL/dvar (:275-299) -> [all-reduce :301-303] -> dx (:305-335)
// for callers whose mini-batch is spread over several ranks: `width` is the local number of
// columns, `statistics_count` the global one (input.Width() in the reference).  The exchange
// format is the reference's: per row sum(x) and sum(x^2), resp. the two gradient sums.
//
// Tiling (all kernels): consecutive lanes take consecutive row items (4 rows = 16 bytes when
// every column start is 16-byte aligned, else single rows), the four waves of a workgroup
// take every fourth column, so a wave instruction reads 1 KiB (256 B) of one column.  The
// summing kernels merge the four waves' partial sums through LDS in a fixed order.
#include "device_utils.hpp"
#include "entrywise_batch_norm_slabs.hpp"
#include "host_utils.hpp"

namespace lbn {

constexpr int kSplitThreads = 256;
constexpr int kSplitWaves = kSplitThreads / kWave;   // column groups of a workgroup
constexpr int kSplitApplyCols = 32;                  // columns per workgroup of the apply kernels

template <int VE>
struct RowItem;
template <>
struct RowItem<4> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) { Vec16<float>::load(p, v); }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { Vec16<float>::store(p, v); }
};
template <>
struct RowItem<1> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[1]) { v[0] = *p; }
  static __device__ __forceinline__ void store(float* p, const float (&v)[1]) { *p = v[0]; }
};

struct SplitArgs {
  int64_t h, w;
  float eps;
  float count;      // statistics_count as a float
  const float* x;
  const float* dy;
  float* out;       // y or dx
  int64_t ldx, lddy, ldo;
  const float* mean;
  const float* var;
  float* sum0;      // column 0 of the (h x 2) result of a summing kernel
  float* sum1;      // column 1
  // Column slabs (gridDim.y of the summing kernels): slab s sums columns [s * slab_cols,
  // (s + 1) * slab_cols) into sum0 / sum1 + s * slab_stride.  One slab: all columns, no offset.
  int64_t slab_cols;
  int64_t slab_stride;
};

// Column range and output offset of a summing workgroup.
struct SplitSlab {
  int64_t c0, c1, out;
};
__device__ __forceinline__ SplitSlab split_slab(const SplitArgs& a, bool ok)
{
  if (gridDim.y == 1) return {0, ok ? a.w : 0, 0};
  const int64_t c0 = static_cast<int64_t>(blockIdx.y) * a.slab_cols;
  const int64_t c1 = c0 + a.slab_cols < a.w ? c0 + a.slab_cols : a.w;
  return {c0, ok ? c1 : c0, static_cast<int64_t>(blockIdx.y) * a.slab_stride};
}

__device__ __forceinline__ float square_rounded(float v)
{
#pragma clang fp contract(off)
  const float sq = v * v;
  return sq;
}

// The four waves' partial pairs of every row item, added in wave order by wave 0.
template <int VE>
__device__ __forceinline__ bool split_merge(float (&a)[VE], float (&b)[VE], float (*lds)[kWave * VE][2])
{
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
#pragma unroll
  for (int r = 0; r < VE; ++r) {
    lds[wave][lane * VE + r][0] = a[r];
    lds[wave][lane * VE + r][1] = b[r];
  }
  __syncthreads();
  if (wave != 0) return false;
#pragma unroll
  for (int r = 0; r < VE; ++r) {
    float sa = lds[0][lane * VE + r][0], sb = lds[0][lane * VE + r][1];
#pragma unroll
    for (int k = 1; k < kSplitWaves; ++k) {
      sa += lds[k][lane * VE + r][0];
      sb += lds[k][lane * VE + r][1];
    }
    a[r] = sa;
    b[r] = sb;
  }
  return true;
}

// sum0 = sum over the local columns of x, sum1 = of x^2 (entrywise_batch_normalization.cpp:78-95).
// Squares are rounded before they are added, as in the reference's loop: the variance
// formula that follows cancels, so a mini-batch of a few samples shows every rounding.
template <int VE>
__global__ void __launch_bounds__(kSplitThreads)
ebn_split_fwd_sums(SplitArgs a)
{
  __shared__ float lds[kSplitWaves][kWave * VE][2];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r0 = (static_cast<int64_t>(blockIdx.x) * kWave + lane) * VE;
  const bool ok = r0 < a.h;
  const int64_t rr = ok ? r0 : 0;
  const SplitSlab sl = split_slab(a, ok);
  const int64_t w = sl.c1;
  float s[VE], q[VE];
#pragma unroll
  for (int r = 0; r < VE; ++r) s[r] = q[r] = 0.f;
  int64_t c = sl.c0 + wave;
  for (; c + kSplitWaves < w; c += 2 * kSplitWaves) {
    float v[2][VE];
    RowItem<VE>::load(a.x + rr + c * a.ldx, v[0]);
    RowItem<VE>::load(a.x + rr + (c + kSplitWaves) * a.ldx, v[1]);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < VE; ++r) {
        s[r] += v[j][r];
        q[r] += square_rounded(v[j][r]);
      }
  }
  for (; c < w; c += kSplitWaves) {
    float v[VE];
    RowItem<VE>::load(a.x + rr + c * a.ldx, v);
#pragma unroll
    for (int r = 0; r < VE; ++r) {
      s[r] += v[r];
      q[r] += square_rounded(v[r]);
    }
  }
  if (split_merge<VE>(s, q, lds) && ok) {
    RowItem<VE>::store(a.sum0 + sl.out + r0, s);
    RowItem<VE>::store(a.sum1 + sl.out + r0, q);
  }
}

// Sums over `count` samples -> mean and Bessel-corrected variance in place, running
// statistics updated (entrywise_batch_normalization.cpp:101-125).  One sample: the sum is
// the mean already, the variance is 1 and the running statistics stay.  The variance is
// clamped at zero where E[x^2] - mean^2 comes out negative.  Every operation is rounded on
// its own, in the reference's order.
// Row r: (sum, sum of squares) -> mean[r], var[r], running statistics updated.
__device__ __forceinline__ void ebn_stats_of_row(int64_t r, float sum, float sumsq, int64_t count, float decay,
                                                 float* mean, float* var, float* rmean, float* rvar)
{
  if (count <= 1) {
    mean[r] = sum;
    var[r] = 1.f;
    return;
  }
  {
#pragma clang fp contract(off)
    const float n = static_cast<float>(count);
    const float m = sum / n;
    const float sqmean = sumsq / n;
    const float mm = m * m;
    const float v = fmaxf(sqmean - mm, 0.f) * n / (n - 1.f);
    const float keep_m = decay * rmean[r];
    const float keep_v = decay * rvar[r];
    const float new_m = (1.f - decay) * m;
    const float new_v = (1.f - decay) * v;
    mean[r] = m;
    var[r] = v;
    rmean[r] = keep_m + new_m;
    rvar[r] = keep_v + new_v;
  }
}

__global__ void __launch_bounds__(256)
ebn_split_fwd_stats(int64_t h, int64_t count, float decay, float* mean, float* var, float* rmean,
                    float* rvar)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= h) return;
  ebn_stats_of_row(r, mean[r], var[r], count, decay, mean, var, rmean, rvar);
}

// Adds the S slabs' partial pairs of every row: a workgroup takes 64 rows, its four waves every
// fourth slab with eight loads in flight, and wave 0 adds the four waves' sums in order.  (One
// thread per row walking 64 slabs by itself took 31 us for 4096 rows.)  STATS: the totals are
// sums of x and x^2 and go on to mean, variance and the running statistics (out0 = mean,
// out1 = variance); otherwise they are stored as they are.
template <bool STATS>
__global__ void __launch_bounds__(kSplitThreads)
ebn_merge_slab_sums(int64_t h, int S, const float* __restrict__ part, int64_t slab_stride, float* out0, float* out1,
                    int64_t count, float decay, float* rmean, float* rvar)
{
  __shared__ float lds[kSplitWaves][kWave][2];
  constexpr int U = 8;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kWave + lane;
  const bool ok = r < h;
  float a = 0.f, b = 0.f;
  if (ok) {
    for (int s0 = wave; s0 < S; s0 += U * kSplitWaves) {
      float va[U], vb[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int sl = s0 + u * kSplitWaves;
        va[u] = sl < S ? part[sl * slab_stride + r] : 0.f;
        vb[u] = sl < S ? part[sl * slab_stride + h + r] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        a += va[u];
        b += vb[u];
      }
    }
  }
  lds[wave][lane][0] = a;
  lds[wave][lane][1] = b;
  __syncthreads();
  if (wave != 0 || !ok) return;
  a = lds[0][lane][0], b = lds[0][lane][1];
#pragma unroll
  for (int k = 1; k < kSplitWaves; ++k) {
    a += lds[k][lane][0];
    b += lds[k][lane][1];
  }
  if (STATS) {
    ebn_stats_of_row(r, a, b, count, decay, out0, out1, rmean, rvar);
  }
  else {
    out0[r] = a;
    out1[r] = b;
  }
}

// y = (x - mean) / sqrt(var + eps) (entrywise_batch_normalization.cpp:131-160).  Grid
// (row blocks, column chunks).
template <int VE>
__global__ void __launch_bounds__(kSplitThreads)
ebn_split_fwd_apply(SplitArgs a)
{
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r0 = (static_cast<int64_t>(blockIdx.x) * kWave + lane) * VE;
  if (r0 >= a.h) return;
  float mean[VE], inv[VE];
  RowItem<VE>::load(a.mean + r0, mean);
  RowItem<VE>::load(a.var + r0, inv);
#pragma unroll
  for (int r = 0; r < VE; ++r) inv[r] = 1.0f / sqrtf(inv[r] + a.eps);
  const int64_t c_begin = static_cast<int64_t>(blockIdx.y) * kSplitApplyCols;
  const int64_t c_end = c_begin + kSplitApplyCols < a.w ? c_begin + kSplitApplyCols : a.w;
  for (int64_t c = c_begin + wave; c < c_end; c += kSplitWaves) {
    float v[VE];
    RowItem<VE>::load(a.x + r0 + c * a.ldx, v);
#pragma unroll
    for (int r = 0; r < VE; ++r) v[r] = (v[r] - mean[r]) * inv[r];
    RowItem<VE>::store(a.out + r0 + c * a.ldo, v);
  }
}

// dx = dy / sqrt(var + eps): the backward pass outside training (:352-392).  Grid as above.
template <int VE>
__global__ void __launch_bounds__(kSplitThreads)
ebn_split_scale_rows(SplitArgs a)
{
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r0 = (static_cast<int64_t>(blockIdx.x) * kWave + lane) * VE;
  if (r0 >= a.h) return;
  float inv[VE];
  RowItem<VE>::load(a.var + r0, inv);
#pragma unroll
  for (int r = 0; r < VE; ++r) inv[r] = 1.0f / sqrtf(inv[r] + a.eps);
  const int64_t c_begin = static_cast<int64_t>(blockIdx.y) * kSplitApplyCols;
  const int64_t c_end = c_begin + kSplitApplyCols < a.w ? c_begin + kSplitApplyCols : a.w;
  for (int64_t c = c_begin + wave; c < c_end; c += kSplitWaves) {
    float g[VE];
    RowItem<VE>::load(a.dy + r0 + c * a.lddy, g);
#pragma unroll
    for (int r = 0; r < VE; ++r) g[r] *= inv[r];
    RowItem<VE>::store(a.out + r0 + c * a.ldo, g);
  }
}

// sum0 = local part of dL/dmean = -sum(dy) / stdev, sum1 = of dL/dvar =
// -sum(dy (x - mean)) / (2 stdev^3) (entrywise_batch_normalization.cpp:275-299).
template <int VE>
__global__ void __launch_bounds__(kSplitThreads)
ebn_split_bwd_sums(SplitArgs a)
{
  __shared__ float lds[kSplitWaves][kWave * VE][2];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r0 = (static_cast<int64_t>(blockIdx.x) * kWave + lane) * VE;
  const bool ok = r0 < a.h;
  const int64_t rr = ok ? r0 : 0;
  float mean[VE], inv[VE];
  RowItem<VE>::load(a.mean + rr, mean);
  RowItem<VE>::load(a.var + rr, inv);
#pragma unroll
  for (int r = 0; r < VE; ++r) inv[r] = 1.0f / sqrtf(inv[r] + a.eps);
  float sa[VE], sb[VE];
#pragma unroll
  for (int r = 0; r < VE; ++r) sa[r] = sb[r] = 0.f;
  const SplitSlab sl = split_slab(a, ok);
  int64_t c = sl.c0 + wave;
  for (; c + kSplitWaves < sl.c1; c += 2 * kSplitWaves) {  // two columns of each tensor in flight
    float v[2][VE], g[2][VE];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      RowItem<VE>::load(a.x + rr + (c + j * kSplitWaves) * a.ldx, v[j]);
      RowItem<VE>::load(a.dy + rr + (c + j * kSplitWaves) * a.lddy, g[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < VE; ++r) {
        sa[r] += g[j][r];
        sb[r] = __builtin_fmaf(g[j][r], v[j][r] - mean[r], sb[r]);
      }
  }
  for (; c < sl.c1; c += kSplitWaves) {
    float v[VE], g[VE];
    RowItem<VE>::load(a.x + rr + c * a.ldx, v);
    RowItem<VE>::load(a.dy + rr + c * a.lddy, g);
#pragma unroll
    for (int r = 0; r < VE; ++r) {
      sa[r] += g[r];
      sb[r] = __builtin_fmaf(g[r], v[r] - mean[r], sb[r]);
    }
  }
  if (split_merge<VE>(sa, sb, lds) && ok) {
#pragma unroll
    for (int r = 0; r < VE; ++r) {
      sa[r] = -sa[r] * inv[r];
      sb[r] = -sb[r] * inv[r] * inv[r] * inv[r] * 0.5f;
    }
    RowItem<VE>::store(a.sum0 + sl.out + r0, sa);
    RowItem<VE>::store(a.sum1 + sl.out + r0, sb);
  }
}

// dx = dy / stdev + dmean / count + dvar (x - mean) 2 / (count - 1)
// (entrywise_batch_normalization.cpp:305-335), with the reduced dmean, dvar in sum0, sum1.
template <int VE>
__global__ void __launch_bounds__(kSplitThreads)
ebn_split_bwd_apply(SplitArgs a)
{
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r0 = (static_cast<int64_t>(blockIdx.x) * kWave + lane) * VE;
  if (r0 >= a.h) return;
  float mean[VE], inv[VE], c0[VE], c1[VE];
  RowItem<VE>::load(a.mean + r0, mean);
  RowItem<VE>::load(a.var + r0, inv);
  RowItem<VE>::load(a.sum0 + r0, c0);
  RowItem<VE>::load(a.sum1 + r0, c1);
#pragma unroll
  for (int r = 0; r < VE; ++r) {
    inv[r] = 1.0f / sqrtf(inv[r] + a.eps);
    c0[r] = c0[r] / a.count;
    c1[r] = c1[r] * 2.f / (a.count - 1.f);
  }
  const int64_t c_begin = static_cast<int64_t>(blockIdx.y) * kSplitApplyCols;
  const int64_t c_end = c_begin + kSplitApplyCols < a.w ? c_begin + kSplitApplyCols : a.w;
  for (int64_t c = c_begin + wave; c < c_end; c += kSplitWaves) {
    float v[VE], g[VE];
    RowItem<VE>::load(a.x + r0 + c * a.ldx, v);
    RowItem<VE>::load(a.dy + r0 + c * a.lddy, g);
#pragma unroll
    for (int r = 0; r < VE; ++r)
      g[r] = __builtin_fmaf(g[r], inv[r], __builtin_fmaf(c1[r], v[r] - mean[r], c0[r]));
    RowItem<VE>::store(a.out + r0 + c * a.ldo, g);
  }
}

__global__ void __launch_bounds__(256)
ebn_split_fill_zero(float* p, int64_t h, int64_t w, int64_t ld)
{
  const int64_t total = h * w;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t c = i / h;
    p[(i - c * h) + c * ld] = 0.f;
  }
}

static bool split_mat_vec_ok(int64_t h, int64_t w, const void* p, int64_t ld)
{
  return h % 4 == 0 && aligned16(p) && (w <= 1 || ld % 4 == 0);
}

static int split_check(int64_t h, int64_t w, const int64_t* lds, int nld)
{
  if (h < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < h) return LBN_ERR_INVALID_ARGUMENT;
  if (h > (int64_t(1) << 36)) return LBN_ERR_UNSUPPORTED;  // gridDim.x < 2^31 with 64 rows per workgroup
  if (w > int64_t(65535) * kSplitApplyCols) return LBN_ERR_UNSUPPORTED;  // gridDim.y of the apply kernels
  return LBN_OK;
}

static dim3 split_grid(int64_t h, int ve, int64_t col_chunks)
{
  return dim3(static_cast<unsigned>(ceil_div(h, int64_t(kWave) * ve)), static_cast<unsigned>(col_chunks));
}

// ------------------------------------------------------------ one rank, column slabs
// Slabs for an (h x w) problem: about four workgroups per compute unit in the summing kernel,
// at least 16 columns (four per wave) a slab.  1: the path does not pay.
constexpr int kSlabMinWidth = 1024;       // narrower mini-batches: one workgroup per 64 rows walks them in less time than four launches take
constexpr int64_t kSlabMaxHeight = 4096;  // taller matrices fill the device well enough without slabs (measured)
constexpr int kSlabMaxSlabs = 64;

static int ebn_slab_count(int64_t h, int64_t w)
{
  if (h % 4 != 0 || h > kSlabMaxHeight || w < kSlabMinWidth) return 1;
  const int64_t row_blocks = ceil_div(h, int64_t(kWave) * 4);
  int64_t S = ceil_div(1024, row_blocks);
  if (S > w / 16) S = w / 16;
  if (S > kSlabMaxSlabs) S = kSlabMaxSlabs;
  return static_cast<int>(S < 1 ? 1 : S);
}

size_t ebn_slab_workspace_bytes(int64_t h, int64_t w)
{
  const int S = ebn_slab_count(h, w);
  return S > 1 ? static_cast<size_t>(S) * 2 * h * sizeof(float) : 0;
}

static bool ebn_slab_ready(int64_t h, int64_t w, void* ws, size_t ws_bytes)
{
  const size_t need = ebn_slab_workspace_bytes(h, w);
  return need > 0 && ws && aligned16(ws) && ws_bytes >= need;
}

bool ebn_slab_fwd(hipStream_t st, int64_t h, int64_t w, float eps, float decay, const float* x, int64_t ldx, float* y,
                  int64_t ldy, float* stats, int64_t ld_stats, float* running_mean, float* running_var, void* ws,
                  size_t ws_bytes)
{
  if (!ebn_slab_ready(h, w, ws, ws_bytes)) return false;
  if (!split_mat_vec_ok(h, w, x, ldx) || !split_mat_vec_ok(h, w, y, ldy) || !aligned16(stats) || ld_stats % 4 != 0)
    return false;
  if (w > int64_t(65535) * kSplitApplyCols) return false;
  const int S = ebn_slab_count(h, w);
  float* part = static_cast<float*>(ws);
  SplitArgs a{};
  a.h = h; a.w = w; a.eps = eps; a.x = x; a.ldx = ldx; a.out = y; a.ldo = ldy;
  a.sum0 = part; a.sum1 = part + h; a.slab_cols = ceil_div(w, S); a.slab_stride = 2 * h;
  hipLaunchKernelGGL((ebn_split_fwd_sums<4>), split_grid(h, 4, S), dim3(kSplitThreads), 0, st, a);
  hipLaunchKernelGGL(ebn_merge_slab_sums<true>, dim3(static_cast<unsigned>(ceil_div(h, kWave))), dim3(kSplitThreads), 0,
                     st, h, S, part, a.slab_stride, stats, stats + ld_stats, w, decay, running_mean, running_var);
  a.mean = stats; a.var = stats + ld_stats;
  hipLaunchKernelGGL((ebn_split_fwd_apply<4>), split_grid(h, 4, ceil_div(w, kSplitApplyCols)), dim3(kSplitThreads), 0,
                     st, a);
  return true;
}

bool ebn_slab_bwd(hipStream_t st, int64_t h, int64_t w, float eps, const float* x, int64_t ldx, const float* dy,
                  int64_t lddy, float* dx, int64_t lddx, const float* stats, int64_t ld_stats, float* stats_grad,
                  int64_t ld_stats_grad, void* ws, size_t ws_bytes)
{
  if (!ebn_slab_ready(h, w, ws, ws_bytes)) return false;
  if (!split_mat_vec_ok(h, w, x, ldx) || !split_mat_vec_ok(h, w, dy, lddy) || !split_mat_vec_ok(h, w, dx, lddx) ||
      !aligned16(stats) || ld_stats % 4 != 0 || !aligned16(stats_grad) || ld_stats_grad % 4 != 0)
    return false;
  if (w > int64_t(65535) * kSplitApplyCols) return false;
  const int S = ebn_slab_count(h, w);
  float* part = static_cast<float*>(ws);
  SplitArgs a{};
  a.h = h; a.w = w; a.eps = eps; a.count = static_cast<float>(w);
  a.x = x; a.ldx = ldx; a.dy = dy; a.lddy = lddy; a.out = dx; a.ldo = lddx;
  a.mean = stats; a.var = stats + ld_stats;
  a.sum0 = part; a.sum1 = part + h; a.slab_cols = ceil_div(w, S); a.slab_stride = 2 * h;
  hipLaunchKernelGGL((ebn_split_bwd_sums<4>), split_grid(h, 4, S), dim3(kSplitThreads), 0, st, a);
  hipLaunchKernelGGL(ebn_merge_slab_sums<false>, dim3(static_cast<unsigned>(ceil_div(h, kWave))), dim3(kSplitThreads),
                     0, st, h, S, part, a.slab_stride, stats_grad, stats_grad + ld_stats_grad, int64_t(0), 0.f,
                     static_cast<float*>(nullptr), static_cast<float*>(nullptr));
  a.sum0 = stats_grad; a.sum1 = stats_grad + ld_stats_grad;
  hipLaunchKernelGGL((ebn_split_bwd_apply<4>), split_grid(h, 4, ceil_div(w, kSplitApplyCols)), dim3(kSplitThreads), 0,
                     st, a);
  return true;
}

void ebn_inference_fwd(hipStream_t st, int64_t h, int64_t w, float eps, const float* x, int64_t ldx, float* y,
                       int64_t ldy, const float* running_mean, const float* running_var)
{
  SplitArgs a{};
  a.h = h; a.w = w; a.eps = eps; a.x = x; a.ldx = ldx; a.out = y; a.ldo = ldy;
  a.mean = running_mean; a.var = running_var;
  const bool vec = split_mat_vec_ok(h, w, x, ldx) && split_mat_vec_ok(h, w, y, ldy) && aligned16(running_mean) &&
                   aligned16(running_var);
  // columns beyond gridDim.y's reach: the call is repeated over column blocks
  const int64_t per_call = int64_t(65535) * kSplitApplyCols;
  for (int64_t c0 = 0; c0 < w; c0 += per_call) {
    SplitArgs b = a;
    b.w = w - c0 < per_call ? w - c0 : per_call;
    b.x = x + c0 * ldx;
    b.out = y + c0 * ldy;
    const int64_t chunks = ceil_div(b.w, kSplitApplyCols);
    if (vec) hipLaunchKernelGGL((ebn_split_fwd_apply<4>), split_grid(h, 4, chunks), dim3(kSplitThreads), 0, st, b);
    else hipLaunchKernelGGL((ebn_split_fwd_apply<1>), split_grid(h, 1, chunks), dim3(kSplitThreads), 0, st, b);
  }
}

void ebn_inference_bwd(hipStream_t st, int64_t h, int64_t w, float eps, const float* dy, int64_t lddy, float* dx,
                       int64_t lddx, const float* running_var)
{
  SplitArgs a{};
  a.h = h; a.w = w; a.eps = eps; a.dy = dy; a.lddy = lddy; a.out = dx; a.ldo = lddx; a.var = running_var;
  const bool vec = split_mat_vec_ok(h, w, dy, lddy) && split_mat_vec_ok(h, w, dx, lddx) && aligned16(running_var);
  const int64_t per_call = int64_t(65535) * kSplitApplyCols;
  for (int64_t c0 = 0; c0 < w; c0 += per_call) {
    SplitArgs b = a;
    b.w = w - c0 < per_call ? w - c0 : per_call;
    b.dy = dy + c0 * lddy;
    b.out = dx + c0 * lddx;
    const int64_t chunks = ceil_div(b.w, kSplitApplyCols);
    if (vec) hipLaunchKernelGGL((ebn_split_scale_rows<4>), split_grid(h, 4, chunks), dim3(kSplitThreads), 0, st, b);
    else hipLaunchKernelGGL((ebn_split_scale_rows<1>), split_grid(h, 1, chunks), dim3(kSplitThreads), 0, st, b);
  }
}

}  // namespace lbn

using namespace lbn;

extern "C" {

int lbn_entrywise_batch_norm_fwd_sums_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                                          int64_t ldx, float* stats, int64_t ld_stats)
{
  const int64_t lds[1] = {ldx};
  if (int e = split_check(height, width, lds, 1)) return e;
  if (height == 0) return LBN_OK;
  if (!stats || ld_stats < height || (width > 0 && !x)) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  SplitArgs a{};
  a.h = height; a.w = width; a.x = x; a.ldx = ldx; a.sum0 = stats; a.sum1 = stats + ld_stats;
  // no local columns: the sums are zero (El::Zero before the loop, :77)
  const bool vec = (width == 0 ? height % 4 == 0 : split_mat_vec_ok(height, width, x, ldx)) &&
                   aligned16(stats) && ld_stats % 4 == 0;
  if (vec) hipLaunchKernelGGL((ebn_split_fwd_sums<4>), split_grid(height, 4, 1), dim3(kSplitThreads), 0, st, a);
  else hipLaunchKernelGGL((ebn_split_fwd_sums<1>), split_grid(height, 1, 1), dim3(kSplitThreads), 0, st, a);
  return launch_status();
}

int lbn_entrywise_batch_norm_fwd_stats_f32(lbn_stream_t stream, int64_t height, int64_t statistics_count,
                                           float decay, float* stats, int64_t ld_stats, float* running_mean,
                                           float* running_var)
{
  if (height < 0 || statistics_count < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0) return LBN_OK;
  if (!stats || ld_stats < height || !running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
  if (height > (int64_t(1) << 36)) return LBN_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(ebn_split_fwd_stats, dim3(static_cast<unsigned>(ceil_div(height, 256))), dim3(256), 0,
                     as_stream(stream), height, statistics_count, decay, stats, stats + ld_stats, running_mean,
                     running_var);
  return launch_status();
}

int lbn_entrywise_batch_norm_fwd_apply_f32(lbn_stream_t stream, int64_t height, int64_t width, float epsilon,
                                           const float* x, int64_t ldx, float* y, int64_t ldy, const float* mean,
                                           const float* var)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = split_check(height, width, lds, 2)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!x || !y || !mean || !var) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  SplitArgs a{};
  a.h = height; a.w = width; a.eps = epsilon; a.x = x; a.ldx = ldx; a.out = y; a.ldo = ldy;
  a.mean = mean; a.var = var;
  const int64_t chunks = ceil_div(width, kSplitApplyCols);
  const bool vec = split_mat_vec_ok(height, width, x, ldx) && split_mat_vec_ok(height, width, y, ldy) &&
                   aligned16(mean) && aligned16(var);
  if (vec) hipLaunchKernelGGL((ebn_split_fwd_apply<4>), split_grid(height, 4, chunks), dim3(kSplitThreads), 0, st, a);
  else hipLaunchKernelGGL((ebn_split_fwd_apply<1>), split_grid(height, 1, chunks), dim3(kSplitThreads), 0, st, a);
  return launch_status();
}

int lbn_entrywise_batch_norm_bwd_sums_f32(lbn_stream_t stream, int64_t height, int64_t width, float epsilon,
                                          const float* x, int64_t ldx, const float* dy, int64_t lddy,
                                          const float* stats, int64_t ld_stats, float* stats_grad,
                                          int64_t ld_stats_grad)
{
  const int64_t lds[2] = {ldx, lddy};
  if (int e = split_check(height, width, lds, 2)) return e;
  if (height == 0) return LBN_OK;
  if (!stats || !stats_grad || ld_stats < height || ld_stats_grad < height || (width > 0 && (!x || !dy)))
    return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  SplitArgs a{};
  a.h = height; a.w = width; a.eps = epsilon; a.x = x; a.ldx = ldx; a.dy = dy; a.lddy = lddy;
  a.mean = stats; a.var = stats + ld_stats; a.sum0 = stats_grad; a.sum1 = stats_grad + ld_stats_grad;
  const bool mats = width == 0 ? height % 4 == 0
                               : split_mat_vec_ok(height, width, x, ldx) && split_mat_vec_ok(height, width, dy, lddy);
  const bool vec = mats && aligned16(stats) && ld_stats % 4 == 0 && aligned16(stats_grad) && ld_stats_grad % 4 == 0;
  if (vec) hipLaunchKernelGGL((ebn_split_bwd_sums<4>), split_grid(height, 4, 1), dim3(kSplitThreads), 0, st, a);
  else hipLaunchKernelGGL((ebn_split_bwd_sums<1>), split_grid(height, 1, 1), dim3(kSplitThreads), 0, st, a);
  return launch_status();
}

int lbn_entrywise_batch_norm_bwd_apply_f32(lbn_stream_t stream, int64_t height, int64_t width,
                                           int64_t statistics_count, float epsilon, const float* x, int64_t ldx,
                                           const float* dy, int64_t lddy, float* dx, int64_t lddx,
                                           const float* stats, int64_t ld_stats, const float* stats_grad,
                                           int64_t ld_stats_grad)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = split_check(height, width, lds, 3)) return e;
  if (statistics_count < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (!dx) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  if (statistics_count <= 1) {  // constant output: zero gradient (:268-271)
    hipLaunchKernelGGL(ebn_split_fill_zero, dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(height * width, 256), 65536))),
                       dim3(256), 0, st, dx, height, width, lddx);
    return launch_status();
  }
  if (!x || !dy || !stats || !stats_grad || ld_stats < height || ld_stats_grad < height)
    return LBN_ERR_INVALID_ARGUMENT;
  SplitArgs a{};
  a.h = height; a.w = width; a.eps = epsilon; a.count = static_cast<float>(statistics_count);
  a.x = x; a.ldx = ldx; a.dy = dy; a.lddy = lddy; a.out = dx; a.ldo = lddx;
  a.mean = stats; a.var = stats + ld_stats;
  a.sum0 = const_cast<float*>(stats_grad); a.sum1 = const_cast<float*>(stats_grad) + ld_stats_grad;
  const int64_t chunks = ceil_div(width, kSplitApplyCols);
  const bool vec = split_mat_vec_ok(height, width, x, ldx) && split_mat_vec_ok(height, width, dy, lddy) &&
                   split_mat_vec_ok(height, width, dx, lddx) && aligned16(stats) && ld_stats % 4 == 0 &&
                   aligned16(stats_grad) && ld_stats_grad % 4 == 0;
  if (vec) hipLaunchKernelGGL((ebn_split_bwd_apply<4>), split_grid(height, 4, chunks), dim3(kSplitThreads), 0, st, a);
  else hipLaunchKernelGGL((ebn_split_bwd_apply<1>), split_grid(height, 1, chunks), dim3(kSplitThreads), 0, st, a);
  return launch_status();
}

}  // extern "C"
