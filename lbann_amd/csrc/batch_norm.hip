// Batch normalization forward and backward for gfx950 (fp32).
//
// Channel c of an NCHW mini-batch is the row range [c*cs, (c+1)*cs) of every matrix
// column, so a per-channel reduction crosses all columns: `width` segments of `cs`
// contiguous floats.  The reduction is split over P workgroups per channel
// (grid P x C) that walk the channel's segments with 128-bit coalesced loads and
// leave one partial pair per workgroup in the workspace; the apply kernel (same
// grid) merges the P partials in a fixed order in its prologue, workgroup 0 of each
// channel writes the statistics, and all P workgroups stream the channel once more
// to write the output.  No atomics: results are bitwise reproducible.
//
// Forward statistics are accumulated about a per-channel pivot (the channel's first
// entry), sum(x-K) and sum((x-K)^2), which removes the cancellation of
// E[x^2]-mean^2 when |mean| >> stdev at no extra cost; LBN_STATS_SUMSQ selects
// K = 0, the reference's formula (batch_normalization.cpp:70-85, :124-128).
#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {

constexpr int kBnThreads = 256;
constexpr int kBnMaxSplit = 64;  // P <= one wave, so a wave merges a channel's partials

// Walks the elements of channel c owned by workgroup p: calls f(offset_in_x, offset_in_y...)
// through index arithmetic shared by all kernels.  `unit` = floats per access (4 or 1),
// `seg` = accesses per column segment (cs / unit).
struct ChannelWalk {
  int64_t cs;    // channel size in floats
  int64_t seg;   // accesses per segment
  int64_t total; // accesses per channel = seg * width
};

template <bool VEC>
__device__ __forceinline__ ChannelWalk make_walk(int64_t cs, int64_t w)
{
  const int64_t seg = VEC ? cs / 4 : cs;
  return {cs, seg, seg * w};
}

// ------------------------------------------------------------------ forward sums
template <bool VEC>
__global__ void __launch_bounds__(kBnThreads)
bn_fwd_sums(const float* __restrict__ x, int64_t ldx, int64_t cs, int64_t w, int use_pivot,
            float2* __restrict__ part)
{
  __shared__ float red[2 * (kBnThreads / kWave)];
  const int P = gridDim.x;
  const int p = blockIdx.x;
  const int64_t c = blockIdx.y;
  const ChannelWalk wk = make_walk<VEC>(cs, w);
  const float* xc = x + c * cs;
  const float K = use_pivot ? xc[0] : 0.f;
  float s = 0.f, q = 0.f;
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const int64_t col = j / wk.seg;
    const int64_t i = j - col * wk.seg;
    if (VEC) {
      float v[4];
      Vec16<float>::load(xc + col * ldx + 4 * i, v);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float d = v[k] - K;
        s += d;
        q += d * d;
      }
    }
    else {
      const float d = xc[col * ldx + i] - K;
      s += d;
      q += d * d;
    }
  }
  team_sum2<kBnThreads / kWave>(s, q, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) part[c * P + p] = make_float2(s, q);
}

// Merges the P partial pairs of channel c; every lane of the calling wave gets the sums.
__device__ __forceinline__ float2 merge_partials(const float2* part, int64_t c, int P)
{
  const int lane = threadIdx.x & (kWave - 1);
  float a = 0.f, b = 0.f;
  if (lane < P) {
    const float2 v = part[c * P + lane];
    a = v.x;
    b = v.y;
  }
  return make_float2(wave_sum(a), wave_sum(b));
}

// Mean / variance from sums about pivot K over n values, with the reference's Bessel
// factor and epsilon floor (batch_normalization.cpp:118-131).
__device__ __forceinline__ void stats_from_sums(float s, float q, float K, int64_t n, int bessel,
                                                float eps, float& mean, float& var)
{
  const float nf = static_cast<float>(n);
  const float dm = s / nf;
  const float sqmean = q / nf;
  mean = K + dm;
  var = nf * (sqmean - dm * dm) / (nf - static_cast<float>(bessel ? 1 : 0));
  var = fmaxf(var, eps);
}

// Raw per-channel sums for callers that all-reduce them: mean[c] = sum, var[c] = sqsum.
__global__ void __launch_bounds__(kWave)
bn_store_sums(const float2* __restrict__ part, int P, float* __restrict__ mean,
              float* __restrict__ var)
{
  const int64_t c = blockIdx.x;
  const float2 r = merge_partials(part, c, P);
  if (threadIdx.x == 0) {
    mean[c] = r.x;
    var[c] = r.y;
  }
}

__global__ void __launch_bounds__(256)
bn_stats_from_sums(int64_t C, int64_t n, int bessel, float eps, float decay,
                   float* __restrict__ mean, float* __restrict__ var,
                   float* __restrict__ rmean, float* __restrict__ rvar)
{
  const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (c >= C) return;
  if (n <= 1) {
    var[c] = 1.f;
    return;
  }
  float m, v;
  stats_from_sums(mean[c], var[c], 0.f, n, bessel, eps, m, v);
  mean[c] = m;
  var[c] = v;
  rmean[c] = decay * rmean[c] + (1.f - decay) * m;
  rvar[c] = decay * rvar[c] + (1.f - decay) * v;
}

// ----------------------------------------------------------------- forward apply
// FROM_PART: statistics come from the partial sums in `part` (training, fused path)
// and workgroup 0 of each channel publishes them; otherwise mean/var are inputs.
template <bool VEC, bool FROM_PART>
__global__ void __launch_bounds__(kBnThreads)
bn_fwd_apply(const float* __restrict__ x, float* __restrict__ y, int64_t ldx, int64_t ldy,
             int64_t cs, int64_t w, int use_pivot, int bessel, float eps, float decay,
             const float2* __restrict__ part, float* __restrict__ mean_io,
             float* __restrict__ var_io, const float* __restrict__ gamma,
             const float* __restrict__ beta, float* __restrict__ rmean, float* __restrict__ rvar)
{
  const int P = gridDim.x;
  const int p = blockIdx.x;
  const int64_t c = blockIdx.y;
  const ChannelWalk wk = make_walk<VEC>(cs, w);
  const float* xc = x + c * cs;
  float* yc = y + c * cs;
  float mean, var;
  if (FROM_PART) {
    const int64_t n = cs * w;
    if (n <= 1) {
      mean = xc[0];
      var = 1.f;
      if (p == 0 && threadIdx.x == 0) {
        mean_io[c] = mean;
        var_io[c] = var;
      }
    }
    else {
      const float K = use_pivot ? xc[0] : 0.f;
      const float2 r = merge_partials(part, c, P);
      stats_from_sums(r.x, r.y, K, n, bessel, eps, mean, var);
      if (p == 0 && threadIdx.x == 0) {
        mean_io[c] = mean;
        var_io[c] = var;
        rmean[c] = decay * rmean[c] + (1.f - decay) * mean;
        rvar[c] = decay * rvar[c] + (1.f - decay) * var;
      }
    }
  }
  else {
    mean = mean_io[c];
    var = var_io[c];
  }
  const float inv_stdev = 1.0f / sqrtf(var + eps);
  const float scale = gamma[c];
  const float bias = beta[c];
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const int64_t col = j / wk.seg;
    const int64_t i = j - col * wk.seg;
    if (VEC) {
      float v[4];
      Vec16<float>::load(xc + col * ldx + 4 * i, v);
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = scale * ((v[k] - mean) * inv_stdev) + bias;
      Vec16<float>::store(yc + col * ldy + 4 * i, v);
    }
    else {
      yc[col * ldy + i] = scale * ((xc[col * ldx + i] - mean) * inv_stdev) + bias;
    }
  }
}

// ----------------------------------------------------------------- backward sums
// Two sums per channel carry all four gradients: A = sum(dy), B = sum(dy * (x - mean)).
template <bool VEC>
__global__ void __launch_bounds__(kBnThreads)
bn_bwd_sums(const float* __restrict__ x, const float* __restrict__ dy, int64_t ldx, int64_t lddy,
            int64_t cs, int64_t w, const float* __restrict__ mean_in, float2* __restrict__ part)
{
  __shared__ float red[2 * (kBnThreads / kWave)];
  const int P = gridDim.x;
  const int p = blockIdx.x;
  const int64_t c = blockIdx.y;
  const ChannelWalk wk = make_walk<VEC>(cs, w);
  const float* xc = x + c * cs;
  const float* gc = dy + c * cs;
  const float mean = mean_in[c];
  float a = 0.f, b = 0.f;
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const int64_t col = j / wk.seg;
    const int64_t i = j - col * wk.seg;
    if (VEC) {
      float v[4], g[4];
      Vec16<float>::load(xc + col * ldx + 4 * i, v);
      Vec16<float>::load(gc + col * lddy + 4 * i, g);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        a += g[k];
        b += g[k] * (v[k] - mean);
      }
    }
    else {
      const float g = gc[col * lddy + i];
      a += g;
      b += g * (xc[col * ldx + i] - mean);
    }
  }
  team_sum2<kBnThreads / kWave>(a, b, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) part[c * P + p] = make_float2(a, b);
}

__device__ __forceinline__ void grads_from_sums(float A, float B, float scale, float inv_stdev,
                                                float& dscale, float& dbias, float& dmean,
                                                float& dvar)
{
  dscale = B * inv_stdev;
  dbias = A;
  dmean = -(scale * inv_stdev) * A;
  dvar = -scale * B * (inv_stdev * inv_stdev * inv_stdev / 2);
}

__global__ void __launch_bounds__(kWave)
bn_store_grads(const float2* __restrict__ part, int P, float eps, const float* __restrict__ mean,
               const float* __restrict__ var, const float* __restrict__ gamma,
               float* __restrict__ dscale, float* __restrict__ dbias, float* __restrict__ dmean,
               float* __restrict__ dvar)
{
  const int64_t c = blockIdx.x;
  const float2 r = merge_partials(part, c, P);
  if (threadIdx.x == 0) {
    const float inv_stdev = 1.0f / sqrtf(var[c] + eps);
    float ds, db, dm, dv;
    grads_from_sums(r.x, r.y, gamma[c], inv_stdev, ds, db, dm, dv);
    dscale[c] = ds;
    dbias[c] = db;
    dmean[c] = dm;
    dvar[c] = dv;
  }
  (void)mean;
}

// ---------------------------------------------------------------- backward apply
// FROM_PART: gradients of the statistics come from the partial sums (fused path) and
// workgroup 0 of each channel publishes dscale, dbias, dmean, dvar; otherwise dmean
// and dvar are inputs (already reduced over ranks by the caller).
template <bool VEC, bool FROM_PART>
__global__ void __launch_bounds__(kBnThreads)
bn_bwd_apply(const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ dx,
             int64_t ldx, int64_t lddy, int64_t lddx, int64_t cs, int64_t w, int64_t num_per_sum,
             int bessel, float eps, int training, const float2* __restrict__ part,
             const float* __restrict__ mean_in, const float* __restrict__ var_in,
             const float* __restrict__ gamma, float* __restrict__ dscale,
             float* __restrict__ dbias, float* __restrict__ dmean_io, float* __restrict__ dvar_io)
{
  const int P = gridDim.x;
  const int p = blockIdx.x;
  const int64_t c = blockIdx.y;
  const ChannelWalk wk = make_walk<VEC>(cs, w);
  const float* xc = x + c * cs;
  const float* gc = dy + c * cs;
  float* dc = dx + c * cs;
  const float mean = mean_in[c];
  const float inv_stdev = 1.0f / sqrtf(var_in[c] + eps);
  const float scale = gamma[c];
  float dmean, dvar;
  if (FROM_PART) {
    const float2 r = merge_partials(part, c, P);
    float ds, db;
    grads_from_sums(r.x, r.y, scale, inv_stdev, ds, db, dmean, dvar);
    if (!training) dmean = dvar = 0.f;  // statistics are constants outside training
    if (p == 0 && threadIdx.x == 0) {
      dscale[c] = ds;
      dbias[c] = db;
      dmean_io[c] = dmean;
      dvar_io[c] = dvar;
    }
  }
  else {
    dmean = dmean_io[c];
    dvar = dvar_io[c];
  }
  const bool zero = num_per_sum <= 1;
  const float k0 = scale * inv_stdev;
  const float dmean_term = dmean / static_cast<float>(num_per_sum);
  const float dvar_term = dvar * 2.f / static_cast<float>(num_per_sum - (bessel ? 1 : 0));
  const int64_t step = static_cast<int64_t>(P) * kBnThreads;
  for (int64_t j = static_cast<int64_t>(p) * kBnThreads + threadIdx.x; j < wk.total; j += step) {
    const int64_t col = j / wk.seg;
    const int64_t i = j - col * wk.seg;
    if (VEC) {
      float v[4], g[4];
      if (!zero) {
        Vec16<float>::load(xc + col * ldx + 4 * i, v);
        Vec16<float>::load(gc + col * lddy + 4 * i, g);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) g[k] = zero ? 0.f : g[k] * k0 + dmean_term + dvar_term * (v[k] - mean);
      Vec16<float>::store(dc + col * lddx + 4 * i, g);
    }
    else {
      dc[col * lddx + i] =
        zero ? 0.f : gc[col * lddy + i] * k0 + dmean_term + dvar_term * (xc[col * ldx + i] - mean);
    }
  }
}

// ==================================================================== host side
// Workgroups per channel: about 4096 workgroups in total, each with at least four
// accesses per thread, at most one wave's worth so a wave can merge the partials.
static int bn_split(int64_t C, int64_t cs, int64_t w)
{
  int64_t P = ceil_div(4096, C);
  const int64_t by_work = ceil_div(cs * w, 4 * 4 * kBnThreads);
  if (P > by_work) P = by_work;
  if (P > kBnMaxSplit) P = kBnMaxSplit;
  if (P < 1) P = 1;
  return static_cast<int>(P);
}

static size_t bn_workspace(int64_t C, int64_t cs, int64_t w)
{
  if (C <= 0 || cs <= 0 || w <= 0) return 0;
  return static_cast<size_t>(C) * bn_split(C, cs, w) * sizeof(float2);
}

struct BnShape {
  int64_t C, cs, w;
  int P;
  bool ok;
};

static int bn_check(int64_t C, int64_t cs, int64_t w, const int64_t* lds, int nld)
{
  if (C < 0 || cs < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < C * cs) return LBN_ERR_INVALID_ARGUMENT;
  if (C > 65535) return LBN_ERR_UNSUPPORTED;  // channels ride on gridDim.y
  return LBN_OK;
}

static bool bn_vec_ok(int64_t cs, int64_t w, const void* a, int64_t lda)
{
  return cs % 4 == 0 && aligned16(a) && (w <= 1 || lda % 4 == 0);
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_batch_norm_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  return bn_workspace(channels, channel_size, width);
}

int lbn_batch_norm_fwd_sums_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                const float* x, int64_t ldx, float* mean, float* var,
                                void* workspace, size_t workspace_bytes)
{
  const int64_t lds[1] = {ldx};
  if (int e = bn_check(C, cs, w, lds, 1)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !mean || !var) return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace);
  const dim3 grid(P, static_cast<unsigned>(C));
  hipStream_t st = as_stream(stream);
  if (bn_vec_ok(cs, w, x, ldx))
    hipLaunchKernelGGL((bn_fwd_sums<true>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, 0, part);
  else
    hipLaunchKernelGGL((bn_fwd_sums<false>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, 0, part);
  hipLaunchKernelGGL(bn_store_sums, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, part, P, mean, var);
  return launch_status();
}

int lbn_batch_norm_fwd_stats_f32(lbn_stream_t stream, int64_t C, int64_t num_per_sum, int bessel,
                                 float epsilon, float decay, float* mean, float* var,
                                 float* running_mean, float* running_var)
{
  if (C < 0 || num_per_sum < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (C == 0) return LBN_OK;
  if (!mean || !var || !running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(bn_stats_from_sums, dim3(static_cast<unsigned>(ceil_div(C, 256))), dim3(256), 0,
                     as_stream(stream), C, num_per_sum, bessel, epsilon, decay, mean, var,
                     running_mean, running_var);
  return launch_status();
}

int lbn_batch_norm_fwd_apply_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                 float epsilon, const float* x, int64_t ldx, float* y, int64_t ldy,
                                 const float* mean, const float* var, const float* scale,
                                 const float* bias)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !y || !mean || !var || !scale || !bias) return LBN_ERR_INVALID_ARGUMENT;
  const int P = bn_split(C, cs, w);
  const dim3 grid(P, static_cast<unsigned>(C));
  hipStream_t st = as_stream(stream);
  float* m = const_cast<float*>(mean);
  float* v = const_cast<float*>(var);
  if (bn_vec_ok(cs, w, x, ldx) && bn_vec_ok(cs, w, y, ldy))
    hipLaunchKernelGGL((bn_fwd_apply<true, false>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs,
                       w, 0, 0, epsilon, 0.f, nullptr, m, v, scale, bias, nullptr, nullptr);
  else
    hipLaunchKernelGGL((bn_fwd_apply<false, false>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs,
                       w, 0, 0, epsilon, 0.f, nullptr, m, v, scale, bias, nullptr, nullptr);
  return launch_status();
}

int lbn_batch_norm_fwd_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                           float epsilon, float decay, int training, const float* x, int64_t ldx,
                           float* y, int64_t ldy, float* mean, float* var, const float* scale,
                           const float* bias, float* running_mean, float* running_var,
                           void* workspace, size_t workspace_bytes, int flags)
{
  if (!training) {
    if (!running_mean || !running_var) return LBN_ERR_INVALID_ARGUMENT;
    return lbn_batch_norm_fwd_apply_f32(stream, C, cs, w, epsilon, x, ldx, y, ldy, running_mean,
                                        running_var, scale, bias);
  }
  const int64_t lds[2] = {ldx, ldy};
  if (int e = bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !y || !mean || !var || !scale || !bias || !running_mean || !running_var)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace);
  const dim3 grid(P, static_cast<unsigned>(C));
  hipStream_t st = as_stream(stream);
  const int pivot = (flags & LBN_STATS_SUMSQ) ? 0 : 1;
  if (bn_vec_ok(cs, w, x, ldx) && bn_vec_ok(cs, w, y, ldy)) {
    hipLaunchKernelGGL((bn_fwd_sums<true>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, pivot, part);
    hipLaunchKernelGGL((bn_fwd_apply<true, true>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs, w,
                       pivot, bessel, epsilon, decay, part, mean, var, scale, bias, running_mean,
                       running_var);
  }
  else {
    hipLaunchKernelGGL((bn_fwd_sums<false>), grid, dim3(kBnThreads), 0, st, x, ldx, cs, w, pivot, part);
    hipLaunchKernelGGL((bn_fwd_apply<false, true>), grid, dim3(kBnThreads), 0, st, x, y, ldx, ldy, cs, w,
                       pivot, bessel, epsilon, decay, part, mean, var, scale, bias, running_mean,
                       running_var);
  }
  return launch_status();
}

int lbn_batch_norm_bwd_sums_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                float epsilon, const float* x, int64_t ldx, const float* dy,
                                int64_t lddy, const float* mean, const float* var,
                                const float* scale, float* dscale, float* dbias, float* dmean,
                                float* dvar, void* workspace, size_t workspace_bytes)
{
  const int64_t lds[2] = {ldx, lddy};
  if (int e = bn_check(C, cs, w, lds, 2)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !dy || !mean || !var || !scale || !dscale || !dbias || !dmean || !dvar)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace);
  const dim3 grid(P, static_cast<unsigned>(C));
  hipStream_t st = as_stream(stream);
  if (bn_vec_ok(cs, w, x, ldx) && bn_vec_ok(cs, w, dy, lddy))
    hipLaunchKernelGGL((bn_bwd_sums<true>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, mean, part);
  else
    hipLaunchKernelGGL((bn_bwd_sums<false>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, mean, part);
  hipLaunchKernelGGL(bn_store_grads, dim3(static_cast<unsigned>(C)), dim3(kWave), 0, st, part, P, epsilon,
                     mean, var, scale, dscale, dbias, dmean, dvar);
  return launch_status();
}

int lbn_batch_norm_bwd_apply_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w,
                                 int64_t num_per_sum, int bessel, float epsilon, const float* x,
                                 int64_t ldx, const float* dy, int64_t lddy, float* dx,
                                 int64_t lddx, const float* mean, const float* var,
                                 const float* scale, const float* dmean, const float* dvar)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = bn_check(C, cs, w, lds, 3)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  if (!x || !dy || !dx || !mean || !var || !scale || !dmean || !dvar) return LBN_ERR_INVALID_ARGUMENT;
  const int P = bn_split(C, cs, w);
  const dim3 grid(P, static_cast<unsigned>(C));
  hipStream_t st = as_stream(stream);
  float* dm = const_cast<float*>(dmean);
  float* dv = const_cast<float*>(dvar);
  if (bn_vec_ok(cs, w, x, ldx) && bn_vec_ok(cs, w, dy, lddy) && bn_vec_ok(cs, w, dx, lddx))
    hipLaunchKernelGGL((bn_bwd_apply<true, false>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, num_per_sum, bessel, epsilon, 1, nullptr, mean, var, scale, nullptr,
                       nullptr, dm, dv);
  else
    hipLaunchKernelGGL((bn_bwd_apply<false, false>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, num_per_sum, bessel, epsilon, 1, nullptr, mean, var, scale, nullptr,
                       nullptr, dm, dv);
  return launch_status();
}

int lbn_batch_norm_bwd_f32(lbn_stream_t stream, int64_t C, int64_t cs, int64_t w, int bessel,
                           float epsilon, int training, const float* x, int64_t ldx,
                           const float* dy, int64_t lddy, float* dx, int64_t lddx,
                           const float* mean, const float* var, const float* running_mean,
                           const float* running_var, const float* scale, float* dscale,
                           float* dbias, float* dmean, float* dvar, void* workspace,
                           size_t workspace_bytes)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = bn_check(C, cs, w, lds, 3)) return e;
  if (C == 0 || cs == 0 || w == 0) return LBN_OK;
  const float* use_mean = training ? mean : running_mean;
  const float* use_var = training ? var : running_var;
  if (!x || !dy || !dx || !use_mean || !use_var || !scale || !dscale || !dbias || !dmean || !dvar)
    return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < bn_workspace(C, cs, w)) return LBN_ERR_WORKSPACE;
  const int P = bn_split(C, cs, w);
  float2* part = static_cast<float2*>(workspace);
  const dim3 grid(P, static_cast<unsigned>(C));
  hipStream_t st = as_stream(stream);
  const int64_t n = cs * w;
  if (bn_vec_ok(cs, w, x, ldx) && bn_vec_ok(cs, w, dy, lddy) && bn_vec_ok(cs, w, dx, lddx)) {
    hipLaunchKernelGGL((bn_bwd_sums<true>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, use_mean, part);
    hipLaunchKernelGGL((bn_bwd_apply<true, true>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, n, bessel, epsilon, training, part, use_mean, use_var, scale, dscale,
                       dbias, dmean, dvar);
  }
  else {
    hipLaunchKernelGGL((bn_bwd_sums<false>), grid, dim3(kBnThreads), 0, st, x, dy, ldx, lddy, cs, w, use_mean, part);
    hipLaunchKernelGGL((bn_bwd_apply<false, true>), grid, dim3(kBnThreads), 0, st, x, dy, dx, ldx, lddy,
                       lddx, cs, w, n, bessel, epsilon, training, part, use_mean, use_var, scale, dscale,
                       dbias, dmean, dvar);
  }
  return launch_status();
}

}  // extern "C"
