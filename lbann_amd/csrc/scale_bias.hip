// Entry-wise and channel-wise scale/bias layers: y = a*x + b with one (a, b) pair per
// entry of the sample tensor (a matrix row) or per channel (a block of channel_size
// rows); backward gives dx = a*dy and the weight gradients da = sum(x*dy), db = sum(dy)
// over everything that shares the pair.
// Reference CPU code: src/layers/learning/entrywise_scale_bias.cpp:35-60 (forward),
// :62-113 (backward); src/layers/learning/channelwise_scale_bias.cpp:33-73, :75-135.
//
// Both are streaming kernels (forward moves 8 bytes per entry, backward 12); the only
// structure is where the weight-gradient sums run:
//  * entry-wise: along the strided direction of the column-major matrix.  A 256-thread
//    block owns 256/GW rows; consecutive lanes take consecutive row quads (16 bytes),
//    the 4*GW column groups of the block each walk every (4*GW)-th column of the block's
//    column slab, and the groups merge their sums by lane exchange and through LDS in a
//    fixed order.  Short matrices are cut into column slabs (grid.y) so that the launch
//    still fills the device; the slabs' partial sums go through the workspace and a
//    second small kernel adds them in slab order.
//  * channel-wise: along a channel, which is `width` segments of channel_size contiguous
//    entries.  grid = (channels, P): the P workgroups of a channel stride over its
//    16-byte vectors, reduce their partial pair, and a one-wave kernel per channel merges
//    the P pairs in order.
// Unaligned shapes take scalar variants of the same kernels.  No atomics: results do
// not depend on scheduling.
#include "device_utils.hpp"
#include "host_utils.hpp"
#include "row_tiles.hpp"

namespace lbn {

constexpr int kSbThreads = 256;
constexpr int kSbWaves = kSbThreads / kWave;
constexpr int kSbMaxParts = 1024;  // workgroups per channel; one wave merges their partial pairs

// ===================================================================== entry-wise
struct EsbArgs {
  int64_t h, w;
  const float* x;
  const float* dy;
  float* out;  // y or dx
  int64_t ldx, lddy, ldo;
  const float* weights;  // (h x 2): scale, bias
  int64_t ld_weights;
  float* wgrad;  // (h x 2)
  int64_t ld_wgrad;
  float2* part;  // [slabs][h] partial (da, db) when the columns are cut into slabs
  int64_t slab_width;
  int64_t cs;  // CH kernels: rows per channel; the pair of row r is weights[r / cs]
};

template <int GW>
using EsbPos = RowTilePos<GW>;

// CH: one (scale, bias) pair per channel of a.cs rows instead of one per row (channel-wise
// scale/bias on channels too small for the channel walk further down).
// ST: inputs through streaming loads (calls that move more than the last-level cache holds).
template <int GW, bool CH = false, bool ST = false>
__global__ void __launch_bounds__(kSbThreads)
esb_fwd_tile(EsbArgs a)
{
  using P = EsbPos<GW>;
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  if (r0 >= a.h) return;  // h is a multiple of 4
  const int64_t c0 = static_cast<int64_t>(blockIdx.y) * a.slab_width;
  const int64_t c1 = imin64(c0 + a.slab_width, a.w);
  float sc[4], bi[4];
  if constexpr (CH) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int64_t ch = (r0 + r) / a.cs;
      sc[r] = a.weights[ch];
      bi[r] = a.weights[ch + a.ld_weights];
    }
  }
  else {
    Vec16<float>::load(a.weights + r0, sc);
    Vec16<float>::load(a.weights + r0 + a.ld_weights, bi);
  }
  int64_t c = c0 + p.g;
  for (; c + 3 * P::kGroups < c1; c += 4 * P::kGroups) {
    float v[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (ST) Vec16<float>::load_stream(a.x + r0 + (c + j * P::kGroups) * a.ldx, v[j]);
      else Vec16<float>::load(a.x + r0 + (c + j * P::kGroups) * a.ldx, v[j]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) v[j][r] = sc[r] * v[j][r] + bi[r];
      Vec16<float>::store(a.out + r0 + (c + j * P::kGroups) * a.ldo, v[j]);
    }
  }
  for (; c < c1; c += P::kGroups) {
    float v[4];
    Vec16<float>::load(a.x + r0 + c * a.ldx, v);
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = sc[r] * v[r] + bi[r];
    Vec16<float>::store(a.out + r0 + c * a.ldo, v);
  }
}

template <int GW, bool CH = false, bool ST = false>
__global__ void __launch_bounds__(kSbThreads)
esb_bwd_tile(EsbArgs a)
{
  using P = EsbPos<GW>;
  __shared__ float lds[kSbWaves][P::kRows][2];
  const P p;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * P::kRows + 4 * p.q;
  const bool row_ok = r0 < a.h;
  const int64_t c0 = static_cast<int64_t>(blockIdx.y) * a.slab_width;
  const int64_t c1 = row_ok ? imin64(c0 + a.slab_width, a.w) : 0;
  const int64_t rr = row_ok ? r0 : 0;
  float sc[4];
  if constexpr (CH) {
#pragma unroll
    for (int r = 0; r < 4; ++r) sc[r] = a.weights[(rr + r) / a.cs];
  }
  else {
    Vec16<float>::load(a.weights + rr, sc);
  }
  float da[4] = {0.f, 0.f, 0.f, 0.f}, db[4] = {0.f, 0.f, 0.f, 0.f};
  int64_t c = c0 + p.g;
  for (; c + P::kGroups < c1; c += 2 * P::kGroups) {
    float v[2][4], g[2][4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (ST) {
        Vec16<float>::load_stream(a.x + rr + (c + j * P::kGroups) * a.ldx, v[j]);
        Vec16<float>::load_stream(a.dy + rr + (c + j * P::kGroups) * a.lddy, g[j]);
      }
      else {
        Vec16<float>::load(a.x + rr + (c + j * P::kGroups) * a.ldx, v[j]);
        Vec16<float>::load(a.dy + rr + (c + j * P::kGroups) * a.lddy, g[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float d[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        da[r] = __builtin_fmaf(v[j][r], g[j][r], da[r]);
        db[r] += g[j][r];
        d[r] = sc[r] * g[j][r];
      }
      Vec16<float>::store(a.out + rr + (c + j * P::kGroups) * a.ldo, d);
    }
  }
  for (; c < c1; c += P::kGroups) {
    float v[4], g[4], d[4];
    Vec16<float>::load(a.x + rr + c * a.ldx, v);
    Vec16<float>::load(a.dy + rr + c * a.lddy, g);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      da[r] = __builtin_fmaf(v[r], g[r], da[r]);
      db[r] += g[r];
      d[r] = sc[r] * g[r];
    }
    Vec16<float>::store(a.out + rr + c * a.ldo, d);
  }
  row_tile_merge<GW>(da, db, lds, p);
  if (p.g != 0 || !row_ok) return;
  if (!CH && gridDim.y == 1) {
    Vec16<float>::store(a.wgrad + r0, da);
    Vec16<float>::store(a.wgrad + r0 + a.ld_wgrad, db);
  }
  else {  // per-row pairs: summed over slabs (and, per channel, over rows) by a second kernel
    float2* dst = a.part + static_cast<int64_t>(blockIdx.y) * a.h + r0;
#pragma unroll
    for (int r = 0; r < 4; ++r) dst[r] = make_float2(da[r], db[r]);
  }
}

// Adds the slabs' partial pairs of every row in slab order.
__global__ void __launch_bounds__(256)
esb_merge_slabs(int64_t h, int slabs, const float2* __restrict__ part, float* __restrict__ wgrad,
                int64_t ld_wgrad)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= h) return;
  float sa = 0.f, sb = 0.f;
  for (int s = 0; s < slabs; ++s) {
    const float2 v = part[static_cast<int64_t>(s) * h + r];
    sa += v.x;
    sb += v.y;
  }
  wgrad[r] = sa;
  wgrad[r + ld_wgrad] = sb;
}

// Channel-wise weight gradients from per-row pairs: one wave per channel adds the pairs of
// its cs rows in every slab (lane-strided, then a wave sum: a fixed order).  WIDE: a whole
// workgroup per channel with four loads per thread in flight, for channels of many rows (one
// wave took 16 us over 3025 rows).
constexpr int64_t kCsbWideChannel = 256;  // rows x slabs from which a channel takes a workgroup

template <bool WIDE>
__global__ void __launch_bounds__(kSbThreads)
csb_merge_rows(int64_t C, int64_t cs, int64_t h, int slabs, const float2* __restrict__ part,
               float* __restrict__ wgrad, int64_t ld_wgrad)
{
  __shared__ float2 red[kSbWaves];
  const int64_t ch = WIDE ? static_cast<int64_t>(blockIdx.x)
                          : static_cast<int64_t>(blockIdx.x) * kSbWaves + wave_index();
  if (ch >= C) return;
  const int lane = threadIdx.x & (kWave - 1);
  constexpr int U = WIDE ? 4 : 1;
  const int64_t first = WIDE ? threadIdx.x : lane;
  const int64_t step = WIDE ? kSbThreads : kWave;
  float a[U], b[U];
#pragma unroll
  for (int u = 0; u < U; ++u) a[u] = b[u] = 0.f;
  for (int s = 0; s < slabs; ++s) {
    const float2* row = part + static_cast<int64_t>(s) * h + ch * cs;
    for (int64_t i0 = first; i0 < cs; i0 += U * step) {
      float2 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = i0 + u * step;
        v[u] = i < cs ? row[i] : make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        a[u] += v[u].x;
        b[u] += v[u].y;
      }
    }
  }
  float ta = a[0], tb = b[0];
  if (WIDE) {
    ta = (a[0] + a[U > 1 ? 1 : 0]) + (a[U > 2 ? 2 : 0] + a[U > 3 ? 3 : 0]);
    tb = (b[0] + b[U > 1 ? 1 : 0]) + (b[U > 2 ? 2 : 0] + b[U > 3 ? 3 : 0]);
  }
  ta = wave_sum(ta);
  tb = wave_sum(tb);
  if (WIDE) {
    if (lane == 0) red[wave_index()] = make_float2(ta, tb);
    __syncthreads();
    if (threadIdx.x != 0) return;
    ta = red[0].x, tb = red[0].y;
#pragma unroll
    for (int k = 1; k < kSbWaves; ++k) {
      ta += red[k].x;
      tb += red[k].y;
    }
  }
  else if (lane != 0) {
    return;
  }
  wgrad[ch] = ta;
  wgrad[ch + ld_wgrad] = tb;
}

// One thread per row, scalar and coalesced: any shape and alignment.
__global__ void __launch_bounds__(256)
esb_fwd_generic(EsbArgs a)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= a.h) return;
  const float sc = a.weights[r], bi = a.weights[r + a.ld_weights];
  const int64_t c0 = static_cast<int64_t>(blockIdx.y) * a.slab_width;
  const int64_t c1 = imin64(c0 + a.slab_width, a.w);
  // eight columns in flight per thread (a row's entries are a leading dimension apart)
  int64_t c = c0;
  for (; c + 8 <= c1; c += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = a.x[r + (c + u) * a.ldx];
#pragma unroll
    for (int u = 0; u < 8; ++u) a.out[r + (c + u) * a.ldo] = sc * v[u] + bi;
  }
  for (; c < c1; ++c) a.out[r + c * a.ldo] = sc * a.x[r + c * a.ldx] + bi;
}

__global__ void __launch_bounds__(256)
esb_bwd_generic(EsbArgs a)
{
  const int64_t r = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (r >= a.h) return;
  const float sc = a.weights[r];
  float da = 0.f, db = 0.f;
  int64_t c = 0;
  for (; c + 8 <= a.w; c += 8) {
    float g[8], v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      g[u] = a.dy[r + (c + u) * a.lddy];
      v[u] = a.x[r + (c + u) * a.ldx];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      da = __builtin_fmaf(v[u], g[u], da);
      db += g[u];
      a.out[r + (c + u) * a.ldo] = sc * g[u];
    }
  }
  for (; c < a.w; ++c) {
    const float g = a.dy[r + c * a.lddy];
    da = __builtin_fmaf(a.x[r + c * a.ldx], g, da);
    db += g;
    a.out[r + c * a.ldo] = sc * g;
  }
  a.wgrad[r] = da;
  a.wgrad[r + a.ld_wgrad] = db;
}

static bool sb_vec_ok(int64_t h, int64_t w, const void* p, int64_t ld) { return row_quads_ok(h, w, p, ld); }

static int sb_check(int64_t h, int64_t w, const int64_t* lds, int nld)
{
  if (h < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < h) return LBN_ERR_INVALID_ARGUMENT;
  if (h > (int64_t(1) << 36) || w > (int64_t(1) << 40)) return LBN_ERR_UNSUPPORTED;  // 64 rows per workgroup, gridDim.x < 2^31
  return LBN_OK;
}

// =================================================================== channel-wise
struct CsbArgs {
  int64_t cs, w;
  const float* x;
  const float* dy;
  float* out;
  int64_t ldx, lddy, ldo;
  const float* weights;  // (C x 2)
  int64_t ld_weights;
  float* wgrad;
  int64_t ld_wgrad;
  float2* part;  // [C][P]
};

template <bool VEC, int T>
__global__ void __launch_bounds__(T)
csb_fwd(CsbArgs a)
{
  const int64_t ch = blockIdx.x;
  const float sc = a.weights[ch], bi = a.weights[ch + a.ld_weights];
  const float* xc = a.x + ch * a.cs;
  float* yc = a.out + ch * a.cs;
  const int64_t seg = VEC ? a.cs / 4 : a.cs;
  const int64_t total = seg * a.w;
  const int64_t step = static_cast<int64_t>(gridDim.y) * T;
  for (int64_t j = static_cast<int64_t>(blockIdx.y) * T + threadIdx.x; j < total; j += step) {
    const unsigned ucol = static_cast<unsigned>(j) / static_cast<unsigned>(seg);  // j < 2^32 (host check)
    const int64_t col = ucol;
    const int64_t i = static_cast<unsigned>(j) - ucol * static_cast<unsigned>(seg);
    if (VEC) {
      float v[4];
      Vec16<float>::load(xc + col * a.ldx + 4 * i, v);
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = sc * v[k] + bi;
      Vec16<float>::store(yc + col * a.ldo + 4 * i, v);
    }
    else {
      yc[col * a.ldo + i] = sc * xc[col * a.ldx + i] + bi;
    }
  }
}

template <bool VEC, int T>
__global__ void __launch_bounds__(T)
csb_bwd(CsbArgs a)
{
  __shared__ float red[2 * (T / kWave)];
  const int64_t ch = blockIdx.x;
  const float sc = a.weights[ch];
  const float* xc = a.x + ch * a.cs;
  const float* gc = a.dy + ch * a.cs;
  float* dc = a.out + ch * a.cs;
  const int64_t seg = VEC ? a.cs / 4 : a.cs;
  const int64_t total = seg * a.w;
  const int64_t step = static_cast<int64_t>(gridDim.y) * T;
  float da = 0.f, db = 0.f;
  for (int64_t j = static_cast<int64_t>(blockIdx.y) * T + threadIdx.x; j < total; j += step) {
    const unsigned ucol = static_cast<unsigned>(j) / static_cast<unsigned>(seg);
    const int64_t col = ucol;
    const int64_t i = static_cast<unsigned>(j) - ucol * static_cast<unsigned>(seg);
    if (VEC) {
      float v[4], g[4], d[4];
      Vec16<float>::load(xc + col * a.ldx + 4 * i, v);
      Vec16<float>::load(gc + col * a.lddy + 4 * i, g);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        da = __builtin_fmaf(v[k], g[k], da);
        db += g[k];
        d[k] = sc * g[k];
      }
      Vec16<float>::store(dc + col * a.ldo + 4 * i, d);
    }
    else {
      const float g = gc[col * a.lddy + i];
      da = __builtin_fmaf(xc[col * a.ldx + i], g, da);
      db += g;
      dc[col * a.ldo + i] = sc * g;
    }
  }
  team_sum2<T / kWave>(da, db, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) {
    if (gridDim.y == 1) {
      a.wgrad[ch] = da;
      a.wgrad[ch + a.ld_wgrad] = db;
    }
    else {
      a.part[ch * gridDim.y + blockIdx.y] = make_float2(da, db);
    }
  }
}

__global__ void __launch_bounds__(kWave)
csb_merge_parts(int P, const float2* __restrict__ part, float* __restrict__ wgrad, int64_t ld_wgrad)
{
  const int64_t ch = blockIdx.x;
  const int lane = threadIdx.x;
  float a = 0.f, b = 0.f;
  for (int p = lane; p < P; p += kWave) {  // lane-strided, then the wave: a fixed order
    const float2 v = part[ch * P + p];
    a += v.x;
    b += v.y;
  }
  a = wave_sum(a);
  b = wave_sum(b);
  if (lane == 0) {
    wgrad[ch] = a;
    wgrad[ch + ld_wgrad] = b;
  }
}

// 256-thread workgroups per channel: about 2048 in total, each thread with at least four
// vectors.
// (three channels of a 299 x 299 image had been held to 64 workgroups each)
static int csb_parts(int64_t C, int64_t vectors_per_channel)
{
  int64_t p = ceil_div(2048, C);
  const int64_t most = ceil_div(vectors_per_channel, 4 * kSbThreads);
  if (p > most) p = most;
  if (p > kSbMaxParts) p = kSbMaxParts;
  return static_cast<int>(p < 1 ? 1 : p);
}

static int csb_check(int64_t C, int64_t cs, int64_t w, const int64_t* lds, int nld)
{
  if (C < 0 || cs < 0 || w < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (C > 0 && cs > (int64_t(1) << 40) / C) return LBN_ERR_UNSUPPORTED;
  for (int i = 0; i < nld; ++i)
    if (w > 1 && lds[i] < C * cs) return LBN_ERR_INVALID_ARGUMENT;
  if (C >= (int64_t(1) << 31) || cs * w >= (int64_t(1) << 32)) return LBN_ERR_UNSUPPORTED;
  return LBN_OK;
}

// Channels shorter than 64 entries (a few 16-byte pieces per column for the channel walk)
// or not a whole number of vectors go through the row tiling when the matrix allows it:
// 4096 x 1 x 1, w = 4096 took 666 us per step with the channel walk.
static bool csb_rows_shape(int64_t cs) { return cs % 4 != 0 || cs < 64; }

static bool csb_vec_ok(int64_t cs, int64_t w, const void* p, int64_t ld)
{
  return cs % 4 == 0 && aligned16(p) && (w <= 1 || ld % 4 == 0);
}

}  // namespace lbn

using namespace lbn;

extern "C" {

int lbn_entrywise_scale_bias_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                                     int64_t ldx, float* y, int64_t ldy, const float* weights,
                                     int64_t ld_weights)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = sb_check(height, width, lds, 2)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!x || !y || !weights || ld_weights < height) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  EsbArgs a{height, width, x, nullptr, y, ldx, 0, ldy, weights, ld_weights, nullptr, 0, nullptr, width};
  if (sb_vec_ok(height, width, x, ldx) && sb_vec_ok(height, width, y, ldy) && aligned16(weights) &&
      ld_weights % 4 == 0) {
    const RowTilePlan p = row_tile_plan(height, width);
    a.slab_width = p.slab_width;
    const dim3 grid(static_cast<unsigned>(p.tiles), static_cast<unsigned>(p.slabs));
    if (p.gw == 1) hipLaunchKernelGGL((esb_fwd_tile<1>), grid, dim3(kSbThreads), 0, st, a);
    else if (stream_call_inputs(2 * height * width * 4))
      hipLaunchKernelGGL((esb_fwd_tile<4, false, true>), grid, dim3(kSbThreads), 0, st, a);
    else hipLaunchKernelGGL((esb_fwd_tile<4>), grid, dim3(kSbThreads), 0, st, a);
    return launch_status();
  }
  const int64_t tiles = ceil_div(height, 256);
  int64_t slabs = ceil_div(1024, tiles);  // as in row_tile_plan, slabs of at least 8 columns
  if (slabs > width / 8) slabs = width / 8;
  if (slabs > kRowTileMaxSlabs) slabs = kRowTileMaxSlabs;
  a.slab_width = ceil_div(width, slabs < 1 ? 1 : slabs);
  const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(ceil_div(width, a.slab_width)));
  hipLaunchKernelGGL(esb_fwd_generic, grid, dim3(256), 0, st, a);
  return launch_status();
}

size_t lbn_entrywise_scale_bias_bwd_workspace_bytes(int64_t height, int64_t width)
{
  if (height <= 0 || width <= 0) return 0;
  const RowTilePlan p = row_tile_plan(height, width);
  return p.slabs > 1 ? static_cast<size_t>(p.slabs) * static_cast<size_t>(height) * sizeof(float2) : 0;
}

int lbn_entrywise_scale_bias_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                                     int64_t ldx, const float* dy, int64_t lddy, float* dx,
                                     int64_t lddx, const float* weights, int64_t ld_weights,
                                     float* weights_grad, int64_t ld_weights_grad, void* workspace,
                                     size_t workspace_bytes)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = sb_check(height, width, lds, 3)) return e;
  if (height == 0 || width == 0) return LBN_OK;
  if (!x || !dy || !dx || !weights || !weights_grad || ld_weights < height || ld_weights_grad < height)
    return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  EsbArgs a{height, width, x, dy, dx, ldx, lddy, lddx, weights, ld_weights, weights_grad, ld_weights_grad,
            static_cast<float2*>(workspace), width};
  if (sb_vec_ok(height, width, x, ldx) && sb_vec_ok(height, width, dy, lddy) &&
      sb_vec_ok(height, width, dx, lddx) && aligned16(weights) && aligned16(weights_grad) &&
      ld_weights_grad % 4 == 0) {
    const RowTilePlan p = row_tile_plan(height, width);
    const int slabs = p.slabs;
    a.slab_width = p.slab_width;
    if (slabs > 1 && (!workspace || !aligned16(workspace) ||
                      workspace_bytes < static_cast<size_t>(slabs) * height * sizeof(float2)))
      return LBN_ERR_WORKSPACE;
    const dim3 grid(static_cast<unsigned>(p.tiles), static_cast<unsigned>(slabs));
    if (p.gw == 1) hipLaunchKernelGGL((esb_bwd_tile<1>), grid, dim3(kSbThreads), 0, st, a);
    else if (stream_call_inputs(3 * height * width * 4))
      hipLaunchKernelGGL((esb_bwd_tile<4, false, true>), grid, dim3(kSbThreads), 0, st, a);
    else hipLaunchKernelGGL((esb_bwd_tile<4>), grid, dim3(kSbThreads), 0, st, a);
    if (slabs > 1)
      hipLaunchKernelGGL(esb_merge_slabs, dim3(static_cast<unsigned>(ceil_div(height, 256))), dim3(256), 0,
                         st, height, slabs, a.part, weights_grad, ld_weights_grad);
    return launch_status();
  }
  hipLaunchKernelGGL(esb_bwd_generic, dim3(static_cast<unsigned>(ceil_div(height, 256))), dim3(256), 0, st, a);
  return launch_status();
}

int lbn_channelwise_scale_bias_fwd_f32(lbn_stream_t stream, int64_t num_channels, int64_t channel_size,
                                       int64_t width, const float* x, int64_t ldx, float* y,
                                       int64_t ldy, const float* weights, int64_t ld_weights)
{
  const int64_t lds[2] = {ldx, ldy};
  if (int e = csb_check(num_channels, channel_size, width, lds, 2)) return e;
  if (num_channels == 0 || channel_size == 0 || width == 0) return LBN_OK;
  if (!x || !y || !weights || ld_weights < num_channels) return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  const int64_t height = num_channels * channel_size;
  if (csb_rows_shape(channel_size) && row_quads_ok(height, width, x, ldx) && row_quads_ok(height, width, y, ldy)) {
    const RowTilePlan p = row_tile_plan(height, width);
    EsbArgs e{height, width, x, nullptr, y, ldx, 0, ldy, weights, ld_weights, nullptr, 0, nullptr, p.slab_width,
              channel_size};
    const dim3 grid(static_cast<unsigned>(p.tiles), static_cast<unsigned>(p.slabs));
    if (p.gw == 1) hipLaunchKernelGGL((esb_fwd_tile<1, true>), grid, dim3(kSbThreads), 0, st, e);
    else hipLaunchKernelGGL((esb_fwd_tile<4, true>), grid, dim3(kSbThreads), 0, st, e);
    return launch_status();
  }
  const CsbArgs a{channel_size, width, x, nullptr, y, ldx, 0, ldy, weights, ld_weights, nullptr, 0, nullptr};
  const bool vec = csb_vec_ok(channel_size, width, x, ldx) && csb_vec_ok(channel_size, width, y, ldy);
  const int64_t units = (vec ? channel_size / 4 : channel_size) * width;
  // one 1024-thread workgroup per channel once there are enough channels to fill the device:
  // measured 64.8 us against 69.7 us for eight 256-thread workgroups per channel (256 x 3136 x 64)
  const bool big = units >= 4 * 1024 && num_channels >= 256;
  const int P = big ? 1 : csb_parts(num_channels, units);
  const dim3 grid(static_cast<unsigned>(num_channels), static_cast<unsigned>(P));
  if (vec && big) hipLaunchKernelGGL((csb_fwd<true, 1024>), grid, dim3(1024), 0, st, a);
  else if (vec) hipLaunchKernelGGL((csb_fwd<true, kSbThreads>), grid, dim3(kSbThreads), 0, st, a);
  else if (big) hipLaunchKernelGGL((csb_fwd<false, 1024>), grid, dim3(1024), 0, st, a);
  else hipLaunchKernelGGL((csb_fwd<false, kSbThreads>), grid, dim3(kSbThreads), 0, st, a);
  return launch_status();
}

size_t lbn_channelwise_scale_bias_bwd_workspace_bytes(int64_t num_channels, int64_t channel_size,
                                                      int64_t width)
{
  if (num_channels <= 0 || channel_size <= 0 || width <= 0) return 0;
  // at most ceil(2048 / channels) workgroups per channel (csb_parts)
  const int64_t parts = ceil_div(2048, num_channels) < kSbMaxParts ? ceil_div(2048, num_channels) : kSbMaxParts;
  size_t need = static_cast<size_t>(num_channels) * parts * sizeof(float2);
  const int64_t height = num_channels * channel_size;
  if (csb_rows_shape(channel_size) && height % 4 == 0) {  // per-row pairs of the row tiling
    const size_t rows = static_cast<size_t>(row_tile_plan(height, width).slabs) * height * sizeof(float2);
    if (rows > need) need = rows;
  }
  return need;
}

int lbn_channelwise_scale_bias_bwd_f32(lbn_stream_t stream, int64_t num_channels, int64_t channel_size,
                                       int64_t width, const float* x, int64_t ldx, const float* dy,
                                       int64_t lddy, float* dx, int64_t lddx, const float* weights,
                                       int64_t ld_weights, float* weights_grad, int64_t ld_weights_grad,
                                       void* workspace, size_t workspace_bytes)
{
  const int64_t lds[3] = {ldx, lddy, lddx};
  if (int e = csb_check(num_channels, channel_size, width, lds, 3)) return e;
  if (num_channels == 0 || channel_size == 0 || width == 0) return LBN_OK;
  if (!x || !dy || !dx || !weights || !weights_grad || ld_weights < num_channels ||
      ld_weights_grad < num_channels)
    return LBN_ERR_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  const int64_t height = num_channels * channel_size;
  if (csb_rows_shape(channel_size) && row_quads_ok(height, width, x, ldx) &&
      row_quads_ok(height, width, dy, lddy) && row_quads_ok(height, width, dx, lddx)) {
    const RowTilePlan p = row_tile_plan(height, width);
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 7u) ||
        workspace_bytes < static_cast<size_t>(p.slabs) * height * sizeof(float2))
      return LBN_ERR_WORKSPACE;
    EsbArgs e{height, width, x, dy, dx, ldx, lddy, lddx, weights, ld_weights, nullptr, 0,
              static_cast<float2*>(workspace), p.slab_width, channel_size};
    const dim3 grid(static_cast<unsigned>(p.tiles), static_cast<unsigned>(p.slabs));
    if (p.gw == 1) hipLaunchKernelGGL((esb_bwd_tile<1, true>), grid, dim3(kSbThreads), 0, st, e);
    else hipLaunchKernelGGL((esb_bwd_tile<4, true>), grid, dim3(kSbThreads), 0, st, e);
    if (channel_size * p.slabs >= kCsbWideChannel)
      hipLaunchKernelGGL(csb_merge_rows<true>, dim3(static_cast<unsigned>(num_channels)), dim3(kSbThreads), 0, st,
                         num_channels, channel_size, height, p.slabs, e.part, weights_grad, ld_weights_grad);
    else
      hipLaunchKernelGGL(csb_merge_rows<false>, dim3(static_cast<unsigned>(ceil_div(num_channels, kSbWaves))),
                         dim3(kSbThreads), 0, st, num_channels, channel_size, height, p.slabs, e.part, weights_grad,
                         ld_weights_grad);
    return launch_status();
  }
  const bool vec = csb_vec_ok(channel_size, width, x, ldx) && csb_vec_ok(channel_size, width, dy, lddy) &&
                   csb_vec_ok(channel_size, width, dx, lddx);
  const int64_t units = (vec ? channel_size / 4 : channel_size) * width;
  // 1024-thread workgroups when that fills the device with one workgroup per channel: no
  // partial sums to merge, so no second kernel
  const bool big = units >= 4 * 1024 && num_channels >= 256;
  const int P = big ? 1 : csb_parts(num_channels, units);
  if (P > 1 && (!workspace || workspace_bytes < static_cast<size_t>(num_channels) * P * sizeof(float2) ||
                (reinterpret_cast<uintptr_t>(workspace) & 7u)))
    return LBN_ERR_WORKSPACE;
  const CsbArgs a{channel_size, width, x, dy, dx, ldx, lddy, lddx, weights, ld_weights, weights_grad,
                  ld_weights_grad, static_cast<float2*>(workspace)};
  const dim3 grid(static_cast<unsigned>(num_channels), static_cast<unsigned>(P));
  if (vec && big) hipLaunchKernelGGL((csb_bwd<true, 1024>), grid, dim3(1024), 0, st, a);
  else if (vec) hipLaunchKernelGGL((csb_bwd<true, kSbThreads>), grid, dim3(kSbThreads), 0, st, a);
  else if (big) hipLaunchKernelGGL((csb_bwd<false, 1024>), grid, dim3(1024), 0, st, a);
  else hipLaunchKernelGGL((csb_bwd<false, kSbThreads>), grid, dim3(kSbThreads), 0, st, a);
  if (P > 1)
    hipLaunchKernelGGL(csb_merge_parts, dim3(static_cast<unsigned>(num_channels)), dim3(kWave), 0, st, P,
                       a.part, weights_grad, ld_weights_grad);
  return launch_status();
}

}  // extern "C"
