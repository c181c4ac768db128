// Entry points that belong to no single layer: version, status strings, diagnostics.
#include <hip/hip_runtime.h>

#include "../../include/lbnorm.h"
#include "cluster_sync.hpp"

namespace lbn {

// The designed exit of a wait that cannot be satisfied: one workgroup acts as member 0 of a
// cluster of two, publishes its pair and polls for member 1, which is never launched.  After
// `max_polls` rounds the wait gives up, raises the workspace's error word and the kernel ends
// like any other.
static __global__ void __launch_bounds__(kWave)
cluster_wait_gives_up(ClusterWorkspace cw, ClusterTag tag, int max_polls, float* out)
{
  cluster_resolve_tag(tag);
  if (threadIdx.x == 0) cluster_publish(1.f, 2.f, cw.slots, 0, tag);
  float a, b;
  cluster_collect(cw.slots, 2, tag, cw.error, -1.f, -1.f, a, b, max_polls);
  if (threadIdx.x < 2) {  // member 0's own pair, and the stand-in values of the absent member 1
    out[2 * threadIdx.x] = a;
    out[2 * threadIdx.x + 1] = b;
  }
}

// A copy with the register pipeline of the batch-norm cluster kernels (three tiles of V 16-byte
// vectors per thread in rotation, persistent workgroups, non-temporal stores) and nothing else: no
// arithmetic, no exchange between workgroups.  CHANNEL_MAJOR walks the matrix in the order of those
// kernels (a cluster of M workgroups takes channel after channel, member m its m-th share of the
// channel's w segments); otherwise workgroup b takes the contiguous tiles b, b + grid, ...
// What this reaches is what the memory system gives that order of accesses.
struct CopyPipelineArgs {
  const float* x;
  float* y;
  int64_t ldx, ldy;
  int64_t channels;
  unsigned cs4;     // 16-byte vectors per channel segment
  unsigned w;
  unsigned share4;  // vectors of a channel per member
  int M;
  int64_t tiles;    // contiguous order: tiles of kCopyThreads * kCopyVectors vectors (height * w / 4 in all)
  int64_t h4;       // vectors per column
};

constexpr int kCopyThreads = 512;
constexpr int kCopyVectors = 4;

template <bool CHANNEL_MAJOR>
static __global__ void __launch_bounds__(kCopyThreads)
selftest_copy_pipeline(CopyPipelineArgs a)
{
  typedef float v4f __attribute__((ext_vector_type(4)));
  constexpr int V = kCopyVectors;
  constexpr int T = kCopyThreads;
  v4f t[3][V];
  int64_t from[3][V], to[3][V];
  const int64_t g = gridDim.x;
  const int ncl = CHANNEL_MAJOR ? static_cast<int>(g) / a.M : 1;
  const int64_t rounds = CHANNEL_MAJOR ? (a.channels + ncl - 1) / ncl : (a.tiles + g - 1) / g;
  // vector i of round r of this workgroup: offsets into x and y in floats, or -1
  auto locate = [&](int64_t r, int i, int64_t& src, int64_t& dst) {
    src = dst = -1;
    if (r >= rounds) return;
    int64_t col, row4;
    if (CHANNEL_MAJOR) {
      const int cl = blockIdx.x / a.M, m = blockIdx.x - cl * a.M;
      const int64_t c = r * ncl + cl;
      const unsigned e = m * a.share4 + threadIdx.x + i * T;
      if (c >= a.channels || threadIdx.x + i * T >= a.share4 || e >= a.w * a.cs4) return;
      col = e / a.cs4;
      row4 = c * a.cs4 + (e - static_cast<unsigned>(col) * a.cs4);
    }
    else {
      const int64_t v = (r * g + blockIdx.x) * (T * V) + threadIdx.x + i * T;
      if (v >= a.h4 * a.w) return;
      col = v / a.h4;
      row4 = v - col * a.h4;
    }
    src = 4 * row4 + col * a.ldx;
    dst = 4 * row4 + col * a.ldy;
  };
  auto load = [&](int slot, int64_t r) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      locate(r, i, from[slot][i], to[slot][i]);
      if (from[slot][i] >= 0) t[slot][i] = *reinterpret_cast<const v4f*>(a.x + from[slot][i]);
    }
  };
  auto store = [&](int slot) {
#pragma unroll
    for (int i = 0; i < V; ++i)
      if (to[slot][i] >= 0) __builtin_nontemporal_store(t[slot][i], reinterpret_cast<v4f*>(a.y + to[slot][i]));
  };
  load(0, 0);
  load(1, 1);
  for (int64_t r = 0; r < rounds; r += 3) {
    load(2, r + 2);
    store(0);
    if (r + 1 < rounds) {
      load(0, r + 3);
      store(1);
    }
    if (r + 2 < rounds) {
      load(1, r + 4);
      store(2);
    }
  }
}

}  // namespace lbn

extern "C" {

int lbn_version(void) { return 100; }  // major*10000 + minor*100 + patch

const char* lbn_status_string(int status)
{
  switch (status) {
  case LBN_OK: return "ok";
  case LBN_ERR_INVALID_ARGUMENT: return "invalid argument (negative size, leading dimension below height, or NULL matrix)";
  case LBN_ERR_WORKSPACE: return "workspace missing, misaligned or smaller than *_workspace_bytes()";
  case LBN_ERR_UNSUPPORTED: return "shape outside the supported index range";
  default: break;
  }
  if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
  return "unknown status";
}

int lbn_selftest_copy_pipeline_f32(lbn_stream_t stream, int64_t num_channels, int64_t channel_size, int64_t width,
                                   const float* x, int64_t ldx, float* y, int64_t ldy, int channel_major)
{
  using namespace lbn;
  if (num_channels < 0 || channel_size < 0 || width < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (num_channels == 0 || channel_size == 0 || width == 0) return LBN_OK;
  const int64_t height = num_channels * channel_size;
  if (!x || !y || (width > 1 && (ldx < height || ldy < height))) return LBN_ERR_INVALID_ARGUMENT;
  // whole 16-byte vectors everywhere, 32-bit vector indices inside a channel
  if (channel_size % 4 || !aligned16(x) || !aligned16(y) || (width > 1 && (ldx % 4 || ldy % 4)) ||
      channel_size / 4 * width >= (int64_t(1) << 31))
    return LBN_ERR_UNSUPPORTED;
  hipStream_t st = as_stream(stream);
  CopyPipelineArgs a{};
  a.x = x, a.y = y, a.ldx = ldx, a.ldy = ldy, a.channels = num_channels;
  a.cs4 = static_cast<unsigned>(channel_size / 4), a.w = static_cast<unsigned>(width), a.h4 = height / 4;
  constexpr int64_t kTile = int64_t(kCopyThreads) * kCopyVectors;
  const int64_t resident = 512;  // two workgroups of 512 threads on each of 256 compute units
  if (channel_major) {
    const int64_t channel4 = static_cast<int64_t>(a.cs4) * a.w;
    const int64_t M = ceil_div(channel4, kTile);
    if (M > resident) return LBN_ERR_UNSUPPORTED;
    a.M = static_cast<int>(M);
    a.share4 = static_cast<unsigned>(ceil_div(channel4, M));
    int64_t ncl = resident / M;
    if (ncl > num_channels) ncl = num_channels;
    hipLaunchKernelGGL((selftest_copy_pipeline<true>), dim3(static_cast<unsigned>(ncl * M)), dim3(kCopyThreads), 0, st, a);
  }
  else {
    a.tiles = ceil_div(a.h4 * a.w, kTile);
    const int64_t grid = a.tiles < resident ? a.tiles : resident;
    hipLaunchKernelGGL((selftest_copy_pipeline<false>), dim3(static_cast<unsigned>(grid)), dim3(kCopyThreads), 0, st, a);
  }
  return launch_status();
}

int lbn_workspace_timed_out(lbn_stream_t stream, const void* workspace, int* timed_out)
{
  if (!timed_out) return LBN_ERR_INVALID_ARGUMENT;
  *timed_out = 0;
  if (!workspace) return LBN_OK;  // shapes that need no workspace have no cross-workgroup wait
  int word = 0;
  hipStream_t st = lbn::as_stream(stream);
  hipError_t e = hipMemcpyAsync(&word, workspace, sizeof(int), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return static_cast<int>(e);
  *timed_out = word == lbn::kClusterTimedOut ? 1 : 0;
  return LBN_OK;
}

int lbn_selftest_cluster_wait_gives_up(lbn_stream_t stream, void* workspace, size_t workspace_bytes,
                                       int max_polls, float* out4)
{
  if (!out4 || max_polls < 1 || max_polls > (1 << 16)) return LBN_ERR_INVALID_ARGUMENT;
  if (!workspace) {  // the library-owned array of the entry point that allocates nothing
    const int status = lbn::static_scratch_address(&workspace);
    if (status != LBN_OK) return status;
    workspace_bytes = lbn::static_scratch_bytes();
  }
  if (workspace_bytes < lbn::cluster_workspace_bytes(1, 2) || !lbn::aligned16(workspace)) return LBN_ERR_WORKSPACE;
  hipStream_t st = lbn::as_stream(stream);
  const lbn::ClusterWorkspace cw = lbn::cluster_workspace(workspace);
  hipLaunchKernelGGL(lbn::cluster_wait_gives_up, dim3(1), dim3(lbn::kWave), 0, st, cw, lbn::cluster_call_tag(st, cw),
                     max_polls, out4);
  return lbn::launch_status();
}

}  // extern "C"
