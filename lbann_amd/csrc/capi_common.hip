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
