// Entry points that belong to no single layer: version, status strings, diagnostics.
#include <hip/hip_runtime.h>

#include "../../include/lbnorm.h"
#include "cluster_sync.hpp"

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

}  // extern "C"
