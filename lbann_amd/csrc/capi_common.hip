// Entry points that belong to no single layer: version and status strings.
#include <hip/hip_runtime.h>

#include "../../include/lbnorm.h"

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

}  // extern "C"
