// ABI bookkeeping shared by all launchers: version, status text, last HIP error.
#include "mops_common.h"

namespace mops {
static thread_local int g_last_hip_error = 0;
int finish_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return MOPS_HIP_ELAUNCH;
  }
  return MOPS_HIP_OK;
}
int record_hip_error(hipError_t e) {
  g_last_hip_error = (int)e;
  return MOPS_HIP_ELAUNCH;
}
}  // namespace mops

extern "C" int mops_hip_abi_version(void) { return 9; }

extern "C" int mops_hip_last_hip_error(void) { return mops::g_last_hip_error; }

extern "C" const char* mops_hip_status_string(int status) {
  switch (status) {
    case MOPS_HIP_OK: return "ok";
    case MOPS_HIP_EINVAL: return "invalid argument (null pointer, negative size or inconsistent sizes)";
    case MOPS_HIP_EUNSUPPORTED: return "unsupported shape for the gfx950 kernels";
    case MOPS_HIP_EALIGN: return "pointer or stride is not 16-byte aligned";
    case MOPS_HIP_EWORKSPACE: return "workspace missing or too small";
    case MOPS_HIP_ELAUNCH: return "HIP runtime call or kernel launch failed";
    case MOPS_HIP_ETOOLARGE: return "problem needs more scratch than the allocation-free entry point holds";
    default: return "unknown status";
  }
}
