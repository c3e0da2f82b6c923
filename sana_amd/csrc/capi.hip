// Entry points that are not tied to one kernel family.
#include "common.h"

extern "C" __attribute__((visibility("default"))) int sana_hip_abi_version(void) { return SANA_HIP_ABI_VERSION; }

extern "C" __attribute__((visibility("default"))) const char* sana_hip_strerror(int code) {
  switch (code) {
    case SANA_OK: return "ok";
    case SANA_ERR_ARG: return "invalid argument (null pointer, non-positive size or unknown enum)";
    case SANA_ERR_SHAPE: return "shape not supported by the gfx950 kernels";
    case SANA_ERR_ALIGN: return "pointer or stride is not 16-byte aligned";
    case SANA_ERR_WORKSPACE: return "workspace missing or too small";
    case SANA_ERR_LAUNCH: return "kernel launch failed";
    case SANA_ERR_DTYPE: return "dtype not supported by this entry point";
    case SANA_ERR_SCRATCH_LIMIT: return "problem needs more scratch than the library's fixed array holds (use the workspace entry point)";
    case SANA_ERR_RUNTIME: return "HIP runtime call failed (no current device, or the scratch symbol could not be resolved)";
    default: return "unknown error code";
  }
}
