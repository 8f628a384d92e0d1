// ABI version and error strings.
#include "common.h"

extern "C" {

int gptq_hip_abi_version(void) { return GPTQ_HIP_ABI_VERSION; }

const char *gptq_hip_error_string(int code) {
  switch (code) {
    case GPTQ_HIP_OK: return "ok";
    case GPTQ_HIP_EINVAL: return "invalid argument (shape, pointer or block size)";
    case GPTQ_HIP_EDTYPE: return "unsupported element type";
    case GPTQ_HIP_EWORKSPACE: return "workspace missing or too small";
    case GPTQ_HIP_ELAUNCH: return "HIP launch failed";
    case GPTQ_HIP_ETOOBIG: return "problem needs more scratch than the call that allocates nothing holds";
    default: return "unknown error";
  }
}

}  // extern "C"
