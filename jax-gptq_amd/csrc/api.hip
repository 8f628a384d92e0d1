// ABI version and error strings.
#include "common.h"

#include <map>
#include <mutex>
#include <utility>

bool gptq_raise_lds_limit(const void *kernel, int bytes) {
  static std::mutex mu;
  static std::map<std::pair<int, const void *>, int> raised;      // (device, kernel) -> limit set
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  std::lock_guard<std::mutex> lock(mu);
  auto it = raised.find({dev, kernel});
  if (it != raised.end() && it->second >= bytes) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  raised[{dev, kernel}] = bytes;
  return true;
}

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
