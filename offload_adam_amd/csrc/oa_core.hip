// Version and error-text entry points of liboffload_adam_hip.so.
#include "oa_common.hpp"

extern "C" int oa_abi_version(void) { return OA_ABI_VERSION; }

extern "C" const char* oa_error_string(int code) {
  switch (code) {
    case 0:
      return "success";
    case OA_EINVAL:
      return "offload_adam_hip: invalid argument (null pointer, negative size or bad enum)";
    case OA_EALIGN:
      return "offload_adam_hip: pointer is not aligned to its element type";
    case OA_ERANGE:
      return "offload_adam_hip: size is beyond what this entry point supports";
    case OA_EOVERLAP:
      return "offload_adam_hip: buffers that must be distinct alias each other";
    case OA_EOS:
      return "offload_adam_hip: an operating-system call failed (see os_errno)";
    case OA_EUNAVAILABLE:
      return "offload_adam_hip: fixed-engine copies are not available on this GPU";
    case OA_ELINKTIMEOUT:
      return "offload_adam_hip: an earlier fixed-engine copy did not complete within its time limit";
    case OA_LINK_OFF:
      return "offload_adam_hip: fixed-engine copies switched off (OFFLOAD_ADAM_COPY_ENGINES)";
    case OA_LINK_NO_RUNTIME:
      return "offload_adam_hip: the ROCr runtime library or one of its entry points was not found";
    case OA_LINK_NO_AGENT:
      return "offload_adam_hip: the HIP device was not found among the HSA agents";
    case OA_LINK_NO_SIGNALS:
      return "offload_adam_hip: signal memory could not be obtained or verified";
    default:
      break;
  }
  if (code > 0) {
    const char* s = hipGetErrorString(static_cast<hipError_t>(code));
    return s ? s : "offload_adam_hip: unknown HIP error";
  }
  return "offload_adam_hip: unknown error code";
}
