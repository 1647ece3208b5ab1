// Status strings and the thread-local error slot.
#include "common.hpp"

namespace sarek_hip {

std::string &last_error_slot() {
  thread_local std::string slot;
  return slot;
}

int fail(int status, const char *fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error_slot() = buf;
  return status;
}

}  // namespace sarek_hip

extern "C" {

int sarek_hip_abi_version(void) { return SAREK_HIP_ABI_VERSION; }

const char *sarek_hip_last_error(void) { return sarek_hip::last_error_slot().c_str(); }

const char *sarek_hip_status_name(int status) {
  switch (status) {
    case SAREK_HIP_OK: return "SAREK_HIP_OK";
    case SAREK_HIP_E_INVALID_ARG: return "SAREK_HIP_E_INVALID_ARG";
    case SAREK_HIP_E_UNSUPPORTED: return "SAREK_HIP_E_UNSUPPORTED";
    case SAREK_HIP_E_COMPILE: return "SAREK_HIP_E_COMPILE";
    case SAREK_HIP_E_NO_DEVICE: return "SAREK_HIP_E_NO_DEVICE";
    case SAREK_HIP_E_WORKSPACE: return "SAREK_HIP_E_WORKSPACE";
    case SAREK_HIP_E_PARSE: return "SAREK_HIP_E_PARSE";
    case SAREK_HIP_E_CODEGEN: return "SAREK_HIP_E_CODEGEN";
    case SAREK_HIP_E_BUFFER_TOO_SMALL: return "SAREK_HIP_E_BUFFER_TOO_SMALL";
    default: break;
  }
  if (status >= 1000) return "HIPRTC_ERROR";
  if (status > 0) return hipGetErrorName(static_cast<hipError_t>(status));
  return "SAREK_HIP_E_UNKNOWN";
}
}
