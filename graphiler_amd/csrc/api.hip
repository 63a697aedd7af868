// Version and error text of the C ABI.
#include "common.h"

extern "C" {

int ga_version(void) { return 100; }

const char *ga_error_string(int code) {
  switch (code) {
    case GA_OK: return "ok";
    case GA_EINVAL: return "invalid argument (null pointer, negative or inconsistent size)";
    case GA_EUNSUPPORTED: return "request not supported by this build";
    case GA_EWORKSPACE: return "workspace missing, too small or not 16-byte aligned";
    case GA_EALIGN: return "pointer not aligned to its element size";
    case GA_ESCRATCH: return "problem needs more partial rows than the library's static scratch buffer holds";
    default:
      return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error code";
  }
}

}  // extern "C"
