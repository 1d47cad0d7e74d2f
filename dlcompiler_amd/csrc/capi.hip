// Version and status helpers of the C ABI.
#include "common.h"

extern "C" int dlb_version(void) { return DLB_ABI_VERSION; }

extern "C" const char* dlb_status_string(int status) {
  switch (status) {
    case DLB_OK:
      return "ok";
    case DLB_ERR_BAD_ARG:
      return "bad argument (null pointer, negative size or inconsistent shapes)";
    case DLB_ERR_UNSUPPORTED:
      return "unsupported shape or dtype";
    case DLB_ERR_LAUNCH:
      return "kernel launch failed";
    case DLB_ERR_WORKSPACE:
      return "workspace missing or too small";
    default:
      return "unknown status";
  }
}
