// Library identification and status strings.
#include "mx_common.h"

extern "C" int mx_version(void) { return 101; }

extern "C" const char* mx_status_string(int status) {
  switch (status) {
    case MX_OK: return "ok";
    case MX_ERR_INVALID_ARG: return "invalid argument";
    case MX_ERR_ALIGNMENT: return "dimension or pointer not aligned to what the kernel needs";
    case MX_ERR_LAUNCH: return "kernel launch failed";
    case MX_ERR_UNSUPPORTED: return "shape not supported";
    case MX_ERR_SCRATCH_TOO_SMALL:
      return "the split of this shape needs more than the library's built-in scratch array holds";
    default: return "unknown status";
  }
}
