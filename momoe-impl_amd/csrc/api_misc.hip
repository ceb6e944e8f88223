// Version and status strings of the C ABI.
#include "common.hpp"

extern "C" int momoe_abi_version(void) { return 1; }

extern "C" const char* momoe_status_string(int status) {
  switch (status) {
    case MOMOE_OK: return "ok";
    case MOMOE_ERR_BAD_ARG: return "bad argument (null/misaligned pointer or non-positive size)";
    case MOMOE_ERR_UNSUPPORTED: return "unsupported shape";
    case MOMOE_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}
