// Library-level entry points of libhalo_moe: ABI version and status names.
#include "common.h"

extern "C" {

int hmoe_abi_version(void) { return 1; }

const char* hmoe_status_string(int status) {
  switch (status) {
    case HMOE_OK: return "ok";
    case HMOE_INVALID_ARGUMENT: return "invalid argument (null pointer, negative size or unknown enum)";
    case HMOE_UNSUPPORTED: return "unsupported shape, alignment or dtype";
    case HMOE_LAUNCH_FAILED: return "kernel launch failed";
    default: return "unknown status";
  }
}

}  // extern "C"
