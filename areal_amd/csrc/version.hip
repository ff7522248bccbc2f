// Library identification for the C ABI.
#include "../../include/areal_amd.h"

extern "C" int aa_version(void) { return 100; /* 0.1.0 */ }

extern "C" const char* aa_status_string(int status) {
  switch (status) {
    case AA_OK: return "ok";
    case AA_ERR_INVALID_ARGUMENT: return "invalid argument";
    case AA_ERR_UNSUPPORTED: return "unsupported configuration";
    case AA_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}
