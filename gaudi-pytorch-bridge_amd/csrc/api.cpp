// Entry points of the C ABI that launch nothing.
#include "../../include/mi355q.h"

extern "C" {

int mi355q_abi_version(void) { return 7; }

const char* mi355q_status_string(int status) {
  switch (status) {
    case MI355Q_OK: return "ok";
    case MI355Q_ERR_INVALID_ARGUMENT: return "invalid argument";
    case MI355Q_ERR_UNSUPPORTED: return "unsupported problem (shape, alignment or size)";
    case MI355Q_ERR_LAUNCH: return "kernel launch failed";
    case MI355Q_ERR_WORKSPACE: return "workspace missing or too small";
    case MI355Q_ERR_TOO_LARGE: return "problem needs more scratch memory than the allocation-free entry point holds";
    default: return "unknown status";
  }
}

}  // extern "C"
