// The library's small host-side state: the per-thread error message.
#include "pyre_api.h"
#include "pyre_common.h"

namespace pyre {
char* error_buffer() {
  static thread_local char buf[512] = "";
  return buf;
}
}  // namespace pyre

extern "C" const char* pyre_last_error() { return pyre::error_buffer(); }
extern "C" int pyre_abi_version() { return 1; }
