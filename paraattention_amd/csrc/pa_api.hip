// Library-wide pieces of the C ABI: version and per-thread error text.
#include "pa_common.h"

namespace pa {
char* error_slot() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace pa

extern "C" int pa_abi_version(void) { return 4; }

extern "C" const char* pa_last_error(void) { return pa::error_slot(); }
