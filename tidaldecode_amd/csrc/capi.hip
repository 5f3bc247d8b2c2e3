// Library-wide state of libtidal_hip.so: error buffer and version.
#include "common.cuh"

namespace tidal {
char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace tidal

extern "C" const char* td_last_error(void) { return tidal::error_buffer(); }
extern "C" int td_version(void) { return 6; }
