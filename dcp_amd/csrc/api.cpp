// Version and error-string entry points of libdcp_hip.so.
#include "common.h"

namespace dcp {
char* last_error_buffer() {
  static thread_local char buffer[512] = {0};
  return buffer;
}
}  // namespace dcp

extern "C" int dcp_version(void) { return 100; }

extern "C" const char* dcp_last_error(void) { return dcp::last_error_buffer(); }
