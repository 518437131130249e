// ABI handshake and per-thread error text of the nestedtensor_amd library.
#include "nt_common.h"

namespace nt {
char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace nt

extern "C" int nt_abi_version(void) { return NT_ABI_VERSION; }

extern "C" const char* nt_last_error(void) { return nt::error_buffer(); }
