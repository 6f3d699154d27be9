// Error reporting and version query of the C ABI.
#include "common.hpp"

#include <string>

namespace siirl {

static thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

}  // namespace siirl

extern "C" int siirl_hip_abi_version(void) { return 1000; }

extern "C" const char* siirl_hip_last_error(void) { return siirl::g_last_error.c_str(); }
