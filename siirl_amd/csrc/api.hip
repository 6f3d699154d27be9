// Error reporting and version query of the C ABI.
#include "common.hpp"

#include <mutex>
#include <set>
#include <string>
#include <utility>

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

int allow_dynamic_lds(const void* kernel, int bytes) {
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> done;  // (kernel, device) pairs already raised
  int dev = 0;
  SIIRL_HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  if (done.count({kernel, dev})) return SIIRL_OK;
  SIIRL_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  done.insert({kernel, dev});
  return SIIRL_OK;
}

}  // namespace siirl

extern "C" int siirl_hip_abi_version(void) { return SIIRL_HIP_ABI_VERSION; }

extern "C" const char* siirl_hip_last_error(void) { return siirl::g_last_error.c_str(); }
