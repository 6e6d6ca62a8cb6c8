// Library-level entry points: version and the thread-local error message.
#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

std::string& last_error() {
  static thread_local std::string msg;
  return msg;
}

int fail_arg(const char* fn, const char* what) {
  last_error() = std::string(fn) + ": " + what;
  return SPX_ERR_ARG;
}

int check_launch(const char* fn) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return SPX_OK;
  last_error() = std::string(fn) + ": " + hipGetErrorString(e);
  return SPX_ERR_HIP;
}

}  // namespace spx

extern "C" int spx_version(void) { return 100; }

extern "C" const char* spx_last_error(void) { return spx::last_error().c_str(); }
