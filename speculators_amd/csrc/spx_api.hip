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

int ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* fn) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    last_error() = std::string(fn) + ": hipGetDevice: " + hipGetErrorString(e);
    return SPX_ERR_HIP;
  }
  const uint64_t bit = (dev >= 0 && dev < 64) ? (1ull << dev) : 0;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return SPX_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    last_error() = std::string(fn) + ": hipFuncSetAttribute: " + hipGetErrorString(e);
    return SPX_ERR_HIP;
  }
  if (bit) done.fetch_or(bit, std::memory_order_release);
  return SPX_OK;
}

}  // namespace spx

extern "C" int spx_version(void) { return 112; }

extern "C" const char* spx_last_error(void) { return spx::last_error().c_str(); }
