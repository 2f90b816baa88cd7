// Library identity and error text of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "common.hpp"

namespace aamd {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  set_error("%s: HIP error %d (%s)", what, (int)e, hipGetErrorString(e));
  return AAMD_ERR_HIP;
}

}  // namespace aamd

extern "C" int aamd_abi_version(void) { return AAMD_ABI_VERSION; }
extern "C" const char* aamd_last_error(void) { return aamd::g_err; }
