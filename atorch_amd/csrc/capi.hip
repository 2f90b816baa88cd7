// Library identity and error text of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "common.hpp"
#ifdef AAMD_TUNING
#include "../../include/atorch_amd_probes.h"
#endif

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

#ifndef AAMD_TUNING
extern "C" int aamd_abi_version(void) { return AAMD_ABI_VERSION; }
extern "C" const char* aamd_last_error(void) { return aamd::g_err; }
#else  // the measurement library keeps its own error text
extern "C" const char* aamd_probes_last_error(void) { return aamd::g_err; }
#endif
