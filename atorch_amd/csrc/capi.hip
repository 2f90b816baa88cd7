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

namespace aamd {
// One wavefront: spins until the shader cycle counter has advanced by min_cycles (the iteration
// bound ends the loop even if the counter stood still).
__global__ void clock_probe_kernel(unsigned long long* out, long long min_cycles) {
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  unsigned long long c1 = c0;
  for (long long it = 0; it < min_cycles && (long long)(c1 - c0) < min_cycles; it++) {
    __builtin_amdgcn_s_sleep(8);
    c1 = __builtin_readcyclecounter();
  }
  const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) {
    out[0] = c1 - c0;
    out[1] = r1 - r0;
  }
}
}  // namespace aamd

extern "C" int aamd_clock_probe(uint64_t* out, int64_t min_cycles, void* stream) {
  AAMD_REQUIRE(out != nullptr, "clock_probe: null pointer");
  AAMD_REQUIRE(min_cycles >= 0 && min_cycles <= (1LL << 31), "clock_probe: min_cycles out of range");
  aamd::clock_probe_kernel<<<1, 64, 0, (hipStream_t)stream>>>(reinterpret_cast<unsigned long long*>(out), min_cycles);
  AAMD_LAUNCH_CHECK("clock_probe");
  return AAMD_OK;
}
