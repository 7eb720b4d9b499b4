// Error channel of the kernel library: every entry point returns 0 on success
// and non-zero after storing a message that he_last_error() hands back.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"
#include "hector_kernels.h"

static thread_local char g_error[1024] = "";

void he_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int he_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    he_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

extern "C" const char* he_last_error(void) { return g_error; }

// Compute units of the current device, asked once per device and process. The grids of the
// products and of the attention kernels count in them; HE_CUS (the MI355X's 256, at which the
// rules were measured) stands in where the device cannot be asked.
int he_cus() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return HE_CUS;
  }
  int n = cached[dev];
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    n = HE_CUS;
  }
  cached[dev] = n;
  return n;
}

extern "C" int he_abi_version(void) { return HE_ABI_VERSION; }
