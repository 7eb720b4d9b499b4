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

extern "C" int he_abi_version(void) { return HE_ABI_VERSION; }
