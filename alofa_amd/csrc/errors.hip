// Error channel of the C entry points: a call returns 0, or 1 after storing a
// message that alofa_last_error() hands out.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

namespace alofa {

static thread_local char g_error[512];

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return 1;
  }
  return 0;
}

}  // namespace alofa

extern "C" const char* alofa_last_error() { return alofa::g_error; }

extern "C" int alofa_abi_version() { return 1; }
