// Error channel of the C entry points (a call returns 0, or 1 after storing a
// message that alofa_last_error() hands out) and the library's one workspace.
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

static Workspace g_workspace = {nullptr, 0, nullptr, 0};
const Workspace& workspace() { return g_workspace; }

int compute_units() {
  static int known = 0;
  if (known == 0) {
    int device = 0, n = 0;
    if (hipGetDevice(&device) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && n > 0) known = n;
    else return 256;      // (what an MI355X has; asked again next time)
  }
  return known;
}

}  // namespace alofa

// Allocates the workspace (once; later calls do nothing). Kernels that would use it fall back to
// forms that need none while it is absent. Not to be called under graph capture.
extern "C" int alofa_workspace_init() {
  using namespace alofa;
  if (g_workspace.tiles != nullptr) return 0;
  constexpr int64_t kTileFloats = 4 << 20;   // 16 MB
  constexpr int kCounters = kGemmCounters;
  void* tiles = nullptr;
  void* counters = nullptr;
  hipError_t e = hipExtMallocWithFlags(&tiles, kTileFloats * sizeof(float), hipDeviceMallocUncached);
  if (e == hipSuccess) e = hipExtMallocWithFlags(&counters, kCounters * sizeof(int), hipDeviceMallocUncached);
  if (e == hipSuccess) e = hipMemset(counters, 0, kCounters * sizeof(int));
  if (e == hipSuccess) e = hipDeviceSynchronize();
  ALOFA_REQUIRE(e == hipSuccess, "workspace_init: %s", hipGetErrorString(e));
  g_workspace = {static_cast<float*>(tiles), kTileFloats, static_cast<int*>(counters), kCounters};
  return 0;
}

extern "C" const char* alofa_last_error() { return alofa::g_error; }

extern "C" int alofa_abi_version() { return 1; }
