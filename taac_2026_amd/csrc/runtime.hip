// Error reporting and ABI version of libtaac_hip.so.
#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace taac {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(TAAC_ERR_LAUNCH, "%s: HIP launch failed: %s", what, hipGetErrorString(e));
  return TAAC_OK;
}

// Compute units of the current device (the persistent kernels launch one workgroup per unit), cached per device.
int compute_units() {
  static int cached[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return -1;
  if (cached[device] > 0) return cached[device];
  int count = 0;
  if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) return -1;
  cached[device] = count;
  return count;
}

// Test hooks (taac_test_hooks): process-wide, changed by tests only.
static std::atomic<int> g_max_workgroups{0};
static std::atomic<int> g_fp8_tiled{0};
int test_max_workgroups() { return g_max_workgroups.load(std::memory_order_relaxed); }
bool test_fp8_tiled() { return g_fp8_tiled.load(std::memory_order_relaxed) != 0; }

}  // namespace taac

extern "C" void taac_test_hooks(int32_t max_workgroups, int32_t fp8_tiled) {
  taac::g_max_workgroups.store(max_workgroups > 0 ? max_workgroups : 0, std::memory_order_relaxed);
  taac::g_fp8_tiled.store(fp8_tiled != 0 ? 1 : 0, std::memory_order_relaxed);
}

extern "C" int taac_abi_version(void) { return TAAC_ABI_VERSION; }
extern "C" const char* taac_last_error(void) { return taac::g_last_error; }
