// Host-only part of libfg_mi355.so: error channel, device facts, stream-K partition arithmetic.
#include <mutex>
#include "fg_common.h"

namespace {
thread_local char g_err[512] = {0};
}

void fg_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fg_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fg_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return FG_ERR_LAUNCH;
  }
  return FG_OK;
}

extern "C" const char* fg_last_error(void) { return g_err; }

extern "C" int fg_abi_version(void) { return 2; }

extern "C" int fg_device_info(int device, int* num_cu, int* lds_bytes, int* gcn_arch) {
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) {
    fg_set_error("device_info: %s", hipGetErrorString(e));
    return FG_ERR_INVALID;
  }
  if (num_cu) *num_cu = p.multiProcessorCount;
  if (lds_bytes) *lds_bytes = (int)p.sharedMemPerBlock;
  if (gcn_arch) {
    int arch = 0;
    const char* s = p.gcnArchName;  // "gfx950:sramecc+:xnack-"
    if (s[0] == 'g' && s[1] == 'f' && s[2] == 'x') {
      // three hex digits after "gfx" (gfx90a exists; gfx950 is all decimal digits)
      for (int i = 3; i < 6 && s[i] && s[i] != ':'; ++i) {
        const char c = s[i];
        arch = arch * 16 + (c >= '0' && c <= '9' ? c - '0' : (c >= 'a' && c <= 'f' ? c - 'a' + 10 : 0));
      }
    }
    *gcn_arch = arch;  // 0x950 for MI355X
  }
  return FG_OK;
}
