// Host-only part of libfg_mi355.so: error channel, device facts, stream-K partition arithmetic.
#include <cstdlib>
#include <cstring>
#include <atomic>
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

namespace {
// The current switches are an immutable snapshot behind an atomic pointer: fg_reload_options() publishes a new one
// and never frees the old (a few dozen bytes per reload), so a thread that reads fg_options() while another reloads
// sees either snapshot whole, and a reference it still holds stays valid.
std::atomic<const FgOptions*> g_opt{nullptr};
std::once_flag g_opt_once;
void load_options() {
  FgOptions o = {};
  o.gemm_no_dma = getenv("FG_GEMM_NO_DMA") != nullptr;
  o.gemm_sk_even = getenv("FG_GEMM_SK_EVEN") != nullptr;
  if (const char* e = getenv("FG_GEMM_TILE")) {
    int a = 0, b = 0;
    if (sscanf(e, "%dx%d", &a, &b) == 2 && a > 0 && b > 0) {
      o.gemm_tile_bm = a; o.gemm_tile_bn = b;
    }
  }
  o.skinny_no_lds = getenv("FG_SKINNY_NO_LDS") != nullptr;
  o.skinny_rows64 = getenv("FG_SKINNY_ROWS64") != nullptr;
  if (const char* e = getenv("FG_SKINNY_TILE")) {
    const int v = atoi(e);
    o.skinny_tile = v == 32 ? 32 : v == 16 ? 16 : 0;
  }
  if (const char* e = getenv("FG_ATTN_KERNEL")) strncpy(o.attn_kernel, e, sizeof(o.attn_kernel) - 1);
  o.attn_mixed = -1;
  if (const char* e = getenv("FG_ATTN_MIXED")) o.attn_mixed = e[0] != '0' ? 1 : 0;
  if (const char* e = getenv("FG_DECODE_MIN_TILES")) {
    const int v = atoi(e);
    if (v >= 4 && v % 4 == 0) o.decode_min_tiles = v;
  }
  if (const char* e = getenv("FG_DECODE_WG_PER_CU")) {
    const int v = atoi(e);
    if (v >= 1 && v <= 64) o.decode_wg_per_cu = v;
  }
  g_opt.store(new FgOptions(o), std::memory_order_release);
}
}  // namespace

const FgOptions& fg_options() {
  std::call_once(g_opt_once, load_options);
  return *g_opt.load(std::memory_order_acquire);
}

extern "C" void fg_reload_options(void) {
  std::call_once(g_opt_once, [] {});
  load_options();
}

extern "C" const char* fg_last_error(void) { return g_err; }

void fg_static_scratch_prime(int device);  // gemm_skinny.hip

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
  // the one piece of per-device set-up the library has: the address of fg_gemm_skinny_static's scratch array
  fg_static_scratch_prime(device);
  return FG_OK;
}
