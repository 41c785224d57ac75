// A stand-in for the few HIP runtime entry points libfg_mi355.so imports, for running the library's host code on a
// machine with no GPU.  Test infrastructure only: it is loaded (RTLD_GLOBAL, before the library) by tests/emu/worker.py
// and by nothing else.  Kernel registrations are recorded, every launch is handed to a callback with the kernel's
// mangled name, its grid, block, dynamic LDS bytes and argument pointers, and the callback runs the kernel's compiled
// assembly in the interpreter (tests/emu/gcn_emu.py).  Nothing here computes anything.
#include <hip/hip_runtime.h>

#include <cstring>
#include <map>
#include <string>

namespace {
typedef int (*launch_cb_t)(const char* name, const unsigned* grid, const unsigned* block, void** args, size_t shmem,
                           void* stream);
typedef void* (*symbol_cb_t)(const char* name, size_t bytes);
launch_cb_t g_launch = nullptr;
symbol_cb_t g_symbol = nullptr;
std::map<const void*, std::string>& functions() {
  static std::map<const void*, std::string> m;
  return m;
}
struct Var {
  std::string name;
  size_t size;
  void* device;
};
std::map<const void*, Var>& variables() {
  static std::map<const void*, Var> m;
  return m;
}
struct Config {
  dim3 grid, block;
  size_t shmem;
  hipStream_t stream;
};
thread_local Config g_cfg;
int g_num_cu = 256;
int g_capturing = 0;
hipError_t g_last_error = hipSuccess;  // what hipGetLastError reports next (a failed launch), as the runtime does
}  // namespace

extern "C" {
void shim_set_callbacks(launch_cb_t l, symbol_cb_t s) {
  g_launch = l;
  g_symbol = s;
}
void shim_set_num_cu(int n) { g_num_cu = n; }
void shim_set_capturing(int on) { g_capturing = on; }
int shim_num_functions() { return (int)functions().size(); }

void** __hipRegisterFatBinary(const void*) {
  static void* handle[1];
  return handle;
}
void __hipUnregisterFatBinary(void**) {}
void __hipRegisterFunction(void**, const void* host, char*, const char* device_name, unsigned, void*, void*, void*, void*,
                           int*) {
  functions()[host] = device_name;
}
void __hipRegisterVar(void**, void* host, char*, char* device_name, int, size_t size, int, int) {
  variables()[host] = Var{device_name, size, nullptr};
}
hipError_t __hipPushCallConfiguration(dim3 grid, dim3 block, size_t shmem, hipStream_t stream) {
  g_cfg = Config{grid, block, shmem, stream};
  return hipSuccess;
}
hipError_t __hipPopCallConfiguration(dim3* grid, dim3* block, size_t* shmem, hipStream_t* stream) {
  *grid = g_cfg.grid;
  *block = g_cfg.block;
  *shmem = g_cfg.shmem;
  *stream = g_cfg.stream;
  return hipSuccess;
}
hipError_t hipLaunchKernel(const void* fn, dim3 grid, dim3 block, void** args, size_t shmem, hipStream_t stream) {
  auto it = functions().find(fn);
  if (it == functions().end() || g_launch == nullptr) return g_last_error = hipErrorInvalidDeviceFunction;
  const unsigned g[3] = {grid.x, grid.y, grid.z}, b[3] = {block.x, block.y, block.z};
  if (g_launch(it->second.c_str(), g, b, args, shmem, (void*)stream) != 0) return g_last_error = hipErrorLaunchFailure;
  return hipSuccess;
}
hipError_t hipGetDevice(int* d) {
  *d = 0;
  return hipSuccess;
}
hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t attr, int) {
  switch (attr) {
    case hipDeviceAttributeMultiprocessorCount: *v = g_num_cu; return hipSuccess;
    case hipDeviceAttributeMaxSharedMemoryPerBlock: *v = 160 * 1024; return hipSuccess;
    case hipDeviceAttributeWarpSize: *v = 64; return hipSuccess;
    default: *v = 0; return hipErrorInvalidValue;
  }
}
hipError_t hipGetDevicePropertiesR0600(hipDeviceProp_tR0600* p, int d) {
  if (d != 0) return hipErrorInvalidDevice;
  std::memset(p, 0, sizeof(*p));
  std::strcpy(p->name, "interpreter");
  std::strcpy(p->gcnArchName, "gfx950:sramecc+:xnack-");
  p->multiProcessorCount = g_num_cu;
  p->sharedMemPerBlock = 160 * 1024;
  p->warpSize = 64;
  p->maxThreadsPerBlock = 1024;
  return hipSuccess;
}
hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
hipError_t hipGetLastError(void) {
  const hipError_t e = g_last_error;
  g_last_error = hipSuccess;
  return e;
}
const char* hipGetErrorString(hipError_t e) {
  return e == hipSuccess ? "no error" : "the interpreter refused the launch (its message is in the test's output)";
}
hipError_t hipGetSymbolAddress(void** ptr, const void* symbol) {
  auto it = variables().find(symbol);
  if (it == variables().end() || g_symbol == nullptr) return hipErrorInvalidSymbol;
  if (it->second.device == nullptr) it->second.device = g_symbol(it->second.name.c_str(), it->second.size);
  *ptr = it->second.device;
  return hipSuccess;
}
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* s) {
  *s = g_capturing ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
  return hipSuccess;
}
hipError_t hipStreamGetCaptureInfo(hipStream_t, hipStreamCaptureStatus* s, unsigned long long* id) {
  *s = g_capturing ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
  if (id) *id = g_capturing ? 1 : 0;
  return hipSuccess;
}
}
