// Error text of the last refused call, per host thread.
#include "common.h"
#include <cstdarg>
#include <cstdio>

namespace ninfer {
static thread_local char g_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int device_cu_count() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}
}  // namespace ninfer

extern "C" const char* ninfer_last_error() { return ninfer::g_error; }

extern "C" int ninfer_device_info(int* cu_count, int* lds_bytes, char* arch, int arch_len) {
  hipDeviceProp_t p;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess)
    return ninfer::set_error(-2, "no HIP device");
  *cu_count = p.multiProcessorCount;
  *lds_bytes = (int)p.sharedMemPerBlock;
  snprintf(arch, arch_len, "%s", p.gcnArchName);
  return 0;
}
