// Error text, device description and ABI version of the kernel library.
#include <stdarg.h>
#include <string.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

// One buffer per thread, as the reference keeps it (backend/shim.cu:8-17).
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// Compute units of the current device, asked once per device.
int device_cus() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    cached[dev] = cus;
  }
  return cached[dev];
}

}  // namespace kllm

extern "C" int kllm_device_cus(void) { return kllm::device_cus(); }

extern "C" int kllm_last_error(char* buf, int len) {
  if (!buf || len <= 0) return 0;
  strncpy(buf, kllm::g_error, len - 1);
  buf[len - 1] = 0;
  return (int)strlen(buf);
}

extern "C" int kllm_abi_version(void) { return 3; }

// Reference: te_device_info, backend/shim.cu:25-34.
extern "C" int kllm_device_info(int device, char* buf, int len) {
  if (!buf || len <= 0) KLLM_FAIL(kllm::ERR_ARG, "device_info: no buffer");
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) KLLM_FAIL((int)e, "device_info: %s", hipGetErrorString(e));
  snprintf(buf, len, "%s (%s), %d CUs, %.1f GiB, LDS %zu KiB per workgroup", p.name, p.gcnArchName,
           p.multiProcessorCount, (double)p.totalGlobalMem / (1024.0 * 1024.0 * 1024.0),
           p.sharedMemPerBlock / 1024);
  return 0;
}
