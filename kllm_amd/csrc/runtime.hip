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

// XCDs (dies with an L2 of their own, which take workgroups round-robin) of the current device,
// asked once per device; 8 if it cannot be asked.
int device_xcds() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 8;
  if (cached[dev] == 0) {
    int xcds = 0;
    if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess || xcds <= 0) xcds = 8;
    cached[dev] = xcds;
  }
  return cached[dev];
}

// ---- what the box reaches with nothing in the way (for quoting figures against) ----------
__global__ __launch_bounds__(256) void calibrate_copy_kernel(floatx4* __restrict__ dst,
                                                             const floatx4* __restrict__ src, long n16) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (long)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// A read-only stream: every lane keeps eight 16-byte loads in flight and adds what it read; one
// float per workgroup goes out, so that the loads cannot be dropped.
__global__ __launch_bounds__(256) void calibrate_read_kernel(const floatx4* __restrict__ src, long n16,
                                                             float* __restrict__ sink) {
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  const long stride = (long)gridDim.x * blockDim.x;
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    floatx4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = src[i + j * stride];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc += v[j];
  }
  for (; i < n16; i += stride) acc += src[i];
  __shared__ float red[16];
  const float total = block_sum(acc[0] + acc[1] + acc[2] + acc[3], red);
  if (threadIdx.x == 0) sink[blockIdx.x] = total;
}

// Four independent accumulator tiles per wave, `iters` rounds of one MFMA each; the result is
// written so that the loop cannot be dropped.
template <bool F32>
__global__ __launch_bounds__(256) void calibrate_mfma_kernel(float* __restrict__ sink, int iters) {
  floatx16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
  const float v = 1.f + threadIdx.x * 1e-6f;
  bf16x8 a8, b8;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a8[e] = (bf16_t)v;
    b8[e] = (bf16_t)(v * 0.5f);
  }
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (F32) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(v, v * 0.5f, acc[j], 0, 0, 0);
      else acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a8, b8, acc[j], 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[j][e];
  if (s == 12345.678f) sink[threadIdx.x % 64] = s;   // never true; keeps the loop alive
}

}  // namespace kllm

extern "C" int kllm_calibrate_copy(void* dst, const void* src, long bytes, hipStream_t stream) {
  KLLM_REQUIRE(dst && src && bytes > 0 && bytes % 16 == 0 && ((uintptr_t)dst & 15) == 0 && ((uintptr_t)src & 15) == 0,
               "calibrate_copy: %ld bytes must be a multiple of 16 and the buffers 16-byte aligned", bytes);
  const int grid = kllm::device_cus() * 16;
  hipLaunchKernelGGL(kllm::calibrate_copy_kernel, dim3(grid), dim3(256), 0, stream, (kllm::floatx4*)dst,
                     (const kllm::floatx4*)src, bytes / 16);
  KLLM_CHECK_LAUNCH("calibrate_copy");
  return 0;
}

extern "C" int kllm_calibrate_read_workgroups(void) { return kllm::device_cus() * 16; }

extern "C" int kllm_calibrate_read(const void* src, long bytes, float* sink, hipStream_t stream) {
  KLLM_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && ((uintptr_t)src & 15) == 0,
               "calibrate_read: %ld bytes must be a multiple of 16 and the buffer 16-byte aligned", bytes);
  hipLaunchKernelGGL(kllm::calibrate_read_kernel, dim3(kllm_calibrate_read_workgroups()), dim3(256), 0, stream,
                     (const kllm::floatx4*)src, bytes / 16, sink);
  KLLM_CHECK_LAUNCH("calibrate_read");
  return 0;
}

// Launches the MFMA loop; *flops receives the floating-point operations of the launch.
extern "C" int kllm_calibrate_mfma(int dtype, int iters, float* sink, double* flops, hipStream_t stream) {
  KLLM_REQUIRE(sink && flops && iters > 0 && iters <= (1 << 20), "calibrate_mfma: bad arguments");
  KLLM_REQUIRE(dtype == kllm::DT_F32 || dtype == kllm::DT_BF16, "calibrate_mfma: unknown dtype %d", dtype);
  const int grid = kllm::device_cus() * 8;          // eight workgroups of four waves per CU
  const double per_mfma = dtype == kllm::DT_F32 ? 2.0 * 32 * 32 * 2 : 2.0 * 32 * 32 * 16;
  *flops = per_mfma * 4.0 * iters * 4.0 * grid;
  if (dtype == kllm::DT_F32)
    hipLaunchKernelGGL(kllm::calibrate_mfma_kernel<true>, dim3(grid), dim3(256), 0, stream, sink, iters);
  else
    hipLaunchKernelGGL(kllm::calibrate_mfma_kernel<false>, dim3(grid), dim3(256), 0, stream, sink, iters);
  KLLM_CHECK_LAUNCH("calibrate_mfma");
  return 0;
}

extern "C" int kllm_device_cus(void) { return kllm::device_cus(); }
extern "C" int kllm_device_xcds(void) { return kllm::device_xcds(); }

extern "C" int kllm_last_error(char* buf, int len) {
  if (!buf || len <= 0) return 0;
  strncpy(buf, kllm::g_error, len - 1);
  buf[len - 1] = 0;
  return (int)strlen(buf);
}

extern "C" int kllm_abi_version(void) { return 8; }

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
