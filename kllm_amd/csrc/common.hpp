// Shared declarations of the gfx950 kernels: storage types, conversions,
// wave reductions, error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

namespace kllm {

constexpr int kWave = 64;  // CDNA wavefront

// Storage types of weights, activations and cache. DT_F32 / DT_BF16 are the
// values of the `dtype` argument of every entry point.
enum : int { DT_F32 = 0, DT_BF16 = 1 };
typedef __bf16 bf16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
// float -> bfloat16 rounds to nearest even (the hardware conversion of gfx950).
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

// The gate's activation of a gated feed-forward, the value of the `act` argument of the
// entry points that apply one.  Another activation is another value here and another case
// in gate_act; every kernel with a gate in its epilogue calls this one function.
enum : int { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_COUNT = 2 };

__device__ __forceinline__ float gate_act(float g, int act) {
  if (act == ACT_GELU_TANH) {   // 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))
    const float u = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.f + tanhf(u));
  }
  return g / (1.f + expf(-g));  // SiLU (reference: backend/model.cu:477-483)
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a workgroup of up to 1024 threads. `red` is LDS of at least 16
// floats. Every thread gets the result; the order of additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // red may still be read from an earlier call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += red[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = red[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, red[w]);
  return total;
}

// ---- errors ---------------------------------------------------------------
// Return convention of every entry point: 0 ok; a positive value is a HIP
// error code; negative values are ERR_ARG (a size or pointer the kernel does
// not take) and ERR_STATE.  The text of the calling thread's last error is
// read with kllm_last_error.
enum : int { ERR_ARG = -2, ERR_STATE = -1 };

void set_error(const char* fmt, ...);

#define KLLM_FAIL(code, ...)            \
  do {                                  \
    ::kllm::set_error(__VA_ARGS__);     \
    return (code);                      \
  } while (0)

#define KLLM_REQUIRE(cond, ...)                   \
  do {                                            \
    if (!(cond)) KLLM_FAIL(::kllm::ERR_ARG, __VA_ARGS__); \
  } while (0)

#define KLLM_CHECK_LAUNCH(name)                                                   \
  do {                                                                            \
    hipError_t e_ = hipGetLastError();                                            \
    if (e_ != hipSuccess)                                                         \
      KLLM_FAIL((int)e_, "%s: launch failed: %s", name, hipGetErrorString(e_));   \
  } while (0)

// Compute units of the current device (cached); 256 if it cannot be asked.
int device_cus();
// XCDs of the current device (cached); 8 if it cannot be asked.
int device_xcds();

inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

}  // namespace kllm
