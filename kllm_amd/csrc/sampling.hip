// Choosing the next token on the device, one workgroup per row of logits.
//
// temperature == 0: the largest logit, the first one on ties (the reference's
// host Argmax, engine/engine.go:216-224).  temperature > 0:
// p = softmax(logits / temperature) with the maximum subtracted, all in
// 32-bit, and the smallest index whose cumulative probability exceeds
// u * total, for a uniform u in [0, 1) that the caller draws.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / kWave;

// (value, index) with the larger value, the smaller index on equal values
__device__ __forceinline__ void better(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    int* __restrict__ out, const float* __restrict__ logits, const float* __restrict__ temperature,
    const float* __restrict__ uniform, int vocab) {
  __shared__ float wave_val[kSampleWaves];
  __shared__ int wave_idx[kSampleWaves];
  __shared__ float wave_tot[kSampleWaves];
  __shared__ int chosen;

  const int r = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const float* row = logits + (long)r * vocab;
  // (asked for here, so that the trip to memory runs beside the logits')
  const float temp = temperature ? temperature[r] : 0.f;
  const float u = uniform ? uniform[r] : 0.f;
  // Each thread owns one contiguous segment, so thread order is index order.
  // Segments are multiples of four logits, so that a row whose length is one too is read
  // in 16-byte pieces, eight of them in flight per thread.
  const int seg = (vocab + 4 * kSampleThreads - 1) / (4 * kSampleThreads) * 4;
  const int lo = min(tid * seg, vocab), hi = min(lo + seg, vocab);

  float bv = -INFINITY;
  int bi = vocab;  // "none": loses against every index
  if (vocab % 4 == 0 && ((uintptr_t)logits & 15) == 0) {
    for (int i0 = lo; i0 < hi; i0 += 32) {
      floatx4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        v[j] = i0 + 4 * j < hi ? *reinterpret_cast<const floatx4*>(row + i0 + 4 * j)
                               : floatx4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = i0 + 4 * j + e;
          if (i < hi && (bi == vocab || v[j][e] > bv)) { bv = v[j][e]; bi = i; }   // strict: the first maximum stays
        }
    }
  } else {
    for (int i = lo; i < hi; ++i) {
      const float v = row[i];
      if (bi == vocab || v > bv) { bv = v; bi = i; }
    }
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (oi < vocab && (bi == vocab || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
  }
  if (lane == 0) {
    wave_val[wave] = bv;
    wave_idx[wave] = bi;
  }
  if (tid == 0) chosen = vocab - 1;
  __syncthreads();
  float mx = wave_val[0];
  int arg = wave_idx[0];
  for (int w = 1; w < kSampleWaves; ++w)
    if (wave_idx[w] < vocab && (arg == vocab || wave_val[w] > mx)) { mx = wave_val[w]; arg = wave_idx[w]; }
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = arg;
    return;
  }
  const float inv_t = 1.f / temp;
  float sum = 0.f;
  for (int i = lo; i < hi; ++i) sum += expf((row[i] - mx) * inv_t);
  // inclusive scan over the wave, then over the waves: thread t's probability
  // mass lies in [incl - sum, incl)
  float incl = sum;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const float up = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += up;
  }
  if (lane == kWave - 1) wave_tot[wave] = incl;
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < kSampleWaves; ++w) {
    if (w < wave) before += wave_tot[w];
    total += wave_tot[w];
  }
  // excl is the previous thread's incl, bit for bit: the ranges leave no gap
  const float prev = __shfl_up(incl, 1, kWave);
  const float excl = before + (lane == 0 ? 0.f : prev);
  incl += before;
  const float target = u * total;
  if (sum > 0.f && target >= excl && target < incl) {
    float c = excl;
    int idx = hi - 1;
    for (int i = lo; i < hi; ++i) {
      c += expf((row[i] - mx) * inv_t);
      if (target < c) { idx = i; break; }
    }
    chosen = idx;
  }
  __syncthreads();
  if (tid == 0) out[r] = chosen;
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_sample(int* out, const float* logits, const float* temperature,
                           const float* uniform, int rows, int vocab, hipStream_t stream) {
  KLLM_REQUIRE(out && logits, "sample: null pointer");
  KLLM_REQUIRE(rows > 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
  KLLM_REQUIRE((temperature == nullptr) == (uniform == nullptr),
               "sample: temperatures and uniforms go together");
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kSampleThreads), 0, stream, out, logits,
                     temperature, uniform, vocab);
  KLLM_CHECK_LAUNCH("sample");
  return 0;
}
