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

constexpr int kSampleThreads = 256;

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    int* __restrict__ out, const float* __restrict__ logits, const float* __restrict__ temperature,
    const float* __restrict__ uniform, int vocab) {
  __shared__ float red[16];
  __shared__ float best_val[kSampleThreads];
  __shared__ int best_idx[kSampleThreads];
  __shared__ float partial[kSampleThreads];
  __shared__ int chosen;

  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + (long)r * vocab;
  // Each thread owns one contiguous segment, so thread order is index order.
  const int seg = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int lo = min(tid * seg, vocab), hi = min(lo + seg, vocab);

  float bv = -INFINITY;
  int bi = vocab;  // "none"
  for (int i = lo; i < hi; ++i) {
    const float v = row[i];
    if (bi == vocab || v > bv) { bv = v; bi = i; }  // strict: the first maximum stays
  }
  best_val[tid] = bv;
  best_idx[tid] = bi;
  __syncthreads();
  if (tid == 0) {
    float v = best_val[0];
    int idx = best_idx[0];
    for (int i = 1; i < kSampleThreads; ++i)
      if (best_idx[i] < vocab && (idx == vocab || best_val[i] > v)) { v = best_val[i]; idx = best_idx[i]; }
    best_val[0] = v;
    chosen = idx;
  }
  __syncthreads();
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = chosen;
    return;
  }
  const float mx = best_val[0];
  const float inv_t = 1.f / temp;
  float sum = 0.f;
  for (int i = lo; i < hi; ++i) sum += expf((row[i] - mx) * inv_t);
  partial[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int i = 0; i < kSampleThreads; ++i) total += partial[i];
    const float target = uniform[r] * total;
    // Segment that holds the target, then the element inside it.
    float before = 0.f;
    int owner = -1;
    for (int i = 0; i < kSampleThreads; ++i) {
      if (target < before + partial[i]) { owner = i; break; }
      before += partial[i];
    }
    int idx = vocab - 1;
    if (owner >= 0) {
      const int olo = min(owner * seg, vocab), ohi = min(olo + seg, vocab);
      float c = before;
      idx = ohi - 1;
      for (int i = olo; i < ohi; ++i) {
        c += expf((row[i] - mx) * inv_t);
        if (target < c) { idx = i; break; }
      }
    }
    out[r] = idx;
  }
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
