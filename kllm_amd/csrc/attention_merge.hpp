// The kernel that merges the partial results of a token's slices of keys; shared by the
// bfloat16 and the float32 decode attention.
#pragma once
#include <math.h>

#include "common.hpp"

namespace kllm {

// out[t, h, :] = sum_s w_s o_s / sum_s w_s l_s with w_s = exp(m_s - max m).
// One wave per (token, head); sixteen slices are read at a time (a token's slices are
// many where contexts are long, and a round of reads costs a trip to memory).
template <typename T>
__global__ __launch_bounds__(64) void attn_merge_kernel(T* __restrict__ out,
                                                        const float* __restrict__ part, int H, int hd,
                                                        int nslices, const int* __restrict__ token_list) {
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int stride = hd + 2;
  const float* p = part + ((long)t * H + h) * nslices * stride;
  float M = -INFINITY;
  for (int s = lane; s < nslices; s += kWave) M = fmaxf(M, p[(long)s * stride + hd]);
  M = wave_max(M);
  float denom = 0.f;
  for (int s = lane; s < nslices; s += kWave) {
    const float ms = p[(long)s * stride + hd];
    if (ms != -INFINITY) denom += expf(ms - M) * p[(long)s * stride + hd + 1];
  }
  denom = wave_sum(denom);
  for (int d = lane; d < hd; d += kWave) {
    float o = 0.f;
    for (int s0 = 0; s0 < nslices; s0 += 16) {
      float ms[16], os[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const bool ok = s0 + j < nslices;
        ms[j] = ok ? p[(long)(s0 + j) * stride + hd] : -INFINITY;
        os[j] = ok ? p[(long)(s0 + j) * stride + d] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (ms[j] != -INFINITY) o += expf(ms[j] - M) * os[j];
    }
    out[((long)t * H + h) * hd + d] = from_f32<T>(o / denom);
  }
}

}  // namespace kllm
