// The kernel that merges the partial results of a token's slices of keys; shared by the
// bfloat16 and the float32 decode attention.
#pragma once
#include <math.h>

#include "common.hpp"

namespace kllm {

// out[t, h, :] = sum_s w_s o_s / sum_s w_s l_s with w_s = exp(m_s - max m).
// One wave per (token, head).  The partial results were written by workgroups on other XCDs, so
// every read is a trip to memory: all reads of sixteen slices (maxima, sums and this lane's
// DV elements of each output) go out together, and every lane works out the weights for
// itself, so that sixteen slices cost one trip and no exchange between lanes.  Further
// rounds of sixteen (long contexts) are merged with a running maximum.  (R: the slices of a
// round, for callers with few.)
template <typename T, int DV, int R = 16>   // DV: elements of a head per lane (head size up to 64 DV); R: slices a round
__device__ __forceinline__ void attn_merge_one(T* __restrict__ out, const float* __restrict__ part, int t, int h, int H,
                                               int hd, int nslices, int lane) {
  const int stride = hd + 2;
  const float* p = part + ((long)t * H + h) * nslices * stride;
  float M = -INFINITY, denom = 0.f, o[DV];
#pragma unroll
  for (int v = 0; v < DV; ++v) o[v] = 0.f;
  for (int s0 = 0; s0 < nslices; s0 += R) {
    float ms[R], ls[R], os[DV][R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const float* q = p + (long)(s0 + j < nslices ? s0 + j : 0) * stride;   // beyond the last slice: a valid address
      ms[j] = q[hd];
      ls[j] = q[hd + 1];
#pragma unroll
      for (int v = 0; v < DV; ++v) os[v][j] = q[lane + 64 * v < hd ? lane + 64 * v : 0];
    }
    float m = M;
#pragma unroll
    for (int j = 0; j < R; ++j)
      if (s0 + j < nslices) m = fmaxf(m, ms[j]);
    if (m == -INFINITY) continue;                      // nothing but empty slices so far
    const float keep = expf(M - m);                    // 0 in the first round that holds a key
    denom *= keep;
#pragma unroll
    for (int v = 0; v < DV; ++v) o[v] *= keep;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      if (s0 + j < nslices && ms[j] != -INFINITY) {
        const float w = expf(ms[j] - m);
        denom += w * ls[j];
#pragma unroll
        for (int v = 0; v < DV; ++v) o[v] += w * os[v][j];
      }
    }
    M = m;
  }
#pragma unroll
  for (int v = 0; v < DV; ++v)
    if (lane + 64 * v < hd) out[((long)t * H + h) * hd + lane + 64 * v] = from_f32<T>(o[v] / denom);
}

template <typename T, int DV>
__global__ __launch_bounds__(64) void attn_merge_kernel(T* __restrict__ out,
                                                        const float* __restrict__ part, int H, int hd,
                                                        int nslices, const int* __restrict__ token_list) {
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x;
  attn_merge_one<T, DV>(out, part, t, blockIdx.y, H, hd, nslices, threadIdx.x);
}

// Launches the merge for `count` tokens (all, or those that token_list names).
template <typename T>
inline void launch_attn_merge(T* out, const float* part, int count, int H, int hd, int nslices,
                              const int* token_list, hipStream_t stream) {
  const dim3 grid(count, H), block(64);
  if (hd <= 64) hipLaunchKernelGGL((attn_merge_kernel<T, 1>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
  else if (hd <= 128) hipLaunchKernelGGL((attn_merge_kernel<T, 2>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
  else if (hd <= 192) hipLaunchKernelGGL((attn_merge_kernel<T, 3>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
  else hipLaunchKernelGGL((attn_merge_kernel<T, 4>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
}

}  // namespace kllm
