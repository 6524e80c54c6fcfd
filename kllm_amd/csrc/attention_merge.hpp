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

// The same for up to 64 slices and heads of up to 128 in one trip to memory instead of one per
// sixteen slices, with fewer loads a lane: every output element of every slice is asked for at once (64 DV
// loads a lane), lane s fetches slice s's maximum and sum and works out its weight, and the
// weights go from lane to lane while the sums are added in the order of the slices.
template <typename T, int DV, int R>   // R: 16, 32 or 64, at least the number of slices
__device__ __forceinline__ void attn_merge_wide(T* __restrict__ out, const float* __restrict__ part, int t, int h, int H,
                                                int hd, int nslices, int lane) {
  const int stride = hd + 2;
  const float* p = part + ((long)t * H + h) * nslices * stride;
  float os[DV][R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const float* q = p + (long)(j < nslices ? j : 0) * stride;      // beyond the last slice: a valid address
#pragma unroll
    for (int v = 0; v < DV; ++v) os[v][j] = q[lane + 64 * v < hd ? lane + 64 * v : 0];
  }
  const bool mine = lane < nslices;
  const float* q = p + (long)(mine ? lane : 0) * stride;
  const float ms = mine ? q[hd] : -INFINITY, ls = mine ? q[hd + 1] : 0.f;
  float M = ms;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
  // (M is finite: some slice holds the token's own key)
  const float w = (ms == -INFINITY) ? 0.f : expf(ms - M);
  float denom = 0.f, o[DV];
#pragma unroll
  for (int v = 0; v < DV; ++v) o[v] = 0.f;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const float wj = __shfl(w, j, 64), lj = __shfl(ls, j, 64);     // 0 beyond the last slice
    denom += wj * lj;
#pragma unroll
    for (int v = 0; v < DV; ++v) o[v] += wj * os[v][j];
  }
#pragma unroll
  for (int v = 0; v < DV; ++v)
    if (lane + 64 * v < hd) out[((long)t * H + h) * hd + lane + 64 * v] = from_f32<T>(o[v] / denom);
}

template <typename T, int DV, int R>
__global__ __launch_bounds__(64) void attn_merge_wide_kernel(T* __restrict__ out, const float* __restrict__ part, int H,
                                                             int hd, int nslices, const int* __restrict__ token_list) {
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x;
  attn_merge_wide<T, DV, R>(out, part, t, blockIdx.y, H, hd, nslices, threadIdx.x);
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
  if (nslices <= 64 && hd <= 128) {
    // (one trip to memory whatever the number of slices, and a lane asks for 2 + slices x DV
    // numbers instead of slices x (2 + DV); 64 slices of a head of 64: the merge 10 us -> 6,
    // 16 slices: a microsecond less)
#define KLLM_MERGE_WIDE(DV, R) \
    hipLaunchKernelGGL((attn_merge_wide_kernel<T, DV, R>), grid, block, 0, stream, out, part, H, hd, nslices, token_list)
    if (hd <= 64) {
      if (nslices <= 16) KLLM_MERGE_WIDE(1, 16); else if (nslices <= 32) KLLM_MERGE_WIDE(1, 32); else KLLM_MERGE_WIDE(1, 64);
    } else {
      if (nslices <= 16) KLLM_MERGE_WIDE(2, 16); else if (nslices <= 32) KLLM_MERGE_WIDE(2, 32); else KLLM_MERGE_WIDE(2, 64);
    }
#undef KLLM_MERGE_WIDE
    return;
  }
  if (hd <= 64) hipLaunchKernelGGL((attn_merge_kernel<T, 1>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
  else if (hd <= 128) hipLaunchKernelGGL((attn_merge_kernel<T, 2>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
  else if (hd <= 192) hipLaunchKernelGGL((attn_merge_kernel<T, 3>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
  else hipLaunchKernelGGL((attn_merge_kernel<T, 4>), grid, block, 0, stream, out, part, H, hd, nslices, token_list);
}

}  // namespace kllm
