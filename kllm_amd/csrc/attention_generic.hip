// Causal attention over the paged cache, one workgroup per (token, head):
// the kernel that takes every size and both dtypes.  The faster kernels for
// prompts and for decode batches are tested against it.
//
// For the token at position p of its request, head h reads KV head
// h / (H/KV) and the keys [max(0, p - window + 1), p] (all keys [0, p] when
// window is 0): reference backend/model.cu:343-408 (scores, maximum, exp,
// sum, values) and :224-225 (window).  Unlike the reference, which keeps all
// scores of a row in shared memory, scores are taken 256 keys at a time with
// a running maximum and sum, so the context is not bounded by a buffer.
//
// Page layout, per page and KV head: keys [slot][hd], values [hd][slot].
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kAttnThreads = 256;
constexpr int kMaxHeadDim = 256;

template <typename T>
__global__ __launch_bounds__(kAttnThreads) void attn_generic_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ span_of_token,
    const int* __restrict__ block_table, int max_pages, int page_size, int H, int KV, int hd,
    int window, float scale) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float ps[kAttnThreads];
  __shared__ float red[16];
  __shared__ float part[kAttnThreads];

  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (H / KV);
  const int pos = positions[t];
  const int len = pos + 1;
  const int start = (window > 0 && len > window) ? len - window : 0;
  const int* table = block_table + (long)span_of_token[t] * max_pages;
  const long block = (long)page_size * hd;

  const T* qrow = q + ((long)t * H + h) * hd;
  for (int i = tid; i < hd; i += kAttnThreads) qs[i] = to_f32(qrow[i]);
  __syncthreads();

  // Values: thread (d, sl) sums over the pages sl, sl + nslice, ... of a chunk.
  const int nslice = kAttnThreads / hd;
  const int d = tid % hd, sl = tid / hd;
  const bool pv_thread = sl < nslice;

  const int chunk_pages = page_size >= kAttnThreads ? 1 : kAttnThreads / page_size;
  const int chunk_keys = chunk_pages * page_size;  // <= 256 (page_size <= 256 is checked on the host)

  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int pg0 = start / page_size; pg0 * page_size < len; pg0 += chunk_pages) {
    const int base = pg0 * page_size;
    // ---- scores of this chunk: thread i <-> key base + i
    float s = -INFINITY;
    const int key = base + tid;
    if (tid < chunk_keys && key >= start && key < len) {
      const int page = table[key / page_size];
      const T* krow = cache + (((long)page * 2 + 0) * KV + kvh) * block + (long)(key % page_size) * hd;
      float dot = 0.f;
      for (int i = 0; i < hd; ++i) dot = fmaf(qs[i], to_f32(krow[i]), dot);
      s = dot * scale;
    }
    const float cmax = block_max(s, red);
    const float m_new = fmaxf(m, cmax);
    const float alpha = expf(m - m_new);  // 0 on the first chunk (m = -inf)
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    ps[tid] = p;
    const float csum = block_sum(p, red);  // its barriers also publish ps
    l = l * alpha + csum;
    m = m_new;
    acc *= alpha;
    // ---- values
    if (pv_thread) {
      for (int pg = sl; pg < chunk_pages; pg += nslice) {
        const int pbase = base + pg * page_size;
        const int lo = max(start - pbase, 0), hi = min(len - pbase, page_size);
        if (lo >= hi) continue;
        const int page = table[pbase / page_size];
        const T* vrow = cache + (((long)page * 2 + 1) * KV + kvh) * block + (long)d * page_size;
        const float* pp = ps + pg * page_size;
        for (int sidx = lo; sidx < hi; ++sidx) acc = fmaf(pp[sidx], to_f32(vrow[sidx]), acc);
      }
    }
    __syncthreads();  // ps is rewritten by the next chunk
  }

  part[tid] = pv_thread ? acc : 0.f;
  __syncthreads();
  if (tid < hd) {
    float o = 0.f;
    for (int s2 = 0; s2 < nslice; ++s2) o += part[s2 * hd + tid];
    out[((long)t * H + h) * hd + tid] = from_f32<T>(o / l);
  }
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_attn_generic(const void* q, void* out, const void* cache, const int* positions,
                                 const int* span_of_token, const int* block_table, int max_pages,
                                 int page_size, int n, int H, int KV, int hd, int window,
                                 float scale, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(q && out && cache && positions && span_of_token && block_table,
               "attn_generic: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && KV > 0 && H % KV == 0, "attn_generic: bad heads n=%d H=%d KV=%d", n,
               H, KV);
  KLLM_REQUIRE(hd > 0 && hd <= kMaxHeadDim, "attn_generic: head_dim %d is outside [1, %d]", hd,
               kMaxHeadDim);
  KLLM_REQUIRE(page_size > 0 && page_size <= kAttnThreads && max_pages > 0,
               "attn_generic: page_size %d is outside [1, %d]", page_size, kAttnThreads);
  KLLM_REQUIRE(window >= 0, "attn_generic: negative window");
  KLLM_REQUIRE(H <= 65535, "attn_generic: too many heads for the grid");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "attn_generic: unknown dtype %d", dtype);
  const dim3 grid(n, H);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(kAttnThreads), 0, stream,
                       (const float*)q, (float*)out, (const float*)cache, positions, span_of_token,
                       block_table, max_pages, page_size, H, KV, hd, window, scale);
  else
    hipLaunchKernelGGL(attn_generic_kernel<bf16_t>, grid, dim3(kAttnThreads), 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, positions,
                       span_of_token, block_table, max_pages, page_size, H, KV, hd, window, scale);
  KLLM_CHECK_LAUNCH("attn_generic");
  return 0;
}
