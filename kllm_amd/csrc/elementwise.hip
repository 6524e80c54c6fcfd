// Embedding, residual add + RMSNorm, rotary tables, rotary + cache append,
// SiLU gate.  One workgroup per token row; 32-bit arithmetic throughout.
//
// Inputs that come from a matrix product may arrive as `nsplit` partial sums
// ([nsplit][n][cols], `split_stride` elements apart); the consumer adds them
// in a fixed order, so a split product needs no pass of its own and gives the
// same bits on every run.
#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kThreads = 256;

// x[t, :] = table[ids[t], :]   (reference: backend/model.cu:89-95).  With `from`, token t
// whose from[t] >= 0 takes its id from sampled[from[t]] instead: the id that the last step's
// sampling left on the device, so that a step can be queued before that id has reached the host.
template <typename T>
__global__ void embed_kernel(float* __restrict__ out, const T* __restrict__ table,
                             const int* __restrict__ ids, const int* __restrict__ from,
                             const int* __restrict__ sampled, int d, int vocab) {
  const long t = blockIdx.x;
  int id = ids[t];
  if (from && from[t] >= 0) id = sampled[from[t]];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host has checked the range
  const T* src = table + (long)id * d;
  float* dst = out + t * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = to_f32(src[i]);
}

// Sum of the nsplit partial values p[0], p[stride], ...: eight loads are in
// flight at a time and the order of additions is fixed.
template <typename TIN>
__device__ __forceinline__ float sum_splits(const TIN* __restrict__ p, int nsplit, long stride) {
  float v = 0.f;
  int s = 0;
  for (; s + 8 <= nsplit; s += 8) {
    float t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = to_f32(p[(long)(s + j) * stride]);
    v += ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
  }
  if (s + 4 <= nsplit) {
    float t[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = to_f32(p[(long)(s + j) * stride]);
    v += (t[0] + t[1]) + (t[2] + t[3]);
    s += 4;
  }
  for (; s < nsplit; ++s) v += to_f32(p[(long)s * stride]);
  return v;
}

// v = x[src] (+ sum of delta splits); optionally x[src] = v;
// out[r] = v * rsqrt(mean(v^2) + eps) * w   (reference: backend/model.cu:101-122, :144-165)
template <typename TIN, typename TOUT, int KEEP>   // KEEP: elements of the row a thread keeps in registers
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TIN* __restrict__ delta, int nsplit,
                                   long split_stride, const float* __restrict__ w,
                                   TOUT* __restrict__ out, const int* __restrict__ rows, int d,
                                   float eps, int write_x) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  const long src = rows ? rows[r] : r;
  float* xr = x + src * d;
  const TIN* dr = delta ? delta + src * d : nullptr;
  const int tid = threadIdx.x, T = blockDim.x;
  // The first KEEP*T elements: every load of the thread goes out before any sum.
  float keep[KEEP], wkeep[KEEP];
#pragma unroll
  for (int it = 0; it < KEEP; ++it) {
    const int i = tid + it * T;
    keep[it] = i < d ? xr[i] : 0.f;
    wkeep[it] = (out && i < d) ? w[i] : 0.f;
  }
  if (dr && KEEP > 4) {                                 // long rows: element by element
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int i = tid + it * T;
      if (i < d) keep[it] += sum_splits(dr + i, nsplit, split_stride);
    }
  } else if (dr) {
    // Eight partial sums of every kept element are loaded before any is added, so that a
    // thread's loads wait for each other once per eight splits, not once per element; the
    // order of additions is that of sum_splits.
    int s = 0;
    for (; s + 8 <= nsplit; s += 8) {
      float t[KEEP][8];
#pragma unroll
      for (int it = 0; it < KEEP; ++it) {
        const int i = tid + it * T;
#pragma unroll
        for (int j = 0; j < 8; ++j) t[it][j] = i < d ? to_f32(dr[i + (long)(s + j) * split_stride]) : 0.f;
      }
#pragma unroll
      for (int it = 0; it < KEEP; ++it)
        keep[it] += ((t[it][0] + t[it][1]) + (t[it][2] + t[it][3])) + ((t[it][4] + t[it][5]) + (t[it][6] + t[it][7]));
    }
    if (s < nsplit) {                                   // up to seven more, again all loaded first
      float t[KEEP][7];
#pragma unroll
      for (int it = 0; it < KEEP; ++it) {
        const int i = tid + it * T;
#pragma unroll
        for (int j = 0; j < 7; ++j)
          t[it][j] = (i < d && s + j < nsplit) ? to_f32(dr[i + (long)(s + j) * split_stride]) : 0.f;
      }
      const int rest = nsplit - s;
#pragma unroll
      for (int it = 0; it < KEEP; ++it) {
        float v = keep[it];
        if (rest >= 4) {
          v += (t[it][0] + t[it][1]) + (t[it][2] + t[it][3]);
#pragma unroll
          for (int j = 4; j < 7; ++j) v += t[it][j];    // zeros beyond the last split
        } else {
#pragma unroll
          for (int j = 0; j < 3; ++j) v += t[it][j];
        }
        keep[it] = v;
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < KEEP; ++it) {
    const int i = tid + it * T;
    if (i < d) {
      if (write_x) xr[i] = keep[it];
      ss += keep[it] * keep[it];
    }
  }
  for (int i = tid + KEEP * T; i < d; i += T) {   // rows longer than KEEP*T
    float v = xr[i];
    if (dr) v += sum_splits(dr + i, nsplit, split_stride);
    if (write_x) xr[i] = v;
    ss += v * v;
  }
  if (!out) return;
  ss = block_sum(ss, red);
  const float scale = rsqrtf(ss / (float)d + eps);
  TOUT* orow = out + r * d;
#pragma unroll
  for (int it = 0; it < KEEP; ++it) {
    const int i = tid + it * T;
    if (i < d) orow[i] = from_f32<TOUT>(keep[it] * scale * wkeep[it]);
  }
  for (int i = tid + KEEP * T; i < d; i += T) {
    float v = xr[i];  // already the sum when write_x (same thread wrote it)
    if (dr && !write_x) v += sum_splits(dr + i, nsplit, split_stride);
    orow[i] = from_f32<TOUT>(v * scale * w[i]);
  }
}

// cos/sin of pos * theta^(-2j/head_dim), angle in double
// (reference: backend/model.cu:176-178)
__global__ void rope_tables_kernel(float* __restrict__ cos_t, float* __restrict__ sin_t,
                                   const int* __restrict__ positions, int n, int half, int head_dim,
                                   double theta) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * half) return;
  const int t = idx / half, j = idx % half;
  const double freq = pow(theta, -2.0 * (double)j / (double)head_dim);
  const double ang = (double)positions[t] * freq;
  cos_t[idx] = (float)cos(ang);
  sin_t[idx] = (float)sin(ang);
}

// Rotate q and k (pairs (j, j + hd/2), reference: backend/model.cu:170-184),
// store q, and put k and v into the token's page (reference: :187-201).
// Page layout, per page and KV head: keys [slot][hd], values [hd][slot].
// How a head is rotated is data: the first `rot` elements of a head are rotated
// (the rest pass through), in pairs (j, j + rot/2) or, `interleaved`, (2j, 2j+1);
// cos and sin are [n][rot/2].  The reference's rotation is rot = hd, not
// interleaved, which is also what the vector kernel below and the fused
// epilogues of the small-batch products take.
template <typename TIN, typename T>
__global__ void rope_append_kernel(const TIN* __restrict__ qkv, int nsplit, long split_stride,
                                   T* __restrict__ q_out, const float* __restrict__ cos_t,
                                   const float* __restrict__ sin_t, T* __restrict__ cache,
                                   const int* __restrict__ positions,
                                   const int* __restrict__ span_of_token,
                                   const int* __restrict__ block_table, int max_pages,
                                   int page_size, int H, int KV, int hd, int rot, int interleaved) {
  const long t = blockIdx.x;
  const int half = hd / 2, rhalf = rot / 2;
  const int qd = H * hd, kvd = cache ? KV * hd : 0;
  const long row = qd + 2 * kvd;
  const TIN* in = qkv + t * row;
  const float* c = cos_t ? cos_t + t * rhalf : nullptr;
  const float* s = sin_t ? sin_t + t * rhalf : nullptr;
  // Items of a token: H*half query pairs, KV*half key pairs, KV*hd values.
  const int q_items = H * half, k_items = cache ? KV * half : 0;
  const int items = q_items + k_items + kvd;
  const long block = (long)page_size * hd;  // one (page, k|v, head) block
  int page = 0, slot = 0;
  if (cache) {
    const int pos = positions[t];
    page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
    slot = pos % page_size;
  }
  for (int item = blockIdx.y * blockDim.x + threadIdx.x; item < items; item += gridDim.y * blockDim.x) {
    if (item < q_items + k_items) {
      const bool is_q = item < q_items;
      const int idx = is_q ? item : item - q_items;
      const int h = idx / half, j = idx % half;
      // the two elements of this item: a rotated pair, or two that pass through
      const bool turns = j < rhalf;
      const int ea = turns ? (interleaved ? 2 * j : j) : rot + 2 * (j - rhalf);
      const int eb = turns ? (interleaved ? 2 * j + 1 : j + rhalf) : ea + 1;
      const TIN* src = in + (is_q ? 0 : qd) + h * hd;
      const float a = sum_splits(src + ea, nsplit, split_stride);
      const float b = sum_splits(src + eb, nsplit, split_stride);
      const float cc = (c && turns) ? c[j] : 1.f, sn = (s && turns) ? s[j] : 0.f;
      T* o = is_q ? q_out + t * qd + h * hd
                  : cache + (((long)page * 2 + 0) * KV + h) * block + (long)slot * hd;
      o[ea] = from_f32<T>(a * cc - b * sn);
      o[eb] = from_f32<T>(b * cc + a * sn);
    } else {
      const int idx = item - q_items - k_items;
      const int h = idx / hd, j = idx % hd;
      const float v = sum_splits(in + qd + kvd + idx, nsplit, split_stride);
      cache[(((long)page * 2 + 1) * KV + h) * block + (long)j * page_size + slot] = from_f32<T>(v);
    }
  }
}

// Four neighbouring sums of the splits at once, added in the order of sum_splits.
__device__ __forceinline__ floatx4 sum_splits4(const float* __restrict__ p, int nsplit, long stride) {
  floatx4 v = {0.f, 0.f, 0.f, 0.f};
  int s = 0;
  for (; s + 8 <= nsplit; s += 8) {
    floatx4 t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = *reinterpret_cast<const floatx4*>(p + (long)(s + j) * stride);
    v += ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
  }
  if (s + 4 <= nsplit) {
    floatx4 t[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = *reinterpret_cast<const floatx4*>(p + (long)(s + j) * stride);
    v += (t[0] + t[1]) + (t[2] + t[3]);
    s += 4;
  }
  for (; s < nsplit; ++s) v += *reinterpret_cast<const floatx4*>(p + (long)s * stride);
  return v;
}

constexpr int kRopeRun = 16;   // neighbouring tokens whose workgroups share an XCD in the kernel below

// The same for float32 sums (whole, or partial sums over slices of K) and head sizes that are
// multiples of 8: a thread takes four neighbouring pairs, or four values, with 16-byte loads,
// and its loads go out before the token's page is looked up, so that the two waits overlap.
// Workgroups are numbered so that a run of kRopeRun neighbouring tokens stays on one XCD (the
// XCDs take workgroups round-robin).  Of a run, `chunks` workgroups per token rotate queries
// and keys (a token's row of each is contiguous in q_out and in its page); `vblocks` more take
// the values of all its tokens, 64 elements of every token each, lanes of neighbouring tokens
// side by side: a value's place in its page is two bytes beside its neighbour token's, so
// sixteen lanes fill a 32-byte sector where a workgroup per token would write two bytes of it.
template <typename T>
__global__ void rope_append_vec_kernel(const float* __restrict__ qkv, int nsplit, long split_stride,
                                       T* __restrict__ q_out,
                                       const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                       T* __restrict__ cache, const int* __restrict__ positions,
                                       const int* __restrict__ span_of_token,
                                       const int* __restrict__ block_table, int max_pages,
                                       int page_size, int H, int KV, int hd, int n, int chunks,
                                       int vblocks, int xcds) {
  typedef T tx4 __attribute__((ext_vector_type(4)));
  const int xcd = blockIdx.x % xcds, seq = blockIdx.x / xcds;
  const int per_run = kRopeRun * chunks + vblocks;
  const int at = seq % per_run;
  const long t0 = ((long)(seq / per_run) * xcds + xcd) * kRopeRun;
  const int half = hd / 2;
  const int qd = H * hd, kvd = cache ? KV * hd : 0;
  const long block = (long)page_size * hd;
  if (at >= kRopeRun * chunks) {
    // values: thread = (token of the run, four neighbouring elements)
    const long t = t0 + threadIdx.x % kRopeRun;
    const int idx = (at - kRopeRun * chunks) * (4 * kThreads / kRopeRun) + (threadIdx.x / kRopeRun) * 4;
    if (t >= n || idx >= kvd) return;
    const floatx4 a = sum_splits4(qkv + t * (qd + 2 * kvd) + qd + kvd + idx, nsplit, split_stride);
    const int pos = positions[t];
    const int page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
    const int h = idx / hd, j = idx % hd;
    T* v = cache + (((long)page * 2 + 1) * KV + h) * block + pos % page_size;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[(long)(j + e) * page_size] = from_f32<T>(a[e]);
    return;
  }
  const long t = t0 + at % kRopeRun;
  if (t >= n) return;
  const float* in = qkv + t * (qd + 2 * kvd);
  const int q_items = H * half / 4, k_items = cache ? KV * half / 4 : 0;
  const int item = (at / kRopeRun) * blockDim.x + threadIdx.x;
  if (item >= q_items + k_items) return;
  const bool is_q = item < q_items;
  const int idx = (is_q ? item : item - q_items) * 4;
  const int h = idx / half, j = idx % half;
  const float* src = in + (is_q ? 0 : qd) + h * hd + j;
  const floatx4 a = sum_splits4(src, nsplit, split_stride);
  const floatx4 b = sum_splits4(src + half, nsplit, split_stride);
  floatx4 cc = {1, 1, 1, 1}, sn = {0, 0, 0, 0};
  if (cos_t) {
    cc = *reinterpret_cast<const floatx4*>(cos_t + t * half + j);
    sn = *reinterpret_cast<const floatx4*>(sin_t + t * half + j);
  }
  int page = 0, slot = 0;
  if (!is_q) {
    const int pos = positions[t];
    page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
    slot = pos % page_size;
  }
  tx4 lo, hi;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    lo[e] = from_f32<T>(a[e] * cc[e] - b[e] * sn[e]);
    hi[e] = from_f32<T>(b[e] * cc[e] + a[e] * sn[e]);
  }
  T* o = is_q ? q_out + t * qd + h * hd : cache + (((long)page * 2 + 0) * KV + h) * block + (long)slot * hd;
  *reinterpret_cast<tx4*>(o + j) = lo;
  *reinterpret_cast<tx4*>(o + j + half) = hi;
}

// out[t, i] = act(gate[t, i]) * up[t, i], gate = cols [0, f), up = cols [f, 2f)
// (reference: backend/model.cu:477-483)
template <typename TIN, typename TOUT>
__global__ void silu_mul_kernel(const TIN* __restrict__ gu, int nsplit, long split_stride,
                                TOUT* __restrict__ out, long n, int f, int act) {
  const long total = n * f;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long t = idx / f;
    const int i = idx % f;
    const TIN* row = gu + t * 2 * f;
    const float g = sum_splits(row + i, nsplit, split_stride);
    const float u = sum_splits(row + f + i, nsplit, split_stride);
    out[idx] = from_f32<TOUT>(gate_act(g, act) * u);
  }
}

// out[i] = sum over splits of in[s][i]
template <typename TOUT>
__global__ void sum_splits_kernel(const float* __restrict__ in, int nsplit, long count,
                                  TOUT* __restrict__ out) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
       i += (long)gridDim.x * blockDim.x)
    out[i] = from_f32<TOUT>(sum_splits(in + i, nsplit, count));
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_sum_splits(const float* in, int nsplit, long count, void* out, int out_dtype,
                               hipStream_t stream) {
  KLLM_REQUIRE(in && out && nsplit >= 1 && count > 0, "sum_splits: bad arguments");
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "sum_splits: unknown dtype");
  int grid = ceil_div(count, kThreads);
  if (grid > 8192) grid = 8192;
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(sum_splits_kernel<float>, dim3(grid), dim3(kThreads), 0, stream, in, nsplit, count,
                       (float*)out);
  else
    hipLaunchKernelGGL(sum_splits_kernel<bf16_t>, dim3(grid), dim3(kThreads), 0, stream, in, nsplit, count,
                       (bf16_t*)out);
  KLLM_CHECK_LAUNCH("sum_splits");
  return 0;
}

extern "C" int kllm_embed(float* out, const void* table, const int* ids, const int* from,
                          const int* sampled, int n, int d, int vocab, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(out && table && ids, "embed: null pointer");
  KLLM_REQUIRE((from == nullptr) == (sampled == nullptr), "embed: from and sampled go together");
  KLLM_REQUIRE(n > 0 && d > 0 && vocab > 0, "embed: bad sizes n=%d d=%d vocab=%d", n, d, vocab);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "embed: unknown dtype %d", dtype);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(n), dim3(kThreads), 0, stream, out,
                       (const float*)table, ids, from, sampled, d, vocab);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(n), dim3(kThreads), 0, stream, out,
                       (const bf16_t*)table, ids, from, sampled, d, vocab);
  KLLM_CHECK_LAUNCH("embed");
  return 0;
}

template <typename TIN>
static int launch_add_rmsnorm(float* x, const void* delta, int nsplit, long split_stride,
                              const float* w, void* out, int out_dtype, const int* rows, int n, int d,
                              float eps, int write_x, hipStream_t stream) {
  // Few rows: more threads per row, so that a row's loads are all in flight.
  const int threads = (n <= 256 && d > 1024) ? 1024 : kThreads;
  const int per_thread = ceil_div(d, threads);
#define KLLM_NORM(TOUT, KEEP)                                                                       \
  hipLaunchKernelGGL((add_rmsnorm_kernel<TIN, TOUT, KEEP>), dim3(n), dim3(threads), 0, stream, x,    \
                     (const TIN*)delta, nsplit, split_stride, w, (TOUT*)out, rows, d, eps, write_x)
  if (out_dtype == DT_F32) {
    if (per_thread <= 2) KLLM_NORM(float, 2);
    else if (per_thread <= 4) KLLM_NORM(float, 4);
    else KLLM_NORM(float, 8);
  } else {
    if (per_thread <= 2) KLLM_NORM(bf16_t, 2);
    else if (per_thread <= 4) KLLM_NORM(bf16_t, 4);
    else KLLM_NORM(bf16_t, 8);
  }
#undef KLLM_NORM
  KLLM_CHECK_LAUNCH("add_rmsnorm");
  return 0;
}

extern "C" int kllm_add_rmsnorm(float* x, const void* delta, int delta_dtype, int nsplit,
                                long split_stride, const float* w, void* out, int out_dtype,
                                const int* rows, int n, int d, float eps, int write_x,
                                hipStream_t stream) {
  KLLM_REQUIRE(x, "add_rmsnorm: null x");
  KLLM_REQUIRE(n > 0 && d > 0, "add_rmsnorm: bad sizes n=%d d=%d", n, d);
  KLLM_REQUIRE(!out || w, "add_rmsnorm: a norm output needs a weight");
  KLLM_REQUIRE(out || (delta && write_x), "add_rmsnorm: nothing to do");
  KLLM_REQUIRE(!delta || nsplit >= 1, "add_rmsnorm: nsplit %d", nsplit);
  KLLM_REQUIRE(!(rows && write_x), "add_rmsnorm: gathered rows cannot be written back");
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "add_rmsnorm: unknown out dtype");
  KLLM_REQUIRE(delta_dtype == DT_F32 || delta_dtype == DT_BF16, "add_rmsnorm: unknown delta dtype");
  if (delta_dtype == DT_F32)
    return launch_add_rmsnorm<float>(x, delta, nsplit, split_stride, w, out, out_dtype, rows, n, d,
                                     eps, write_x, stream);
  return launch_add_rmsnorm<bf16_t>(x, delta, nsplit, split_stride, w, out, out_dtype, rows, n, d,
                                    eps, write_x, stream);
}

extern "C" int kllm_rope_tables(float* cos_t, float* sin_t, const int* positions, int n,
                                int head_dim, double theta, hipStream_t stream) {
  KLLM_REQUIRE(cos_t && sin_t && positions, "rope_tables: null pointer");
  KLLM_REQUIRE(n > 0 && head_dim > 0 && head_dim % 2 == 0, "rope_tables: bad sizes n=%d hd=%d", n,
               head_dim);
  KLLM_REQUIRE(theta > 0, "rope_tables: theta must be positive");
  const int half = head_dim / 2;
  const long total = (long)n * half;
  hipLaunchKernelGGL(rope_tables_kernel, dim3(ceil_div(total, kThreads)), dim3(kThreads), 0, stream,
                     cos_t, sin_t, positions, n, half, head_dim, theta);
  KLLM_CHECK_LAUNCH("rope_tables");
  return 0;
}

template <typename TIN, typename T>
static int launch_rope_append(const void* qkv, int nsplit, long split_stride, void* q_out,
                              const float* cos_t, const float* sin_t, void* cache,
                              const int* positions, const int* span_of_token,
                              const int* block_table, int max_pages, int page_size, int n, int H,
                              int KV, int hd, int rot, int interleaved, hipStream_t stream) {
  const int items = H * (hd / 2) + (cache ? KV * (hd / 2) + KV * hd : 0);
  int chunks = ceil_div(items, kThreads);
  if ((long)n * chunks > 16384) chunks = ceil_div(16384, n);   // many tokens: fewer, longer workgroups
  if (rot == hd && !interleaved && sizeof(TIN) == 4 && hd % 8 == 0 && ((uintptr_t)qkv & 15) == 0 &&
      (nsplit == 1 || split_stride % 4 == 0) && (H * hd + (cache ? 2 * KV * hd : 0)) % 4 == 0 &&
      ((uintptr_t)q_out & 15) == 0 && (!cache || ((uintptr_t)cache & 15) == 0) &&
      (!cos_t || (((uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0)) {
    const int pairs = H * (hd / 2) + (cache ? KV * (hd / 2) : 0);
    const int vchunks = ceil_div(pairs, 4 * kThreads), xcds = device_xcds();
    const int vblocks = cache ? ceil_div((long)KV * hd, 4 * kThreads / kRopeRun) : 0;
    const long runs = ceil_div(ceil_div(n, kRopeRun), xcds) * xcds;     // padded: every XCD gets as many
    hipLaunchKernelGGL((rope_append_vec_kernel<T>), dim3(runs * (kRopeRun * vchunks + vblocks)), dim3(kThreads), 0,
                       stream, (const float*)qkv, nsplit, split_stride, (T*)q_out, cos_t, sin_t, (T*)cache, positions, span_of_token,
                       block_table, max_pages, page_size, H, KV, hd, n, vchunks, vblocks, xcds);
    KLLM_CHECK_LAUNCH("rope_append");
    return 0;
  }
  hipLaunchKernelGGL((rope_append_kernel<TIN, T>), dim3(n, chunks), dim3(kThreads), 0, stream,
                     (const TIN*)qkv, nsplit, split_stride, (T*)q_out, cos_t, sin_t, (T*)cache,
                     positions, span_of_token, block_table, max_pages, page_size, H, KV, hd, rot, interleaved);
  KLLM_CHECK_LAUNCH("rope_append");
  return 0;
}

extern "C" int kllm_rope_append(const void* qkv, int in_dtype, int nsplit, long split_stride,
                                void* q_out, const float* cos_t, const float* sin_t, void* cache,
                                const int* positions, const int* span_of_token,
                                const int* block_table, int max_pages, int page_size, int n, int H,
                                int KV, int hd, int rot, int interleaved, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(qkv && q_out, "rope_append: null pointer");
  KLLM_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0 && (interleaved == 0 || interleaved == 1),
               "rope_append: rotary dimension %d of a head of %d (even, at most the head), interleaved %d", rot, hd,
               interleaved);
  KLLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "rope_append: cos and sin go together");
  KLLM_REQUIRE(n > 0 && H > 0 && hd > 0 && hd % 2 == 0, "rope_append: bad sizes n=%d H=%d hd=%d", n,
               H, hd);
  KLLM_REQUIRE(nsplit >= 1, "rope_append: nsplit %d", nsplit);
  if (cache) {
    KLLM_REQUIRE(positions && span_of_token && block_table, "rope_append: null index array");
    KLLM_REQUIRE(KV > 0 && max_pages > 0 && page_size > 0,
                 "rope_append: bad cache sizes KV=%d max_pages=%d page_size=%d", KV, max_pages,
                 page_size);
  }
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "rope_append: unknown dtype");
  KLLM_REQUIRE(in_dtype == DT_F32 || in_dtype == DT_BF16, "rope_append: unknown input dtype");
#define KLLM_RA(TIN, T)                                                                         \
  return launch_rope_append<TIN, T>(qkv, nsplit, split_stride, q_out, cos_t, sin_t, cache,      \
                                    positions, span_of_token, block_table, max_pages, page_size, \
                                    n, H, KV, hd, rot, interleaved, stream)
  if (in_dtype == DT_F32 && dtype == DT_F32) KLLM_RA(float, float);
  if (in_dtype == DT_F32 && dtype == DT_BF16) KLLM_RA(float, bf16_t);
  if (in_dtype == DT_BF16 && dtype == DT_BF16) KLLM_RA(bf16_t, bf16_t);
#undef KLLM_RA
  KLLM_FAIL(ERR_ARG, "rope_append: bfloat16 input with a float32 cache is not built");
}

extern "C" int kllm_silu_mul(const void* gu, int in_dtype, int nsplit, long split_stride, void* out,
                             int out_dtype, int n, int f, int act, hipStream_t stream) {
  KLLM_REQUIRE(gu && out, "silu_mul: null pointer");
  KLLM_REQUIRE(act >= 0 && act < ACT_COUNT, "silu_mul: unknown activation %d", act);
  KLLM_REQUIRE(n > 0 && f > 0 && nsplit >= 1, "silu_mul: bad sizes n=%d f=%d nsplit=%d", n, f,
               nsplit);
  const long total = (long)n * f;
  int grid = ceil_div(total, kThreads);
  if (grid > 8192) grid = 8192;
#define KLLM_SM(TIN, TOUT)                                                                      \
  hipLaunchKernelGGL((silu_mul_kernel<TIN, TOUT>), dim3(grid), dim3(kThreads), 0, stream,       \
                     (const TIN*)gu, nsplit, split_stride, (TOUT*)out, (long)n, f, act)
  if (in_dtype == DT_F32 && out_dtype == DT_F32) KLLM_SM(float, float);
  else if (in_dtype == DT_F32 && out_dtype == DT_BF16) KLLM_SM(float, bf16_t);
  else if (in_dtype == DT_BF16 && out_dtype == DT_BF16) KLLM_SM(bf16_t, bf16_t);
  else KLLM_FAIL(ERR_ARG, "silu_mul: dtype pair %d -> %d is not built", in_dtype, out_dtype);
#undef KLLM_SM
  KLLM_CHECK_LAUNCH("silu_mul");
  return 0;
}
