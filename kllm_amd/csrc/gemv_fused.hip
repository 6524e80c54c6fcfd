// Matrix products for up to 8 rows of X (the decode batches where every other
// cost is a launch): Y = X . W^T with the whole of K in one wave, so that no
// partial sums cross memory, and with the next elementwise step done in the
// epilogue while the sums are still in registers.
//
// A workgroup puts X (all rows, a chunk of K) into LDS; each of its four waves
// then owns a *pair* of rows of W, streams them from memory with several
// 16-byte loads per lane in flight, multiplies with X from LDS and reduces
// over its lanes.  What a pair is depends on the epilogue:
//
//   plain    rows (2p, 2p+1)              -> y[t][row] in float32
//   swiglu   rows (p, f+p): gate and up   -> h[t][p] = silu(gate) * up
//                                            (reference: backend/model.cu:477-483)
//   rope     rows (j, j+hd/2) of one head -> rotated q or k; rows (2p, 2p+1) of v
//            -> q_out and the token's page (reference: backend/model.cu:170-201)
//   resid    rows (2p, 2p+1): the sums are added to the residual stream in
//            place, and the workgroup's partial sums of squares of the new rows
//            are left for the consumer of the RMS norm behind the addition
//            (reference: the fused add + norm, backend/model.cu:144-165, here
//            without a launch of its own)
//
// The consumer of a resid product is given the residual stream (`norm_x`,
// float32) instead of X, the norm's weight and those partial sums, and
// normalises while it stages X: x * rsqrt(sum of squares / d + eps) * w,
// rounded to the storage type, the norm kernel's numbers in its order.
//
// Works for float32 and bfloat16 storage (32-bit accumulation in both).
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int GV_WAVES = 4;
constexpr int GV_MAXN = 8;
constexpr int GV_U = 4;                       // loads in flight per row and lane
constexpr int GV_LDS_BYTES = 32 * 1024;       // X chunk staged per workgroup

enum : int { GV_PLAIN = 0, GV_SWIGLU = 1, GV_ROPE = 2, GV_RESID = 3 };
constexpr int GV_SS_MAX = 512;                // partial sums of squares per row at most
constexpr int GV_NORMED_MAXN = 4;             // rows of X that are normalised while staged, at most

struct GvRope {
  void* q_out;
  const float* cos_t;
  const float* sin_t;
  void* cache;
  const int* positions;
  const int* span_of_token;
  const int* block_table;
  int max_pages, page_size, H, KV, hd;
  int act;                      // the gate's activation (GV_SWIGLU)
  const float* norm_x;          // the residual stream [n][k] that X is the RMS norm of, or null (then X is read)
  const float* norm_w;          // ... the norm's weight [k]
  const float* ss_in;           // ... [n][ss_parts rounded up to 4] partial sums of squares of its rows
  int ss_parts;
  float eps_in;
  float* resid;                 // GV_RESID: x [n][m], the sums are added in place
  float* ss_out;                // GV_RESID: [n][workgroups rounded up to 4]
};

template <typename T, int NT, int MODE, bool NORMED>   // NORMED: X is made from rp.norm_x while it is staged
__global__ __launch_bounds__(64 * GV_WAVES) void gemv_fused_kernel(
    const T* __restrict__ X, const T* __restrict__ W, void* __restrict__ Y, int n, int m, int k,
    int kchunk, int f, GvRope rp) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* xs = reinterpret_cast<T*>(lds_raw);       // [NT][kchunk]
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const long pair = (long)blockIdx.x * GV_WAVES + wave;
  const long pairs = m / 2;

  // ---- the two rows of this wave
  long row_a = 0, row_b = 0;
  bool live = pair < pairs;
  int region = 0, head = 0, j = 0;              // rope: 0 q, 1 k, 2 v
  // The rows' partial sums of squares go out first (two 16-byte loads a lane and row).
  floatx4 ss_v[NORMED ? NT : 1][2];
  if (NORMED) {
    const float* ssp = rp.ss_in;
    const int stride = (rp.ss_parts + 3) / 4 * 4;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int at = 4 * (lane + 64 * jj);
        ss_v[t][jj] = *reinterpret_cast<const floatx4*>(ssp + (long)min(t, n - 1) * stride + (at < stride ? at : 0));
      }
  }
  if (live) {
    if (MODE == GV_PLAIN || MODE == GV_RESID) {
      row_a = 2 * pair;
      row_b = row_a + 1;
    } else if (MODE == GV_SWIGLU) {
      row_a = pair;
      row_b = f + pair;
    } else {
      const int half = rp.hd / 2;
      const long q_pairs = (long)rp.H * half, k_pairs = rp.cache ? (long)rp.KV * half : 0;
      if (pair < q_pairs + k_pairs) {
        region = pair < q_pairs ? 0 : 1;
        const long p = region ? pair - q_pairs : pair;
        head = p / half;
        j = p % half;
        row_a = (region ? (long)rp.H * rp.hd : 0) + (long)head * rp.hd + j;
        row_b = row_a + half;
      } else {
        region = 2;
        const long p = pair - q_pairs - k_pairs;
        const long e = 2 * p;                   // element of the value vector
        head = e / rp.hd;
        j = e % rp.hd;
        row_a = (long)(rp.H + rp.KV) * rp.hd + e;
        row_b = row_a + 1;
      }
    }
  }

  // GV_RESID: lane t adds to x[t][row_a], x[t][row_b]; asked for now, needed at the very end
  float res_a = 0.f, res_b = 0.f;
  if (MODE == GV_RESID) {
    const bool ok = live && lane < n;
    const float* xp = rp.resid + (long)(ok ? lane : 0) * m;
    res_a = xp[ok ? row_a : 0];
    res_b = xp[ok ? row_b : 0];
  }
  // the rows' scales: sums in a fixed order, then across the wave (every wave gets all rows')
  float rs[NORMED ? NT : 1];
  if (NORMED) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float v = 0.f;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int e = 0; e < 4; ++e) v += 4 * (lane + 64 * jj) + e < rp.ss_parts ? ss_v[t][jj][e] : 0.f;
      rs[t] = rsqrtf(wave_sum(v) / (float)k + rp.eps_in);
    }
  }

  float acc[2][NT];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[r][t] = 0.f;
  const T* wa = W + row_a * k;
  const T* wb = W + row_b * k;

  for (int kc = 0; kc < k; kc += kchunk) {
    const int klen = min(kchunk, k - kc);        // a multiple of V
    // first loads of W go out before X is staged
    vec_t pre[2][GV_U];
#pragma unroll
    for (int u = 0; u < GV_U; ++u) {
      const int kk = (u * kWave + lane) * V;
      const bool ok = live && kk < klen;
      pre[0][u] = ok ? *reinterpret_cast<const vec_t*>(wa + kc + kk) : vec_t{};
      pre[1][u] = ok ? *reinterpret_cast<const vec_t*>(wb + kc + kk) : vec_t{};
    }
    if (kc) __syncthreads();                      // the last chunk is no longer read
    const int vecs = klen / V;
    const int total = NT * vecs;
    if (NORMED) {
      // normalising while staging: x and the norm's weight in float32, four pieces a thread at a time
      for (int base = tid; base < total; base += 64 * GV_WAVES * 4) {
        floatx4 xa[4][V / 4], wv[4][V / 4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int idx = min(base + i * 64 * GV_WAVES, total - 1);
          const int t = min(idx / vecs, n - 1), ch = idx % vecs;
#pragma unroll
          for (int q = 0; q < V / 4; ++q) {
            xa[i][q] = *reinterpret_cast<const floatx4*>(rp.norm_x + (long)t * k + kc + ch * V + 4 * q);
            wv[i][q] = *reinterpret_cast<const floatx4*>(rp.norm_w + kc + ch * V + 4 * q);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int idx = base + i * 64 * GV_WAVES;
          if (idx < total) {
            const int t = idx / vecs, ch = idx % vecs;
            float r = rs[0];
#pragma unroll
            for (int tt = 1; tt < NT; ++tt) r = t == tt ? rs[tt] : r;
            vec_t v;
#pragma unroll
            for (int e = 0; e < V; ++e)
              v[e] = t < n ? from_f32<T>(xa[i][e / 4][e % 4] * r * wv[i][e / 4][e % 4]) : from_f32<T>(0.f);
            *reinterpret_cast<vec_t*>(xs + (long)t * kchunk + ch * V) = v;
          }
        }
      }
    } else
    for (int base = tid; base < total; base += 64 * GV_WAVES * 8) {   // eight loads in flight
      vec_t v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int idx = base + i * 64 * GV_WAVES;
        const int t = idx / vecs, ch = idx % vecs;
        v[i] = (idx < total && t < n) ? *reinterpret_cast<const vec_t*>(X + (long)t * k + kc + ch * V)
                                      : vec_t{};
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int idx = base + i * 64 * GV_WAVES;
        if (idx < total) {
          const int t = idx / vecs, ch = idx % vecs;
          *reinterpret_cast<vec_t*>(xs + (long)t * kchunk + ch * V) = v[i];
        }
      }
    }
    __syncthreads();
    for (int k0 = 0; k0 < klen; k0 += GV_U * kWave * V) {
      vec_t cur[2][GV_U];
#pragma unroll
      for (int u = 0; u < GV_U; ++u) {
        cur[0][u] = pre[0][u];
        cur[1][u] = pre[1][u];
      }
      const int k1 = k0 + GV_U * kWave * V;
#pragma unroll
      for (int u = 0; u < GV_U; ++u) {            // the next round's loads
        const int kk = k1 + (u * kWave + lane) * V;
        const bool ok = live && kk < klen;
        pre[0][u] = ok ? *reinterpret_cast<const vec_t*>(wa + kc + kk) : vec_t{};
        pre[1][u] = ok ? *reinterpret_cast<const vec_t*>(wb + kc + kk) : vec_t{};
      }
#pragma unroll
      for (int u = 0; u < GV_U; ++u) {
        const int kk = k0 + (u * kWave + lane) * V;
        if (kk < klen) {
          float wf[2][V];
#pragma unroll
          for (int e = 0; e < V; ++e) {
            wf[0][e] = to_f32(cur[0][u][e]);
            wf[1][e] = to_f32(cur[1][u][e]);
          }
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const vec_t xv = *reinterpret_cast<const vec_t*>(xs + (long)t * kchunk + kk);
#pragma unroll
            for (int e = 0; e < V; ++e) {
              const float xf = to_f32(xv[e]);
              acc[0][t] = fmaf(wf[0][e], xf, acc[0][t]);
              acc[1][t] = fmaf(wf[1][e], xf, acc[1][t]);
            }
          }
        }
      }
    }
  }

  // ---- reduce over the wave; afterwards lane t finishes row t of X
  float mine_a = 0.f, mine_b = 0.f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const float sa = wave_sum(acc[0][t]), sb = wave_sum(acc[1][t]);
    if (lane == t) {
      mine_a = sa;
      mine_b = sb;
    }
  }
  if (MODE == GV_RESID) {
    // every wave reaches the barrier; a wave without rows of W counts zero
    __shared__ float sq_lds[GV_WAVES][GV_MAXN];
    const int t = lane;
    float sq = 0.f;
    if (live && t < n) {
      float* xp = rp.resid + (long)t * m;
      const float xa = res_a + mine_a, xb = res_b + mine_b;
      xp[row_a] = xa;
      xp[row_b] = xb;
      sq = xa * xa + xb * xb;
    }
    if (t < GV_MAXN) sq_lds[wave][t] = sq;
    __syncthreads();
    if (wave == 0 && t < n) {
      const float total = (sq_lds[0][t] + sq_lds[1][t]) + (sq_lds[2][t] + sq_lds[3][t]);
      rp.ss_out[(long)t * (((int)gridDim.x + 3) / 4 * 4) + blockIdx.x] = total;
    }
    return;
  }
  if (!live || lane >= n) return;
  const int t = lane;
  if (MODE == GV_PLAIN) {
    float* y = reinterpret_cast<float*>(Y);
    y[(long)t * m + row_a] = mine_a;
    y[(long)t * m + row_b] = mine_b;
  } else if (MODE == GV_SWIGLU) {
    T* h = reinterpret_cast<T*>(Y);
    h[(long)t * f + pair] = from_f32<T>(gate_act(mine_a, rp.act) * mine_b);
  } else {
    const int half = rp.hd / 2;
    int page = 0, slot = 0;
    if (region) {
      const int pos = rp.positions[t];
      page = rp.block_table[(long)rp.span_of_token[t] * rp.max_pages + pos / rp.page_size];
      slot = pos % rp.page_size;
    }
    const long block = (long)rp.page_size * rp.hd;
    if (region < 2) {
      const float cc = rp.cos_t ? rp.cos_t[(long)t * half + j] : 1.f;
      const float sn = rp.sin_t ? rp.sin_t[(long)t * half + j] : 0.f;
      const float ra = mine_a * cc - mine_b * sn, rb = mine_b * cc + mine_a * sn;
      T* o = region == 0
                 ? reinterpret_cast<T*>(rp.q_out) + ((long)t * rp.H + head) * rp.hd
                 : reinterpret_cast<T*>(rp.cache) + (((long)page * 2 + 0) * rp.KV + head) * block +
                       (long)slot * rp.hd;
      o[j] = from_f32<T>(ra);
      o[j + half] = from_f32<T>(rb);
    } else {
      T* v = reinterpret_cast<T*>(rp.cache) + (((long)page * 2 + 1) * rp.KV + head) * block;
      v[(long)j * rp.page_size + slot] = from_f32<T>(mine_a);
      v[(long)(j + 1) * rp.page_size + slot] = from_f32<T>(mine_b);
    }
  }
}

template <typename T, int MODE, bool NORMED>
static int launch_gv_n(const void* x, const void* w, void* y, int n, int m, int k, int f, const GvRope& rp,
                       hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  const int nt = n <= 1 ? 1 : n <= 2 ? 2 : n <= 4 ? 4 : 8;
  int kchunk = GV_LDS_BYTES / (nt * (int)sizeof(T));
  kchunk = kchunk / (GV_U * kWave * V) * (GV_U * kWave * V);   // whole rounds of loads
  if (kchunk > k) kchunk = k;
  const size_t lds = (size_t)nt * kchunk * sizeof(T);
  const dim3 grid(ceil_div(m / 2, GV_WAVES));
#define KLLM_GV(NT)                                                                              \
  hipLaunchKernelGGL((gemv_fused_kernel<T, NT, MODE, NORMED>), grid, dim3(64 * GV_WAVES), lds, stream,   \
                     (const T*)x, (const T*)w, y, n, m, k, kchunk, f, rp)
  if (nt == 1) KLLM_GV(1);
  else if (nt == 2) KLLM_GV(2);
  else if (nt == 4) KLLM_GV(4);
  else if (!NORMED) KLLM_GV(8);
  else KLLM_FAIL(ERR_ARG, "gemv: normalising while staging is built for up to %d rows, not %d", GV_NORMED_MAXN, n);
#undef KLLM_GV
  return 0;
}

template <typename T, int MODE>
static int launch_gv(const void* x, const void* w, void* y, int n, int m, int k, int f, const GvRope& rp,
                     hipStream_t stream) {
  if (rp.norm_x && MODE != GV_RESID) return launch_gv_n<T, MODE, true>(x, w, y, n, m, k, f, rp, stream);
  return launch_gv_n<T, MODE, false>(x, w, y, n, m, k, f, rp, stream);
}

}  // namespace kllm

using namespace kllm;

static int check_common(const char* what, const void* x, const void* w, const void* y, int n, int m,
                        int k, int dtype) {
  KLLM_REQUIRE(x && w && y, "%s: null pointer", what);
  KLLM_REQUIRE(n > 0 && n <= GV_MAXN, "%s: n=%d is outside [1, %d]", what, n, GV_MAXN);
  KLLM_REQUIRE(m > 0 && m % 2 == 0 && k > 0, "%s: bad sizes m=%d k=%d (m must be even)", what, m, k);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "%s: unknown dtype %d", what, dtype);
  const int v = dtype == DT_F32 ? 4 : 8;
  KLLM_REQUIRE(k % v == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0,
               "%s: K=%d must be a multiple of %d and the operands 16-byte aligned", what, k, v);
  return 0;
}

// X as the RMS norm of a residual stream, made while staging: checked and put into the
// kernel's arguments.  With it `x` is not read.
static int set_norm(const char* what, GvRope& rp, const KllmNormedInput* in, int n) {
  if (!in || !in->x) return 0;
  KLLM_REQUIRE(n <= GV_NORMED_MAXN, "%s: normalising while staging is built for up to %d rows, not %d", what,
               GV_NORMED_MAXN, n);
  KLLM_REQUIRE(in->weight && in->ss && in->parts >= 1 && in->parts <= GV_SS_MAX && in->eps >= 0.f,
               "%s: normalising while staging needs the norm's weight and 1 to %d partial sums of squares per row (got %d)",
               what, GV_SS_MAX, in->parts);
  KLLM_REQUIRE(((uintptr_t)in->x & 15) == 0 && ((uintptr_t)in->weight & 15) == 0 && ((uintptr_t)in->ss & 15) == 0,
               "%s: the residual stream, the norm's weight and the sums of squares must be 16-byte aligned", what);
  rp.norm_x = in->x;
  rp.norm_w = in->weight;
  rp.ss_in = in->ss;
  rp.ss_parts = in->parts;
  rp.eps_in = in->eps;
  return 0;
}

extern "C" int kllm_gemv_resid(const void* x, const void* w, float* resid, float* ss_out, int n, int m,
                               int k, int dtype, hipStream_t stream) {
  if (int rc = check_common("gemv_resid", x, w, resid, n, m, k, dtype)) return rc;
  KLLM_REQUIRE(ss_out, "gemv_resid: null pointer");
  GvRope rp = {};
  rp.resid = resid;
  rp.ss_out = ss_out;
  if (int rc = dtype == DT_F32 ? launch_gv<float, GV_RESID>(x, w, resid, n, m, k, 0, rp, stream)
                                 : launch_gv<bf16_t, GV_RESID>(x, w, resid, n, m, k, 0, rp, stream))
    return rc;
  KLLM_CHECK_LAUNCH("gemv_resid");
  return 0;
}

extern "C" int kllm_gemv_resid_parts(int m) { return ceil_div(m / 2, GV_WAVES); }
extern "C" int kllm_gemv_max_rows(void) { return GV_MAXN; }
extern "C" int kllm_gemv_normed_max_rows(void) { return GV_NORMED_MAXN; }
extern "C" int kllm_gemv_normed_max_parts(void) { return GV_SS_MAX; }

extern "C" int kllm_gemv_plain(const void* x, const void* w, float* y, int n, int m, int k, int dtype,
                               const KllmNormedInput* normed, hipStream_t stream) {
  if (normed && normed->x && !x) x = normed->x;
  if (int rc = check_common("gemv_plain", x, w, y, n, m, k, dtype)) return rc;
  GvRope rp = {};
  if (int rc = set_norm("gemv_plain", rp, normed, n)) return rc;
  if (int rc = dtype == DT_F32 ? launch_gv<float, GV_PLAIN>(x, w, y, n, m, k, 0, rp, stream)
                                 : launch_gv<bf16_t, GV_PLAIN>(x, w, y, n, m, k, 0, rp, stream))
    return rc;
  KLLM_CHECK_LAUNCH("gemv_plain");
  return 0;
}

extern "C" int kllm_gemv_swiglu(const void* x, const void* w_gate_up, void* h, int n, int f, int k,
                                int dtype, int act, const KllmNormedInput* normed, hipStream_t stream) {
  if (normed && normed->x && !x) x = normed->x;
  if (int rc = check_common("gemv_swiglu", x, w_gate_up, h, n, 2 * f, k, dtype)) return rc;
  KLLM_REQUIRE(act >= 0 && act < ACT_COUNT, "gemv_swiglu: unknown activation %d", act);
  GvRope rp = {};
  rp.act = act;
  if (int rc = set_norm("gemv_swiglu", rp, normed, n)) return rc;
  if (int rc = dtype == DT_F32 ? launch_gv<float, GV_SWIGLU>(x, w_gate_up, h, n, 2 * f, k, f, rp, stream)
                                 : launch_gv<bf16_t, GV_SWIGLU>(x, w_gate_up, h, n, 2 * f, k, f, rp, stream))
    return rc;
  KLLM_CHECK_LAUNCH("gemv_swiglu");
  return 0;
}

extern "C" int kllm_gemv_rope_append(const void* x, const void* w_qkv, void* q_out, const float* cos_t,
                                     const float* sin_t, void* cache, const int* positions,
                                     const int* span_of_token, const int* block_table, int max_pages,
                                     int page_size, int n, int H, int KV, int hd, int k, int dtype,
                                     const KllmNormedInput* normed, hipStream_t stream) {
  if (normed && normed->x && !x) x = normed->x;
  const int m = H * hd + (cache ? 2 * KV * hd : 0);
  if (int rc = check_common("gemv_rope_append", x, w_qkv, q_out, n, m, k, dtype)) return rc;
  KLLM_REQUIRE(H > 0 && hd > 0 && hd % 2 == 0, "gemv_rope_append: bad heads H=%d hd=%d", H, hd);
  KLLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "gemv_rope_append: cos and sin go together");
  if (cache)
    KLLM_REQUIRE(KV > 0 && positions && span_of_token && block_table && max_pages > 0 && page_size > 0,
                 "gemv_rope_append: bad cache arguments");
  GvRope rp = {};
  rp.q_out = q_out; rp.cos_t = cos_t; rp.sin_t = sin_t; rp.cache = cache;
  rp.positions = positions; rp.span_of_token = span_of_token; rp.block_table = block_table;
  rp.max_pages = max_pages; rp.page_size = page_size; rp.H = H; rp.KV = KV; rp.hd = hd;
  if (int rc = set_norm("gemv_rope_append", rp, normed, n)) return rc;
  if (int rc = dtype == DT_F32 ? launch_gv<float, GV_ROPE>(x, w_qkv, q_out, n, m, k, 0, rp, stream)
                                 : launch_gv<bf16_t, GV_ROPE>(x, w_qkv, q_out, n, m, k, 0, rp, stream))
    return rc;
  KLLM_CHECK_LAUNCH("gemv_rope_append");
  return 0;
}
