// Matrix products of a decode batch (up to 32 rows of X, bfloat16) on MFMA, with
// the step after the product done in the same launch.  Y = X . W^T, then
//
//   PARTS    float32 sums [nsplit, n, m] (only this one may split K);
//   SWIGLU   silu(gate) * up in bfloat16 (reference backend/model.cu:477-483);
//   ROPE     rotated queries and keys, and values, written to q_out and to
//            the tokens' pages (reference backend/model.cu:170-201).
//
// A workgroup owns tiles of 16 rows of W and one slice of K (all of K unless
// the caller splits).  It puts its slice of X, all rows, into LDS once.  Each
// of its four waves takes a quarter of the slice: it streams its part of the 16
// rows of W straight from memory, sixteen 16-byte loads per lane in flight, the
// first of them before X is staged, and multiplies with X from LDS
// (MFMA 16x16x32: A = W tile, B = X^T, D[w row][x row]).  The four partial
// tiles meet in LDS, are added in a fixed order, and the epilogue runs on the
// sums; no partial sum crosses memory unless the caller splits K.
//
// What the 16 MFMA rows of a tile are depends on the epilogue: 16 consecutive
// rows of W, or 8 pairs (gate row p and up row p; rows j and j + hd/2 of one
// head; two neighbouring value rows) with the first members in MFMA rows 0-7
// and the second in rows 8-15.
//
// The kernel is kept small on purpose (loops over rounds and tiles, one copy of
// the epilogue): a decode step runs a few workgroups of it per CU between other
// kernels, with a cold instruction cache every time, and a version with the
// epilogue unrolled into every round (74 KB of code) took half as long again.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int FL_AHEAD = 8;        // W loads per lane in one of the two buffers
constexpr int FL_PAD = 136;        // LDS row padding (elements): 128 of zeros behind K, 8 to shift banks
constexpr int FL_LDS_MAX = 160 * 1024;
constexpr int FL_TILE = 16 * 17;    // floats of one wave's partial tile in LDS: [x row][w row], padded

enum : int { FL_PARTS = 0, FL_SWIGLU = 2, FL_ROPE = 3 };

struct FlOut {
  void* y;
  const float* cos_t;
  const float* sin_t;
  void* cache;
  const int* positions;
  const int* span_of_token;
  const int* block_table;
  int max_pages, page_size, H, KV, hd;
  int act;                      // the gate's activation (FL_SWIGLU)
};

// Row of W behind MFMA row c of a tile, or -1.  Pair epilogues: unit = pair.
template <int EP>
__device__ __forceinline__ long fl_row(int tile, int c, int m, const FlOut& o) {
  if (EP == FL_PARTS) {
    const long r = (long)tile * 16 + c;
    return r < m ? r : -1;
  }
  const int pair = tile * 8 + (c & 7);          // m < 2^31, so pairs and tiles fit an int
  const int pairs = m / 2;
  if (pair >= pairs) return -1;
  const bool second = c >= 8;
  if (EP == FL_SWIGLU) return second ? pairs + pair : pair;
  const int half = o.hd / 2;
  const int rot_pairs = (o.H + (o.cache ? o.KV : 0)) * half;
  if (pair < rot_pairs) {
    const long a = (long)(pair / half) * o.hd + pair % half;   // q and k rows follow each other in W
    return second ? a + half : a;
  }
  const long e = 2 * (long)(pair - rot_pairs);
  return (long)(o.H + o.KV) * o.hd + e + (second ? 1 : 0);
}

// A workgroup barrier for data in LDS.  Unlike __syncthreads it does not wait for loads from
// memory: the weights asked for ahead stay in flight while the waves meet.
__device__ __forceinline__ void fl_lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);        // lgkmcnt(0): this wave's LDS operations are done
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int NT, int EP>
__global__ __launch_bounds__(256) void fused_linear_kernel(const bf16_t* __restrict__ X, FlOut out,
                                                           const bf16_t* __restrict__ W, int n, int m,
                                                           int k, int kslice, int tiles, int tiles_per_wg,
                                                           int x_stride) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int ld = kslice + FL_PAD;
  bf16_t* xs = reinterpret_cast<bf16_t*>(lds_raw);                            // [n][ld]
  float* part = reinterpret_cast<float*>(lds_raw + (size_t)n * ld * sizeof(bf16_t));   // [2][4][NT][x row 16][17]

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int g = lane / 16, c = lane % 16;
  const int kbeg = blockIdx.y * kslice;
  const int klen = min(k, kbeg + kslice) - kbeg;            // a multiple of 8
  const int kw = ((klen + 3) / 4 + 31) / 32 * 32;           // K of one wave
  const int wk0 = wave * kw;                                // this wave's offset in the slice
  const int wlen = max(0, min(klen, wk0 + kw) - wk0);
  const int steps = kw / 32;
  const int tile0 = blockIdx.x * tiles_per_wg;
  const int my_tiles = min(tiles_per_wg, tiles - tile0);
  const int rsteps = (steps + 2 * FL_AHEAD - 1) / (2 * FL_AHEAD) * (2 * FL_AHEAD);   // whole turns of both buffers
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // ---- rotate-and-append epilogue: thread (pair tid % 8, token tid / 8) needs the token's
  // page and slot, and cos and sin of its pair.  Loads return in order, so the position and
  // the span are asked for before the weights, and what depends on them after X is on its
  // way: none of it then holds up the weights or X, and all of it is there at the epilogue.
  int ep_pos[NT], ep_span[NT];
  if (EP == FL_ROPE) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int xr = t * 16 + tid / 8;
      const bool ok = out.cache && xr < n && tid < 128;
      ep_pos[t] = ok ? out.positions[xr] : 0;
      ep_span[t] = ok ? out.span_of_token[xr] : 0;
    }
  }

  // ---- X: wave w stages rows w, w + 4, ... of the slice, eight 16-byte loads a lane at a
  // time.  Loads return in order, so the last batch goes out before the weights: X is
  // then in LDS and the workgroup past its barrier while the weights are still arriving.
  // No load carries a branch (an index beyond the wave's share reads its last item again), so
  // that the compiler can count what is in flight and wait for X alone.
  const int chunks = klen / 8;
  const int mine = (n - wave + 3) / 4;                    // rows of this wave
  const int items = mine * chunks;
  auto x_load = [&](int base, bf16x8 (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = min(base + j * kWave, max(items - 1, 0));
      const int ri = idx / chunks, ch = idx - ri * chunks;
      const int row = min(wave + 4 * ri, n - 1);          // a wave without rows reads the last row
      v[j] = *reinterpret_cast<const bf16x8*>(X + (long)row * x_stride + kbeg + ch * 8);
    }
  };
  auto x_store = [&](int base, const bf16x8 (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * kWave;
      if (idx < items) {
        const int ri = idx / chunks, ch = idx - ri * chunks;
        *reinterpret_cast<bf16x8*>(&xs[(wave + 4 * ri) * ld + ch * 8]) = v[j];
      }
    }
  };
  bf16x8 xv0[8];
  int xbase = lane;
  for (; xbase + kWave * 8 < items; xbase += kWave * 8) {   // all but the last batch (more than eight rows)
    x_load(xbase, xv0);
    x_store(xbase, xv0);
  }
  x_load(xbase, xv0);

  // ---- W: two buffers of FL_AHEAD loads each, used in turn: while one is multiplied the
  // other is on its way, and it is asked for again as soon as it has been used.  No register
  // is copied from one buffer to the other (a copy would have to wait for its load).  A tile's
  // steps are padded to whole turns of both buffers.  A row, a tile or a K that does not exist
  // reads the first K of a row that does (finite numbers): the X beside it in LDS is zero, or
  // the output row is ignored.
  const bf16_t* far_row;                                    // first K of this lane's row of W
  int far_lane_off;                                         // this lane's offset in it, or -1: no such row
  int far_tile = 0, far_s0 = 0;                             // the steps that are loaded next
  auto tile_ptr = [&](int t) {
    const long r = t < my_tiles ? fl_row<EP>((int)tile0 + t, c, m, out) : -1;
    far_row = W + (r >= 0 ? r : 0) * k + kbeg;
    far_lane_off = r >= 0 ? wk0 + 8 * g : -1;
  };
  auto fill = [&](bf16x8 (&buf)[FL_AHEAD]) {
#pragma unroll
    for (int i = 0; i < FL_AHEAD; ++i) {
      const int s = far_s0 + i;
      const bool valid = far_lane_off >= 0 && s < steps && 32 * s + 8 * g < wlen;
      buf[i] = *reinterpret_cast<const bf16x8*>(far_row + (valid ? far_lane_off + 32 * s : 0));
    }
    far_s0 += FL_AHEAD;
    if (far_s0 == rsteps) {
      far_s0 = 0;
      tile_ptr(++far_tile);
    }
  };
  bf16x8 bufa[FL_AHEAD], bufb[FL_AHEAD];
  tile_ptr(0);
  fill(bufa);
  fill(bufb);

  // ---- X into LDS: what was asked for before the weights has arrived first
  x_store(xbase, xv0);
  {   // zeros in X's columns [klen, klen + 128): what the waves' slices of K reach beyond klen
    const int r = tid / 16, ch = tid % 16;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (t * 16 + r < n) *reinterpret_cast<bf16x8*>(&xs[(t * 16 + r) * ld + klen + 8 * ch]) = zero;
  }
  int ep_page[NT], ep_slot[NT];
  float ep_cos[NT], ep_sin[NT];
  auto rope_angles = [&](int tile_index) {
    if (EP != FL_ROPE || tid >= 128) return;
    const int half = out.hd / 2;
    const int pair = (tile0 + tile_index) * 8 + tid % 8;
    const int rot_pairs = (out.H + (out.cache ? out.KV : 0)) * half;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int xr = t * 16 + tid / 8;
      const bool ok = out.cos_t && xr < n && pair < rot_pairs && tile_index < my_tiles;
      ep_cos[t] = ok ? out.cos_t[(long)xr * half + pair % half] : 1.f;
      ep_sin[t] = ok ? out.sin_t[(long)xr * half + pair % half] : 0.f;
    }
  };
  if (EP == FL_ROPE) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int xr = t * 16 + tid / 8;
      ep_page[t] = ep_slot[t] = 0;
      if (out.cache && xr < n && tid < 128) {
        ep_page[t] = out.block_table[(long)ep_span[t] * out.max_pages + ep_pos[t] / out.page_size];
        ep_slot[t] = ep_pos[t] % out.page_size;
      }
    }
    rope_angles(0);
  }
  fl_lds_barrier();

  floatx4 acc[NT];
  const bf16_t* xrow[NT];                                   // rows beyond n are ignored: they read row n - 1
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    xrow[t] = xs + min(t * 16 + c, n - 1) * ld + wk0 + 8 * g;
  }
  auto multiply = [&](const bf16x8 (&buf)[FL_AHEAD], int s0) {
#pragma unroll
    for (int i = 0; i < FL_AHEAD; ++i) {
      if (s0 + i < steps) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const bf16x8 b = *reinterpret_cast<const bf16x8*>(xrow[t] + 32 * (s0 + i));
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[i], b, acc[t], 0, 0, 0);
        }
      }
    }
  };

  for (int tile = 0; tile < my_tiles; ++tile) {
    for (int s0 = 0; s0 < rsteps; s0 += 2 * FL_AHEAD) {
      multiply(bufa, s0);
      fill(bufa);
      multiply(bufb, s0 + FL_AHEAD);
      fill(bufb);
    }
    // ---- the tile is complete in this wave: meet the other waves in LDS
    float* pb = part + (tile & 1) * 4 * NT * FL_TILE;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) pb[(wave * NT + t) * FL_TILE + c * 17 + 4 * g + i] = acc[t][i];
      acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    fl_lds_barrier();
    const int tl = tile0 + tile;
    // Neighbouring threads take neighbouring rows of W: their stores share cache lines.
    if (EP == FL_PARTS) {
      const int r16 = tid % 16, xc = tid / 16;
      const long row = (long)tl * 16 + r16;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int xr = t * 16 + xc;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) v += pb[(w * NT + t) * FL_TILE + xc * 17 + r16];
        if (row < m && xr < n) reinterpret_cast<float*>(out.y)[((long)blockIdx.y * n + xr) * m + row] = v;
      }
    } else if (tid < 128) {
      const int p8 = tid % 8, xc = tid / 8;
      const int pair = tl * 8 + p8, pairs = m / 2;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int xr = t * 16 + xc;
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          a += pb[(w * NT + t) * FL_TILE + xc * 17 + p8];
          b += pb[(w * NT + t) * FL_TILE + xc * 17 + p8 + 8];
        }
        if (pair >= pairs || xr >= n) continue;
        if (EP == FL_SWIGLU) {
          bf16_t* h = reinterpret_cast<bf16_t*>(out.y);
          h[(long)xr * pairs + pair] = from_f32<bf16_t>(gate_act(a, out.act) * b);
        } else {
          const int half = out.hd / 2;
          const int q_pairs = out.H * half, k_pairs = out.cache ? out.KV * half : 0;
          const int region = pair < q_pairs ? 0 : pair < q_pairs + k_pairs ? 1 : 2;
          const int page = ep_page[t], slot = ep_slot[t];
          const long block = (long)out.page_size * out.hd;
          if (region < 2) {
            const int p = region ? pair - q_pairs : pair;
            const int head = p / half, j = p % half;
            const float cc = ep_cos[t], sn = ep_sin[t];
            const float ra = a * cc - b * sn, rb = b * cc + a * sn;
            bf16_t* o = region == 0
                            ? reinterpret_cast<bf16_t*>(out.y) + ((long)xr * out.H + head) * out.hd
                            : reinterpret_cast<bf16_t*>(out.cache) +
                                  (((long)page * 2 + 0) * out.KV + head) * block + (long)slot * out.hd;
            o[j] = from_f32<bf16_t>(ra);
            o[j + half] = from_f32<bf16_t>(rb);
          } else {
            const int e = 2 * (pair - q_pairs - k_pairs);
            const int head = e / out.hd, j = e % out.hd;
            bf16_t* v = reinterpret_cast<bf16_t*>(out.cache) + (((long)page * 2 + 1) * out.KV + head) * block;
            v[(long)j * out.page_size + slot] = from_f32<bf16_t>(a);
            v[(long)(j + 1) * out.page_size + slot] = from_f32<bf16_t>(b);
          }
        }
      }
    }
    rope_angles(tile + 1);
  }
}

static size_t fl_lds_bytes(int n, int nt, int kslice) {
  return (size_t)n * (kslice + FL_PAD) * sizeof(bf16_t) + (size_t)(2 * 4 * nt * FL_TILE) * sizeof(float);
}

template <int NT, int EP>
static int fl_launch(const void* x, const FlOut& out, const void* w, int n, int m, int k, int kslice,
                     int nsplit, int tiles, int tiles_per_wg, int x_stride, hipStream_t stream) {
  const size_t lds = fl_lds_bytes(n, NT, kslice);
  static size_t allowed = 64 * 1024;
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)fused_linear_kernel<NT, EP>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, FL_LDS_MAX);
    if (e != hipSuccess) KLLM_FAIL((int)e, "fused_linear: cannot raise the LDS limit: %s", hipGetErrorString(e));
    allowed = FL_LDS_MAX;
  }
  const dim3 grid(ceil_div(tiles, tiles_per_wg), nsplit);
  hipLaunchKernelGGL((fused_linear_kernel<NT, EP>), grid, dim3(256), lds, stream, (const bf16_t*)x, out,
                     (const bf16_t*)w, n, m, k, kslice, tiles, tiles_per_wg, x_stride);
  return 0;
}

template <int NT>
static int fl_launch_ep(int ep, const void* x, const FlOut& out, const void* w, int n, int m, int k,
                        int kslice, int nsplit, int tiles, int tpw, int xs, hipStream_t st) {
  switch (ep) {
    case FL_PARTS: return fl_launch<NT, FL_PARTS>(x, out, w, n, m, k, kslice, nsplit, tiles, tpw, xs, st);
    case FL_SWIGLU: return fl_launch<NT, FL_SWIGLU>(x, out, w, n, m, k, kslice, nsplit, tiles, tpw, xs, st);
    default: return fl_launch<NT, FL_ROPE>(x, out, w, n, m, k, kslice, nsplit, tiles, tpw, xs, st);
  }
}

}  // namespace kllm

using namespace kllm;

static bool fl_aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

extern "C" long kllm_fused_linear_lds_bytes(int n, int k, int nsplit) {
  if (n <= 0 || k <= 0 || nsplit <= 0) return -1;
  const int kslice = ceil_div(ceil_div(k, nsplit), 32) * 32;
  return (long)fl_lds_bytes(n, ceil_div(n, 16), kslice);
}

extern "C" int kllm_fused_linear(const void* x, int x_stride, const KllmLinearOut* yout, const void* w,
                                 int n, int m, int k, int tiles_per_wg, hipStream_t stream) {
  KLLM_REQUIRE(x && yout && w && yout->y, "fused_linear: null pointer");
  KLLM_REQUIRE(n > 0 && n <= KLLM_FUSED_LINEAR_MAX_ROWS, "fused_linear: n=%d is outside [1, %d]", n,
               KLLM_FUSED_LINEAR_MAX_ROWS);
  KLLM_REQUIRE(m > 0 && k > 0 && k % 8 == 0, "fused_linear: bad sizes m=%d k=%d (K must be a multiple of 8)", m, k);
  KLLM_REQUIRE((long)m * k < (1L << 40) && m < (1 << 30), "fused_linear: sizes overflow");
  KLLM_REQUIRE(fl_aligned16(w) && fl_aligned16(x), "fused_linear: operands must be 16-byte aligned");
  KLLM_REQUIRE(tiles_per_wg >= 1 && tiles_per_wg <= 64, "fused_linear: %d tiles per workgroup", tiles_per_wg);
  const int ep = yout->kind;
  KLLM_REQUIRE(ep == FL_PARTS || ep == FL_SWIGLU || ep == FL_ROPE, "fused_linear: unknown output kind %d", ep);
  const int nsplit = yout->nsplit;
  KLLM_REQUIRE(nsplit >= 1 && nsplit <= 64, "fused_linear: nsplit %d is outside [1, 64]", nsplit);
  KLLM_REQUIRE(nsplit == 1 || ep == FL_PARTS, "fused_linear: K is split only for partial sums");
  const int kslice = ceil_div(ceil_div(k, nsplit), 32) * 32;
  KLLM_REQUIRE((long)kslice * (nsplit - 1) < k, "fused_linear: nsplit %d leaves an empty slice of K=%d", nsplit, k);
  const int nt = ceil_div(n, 16);
  KLLM_REQUIRE(fl_lds_bytes(n, nt, kslice) <= (size_t)FL_LDS_MAX,
               "fused_linear: %d rows of K=%d need %zu bytes of LDS, more than %d", n, kslice,
               fl_lds_bytes(n, nt, kslice), FL_LDS_MAX);
  if (x_stride <= 0) x_stride = k;
  KLLM_REQUIRE(x_stride >= k && x_stride % 8 == 0, "fused_linear: row stride %d of x does not fit K=%d", x_stride, k);

  FlOut out = {};
  out.y = yout->y;
  out.act = yout->act;
  KLLM_REQUIRE(ep != FL_SWIGLU || (out.act >= 0 && out.act < ACT_COUNT), "fused_linear: unknown activation %d", out.act);
  int tiles = ceil_div(m, 16);
  if (ep == FL_SWIGLU || ep == FL_ROPE) {
    KLLM_REQUIRE(m % 2 == 0, "fused_linear: m=%d must be even for a pair epilogue", m);
    tiles = ceil_div(m / 2, 8);
  }
  if (ep == FL_ROPE) {
    const int H = yout->H, KV = yout->KV, hd = yout->hd;
    KLLM_REQUIRE(H > 0 && hd > 0 && hd % 2 == 0, "fused_linear: bad heads H=%d hd=%d", H, hd);
    KLLM_REQUIRE((yout->cos_t == nullptr) == (yout->sin_t == nullptr), "fused_linear: cos and sin go together");
    if (yout->cache)
      KLLM_REQUIRE(KV > 0 && yout->positions && yout->span_of_token && yout->block_table &&
                       yout->max_pages > 0 && yout->page_size > 0,
                   "fused_linear: bad cache arguments");
    KLLM_REQUIRE(m == H * hd + (yout->cache ? 2 * KV * hd : 0), "fused_linear: m=%d does not fit the heads", m);
    out.cos_t = yout->cos_t;
    out.sin_t = yout->sin_t;
    out.cache = yout->cache;
    out.positions = yout->positions;
    out.span_of_token = yout->span_of_token;
    out.block_table = yout->block_table;
    out.max_pages = yout->max_pages;
    out.page_size = yout->page_size;
    out.H = H;
    out.KV = KV;
    out.hd = hd;
  }
  const int rc = nt == 1 ? fl_launch_ep<1>(ep, x, out, w, n, m, k, kslice, nsplit, tiles, tiles_per_wg, x_stride, stream)
                         : fl_launch_ep<2>(ep, x, out, w, n, m, k, kslice, nsplit, tiles, tiles_per_wg, x_stride, stream);
  if (rc) return rc;
  KLLM_CHECK_LAUNCH("fused_linear");
  return 0;
}
