// Matrix products of a decode batch (up to 32 rows of X, bfloat16) on MFMA, with
// the step after the product done in the same launch.  Y = X . W^T, then
//
//   PARTS    float32 sums [nsplit, n, m] (only this one may split K);
//   RESID    the sums are added to the float32 residual stream in place; the
//            new rows times the weight of the RMS norm behind the addition go
//            out in bfloat16, and each workgroup leaves the sums of squares of
//            its columns of the new rows (reference: the fused add + norm,
//            backend/model.cu:144-165, here without a launch of its own);
//   SWIGLU   silu(gate) * up in bfloat16 (reference backend/model.cu:477-483);
//   ROPE     rotated queries and keys, and values, written to q_out and to
//            the tokens' pages (reference backend/model.cu:170-201).
//
// The consumer of a RESID product (SWIGLU or ROPE, `SCALED`) reads those
// bfloat16 rows x * w as its X and multiplies its float32 sums by the row's
// rsqrt(sum of squares / K + eps): the RMS norm without a kernel of its own
// and with 16-bit staging.  Against the norm kernel the rounding to bfloat16
// happens before the row scale instead of after it; both round every element
// of the normalised row once.
//
// A workgroup owns tiles of 16 rows of W and one slice of K (all of K unless
// the caller splits).  It puts its slice of X, all rows, into LDS once (where
// they do not fit, in several passes over K, with one tile to a workgroup whose
// sums stay in registers from pass to pass).  Each
// of its four or eight waves (see fl_waves) takes its share of the slice: it
// streams its part of the 16 rows of W straight from memory, eight 16-byte loads
// per lane in flight, the first of them before X is staged, and multiplies with
// X from LDS (MFMA 16x16x32: A = W tile, B = X^T, D[w row][x row]).  The waves'
// partial tiles meet in LDS, are added in a fixed order, and the epilogue runs on
// the sums; no partial sum crosses memory unless the caller splits K.
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

// W loads per lane in one of the two buffers.  Four, not more: in a decode step the kernel runs
// with a cold instruction cache, and its time follows its code size (8 ahead: 2,000 instructions
// and 6.7 us for 2,048 x 2,048 weights at 8 rows; 4 ahead: 1,660 and 6.0 us; more waves to a
// workgroup or more of X in registers measured slower for the same reason).
constexpr int FL_AHEAD = 4;
// LDS row padding (elements): zeros behind K as far as the waves' slices reach beyond it
// (less than 32 per wave), 8 to shift banks
constexpr int fl_pad(int nw) { return 32 * nw + 8; }
constexpr int FL_SS_LOADS = 4;     // 16-byte loads per lane of a row's partial sums of squares: 16 lanes a row
constexpr int FL_SS_MAX = 16 * 4 * FL_SS_LOADS;   // partial sums of squares per row at most
constexpr int FL_LDS_MAX = 160 * 1024;
constexpr int FL_TILE = 16 * 17;    // floats of one wave's partial tile in LDS: [x row][w row], padded

enum : int { FL_PARTS = 0, FL_RESID = 1, FL_SWIGLU = 2, FL_ROPE = 3 };

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
  float* resid;                 // FL_RESID: the residual stream [n][m]; y receives bfloat16 resid * norm_w
  const float* norm_w;          // FL_RESID: weight [m] of the norm behind the addition
  float* ss_out;                // FL_RESID: [n][workgroups rounded up to 4] sums of squares of the new rows
  const float* ss_in;           // SCALED: [n][ss_parts rounded up to 4], what a FL_RESID product left
  int ss_parts;
  float eps;
  int tiled;                    // W is the copy that fl_tile_kernel made for this epilogue (see there)
};

// Row of W behind MFMA row c of a tile, or -1.  Pair epilogues: unit = pair.
template <int EP>
__device__ __forceinline__ long fl_row(int tile, int c, int m, const FlOut& o) {
  if (EP == FL_PARTS || EP == FL_RESID) {
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

// NW waves share a tile's K; SCALED: the sums are multiplied by a row scale made from out.ss_in;
// PASSES: the rows of X do not fit into LDS at once and go in passes of kpass of K (a kernel of
// its own, so that the one for rows that fit carries none of it).
template <int NT, int EP, int NW, bool SCALED, bool PASSES>
__global__ __launch_bounds__(64 * NW) void fused_linear_kernel(const bf16_t* __restrict__ X, FlOut out,
                                                           const bf16_t* __restrict__ W, int n, int m,
                                                           int k, int kslice, int tiles, int tiles_per_wg,
                                                           int x_stride, int kpass) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int ld = kpass + fl_pad(NW);
  bf16_t* xs = reinterpret_cast<bf16_t*>(lds_raw);                            // [n][ld]
  float* part = reinterpret_cast<float*>(lds_raw + (size_t)n * ld * sizeof(bf16_t));   // [2][NW][NT][x row 16][17]
  float* row_scale = part + 2 * NW * NT * FL_TILE;                            // [32]

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int g = lane / 16, c = lane % 16;
  const int kbeg = blockIdx.y * kslice;
  const int klen = min(k, kbeg + kslice) - kbeg;            // a multiple of 8
  // The slice is staged and multiplied in passes of kpass of K (one pass where all rows of the slice
  // fit into LDS; several only with one tile to a workgroup, whose sums then stay in registers).
  const int npass = PASSES ? (klen + kpass - 1) / kpass : 1;
  auto pass_len = [&](int pass) { return PASSES ? min(klen - pass * kpass, kpass) : klen; };
  const int kw = ((pass_len(0) + NW - 1) / NW + 31) / 32 * 32;     // K of one wave in a pass
  const int wk0 = wave * kw;                                // this wave's offset in the pass
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

  // ---- X: wave w stages rows w, w + NW, ... of the slice straight into LDS, a kilobyte (512 of
  // K) per instruction, without passing registers: all of them are in flight at once however
  // many rows there are, before the weights are asked for (loads return in order).
  auto stage = [&](int pass) {
    const int plen = pass_len(pass);
    const int kchunks = (plen + 511) / 512;
    for (int r = wave; r < n; r += NW) {
      const bf16_t* src = X + (long)r * x_stride + kbeg + pass * kpass + lane * 8;
      bf16_t* dst = xs + r * ld;
      for (int ch = 0; ch < kchunks; ++ch)
        if (ch * 512 + lane * 8 < plen)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + ch * 512),
                                           (__attribute__((address_space(3))) void*)(dst + ch * 512), 16, 0, 0);
    }
  };
  stage(0);
  asm volatile("" ::: "memory");     // no later load moves in front of these: the wait below counts on it

  // ---- SCALED: a row's partial sums of squares, sixteen lanes to a row, asked for behind X
  // and before the weights (loads return in order)
  floatx4 ssv[SCALED ? NT : 1][FL_SS_LOADS];
  if (SCALED) {
    const int stride = (out.ss_parts + 3) / 4 * 4;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < FL_SS_LOADS; ++i) {
        const int at = 4 * (tid % 16 + 16 * i);
        ssv[t][i] = *reinterpret_cast<const floatx4*>(out.ss_in + (long)min(t * 16 + (tid / 16) % 16, n - 1) * stride +
                                                      (at < stride ? at : 0));
      }
  }
  // ---- FL_RESID: thread (w row tid % 16, x row tid / 16) adds to resid[x row][w row]; the old
  // value and the norm's weight are asked for now and needed in the epilogue
  float res_old[EP == FL_RESID ? NT : 1], res_w = 0.f;
  float ss_acc[EP == FL_RESID ? NT : 1];
  auto resid_load = [&](int tile_index) {
    if (EP != FL_RESID) return;
    const long row = (long)(tile0 + tile_index) * 16 + tid % 16;
    const bool live = tid < 256 && row < m && tile_index < my_tiles;
    // The indices pass through a register that the compiler cannot see into: left to itself it
    // turns the choice of an index into a branch around two loads, and with a load inside a branch
    // every wait of the loop becomes a wait for all loads in flight.
    long at = live ? row : 0;
    asm volatile("" : "+v"(at));
    res_w = out.norm_w[at];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int xr = t * 16 + tid / 16;
      at = live && xr < n ? (long)xr * m + row : 0;
      asm volatile("" : "+v"(at));
      res_old[t] = out.resid[at];
    }
  };
  if (EP == FL_RESID) {
#pragma unroll
    for (int t = 0; t < NT; ++t) ss_acc[t] = 0.f;
    resid_load(0);
  }

  // ---- W: two buffers of FL_AHEAD loads each, used in turn: while one is multiplied the
  // other is on its way, and it is asked for again as soon as it has been used.  No register
  // is copied from one buffer to the other (a copy would have to wait for its load).  A tile's
  // steps are padded to whole turns of both buffers.  A row, a tile or a K that does not exist
  // reads the first K of a row that does (finite numbers): the X beside it in LDS is zero, or
  // the output row is ignored.
  // With a tiled copy of W (out.tiled) a tile's step is 1 KB in the order the lanes want it:
  // a load instruction reads one contiguous kilobyte instead of 64 bytes of each of 16 rows
  // (streamed alone, 2,048 x 5,632 weights: 8.5 -> 6.7 us; 11,264 x 2,048: 12.0 -> 9.9).
  const bf16_t* far_row;                                    // first K of this lane's row of W
  int far_lane_off;                                         // this lane's offset in it, or -1: no such row
  const int far_stride = out.tiled ? 512 : 32;              // elements from a step to the next
  int far_tile = 0, far_s0 = 0;                             // the steps that are loaded next; a tile's passes count as tiles
  int far_wlen = 0;                                         // this wave's K in that pass
  auto tile_ptr = [&](int u) {
    const int t = PASSES ? u / npass : u, pass = PASSES ? u % npass : 0;
    const int pbeg = kbeg + pass * kpass;
    far_wlen = max(0, min(pass_len(pass), wk0 + kw) - wk0);
    if (out.tiled) {     // rows that do not exist hold zeros there; a tile that does not exist reads the first
      const long tl = t < my_tiles ? tile0 + t : tile0;
      far_row = W + ((tl * ((k + 31) / 32) + pbeg / 32) * kWave + lane) * 8;
      far_lane_off = (wk0 / 32) * 512;
      return;
    }
    const long r = t < my_tiles ? fl_row<EP>((int)tile0 + t, c, m, out) : -1;
    far_row = W + (r >= 0 ? r : 0) * k + pbeg;
    far_lane_off = r >= 0 ? wk0 + 8 * g : -1;
  };
  auto fill = [&](bf16x8 (&buf)[FL_AHEAD]) {
#pragma unroll
    for (int i = 0; i < FL_AHEAD; ++i) {
      const int s = far_s0 + i;
      const bool valid = far_lane_off >= 0 && s < steps && 32 * s + 8 * g < far_wlen;
      buf[i] = *reinterpret_cast<const bf16x8*>(far_row + (valid ? far_lane_off + far_stride * s : 0));
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

  auto zero_behind = [&](int pass) {   // zeros in X's columns from the K of the pass to where the waves' slices reach
    constexpr int per_row = 4 * NW;                         // threads to 32 * NW zeros of a row: 16 rows at a time
    const int plen = pass_len(pass);                        // (a last pass may be shorter than the others)
    const int r = tid / per_row;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (t * 16 + r < n) {
        if (!PASSES) {   // all passes alike: the slices reach less than 32 NW beyond
          *reinterpret_cast<bf16x8*>(&xs[(t * 16 + r) * ld + plen + 8 * (tid % per_row)]) = zero;
        } else {
          for (int at = plen + 8 * (tid % per_row); at < NW * kw; at += 8 * per_row)
            *reinterpret_cast<bf16x8*>(&xs[(t * 16 + r) * ld + at]) = zero;
        }
      }
  };
  zero_behind(0);
  if (SCALED) {   // the rows' scales: sums in a fixed order, then across the row's sixteen lanes
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float v = 0.f;
#pragma unroll
      for (int i = 0; i < FL_SS_LOADS; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) v += 4 * (tid % 16 + 16 * i) + e < out.ss_parts ? ssv[t][i][e] : 0.f;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
      if (tid % 16 == 0 && tid < 256) row_scale[t * 16 + tid / 16] = rsqrtf(v / (float)k + out.eps);
    }
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
  {
    // X has landed in LDS when at most the loads that every wave issued behind it are still in
    // flight: the sums of squares, the residual values and the two buffers of weights (loads of
    // the rotation epilogue, which not every wave issues, come behind those and only make
    // the wait a little longer).
    constexpr int behind = (SCALED ? NT * FL_SS_LOADS : 0) + (EP == FL_RESID ? 1 + NT : 0) + 2 * FL_AHEAD;
    static_assert(behind < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt((behind & 0xF) | ((behind >> 4) << 14) | 0x0F70);
  }
  fl_lds_barrier();

  floatx4 acc[NT];
  const bf16_t* xrow[NT];                                   // rows beyond n are ignored: they read row n - 1
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    xrow[t] = xs + min(t * 16 + c, n - 1) * ld + wk0 + 8 * g;
  }
  // A buffer's steps: all their rows of X are asked of LDS first, without a branch between them, so
  // that LDS answers while the wave still waits for the weights; a step beyond the wave's last
  // multiplies with zeros (its weights are whatever the first K of the row holds).
  auto multiply = [&](const bf16x8 (&buf)[FL_AHEAD], int s0) {
    bf16x8 b[FL_AHEAD][NT];
#pragma unroll
    for (int i = 0; i < FL_AHEAD; ++i)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        b[i][t] = *reinterpret_cast<const bf16x8*>(xrow[t] + 32 * min(s0 + i, steps - 1));
#pragma unroll
    for (int i = 0; i < FL_AHEAD; ++i) {
      const bool live = s0 + i < steps;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[i], live ? b[i][t] : zero, acc[t], 0, 0, 0);
    }
  };

  for (int tile = 0; tile < my_tiles; ++tile) {
    for (int pass = 0; pass < npass; ++pass) {
      if (PASSES && pass > 0) {
        // the next columns of X take the place of the ones that every wave has multiplied; the
        // weights asked for ahead are older loads and arrive on the way
        fl_lds_barrier();
        stage(pass);
        zero_behind(pass);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70);                 // vmcnt(0)
        fl_lds_barrier();
      }
      for (int s0 = 0; s0 < rsteps; s0 += 2 * FL_AHEAD) {
        multiply(bufa, s0);
        fill(bufa);
        multiply(bufb, s0 + FL_AHEAD);
        fill(bufb);
      }
    }
    // ---- the tile is complete in this wave: meet the other waves in LDS
    float* pb = part + (tile & 1) * NW * NT * FL_TILE;
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
      const int r16 = tid % 16, xc = (tid / 16) % 16;       // (with more than four waves the others repeat the stores)
      const long row = (long)tl * 16 + r16;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int xr = t * 16 + xc;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += pb[(w * NT + t) * FL_TILE + xc * 17 + r16];
        if (row < m && xr < n) reinterpret_cast<float*>(out.y)[((long)blockIdx.y * n + xr) * m + row] = v;
      }
    } else if (EP == FL_RESID) {
      if (tid < 256) {
        const int r16 = tid % 16, xc = tid / 16;
        const long row = (long)tl * 16 + r16;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const int xr = t * 16 + xc;
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < NW; ++w) v += pb[(w * NT + t) * FL_TILE + xc * 17 + r16];
          if (row < m && xr < n) {
            const float x = res_old[t] + v;
            out.resid[(long)xr * m + row] = x;
            reinterpret_cast<bf16_t*>(out.y)[(long)xr * m + row] = from_f32<bf16_t>(x * res_w);
            ss_acc[t] += x * x;
          }
        }
      }
      resid_load(tile + 1);
    } else if (tid < 128) {
      const int p8 = tid % 8, xc = tid / 8;
      const int pair = tl * 8 + p8, pairs = m / 2;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int xr = t * 16 + xc;
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
          a += pb[(w * NT + t) * FL_TILE + xc * 17 + p8];
          b += pb[(w * NT + t) * FL_TILE + xc * 17 + p8 + 8];
        }
        if (pair >= pairs || xr >= n) continue;
        if (SCALED) {
          const float rs = row_scale[xr];
          a *= rs;
          b *= rs;
        }
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
  if (EP == FL_RESID && tid < 256) {   // the workgroup's sums of squares, one per row of X
    const int stride = ((int)gridDim.x + 3) / 4 * 4;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float v = ss_acc[t];
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
      const int xr = t * 16 + tid / 16;
      if (tid % 16 == 0 && xr < n) out.ss_out[(long)xr * stride + blockIdx.x] = v;
    }
  }
}

// The tiled copy of W for an epilogue: [tile][step of 32 of K][lane][8 elements], lane (g, c)
// holding W[row of MFMA row c][32 step + 8 g ...], zeros where the row or the K is not there.
// One workgroup of 64 lanes per (tile, step).
template <int EP>
__global__ __launch_bounds__(64) void fl_tile_kernel(const bf16_t* __restrict__ W, bf16_t* __restrict__ Wt, FlOut out,
                                                     int m, int k) {
  const int lane = threadIdx.x, g = lane / 16, c = lane % 16;
  const int step = blockIdx.y, ksteps = gridDim.y;
  const long tile = blockIdx.x;
  const long r = fl_row<EP>((int)tile, c, m, out);
  const int kk = 32 * step + 8 * g;
  bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (r >= 0 && kk < k) v = *reinterpret_cast<const bf16x8*>(W + r * k + kk);      // k is a multiple of 8
  *reinterpret_cast<bf16x8*>(Wt + ((tile * ksteps + step) * kWave + lane) * 8) = v;
}

static size_t fl_lds_bytes(int n, int nt, int kslice, int nw = 4) {
  return (size_t)n * (kslice + fl_pad(nw)) * sizeof(bf16_t) + (size_t)(2 * nw * nt * FL_TILE + 32) * sizeof(float);
}

template <int NT, int EP, int NW, bool SCALED, bool PASSES>
static int fl_launch_passes(const void* x, const FlOut& out, const void* w, int n, int m, int k, int kslice, int kpass,
                     int nsplit, int tiles, int tiles_per_wg, int x_stride, hipStream_t stream) {
  size_t lds = fl_lds_bytes(n, NT, kpass, NW);
  static size_t allowed = 64 * 1024;          // one per instantiation
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)fused_linear_kernel<NT, EP, NW, SCALED, PASSES>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, FL_LDS_MAX);
    if (e != hipSuccess) KLLM_FAIL((int)e, "fused_linear: cannot raise the LDS limit: %s", hipGetErrorString(e));
    allowed = FL_LDS_MAX;
  }
  const dim3 grid(ceil_div(tiles, tiles_per_wg), nsplit);
  hipLaunchKernelGGL((fused_linear_kernel<NT, EP, NW, SCALED, PASSES>), grid, dim3(64 * NW), lds, stream, (const bf16_t*)x,
                     out, (const bf16_t*)w, n, m, k, kslice, tiles, tiles_per_wg, x_stride, kpass);
  return 0;
}

template <int NT, int EP, int NW, bool SCALED>
static int fl_launch(const void* x, const FlOut& out, const void* w, int n, int m, int k, int kslice, int kpass,
                     int nsplit, int tiles, int tiles_per_wg, int x_stride, hipStream_t stream) {
  if (kpass < kslice)
    return fl_launch_passes<NT, EP, NW, SCALED, true>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tiles_per_wg,
                                                      x_stride, stream);
  return fl_launch_passes<NT, EP, NW, SCALED, false>(x, out, w, n, m, k, kslice, kslice, nsplit, tiles, tiles_per_wg,
                                                     x_stride, stream);
}

template <int NT, int NW>
static int fl_launch_nw(int ep, bool scaled, const void* x, const FlOut& out, const void* w, int n, int m, int k,
                        int kslice, int kpass, int nsplit, int tiles, int tpw, int xs, hipStream_t st) {
  switch (ep) {
    case FL_PARTS: return fl_launch<NT, FL_PARTS, NW, false>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st);
    case FL_RESID: return fl_launch<NT, FL_RESID, NW, false>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st);
    case FL_SWIGLU:
      return scaled ? fl_launch<NT, FL_SWIGLU, NW, true>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st)
                    : fl_launch<NT, FL_SWIGLU, NW, false>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st);
    default:
      return scaled ? fl_launch<NT, FL_ROPE, NW, true>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st)
                    : fl_launch<NT, FL_ROPE, NW, false>(x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st);
  }
}

template <int NT>
static int fl_launch_ep(int ep, bool scaled, int nw, const void* x, const FlOut& out, const void* w, int n, int m, int k,
                        int kslice, int kpass, int nsplit, int tiles, int tpw, int xs, hipStream_t st) {
  if (nw == 8) return fl_launch_nw<NT, 8>(ep, scaled, x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st);
  return fl_launch_nw<NT, 4>(ep, scaled, x, out, w, n, m, k, kslice, kpass, nsplit, tiles, tpw, xs, st);
}

}  // namespace kllm

using namespace kllm;

static bool fl_aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

extern "C" long kllm_fused_linear_lds_bytes(int n, int k, int nsplit) {
  if (n <= 0 || k <= 0 || nsplit <= 0) return -1;
  const int kslice = ceil_div(ceil_div(k, nsplit), 32) * 32;
  return (long)fl_lds_bytes(n, ceil_div(n, 16), kslice);
}

// K of a pass for n rows of a slice of kslice: the slice itself where its rows fit into LDS, else
// the least number of equal passes (up to FL_MAX_PASSES) whose rows do; 0 if none does.
constexpr int FL_MAX_PASSES = 8;
static int fl_pass_k(int n, int kslice, int nw = 4) {
  const int nt = ceil_div(n, 16);
  for (int passes = 1; passes <= FL_MAX_PASSES; ++passes) {
    const int kpass = ceil_div(ceil_div(kslice, passes), 32) * 32;
    if (fl_lds_bytes(n, nt, kpass, nw) <= (size_t)FL_LDS_MAX) return kpass;
  }
  return 0;
}

// Waves of a workgroup.  Eight for the epilogues whose products run on few workgroups, on five
// eighths of the CUs at most (the residual product: 128 for 2,048 columns; the rotation: 160 for 2,560): a wave's
// chain of loads is half as long (8 rows of X, 2,048 x 5,632: 9.4 -> 8.2 us; 2,048 x 2,048: 5.2 ->
// 4.9; a decode step of 8 tokens at 1.1B sizes 1.080 -> 1.042 ms).  Four for the gate, whose
// workgroups already share their CUs (eight: 1.042 -> 1.078 ms), for the logits (no difference),
// and wherever eight waves' partial tiles and padding leave no room for the rows of X; sixteen
// are slower than eight everywhere.
static int fl_waves(int ep, int n, int kslice, int kpass4, int workgroups, int tiles_per_wg) {
  if (ep != FL_RESID && ep != FL_ROPE) return 4;
  if (8 * workgroups > 5 * device_cus()) return 4;   // (4,096 x 4,096 on 256 workgroups: a step of 8 tokens at 8B sizes 4.09 -> 4.12 ms with eight)
  // Eight waves' partial tiles and padding take room from the rows of X: they may need a pass
  // more than four waves would, and still win (13 tokens at 1.1B sizes: 1.172 -> 1.16 ms; 16
  // tokens, two passes either way: 1.207 -> 1.176), but passes want one tile to a workgroup.
  // From 17 rows on a pass more loses (28 tokens: 1.59 against 1.55 ms).
  const int kpass8 = fl_pass_k(n, kslice, 8);
  if (!kpass8 || (kpass8 < kslice && (tiles_per_wg > 1 || (n > 16 && kpass4 >= kslice)))) return 4;
  return 8;
}

extern "C" int kllm_fused_linear_passes(int n, int k, int nsplit) {
  if (n <= 0 || n > KLLM_FUSED_LINEAR_MAX_ROWS || k <= 0 || nsplit <= 0) return 0;
  const int kslice = ceil_div(ceil_div(k, nsplit), 32) * 32;
  const int kpass = fl_pass_k(n, kslice);
  return kpass ? ceil_div(kslice < k ? kslice : k, kpass) : 0;
}

extern "C" int kllm_fused_linear_resid_parts(int m, int tiles_per_wg) {
  if (m <= 0 || tiles_per_wg <= 0) return -1;
  return ceil_div(ceil_div(m, 16), tiles_per_wg);
}

extern "C" int kllm_fused_linear_max_parts(void) { return FL_SS_MAX; }

static int fl_tiles(int kind, int m) { return kind == FL_SWIGLU || kind == FL_ROPE ? ceil_div(m / 2, 8) : ceil_div(m, 16); }

extern "C" long kllm_fused_linear_tiled_elements(int kind, int m, int k) {
  if (m <= 0 || k <= 0 || k % 8) return -1;
  return (long)fl_tiles(kind, m) * ceil_div(k, 32) * 512;
}

extern "C" int kllm_fused_linear_tile(const void* w, void* wt, int kind, int m, int k, int H, int KV, int hd,
                                      int with_kv, hipStream_t stream) {
  KLLM_REQUIRE(w && wt && fl_aligned16(w) && fl_aligned16(wt), "fused_linear_tile: null or unaligned pointer");
  KLLM_REQUIRE(m > 0 && k > 0 && k % 8 == 0 && m < (1 << 30), "fused_linear_tile: bad sizes m=%d k=%d", m, k);
  KLLM_REQUIRE(kind == FL_PARTS || kind == FL_RESID || kind == FL_SWIGLU || kind == FL_ROPE,
               "fused_linear_tile: unknown output kind %d", kind);
  FlOut out = {};
  if (kind == FL_SWIGLU || kind == FL_ROPE) KLLM_REQUIRE(m % 2 == 0, "fused_linear_tile: m=%d must be even for a pair epilogue", m);
  if (kind == FL_ROPE) {
    KLLM_REQUIRE(H > 0 && hd > 0 && hd % 2 == 0 && (!with_kv || KV > 0) && m == H * hd + (with_kv ? 2 * KV * hd : 0),
                 "fused_linear_tile: m=%d does not fit H=%d KV=%d hd=%d", m, H, KV, hd);
    out.H = H;
    out.KV = KV;
    out.hd = hd;
    out.cache = with_kv ? const_cast<void*>(w) : nullptr;     // only "is there a cache" is read
  }
  const dim3 grid(fl_tiles(kind, m), ceil_div(k, 32));
  KLLM_REQUIRE(grid.y <= 65535u, "fused_linear_tile: K=%d is too long", k);
  const bf16_t* wp = (const bf16_t*)w;
  bf16_t* tp = (bf16_t*)wt;
  if (kind == FL_SWIGLU) hipLaunchKernelGGL(fl_tile_kernel<FL_SWIGLU>, grid, dim3(64), 0, stream, wp, tp, out, m, k);
  else if (kind == FL_ROPE) hipLaunchKernelGGL(fl_tile_kernel<FL_ROPE>, grid, dim3(64), 0, stream, wp, tp, out, m, k);
  else hipLaunchKernelGGL(fl_tile_kernel<FL_PARTS>, grid, dim3(64), 0, stream, wp, tp, out, m, k);
  KLLM_CHECK_LAUNCH("fused_linear_tile");
  return 0;
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
  KLLM_REQUIRE(ep == FL_PARTS || ep == FL_RESID || ep == FL_SWIGLU || ep == FL_ROPE,
               "fused_linear: unknown output kind %d", ep);
  const int nsplit = yout->nsplit;
  KLLM_REQUIRE(nsplit >= 1 && nsplit <= 64, "fused_linear: nsplit %d is outside [1, 64]", nsplit);
  KLLM_REQUIRE(nsplit == 1 || ep == FL_PARTS, "fused_linear: K is split only for partial sums");
  const int kslice = ceil_div(ceil_div(k, nsplit), 32) * 32;
  KLLM_REQUIRE((long)kslice * (nsplit - 1) < k, "fused_linear: nsplit %d leaves an empty slice of K=%d", nsplit, k);
  const int nt = ceil_div(n, 16);
  const int kpass = fl_pass_k(n, kslice);
  KLLM_REQUIRE(kpass > 0, "fused_linear: %d rows of K=%d need %zu bytes of LDS, more than %d even in %d passes", n,
               kslice, fl_lds_bytes(n, nt, kslice), FL_LDS_MAX, FL_MAX_PASSES);
  KLLM_REQUIRE(kpass >= kslice || tiles_per_wg == 1,
               "fused_linear: %d rows of K=%d do not fit into LDS at once; in passes a workgroup takes one tile, not %d",
               n, kslice, tiles_per_wg);
  if (x_stride <= 0) x_stride = k;
  KLLM_REQUIRE(x_stride >= k && x_stride % 8 == 0, "fused_linear: row stride %d of x does not fit K=%d", x_stride, k);

  FlOut out = {};
  out.y = yout->y;
  out.act = yout->act;
  out.tiled = yout->tiled ? 1 : 0;
  KLLM_REQUIRE(ep != FL_SWIGLU || (out.act >= 0 && out.act < ACT_COUNT), "fused_linear: unknown activation %d", out.act);
  int tiles = ceil_div(m, 16);
  const bool scaled = yout->ss_in != nullptr;
  if (scaled) {
    KLLM_REQUIRE(ep == FL_SWIGLU || ep == FL_ROPE, "fused_linear: only the gate and the rotation epilogues scale their rows");
    KLLM_REQUIRE(yout->ss_parts >= 1 && yout->ss_parts <= FL_SS_MAX && fl_aligned16(yout->ss_in) && yout->eps >= 0.f,
                 "fused_linear: %d partial sums of squares per row are outside [1, %d], or they are not 16-byte aligned",
                 yout->ss_parts, FL_SS_MAX);
    out.ss_in = yout->ss_in;
    out.ss_parts = yout->ss_parts;
    out.eps = yout->eps;
  }
  if (ep == FL_RESID) {
    KLLM_REQUIRE(yout->resid && yout->norm_w && yout->ss_out, "fused_linear: the residual epilogue needs the stream, "
                 "the norm's weight and room for the sums of squares");
    KLLM_REQUIRE(ceil_div(tiles, tiles_per_wg) <= FL_SS_MAX, "fused_linear: %d workgroups leave more than %d sums of "
                 "squares per row (take more tiles per workgroup)", ceil_div(tiles, tiles_per_wg), FL_SS_MAX);
    out.resid = yout->resid;
    out.norm_w = yout->norm_w;
    out.ss_out = yout->ss_out;
  }
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
  const int nw = fl_waves(ep, n, kslice, kpass, ceil_div(tiles, tiles_per_wg) * nsplit, tiles_per_wg);
  const int kpass_run = nw == 4 ? kpass : fl_pass_k(n, kslice, nw);    // eight waves' partial tiles take room from the rows
  const int rc = nt == 1 ? fl_launch_ep<1>(ep, scaled, nw, x, out, w, n, m, k, kslice, kpass_run, nsplit, tiles, tiles_per_wg, x_stride, stream)
                         : fl_launch_ep<2>(ep, scaled, nw, x, out, w, n, m, k, kslice, kpass_run, nsplit, tiles, tiles_per_wg, x_stride, stream);
  if (rc) return rc;
  KLLM_CHECK_LAUNCH("fused_linear");
  return 0;
}
