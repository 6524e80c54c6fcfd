// Prompt attention over the paged cache on the matrix cores (bfloat16).
//
// One wave takes 32 consecutive tokens of one request (a query tile) and one
// head, and walks the request's keys in tiles of 32, from the first key any of
// its queries may read to the last: earlier pages of the cache and the rows
// this step has just written alike, so a prompt's portion at a position > 0
// needs no other path.  Running maximum and sum per query (online softmax), no
// score matrix in memory, context bounded by pages only.  Formulas as in the
// generic kernel (reference: backend/model.cu:343-408, window :224-225), in
// 32-bit; probabilities are rounded to bfloat16 for the product with the values.
//
// The scores are computed transposed, S^T = K Q^T, so that a query is a
// column: MFMA 32x32x16, lane l (g = l/32, c = l%32) holds A[c][8g..8g+7],
// B[8g..8g+7][c] and D[8(i/4) + 4g + i%4][c], i = 0..15.  A = 32 keys x 16 of
// hd, one key row per lane straight from its page; B = q of 32 tokens.  A lane
// then holds 16 scores of one query, its partner lane (l ^ 32) the other 16:
// maximum and sum need one exchange.  For the values, O^T += V^T P^T, the 16 k
// slots of MFMA u are the keys 16u + 8(j/4) + 4g + j%4, j = 0..7 -- exactly the
// scores D[8u + j] a lane holds -- and A = values [hd row c][those keys], two
// 8-byte reads from the [hd][slot] value layout of one page.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kPrefillWaves = 4;
constexpr int kQueryTile = 32;

template <int HDT>  // head_dim = 32 * HDT
__global__ __launch_bounds__(64 * kPrefillWaves) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ query_tiles, int n_tiles, const int* __restrict__ span_start,
    const int* __restrict__ span_pos, const int* __restrict__ block_table, int max_pages,
    int page_size, int H, int KV, int window, float scale) {
  constexpr int hd = 32 * HDT;
  constexpr int KS = hd / 16;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 32, c = lane % 32;
  const long item = (long)blockIdx.x * kPrefillWaves + wave;   // (tile, head), head fastest
  if (item >= (long)n_tiles * H) return;
  const int tile = n_tiles - 1 - (int)(item / H), h = item % H;   // later tiles read more keys: start them first
  const int kvh = h / (H / KV);
  const int t0 = query_tiles[2 * tile], span = query_tiles[2 * tile + 1];
  const int s_begin = span_start[span], s_end = span_start[span + 1];
  const int pos0 = span_pos[span];
  const int kv_len = pos0 + (s_end - s_begin);              // keys of the request after this step
  const int nq = min(kQueryTile, s_end - t0);               // queries of this tile
  const int tq = t0 + min(c, nq - 1);                       // this lane's query (clamped)
  const int qpos = pos0 + (tq - s_begin);
  const int qpos_min = pos0 + (t0 - s_begin), qpos_max = qpos_min + nq - 1;
  const int lowest = (window > 0) ? max(0, qpos_min - window + 1) : 0;   // first key any query reads
  const int my_start = (window > 0) ? max(0, qpos - window + 1) : 0;
  const int* table = block_table + (long)span * max_pages;
  const long block = (long)page_size * hd;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const float c2 = scale * 1.4426950408889634f;             // scale * log2(e)

  bf16x8 qb[KS];
#pragma unroll
  for (int kk = 0; kk < KS; ++kk)
    qb[kk] = *reinterpret_cast<const bf16x8*>(q + ((long)tq * H + h) * hd + 16 * kk + 8 * g);

  float m = -INFINITY, l = 0.f;
  floatx16 acc[HDT];
#pragma unroll
  for (int r = 0; r < HDT; ++r)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[r][i] = 0.f;

  // One tile's operands.  The loads of tile i+1 go out before tile i is
  // computed; its page ids were read one tile earlier still.
  struct Tile {
    bf16x8 k[KS];
    bf16x4 vlo[HDT][2], vhi[HDT][2];
    bool row_ok, live[2];
  };
  const int kb0 = lowest / 32 * 32;
  const int first_page_key = lowest / page_size * page_size;   // pages before this may be gone
  auto pages_of = [&](int kb, int& prow, int& p0, int& p1) {
    const int key_row = kb + c;
    const bool in = kb <= qpos_max;
    prow = (in && key_row < kv_len && key_row >= first_page_key) ? table[key_row / page_size] : -1;
    p0 = (in && kb < kv_len && kb + 16 > lowest) ? table[kb / page_size] : -1;
    p1 = (in && kb + 16 < kv_len && kb + 32 > lowest) ? table[(kb + 16) / page_size] : -1;
  };
  auto fetch = [&](int kb, int prow, int p0, int p1) -> Tile {
    Tile T;
    const int key_row = kb + c;
    T.row_ok = prow >= 0;
    const bf16_t* krow = cache + (((long)(T.row_ok ? prow : 0) * 2 + 0) * KV + kvh) * block +
                         (long)(key_row % page_size) * hd;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      T.k[kk] = T.row_ok ? *reinterpret_cast<const bf16x8*>(krow + 16 * kk + 8 * g) : zero8;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int vp = u ? p1 : p0;
      const int k0 = kb + 16 * u;
      T.live[u] = vp >= 0;
      const bf16_t* vbase = cache + (((long)(T.live[u] ? vp : 0) * 2 + 1) * KV + kvh) * block + (k0 % page_size);
#pragma unroll
      for (int r = 0; r < HDT; ++r) {
        const bf16_t* vrow = vbase + (long)(32 * r + c) * page_size;
        T.vlo[r][u] = T.live[u] ? *reinterpret_cast<const bf16x4*>(vrow + 4 * g) : bf16x4{0, 0, 0, 0};
        T.vhi[r][u] = T.live[u] ? *reinterpret_cast<const bf16x4*>(vrow + 8 + 4 * g) : bf16x4{0, 0, 0, 0};
      }
    }
    return T;
  };

  int prow, pg0, pg1;
  pages_of(kb0, prow, pg0, pg1);
  Tile nxt = fetch(kb0, prow, pg0, pg1);
  pages_of(kb0 + 32, prow, pg0, pg1);
  for (int kb = kb0; kb <= qpos_max; kb += 32) {
    const Tile cur = nxt;
    nxt = fetch(kb + 32, prow, pg0, pg1);
    pages_of(kb + 64, prow, pg0, pg1);
    // ---- scores: this lane's key row is kb + c
    floatx16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur.k[kk], qb[kk], s, 0, 0, 0);
    // ---- mask (only where a tile touches an edge), maximum, probabilities.
    // exp(x) is taken as exp2(x * log2 e) with the hardware's exp2.
    const bool inner = kb >= my_start && kb + 31 <= qpos && kb + 32 <= kv_len;   // no mask needed
    if (__any(!inner)) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = kb + 8 * (i / 4) + 4 * g + i % 4;
        const bool ok = inner || (key <= qpos && key >= my_start);
        s[i] = ok ? s[i] : -INFINITY;
      }
    }
    float tmax = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) tmax = fmaxf(tmax, s[i]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m, tmax);                       // in units of raw scores
    const float mc = (m_new == -INFINITY) ? 0.f : m_new * c2;
    const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m * c2 - mc);
    bf16x8 pb[2];
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = __builtin_amdgcn_exp2f(fmaf(s[i], c2, -mc));   // exp2(-inf) = 0
      pb[i / 8][i % 8] = (bf16_t)p;
      psum += p;
    }
    l = l * alpha + psum;
    m = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[r][i] *= alpha;
    }
    // ---- values: page u of this tile holds keys kb + 16u .. kb + 16u + 15
    const bool v_edge = kb < lowest || kb + 32 > kv_len;     // slots that may hold anything
    if (!v_edge) {
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          bf16x8 a;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            a[j] = cur.vlo[r][u][j];
            a[4 + j] = cur.vhi[r][u][j];
          }
          acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[u], acc[r], 0, 0, 0);
        }
    } else {
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int k0 = kb + 16 * u;
          bf16x8 a;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int key_lo = k0 + 4 * g + j, key_hi = k0 + 8 + 4 * g + j;
            a[j] = (cur.live[u] && key_lo >= lowest && key_lo < kv_len) ? cur.vlo[r][u][j] : (bf16_t)0.f;
            a[4 + j] = (cur.live[u] && key_hi >= lowest && key_hi < kv_len) ? cur.vhi[r][u][j] : (bf16_t)0.f;
          }
          acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[u], acc[r], 0, 0, 0);
        }
    }
  }

  l += __shfl_xor(l, 32, kWave);
  if (c >= nq) return;
  const float inv = 1.f / l;
  bf16_t* orow = out + ((long)tq * H + h) * hd;
#pragma unroll
  for (int r = 0; r < HDT; ++r)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      bf16x4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (bf16_t)(acc[r][4 * b + j] * inv);
      *reinterpret_cast<bf16x4*>(orow + 32 * r + 8 * b + 4 * g) = v;
    }
}

template <int HDT>
static void launch_prefill(int grid, hipStream_t stream, const void* q, void* out, const void* cache,
                           const int* query_tiles, int n_tiles, const int* span_start,
                           const int* span_pos, const int* block_table, int max_pages, int page_size,
                           int H, int KV, int window, float scale) {
  hipLaunchKernelGGL(attn_prefill_mfma_kernel<HDT>, dim3(grid), dim3(64 * kPrefillWaves), 0, stream,
                     (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, query_tiles, n_tiles,
                     span_start, span_pos, block_table, max_pages, page_size, H, KV, window, scale);
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_attn_prefill(const void* q, void* out, const void* cache, const int* query_tiles,
                                 int n_tiles, const int* span_start, const int* span_pos,
                                 const int* block_table, int max_pages, int page_size, int H, int KV,
                                 int hd, int window, float scale, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(q && out && cache && query_tiles && span_start && span_pos && block_table,
               "attn_prefill: null pointer");
  KLLM_REQUIRE(dtype == DT_BF16, "attn_prefill: bfloat16 only (float32 uses the generic kernel)");
  KLLM_REQUIRE(n_tiles > 0 && H > 0 && KV > 0 && H % KV == 0, "attn_prefill: bad sizes tiles=%d H=%d KV=%d",
               n_tiles, H, KV);
  KLLM_REQUIRE(hd % 32 == 0 && hd >= 32 && hd <= 256 && (hd <= 128 || hd == 192 || hd == 256),
               "attn_prefill: head_dim %d is not built (32, 64, 96, 128, 192, 256)", hd);
  KLLM_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_prefill: page_size %d must be a multiple of 16",
               page_size);
  KLLM_REQUIRE(max_pages > 0 && window >= 0, "attn_prefill: bad table width or window");
  const long items = (long)n_tiles * H;
  KLLM_REQUIRE(items < (1L << 31), "attn_prefill: too many tiles");
  const int grid = ceil_div(items, kPrefillWaves);
#define KLLM_PF(HDT)                                                                              \
  case HDT:                                                                                       \
    launch_prefill<HDT>(grid, stream, q, out, cache, query_tiles, n_tiles, span_start, span_pos,  \
                        block_table, max_pages, page_size, H, KV, window, scale);                 \
    break
  switch (hd / 32) {
    KLLM_PF(1); KLLM_PF(2); KLLM_PF(3); KLLM_PF(4); KLLM_PF(6); KLLM_PF(8);
    default: KLLM_FAIL(ERR_ARG, "attn_prefill: head_dim %d is not built", hd);
  }
#undef KLLM_PF
  KLLM_CHECK_LAUNCH("attn_prefill");
  return 0;
}
