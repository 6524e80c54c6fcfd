// Prompt attention over the paged cache on the matrix cores (bfloat16).
//
// A workgroup takes 32 consecutive tokens of one request (a query tile) and one
// head; its four waves share out the request's keys in tiles of 32, round
// robin, from the first key any of the queries may read to the last: earlier
// pages of the cache and the rows this step has just written alike, so a
// prompt's portion at a position > 0 needs no other path.  Running maximum and
// sum per query (online softmax) in every wave, merged in LDS at the end; no
// score matrix in memory, context bounded by pages only.  Sharing a tile's keys
// out over waves keeps the longest chain of dependent tiles short (a late
// query tile of a long prompt has many) and gives the chip four times as many
// workgroups as one wave per tile would, so that late and early tiles balance.  Formulas as in the
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
__global__ __launch_bounds__(64 * kPrefillWaves) __attribute__((amdgpu_waves_per_eu(HDT <= 2 ? 3 : 1))) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ query_tiles, int n_tiles, const int* __restrict__ span_start,
    const int* __restrict__ span_pos, const int* __restrict__ block_table, int max_pages,
    int page_size, int H, int KV, int window, float scale) {
  constexpr int hd = 32 * HDT;
  constexpr int KS = hd / 16;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 32, c = lane % 32;
  const long item = blockIdx.x;                               // (tile, head), head fastest
  const int tile = n_tiles - 1 - (int)(item / H), h = item % H;   // later tiles read more keys: start them first
  const int kvh = h / (H / KV);
  // The same for every lane: said so explicitly, which keeps the loop's page lookups and
  // address arithmetic on the scalar unit.
  const int t0 = __builtin_amdgcn_readfirstlane(query_tiles[2 * tile]);
  const int span = __builtin_amdgcn_readfirstlane(query_tiles[2 * tile + 1]);
  const int s_begin = __builtin_amdgcn_readfirstlane(span_start[span]);
  const int s_end = __builtin_amdgcn_readfirstlane(span_start[span + 1]);
  const int pos0 = __builtin_amdgcn_readfirstlane(span_pos[span]);
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

  // One tile's operands.  Two tiles are in registers: while one is multiplied the loads of
  // the wave's next one are on their way, and the page ids of the one after that.  Loads
  // carry no branch (a page or a row that does not exist reads page 0 and is masked or
  // zeroed where it is used), so that the waits count them exactly.
  struct Tile {
    bf16x8 k[KS];
    bf16x4 vlo[HDT][2], vhi[HDT][2];
    bool live[2];
  };
  const int kb0 = lowest / 32 * 32;
  // page and slot of a key: a shift and a mask when the page size is a power of two
  const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
  auto page_index = [&](int key) { return page_shift >= 0 ? key >> page_shift : key / page_size; };
  auto page_slot = [&](int key) { return page_shift >= 0 ? key & (page_size - 1) : key % page_size; };
  const int first_page_key = page_index(lowest) * page_size;   // pages before this may be gone
  struct Pages {
    int row, p0, p1;
  };
  auto pages_of = [&](int kb) -> Pages {
    Pages P = {-1, -1, -1};
    if (kb > qpos_max) return P;
    const int key_row = kb + c;
    const bool in = true;
    const bool rok = in && key_row < kv_len && key_row >= first_page_key;
    const bool ok0 = in && kb < kv_len && kb + 16 > lowest;
    const bool ok1 = in && kb + 16 < kv_len && kb + 32 > lowest;
    P.row = table[rok ? page_index(key_row) : 0];
    P.p0 = table[ok0 ? page_index(kb) : 0];
    P.p1 = table[ok1 ? page_index(kb + 16) : 0];
    P.row = rok ? P.row : -1;
    P.p0 = ok0 ? P.p0 : -1;
    P.p1 = ok1 ? P.p1 : -1;
    return P;
  };
  auto fetch = [&](int kb, const Pages& P) -> Tile {
    Tile T = {};
    if (kb > qpos_max) return T;                              // beyond the last tile: same for all lanes
    const int key_row = kb + c;
    const bf16_t* krow = cache + (((long)max(P.row, 0) * 2 + 0) * KV + kvh) * block +
                         (long)page_slot(key_row) * hd;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) T.k[kk] = *reinterpret_cast<const bf16x8*>(krow + 16 * kk + 8 * g);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int vp = u ? P.p1 : P.p0;
      T.live[u] = vp >= 0;
      const bf16_t* vbase = cache + (((long)max(vp, 0) * 2 + 1) * KV + kvh) * block + page_slot(kb + 16 * u);
#pragma unroll
      for (int r = 0; r < HDT; ++r) {
        const bf16_t* vrow = vbase + (long)(32 * r + c) * page_size;
        T.vlo[r][u] = *reinterpret_cast<const bf16x4*>(vrow + 4 * g);
        T.vhi[r][u] = *reinterpret_cast<const bf16x4*>(vrow + 8 + 4 * g);
      }
    }
    return T;
  };

  auto compute = [&](const Tile& cur, int kb) {
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
  };

  // A and B take turns, so that no tile is copied from register to register.
  constexpr int kStride = 32 * kPrefillWaves;                 // keys between a wave's tiles
  const int kfirst = kb0 + 32 * wave;
  Pages P = pages_of(kfirst);
  Tile A = fetch(kfirst, P);
  P = pages_of(kfirst + kStride);
  for (int kb = kfirst; kb <= qpos_max; kb += 2 * kStride) {
    const Tile B = fetch(kb + kStride, P);
    P = pages_of(kb + 2 * kStride);
    compute(A, kb);
    if (kb + kStride > qpos_max) break;
    A = fetch(kb + 2 * kStride, P);
    P = pages_of(kb + 3 * kStride);
    compute(B, kb + kStride);
  }

  l += __shfl_xor(l, 32, kWave);

  // ---- the waves meet: waves 1..3 leave maximum, sum and output in LDS (lane-contiguous),
  // wave 0 adds them in a fixed order with weights exp(m_w - max m) and writes the tile.
  extern __shared__ float red[];                              // [3][HDT*16 + 2][64]
  constexpr int kRows = HDT * 16 + 2;
  if (wave > 0) {
    float* mine = red + (wave - 1) * kRows * kWave + lane;
#pragma unroll
    for (int r = 0; r < HDT; ++r)
#pragma unroll
      for (int i = 0; i < 16; ++i) mine[(16 * r + i) * kWave] = acc[r][i];
    mine[(HDT * 16) * kWave] = m;
    mine[(HDT * 16 + 1) * kWave] = l;
  }
  __syncthreads();
  if (wave > 0 || c >= nq) return;
  float mw[kPrefillWaves - 1], M = m;
#pragma unroll
  for (int w = 0; w < kPrefillWaves - 1; ++w) {
    mw[w] = red[(w * kRows + HDT * 16) * kWave + lane];
    M = fmaxf(M, mw[w]);
  }
  // M is finite: the wave that holds the query's own key has a finite maximum
  const float w0 = __builtin_amdgcn_exp2f((m - M) * c2);      // exp2(-inf) = 0 for a wave without keys
  float ww[kPrefillWaves - 1];
  l *= w0;
#pragma unroll
  for (int w = 0; w < kPrefillWaves - 1; ++w) {
    ww[w] = __builtin_amdgcn_exp2f((mw[w] - M) * c2);
    l += ww[w] * red[(w * kRows + HDT * 16 + 1) * kWave + lane];
  }
  const float inv = 1.f / l;
  bf16_t* orow = out + ((long)tq * H + h) * hd;
#pragma unroll
  for (int r = 0; r < HDT; ++r)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      bf16x4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = 4 * b + j;
        float o = acc[r][i] * w0;
#pragma unroll
        for (int w = 0; w < kPrefillWaves - 1; ++w) o += ww[w] * red[(w * kRows + 16 * r + i) * kWave + lane];
        v[j] = (bf16_t)(o * inv);
      }
      *reinterpret_cast<bf16x4*>(orow + 32 * r + 8 * b + 4 * g) = v;
    }
}

template <int HDT>
static void launch_prefill(int grid, hipStream_t stream, const void* q, void* out, const void* cache,
                           const int* query_tiles, int n_tiles, const int* span_start,
                           const int* span_pos, const int* block_table, int max_pages, int page_size,
                           int H, int KV, int window, float scale) {
  const size_t lds = (size_t)(kPrefillWaves - 1) * (HDT * 16 + 2) * kWave * sizeof(float);
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    (void)hipFuncSetAttribute((const void*)attn_prefill_mfma_kernel<HDT>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = 1;
  }
  hipLaunchKernelGGL(attn_prefill_mfma_kernel<HDT>, dim3(grid), dim3(64 * kPrefillWaves), lds, stream,
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
  const int grid = (int)items;
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
