// Float32 attention over the paged cache on the matrix cores, for prompts and
// for decode tokens: one kernel, two ways of filling its 32 columns.
//
// Operands, products and sums are 32-bit throughout (MFMA 32x32x2 with float32
// inputs; expf; no reduced precision anywhere).  Formulas as in the generic
// kernel (reference: backend/model.cu:343-408, window :224-225): score =
// (q.k) * scale over keys [max(0, p - window + 1), p], softmax with the maximum
// subtracted, online over tiles of 32 keys so that no score matrix exists.
//
// One wave is one work item with 32 columns:
//   prompt   32 consecutive tokens of one request and one head: column c is
//            token t0 + c, each with its own causal bound
//   decode   one token, one KV head and up to 32 query heads of its group:
//            column c is head c, all with the token's bound; the token's keys
//            are cut into slices, a wave takes one and leaves a partial result
//            (maximum, sum, unnormalised output) that a second kernel merges
// A key tile is then read once for all 32 columns.
//
// MFMA 32x32x2 (lane l, g = l/32, c = l%32): A[c][g], B[g][c], D[8(i/4) + 4g +
// i%4][c] in accumulator register i.  Which element of the inner dimension a
// lane's operand stands for is free as long as A and B agree, so a lane reads
// four consecutive floats (16 bytes) and issues four MFMAs, one per float.
//   scores  S^T = K Q^T: A = key row c of the tile, floats 8kk + 4g .. + 3 of
//           head_dim, straight from the page; B = the same floats of column c's
//           query, from LDS.  The lane then holds, of column c, the scores of
//           keys 8(i/4) + 4g + i%4.
//   values  O^T += V^T P^T: A = values [head_dim row 32r + c][keys 8j + 4g .. +
//           3], one 16-byte read of the [head_dim][slot] value layout; B = the
//           probabilities of exactly those keys, which are registers 4j .. 4j +
//           3 of the scores.
//
// Loads carry no branch: a key outside the range the item reads is replaced by
// one inside it (a valid page) and masked (scores) or zeroed (values), so that
// pages given back behind a window or slots not yet written are never read.
// The next tile's keys are on their way during softmax and values, this tile's
// values during its scores (head sizes up to 128; larger ones load in turn,
// for registers).
#include <math.h>

#include "attention_f32.hpp"
#include "attention_merge.hpp"
#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kF32Waves = 4;

struct AttnF32Args {
  const float* q;
  float* out;
  float* part;
  const float* cache;
  const int* positions;        // decode
  const int* span_of_token;    // decode
  const int* token_list;       // decode: the tokens (null: 0 .. count - 1)
  const int* query_tiles;      // prompt
  const int* span_start;       // prompt
  const int* span_pos;         // prompt
  const int* block_table;
  int count;                   // decode: tokens; prompt: blocks of 128
  int max_pages, page_size, H, KV, hd, window;
  float scale;
  int nslices, col_blocks;     // decode: slices of the keys, blocks of 32 heads per group
  int wg_merge;                // decode: a workgroup's four slices leave one partial result
};

template <int HDT, bool DECODE>   // head_dim <= 32 * HDT
__global__ __launch_bounds__(64 * kF32Waves) void attn_f32_mfma_kernel(const AttnF32Args a) {
  constexpr int KC = 4 * HDT;                   // chunks of 8 floats of head_dim, at most
  constexpr bool AHEAD = HDT <= 4;              // next keys in flight while this tile is multiplied
  extern __shared__ __attribute__((aligned(16))) float q_lds[];   // [waves][32][hd + 4]
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int g = lane / 32, c = lane % 32;
  const int hd = a.hd, H = a.H, KV = a.KV, G = H / KV, page_size = a.page_size, window = a.window;
  const int kc = hd / 8;
  const int QLD = hd + 4;
  float* qs = q_lds + wave * 32 * QLD;
  const long item = (long)blockIdx.x * kF32Waves + wave;

  // ---- what this wave takes (the same in every lane)
  bool live;
  int t_base = 0, ncol = 1, h_base = 0, kvh = 0, span = 0, pos_base = 0, slice = 0;
  if (DECODE) {
    const long total = (long)a.count * KV * a.col_blocks * a.nslices;
    live = item < total;
    if (live) {
      slice = (int)(item % a.nslices);
      long r = item / a.nslices;
      const int cb = (int)(r % a.col_blocks);
      r /= a.col_blocks;
      kvh = (int)(r % KV);
      const int ti = (int)(r / KV);
      t_base = a.token_list ? a.token_list[ti] : ti;
      span = a.span_of_token[t_base];
      pos_base = a.positions[t_base];
      h_base = kvh * G + cb * 32;
      ncol = min(32, G - cb * 32);
    }
  } else {
    const long total = (long)a.count * 4 * H;
    live = item < total;
    if (live) {
      // Later tokens read more keys.  The later half of the (block, 32 tokens) pairs is
      // started first, longest first, then the earlier half, shortest first: a CU that
      // holds a workgroup of each half gets a long and a short one.
      const int h = (int)(item % H), place = (int)(item / H);
      const int npairs = a.count * 4, n_late = (npairs + 1) / 2;
      const int pair = place < n_late ? npairs - 1 - place : place - n_late;
      const int blk = pair / 4, sub = pair % 4;
      const int t0 = a.query_tiles[2 * blk] + 32 * sub;
      span = a.query_tiles[2 * blk + 1];
      const int s_begin = a.span_start[span], s_end = a.span_start[span + 1];
      if (t0 >= s_end) {
        live = false;                           // the block ends before these 32 tokens
      } else {
        t_base = t0;
        ncol = min(32, s_end - t0);
        pos_base = a.span_pos[span] + (t0 - s_begin);
        h_base = h;
        kvh = h / G;
      }
    }
  }

  // ---- the columns' queries into LDS
  if (live) {
    const int chunks = hd / 4;
    for (int idx = lane; idx < 32 * chunks; idx += kWave) {
      const int col = idx / chunks, ch = idx % chunks;
      const int cc = min(col, ncol - 1);
      const int tok = DECODE ? t_base : t_base + cc;
      const int head = DECODE ? h_base + cc : h_base;
      const floatx4 v = *reinterpret_cast<const floatx4*>(a.q + ((long)tok * H + head) * hd + 4 * ch);
      *reinterpret_cast<floatx4*>(qs + col * QLD + 4 * ch) = v;
    }
  }
  __syncthreads();
  if (!live) return;

  const bool col_ok = c < ncol;
  const int cc = min(c, ncol - 1);
  const int my_tok = DECODE ? t_base : t_base + cc;
  const int my_head = DECODE ? h_base + cc : h_base;
  const int my_pos = DECODE ? pos_base : pos_base + cc;
  const int my_start = window > 0 ? max(0, my_pos - window + 1) : 0;
  const int qmax = DECODE ? pos_base : pos_base + ncol - 1;            // last key any column reads
  const int lowest = window > 0 ? max(0, pos_base - window + 1) : 0;   // first key any column reads
  const int first = lowest / 32 * 32;
  const int tiles = (qmax - first) / 32 + 1;
  const int nslices = DECODE ? a.nslices : 1;
  const int per = (tiles + nslices - 1) / nslices;
  const int tile0 = slice * per, tile1 = min(tile0 + per, tiles);
  const int first_page_key = lowest / page_size * page_size;           // pages before this may be gone

  const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
  auto page_index = [&](int key) { return page_shift >= 0 ? key >> page_shift : key / page_size; };
  auto page_slot = [&](int key) { return page_shift >= 0 ? key & (page_size - 1) : key % page_size; };
  auto inside = [&](int key) { return min(max(key, first_page_key), qmax); };   // a key whose page exists
  const int* table = a.block_table + (long)span * a.max_pages;
  const long block = (long)page_size * hd;
  const float* kcache = a.cache + (long)kvh * block;                   // + page * 2 * KV * block
  const float* vcache = a.cache + ((long)KV + kvh) * block;
  const long page_stride = 2L * KV * block;

  float m = -INFINITY, l = 0.f;
  floatx16 acc[HDT];
#pragma unroll
  for (int r = 0; r < HDT; ++r)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[r][i] = 0.f;

  struct VPages {
    int page[4];
  };
  auto lookup_k = [&](int tile) -> int { return table[page_index(inside(first + 32 * tile + c))]; };
  auto lookup_v = [&](int tile) -> VPages {
    VPages P;
#pragma unroll
    for (int j = 0; j < 4; ++j) P.page[j] = table[page_index(inside(first + 32 * tile + 8 * j + 4 * g) & ~3)];
    return P;
  };
  auto fetch_k = [&](int tile, int page, floatx4 (&K)[KC]) {
    const int key = inside(first + 32 * tile + c);
    const float* row = kcache + page * page_stride + (long)page_slot(key) * hd + 4 * g;
#pragma unroll
    for (int kk = 0; kk < KC; ++kk) K[kk] = *reinterpret_cast<const floatx4*>(row + 8 * min(kk, kc - 1));
  };
  auto fetch_v = [&](int tile, const VPages& P, floatx4 (&V)[HDT][4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int key0 = inside(first + 32 * tile + 8 * j + 4 * g) & ~3;
      const float* base = vcache + P.page[j] * page_stride + page_slot(key0);
#pragma unroll
      for (int r = 0; r < HDT; ++r)
        V[r][j] = *reinterpret_cast<const floatx4*>(base + (long)min(32 * r + c, hd - 1) * page_size);
    }
  };

  floatx16 s;
  auto scores = [&](const floatx4 (&K)[KC]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KC; ++kk) {
      if (kk < kc) {
        const floatx4 b = *reinterpret_cast<const floatx4*>(qs + c * QLD + 8 * kk + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) s = __builtin_amdgcn_mfma_f32_32x32x2f32(K[kk][e], b[e], s, 0, 0, 0);
      }
    }
  };
  // mask, running maximum and sum; s becomes the probabilities
  auto softmax = [&](int tile) {
    const int kb = first + 32 * tile;
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb + 8 * (i / 4) + 4 * g + i % 4;
      const bool ok = key <= my_pos && key >= my_start;
      s[i] = ok ? s[i] * a.scale : -INFINITY;
      tmax = fmaxf(tmax, s[i]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m, tmax);
    const float mref = (m_new == -INFINITY) ? 0.f : m_new;   // a column with no key yet
    const float alpha = expf(m - mref);                      // exp(-inf) = 0
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = expf(s[i] - mref);
      psum += s[i];
    }
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int r = 0; r < HDT; ++r)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[r][i] *= alpha;
  };
  auto values = [&](int tile, floatx4 (&V)[HDT][4]) {
    const int kb = first + 32 * tile;
    if (kb < first_page_key || kb + 31 > qmax) {            // slots that were replaced or may hold anything
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = kb + 8 * j + 4 * g + e;
          const bool ok = key >= first_page_key && key <= qmax;
#pragma unroll
          for (int r = 0; r < HDT; ++r) V[r][j][e] = ok ? V[r][j][e] : 0.f;
        }
    }
#pragma unroll
    for (int r = 0; r < HDT; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[r] = __builtin_amdgcn_mfma_f32_32x32x2f32(V[r][j][e], s[4 * j + e], acc[r], 0, 0, 0);
  };

  if (tile0 < tile1) {
    floatx4 K[KC];
    floatx4 V[HDT][4];
    if (AHEAD) {
      int kp = lookup_k(tile0);
      VPages vp = lookup_v(tile0);
      fetch_k(tile0, kp, K);
      kp = lookup_k(tile0 + 1);
      for (int tile = tile0; tile < tile1; ++tile) {
        fetch_v(tile, vp, V);
        vp = lookup_v(tile + 1);
        scores(K);
        fetch_k(tile + 1, kp, K);                            // a tile beyond the last: valid addresses, dropped
        kp = lookup_k(tile + 2);
        softmax(tile);
        values(tile, V);
      }
    } else {
      for (int tile = tile0; tile < tile1; ++tile) {
        fetch_k(tile, lookup_k(tile), K);
        const VPages vp = lookup_v(tile);
        scores(K);
        fetch_v(tile, vp, V);
        softmax(tile);
        values(tile, V);
      }
    }
  }
  l += __shfl_xor(l, 32, kWave);
  if (DECODE && a.wg_merge) {
    // The four waves of a workgroup hold four neighbouring slices of the same token and heads
    // (the number of slices is a multiple of four): they meet in LDS, each in the place of its
    // queries, and leave one partial result, so that the second kernel reads a quarter.
    if (col_ok) {
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int d = 32 * r + 8 * b + 4 * g;
          if (d < hd) {
#pragma unroll
            for (int j = 0; j < 4; ++j) qs[c * QLD + d + j] = acc[r][4 * b + j];
          }
        }
      if (g == 0) {
        qs[c * QLD + hd] = m;                                // -inf and 0 for a slice without keys
        qs[c * QLD + hd + 1] = l;
      }
    }
    __syncthreads();
    const int nout = nslices / kF32Waves, sout = slice / kF32Waves;
    for (int idx = threadIdx.x; idx < ncol * hd; idx += 64 * kF32Waves) {
      const int col = idx / hd, d = idx % hd;
      float mw[kF32Waves], M = -INFINITY;
#pragma unroll
      for (int w = 0; w < kF32Waves; ++w) {
        mw[w] = q_lds[(w * 32 + col) * QLD + hd];
        M = fmaxf(M, mw[w]);
      }
      float o = 0.f, L = 0.f;
#pragma unroll
      for (int w = 0; w < kF32Waves; ++w) {
        const float wt = mw[w] == -INFINITY ? 0.f : expf(mw[w] - M);
        o += wt * q_lds[(w * 32 + col) * QLD + d];
        L += wt * q_lds[(w * 32 + col) * QLD + hd + 1];
      }
      float* prow = a.part + (((long)t_base * H + h_base + col) * nout + sout) * (hd + 2);
      prow[d] = o;
      if (d == 0) {
        prow[hd] = M;
        prow[hd + 1] = L;
      }
    }
    return;
  }
  if (!col_ok) return;

  // acc[r][i] is output element 32r + 8(i/4) + 4g + i%4 of this lane's column
  if (nslices == 1) {
    const float inv = 1.f / l;                               // finite: a column reads its own key
    float* orow = a.out + ((long)my_tok * H + my_head) * hd;
#pragma unroll
    for (int r = 0; r < HDT; ++r)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int d = 32 * r + 8 * b + 4 * g;
        if (d < hd) {
          floatx4 v;
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = acc[r][4 * b + j] * inv;
          *reinterpret_cast<floatx4*>(orow + d) = v;
        }
      }
    return;
  }
  float* prow = a.part + (((long)my_tok * H + my_head) * nslices + slice) * (hd + 2);
#pragma unroll
  for (int r = 0; r < HDT; ++r)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int d = 32 * r + 8 * b + 4 * g;
      if (d < hd) {
#pragma unroll
        for (int j = 0; j < 4; ++j) prow[d + j] = acc[r][4 * b + j];
      }
    }
  if (g == 0) {
    prow[hd] = m;                                            // -inf and 0 for a slice without keys
    prow[hd + 1] = l;
  }
}

template <int HDT, bool DECODE>
static int launch_f32(const AttnF32Args& a, long items, hipStream_t stream) {
  const size_t lds = (size_t)kF32Waves * 32 * (a.hd + 4) * sizeof(float);
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_f32_mfma_kernel<HDT, DECODE>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) KLLM_FAIL((int)e, "attention float32: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = 1;
  }
  const long grid = (items + kF32Waves - 1) / kF32Waves;
  KLLM_REQUIRE(grid > 0 && grid < (1L << 31), "attention float32: %ld work items do not fit a grid", items);
  hipLaunchKernelGGL((attn_f32_mfma_kernel<HDT, DECODE>), dim3((unsigned)grid), dim3(64 * kF32Waves), lds, stream, a);
  return 0;
}

template <bool DECODE>
static int dispatch_f32(const AttnF32Args& a, long items, hipStream_t stream) {
  const int hdt = (a.hd + 31) / 32;
  if (hdt <= 1) return launch_f32<1, DECODE>(a, items, stream);
  if (hdt <= 2) return launch_f32<2, DECODE>(a, items, stream);
  if (hdt <= 3) return launch_f32<3, DECODE>(a, items, stream);
  if (hdt <= 4) return launch_f32<4, DECODE>(a, items, stream);
  if (hdt <= 6) return launch_f32<6, DECODE>(a, items, stream);
  return launch_f32<8, DECODE>(a, items, stream);
}

bool attn_f32_fits(int hd, int page_size) {
  return hd >= 8 && hd <= 256 && hd % 8 == 0 && page_size > 0 && page_size % 4 == 0;
}

extern "C" int kllm_attn_f32_fits(int hd, int page_size) { return attn_f32_fits(hd, page_size) ? 1 : 0; }

int attn_f32_slices(int n, int KV, int H, int max_keys) {
  // About four waves per CU across the chip (eight from one group per CU on, where partial
  // results cost little beside the keys), shared out over tokens x KV heads x blocks of 32
  // heads; a slice is one wave and should have 32 keys at least (measured: 64 tokens at 2,048
  // keys 61 us with 8 slices against 68 with 4; one token at 32,768 keys 47 us with 256 against
  // 69 with 64; 8 tokens at 512 keys 13 us with 16 against 15 with 32).
  const int col_blocks = (H / KV + 31) / 32;
  const long groups = (long)n * KV * col_blocks;
  const int cus = device_cus();
  long want = (groups >= cus ? 8L : 4L) * cus / (groups > 0 ? groups : 1);
  long most = max_keys > 0 ? max_keys / 32 : 64;
  if (most > kAttnF32MaxSlices) most = kAttnF32MaxSlices;
  if (want > most) want = most;
  if (want < 1) want = 1;
  return (int)want;
}

int attn_f32_decode(const float* q, float* out, float* part, const float* cache, const int* positions,
                    const int* span_of_token, const int* block_table, int max_pages, int page_size,
                    int H, int KV, int hd, int window, float scale, int nslices, const int* token_list,
                    int count, hipStream_t stream) {
  KLLM_REQUIRE(attn_f32_fits(hd, page_size),
               "attn_decode float32: head_dim %d must be a multiple of 8 up to 256 and page_size %d a multiple of 4",
               hd, page_size);
  KLLM_REQUIRE(nslices >= 1 && nslices <= kAttnF32MaxSlices, "attn_decode float32: nslices %d is outside [1, %d]",
               nslices, kAttnF32MaxSlices);
  AttnF32Args a = {};
  a.q = q; a.out = out; a.part = part; a.cache = cache;
  a.positions = positions; a.span_of_token = span_of_token; a.token_list = token_list;
  a.block_table = block_table; a.count = count;
  a.max_pages = max_pages; a.page_size = page_size; a.H = H; a.KV = KV; a.hd = hd; a.window = window;
  a.scale = scale; a.nslices = nslices; a.col_blocks = (H / KV + 31) / 32;
  a.wg_merge = nslices % kF32Waves == 0;
  const long items = (long)count * KV * a.col_blocks * nslices;
  if (int rc = dispatch_f32<true>(a, items, stream)) return rc;
  KLLM_CHECK_LAUNCH("attn_decode float32");
  if (nslices > 1) {
    launch_attn_merge<float>(out, part, count, H, hd, a.wg_merge ? nslices / kF32Waves : nslices, token_list, stream);
    KLLM_CHECK_LAUNCH("attn_merge float32");
  }
  return 0;
}

int attn_f32_prefill(const float* q, float* out, const float* cache, const int* query_tiles, int n_tiles,
                     const int* span_start, const int* span_pos, const int* block_table, int max_pages,
                     int page_size, int H, int KV, int hd, int window, float scale, hipStream_t stream) {
  KLLM_REQUIRE(attn_f32_fits(hd, page_size),
               "attn_prefill float32: head_dim %d must be a multiple of 8 up to 256 and page_size %d a multiple of 4",
               hd, page_size);
  AttnF32Args a = {};
  a.q = q; a.out = out; a.cache = cache;
  a.query_tiles = query_tiles; a.span_start = span_start; a.span_pos = span_pos;
  a.block_table = block_table; a.count = n_tiles;
  a.max_pages = max_pages; a.page_size = page_size; a.H = H; a.KV = KV; a.hd = hd; a.window = window;
  a.scale = scale; a.nslices = 1; a.col_blocks = 1;
  const long items = (long)n_tiles * 4 * H;
  if (int rc = dispatch_f32<false>(a, items, stream)) return rc;
  KLLM_CHECK_LAUNCH("attn_prefill float32");
  return 0;
}

}  // namespace kllm
