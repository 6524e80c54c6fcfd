// Decode attention over the paged cache on the matrix cores (bfloat16).
//
// One wave takes one token, one KV head with up to 16 of its query heads, and
// one slice of the token's keys; it streams that slice's pages from memory
// once, for all heads of the group.  The waves of a workgroup (four or eight)
// merge their results in LDS.  Where one workgroup covers all keys of its token it writes the
// output itself; otherwise it leaves one partial result (running maximum, sum,
// unnormalised output) and a second kernel merges the workgroups' partials.
// The launch does not depend on any context length, so a recorded step can be
// replayed as contexts grow.
//
// Formulas as in the generic kernel (reference: backend/model.cu:343-408):
// score = (q.k)/sqrt(hd) over keys [max(0, p-window+1), p], softmax with the
// maximum subtracted, all in 32-bit; probabilities are rounded to bfloat16 for
// the product with the values and their sum is taken over the rounded numbers.
//
// MFMA 16x16x32 (lane l: g = l/16, c = l%16): A[c][8g..8g+7], B[8g..8g+7][c],
// D[4g+i][c].  Scores: A = 16 keys x 32 of hd (one key row per lane, straight
// from its page), B = q of 16 heads, D[key 4g+i][head c].  Values: the 32 k
// slots of one MFMA are keys (4g+j) of page-tile 0 for j < 4 and of page-tile 1
// for j >= 4, which is exactly how a lane holds its probabilities; A = values
// [hd row c][those keys], two 8-byte reads from the [hd][slot] value layout.
#include <math.h>

#include <mutex>

#include "attention_f32.hpp"
#include "attention_merge.hpp"
#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

// Waves of a workgroup: four where a token's keys are shared out over several workgroups
// (small batches: many small workgroups start sooner than few large ones; 8 tokens at 2,048
// keys: 6.1 us with 16 workgroups of 4 waves to a token and KV head, 9.7 us with 4 of 16),
// and eight, where the registers of the head size allow them, where one workgroup takes all
// keys of its token and writes the output itself.  Measured with 4 / 8 / 16 waves, in us:
// 64 tokens x 4 KV heads of 64 at 2,048 keys 37.1 / 25.8 / 25.9 (two workgroups of four waves
// and their merge: 29.9); 128 such tokens 44.0 / 44.7 / 48.9; 64 tokens x 8 KV heads of 128 at
// 4,096 keys 220 / 195; 32 tokens x 32 KV heads of 128 at 2,048 keys 221 / 208.
constexpr int kDecodeWavesShared = 4;
constexpr int decode_waves_whole(int hdt) { return hdt <= 8 ? 8 : 4; }
// Tiles of 32 keys in a group; two groups are in registers.
constexpr int decode_ahead(int hdt) { return 1; }

__device__ __forceinline__ float group4_max(float v) {   // over lanes c, c+16, c+32, c+48
  v = fmaxf(v, __shfl_xor(v, 16, kWave));
  return fmaxf(v, __shfl_xor(v, 32, kWave));
}
__device__ __forceinline__ float group4_sum(float v) {
  v += __shfl_xor(v, 16, kWave);
  return v + __shfl_xor(v, 32, kWave);
}

template <int HDT, int kDecodeWaves>  // head_dim = 16 * HDT
__global__ __launch_bounds__(64 * kDecodeWaves) void attn_decode_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ final_out, float* __restrict__ part,
    const bf16_t* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ span_of_token,
    const int* __restrict__ block_table, int max_pages, int page_size, int H, int KV, int window,
    float scale, int head_tiles, const int* __restrict__ token_list) {
  constexpr int hd = 16 * HDT;
  constexpr int KS = (hd + 31) / 32;           // MFMA steps over head_dim for the scores
  constexpr int kDecodeAhead = decode_ahead(HDT);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 16, c = lane % 16;
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y % head_tiles;
  const int G = H / KV;
  const int nslices = gridDim.z * kDecodeWaves;
  const int slice = blockIdx.z * kDecodeWaves + wave;

  const int len = positions[t] + 1;
  const int start = (window > 0 && len > window) ? len - window : 0;
  const int first = start / 32 * 32;                       // tiles of 32 keys from here
  const int tiles = (len - first + 31) / 32;
  const int per = (tiles + nslices - 1) / nslices;
  const int tile0 = slice * per, tile1 = min(tile0 + per, tiles);
  const int* table = block_table + (long)span_of_token[t] * max_pages;
  const long block = (long)page_size * hd;

  const int head_in_group = ht * 16 + c;                   // this lane's column
  const bool head_ok = head_in_group < G;
  const int head = kvh * G + (head_ok ? head_in_group : 0);
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8 qb[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = 32 * ks + 8 * g;
    qb[ks] = (head_ok && d0 < hd)
                 ? *reinterpret_cast<const bf16x8*>(q + ((long)t * H + head) * hd + d0)
                 : zero8;
  }

  float m = -INFINITY, l = 0.f;
  floatx4 acc[HDT];
#pragma unroll
  for (int i = 0; i < HDT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

  // One tile's operands.
  struct Tile {
    bf16x8 k[2][KS];
    bf16x4 v[2][HDT];
    bool live[2];
  };
  // Loads carry no branch: a tile or a page that does not exist reads a valid address
  // (table entry 0, page 0) and is marked dead, so that the compiler can count the loads in
  // flight and a tile's arithmetic waits for its own operands only.
  auto page_of = [&](int tile, int u) -> int {
    const int k0 = first + tile * 32 + 16 * u;
    const bool ok = tile < tile1 && k0 < len && k0 + 16 > start;
    const int page = table[ok ? k0 / page_size : 0];
    return ok ? page : -1;
  };
  auto fetch = [&](int tile, int page0, int page1) -> Tile {
    Tile T;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int page = u ? page1 : page0;
      const int k0 = first + tile * 32 + 16 * u;
      T.live[u] = page >= 0;
      const long base = ((long)(T.live[u] ? page : 0) * 2 * KV + kvh) * block;
      const bf16_t* kp = cache + base + (long)(k0 % page_size + c) * hd;        // keys [slot][hd]
      const bf16_t* vp = cache + base + (long)KV * block + (k0 % page_size);     // values [hd][slot]
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        T.k[u][ks] = *reinterpret_cast<const bf16x8*>(kp + (d0 < hd ? d0 : 0));
      }
#pragma unroll
      for (int r = 0; r < HDT; ++r)
        T.v[u][r] = *reinterpret_cast<const bf16x4*>(vp + (long)(16 * r + c) * page_size + 4 * g);
    }
    return T;
  };

  // Tiles go in groups of kDecodeAhead: while one group is multiplied the next group's
  // operands are on their way, and the page ids of the group after that.
  int pg[kDecodeAhead][2];
  Tile cur[kDecodeAhead];
#pragma unroll
  for (int j = 0; j < kDecodeAhead; ++j) {
    pg[j][0] = page_of(tile0 + j, 0);
    pg[j][1] = page_of(tile0 + j, 1);
  }
#pragma unroll
  for (int j = 0; j < kDecodeAhead; ++j) {
    cur[j] = fetch(tile0 + j, pg[j][0], pg[j][1]);
    pg[j][0] = page_of(tile0 + kDecodeAhead + j, 0);
    pg[j][1] = page_of(tile0 + kDecodeAhead + j, 1);
  }
  auto compute = [&](const Tile& cur, int tile) {
    const int kb = first + tile * 32;
    const bool edge = kb < start || kb + 32 > len;
    floatx4 s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      s[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bool kin = cur.live[u] && 32 * ks + 8 * g < hd;   // a dead page may hold anything
        s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kin ? cur.k[u][ks] : zero8, qb[ks], s[u], 0, 0, 0);
      }
    }
    // ---- online softmax for this lane's head over its 8 keys, then the 4 lanes of the column
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb + 16 * u + 4 * g + i;
        const bool ok = cur.live[u] && key >= start && key < len;
        s[u][i] = ok ? s[u][i] * scale : -INFINITY;
        tmax = fmaxf(tmax, s[u][i]);
      }
    tmax = group4_max(tmax);
    const float m_new = fmaxf(m, tmax);                    // finite: every tile holds a readable key
    const float alpha = expf(m - m_new);
    bf16x8 pb;
    float psum = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = (s[u][i] == -INFINITY) ? 0.f : expf(s[u][i] - m_new);
        const bf16_t pr = (bf16_t)p;
        pb[4 * u + i] = pr;
        psum += (float)pr;
      }
    l = l * alpha + psum;
    m = m_new;
    // ---- values
#pragma unroll
    for (int r = 0; r < HDT; ++r) {
      acc[r] *= alpha;
      bf16x8 a;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb + 16 * u + 4 * g + i;
          const bool ok = cur.live[u] && (!edge || (key >= start && key < len));   // stale slots may hold anything
          a[4 * u + i] = ok ? cur.v[u][r][i] : (bf16_t)0.f;
        }
      acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[r], 0, 0, 0);
    }
  };
  for (int tile = tile0; tile < tile1; tile += kDecodeAhead) {
    Tile nxt[kDecodeAhead];
#pragma unroll
    for (int j = 0; j < kDecodeAhead; ++j) {
      nxt[j] = fetch(tile + kDecodeAhead + j, pg[j][0], pg[j][1]);
      pg[j][0] = page_of(tile + 2 * kDecodeAhead + j, 0);
      pg[j][1] = page_of(tile + 2 * kDecodeAhead + j, 1);
    }
#pragma unroll
    for (int j = 0; j < kDecodeAhead; ++j)
      if (tile + j < tile1) compute(cur[j], tile + j);
#pragma unroll
    for (int j = 0; j < kDecodeAhead; ++j) cur[j] = nxt[j];
  }

  l = group4_sum(l);

  // ---- the waves' results meet in LDS; then a thread merges, in the order of the waves,
  // four elements of one head and writes them: the output itself where this workgroup had
  // all the keys, else the workgroup's partial result
  extern __shared__ __attribute__((aligned(16))) float red[];   // [waves][heads of the tile][hd + 4]
  constexpr int RS = hd + 4;                                 // row stride: 16-byte rows
  const int heads_here = min(16, G - ht * 16);
  if (head_ok) {
    float* mine = red + (wave * heads_here + c) * RS;
#pragma unroll
    for (int r = 0; r < HDT; ++r) *reinterpret_cast<floatx4*>(mine + 16 * r + 4 * g) = acc[r];
    if (g == 0) {
      mine[hd] = m;
      mine[hd + 1] = l;
    }
  }
  __syncthreads();
  const bool whole = gridDim.z == 1;
  constexpr int CH = hd / 4;                                 // pieces of four elements in a head
  for (int idx = threadIdx.x; idx < heads_here * CH; idx += 64 * kDecodeWaves) {
    const int hc = idx / CH, d4 = (idx % CH) * 4;
    const float* col = red + hc * RS;
    float mj[kDecodeWaves], M = -INFINITY;
#pragma unroll
    for (int j = 0; j < kDecodeWaves; ++j) {
      mj[j] = col[j * heads_here * RS + hd];
      M = fmaxf(M, mj[j]);
    }
    const bool any = M != -INFINITY;                         // a workgroup beyond the last key has nothing
    floatx4 v = {0.f, 0.f, 0.f, 0.f};
    float L = 0.f;
#pragma unroll
    for (int j = 0; j < kDecodeWaves; ++j) {
      const float* w = col + j * heads_here * RS;
      const float wj = any ? expf(mj[j] - M) : 0.f;
      L += wj * w[hd + 1];
      v += wj * *reinterpret_cast<const floatx4*>(w + d4);
    }
    const int head_o = kvh * G + ht * 16 + hc;
    if (whole) {
      const float inv = 1.f / L;
      bf16x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (bf16_t)(v[i] * inv);
      *reinterpret_cast<bf16x4*>(final_out + ((long)t * H + head_o) * hd + d4) = o;
    } else {
      float* out = part + (((long)t * H + head_o) * gridDim.z + blockIdx.z) * (hd + 2);   // 8-byte rows
      *reinterpret_cast<floatx2*>(out + d4) = floatx2{v[0], v[1]};
      *reinterpret_cast<floatx2*>(out + d4 + 2) = floatx2{v[2], v[3]};
      if (d4 == 0) *reinterpret_cast<floatx2*>(out + hd) = floatx2{M, L};
    }
  }
}

template <int HDT, int W>
static int launch_decode(dim3 grid, hipStream_t stream, const void* q, void* out, float* part,
                         const void* cache, const int* positions, const int* span_of_token,
                         const int* block_table, int max_pages, int page_size, int H, int KV, int window,
                         float scale, int head_tiles, const int* token_list) {
  const int heads = H / KV < 16 ? H / KV : 16;
  const size_t lds = (size_t)W * heads * (16 * HDT + 4) * sizeof(float);
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_decode_mfma_kernel<HDT, W>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       W * 16 * (16 * HDT + 4) * (int)sizeof(float));
    if (e != hipSuccess) KLLM_FAIL((int)e, "attn_decode: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = 1;
  }
  hipLaunchKernelGGL((attn_decode_mfma_kernel<HDT, W>), grid, dim3(64 * W), lds, stream,
                     (const bf16_t*)q, (bf16_t*)out, part, (const bf16_t*)cache, positions, span_of_token,
                     block_table, max_pages, page_size, H, KV, window, scale, head_tiles, token_list);
  return 0;
}

// Workgroups that one CU holds at a time (registers and LDS decide: four of the shared
// variant's for heads of 64, two for heads of 128; of the variant that takes all keys, two and
// one), asked of the runtime once per head size; `heads` as in launch_decode.
template <int HDT, int W>
static int decode_resident_of(int heads) {
  int blocks = 0;
  const size_t lds = (size_t)W * heads * (16 * HDT + 4) * sizeof(float);
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, attn_decode_mfma_kernel<HDT, W>, 64 * W, lds) !=
          hipSuccess || blocks < 1) {
    (void)hipGetLastError();
    blocks = W > kDecodeWavesShared ? 1 : 2;
  }
  return blocks;
}

static int decode_resident(int hdt, int heads, bool whole) {
  static int known[2][17][17];                    // by variant, head size / 16 and heads of a group; 0: not asked yet
  if (hdt < 1 || hdt > 16 || heads < 1 || heads > 16) return whole ? 1 : 2;
  int& r = known[whole][hdt][heads];
  if (r) return r;
#define KLLM_RES(HDT)                                                                          \
  case HDT:                                                                                    \
    r = whole ? decode_resident_of<HDT, decode_waves_whole(HDT)>(heads)                        \
              : decode_resident_of<HDT, kDecodeWavesShared>(heads);                            \
    break
  switch (hdt) {
    KLLM_RES(1); KLLM_RES(2); KLLM_RES(3); KLLM_RES(4); KLLM_RES(5); KLLM_RES(6); KLLM_RES(7);
    KLLM_RES(8); KLLM_RES(12); KLLM_RES(16);
    default: r = whole ? 1 : 2;
  }
#undef KLLM_RES
  return r;
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_attn_decode_slices(int n, int KV, int H, int hd, int dtype, int max_keys) {
  if (KV <= 0 || H <= 0 || n <= 0 || hd <= 0) return 1;
  if (dtype == DT_F32) return attn_f32_slices(n, KV, H, max_keys);
  // Three quarters as many token x KV head x head tile groups as CUs, or more: one workgroup
  // takes all keys of its group and writes the output.  Otherwise workgroups of four waves
  // that each leave a partial result: about two per CU across the chip, their number per
  // group rounded up to a power of two (the keys of a context then go evenly to slices and
  // waves: 10 tokens x 4 KV heads of 64 at 2,048 keys, attention and merge: 11.7 us with 16,
  // 12.6 us with 13), but no more than the chip holds at a time (10 tokens x 8 KV heads of
  // 128 at 4,096 keys, two workgroups a CU: 35.5 us with 6, 41.1 us with 8, which is 640
  // workgroups).  A wave should have two tiles of 16 keys at least: 16 workgroups to a group
  // at contexts of 2,048, 32 at 4,096 and 64 from 8,192 keys on: every workgroup more is a
  // partial result more to merge, but the merge asks for all of them at once (one token, 4 KV
  // heads of 64, attention and merge in us with 16 / 32 / 64 workgroups to a group: 2,048 keys
  // 7.2 / 7.4 / 8.2, 4,096 keys 9.5 / 7.9 / 8.5, 8,192 keys 13.5 / 10.4 / 9.3, 16,384 keys
  // 21.5 / 14.2 / 12.8, 32,768 keys 37.4 / 22.9 / 16.7, 131,072 keys 143 / 76.4 / 45.9; four
  // tokens: 2,048 keys 8.2 / 8.7 / 9.8, 8,192 keys 15.7 / 13.1 / 15.5; when the merge took
  // sixteen at a time, 64 workgroups at 32,768 keys took 23.2 us and 16 at 2,048 keys 8.6).
  const int head_tiles = (H / KV + 15) / 16;
  long groups = (long)n * KV * head_tiles;
  const int hdt = (hd + 15) / 16;
  // (measured at 2,048 keys, one workgroup against the rule below: 192 groups 23.4 against
  // 28.7 us, 128 groups 22.6 against 20.0 us)
  const int heads = H / KV < 16 ? H / KV : 16;
  if (decode_waves_whole(hdt) > kDecodeWavesShared && 4 * groups >= 3L * device_cus()) {
    // ... unless the groups are a few more than the chip holds of such workgroups at a time:
    // the CUs that get a second one take twice as long as the others, and four workgroups
    // to a group spread the keys evenly (33 tokens x 8 KV heads of 128 at 2,048 keys, one
    // workgroup a CU: 71.2 us with one, 57.9 us with four and the merge; 40 tokens: 83.7 and
    // 75.7; 48 tokens: the same; 9 tokens x 32 KV heads: 78.4 and 62.4)
    // Where a CU holds two such workgroups (heads of 64) the second one shares the CU's
    // bandwidth with the first and nothing is gained (160 tokens x 4 KV heads of 64: 67.1 us
    // with one, 77.0 us with four).
    const int resident = decode_resident(hdt, heads, true);
    const long held = (long)resident * device_cus();
    if (resident > 1 || groups <= held || 5 * groups >= 8 * held) return 1;
    return 4;
  }
  if (groups < 1) groups = 1;
  int wg = 1;
  while ((long)wg * groups < 2L * device_cus()) wg *= 2;
  const long fit = (long)decode_resident(hdt, heads, false) * device_cus() / groups;   // what the chip holds at a time
  if (wg > fit) wg = (int)fit;
  int most = max_keys > 2048 ? max_keys / (32 * kDecodeWavesShared) : 16;
  const int cap = max_keys >= 8192 ? 64 : 32;
  if (most > cap) most = cap;
  if (wg > most) wg = most;
  if (wg < 1) wg = 1;
  return wg;
}

// Checks and launches shared by both entry points; `part` holds at least part_floats floats.
static int attn_decode_run(const char* who, const void* q, void* out, float* part, long part_floats,
                           const void* cache, const int* positions, const int* span_of_token,
                           const int* block_table, int max_pages, int page_size, int n, int H, int KV,
                           int hd, int window, float scale, int nslices, int dtype,
                           const int* token_list, int n_listed, hipStream_t stream) {
  KLLM_REQUIRE(q && out && part && cache && positions && span_of_token && block_table,
               "%s: null pointer", who);
  KLLM_REQUIRE(dtype == DT_BF16 || dtype == DT_F32, "%s: unknown dtype %d", who, dtype);
  KLLM_REQUIRE(n > 0 && H > 0 && KV > 0 && H % KV == 0, "%s: bad heads n=%d H=%d KV=%d", who, n, H, KV);
  if (dtype == DT_F32) {
    KLLM_REQUIRE(max_pages > 0 && window >= 0, "%s: bad table width or window", who);
    KLLM_REQUIRE(nslices >= 1 && part_floats >= (long)n * H * nslices * (hd + 2),
                 "%s: the partial results of n=%d H=%d nslices=%d head_dim=%d need %ld floats, the workspace has %ld",
                 who, n, H, nslices, hd, (long)n * H * nslices * (hd + 2), part_floats);
    KLLM_REQUIRE(H <= 65535, "%s: too many heads for the grid", who);
    KLLM_REQUIRE(!token_list || (n_listed > 0 && n_listed <= n), "%s: bad token list", who);
    return attn_f32_decode((const float*)q, (float*)out, part, (const float*)cache, positions, span_of_token,
                           block_table, max_pages, page_size, H, KV, hd, window, scale, nslices, token_list,
                           token_list ? n_listed : n, stream);
  }
  KLLM_REQUIRE(hd % 16 == 0 && hd >= 16 && hd <= 256 && (hd <= 128 || hd == 192 || hd == 256),
               "%s: head_dim %d is not built (16..128 in steps of 16, 192, 256)", who, hd);
  KLLM_REQUIRE(page_size % 16 == 0 && page_size > 0 && max_pages > 0,
               "%s: page_size %d must be a multiple of 16", who, page_size);
  KLLM_REQUIRE(nslices >= 1 && nslices <= 256, "%s: nslices %d is outside [1, 256]", who, nslices);
  KLLM_REQUIRE(window >= 0, "%s: negative window", who);
  KLLM_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)cache & 15) == 0 &&
                   ((uintptr_t)part & 15) == 0,
               "%s: q, out, cache and part must be 16-byte aligned", who);
  KLLM_REQUIRE(part_floats >= (long)n * H * nslices * (hd + 2),
               "%s: the partial results of n=%d H=%d nslices=%d head_dim=%d need %ld floats, the workspace has %ld",
               who, n, H, nslices, hd, (long)n * H * nslices * (hd + 2), part_floats);
  const int head_tiles = (H / KV + 15) / 16;
  KLLM_REQUIRE((long)KV * head_tiles <= 65535 && H <= 65535, "%s: too many heads for the grid", who);
  KLLM_REQUIRE(!token_list || (n_listed > 0 && n_listed <= n), "%s: bad token list", who);
  const int count = token_list ? n_listed : n;     // part and out are indexed by token, not by list place
  const dim3 grid(count, KV * head_tiles, nslices);
#define KLLM_DEC(HDT)                                                                             \
  case HDT:                                                                                       \
    if (int rc = nslices == 1                                                                     \
                     ? launch_decode<HDT, decode_waves_whole(HDT)>(                               \
                           grid, stream, q, out, part, cache, positions, span_of_token,           \
                           block_table, max_pages, page_size, H, KV, window, scale, head_tiles,   \
                           token_list)                                                            \
                     : launch_decode<HDT, kDecodeWavesShared>(                                    \
                           grid, stream, q, out, part, cache, positions, span_of_token,           \
                           block_table, max_pages, page_size, H, KV, window, scale, head_tiles,   \
                           token_list))                                                           \
      return rc;                                                                                  \
    break
  switch (hd / 16) {
    KLLM_DEC(1); KLLM_DEC(2); KLLM_DEC(3); KLLM_DEC(4); KLLM_DEC(5); KLLM_DEC(6); KLLM_DEC(7);
    KLLM_DEC(8); KLLM_DEC(12); KLLM_DEC(16);
    default: KLLM_FAIL(ERR_ARG, "%s: head_dim %d is not built", who, hd);
  }
#undef KLLM_DEC
  KLLM_CHECK_LAUNCH(who);
  if (nslices == 1) return 0;                      // the one workgroup of a token has written the output
  launch_attn_merge<bf16_t>((bf16_t*)out, part, count, H, hd, nslices, token_list, stream);
  KLLM_CHECK_LAUNCH("attn_merge");
  return 0;
}

extern "C" int kllm_attn_decode(const void* q, void* out, float* part, long part_floats,
                                const void* cache, const int* positions, const int* span_of_token,
                                const int* block_table, int max_pages, int page_size, int n, int H,
                                int KV, int hd, int window, float scale, int nslices, int dtype,
                                const int* token_list, int n_listed, hipStream_t stream) {
  return attn_decode_run("attn_decode", q, out, part, part_floats, cache, positions, span_of_token,
                         block_table, max_pages, page_size, n, H, KV, hd, window, scale, nslices, dtype,
                         token_list, n_listed, stream);
}

// ---- the entry point that allocates nothing -------------------------------------------------
// The partial results of the slices live in this array instead of a workspace of the caller's.
// Every GPU that the library runs on holds its own copy (4 MiB) until the process ends.  In
// host code the array's name is only a stand-in: its address on the current device comes
// from hipGetSymbolAddress, once per device, and only that pointer is ever handed to a kernel.
static __device__ __align__(256) float scratch[KLLM_ATTN_DECODE_STATIC_FLOATS];

constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices];        // per device, null until looked up
static std::mutex g_scratch_mutex;

// The array's address on the current device (looked up at the first call there).  The lookup
// may load the module's device variables, which a thread that is recording a graph must not
// do: a first call on a device while `stream` is being captured is refused.
static int scratch_on_current_device(float** ptr, hipStream_t stream, bool check_capture) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) KLLM_FAIL((int)e, "attn_decode_static: hipGetDevice: %s", hipGetErrorString(e));
  KLLM_REQUIRE(dev >= 0 && dev < kMaxDevices, "attn_decode_static: device %d is outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    if (check_capture) {
      hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
      e = hipStreamIsCapturing(stream, &st);
      if (e != hipSuccess) KLLM_FAIL((int)e, "attn_decode_static: hipStreamIsCapturing: %s", hipGetErrorString(e));
      if (st != hipStreamCaptureStatusNone)
        KLLM_FAIL(ERR_STATE, "attn_decode_static: the first call on device %d came while its stream is being "
                  "captured; call kllm_attn_decode_static_init() on the device before recording", dev);
    }
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      KLLM_FAIL(e != hipSuccess ? (int)e : ERR_STATE, "attn_decode_static: hipGetSymbolAddress on device %d: %s",
                dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" int kllm_attn_decode_static_init(void) {
  float* part = nullptr;
  return scratch_on_current_device(&part, nullptr, false);
}

extern "C" int kllm_attn_decode_static(const void* q, void* out, const void* cache, const int* positions,
                                       const int* span_of_token, const int* block_table, int max_pages,
                                       int page_size, int n, int H, int KV, int hd, int window, float scale,
                                       int nslices, int dtype, const int* token_list, int n_listed,
                                       hipStream_t stream) {
  KLLM_REQUIRE(n > 0 && H > 0 && nslices >= 1 && hd > 0, "attn_decode_static: bad sizes n=%d H=%d nslices=%d hd=%d",
               n, H, nslices, hd);
  const long need = (long)n * H * nslices * (hd + 2);
  KLLM_REQUIRE(need <= (long)KLLM_ATTN_DECODE_STATIC_FLOATS,
               "attn_decode_static: n=%d tokens x H=%d heads x nslices=%d slices x (head_dim=%d + 2) = %ld floats of "
               "partial results exceed the built-in scratch of %ld floats; use fewer slices or kllm_attn_decode "
               "with a workspace",
               n, H, nslices, hd, need, (long)KLLM_ATTN_DECODE_STATIC_FLOATS);
  float* part = nullptr;
  if (int rc = scratch_on_current_device(&part, stream, true)) return rc;
  // Nothing in the scratch has to start at zero: the first kernel writes every partial result
  // (maximum, sum, output of each token, head and slice) that the second one reads.
  return attn_decode_run("attn_decode_static", q, out, part, (long)KLLM_ATTN_DECODE_STATIC_FLOATS, cache,
                         positions, span_of_token, block_table, max_pages, page_size, n, H, KV, hd, window,
                         scale, nslices, dtype, token_list, n_listed, stream);
}
