// Prompt attention over the paged cache on the matrix cores (bfloat16), two
// kernels with the same arithmetic; which one runs is decided per launch (see
// launch_prefill at the end of this file).
//
// Both read a request's keys from the first key any of a workgroup's queries
// may read to the last -- earlier pages of the cache and the rows this step
// has just written alike, so a prompt's portion at a position > 0 needs no
// other path.  Running maximum and sum per query (online softmax), no score
// matrix in memory, context bounded by pages only.  Formulas as in the generic
// kernel (reference: backend/model.cu:343-408, window :224-225), in 32-bit;
// probabilities are rounded to bfloat16 for the product with the values and
// their sum is taken over the rounded numbers, as in the decode kernel.
//
// The first kernel (attn_prefill_mfma_kernel): a workgroup takes up to 128
// consecutive tokens of one request (a query block) and one head; each wave of
// a group of four owns 32 of the queries.  Keys and values pass through LDS in
// tiles of 64 keys (two blocks of 32; 32 keys for head sizes above 128, for
// registers), and every tile is read from memory once for the 128 queries: one
// workgroup per 32 queries reading its own keys takes four times the traffic
// between L2 and the CUs, and with many workgroups that traffic bounds the
// kernel.  The tiles after the one being multiplied are on their way: the next
// one being written to the other LDS buffer, two more in registers, the page
// ids two tiles before their loads.  A wave's chain of dependent steps per tile
// is long (LDS, scores, maximum across lanes, exponentials, values, barrier), so
// 64 keys share one chain, and with PAR = 2 two groups of four waves take the
// tiles in turn and meet in LDS at the end: two chains of half the length.
//
// The scores are computed transposed, S^T = K Q^T, so that a query is a
// column: MFMA 32x32x16, lane l (g = l/32, c = l%32) holds A[c][8g..8g+7],
// B[8g..8g+7][c] and D[8(i/4) + 4g + i%4][c], i = 0..15.  A = 32 keys x 16 of
// hd, one key row per lane from LDS; B = q of 32 tokens.  A lane then holds 16
// scores of one query, its partner lane (l ^ 32) the other 16: maximum and sum
// need one exchange.  For the values, O^T += V^T P^T, the 16 k slots of MFMA u
// are the keys 16u + 8(j/4) + 4g + j%4, j = 0..7 -- exactly the scores
// D[8u + j] a lane holds -- and A = values [hd row c][those keys], two 8-byte
// reads from the [hd][key] tile in LDS.
//
// LDS rows are padded so that the lanes of a read fall into different banks:
// keys [64][hd + 8], values [hd][64 + 4] (tiles of 32 keys for head sizes above 128).
#include <math.h>

#include <type_traits>

#include "attention_f32.hpp"
#include "attention_merge.hpp"
#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kPrefillWaves = 4;
constexpr int kQueryBlock = 32 * kPrefillWaves;   // queries of a workgroup
// Limits of the division-free page arithmetic (page_magic in the first kernel).
constexpr int kPrefillMaxPage = 2048;
constexpr int kPrefillMaxKeys = 1 << 24;
constexpr int kPrefillMaxSlices = 4;              // workgroups that may share out the keys of one block and head
constexpr int kPrefillSliceFromKeys = 1280;       // ... when the longest block reads at least this many

template <int HDT>
struct PrefillShape {
  static constexpr int hd = 32 * HDT;
  static constexpr int KS = hd / 16;
  static constexpr int NB = HDT <= 4 ? 2 : 1;       // blocks of 32 keys in a tile (large heads leave registers for one)
  static constexpr int KT = 32 * NB;                // keys of a tile
  static constexpr int KLD = hd + 8;                // elements of a key row in LDS
  static constexpr int VLD = KT + 4;                // elements of a value row in LDS
  static constexpr int kBuf = KT * KLD + hd * VLD;  // elements of one buffer: a tile's keys, then its values
  static constexpr int kPieces = KT * hd / 8;       // 16-byte pieces of a tile's keys, and of its values
  static constexpr int CPT = kPieces / 256;         // pieces per thread
  static constexpr int kMaxPar = HDT <= 4 ? 2 : 1;  // groups of four waves that may take the tiles in turn (registers)
};

template <int HDT, int PAR>  // head_dim = 32 * HDT; PAR groups of four waves
__global__ __launch_bounds__(64 * kPrefillWaves * PAR) __attribute__((amdgpu_waves_per_eu(HDT <= 2 && PAR == 1 ? 3 : (HDT <= 4 ? 2 : 1)))) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ query_tiles, int n_tiles, const int* __restrict__ span_start,
    const int* __restrict__ span_pos, const int* __restrict__ block_table, int max_pages,
    int page_size, unsigned page_magic, int H, int KV, int window, float scale, float* __restrict__ part) {
  typedef PrefillShape<HDT> S;
  constexpr int hd = S::hd, KS = S::KS, NB = S::NB, KT = S::KT, KLD = S::KLD, VLD = S::VLD, CPT = S::CPT;
  extern __shared__ __attribute__((aligned(16))) bf16_t tiles_lds[];   // [PAR][2][kBuf]
  const int lane = threadIdx.x % kWave;
  const int tid = threadIdx.x % 256;                          // within the group of four waves
  const int par = PAR == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x / 256) : 0;   // the group: tiles par, par + PAR, ...
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) % kPrefillWaves;
  const int g = lane / 32, c = lane % 32;
  const long item = blockIdx.x;                               // (block, head), head fastest
  // Later blocks read more keys.  With three workgroups a CU (one group of waves) the later
  // half of the list is started first, longest block first, then the earlier half, shortest
  // first: a CU that holds one workgroup of each half gets a long and a short one, and all CUs
  // about the same number of keys.  With one workgroup a CU (two groups) a CU takes the next
  // block when it is done with one: longest first throughout.
  const int place = (int)(item / H), h = item % H, n_late = (n_tiles + 1) / 2;
  const int blk = (PAR == 2 || place < n_late) ? n_tiles - 1 - place : place - n_late;
  const int kvh = h / (H / KV);
  // The same for every lane: said so explicitly, which keeps the loop's address arithmetic on
  // the scalar unit.
  const int t0 = __builtin_amdgcn_readfirstlane(query_tiles[2 * blk]);
  const int span = __builtin_amdgcn_readfirstlane(query_tiles[2 * blk + 1]);
  const int s_begin = __builtin_amdgcn_readfirstlane(span_start[span]);
  const int s_end = __builtin_amdgcn_readfirstlane(span_start[span + 1]);
  const int pos0 = __builtin_amdgcn_readfirstlane(span_pos[span]);
  const int kv_len = pos0 + (s_end - s_begin);              // keys of the request after this step
  // the block's queries, and this wave's
  const int nq_blk = min(kQueryBlock, s_end - t0);
  const int blk_qmin = pos0 + (t0 - s_begin), blk_qmax = blk_qmin + nq_blk - 1;
  const int wq0 = t0 + 32 * wave;
  const int nq = max(0, min(32, s_end - wq0));
  const bool active = nq > 0;
  const int tq = active ? wq0 + min(c, nq - 1) : t0;        // this lane's query (clamped)
  const int qpos = pos0 + (tq - s_begin);
  const int w_qmin = pos0 + (wq0 - s_begin), w_qmax = w_qmin + nq - 1;
  const int lowest = (window > 0) ? max(0, blk_qmin - window + 1) : 0;   // first key any query reads
  const int w_lowest = (window > 0) ? max(0, w_qmin - window + 1) : 0;   // ... any query of this wave
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

  const int kb0 = lowest / 32 * 32;
  const int ntiles_all = (blk_qmax - kb0) / KT + 1;
  // The tiles go in turn to the slices (workgroups of the same block and head, blockIdx.y: where
  // the blocks alone leave CUs idle) and, within a slice, to the groups of waves.
  const int nslices = gridDim.y, slice = blockIdx.y;
  const int ntiles = (ntiles_all + PAR * nslices - 1) / (PAR * nslices);   // steps of the loop: the same for all
  auto tile_no = [&](int t) { return nslices * (PAR * t + par) + slice; };
  auto tile_key = [&](int t) { return kb0 + KT * tile_no(t); };   // first key of this group's t-th tile
  // page and slot of a key: a shift and a mask when the page size is a power of two
  // Page of a key without a division: page_magic = ceil(2^35 / page_size) from the host, exact
  // for keys below 2^24 and pages of up to 2,048 tokens (kPrefillMaxKeys, checked at the launch).
  auto page_index = [&](int key) { return (int)(__umulhi((unsigned)key, page_magic) >> 3); };
  const int first_page_key = page_index(lowest) * page_size;   // pages before this may be gone

  // ---- a tile's way from memory to LDS.  Thread tid moves the same pieces of every tile:
  // piece i = tid + 256 j of the keys is 16 bytes of key row i / (hd/8); piece i of the values
  // is 8 keys of one hd row of one half of the tile.  A half (16 keys) lies in one page, and
  // the pieces of one wave lie in one half: page, slot and base address are the same for the
  // whole wave and are worked out on the scalar unit; what differs between lanes is constant
  // over the tiles and kept in registers.  Loads carry no branch: a half that does not exist
  // reads page 0 and is masked (keys) or zeroed (values).
  int half_of[CPT], k_off[CPT], v_off[CPT], k_lds[CPT], v_lds[CPT], v_key[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int i = tid + 256 * j;
    half_of[j] = __builtin_amdgcn_readfirstlane(i / (2 * hd));
    const int krow = i / (hd / 8), kcol = i % (hd / 8) * 8;
    const int rest = i % (2 * hd), d = rest / 2, part = rest % 2;
    k_off[j] = ((krow % 16) * hd + kcol) * (int)sizeof(bf16_t);   // bytes from the half's first key row in its page
    v_off[j] = (d * page_size + 8 * part) * (int)sizeof(bf16_t);  // bytes from the half's first slot of the page's values
    k_lds[j] = krow * KLD + kcol;
    v_lds[j] = KT * KLD + d * VLD + 16 * half_of[j] + 8 * part;
    v_key[j] = 16 * half_of[j] + 8 * part;                  // first key of the values piece, from the tile's
  }
  struct Pages {
    int page[CPT];
  };
  struct Stage {
    bf16x8 k[CPT], v[CPT];
  };
  auto key_ok = [&](int key) { return key < kv_len && key >= first_page_key; };
  auto lookup = [&](int t) -> Pages {
    Pages P;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      const int key0 = tile_key(t) + 16 * half_of[j];
      const bool ok = tile_no(t) < ntiles_all && key_ok(key0);
      // A vector load although the address is the same in every lane: a scalar load would be
      // counted together with the LDS operations, and every wait for LDS would wait for it.
      int index = ok ? page_index(key0) : 0;
      asm volatile("" : "+v"(index));
      P.page[j] = table[index];                             // made uniform, and clamped, in fetch
    }
    return P;
  };
  // A page's bytes are addressed from its first: one 64-bit product per page, the rest in 32 bits
  // (a page of all heads' keys and values is far below 4 GB), so that the scalar unit has little
  // to do per tile.
  const unsigned page_bytes = (unsigned)(2 * KV * block * sizeof(bf16_t));
  const unsigned k_head = (unsigned)(kvh * block * sizeof(bf16_t));
  const unsigned v_head = (unsigned)((KV + kvh) * block * sizeof(bf16_t));
  const char* const cache_bytes = reinterpret_cast<const char*>(cache);
  auto fetch = [&](int t, const Pages& P) -> Stage {
    Stage T;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      const int key0 = tile_key(t) + 16 * half_of[j];
      const unsigned slot0 = (unsigned)(key0 - page_index(key0) * page_size);
      const unsigned page = (unsigned)max(__builtin_amdgcn_readfirstlane(P.page[j]), 0);
      const char* pbase = cache_bytes + (unsigned long)page * page_bytes;
      const unsigned kb_off = k_head + slot0 * (unsigned)(hd * sizeof(bf16_t));
      const unsigned vb_off = v_head + slot0 * (unsigned)sizeof(bf16_t);
      T.k[j] = *reinterpret_cast<const bf16x8*>(pbase + (kb_off + (unsigned)k_off[j]));
      T.v[j] = *reinterpret_cast<const bf16x8*>(pbase + (vb_off + (unsigned)v_off[j]));
    }
    return T;
  };
  auto stash = [&](const Stage& T, int t, bf16_t* buf) {
    if (tile_no(t) >= ntiles_all) return;
    const int kb = tile_key(t);
    const bool v_edge = kb < first_page_key || kb + KT > kv_len;   // slots that may hold anything
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      {
        *reinterpret_cast<bf16x8*>(&buf[k_lds[j]]) = T.k[j];
        bf16x8 v = T.v[j];
        if (v_edge) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = key_ok(kb + v_key[j] + e) ? v[e] : (bf16_t)0.f;
        }
        bf16_t* dst = &buf[v_lds[j]];                                   // 8-byte aligned
        bf16x4 lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
        *reinterpret_cast<bf16x4*>(dst) = lo;
        *reinterpret_cast<bf16x4*>(dst + 4) = hi;
      }
    }
  };
  auto lds_barrier = [&]() {   // for data in LDS only: loads from memory stay in flight
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  // One tile's arithmetic for this wave's 32 queries.  `masked` is a type (a constant of the
  // code): tiles whose every key is read by every query of the wave, the bulk, carry no mask
  // (head sizes up to 128; for larger ones, where the matrix unit bounds the time, one code).
  // The vector unit's share is kept small, it bounds the kernel: one multiply-add, one exp2 and
  // half a conversion per score, a sixth of a three-way maximum; the sum of the probabilities is
  // a matrix product with ones (of the rounded probabilities, as they multiply the values), and
  // the output is brought to a new maximum only when the maximum has grown by more than
  // kGrow binary orders (probabilities then stay below 2^kGrow instead of 1; the quotient at
  // the end is the same).
  constexpr float kGrow = 8.f;
  const bf16_t one = (bf16_t)1.f;
  const bf16x8 ones = {one, one, one, one, one, one, one, one};
  const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float grow_raw = kGrow / c2;                        // kGrow in units of raw scores
  float mc = 0.f;                                           // m * c2, 0 while m is -inf
  float m_limit = -INFINITY;                                // m + grow_raw
  auto tile_math = [&](auto masked, int kb, const bf16_t* buf) {
    // ---- scores: this lane's key rows are kb + c and kb + 32 + c
    floatx16 s[NB];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&buf[(32 * b + c) * KLD + 16 * kk + 8 * g]);
        s[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qb[kk], kk == 0 ? zero16 : s[b], 0, 0, 0);
      }
    if constexpr (decltype(masked)::value) {
      const int hi = min(qpos, kv_len - 1) - kb - 4 * g, lo = my_start - kb - 4 * g;   // offsets in the tile this lane's query reads
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int e = 32 * b + 8 * (i / 4) + i % 4;
          const bool ok = (e <= hi) & (e >= lo);
          s[b][i] = ok ? s[b][i] : -INFINITY;
        }
    }
    // ---- maximum; exp(x) is taken as exp2(x * log2 e) with the hardware's exp2
    float tmax = s[0][0];
#pragma unroll
    for (int e = 1; e < 16 * NB; ++e) tmax = fmaxf(tmax, s[e / 16][e % 16]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const bool grow = tmax > m_limit;                         // never for a maximum of -inf
    const bool any_grow = __any(grow);
    float a0 = 1.f;
    if (any_grow) {
      const float m_new = grow ? tmax : m;
      const float alpha = grow ? __builtin_amdgcn_exp2f(mc - m_new * c2) : 1.f;   // m = -inf: what was accumulated is 0 anyway
      a0 = (m == -INFINITY) ? 0.f : alpha;
      l *= a0;
      m = m_new;
      mc = (m == -INFINITY) ? 0.f : m * c2;
      m_limit = m + grow_raw;
    }
    // ---- probabilities, rounded, and their sum
    bf16x8 pb[NB][2];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        pb[b][i / 8][i % 8] = (bf16_t)__builtin_amdgcn_exp2f(fmaf(s[b][i], c2, -mc));   // exp2(-inf) = 0
    floatx16 ls = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[0][0], zero16, 0, 0, 0);
    ls = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[0][1], ls, 0, 0, 0);
    if (NB == 2) {
      ls = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[NB - 1][0], ls, 0, 0, 0);
      ls = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[NB - 1][1], ls, 0, 0, 0);
    }
    // ---- values: half u of block b holds keys kb + 32b + 16u .. + 15.  For head sizes up to
    // 128 the products follow the rescaling inside each branch, not behind their join: the
    // accumulators then stay where they are on the common path (behind the join the compiler
    // copies all of them every tile).
    const bf16_t* vt = buf + KT * KLD;
    auto values = [&]() {
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < HDT; ++r)
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const bf16_t* vrow = vt + (32 * r + c) * VLD + 32 * b + 16 * u + 4 * g;
            const bf16x4 lo = *reinterpret_cast<const bf16x4*>(vrow);
            const bf16x4 hi = *reinterpret_cast<const bf16x4*>(vrow + 8);
            const bf16x8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[b][u], acc[r], 0, 0, 0);
          }
    };
    auto rescale = [&]() {
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[r][i] *= a0;
    };
    if constexpr (HDT <= 4) {
      if (any_grow) {
        rescale();
        values();
      } else {
        values();
      }
    } else {                                                  // large heads: their code is long as it is
      if (any_grow) rescale();
      values();
    }
    l += ls[0];                                               // every row of ls is the sum over the tile's keys
  };
  const int w_highstart = (window > 0) ? max(0, w_qmax - window + 1) : 0;   // from here on no query of the wave masks a key below it
  auto compute = [&](int t, const bf16_t* buf) {
    const int kb = tile_key(t);
    if (!active || kb > w_qmax || kb + KT <= w_lowest) return;   // nothing here for this wave's queries
    if (HDT <= 4 && kb >= w_highstart && kb + KT - 1 <= w_qmin)   // every key for every query of the wave
      tile_math(std::false_type(), kb, buf);
    else
      tile_math(std::true_type(), kb, buf);
  };

  // Tiles in registers on their way to LDS: two for head size 96; one for the small heads, whose
  // registers buy a third wave per SIMD instead (8,192 tokens x 32 heads of 64: 469 -> 411 us),
  // and for the large ones, which have none to spare.
  constexpr int kAhead = HDT == 3 ? 2 : 1;
  constexpr int kRound = kAhead > 2 ? kAhead : 2;            // steps of a round: even, so that buffers alternate
  bf16_t* const bufs[2] = {tiles_lds + (2 * par) * S::kBuf, tiles_lds + (2 * par + 1) * S::kBuf};
  Pages pg[2];                                              // pg[x % 2]: the pages of tile x, then of x + 2
  Stage st[kAhead];
  pg[0] = lookup(0);
  pg[1] = lookup(1);
#pragma unroll
  for (int i = 0; i < kAhead; ++i) {
    st[i] = fetch(i, pg[i % 2]);
    pg[i % 2] = lookup(i + 2);
  }
  stash(st[0], 0, bufs[0]);
  lds_barrier();
  st[0] = fetch(kAhead, pg[kAhead % 2]);
  pg[kAhead % 2] = lookup(kAhead + 2);
  // Whole rounds, every step of every round the same for all waves and without a branch
  // around a load, so that the compiler can count the loads in flight: a tile beyond the last
  // is asked for (a valid address) and dropped.
  for (int round0 = 0; round0 < ntiles; round0 += kRound) {
#pragma unroll
    for (int i = 0; i < kRound; ++i) {
      const int t = round0 + i;
      compute(t, bufs[i % 2]);
      stash(st[(i + 1) % kAhead], t + 1, bufs[(i + 1) % 2]);
      lds_barrier();
      st[(i + 1) % kAhead] = fetch(t + 1 + kAhead, pg[(i + 1 + kAhead) % 2]);
      pg[(i + 1 + kAhead) % 2] = lookup(t + 3 + kAhead);
    }
  }

  // ---- the two groups meet: the second leaves maximum, sum and output in LDS (lane-contiguous,
  // in place of the tiles), the first adds them with weights exp(m - max m) and writes.
  if (PAR == 2) {
    float* red = reinterpret_cast<float*>(tiles_lds);         // [4 waves][HDT*16 + 2][64]
    constexpr int kRows = HDT * 16 + 2;
    lds_barrier();                                            // the last tiles have been read
    float* mine = red + (wave * kRows) * kWave + lane;
    if (par == 1) {
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) mine[(16 * r + i) * kWave] = acc[r][i];
      mine[(HDT * 16) * kWave] = m;
      mine[(HDT * 16 + 1) * kWave] = l;
    }
    lds_barrier();
    if (par == 1) return;
    const float m1 = mine[(HDT * 16) * kWave], l1 = mine[(HDT * 16 + 1) * kWave];
    const float M = fmaxf(m, m1);
    // (M is -inf where neither group had a key for the lane's query: a slice of the keys that ends before it)
    const float w0 = (M == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m - M) * c2);   // exp2(-inf) = 0
    const float w1 = (M == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m1 - M) * c2);
    l = l * w0 + l1 * w1;
#pragma unroll
    for (int r = 0; r < HDT; ++r)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[r][i] = acc[r][i] * w0 + mine[(16 * r + i) * kWave] * w1;
    m = M;
  }
  if (!active || c >= nq) return;
  if (nslices > 1) {
    // Keys in slices: the slice's sums as they are, with its maximum (in units of the scaled
    // scores, as the merge takes it) and its sum of probabilities; a slice without a key for
    // this query leaves a maximum of -inf.  Rows of hd + 2 floats are 8-byte aligned.
    float* prow = part + (((long)tq * H + h) * nslices + slice) * (hd + 2);
#pragma unroll
    for (int r = 0; r < HDT; ++r)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float* dst = prow + 32 * r + 8 * b + 4 * g;
        *reinterpret_cast<floatx2*>(dst) = floatx2{acc[r][4 * b], acc[r][4 * b + 1]};
        *reinterpret_cast<floatx2*>(dst + 2) = floatx2{acc[r][4 * b + 2], acc[r][4 * b + 3]};
      }
    if (g == 0) *reinterpret_cast<floatx2*>(prow + hd) = floatx2{m * scale, l};
    return;
  }
  const float inv = 1.f / l;                                  // finite: a query reads its own key
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

// The merge of the slices' results, one wave per (query, head); a block's queries are the
// rows from its first to the end of its span, at most kQueryBlock.
constexpr int kMergeWaves = 8;   // (query, head) pairs of a workgroup of the merge below

template <int DV>
__global__ __launch_bounds__(64 * kMergeWaves) void attn_prefill_merge_kernel(
    bf16_t* __restrict__ out, const float* __restrict__ part, const int* __restrict__ query_tiles,
    const int* __restrict__ span_start, int H, int hd, int nslices) {
  const int tile = blockIdx.x / kQueryBlock;
  const int t = query_tiles[2 * tile] + blockIdx.x % kQueryBlock;
  if (t >= span_start[query_tiles[2 * tile + 1] + 1]) return;
  const int h = blockIdx.y * kMergeWaves + threadIdx.x / kWave;
  if (h >= H) return;
  attn_merge_wide<bf16_t, DV, kPrefillMaxSlices>(out, part, t, h, H, hd, nslices, threadIdx.x % kWave);
}

// ---------------------------------------------------------------------------
// The same attention for steps with few query blocks (short prompts, a portion
// of a prompt at a long context, few heads): there the longest chain of key
// tiles bounds the time, not the traffic, and the keys are better shared out
// more finely.  A workgroup takes 32 of a block's queries and one head; its
// four waves share out the request's keys in tiles of 32, round robin, each
// streaming its tiles straight from the pages into registers (no LDS on the
// way), and meet in LDS at the end.  Four times the workgroups, a quarter of
// the chain, four times the reads from L2.
constexpr int kQueryTile = 32;

template <int HDT>  // head_dim = 32 * HDT
__global__ __launch_bounds__(64 * kPrefillWaves) __attribute__((amdgpu_waves_per_eu(HDT <= 2 ? 3 : 1))) void attn_prefill_split_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ query_tiles, int n_tiles, const int* __restrict__ span_start,
    const int* __restrict__ span_pos, const int* __restrict__ block_table, int max_pages,
    int page_size, int H, int KV, int window, float scale) {
  constexpr int hd = 32 * HDT;
  constexpr int KS = hd / 16;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 32, c = lane % 32;
  const long item = blockIdx.x;                               // (block, tile of 32 in it, head), head fastest
  const int tiles32 = kQueryBlock / kQueryTile;
  const int tile = n_tiles - 1 - (int)(item / ((long)H * tiles32));   // later blocks read more keys: start them first
  const int sub = tiles32 - 1 - (int)(item / H % tiles32), h = item % H;
  const int kvh = h / (H / KV);
  // The same for every lane: said so explicitly, which keeps the loop's page lookups and
  // address arithmetic on the scalar unit.
  const int t0 = __builtin_amdgcn_readfirstlane(query_tiles[2 * tile]) + kQueryTile * sub;
  const int span = __builtin_amdgcn_readfirstlane(query_tiles[2 * tile + 1]);
  const int s_begin = __builtin_amdgcn_readfirstlane(span_start[span]);
  const int s_end = __builtin_amdgcn_readfirstlane(span_start[span + 1]);
  const int pos0 = __builtin_amdgcn_readfirstlane(span_pos[span]);
  const int kv_len = pos0 + (s_end - s_begin);              // keys of the request after this step
  if (t0 >= s_end) return;                                  // the block ends before this tile
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

  // The vector unit's share per score as in the first kernel: the sum of the rounded
  // probabilities is a product with ones, and the output is brought to a new maximum only when
  // the maximum has grown by more than kGrow binary orders.
  constexpr float kGrow = 8.f;
  const bf16_t one = (bf16_t)1.f;
  const bf16x8 ones = {one, one, one, one, one, one, one, one};
  const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float grow_raw = kGrow / c2;                        // kGrow in units of raw scores
  float mc = 0.f;                                           // m * c2, 0 while m is -inf
  float m_limit = -INFINITY;                                // m + grow_raw
  auto compute = [&](const Tile& cur, int kb) {
    // ---- scores: this lane's key row is kb + c
    floatx16 s;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur.k[kk], qb[kk], kk == 0 ? zero16 : s, 0, 0, 0);
    // ---- mask (only where a tile touches an edge), maximum, probabilities.
    // exp(x) is taken as exp2(x * log2 e) with the hardware's exp2.
    const bool inner = kb >= my_start && kb + 31 <= qpos && kb + 32 <= kv_len;   // no mask needed
    if (__any(!inner)) {
      const int hi = min(qpos, kv_len - 1) - kb - 4 * g, lo = my_start - kb - 4 * g;   // offsets in the tile this lane's query reads
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int e = 8 * (i / 4) + i % 4;
        const bool ok = (e <= hi) & (e >= lo);
        s[i] = ok ? s[i] : -INFINITY;
      }
    }
    float tmax = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) tmax = fmaxf(tmax, s[i]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const bool grow = tmax > m_limit;                         // never for a maximum of -inf
    if (__any(grow)) {
      const float m_new = grow ? tmax : m;
      const float alpha = grow ? __builtin_amdgcn_exp2f(mc - m_new * c2) : 1.f;   // m = -inf: what was accumulated is 0 anyway
      const float a0 = (m == -INFINITY) ? 0.f : alpha;
      l *= a0;
#pragma unroll
      for (int r = 0; r < HDT; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[r][i] *= a0;
      m = m_new;
      mc = (m == -INFINITY) ? 0.f : m * c2;
      m_limit = m + grow_raw;
    }
    bf16x8 pb[2];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      pb[i / 8][i % 8] = (bf16_t)__builtin_amdgcn_exp2f(fmaf(s[i], c2, -mc));   // exp2(-inf) = 0
    floatx16 ls = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[0], zero16, 0, 0, 0);
    ls = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[1], ls, 0, 0, 0);
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
    l += ls[0];                                               // every row of ls is the sum over the tile's keys
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

template <int HDT, int PAR>
static void launch_prefill_par(int grid, hipStream_t stream, const void* q, void* out, const void* cache,
                               const int* query_tiles, int n_tiles, const int* span_start,
                               const int* span_pos, const int* block_table, int max_pages, int page_size,
                               int H, int KV, int window, float scale, float* part = nullptr, int nslices = 1) {
  typedef PrefillShape<HDT> S;
  const size_t lds = (size_t)PAR * 2 * S::kBuf * sizeof(bf16_t);   // also holds the groups' merge
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    (void)hipFuncSetAttribute((const void*)attn_prefill_mfma_kernel<HDT, PAR>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = 1;
  }
  const unsigned page_magic = (unsigned)(((1UL << 35) + page_size - 1) / page_size);   // ceil(2^35 / page_size)
  hipLaunchKernelGGL((attn_prefill_mfma_kernel<HDT, PAR>), dim3(grid, nslices), dim3(64 * kPrefillWaves * PAR), lds, stream,
                     (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, query_tiles, n_tiles,
                     span_start, span_pos, block_table, max_pages, page_size, page_magic, H, KV, window, scale, part);
  if (nslices > 1) {
    const dim3 mgrid(n_tiles * kQueryBlock, ceil_div(H, kMergeWaves));
    hipLaunchKernelGGL((attn_prefill_merge_kernel<(HDT + 1) / 2>), mgrid, dim3(64 * kMergeWaves), 0, stream,
                       (bf16_t*)out, part, query_tiles, span_start, H, 32 * HDT, nslices);
  }
}

template <int HDT>
static void launch_prefill_split(int n_tiles, hipStream_t stream, const void* q, void* out, const void* cache,
                                 const int* query_tiles, const int* span_start, const int* span_pos,
                                 const int* block_table, int max_pages, int page_size, int H, int KV,
                                 int window, float scale) {
  const size_t lds = (size_t)(kPrefillWaves - 1) * (HDT * 16 + 2) * kWave * sizeof(float);
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    (void)hipFuncSetAttribute((const void*)attn_prefill_split_kernel<HDT>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = 1;
  }
  const int grid = n_tiles * (kQueryBlock / kQueryTile) * H;
  hipLaunchKernelGGL(attn_prefill_split_kernel<HDT>, dim3(grid), dim3(64 * kPrefillWaves), lds, stream,
                     (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, query_tiles, n_tiles,
                     span_start, span_pos, block_table, max_pages, page_size, H, KV, window, scale);
}

// Which kernel.  One group of waves with the keys through LDS (three workgroups a CU) when
// there are more than two query blocks per CU: the CUs are full and the traffic decides.  With
// fewer, a block's chain of tiles takes about 2,700 cycles a tile whatever else the CU holds;
// two groups of waves that take the tiles in turn (one workgroup a CU, longest blocks first)
// bring a pair of tiles to 3,900 cycles.  That pays when the longest chain bounds the time:
// whole prompts, whose later blocks read more keys (32 heads, one prompt, us with one group ->
// two: head 64, 2,048 tokens 47.7 -> 42.9, 1,500 tokens 36.3 -> 27.9; 24 heads of 96, 2,048
// tokens 60.7 -> 46.8; head 128, 2,048 tokens 74.4 -> 69.6), or one block per CU.  It does not
// when every block has a long chain and a CU holds two of them, a portion of a prompt far into
// its context: then the CU's tiles bound the time, and one group with its blocks side by side
// takes fewer cycles a tile (32,768 tokens in portions of 2,048: 237 ms against 252).  The
// caller says how many keys the blocks read together and the longest block alone
// (`keys_total`, `keys_longest`; 0: not known, the prompt is taken to start at its beginning).
// For heads below 128 and no more blocks than three quarters of the CUs, the keys are shared
// out over the waves of small workgroups instead (512 tokens: 11.2 us against 12.4 with two
// groups; 8 heads, 2,048 tokens: 28.4 against 31.8; 1,024 tokens of 32 heads, one block per CU:
// 22.6 against 20.0).
template <int HDT>
static void launch_prefill(int grid, hipStream_t stream, const void* q, void* out, const void* cache,
                           const int* query_tiles, int n_tiles, const int* span_start,
                           const int* span_pos, const int* block_table, int max_pages, int page_size,
                           int H, int KV, int window, float scale, long keys_total, int keys_longest,
                           float* part, int nslices) {
  const int cus = device_cus();
  // (the caller asked kllm_attn_prefill_slices: few blocks of a large head.  The slices' results
  // pass through memory and a second kernel, about 10 us for 512 queries of 32 heads; they pay
  // from about 1,280 keys to the longest block on, see there.)
  if (nslices > 1 && keys_longest >= kPrefillSliceFromKeys) {
    launch_prefill_par<HDT, PrefillShape<HDT>::kMaxPar>(grid, stream, q, out, cache, query_tiles, n_tiles, span_start,
                                                        span_pos, block_table, max_pages, page_size, H, KV, window,
                                                        scale, part, nslices);
    return;
  }
  bool chain_bound = true;
  if (keys_total > 0 && keys_longest > 0)   // tiles of a CU's share of all blocks against the longest block's
    chain_bound = 5 * (keys_total * H / cus) < 6 * (long)keys_longest;
  if (grid > 2 * cus || PrefillShape<HDT>::kMaxPar == 1 || (grid > cus && !chain_bound))
    launch_prefill_par<HDT, 1>(grid, stream, q, out, cache, query_tiles, n_tiles, span_start, span_pos,
                               block_table, max_pages, page_size, H, KV, window, scale);
  else if (HDT >= 4 || 4 * grid > 3 * cus)
    launch_prefill_par<HDT, PrefillShape<HDT>::kMaxPar>(grid, stream, q, out, cache, query_tiles, n_tiles,
                                                        span_start, span_pos, block_table, max_pages, page_size,
                                                        H, KV, window, scale);
  else
    launch_prefill_split<HDT>(n_tiles, stream, q, out, cache, query_tiles, span_start, span_pos, block_table,
                              max_pages, page_size, H, KV, window, scale);
}

}  // namespace kllm

using namespace kllm;

// Slices of the keys over workgroups (with a merge behind them) for a step of n_tiles blocks:
// for heads of 128 and more, whose blocks have no kernel that shares out the keys more finely,
// as many (2 or 4) as still leave no more workgroups than CUs.  512 queries of 32 heads of 128
// behind 1,536 cached keys: 52 us in one slice, 44 in two (34 for the slices, the rest for their
// results' way through memory and the merge); behind 3,584: 92 and 65; behind 512: 30 and 33,
// from the first token 20 and 28; 256 queries behind 1,024: 33 and 28 in four.  1,024 queries
// (one block per CU): no gain.  The launch takes the slices when the longest block reads at
// least kPrefillSliceFromKeys keys (keys_longest; not when the caller does not say).
extern "C" int kllm_attn_prefill_slices(int n_tiles, int H, int hd) {
  if (hd < 128 || n_tiles <= 0 || H <= 0) return 1;
  const long blocks = (long)n_tiles * H;
  int slices = 1;
  while (slices < kPrefillMaxSlices && blocks * slices * 2 <= device_cus()) slices *= 2;
  return slices;
}

extern "C" int kllm_attn_prefill(const void* q, void* out, const void* cache, const int* query_tiles,
                                 int n_tiles, const int* span_start, const int* span_pos,
                                 const int* block_table, int max_pages, int page_size, int H, int KV,
                                 int hd, int window, float scale, long keys_total, int keys_longest, float* part,
                                 long part_floats, int nslices, int n_rows, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(q && out && cache && query_tiles && span_start && span_pos && block_table,
               "attn_prefill: null pointer");
  KLLM_REQUIRE(keys_total >= 0 && keys_longest >= 0, "attn_prefill: negative numbers of keys");
  KLLM_REQUIRE(dtype == DT_BF16 || dtype == DT_F32, "attn_prefill: unknown dtype %d", dtype);
  KLLM_REQUIRE(n_tiles > 0 && H > 0 && KV > 0 && H % KV == 0, "attn_prefill: bad sizes tiles=%d H=%d KV=%d",
               n_tiles, H, KV);
  if (dtype == DT_F32) {
    KLLM_REQUIRE(max_pages > 0 && window >= 0, "attn_prefill: bad table width or window");
    return attn_f32_prefill((const float*)q, (float*)out, (const float*)cache, query_tiles, n_tiles, span_start,
                            span_pos, block_table, max_pages, page_size, H, KV, hd, window, scale, stream);
  }
  KLLM_REQUIRE(hd % 32 == 0 && hd >= 32 && hd <= 256 && (hd <= 128 || hd == 192 || hd == 256),
               "attn_prefill: head_dim %d is not built (32, 64, 96, 128, 192, 256)", hd);
  KLLM_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_prefill: page_size %d must be a multiple of 16",
               page_size);
  KLLM_REQUIRE(max_pages > 0 && window >= 0, "attn_prefill: bad table width or window");
  KLLM_REQUIRE(page_size <= kPrefillMaxPage && (long)max_pages * page_size <= kPrefillMaxKeys,
               "attn_prefill: page_size %d x table width %d beyond %d tokens per page or %d per request", page_size,
               max_pages, kPrefillMaxPage, kPrefillMaxKeys);
  const long items = (long)n_tiles * H;
  KLLM_REQUIRE(items < (1L << 31), "attn_prefill: too many tiles");
  KLLM_REQUIRE(nslices >= 1 && nslices <= kPrefillMaxSlices && (nslices == 1 || kllm_attn_prefill_slices(n_tiles, H, hd) > 1),
               "attn_prefill: %d slices of the keys for %d blocks of %d heads of %d (kllm_attn_prefill_slices says how many)",
               nslices, n_tiles, H, hd);
  KLLM_REQUIRE(nslices == 1 || (part && n_rows > 0 && part_floats >= (long)n_rows * H * nslices * (hd + 2)),
               "attn_prefill: %d slices need room for %d rows x %d heads x %d slices x (%d + 2) floats", nslices, n_rows,
               H, nslices, hd);
  const int grid = (int)items;
#define KLLM_PF(HDT)                                                                              \
  case HDT:                                                                                       \
    launch_prefill<HDT>(grid, stream, q, out, cache, query_tiles, n_tiles, span_start, span_pos,  \
                        block_table, max_pages, page_size, H, KV, window, scale, keys_total,      \
                        keys_longest, part, nslices);                                             \
    break
  switch (hd / 32) {
    KLLM_PF(1); KLLM_PF(2); KLLM_PF(3); KLLM_PF(4); KLLM_PF(6); KLLM_PF(8);
    default: KLLM_FAIL(ERR_ARG, "attn_prefill: head_dim %d is not built", hd);
  }
#undef KLLM_PF
  KLLM_CHECK_LAUNCH("attn_prefill");
  return 0;
}
