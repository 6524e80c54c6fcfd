// Matrix products Y[n, m] = X[n, k] . W[m, k]^T (weights are [out, in], as the
// reference keeps them: backend/model.cu:494-503).  Accumulation is always in
// 32-bit.  Five kernels:
//
//   plain   one thread per output; any size; the yardstick the others are
//           tested against
//   tiled   true 32-bit FMA tiles through LDS, for the float32 engine
//   mfma    MFMA tiles through LDS, for prompts: bfloat16 on 32x32x16, float32 on
//           32x32x2 (32-bit operands, products and sums: no reduced precision)
//   skinny  bfloat16 MFMA 16x16x32, weights streamed straight from memory,
//           for up to 64 rows of X (decode batches); K may be split
//   gemv    one wave per weight row, up to 8 rows of X; K may be split
//
// A split product writes `nsplit` partial results [nsplit][n][m] in float32;
// the consumer adds them.
#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

// ------------------------------------------------------------------ plain
template <typename T, typename TOUT>
__global__ void gemm_plain_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                  TOUT* __restrict__ Y, int n, int m, int k) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * m) return;
  const int r = idx / m, c = idx % m;
  const T* x = X + (long)r * k;
  const T* w = W + (long)c * k;
  float acc = 0.f;
  for (int i = 0; i < k; ++i) acc = fmaf(to_f32(x[i]), to_f32(w[i]), acc);
  Y[idx] = from_f32<TOUT>(acc);
}

// ------------------------------------------------------------------ tiled f32
constexpr int TBM = 64, TBN = 64, TBK = 16;

template <typename TOUT>
__global__ __launch_bounds__(256) void gemm_f32_tiled_kernel(const float* __restrict__ X,
                                                             const float* __restrict__ W,
                                                             TOUT* __restrict__ Y, int n, int m,
                                                             int k, int vec_ok) {
  __shared__ float Xs[TBK][TBM + 4];
  __shared__ float Ws[TBK][TBN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const long row0 = (long)blockIdx.y * TBM, col0 = (long)blockIdx.x * TBN;
  const int lr = tid / 4, lk = (tid % 4) * 4;  // this thread's part of a tile load

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < k; k0 += TBK) {
    float xv[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    const long xr = row0 + lr, wr = col0 + lr;
    const int kk = k0 + lk;
    if (xr < n) {
      const float* p = X + xr * k + kk;
      if (vec_ok && kk + 3 < k) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) if (kk + i < k) xv[i] = p[i];
      }
    }
    if (wr < m) {
      const float* p = W + wr * k + kk;
      if (vec_ok && kk + 3 < k) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        wv[0] = v.x; wv[1] = v.y; wv[2] = v.z; wv[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) if (kk + i < k) wv[i] = p[i];
      }
    }
    __syncthreads();  // the previous tile is no longer read
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      Xs[lk + i][lr] = xv[i];
      Ws[lk + i][lr] = wv[i];
    }
    __syncthreads();
#pragma unroll
    for (int kk2 = 0; kk2 < TBK; ++kk2) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = Xs[kk2][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk2][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long r = row0 + ty * 4 + i;
    if (r >= n) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long c = col0 + tx * 4 + j;
      if (c < m) Y[r * m + c] = from_f32<TOUT>(acc[i][j]);
    }
  }
}

// ------------------------------------------------------------------ MFMA tiles
// Workgroup tile 128 (rows of X) x 128 (rows of W), 128 bytes of K per stage
// (64 bfloat16 or 32 float32), two or three LDS stages.  Four waves in 2 x 2,
// each 2 x 2 MFMA tiles of 32 x 32.
// MFMA 32x32x16 (bfloat16): lane l holds A[l%32][8*(l/32)..+7], B[l%32][...]
// likewise, and D[8*(i/4) + 4*(l/32) + i%4][l%32] in accumulator register i.
// MFMA 32x32x2 (float32): lane l holds A[l%32][l/32] and B[l%32][l/32], D as
// above.  Which element of K a lane's operand stands for is free as long as A
// and B agree, so a lane reads the same 16 bytes as in bfloat16 -- four
// consecutive floats, lanes 0..31 the first four of eight and lanes 32..63 the
// second four -- and issues four MFMAs, one per float: the tile loads, the LDS
// layout and the reads are the same code for both types.
//
// Operands go from memory to LDS directly (global_load_lds, 16 bytes per
// lane), one or two stages ahead of the MFMAs, without passing through
// registers: nothing waits on a register stage and no ds_write is issued.
// Such a load puts lane l's 16 bytes at LDS base + 16 l, so a wave's
// instruction fills 8 rows x 128 bytes of an unpadded tile -- whole cache
// lines of both operands, which measured a third faster than 64-byte rows.
// Bank conflicts of the 16-byte reads are avoided by a swizzle instead of
// padding: row r keeps its chunk c (8 elements) in slot c ^ swz(r), which the
// loading lane arranges by choosing which chunk it fetches.  Rows beyond the
// matrices are clamped to the last row (their results are never stored) and
// chunks beyond K come from a page of zeros.
//
// Stages: two (64 KB of LDS, two workgroups per CU) when the product has more
// tiles than CUs; three (one workgroup per CU, a deeper queue of loads) when
// every CU gets at most one tile.
//
// DUAL: W is [gate rows; up rows] = [2m, k]; a workgroup takes 64 gate rows and
// the 64 up rows that belong to them, and writes act(gate) * up for m columns
// (reference: backend/model.cu:477-483, :1112-1114) -- the gated activation
// never exists in 32-bit in memory.
//
// Workgroups are numbered so that the XCDs (which take workgroups round-robin,
// each with an L2 of its own; their number is asked of the runtime) each get a
// contiguous run of tiles that share rows of X.
constexpr int MBN = 128;
constexpr int MROW = 128;                     // bytes of a tile row in LDS: one stage of K

__device__ __attribute__((aligned(16))) unsigned char g_zero_chunk[16];   // zero-initialised

template <typename T> struct MfmaOperand;
template <> struct MfmaOperand<bf16_t> { typedef bf16x8 type; };
template <> struct MfmaOperand<float> { typedef floatx4 type; };

// One step of 32 bytes of K per row: acc += A . B^T for a 32 x 32 tile.
__device__ __forceinline__ floatx16 mfma_tile_step(bf16x8 a, bf16x8 b, floatx16 acc) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mfma_tile_step(floatx4 a, floatx4 b, floatx16 acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
  return acc;
}

// Slot permutation of a row's eight chunks: rows of equal parity among 16 neighbours get
// different slots, so that the 16-byte reads of 16 lanes spread over all 64 banks.
__device__ __forceinline__ int mfma_swz(int row) { return (row >> 1) & 7; }

// WR x WC waves, each with WTM x 2 MFMA tiles of 32 x 32: a workgroup's tile is 32 WTM WR rows
// of X by 64 WC rows of W (128 x 128 with four waves, 256 x 128 and 256 x 256 with eight; for
// decode batches 64 x 128 and 64 x 64 with two).
template <typename T, typename TOUT, bool DUAL, int WR, int MSTAGES, int WC = 2, int WTM = 2, int WTN = 2>
__global__ __launch_bounds__(64 * WR * WC) __attribute__((amdgpu_waves_per_eu(2))) void gemm_mfma_kernel(const T* __restrict__ X,
                                                             const T* __restrict__ W,
                                                             TOUT* __restrict__ Y, int n, int m,
                                                             int k, int tiles_x, int tiles_y, int kslice, int act,
                                                             int xcds) {
  typedef typename MfmaOperand<T>::type op_t;   // 16 bytes of a row
  constexpr int EPC = 16 / sizeof(T);           // elements of a 16-byte chunk
  constexpr int MBK = MROW / sizeof(T);         // elements of K per stage
  constexpr int BM = 32 * WTM * WR;             // rows of X per workgroup
  constexpr int BN = 32 * WTN * WC;             // rows of W per workgroup
  constexpr int NW = WR * WC;                   // waves
  // DUAL with an odd number of column tiles a wave: gate and up rows share every tile of 32
  // columns, 16 each (see the epilogue); with an even number they have tiles of their own.
  constexpr bool PAIRED = DUAL && WTN % 2 == 1;
  static_assert(!DUAL || PAIRED || WTN == 2, "DUAL: two column tiles a wave (gate, up) or an odd number of shared ones");
  constexpr int XI = BM / 8 / NW;               // load instructions of X per wave and stage (8 rows each)
  constexpr int WI = BN / 8 / NW;
  constexpr int XBYTES = BM * MROW, WBYTES = BN * MROW;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];   // [MSTAGES][X tile | W tile]
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wr = wave / WC, wc = wave % WC;
  const long total = (long)tiles_x * tiles_y;
  const long per_xcd = (total + xcds - 1) / xcds;
  const long id = (long)(blockIdx.x % xcds) * per_xcd + blockIdx.x / xcds;
  if (id >= total) return;
  // An XCD's run of tiles walks the shorter side fastest: it then reads only its share
  // of the larger operand and shares the smaller one.
  const bool x_major = tiles_x >= tiles_y;
  const long trow = x_major ? id % tiles_y : id / tiles_x;
  const long tcol = x_major ? id / tiles_y : id % tiles_x;
  const long row0 = trow * BM, col0 = tcol * (DUAL ? BN / 2 : BN);

  // Wave w loads rows [8 XI w, 8 XI (w+1)) of the X tile and [8 WI w, 8 WI (w+1)) of the W
  // tile.  In one instruction lane l serves row l / 8 (of 8), slot l % 8.
  const T* xsrc[XI];
  const T* wsrc[WI];
  int xchunk[XI], wchunk[WI];
#pragma unroll
  for (int i = 0; i < XI; ++i) {
    const int r = 8 * (XI * wave + i) + lane / 8;
    xchunk[i] = ((lane % 8) ^ mfma_swz(r)) * EPC;
    xsrc[i] = X + min(row0 + r, (long)n - 1) * k + xchunk[i];
  }
#pragma unroll
  for (int i = 0; i < WI; ++i) {
    const int r = 8 * (WI * wave + i) + lane / 8;             // DUAL: the first half of the rows gate, the second up
    wchunk[i] = ((lane % 8) ^ mfma_swz(r)) * EPC;
    long col, up;
    if (PAIRED) {                                              // ... or 16 gate rows and their 16 up rows in turn
      col = col0 + 16 * (r / 32) + r % 16;
      up = r % 32 >= 16;
    } else {
      col = DUAL ? col0 + r % (BN / 2) : col0 + r;
      up = DUAL && r >= BN / 2;
    }
    const long wrow = min(col, (long)m - 1) + (up ? m : 0);
    wsrc[i] = W + wrow * k + wchunk[i];
  }
  // blockIdx.y: a slice of K (kslice a multiple of a stage); its sums go to Y[blockIdx.y]
  const int kbeg = blockIdx.y * kslice, kend = min(k, kbeg + kslice);
  Y += (long)blockIdx.y * n * m;
  auto issue = [&](int kt) {
    unsigned char* base = lds + (kt % MSTAGES) * (XBYTES + WBYTES);
    const int kk = kbeg + kt * MBK;
#pragma unroll
    for (int i = 0; i < XI; ++i) {
      const T* src = kk + xchunk[i] < kend ? xsrc[i] + kk : reinterpret_cast<const T*>(g_zero_chunk);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(base + 8 * (XI * wave + i) * MROW),
                                       16, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < WI; ++i) {
      const T* src = kk + wchunk[i] < kend ? wsrc[i] + kk : reinterpret_cast<const T*>(g_zero_chunk);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(base + XBYTES + 8 * (WI * wave + i) * MROW),
                                       16, 0, 0);
    }
  };

  floatx16 acc[WTM][WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int ktiles = (kend - kbeg + MBK - 1) / MBK;
  issue(0);
  if (MSTAGES > 2 && ktiles > 1) issue(1);
  for (int kt = 0; kt < ktiles; ++kt) {
    // This wave's loads of stage kt have landed when at most the newer stage's (XI + WI
    // instructions, with three stages) are still in flight; after the barrier so have every
    // wave's, and every wave is done reading the stage that the next loads overwrite.  The
    // barrier is a bare s_barrier: a fence here would also wait for the newest loads.
    if (MSTAGES > 2 && kt + 1 < ktiles) __builtin_amdgcn_s_waitcnt(0x0F70 | (XI + WI));   // vmcnt(XI + WI)
    else __builtin_amdgcn_s_waitcnt(0x0F70);                                             // vmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (kt + MSTAGES - 1 < ktiles) issue(kt + MSTAGES - 1);
    const unsigned char* xs = lds + (kt % MSTAGES) * (XBYTES + WBYTES);
    const unsigned char* ws = xs + XBYTES;
    // The operands of step ks + 1 are asked for before the MFMAs of step ks are issued, so
    // that LDS answers while the matrix unit works.
    op_t a[2][WTM], b[2][WTN];
    auto read_step = [&](int ks, op_t (&ar)[WTM], op_t (&br)[WTN]) {
      const int chunk = ks * 2 + lane / 32;
#pragma unroll
      for (int i = 0; i < WTM; ++i) {
        const int r = wr * 32 * WTM + i * 32 + lane % 32;
        ar[i] = *reinterpret_cast<const op_t*>(xs + r * MROW + (chunk ^ mfma_swz(r)) * 16);
      }
#pragma unroll
      for (int j = 0; j < WTN; ++j) {
        const int r = (DUAL && !PAIRED ? j * (BN / 2) + wc * 32 : wc * 32 * WTN + j * 32) + lane % 32;
        br[j] = *reinterpret_cast<const op_t*>(ws + r * MROW + (chunk ^ mfma_swz(r)) * 16);
      }
    };
    read_step(0, a[0], b[0]);
#pragma unroll
    for (int ks = 0; ks < MROW / 32; ++ks) {
      if (ks + 1 < MROW / 32) read_step(ks + 1, a[(ks + 1) & 1], b[(ks + 1) & 1]);
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WTN; ++j)
          acc[i][j] = mfma_tile_step(a[ks & 1][i], b[ks & 1][j], acc[i][j]);
    }
  }

  if (PAIRED) {
    // Lanes c and c + 16 of a tile of 32 columns hold the gate and the up sum of one output
    // column, for 16 rows each.  They share the rows out: the lane with the gates takes the
    // first eight and is sent their up sums, the lane with the up sums the other eight and is
    // sent their gates; every lane then has eight outputs to gate and to store.
    const int cl = lane % 32;
    const bool has_gate = cl < 16;
#pragma unroll
    for (int j = 0; j < WTN; ++j) {
      const long c = col0 + 16 * (wc * WTN + j) + cl % 16;
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const float lo = acc[i][j][t], hi = acc[i][j][8 + t];
          const float got = __shfl_xor(has_gate ? hi : lo, 16, kWave);
          const float gate = has_gate ? lo : got, up = has_gate ? got : hi;
          const int e = has_gate ? t : 8 + t;
          const long r = row0 + wr * 32 * WTM + i * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          if (c < m && r < n) Y[r * m + c] = from_f32<TOUT>(gate_act(gate, act) * up);
        }
    }
    return;
  }
  if (DUAL) {
    const long c = col0 + wc * 32 + lane % 32;
    if (c >= m) return;
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const long r = row0 + wr * 32 * WTM + i * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
        const float gate = acc[i][0][e], up = acc[i][1][e];
        if (r < n) Y[r * m + c] = from_f32<TOUT>(gate_act(gate, act) * up);
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j) {
      const long c = col0 + wc * 32 * WTN + j * 32 + lane % 32;
      if (c >= m) continue;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const long r = row0 + wr * 32 * WTM + i * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
        if (r < n) Y[r * m + c] = from_f32<TOUT>(acc[i][j][e]);
      }
    }
}

template <typename T, typename TOUT, bool DUAL, int WR, int MSTAGES, int WC = 2, int WTM = 2, int WTN = 2>
static int launch_mfma_tile(const void* x, const void* w, void* y, int n, int m, int k, int nsplit, int act,
                            hipStream_t stream) {
  constexpr int MBK = MROW / sizeof(T);
  constexpr int BM = 32 * WTM * WR, BN = 32 * WTN * WC;
  const int tx = ceil_div(m, DUAL ? BN / 2 : BN), ty = ceil_div(n, BM);
  const int kslice = ceil_div(ceil_div(k, nsplit), MBK) * MBK;
  const int xcds = device_xcds();
  const dim3 grid(ceil_div((long)tx * ty, xcds) * xcds, nsplit);   // padded so that every XCD gets as many
  const size_t lds = (size_t)MSTAGES * (BM + BN) * MROW;
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_mfma_kernel<T, TOUT, DUAL, WR, MSTAGES, WC, WTM, WTN>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) KLLM_FAIL((int)e, "gemm mfma: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = 1;
  }
  hipLaunchKernelGGL((gemm_mfma_kernel<T, TOUT, DUAL, WR, MSTAGES, WC, WTM, WTN>), grid, dim3(64 * WR * WC), lds, stream,
                     (const T*)x, (const T*)w, (TOUT*)y, n, m, k, tx, ty, kslice, act, xcds);
  return 0;
}

constexpr long kNarrowBelow = 40000000;   // weights (elements) below which a decode batch gets tiles of 64 columns

// Tiles of 256 rows of X (eight waves) fetch a quarter less per flop than two tiles of 128;
// they are taken when they still give every CU two rounds of work and the last round is not
// mostly idle (8,192 x 2,560 x 2,048, two and a half rounds: 113 us against 101 us with 128 rows).  The thresholds follow
// the chip's number of CUs.
template <typename T, typename TOUT, bool DUAL>
static int launch_mfma(const void* x, const void* w, void* y, int n, int m, int k, int nsplit, int act,
                       hipStream_t stream) {
  const int cus = device_cus();
  const int tx = ceil_div(m, DUAL ? MBN / 2 : MBN);
  // A decode batch: tiles of 64 rows, half the products and half the loads of X of 128.  In
  // bfloat16 a product of few tiles keeps three stages of loads in flight (one workgroup a CU).
  if (n <= 64) {
    // ... and against weights below 40 M elements tiles of 64 columns (two waves of 32 x 64):
    // twice the workgroups, which is what a product of few column tiles lacks (64 rows, 2,048
    // x 5,632 in 8 slices: 9.8 us against 13.2 us; 11,264 x 2,048 in 4: 14.3 against 16.2; 4,096
    // x 14,336 in 8: 32.9 against 28.7).  In float32, where a wave's chain of products bounds
    // the time, the same halves the chain (a decode step of 64 tokens at 1.1B sizes: 4.75 ->
    // 4.30 ms).
    if constexpr (!DUAL) {
      if ((long)m * k < kNarrowBelow) {
        if ((long)ceil_div(m, 64) * nsplit <= cus)
          return launch_mfma_tile<T, TOUT, DUAL, 2, 3, 1, 1>(x, w, y, n, m, k, nsplit, act, stream);
        return launch_mfma_tile<T, TOUT, DUAL, 2, 2, 1, 1>(x, w, y, n, m, k, nsplit, act, stream);
      }
    }
    if (sizeof(T) == 2 && (long)tx * nsplit <= cus)
      return launch_mfma_tile<T, TOUT, DUAL, 1, 3>(x, w, y, n, m, k, nsplit, act, stream);
    return launch_mfma_tile<T, TOUT, DUAL, 1, 2>(x, w, y, n, m, k, nsplit, act, stream);
  }
  // 256 x 256 tiles (eight waves of 128 x 64, one workgroup a CU) fetch a third less again and
  // are 10-27 % faster (2,048 x 28,672 x 4,096: 499 us against 561 us) where their rounds fill
  // the chip: three quarters of the CUs busy on average, counting the last round.  With 80, 128,
  // 320 or 352 such tiles on 256 CUs they lose by as much.  bfloat16 only: float32 is bound by
  // its products, not its loads.  Tiles of 256 rows are for more than 128 rows: below, half of
  // every tile's products would be of rows that are not there (a decode step of 72 tokens at
  // 1.1B sizes: 2.60 -> 2.54 ms, of 128 at Llama-3-8B sizes: 11.98 -> 11.84 ms).
  if (sizeof(T) == 2 && n > 128) {
    const long big = (long)ceil_div(n, 256) * ceil_div(m, DUAL ? 128 : 256) * nsplit;
    const long rounds = ceil_div(big, (long)cus);
    const bool big_fits = 4 * big >= 3 * rounds * cus;
    // 256 x 192 tiles (eight waves of 64 x 96; with the gate, 96 output columns whose gate and
    // up rows share the column tiles): the fastest tile here where its rounds fill the chip
    // (2,048 x 11,264 x 2,048: 103 us against 123 us with 256 x 128; 2,048 x 12,288 x 4,096: 195
    // against 227 us with 128 x 128 and 241 us with 256 x 256; 512 x 22,016 x 4,096: 93 against
    // 113 us with 256 x 256), taken when its last round is at least 85 % full and it does not
    // need more time than 256 x 256 by their tiles' sizes and rounds.
    const long mid = (long)ceil_div(n, 256) * ceil_div(m, DUAL ? 96 : 192) * nsplit;
    const long mid_rounds = ceil_div(mid, (long)cus);
    // (a single round of them from three fifths of the CUs on: 768 x 11,264 x 2,048 on 177 tiles 50 us
    // against 63 us, 1,536 x 6,144 x 4,096 on 192 tiles 92 against 115; on 118 tiles, 512 rows,
    // 50 against 39)
    // for a product that is not cut along K, counting only the rows that are there (640 rows
    // in three tiles of 256: slower, 3.34 -> 3.63 ms for the whole step at 1.1B sizes)
    const bool one_round = mid_rounds == 1 && nsplit == 1 &&
                           5L * mid * n >= 3L * cus * 256 * ceil_div(n, 256);
    const bool mid_fits = 100 * mid >= 85 * mid_rounds * cus || one_round;
    if (mid_fits && (!big_fits || 3 * mid_rounds <= 4 * rounds))
      return launch_mfma_tile<T, TOUT, DUAL, 4, 2, 2, 2, 3>(x, w, y, n, m, k, nsplit, act, stream);
    if (big_fits)
      return launch_mfma_tile<T, TOUT, DUAL, 2, 2, 4, 4>(x, w, y, n, m, k, nsplit, act, stream);
  }
  const long tall = (long)ceil_div(n, 256) * tx * nsplit;
  if (tall >= 2L * cus && 10 * tall >= 9L * ceil_div(tall, (long)cus) * cus)   // two rounds at least, nine tenths full
    return launch_mfma_tile<T, TOUT, DUAL, 4, 2>(x, w, y, n, m, k, nsplit, act, stream);
  const long tiles = (long)ceil_div(n, 128) * tx * nsplit;
  if (tiles <= cus) return launch_mfma_tile<T, TOUT, DUAL, 2, 3>(x, w, y, n, m, k, nsplit, act, stream);   // one per CU at most
  return launch_mfma_tile<T, TOUT, DUAL, 2, 2>(x, w, y, n, m, k, nsplit, act, stream);
}

// ------------------------------------------------------------------ bf16 MFMA skinny
// Up to 16*NT rows of X (decode batches).  A workgroup takes 64 rows of W and
// one slice of K: it first puts its slice of X into LDS, then each of its four
// waves streams 16 rows of W straight from memory, eight 16-byte loads ahead,
// and multiplies them with X from LDS.  MFMA 16x16x32 with A = W tile,
// B = X^T, so D[w row][x row]: lane l (g = l/16, c = l%16) holds
// A[c][8g..8g+7], B[8g..8g+7][c], D[4g+i][c].
constexpr int SK_SLICE_MAX = 512;             // K per workgroup at most
constexpr int SK_LD = SK_SLICE_MAX + 8;       // LDS row stride (elements): 16-byte reads conflict-free
constexpr int SK_AHEAD = 8;                   // W loads in flight per lane

template <int NT, int RT>   // NT: 16-row tiles of X; RT: 16-row tiles of W per wave (1 or 2)
__global__ __launch_bounds__(256) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ X,
                                                               const bf16_t* __restrict__ W,
                                                               float* __restrict__ Y, int n, int m,
                                                               int k, int kslice) {
  extern __shared__ __attribute__((aligned(16))) bf16_t xs[];   // [NT*16][SK_LD]
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int g = lane / 16, c = lane % 16;
  const int kbeg = blockIdx.y * kslice;
  const int kend = min(k, kbeg + kslice);
  const int klen = kend - kbeg;                                  // a multiple of 8
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // This wave's rows of W; their first loads go out before X is staged.  With RT = 2 a
  // wave multiplies every piece of X it reads from LDS with two tiles of W, and a
  // workgroup stages X once for 128 rows of W instead of 64.
  const long m0 = ((long)blockIdx.x * 4 + wave) * 16 * RT;
  const bf16_t* wp[RT];
  bool wok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const long wrow = m0 + rt * 16 + c;
    wok[rt] = wrow < m;
    wp[rt] = W + (wok[rt] ? wrow : 0) * k + kbeg + 8 * g;
  }
  const int steps = (klen + 31) / 32;
  auto load_a = [&](int rt, int s) -> bf16x8 {
    return (wok[rt] && s < steps && 32 * s + 8 * g < klen) ? *reinterpret_cast<const bf16x8*>(wp[rt] + 32 * s)
                                                            : zero;
  };
  bf16x8 cur[RT][SK_AHEAD], nxt[RT][SK_AHEAD];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int u = 0; u < SK_AHEAD; ++u) cur[rt][u] = load_a(rt, u);

  // Stage X[0..16*NT)[kbeg..kend) in LDS, eight 16-byte loads in flight per thread.
  const int chunks = (klen + 7) / 8;
  const int total = NT * 16 * chunks;
  for (int base = tid; base < total; base += 256 * 8) {
    bf16x8 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * 256;
      const int r = idx / chunks, ch = idx % chunks;
      v[j] = (idx < total && r < n) ? *reinterpret_cast<const bf16x8*>(X + (long)r * k + kbeg + ch * 8) : zero;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * 256;
      if (idx < total) {
        const int r = idx / chunks, ch = idx % chunks;
        *reinterpret_cast<bf16x8*>(&xs[r * SK_LD + ch * 8]) = v[j];
      }
    }
  }
  __syncthreads();
  if (m0 >= m) return;

  floatx4 acc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[rt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int s0 = 0; s0 < steps; s0 += SK_AHEAD) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int u = 0; u < SK_AHEAD; ++u) nxt[rt][u] = load_a(rt, s0 + SK_AHEAD + u);
#pragma unroll
    for (int u = 0; u < SK_AHEAD; ++u) {
      const int s1 = s0 + u;
      if (s1 < steps) {
        const bool kin = 32 * s1 + 8 * g < klen;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const bf16x8 b = kin ? *reinterpret_cast<const bf16x8*>(&xs[(t * 16 + c) * SK_LD + 32 * s1 + 8 * g])
                               : zero;
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[rt][u], b, acc[rt][t], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int u = 0; u < SK_AHEAD; ++u) cur[rt][u] = nxt[rt][u];
  }

  // A lane holds four neighbouring columns of one row of X: one 16-byte store where the
  // row length allows it.
  float* out = Y + (long)blockIdx.y * n * m;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const long col0 = m0 + rt * 16 + 4 * g;
    const bool vec = m % 4 == 0 && col0 + 3 < m && ((uintptr_t)Y & 15) == 0;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int xr = t * 16 + c;
      if (xr >= n) continue;
      if (vec) {
        *reinterpret_cast<floatx4*>(&out[(long)xr * m + col0]) = acc[rt][t];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col0 + i < m) out[(long)xr * m + col0 + i] = acc[rt][t][i];
      }
    }
  }
}

// ------------------------------------------------------------------ gemv
// One wave per row of W, NT (<= 8) rows of X; lanes stride over K in chunks
// of 8 elements.  Four rows of W per workgroup.
template <typename T, int NT>
__global__ __launch_bounds__(256) void gemv_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                   float* __restrict__ Y, int n, int m, int k,
                                                   int kslice, int vec_ok) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const long row = (long)blockIdx.x * 4 + wave;
  if (row >= m) return;
  const int kbeg = blockIdx.y * kslice;
  const int kend = min(k, kbeg + kslice);
  const T* w = W + row * k;
  float acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = 0.f;

  constexpr int V = 16 / sizeof(T);  // elements per 16-byte load
  typedef T vec_t __attribute__((ext_vector_type(V)));
  if (vec_ok) {
    for (int i = kbeg + lane * V; i < kend; i += kWave * V) {
      const vec_t wv = *reinterpret_cast<const vec_t*>(w + i);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (t < n) {
          const vec_t xv = *reinterpret_cast<const vec_t*>(X + (long)t * k + i);
#pragma unroll
          for (int e = 0; e < V; ++e) acc[t] = fmaf(to_f32(wv[e]), to_f32(xv[e]), acc[t]);
        }
      }
    }
  } else {
    for (int i = kbeg + lane; i < kend; i += kWave) {
      const float wv = to_f32(w[i]);
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n) acc[t] = fmaf(wv, to_f32(X[(long)t * k + i]), acc[t]);
    }
  }
  float* out = Y + (long)blockIdx.y * n * m;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const float s = wave_sum(acc[t]);
    if (lane == 0 && t < n) out[(long)t * m + row] = s;
  }
}

// ------------------------------------------------------------------ streaming gemv
// Up to 4 rows of X.  A wave takes R rows of W and one slice of K and has all
// of a slice's loads in flight at once: U steps of 64 lanes x 16 bytes per row.
template <typename T, int NT, int R, int U>
__global__ __launch_bounds__(256) void gemv_stream_kernel(const T* __restrict__ X,
                                                          const T* __restrict__ W,
                                                          float* __restrict__ Y, int n, int m, int k,
                                                          int kslice) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const long row0 = ((long)blockIdx.x * 4 + wave) * R;
  if (row0 >= m) return;
  const int kbeg = blockIdx.y * kslice;
  const int kend = min(k, kbeg + kslice);
  float acc[R][NT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[r][t] = 0.f;

  for (int k0 = kbeg + lane * V; k0 < kend; k0 += U * kWave * V) {
    vec_t wv[U][R], xv[U][NT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * kWave * V;
      const bool kin = kk < kend;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const bool ok = kin && row0 + r < m;
        wv[u][r] = ok ? *reinterpret_cast<const vec_t*>(W + (row0 + r) * k + kk) : vec_t{};
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const bool ok = kin && t < n;
        xv[u][t] = ok ? *reinterpret_cast<const vec_t*>(X + (long)t * k + kk) : vec_t{};
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < V; ++e)
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const float wf = to_f32(wv[u][r][e]);
#pragma unroll
          for (int t = 0; t < NT; ++t) acc[r][t] = fmaf(wf, to_f32(xv[u][t][e]), acc[r][t]);
        }
  }
  float* out = Y + (long)blockIdx.y * n * m;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const float sum = wave_sum(acc[r][t]);
      if (lane == 0 && t < n && row0 + r < m) out[(long)t * m + row0 + r] = sum;
    }
}

}  // namespace kllm

using namespace kllm;

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// The 64-row variant of the skinny kernel stages 66,560 bytes of LDS, above the
// default limit of a launch; raise it once per kernel.
template <int NT, int RT>
static int launch_skinny(const bf16_t* x, const bf16_t* w, float* y, int n, int m, int k, int kslice,
                         int nsplit, hipStream_t stream) {
  static int raised = 0;
  const size_t lds = (size_t)NT * 16 * SK_LD * sizeof(bf16_t);
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_skinny_kernel<NT, RT>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) KLLM_FAIL((int)e, "gemm skinny: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = 1;
  }
  const dim3 grid(ceil_div(m, 64 * RT), nsplit);
  hipLaunchKernelGGL((gemm_bf16_skinny_kernel<NT, RT>), grid, dim3(256), lds, stream, x, w, y, n, m, k, kslice);
  return 0;
}

extern "C" int kllm_gemm_decode_tile_cols(int n, int m, int k) {
  return n <= 64 && (long)m * k < kNarrowBelow ? 64 : MBN;
}

extern "C" int kllm_gemm(const void* x, const void* w, void* y, int n, int m, int k, int dtype,
                         int out_dtype, int algo, int nsplit, hipStream_t stream) {
  KLLM_REQUIRE(x && w && y, "gemm: null pointer");
  KLLM_REQUIRE(n > 0 && m > 0 && k > 0, "gemm: bad sizes n=%d m=%d k=%d", n, m, k);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "gemm: unknown dtype %d", dtype);
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == dtype, "gemm: output dtype %d with input %d",
               out_dtype, dtype);
  KLLM_REQUIRE(nsplit >= 1 && nsplit <= 256, "gemm: nsplit %d is outside [1, 256]", nsplit);
  KLLM_REQUIRE((long)n * m < (1L << 31) && (long)m * k < (1L << 40), "gemm: sizes overflow");

  if (algo == KLLM_GEMM_PLAIN) {
    KLLM_REQUIRE(nsplit == 1, "gemm plain: no split");
    const long total = (long)n * m;
    const dim3 grid(ceil_div(total, 256));
    if (dtype == DT_F32)
      hipLaunchKernelGGL((gemm_plain_kernel<float, float>), grid, dim3(256), 0, stream,
                         (const float*)x, (const float*)w, (float*)y, n, m, k);
    else if (out_dtype == DT_F32)
      hipLaunchKernelGGL((gemm_plain_kernel<bf16_t, float>), grid, dim3(256), 0, stream,
                         (const bf16_t*)x, (const bf16_t*)w, (float*)y, n, m, k);
    else
      hipLaunchKernelGGL((gemm_plain_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream,
                         (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, n, m, k);
    KLLM_CHECK_LAUNCH("gemm plain");
    return 0;
  }

  if (algo == KLLM_GEMM_TILED_F32) {
    KLLM_REQUIRE(dtype == DT_F32 && out_dtype == DT_F32, "gemm tiled: float32 only");
    KLLM_REQUIRE(nsplit == 1, "gemm tiled: no split");
    const int vec_ok = (k % 4 == 0) && aligned16(x) && aligned16(w);
    const dim3 grid(ceil_div(m, TBN), ceil_div(n, TBM));
    hipLaunchKernelGGL((gemm_f32_tiled_kernel<float>), grid, dim3(256), 0, stream, (const float*)x,
                       (const float*)w, (float*)y, n, m, k, vec_ok);
    KLLM_CHECK_LAUNCH("gemm tiled");
    return 0;
  }

  if (algo == KLLM_GEMM_MFMA_BF16 || algo == KLLM_GEMM_MFMA_F32) {
    const bool f32 = algo == KLLM_GEMM_MFMA_F32;
    const int stage = f32 ? MROW / 4 : MROW / 2, chunk = f32 ? 4 : 8;   // elements of K per stage, per 16 bytes
    KLLM_REQUIRE(dtype == (f32 ? DT_F32 : DT_BF16), "gemm mfma: algorithm %d does not take dtype %d", algo, dtype);
    KLLM_REQUIRE(nsplit == 1 || out_dtype == DT_F32, "gemm mfma: K is split only for float32 partial sums");
    KLLM_REQUIRE(nsplit <= 16 && (long)(ceil_div(ceil_div(k, nsplit), stage) * stage) * (nsplit - 1) < k,
                 "gemm mfma: nsplit %d leaves an empty slice of K=%d", nsplit, k);
    KLLM_REQUIRE(k % chunk == 0 && aligned16(x) && aligned16(w),
                 "gemm mfma: K=%d must be a multiple of %d and the operands 16-byte aligned", k, chunk);
    int rc = f32 ? launch_mfma<float, float, false>(x, w, y, n, m, k, nsplit, 0, stream)
             : out_dtype == DT_F32 ? launch_mfma<bf16_t, float, false>(x, w, y, n, m, k, nsplit, 0, stream)
                                   : launch_mfma<bf16_t, bf16_t, false>(x, w, y, n, m, k, 1, 0, stream);
    if (rc) return rc;
    KLLM_CHECK_LAUNCH("gemm mfma");
    return 0;
  }

  if (algo == KLLM_GEMM_SKINNY_BF16) {
    KLLM_REQUIRE(dtype == DT_BF16 && out_dtype == DT_F32,
                 "gemm skinny: bfloat16 in, float32 partial sums out");
    KLLM_REQUIRE(n <= 64, "gemm skinny: n=%d exceeds 64", n);
    KLLM_REQUIRE(k % 8 == 0 && aligned16(x) && aligned16(w),
                 "gemm skinny: K=%d must be a multiple of 8 and the operands 16-byte aligned", k);
    const int kslice = ceil_div(ceil_div(k, nsplit), 32) * 32;
    KLLM_REQUIRE(kslice <= SK_SLICE_MAX, "gemm skinny: K=%d in %d slices exceeds %d per slice", k,
                 nsplit, SK_SLICE_MAX);
    KLLM_REQUIRE((long)kslice * (nsplit - 1) < k, "gemm skinny: nsplit %d leaves an empty slice of K=%d",
                 nsplit, k);
    const bf16_t *xp = (const bf16_t*)x, *wp = (const bf16_t*)w;
    float* yp = (float*)y;
    const int nt = ceil_div(n, 16);
    // Many rows of X and of W: two tiles of W per wave, while that still leaves a workgroup
    // for every CU (measured: a gain from 33 rows of X on, a loss below).
    const bool wide = nt >= 3 && (long)ceil_div(m, 128) * nsplit >= 256;
    int rc;
    if (nt == 1) rc = launch_skinny<1, 1>(xp, wp, yp, n, m, k, kslice, nsplit, stream);
    else if (nt == 2) rc = launch_skinny<2, 1>(xp, wp, yp, n, m, k, kslice, nsplit, stream);
    else if (nt == 3) rc = wide ? launch_skinny<3, 2>(xp, wp, yp, n, m, k, kslice, nsplit, stream)
                                : launch_skinny<3, 1>(xp, wp, yp, n, m, k, kslice, nsplit, stream);
    else rc = wide ? launch_skinny<4, 2>(xp, wp, yp, n, m, k, kslice, nsplit, stream)
                   : launch_skinny<4, 1>(xp, wp, yp, n, m, k, kslice, nsplit, stream);
    if (rc) return rc;
    KLLM_CHECK_LAUNCH("gemm skinny");
    return 0;
  }

  if (algo == KLLM_GEMM_GEMV) {
    KLLM_REQUIRE(out_dtype == DT_F32, "gemv: float32 partial sums out");
    KLLM_REQUIRE(n <= 8, "gemv: n=%d exceeds 8", n);
    const int vlen = dtype == DT_F32 ? 4 : 8;
    const int vec_ok = (k % vlen == 0) && aligned16(x) && aligned16(w);
    const int unit = kWave * vlen;
    if (vec_ok && n <= 4) {
      constexpr int R = 2, U = 4;
      const int ks = ceil_div(ceil_div(k, nsplit), unit) * unit;
      KLLM_REQUIRE((long)ks * (nsplit - 1) < k, "gemv: nsplit %d leaves an empty slice of K=%d", nsplit, k);
      const dim3 sgrid(ceil_div(m, 4 * R), nsplit);
#define KLLM_GS(T, NT)                                                                           \
  hipLaunchKernelGGL((gemv_stream_kernel<T, NT, R, U>), sgrid, dim3(256), 0, stream, (const T*)x, \
                     (const T*)w, (float*)y, n, m, k, ks)
      if (dtype == DT_F32) {
        if (n == 1) KLLM_GS(float, 1);
        else if (n == 2) KLLM_GS(float, 2);
        else KLLM_GS(float, 4);
      } else {
        if (n == 1) KLLM_GS(bf16_t, 1);
        else if (n == 2) KLLM_GS(bf16_t, 2);
        else KLLM_GS(bf16_t, 4);
      }
#undef KLLM_GS
      KLLM_CHECK_LAUNCH("gemv stream");
      return 0;
    }
    int kslice = ceil_div(ceil_div(k, nsplit), unit) * unit;
    KLLM_REQUIRE((long)kslice * (nsplit - 1) < k, "gemv: nsplit %d leaves an empty slice of K=%d",
                 nsplit, k);
    const dim3 grid(ceil_div(m, 4), nsplit);
#define KLLM_GEMV(T, NT)                                                                        \
  hipLaunchKernelGGL((gemv_kernel<T, NT>), grid, dim3(256), 0, stream, (const T*)x, (const T*)w, \
                     (float*)y, n, m, k, kslice, vec_ok)
    if (dtype == DT_F32) {
      if (n == 1) KLLM_GEMV(float, 1);
      else if (n == 2) KLLM_GEMV(float, 2);
      else if (n <= 4) KLLM_GEMV(float, 4);
      else KLLM_GEMV(float, 8);
    } else {
      if (n == 1) KLLM_GEMV(bf16_t, 1);
      else if (n == 2) KLLM_GEMV(bf16_t, 2);
      else if (n <= 4) KLLM_GEMV(bf16_t, 4);
      else KLLM_GEMV(bf16_t, 8);
    }
#undef KLLM_GEMV
    KLLM_CHECK_LAUNCH("gemv");
    return 0;
  }
  KLLM_FAIL(ERR_ARG, "gemm: unknown algorithm %d", algo);
}

extern "C" int kllm_gemm_swiglu(const void* x, const void* w_gate_up, void* h, int n, int f, int k,
                                int dtype, int act, hipStream_t stream) {
  KLLM_REQUIRE(x && w_gate_up && h, "gemm_swiglu: null pointer");
  KLLM_REQUIRE(act >= 0 && act < ACT_COUNT, "gemm_swiglu: unknown activation %d", act);
  KLLM_REQUIRE(n > 0 && f > 0 && k > 0, "gemm_swiglu: bad sizes n=%d f=%d k=%d", n, f, k);
  KLLM_REQUIRE(dtype == DT_BF16 || dtype == DT_F32, "gemm_swiglu: unknown dtype %d", dtype);
  const int chunk = dtype == DT_F32 ? 4 : 8;
  KLLM_REQUIRE(k % chunk == 0 && aligned16(x) && aligned16(w_gate_up),
               "gemm_swiglu: K=%d must be a multiple of %d and the operands 16-byte aligned", k, chunk);
  KLLM_REQUIRE((long)n * f < (1L << 31), "gemm_swiglu: sizes overflow");
  if (int rc = dtype == DT_F32 ? launch_mfma<float, float, true>(x, w_gate_up, h, n, f, k, 1, act, stream)
                               : launch_mfma<bf16_t, bf16_t, true>(x, w_gate_up, h, n, f, k, 1, act, stream))
    return rc;
  KLLM_CHECK_LAUNCH("gemm_swiglu");
  return 0;
}
