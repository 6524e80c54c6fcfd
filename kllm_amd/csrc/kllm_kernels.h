/* C ABI of the gfx950 kernel library.
 *
 * Every function takes device pointers and the HIP stream to launch on, checks
 * on the host that the sizes fit what its kernel and grid assume, and returns
 * 0, a positive HIP error code, or a negative KLLM_ERR_* value; the text of the
 * calling thread's last error is read with kllm_last_error.  The role is the
 * one backend/shim.h plays in the reference (error codes :19-27), but the
 * boundary lies lower: the host keeps the model, the cache tables and the
 * batch, and calls one kernel at a time.
 *
 * dtype arguments: 0 = float32, 1 = bfloat16.
 */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KLLM_ERR_STATE (-1)
#define KLLM_ERR_ARG (-2)

#define KLLM_GEMM_PLAIN 0
#define KLLM_GEMM_TILED_F32 1
#define KLLM_GEMM_MFMA_BF16 2
#define KLLM_GEMM_SKINNY_BF16 3
#define KLLM_GEMM_GEMV 4
#define KLLM_GEMM_GEMV_LDS 5 /* kllm_gemv_plain, reached through the Python wrapper */
#define KLLM_GEMM_MFMA_F32 6 /* MFMA 32x32x2 with 32-bit operands: no reduced precision */

/* Copies the calling thread's last error text; returns its length. */
int kllm_last_error(char* buf, int len);
/* One line about the device: name, architecture, compute units, memory. */
int kllm_device_info(int device, char* buf, int len);
/* ABI version, bumped when a signature changes. */
int kllm_abi_version(void);
/* Compute units and XCDs of the current device (the launch heuristics scale with them). */
int kllm_device_cus(void);
int kllm_device_xcds(void);

/* What the box reaches with nothing in the way, for quoting measured figures against: a
 * plain copy of `bytes` (a multiple of 16) and a loop of `iters` rounds of four independent
 * MFMAs per wave on every CU (bfloat16 32x32x16 or float32 32x32x2); *flops receives the
 * floating-point operations of the launch.  The caller times them. */
int kllm_calibrate_copy(void* dst, const void* src, long bytes, hipStream_t stream);
/* A read-only stream over `bytes`: sink receives one float per workgroup
 * (kllm_calibrate_read_workgroups() of them). */
int kllm_calibrate_read(const void* src, long bytes, float* sink, hipStream_t stream);
int kllm_calibrate_read_workgroups(void);
int kllm_calibrate_mfma(int dtype, int iters, float* sink, double* flops, hipStream_t stream);

/* out[t] = table[ids[t]]; with `from` (and `sampled`), token t whose from[t] >= 0 takes its id
 * from sampled[from[t]], a token id that an earlier launch left on the device. */
int kllm_embed(float* out, const void* table, const int* ids, const int* from, const int* sampled,
               int n, int d, int vocab, int dtype, hipStream_t stream);

/* v = x[src] + sum of the nsplit partial deltas (delta may be null);
 * x[src] = v when write_x; out[r] = rmsnorm(v) * w when out is not null.
 * src = rows[r] when rows is given (then write_x must be 0), else r. */
int kllm_add_rmsnorm(float* x, const void* delta, int delta_dtype, int nsplit, long split_stride,
                     const float* w, void* out, int out_dtype, const int* rows, int n, int d,
                     float eps, int write_x, hipStream_t stream);

/* cos and sin [n][head_dim/2] of positions[t] * theta^(-2j/head_dim), angle in double. */
int kllm_rope_tables(float* cos_t, float* sin_t, const int* positions, int n, int head_dim,
                     double theta, hipStream_t stream);

/* qkv: [nsplit][n][H*hd + 2*KV*hd] (only [n][H*hd] when cache is null).
 * Rotates q and k when cos/sin ([n][rot/2]) are given, writes q_out [n][H*hd]
 * and puts k, v into the pages of `cache` ([pages][2][KV][page_size*hd]; keys
 * [slot][hd], values [hd][slot]).  The first `rot` elements of a head are
 * rotated (rot even, at most hd; the rest pass through), in pairs (j, j + rot/2)
 * or, `interleaved`, (2j, 2j + 1). */
int kllm_rope_append(const void* qkv, int in_dtype, int nsplit, long split_stride, void* q_out,
                     const float* cos_t, const float* sin_t, void* cache, const int* positions,
                     const int* span_of_token, const int* block_table, int max_pages,
                     int page_size, int n, int H, int KV, int hd, int rot, int interleaved, int dtype,
                     hipStream_t stream);

/* The gate's activation of a gated feed-forward (`act` below). */
#define KLLM_ACT_SILU 0
#define KLLM_ACT_GELU_TANH 1

/* out[n][f] = act(gu[:, :f]) * gu[:, f:], gu = [nsplit][n][2f]. */
int kllm_silu_mul(const void* gu, int in_dtype, int nsplit, long split_stride, void* out,
                  int out_dtype, int n, int f, int act, hipStream_t stream);

/* out[count] = sum over s of in[s][count], rounded to out_dtype. */
int kllm_sum_splits(const float* in, int nsplit, long count, void* out, int out_dtype,
                    hipStream_t stream);

/* Columns of the tiles that a decode batch of n rows (at most 64) gets against w[m][k] on the
 * MFMA kernel: a caller that cuts K into slices counts its workgroups with it. */
int kllm_gemm_decode_tile_cols(int n, int m, int k);
/* y[nsplit][n][m] = x[n][k] . w[m][k]^T, 32-bit accumulation. */
int kllm_gemm(const void* x, const void* w, void* y, int n, int m, int k, int dtype, int out_dtype,
              int algo, int nsplit, hipStream_t stream);

/* h[n][f] = act(x . w[0:f]^T) * (x . w[f:2f]^T) on the MFMA tiles, h in dtype. */
int kllm_gemm_swiglu(const void* x, const void* w_gate_up, void* h, int n, int f, int k, int dtype,
                     int act, hipStream_t stream);

/* Products for up to 8 rows of x with the whole of K in one wave (no partial
 * sums) and the next elementwise step in the epilogue.  m even, K a multiple
 * of 8 (bfloat16) or 4 (float32).
 *   plain:       y[n][m] float32 = x . w^T
 *   swiglu:      h[n][f] = act(x . w[0:f]^T) * (x . w[f:2f]^T), h in dtype
 *   rope_append: w = [q; k; v] rows (only q when cache is null); rotates q and k
 *                with cos/sin [n][hd/2] (if given), writes q_out [n][H*hd] and
 *                puts k, v into the pages of `cache`
 * With `normed` (may be null) x is not read (it may be null): the kernel stages
 * normed->x * rsqrt(sum of normed->ss[row][:] / k + eps) * normed->weight, rounded to dtype,
 * the RMS norm of the residual stream that a resid product (kllm_gemv_resid) has just
 * updated, without a launch of its own; built for up to 4 rows. */
typedef struct {
  const float* x;      /* the residual stream [n][k], float32 */
  const float* weight; /* the norm's weight [k] */
  const float* ss;     /* [n][parts rounded up to 4] partial sums of squares of x's rows */
  int parts;           /* at most 512 */
  float eps;
} KllmNormedInput;     /* all three 16-byte aligned */
int kllm_gemv_plain(const void* x, const void* w, float* y, int n, int m, int k, int dtype,
                    const KllmNormedInput* normed, hipStream_t stream);
int kllm_gemv_swiglu(const void* x, const void* w_gate_up, void* h, int n, int f, int k, int dtype,
                     int act, const KllmNormedInput* normed, hipStream_t stream);
/* resid [n][m] float32 += x . w^T in place; ss_out [n][P rounded up to 4] = the
 * workgroups' partial sums of squares of resid's new rows, P = kllm_gemv_resid_parts(m). */
int kllm_gemv_resid(const void* x, const void* w, float* resid, float* ss_out, int n, int m, int k,
                    int dtype, hipStream_t stream);
int kllm_gemv_resid_parts(int m);
/* Limits of the kernels above: rows of x, rows when `normed` is given, normed->parts. */
int kllm_gemv_max_rows(void);
int kllm_gemv_normed_max_rows(void);
int kllm_gemv_normed_max_parts(void);
int kllm_gemv_rope_append(const void* x, const void* w_qkv, void* q_out, const float* cos_t,
                          const float* sin_t, void* cache, const int* positions,
                          const int* span_of_token, const int* block_table, int max_pages,
                          int page_size, int n, int H, int KV, int hd, int k, int dtype,
                          const KllmNormedInput* normed, hipStream_t stream);

/* Products of a decode batch (bfloat16, up to KLLM_FUSED_LINEAR_MAX_ROWS rows)
 * on the matrix cores, fused with the step after them.  x is [n][k] with a row
 * stride of x_stride elements (0 = k), w is [m][k].  Output:
 *   PARTS   y float32 [nsplit][n][m]; only this one may split K
 *   RESID   resid float32 [n][m] += x . w^T in place; y bfloat16 [n][m] = the new rows times
 *           norm_w [m] (the weight of the RMS norm behind the addition); ss_out
 *           [n][P rounded up to 4] = the workgroups' sums of squares of the new rows,
 *           P = kllm_fused_linear_resid_parts(m, tiles_per_wg), at most
 *           kllm_fused_linear_max_parts()
 *   SWIGLU  y bfloat16 [n][m/2] = act(x . w[0:m/2]^T) * (x . w[m/2:m]^T)
 *   ROPE    w = [q; k; v] rows (only q when cache is null): q and k rotated with
 *           cos/sin [n][hd/2] (if given); y = q_out [n][H*hd], k and v go to the
 *           tokens' pages of `cache`
 * With ss_in (SWIGLU and ROPE only) x is such a y and the sums are multiplied by the row's
 * rsqrt(sum of ss_in[row][0:ss_parts] / k + eps) before the epilogue: the RMS norm of the
 * stream, rounded to bfloat16 before the row scale instead of after it.
 * All of a workgroup's slice of K for all rows is staged in LDS:
 * kllm_fused_linear_lds_bytes says how much that needs; beyond 160 KiB see
 * kllm_fused_linear_passes. */
#define KLLM_FUSED_LINEAR_MAX_ROWS 32
#define KLLM_LINEAR_OUT_PARTS 0
#define KLLM_LINEAR_OUT_RESID 1
#define KLLM_LINEAR_OUT_SWIGLU 2
#define KLLM_LINEAR_OUT_ROPE 3
typedef struct {
  void* y;
  const float* cos_t;
  const float* sin_t;
  void* cache;
  const int* positions;
  const int* span_of_token;
  const int* block_table;
  int kind;
  int nsplit;
  int max_pages, page_size, H, KV, hd;
  int act;
  float* resid;         /* RESID */
  const float* norm_w;  /* RESID */
  float* ss_out;        /* RESID */
  const float* ss_in;   /* row scale of the sums, or null; 16-byte aligned */
  int ss_parts;
  float eps;
  int tiled;            /* w is the copy that kllm_fused_linear_tile made of the weights for this kind */
} KllmLinearOut;
long kllm_fused_linear_lds_bytes(int n, int k, int nsplit);
/* Where that is more than LDS holds, the rows are staged and multiplied in passes over K, with
 * one tile to a workgroup (tiles_per_wg = 1): how many passes a call needs (1: all at once; 0:
 * the kernel does not take the sizes). */
int kllm_fused_linear_passes(int n, int k, int nsplit);
/* A copy of w[m][k] in the order the kernel's lanes read it (a load instruction then reads one
 * contiguous kilobyte instead of 64 bytes of each of 16 rows: weights stream 20-30 % faster),
 * for one output kind (PARTS and RESID share theirs; ROPE with the heads it will be called
 * with, with_kv: whether k and v rows follow q's): wt holds
 * kllm_fused_linear_tiled_elements(kind, m, k) elements.  Pass it as w with out->tiled = 1. */
long kllm_fused_linear_tiled_elements(int kind, int m, int k);
int kllm_fused_linear_tile(const void* w, void* wt, int kind, int m, int k, int H, int KV, int hd, int with_kv,
                           hipStream_t stream);
int kllm_fused_linear_resid_parts(int m, int tiles_per_wg);
int kllm_fused_linear_max_parts(void);
int kllm_fused_linear(const void* x, int x_stride, const KllmLinearOut* out, const void* w, int n, int m,
                      int k, int tiles_per_wg, hipStream_t stream);

/* Causal attention of n tokens over the paged cache; any head size up to 256. */
int kllm_attn_generic(const void* q, void* out, const void* cache, const int* positions,
                      const int* span_of_token, const int* block_table, int max_pages,
                      int page_size, int n, int H, int KV, int hd, int window, float scale,
                      int dtype, hipStream_t stream);

/* Decode attention on the matrix cores: every token's keys are cut into
 * `nslices` slices (1..256) that run side by side (bfloat16: a workgroup of 4
 * or 8 waves to a slice; head sizes 16..128 in steps of 16, 192,
 * 256, pages a multiple of 16; float32: one wave to a slice, 32-bit MFMA, head
 * sizes in steps of 8, pages a multiple of 4); `part` is float32 scratch of
 * n*H*nslices*(hd+2) elements (bfloat16 with one slice writes the output at once
 * and leaves it untouched).  kllm_attn_decode_slices proposes nslices for a batch
 * whose longest request has at most max_keys keys (0: unknown, as for contexts
 * of 2,048).  With token_list only the n_listed tokens it names are computed (q,
 * out and part stay indexed by token row). */
int kllm_attn_decode_slices(int n, int KV, int H, int hd, int dtype, int max_keys);
/* Whether the float32 attention on the matrix cores takes this head size and page size. */
int kllm_attn_f32_fits(int hd, int page_size);
int kllm_attn_decode(const void* q, void* out, float* part, long part_floats, const void* cache,
                     const int* positions, const int* span_of_token, const int* block_table,
                     int max_pages, int page_size, int n, int H, int KV, int hd, int window,
                     float scale, int nslices, int dtype, const int* token_list, int n_listed,
                     hipStream_t stream);

/* kllm_attn_decode without a workspace argument and without any allocation: for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The partial
 * results go to an array that the library holds on every GPU it runs on
 * (KLLM_ATTN_DECODE_STATIC_FLOATS floats = 4 MiB, kept until the process ends); a call whose
 * n * H * nslices * (hd + 2) exceeds that is refused.  The array's address is looked up at
 * the first call on a device, which must be the current device (and the stream's), or by
 * kllm_attn_decode_static_init(); a first call while the stream is being captured is refused
 * (the lookup is not graph work): call the init function on the device before recording.
 * All calls on one GPU share the array and it keeps the last call's contents: the caller
 * must serialise them on one stream per GPU (calls that overlap on one GPU, from two streams
 * or two threads, a replayed graph beside eager calls, race on it); nothing in it needs
 * clearing between calls.  Same kernels, same results as kllm_attn_decode. */
#define KLLM_ATTN_DECODE_STATIC_FLOATS (1 << 20)
int kllm_attn_decode_static_init(void);
int kllm_attn_decode_static(const void* q, void* out, const void* cache, const int* positions,
                            const int* span_of_token, const int* block_table, int max_pages,
                            int page_size, int n, int H, int KV, int hd, int window, float scale,
                            int nslices, int dtype, const int* token_list, int n_listed,
                            hipStream_t stream);

/* Prompt attention on the matrix cores (bfloat16, or float32 with 32-bit MFMA).
 * query_tiles holds (first token row, span) pairs: up to 128 consecutive tokens
 * of one span.  bfloat16: head sizes 32, 64, 96, 128, 192, 256, pages a multiple
 * of 16 and of at most 2,048 tokens, max_pages * page_size at most 2^24.
 * keys_total / keys_longest: the keys that the blocks read, all together and the
 * longest block alone, for the choice of the kernel (0: not known). */
int kllm_attn_prefill(const void* q, void* out, const void* cache, const int* query_tiles,
                      int n_tiles, const int* span_start, const int* span_pos,
                      const int* block_table, int max_pages, int page_size, int H, int KV, int hd,
                      int window, float scale, long keys_total, int keys_longest, float* part,
                      long part_floats, int nslices, int n_rows, int dtype, hipStream_t stream);
/* nslices of kllm_attn_prefill: how many workgroups share out the keys of a block and head
 * (1: none; more where few blocks of a large head would leave CUs idle; taken only when
 * keys_longest says that the longest block reads 1,280 keys or more).  With more than one,
 * `part` is room for n_rows (the rows of q) x H x nslices x (hd + 2) floats, and the results
 * are merged by a second kernel of the same call. */
int kllm_attn_prefill_slices(int n_tiles, int H, int hd);

/* out[r] = sampled index of logits[r][:]; temperature/uniform null: greedy. */
int kllm_sample(int* out, const float* logits, const float* temperature, const float* uniform,
                int rows, int vocab, hipStream_t stream);

/* A step's launches in one call.  `words` is a buffer of n_words 64-bit words holding commands
 * (executor.hpp describes the layout: entry point, argument words, structs that arguments
 * point to); they run in order on `stream`, whatever stream argument was recorded.
 * kllm_command_op gives the number that names an entry point of this header in a command
 * (-1: it cannot be recorded), kllm_command_nargs its number of arguments.  Returns 0, or the
 * code of the first command that failed with *failed = its index (-3: the buffer itself is
 * malformed); commands before it have run, none after it.  The role of the reference's
 * te_forward_batch (backend/shim.h:106-117): one call across the language boundary for the
 * whole forward pass. */
int kllm_command_op(const char* name);
int kllm_command_nargs(int op);
int kllm_run_commands(const uint64_t* words, long n_words, int* failed, hipStream_t stream);

#ifdef __cplusplus
}
#endif
