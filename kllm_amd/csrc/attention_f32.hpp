// Float32 attention over the paged cache on the matrix cores (attention_f32.hip).
// Internal to the library: the entry points kllm_attn_decode and kllm_attn_prefill
// hand float32 calls to these two functions after their own checks.
#pragma once
#include <hip/hip_runtime.h>

namespace kllm {

// Largest number of slices of a token's keys (one wave each) the decode launch takes.
constexpr int kAttnF32MaxSlices = 256;

// Whether the float32 kernels take these sizes (head_dim a multiple of 8 up to 256,
// page_size a multiple of 4).
bool attn_f32_fits(int hd, int page_size);

// Decode tokens: every token's keys in `nslices` slices, one wave per (token, KV head,
// 32 heads of its group, slice); partial results in `part`, merged by a second launch
// when nslices > 1.  Returns 0 or an error code (text set).
int attn_f32_decode(const float* q, float* out, float* part, const float* cache, const int* positions,
                    const int* span_of_token, const int* block_table, int max_pages, int page_size,
                    int H, int KV, int hd, int window, float scale, int nslices, const int* token_list,
                    int count, hipStream_t stream);

// Prompt tokens: query_tiles lists (first token row, span) of blocks of up to 128
// consecutive tokens of one span; one wave per (32 tokens of a block, head).
int attn_f32_prefill(const float* q, float* out, const float* cache, const int* query_tiles, int n_tiles,
                     const int* span_start, const int* span_pos, const int* block_table, int max_pages,
                     int page_size, int H, int KV, int hd, int window, float scale, hipStream_t stream);

// Slices proposed for a decode batch of n tokens whose longest request has at most max_keys
// keys (0: unknown).
int attn_f32_slices(int n, int KV, int H, int max_keys);

}  // namespace kllm
