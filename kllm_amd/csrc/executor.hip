// The entry points that a command buffer may name, and the call that runs one
// (see executor.hpp for the buffer and the loop).
#include "executor.hpp"

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {
namespace cmd {

template <> struct Decode<hipStream_t> : TheStream<hipStream_t> {};
template <> struct Decode<const KllmNormedInput*> : InBuffer<KllmNormedInput> {};
template <> struct Decode<const KllmLinearOut*> : InBuffer<KllmLinearOut> {};

// Every entry point that launches work on a stream.  A command names one by its index here;
// the host asks for the index by name (kllm_command_op), so the order is free to change.
static const Op kOps[] = {
    KLLM_CMD_OP(kllm_embed),
    KLLM_CMD_OP(kllm_add_rmsnorm),
    KLLM_CMD_OP(kllm_rope_tables),
    KLLM_CMD_OP(kllm_rope_append),
    KLLM_CMD_OP(kllm_silu_mul),
    KLLM_CMD_OP(kllm_sum_splits),
    KLLM_CMD_OP(kllm_gemm),
    KLLM_CMD_OP(kllm_gemm_swiglu),
    KLLM_CMD_OP(kllm_gemv_plain),
    KLLM_CMD_OP(kllm_gemv_swiglu),
    KLLM_CMD_OP(kllm_gemv_resid),
    KLLM_CMD_OP(kllm_gemv_rope_append),
    KLLM_CMD_OP(kllm_fused_linear),
    KLLM_CMD_OP(kllm_attn_generic),
    KLLM_CMD_OP(kllm_attn_decode),
    KLLM_CMD_OP(kllm_attn_prefill),
    KLLM_CMD_OP(kllm_sample),
};
constexpr int kNumOps = (int)(sizeof(kOps) / sizeof(kOps[0]));

}  // namespace cmd
}  // namespace kllm

using namespace kllm;

extern "C" int kllm_command_op(const char* name) {
  if (!name) return -1;
  for (int i = 0; i < cmd::kNumOps; ++i)
    if (strcmp(cmd::kOps[i].name, name) == 0) return i;
  return -1;
}

extern "C" int kllm_command_nargs(int op) { return op >= 0 && op < cmd::kNumOps ? cmd::kOps[op].nargs : -1; }

extern "C" int kllm_run_commands(const uint64_t* words, long n_words, int* failed, hipStream_t stream) {
  if (failed) *failed = -1;
  KLLM_REQUIRE(words && n_words >= 0 && ((uintptr_t)words & 7) == 0, "run_commands: no buffer, or it is not 8-byte aligned");
  const char* why = nullptr;
  const int rc = cmd::run(cmd::kOps, cmd::kNumOps, words, n_words, (void*)stream, failed, &why);
  if (rc == cmd::RUN_MALFORMED) set_error("run_commands: command %d: %s", failed ? *failed : -1, why ? why : "malformed");
  return rc;
}
