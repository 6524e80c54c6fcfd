// The command-buffer loop of kllm_amd/csrc/executor.hpp built for the CPU with stand-in entry
// points, to be run under AddressSanitizer and UndefinedBehaviorSanitizer: every argument kind
// decodes to what was packed, structs travel inside their command, commands run in order and
// stop at the first failure, and malformed buffers are refused without a stray read.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "executor.hpp"

struct FakeStream {};
typedef FakeStream* fake_stream_t;
struct Pair {
  const float* p;
  int parts;
  float eps;
};

static std::vector<int> g_log;
static FakeStream g_stream;

extern "C" int op_all_kinds(const void* a, float* b, int i, long l, float f, double d, const Pair* s, fake_stream_t st) {
  const bool ok = a == (const void*)0x1000 && b == (float*)0x2000 && i == -7 && l == -(1L << 40) && f == 1.5f &&
                  d == -2.25 && s && s->p == (const float*)0x3000 && s->parts == 9 && s->eps == 0.125f && st == &g_stream;
  g_log.push_back(ok ? 1 : -1);
  return 0;
}
extern "C" int op_null_struct(const Pair* s, int v, fake_stream_t st) {
  g_log.push_back(s == nullptr && st == &g_stream ? 100 + v : -100);
  return 0;
}
extern "C" int op_fails(int code, fake_stream_t) {
  g_log.push_back(200);
  return code;
}

namespace kllm {
namespace cmd {
template <> struct Decode<fake_stream_t> : TheStream<fake_stream_t> {};
template <> struct Decode<const Pair*> : InBuffer<Pair> {};
}  // namespace cmd
}  // namespace kllm

using namespace kllm::cmd;
static const Op kOps[] = {KLLM_CMD_OP(op_all_kinds), KLLM_CMD_OP(op_null_struct), KLLM_CMD_OP(op_fails)};

static uint64_t bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static uint64_t bits(double d) { uint64_t u; memcpy(&u, &d, 8); return u; }
static uint64_t head(int op, int nargs, long words) { return (uint64_t)op | ((uint64_t)nargs << 16) | ((uint64_t)words << 32); }

#define CHECK(c) do { if (!(c)) { printf("FAILED line %d: %s\n", __LINE__, #c); return 1; } } while (0)

int main() {
  // exactly sized heap buffers, so that a read past the end is seen
  const long pair_words = (sizeof(Pair) + 7) / 8;
  Pair pr = {(const float*)0x3000, 9, 0.125f};
  std::vector<uint64_t> all = {head(0, 8, 9 + pair_words), 0x1000, 0x2000, (uint64_t)(int64_t)-7,
                               (uint64_t)(-(1L << 40)), bits(1.5f), bits(-2.25), 9, 0xdeadbeef};
  all.resize(9 + pair_words);
  memcpy(&all[9], &pr, sizeof pr);
  std::vector<uint64_t> null_s = {head(1, 3, 4), 0, 5, 0};
  std::vector<uint64_t> fails = {head(2, 2, 3), (uint64_t)(int64_t)-2, 0};
  int failed = 123;
  const char* why = "x";

  {   // three commands in order; the struct offset is relative to its own command, so joining is free
    std::vector<uint64_t> buf(null_s);
    buf.insert(buf.end(), all.begin(), all.end());
    buf.insert(buf.end(), null_s.begin(), null_s.end());
    g_log.clear();
    CHECK(run(kOps, 3, buf.data(), (long)buf.size(), &g_stream, &failed, &why) == RUN_OK);
    CHECK(failed == -1 && why == nullptr);
    CHECK(g_log == (std::vector<int>{105, 1, 105}));
  }
  {   // stops at the first failing command and names it
    std::vector<uint64_t> buf(null_s);
    buf.insert(buf.end(), fails.begin(), fails.end());
    buf.insert(buf.end(), null_s.begin(), null_s.end());
    g_log.clear();
    CHECK(run(kOps, 3, buf.data(), (long)buf.size(), &g_stream, &failed, &why) == -2);
    CHECK(failed == 1 && why == nullptr && g_log == (std::vector<int>{105, 200}));
  }
  {   // an empty buffer is fine
    g_log.clear();
    CHECK(run(kOps, 3, nullptr, 0, &g_stream, &failed, &why) == RUN_OK && failed == -1 && g_log.empty());
  }
  // malformed buffers: refused, nothing behind them runs, nothing outside them is read
  auto refused = [&](std::vector<uint64_t> buf, int at) {
    g_log.clear();
    failed = 99;
    const int rc = run(kOps, 3, buf.data(), (long)buf.size(), &g_stream, &failed, &why);
    return rc == RUN_MALFORMED && failed == at && why != nullptr;
  };
  {
    std::vector<uint64_t> b(all.begin(), all.end() - 1);     // a command cut short
    CHECK(refused(b, 0) && g_log.empty());
    b = null_s; b[0] = head(1, 3, 3);                          // fewer words than arguments
    CHECK(refused(b, 0));
    b = null_s; b[0] = head(7, 3, 4);                          // unknown entry point
    CHECK(refused(b, 0));
    b = null_s; b[0] = head(1, 2, 4);                          // wrong argument count
    CHECK(refused(b, 0));
    b = all; b[7] = (uint64_t)b.size() - pair_words + 1;        // the struct would end outside its command
    CHECK(refused(b, 0) && g_log.empty());
    b = all; b[7] = 1u << 30;                                  // ... or start far outside
    CHECK(refused(b, 0) && g_log.empty());
    b = null_s; b.insert(b.end(), all.begin(), all.end() - 2); // a good command, then a cut one
    CHECK(refused(b, 1) && g_log == (std::vector<int>{105}));
  }
  printf("executor host check: ok\n");
  return 0;
}
