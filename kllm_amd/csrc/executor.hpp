// The command buffer of a step and the loop that runs it: the host side of "one native call
// issues a step's launches".  The parts of a model do not call the kernel library launch by
// launch; they record (entry point, arguments) into one buffer of 64-bit words, and a single
// call walks the buffer and calls the entry points in order, on one stream.  The role is the
// reference's te_forward_batch (backend/shim.h:106-117, backend/model.cu:995-1195): one call
// across the language boundary runs the whole forward pass; here the pass itself stays
// described by the model's parts, so any arrangement of parts runs this way.
//
// This header is plain C++ (no GPU headers): the table of entry points is handed in, so the
// loop can be built for the CPU with stand-in entry points and run under sanitizers.
//
// Layout.  A command is
//     word 0      op | nargs << 16 | words << 32   (words: the whole command, this word included)
//     word 1..    nargs argument words
//     then        payload words (structs that arguments point to)
// An argument word holds, by the C type of the parameter it stands for: a pointer or an
// integer as it is (integers sign-extended), a float's bits in the low half, a double's bits,
// nothing for the stream parameter (the loop passes its own), and for a pointer to a struct
// that travels in the buffer the offset of the struct in words from the command's word 0
// (0: null pointer), so that commands can be copied and joined without touching them.
#pragma once

#include <stdint.h>
#include <string.h>

#include <utility>

namespace kllm {
namespace cmd {

struct Context {
  const uint64_t* base;   // word 0 of the command that is being decoded: struct offsets count from here
  long words;             // the command's length
  void* stream;           // the stream every command runs on
  bool bad_offset;        // set when a struct offset points outside the command
};

// A parameter type T is decoded from its argument word by Decode<T>::get.  Pointers to
// device memory and integers are decoded here; the stream type and the structs that travel
// in the buffer are specialised where the table of entry points is defined.
template <typename T> struct Decode;
template <typename T> struct Decode<T*> {
  static T* get(uint64_t w, Context&) { return reinterpret_cast<T*>(static_cast<uintptr_t>(w)); }
};
template <> struct Decode<int> {
  static int get(uint64_t w, Context&) { return static_cast<int>(static_cast<int64_t>(w)); }
};
template <> struct Decode<long> {
  static long get(uint64_t w, Context&) { return static_cast<long>(static_cast<int64_t>(w)); }
};
template <> struct Decode<float> {
  static float get(uint64_t w, Context&) {
    const uint32_t lo = static_cast<uint32_t>(w);
    float f;
    memcpy(&f, &lo, sizeof f);
    return f;
  }
};
template <> struct Decode<double> {
  static double get(uint64_t w, Context&) {
    double d;
    memcpy(&d, &w, sizeof d);
    return d;
  }
};

// For a struct S that travels in the buffer: `template <> struct Decode<const S*> : InBuffer<S> {};`
template <typename S> struct InBuffer {
  static const S* get(uint64_t w, Context& c) {
    if (w == 0) return nullptr;
    const long need = (long)((sizeof(S) + 7) / 8);
    if (w >= (uint64_t)c.words || (long)w + need > c.words) {
      c.bad_offset = true;
      return nullptr;
    }
    return reinterpret_cast<const S*>(c.base + w);
  }
};
// For the stream type: `template <> struct Decode<stream_t> : TheStream<stream_t> {};`
template <typename S> struct TheStream {
  static S get(uint64_t, Context& c) { return static_cast<S>(c.stream); }
};

template <typename... A, size_t... I>
int invoke(int (*fn)(A...), const uint64_t* a, Context& c, std::index_sequence<I...>) {
  // every argument is decoded before the call, so that a bad offset stops it
  auto run = [&](A... v) { return c.bad_offset ? -2 : fn(v...); };
  return run(Decode<A>::get(a[I], c)...);
}

struct Op {
  const char* name;
  int nargs;
  int (*run)(const uint64_t* args, Context& c);
};

template <typename... A> constexpr int count_args(int (*)(A...)) { return (int)sizeof...(A); }
template <typename... A> int call(int (*fn)(A...), const uint64_t* a, Context& c) {
  return invoke(fn, a, c, std::index_sequence_for<A...>{});
}

// One entry of a table: KLLM_CMD_OP(kllm_embed)
#define KLLM_CMD_OP(f)                                                                     \
  ::kllm::cmd::Op {                                                                        \
    #f, ::kllm::cmd::count_args(&f),                                                       \
        [](const uint64_t* a, ::kllm::cmd::Context& c) { return ::kllm::cmd::call(&f, a, c); } \
  }

enum : int {
  RUN_OK = 0,
  RUN_MALFORMED = -3,   // the buffer itself is wrong (a length, an op, an argument count, an offset)
};

// Walks `words` 64-bit words of commands and calls their entry points in order.  Stops at the
// first command that fails: returns its code (an entry point's own, or RUN_MALFORMED for a
// command that cannot be decoded) with *failed = the command's index and *why = a static text
// for RUN_MALFORMED (else null); commands before it have run, none after it.  Returns 0 with
// *failed = -1 when all ran.
inline int run(const Op* ops, int n_ops, const uint64_t* buf, long words, void* stream, int* failed,
               const char** why) {
  Context c{buf, 0, stream, false};
  if (why) *why = nullptr;
  long at = 0;
  int index = 0;
  auto fail = [&](int code, const char* text) {
    if (failed) *failed = index;
    if (why) *why = text;
    return code;
  };
  for (; at < words; ++index) {
    const uint64_t head = buf[at];
    const int op = (int)(head & 0xFFFF), nargs = (int)((head >> 16) & 0xFFFF);
    const long len = (long)(head >> 32);
    if (len < 1 + nargs || at + len > words) return fail(RUN_MALFORMED, "a command runs past the end of the buffer");
    if (op >= n_ops) return fail(RUN_MALFORMED, "unknown entry point");
    if (nargs != ops[op].nargs) return fail(RUN_MALFORMED, "wrong number of arguments for the entry point");
    c.base = buf + at;
    c.words = len;
    c.bad_offset = false;
    const int rc = ops[op].run(buf + at + 1, c);
    if (c.bad_offset) return fail(RUN_MALFORMED, "a struct argument points outside its command");
    if (rc != 0) return fail(rc, nullptr);
    at += len;
  }
  if (failed) *failed = -1;
  return RUN_OK;
}

}  // namespace cmd
}  // namespace kllm
