// Internal helpers of the host layer.
#pragma once
#include <signal.h>
#include <stdio.h>

#include <mutex>

#include "llama_cu_hip.h"
#include "llama_cu_host.hpp"

// A failing device call is fatal, as the reference's CHECK_CUDA (llama_cu.h:48-56): print, raise.
#define LCU_CHECK(expr)                                                                              \
  do {                                                                                               \
    int lcu_status__ = (expr);                                                                       \
    if (lcu_status__ != 0) {                                                                         \
      fprintf(stderr, "%s(%d): gpu error %d: %s (source: " #expr ")\n", __func__, __LINE__,        \
              lcu_status__, lcu_last_error());                                                       \
      raise(SIGSEGV);                                                                                \
    }                                                                                                \
  } while (0)

#define RETURN_UNLESS(x) \
  if (!(x)) {            \
    return false;        \
  }

namespace llama_cu {
// Several host threads may drive contexts of one process.  Kernel launches and copies from several
// threads are everyday use of the runtime; what changes the device's set of streams, allocations
// and graphs is done by one thread at a time: stream creation and destruction, device allocation
// and release (both wait for the whole device), and everything about a graph (its capture runs in
// the capturing thread's own capture mode, and nobody allocates, frees or creates a stream under
// it; instantiation; launch; destruction).  Recursive: a context's constructor takes it around
// members that take it themselves.
inline std::recursive_mutex& device_structure_mutex() {
  static std::recursive_mutex m;
  return m;
}
using device_structure_lock = std::lock_guard<std::recursive_mutex>;

inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
inline size_t round_up(size_t a, size_t b) { return ceil_div(a, b) * b; }
}  // namespace llama_cu
