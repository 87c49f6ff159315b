// Internal helpers of the host layer.
#pragma once
#include <signal.h>
#include <stdio.h>

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
inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
inline size_t round_up(size_t a, size_t b) { return ceil_div(a, b) * b; }
}  // namespace llama_cu
