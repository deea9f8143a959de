// Error convention of the C++ mirrors: die() prints to stderr and aborts, as the reference engine's does
// (altar1-4xgx10-switchless/engine/common/check.h:8-21). A non-zero status of the C ABI becomes a die().
#pragma once
#include <cstdarg>
#include <cstdio>
#include <cstdlib>

#include "../dsgx.h"

[[noreturn]] inline void die(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::vfprintf(stderr, fmt, ap);
  va_end(ap);
  std::fputc('\n', stderr);
  std::abort();
}
#define DSGX_DIE_ON(rc)                                   \
  do {                                                    \
    if ((rc) != 0) die("%s", dsgx_last_error());          \
  } while (0)
