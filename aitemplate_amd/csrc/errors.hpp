// Thread-local error message behind aitamd_last_error(): launchers return a
// non-zero code and never throw across the C boundary.
#pragma once

#include <stdarg.h>
#include <stdio.h>

#include <string>

namespace aitamd {

inline std::string& last_error() {
  static thread_local std::string msg;
  return msg;
}

inline int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
inline int fail(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error() = buf;
  return 1;
}

}  // namespace aitamd
