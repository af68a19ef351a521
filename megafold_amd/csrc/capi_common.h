// Argument-checking helpers shared by the C-ABI entry points.
#pragma once
#include <cstdarg>
#include <cstdio>
#include <cstdint>

namespace mf {

inline char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}
inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}
inline void clear_error() { last_error_buf()[0] = 0; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline uint64_t align256(uint64_t v) { return (v + 255u) & ~uint64_t(255); }
inline int dtype_size(int dt) { return dt == 0 ? 4 : (dt == 1 || dt == 2) ? 2 : dt == 3 ? 1 : 0; }

}  // namespace mf
