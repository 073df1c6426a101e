// Error plumbing shared by the extern "C" entry points: every entry point returns 0 on success, -1 for an argument it
// rejects (message via gaac_last_error()), or the positive hipError_t of a failed launch.  Entry points allocate no
// memory, never synchronize, and enqueue all work on the stream they are given.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdarg>

namespace gaac {
char* last_error_buffer();      // thread-local, 512 bytes
inline int fail(const char* fmt, ...) {
  va_list ap; va_start(ap, fmt); vsnprintf(last_error_buffer(), 512, fmt, ap); va_end(ap);
  return -1;
}
inline int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { snprintf(last_error_buffer(), 512, "%s: %s", what, hipGetErrorString(e)); return (int)e; }
  return 0;
}
}  // namespace gaac

#define GAAC_REQUIRE(cond, ...) do { if (!(cond)) return gaac::fail(__VA_ARGS__); } while (0)
