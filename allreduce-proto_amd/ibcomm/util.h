// Error codes and helpers with the names PFNProto's ibcomm/util.h gives them, for code written
// against the reference (ibcomm/util.h:32-60, 151-175).  Header only.
#pragma once

#include <cstdio>
#include <cstdlib>

#include <unistd.h>

namespace util {

enum class IBCOMM_ERROR_CODE : int {
  INVALID_ARGUMENT = 1,
  IBVERBS_ERROR = 2,  // raised here for loopback protocol violations
  CUDA_ERROR = 3,     // raised here for HIP failures
  NOT_SUPPORTED = 4
};

// Prints where and why, then ends the process with the error code as exit status: callers of the
// reference (and its tests, tests/allreduce_test.py:95-97) rely on that exit status.  Several
// emulated ranks of one process usually hit the same error at the same moment, and exit() must not
// run its handlers on two threads at once, so the process ends with _exit() after flushing.
[[noreturn]] inline void EndProcess(IBCOMM_ERROR_CODE error_code) {
  fflush(stdout);
  fflush(stderr);
  _exit(static_cast<int>(error_code));
}

[[noreturn]] inline void IbcommError(const char* filename, int line, IBCOMM_ERROR_CODE error_code, const char* message) {
  fprintf(stderr, "Error occured at %s:L%d.\n%s\n", filename, line, message);
  EndProcess(error_code);
}

template <typename A, typename... Args>
[[noreturn]] void IbcommError(const char* filename, int line, IBCOMM_ERROR_CODE error_code, const char* format, A const& a,
                              Args const&... args) {
  fprintf(stderr, "Error occured at %s:L%d.\n", filename, line);
  fprintf(stderr, format, a, args...);
  fputs("\n", stderr);
  EndProcess(error_code);
}

inline void IbcommWarning(const char* filename, int line, const char* message) {
  fprintf(stderr, "Warning occured at %s:L%d.\n%s\n", filename, line, message);
}

template <typename A, typename... Args>
void IbcommWarning(const char* filename, int line, const char* format, A const& a, Args const&... args) {
  fprintf(stderr, "Warning occured at %s:L%d.\n", filename, line);
  fprintf(stderr, format, a, args...);
  fputs("\n", stderr);
}

template <typename T>
inline T ceilDiv(T v1, T v2) {
  return v1 % v2 ? v1 / v2 + 1 : v1 / v2;
}

// log2(n) for a power of two, 0 for anything else (including 1).
inline int GetExpOfTwo(int n) {
  if (n <= 0 || (n & (n - 1)) != 0) return 0;
  int p = 0;
  while ((1 << p) != n) p++;
  return p;
}

}  // namespace util
