// Error reporting for the HIP allreduce library.
//
// The reference reports every failure on this path by printing a message and
// calling exit(code) (ibcomm/util.h:44-52) with the codes of util.h:32-42.  The
// C ABI returns those same codes instead and keeps the message per thread; the
// C++ IBVerbsCommunicator facade turns a non-zero return back into
// print-and-exit, so a drop-in user sees the reference's behaviour.
#pragma once

#include <stdarg.h>
#include <stdio.h>

namespace ibcomm_hip {

enum Status : int {
  kOk = 0,
  kInvalidArgument = 1,  // IBCOMM_ERROR_CODE::INVALID_ARGUMENT
  kTransportError = 2,   // IBCOMM_ERROR_CODE::IBVERBS_ERROR (loopback protocol violations)
  kDeviceError = 3,      // IBCOMM_ERROR_CODE::CUDA_ERROR (any HIP failure)
  kNotSupported = 4,     // IBCOMM_ERROR_CODE::NOT_SUPPORTED
};

inline char* LastErrorBuffer() {
  static thread_local char buf[512] = "";
  return buf;
}

inline int Fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(LastErrorBuffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline void Warn(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  fputs("ibcomm-hip warning: ", stderr);
  vfprintf(stderr, fmt, ap);
  fputc('\n', stderr);
  va_end(ap);
}

}  // namespace ibcomm_hip

#define IBCOMM_RETURN_IF_ERROR(expr) \
  do {                               \
    int _rc = (expr);                \
    if (_rc != 0) return _rc;        \
  } while (0)
