// Error reporting and version entry points of libpith_hip.so.
#include <cstdarg>
#include <cstdio>

#include "pith_common.h"

namespace pith {
namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PITH_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return PITH_OK;
}
}  // namespace pith

extern "C" int pith_version(void) { return 100; /* 0.1.0 */ }

extern "C" const char* pith_last_error(void) { return pith::g_last_error; }

extern "C" const char* pith_error_name(int code) {
  switch (code) {
    case PITH_OK: return "PITH_OK";
    case PITH_ERR_NULL_POINTER: return "PITH_ERR_NULL_POINTER";
    case PITH_ERR_BAD_SHAPE: return "PITH_ERR_BAD_SHAPE";
    case PITH_ERR_BAD_DTYPE: return "PITH_ERR_BAD_DTYPE";
    case PITH_ERR_UNSUPPORTED: return "PITH_ERR_UNSUPPORTED";
    case PITH_ERR_MISALIGNED: return "PITH_ERR_MISALIGNED";
    case PITH_ERR_LAUNCH: return "PITH_ERR_LAUNCH";
    default: return "PITH_ERR_UNKNOWN";
  }
}
