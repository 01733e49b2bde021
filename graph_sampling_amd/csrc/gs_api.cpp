// Status text and version of the C ABI.
#include <cstdarg>
#include <cstdio>

#include "../../include/gs_hip.h"

namespace gs {
namespace {
thread_local char g_error_text[512] = "";
}

void set_error_text(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error_text, sizeof(g_error_text), fmt, ap);
  va_end(ap);
}
}  // namespace gs

extern "C" {

const char* gs_status_string(int status) {
  switch (status) {
    case GS_OK:
      return "ok";
    case GS_ERR_INVALID_ARG:
    case GS_ERR_WORKSPACE:
    case GS_ERR_UNSUPPORTED:
    case GS_ERR_LAUNCH:
      return gs::g_error_text[0] ? gs::g_error_text : "error (no detail recorded)";
    default:
      return "unknown status";
  }
}

int gs_version(void) { return 100; }

}  // extern "C"
