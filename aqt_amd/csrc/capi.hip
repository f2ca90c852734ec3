// Error state and version of the aqtx C-ABI.
#include "common.h"

namespace aqtx {
namespace {
thread_local char g_error[512] = {0};
}

int set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

void clear_error() { g_error[0] = 0; }

}  // namespace aqtx

extern "C" const char* aqtx_last_error(void) { return aqtx::g_error; }
extern "C" int aqtx_version(void) { return AQTX_VERSION; }
