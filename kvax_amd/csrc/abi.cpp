// Error plumbing and version of the C ABI.
#include "common.h"

namespace kvax {
namespace {
thread_local char g_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace kvax

extern "C" int kvax_abi_version(void) { return 1; }
extern "C" const char* kvax_last_error(void) { return kvax::g_error; }
