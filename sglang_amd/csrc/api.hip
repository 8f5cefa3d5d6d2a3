// Error reporting and ABI version of the fp8k library.
#include "fp8k_common.h"

namespace fp8k {

static thread_local char g_err[512] = {0};

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_err[0] = 0; }

}  // namespace fp8k

extern "C" const char* fp8k_last_error(void) { return fp8k::g_err; }
extern "C" int fp8k_abi_version(void) { return 2; }
