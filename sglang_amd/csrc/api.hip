// Error reporting and ABI version of the fp8k library.
#include <atomic>

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

// Compute units of the current device, read once per device (a read-only cache; 256 on MI355X, which is also the
// answer when no device is visible, so that the workspace queries work on a machine without a GPU).
int num_cu() {
  constexpr int kMaxDev = 64;
  static std::atomic<int> cache[kMaxDev];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) {
    (void)hipGetLastError();
    return 256;
  }
  int n = cache[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    n = 256;
  }
  cache[dev].store(n, std::memory_order_relaxed);
  return n;
}

}  // namespace fp8k

extern "C" const char* fp8k_last_error(void) { return fp8k::g_err; }
extern "C" int fp8k_abi_version(void) { return 3; }
