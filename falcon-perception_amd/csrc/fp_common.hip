// Error reporting shared by every entry point of libfp_paged_kv.so.
#include "fp_common.h"

#include <stdarg.h>

namespace fp {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FP_OK;
}

}  // namespace fp

extern "C" int fp_abi_version(void) { return FP_ABI_VERSION; }

extern "C" const char* fp_last_error(void) { return fp::error_buffer(); }

int fp::compute_units() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached[dev] = n;
  }
  return cached[dev];
}
