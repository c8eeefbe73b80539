// Process-wide state behind the C ABI: error text and device facts.
#include "api_util.h"

namespace distca {

char *error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int num_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

}  // namespace distca

extern "C" const char *distca_last_error(void) { return distca::error_buffer(); }
extern "C" int distca_abi_version(void) { return 1; }
