// Host-side helpers shared by the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/distca_ca.h"

namespace distca {

char *error_buffer();  // thread-local, 512 bytes

inline int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(DISTCA_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return DISTCA_OK;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Brackets a kernel launch with events when timing is enabled (see distca_timing_enable).
void timer_begin(int which, hipStream_t stream);
void timer_end(int which, hipStream_t stream);
struct ScopedTimer {
  int which;
  hipStream_t stream;
  ScopedTimer(int w, hipStream_t s) : which(w), stream(s) { timer_begin(w, s); }
  ~ScopedTimer() { timer_end(which, stream); }
};

// Number of compute units of the current device (cached per device id).
int num_compute_units();
// Per-device set-up such as raising a kernel's dynamic LDS limit is done once for each GPU the library runs
// on: pending() is true until done() has been called for `slot` on the current device.  The flag is set only
// after the set-up calls have succeeded, so a second host thread never launches ahead of them (two threads
// may both do the set-up, which is idempotent).
bool device_setup_pending(int slot);
void device_setup_done(int slot);
// Every kernel that needs such set-up exists once per element type; the fp16 builds of the sources use the upper half.
enum { kSlotPerType = 3, kSlotCount = 2 * kSlotPerType };
#ifdef DISTCA_F16
enum { kSlotFwdLds = kSlotPerType + 0, kSlotBwdDq64 = kSlotPerType + 1, kSlotBwdLds64 = kSlotPerType + 2 };
#else
enum { kSlotFwdLds = 0, kSlotBwdDq64 = 1, kSlotBwdLds64 = 2 };
#endif

}  // namespace distca
