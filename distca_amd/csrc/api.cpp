// Process-wide state behind the C ABI: error text and device facts.
#include "api_util.h"

#include <atomic>
#include <utility>
#include <vector>

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

namespace {
std::atomic<unsigned char> &setup_flag(int slot, bool *ok) {
  static std::atomic<unsigned char> done[64][kSlotCount];
  static std::atomic<unsigned char> none;
  int dev = 0;
  *ok = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && slot >= 0 && slot < kSlotCount;
  return *ok ? done[dev][slot] : none;
}
}  // namespace

bool device_setup_pending(int slot) {
  bool ok;
  std::atomic<unsigned char> &f = setup_flag(slot, &ok);
  return !ok || f.load(std::memory_order_acquire) == 0;
}

void device_setup_done(int slot) {
  bool ok;
  std::atomic<unsigned char> &f = setup_flag(slot, &ok);
  if (ok) f.store(1, std::memory_order_release);
}

namespace {
struct TimerState {
  bool enabled = false;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> pending[DISTCA_TIMER_COUNT];
  std::vector<std::pair<hipEvent_t, hipEvent_t>> pool;
};
TimerState &timers() {
  static TimerState t;
  return t;
}
}  // namespace

void timer_begin(int which, hipStream_t stream) {
  TimerState &t = timers();
  if (!t.enabled || which < 0 || which >= DISTCA_TIMER_COUNT) return;
  std::pair<hipEvent_t, hipEvent_t> ev;
  if (!t.pool.empty()) {
    ev = t.pool.back();
    t.pool.pop_back();
  } else if (hipEventCreate(&ev.first) != hipSuccess || hipEventCreate(&ev.second) != hipSuccess) {
    return;
  }
  (void)hipEventRecord(ev.first, stream);
  t.pending[which].push_back(ev);
}

void timer_end(int which, hipStream_t stream) {
  TimerState &t = timers();
  if (!t.enabled || which < 0 || which >= DISTCA_TIMER_COUNT || t.pending[which].empty()) return;
  (void)hipEventRecord(t.pending[which].back().second, stream);
}

}  // namespace distca

extern "C" void distca_timing_enable(int on) { distca::timers().enabled = on != 0; }

extern "C" int distca_timing_read(int which, double *total_ms, int64_t *launches) {
  using namespace distca;
  if (which < 0 || which >= DISTCA_TIMER_COUNT || !total_ms || !launches) return fail(DISTCA_E_INVALID, "timing_read: bad argument");
  TimerState &t = timers();
  double sum = 0;
  int64_t n = 0;
  for (auto &ev : t.pending[which]) {
    float ms = 0.f;
    if (hipEventSynchronize(ev.second) == hipSuccess && hipEventElapsedTime(&ms, ev.first, ev.second) == hipSuccess) {
      sum += ms;
      ++n;
    }
    t.pool.push_back(ev);
  }
  t.pending[which].clear();
  *total_ms = sum;
  *launches = n;
  return DISTCA_OK;
}

extern "C" const char *distca_last_error(void) { return distca::error_buffer(); }
extern "C" int distca_abi_version(void) { return 4; }
