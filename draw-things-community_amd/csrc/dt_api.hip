// Library identification and the device check shared by all entry points.
#include <atomic>

#include "dt_common.h"
#include "dt_layout.h"

namespace dt {

bool device_ok() {
  // 0 = unknown, 1 = gfx950, 2 = other.  Per-process; a process drives one GPU.
  static std::atomic<int> state{0};
  int s = state.load(std::memory_order_acquire);
  if (s == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    s = 2;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
      const char* a = prop.gcnArchName;
      if (a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0') s = 1;
    }
    state.store(s, std::memory_order_release);
  }
  return s == 1;
}

}  // namespace dt

DT_EXPORT const char* dt_version(void) { return "dthip 0.1 (gfx950)"; }

DT_EXPORT dt_status dt_init(int device) {
  if (hipSetDevice(device) != hipSuccess) return DT_INVALID;
  return dt::device_ok() ? DT_OK : DT_NO_KERNEL;
}

DT_EXPORT int64_t dt_qx_bytes(int32_t qbits, int32_t nib, int64_t count) {
  return dt::qx_total_bytes(qbits, nib, count);
}
