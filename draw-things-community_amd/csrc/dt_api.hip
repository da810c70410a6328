// Library identification and the device check shared by all entry points.
#include <atomic>

#include "dt_common.h"
#include "dt_layout.h"
#include "dt_sdpa.h"

namespace dt {

constexpr int kMaxDevices = 64;

// Errors after which the device (or the process's use of it) is gone: a faulted kernel, a lost or torn-down context.
// The runtime keeps reporting these whatever is called next.
static bool fatal_error(hipError_t e) {
  switch (e) {
    case hipErrorIllegalAddress:
    case hipErrorLaunchFailure:
    case hipErrorLaunchTimeOut:
    case hipErrorPriorLaunchFailure:
    case hipErrorAssert:
    case hipErrorECCNotCorrectable:
    case hipErrorDeinitialized:
    case hipErrorContextIsDestroyed:
    case hipErrorNoDevice:
    case hipErrorUnknown:
    case hipErrorRuntimeMemory:
    case hipErrorRuntimeOther: return true;
    default: return false;
  }
}

dt_status device_ready() {
  // per device ordinal: 0 = unknown, 1 = gfx950, 2 = other
  static std::atomic<int> state[kMaxDevices];
  if (const hipError_t pending = hipPeekAtLastError(); pending != hipSuccess) {
    // A fault of earlier work stays where it is, for its owner to read, and nothing is enqueued on top of it.
    if (fatal_error(pending)) return DT_DEVICE_ERROR;
    // Anything else in the thread's slot (a rejected argument, a pointer-attribute probe on host memory, peer
    // access enabled twice, an unsupported query, a stream query's "not ready") is the result of a call that has
    // already handed that code to its caller.  It is cleared so that the status read after this entry point's launch
    // belongs to that launch.
    (void)hipGetLastError();
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();  // this query's own failure
    return DT_DEVICE_ERROR;
  }
  if (dev < 0 || dev >= kMaxDevices) return DT_NO_KERNEL;
  int s = state[dev].load(std::memory_order_acquire);
  if (s == 0) {
    hipDeviceProp_t prop;
    s = 2;
    if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
      const char* a = prop.gcnArchName;
      if (a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0') s = 1;
    } else {
      (void)hipGetLastError();
    }
    state[dev].store(s, std::memory_order_release);
  }
  return s == 1 ? DT_OK : DT_NO_KERNEL;
}

}  // namespace dt

DT_EXPORT const char* dt_version(void) { return "dthip 0.1 (gfx950)"; }

DT_EXPORT dt_status dt_init(int device) {
  if (hipSetDevice(device) != hipSuccess) return DT_INVALID;
  const dt_status st = dt::device_ready();
  // the device address of this GPU's static scratch (dt_sdpa_f16_static), looked up while `device` is current
  if (st == DT_OK && !dt::sdpa_static_scratch()) return DT_DEVICE_ERROR;
  return st;
}

DT_EXPORT int64_t dt_qx_bytes(int32_t qbits, int32_t nib, int64_t count) {
  return dt::qx_total_bytes(qbits, nib, count);
}
