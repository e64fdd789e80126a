// Status strings and ABI version of the C interface, and the per-device facts the launch planners ask for.
#include <atomic>

#include "tmx_kernels.h"

namespace tmx {

// Compute units of the current device, looked up once per device (256 when no device answers: the
// workspace-size queries also run on machines without a GPU).  The in-launch hand-overs use it to
// decide whether every workgroup of a launch is resident at once.
int device_cus() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return 256;
  }
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    n = 256;
  }
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

}  // namespace tmx

extern "C" const char* tmx_status_string(int status) {
  switch (status) {
    case TMX_OK: return "ok";
    case TMX_ERR_ARG: return "invalid argument (null pointer or inconsistent optional arguments)";
    case TMX_ERR_SHAPE: return "shape violates the kernel's tiling rules";
    case TMX_ERR_LAUNCH: return "HIP launch failed";
    case TMX_ERR_UNSUPPORTED: return "unsupported configuration";
    case TMX_ERR_SCRATCH: return "the request needs more scratch memory than the library's static buffer holds";
    case TMX_ERR_DEVICE_WAIT: return "a bounded wait inside a kernel ran out: results since the last status check are invalid";
    default: return "unknown status";
  }
}

extern "C" int tmx_abi_version(void) { return TMX_ABI_VERSION; }
