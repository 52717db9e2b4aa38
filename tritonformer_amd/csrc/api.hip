// Status strings and version of the C ABI.
#include <atomic>
#include "common.h"

extern "C" const char* tf_status_string(int status) {
  switch (status) {
    case TF_OK: return "ok";
    case TF_EINVAL: return "invalid argument (size, null pointer or unsupported combination)";
    case TF_EDTYPE: return "dtype not supported by this entry point";
    case TF_EALIGN: return "pointer or stride violates an alignment requirement";
    case TF_ESHAPE: return "shape precondition violated";
    case TF_EWORKSPACE: return "workspace missing or too small";
    case TF_ELAUNCH: return "HIP kernel launch failed";
  }
  return "unknown status";
}

extern "C" int tf_version(void) { return 200; }

#ifndef TF_SOURCE_HASH
#define TF_SOURCE_HASH ""
#endif
extern "C" const char* tf_source_hash(void) { return TF_SOURCE_HASH; }

namespace tfa {

DeviceShape device_shape() {
  constexpr int kMaxDevices = 64;
  static std::atomic<uint32_t> cache[kMaxDevices];  // 0 = not read yet; else cus << 8 | xcds
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
  uint32_t packed = cache[dev].load(std::memory_order_relaxed);
  if (packed == 0) {
    int cus = 0, xcds = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess || xcds <= 0) xcds = 8;
    (void)hipGetLastError();
    if (xcds > 255) xcds = 255;
    packed = ((uint32_t)cus << 8) | (uint32_t)xcds;
    cache[dev].store(packed, std::memory_order_relaxed);  // every thread computes the same value
  }
  return {(int)(packed >> 8), (int)(packed & 255u)};
}

}  // namespace tfa

extern "C" int tf_device_info(int* cus, int* xcds) {
  if (!cus || !xcds) return TF_EINVAL;
  const tfa::DeviceShape d = tfa::device_shape();
  *cus = d.cus;
  *xcds = d.xcds;
  return TF_OK;
}
