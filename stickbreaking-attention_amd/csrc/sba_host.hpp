// Host-side launch facts that do not change while the process lives, looked up once per device instead of on every
// call: the compute-unit count, and which kernels have had their dynamic-LDS limit raised on which device.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

namespace sba {

inline hipError_t device_cus(int* dev_out, int* cus_out) {
  static std::atomic<int> cached[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  int cus = (dev >= 0 && dev < 64) ? cached[dev].load(std::memory_order_relaxed) : 0;
  if (cus == 0) {
    if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
    if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
  }
  *dev_out = dev; *cus_out = cus;
  return hipSuccess;
}

template <typename Kernel>
inline hipError_t raise_lds_limit(Kernel kernel, std::atomic<uint64_t>& done, int dev, size_t lds_bytes) {
  const uint64_t bit = (dev >= 0 && dev < 64) ? (uint64_t)1 << dev : 0;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e == hipSuccess && bit) done.fetch_or(bit, std::memory_order_release);
  return e;
}

}  // namespace sba
