// Host-side launch helpers: per-device launch geometry, looked up the first time a device is
// used by a launcher and cached after that.  A process may drive several devices; attributes set
// with hipFuncSetAttribute and occupancy figures belong to the device that was current when
// they were set or asked for.
#pragma once
#include "of3_tiles.h"

#include <hip/hip_runtime.h>

namespace of3 {

constexpr int kMaxDevices = 64;

// cache: one slot per device, zero-initialised storage of the calling launcher (a function-local
// static).  setup(dev, &value) runs with `dev` current the first time the launcher sees it; the
// value it produces (at least 1) is returned from then on.  Concurrent first calls compute the
// same value twice, which is harmless.
template <typename Setup>
inline hipError_t per_device(int (&cache)[kMaxDevices], Setup&& setup, int* out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  if (cache[dev] == 0) {
    int v = 0;
    e = setup(dev, &v);
    if (e != hipSuccess) return e;
    cache[dev] = v > 0 ? v : 1;
  }
  *out = cache[dev];
  return hipSuccess;
}

inline hipError_t cu_count(int dev, int* n) {
  return hipDeviceGetAttribute(n, hipDeviceAttributeMultiprocessorCount, dev);
}

// work-groups of `threads` threads (no dynamic LDS) that fit the device at once
template <typename Kernel>
inline hipError_t resident_blocks(Kernel kern, int threads, int dev, int* out) {
  int cus = 0, per_cu = 0;
  hipError_t e = cu_count(dev, &cus);
  if (e != hipSuccess) return e;
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, threads, 0);
  if (e != hipSuccess) return e;
  *out = cus * (per_cu > 0 ? per_cu : 1);
  return hipSuccess;
}

// lets work-groups of Kern ask for up to max_bytes of dynamic LDS (beyond the 64 KB a kernel may use
// without asking); once per kernel and device
template <auto Kern>
inline hipError_t allow_dynamic_lds(size_t max_bytes) {
  static int cache[kMaxDevices];  // one per kernel: Kern is part of the function's identity
  int done = 0;
  return per_device(
      cache,
      [&](int, int* v) {
        *v = 1;
        return hipFuncSetAttribute(reinterpret_cast<const void*>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)max_bytes);
      },
      &done);
}

}  // namespace of3
