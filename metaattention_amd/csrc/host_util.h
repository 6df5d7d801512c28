// Host-side helpers shared by the launchers: the HIP error behind a failed launch, and what the library caches per
// device on a first call (kernel attributes, the number of CUs) in a way that concurrent first calls cannot break.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstddef>
#include <cstdint>

namespace ma {

// hipGetLastError() clears what it returns, so the launcher that sees an error keeps it here (per host thread) for the
// message the C entry point builds.
inline thread_local hipError_t t_hip_error = hipSuccess;
inline int hip_check(hipError_t e) {
  if (e == hipSuccess) return 0;
  t_hip_error = e;
  return -1;
}
// 0, or -1 after recording the error of the launches since the last check
inline int launch_status() { return hip_check(hipGetLastError()); }

inline int current_device() {
  int dev = 0;
  return hip_check(hipGetDevice(&dev)) == 0 ? dev : -1;
}

// Raises the dynamic LDS limit of the given kernels once per device.  `done` holds a bit per device ordinal.  Threads
// that meet in a first call each set the attribute (setting it twice is harmless) and none launches before it is set.
template <typename... K>
int allow_lds(std::atomic<uint64_t>& done, size_t bytes, K... kerns) {
  const int dev = current_device();
  if (dev < 0) return -1;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return 0;
  const void* list[] = {(const void*)kerns...};
  for (const void* k : list)
    if (hip_check(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes)) != 0) return -1;
  done.fetch_or(bit, std::memory_order_release);
  return 0;
}

// Number of CUs of the current device (asked once per device); 0 if there is no device.
inline int device_cus() {
  static std::atomic<int> cached[64];
  const int dev = current_device();
  if (dev < 0) return 0;
  int n = cached[dev & 63].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hip_check(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev)) != 0 || n <= 0) return 0;
  cached[dev & 63].store(n, std::memory_order_relaxed);
  return n;
}

}  // namespace ma
