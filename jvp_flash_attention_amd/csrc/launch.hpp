// Host-side launch helpers shared by the per-instance translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <mutex>
#include <unordered_map>

namespace jvpfa {

// Workgroups here use more than the 64 KB of LDS a kernel gets by default; gfx950 has 160 KB
// per CU.  Raising the limit is per function and per device: it is done on a kernel's first launch
// on a device and remembered (a small table under a mutex; callers come from any thread).
inline int allow_lds(const void *kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return 0;
  static std::mutex mu;
  static std::unordered_map<const void *, uint64_t> done;  // kernel -> bit per device on which the limit is raised
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return -6;
  const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = done.find(kernel);
    if (bit && it != done.end() && (it->second & bit)) return 0;
  }
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return -6;
  std::lock_guard<std::mutex> lock(mu);
  done[kernel] |= bit;
  return 0;
}

}  // namespace jvpfa
