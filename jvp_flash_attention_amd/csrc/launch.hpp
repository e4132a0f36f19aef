// Host-side launch helpers shared by the per-instance translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace jvpfa {

// Workgroups here use more than the 64 KB of LDS a kernel gets by default; gfx950 has 160 KB
// per CU.  Raising the limit is per function and idempotent, so it is simply done on every
// launch (a host-side table lookup in the HIP runtime, no device work).
inline int allow_lds(const void *kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  return e == hipSuccess ? 0 : -6;
}

}  // namespace jvpfa
