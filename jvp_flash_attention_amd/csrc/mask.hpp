// Mask access shared by forward and backward: eight consecutive keys of one query row.
#pragma once
#include "common.hpp"
#include "params.hpp"

namespace jvpfa {

// Boolean mask bytes (nonzero = attend) for keys key0 .. key0+7 of one query row.
// Keys >= L read as "masked".
__device__ __forceinline__ void mask_keep8(const Problem &pr, int64_t rowoff, int key0, bool keep[8]) {
  const uint8_t *base = reinterpret_cast<const uint8_t *>(pr.mask) + rowoff;
  if (pr.ms[3] == 1 && key0 + 8 <= pr.L && ((reinterpret_cast<uintptr_t>(base + key0) & 7) == 0)) {
    uint64_t w = *reinterpret_cast<const uint64_t *>(base + key0);
#pragma unroll
    for (int e = 0; e < 8; ++e) keep[e] = ((w >> (8 * e)) & 0xff) != 0;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) keep[e] = (key0 + e < pr.L) ? base[(int64_t)(key0 + e) * pr.ms[3]] != 0 : false;
  }
}

// Additive mask values (element type T) for keys key0 .. key0+7, already multiplied by log2(e).
template <typename T>
__device__ __forceinline__ void mask_bias8(const Problem &pr, int64_t rowoff, int key0, float bias[8]) {
  const T *base = reinterpret_cast<const T *>(pr.mask) + rowoff;
  if (pr.ms[3] == 1 && key0 + 8 <= pr.L && ((reinterpret_cast<uintptr_t>(base + key0) & 15) == 0)) {
    Frag<T> w = ld8<T>(base + key0);
#pragma unroll
    for (int e = 0; e < 8; ++e) bias[e] = (float)w[e] * LOG2E;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      bias[e] = (key0 + e < pr.L) ? (float)base[(int64_t)(key0 + e) * pr.ms[3]] * LOG2E : 0.f;
  }
}

}  // namespace jvpfa
